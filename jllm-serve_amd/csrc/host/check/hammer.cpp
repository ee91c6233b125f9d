// Hammers the native host library (page pool, step layout) with random work, for a build under AddressSanitizer and
// UndefinedBehaviorSanitizer on the CPU: every buffer handed to the library is allocated at exactly its stated
// length, so a read or write one element too far is a report. The reference hammers its pool the same way
// (src/test/java/org/robomiri/jllm/KvPoolTest.java:147). Prints "hammer ok" and returns 0, or says what disagreed.
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <map>
#include <random>
#include <vector>

#include "../host_core.h"

namespace {

int failures = 0;
#define EXPECT(cond, ...)                    \
  do {                                       \
    if (!(cond)) {                           \
      std::fprintf(stderr, "hammer: ");      \
      std::fprintf(stderr, __VA_ARGS__);     \
      std::fprintf(stderr, " (%s)\n", #cond); \
      if (++failures > 20) std::exit(1);     \
    }                                        \
  } while (0)

void hammer_pool(std::mt19937& rng, int pages, int steps) {
  void* pool = jllm_pool_new(pages);
  std::map<int, int> refs;
  for (int s = 0; s < steps; ++s) {
    const int op = (int)(rng() % 100);
    if (op < 45) {
      const int p = jllm_pool_alloc(pool);
      if ((int)refs.size() == pages) {
        EXPECT(p == -1, "alloc from a full pool gave page %d", p);
      } else {
        EXPECT(p >= 0 && p < pages && !refs.count(p), "alloc gave page %d", p);
        refs[p] = 1;
      }
    } else if (op < 60 && !refs.empty()) {
      auto it = refs.begin();
      std::advance(it, rng() % refs.size());
      EXPECT(jllm_pool_retain(pool, it->first) == 0, "retain of a held page failed");
      ++it->second;
    } else if (op < 95 && !refs.empty()) {
      auto it = refs.begin();
      std::advance(it, rng() % refs.size());
      const int left = jllm_pool_release(pool, it->first);
      EXPECT(left == it->second - 1, "release said %d references left", left);
      if (--it->second == 0) refs.erase(it);
    } else if (op < 97) {
      // pages that do not exist or are not held: refused, nothing touched
      const int bad = (rng() & 1) ? -1 - (int)(rng() % 5) : pages + (int)(rng() % 5);
      EXPECT(jllm_pool_release(pool, bad) == -1 && jllm_pool_retain(pool, bad) == -1 && jllm_pool_refs(pool, bad) == -1,
             "a page that does not exist was accepted");
    } else {
      // the free list in another order; a list of the wrong length or with a held page is refused
      std::vector<int32_t> list((size_t)jllm_pool_free_pages(pool));
      EXPECT(jllm_pool_free_list(pool, list.data()) == (int)list.size(), "free list length");
      for (size_t i = list.size(); i > 1; --i) std::swap(list[i - 1], list[rng() % i]);
      EXPECT(jllm_pool_set_free_list(pool, list.data(), (int)list.size()) == 0, "a reordered free list was refused");
      if (!list.empty() && !refs.empty()) {
        std::vector<int32_t> wrong(list);
        wrong[0] = refs.begin()->first;
        EXPECT(jllm_pool_set_free_list(pool, wrong.data(), (int)wrong.size()) == -1, "a held page on the free list");
      }
      std::vector<int32_t> many((size_t)pages + 1);
      EXPECT(jllm_pool_alloc_many(pool, jllm_pool_free_pages(pool) + 1, many.data()) == -1, "more pages than are free");
    }
    if (s % 64 == 0) {
      int page = -1;
      EXPECT(jllm_pool_check(pool, &page) == 0, "pool check failed at page %d", page);
      EXPECT(jllm_pool_free_pages(pool) == pages - (int)refs.size(), "free count");
    }
  }
  jllm_pool_delete(pool);
}

struct Arena {  // one group's block tables: rows x stride, each allocation exactly as long as it says
  int rows, stride;
  std::vector<int32_t> data, lens;
};

void hammer_layout(std::mt19937& rng, int rounds) {
  for (int round = 0; round < rounds; ++round) {
    const int page_size = 1 << (rng() % 6);
    const int n_groups = (int)(rng() % 3);
    const int rows = 1 + (int)(rng() % 8);
    const bool decode = rng() % 3 == 0;
    const int n_entries = 1 + (int)(rng() % rows);
    std::vector<int32_t> n_tokens, pos0, slots, want_counts, tokens, wants, table_rows;
    std::vector<int> order(rows);
    for (int i = 0; i < rows; ++i) order[i] = i;
    for (int i = rows; i > 1; --i) std::swap(order[i - 1], order[rng() % i]);
    int max_ctx = 1;
    for (int i = 0; i < n_entries; ++i) {
      const int n = decode ? 1 : 1 + (int)(rng() % 40);
      const int p0 = (int)(rng() % 100);
      n_tokens.push_back(n);
      pos0.push_back(p0);
      slots.push_back(order[i]);
      table_rows.push_back(order[i]);
      max_ctx = std::max(max_ctx, p0 + n);
      for (int j = 0; j < n; ++j) tokens.push_back((int32_t)(rng() % 50000));
      int nw = (int)(rng() % 3);
      if (nw > n) nw = n;
      want_counts.push_back(nw);
      for (int j = 0; j < nw; ++j) wants.push_back(j == 0 ? n - 1 : (int32_t)(rng() % n));  // the last place among them
    }
    // tables exactly as wide as the longest request needs: the last column is in use
    const int stride = (max_ctx + page_size - 1) / page_size;
    std::vector<Arena> arenas((size_t)n_groups);
    for (auto& a : arenas) {
      a.rows = rows;
      a.stride = stride;
      a.data.assign((size_t)rows * stride, -7);
      a.lens.assign((size_t)rows, 0);
      for (int i = 0; i < n_entries; ++i) {
        const int need = (pos0[i] + n_tokens[i] + page_size - 1) / page_size;
        a.lens[table_rows[i]] = need;
        for (int k = 0; k < need; ++k) a.data[(size_t)table_rows[i] * stride + k] = (int32_t)(rng() % 1000);
      }
    }
    std::vector<const int32_t*> ap, lp;
    std::vector<int64_t> st;
    for (auto& a : arenas) {
      ap.push_back(a.data.data());
      lp.push_back(a.lens.data());
      st.push_back(a.stride);
    }
    const int pad_rows = decode && rng() % 2 ? n_entries + (int)(rng() % 9) : 0;
    JllmStepBatch b{};
    b.n_entries = n_entries;
    b.n_tokens = n_tokens.data();
    b.pos0 = pos0.data();
    b.state_slots = slots.data();
    b.tokens = tokens.data();
    b.tokens_len = (int64_t)tokens.size();
    b.want_counts = want_counts.data();
    b.wants = wants.data();
    b.wants_len = (int64_t)wants.size();
    b.pad_rows = pad_rows;
    b.pad_state_slot = rows;
    b.min_width = rng() % 4 == 0 ? stride + 3 : 0;
    b.page_size = page_size;
    b.n_groups = n_groups;
    b.arena_rows = rows;
    b.arena = ap.data();
    b.arena_stride = st.data();
    b.table_rows = table_rows.data();
    b.table_lens = lp.data();
    JllmStepSizes sizes{};
    int32_t none = 0;
    EXPECT(jllm_step_layout(&b, &none, 0, &sizes) == -1, "round %d: a buffer of no room was written", round);
    const int64_t total = 3 * (int64_t)sizes.T + sizes.R + sizes.S + (int64_t)n_groups * (sizes.T + (int64_t)sizes.R * sizes.width);
    std::vector<int32_t> out((size_t)total);  // exactly as long as the builder says it needs
    const int64_t got = jllm_step_layout(&b, out.data(), total, &sizes);
    EXPECT(got == total, "round %d: wrote %lld of %lld", round, (long long)got, (long long)total);
    if (got == total) {
      // spot checks: positions follow pos0, selected rows lie inside the step, slots name the table's page
      int64_t row = 0;
      for (int i = 0; i < n_entries; ++i) {
        EXPECT(out[(size_t)(sizes.T + row)] == pos0[i], "round %d: first position of entry %d", round, i);
        row += n_tokens[i];
      }
      for (int s = 0; s < sizes.S; ++s) {
        const int32_t r = out[(size_t)(3 * (int64_t)sizes.T + sizes.R + s)];
        EXPECT(r >= 0 && r < sizes.T, "round %d: selected row %d outside the step", round, r);
      }
      for (int64_t r = n_entries; r < sizes.R; ++r)
        EXPECT(out[(size_t)(3 * (int64_t)sizes.T + r)] == rows, "round %d: a padding request with a live state slot", round);
    }
    // the same batch made wrong in one place is refused before anything is read through the wrong value
    JllmStepBatch bad = b;
    std::vector<int32_t> w2(wants), rows2(table_rows), n2(n_tokens), lens2;
    switch (rng() % 5) {
      case 0:
        if (!w2.empty()) {
          w2[0] = n_tokens[0] + (int32_t)(rng() % 1000);
          for (int i = 0, k = 0; i < n_entries; ++i) {
            if (want_counts[i]) { w2[(size_t)k] = n_tokens[i] + (int32_t)(rng() % 1000); break; }
            k += want_counts[i];
          }
          bad.wants = w2.data();
          EXPECT(jllm_step_layout(&bad, out.data(), total, &sizes) == -3, "round %d: a wanted place beyond its entry", round);
        }
        break;
      case 1:
        if (n_groups) {
          rows2[0] = rows + (int32_t)(rng() % 1000);
          bad.table_rows = rows2.data();
          EXPECT(jllm_step_layout(&bad, out.data(), total, &sizes) == -3, "round %d: a table row beyond the arena", round);
        }
        break;
      case 2:
        bad.tokens_len = b.tokens_len + 1;
        EXPECT(jllm_step_layout(&bad, out.data(), total, &sizes) == -3, "round %d: a token list of another length", round);
        break;
      case 3:
        if (n_groups) {
          lens2 = arenas[0].lens;
          lens2[(size_t)table_rows[0]] = stride + 1 + (int32_t)(rng() % 1000);
          std::vector<const int32_t*> lp2(lp);
          lp2[0] = lens2.data();
          bad.table_lens = lp2.data();
          EXPECT(jllm_step_layout(&bad, out.data(), total, &sizes) == -3, "round %d: a table longer than its row", round);
        }
        break;
      default:
        n2[0] = -(int32_t)(rng() % 5);
        bad.n_tokens = n2.data();
        EXPECT(jllm_step_layout(&bad, out.data(), total, &sizes) == -3, "round %d: an entry without tokens", round);
    }
    // a page that was given back under a row that is written: refused with -2
    if (n_groups && n_tokens[0] > 0) {
      Arena& a = arenas[0];
      const int k = pos0[0] / page_size;
      const int32_t keep = a.data[(size_t)table_rows[0] * stride + k];
      a.data[(size_t)table_rows[0] * stride + k] = -1;
      EXPECT(jllm_step_layout(&b, out.data(), total, &sizes) == -2, "round %d: a row in a page that was given back", round);
      a.data[(size_t)table_rows[0] * stride + k] = keep;
    }
  }
}

}  // namespace

int main(int argc, char** argv) {
  const unsigned seed = argc > 1 ? (unsigned)std::atoi(argv[1]) : 1u;
  const int rounds = argc > 2 ? std::atoi(argv[2]) : 3000;
  std::mt19937 rng(seed);
  for (int pages : {1, 2, 37, 300}) hammer_pool(rng, pages, 20000);
  hammer_layout(rng, rounds);
  if (failures) {
    std::fprintf(stderr, "hammer: %d checks failed\n", failures);
    return 1;
  }
  std::printf("hammer ok (seed %u, %d layout rounds)\n", seed, rounds);
  return 0;
}
