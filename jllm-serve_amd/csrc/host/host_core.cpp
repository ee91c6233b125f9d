#include "host_core.h"

#include <algorithm>
#include <cstdint>
#include <cstring>
#include <vector>

namespace {

struct PagePool {
  std::vector<int32_t> free;  // back() is handed out next
  std::vector<int32_t> refs;
  int high_water = 0;
  int64_t allocations = 0;
  int used() const { return (int)refs.size() - (int)free.size(); }
};

inline int ctz32(int v) { return __builtin_ctz((unsigned)v); }

}  // namespace

extern "C" {

int jllm_host_abi_version() { return 2; }

void* jllm_pool_new(int num_pages) {
  if (num_pages < 1) return nullptr;
  PagePool* p = new PagePool;
  p->refs.assign(num_pages, 0);
  p->free.resize(num_pages);
  for (int i = 0; i < num_pages; ++i) p->free[i] = num_pages - 1 - i;  // page 0 first
  return p;
}

void jllm_pool_delete(void* pool) { delete (PagePool*)pool; }

int jllm_pool_alloc(void* pool) {
  PagePool* p = (PagePool*)pool;
  if (p->free.empty()) return -1;
  const int page = p->free.back();
  p->free.pop_back();
  p->refs[page] = 1;
  ++p->allocations;
  p->high_water = std::max(p->high_water, p->used());
  return page;
}

int jllm_pool_alloc_many(void* pool, int n, int32_t* out) {
  PagePool* p = (PagePool*)pool;
  if (n < 0 || (size_t)n > p->free.size()) return -1;
  for (int i = 0; i < n; ++i) out[i] = jllm_pool_alloc(pool);
  return 0;
}

int jllm_pool_retain(void* pool, int page) {
  PagePool* p = (PagePool*)pool;
  if (page < 0 || page >= (int)p->refs.size() || p->refs[page] <= 0) return -1;
  ++p->refs[page];
  return 0;
}

int jllm_pool_release(void* pool, int page) {
  PagePool* p = (PagePool*)pool;
  if (page < 0 || page >= (int)p->refs.size() || p->refs[page] <= 0) return -1;
  if (--p->refs[page] == 0) p->free.push_back(page);
  return p->refs[page];
}

int jllm_pool_refs(void* pool, int page) {
  PagePool* p = (PagePool*)pool;
  return page < 0 || page >= (int)p->refs.size() ? -1 : p->refs[page];
}

int jllm_pool_free_pages(void* pool) { return (int)((PagePool*)pool)->free.size(); }
int jllm_pool_high_water(void* pool) { return ((PagePool*)pool)->high_water; }
int64_t jllm_pool_allocations(void* pool) { return ((PagePool*)pool)->allocations; }

int jllm_pool_free_list(void* pool, int32_t* out) {
  PagePool* p = (PagePool*)pool;
  if (!p->free.empty()) std::memcpy(out, p->free.data(), p->free.size() * sizeof(int32_t));  // no copy from or to nowhere
  return (int)p->free.size();
}

int jllm_pool_set_free_list(void* pool, const int32_t* order, int n) {
  PagePool* p = (PagePool*)pool;
  if (n != (int)p->free.size()) return -1;
  std::vector<char> seen(p->refs.size(), 0);
  for (int i = 0; i < n; ++i) {
    const int page = order[i];
    if (page < 0 || page >= (int)p->refs.size() || p->refs[page] != 0 || seen[page]) return -1;
    seen[page] = 1;
  }
  if (n > 0) std::memcpy(p->free.data(), order, (size_t)n * sizeof(int32_t));
  return 0;
}

int jllm_pool_check(void* pool, int* page) {
  PagePool* p = (PagePool*)pool;
  std::vector<char> on_list(p->refs.size(), 0);
  for (int32_t f : p->free) {
    if (on_list[f]) {
      *page = f;
      return 1;
    }
    on_list[f] = 1;
  }
  for (int i = 0; i < (int)p->refs.size(); ++i)
    if ((p->refs[i] == 0) != (on_list[i] != 0)) {
      *page = i;
      return 2;
    }
  return 0;
}

int64_t jllm_step_layout(const JllmStepBatch* b, int32_t* out, int64_t capacity, JllmStepSizes* sizes) {
  // the arguments are checked against their own stated lengths before anything is read through them
  if (b->n_entries < 0 || b->pad_rows < 0 || b->n_groups < 0 || b->page_size < 1 ||
      (b->page_size & (b->page_size - 1)) != 0 || b->arena_rows < 0)
    return -3;
  int64_t n_real = 0, n_want = 0;
  int max_ctx = 1;
  for (int i = 0; i < b->n_entries; ++i) {
    const int n = b->n_tokens[i];
    if (n < 1 || b->pos0[i] < 0 || (int64_t)b->pos0[i] + n > INT32_MAX || b->want_counts[i] < 0) return -3;
    if (b->n_groups > 0 && (b->table_rows[i] < 0 || b->table_rows[i] >= b->arena_rows)) return -3;
    for (int j = 0; j < b->want_counts[i]; ++j) {
      if (n_want + j >= b->wants_len) return -3;
      const int32_t w = b->wants[n_want + j];
      if (w < 0 || w >= n) return -3;
    }
    n_real += n;
    n_want += b->want_counts[i];
    max_ctx = std::max(max_ctx, b->pos0[i] + n);
  }
  if (n_real != b->tokens_len || n_want != b->wants_len) return -3;
  const int64_t T = std::max<int64_t>(n_real, b->pad_rows);
  const int64_t R = b->n_entries + (T - n_real);
  const int64_t S = b->pad_rows ? T : n_want;
  const int page_size = b->page_size;
  const int shift = ctz32(page_size);
  const int64_t width = std::max<int64_t>(std::max(b->min_width, 1), ((int64_t)max_ctx + page_size - 1) >> shift);
  sizes->T = (int32_t)T;
  sizes->R = (int32_t)R;
  sizes->S = (int32_t)S;
  sizes->width = (int32_t)width;
  sizes->max_context = max_ctx;
  const int64_t total = 3 * T + R + S + (int64_t)b->n_groups * (T + R * width);
  if (total > capacity) return -1;
  for (int g = 0; g < b->n_groups; ++g)
    for (int i = 0; i < b->n_entries; ++i) {
      const int len = b->table_lens[g][b->table_rows[i]];
      if (len < 0 || len > b->arena_stride[g]) return -3;
    }
  int32_t* tok = out;
  int32_t* pos = tok + T;
  int32_t* req = pos + T;
  int32_t* slots_of = req + T;
  int32_t* sel = slots_of + R;
  int32_t* next = sel + S;
  int64_t row = 0, w = 0, s = 0;
  for (int i = 0; i < b->n_entries; ++i) {
    const int n = b->n_tokens[i];
    for (int j = 0; j < n; ++j) {
      tok[row + j] = b->tokens[row + j];
      pos[row + j] = b->pos0[i] + j;
      req[row + j] = i;
    }
    if (!b->pad_rows)
      for (int j = 0; j < b->want_counts[i]; ++j) sel[s++] = (int32_t)row + b->wants[w + j];
    w += b->want_counts[i];
    slots_of[i] = b->state_slots[i];
    row += n;
  }
  for (int64_t r = n_real; r < T; ++r) {  // padded rows: one request each
    tok[r] = 0;
    pos[r] = 0;
    req[r] = (int32_t)(b->n_entries + (r - n_real));
  }
  // a padded request's state is a row that no live request can hold
  for (int64_t r = b->n_entries; r < R; ++r) slots_of[r] = b->pad_state_slot;
  if (b->pad_rows)
    for (int64_t r = 0; r < T; ++r) sel[r] = (int32_t)r;
  for (int g = 0; g < b->n_groups; ++g) {
    int32_t* slots = next;
    int32_t* table = slots + T;
    next = table + R * width;
    std::fill(slots, slots + T, -1);
    std::memset(table, 0, (size_t)(R * width) * sizeof(int32_t));
    row = 0;
    for (int i = 0; i < b->n_entries; ++i) {
      const int32_t* t = b->arena[g] + (int64_t)b->table_rows[i] * b->arena_stride[g];
      const int len = b->table_lens[g][b->table_rows[i]];
      int32_t* dst = table + (int64_t)i * width;
      const int copy = (int)std::min<int64_t>(len, width);
      for (int k = 0; k < copy; ++k) dst[k] = std::max(t[k], 0);
      for (int j = 0; j < b->n_tokens[i]; ++j) {
        const int p = b->pos0[i] + j;
        const int k = p >> shift;
        if (k >= len || t[k] < 0) return -2;
        slots[row + j] = t[k] * page_size + (p & (page_size - 1));
      }
      row += b->n_tokens[i];
    }
  }
  return total;
}

}  // extern "C"
