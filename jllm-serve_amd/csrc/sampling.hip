// Token selection on the device.
//
// Order of operations as sampling/Sampler.java:346-432: penalties, bias, then greedy (temperature 0 or
// top_k 1: the lowest index among equal maxima, :458-466) or: candidates = the top_k largest logits (all
// when top_k is 0 or >= vocab), weights exp((z - max) / T), top-p = the shortest prefix of the candidates
// in descending order whose share of the candidates' mass reaches top_p, min-p drops weights below min_p
// (the top token has weight 1), and one draw in proportion to the kept weights.
//
// No sort: the k-th largest logit and the value at which the descending cumulative mass reaches top_p are
// found by a radix descent over order-preserving keys (four passes of 256 buckets each). Masses are summed
// as 64-bit fixed point (weight * 2^40), so every sum is exact and independent of the order of the
// additions: the same logits, parameters and uniform number always select the same token. Entries equal
// to a threshold value are all kept. The draw walks the kept entries in index order.
//
// A scan of a long row by one workgroup takes about 20 us (151,936 logits), and a radix descent is four of them. So
// the row is first counted and weighed once into 2,048 buckets of 1/64 below the maximum (a bucket is a range of
// keys: a larger logit never lies in a later bucket); running sums over the buckets say in which one a threshold
// lies, that bucket's entries are gathered into LDS with one more scan, and the radix descent runs over the list.
// A bucket with more entries than the list holds (many equal logits) is handled by the descent over the whole row,
// as before: the thresholds are the same either way.
//
// Most of that time is not the scans (10 to 25 us each) but what lies between them: a radix descent is four rounds of
// a histogram and a walk over it by one thread, a sum over the workgroup is ten barriers, the draw walks a run of the
// row group by group. With top-k, or with top-p on a peaked row, everything that can be kept is among the few largest
// entries, so there is a short way first. The scan for the maximum leaves every thread's own maximum; the threads in
// m groups (m = top_k, or 64 for top-p alone) have m maxima that are m different entries, so at least m entries reach
// the smallest of them, and a few times m do, whatever the spread of the row. One more scan collects the entries that reach it, with their indices,
// into a list (up to 1,024) and weighs the rest all together. If the list is whole, each of its entries looks at all
// the others once per question: how many are larger (top-k), how much mass lies above it (top-p), how much kept mass
// has a lower index (the draw). The thresholds and the drawn token are the same as the long way's, which every other
// row still takes (top_k above 128, top-p reached beyond the list, thousands of equal logits).
#include <math.h>
#include <stddef.h>

#include "common.h"

#define SAMPLE_THREADS 1024
#define FX_ONE 1099511627776.0f  // 2^40

__device__ __forceinline__ uint32_t order_key(float f) {
  const uint32_t u = __float_as_uint(f);
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

__device__ __forceinline__ unsigned long long fx_weight(float z, float zmax, float inv_t) {
  const float x = (z - zmax) * inv_t;
  if (x < -27.8f) return 0ull;  // exp(x) * 2^40 < 1 from -27.73 down: the same zero without the exponential
  return (unsigned long long)(expf(x) * FX_ONE);
}

struct BlockScratch {
  unsigned long long hist[256];
  unsigned long long partial[SAMPLE_THREADS];
  float fv[SAMPLE_THREADS / 64];
  int iv[SAMPLE_THREADS / 64];
  unsigned long long bcast;
  uint32_t ubcast;
};

// f(i, z[i]) for every entry lo <= i < hi of a row, the lanes `first` of `stride` side by side. A scan by one
// workgroup is bound by memory latency, not by bandwidth, so a lane has 16 entries on their way at a time: four
// 16-byte loads where the run starts on a 16-byte boundary, else eight single ones. A lane sees its entries in
// ascending order.
template <typename F>
__device__ __forceinline__ void scan_row(const float* __restrict__ z, int lo, int hi, int first, int stride, F f) {
  if ((((uintptr_t)(z + lo)) & 15) == 0) {
    const int n4 = (hi - lo) >> 2;
    const float4* z4 = (const float4*)(z + lo);
    for (int q0 = first; q0 < n4; q0 += stride * 4) {
      float4 v[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int q = q0 + u * stride;
        v[u] = q < n4 ? z4[q] : float4{0.f, 0.f, 0.f, 0.f};
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int q = q0 + u * stride;
        if (q < n4) {
          const int i = lo + 4 * q;
          f(i, v[u].x);
          f(i + 1, v[u].y);
          f(i + 2, v[u].z);
          f(i + 3, v[u].w);
        }
      }
    }
    for (int i = lo + 4 * n4 + first; i < hi; i += stride) f(i, z[i]);
    return;
  }
  for (int i0 = lo + first; i0 < hi; i0 += stride * 8) {
    float v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int i = i0 + u * stride;
      v[u] = i < hi ? z[i] : 0.f;
    }
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int i = i0 + u * stride;
      if (i < hi) f(i, v[u]);
    }
  }
}

// (value, index) of the row maximum, lowest index among equals; every thread gets the result. With m > 0 (at most
// SAMPLE_THREADS), `cut_key` becomes the order key of a value that at least m entries of the row reach: the threads
// form m groups, every group's maximum is an entry of its own, and the smallest of those is taken. 0 where a group
// saw no number.
__device__ void block_argmax(const float* z, int vocab, BlockScratch& s, float& best_out, int& idx_out, int m = 0,
                             uint32_t* cut_key = nullptr) {
  float best = -INFINITY;
  int idx = 0x7fffffff;
  // ascending i per lane keeps the lower index on ties
  scan_row(z, 0, vocab, threadIdx.x, SAMPLE_THREADS, [&](int i, float v) {
    if (idx == 0x7fffffff || v > best) {
      best = v;
      idx = i;
    }
  });
  if (m > 0) {
    float* mx = (float*)s.partial;  // [SAMPLE_THREADS]
    __syncthreads();
    mx[threadIdx.x] = idx != 0x7fffffff ? best : __uint_as_float(0x7fc00000u);
    if (threadIdx.x == 0) *cut_key = 0xffffffffu;
    __syncthreads();
    if ((int)threadIdx.x < m) {
      const int lo = (int)threadIdx.x * SAMPLE_THREADS / m, hi = ((int)threadIdx.x + 1) * SAMPLE_THREADS / m;
      float gmax = -INFINITY;
      bool any = false;
      for (int t = lo; t < hi; ++t) {
        const float o = mx[t];
        if (o == o) {
          any = true;
          gmax = fmaxf(gmax, o);
        }
      }
      atomicMin(cut_key, any ? order_key(gmax) : 0u);
    }
    __syncthreads();
  }
  for (int o = 32; o > 0; o >>= 1) {
    const float ov = __shfl_xor(best, o, 64);
    const int oi = __shfl_xor(idx, o, 64);
    if (oi != 0x7fffffff && (idx == 0x7fffffff || ov > best || (ov == best && oi < idx))) {
      best = ov;
      idx = oi;
    }
  }
  __syncthreads();
  if ((threadIdx.x & 63) == 0) {
    s.fv[threadIdx.x >> 6] = best;
    s.iv[threadIdx.x >> 6] = idx;
  }
  __syncthreads();
  best = s.fv[0];
  idx = s.iv[0];
  for (int w = 1; w < SAMPLE_THREADS / 64; ++w) {
    const float ov = s.fv[w];
    const int oi = s.iv[w];
    if (oi != 0x7fffffff && (idx == 0x7fffffff || ov > best || (ov == best && oi < idx))) {
      best = ov;
      idx = oi;
    }
  }
  best_out = best;
  idx_out = idx == 0x7fffffff ? 0 : idx;
}

__device__ __forceinline__ unsigned long long wave_sum_u64(unsigned long long v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}

// Radix descent over the entries that `each(f)` hands to f. With `weighted` false: the key of the k-th largest entry
// (target = k) among entries with key >= floor_key. With `weighted` true: the key at which the descending cumulative
// mass of those entries reaches `target`.
template <typename Each>
__device__ uint32_t radix_descent(Each each, bool weighted, unsigned long long target, uint32_t floor_key, float zmax,
                                  float inv_t, BlockScratch& s) {
  uint32_t prefix = 0;
  unsigned long long remaining = target;
  for (int shift = 24; shift >= 0; shift -= 8) {
    for (int b = threadIdx.x; b < 256; b += SAMPLE_THREADS) s.hist[b] = 0ull;
    __syncthreads();
    const uint32_t high_mask = shift == 24 ? 0u : (0xffffffffu << (shift + 8));
    each([&](float v) {
      const uint32_t key = order_key(v);
      if (key < floor_key || (key & high_mask) != prefix) return;
      const unsigned long long m = weighted ? fx_weight(v, zmax, inv_t) : 1ull;
      if (m) atomicAdd(&s.hist[(key >> shift) & 0xffu], m);
    });
    __syncthreads();
    if (threadIdx.x == 0) {
      int chosen = -1;
      int lowest_nonempty = -1;
      unsigned long long rem = remaining;
      for (int b = 255; b >= 0; --b) {
        const unsigned long long h = s.hist[b];
        if (h == 0ull) continue;
        lowest_nonempty = b;
        if (h < rem) {
          rem -= h;
        } else {
          chosen = b;
          break;
        }
      }
      if (chosen < 0) {  // the target exceeds what is there (k > count): everything stays
        chosen = lowest_nonempty < 0 ? 0 : lowest_nonempty;
        rem = 1ull;
      }
      s.ubcast = (uint32_t)chosen;
      s.bcast = rem;
    }
    __syncthreads();
    prefix |= s.ubcast << shift;
    remaining = s.bcast;
    __syncthreads();
  }
  return prefix;
}

// over a whole row
__device__ uint32_t radix_threshold(const float* z, int vocab, bool weighted, unsigned long long target,
                                    uint32_t floor_key, float zmax, float inv_t, BlockScratch& s) {
  return radix_descent([&](auto f) { scan_row(z, 0, vocab, threadIdx.x, SAMPLE_THREADS, [&](int, float v) { f(v); }); },
                       weighted, target, floor_key, zmax, inv_t, s);
}

// sum over the block of a 64-bit value; every thread gets the result
__device__ unsigned long long block_sum_u64(unsigned long long v, BlockScratch& s) {
  __syncthreads();
  s.partial[threadIdx.x] = v;
  __syncthreads();
  for (int o = SAMPLE_THREADS / 2; o > 0; o >>= 1) {
    if (threadIdx.x < o) s.partial[threadIdx.x] += s.partial[threadIdx.x + o];
    __syncthreads();
  }
  const unsigned long long r = s.partial[0];
  __syncthreads();
  return r;
}

#define SB_BUCKETS 2048   // of 1/64 below the row's maximum; the last one takes everything further down
#define SB_SCALE 64.0f
#define SB_LIST 4096      // entries of one bucket that the list in LDS holds

struct BucketScratch {
  unsigned long long mass[SB_BUCKETS];
  uint32_t cnt[SB_BUCKETS];
  float list[SB_LIST];
  int n_list;
};

#define NL_CAP 1024      // entries that the list of the largest entries holds
#define NL_MAX_K 128     // the largest top_k for which it is tried (the list then has a few hundred entries)
#define NL_TOP_P_M 64    // top-p alone: the list takes what reaches the smallest of 64 groups' maxima

struct NearList {
  float v[NL_CAP];
  int i[NL_CAP];
  int n;  // how many entries belong in the list; more than it holds: it is not whole and not used
  uint32_t key_k, key_p, key_cut;
};
static_assert(NL_CAP * sizeof(unsigned long long) <= SB_LIST * sizeof(float), "the weights of the list's entries lie where the bucket list would");

__device__ __forceinline__ float key_value(uint32_t key) {  // the float whose order_key is `key`
  return __uint_as_float((key & 0x80000000u) ? (key & 0x7fffffffu) : ~key);
}

// An entry joins the list. The lanes of a wave that come here together take their places with one atomic; a thread
// that has seen the list full stops asking (`lost`): the list will not be used.
__device__ __forceinline__ void near_append(NearList& nl, bool& lost, float v, int i) {
  const bool want = !lost;
  const unsigned long long m = __ballot(want);
  if (!want) return;
  const int lane = threadIdx.x & 63;
  const int leader = __builtin_ctzll(m);
  int base = 0;
  if (lane == leader) base = atomicAdd(&nl.n, __popcll(m));
  base = __builtin_amdgcn_readlane(base, leader);
  const int at = base + __popcll(m & ((1ull << lane) - 1ull));
  if (at < NL_CAP) {
    nl.v[at] = v;
    nl.i[at] = i;
  } else {
    lost = true;
  }
}

// a larger logit never has a larger bucket: the difference and the product round monotonically
__device__ __forceinline__ int bucket_of(float v, float zmax) {
  const float t = (zmax - v) * SB_SCALE;
  return t < (float)(SB_BUCKETS - 1) ? (int)t : SB_BUCKETS - 1;  // also what is not a number
}

// The first bucket at which the running sum of val[] reaches `target` (>= 1, at most the whole sum), and the sum
// before that bucket; every thread gets both.
template <typename T>
__device__ void find_bucket(const T* val, unsigned long long target, BlockScratch& s, int& bucket,
                            unsigned long long& before) {
  constexpr int PER = SB_BUCKETS / SAMPLE_THREADS;
  unsigned long long mine = 0ull;
#pragma unroll
  for (int e = 0; e < PER; ++e) mine += val[threadIdx.x * PER + e];
  __syncthreads();
  s.partial[threadIdx.x] = mine;
  __syncthreads();
  for (int o = 1; o < SAMPLE_THREADS; o <<= 1) {  // running sums over the threads
    const unsigned long long add = threadIdx.x >= o ? s.partial[threadIdx.x - o] : 0ull;
    __syncthreads();
    s.partial[threadIdx.x] += add;
    __syncthreads();
  }
  const unsigned long long upto = s.partial[threadIdx.x];
  unsigned long long acc = upto - mine;
  if (acc < target && target <= upto) {  // exactly one thread
#pragma unroll
    for (int e = 0; e < PER; ++e) {
      const unsigned long long v = val[threadIdx.x * PER + e];
      if (acc + v >= target) {
        s.ubcast = (uint32_t)(threadIdx.x * PER + e);
        s.bcast = acc;
        break;
      }
      acc += v;
    }
  }
  __syncthreads();
  bucket = (int)s.ubcast;
  before = s.bcast;
  __syncthreads();
}

// the entries of one bucket with key >= floor_key go into the list, as many as fit; returns how many there are
__device__ int gather_bucket(const float* z, int vocab, float zmax, int bucket, uint32_t floor_key, BucketScratch& b) {
  __syncthreads();
  if (threadIdx.x == 0) b.n_list = 0;
  __syncthreads();
  scan_row(z, 0, vocab, threadIdx.x, SAMPLE_THREADS, [&](int, float v) {
    if (bucket_of(v, zmax) == bucket && order_key(v) >= floor_key) {
      const int at = atomicAdd(&b.n_list, 1);
      if (at < SB_LIST) b.list[at] = v;
    }
  });
  __syncthreads();
  return b.n_list;
}

__device__ uint32_t radix_list(const BucketScratch& b, int n, bool weighted, unsigned long long target, uint32_t floor_key,
                               float zmax, float inv_t, BlockScratch& s) {
  return radix_descent([&](auto f) { for (int i = threadIdx.x; i < n; i += SAMPLE_THREADS) f(b.list[i]); }, weighted,
                       target, floor_key, zmax, inv_t, s);
}

__global__ __launch_bounds__(SAMPLE_THREADS) void sample_kernel(
    const float* __restrict__ logits, int ld, int vocab, const float* __restrict__ temperature,
    const int* __restrict__ top_k, const float* __restrict__ top_p, const float* __restrict__ min_p,
    const double* __restrict__ uniform, int* __restrict__ out) {
  __shared__ BlockScratch s;
  const int row = blockIdx.x;
  const float* z = logits + (size_t)row * ld;
  float zmax;
  int imax;
  const float T = temperature[row];
  const int k = top_k[row];
  const bool greedy = T == 0.f || k == 1;
  const bool need_k = k > 0 && k < vocab;
  const float p = top_p[row];
  const bool need_p = p < 1.0f;
  __shared__ NearList nl;
  // the short way is tried where a threshold keeps few entries: top_k up to NL_MAX_K, or top-p alone
  const int short_m = greedy || !(need_k || need_p) ? 0 : need_k ? (k <= NL_MAX_K ? k : 0) : NL_TOP_P_M;
  block_argmax(z, vocab, s, zmax, imax, short_m, &nl.key_cut);
  if (greedy) {
    if (threadIdx.x == 0) out[row] = imax;
    return;
  }
  const float inv_t = 1.0f / T;
  uint32_t floor_key = 0u;
  const unsigned long long min_w = (unsigned long long)(min_p[row] * FX_ONE);
  __shared__ BucketScratch b;
  const uint32_t key_cut = short_m > 0 ? nl.key_cut : 0u;
  if (key_cut != 0u) {
    const float cut = key_value(key_cut);
    // ---- the short way: thresholds and draw from the list of the entries that reach `cut`
    __syncthreads();
    if (threadIdx.x == 0) {
      nl.n = 0;
      nl.key_k = nl.key_p = 0xffffffffu;
    }
    __syncthreads();
    unsigned long long far = 0ull;  // the mass of the entries that are not in the list (top-p alone weighs the whole row)
    bool lost = false;
    scan_row(z, 0, vocab, threadIdx.x, SAMPLE_THREADS, [&](int i, float v) {
      if (v >= cut)
        near_append(nl, lost, v, i);
      else if (!need_k)
        far += fx_weight(v, zmax, inv_t);
    });
    if (!need_k) far = block_sum_u64(far, s);
    __syncthreads();
    const int n = nl.n;
    if (n <= NL_CAP) {  // whole; it holds at least short_m entries, so with top-k the k-th largest is among them
      unsigned long long* lw = (unsigned long long*)b.list;  // the weights of the list's entries
      const bool have = threadIdx.x < n;
      const float v_i = have ? nl.v[threadIdx.x] : 0.f;
      const uint32_t key_i = order_key(v_i);
      const unsigned long long w_i = have ? fx_weight(v_i, zmax, inv_t) : 0ull;
      if (have) lw[threadIdx.x] = w_i;
      __syncthreads();
      uint32_t floor_k = 0u;
      if (need_k) {  // the k-th largest key: the smallest among the entries with fewer than k larger ones
        if (have) {
          int larger = 0;
          for (int j = 0; j < n; ++j) larger += order_key(nl.v[j]) > key_i;
          if (larger < k) atomicMin(&nl.key_k, key_i);
        }
        __syncthreads();
        floor_k = nl.key_k;
      }
      bool inside = true;  // top-p is reached inside the list
      uint32_t floor_p = 0u;
      if (need_p) {  // the key at which the descending mass of the candidates reaches top_p of all of it
        unsigned long long all = 0ull, above = 0ull;
        for (int j = 0; j < n; ++j) {
          const uint32_t kj = order_key(nl.v[j]);
          if (kj < floor_k) continue;
          all += lw[j];
          if (kj > key_i) above += lw[j];
        }
        unsigned long long target = (unsigned long long)ceil((double)p * (double)(all + far));  // far: 0 with top-k
        if (target < 1ull) target = 1ull;
        inside = target <= all;  // the same in every thread
        if (inside) {
          if (have && key_i >= floor_k && above < target) atomicMin(&nl.key_p, key_i);
          __syncthreads();
          floor_p = nl.key_p;
        }
      }
      if (inside) {
        const uint32_t fl = max(floor_k, floor_p);
        // the draw: the kept entry whose kept entries of lower index weigh at most r and, with it, more
        unsigned long long total = 0ull, before = 0ull;
        const int idx_i = have ? nl.i[threadIdx.x] : 0;
        for (int j = 0; j < n; ++j) {
          if (order_key(nl.v[j]) < fl || lw[j] < min_w) continue;
          total += lw[j];
          if (nl.i[j] < idx_i) before += lw[j];
        }
        if (total > 0ull) {  // always: the maximum weighs 2^40 and is kept
          unsigned long long r = (unsigned long long)(uniform[row] * (double)total);
          if (r >= total) r = total - 1ull;
          if (have && key_i >= fl && w_i >= min_w && before <= r && r < before + w_i) out[row] = idx_i;
          return;
        }
      }
    }
    __syncthreads();
  }
  // ---- the long way
  if (need_k || need_p) {
    for (int j = threadIdx.x; j < SB_BUCKETS; j += SAMPLE_THREADS) {
      b.cnt[j] = 0u;
      b.mass[j] = 0ull;
    }
    __syncthreads();
    scan_row(z, 0, vocab, threadIdx.x, SAMPLE_THREADS, [&](int, float v) {
      const int j = bucket_of(v, zmax);
      atomicAdd(&b.cnt[j], 1u);
      const unsigned long long w = fx_weight(v, zmax, inv_t);
      if (w) atomicAdd(&b.mass[j], w);
    });
    __syncthreads();
    bool listed = true;   // the thresholds so far came from bucket lists (else: from descents over the whole row)
    int jk = -1, n_list = 0;
    if (need_k) {
      unsigned long long before;
      find_bucket(b.cnt, (unsigned long long)k, s, jk, before);
      if (b.cnt[jk] <= SB_LIST) {
        n_list = gather_bucket(z, vocab, zmax, jk, 0u, b);
        floor_key = radix_list(b, n_list, false, (unsigned long long)k - before, 0u, zmax, inv_t, s);
      } else {
        floor_key = radix_threshold(z, vocab, false, (unsigned long long)k, 0u, zmax, inv_t, s);
        listed = false;
      }
    }
    if (need_p && listed) {
      if (need_k) {  // what is kept of the threshold's bucket; the buckets behind it hold nothing that is kept
        unsigned long long kept = 0ull;
        for (int i = threadIdx.x; i < n_list; i += SAMPLE_THREADS)
          if (order_key(b.list[i]) >= floor_key) kept += fx_weight(b.list[i], zmax, inv_t);
        kept = block_sum_u64(kept, s);
        for (int j = jk + threadIdx.x; j < SB_BUCKETS; j += SAMPLE_THREADS) b.mass[j] = j == jk ? kept : 0ull;
        __syncthreads();
      }
      unsigned long long mass = 0ull;
      for (int j = threadIdx.x; j < SB_BUCKETS; j += SAMPLE_THREADS) mass += b.mass[j];
      mass = block_sum_u64(mass, s);
      unsigned long long target = (unsigned long long)ceil((double)p * (double)mass);
      if (target < 1ull) target = 1ull;
      uint32_t tp = 0u;
      if (mass > 0ull) {
        int jp;
        unsigned long long before;
        find_bucket(b.mass, target, s, jp, before);
        if (need_k && jp == jk) {
          tp = radix_list(b, n_list, true, target - before, floor_key, zmax, inv_t, s);
        } else if (b.cnt[jp] <= SB_LIST) {
          n_list = gather_bucket(z, vocab, zmax, jp, floor_key, b);
          tp = radix_list(b, n_list, true, target - before, floor_key, zmax, inv_t, s);
        } else {
          tp = radix_threshold(z, vocab, true, target, floor_key, zmax, inv_t, s);
        }
      }
      floor_key = max(floor_key, tp);
    } else if (need_p) {
      unsigned long long mass = 0ull;
      scan_row(z, 0, vocab, threadIdx.x, SAMPLE_THREADS, [&](int, float v) {
        if (order_key(v) >= floor_key) mass += fx_weight(v, zmax, inv_t);
      });
      mass = block_sum_u64(mass, s);
      unsigned long long target = (unsigned long long)ceil((double)p * (double)mass);
      if (target < 1ull) target = 1ull;
      const uint32_t tp = radix_threshold(z, vocab, true, target, floor_key, zmax, inv_t, s);
      floor_key = max(floor_key, tp);
    }
  }
  // The draw takes the kept entries in index order. The row is cut into chunks of 256 entries (more where a row has
  // more chunks than fit); the waves take them in turn, four in flight each, and leave every chunk's kept mass in
  // LDS, where the buckets were. The sums say which chunk holds the drawn mass, and one wave finds the entry in it.
  constexpr int NW = SAMPLE_THREADS / 64;
  constexpr int MAX_CHUNKS = (int)((sizeof(b.mass) + sizeof(b.cnt)) / sizeof(unsigned long long));
  static_assert(offsetof(BucketScratch, mass) == 0 && offsetof(BucketScratch, cnt) == sizeof(b.mass), "the chunk sums lie over mass and cnt");
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int per = 256 * ((vocab + 256 * MAX_CHUNKS - 1) / (256 * MAX_CHUNKS));  // entries per chunk
  const int nchunks = (vocab + per - 1) / per;
  unsigned long long* csum = (unsigned long long*)&b;
  auto kept = [&](float v) -> unsigned long long {
    if (order_key(v) < floor_key) return 0ull;
    const unsigned long long w = fx_weight(v, zmax, inv_t);
    return w >= min_w ? w : 0ull;
  };
  __syncthreads();  // the buckets are done with
  for (int c0 = wave; c0 < nchunks; c0 += NW * 4) {
    unsigned long long acc[4] = {0ull, 0ull, 0ull, 0ull};
    for (int o = 0; o < per; o += 256) {
      float v[4][4];
      bool ok[4][4];
#pragma unroll
      for (int q = 0; q < 4; ++q)
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          const int c = c0 + q * NW;
          const long long i = (long long)c * per + o + u * 64 + lane;
          ok[q][u] = c < nchunks && i < vocab;
          v[q][u] = ok[q][u] ? z[i] : 0.f;
        }
#pragma unroll
      for (int q = 0; q < 4; ++q)
#pragma unroll
        for (int u = 0; u < 4; ++u)
          if (ok[q][u]) acc[q] += kept(v[q][u]);
    }
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const unsigned long long sum = wave_sum_u64(acc[q]);
      if (lane == 0 && c0 + q * NW < nchunks) csum[c0 + q * NW] = sum;
    }
  }
  __syncthreads();
  if (wave != 0) return;
  // wave 0: every lane adds a run of consecutive chunks, running sums over the lanes say which lane's run holds the
  // drawn mass, and that lane walks its run
  const int cpl = (nchunks + 63) / 64;
  const int c_lo = min(nchunks, lane * cpl), c_hi = min(nchunks, c_lo + cpl);
  unsigned long long mine = 0ull;
  for (int c = c_lo; c < c_hi; ++c) mine += csum[c];
  unsigned long long upto = mine;  // the sum of the runs up to and with this lane's
#pragma unroll
  for (int d = 1; d < 64; d <<= 1) {
    const unsigned long long up = __shfl_up(upto, d, 64);
    if (lane >= d) upto += up;
  }
  const unsigned long long total = __shfl(upto, 63, 64);
  if (total == 0ull) {
    if (lane == 0) out[row] = imax;
    return;
  }
  unsigned long long r = (unsigned long long)(uniform[row] * (double)total);
  if (r >= total) r = total - 1ull;
  const int holder = __builtin_ctzll(__ballot(r < upto));  // the first lane whose running sum passes r
  int hold = 0;
  unsigned long long before = upto - mine;
  if (lane == holder) {
    hold = c_lo;
    while (hold + 1 < c_hi && r >= before + csum[hold]) before += csum[hold++];
  }
  hold = __shfl(hold, holder, 64);
  before = __shfl(before, holder, 64);
  int pick = imax;
  bool found = false;
  for (int o = 0; o < per && !found; o += 256) {
    unsigned long long wv[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const long long i = (long long)hold * per + o + u * 64 + lane;
      wv[u] = i < vocab ? kept(z[i]) : 0ull;
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      if (found) continue;
      const unsigned long long group = wave_sum_u64(wv[u]);
      if (r < before + group) {  // the entry lies in this group of 64: running sums over its lanes, in index order
        unsigned long long run = wv[u];
#pragma unroll
        for (int d = 1; d < 64; d <<= 1) {
          const unsigned long long up = __shfl_up(run, d, 64);
          if (lane >= d) run += up;
        }
        const unsigned long long passed = __ballot(r < before + run);
        pick = hold * per + o + u * 64 + __builtin_ctzll(passed);
        found = true;
      } else {
        before += group;
      }
    }
  }
  if (lane == 0) out[row] = pick;
}

extern "C" int jllm_sample(const float* logits, int ld, int n_rows, int vocab, const float* temperature,
                           const int* top_k, const float* top_p, const float* min_p, const double* uniform, int* out,
                           hipStream_t stream) {
  if (n_rows <= 0) return 0;
  if (vocab <= 0 || ld < vocab) JLLM_FAIL("sample: vocab %d stride %d", vocab, ld);
  sample_kernel<<<n_rows, SAMPLE_THREADS, 0, stream>>>(logits, ld, vocab, temperature, top_k, top_p, min_p, uniform, out);
  JLLM_CHECK_LAUNCH("sample");
  return 0;
}

// ---------------------------------------------------------------------------------------------------------
__global__ __launch_bounds__(1024) void argmax_kernel(const float* __restrict__ logits, int ld, int vocab,
                                                      int* __restrict__ out) {
  __shared__ BlockScratch s;
  float best;
  int idx;
  block_argmax(logits + (size_t)blockIdx.x * ld, vocab, s, best, idx);
  if (threadIdx.x == 0) out[blockIdx.x] = idx;
}

// The same in two launches for long rows: a scan of one row by one workgroup is a chain of memory latencies (20 us
// for 151,936 logits). ARGMAX_CHUNKS workgroups per row each take a run of the row with all of their loads in flight
// and leave (value, index) candidates; one wave per row then picks among them, the lower index among equals.
#define ARGMAX_CHUNKS 32
#define ARGMAX_LONG_ROW 16384

__global__ __launch_bounds__(256) void argmax_chunks_kernel(const float* __restrict__ logits, int ld, int vocab, int per,
                                                            float* __restrict__ cand_v, int* __restrict__ cand_i) {
  __shared__ float fv[4];
  __shared__ int iv[4];
  const float* z = logits + (size_t)blockIdx.x * ld;
  const int lo = blockIdx.y * per, hi = min(vocab, lo + per);
  float best = -INFINITY;
  int idx = 0x7fffffff;
  for (int i0 = lo + threadIdx.x; i0 < hi; i0 += 256 * 8) {  // ascending i per lane keeps the lower index on ties
    float v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int i = i0 + u * 256;
      v[u] = i < hi ? z[i] : -INFINITY;
    }
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int i = i0 + u * 256;
      if (i < hi && (idx == 0x7fffffff || v[u] > best)) {
        best = v[u];
        idx = i;
      }
    }
  }
  for (int o = 32; o > 0; o >>= 1) {
    const float ov = __shfl_xor(best, o, 64);
    const int oi = __shfl_xor(idx, o, 64);
    if (oi != 0x7fffffff && (idx == 0x7fffffff || ov > best || (ov == best && oi < idx))) {
      best = ov;
      idx = oi;
    }
  }
  if ((threadIdx.x & 63) == 0) {
    fv[threadIdx.x >> 6] = best;
    iv[threadIdx.x >> 6] = idx;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < 4; ++w)
      if (iv[w] != 0x7fffffff && (idx == 0x7fffffff || fv[w] > best || (fv[w] == best && iv[w] < idx))) {
        best = fv[w];
        idx = iv[w];
      }
    cand_v[blockIdx.x * ARGMAX_CHUNKS + blockIdx.y] = best;
    cand_i[blockIdx.x * ARGMAX_CHUNKS + blockIdx.y] = idx;
  }
}

__global__ __launch_bounds__(64) void argmax_pick_kernel(const float* __restrict__ cand_v, const int* __restrict__ cand_i,
                                                         int* __restrict__ out) {
  const int lane = threadIdx.x;
  float best = lane < ARGMAX_CHUNKS ? cand_v[blockIdx.x * ARGMAX_CHUNKS + lane] : -INFINITY;
  int idx = lane < ARGMAX_CHUNKS ? cand_i[blockIdx.x * ARGMAX_CHUNKS + lane] : 0x7fffffff;
  for (int o = 32; o > 0; o >>= 1) {
    const float ov = __shfl_xor(best, o, 64);
    const int oi = __shfl_xor(idx, o, 64);
    if (oi != 0x7fffffff && (idx == 0x7fffffff || ov > best || (ov == best && oi < idx))) {
      best = ov;
      idx = oi;
    }
  }
  if (lane == 0) out[blockIdx.x] = idx == 0x7fffffff ? 0 : idx;
}

// `scratch`: n_rows * 64 words for the candidates of long rows, or null (then one workgroup scans each row)
extern "C" int jllm_argmax(const float* logits, int ld, int n_rows, int vocab, int* out, void* scratch, hipStream_t stream) {
  if (n_rows <= 0) return 0;
  if (vocab <= 0 || ld < vocab) JLLM_FAIL("argmax: vocab %d stride %d", vocab, ld);
  if (scratch && vocab >= ARGMAX_LONG_ROW && n_rows <= 65535) {
    float* cand_v = (float*)scratch;
    int* cand_i = (int*)scratch + (size_t)n_rows * ARGMAX_CHUNKS;
    const int per = (vocab + ARGMAX_CHUNKS - 1) / ARGMAX_CHUNKS;
    argmax_chunks_kernel<<<dim3(n_rows, ARGMAX_CHUNKS), 256, 0, stream>>>(logits, ld, vocab, per, cand_v, cand_i);
    JLLM_CHECK_LAUNCH("argmax_chunks");
    argmax_pick_kernel<<<n_rows, 64, 0, stream>>>(cand_v, cand_i, out);
    JLLM_CHECK_LAUNCH("argmax_pick");
    return 0;
  }
  argmax_kernel<<<n_rows, SAMPLE_THREADS, 0, stream>>>(logits, ld, vocab, out);
  JLLM_CHECK_LAUNCH("argmax");
  return 0;
}

// ---------------------------------------------------------------------------------------------------------
// Log-probabilities (engine/TokenLogprob.java:22-54): logprob(t) = z_t - (max + log(sum_j exp(z_j - max))) from
// the raw logits, the sum in double; and the `top` most likely tokens, most likely first, the lower index first
// among equal logits. One workgroup per row; each alternative is one more scan of the row for the largest entry
// that comes after the previous one in that order.
__device__ void block_argmax_after(const float* z, int vocab, BlockScratch& s, float pv, int pi, float& best_out,
                                   int& idx_out) {
  float best = -INFINITY;
  int idx = 0x7fffffff;
  for (int i = threadIdx.x; i < vocab; i += SAMPLE_THREADS) {
    const float v = z[i];
    const bool after = v < pv || (v == pv && i > pi);
    if (after && (idx == 0x7fffffff || v > best)) {
      best = v;
      idx = i;
    }
  }
  for (int o = 32; o > 0; o >>= 1) {
    const float ov = __shfl_xor(best, o, 64);
    const int oi = __shfl_xor(idx, o, 64);
    if (oi != 0x7fffffff && (idx == 0x7fffffff || ov > best || (ov == best && oi < idx))) {
      best = ov;
      idx = oi;
    }
  }
  __syncthreads();
  if ((threadIdx.x & 63) == 0) {
    s.fv[threadIdx.x >> 6] = best;
    s.iv[threadIdx.x >> 6] = idx;
  }
  __syncthreads();
  best = s.fv[0];
  idx = s.iv[0];
  for (int w = 1; w < SAMPLE_THREADS / 64; ++w) {
    const float ov = s.fv[w];
    const int oi = s.iv[w];
    if (oi != 0x7fffffff && (idx == 0x7fffffff || ov > best || (ov == best && oi < idx))) {
      best = ov;
      idx = oi;
    }
  }
  best_out = best;
  idx_out = idx;
  __syncthreads();
}

__global__ __launch_bounds__(SAMPLE_THREADS) void logprob_kernel(const float* __restrict__ logits, int ld, int vocab,
                                                                 const int* __restrict__ tokens, int top,
                                                                 float* __restrict__ out_lp, int* __restrict__ top_ids,
                                                                 float* __restrict__ top_lp) {
  __shared__ BlockScratch s;
  __shared__ double wsum[SAMPLE_THREADS / 64];
  const int row = blockIdx.x;
  const float* z = logits + (size_t)row * ld;
  float zmax;
  int imax;
  block_argmax(z, vocab, s, zmax, imax);
  double mine = 0.0;
  for (int i = threadIdx.x; i < vocab; i += SAMPLE_THREADS) mine += exp((double)z[i] - (double)zmax);
  for (int o = 32; o > 0; o >>= 1) mine += __shfl_xor(mine, o, 64);
  __syncthreads();
  if ((threadIdx.x & 63) == 0) wsum[threadIdx.x >> 6] = mine;
  __syncthreads();
  double total = 0.0;
  for (int w = 0; w < SAMPLE_THREADS / 64; ++w) total += wsum[w];
  const double lse = (double)zmax + log(total);
  if (threadIdx.x == 0) out_lp[row] = (float)((double)z[tokens[row]] - lse);
  float pv = zmax;
  int pi = imax;
  for (int n = 0; n < top; ++n) {
    if (threadIdx.x == 0) {
      top_ids[(size_t)row * top + n] = pi;
      top_lp[(size_t)row * top + n] = (float)((double)pv - lse);
    }
    if (n + 1 < top) block_argmax_after(z, vocab, s, pv, pi, pv, pi);
  }
}

extern "C" int jllm_token_logprobs(const float* logits, int ld, int n_rows, int vocab, const int* tokens, int top,
                                   float* out_lp, int* top_ids, float* top_lp, hipStream_t stream) {
  if (n_rows <= 0) return 0;
  if (vocab <= 0 || ld < vocab) JLLM_FAIL("logprobs: vocab %d stride %d", vocab, ld);
  if (top < 0 || top > vocab) JLLM_FAIL("logprobs: %d alternatives of a vocabulary of %d", top, vocab);
  if (top > 0 && (!top_ids || !top_lp)) JLLM_FAIL("logprobs: no room for the alternatives");
  logprob_kernel<<<n_rows, SAMPLE_THREADS, 0, stream>>>(logits, ld, vocab, tokens, top, out_lp, top_ids, top_lp);
  JLLM_CHECK_LAUNCH("logprobs");
  return 0;
}

// ---------------------------------------------------------------------------------------------------------
// Penalties and bias of one row (sampling/Sampler.java:434-456). `ids` lists each token seen in the prompt
// or the output once, `counts` how often it was generated: z = z > 0 ? z / rep : z * rep for every seen
// token, then z -= presence + frequency * count for generated ones; then the bias entries are added.
__global__ void adjust_logits_kernel(float* __restrict__ z, const int* __restrict__ ids, const int* __restrict__ counts,
                                     int n_seen, float rep, float presence, float frequency,
                                     const int* __restrict__ bias_ids, const float* __restrict__ bias_vals, int n_bias,
                                     int vocab) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n_seen) {
    const int t = ids[i];
    if (t >= 0 && t < vocab) {
      float v = z[t];
      if (rep != 1.0f) v = v > 0.f ? v / rep : v * rep;
      const int c = counts[i];
      if (c > 0) v -= presence + frequency * (float)c;
      z[t] = v;
    }
  }
}

__global__ void bias_logits_kernel(float* __restrict__ z, const int* __restrict__ bias_ids,
                                   const float* __restrict__ bias_vals, int n_bias, int vocab) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n_bias) {
    const int t = bias_ids[i];
    if (t >= 0 && t < vocab) z[t] += bias_vals[i];
  }
}

extern "C" int jllm_adjust_logits(float* row, int vocab, const int* ids, const int* counts, int n_seen, float rep,
                                  float presence, float frequency, const int* bias_ids, const float* bias_vals,
                                  int n_bias, hipStream_t stream) {
  if (n_seen > 0) {
    adjust_logits_kernel<<<(n_seen + 255) / 256, 256, 0, stream>>>(row, ids, counts, n_seen, rep, presence, frequency,
                                                                   nullptr, nullptr, 0, vocab);
    JLLM_CHECK_LAUNCH("adjust_logits");
  }
  if (n_bias > 0) {
    bias_logits_kernel<<<(n_bias + 255) / 256, 256, 0, stream>>>(row, bias_ids, bias_vals, n_bias, vocab);
    JLLM_CHECK_LAUNCH("bias_logits");
  }
  return 0;
}
