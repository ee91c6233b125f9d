// Causal grouped-query attention over a paged cache for any head size, any head counts and any page
// size, fp32 or bf16 storage, all arithmetic in fp32. One workgroup of four 64-lane waves per (token row, query head).
//
// The row at absolute position p sees keys [first, p], first = max(0, p + 1 - window) with a window,
// else 0. Keys are walked in blocks of 64 aligned to absolute positions (block c covers 64c .. 64c+63); wave w takes
// the blocks with c % 4 == w in ascending order with a running maximum and sum of its own, and the four waves' results
// are merged in the order of the waves. So the result of a row depends only on its own position and keys: not on how
// the request was cut into steps, on the other rows of the batch, or on which pages hold the keys. Within a block a
// lane owns one key for the scores (the dot product in ascending order of the dims) and 64-strided dims for the
// weighted sum (the keys in ascending order). Up to four query heads of one kv head share a workgroup, and with it
// every key and value it reads; a head's arithmetic is the same whichever heads sit beside it.
//
// A position encoding may add a bias to the scores instead of (or beside) rotating q and k: with `slopes` (one fp32
// number per query head) the score of key j for the row at p gets slopes[h] * (j - p) added after the scaling.
//
// Cache layout of one layer: [page][kv_head][page_size][head_dim]; position j of request r lives in page
// block_table[r][j / page_size] at offset j % page_size. Table entries of positions before `first` are
// never read (they may have been given back).
#include <math.h>

#include "common.h"

#define ATT_MAX_ACC 8  // head_dim <= 512
#define ATT_WAVES 4

// four consecutive elements as floats; `wide`: they start on a 16-byte (fp32) or 8-byte (bf16) boundary
template <typename T>
__device__ __forceinline__ void load4f(const T* __restrict__ p, bool wide, float (&v)[4]);
template <>
__device__ __forceinline__ void load4f<float>(const float* __restrict__ p, bool wide, float (&v)[4]) {
  if (wide) {
    const float4 t = *(const float4*)p;
    v[0] = t.x, v[1] = t.y, v[2] = t.z, v[3] = t.w;
  } else {
    v[0] = p[0], v[1] = p[1], v[2] = p[2], v[3] = p[3];
  }
}
template <>
__device__ __forceinline__ void load4f<bf16_t>(const bf16_t* __restrict__ p, bool wide, float (&v)[4]) {
  if (wide) {
    const uint2 t = *(const uint2*)p;
    v[0] = __builtin_bit_cast(float, t.x << 16), v[1] = __builtin_bit_cast(float, t.x & 0xffff0000u);
    v[2] = __builtin_bit_cast(float, t.y << 16), v[3] = __builtin_bit_cast(float, t.y & 0xffff0000u);
  } else {
#pragma unroll
    for (int e = 0; e < 4; ++e) v[e] = ldf(p, e);
  }
}

// GC: query heads of one kv head that a workgroup takes together (they read the same keys and values); a workgroup
// whose share of the group has fewer does the last head again in the spare places and stores it once.
template <typename T, int GC>
__global__ __launch_bounds__(64 * ATT_WAVES) void paged_attention_generic_kernel(
    const T* __restrict__ q, int ldq, T* __restrict__ out, int ldo, const T* __restrict__ kcache,
    const T* __restrict__ vcache, const int* __restrict__ block_table, int max_blocks,
    const int* __restrict__ row_req, const int* __restrict__ positions, int H, int Hkv, int hd, int page_size,
    int window, float scale, const float* __restrict__ slopes, int wide) {
  extern __shared__ float smem[];
  float* qs = smem;            // GC x hd
  float* mg = smem + GC * hd;  // ATT_WAVES x GC x (2 + hd): every wave's maximum, sum and weighted sums per head
  const int t = blockIdx.x;
  const int G = H / Hkv;
  const int chunks = (G + GC - 1) / GC;
  const int kvh = blockIdx.y / chunks;
  const int h0 = kvh * G + (blockIdx.y % chunks) * GC;  // the first head of this workgroup
  const int gn = min(GC, kvh * G + G - h0);              // how many it has
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int pos = positions[t];
  const int* tbl = block_table + (size_t)row_req[t] * max_blocks;
  const int first = window > 0 ? max(0, pos + 1 - window) : 0;
  for (int i = threadIdx.x; i < GC * hd; i += 64 * ATT_WAVES) {
    const int g = min(i / hd, gn - 1);
    qs[i] = ldf(q + (size_t)t * ldq + (size_t)(h0 + g) * hd, i % hd);
  }
  __syncthreads();
  const int nacc = (hd + 63) >> 6;
  const int hd4 = hd & ~3;
  float acc[GC][ATT_MAX_ACC];
  float m[GC], l[GC];
#pragma unroll
  for (int g = 0; g < GC; ++g) {
    m[g] = -INFINITY, l[g] = 0.f;
#pragma unroll
    for (int a = 0; a < ATT_MAX_ACC; ++a) acc[g][a] = 0.f;
  }
  const int b_first = first >> 6;
  for (int blk = b_first + ((wave - b_first) & (ATT_WAVES - 1)); blk * 64 <= pos; blk += ATT_WAVES) {
    const int c0 = blk * 64;
    const int kj = c0 + lane;
    const bool valid = kj >= first && kj <= pos;
    float s[GC];
#pragma unroll
    for (int g = 0; g < GC; ++g) s[g] = -INFINITY;
    size_t row_at = 0;  // where this lane's key (and value) starts in the cache, in elements
    if (valid) {
      const int page = tbl[kj / page_size];
      row_at = (((size_t)page * Hkv + kvh) * page_size + kj % page_size) * hd;
      const T* kr = kcache + row_at;
      float d[GC];
#pragma unroll
      for (int g = 0; g < GC; ++g) d[g] = 0.f;
#pragma unroll 4
      for (int i = 0; i < hd4; i += 4) {
        float kv[4];
        load4f<T>(kr + i, wide != 0, kv);
#pragma unroll
        for (int g = 0; g < GC; ++g)
#pragma unroll
          for (int e = 0; e < 4; ++e) d[g] = fmaf(qs[g * hd + i + e], kv[e], d[g]);
      }
      for (int i = hd4; i < hd; ++i) {
        const float kv = ldf(kr, i);
#pragma unroll
        for (int g = 0; g < GC; ++g) d[g] = fmaf(qs[g * hd + i], kv, d[g]);
      }
#pragma unroll
      for (int g = 0; g < GC; ++g) {
        s[g] = d[g] * scale;
        if (slopes) s[g] += slopes[h0 + min(g, gn - 1)] * (float)(kj - pos);  // a position encoding that biases scores by distance
      }
    }
    float p[GC];
#pragma unroll
    for (int g = 0; g < GC; ++g) {
      const float m_new = fmaxf(m[g], wave_max(s[g]));
      p[g] = valid ? expf(s[g] - m_new) : 0.f;
      const float alpha = expf(m[g] - m_new);
      l[g] = l[g] * alpha + wave_sum(p[g]);
#pragma unroll
      for (int a = 0; a < ATT_MAX_ACC; ++a) acc[g][a] *= alpha;
      m[g] = m_new;
    }
    const int j0 = max(0, first - c0);
    const int j1 = min(63, pos - c0);
    // the block's values in ascending order of the keys; lane j knows where key j lies. Four keys' values are
    // requested before any is used (one at a time, a block was 64 memory latencies long); a key outside the row's
    // range has probability 0 and reads the nearest key inside it, so nothing that is not a value is ever multiplied
    for (int jb = 0; jb < 64; jb += 4) {
      if (jb + 3 < j0 || jb > j1) continue;
      float pj[4][GC], vv[4][ATT_MAX_ACC];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int j = jb + u;
        const int jj = min(max(j, j0), j1);
#pragma unroll
        for (int g = 0; g < GC; ++g) pj[u][g] = __shfl(p[g], j, 64);
        const unsigned lo = __shfl((unsigned)(row_at & 0xffffffffu), jj, 64), hi = __shfl((unsigned)(row_at >> 32), jj, 64);
        const T* vr = vcache + (((size_t)hi << 32) | lo);
#pragma unroll
        for (int a = 0; a < ATT_MAX_ACC; ++a) {
          const int d = lane + a * 64;
          vv[u][a] = (a < nacc && d < hd) ? ldf(vr, d) : 0.f;
        }
      }
#pragma unroll
      for (int u = 0; u < 4; ++u)
#pragma unroll
        for (int g = 0; g < GC; ++g)
#pragma unroll
          for (int a = 0; a < ATT_MAX_ACC; ++a)
            if (a < nacc) acc[g][a] = fmaf(pj[u][g], vv[u][a], acc[g][a]);
    }
  }
  // the waves' results, merged in the order of the waves
#pragma unroll
  for (int g = 0; g < GC; ++g) {
    float* mine = mg + (size_t)(wave * GC + g) * (2 + hd);
    if (lane == 0) {
      mine[0] = m[g];
      mine[1] = l[g];
    }
#pragma unroll
    for (int a = 0; a < ATT_MAX_ACC; ++a) {
      const int d = lane + a * 64;
      if (a < nacc && d < hd) mine[2 + d] = acc[g][a];
    }
  }
  __syncthreads();
  if (wave != 0) return;
#pragma unroll
  for (int g = 0; g < GC; ++g) {
    if (g >= gn) continue;
    float mm = m[g], ll = l[g];
    for (int w = 1; w < ATT_WAVES; ++w) {
      const float* theirs = mg + (size_t)(w * GC + g) * (2 + hd);
      const float om = theirs[0], ol = theirs[1];
      if (ol == 0.f) continue;  // that wave had no key
      const float m_new = fmaxf(mm, om);
      const float ca = expf(mm - m_new), cb = expf(om - m_new);
      ll = ll * ca + ol * cb;
#pragma unroll
      for (int a = 0; a < ATT_MAX_ACC; ++a) {
        const int d = lane + a * 64;
        if (a < nacc && d < hd) acc[g][a] = acc[g][a] * ca + theirs[2 + d] * cb;
      }
      mm = m_new;
    }
    const float inv = 1.0f / ll;
    T* o = out + (size_t)t * ldo + (size_t)(h0 + g) * hd;
#pragma unroll
    for (int a = 0; a < ATT_MAX_ACC; ++a) {
      const int d = lane + a * 64;
      if (a < nacc && d < hd) stf(o, d, acc[g][a] * inv);
    }
  }
}

extern "C" int jllm_paged_attention_generic(const void* q, int ldq, void* out, int ldo, int dtype, const void* kcache,
                                            const void* vcache, const int* block_table, int max_blocks,
                                            const int* row_req, const int* positions, int n_tokens, int H, int Hkv,
                                            int hd, int page_size, int window, float scale, const float* slopes,
                                            hipStream_t stream) {
  if (n_tokens <= 0) return 0;
  if (H <= 0 || Hkv <= 0 || H % Hkv != 0) JLLM_FAIL("attention: %d query heads over %d kv heads", H, Hkv);
  if (hd <= 0 || hd > 64 * ATT_MAX_ACC) JLLM_FAIL("attention: head_dim %d (this kernel takes 1..%d)", hd, 64 * ATT_MAX_ACC);
  if (page_size <= 0 || max_blocks <= 0) JLLM_FAIL("attention: page_size %d max_blocks %d", page_size, max_blocks);
  if (ldq < H * hd || ldo < H * hd) JLLM_FAIL("attention: row strides %d/%d < %d", ldq, ldo, H * hd);
  if (window < 0) JLLM_FAIL("attention: window %d", window);
  if (H > 65535) JLLM_FAIL("attention: too many heads");
  // up to four heads of a kv head per workgroup where the accumulators fit in registers (head sizes up to 256) and
  // the step still has two workgroups for every compute unit (a head's result is the same bits either way)
  const int G = H / Hkv;
  int cus = jllm_compute_units();
  if (cus <= 0) cus = 256;
  int gc = 1;
  if (hd <= 256) {
    if (G >= 3 && (long)n_tokens * Hkv * ((G + 3) / 4) >= 2L * cus)
      gc = 4;
    else if (G >= 2 && (long)n_tokens * Hkv * ((G + 1) / 2) >= 2L * cus)
      gc = 2;
  }
  dim3 grid(n_tokens, Hkv * ((G + gc - 1) / gc));
  const size_t smem = (size_t)(gc * hd + ATT_WAVES * gc * (2 + hd)) * sizeof(float);
  // a key's row can be read four elements at a time where every row starts on such a boundary
  const size_t esz = dtype == JLLM_F32 ? 4 : 2;
  const int wide = ((size_t)hd * esz) % (4 * esz) == 0 && ((uintptr_t)kcache % (4 * esz)) == 0;
#define ATT_LAUNCH(GC)                                                                                                \
  paged_attention_generic_kernel<T, GC><<<grid, 64 * ATT_WAVES, smem, stream>>>(                                      \
      (const T*)q, ldq, (T*)out, ldo, (const T*)kcache, (const T*)vcache, block_table, max_blocks, row_req, positions, H, Hkv, \
      hd, page_size, window, scale, slopes, wide)
  JLLM_DISPATCH_1(dtype, T, {
    if (gc == 4)
      ATT_LAUNCH(4);
    else if (gc == 2)
      ATT_LAUNCH(2);
    else
      ATT_LAUNCH(1);
  })
#undef ATT_LAUNCH
  JLLM_CHECK_LAUNCH("paged_attention_generic");
  return 0;
}
