// Causal grouped-query attention over a paged cache for any head size, any head counts and any page
// size, fp32 or bf16 storage, all arithmetic in fp32. One 64-lane wave per (token row, query head).
//
// The row at absolute position p sees keys [first, p], first = max(0, p + 1 - window) with a window,
// else 0. Keys are walked in blocks of 64 aligned to absolute positions (block c covers 64c .. 64c+63)
// with a running maximum and sum, so the result of a row depends only on its own position and keys: not
// on how the request was cut into steps, on the other rows of the batch, or on which pages hold the keys.
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

template <typename T>
__global__ __launch_bounds__(64) void paged_attention_generic_kernel(
    const T* __restrict__ q, int ldq, T* __restrict__ out, int ldo, const T* __restrict__ kcache,
    const T* __restrict__ vcache, const int* __restrict__ block_table, int max_blocks,
    const int* __restrict__ row_req, const int* __restrict__ positions, int H, int Hkv, int hd, int page_size,
    int window, float scale, const float* __restrict__ slopes) {
  extern __shared__ float smem[];
  float* qs = smem;       // hd
  float* ps = smem + hd;  // 64
  const int t = blockIdx.x;
  const int h = blockIdx.y;
  const int lane = threadIdx.x;
  const int pos = positions[t];
  const int* tbl = block_table + (size_t)row_req[t] * max_blocks;
  const int first = window > 0 ? max(0, pos + 1 - window) : 0;
  const int kvh = h / (H / Hkv);
  const T* qr = q + (size_t)t * ldq + (size_t)h * hd;
  for (int i = lane; i < hd; i += 64) qs[i] = ldf(qr, i);
  __syncthreads();
  const int nacc = (hd + 63) >> 6;
  float acc[ATT_MAX_ACC];
#pragma unroll
  for (int a = 0; a < ATT_MAX_ACC; ++a) acc[a] = 0.f;
  float m = -INFINITY, l = 0.f;
  for (int c0 = (first >> 6) << 6; c0 <= pos; c0 += 64) {
    const int kj = c0 + lane;
    const bool valid = kj >= first && kj <= pos;
    float s = -INFINITY;
    if (valid) {
      const int page = tbl[kj / page_size];
      const int off = kj % page_size;
      const T* kr = kcache + (((size_t)page * Hkv + kvh) * page_size + off) * hd;
      float d = 0.f;
      for (int i = 0; i < hd; ++i) d = fmaf(qs[i], ldf(kr, i), d);
      s = d * scale;
      if (slopes) s += slopes[h] * (float)(kj - pos);  // a position encoding that biases scores by distance
    }
    const float m_new = fmaxf(m, wave_max(s));
    const float p = valid ? expf(s - m_new) : 0.f;
    const float alpha = expf(m - m_new);
    l = l * alpha + wave_sum(p);
    ps[lane] = p;
    __syncthreads();
#pragma unroll
    for (int a = 0; a < ATT_MAX_ACC; ++a) acc[a] *= alpha;
    const int j0 = max(0, first - c0);
    const int j1 = min(63, pos - c0);
    for (int j = j0; j <= j1; ++j) {
      const float pj = ps[j];
      const int kk = c0 + j;
      const int page = tbl[kk / page_size];
      const int off = kk % page_size;
      const T* vr = vcache + (((size_t)page * Hkv + kvh) * page_size + off) * hd;
#pragma unroll
      for (int a = 0; a < ATT_MAX_ACC; ++a) {
        const int d = lane + a * 64;
        if (a < nacc && d < hd) acc[a] = fmaf(pj, ldf(vr, d), acc[a]);
      }
    }
    __syncthreads();
    m = m_new;
  }
  const float inv = 1.0f / l;
  T* o = out + (size_t)t * ldo + (size_t)h * hd;
#pragma unroll
  for (int a = 0; a < ATT_MAX_ACC; ++a) {
    const int d = lane + a * 64;
    if (a < nacc && d < hd) stf(o, d, acc[a] * inv);
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
  dim3 grid(n_tokens, H);
  const size_t smem = (size_t)(hd + 64) * sizeof(float);
  JLLM_DISPATCH_1(dtype, T, {
    paged_attention_generic_kernel<T><<<grid, 64, smem, stream>>>((const T*)q, ldq, (T*)out, ldo, (const T*)kcache,
                                                                  (const T*)vcache, block_table, max_blocks, row_req,
                                                                  positions, H, Hkv, hd, page_size, window, scale, slopes);
  })
  JLLM_CHECK_LAUNCH("paged_attention_generic");
  return 0;
}
