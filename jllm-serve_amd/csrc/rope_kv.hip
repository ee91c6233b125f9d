// Per-head q/k RMSNorm, rotary position encoding and the write of k and v into cache pages, in one pass
// over the fused projection output qkv[t] = [q (H*hd) | k (Hkv*hd) | v (Hkv*hd)].
//
// q is normalised and rotated in place. k is normalised and rotated in fp32 and rounded once when it is
// stored in its page; v is copied. Rotation pairs (i, i + rot/2) for i < rot/2 ("half" pairing); the
// angles come from a host-made fp32 table cos/sin[position][rot/2]; dimensions >= rot stay as they are.
//
// Cache layout of one layer: [page][kv_head][page_size][head_dim]; `slots[t]` = page * page_size + offset
// of token t, or < 0 for "do not store".
#include "common.h"
#include "head_lanes.h"

template <typename T, typename TG>
__global__ __launch_bounds__(64) void qk_norm_rope_store_kernel(
    T* __restrict__ qkv, int ld, const int* __restrict__ positions, const int* __restrict__ slots,
    const float* __restrict__ cos_t, const float* __restrict__ sin_t, const TG* __restrict__ gq,
    const TG* __restrict__ gk, float eps, int H, int Hkv, int hd, int rot, int page_size, T* __restrict__ kcache,
    T* __restrict__ vcache, int write_kv) {
  extern __shared__ float vals[];  // hd
  const int t = blockIdx.x;
  const int h = blockIdx.y;  // 0..H-1 q heads, then Hkv k heads, then Hkv v heads
  const int lane = threadIdx.x;
  const bool is_q = h < H;
  const bool is_k = !is_q && h < H + Hkv;
  if (!is_q && !write_kv) return;
  T* src = qkv + (size_t)t * ld + (size_t)h * hd;
  const int slot = slots ? slots[t] : -1;
  if (!is_q && slot < 0) return;
  size_t dst = 0;
  if (!is_q) {
    const int kvh = is_k ? h - H : h - H - Hkv;
    const int page = slot / page_size;
    const int off = slot - page * page_size;
    dst = (((size_t)page * Hkv + kvh) * page_size + off) * hd;
  }
  if (!is_q && !is_k) {  // v: a copy
    for (int i = lane; i < hd; i += 64) vcache[dst + i] = src[i];
    return;
  }
  float ss = 0.f;
  for (int i = lane; i < hd; i += 64) {
    float v = ldf(src, i);
    vals[i] = v;
    ss += v * v;
  }
  const TG* g = is_q ? gq : gk;
  if (g) {
    ss = wave_sum(ss);
    const float s = norm_scale(ss, hd, eps);
    for (int i = lane; i < hd; i += 64) vals[i] = (vals[i] * s) * ldf(g, i);
  }
  __syncthreads();
  const int half = rot >> 1;
  T* o = is_q ? src : kcache + dst;
  if (cos_t) {
    const float* c = cos_t + (size_t)positions[t] * half;
    const float* s = sin_t + (size_t)positions[t] * half;
    for (int i = lane; i < half; i += 64) {
      const float a = vals[i], b = vals[i + half];
      const float cs = c[i], sn = s[i];
      stf(o, i, a * cs - b * sn);
      stf(o, i + half, b * cs + a * sn);
    }
    for (int i = rot + lane; i < hd; i += 64) stf(o, i, vals[i]);
  } else {
    for (int i = lane; i < hd; i += 64) stf(o, i, vals[i]);
  }
}

// The same for bf16 with head_dim % 8 == 0 and rotary width % 16 == 0 (what models have): a head lies over LPK
// lanes with 16 bytes each, a wave handles 64 / LPK heads of a token, a workgroup four times as many; every
// access is a 16-byte one.
template <int LPK>
__global__ __launch_bounds__(256) void qk_norm_rope_store_lanes_kernel(
    bf16_t* qkv, int ld, const int* __restrict__ positions, const int* __restrict__ slots,
    const float* __restrict__ cos_t, const float* __restrict__ sin_t, const void* __restrict__ gq,
    const void* __restrict__ gk, int gain_dtype, float eps, int H, int Hkv, int hd, int rot, int page_size,
    bf16_t* kcache, bf16_t* vcache, int write_kv) {
  constexpr int HPW = 64 / LPK;  // heads per wave
  const int t = blockIdx.x;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int sub = lane % LPK;
  const int h = (blockIdx.y * 4 + wave) * HPW + lane / LPK;  // 0..H-1 q heads, then Hkv k heads, then Hkv v heads
  const int d0 = sub * 8;
  const bool inside = h < H + 2 * Hkv;
  const bool active = inside && d0 < hd;
  const bool is_q = h < H;
  const bool is_k = !is_q && h < H + Hkv;
  const int pos = positions[t];
  const int slot = slots ? slots[t] : -1;
  const bool rotate = cos_t != nullptr;
  bf16_t* src = qkv + (size_t)t * ld + (size_t)(inside ? h : 0) * hd + d0;
  uint4 raw = uint4{0u, 0u, 0u, 0u};
  const bool wanted = active && (is_q || (write_kv && slot >= 0));
  if (wanted) raw = *(const uint4*)src;
  LaneAngles an;
  const int half = rot >> 1;
  an.low = rotate && d0 < half;
  an.high = rotate && d0 >= half && d0 < rot;
  an.src = lane + (an.low ? (half >> 3) : an.high ? -(half >> 3) : 0);
  float gn[8];
  const void* gain = is_q ? gq : gk;
  const bool normed = gain != nullptr && (is_q || is_k);
  if (wanted && (is_q || is_k)) {
    if (an.low || an.high) {
      const size_t at = (size_t)pos * half + (an.low ? d0 : d0 - half);
      load8(cos_t, JLLM_F32, at, an.c);
      load8(sin_t, JLLM_F32, at, an.s);
    }
    if (normed) load8(gain, gain_dtype, d0, gn);
  }
  size_t dst = 0;
  if (!is_q && inside && slot >= 0) {
    const int kvh = is_k ? h - H : h - H - Hkv;
    const int page = slot / page_size;
    dst = (((size_t)page * Hkv + kvh) * page_size + (slot - page * page_size)) * hd + d0;
  }
  float x[8];
  unpack8(raw, x);
  // every lane takes part in the exchanges; v heads and lanes outside pass through unchanged
  norm_rope8<LPK>(x, gn, normed, an, rotate && (is_q || is_k) && inside, eps, hd, wanted && (is_q || is_k));
  if (!wanted) return;
  const uint4 o = uint4{pack2(x[0], x[1]), pack2(x[2], x[3]), pack2(x[4], x[5]), pack2(x[6], x[7])};
  if (is_q)
    *(uint4*)src = o;
  else if (is_k)
    *(uint4*)(kcache + dst) = o;
  else
    *(uint4*)(vcache + dst) = raw;
}

template <int LPK>
static void launch_rope_lanes(int n_tokens, int heads, hipStream_t stream, void* qkv, int ld, const int* positions,
                              const int* slots, const float* cos_t, const float* sin_t, const void* gq, const void* gk,
                              int gain_dtype, float eps, int H, int Hkv, int hd, int rot, int page_size, void* kcache,
                              void* vcache, int write_kv) {
  const int per_block = 4 * (64 / LPK);
  dim3 grid(n_tokens, (heads + per_block - 1) / per_block);
  qk_norm_rope_store_lanes_kernel<LPK><<<grid, 256, 0, stream>>>((bf16_t*)qkv, ld, positions, slots, cos_t, sin_t, gq, gk,
                                                                 gain_dtype, eps, H, Hkv, hd, rot, page_size,
                                                                 (bf16_t*)kcache, (bf16_t*)vcache, write_kv);
}

extern "C" int jllm_qk_norm_rope_store(void* qkv, int dtype, int ld, const int* positions, const int* slots,
                                       const float* cos_t, const float* sin_t, const void* gq, const void* gk,
                                       int gain_dtype, float eps, int n_tokens, int H, int Hkv, int hd, int rot,
                                       int page_size, void* kcache, void* vcache, int write_kv, hipStream_t stream) {
  if (n_tokens <= 0) return 0;
  if (H <= 0 || Hkv <= 0 || hd <= 0 || hd > 8192) JLLM_FAIL("rope: heads %d/%d head_dim %d", H, Hkv, hd);
  if (cos_t && (rot < 2 || rot > hd || (rot & 1))) JLLM_FAIL("rope: rotary width %d of head_dim %d", rot, hd);
  if ((gq == nullptr) != (gk == nullptr)) JLLM_FAIL("rope: q and k gains come together");
  if (write_kv && (!kcache || !vcache || !slots || page_size <= 0)) JLLM_FAIL("rope: cache write without a cache");
  if (ld < (H + 2 * Hkv) * hd) JLLM_FAIL("rope: row stride %d < %d", ld, (H + 2 * Hkv) * hd);
  if (H + 2 * Hkv > 65535) JLLM_FAIL("rope: too many heads");
  if (dtype == JLLM_BF16 && (hd & 7) == 0 && hd <= 256 && (!cos_t || (rot & 15) == 0) && (ld & 7) == 0 &&
      ((uintptr_t)qkv & 15) == 0 && ((uintptr_t)gq & 15) == 0 && ((uintptr_t)gk & 15) == 0 &&
      ((uintptr_t)kcache & 15) == 0 && ((uintptr_t)vcache & 15) == 0) {
    const int heads = write_kv ? H + 2 * Hkv : H;
    int lpk = 2;
    while (lpk * 8 < hd) lpk <<= 1;
#define ROPE_LANES(L)                                                                                                \
  launch_rope_lanes<L>(n_tokens, heads, stream, qkv, ld, positions, slots, cos_t, sin_t, gq, gk, gain_dtype, eps, H, \
                       Hkv, hd, rot, page_size, kcache, vcache, write_kv)
    switch (lpk) {
      case 2: ROPE_LANES(2); break;
      case 4: ROPE_LANES(4); break;
      case 8: ROPE_LANES(8); break;
      case 16: ROPE_LANES(16); break;
      default: ROPE_LANES(32); break;
    }
#undef ROPE_LANES
    JLLM_CHECK_LAUNCH("qk_norm_rope_store");
    return 0;
  }
  dim3 grid(n_tokens, H + 2 * Hkv);
  const size_t smem = (size_t)hd * sizeof(float);
  JLLM_DISPATCH_1(dtype, T, {
    JLLM_DISPATCH_1(gain_dtype, TG, {
      qk_norm_rope_store_kernel<T, TG><<<grid, 64, smem, stream>>>((T*)qkv, ld, positions, slots, cos_t, sin_t,
                                                                   (const TG*)gq, (const TG*)gk, eps, H, Hkv, hd, rot,
                                                                   page_size, (T*)kcache, (T*)vcache, write_kv);
    })
  })
  JLLM_CHECK_LAUNCH("qk_norm_rope_store");
  return 0;
}

// ---------------------------------------------------------------------------------------------------------
// Copies the first `rows` positions of page `src` to page `dst` in every layer run of a group (what a
// copy-on-write of a partly filled page needs; the reference's KvStorage.copy, kv/KvStorage.java:43).
// storage: [runs][pages][outer][page_size][inner] of any element type, `inner_bytes` bytes per (outer, position);
// grid (runs * outer, rows). Moves 4-byte words where everything is a multiple of four, else bytes.
template <typename W>
__global__ void copy_page_rows_kernel(W* __restrict__ storage, size_t run_stride, size_t page_stride, int outer,
                                      int page_size, int inner, int src, int dst) {
  const int run = blockIdx.x / outer;
  const int o = blockIdx.x % outer;
  const int row = blockIdx.y;
  const size_t off = (size_t)run * run_stride + ((size_t)o * page_size + row) * inner;
  const W* s = storage + off + (size_t)src * page_stride;
  W* d = storage + off + (size_t)dst * page_stride;
  for (int i = threadIdx.x; i < inner; i += blockDim.x) d[i] = s[i];
}

extern "C" int jllm_copy_page_rows(void* storage, int runs, int pages, int outer, int page_size, long long inner_bytes,
                                   int src, int dst, int rows, hipStream_t stream) {
  if (rows <= 0 || src == dst) return 0;
  if (src < 0 || dst < 0 || src >= pages || dst >= pages) JLLM_FAIL("copy_page: pages %d -> %d of %d", src, dst, pages);
  if (rows > page_size) JLLM_FAIL("copy_page: %d rows of a page of %d", rows, page_size);
  if (runs <= 0 || outer <= 0 || inner_bytes <= 0 || inner_bytes > 2147483647ll) JLLM_FAIL("copy_page: %d runs, %d x %lld bytes", runs, outer, inner_bytes);
  dim3 grid((unsigned)runs * (unsigned)outer, rows);
  if ((long long)runs * outer > 2147483647ll / 2 || grid.y > 65535) JLLM_FAIL("copy_page: grid too large");
  if ((inner_bytes & 3) == 0 && ((uintptr_t)storage & 3) == 0) {
    const int inner = (int)(inner_bytes / 4);
    const size_t page_stride = (size_t)outer * page_size * inner;
    copy_page_rows_kernel<uint32_t><<<grid, 64, 0, stream>>>((uint32_t*)storage, (size_t)pages * page_stride, page_stride, outer,
                                                             page_size, inner, src, dst);
  } else {
    const int inner = (int)inner_bytes;
    const size_t page_stride = (size_t)outer * page_size * inner;
    copy_page_rows_kernel<uint8_t><<<grid, 64, 0, stream>>>((uint8_t*)storage, (size_t)pages * page_stride, page_stride, outer,
                                                            page_size, inner, src, dst);
  }
  JLLM_CHECK_LAUNCH("copy_page_rows");
  return 0;
}
