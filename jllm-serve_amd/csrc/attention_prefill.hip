// Causal attention of prompt portions over a paged bf16 cache on the matrix cores (flash style: no score matrix
// in memory, running maximum and sum in fp32).
//
// Grid (tile, query head). A tile is up to 128 consecutive rows of one request (4 waves x 32 rows); the host lists
// the tiles as (request, first row, rows, position of the first row). Keys are walked in blocks of 64 aligned to
// absolute positions. Per block the workgroup stages K as it lies ([key][dim]) and V transposed ([dim][key]) in
// LDS; positions outside the tile's visible range are stored as zeros and their table entries are never read.
//
// Each wave computes the TRANSPOSED scores S^T[key][row] = K Q^T (v_mfma_f32_32x32x16_bf16, A = K from LDS,
// B = Q held in registers), so a lane owns one query row: the row maximum and sum are in-lane reductions plus
// one exchange between the two half-waves, and the rescale of the output is a per-lane scalar. The
// probabilities, rounded to bf16, are already laid out as the B operand of O^T[dim][row] += V^T P^T: the k slots
// of that product are assigned to keys in the order the score accumulators hold them, and the A operand (V^T
// from LDS) is read in the same order.
//
// Needs bf16, head_dim a multiple of 16 up to 128, or 192; the caller falls back to the general kernel otherwise.
#include <math.h>

#include "common.h"
#include "mfma.h"

#define PA_ROWS 128
#define PA_KEYS 64

template <int HD16>
__global__ __launch_bounds__(256) void prefill_attention_kernel(
    const bf16_t* __restrict__ q, int ldq, bf16_t* __restrict__ out, int ldo, const bf16_t* __restrict__ kc,
    const bf16_t* __restrict__ vc, const int* __restrict__ block_table, int max_blocks, const int* __restrict__ tiles,
    int H, int Hkv, int page_size, int window, float scale_log2e) {
  constexpr int HD = HD16 * 16;
  constexpr int DB = (HD + 31) / 32;
  constexpr int HDP = DB * 32;
  constexpr int KLD = HD + 8;
  constexpr int VLD = PA_KEYS + 8;
  __shared__ __align__(16) bf16_t Ks[PA_KEYS * KLD];
  __shared__ __align__(16) bf16_t Vt[HDP * VLD];
  const int* tile = tiles + (size_t)blockIdx.x * 4;
  const int req = tile[0], row0 = tile[1], nrows = tile[2], pos0 = tile[3];
  const int h = blockIdx.y;
  const int kvh = h / (H / Hkv);
  const int tid = threadIdx.x;
  const int wave = tid >> 6, lane = tid & 63;
  const int qi = lane & 31, half = lane >> 5;
  const int wq = wave * 32 + qi;
  const int pos_q = pos0 + min(wq, nrows - 1);
  const int first_q = window > 0 ? max(0, pos_q + 1 - window) : 0;
  const int* tbl = block_table + (size_t)req * max_blocks;
  const int k_lo = window > 0 ? max(0, pos0 + 1 - window) : 0;  // oldest key any row of the tile sees
  const int k_hi = pos0 + nrows - 1;
  const int wave_hi = pos0 + min(nrows - 1, wave * 32 + 31);  // newest key this wave needs
  const bool wave_on = wave * 32 < nrows;
  // Q as the B operand: lane holds Q[row][ks * 16 + half * 8 .. + 8]
  uint4 qf[HD16];
  {
    const bf16_t* qr = q + (size_t)(row0 + min(wq, nrows - 1)) * ldq + (size_t)h * HD + half * 8;
#pragma unroll
    for (int ks = 0; ks < HD16; ++ks) qf[ks] = *(const uint4*)(qr + ks * 16);
  }
  if (HD != HDP) {  // dims beyond head_dim of the transposed V stay zero
    for (int i = tid; i < (HDP - HD) * VLD; i += 256) Vt[HD * VLD + i].bits = 0;
  }
  floatx16 o[DB];
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int e = 0; e < 16; ++e) o[db][e] = 0.f;
  float m = -INFINITY, l = 0.f;
  for (int kt = (k_lo / PA_KEYS) * PA_KEYS; kt <= k_hi; kt += PA_KEYS) {
    __syncthreads();
    for (int c = tid; c < PA_KEYS * HD16 * 2; c += 256) {
      const int key = c / (HD16 * 2), pc = c % (HD16 * 2);
      const int kabs = kt + key;
      uint4 kv = uint4{0u, 0u, 0u, 0u}, vv = uint4{0u, 0u, 0u, 0u};
      if (kabs >= k_lo && kabs <= k_hi) {
        const int page = tbl[kabs / page_size];
        const size_t base = (((size_t)page * Hkv + kvh) * page_size + (kabs % page_size)) * HD + pc * 8;
        kv = *(const uint4*)(kc + base);
        vv = *(const uint4*)(vc + base);
      }
      *(uint4*)(Ks + (size_t)key * KLD + pc * 8) = kv;
      const uint32_t w[4] = {vv.x, vv.y, vv.z, vv.w};
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        Vt[(size_t)(pc * 8 + 2 * e) * VLD + key].bits = (uint16_t)(w[e] & 0xffffu);
        Vt[(size_t)(pc * 8 + 2 * e + 1) * VLD + key].bits = (uint16_t)(w[e] >> 16);
      }
    }
    __syncthreads();
    if (!wave_on || kt > wave_hi) continue;
    // transposed scores of 64 keys x 32 rows
    floatx16 s[2];
#pragma unroll
    for (int kb = 0; kb < 2; ++kb) {
#pragma unroll
      for (int e = 0; e < 16; ++e) s[kb][e] = 0.f;
      const bf16_t* kr = Ks + (size_t)(kb * 32 + qi) * KLD + half * 8;
#pragma unroll
      for (int ks = 0; ks < HD16; ++ks) s[kb] = mfma32(*(const uint4*)(kr + ks * 16), qf[ks], s[kb]);
    }
    float mx = -INFINITY;
#pragma unroll
    for (int kb = 0; kb < 2; ++kb)
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const int key = kt + kb * 32 + 8 * (e >> 2) + half * 4 + (e & 3);
        const float v = (key >= first_q && key <= pos_q) ? s[kb][e] * scale_log2e : -INFINITY;
        s[kb][e] = v;
        mx = fmaxf(mx, v);
      }
    mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
    const float m_new = fmaxf(m, mx);
    uint4 pb[2][2];
    if (m_new == -INFINITY) {  // this row sees none of the block's keys
#pragma unroll
      for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int st = 0; st < 2; ++st) pb[kb][st] = uint4{0u, 0u, 0u, 0u};
    } else {
      const float alpha = exp2f(m - m_new);
      float rs = 0.f;
#pragma unroll
      for (int kb = 0; kb < 2; ++kb) {
        float p[16];
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          p[e] = exp2f(s[kb][e] - m_new);
          rs += p[e];
        }
#pragma unroll
        for (int st = 0; st < 2; ++st) {
          uint32_t w[4];
#pragma unroll
          for (int j = 0; j < 4; ++j)
            w[j] = (uint32_t)f32_to_bf16(p[8 * st + 2 * j]).bits | ((uint32_t)f32_to_bf16(p[8 * st + 2 * j + 1]).bits << 16);
          pb[kb][st] = uint4{w[0], w[1], w[2], w[3]};
        }
      }
      rs += __shfl_xor(rs, 32, 64);
      l = l * alpha + rs;
      m = m_new;
#pragma unroll
      for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int e = 0; e < 16; ++e) o[db][e] *= alpha;
    }
    // O^T[dim][row] += V^T[dim][key] P^T[key][row]
#pragma unroll
    for (int db = 0; db < DB; ++db) {
      const bf16_t* vr = Vt + (size_t)(db * 32 + qi) * VLD + half * 4;
#pragma unroll
      for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int st = 0; st < 2; ++st) {
          const uint2 lo = *(const uint2*)(vr + kb * 32 + 16 * st);
          const uint2 hi = *(const uint2*)(vr + kb * 32 + 16 * st + 8);
          o[db] = mfma32(uint4{lo.x, lo.y, hi.x, hi.y}, pb[kb][st], o[db]);
        }
    }
  }
  if (!wave_on || wq >= nrows) return;
  const float inv = 1.0f / l;
  bf16_t* orow = out + (size_t)(row0 + wq) * ldo + (size_t)h * HD;
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int e4 = 0; e4 < 4; ++e4) {
      const int d = db * 32 + 8 * e4 + half * 4;
      if (d < HD) {
        const uint32_t w0 = (uint32_t)f32_to_bf16(o[db][4 * e4] * inv).bits | ((uint32_t)f32_to_bf16(o[db][4 * e4 + 1] * inv).bits << 16);
        const uint32_t w1 = (uint32_t)f32_to_bf16(o[db][4 * e4 + 2] * inv).bits | ((uint32_t)f32_to_bf16(o[db][4 * e4 + 3] * inv).bits << 16);
        *(uint2*)(orow + d) = uint2{w0, w1};
      }
    }
}

// tiles: int32 [n_tiles][4] = (request index, first row in the batch, rows (1..128), position of the first row)
// returns 0 when it ran, 1 when the shape is not one it takes, -1 on errors
extern "C" int jllm_prefill_attention_bf16(const void* q, int ldq, void* out, int ldo, const void* kcache,
                                           const void* vcache, const int* block_table, int max_blocks, const int* tiles,
                                           const int* positions, int n_tiles, int n_requests, int H, int Hkv, int hd,
                                           int page_size, int window, int max_context, float scale,
                                           hipStream_t stream) {
  (void)positions;
  (void)n_requests;
  (void)max_context;
  if (n_tiles <= 0) return 0;
  if (Hkv <= 0 || H % Hkv != 0) JLLM_FAIL("prefill attention: %d query heads over %d kv heads", H, Hkv);
  if ((hd & 15) || hd > 192 || hd < 16 || (ldq & 7) || (ldo & 3) || ((uintptr_t)q & 15) || ((uintptr_t)out & 7)) return 1;
  if (page_size <= 0 || H > 65535) return 1;
  dim3 grid(n_tiles, H);
  const float sl = scale * 1.4426950408889634f;
#define PA_CASE(N)                                                                                                     \
  case N:                                                                                                              \
    prefill_attention_kernel<N><<<grid, 256, 0, stream>>>((const bf16_t*)q, ldq, (bf16_t*)out, ldo,                    \
                                                          (const bf16_t*)kcache, (const bf16_t*)vcache, block_table,   \
                                                          max_blocks, tiles, H, Hkv, page_size, window, sl);           \
    break;
  switch (hd / 16) {
    PA_CASE(1) PA_CASE(2) PA_CASE(3) PA_CASE(4) PA_CASE(5) PA_CASE(6) PA_CASE(7) PA_CASE(8) PA_CASE(12)
    default: return 1;
  }
#undef PA_CASE
  JLLM_CHECK_LAUNCH("prefill_attention");
  return 0;
}
