// The epilogue of the tiled products: what a wave does with its FM x FN accumulators of 32 x 32 once K is done.
//
// The weight fragment went in as the first MFMA operand, so an accumulator holds its tile transposed: element e of
// lane l is output column 8 * (e / 4) + (l / 32) * 4 + e % 4 of the 32-column block and output row l % 32 of the
// 32-row block; a lane owns four consecutive output columns of one row and stores them at once. Epilogues: store
// (fp32 or bf16), add into the fp32 residual, gated (accumulators [.][0] and [.][1] are gate and up of the same 32
// outputs: silu(gate) * up). With `split_z` the wave leaves an fp32 partial tile instead (K cut over workgroups;
// a reduction kernel applies bias and epilogue).
#pragma once
#include "common.h"
#include "mfma.h"

template <bool GATED, int FM, int FN, int TBM, int TBN>
__device__ __forceinline__ void tile_epilogue(floatx16 (&acc)[FM][FN], int lane, int wm, int wn, int m0, int n0,
                                              const void* __restrict__ bias, int bias_dtype, void* __restrict__ out,
                                              int out_dtype, int ldo, int M, int N, int epilogue, float* __restrict__ partial,
                                              int split_z, int n_splits) {
  // epilogue: accumulator element e of lane l is output column 8 * (e / 4) + (l / 32) * 4 + e % 4 of the 32-column
  // block and output row l % 32 of the 32-row block
  const int row_in = lane & 31;
  const int col_in = (lane >> 5) * 4;
  if (n_splits > 1) {  // partial sums [z][M][N]; the reduction kernel applies bias and epilogue
    float* pz = partial + (size_t)split_z * M * N;
#pragma unroll
    for (int mi = 0; mi < FM; ++mi) {
      const int m = m0 + (wm * FM + mi) * 32 + row_in;
      if (m >= M) continue;
#pragma unroll
      for (int ni = 0; ni < FN; ++ni)
#pragma unroll
        for (int e4 = 0; e4 < 4; ++e4) {
          const int n = n0 + (wn * FN + ni) * 32 + 8 * e4 + col_in;
          float* dst = pz + (size_t)m * N + n;
          if (n + 3 < N && (N & 3) == 0) {
            *(floatx4*)dst = floatx4{acc[mi][ni][4 * e4], acc[mi][ni][4 * e4 + 1], acc[mi][ni][4 * e4 + 2], acc[mi][ni][4 * e4 + 3]};
          } else {
#pragma unroll
            for (int c = 0; c < 4; ++c)
              if (n + c < N) dst[c] = acc[mi][ni][4 * e4 + c];
          }
        }
    }
    return;
  }
  const bool vec_ok = (ldo & 3) == 0 && (((uintptr_t)out) & 15) == 0;
  // Tiles that lie wholly inside the output (nearly all of a large product) take a path without per-element checks:
  // the kind of epilogue, the output type and the bias are decided once, outside the loops, and the gate's
  // 1 / (1 + exp(-x)) uses the hardware's exp2 and reciprocal (the result is rounded to bf16 or added in fp32 anyway).
  if (vec_ok && m0 + TBM <= M && n0 + (GATED ? TBN / 2 : TBN) <= N) {
    constexpr int NI = GATED ? 1 : FN;
    float bv[NI][4][4];
#pragma unroll
    for (int ni = 0; ni < NI; ++ni)
#pragma unroll
      for (int e4 = 0; e4 < 4; ++e4) {
        const int n = GATED ? n0 + wn * 32 + 8 * e4 + col_in : n0 + (wn * FN + ni) * 32 + 8 * e4 + col_in;
#pragma unroll
        for (int c = 0; c < 4; ++c)
          bv[ni][e4][c] = !bias ? 0.f : (bias_dtype == JLLM_BF16) ? ldf((const bf16_t*)bias, n + c) : ldf((const float*)bias, n + c);
      }
    const int kind = GATED ? 3 : epilogue == 1 ? 1 : out_dtype == JLLM_BF16 ? 2 : 0;  // store fp32, add, store bf16, gated
#pragma unroll
    for (int mi = 0; mi < FM; ++mi) {
      const size_t row = (size_t)(m0 + (wm * FM + mi) * 32 + row_in) * ldo;
#pragma unroll
      for (int ni = 0; ni < NI; ++ni)
#pragma unroll
        for (int e4 = 0; e4 < 4; ++e4) {
          const int n = GATED ? n0 + wn * 32 + 8 * e4 + col_in : n0 + (wn * FN + ni) * 32 + 8 * e4 + col_in;
          float v[4];
#pragma unroll
          for (int c = 0; c < 4; ++c) {
            float x = acc[mi][ni][4 * e4 + c] + bv[ni][e4][c];
            if (GATED) x = gate_fn<true>(x) * acc[mi][1][4 * e4 + c];
            v[c] = x;
          }
          const size_t o = row + n;
          if (kind == 1) {
            floatx4* dst = (floatx4*)((float*)out + o);
            const floatx4 cur = *dst;
            *dst = floatx4{cur[0] + v[0], cur[1] + v[1], cur[2] + v[2], cur[3] + v[3]};
          } else if (kind == 0 || (GATED && out_dtype != JLLM_BF16)) {
            *(floatx4*)((float*)out + o) = floatx4{v[0], v[1], v[2], v[3]};
          } else {
            *(u32x2*)((bf16_t*)out + o) = u32x2{pack_bf16(v[0], v[1]), pack_bf16(v[2], v[3])};
          }
        }
    }
    return;
  }
#pragma unroll
  for (int mi = 0; mi < FM; ++mi) {
    const int m = m0 + (wm * FM + mi) * 32 + row_in;
    if (m >= M) continue;
#pragma unroll
    for (int ni = 0; ni < (GATED ? 1 : FN); ++ni) {
#pragma unroll
      for (int e4 = 0; e4 < 4; ++e4) {
        const int n = GATED ? n0 + wn * 32 + 8 * e4 + col_in : n0 + (wn * FN + ni) * 32 + 8 * e4 + col_in;
        if (n >= N) continue;
        float v[4];
#pragma unroll
        for (int c = 0; c < 4; ++c) {
          float x = acc[mi][ni][4 * e4 + c];
          if (bias && n + c < N) x += (bias_dtype == JLLM_BF16) ? ldf((const bf16_t*)bias, n + c) : ldf((const float*)bias, n + c);
          if (GATED) x = gate_fn<true>(x) * acc[mi][1][4 * e4 + c];
          v[c] = x;
        }
        const size_t o = (size_t)m * ldo + n;
        if (n + 3 < N && vec_ok) {
          if (epilogue == 1) {
            floatx4* dst = (floatx4*)((float*)out + o);
            floatx4 cur = *dst;
            *dst = floatx4{cur[0] + v[0], cur[1] + v[1], cur[2] + v[2], cur[3] + v[3]};
          } else if (out_dtype == JLLM_BF16) {
            *(u32x2*)((bf16_t*)out + o) = u32x2{pack_bf16(v[0], v[1]), pack_bf16(v[2], v[3])};
          } else {
            *(floatx4*)((float*)out + o) = floatx4{v[0], v[1], v[2], v[3]};
          }
        } else {
#pragma unroll
          for (int c = 0; c < 4; ++c) {
            if (n + c >= N) continue;
            if (epilogue == 1)
              ((float*)out)[o + c] += v[c];
            else if (out_dtype == JLLM_BF16)
              stf((bf16_t*)out, o + c, v[c]);
            else
              stf((float*)out, o + c, v[c]);
          }
        }
      }
    }
  }
}
