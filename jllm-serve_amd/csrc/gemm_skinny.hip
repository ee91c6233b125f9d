// out[M,N] = A[M,K] * W[N,K]^T for few rows (decode steps): bf16 operands, fp32 accumulation on the matrix
// cores, bound by streaming W from HBM once.
//
// One workgroup of 8 (or 4) waves owns 16 weight rows (16 outputs per activation row). The K dimension is cut in
// blocks of 128; wave w takes blocks w, w+8, ...: per block each lane issues 4 loads of 16 bytes of its weight
// row (lane l, load j: row l%16, k = block*128 + j*32 + (l/16)*8 .. +8), so every load instruction covers whole
// 64-byte pieces of 16 rows (no sector is fetched for a quarter of its bytes) and a block is 16 rows x 256
// contiguous bytes; each load feeds one MFMA (16x16x32) per 16 activation rows. The two operands use the same k assignment, which
// is all a dot product needs. The 8 partial tiles are summed through LDS in wave order, so a result does not
// depend on M or on the other rows. Epilogues: store, add into the fp32 residual, gated (two weights).
//
// An RMSNorm between two such products costs no launch of its own. The product that adds into the residual
// ("emit") also leaves, for the norm that follows, the new residual values times that norm's gain as bf16
// [M, N] and the sum of their squares over its 16 columns as partial[m][block]. The product that consumes the
// norm ("normed") takes those bf16 rows as its input and multiplies its sums by rsqrt(sum of the partials / K +
// eps) at the end: sum_k W[n,k] (x[k] g[k]) s = the product over the normalised row. The partials are summed in
// an order that depends on nothing but their count.
//
// Needs K % 128 == 0, N % 16 == 0, M <= 64, 16-byte aligned rows; the caller falls back otherwise.
#include "common.h"
#include "mfma.h"


// what the two norm-carrying forms need beyond the plain product
struct SkinnyNorm {
  bf16_t* emit_rows;          // emit: [M, N] bf16, (residual after the add) * emit_gain
  const void* emit_gain;      // [N]
  int emit_gain_dtype;
  float* emit_partial;        // [M][N / 16]
  const float* norm_partial;  // normed: [M][norm_parts] sums of squares of the input rows
  int norm_parts;
  float norm_eps;
};

// sum over the 16 lanes of a row of lanes (the 16 columns of a tile), left in all of them
__device__ __forceinline__ float row16_sum(float d) {
  d += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, d), 0xB1, 0xF, 0xF, true));
  d += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, d), 0x4E, 0xF, 0xF, true));
  d += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, d), 0x141, 0xF, 0xF, true));
  d += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, d), 0x140, 0xF, 0xF, true));
  return d;
}

// TWO: the workgroup owns 16 + rows2 weight rows (rows2 = 1 .. 16), the second tile in the place the up weight
// has with the gated epilogue: the activations are read once for both, and N / 24 (or N / 20, N / 28) workgroups may
// fill the compute units where N / 16 leaves some of them with one workgroup more. Store and accumulate epilogues,
// the norm forms included: the squares of the second tile's columns go into the workgroup's one partial sum, and the
// places of the [M][N / 16] partial sums that no workgroup owns are set to zero.
template <int MT, bool GATED, int SK_WAVES, bool TWO = false>
__global__ __launch_bounds__(SK_WAVES * 64) void gemm_skinny_kernel(
    const bf16_t* __restrict__ A, int lda, const bf16_t* __restrict__ W, const bf16_t* __restrict__ W2,
    const void* __restrict__ bias, int bias_dtype, void* __restrict__ out, int out_dtype, int ldo, int M, int N,
    int K, int epilogue, SkinnyNorm nm, int rows2) {
  static_assert(!(GATED && TWO) && (!TWO || MT == 1), "a second tile of weight rows: one weight, one tile of rows");
  constexpr bool DUAL = GATED || TWO;  // a second set of weight registers and sums
  __shared__ float red[SK_WAVES - 1][MT][64][4];
  __shared__ float ssq[SK_WAVES][MT][16];  // normed: each wave's share of the rows' sums of squares
  const int wave = threadIdx.x >> 6;
  const int lane = threadIdx.x & 63;
  const int col = lane & 15;
  const int g = lane >> 4;
  const int n0 = blockIdx.x * (TWO ? 16 + rows2 : 16);
  const int nblk = K >> 7;
  const int rot = (int)((blockIdx.x * 7u) % (unsigned)nblk);
  const bf16_t* wrow = W + (size_t)(n0 + col) * K + g * 8;
  const bf16_t* urow = GATED ? W2 + (size_t)(n0 + col) * K + g * 8
                       : TWO ? W + (size_t)(n0 + 16 + min(col, rows2 - 1)) * K + g * 8 : nullptr;
  const bf16_t* arow[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) arow[mt] = A + (size_t)min(mt * 16 + col, M - 1) * lda + g * 8;
  floatx4 acc[MT];
  floatx4 acc2[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    acc[mt] = floatx4{0.f, 0.f, 0.f, 0.f};
    acc2[mt] = floatx4{0.f, 0.f, 0.f, 0.f};
  }
  // wave 0 writes the outputs: what it adds into (the residual, the bias) is requested now, long before it is needed
  float prev[MT][4];
  float rscale[MT][4];  // normed: rsqrt(mean of squares + eps) of the rows this lane writes
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int i = 0; i < 4; ++i) rscale[mt][i] = 1.0f;
  float b = 0.f, eg = 0.f, b2 = 0.f, eg2 = 0.f;
  float prev2[4] = {0.f, 0.f, 0.f, 0.f};  // the second tile's share of the residual
  if (wave == 0) {
    const int n = n0 + col;
    if (bias) b = (bias_dtype == JLLM_BF16) ? ldf((const bf16_t*)bias, n) : ldf((const float*)bias, n);
    if (TWO) {
      const int n2 = n0 + 16 + min(col, rows2 - 1);
      if (bias) b2 = (bias_dtype == JLLM_BF16) ? ldf((const bf16_t*)bias, n2) : ldf((const float*)bias, n2);
      if (nm.emit_rows) eg2 = (nm.emit_gain_dtype == JLLM_BF16) ? ldf((const bf16_t*)nm.emit_gain, n2) : ldf((const float*)nm.emit_gain, n2);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int m = g * 4 + i;
        prev2[i] = (epilogue == 1 && m < M) ? ((const float*)out)[(size_t)m * ldo + n2] : 0.f;
      }
    }
    if (nm.emit_rows) eg = (nm.emit_gain_dtype == JLLM_BF16) ? ldf((const bf16_t*)nm.emit_gain, n) : ldf((const float*)nm.emit_gain, n);
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int m = mt * 16 + g * 4 + i;
        prev[mt][i] = (epilogue == 1 && m < M) ? ((const float*)out)[(size_t)m * ldo + n] : 0.f;
      }
  }
  // UB K blocks per turn. What bounds this kernel is how many weight bytes are in flight, so the loads of a turn are
  // asked for before the turn before it is multiplied. Loads come back in the order they were asked for, and a wait
  // can only name how many of the latest may still be out: the loads of the next turn therefore stand in straight
  // code (a branch around them makes the compiler wait for all of them), and the registers of two turns take turns
  // instead of being copied (a copy waits for its load).
  constexpr int UB = DUAL ? 1 : 2;
  constexpr int STEP = UB * SK_WAVES;
  constexpr bool PINGPONG = MT == 1 && !GATED;
  auto block_of = [&](int blk, int b) {
    // past the end: a harmless reload of the last block. Workgroups walk K from different starting blocks, so that
    // at any moment they ask the L2 for different parts of the (shared) activations
    int bb = min(blk + b * SK_WAVES, nblk - 1) + rot;
    return bb >= nblk ? bb - nblk : bb;
  };
  // the ping-pong form: weights and activations of a turn together
  struct Turn {
    u32x4 w[UB][4], a[UB][4], u[TWO ? UB : 1][4];  // u: the second tile's weights
  };
  auto load = [&](Turn& t, int blk) {
#pragma unroll
    for (int b = 0; b < UB; ++b) {
      const size_t k = (size_t)block_of(blk, b) * 128;
#pragma unroll
      for (int j = 0; j < 4; ++j) t.a[b][j] = *(const u32x4*)(arow[0] + k + j * 32);  // rows beyond M: row M - 1 again
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        t.w[b][j] = *(const u32x4*)(wrow + k + j * 32);
        if (TWO) t.u[b][j] = *(const u32x4*)(urow + k + j * 32);
      }
    }
  };
  // the other form: the weights a turn ahead, copied into place after the products
  u32x4 wv[UB][4], uv[UB][4];
  auto fetch = [&](int blk, u32x4 (*w)[4], u32x4 (*u)[4]) {
#pragma unroll
    for (int b = 0; b < UB; ++b) {
      const size_t k = (size_t)block_of(blk, b) * 128;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        w[b][j] = *(const u32x4*)(wrow + k + j * 32);
        if (DUAL) u[b][j] = *(const u32x4*)(urow + k + j * 32);
      }
    }
  };
  Turn t0, t1;
  if (PINGPONG)
    load(t0, wave);  // a wave beyond the last block: a harmless load, no products
  else if (wave < nblk)
    fetch(wave, wv, uv);
  if (nm.norm_partial) {
    // normed: the sums of squares of the input rows, while the first weights are on their way. Every wave takes a
    // share: lane `col` of wave w the four partials 4 (16 w + col) .., then those 64 SK_WAVES further on; the
    // shares meet in LDS below, in wave order
    const int p4n = nm.norm_parts >> 2;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int i = 0; i < 4; ++i) rscale[mt][i] = 0.f;
    for (int p4 = wave * 16 + col; p4 < p4n; p4 += SK_WAVES * 16) {
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int m = mt * 16 + g * 4 + i;
          if (m < M) {
            const floatx4 v = ((const floatx4*)(nm.norm_partial + (size_t)m * nm.norm_parts))[p4];
            rscale[mt][i] += (v[0] + v[1]) + (v[2] + v[3]);
          }
        }
    }
  }
  const int turns = wave < nblk ? (nblk - wave + STEP - 1) / STEP : 0;
  if constexpr (PINGPONG) {
    // every turn but the last has all of its blocks
    auto products = [&](const Turn& t, int blk, bool whole) {
#pragma unroll
      for (int b = 0; b < UB; ++b) {
        if (whole || blk + b * SK_WAVES < nblk) {
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            acc[0] = mfma16(t.a[b][j], t.w[b][j], acc[0]);
            if (TWO) acc2[0] = mfma16(t.a[b][j], t.u[b][j], acc2[0]);
          }
        }
      }
    };
    int i = 0, blk = wave;
    for (; i + 2 < turns; i += 2, blk += 2 * STEP) {
      load(t1, blk + STEP);
      products(t0, blk, true);
      load(t0, blk + 2 * STEP);
      products(t1, blk + STEP, true);
    }
    if (turns - i == 2) {
      load(t1, blk + STEP);
      products(t0, blk, true);
      products(t1, blk + STEP, false);
    } else if (turns - i == 1) {
      products(t0, blk, false);
    }
  } else {
    // several tiles of rows, or two weights: too many registers for two turns of activations, and more activation
    // loads in flight only crowd out weight loads. The weights a turn ahead, the activations (L2) in their own turn
    for (int blk = wave; blk < nblk; blk += STEP) {
      u32x4 wn[UB][4], un[UB][4];
      if (blk + STEP < nblk) fetch(blk + STEP, wn, un);
#pragma unroll
      for (int b = 0; b < UB; ++b) {
        if (blk + b * SK_WAVES < nblk) {
          const size_t k = (size_t)block_of(blk, b) * 128;
#pragma unroll
          for (int mt = 0; mt < MT; ++mt) {
            u32x4 av[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
              if (MT == 1)  // rows beyond M read row M - 1 again
                av[j] = *(const u32x4*)(arow[mt] + k + j * 32);
              else  // lanes of row tiles beyond M load nothing: their operand rows are zeros
                av[j] = mt * 16 + col < M ? *(const u32x4*)(arow[mt] + k + j * 32) : u32x4{0u, 0u, 0u, 0u};
            }
#pragma unroll
            for (int j = 0; j < 4; ++j) {
              acc[mt] = mfma16(av[j], wv[b][j], acc[mt]);
              if (DUAL) acc2[mt] = mfma16(av[j], uv[b][j], acc2[mt]);
            }
          }
        }
      }
#pragma unroll
      for (int b = 0; b < UB; ++b)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          wv[b][j] = wn[b][j];
          if (DUAL) uv[b][j] = un[b][j];
        }
    }
  }
  if (nm.norm_partial) {
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float t = row16_sum(rscale[mt][i]);
        if (col == 0) ssq[wave][mt][g * 4 + i] = t;
      }
  }
  // sum the 8 partial tiles in wave order (gate first, then up, or the second tile, through the same buffer)
  for (int pass = 0; pass < (DUAL ? 2 : 1); ++pass) {
    if (pass == 1) __syncthreads();
    if (wave > 0) {
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int i = 0; i < 4; ++i) red[wave - 1][mt][lane][i] = pass == 0 ? acc[mt][i] : acc2[mt][i];
    }
    __syncthreads();
    if (wave == 0) {
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          float s = pass == 0 ? acc[mt][i] : acc2[mt][i];
#pragma unroll
          for (int w = 0; w < SK_WAVES - 1; ++w) s += red[w][mt][lane][i];
          if (pass == 0)
            acc[mt][i] = s;
          else
            acc2[mt][i] = s;
        }
    }
  }
  if (wave != 0) return;
  if (nm.norm_partial) {
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        float t = 0.f;
#pragma unroll
        for (int w = 0; w < SK_WAVES; ++w) t += ssq[w][mt][g * 4 + i];
        rscale[mt][i] = 1.0f / sqrtf(t / (float)K + nm.norm_eps);
      }
  }
  const int n = n0 + col;
  float sq2[4] = {0.f, 0.f, 0.f, 0.f};  // the squares of the second tile's columns, per row of this lane
  if (TWO) {  // the second tile: columns n0 + 16 .. n0 + 16 + rows2 - 1
    const bool mine = col < rows2;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int m = g * 4 + i;
      const float v = acc2[0][i] * rscale[0][i] + b2;
      const float now = prev2[i] + v;
      if (nm.emit_rows) sq2[i] = row16_sum(mine && m < M ? now * now : 0.f);
      if (m >= M || !mine) continue;
      const size_t o = (size_t)m * ldo + n + 16;
      if (nm.emit_rows) nm.emit_rows[(size_t)m * N + n + 16] = f32_to_bf16(now * eg2);
      if (epilogue == 1)
        ((float*)out)[o] = now;
      else if (out_dtype == JLLM_BF16)
        stf((bf16_t*)out, o, v);
      else
        stf((float*)out, o, v);
    }
    if (nm.emit_rows && col == 0) {  // the partial sums beyond the workgroups' own: zeros
      const int spare = (N >> 4) - (int)gridDim.x;
      if ((int)blockIdx.x < spare)
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (g * 4 + i < M) nm.emit_partial[(size_t)(g * 4 + i) * (N >> 4) + gridDim.x + blockIdx.x] = 0.f;
    }
  }
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int m = mt * 16 + g * 4 + i;
      float v = acc[mt][i] * rscale[mt][i] + b;
      if (GATED) v = gate_fn<false>(v) * (acc2[mt][i] * rscale[mt][i]);
      const float now = prev[mt][i] + v;
      if (nm.emit_rows) {  // every lane of the row takes part in the sum, rows beyond M with zeros
        const float sq = row16_sum(m < M ? now * now : 0.f) + (TWO ? sq2[i] : 0.f);
        if (m < M) {
          nm.emit_rows[(size_t)m * N + n] = f32_to_bf16(now * eg);
          if (col == 0) nm.emit_partial[(size_t)m * (N >> 4) + blockIdx.x] = sq;
        }
      }
      if (m >= M) continue;
      const size_t o = (size_t)m * ldo + n;
      if (epilogue == 1)
        ((float*)out)[o] = now;
      else if (out_dtype == JLLM_BF16)
        stf((bf16_t*)out, o, v);
      else
        stf((float*)out, o, v);
    }
}

template <int MT, int WAVES>
static void launch_skinny(dim3 grid, hipStream_t stream, const void* A, int lda, const void* W, const void* W2,
                          const void* bias, int bias_dtype, void* out, int out_dtype, int ldo, int M, int N, int K,
                          int epilogue, const SkinnyNorm& nm) {
  if (W2)
    gemm_skinny_kernel<MT, true, WAVES><<<grid, WAVES * 64, 0, stream>>>((const bf16_t*)A, lda, (const bf16_t*)W,
                                                                         (const bf16_t*)W2, bias, bias_dtype, out,
                                                                         out_dtype, ldo, M, N, K, epilogue, nm, 0);
  else
    gemm_skinny_kernel<MT, false, WAVES><<<grid, WAVES * 64, 0, stream>>>((const bf16_t*)A, lda, (const bf16_t*)W,
                                                                          nullptr, bias, bias_dtype, out, out_dtype,
                                                                          ldo, M, N, K, epilogue, nm, 0);
}

template <int WAVES>
static void launch_skinny_mt(int mt, dim3 grid, hipStream_t stream, const void* A, int lda, const void* W,
                             const void* W2, const void* bias, int bias_dtype, void* out, int out_dtype, int ldo, int M,
                             int N, int K, int epilogue, const SkinnyNorm& nm) {
  switch (mt) {
    case 1: launch_skinny<1, WAVES>(grid, stream, A, lda, W, W2, bias, bias_dtype, out, out_dtype, ldo, M, N, K, epilogue, nm); break;
    case 2: launch_skinny<2, WAVES>(grid, stream, A, lda, W, W2, bias, bias_dtype, out, out_dtype, ldo, M, N, K, epilogue, nm); break;
    case 3: launch_skinny<3, WAVES>(grid, stream, A, lda, W, W2, bias, bias_dtype, out, out_dtype, ldo, M, N, K, epilogue, nm); break;
    default: launch_skinny<4, WAVES>(grid, stream, A, lda, W, W2, bias, bias_dtype, out, out_dtype, ldo, M, N, K, epilogue, nm); break;
  }
}

static int skinny_checked(const void* A, int lda, const void* W, const void* W2, const void* bias, int bias_dtype,
                          void* out, int out_dtype, int ldo, int M, int N, int K, int epilogue, const SkinnyNorm& nm,
                          int rows2, hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (M > 64 || (K & 127) || (N & 15) || (lda & 7) || K <= 0) return 1;
  if (((uintptr_t)A & 15) || ((uintptr_t)W & 15) || (W2 && ((uintptr_t)W2 & 15))) return 1;
  JLLM_TAKE_GATE("gemm_skinny", epilogue);
  if (epilogue < 0 || epilogue > 2 || (epilogue == 2) != (W2 != nullptr)) JLLM_FAIL("gemm_skinny: epilogue %d", epilogue);
  if (epilogue == 1 && out_dtype != JLLM_F32) JLLM_FAIL("gemm_skinny: the accumulate epilogue adds into fp32");
  if (ldo < N) JLLM_FAIL("gemm_skinny: ldo %d < N %d", ldo, N);
  if (nm.emit_rows && (epilogue != 1 || !nm.emit_gain || !nm.emit_partial)) JLLM_FAIL("gemm_skinny: rows for a norm come from the accumulate epilogue, with gain and partial sums");
  if (nm.norm_partial && nm.norm_parts <= 0) JLLM_FAIL("gemm_skinny: %d partial sums", nm.norm_parts);
  if (nm.norm_partial && ((nm.norm_parts & 3) || ((uintptr_t)nm.norm_partial & 15))) return 1;
  const int mt = (M + 15) / 16;
  int cus = jllm_compute_units();
  if (cus <= 0) JLLM_FAIL("gemm_skinny: the GPU's compute units could not be read");
  // `rows2` > 0: one tile of rows, one weight; a workgroup owns 16 + rows2 weight rows, which the caller asks for
  // where that many fewer workgroups fill the compute units and N / 16 do not (N = 6144 on 256 compute units: 256
  // workgroups of 24 against 384, which leaves every other compute unit with two). Measured on that shape: the same
  // at 1 row, 16.0 -> 14.9 us at 8 rows, 18.8 -> 16.4 at 16 (a third less activation traffic as well). 32 rows per
  // workgroup for the output head, which has thousands of tiles, were measured too: slower below 8 rows (202 ->
  // 218 us at one), so it keeps 16.
  if (rows2 != 0) {
    if (rows2 < 1 || rows2 > 16 || mt != 1 || W2 || N % (16 + rows2))
      JLLM_FAIL("gemm_skinny: %d + 16 weight rows per workgroup need one weight, up to 16 rows and N %% (16 + %d) == 0", rows2, rows2);
    const int groups = N / (16 + rows2);
    if (groups > cus)
      gemm_skinny_kernel<1, false, 4, true><<<groups, 4 * 64, 0, stream>>>((const bf16_t*)A, lda, (const bf16_t*)W, nullptr, bias, bias_dtype,
                                                                           out, out_dtype, ldo, M, N, K, epilogue, nm, rows2);
    else
      gemm_skinny_kernel<1, false, 8, true><<<groups, 8 * 64, 0, stream>>>((const bf16_t*)A, lda, (const bf16_t*)W, nullptr, bias, bias_dtype,
                                                                           out, out_dtype, ldo, M, N, K, epilogue, nm, rows2);
    JLLM_CHECK_LAUNCH("gemm_skinny");
    return 0;
  }
  dim3 grid(N / 16);
  // Every workgroup should be resident at once (a second round of workgroups starts late and runs at half load):
  // with more than one 16-row tile per compute unit the K split is 4 waves instead of 8, so that three workgroups
  // fit on a compute unit.
  if (N / 16 > cus)
    launch_skinny_mt<4>(mt, grid, stream, A, lda, W, W2, bias, bias_dtype, out, out_dtype, ldo, M, N, K, epilogue, nm);
  else
    launch_skinny_mt<8>(mt, grid, stream, A, lda, W, W2, bias, bias_dtype, out, out_dtype, ldo, M, N, K, epilogue, nm);
  JLLM_CHECK_LAUNCH("gemm_skinny");
  return 0;
}

// `rows2`: 0, or the weight rows a workgroup owns beyond its 16 (1 .. 16; one weight, up to 16 rows of activations,
// N a multiple of 16 + rows2). returns 0 when it ran, 1 when the shape is not one it takes (the caller uses another
// kernel), -1 on errors
extern "C" int jllm_gemm_skinny_bf16(const void* A, int lda, const void* W, const void* W2, const void* bias,
                                     int bias_dtype, void* out, int out_dtype, int ldo, int M, int N, int K,
                                     int epilogue, int rows2, hipStream_t stream) {
  return skinny_checked(A, lda, W, W2, bias, bias_dtype, out, out_dtype, ldo, M, N, K, epilogue, SkinnyNorm{}, rows2, stream);
}

// The same with an RMSNorm on either side (see the head of this file). emit_rows [M, N] bf16, emit_gain [N] and
// emit_partial [M][N / 16] fp32 go with the accumulate epilogue; norm_partial [M][norm_parts] with any.
extern "C" int jllm_gemm_skinny_norm_bf16(const void* A, int lda, const void* W, const void* W2, const void* bias,
                                          int bias_dtype, void* out, int out_dtype, int ldo, int M, int N, int K,
                                          int epilogue, int rows2, void* emit_rows, const void* emit_gain,
                                          int emit_gain_dtype, float* emit_partial, const float* norm_partial,
                                          int norm_parts, float norm_eps, hipStream_t stream) {
  SkinnyNorm nm{(bf16_t*)emit_rows, emit_gain, emit_gain_dtype, emit_partial, norm_partial, norm_parts, norm_eps};
  return skinny_checked(A, lda, W, W2, bias, bias_dtype, out, out_dtype, ldo, M, N, K, epilogue, nm, rows2, stream);
}
