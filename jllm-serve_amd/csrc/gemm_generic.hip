// C[M,N] = A[M,K] * W[N,K]^T for any sizes and for fp32 or bf16 operands, accumulated in true fp32 with
// plain FMAs in ascending k (no matrix-core shortcuts): the 32-bit path of every linear layer, and the
// fallback for shapes the MFMA kernels refuse. One output element's sum never depends on M or on the
// other rows of the batch.
//
// Epilogues: 0 store (fp32 or bf16), 1 add into an fp32 matrix (the residual stream), 2 gated:
// out = silu(A*Wg^T) * (A*Wu^T) with two weight matrices sharing the A tile.
#include "common.h"

#define GBM 64
#define GBN 64
#define GBK 16

template <typename T>
__device__ __forceinline__ void load_tile(const T* __restrict__ base, int ld, int row0, int nrows, int k0, int K,
                                          float (*dst)[GBM + 4]) {
  // 64 rows x 16 k; thread i: row i/4, k (i%4)*4 .. +4
  const int r = threadIdx.x >> 2;
  const int kq = (threadIdx.x & 3) * 4;
  const int row = row0 + r;
  const T* p = base + (size_t)row * ld + k0 + kq;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    float v = 0.f;
    if (row < nrows && k0 + kq + j < K) v = ldf(p, j);
    dst[kq + j][r] = v;
  }
}

// bias, gate and store of one output: the same arithmetic in both kernels of this file
template <bool GATED>
__device__ __forceinline__ void finish_output(float v, float up, int m, int n, const void* __restrict__ bias, int bias_dtype,
                                              void* __restrict__ out, int out_dtype, int ldo, int epilogue) {
  if (bias) v += (bias_dtype == JLLM_BF16) ? ldf((const bf16_t*)bias, n) : ldf((const float*)bias, n);
  const size_t o = (size_t)m * ldo + n;
  if (GATED) {
    const float g = v;
    v = gate_fn<false>(g) * up;
  }
  if (epilogue == 1) {
    ((float*)out)[o] += v;
  } else if (out_dtype == JLLM_BF16) {
    stf((bf16_t*)out, o, v);
  } else {
    stf((float*)out, o, v);
  }
}

template <typename TA, typename TW, bool GATED>
__global__ __launch_bounds__(256) void gemm_generic_kernel(const TA* __restrict__ A, int lda, const TW* __restrict__ W,
                                                           const TW* __restrict__ W2, const void* __restrict__ bias,
                                                           int bias_dtype, void* __restrict__ out, int out_dtype,
                                                           int ldo, int M, int N, int K, int epilogue) {
  __shared__ float As[GBK][GBM + 4];
  __shared__ float Ws[GBK][GBN + 4];
  __shared__ float Us[GATED ? GBK : 1][GBN + 4];
  const int tx = threadIdx.x & 15;
  const int ty = threadIdx.x >> 4;
  const int m0 = blockIdx.y * GBM;
  const int n0 = blockIdx.x * GBN;
  float acc[4][4] = {};
  float acc2[4][4] = {};
  for (int k0 = 0; k0 < K; k0 += GBK) {
    load_tile<TA>(A, lda, m0, M, k0, K, As);
    load_tile<TW>(W, K, n0, N, k0, K, Ws);
    if (GATED) load_tile<TW>(W2, K, n0, N, k0, K, Us);
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < GBK; ++kk) {
      float a[4], w[4], u[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = As[kk][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) w[j] = Ws[kk][tx * 4 + j];
      if (GATED) {
#pragma unroll
        for (int j = 0; j < 4; ++j) u[j] = Us[kk][tx * 4 + j];
      }
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          acc[i][j] = fmaf(a[i], w[j], acc[i][j]);
          if (GATED) acc2[i][j] = fmaf(a[i], u[j], acc2[i][j]);
        }
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int m = m0 + ty * 4 + i;
    if (m >= M) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tx * 4 + j;
      if (n >= N) continue;
      finish_output<GATED>(acc[i][j], acc2[i][j], m, n, bias, bias_dtype, out, out_dtype, ldo, epilogue);
    }
  }
}

// The same sums for up to 16 rows (decode steps of the 32-bit path), where a 64 x 64 tile would leave most of the
// GPU idle: a thread owns one weight row and RM activation rows, one accumulator per output, ascending k, fmaf, as
// above, so an output has the same bits whichever of the two kernels computed it. The weights stream through 16-byte
// loads (eight k per turn where K and the alignment allow); the activations of a turn are the same for every lane.
template <typename T>
__device__ __forceinline__ void load8(const T* __restrict__ p, float (&v)[8]);
template <>
__device__ __forceinline__ void load8<float>(const float* __restrict__ p, float (&v)[8]) {
  const float4 a = *(const float4*)p, b = *(const float4*)(p + 4);
  v[0] = a.x, v[1] = a.y, v[2] = a.z, v[3] = a.w, v[4] = b.x, v[5] = b.y, v[6] = b.z, v[7] = b.w;
}
template <>
__device__ __forceinline__ void load8<bf16_t>(const bf16_t* __restrict__ p, float (&v)[8]) {
  const uint4 r = *(const uint4*)p;
  const unsigned w[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    v[2 * i] = __builtin_bit_cast(float, w[i] << 16);
    v[2 * i + 1] = __builtin_bit_cast(float, w[i] & 0xffff0000u);
  }
}

template <typename TA, typename TW, bool GATED, int RM>
__global__ __launch_bounds__(256) void gemm_rows_kernel(const TA* __restrict__ A, int lda, const TW* __restrict__ W,
                                                        const TW* __restrict__ W2, const void* __restrict__ bias,
                                                        int bias_dtype, void* __restrict__ out, int out_dtype, int ldo,
                                                        int M, int N, int K, int epilogue, int wide) {
  const int n = blockIdx.x * 256 + threadIdx.x;
  const int m0 = blockIdx.y * RM;
  if (n >= N) return;
  const TW* w = W + (size_t)n * K;
  const TW* u = GATED ? W2 + (size_t)n * K : nullptr;
  const TA* a[RM];
#pragma unroll
  for (int i = 0; i < RM; ++i) a[i] = A + (size_t)min(m0 + i, M - 1) * lda;  // rows beyond M: the last row, never stored
  float acc[RM], acc2[RM];
#pragma unroll
  for (int i = 0; i < RM; ++i) acc[i] = acc2[i] = 0.f;
  int k = 0;
  if (wide) {  // K % 8 == 0 and 16-byte aligned weight rows
#pragma unroll 2
    for (; k < K; k += 8) {
      float wv[8], uv[8];
      load8<TW>(w + k, wv);
      if (GATED) load8<TW>(u + k, uv);
#pragma unroll
      for (int i = 0; i < RM; ++i) {
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const float av = ldf(a[i], k + j);
          acc[i] = fmaf(av, wv[j], acc[i]);
          if (GATED) acc2[i] = fmaf(av, uv[j], acc2[i]);
        }
      }
    }
  }
  for (; k < K; ++k) {
    const float wv = ldf(w, k), uv = GATED ? ldf(u, k) : 0.f;
#pragma unroll
    for (int i = 0; i < RM; ++i) {
      const float av = ldf(a[i], k);
      acc[i] = fmaf(av, wv, acc[i]);
      if (GATED) acc2[i] = fmaf(av, uv, acc2[i]);
    }
  }
#pragma unroll
  for (int i = 0; i < RM; ++i)
    if (m0 + i < M) finish_output<GATED>(acc[i], acc2[i], m0 + i, n, bias, bias_dtype, out, out_dtype, ldo, epilogue);
}

template <typename TA, typename TW, int RM>
static void launch_rows(const void* A, int lda, const void* W, const void* W2, const void* bias, int bias_dtype, void* out,
                        int out_dtype, int ldo, int M, int N, int K, int epilogue, hipStream_t stream) {
  dim3 grid((N + 255) / 256, (M + RM - 1) / RM);
  const int esz = (int)sizeof(TW);
  const int wide = (K % 8 == 0) && (((uintptr_t)W % 16) == 0) && (!W2 || ((uintptr_t)W2 % 16) == 0) && ((size_t)K * esz % 16 == 0);
  if (W2)
    gemm_rows_kernel<TA, TW, true, RM><<<grid, 256, 0, stream>>>((const TA*)A, lda, (const TW*)W, (const TW*)W2, bias,
                                                                 bias_dtype, out, out_dtype, ldo, M, N, K, epilogue, wide);
  else
    gemm_rows_kernel<TA, TW, false, RM><<<grid, 256, 0, stream>>>((const TA*)A, lda, (const TW*)W, nullptr, bias,
                                                                  bias_dtype, out, out_dtype, ldo, M, N, K, epilogue, wide);
}

#define GEMM_ROWS_MAX 16

extern "C" int jllm_gemm_generic(const void* A, int a_dtype, int lda, const void* W, const void* W2, int w_dtype,
                                 const void* bias, int bias_dtype, void* out, int out_dtype, int ldo, int M, int N,
                                 int K, int epilogue, hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (K <= 0) JLLM_FAIL("gemm: K=%d", K);
  if (lda < K || ldo < N) JLLM_FAIL("gemm: leading dimensions lda=%d K=%d ldo=%d N=%d", lda, K, ldo, N);
  JLLM_TAKE_GATE("gemm", epilogue);
  if (epilogue < 0 || epilogue > 2) JLLM_FAIL("gemm: epilogue %d", epilogue);
  if ((epilogue == 2) != (W2 != nullptr)) JLLM_FAIL("gemm: the gated epilogue needs exactly two weight matrices");
  if (epilogue == 1 && out_dtype != JLLM_F32) JLLM_FAIL("gemm: the accumulate epilogue adds into fp32");
  if (M <= GEMM_ROWS_MAX) {
    JLLM_DISPATCH_1(a_dtype, TA, {
      JLLM_DISPATCH_1(w_dtype, TW, {
        if (M >= 4)
          launch_rows<TA, TW, 4>(A, lda, W, W2, bias, bias_dtype, out, out_dtype, ldo, M, N, K, epilogue, stream);
        else if (M >= 2)
          launch_rows<TA, TW, 2>(A, lda, W, W2, bias, bias_dtype, out, out_dtype, ldo, M, N, K, epilogue, stream);
        else
          launch_rows<TA, TW, 1>(A, lda, W, W2, bias, bias_dtype, out, out_dtype, ldo, M, N, K, epilogue, stream);
      })
    })
    JLLM_CHECK_LAUNCH("gemm_rows");
    return 0;
  }
  dim3 grid((N + GBN - 1) / GBN, (M + GBM - 1) / GBM);
  if (grid.y > 65535) JLLM_FAIL("gemm: M=%d is too large for this kernel", M);
  JLLM_DISPATCH_1(a_dtype, TA, {
    JLLM_DISPATCH_1(w_dtype, TW, {
      if (W2)
        gemm_generic_kernel<TA, TW, true><<<grid, 256, 0, stream>>>((const TA*)A, lda, (const TW*)W, (const TW*)W2, bias,
                                                                     bias_dtype, out, out_dtype, ldo, M, N, K, epilogue);
      else
        gemm_generic_kernel<TA, TW, false><<<grid, 256, 0, stream>>>((const TA*)A, lda, (const TW*)W, nullptr, bias,
                                                                      bias_dtype, out, out_dtype, ldo, M, N, K, epilogue);
    })
  })
  JLLM_CHECK_LAUNCH("gemm_generic");
  return 0;
}
