// C[M,N] = A[M,K] * W[N,K]^T for any sizes and for fp32 or bf16 operands, accumulated in true fp32 with
// plain FMAs in ascending k (no matrix-core shortcuts): the 32-bit path of every linear layer, and the
// fallback for shapes the MFMA kernels refuse. One output element's sum never depends on M or on the
// other rows of the batch.
//
// Epilogues: 0 store (fp32 or bf16), 1 add into an fp32 matrix (the residual stream), 2 gated:
// out = silu(A*Wg^T) * (A*Wu^T) with two weight matrices sharing the A tile.
#include "common.h"

#define GBN 64
#define GBK 32

// rows x GBK k of a row-major matrix into dst[k][row]; thread i: row i / (GBK / 4) (+ a round's rows), four k
template <typename T, int ROWS>
__device__ __forceinline__ void load_tile(const T* __restrict__ base, int ld, int row0, int nrows, int k0, int K,
                                          float (*dst)[ROWS + 4]) {
  constexpr int TPR = GBK / 4;  // threads per row
  const int kq = (threadIdx.x % TPR) * 4;
#pragma unroll
  for (int r0 = 0; r0 < ROWS; r0 += 256 / TPR) {
    const int r = r0 + (threadIdx.x / TPR);
    const int row = row0 + r;
    const T* p = base + (size_t)row * ld + k0 + kq;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      float v = 0.f;
      if (row < nrows && k0 + kq + j < K) v = ldf(p, j);
      dst[kq + j][r] = v;
    }
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

// TM rows by 4 columns of outputs per thread: a tile of 16 TM rows by 64 columns. With TM = 8 a k step is 32
// multiply-adds for 12 values read from LDS, which the vector units, not LDS, then bound; TM = 4 for few rows, where a
// tile of 128 would be mostly empty.
template <typename TA, typename TW, bool GATED, int TM>
__global__ __launch_bounds__(256) void gemm_generic_kernel(const TA* __restrict__ A, int lda, const TW* __restrict__ W,
                                                           const TW* __restrict__ W2, const void* __restrict__ bias,
                                                           int bias_dtype, void* __restrict__ out, int out_dtype,
                                                           int ldo, int M, int N, int K, int epilogue) {
  constexpr int GBM = 16 * TM;
  __shared__ float As[GBK][GBM + 4];
  __shared__ float Ws[GBK][GBN + 4];
  __shared__ float Us[GATED ? GBK : 1][GBN + 4];
  const int tx = threadIdx.x & 15;
  const int ty = threadIdx.x >> 4;
  const int m0 = blockIdx.y * GBM;
  const int n0 = blockIdx.x * GBN;
  float acc[TM][4] = {};
  float acc2[TM][4] = {};
  for (int k0 = 0; k0 < K; k0 += GBK) {
    load_tile<TA, GBM>(A, lda, m0, M, k0, K, As);
    load_tile<TW, GBN>(W, K, n0, N, k0, K, Ws);
    if (GATED) load_tile<TW, GBN>(W2, K, n0, N, k0, K, Us);
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < GBK; ++kk) {
      float a[TM], w[4], u[4];
#pragma unroll
      for (int i = 0; i < TM; ++i) a[i] = As[kk][ty * TM + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) w[j] = Ws[kk][tx * 4 + j];
      if (GATED) {
#pragma unroll
        for (int j = 0; j < 4; ++j) u[j] = Us[kk][tx * 4 + j];
      }
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          acc[i][j] = fmaf(a[i], w[j], acc[i][j]);
          if (GATED) acc2[i][j] = fmaf(a[i], u[j], acc2[i][j]);
        }
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < TM; ++i) {
    const int m = m0 + ty * TM + i;
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
// GPU idle: one accumulator per output, ascending k, fmaf, as above, so an output has the same bits whichever of the
// two kernels computed it. A workgroup owns 32 weight rows and all the activation rows: thread (r, q) has weight row r
// and activation rows q and q + 8. K advances in turns of 64 through two LDS buffers: the workgroup fetches the turn's
// 32 x 64 weights with every 16 lanes reading 256 contiguous bytes of a row (whole cache lines; a thread walking
// along a row of its own reads 16 bytes of 64 different lines per load instruction, and the loads of such a kernel took
// 3 us a turn), and the activations, which lanes share. A K that is not a multiple of 64 ends in a turn filled up with
// zeros, which add nothing.
#define GR_ROWS 32   // weight rows per workgroup
#define GR_K 64      // k per turn
#define GR_WLD 65    // row stride of the weights in LDS: the lanes of a wave read one column of 32 rows
#define GR_ALD 68    // of the activations: rows q and q + 1 in different banks

template <typename TA, typename TW, bool GATED>
__global__ __launch_bounds__(256) void gemm_rows_kernel(const TA* __restrict__ A, int lda, const TW* __restrict__ W,
                                                        const TW* __restrict__ W2, const void* __restrict__ bias,
                                                        int bias_dtype, void* __restrict__ out, int out_dtype, int ldo,
                                                        int M, int N, int K, int epilogue) {
  __shared__ float ws[2][GATED ? 2 : 1][GR_ROWS][GR_WLD];
  __shared__ float as[2][16][GR_ALD];
  const int r = threadIdx.x & (GR_ROWS - 1), q = threadIdx.x / GR_ROWS;  // q = 0 .. 7
  const int n0 = blockIdx.x * GR_ROWS;
  // staging: element e = threadIdx.x + 256 i of the 32 x 64 tile is (row e / 64, k e % 64): a wave reads one row's 256
  // bytes; of the 16 x 64 activations likewise
  struct Staged {
    float w[8], u[GATED ? 8 : 1], a[4];
  };
  auto fetch = [&](Staged& st, int k0) {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int e = threadIdx.x + 256 * i;
      const int row = min(n0 + e / GR_K, N - 1), k = k0 + e % GR_K;
      st.w[i] = k < K ? ldf(W + (size_t)row * K, k) : 0.f;
      if (GATED) st.u[i] = k < K ? ldf(W2 + (size_t)row * K, k) : 0.f;
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int e = threadIdx.x + 256 * i;
      const int m = e / GR_K, k = k0 + e % GR_K;
      st.a[i] = (m < M && k < K) ? ldf(A + (size_t)m * lda, k) : 0.f;
    }
  };
  auto put = [&](const Staged& st, int buf) {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int e = threadIdx.x + 256 * i;
      ws[buf][0][e / GR_K][e % GR_K] = st.w[i];
      if (GATED) ws[buf][GATED ? 1 : 0][e / GR_K][e % GR_K] = st.u[i];
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int e = threadIdx.x + 256 * i;
      as[buf][e / GR_K][e % GR_K] = st.a[i];
    }
  };
  float acc[2] = {0.f, 0.f}, acc2[2] = {0.f, 0.f};
  const int turns = (K + GR_K - 1) / GR_K;
  Staged st;
  fetch(st, 0);
  put(st, 0);
  __syncthreads();
  for (int turn = 0; turn < turns; ++turn) {
    const int buf = turn & 1;
    if (turn + 1 < turns) fetch(st, (turn + 1) * GR_K);
#pragma unroll 8
    for (int k = 0; k < GR_K; ++k) {
      const float wv = ws[buf][0][r][k];
      const float uv = GATED ? ws[buf][GATED ? 1 : 0][r][k] : 0.f;
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        const float av = as[buf][q + 8 * i][k];
        acc[i] = fmaf(av, wv, acc[i]);
        if (GATED) acc2[i] = fmaf(av, uv, acc2[i]);
      }
    }
    if (turn + 1 < turns) put(st, buf ^ 1);
    __syncthreads();
  }
  const int n = n0 + r;
  if (n >= N) return;
#pragma unroll
  for (int i = 0; i < 2; ++i)
    if (q + 8 * i < M) finish_output<GATED>(acc[i], acc2[i], q + 8 * i, n, bias, bias_dtype, out, out_dtype, ldo, epilogue);
}

template <typename TA, typename TW>
static void launch_rows(const void* A, int lda, const void* W, const void* W2, const void* bias, int bias_dtype, void* out,
                        int out_dtype, int ldo, int M, int N, int K, int epilogue, hipStream_t stream) {
  dim3 grid((N + GR_ROWS - 1) / GR_ROWS);
  if (W2)
    gemm_rows_kernel<TA, TW, true><<<grid, 256, 0, stream>>>((const TA*)A, lda, (const TW*)W, (const TW*)W2, bias,
                                                             bias_dtype, out, out_dtype, ldo, M, N, K, epilogue);
  else
    gemm_rows_kernel<TA, TW, false><<<grid, 256, 0, stream>>>((const TA*)A, lda, (const TW*)W, nullptr, bias,
                                                              bias_dtype, out, out_dtype, ldo, M, N, K, epilogue);
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
        launch_rows<TA, TW>(A, lda, W, W2, bias, bias_dtype, out, out_dtype, ldo, M, N, K, epilogue, stream);
      })
    })
    JLLM_CHECK_LAUNCH("gemm_rows");
    return 0;
  }
  const bool tall = M > 64;  // tiles of 128 rows
  dim3 grid((N + GBN - 1) / GBN, tall ? (M + 127) / 128 : (M + 63) / 64);
  if (grid.y > 65535) JLLM_FAIL("gemm: M=%d is too large for this kernel", M);
  JLLM_DISPATCH_1(a_dtype, TA, {
    JLLM_DISPATCH_1(w_dtype, TW, {
      if (W2 && tall)
        gemm_generic_kernel<TA, TW, true, 8><<<grid, 256, 0, stream>>>((const TA*)A, lda, (const TW*)W, (const TW*)W2, bias,
                                                                        bias_dtype, out, out_dtype, ldo, M, N, K, epilogue);
      else if (W2)
        gemm_generic_kernel<TA, TW, true, 4><<<grid, 256, 0, stream>>>((const TA*)A, lda, (const TW*)W, (const TW*)W2, bias,
                                                                        bias_dtype, out, out_dtype, ldo, M, N, K, epilogue);
      else if (tall)
        gemm_generic_kernel<TA, TW, false, 8><<<grid, 256, 0, stream>>>((const TA*)A, lda, (const TW*)W, nullptr, bias,
                                                                         bias_dtype, out, out_dtype, ldo, M, N, K, epilogue);
      else
        gemm_generic_kernel<TA, TW, false, 4><<<grid, 256, 0, stream>>>((const TA*)A, lda, (const TW*)W, nullptr, bias,
                                                                         bias_dtype, out, out_dtype, ldo, M, N, K, epilogue);
    })
  })
  JLLM_CHECK_LAUNCH("gemm_generic");
  return 0;
}
