// out[M,N] = A[M,K] * W[N,K]^T for many rows (prompt portions): bf16 operands staged through LDS, fp32
// accumulation on the matrix cores (v_mfma_f32_32x32x16_bf16).
//
// Two tile shapes. The small one: 4 waves in a 2 x 2 arrangement over a 128 x 128 output tile, each wave owning
// 64 x 64 = four 32 x 32 accumulators; two such workgroups share a compute unit. The large one, for products
// with many tiles: 8 waves in a 2 x 4 arrangement over 256 x 256, each wave owning 128 x 64 (fewer LDS bytes per
// multiply). K advances in steps of 64 through two LDS buffers: while the waves multiply out of
// one, the 16-byte global loads of the next step are already in registers and are stored into the other.
// LDS rows are padded by 16 bytes so that the 16-byte operand reads of neighbouring rows fall into
// different banks. With gridDim.x a multiple of 8, the workgroups that share a weight tile run on the same
// XCD (workgroups go round-robin to the 8 XCDs by linear id), so the tile is fetched into one L2.
//
// Epilogues: store, add into the fp32 residual, gated. For the gated one the LDS rows of the weight tile are,
// per 64 rows, 32 gate rows and the 32 matching up rows, so that every wave holds gate and up of the same 32
// outputs in neighbouring accumulators and silu(gate) * up is formed in registers.
//
// Needs K % 64 == 0 and 16-byte aligned rows; any M and N. The caller falls back otherwise.
#include "common.h"
#include "gemm_epilogue.h"
#include "mfma.h"

#define TBK 64
#define TPCS (TBK / 8)  // 16-byte pieces per tile row
#define TLD (TBK + 8)   // LDS row stride in elements

// WGM x WGN waves, each with FM x FN accumulators of 32 x 32 (FN = 2 for the gated epilogue: gate and up)
template <bool GATED, int WGM, int WGN, int FM, int FN, bool DEEP>
__global__ __launch_bounds__(WGM* WGN * 64) void gemm_mfma_kernel(
    const bf16_t* __restrict__ A, int lda, const bf16_t* __restrict__ W, const bf16_t* __restrict__ W2,
    const void* __restrict__ bias, int bias_dtype, void* __restrict__ out, int out_dtype, int ldo, int M, int N, int K,
    int epilogue, float* __restrict__ partial) {
  static_assert(FN == 2, "a wave's columns are two 32-wide accumulators (gate and up with the gated epilogue)");
  constexpr int NT = WGM * WGN * 64;
  constexpr int TBM = WGM * FM * 32, TBN = WGN * FN * 32;
  constexpr int TRSTEP = NT / TPCS;        // rows between a thread's pieces
  constexpr int PA = TBM / TRSTEP, PB = TBN / TRSTEP;  // pieces per thread
  extern __shared__ __align__(16) unsigned char smem_raw[];
  bf16_t* As = (bf16_t*)smem_raw;             // [2][TBM][TLD]
  bf16_t* Bs = As + 2 * TBM * TLD;            // [2][TBN][TLD]
  const int tid = threadIdx.x;
  const int wave = tid >> 6, lane = tid & 63;
  const int wm = wave / WGN, wn = wave % WGN;
  const int m0 = blockIdx.y * TBM;
  const int n0 = blockIdx.x * (GATED ? TBN / 2 : TBN);  // output columns covered by this workgroup start here
  // global -> register staging: piece c = tid + NT j: row c / TPCS, 16 bytes number c % TPCS
  const int lrow = tid / TPCS, lpc = tid % TPCS;
  const bf16_t* aptr[PA];
  const bf16_t* bptr[PB];
#pragma unroll
  for (int j = 0; j < PA; ++j) aptr[j] = A + (size_t)min(m0 + lrow + TRSTEP * j, M - 1) * lda + lpc * 8;
#pragma unroll
  for (int j = 0; j < PB; ++j) {
    const int r = lrow + TRSTEP * j;
    int wr;
    const bf16_t* wb = W;
    if (GATED) {  // LDS row r: quarter r / 32: even = gate, odd = up of the outputs n0 + (quarter / 2) * 32 ..
      const int quarter = r >> 5;
      wr = n0 + (quarter >> 1) * 32 + (r & 31);
      wb = (quarter & 1) ? W2 : W;
    } else {
      wr = n0 + r;
    }
    bptr[j] = wb + (size_t)min(wr, N - 1) * K + lpc * 8;
  }
  // gridDim.z > 1: this workgroup multiplies only its share of K and leaves an fp32 partial tile
  const int nk_all = K / TBK;
  const int nk_per = (nk_all + gridDim.z - 1) / gridDim.z;
  const int kt0 = blockIdx.z * nk_per;
  const int nk = max(0, min(nk_all, kt0 + nk_per) - kt0);
  floatx16 acc[FM][FN];
#pragma unroll
  for (int i = 0; i < FM; ++i)
#pragma unroll
    for (int j = 0; j < FN; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;
#pragma unroll
  for (int j = 0; j < PA; ++j) aptr[j] += (size_t)kt0 * TBK;
#pragma unroll
  for (int j = 0; j < PB; ++j) bptr[j] += (size_t)kt0 * TBK;
  struct Staged {
    u32x4 a[PA], b[PB];
  };
  auto request = [&](Staged& r, int kt) {  // the global loads of K step kt
#pragma unroll
    for (int j = 0; j < PA; ++j) r.a[j] = *(const u32x4*)(aptr[j] + (size_t)kt * TBK);
#pragma unroll
    for (int j = 0; j < PB; ++j) r.b[j] = *(const u32x4*)(bptr[j] + (size_t)kt * TBK);
  };
  auto put = [&](const Staged& r, int buf) {  // into LDS buffer buf
#pragma unroll
    for (int j = 0; j < PA; ++j) *(u32x4*)(As + (size_t)buf * TBM * TLD + (size_t)(lrow + TRSTEP * j) * TLD + lpc * 8) = r.a[j];
#pragma unroll
    for (int j = 0; j < PB; ++j) *(u32x4*)(Bs + (size_t)buf * TBN * TLD + (size_t)(lrow + TRSTEP * j) * TLD + lpc * 8) = r.b[j];
  };
  const int fr = lane & 31;        // fragment row / column
  const int fk = (lane >> 5) * 8;  // fragment k offset
  auto multiply = [&](int cur) {
    const bf16_t* Ac = As + (size_t)cur * TBM * TLD + (size_t)(wm * FM * 32 + fr) * TLD + fk;
    const bf16_t* Bc = Bs + (size_t)cur * TBN * TLD + (size_t)(wn * FN * 32 + fr) * TLD + fk;
    // the weight fragment goes in as the first operand: the accumulator then holds the tile transposed (rows =
    // output columns), so a lane owns four consecutive output columns of one row and stores them at once
    constexpr int KS = DEEP ? 2 : TBK / 16;  // k16 steps whose fragments are in registers together
#pragma unroll
    for (int k0 = 0; k0 < TBK / 16; k0 += KS) {
      u32x4 af[KS][FM], bf[KS][FN];
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
#pragma unroll
        for (int i = 0; i < FM; ++i) af[ks][i] = *(const u32x4*)(Ac + i * 32 * TLD + (k0 + ks) * 16);
#pragma unroll
        for (int j = 0; j < FN; ++j) bf[ks][j] = *(const u32x4*)(Bc + j * 32 * TLD + (k0 + ks) * 16);
      }
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
#pragma unroll
        for (int i = 0; i < FM; ++i)
#pragma unroll
          for (int j = 0; j < FN; ++j) acc[i][j] = mfma32(bf[ks][j], af[ks][i], acc[i][j]);
      }
      // the order of issue: the LDS reads of step ks + 1 go out before the multiplies of step ks
      __builtin_amdgcn_sched_group_barrier(0x100, FM + FN, 0);
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        if (ks + 1 < KS) __builtin_amdgcn_sched_group_barrier(0x100, FM + FN, 0);
        __builtin_amdgcn_sched_group_barrier(0x008, FM * FN, 0);
      }
    }
  };
  if (nk > 0) {
    if constexpr (DEEP) {
      // Two K steps on their way while a third is multiplied: a step of the small tile is 0.2 us of work, and with
      // one step in flight every step waited a memory latency (1.1 us a step for weights that come from HBM once).
      // Two register sets take turns, so the wait before a set is stored names only the older of the two requests.
      // No branch stands around a request (the compiler would wait for every load behind one): a step beyond the
      // last is the last step once more, stored where nobody reads it again.
      Staged r0, r1;
      const int last = nk - 1;
      request(r0, 0);
      request(r1, min(1, last));
      put(r0, 0);
      request(r0, min(2, last));
      __syncthreads();
      for (int kt = 0; kt < nk; kt += 2) {
        multiply(0);
        put(r1, 1);
        request(r1, min(kt + 3, last));
        __syncthreads();
        if (kt + 1 >= nk) break;
        multiply(1);
        put(r0, 0);
        request(r0, min(kt + 4, last));
        __syncthreads();
      }
    } else {
      Staged r;
      request(r, 0);
      put(r, 0);
      __syncthreads();
      for (int kt = 0; kt < nk; ++kt) {
        const int cur = kt & 1;
        if (kt + 1 < nk) request(r, kt + 1);
        multiply(cur);
        if (kt + 1 < nk) put(r, cur ^ 1);
        __syncthreads();
      }
    }
  }
  tile_epilogue<GATED, FM, FN, TBM, TBN>(acc, lane, wm, wn, m0, n0, bias, bias_dtype, out, out_dtype, ldo, M, N, epilogue, partial,
                                         (int)blockIdx.z, (int)gridDim.z);
}

// sums the K-split partials in ascending order of the split and applies bias and epilogue; V outputs per thread
// (4 when the rows allow 16-byte accesses)
template <int V>
__global__ __launch_bounds__(256) void splitk_reduce_kernel(const float* __restrict__ partial, int splits,
                                                            const void* __restrict__ bias, int bias_dtype,
                                                            void* __restrict__ out, int out_dtype, int ldo, int M, int N,
                                                            int epilogue) {
  const size_t i = ((size_t)blockIdx.x * 256 + threadIdx.x) * V;
  if (i >= (size_t)M * N) return;
  const int m = (int)(i / N), n = (int)(i % N);
  float v[V];
#pragma unroll
  for (int e = 0; e < V; ++e) v[e] = 0.f;
  for (int z = 0; z < splits; ++z) {
    const float* p = partial + (size_t)z * M * N + i;
    if (V == 4) {
      const float4 t = *(const float4*)p;
      v[0] += t.x, v[1 % V] += t.y, v[2 % V] += t.z, v[3 % V] += t.w;
    } else {
      v[0] += p[0];
    }
  }
  if (bias) {
#pragma unroll
    for (int e = 0; e < V; ++e)
      v[e] += (bias_dtype == JLLM_BF16) ? ldf((const bf16_t*)bias, n + e) : ldf((const float*)bias, n + e);
  }
  const size_t o = (size_t)m * ldo + n;
  if (epilogue == 1) {
    float* r = (float*)out + o;
    if (V == 4) {
      float4 t = *(float4*)r;
      t.x += v[0], t.y += v[1 % V], t.z += v[2 % V], t.w += v[3 % V];
      *(float4*)r = t;
    } else {
      r[0] += v[0];
    }
  } else if (out_dtype == JLLM_BF16) {
#pragma unroll
    for (int e = 0; e < V; ++e) stf((bf16_t*)out, o + e, v[e]);
  } else {
#pragma unroll
    for (int e = 0; e < V; ++e) stf((float*)out, o + e, v[e]);
  }
}

int jllm_splitk_reduce(const float* partial, int splits, const void* bias, int bias_dtype, void* out, int out_dtype,
                       int ldo, int M, int N, int epilogue, hipStream_t stream) {
  const size_t total = (size_t)M * N;
  if ((N & 3) == 0 && (ldo & 3) == 0 && ((uintptr_t)out & 15) == 0 && ((uintptr_t)partial & 15) == 0) {
    splitk_reduce_kernel<4><<<(unsigned)((total / 4 + 255) / 256), 256, 0, stream>>>(partial, splits, bias, bias_dtype, out,
                                                                                   out_dtype, ldo, M, N, epilogue);
  } else {
    splitk_reduce_kernel<1><<<(unsigned)((total + 255) / 256), 256, 0, stream>>>(partial, splits, bias, bias_dtype, out,
                                                                               out_dtype, ldo, M, N, epilogue);
  }
  JLLM_CHECK_LAUNCH("splitk_reduce");
  return 0;
}

template <int WGM, int WGN, int FM, int FN, bool DEEP>
static int launch_tiled(const void* A, int lda, const void* W, const void* W2, const void* bias, int bias_dtype,
                        void* out, int out_dtype, int ldo, int M, int N, int K, int epilogue, int splits,
                        float* partial, hipStream_t stream) {
  constexpr int TBM = WGM * FM * 32, TBN = WGN * FN * 32;
  const int cols = W2 ? TBN / 2 : TBN;
  dim3 grid((N + cols - 1) / cols, (M + TBM - 1) / TBM, splits);
  if (grid.y > 65535) return 1;
  const size_t smem = (size_t)2 * (TBM + TBN) * TLD * sizeof(bf16_t);
  static bool configured = false;
  if (!configured) {
    hipError_t e1 = hipFuncSetAttribute((const void*)gemm_mfma_kernel<true, WGM, WGN, FM, FN, DEEP>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    hipError_t e2 = hipFuncSetAttribute((const void*)gemm_mfma_kernel<false, WGM, WGN, FM, FN, DEEP>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    if (e1 != hipSuccess || e2 != hipSuccess) JLLM_FAIL("gemm_mfma: cannot reserve %zu bytes of LDS", smem);
    configured = true;
  }
  if (W2)
    gemm_mfma_kernel<true, WGM, WGN, FM, FN, DEEP><<<grid, WGM * WGN * 64, smem, stream>>>(
        (const bf16_t*)A, lda, (const bf16_t*)W, (const bf16_t*)W2, bias, bias_dtype, out, out_dtype, ldo, M, N, K, epilogue, partial);
  else
    gemm_mfma_kernel<false, WGM, WGN, FM, FN, DEEP><<<grid, WGM * WGN * 64, smem, stream>>>(
        (const bf16_t*)A, lda, (const bf16_t*)W, nullptr, bias, bias_dtype, out, out_dtype, ldo, M, N, K, epilogue, partial);
  return 0;
}

// `splits` > 1 cuts K over gridDim.z (not with the gated epilogue); `partial` then holds splits * M * N floats.
// returns 0 when it ran, 1 when the shape is not one it takes, -1 on errors
extern "C" int jllm_gemm_mfma_bf16(const void* A, int lda, const void* W, const void* W2, const void* bias,
                                   int bias_dtype, void* out, int out_dtype, int ldo, int M, int N, int K, int epilogue,
                                   int splits, float* partial, hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (K <= 0 || (K % TBK) || (lda & 7)) return 1;
  if (((uintptr_t)A & 15) || ((uintptr_t)W & 15) || (W2 && ((uintptr_t)W2 & 15))) return 1;
  JLLM_TAKE_GATE("gemm_mfma", epilogue);
  if (epilogue < 0 || epilogue > 2 || (epilogue == 2) != (W2 != nullptr)) JLLM_FAIL("gemm_mfma: epilogue %d", epilogue);
  if (epilogue == 1 && out_dtype != JLLM_F32) JLLM_FAIL("gemm_mfma: the accumulate epilogue adds into fp32");
  if (ldo < N) JLLM_FAIL("gemm_mfma: ldo %d < N %d", ldo, N);
  if (splits < 1) splits = 1;
  if (splits > 1 && (W2 || !partial || (K / TBK) % splits != 0)) JLLM_FAIL("gemm_mfma: %d K splits are not possible here", splits);
  // the large tile when it still gives every compute unit two rounds of work, or when one round of it fills three
  // quarters of the compute units or more (the small tile would then need a second, half-empty round)
  const long big_tiles = (long)((N + (W2 ? 127 : 255)) / (W2 ? 128 : 256)) * ((M + 255) / 256);
  int rc;
  if (splits == 1 && (big_tiles >= 512 || (big_tiles >= 192 && big_tiles <= 256)))
    rc = launch_tiled<2, 4, 4, 2, false>(A, lda, W, W2, bias, bias_dtype, out, out_dtype, ldo, M, N, K, epilogue, 1, partial, stream);
  else {
    // The small tile with two K steps requested ahead where every workgroup has a compute unit to itself: then a step
    // takes 0.85 us instead of 1.1 (gate/up at 128 rows of the 8B shape, 192 workgroups: 68 -> 54 us; down, 256: 38 ->
    // 33). Where compute units hold two workgroups the deeper requests of both only crowd the one path into LDS
    // (384 workgroups: 73 -> 89 us), so those keep one step ahead.
    const long groups = (long)((N + (W2 ? 63 : 127)) / (W2 ? 64 : 128)) * ((M + 127) / 128) * splits;
    const int cus = jllm_compute_units();
    if (cus > 0 && groups <= cus)
      rc = launch_tiled<2, 2, 2, 2, true>(A, lda, W, W2, bias, bias_dtype, out, out_dtype, ldo, M, N, K, epilogue, splits, partial, stream);
    else
      rc = launch_tiled<2, 2, 2, 2, false>(A, lda, W, W2, bias, bias_dtype, out, out_dtype, ldo, M, N, K, epilogue, splits, partial, stream);
  }
  if (rc != 0) return rc;
  JLLM_CHECK_LAUNCH("gemm_mfma");
  if (splits > 1) return jllm_splitk_reduce(partial, splits, bias, bias_dtype, out, out_dtype, ldo, M, N, epilogue, stream);
  return 0;
}
