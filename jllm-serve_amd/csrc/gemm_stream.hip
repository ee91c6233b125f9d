// out[M,N] = A[M,K] * W[N,K]^T for 17 to 64 rows (decode steps of many requests, small prompt portions): bf16
// operands, fp32 accumulation on the matrix cores (16x16x32), bound by streaming W from HBM once.
//
// A workgroup of 8 waves owns 128 weight rows and a range of K; wave w owns rows 16 w .. 16 w + 15 and keeps their
// sums for all the activation rows (up to four 16-row tiles), so nothing is reduced inside the workgroup. The weights
// go straight from memory into the registers that feed the matrix cores, 16 bytes per lane and load, requested
// two steps of K ahead (lane l, load j of a 128-wide block: row l%16, k = block * 128 + j * 32 + (l/16) * 8 .. + 8;
// both operands use this k assignment). The activations, which all 8 waves share, go through LDS: the chunk of
// the next step is requested before this step's products and stored behind them, one barrier per step. Rows are
// padded by 16 bytes so that the 16 lanes of a tile row read different banks.
//
// Products with few column tiles cut K over gridDim.y; each part leaves an fp32 partial [part][matrix][M][N] and
// a second kernel adds the parts in ascending order and applies bias and epilogue (store, add into the fp32
// residual, gated with two weights). How K is cut depends on N and K only, never on M: a row's result does not
// depend on the rows beside it.
//
// Needs K % 128 == 0, N % 16 == 0, M <= 64, 16-byte aligned rows; the caller uses another kernel otherwise.
#include "common.h"
#include "mfma.h"

#define GS_WAVES 8
#define GS_COLS (GS_WAVES * 16)

template <int MT, bool GATED>
__global__ __launch_bounds__(GS_WAVES * 64) void gemm_stream_kernel(
    const bf16_t* __restrict__ A, int lda, const bf16_t* __restrict__ W, const bf16_t* __restrict__ W2,
    const void* __restrict__ bias, int bias_dtype, void* __restrict__ out, int out_dtype, int ldo, int M, int N, int K,
    int epilogue, float* __restrict__ partial, int blocks_per_part) {
  constexpr int UB = GATED ? 1 : 2;            // 128-wide K blocks per step
  constexpr int LD = UB * 128 + 8;             // LDS row stride in elements
  constexpr int PIECES = MT * 16 * UB * 16;    // 16-byte pieces of an activation chunk
  constexpr int PPT = (PIECES + GS_WAVES * 64 - 1) / (GS_WAVES * 64);
  extern __shared__ __align__(16) unsigned char smem_raw[];
  bf16_t(*As)[MT * 16][LD] = (bf16_t(*)[MT * 16][LD])smem_raw;  // [2][MT * 16][LD]
  const int tid = threadIdx.x;
  const int wave = tid >> 6, lane = tid & 63;
  const int col = lane & 15, g = lane >> 4;
  const int n0 = blockIdx.x * GS_COLS + wave * 16;
  const bool live = n0 < N;  // N is a multiple of 16: a wave has all of its rows or none
  const int nblk = K >> 7;
  const int b_begin = blockIdx.y * blocks_per_part;
  const int b_end = min(nblk, b_begin + blocks_per_part);
  const int steps = (b_end - b_begin + UB - 1) / UB;
  const bf16_t* wrow = W + (size_t)(live ? n0 + col : 0) * K + g * 8;
  const bf16_t* urow = GATED ? W2 + (size_t)(live ? n0 + col : 0) * K + g * 8 : nullptr;
  floatx4 acc[MT], acc2[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    acc[mt] = floatx4{0.f, 0.f, 0.f, 0.f};
    acc2[mt] = floatx4{0.f, 0.f, 0.f, 0.f};
  }
  // the blocks of step s are b_begin + s UB .. ; past the end of the range: a harmless reload of its last block,
  // whose products are skipped
  auto block_of = [&](int s, int b) { return min(b_begin + s * UB + b, b_end - 1); };
  u32x4 wv[UB][4], uv[UB][4];
  auto fetch_w = [&](int s, u32x4 (*w)[4], u32x4 (*u)[4]) {
#pragma unroll
    for (int b = 0; b < UB; ++b) {
      const size_t k = (size_t)block_of(s, b) * 128;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        w[b][j] = *(const u32x4*)(wrow + k + j * 32);
        if (GATED) u[b][j] = *(const u32x4*)(urow + k + j * 32);
      }
    }
  };
  // activation chunk of a step: piece q = tid + 512 i: row q / (16 UB), 16 bytes number q % (16 UB)
  u32x4 areg[PPT];
  auto fetch_a = [&](int s) {
#pragma unroll
    for (int i = 0; i < PPT; ++i) {
      const int q = tid + GS_WAVES * 64 * i;
      const int row = q / (16 * UB), pc = q % (16 * UB);
      areg[i] = u32x4{0u, 0u, 0u, 0u};
      if (q < PIECES && row < M) {
        const int blk = block_of(s, pc >> 4);
        areg[i] = *(const u32x4*)(A + (size_t)row * lda + (size_t)blk * 128 + (pc & 15) * 8);
      }
    }
  };
  auto store_a = [&](int buf) {
#pragma unroll
    for (int i = 0; i < PPT; ++i) {
      const int q = tid + GS_WAVES * 64 * i;
      if (q < PIECES) *(u32x4*)(&As[buf][q / (16 * UB)][(q % (16 * UB)) * 8]) = areg[i];
    }
  };
  if (steps > 0) {
    if (live) fetch_w(0, wv, uv);
    fetch_a(0);
    store_a(0);
  }
  __syncthreads();
  for (int s = 0; s < steps; ++s) {
    const int buf = s & 1;
    u32x4 wn[UB][4], un[UB][4];
    if (s + 1 < steps) {
      if (live) fetch_w(s + 1, wn, un);
      fetch_a(s + 1);
    }
    if (live) {
#pragma unroll
      for (int b = 0; b < UB; ++b) {
        if (b_begin + s * UB + b < b_end) {
#pragma unroll
          for (int j = 0; j < 4; ++j) {
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
              const u32x4 a = *(const u32x4*)(&As[buf][mt * 16 + col][b * 128 + j * 32 + g * 8]);
              acc[mt] = mfma16(a, wv[b][j], acc[mt]);
              if (GATED) acc2[mt] = mfma16(a, uv[b][j], acc2[mt]);
            }
          }
        }
      }
    }
    if (s + 1 < steps) store_a(buf ^ 1);
#pragma unroll
    for (int b = 0; b < UB; ++b)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        wv[b][j] = wn[b][j];
        if (GATED) uv[b][j] = un[b][j];
      }
    __syncthreads();
  }
  if (!live) return;
  const int n = n0 + col;
  if (gridDim.y > 1) {  // partial sums [part][matrix][M][N]; the second kernel applies bias and epilogue
    float* pz = partial + (size_t)blockIdx.y * (GATED ? 2 : 1) * M * N;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int m = mt * 16 + g * 4 + i;
        if (m >= M) continue;
        pz[(size_t)m * N + n] = acc[mt][i];
        if (GATED) pz[(size_t)M * N + (size_t)m * N + n] = acc2[mt][i];
      }
    return;
  }
  float b = 0.f;
  if (bias) b = (bias_dtype == JLLM_BF16) ? ldf((const bf16_t*)bias, n) : ldf((const float*)bias, n);
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int m = mt * 16 + g * 4 + i;
      if (m >= M) continue;
      float v = acc[mt][i] + b;
      if (GATED) v = gate_fn<false>(v) * acc2[mt][i];
      const size_t o = (size_t)m * ldo + n;
      if (epilogue == 1)
        ((float*)out)[o] += v;
      else if (out_dtype == JLLM_BF16)
        stf((bf16_t*)out, o, v);
      else
        stf((float*)out, o, v);
    }
}

// what the reduction needs when an RMSNorm rides on the product (the same two forms as in the kernel for up to 16
// rows): "emit" leaves bf16(new residual * gain) and the sums of squares per 16 columns for the norm that follows,
// "normed" multiplies the sums by rsqrt(sum of the input rows' partial sums of squares / K + eps)
struct StreamNorm {
  bf16_t* emit_rows;
  const void* emit_gain;
  int emit_gain_dtype;
  float* emit_partial;
  const float* norm_partial;
  int norm_parts;
  float norm_eps;
  int K;
};

// adds the K parts in ascending order and applies bias and epilogue; `mats` = 2: gate and up sums side by side.
// One wave per workgroup, V consecutive outputs per lane (4 when rows allow 16-byte accesses): 64 V outputs, which
// lie in one row when a norm form is asked for (N is then a multiple of 256). The kernel is a chain of memory
// latencies, so everything it reads (the norm's partial sums, the residual, up to eight parts at a time) is
// requested before anything is added.
template <int V>
__global__ __launch_bounds__(64) void stream_reduce_kernel(const float* __restrict__ partial, int parts, int mats,
                                                           const void* __restrict__ bias, int bias_dtype,
                                                           void* __restrict__ out, int out_dtype, int ldo, int M, int N,
                                                           int epilogue, StreamNorm nm) {
  typedef float vec_t __attribute__((ext_vector_type(V)));
  const size_t i = ((size_t)blockIdx.x * 64 + threadIdx.x) * V;
  const size_t MN = (size_t)M * N;
  const bool inside = i < MN;  // N is a multiple of V: the V outputs are inside together
  const size_t ic = inside ? i : MN - V;
  const int m = (int)(ic / N), n = (int)(ic % N);
  const size_t o = (size_t)m * ldo + n;
  float t = 0.f;
  if (nm.norm_partial)  // lane l adds the partials l, l + 64, ..., then the wave adds up in a fixed order
    for (int p = threadIdx.x; p < nm.norm_parts; p += 64) t += nm.norm_partial[(size_t)m * nm.norm_parts + p];
  vec_t res = 0.f;
  if (epilogue == 1) res = *(const vec_t*)((const float*)out + o);
  vec_t v = 0.f, u = 0.f;
  const size_t zs = (size_t)mats * MN;
  for (int z0 = 0; z0 < parts; z0 += 8) {
    vec_t pv[8], pu[8];
#pragma unroll
    for (int z = 0; z < 8; ++z) {
      const size_t at = (size_t)min(z0 + z, parts - 1) * zs + ic;
      pv[z] = *(const vec_t*)(partial + at);
      if (mats == 2) pu[z] = *(const vec_t*)(partial + at + MN);
    }
#pragma unroll
    for (int z = 0; z < 8; ++z)
      if (z0 + z < parts) {
        v += pv[z];
        if (mats == 2) u += pu[z];
      }
  }
  float scale = 1.0f;
  if (nm.norm_partial) scale = 1.0f / sqrtf(wave_sum(t) / (float)nm.K + nm.norm_eps);
  v *= scale;
  float r[V];
#pragma unroll
  for (int e = 0; e < V; ++e) {
    float x = v[e];
    if (bias) x += (bias_dtype == JLLM_BF16) ? ldf((const bf16_t*)bias, n + e) : ldf((const float*)bias, n + e);
    if (mats == 2) x = gate_fn<false>(x) * (u[e] * scale);
    r[e] = x;
  }
  if (nm.emit_rows) {  // epilogue 1; the lanes of 16 consecutive columns add their squares (all lanes take part)
    float sq = 0.f;
#pragma unroll
    for (int e = 0; e < V; ++e) {
      r[e] = inside ? res[e] + r[e] : 0.f;
      sq += r[e] * r[e];
    }
    sq += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, sq), 0xB1, 0xF, 0xF, true));
    sq += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, sq), 0x4E, 0xF, 0xF, true));
    if (V == 1) {
      sq += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, sq), 0x141, 0xF, 0xF, true));
      sq += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, sq), 0x140, 0xF, 0xF, true));
    }
    if (!inside) return;
#pragma unroll
    for (int e = 0; e < V; ++e) {
      const float eg = (nm.emit_gain_dtype == JLLM_BF16) ? ldf((const bf16_t*)nm.emit_gain, n + e) : ldf((const float*)nm.emit_gain, n + e);
      ((float*)out)[o + e] = r[e];
      nm.emit_rows[(size_t)m * N + n + e] = f32_to_bf16(r[e] * eg);
    }
    if ((n & 15) == 0) nm.emit_partial[(size_t)m * (N >> 4) + (n >> 4)] = sq;
    return;
  }
  if (!inside) return;
#pragma unroll
  for (int e = 0; e < V; ++e) {
    if (epilogue == 1)
      ((float*)out)[o + e] = res[e] + r[e];
    else if (out_dtype == JLLM_BF16)
      stf((bf16_t*)out, o + e, r[e]);
    else
      stf((float*)out, o + e, r[e]);
  }
}

template <int MT>
static void launch_stream(dim3 grid, hipStream_t stream, const void* A, int lda, const void* W, const void* W2,
                          const void* bias, int bias_dtype, void* out, int out_dtype, int ldo, int M, int N, int K,
                          int epilogue, float* partial, int bpp) {
  const size_t smem_g = (size_t)2 * MT * 16 * (128 + 8) * sizeof(bf16_t), smem_p = (size_t)2 * MT * 16 * (256 + 8) * sizeof(bf16_t);
  static bool configured = false;
  if (!configured) {  // above 64 KB the size has to be allowed first
    (void)hipFuncSetAttribute((const void*)gemm_stream_kernel<MT, true>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem_g);
    (void)hipFuncSetAttribute((const void*)gemm_stream_kernel<MT, false>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem_p);
    configured = true;
  }
  if (W2)
    gemm_stream_kernel<MT, true><<<grid, GS_WAVES * 64, smem_g, stream>>>((const bf16_t*)A, lda, (const bf16_t*)W,
                                                                          (const bf16_t*)W2, bias, bias_dtype, out,
                                                                          out_dtype, ldo, M, N, K, epilogue, partial, bpp);
  else
    gemm_stream_kernel<MT, false><<<grid, GS_WAVES * 64, smem_p, stream>>>((const bf16_t*)A, lda, (const bf16_t*)W,
                                                                           nullptr, bias, bias_dtype, out, out_dtype, ldo,
                                                                           M, N, K, epilogue, partial, bpp);
}

static int stream_checked(const void* A, int lda, const void* W, const void* W2, const void* bias, int bias_dtype,
                          void* out, int out_dtype, int ldo, int M, int N, int K, int epilogue, int parts, float* partial,
                          const StreamNorm& nm, hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (M > 64 || (K & 127) || (N & 15) || (lda & 7) || K <= 0) return 1;
  if (((uintptr_t)A & 15) || ((uintptr_t)W & 15) || (W2 && ((uintptr_t)W2 & 15))) return 1;
  JLLM_TAKE_GATE("gemm_stream", epilogue);
  if (epilogue < 0 || epilogue > 2 || (epilogue == 2) != (W2 != nullptr)) JLLM_FAIL("gemm_stream: epilogue %d", epilogue);
  if (epilogue == 1 && out_dtype != JLLM_F32) JLLM_FAIL("gemm_stream: the accumulate epilogue adds into fp32");
  if (ldo < N) JLLM_FAIL("gemm_stream: ldo %d < N %d", ldo, N);
  const int nblk = K >> 7;
  if (parts < 1) parts = 1;
  if (parts > nblk) parts = nblk;
  if (parts > 1 && !partial) JLLM_FAIL("gemm_stream: %d parts of K need a buffer for the partial sums", parts);
  const int ub = W2 ? 1 : 2;
  int bpp = (nblk + parts - 1) / parts;
  bpp = (bpp + ub - 1) / ub * ub;           // whole steps
  const int used = (nblk + bpp - 1) / bpp;  // parts that have any block
  const bool with_norm = nm.emit_rows || nm.norm_partial;
  if (with_norm) {  // the norm forms live in the reduction kernel, one output row per workgroup
    if (used < 2 || (N & 255)) return 1;
    if (nm.emit_rows && (epilogue != 1 || !nm.emit_gain || !nm.emit_partial)) JLLM_FAIL("gemm_stream: rows for a norm come from the accumulate epilogue, with gain and partial sums");
    if (nm.norm_partial && nm.norm_parts <= 0) JLLM_FAIL("gemm_stream: %d partial sums", nm.norm_parts);
  }
  dim3 grid((N + GS_COLS - 1) / GS_COLS, used);
  if (grid.y > 65535) return 1;
  switch ((M + 15) / 16) {
    case 1: launch_stream<1>(grid, stream, A, lda, W, W2, bias, bias_dtype, out, out_dtype, ldo, M, N, K, epilogue, partial, bpp); break;
    case 2: launch_stream<2>(grid, stream, A, lda, W, W2, bias, bias_dtype, out, out_dtype, ldo, M, N, K, epilogue, partial, bpp); break;
    case 3: launch_stream<3>(grid, stream, A, lda, W, W2, bias, bias_dtype, out, out_dtype, ldo, M, N, K, epilogue, partial, bpp); break;
    default: launch_stream<4>(grid, stream, A, lda, W, W2, bias, bias_dtype, out, out_dtype, ldo, M, N, K, epilogue, partial, bpp); break;
  }
  JLLM_CHECK_LAUNCH("gemm_stream");
  if (used > 1) {
    const size_t total = (size_t)M * N;
    const bool wide = !(N & 3) && !(ldo & 3) && !((uintptr_t)out & 15) && !((uintptr_t)partial & 15);
    if (wide)
      stream_reduce_kernel<4><<<(unsigned)((total / 4 + 63) / 64), 64, 0, stream>>>(partial, used, W2 ? 2 : 1, bias, bias_dtype,
                                                                                  out, out_dtype, ldo, M, N, epilogue, nm);
    else
      stream_reduce_kernel<1><<<(unsigned)((total + 63) / 64), 64, 0, stream>>>(partial, used, W2 ? 2 : 1, bias, bias_dtype,
                                                                              out, out_dtype, ldo, M, N, epilogue, nm);
    JLLM_CHECK_LAUNCH("gemm_stream_reduce");
  }
  return 0;
}

// `parts` > 1 cuts K over gridDim.y; `partial` then holds parts * (W2 ? 2 : 1) * M * N floats.
// returns 0 when it ran, 1 when the shape is not one it takes (the caller uses another kernel), -1 on errors
extern "C" int jllm_gemm_stream_bf16(const void* A, int lda, const void* W, const void* W2, const void* bias,
                                     int bias_dtype, void* out, int out_dtype, int ldo, int M, int N, int K, int epilogue,
                                     int parts, float* partial, hipStream_t stream) {
  return stream_checked(A, lda, W, W2, bias, bias_dtype, out, out_dtype, ldo, M, N, K, epilogue, parts, partial, StreamNorm{},
                        stream);
}

// The same with an RMSNorm on either side (the forms of jllm_gemm_skinny_norm_bf16); needs K in at least two parts
// and N % 256 == 0, declines otherwise.
extern "C" int jllm_gemm_stream_norm_bf16(const void* A, int lda, const void* W, const void* W2, const void* bias,
                                          int bias_dtype, void* out, int out_dtype, int ldo, int M, int N, int K,
                                          int epilogue, int parts, float* partial, void* emit_rows, const void* emit_gain,
                                          int emit_gain_dtype, float* emit_partial, const float* norm_partial,
                                          int norm_parts, float norm_eps, hipStream_t stream) {
  StreamNorm nm{(bf16_t*)emit_rows, emit_gain, emit_gain_dtype, emit_partial, norm_partial, norm_parts, norm_eps, K};
  return stream_checked(A, lda, W, W2, bias, bias_dtype, out, out_dtype, ldo, M, N, K, epilogue, parts, partial, nm, stream);
}
