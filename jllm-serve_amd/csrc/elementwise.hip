// Embedding gather, RMSNorm, and the error channel of the library.
#include <stdarg.h>
#include <string.h>

#include "common.h"

static thread_local char g_error[512] = "";

void jllm_set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
}

extern "C" const char* jllm_last_error() { return g_error; }

extern "C" int jllm_abi_version() { return 5; }

// Compute units of the current GPU, read from the device's properties once per device (0 on errors).
extern "C" int jllm_compute_units() {
  static int cached[64];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 0;
  if (cached[dev] == 0) {
    int n = 0;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) return 0;
    cached[dev] = n;
  }
  return cached[dev];
}

// ---------------------------------------------------------------------------------------------------------
// x[t, :] = scale * E[ids[t], :]   (the residual stream is fp32 whatever the table's type)
template <typename T>
__global__ void embed_kernel(const T* __restrict__ table, const int* __restrict__ ids, float* __restrict__ out,
                             int d, float scale) {
  const int t = blockIdx.x;
  const size_t row = (size_t)ids[t] * d;
  float* o = out + (size_t)t * d;
  for (int i = threadIdx.x; i < d; i += blockDim.x) o[i] = ldf(table, row + i) * scale;
}

extern "C" int jllm_embed(const void* table, int table_dtype, const int* ids, float* out, int n_tokens, int d,
                          float scale, hipStream_t stream) {
  if (n_tokens <= 0) return 0;
  if (d <= 0) JLLM_FAIL("embed: width %d", d);
  JLLM_DISPATCH_1(table_dtype, T, {
    embed_kernel<T><<<n_tokens, 256, 0, stream>>>((const T*)table, ids, out, d, scale);
  })
  JLLM_CHECK_LAUNCH("embed");
  return 0;
}

// ---------------------------------------------------------------------------------------------------------
// RMSNorm of fp32 rows: y = (x * rsqrt(mean(x^2) + eps)) * g. One block per output row; `rows` (optional)
// picks the input row of each output row; output rows lie `ldo` elements apart. Sum of squares, the reciprocal root and both products are fp32.
// Rows of up to 8192 values whose width is a multiple of 4 are read once, 16 bytes per lane, and held in
// registers (every load is in flight at the same time: the kernel is bound by latency, not by bytes);
// other widths take the two-pass loop.
template <typename TG, typename TO>
__global__ __launch_bounds__(256) void rmsnorm_kernel(const float* __restrict__ x, const int* __restrict__ rows,
                                                      const TG* __restrict__ gain, TO* __restrict__ out, int ldo, int d,
                                                      float eps) {
  __shared__ float red[4];
  const int r = blockIdx.x;
  const float* xi = x + (size_t)(rows ? rows[r] : r) * d;
  TO* o = out + (size_t)r * ldo;
  if ((d & 3) == 0 && d <= 8192) {
    const int nv = d >> 2;
    float4 v[8], gn[8];
    float ss = 0.f;
    // the gains are requested together with the row, as 8- or 16-byte loads, so that nothing is waited for twice
    const bool gvec = (((uintptr_t)gain) & 15) == 0;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int i = threadIdx.x + 256 * j;
      v[j] = i < nv ? ((const float4*)xi)[i] : float4{0.f, 0.f, 0.f, 0.f};
      gn[j] = float4{0.f, 0.f, 0.f, 0.f};
      if (i < nv) {
        if (!gvec) {
          gn[j] = float4{ldf(gain, 4 * i), ldf(gain, 4 * i + 1), ldf(gain, 4 * i + 2), ldf(gain, 4 * i + 3)};
        } else if (sizeof(TG) == 2) {
          const uint2 u = ((const uint2*)gain)[i];
          gn[j] = float4{__uint_as_float(u.x << 16), __uint_as_float(u.x & 0xffff0000u), __uint_as_float(u.y << 16),
                         __uint_as_float(u.y & 0xffff0000u)};
        } else {
          gn[j] = ((const float4*)gain)[i];
        }
      }
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) ss += v[j].x * v[j].x + v[j].y * v[j].y + v[j].z * v[j].z + v[j].w * v[j].w;
    ss = block_sum<4>(ss, red);
    const float s = norm_scale(ss, d, eps);
    const bool ovec = (((uintptr_t)o) & 15) == 0;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int i = threadIdx.x + 256 * j;
      if (i < nv) {
        const float a = (v[j].x * s) * gn[j].x, b = (v[j].y * s) * gn[j].y, c = (v[j].z * s) * gn[j].z, e = (v[j].w * s) * gn[j].w;
        if (!ovec) {
          stf(o, 4 * i, a);
          stf(o, 4 * i + 1, b);
          stf(o, 4 * i + 2, c);
          stf(o, 4 * i + 3, e);
        } else if (sizeof(TO) == 2) {
          ((uint2*)o)[i] = uint2{(uint32_t)f32_to_bf16(a).bits | ((uint32_t)f32_to_bf16(b).bits << 16),
                                 (uint32_t)f32_to_bf16(c).bits | ((uint32_t)f32_to_bf16(e).bits << 16)};
        } else {
          ((float4*)o)[i] = float4{a, b, c, e};
        }
      }
    }
    return;
  }
  float ss = 0.f;
  for (int i = threadIdx.x; i < d; i += 256) {
    float v = xi[i];
    ss += v * v;
  }
  ss = block_sum<4>(ss, red);
  const float s = norm_scale(ss, d, eps);
  for (int i = threadIdx.x; i < d; i += 256) stf(o, i, (xi[i] * s) * ldf(gain, i));
}

extern "C" int jllm_rmsnorm(const float* x, const int* rows, int n_rows, int d, const void* gain, int gain_dtype,
                            float eps, void* out, int out_dtype, int ldo, hipStream_t stream) {
  if (n_rows <= 0) return 0;
  if (d <= 0) JLLM_FAIL("rmsnorm: width %d", d);
  if (ldo < d) JLLM_FAIL("rmsnorm: output row stride %d < width %d", ldo, d);
  JLLM_DISPATCH_1(gain_dtype, TG, {
    JLLM_DISPATCH_1(out_dtype, TO, {
      rmsnorm_kernel<TG, TO><<<n_rows, 256, 0, stream>>>(x, rows, (const TG*)gain, (TO*)out, ldo, d, eps);
    })
  })
  JLLM_CHECK_LAUNCH("rmsnorm");
  return 0;
}

// ---------------------------------------------------------------------------------------------------------
// Copies n 32-bit words. The source may be pinned host memory: the step's description (token ids, positions, block
// tables) reaches the device inside the stream of kernels, with no copy engine to start and wait for.
__global__ __launch_bounds__(256) void copy_words_kernel(const uint32_t* __restrict__ src, uint32_t* __restrict__ dst, size_t n) {
  const size_t n4 = n / 4;
  const size_t stride = (size_t)gridDim.x * 256;
  if ((((uintptr_t)src | (uintptr_t)dst) & 15) == 0) {
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n4; i += stride) ((uint4*)dst)[i] = ((const uint4*)src)[i];
    for (size_t i = n4 * 4 + (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += stride) dst[i] = src[i];
  } else {
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += stride) dst[i] = src[i];
  }
}

extern "C" int jllm_copy_words(const void* src, void* dst, long long n_words, hipStream_t stream) {
  if (n_words <= 0) return 0;
  if (((uintptr_t)src & 3) || ((uintptr_t)dst & 3)) JLLM_FAIL("copy_words: pointers must be 4-byte aligned");
  const long long groups = (n_words / 4 + 255) / 256;
  copy_words_kernel<<<(unsigned)(groups < 1 ? 1 : groups > 64 ? 64 : groups), 256, 0, stream>>>((const uint32_t*)src, (uint32_t*)dst,
                                                                                              (size_t)n_words);
  JLLM_CHECK_LAUNCH("copy_words");
  return 0;
}
