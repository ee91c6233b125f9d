// Shared device helpers for the gfx950 kernels: element types, 64-lane wave reductions, error reporting.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

#define JLLM_WAVE 64

// dtype codes shared with the Python side
enum { JLLM_F32 = 0, JLLM_BF16 = 1 };

struct bf16_t {
  uint16_t bits;
};

__device__ __forceinline__ float bf16_to_f32(bf16_t v) { return __uint_as_float(((uint32_t)v.bits) << 16); }

// round to nearest even; NaN stays NaN (quiet)
__device__ __forceinline__ bf16_t f32_to_bf16(float f) {
  uint32_t u = __float_as_uint(f);
  bf16_t r;
  if ((u & 0x7fffffffu) > 0x7f800000u) {
    r.bits = (uint16_t)((u >> 16) | 0x0040u);
    return r;
  }
  uint32_t lsb = (u >> 16) & 1u;
  u += 0x7fffu + lsb;
  r.bits = (uint16_t)(u >> 16);
  return r;
}

__device__ __forceinline__ float ldf(const float* p, size_t i) { return p[i]; }
__device__ __forceinline__ float ldf(const bf16_t* p, size_t i) { return bf16_to_f32(p[i]); }
__device__ __forceinline__ void stf(float* p, size_t i, float v) { p[i] = v; }
__device__ __forceinline__ void stf(bf16_t* p, size_t i, float v) { p[i] = f32_to_bf16(v); }

// what a value becomes when it is stored in T and read back
template <typename T>
__device__ __forceinline__ float round_to(float v);
template <>
__device__ __forceinline__ float round_to<float>(float v) { return v; }
template <>
__device__ __forceinline__ float round_to<bf16_t>(float v) { return bf16_to_f32(f32_to_bf16(v)); }

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = JLLM_WAVE / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, JLLM_WAVE);
  return v;
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = JLLM_WAVE / 2; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, JLLM_WAVE));
  return v;
}

// Sum over a block of NW waves in a fixed order; every thread gets the result. `red` holds NW floats.
template <int NW>
__device__ __forceinline__ float block_sum(float v, float* red) {
  v = wave_sum(v);
  const int lane = threadIdx.x & (JLLM_WAVE - 1);
  const int w = threadIdx.x / JLLM_WAVE;
  __syncthreads();
  if (lane == 0) red[w] = v;
  __syncthreads();
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < NW; ++i) s += red[i];
  return s;
}

// host side -----------------------------------------------------------------------------------------------
void jllm_set_error(const char* fmt, ...);
extern "C" int jllm_compute_units();  // of the current GPU (elementwise.hip)
// sums fp32 partials [splits][M][N] in ascending order of the split, adds the bias, applies the epilogue (gemm_mfma.hip)
int jllm_splitk_reduce(const float* partial, int splits, const void* bias, int bias_dtype, void* out, int out_dtype,
                       int ldo, int M, int N, int epilogue, hipStream_t stream);

#define JLLM_FAIL(...)           \
  do {                           \
    jllm_set_error(__VA_ARGS__); \
    return -1;                   \
  } while (0)

#define JLLM_CHECK_LAUNCH(name)                                               \
  do {                                                                        \
    hipError_t e_ = hipGetLastError();                                        \
    if (e_ != hipSuccess) JLLM_FAIL("%s: launch failed: %s", name, hipGetErrorString(e_)); \
  } while (0)

#define JLLM_DISPATCH_1(code, T, ...)                 \
  if ((code) == JLLM_F32) {                           \
    typedef float T;                                  \
    __VA_ARGS__                                       \
  } else if ((code) == JLLM_BF16) {                   \
    typedef bf16_t T;                                 \
    __VA_ARGS__                                       \
  } else {                                            \
    JLLM_FAIL("unknown dtype code %d", (int)(code));  \
  }
