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

// The gate function of the gated epilogue, out = gate(a . Wg) * (a . Wu), has a code that rides in bits 8 and up of an
// entry point's `epilogue` argument (bits 0..7: 0 store, 1 add into fp32, 2 gated). One gate function is built:
// code 0, SiLU, z / (1 + exp(-z)) (cpu/VectorKernels.java:637-639 of the reference). Every product kernel applies
// gate_fn below and every entry point takes its argument apart with JLLM_TAKE_GATE, which refuses a code that is not
// built with a message; another gate function is a case in gate_fn, a larger JLLM_GATE_COUNT, and the code handed
// on to the kernels.
#define JLLM_GATE_SILU 0
#define JLLM_GATE_COUNT 1
#define JLLM_TAKE_GATE(name, epilogue)                                                                       \
  do {                                                                                                       \
    const int gate_ = (epilogue) >> 8;                                                                       \
    (epilogue) &= 0xff;                                                                                      \
    if (gate_ < 0 || gate_ >= JLLM_GATE_COUNT)                                                               \
      JLLM_FAIL("%s: gate function %d of the gated epilogue is not built (0 = silu is)", name, gate_);        \
    if (gate_ != 0 && (epilogue) != 2) JLLM_FAIL("%s: a gate function without the gated epilogue", name);    \
  } while (0)
// FAST: the hardware's exp2 and reciprocal (where the result is rounded to bf16 or added in fp32 anyway)
template <bool FAST>
__device__ __forceinline__ float gate_fn(float z) {
  if (FAST) return z * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.4426950408889634f * z));
  return z / (1.0f + expf(-z));
}

// The scale of an RMSNorm from a row's sum of squares: the mean and the sum with eps in fp32, the inverse square root in
// double, rounded once to fp32 (cpu/VectorKernels.java:630-632 of the reference: (float)(1.0 / Math.sqrt(ss / n + eps))).
// The general kernels, which are the whole of a float32 run, use it; the bf16 matrix-core kernels keep an fp32 1/sqrt,
// which differs by at most one unit in the last place.
__device__ __forceinline__ float norm_scale(float ss, int n, float eps) {
  return (float)(1.0 / sqrt((double)(ss / (float)n + eps)));
}

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
