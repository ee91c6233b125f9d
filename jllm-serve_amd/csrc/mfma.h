// gfx950 matrix-core helpers: operand types and the two bf16 MFMA shapes used by the kernels.
//
// v_mfma_f32_16x16x32_bf16: D[16x16] += A[16x32] * B[32x16]. Lane l holds, of A, row l%16, k (l/16)*8 .. +8;
// of B, column l%16, k (l/16)*8 .. +8; of D, rows (l/16)*4 + i (i = 0..3), column l%16.
// v_mfma_f32_32x32x16_bf16: D[32x32] += A[32x16] * B[16x32]. Lane l holds, of A, row l%32, k (l/32)*8 .. +8;
// of B, column l%32, k (l/32)*8 .. +8; of D, rows 8*(i/4) + (l/32)*4 + i%4 (i = 0..15), column l%32.
// Both operands are read "k-contiguous", which is how activations [rows, K] and weights [N, K] lie in memory.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef float floatx16 __attribute__((ext_vector_type(16)));

typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ floatx16 mfma32(u32x4 a, u32x4 b, floatx16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
}

__device__ __forceinline__ floatx4 mfma16(u32x4 a, u32x4 b, floatx4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
}

// v_mfma_f32_16x16x16_bf16: D[16x16] += A[16x16] * B[16x16]. Lane l holds, of A, row l%16, k (l/16)*4 .. +4; of B,
// column l%16, k (l/16)*4 .. +4; of D, rows (l/16)*4 + i (i = 0..3), column l%16.
__device__ __forceinline__ floatx4 mfma16k16(u32x2 a, u32x2 b, floatx4 c) {
  typedef short short4_t __attribute__((ext_vector_type(4)));
  return __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(short4_t, a), __builtin_bit_cast(short4_t, b), c, 0, 0, 0);
}

// 8 bytes per lane through the transposing LDS load of gfx950 (ds_read_b64_tr_b16): within 16 lanes, lane r names 8
// bytes (a row of four 16-bit values) and lane i receives column i % 4 of the rows i / 4 + 4 e (e = 0..3)
__device__ __forceinline__ u32x2 lds_read_tr16(const void* p) {
  typedef short short4_t __attribute__((ext_vector_type(4)));
  const short4_t v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((short4_t __attribute__((address_space(3)))*)p);
  return __builtin_bit_cast(u32x2, v);
}

// two floats -> two bf16 in one register (round to nearest even; the hardware conversion of gfx950)
__device__ __forceinline__ uint32_t pack_bf16(float a, float b) {
  typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
  typedef float floatx2_t __attribute__((ext_vector_type(2)));
  const bf16x2_t v = __builtin_convertvector(floatx2_t{a, b}, bf16x2_t);
  return __builtin_bit_cast(uint32_t, v);
}

union Pack16 {
  uint4 u;
  bf16x8_t v;
};

__device__ __forceinline__ bf16x8_t as_bf16x8(uint4 u) {
  Pack16 p;
  p.u = u;
  return p.v;
}

__device__ __forceinline__ floatx4 mfma16(uint4 a, uint4 b, floatx4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(a), as_bf16x8(b), c, 0, 0, 0);
}

__device__ __forceinline__ floatx16 mfma32(uint4 a, uint4 b, floatx16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(as_bf16x8(a), as_bf16x8(b), c, 0, 0, 0);
}
