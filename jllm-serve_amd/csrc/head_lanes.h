// A head's values spread over LPK lanes of a wave, 8 consecutive dims (16 bytes of bf16) per lane: what the decode
// attention and the q/k norm + rotation kernels share. LPK is the power of two with LPK * 8 >= head_dim; lanes
// whose dims lie beyond head_dim hold zeros.
#pragma once
#include "common.h"

typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef float floatx2_t __attribute__((ext_vector_type(2)));


__device__ __forceinline__ void unpack8(uint4 v, float* f) {
  f[0] = __uint_as_float(v.x << 16);
  f[1] = __uint_as_float(v.x & 0xffff0000u);
  f[2] = __uint_as_float(v.y << 16);
  f[3] = __uint_as_float(v.y & 0xffff0000u);
  f[4] = __uint_as_float(v.z << 16);
  f[5] = __uint_as_float(v.z & 0xffff0000u);
  f[6] = __uint_as_float(v.w << 16);
  f[7] = __uint_as_float(v.w & 0xffff0000u);
}


// two floats -> two bf16 in one register (round to nearest even; the hardware conversion of gfx950)
__device__ __forceinline__ uint32_t pack2(float a, float b) {
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(floatx2_t{a, b}, bf16x2_t));
}


// sum over the LPK lanes that share a key, left in every one of them; data-parallel-primitive moves inside a
// row of 16 lanes (quad swaps, then mirrors of 8 and 16 lanes), one cross-row exchange for 32
template <int LPK>
__device__ __forceinline__ float group_sum(float d) {
  if (LPK >= 2) d += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, d), 0xB1, 0xF, 0xF, true));
  if (LPK >= 4) d += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, d), 0x4E, 0xF, 0xF, true));
  if (LPK >= 8) d += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, d), 0x141, 0xF, 0xF, true));
  if (LPK >= 16) d += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, d), 0x140, 0xF, 0xF, true));
  if (LPK >= 32) d += __shfl_xor(d, 16, 64);
  return d;
}


// the 8 gains, cosines and sines that belong to this lane's dims, loaded with 16-byte loads ahead of their use
struct LaneAngles {
  float c[8], s[8];
  int src;          // lane that holds the rotation partners of this lane's dims
  bool low, high;   // first / second half of the rotated dims (neither: not rotated)
};

__device__ __forceinline__ void load8(const void* p, int dtype, int at, float* out) {
  if (dtype == JLLM_BF16) {
    const uint4 v = *(const uint4*)((const bf16_t*)p + at);
    out[0] = __uint_as_float(v.x << 16);
    out[1] = __uint_as_float(v.x & 0xffff0000u);
    out[2] = __uint_as_float(v.y << 16);
    out[3] = __uint_as_float(v.y & 0xffff0000u);
    out[4] = __uint_as_float(v.z << 16);
    out[5] = __uint_as_float(v.z & 0xffff0000u);
    out[6] = __uint_as_float(v.w << 16);
    out[7] = __uint_as_float(v.w & 0xffff0000u);
  } else {
    const float4 a = *(const float4*)((const float*)p + at), b = *(const float4*)((const float*)p + at + 4);
    out[0] = a.x, out[1] = a.y, out[2] = a.z, out[3] = a.w, out[4] = b.x, out[5] = b.y, out[6] = b.z, out[7] = b.w;
  }
}

// one head's 8 values of this lane: per-head RMSNorm over the LPK lanes of the group (normed false: none), then the
// rotation by the row's angles; partners (i, i + rot/2) sit rot/16 lanes apart at the same place in the lane
template <int LPK>
__device__ __forceinline__ void norm_rope8(float* x, const float* gain, bool normed, const LaneAngles& an, bool rotate,
                                           float eps, int hd, bool active) {
  if (normed) {
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) ss += x[i] * x[i];
    ss = group_sum<LPK>(ss);
    const float sc = 1.0f / sqrtf(ss / (float)hd + eps);
    if (active) {
#pragma unroll
      for (int i = 0; i < 8; ++i) x[i] = (x[i] * sc) * gain[i];
    }
  }
  if (!rotate) return;
  float other[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) other[i] = __shfl(x[i], an.src, 64);
  if (an.low || an.high) {
#pragma unroll
    for (int i = 0; i < 8; ++i) x[i] = an.low ? x[i] * an.c[i] - other[i] * an.s[i] : x[i] * an.c[i] + other[i] * an.s[i];
  }
}


// --- scores of GP heads (a power of two <= LPK) per key, each a partial sum held by every lane of the group ---------
// Exchanges for the reductions below: with lane ^ 1 and lane ^ 2 inside a quad (DPP), lane ^ 4 (through the LDS
// crossbar), and a rotation by N lanes inside a row of 16 (DPP), which keeps a lane's place in its quad.
template <int X>
__device__ __forceinline__ float xor_lane(float v) {
  if (X == 1) return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1, 0xF, 0xF, true));
  if (X == 2) return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4E, 0xF, 0xF, true));
  return __shfl_xor(v, X, 64);
}
template <int N>
__device__ __forceinline__ float row_rotate(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x120 + N, 0xF, 0xF, true));
}

// Transposing reduction: on entry every lane of a group holds its partial sums a[0 .. GP) for GP heads; on return
// each lane holds the complete sum (over the LPK lanes of the group) of ONE head, head_slot<GP>(sub). Every step
// halves the values a lane carries: of a pair of lanes one keeps the lower half and the other the upper half, and
// each sends the other half across. About half the exchanges of GP separate reductions, and the softmax that
// follows is spread over the lanes instead of being repeated in all of them.
template <int LPK, int GP>
__device__ __forceinline__ float heads_to_lanes(float* a, int sub) {
  static_assert(GP <= LPK && GP <= 8, "one head per lane needs at least as many lanes as heads");
  if (GP >= 2) {
    const bool up = sub & 1;
#pragma unroll
    for (int j = 0; j < GP / 2; ++j) {
      const float send = up ? a[j] : a[j + GP / 2], keep = up ? a[j + GP / 2] : a[j];
      a[j] = keep + xor_lane<1>(send);
    }
  }
  if (GP >= 4) {
    const bool up = sub & 2;
#pragma unroll
    for (int j = 0; j < GP / 4; ++j) {
      const float send = up ? a[j] : a[j + GP / 4], keep = up ? a[j + GP / 4] : a[j];
      a[j] = keep + xor_lane<2>(send);
    }
  }
  if (GP >= 8) {
    const bool up = sub & 4;
    const float send = up ? a[0] : a[1], keep = up ? a[1] : a[0];
    a[0] = keep + xor_lane<4>(send);
  }
  float d = a[0];
  // the lanes that hold the same head: sub + GP, sub + 2 GP, ... (plain sums from here on)
  if (GP == 1) return group_sum<LPK>(d);
  if (GP == 2) {
    if (LPK >= 4) d += xor_lane<2>(d);
    if (LPK >= 8) d += xor_lane<4>(d);
    if (LPK >= 16) d += row_rotate<8>(d);
  } else if (GP == 4) {
    if (LPK == 8) d += xor_lane<4>(d);
    if (LPK >= 16) {
      d += row_rotate<8>(d);
      d += row_rotate<4>(d);
    }
  } else {
    if (LPK >= 16) d += row_rotate<8>(d);
  }
  if (LPK >= 32) d += __shfl_xor(d, 16, 64);
  return d;
}

// which head a lane ends up with: the first step splits by bit 0 of sub into lower / upper half of the heads, the
// second by bit 1 into quarters, the third by bit 2
template <int GP>
__device__ __forceinline__ int head_slot(int sub) {
  int h = 0;
  if (GP >= 2) h += (sub & 1) * (GP / 2);
  if (GP >= 4) h += ((sub >> 1) & 1) * (GP / 4);
  if (GP >= 8) h += ((sub >> 2) & 1);
  return h;
}

// the value that the lane with head `g` holds, in every lane of its block of GP lanes (g known at compile time)
template <int GP, int g>
__device__ __forceinline__ float from_head(float v) {
  // the lane of head g inside a block of GP lanes: the inverse of head_slot
  constexpr int s = (GP >= 2 ? ((g / (GP / 2)) & 1) : 0) + (GP >= 4 ? ((g / (GP / 4)) & 1) * 2 : 0) + (GP >= 8 ? (g & 1) * 4 : 0);
  if (GP == 1) return v;
  if (GP == 2) {  // blocks of two lanes inside a quad: lanes 0,1 take from s, lanes 2,3 from 2 + s
    constexpr int ctrl = s | (s << 2) | ((2 + s) << 4) | ((2 + s) << 6);
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), ctrl, 0xF, 0xF, true));
  }
  if (GP == 4) {
    constexpr int ctrl = s | (s << 2) | (s << 4) | (s << 6);
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), ctrl, 0xF, 0xF, true));
  }
  return __shfl(v, ((threadIdx.x & 63) & ~7) | s, 64);
}
