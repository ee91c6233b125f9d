// Attention of single rows (decode steps) over a paged bf16 cache: bound by reading the keys and values once.
//
// Grid (row, kv head, split). A split is a range of `split` absolute key positions (a power of two, 64 to 512, that
// the caller chooses so that the workgroups of the step just fill the GPU): for one choice, which keys are summed
// together depends only on the row's own position; between choices results differ by rounding. The G query heads of a kv
// head share every key and value that is loaded.
//
// A key's head_dim values are spread over LPK lanes (8 values = 16 bytes per lane), so one wave load covers
// 64/LPK consecutive keys = one contiguous piece of a page. Each group of LPK lanes walks its own keys with
// its own running maximum and sum (four keys in flight), and the groups are merged at the end in a fixed
// order: inside the wave by a butterfly, across the four waves through LDS. A row whose keys lie in one split
// is normalised and written at once; otherwise the split's (max, sum, weighted values) go to a scratch buffer
// and a second kernel merges the splits in ascending order.
//
// The fused form does the whole attention of a decode step in one launch: it takes the projection output
// qkv[t] = [q | k | v] as it comes from the product, normalises and rotates q in registers (every workgroup for
// its own heads), lets the workgroup of a row's last split normalise, rotate and store the new key and copy the
// new value into their page before the keys are read. The splits are merged by the same second kernel. (Merging
// them in the first kernel, by the workgroup that finishes last, was measured: the device-wide fences it needs
// cost far more than the launch it saves.)
//
// Needs bf16, head_dim % 8 == 0, head_dim <= 256, G <= 8 (the fused form: rotary width % 16 == 0); the caller
// falls back to the general kernels otherwise.
#include <math.h>

#include <mutex>
#include <type_traits>

#include "common.h"
#include "head_lanes.h"
#include "mfma.h"
#include "no_alloc.h"

#define DA_MAX_SPLIT 2048  // keys per split: a power of two up to this, chosen by the caller
#define DA_WAVES 4
#define DA_U 4  // keys per group and turn; the packed weighted sum below is written for exactly four

// a.lo * b.lo + a.hi * b.hi + c with a, b holding two bf16 each (v_dot2_f32_bf16: exact products, fp32 sum)
__device__ __forceinline__ float dot2(uint32_t a, uint32_t b, float c) {
  return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, a), __builtin_bit_cast(bf16x2_t, b), c, false);
}

// scores are kept in units of log2(e), so the exponentials are single v_exp_f32 instructions
__device__ __forceinline__ float safe_exp_diff(float a, float m) {
  return a == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(a - m);
}

// merges the splits s_lo..s_hi of one (row, head) in ascending order and writes the normalised output; one wave,
// lane s reads the (max, sum) of split s, so all of them are requested at once
__device__ __forceinline__ void combine_head(const float* part_acc, const float* part_ml, size_t base, int s_lo, int s_hi,
                                             int hd, bf16_t* o, int lane) {
  const int ns = s_hi - s_lo + 1;
  float acc[4] = {0.f, 0.f, 0.f, 0.f};
  if (ns <= 8) {
    // the common case (up to 2,048 keys): every value and every (max, sum) is requested before anything is computed
    float pv[8][4];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const float* pa = part_acc + (base + s_lo + min(j, ns - 1)) * hd;
#pragma unroll
      for (int a = 0; a < 4; ++a) {
        const int d = lane + 64 * a;
        pv[j][a] = d < hd ? pa[d] : 0.f;
      }
    }
    const int s = s_lo + lane;
    const float ms = s <= s_hi ? part_ml[(base + s) * 2] : -INFINITY;
    const float ls = s <= s_hi ? part_ml[(base + s) * 2 + 1] : 0.f;
    const float m = wave_max(ms);
    const float w = s <= s_hi ? __builtin_amdgcn_exp2f(ms - m) : 0.f;
    const float l = wave_sum(ls * w);
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const float wl = __shfl(w, j, 64);
      const float wj = j < ns ? wl : 0.f;
#pragma unroll
      for (int a = 0; a < 4; ++a) acc[a] = fmaf(pv[j][a], wj, acc[a]);
    }
    const float inv = 1.0f / l;
#pragma unroll
    for (int a = 0; a < 4; ++a) {
      const int d = lane + 64 * a;
      if (d < hd) o[d] = f32_to_bf16(acc[a] * inv);
    }
    return;
  }
  float m = -INFINITY;
  for (int c = 0; c < ns; c += 64) {
    const int s = s_lo + c + lane;
    m = fmaxf(m, s <= s_hi ? part_ml[(base + s) * 2] : -INFINITY);
  }
  m = wave_max(m);
  float l = 0.f;
  for (int c = 0; c < ns; c += 64) {  // ascending blocks of 64 splits, ascending inside a block
    const int s = s_lo + c + lane;
    const float w = s <= s_hi ? __builtin_amdgcn_exp2f(part_ml[(base + s) * 2] - m) : 0.f;
    const float lw = s <= s_hi ? part_ml[(base + s) * 2 + 1] * w : 0.f;
    l += wave_sum(lw);
    const int nb = min(64, ns - c);
    for (int j0 = 0; j0 < nb; j0 += 8) {  // eight splits' values are requested before any is used
      float pv[8][4];
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const float* pa = part_acc + (base + s_lo + c + min(j0 + j, nb - 1)) * hd;
#pragma unroll
        for (int a = 0; a < 4; ++a) {
          const int d = lane + 64 * a;
          pv[j][a] = d < hd ? pa[d] : 0.f;
        }
      }
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const float wl = __shfl(w, min(j0 + j, 63), 64);
        const float wj = j0 + j < nb ? wl : 0.f;
#pragma unroll
        for (int a = 0; a < 4; ++a) acc[a] = fmaf(pv[j][a], wj, acc[a]);
      }
    }
  }
  const float inv = 1.0f / l;
#pragma unroll
  for (int a = 0; a < 4; ++a) {
    const int d = lane + 64 * a;
    if (d < hd) o[d] = f32_to_bf16(acc[a] * inv);
  }
}

// what the fused form needs beyond the plain one
struct DecodeFusion {
  const int* slots;       // cache slot of each row's new token, < 0: store nothing
  const float* cos_t;     // [positions][rot / 2], null: no rotation
  const float* sin_t;
  const void* gq;         // gains of the per-head q / k norm (null: no norm), bf16 or fp32
  const void* gk;
  int gain_dtype;
  float eps;
  int rot;                // rotary width
  int write_kv;           // 0: the cache belongs to another layer, which has stored this token already
  bf16_t* kc_w;           // the caches again, writable
  bf16_t* vc_w;
};

template <int LPK, int G, bool FUSED>
__global__ __launch_bounds__(DA_WAVES * 64) __attribute__((amdgpu_waves_per_eu(G <= 4 ? 4 : 1, 8))) void decode_attention_kernel(
    const bf16_t* q, int ldq, const bf16_t* kc, const bf16_t* vc, const int* __restrict__ block_table, int max_blocks,
    const int* __restrict__ row_req, const int* __restrict__ positions, int Hkv, int hd, int page_size, int window,
    float scale, float* part_acc, float* part_ml, int max_splits, int split, bf16_t* out, int ldo, DecodeFusion fu) {
  constexpr int KG = 64 / LPK;         // key groups per wave
  constexpr int NG = DA_WAVES * KG;    // key groups per workgroup
  __shared__ int tb[DA_MAX_SPLIT + 4];
  __shared__ float mrg[DA_WAVES - 1][G][LPK][10];
  const int t = blockIdx.x;
  const int kvh = blockIdx.y;
  const int s = blockIdx.z;
  const int pos = positions[t];
  const int first = window > 0 ? max(0, pos + 1 - window) : 0;
  const int s_lo = first / split, s_hi = pos / split;
  if (s < s_lo || s > s_hi) return;
  const int kb = max(first, s * split);
  const int ke = min(pos, s * split + split - 1);
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int sub = lane % LPK;
  const int grp = wave * KG + lane / LPK;
  const bool active = sub * 8 < hd;
  const int H = Hkv * G;
  // the block-table entries this split touches
  const int* tbl = block_table + (size_t)row_req[t] * max_blocks;
  const int psh = __builtin_ctz(page_size);  // pages hold a power of two of positions: shifts, not divisions
  const int b0 = kb >> psh;
  const int nb = (ke >> psh) - b0 + 1;
  for (int i = threadIdx.x; i < nb; i += DA_WAVES * 64) tb[i] = tbl[b0 + i];
  // everything the prologue needs is requested at once: q, and in the fused form the gains and the row's angles
  uint4 qraw[G];
#pragma unroll
  for (int g = 0; g < G; ++g) {
    qraw[g] = uint4{0u, 0u, 0u, 0u};
    if (active) qraw[g] = *(const uint4*)(q + (size_t)t * ldq + (size_t)(kvh * G + g) * hd + sub * 8);
  }
  LaneAngles an;
  float gq8[8];
  const bool rotate = FUSED && fu.cos_t != nullptr;
  if (FUSED) {
    const int d0 = sub * 8, half = fu.rot >> 1;
    an.low = rotate && d0 < half;
    an.high = rotate && d0 >= half && d0 < fu.rot;
    an.src = lane + (an.low ? (half >> 3) : an.high ? -(half >> 3) : 0);
    if (an.low || an.high) {
      const size_t at = (size_t)pos * half + (an.low ? d0 : d0 - half);
      load8(fu.cos_t, JLLM_F32, at, an.c);
      load8(fu.sin_t, JLLM_F32, at, an.s);
    }
    if (fu.gq && active) load8(fu.gq, fu.gain_dtype, d0, gq8);
  }
  if (FUSED && fu.write_kv && s == s_hi && wave == 0 && lane < LPK) {
    // the new token's key and value go into their page before anyone reads the keys of this split
    const int slot = fu.slots[t];
    if (slot >= 0) {
      const int page = slot >> psh;
      const size_t dst = ((((size_t)page * Hkv + kvh) << psh) + (slot & (page_size - 1))) * hd + sub * 8;
      const bf16_t* kin = q + (size_t)t * ldq + (size_t)(H + kvh) * hd + sub * 8;
      uint4 kv_ = uint4{0u, 0u, 0u, 0u}, vv = uint4{0u, 0u, 0u, 0u};
      float gk8[8];
      if (active) {
        kv_ = *(const uint4*)kin;
        vv = *(const uint4*)(kin + (size_t)Hkv * hd);
        if (fu.gk) load8(fu.gk, fu.gain_dtype, sub * 8, gk8);
      }
      float x[8];
      unpack8(kv_, x);
      norm_rope8<LPK>(x, gk8, fu.gk != nullptr, an, rotate, fu.eps, hd, active);
      if (active) {
        *(uint4*)(fu.kc_w + dst) = uint4{pack2(x[0], x[1]), pack2(x[2], x[3]), pack2(x[4], x[5]), pack2(x[6], x[7])};
        *(uint4*)(fu.vc_w + dst) = vv;
      }
    }
    __threadfence_block();
  }
  // With at least as many lanes per key as heads, each lane keeps the running maximum and sum of ONE head
  // (head_slot of its place in the group) and the scores reach it by a transposing reduction; otherwise every lane
  // keeps them for all heads.
  constexpr int GP = G <= 1 ? 1 : G <= 2 ? 2 : G <= 4 ? 4 : 8;
  constexpr bool DIST = GP >= 2 && GP <= LPK;
  const int my_head = DIST ? head_slot<GP>(sub) : 0;
  float m1 = -INFINITY, l1 = 0.f;  // DIST: of head my_head
  float m[G], l[G], acc[G][8];
#pragma unroll
  for (int g = 0; g < G; ++g) {
    m[g] = -INFINITY;
    l[g] = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[g][i] = 0.f;
  }
  __syncthreads();
  // the keys and values of the next four positions are requested before the current four are used
  uint4 kraw[DA_U], vraw[DA_U];
  auto fetch = [&](int k0, uint4* kr, uint4* vr) {
#pragma unroll
    for (int u = 0; u < DA_U; ++u) {
      const int kj = k0 + u * NG;
      kr[u] = uint4{0u, 0u, 0u, 0u};
      vr[u] = uint4{0u, 0u, 0u, 0u};
      if (kj <= ke && active) {
        const int page = tb[(kj >> psh) - b0];
        const size_t base = ((((size_t)page * Hkv + kvh) << psh) + (kj & (page_size - 1))) * hd + sub * 8;
        kr[u] = *(const uint4*)(kc + base);
        vr[u] = *(const uint4*)(vc + base);
      }
    }
  };
  fetch(kb + grp, kraw, vraw);
  // q stays as four bf16 pairs: the dot products take packed operands. In the fused form it is normalised and
  // rotated in fp32 here, while the first keys are on their way, and rounded to bf16 once, as if it had gone
  // through memory
  uint32_t qp[G][4];
#pragma unroll
  for (int g = 0; g < G; ++g) {
    uint4 v = qraw[g];
    if (FUSED) {
      float x[8];
      unpack8(v, x);
      norm_rope8<LPK>(x, gq8, fu.gq != nullptr, an, rotate, fu.eps, hd, active);
      v = uint4{pack2(x[0], x[1]), pack2(x[2], x[3]), pack2(x[4], x[5]), pack2(x[6], x[7])};
    }
    qp[g][0] = v.x;
    qp[g][1] = v.y;
    qp[g][2] = v.z;
    qp[g][3] = v.w;
  }
  for (int k0 = kb + grp; k0 <= ke; k0 += NG * DA_U) {
    uint4 knext[DA_U], vnext[DA_U];
    fetch(k0 + NG * DA_U, knext, vnext);
    bool valid[DA_U];
#pragma unroll
    for (int u = 0; u < DA_U; ++u) valid[u] = k0 + u * NG <= ke;
    float sc[DA_U][G];
    float sc1[DA_U];  // DIST: the scores of this lane's head
#pragma unroll
    for (int u = 0; u < DA_U; ++u) {
      float part[GP];
#pragma unroll
      for (int g = 0; g < GP; ++g) {
        float d = 0.f;
        if (g < G) {
          d = dot2(qp[g < G ? g : 0][0], kraw[u].x, 0.f);
          d = dot2(qp[g < G ? g : 0][1], kraw[u].y, d);
          d = dot2(qp[g < G ? g : 0][2], kraw[u].z, d);
          d = dot2(qp[g < G ? g : 0][3], kraw[u].w, d);
        }
        part[g] = d;
      }
      if constexpr (DIST) {
        const float d = heads_to_lanes<LPK, GP>(part, sub);
        sc1[u] = (valid[u] && my_head < G) ? d * scale : -INFINITY;
      } else {
#pragma unroll
        for (int g = 0; g < G; ++g) sc[u][g] = valid[u] ? group_sum<LPK>(part[g]) * scale : -INFINITY;
      }
    }
    // values of two keys side by side per dim (v_perm_b32), so that the weighted sum is two packed dot products per
    // dim and head; the weights are rounded to bf16 for it (the running sum l keeps them in fp32)
    uint32_t v01[8], v23[8];
    {
      const uint32_t w0[4] = {vraw[0].x, vraw[0].y, vraw[0].z, vraw[0].w};
      const uint32_t w1[4] = {vraw[1].x, vraw[1].y, vraw[1].z, vraw[1].w};
      const uint32_t w2[4] = {vraw[2].x, vraw[2].y, vraw[2].z, vraw[2].w};
      const uint32_t w3[4] = {vraw[3].x, vraw[3].y, vraw[3].z, vraw[3].w};
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        v01[2 * j] = __builtin_amdgcn_perm(w1[j], w0[j], 0x05040100u);
        v01[2 * j + 1] = __builtin_amdgcn_perm(w1[j], w0[j], 0x07060302u);
        v23[2 * j] = __builtin_amdgcn_perm(w3[j], w2[j], 0x05040100u);
        v23[2 * j + 1] = __builtin_amdgcn_perm(w3[j], w2[j], 0x07060302u);
      }
    }
    if constexpr (DIST) {
      // the softmax step of this lane's head, then its three numbers (rescale, two packed weight pairs) go to all
      // lanes. A lane whose place has no head (G < GP) carries zeros.
      float mn = m1;
#pragma unroll
      for (int u = 0; u < DA_U; ++u) mn = fmaxf(mn, sc1[u]);
      const float alpha1 = safe_exp_diff(m1, mn);  // mn is finite for real heads: a group's first key is valid
      float p[DA_U];
      float ps = 0.f;
#pragma unroll
      for (int u = 0; u < DA_U; ++u) {
        p[u] = safe_exp_diff(sc1[u], mn);
        ps += p[u];
      }
      l1 = l1 * alpha1 + ps;
      m1 = mn;
      const float p01_1 = __uint_as_float(pack2(p[0], p[1])), p23_1 = __uint_as_float(pack2(p[2], p[3]));
      auto head_step = [&](auto gc) {
        constexpr int g = decltype(gc)::value;
        if constexpr (g < G) {
          const float alpha = from_head<GP, g>(alpha1);
          const uint32_t p01 = __float_as_uint(from_head<GP, g>(p01_1)), p23 = __float_as_uint(from_head<GP, g>(p23_1));
#pragma unroll
          for (int i = 0; i < 8; ++i) acc[g][i] = dot2(v23[i], p23, dot2(v01[i], p01, acc[g][i] * alpha));
        }
      };
      head_step(std::integral_constant<int, 0>{});
      head_step(std::integral_constant<int, 1>{});
      head_step(std::integral_constant<int, 2>{});
      head_step(std::integral_constant<int, 3>{});
      head_step(std::integral_constant<int, 4>{});
      head_step(std::integral_constant<int, 5>{});
      head_step(std::integral_constant<int, 6>{});
      head_step(std::integral_constant<int, 7>{});
    } else {
#pragma unroll
    for (int g = 0; g < G; ++g) {
      float mn = m[g];
#pragma unroll
      for (int u = 0; u < DA_U; ++u) mn = fmaxf(mn, sc[u][g]);
      // the first key of a group is always valid, so mn is finite here
      const float alpha = safe_exp_diff(m[g], mn);
      float p[DA_U];
      float ps = 0.f;
#pragma unroll
      for (int u = 0; u < DA_U; ++u) {
        p[u] = safe_exp_diff(sc[u][g], mn);
        ps += p[u];
      }
      l[g] = l[g] * alpha + ps;
      const uint32_t p01 = pack2(p[0], p[1]), p23 = pack2(p[2], p[3]);
#pragma unroll
      for (int i = 0; i < 8; ++i) acc[g][i] = dot2(v23[i], p23, dot2(v01[i], p01, acc[g][i] * alpha));
      m[g] = mn;
    }
    }
#pragma unroll
    for (int u = 0; u < DA_U; ++u) {
      kraw[u] = knext[u];
      vraw[u] = vnext[u];
    }
  }
  if constexpr (DIST) {  // from here on every lane knows the maximum and sum of every head, as in the other form
    auto spread = [&](auto gc) {
      constexpr int g = decltype(gc)::value;
      if constexpr (g < G) {
        m[g] = from_head<GP, g>(m1);
        l[g] = from_head<GP, g>(l1);
      }
    };
    spread(std::integral_constant<int, 0>{});
    spread(std::integral_constant<int, 1>{});
    spread(std::integral_constant<int, 2>{});
    spread(std::integral_constant<int, 3>{});
    spread(std::integral_constant<int, 4>{});
    spread(std::integral_constant<int, 5>{});
    spread(std::integral_constant<int, 6>{});
    spread(std::integral_constant<int, 7>{});
  }
  // merge the key groups of the wave: butterfly over the lanes that hold the same dims
#pragma unroll
  for (int o = LPK; o < 64; o <<= 1) {
#pragma unroll
    for (int g = 0; g < G; ++g) {
      const float om = __shfl_xor(m[g], o, 64);
      const float ol = __shfl_xor(l[g], o, 64);
      const float mn = fmaxf(m[g], om);
      const float a = safe_exp_diff(m[g], mn), b = safe_exp_diff(om, mn);
      l[g] = l[g] * a + ol * b;
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const float oa = __shfl_xor(acc[g][i], o, 64);
        acc[g][i] = acc[g][i] * a + oa * b;
      }
      m[g] = mn;
    }
  }
  // and the waves, in order, through LDS
  if (wave > 0 && lane < LPK) {
#pragma unroll
    for (int g = 0; g < G; ++g) {
      mrg[wave - 1][g][lane][0] = m[g];
      mrg[wave - 1][g][lane][1] = l[g];
#pragma unroll
      for (int i = 0; i < 8; ++i) mrg[wave - 1][g][lane][2 + i] = acc[g][i];
    }
  }
  __syncthreads();
  const bool single = s_lo == s_hi;
  if (wave == 0 && lane < LPK && active) {
#pragma unroll
    for (int g = 0; g < G; ++g) {
#pragma unroll
      for (int w = 0; w < DA_WAVES - 1; ++w) {
        const float om = mrg[w][g][lane][0], ol = mrg[w][g][lane][1];
        const float mn = fmaxf(m[g], om);
        const float a = safe_exp_diff(m[g], mn), b = safe_exp_diff(om, mn);
        l[g] = l[g] * a + ol * b;
#pragma unroll
        for (int i = 0; i < 8; ++i) acc[g][i] = acc[g][i] * a + mrg[w][g][lane][2 + i] * b;
        m[g] = mn;
      }
      const int h = kvh * G + g;
      if (single) {
        const float inv = 1.0f / l[g];
        bf16_t* o = out + (size_t)t * ldo + (size_t)h * hd + sub * 8;
#pragma unroll
        for (int i = 0; i < 8; ++i) o[i] = f32_to_bf16(acc[g][i] * inv);
      } else {
        const size_t pi = ((size_t)t * H + h) * max_splits + s;
        float* pa = part_acc + pi * hd + sub * 8;
#pragma unroll
        for (int i = 0; i < 8; ++i) pa[i] = acc[g][i];
        if (sub == 0) {
          part_ml[pi * 2] = m[g];
          part_ml[pi * 2 + 1] = l[g];
        }
      }
    }
  }
}

// The same for head_dim 128 with the scores on the matrix cores. A wave takes 16 consecutive keys per turn (the
// workgroup 64): S^T[key][head] = K Q^T is four v_mfma_f32_16x16x32_bf16 with K straight from the cache as the A
// operand (lane l: key l%16, dims 32 j + (l/16) 8 .. + 8) and Q as the B operand (column = head; columns beyond G
// are zeros). A lane then holds the scores of keys 4 (l/16) .. + 3 for head l%16: one head per lane, as above.
// The weighted sum is on the matrix cores too: O^T[dim][head] += V^T[dim][key] P^T[key][head], eight
// v_mfma_f32_16x16x16_bf16 per turn. Their B operand (head l%16, keys 4 (l/16) .. + 3) is exactly the lane's four
// probabilities; their A operand, V transposed, comes from a wave-private LDS copy of the turn's values, written
// as it lies in the cache and read with the transposing load ds_read_b64_tr_b16 (lane r of 16 names 8 bytes, lane i
// receives column i % 4 of rows i / 4 + 4 e: lane r names key 4 (l/16) + r / 4, dims 4 (r % 4) .. + 4, and lane i
// receives dim i of the group's four keys). One running maximum per head serves all four key groups of a wave; it
// moves only when a turn's maximum exceeds it by more than 2^8, so the accumulators are rarely rescaled.
template <int G, bool FUSED>
__global__ __launch_bounds__(DA_WAVES * 64) __attribute__((amdgpu_waves_per_eu(1, 3))) void decode_attention_mfma_kernel(
    const bf16_t* q, int ldq, const bf16_t* kc, const bf16_t* vc, const int* __restrict__ block_table, int max_blocks,
    const int* __restrict__ row_req, const int* __restrict__ positions, int Hkv, int page_size, int window, float scale,
    float* part_acc, float* part_ml, int max_splits, int split, bf16_t* out, int ldo, DecodeFusion fu) {
  constexpr int hd = 128, LPK = 16;
  constexpr int VLD = hd + 16;  // row stride of the V copy: 72 words, so the 16 rows of a transposing load spread over the banks
  __shared__ int tb[DA_MAX_SPLIT + 4];
  // the waves' copies of a turn's values during the loop; afterwards, per lane of the waves 1..: maximum, sum, 32 accumulators
  constexpr int VS_BYTES = DA_WAVES * 16 * VLD * 2, MRG_BYTES = (DA_WAVES - 1) * 64 * 34 * 4;
  __shared__ __align__(16) unsigned char pool[VS_BYTES > MRG_BYTES ? VS_BYTES : MRG_BYTES];
  float (*mrg)[64][34] = (float (*)[64][34])pool;
  __shared__ __align__(16) bf16_t qs[G][hd];  // fused form: q after norm and rotation, to be read as the B operand
  const int t = blockIdx.x;
  const int kvh = blockIdx.y;
  const int s = blockIdx.z;
  const int pos = positions[t];
  const int first = window > 0 ? max(0, pos + 1 - window) : 0;
  const int s_lo = first / split, s_hi = pos / split;
  if (s < s_lo || s > s_hi) return;
  const int kb = max(first, s * split);
  const int ke = min(pos, s * split + split - 1);
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int sub = lane & 15, q4 = lane >> 4;
  const int H = Hkv * G;
  const int* tbl = block_table + (size_t)row_req[t] * max_blocks;
  const int psh = __builtin_ctz(page_size);  // pages hold a power of two of positions: shifts, not divisions
  const int b0 = kb >> psh;
  const int nb = (ke >> psh) - b0 + 1;
  for (int i = threadIdx.x; i < nb; i += DA_WAVES * 64) tb[i] = tbl[b0 + i];
  const bf16_t* qrow = q + (size_t)t * ldq + (size_t)kvh * G * hd;
  u32x4 qf[4];  // B operand: head `sub`, dims 32 j + 8 q4 .. + 8
  if (FUSED) {
    // wave 0 prepares q: lane group q4 takes heads q4, q4 + 4, ..; norm and rotation in the 8-dims-per-lane layout
    const bool rotate = fu.cos_t != nullptr;
    if (wave == 0) {
      LaneAngles an;
      float gq8[8];
      const int d0 = sub * 8, half = fu.rot >> 1;
      an.low = rotate && d0 < half;
      an.high = rotate && d0 >= half && d0 < fu.rot;
      an.src = lane + (an.low ? (half >> 3) : an.high ? -(half >> 3) : 0);
      if (an.low || an.high) {
        const size_t at = (size_t)pos * half + (an.low ? d0 : d0 - half);
        load8(fu.cos_t, JLLM_F32, at, an.c);
        load8(fu.sin_t, JLLM_F32, at, an.s);
      }
      if (fu.gq) load8(fu.gq, fu.gain_dtype, d0, gq8);
#pragma unroll
      for (int g0 = 0; g0 < G; g0 += 4) {
        const int g = g0 + q4;
        uint4 v = uint4{0u, 0u, 0u, 0u};
        if (g < G) v = *(const uint4*)(qrow + (size_t)g * hd + d0);
        float x[8];
        unpack8(v, x);
        norm_rope8<LPK>(x, gq8, fu.gq != nullptr, an, rotate, fu.eps, hd, true);
        if (g < G) *(uint4*)(&qs[g][d0]) = uint4{pack2(x[0], x[1]), pack2(x[2], x[3]), pack2(x[4], x[5]), pack2(x[6], x[7])};
      }
      if (fu.write_kv && s == s_hi && q4 == 0) {
        // the new token's key and value go into their page before anyone reads the keys of this split
        const int slot = fu.slots[t];
        if (slot >= 0) {
          const int page = slot >> psh;
          const size_t dst = ((((size_t)page * Hkv + kvh) << psh) + (slot & (page_size - 1))) * hd + d0;
          const bf16_t* kin = q + (size_t)t * ldq + (size_t)(H + kvh) * hd + d0;
          const uint4 kv_ = *(const uint4*)kin;
          const uint4 vv = *(const uint4*)(kin + (size_t)Hkv * hd);
          float gk8[8];
          if (fu.gk) load8(fu.gk, fu.gain_dtype, d0, gk8);
          float x[8];
          unpack8(kv_, x);
          norm_rope8<LPK>(x, gk8, fu.gk != nullptr, an, rotate, fu.eps, hd, true);
          *(uint4*)(fu.kc_w + dst) = uint4{pack2(x[0], x[1]), pack2(x[2], x[3]), pack2(x[4], x[5]), pack2(x[6], x[7])};
          *(uint4*)(fu.vc_w + dst) = vv;
        }
        __threadfence_block();
      }
    }
  } else {
#pragma unroll
    for (int j = 0; j < 4; ++j)
      qf[j] = sub < G ? *(const u32x4*)(qrow + (size_t)sub * hd + j * 32 + q4 * 8) : u32x4{0u, 0u, 0u, 0u};
  }
  floatx4 acc[8];  // O^T: dims 16 j + 4 q4 .. + 3 of head `sub`
#pragma unroll
  for (int j = 0; j < 8; ++j) acc[j] = floatx4{0.f, 0.f, 0.f, 0.f};
  float m1 = -INFINITY, l1 = 0.f;  // of head `sub`: the wave's running maximum, and the sum over this lane's key group
  bf16_t* vw = (bf16_t*)pool + wave * 16 * VLD;
  const bf16_t* v_tr = vw + (4 * q4 + (sub >> 2)) * VLD + 4 * (sub & 3);  // what this lane names in a transposing load
  __syncthreads();
  if (FUSED) {
#pragma unroll
    for (int j = 0; j < 4; ++j)
      qf[j] = sub < G ? *(const u32x4*)(&qs[sub < G ? sub : 0][j * 32 + q4 * 8]) : u32x4{0u, 0u, 0u, 0u};
  }
  // a turn: keys k0 .. k0 + 15 of this wave. K for the scores: key k0 + sub, dims 32 j + 8 q4; V for the sums: key
  // k0 + 4 q4 + u, dims 8 sub. The next turn's are requested before this turn's are used.
  struct Turn {
    u32x4 k[4];
    uint4 v[4];
  };
  const bool one_page = page_size >= 4 && (kb & 3) == 0;
  // keys beyond the end of the range are read as the last key of the range (a valid one): no branches and nothing to
  // clear; their scores are masked below and their probabilities are zero
  auto fetch = [&](int k0, Turn& tn) {
    const int kk = min(k0 + sub, ke);
    {
      const int page = tb[(kk >> psh) - b0];
      const bf16_t* kp = kc + ((((size_t)page * Hkv + kvh) << psh) + (kk & (page_size - 1))) * hd + q4 * 8;
#pragma unroll
      for (int j = 0; j < 4; ++j) tn.k[j] = *(const u32x4*)(kp + j * 32);
    }
    if (one_page) {  // the lane's four keys start at a multiple of four and pages hold at least four: one table entry
      const int kv0 = k0 + 4 * q4;
      const int page = tb[(min(kv0, ke) >> psh) - b0];
      const bf16_t* vp = vc + (((size_t)page * Hkv + kvh) << psh) * hd + sub * 8;
#pragma unroll
      for (int u = 0; u < 4; ++u) tn.v[u] = *(const uint4*)(vp + (size_t)(min(kv0 + u, ke) & (page_size - 1)) * hd);
    } else {
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int kv = min(k0 + 4 * q4 + u, ke);
        const int page = tb[(kv >> psh) - b0];
        tn.v[u] = *(const uint4*)(vc + ((((size_t)page * Hkv + kvh) << psh) + (kv & (page_size - 1))) * hd + sub * 8);
      }
    }
  };
  const int k_first = kb + wave * 16;
  auto turn = [&](int k0, const Turn& tn) {
    floatx4 sc = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int j = 0; j < 4; ++j) sc = mfma16(tn.k[j], qf[j], sc);
    float z[4];
    float mx = -INFINITY;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      z[i] = (k0 + 4 * q4 + i <= ke && sub < G) ? sc[i] * scale : -INFINITY;
      mx = fmaxf(mx, z[i]);
    }
    mx = fmaxf(mx, __shfl_xor(mx, 16, 64));  // over the four key groups: the head's maximum in this turn
    mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
    if (mx > m1 + 8.0f) {  // also the first turn with a visible key (m1 = -inf)
      const float alpha = safe_exp_diff(m1, mx);
      l1 *= alpha;
#pragma unroll
      for (int j = 0; j < 8; ++j) acc[j] *= alpha;
      m1 = mx;
    }
    float p[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      p[i] = safe_exp_diff(z[i], m1);  // m1 = -inf only while every key so far was beyond the end: then z is too
      l1 += p[i];
    }
    const u32x2 pb = u32x2{pack2(p[0], p[1]), pack2(p[2], p[3])};
    // the turn's values as they lie in the cache: key 4 q4 + u, dims 8 sub .. + 7; the wave's own LDS region, and
    // LDS operations of one wave complete in order, so no barrier stands between the turns
#pragma unroll
    for (int u = 0; u < 4; ++u) *(uint4*)(vw + (4 * q4 + u) * VLD + sub * 8) = tn.v[u];
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[j] = mfma16k16(lds_read_tr16(v_tr + 16 * j), pb, acc[j]);
  };
  // two sets of registers take turns: while one turn is computed the next one's keys and values arrive in the other
  Turn ta, tb2;
  fetch(k_first, ta);
  for (int k0 = k_first; k0 <= ke; k0 += 2 * DA_WAVES * 16) {
    fetch(k0 + DA_WAVES * 16, tb2);
    turn(k0, ta);
    if (k0 + DA_WAVES * 16 > ke) break;
    fetch(k0 + 2 * DA_WAVES * 16, ta);
    turn(k0 + DA_WAVES * 16, tb2);
  }
  // the sum over the four key groups; then the waves merge, in order, through LDS
  l1 += __shfl_xor(l1, 16, 64);
  l1 += __shfl_xor(l1, 32, 64);
  __syncthreads();  // every wave is done with its copy of the values: the memory now carries the merge
  if (wave > 0) {
    float* dst = &mrg[wave - 1][lane][0];
    dst[0] = m1;
    dst[1] = l1;
#pragma unroll
    for (int j = 0; j < 8; ++j)
#pragma unroll
      for (int i = 0; i < 4; ++i) dst[2 + 4 * j + i] = acc[j][i];
  }
  __syncthreads();
  const bool single = s_lo == s_hi;
  if (wave == 0 && sub < G) {
#pragma unroll
    for (int w = 0; w < DA_WAVES - 1; ++w) {
      const float* src = &mrg[w][lane][0];
      const float om = src[0], ol = src[1];
      const float mn = fmaxf(m1, om);
      const float a = safe_exp_diff(m1, mn), b = safe_exp_diff(om, mn);
      l1 = l1 * a + ol * b;
#pragma unroll
      for (int j = 0; j < 8; ++j)
#pragma unroll
        for (int i = 0; i < 4; ++i) acc[j][i] = acc[j][i] * a + src[2 + 4 * j + i] * b;
      m1 = mn;
    }
    const int h = kvh * G + sub;
    if (single) {
      const float inv = 1.0f / l1;
      bf16_t* o = out + (size_t)t * ldo + (size_t)h * hd + 4 * q4;
#pragma unroll
      for (int j = 0; j < 8; ++j)
        *(u32x2*)(o + 16 * j) = u32x2{pack2(acc[j][0] * inv, acc[j][1] * inv), pack2(acc[j][2] * inv, acc[j][3] * inv)};
    } else {
      const size_t pi = ((size_t)t * H + h) * max_splits + s;
      float* pa = part_acc + pi * hd + 4 * q4;
#pragma unroll
      for (int j = 0; j < 8; ++j) *(floatx4*)(pa + 16 * j) = acc[j];
      if (q4 == 0) {
        part_ml[pi * 2] = m1;
        part_ml[pi * 2 + 1] = l1;
      }
    }
  }
}

// rows that had a single split were written by the first kernel; one wave per (row, head)
__global__ __launch_bounds__(64) void decode_attention_combine_kernel(const float* __restrict__ part_acc,
                                                                      const float* __restrict__ part_ml,
                                                                      const int* __restrict__ positions, int H, int hd,
                                                                      int window, int max_splits, int split,
                                                                      bf16_t* __restrict__ out, int ldo) {
  const int t = blockIdx.x;
  const int h = blockIdx.y;
  const int pos = positions[t];
  const int first = window > 0 ? max(0, pos + 1 - window) : 0;
  const int s_lo = first / split, s_hi = pos / split;
  if (s_lo == s_hi) return;
  combine_head(part_acc, part_ml, ((size_t)t * H + h) * max_splits, s_lo, s_hi, hd, out + (size_t)t * ldo + (size_t)h * hd,
               threadIdx.x);
}

template <int LPK, bool FUSED>
static int launch_decode(int G, dim3 grid, hipStream_t st, const bf16_t* q, int ldq, const bf16_t* kc, const bf16_t* vc,
                         const int* bt, int mb, const int* rr, const int* ps, int Hkv, int hd, int page, int window,
                         float scale, float* pa, float* pm, int ms, int split, bf16_t* out, int ldo, const DecodeFusion& fu) {
#define DA_CASE(GG)                                                                                              \
  case GG:                                                                                                       \
    decode_attention_kernel<LPK, GG, FUSED><<<grid, DA_WAVES * 64, 0, st>>>(q, ldq, kc, vc, bt, mb, rr, ps, Hkv, \
                                                                            hd, page, window, scale, pa, pm, ms, \
                                                                            split, out, ldo, fu);                \
    return 0;
  switch (G) {
    DA_CASE(1) DA_CASE(2) DA_CASE(3) DA_CASE(4) DA_CASE(5) DA_CASE(6) DA_CASE(7) DA_CASE(8)
    default: return 1;
  }
#undef DA_CASE
}

template <bool FUSED>
static int decode_attention(const void* q, int ldq, void* out, int ldo, const void* kcache, const void* vcache,
                            const int* block_table, int max_blocks, const int* row_req, const int* positions, int n_rows,
                            int H, int Hkv, int hd, int page_size, int window, float scale, int max_pos, float* part_acc,
                            float* part_ml, int max_splits, int split, const DecodeFusion& fu, hipStream_t stream) {
  if (n_rows <= 0) return 0;
  if (Hkv <= 0 || H % Hkv != 0) JLLM_FAIL("decode attention: %d query heads over %d kv heads", H, Hkv);
  const int G = H / Hkv;
  if (G > 8 || (hd & 7) || hd > 256 || hd < 8 || (ldq & 7) || ((uintptr_t)q & 15)) return 1;
  if (page_size <= 0 || (page_size & (page_size - 1))) return 1;
  if (Hkv > 65535 || max_splits > 65535) return 1;
  if (split < 16 || split > DA_MAX_SPLIT || (split & (split - 1))) JLLM_FAIL("decode attention: split of %d keys", split);
  if (max_splits < max_pos / split + 1) JLLM_FAIL("decode attention: %d splits for positions up to %d", max_splits, max_pos);
  if (ldo < H * hd) JLLM_FAIL("decode attention: output stride %d < %d", ldo, H * hd);
  int lpk = 2;
  while (lpk * 8 < hd) lpk <<= 1;
  const int used = max_pos / split + 1;
  dim3 grid(n_rows, Hkv, used);
  int rc;
#define DA_ARGS G, grid, stream, (const bf16_t*)q, ldq, (const bf16_t*)kcache, (const bf16_t*)vcache, block_table,    \
                max_blocks, row_req, positions, Hkv, hd, page_size, window, scale * 1.4426950408889634f, part_acc,  \
                part_ml, max_splits, split, (bf16_t*)out, ldo, fu
  if (hd == 128) {
#define DA_MCASE(GG)                                                                                                    \
  case GG:                                                                                                              \
    decode_attention_mfma_kernel<GG, FUSED><<<grid, DA_WAVES * 64, 0, stream>>>(                                        \
        (const bf16_t*)q, ldq, (const bf16_t*)kcache, (const bf16_t*)vcache, block_table, max_blocks, row_req, positions, \
        Hkv, page_size, window, scale * 1.4426950408889634f, part_acc, part_ml, max_splits, split, (bf16_t*)out, ldo, fu); \
    break;
    switch (G) {
      DA_MCASE(1) DA_MCASE(2) DA_MCASE(3) DA_MCASE(4) DA_MCASE(5) DA_MCASE(6) DA_MCASE(7) DA_MCASE(8)
    }
#undef DA_MCASE
    rc = 0;
  } else
  switch (lpk) {
    case 2: rc = launch_decode<2, FUSED>(DA_ARGS); break;
    case 4: rc = launch_decode<4, FUSED>(DA_ARGS); break;
    case 8: rc = launch_decode<8, FUSED>(DA_ARGS); break;
    case 16: rc = launch_decode<16, FUSED>(DA_ARGS); break;
    default: rc = launch_decode<32, FUSED>(DA_ARGS); break;
  }
#undef DA_ARGS
  if (rc != 0) return rc;
  JLLM_CHECK_LAUNCH("decode_attention");
  if (used > 1) {
    dim3 cg(n_rows, H);
    decode_attention_combine_kernel<<<cg, 64, 0, stream>>>(part_acc, part_ml, positions, H, hd, window, max_splits, split,
                                                           (bf16_t*)out, ldo);
    JLLM_CHECK_LAUNCH("decode_attention_combine");
  }
  return 0;
}

// scratch: part_acc needs n_rows * H * max_splits * hd floats, part_ml n_rows * H * max_splits * 2 floats, where
// max_splits counts from split 0: max_pos / split + 1.
// returns 0 when it ran, 1 when the shape is not one it takes, -1 on errors
extern "C" int jllm_decode_attention_bf16(const void* q, int ldq, void* out, int ldo, const void* kcache,
                                          const void* vcache, const int* block_table, int max_blocks,
                                          const int* row_req, const int* positions, int n_rows, int H, int Hkv, int hd,
                                          int page_size, int window, float scale, int max_pos, float* part_acc,
                                          float* part_ml, int max_splits, int split, hipStream_t stream) {
  return decode_attention<false>(q, ldq, out, ldo, kcache, vcache, block_table, max_blocks, row_req, positions, n_rows, H,
                                 Hkv, hd, page_size, window, scale, max_pos, part_acc, part_ml, max_splits, split,
                                 DecodeFusion{}, stream);
}

// The whole attention of a decode step from the projection output qkv [rows, (H + 2 Hkv) * hd]: q/k norm (gains
// null: none), rotation (tables null: none), store of the new key and value at `slots` (write_kv = 0: not stored),
// attention over the pages, merge of the splits.
extern "C" int jllm_decode_attention_fused_bf16(const void* qkv, int ldqkv, void* out, int ldo, void* kcache,
                                                void* vcache, const int* block_table, int max_blocks,
                                                const int* row_req, const int* positions, const int* slots,
                                                const float* cos_t, const float* sin_t, const void* gq, const void* gk,
                                                int gain_dtype, float eps, int rot, int write_kv, int n_rows, int H,
                                                int Hkv, int hd, int page_size, int window, float scale, int max_pos,
                                                float* part_acc, float* part_ml, int max_splits, int split,
                                                hipStream_t stream) {
  if ((cos_t == nullptr) != (sin_t == nullptr)) JLLM_FAIL("decode attention: cos and sin tables come together");
  if ((gq == nullptr) != (gk == nullptr)) JLLM_FAIL("decode attention: q and k gains come together");
  if (cos_t && (rot < 16 || rot > hd || (rot & 15))) return 1;
  if (ldqkv < (H + 2 * Hkv) * hd) JLLM_FAIL("decode attention: row stride %d < %d", ldqkv, (H + 2 * Hkv) * hd);
  if (write_kv && !slots) JLLM_FAIL("decode attention: cache write without slots");
  if (((uintptr_t)gq & 15) || ((uintptr_t)gk & 15)) return 1;
  DecodeFusion fu{slots, cos_t, sin_t, gq, gk, gain_dtype, eps, rot, write_kv, (bf16_t*)kcache, (bf16_t*)vcache};
  return decode_attention<true>(qkv, ldqkv, out, ldo, kcache, vcache, block_table, max_blocks, row_req, positions, n_rows,
                                H, Hkv, hd, page_size, window, scale, max_pos, part_acc, part_ml, max_splits, split, fu,
                                stream);
}

// ---------------------------------------------------------------------------------------- without allocation
// The scratch of the split keys inside the library's device image (no_alloc.h). On the host `scratch` is only a
// stand-in for the symbol: the address that kernels and copies may use is looked up per GPU and kept.
static __device__ __align__(256) float scratch[JLLM_NO_ALLOC_SCRATCH_FLOATS];

#define JLLM_MAX_DEVICES 64
static float* g_scratch_ptr[JLLM_MAX_DEVICES];
static std::mutex g_scratch_lock;

static int scratch_of_current_device(float** ptr) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) JLLM_FAIL("no-alloc decode attention: hipGetDevice: %s", hipGetErrorString(e));
  if (dev < 0 || dev >= JLLM_MAX_DEVICES) JLLM_FAIL("no-alloc decode attention: device %d is beyond the %d it keeps addresses for", dev, JLLM_MAX_DEVICES);
  std::lock_guard<std::mutex> hold(g_scratch_lock);
  if (g_scratch_ptr[dev] == nullptr) {
    float* p = nullptr;
    e = hipGetSymbolAddress((void**)&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || p == nullptr)
      JLLM_FAIL("no-alloc decode attention: hipGetSymbolAddress on device %d: %s", dev, hipGetErrorString(e));
    g_scratch_ptr[dev] = p;
  }
  *ptr = g_scratch_ptr[dev];
  return 0;
}

extern "C" int jllm_decode_attention_bf16_no_alloc(const void* q, int ldq, void* out, int ldo, const void* kcache,
                                                   const void* vcache, const int* block_table, int max_blocks,
                                                   const int* row_req, const int* positions, int n_rows, int H,
                                                   int Hkv, int hd, int page_size, int window, float scale,
                                                   int max_pos, int split, hipStream_t stream) {
  if (n_rows <= 0) return 0;
  if (H <= 0 || hd <= 0 || max_pos < 0) JLLM_FAIL("no-alloc decode attention: %d heads of %d, positions up to %d", H, hd, max_pos);
  if (split < 16 || split > DA_MAX_SPLIT || (split & (split - 1))) JLLM_FAIL("decode attention: split of %d keys", split);
  const size_t max_splits = (size_t)max_pos / split + 1;
  const size_t entries = (size_t)n_rows * H * max_splits;  // (row, head, split) triples
  const size_t acc_floats = (entries * hd + 63) / 64 * 64;  // the (max, sum) pairs start on a 256-byte boundary
  const size_t need = acc_floats + entries * 2;
  if (need > (size_t)JLLM_NO_ALLOC_SCRATCH_FLOATS)
    JLLM_FAIL("no-alloc decode attention: %d rows x %d heads x %zu splits of head size %d need %zu floats of scratch, the "
              "library holds %u; use jllm_decode_attention_bf16 with a scratch of the caller's",
              n_rows, H, max_splits, hd, need, (unsigned)JLLM_NO_ALLOC_SCRATCH_FLOATS);
  float* base = nullptr;
  if (scratch_of_current_device(&base) != 0) return -1;
  return decode_attention<false>(q, ldq, out, ldo, kcache, vcache, block_table, max_blocks, row_req, positions, n_rows, H,
                                 Hkv, hd, page_size, window, scale, max_pos, base, base + acc_floats, (int)max_splits, split,
                                 DecodeFusion{}, stream);
}
