// Causal attention of prompt portions over a paged bf16 cache on the matrix cores (flash style: no score matrix
// in memory, running maximum and sum in fp32).
//
// Grid (query head, tile): the heads of a tile are neighbours in the order of dispatch, and the caller lists the
// tiles with the most keys first, so that the long ones start first and the short ones fill the gaps. A tile is up to 128 consecutive rows of one request (4 waves x 32 rows); the host lists
// the tiles as (request, first row, rows, position of the first row). Keys are walked in blocks of 64 aligned to
// absolute positions. Per block the workgroup stages K and V as they lie ([key][dim]) in LDS (two buffers: the
// next block's global loads are in flight while the current one is multiplied); positions outside the tile's
// visible range are stored as zeros and their table entries are never read.
//
// Each wave computes the TRANSPOSED scores S^T[key][row] = K Q^T (v_mfma_f32_32x32x16_bf16, A = K from LDS,
// B = Q held in registers), so a lane owns one query row: the row maximum and sum are in-lane reductions plus
// one exchange between the two half-waves, and the rescale of the output is a per-lane scalar. The
// probabilities, rounded to bf16, are already laid out as the B operand of O^T[dim][row] += V^T P^T: the k slots
// of that product are assigned to keys in the order the score accumulators hold them, and the A operand V^T is
// read in the same order with the transposing LDS load of gfx950 (ds_read_b64_tr_b16): within 16 lanes, lane r
// names 8 bytes (4 dims) and lane i receives, of the 16 x 4 elements named, column i % 4 of rows i / 4 + 4 e
// (e = 0..3). Lane r therefore names key r / 4, dims 4 (r % 4) .. + 4, and lane i receives dim i of keys 0..3.
//
// A step with few tiles (all workgroups resident at once, two per compute unit) waits for the tile with the most
// keys. For such steps, with head sizes up to 128, a workgroup has two such groups of four waves (NG = 2) for the
// same 128 rows: the first takes the first half of the tile's key blocks, the second the rest, each through LDS
// buffers of its own, and at the end the second group hands its maxima, sums and outputs to the first through LDS
// (its state is merged behind the first group's, always in that order). A tile's longest chain of blocks is then
// half as long, one workgroup fills a compute unit (8 waves, 152 KB of LDS at head size 128), and with the tiles
// listed longest first a unit that gets a long tile takes a short one afterwards. Measured at 32 heads: one
// 2,048-token prompt 85 -> 70 us, one of 1,024 tokens 42 -> 32; from two 2,048-token prompts on (or 40 heads) the
// one-group form is faster (115 against 139 us): two independent workgroups on a unit overlap better than one whose
// eight waves meet at a barrier after every block.
//
// Head size 128 has a third form further down (prefill_attention_turns_kernel): two groups that take turns at the
// matrix cores, keys and values loaded straight into LDS; the entry point says when it is taken.
//
// Needs bf16, head_dim a multiple of 16 up to 128, or 192; the caller falls back to the general kernel otherwise.
#include <math.h>

#include "common.h"
#include "mfma.h"

#define PA_ROWS 128
#define PA_KEYS 64


template <int HD16, int NG>
__global__ __launch_bounds__(256 * NG, NG == 1 ? 2 : 1) void prefill_attention_kernel(
    const bf16_t* __restrict__ q, int ldq, bf16_t* __restrict__ out, int ldo, const bf16_t* __restrict__ kc,
    const bf16_t* __restrict__ vc, const int* __restrict__ block_table, int max_blocks, const int* __restrict__ tiles,
    int H, int Hkv, int page_shift, int window, float scale_log2e) {
  constexpr int HD = HD16 * 16;
  constexpr int DB = (HD + 31) / 32;
  constexpr int HDP = DB * 32;
  constexpr int KLD = HD + 8;
  // rows of V are 16 words apart (mod 64 banks) where the head size allows it: the four keys that 32 lanes read
  // at once then fall into different banks; K rows are 4 words apart for its 16-byte reads of 16 keys
  constexpr int VLD = HD + 32;
  constexpr int KSZ = PA_KEYS * KLD;  // elements of one K buffer
  constexpr int VSZ = PA_KEYS * VLD;
  constexpr int NCH = (PA_KEYS * HD16 * 2 + 255) / 256;  // 16-byte pieces of K (and of V) per thread and block
  extern __shared__ __align__(16) unsigned char smem_raw[];
  // (the wave's number is the same in all its lanes: said so, what follows from it stays in scalar registers and a
  // branch on it is a jump instead of a lane mask)
  const int grp = NG > 1 ? __builtin_amdgcn_readfirstlane((int)threadIdx.x >> 8) : 0;  // key group: four waves with their own buffers
  bf16_t* Ks = (bf16_t*)smem_raw + (size_t)grp * 2 * (KSZ + VSZ);  // [2][KSZ]
  bf16_t* Vs = Ks + 2 * KSZ;                                       // [2][VSZ]
  const int* tile = tiles + (size_t)blockIdx.y * 4;
  const int req = tile[0], row0 = tile[1], nrows = tile[2], pos0 = tile[3];
  const int h = blockIdx.x;
  const int kvh = h / (H / Hkv);
  const int tid = threadIdx.x & 255;  // within the group
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
  const int qi = lane & 31, half = lane >> 5;
  const int wq = wave * 32 + qi;
  const int pos_q = pos0 + min(wq, nrows - 1);
  const int first_q = window > 0 ? max(0, pos_q + 1 - window) : 0;
  const int* tbl = block_table + (size_t)req * max_blocks;
  const int k_lo = window > 0 ? max(0, pos0 + 1 - window) : 0;  // oldest key any row of the tile sees
  const int k_hi = pos0 + nrows - 1;
  const int wave_lo_pos = pos0 + min(nrows - 1, wave * 32);        // position of this wave's first row
  const int wave_hi = pos0 + min(nrows - 1, wave * 32 + 31);       // newest key this wave needs
  const int wave_first = window > 0 ? max(0, wave_hi + 1 - window) : 0;  // oldest key its last row sees
  const bool wave_on = wave * 32 < nrows;
  // Q as the B operand: lane holds Q[row][ks * 16 + half * 8 .. + 8]
  u32x4 qf[HD16];
  {
    const bf16_t* qr = q + (size_t)(row0 + min(wq, nrows - 1)) * ldq + (size_t)h * HD + half * 8;
#pragma unroll
    for (int ks = 0; ks < HD16; ++ks) qf[ks] = *(const u32x4*)(qr + ks * 16);
  }
  if (HD != HDP) {  // dims beyond head_dim are read with the last 32-dim block: they stay zero in both buffers
    for (int i = tid; i < 2 * VSZ; i += 256) Vs[i].bits = 0;
    __syncthreads();
  }
  // this group's blocks: the tile's blocks of 64 keys cut into NG runs of equal length (the last may be shorter)
  const int kt_tile = (k_lo / PA_KEYS) * PA_KEYS;
  const int n_blocks = (k_hi - kt_tile) / PA_KEYS + 1;
  const int per_group = (n_blocks + NG - 1) / NG;
  const int kt_first = kt_tile + grp * per_group * PA_KEYS;
  const int kt_last = min(k_hi, kt_first + per_group * PA_KEYS - 1);  // newest key of the group's run (< kt_first: none)
  // staging: this thread's pieces of a block: piece c = tid + 256 j: key c / (HD16*2), 16 bytes number c % (HD16*2)
  u32x4 kreg[NCH], vreg[NCH];
  // The table entries of a block are requested one block before its keys and values (-1: nothing to read), so that
  // the loads of a block do not wait for a table entry first: two latencies in a row are more than a block's products.
  int pg[NCH];
  auto load_pages = [&](int kt) {
#pragma unroll
    for (int j = 0; j < NCH; ++j) {
      const int c = tid + 256 * j;
      const int kabs = kt + c / (HD16 * 2);
      pg[j] = (c < PA_KEYS * HD16 * 2 && kabs >= k_lo && kabs <= kt_last) ? tbl[kabs >> page_shift] : -1;
    }
  };
  auto load_block = [&](int kt) {  // with the entries that load_pages(kt) left in pg
#pragma unroll
    for (int j = 0; j < NCH; ++j) {
      const int c = tid + 256 * j;
      const int key = c / (HD16 * 2), pc = c % (HD16 * 2);
      const int kabs = kt + key;
      kreg[j] = u32x4{0u, 0u, 0u, 0u};
      vreg[j] = u32x4{0u, 0u, 0u, 0u};
      if (pg[j] >= 0) {  // pages hold a power of two of positions
        const size_t base = ((((size_t)pg[j] * Hkv + kvh) << page_shift) + (kabs & ((1 << page_shift) - 1))) * HD + pc * 8;
        kreg[j] = *(const u32x4*)(kc + base);
        vreg[j] = *(const u32x4*)(vc + base);
      }
    }
  };
  auto store_block = [&](int buf) {
    bf16_t* kd = Ks + buf * KSZ;
    bf16_t* vd = Vs + buf * VSZ;
#pragma unroll
    for (int j = 0; j < NCH; ++j) {
      const int c = tid + 256 * j;
      if (c >= PA_KEYS * HD16 * 2) continue;
      const int key = c / (HD16 * 2), pc = c % (HD16 * 2);
      *(u32x4*)(kd + (size_t)key * KLD + pc * 8) = kreg[j];
      *(u32x4*)(vd + (size_t)key * VLD + pc * 8) = vreg[j];
    }
  };
  // what this lane names in a transposing load of V: key 4 half + (lane % 16) / 4, dims 16 ((lane / 16) % 2) + 4 (lane % 4)
  const int v_lane = (half * 4 + ((lane & 15) >> 2)) * VLD + 16 * ((lane >> 4) & 1) + 4 * (lane & 3);
  floatx16 o[DB];
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int e = 0; e < 16; ++e) o[db][e] = 0.f;
  float m = -INFINITY, l = 0.f;
  load_pages(kt_first);
  load_block(kt_first);
  load_pages(kt_first + PA_KEYS);
  store_block(0);
  __syncthreads();
  int buf = 0;
  // every group takes as many steps as the longest run, so that the barriers match
  for (int it = 0, kt = kt_first; it < per_group; ++it, kt += PA_KEYS, buf ^= 1) {
    const bool more = kt + PA_KEYS <= kt_last;
    if (more) {
      load_block(kt + PA_KEYS);  // in flight while this block is multiplied
      load_pages(kt + 2 * PA_KEYS);
    }
    if (wave_on && kt <= wave_hi && kt <= kt_last) {
      const bf16_t* Kb = Ks + buf * KSZ;
      const bf16_t* Vb = Vs + buf * VSZ + v_lane;
      // transposed scores of 64 keys x 32 rows
      floatx16 s[2];
#pragma unroll
      for (int kb = 0; kb < 2; ++kb) {
#pragma unroll
        for (int e = 0; e < 16; ++e) s[kb][e] = 0.f;
        const bf16_t* kr = Kb + (size_t)(kb * 32 + qi) * KLD + half * 8;
#pragma unroll
        for (int ks = 0; ks < HD16; ++ks) s[kb] = mfma32(*(const u32x4*)(kr + ks * 16), qf[ks], s[kb]);
      }
      // every key of the block is visible to every row of this wave: no comparisons needed
      const bool all_visible = kt + PA_KEYS - 1 <= wave_lo_pos && kt >= wave_first;
      // the maximum is taken over the raw scores (the scale is positive); masked scores become -inf
      float mx = -INFINITY;
      if (!all_visible) {
        const int key0 = kt + half * 4;
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
          for (int e = 0; e < 16; ++e) {
            const int key = key0 + kb * 32 + 8 * (e >> 2) + (e & 3);
            s[kb][e] = (key >= first_q && key <= pos_q) ? s[kb][e] : -INFINITY;
          }
      }
#pragma unroll
      for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int e = 0; e < 16; ++e) mx = fmaxf(mx, s[kb][e]);
      mx = fmaxf(mx, __shfl_xor(mx, 32, 64)) * scale_log2e;
      // the running maximum moves only when the new one exceeds it by more than 2^8: probabilities up to 256 lose
      // nothing in fp32 sums or in bf16, and the output is rescaled a few times per row instead of at every block
      const float m_new = (mx > m + 8.0f) ? mx : m;
      u32x4 pb[2][2];
      if (m_new == -INFINITY) {  // this row sees none of the block's keys
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
          for (int st = 0; st < 2; ++st) pb[kb][st] = u32x4{0u, 0u, 0u, 0u};
      } else {
        float rs = 0.f;
#pragma unroll
        for (int kb = 0; kb < 2; ++kb) {
          float p[16];
#pragma unroll
          for (int e = 0; e < 16; ++e) {
            p[e] = __builtin_amdgcn_exp2f(fmaf(s[kb][e], scale_log2e, -m_new));
            rs += p[e];
          }
#pragma unroll
          for (int st = 0; st < 2; ++st)
            pb[kb][st] = u32x4{pack_bf16(p[8 * st], p[8 * st + 1]), pack_bf16(p[8 * st + 2], p[8 * st + 3]),
                               pack_bf16(p[8 * st + 4], p[8 * st + 5]), pack_bf16(p[8 * st + 6], p[8 * st + 7])};
        }
        rs += __shfl_xor(rs, 32, 64);
        if (m_new != m) {
          const float alpha = __builtin_amdgcn_exp2f(m - m_new);
          l *= alpha;
#pragma unroll
          for (int db = 0; db < DB; ++db)
#pragma unroll
            for (int e = 0; e < 16; ++e) o[db][e] *= alpha;
          m = m_new;
        }
        l += rs;
      }
      // O^T[dim][row] += V^T[dim][key] P^T[key][row]
#pragma unroll
      for (int db = 0; db < DB; ++db) {
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
          for (int st = 0; st < 2; ++st) {
            const int k0 = kb * 32 + 16 * st;  // this lane's half takes keys k0 + 4 half .. + 4 and those 8 further
            const u32x2 lo = lds_read_tr16(Vb + k0 * VLD + db * 32);
            const u32x2 hi = lds_read_tr16(Vb + (k0 + 8) * VLD + db * 32);
            o[db] = mfma32(u32x4{lo.x, lo.y, hi.x, hi.y}, pb[kb][st], o[db]);
          }
      }
    }
    if (more) store_block(buf ^ 1);  // nobody reads that buffer: the barrier below ended the block before
    __syncthreads();
  }
  if (NG > 1) {
    // the second group's state goes to the first through LDS ([value][wave][lane]: no bank conflicts), which merges it
    // behind its own; the last barrier of the loop has ended every read of the buffers
    float* mrg = (float*)smem_raw;
    const int at = wave * 64 + lane;
    if (grp == 1) {
      mrg[at] = m;
      mrg[256 + at] = l;
#pragma unroll
      for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int e = 0; e < 16; ++e) mrg[(2 + db * 16 + e) * 256 + at] = o[db][e];
    }
    __syncthreads();
    if (grp == 1) return;
    const float m1 = mrg[at], l1 = mrg[256 + at];
    const float mn = fmaxf(m, m1);
    const float a0 = m == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(m - mn);
    const float a1 = m1 == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(m1 - mn);
    l = l * a0 + l1 * a1;
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int e = 0; e < 16; ++e) o[db][e] = o[db][e] * a0 + mrg[(2 + db * 16 + e) * 256 + at] * a1;
  }
  if (!wave_on || wq >= nrows) return;
  const float inv = 1.0f / l;
  bf16_t* orow = out + (size_t)(row0 + wq) * ldo + (size_t)h * HD;
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int e4 = 0; e4 < 4; ++e4) {
      const int d = db * 32 + 8 * e4 + half * 4;
      if (d < HD)
        *(u32x2*)(orow + d) = u32x2{pack_bf16(o[db][4 * e4] * inv, o[db][4 * e4 + 1] * inv),
                                    pack_bf16(o[db][4 * e4 + 2] * inv, o[db][4 * e4 + 3] * inv)};
    }
}

// ---------------------------------------------------------------------------------------------------------
// Head size 128, two groups of four waves that take turns at the matrix cores.
//
// The kernel above spends a block of keys in phases that follow each other (products, exponentials, products), and
// all waves of a workgroup are in the same phase at the same time: the matrix cores idle while the exponentials
// are taken, and the other way round. Here a workgroup has two groups of four waves for the same 128 rows, one wave
// of each on every SIMD. Both walk the tile's blocks of 64 keys, the first group the even blocks, the second the
// odd ones, half a step apart: while one group multiplies (the weighted sum of its block before, then the scores of
// its next block: 32 MFMAs), the other takes the exponentials of the block it has just scored and issues its
// loads. A workgroup barrier ends every phase. At the end the second group hands its maxima, sums and outputs to
// the first through LDS, as in the two-group form above.
//
// Keys and values go from the cache straight into LDS (global_load_lds_dwordx4: 16 bytes per lane, no registers, no
// LDS stores), each into a ring of two blocks per group: in the phase after the scores of block i the group asks
// for the keys of block i + 2 (their slot was read last by those scores) and the values of block i + 1 (their slot
// was read last by the weighted sum of block i - 1), and both have two phases to arrive. A lane's place in LDS is fixed by
// its number, so the bank swizzle is applied on the global side: slot s of key k holds the key's 16-byte piece
// s ^ swz(k), with swz(k) = 4 (k % 4) + (k / 4) % 4, which spreads the 16 keys that a score fragment reads, and the 4
// keys x 64 bytes that a transposing read of values names, over all banks. Keys outside the tile's visible range
// are read as the nearest visible key (finite numbers in a page the request holds) and masked as before.
#define PP_KEYS 64
#define PP_ROWB 256                   // bytes of one key (or value) row of head size 128
#define PP_BUF (PP_KEYS * PP_ROWB)    // one block of keys, or of values: 16 KB

#define PA_VMCNT(n) __builtin_amdgcn_s_waitcnt(((n) & 15) | (((n) >> 4) << 14) | (7 << 4) | (15 << 8))
#define PA_LGKMCNT0() __builtin_amdgcn_s_waitcnt((15) | (3 << 14) | (7 << 4) | (0 << 8))

// One load of 16 bytes per lane from global memory straight into LDS, written as the instruction itself. Through the
// compiler's builtin the compiler knows of a load into LDS that is on its way, and from then on it waits for all
// outstanding loads and LDS reads before every use of either (it cannot tell which of them that load might be): the
// waits below are written out by hand instead, as the pipeline needs them, and nothing else in the loop of the kernel
// is a vector memory load (table entries come through the scalar cache where pages hold 16 positions or more).
// `lds` is the byte address in LDS of the wave's 1 KB (lane l's 16 bytes land at lds + 16 l).
__device__ __forceinline__ void load_to_lds_16(const void* base, uint32_t offset, uint32_t lds) {
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" : : "v"(offset), "s"(base), "s"(lds) : "memory", "m0");
}
__device__ __forceinline__ void load_to_lds_16(const void* address, uint32_t lds) {
  asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" : : "v"(address), "s"(lds) : "memory", "m0");
}

// WIDE: pages hold 16 positions or more, so the 16 keys a wave brings per block lie in one page and its table entry is
// the same in all lanes
template <bool WIDE>
__global__ __launch_bounds__(512, 1) void prefill_attention_turns_kernel(
    const bf16_t* __restrict__ q, int ldq, bf16_t* __restrict__ out, int ldo, const bf16_t* __restrict__ kc,
    const bf16_t* __restrict__ vc, const int* __restrict__ block_table, int max_blocks, const int* __restrict__ tiles,
    int H, int Hkv, int page_shift, int window, float scale_log2e) {
  constexpr int HD = 128, DB = 4, HD16 = 8;
  extern __shared__ __align__(1024) unsigned char smem_raw[];
  // the wave's number is the same in all its lanes: said so, everything that follows from it (which rows, which blocks,
  // whether a block needs the mask) stays in scalar registers and every branch on it is a jump, not a lane mask
  const int grp = __builtin_amdgcn_readfirstlane((int)threadIdx.x >> 8);
  unsigned char* Kb = smem_raw + (size_t)grp * 4 * PP_BUF;  // [2][PP_BUF]
  unsigned char* Vb = Kb + 2 * PP_BUF;                      // [2][PP_BUF]
  const int* tile = tiles + (size_t)blockIdx.y * 4;
  const int req = tile[0], row0 = tile[1], nrows = tile[2], pos0 = tile[3];
  const int h = blockIdx.x;
  const int kvh = h / (H / Hkv);
  const int tid = threadIdx.x & 255;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
  const int qi = lane & 31, half = lane >> 5;
  const int wq = wave * 32 + qi;
  const int pos_q = pos0 + min(wq, nrows - 1);
  const int first_q = window > 0 ? max(0, pos_q + 1 - window) : 0;
  const int* tbl = block_table + (size_t)req * max_blocks;
  const int k_lo = window > 0 ? max(0, pos0 + 1 - window) : 0;
  const int k_hi = pos0 + nrows - 1;
  const int wave_lo_pos = pos0 + min(nrows - 1, wave * 32);
  const int wave_hi = pos0 + min(nrows - 1, wave * 32 + 31);
  const int wave_first = window > 0 ? max(0, wave_hi + 1 - window) : 0;
  const int kt_tile = (k_lo / PP_KEYS) * PP_KEYS;
  const int n_blocks = (k_hi - kt_tile) / PP_KEYS + 1;
  const int iters = (n_blocks + 1) / 2;  // steps of both groups: the second group's last block may not exist (all masked)
  const int page_mask = (1 << page_shift) - 1;
  // ---- global side of the loads: instruction c of this wave brings keys wave * 16 + 4 c .. + 4 of a block, lane l the
  // piece that belongs into slot l % 16 of key l / 16 of those. Keys outside [k_lo, k_hi] are read as the nearest
  // inside: finite numbers from a page the request holds, masked where the scores are taken.
  const int lkey = lane >> 4;
  const uint32_t lds_k = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char*)Kb;
  const uint32_t lds_v = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char*)Vb;
  // The table entries of a block's keys are loaded a phase before the loads that use them are issued.
  struct Pages {
    int pg[WIDE ? 1 : 4];
  };
  auto pages_of = [&](int i, Pages& p) {  // block i of this group
    const int kw = kt_tile + (grp + 2 * i) * PP_KEYS + wave * 16;
    if (WIDE) {
      // the wave's 16 keys, aligned to 16: wholly before k_lo they are all read as k_lo, wholly after k_hi as k_hi,
      // else the ones outside are read as one inside the same 16: one page in every case
      const int k = kw + 15 < k_lo ? k_lo : kw > k_hi ? k_hi : kw;
      p.pg[0] = __builtin_amdgcn_readfirstlane(tbl[k >> page_shift]);
    } else {
#pragma unroll
      for (int c = 0; c < 4; ++c) p.pg[c] = tbl[min(max(kw + 4 * c + lkey, k_lo), k_hi) >> page_shift];
    }
  };
  auto issue = [&](const bf16_t* cache, uint32_t dst, int i, const Pages& p) {  // into the ring slot at LDS address dst
    const int kw = kt_tile + (grp + 2 * i) * PP_KEYS + wave * 16;
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      const int kabs = min(max(kw + 4 * c + lkey, k_lo), k_hi);
      const int piece = (lane & 15) ^ ((lkey << 2) | c);  // swz of key 4 c + lkey (+ 16 wave)
      const uint32_t off = (uint32_t)(kabs & page_mask) * PP_ROWB + piece * 16;
      if (WIDE) {
        const unsigned char* base = (const unsigned char*)cache + ((((size_t)p.pg[0] * Hkv + kvh) << page_shift) * PP_ROWB);
        load_to_lds_16(base, off, dst + (wave * 4 + c) * 1024);
      } else {
        const unsigned char* src = (const unsigned char*)cache + ((((size_t)p.pg[c] * Hkv + kvh) << page_shift) * PP_ROWB) + off;
        load_to_lds_16(src, dst + (wave * 4 + c) * 1024);
      }
    }
  };
  // ---- LDS side. Scores: the fragment of key block kb, k16 step ks is key kb * 32 + qi, piece 2 ks + half.
  // byte offset of piece (2 ks + half) ^ swz(qi) of key qi: kbase ^ 32 ks (the swizzle's bits and the 32 ks do not carry)
  const int kbase = qi * PP_ROWB + ((half ^ (((qi & 3) << 2) | ((qi >> 2) & 3))) * 16);
  // Values, through the transposing read: this lane names key k0 + 4 half + j (and the one 8 further), j = (lane % 16) / 4,
  // dims 32 db + 16 a + 4 (lane % 4) .. + 4 with a = (lane / 16) % 2: piece 4 db + 2 a + (lane % 4) / 2, swizzled
  // with 4 j + half (and 4 j + half + 2 for the key 8 further: the same piece with its bit 1 turned)
  const int vj = (lane & 15) >> 2;
  const int vbase_lo = (half * 4 + vj) * PP_ROWB + (((2 * ((lane >> 4) & 1) + ((lane & 3) >> 1)) ^ half) * 16) + 8 * (lane & 1);
  const int vbase_hi = (vbase_lo ^ 32) + 8 * PP_ROWB;
  int vdb[DB];
#pragma unroll
  for (int db = 0; db < DB; ++db) vdb[db] = (db ^ vj) * 64;
  // ---- prologue: the keys of the first block on their way, the table entries of what the first step asks for; Q as
  // the B operand
  {
    Pages p0, p1;
    pages_of(0, p0);
    pages_of(1, p1);
    issue(kc, lds_k, 0, p0);
    issue(vc, lds_v, 0, p0);
    issue(kc, lds_k + PP_BUF, 1, p1);
  }
  u32x4 qf[HD16];
  {
    const bf16_t* qr = q + (size_t)(row0 + min(wq, nrows - 1)) * ldq + (size_t)h * HD + half * 8;
#pragma unroll
    for (int ks = 0; ks < HD16; ++ks) qf[ks] = *(const u32x4*)(qr + ks * 16);
  }
  floatx16 o[DB];
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int e = 0; e < 16; ++e) o[db][e] = 0.f;
  floatx16 s[2];
  u32x4 pb[2][2];
#pragma unroll
  for (int kb = 0; kb < 2; ++kb)
#pragma unroll
    for (int st = 0; st < 2; ++st) pb[kb][st] = u32x4{0u, 0u, 0u, 0u};
  float m = -INFINITY, l = 0.f;
  PA_VMCNT(0);
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_sched_barrier(0);
  if (grp == 1) {  // half a step behind
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
  }
  // Step i of a group: a multiply phase (the weighted sum of block i - 1, then the scores of block i), a barrier, an
  // exponentials phase (which also issues the loads), a barrier. Every wave takes every block of its group; what a
  // wave's rows do not see is masked (the last blocks of a tile).
  // a block that starts beyond the wave's last row is skipped by the wave (the last blocks of a tile on the diagonal)
  auto seen = [&](int i) { return kt_tile + (grp + 2 * i) * PP_KEYS <= wave_hi; };
  auto weighted_sum = [&](int i) {  // O^T[dim][row] += V^T[dim][key] P^T[key][row] of block i
    if (!seen(i)) return;
    const unsigned char* Vp = Vb + (i & 1) * PP_BUF;
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int st = 0; st < 2; ++st) {
          const int k0 = kb * 32 + 16 * st;
          const u32x2 lo = lds_read_tr16(Vp + k0 * PP_ROWB + vbase_lo + vdb[db]);
          const u32x2 hi = lds_read_tr16(Vp + k0 * PP_ROWB + vbase_hi + vdb[db]);
          o[db] = mfma32(u32x4{lo.x, lo.y, hi.x, hi.y}, pb[kb][st], o[db]);
        }
  };
  auto scores = [&](int i) {  // transposed scores of 64 keys x 32 rows
    if (!seen(i)) return;
    const unsigned char* Kp = Kb + (i & 1) * PP_BUF;
    const floatx16 zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    s[0] = zero;
    s[1] = zero;
#pragma unroll
    for (int ks = 0; ks < HD16; ++ks)
#pragma unroll
      for (int kb = 0; kb < 2; ++kb)
        s[kb] = mfma32(*(const u32x4*)(Kp + kb * 32 * PP_ROWB + (kbase ^ (32 * ks))), qf[ks], s[kb]);
  };
  auto phase_end = [&]() {
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
  };
  auto exponentials = [&](int i) {
    const int kt = kt_tile + (grp + 2 * i) * PP_KEYS;
    // the table entries of what this phase asks for at its end go first
    Pages pgk, pgv;
    pages_of(i + 2, pgk);
    pages_of(i + 1, pgv);
    const bool all_visible = kt + PP_KEYS - 1 <= wave_lo_pos && kt >= wave_first;
    if (seen(i)) {
    if (!all_visible) {  // a block on the diagonal, at the window's edge or beyond the tile: unseen keys score -inf
      const int key0 = kt + half * 4;
#pragma unroll
      for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          const int key = key0 + kb * 32 + 8 * (e >> 2) + (e & 3);
          s[kb][e] = (key >= first_q && key <= pos_q) ? s[kb][e] : -INFINITY;
        }
    }
    float mx = -INFINITY;
#pragma unroll
    for (int kb = 0; kb < 2; ++kb)
#pragma unroll
      for (int e = 0; e < 16; ++e) mx = fmaxf(mx, s[kb][e]);
    mx = fmaxf(mx, __shfl_xor(mx, 32, 64)) * scale_log2e;
    // the running maximum moves only when the new one exceeds it by more than 2^8: probabilities up to 256 lose
    // nothing in fp32 sums or in bf16, and the output is rescaled a few times per row instead of at every block
    const float m_new = (mx > m + 8.0f) ? mx : m;
    const float m_use = m_new == -INFINITY ? 0.f : m_new;  // a row that has seen no key yet: every exponential is 0
    float rs = 0.f;
#pragma unroll
    for (int kb = 0; kb < 2; ++kb) {
      float p[16];
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        p[e] = __builtin_amdgcn_exp2f(fmaf(s[kb][e], scale_log2e, -m_use));
        rs += p[e];
      }
#pragma unroll
      for (int st = 0; st < 2; ++st)
        pb[kb][st] = u32x4{pack_bf16(p[8 * st], p[8 * st + 1]), pack_bf16(p[8 * st + 2], p[8 * st + 3]),
                           pack_bf16(p[8 * st + 4], p[8 * st + 5]), pack_bf16(p[8 * st + 6], p[8 * st + 7])};
    }
    rs += __shfl_xor(rs, 32, 64);
    if (__builtin_amdgcn_ballot_w64(m_new != m) != 0) {  // some row's maximum moved: rescale (a factor of 1 elsewhere)
      const float alpha = m_new == m ? 1.0f : __builtin_amdgcn_exp2f(m - m_new);
      l *= alpha;
#pragma unroll
      for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int e = 0; e < 16; ++e) o[db][e] *= alpha;
      m = m_new;
    }
    l += rs;
    }
    // The loads are issued here, by the group that is not multiplying: a compute unit takes a load of 1 KB about
    // every 40 cycles and the issuing wave waits meanwhile, which would hold up its own multiplies. The keys of block
    // i + 2 go where the scores of block i were just read, the values of block i + 1 where the weighted sum of block
    // i - 1 was. What the phase before asked for (keys of i + 1, values of i) is needed next and must have landed:
    // loads complete in order, so all but the 8 just issued.
    __builtin_amdgcn_sched_barrier(0);
    issue(kc, lds_k + (i & 1) * PP_BUF, i + 2, pgk);
    issue(vc, lds_v + ((i + 1) & 1) * PP_BUF, i + 1, pgv);
    PA_VMCNT(8);
  };
  scores(0);
  phase_end();
  exponentials(0);
  phase_end();
  for (int i = 1; i < iters; ++i) {
    weighted_sum(i - 1);
    scores(i);
    phase_end();
    exponentials(i);
    phase_end();
  }
  weighted_sum(iters - 1);
  // the second group's state goes to the first through LDS ([value][wave][lane]), which merges it behind its own
  PA_VMCNT(0);                   // nothing is on its way into LDS any more
  __builtin_amdgcn_s_barrier();  // the multiply phase of the other group has ended (the first group's extra barrier)
  if (grp == 0) __builtin_amdgcn_s_barrier();
  float* mrg = (float*)smem_raw;
  const int at = wave * 64 + lane;
  if (grp == 1) {
    mrg[at] = m;
    mrg[256 + at] = l;
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int e = 0; e < 16; ++e) mrg[(2 + db * 16 + e) * 256 + at] = o[db][e];
  }
  __syncthreads();
  if (grp == 1) return;
  const float m1 = mrg[at], l1 = mrg[256 + at];
  const float mn = fmaxf(m, m1);
  const float a0 = m == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(m - mn);
  const float a1 = m1 == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(m1 - mn);
  l = l * a0 + l1 * a1;
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int e = 0; e < 16; ++e) o[db][e] = o[db][e] * a0 + mrg[(2 + db * 16 + e) * 256 + at] * a1;
  if (wq >= nrows) return;
  const float inv = 1.0f / l;
  bf16_t* orow = out + (size_t)(row0 + wq) * ldo + (size_t)h * HD;
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int e4 = 0; e4 < 4; ++e4) {
      const int d = db * 32 + 8 * e4 + half * 4;
      *(u32x2*)(orow + d) = u32x2{pack_bf16(o[db][4 * e4] * inv, o[db][4 * e4 + 1] * inv),
                                  pack_bf16(o[db][4 * e4 + 2] * inv, o[db][4 * e4 + 3] * inv)};
    }
}

static int launch_prefill_turns(dim3 grid, hipStream_t stream, const bf16_t* q, int ldq, bf16_t* out, int ldo, const bf16_t* kc,
                                const bf16_t* vc, const int* bt, int mb, const int* tiles, int H, int Hkv, int page, int window,
                                float sl) {
  constexpr size_t smem = 8 * PP_BUF;  // two groups x (two blocks of keys + two of values); the merge needs 66 KB of it
  static bool configured = false;
  if (!configured) {
    if (hipFuncSetAttribute((const void*)prefill_attention_turns_kernel<true>, hipFuncAttributeMaxDynamicSharedMemorySize,
                            (int)smem) != hipSuccess ||
        hipFuncSetAttribute((const void*)prefill_attention_turns_kernel<false>, hipFuncAttributeMaxDynamicSharedMemorySize,
                            (int)smem) != hipSuccess)
      return -1;
    configured = true;
  }
  int shift = 0;
  while ((1 << shift) < page) ++shift;
  if (page >= 16)
    prefill_attention_turns_kernel<true><<<grid, 512, smem, stream>>>(q, ldq, out, ldo, kc, vc, bt, mb, tiles, H, Hkv, shift, window, sl);
  else
    prefill_attention_turns_kernel<false><<<grid, 512, smem, stream>>>(q, ldq, out, ldo, kc, vc, bt, mb, tiles, H, Hkv, shift, window, sl);
  return 0;
}

template <int HD16, int NG>
static int launch_prefill(dim3 grid, hipStream_t stream, const bf16_t* q, int ldq, bf16_t* out, int ldo, const bf16_t* kc,
                          const bf16_t* vc, const int* bt, int mb, const int* tiles, int H, int Hkv, int page, int window,
                          float sl) {
  constexpr int HD = HD16 * 16;
  // buffers of the groups; afterwards the merge of two groups: (2 + accumulators) x 256 floats
  constexpr size_t stage = (size_t)NG * 2 * (PA_KEYS * (HD + 8) + PA_KEYS * (HD + 32)) * sizeof(bf16_t);
  constexpr size_t merge = NG > 1 ? (size_t)(2 + ((HD + 31) / 32) * 16) * 256 * sizeof(float) : 0;
  constexpr size_t smem = stage > merge ? stage : merge;
  static bool configured = false;
  if (!configured) {
    if (hipFuncSetAttribute((const void*)prefill_attention_kernel<HD16, NG>, hipFuncAttributeMaxDynamicSharedMemorySize,
                            (int)smem) != hipSuccess)
      return -1;
    configured = true;
  }
  int shift = 0;
  while ((1 << shift) < page) ++shift;
  prefill_attention_kernel<HD16, NG><<<grid, 256 * NG, smem, stream>>>(q, ldq, out, ldo, kc, vc, bt, mb, tiles, H, Hkv,
                                                                      shift, window, sl);
  return 0;
}

// tiles: int32 [n_tiles][4] = (request index, first row in the batch, rows (1..128), position of the first row);
// key_groups: the caller's advice on the form (below)
// returns 0 when it ran, 1 when the shape is not one it takes, -1 on errors
extern "C" int jllm_prefill_attention_bf16(const void* q, int ldq, void* out, int ldo, const void* kcache,
                                           const void* vcache, const int* block_table, int max_blocks, const int* tiles,
                                           const int* positions, int n_tiles, int n_requests, int H, int Hkv, int hd,
                                           int page_size, int window, int max_context, float scale, int key_groups,
                                           hipStream_t stream) {
  (void)positions;
  (void)n_requests;
  if (n_tiles <= 0) return 0;
  if (Hkv <= 0 || H % Hkv != 0) JLLM_FAIL("prefill attention: %d query heads over %d kv heads", H, Hkv);
  if ((hd & 15) || hd > 192 || hd < 16 || (ldq & 7) || (ldo & 3) || ((uintptr_t)q & 15) || ((uintptr_t)out & 7)) return 1;
  if (page_size <= 0 || (page_size & (page_size - 1)) || n_tiles > 65535) return 1;
  dim3 grid(H, n_tiles);
  const float sl = scale * 1.4426950408889634f;
  // Two key groups per workgroup while one-group workgroups would all be resident at once (two per compute unit):
  // then the step waits for the tile with the most keys, and halving every tile's chain of blocks is what helps.
  // With more workgroups than that the units stay busy anyway, and two independent workgroups of four waves on a
  // unit overlap better than one of eight that meets at a barrier after every block.
  // `key_groups`: 1 when the caller knows that the tiles have about the same number of keys (portions deep inside
  // long requests: nothing waits for one long tile, and the one-group form is the faster one), 2 or 0 otherwise.
  const bool older = (key_groups & 4) != 0;  // + 4: never the form with turns (to measure the forms against each other)
  key_groups &= 3;
  const bool few = (long)H * n_tiles <= 2L * jllm_compute_units();
  const bool two_groups = hd <= 128 && key_groups != 1 && few;
  // Head size 128: the form whose two groups take turns at the matrix cores holds a compute unit alone (128 KB of
  // LDS), so its start (the first blocks' loads with nothing to hide them) and its end (the merge) are not covered by
  // another workgroup's work. It wins where tiles are long or few: a step whose workgroups are all resident at
  // once (one 2,048-token prompt at 32 heads: 53 against 59 us), and tiles deep inside long requests (2,048 rows
  // from position 6,144: 255 against 300 us, 0.94 PFLOP/s; from 14,336: 520 against 620, 0.99 PFLOP/s). Four
  // 2,048-token prompts from their start (17 blocks a tile on average, eight rounds of workgroups) take 204 us
  // against 196 in the one-group form. (Best of three runs of 50 calls each, the kernel alone.)
  if (hd == 128 && !older && (few || (key_groups == 1 && max_context >= 3072))) {
    if (launch_prefill_turns(grid, stream, (const bf16_t*)q, ldq, (bf16_t*)out, ldo, (const bf16_t*)kcache, (const bf16_t*)vcache,
                             block_table, max_blocks, tiles, H, Hkv, page_size, window, sl) != 0)
      JLLM_FAIL("prefill attention: cannot reserve LDS");
    JLLM_CHECK_LAUNCH("prefill_attention");
    return 0;
  }
#define PA_CASE(N)                                                                                                     \
  case N: {                                                                                                            \
    const int rc_ = two_groups && N <= 8                                                                               \
        ? launch_prefill<N, (N <= 8 ? 2 : 1)>(grid, stream, (const bf16_t*)q, ldq, (bf16_t*)out, ldo, (const bf16_t*)kcache, \
                          (const bf16_t*)vcache, block_table, max_blocks, tiles, H, Hkv, page_size, window, sl)        \
        : launch_prefill<N, 1>(grid, stream, (const bf16_t*)q, ldq, (bf16_t*)out, ldo, (const bf16_t*)kcache,          \
                          (const bf16_t*)vcache, block_table, max_blocks, tiles, H, Hkv, page_size, window, sl);       \
    if (rc_ != 0) JLLM_FAIL("prefill attention: cannot reserve LDS");                                                  \
    break;                                                                                                             \
  }
  switch (hd / 16) {
    PA_CASE(1) PA_CASE(2) PA_CASE(3) PA_CASE(4) PA_CASE(5) PA_CASE(6) PA_CASE(7) PA_CASE(8) PA_CASE(12)
    default: return 1;
  }
#undef PA_CASE
  JLLM_CHECK_LAUNCH("prefill_attention");
  return 0;
}
