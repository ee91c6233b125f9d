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
  const int grp = NG > 1 ? (int)threadIdx.x >> 8 : 0;  // key group: four waves with their own buffers
  bf16_t* Ks = (bf16_t*)smem_raw + (size_t)grp * 2 * (KSZ + VSZ);  // [2][KSZ]
  bf16_t* Vs = Ks + 2 * KSZ;                                       // [2][VSZ]
  const int* tile = tiles + (size_t)blockIdx.y * 4;
  const int req = tile[0], row0 = tile[1], nrows = tile[2], pos0 = tile[3];
  const int h = blockIdx.x;
  const int kvh = h / (H / Hkv);
  const int tid = threadIdx.x & 255;  // within the group
  const int wave = tid >> 6, lane = tid & 63;
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
#pragma unroll
      for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          float v = s[kb][e];
          if (!all_visible) {
            const int key = kt + kb * 32 + 8 * (e >> 2) + half * 4 + (e & 3);
            v = (key >= first_q && key <= pos_q) ? v : -INFINITY;
            s[kb][e] = v;
          }
          mx = fmaxf(mx, v);
        }
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
  (void)max_context;
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
  const bool two_groups = hd <= 128 && key_groups != 1 && (long)H * n_tiles <= 2L * jllm_compute_units();
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
