// out[M,N] = A[M,K] * W[N,K]^T for many rows, bf16 on the matrix cores (v_mfma_f32_32x32x16_bf16), built so that the
// matrix cores of a compute unit never wait for operands:
//
//  * A workgroup of 8 waves (2 x 4) owns a 256 x 256 output tile (a wave 128 x 64: FM = 4 by FN = 2 accumulators of
//    32 x 32). K advances in stages of 32 through a ring of NS stages in LDS.
//  * Global -> LDS without registers: global_load_lds_dwordx4 writes 16 bytes per lane straight into LDS, 1 KB
//    (16 tile rows of 64 bytes) per instruction, NS - 1 stages ahead of the multiplies. A lane's place in LDS is
//    fixed by its number, so the bank swizzle is applied on the global side: the lane that fills slot s of row r
//    fetches the row's 16-byte piece s ^ f(r).
//  * The waves form two groups, one wave of each on every SIMD, that run half a stage apart: while one group
//    multiplies (16 MFMAs from registers, nothing else), the other reads the next stage's fragments from LDS and
//    issues its share of the global loads; a workgroup barrier after every phase keeps them apart. A SIMD's matrix
//    core so always has a wave with all operands in registers.
//
// Phases are the times between two workgroup barriers. In phase 2t group 0 is in its memory phase of stage t (it reads
// the stage's second half of fragments from LDS and issues the loads of stage t + NS - 1) while group 1 multiplies
// stage t - 1 and, between the multiplies, reads the first half of stage t's fragments; in phase 2t + 1 the groups
// have swapped (group 0 multiplies stage t and reads the first half of stage t + 1). So stage s is read from phase
// 2s - 1 on and must have landed when that phase starts: before the barrier in front of it every wave waits until
// its own loads of stages <= s are complete (loads complete in order; group 0 has issued two stages beyond s by
// then, group 1 one). The loads of stage t + NS - 1 go to the slot of stage t - 1, whose last reader (group 1, second
// half, phase 2t - 1) has waited for its LDS reads before the barrier that ends that phase.
//
// Epilogues as in the other tiled kernel (gemm_epilogue.h). Needs K % 32 == 0 and at least NS - 1 stages, 16-byte
// aligned rows; any M and N (rows beyond the end are read as the last row and never stored).
#include "common.h"
#include "gemm_epilogue.h"
#include "mfma.h"

#define PP_BK 32
#define PP_ROW_BYTES (PP_BK * 2)  // a tile row in LDS: 64 bytes = 4 pieces of 16
#define PP_WAVES 8

// The piece of row r that lies in slot s is s ^ pp_swz(r): 16 lanes that read the same piece of 16 consecutive rows,
// and 8 lanes of 8 rows, then cover every bank once, whichever of the two the LDS takes per pass.
__device__ __forceinline__ int pp_swz(int r) { return (((r >> 1) ^ (r >> 3)) & 1) | (((r >> 2) & 1) << 1); }

#define PP_VMCNT(n) __builtin_amdgcn_s_waitcnt(((n) & 15) | (((n) >> 4) << 14) | (7 << 4) | (15 << 8))
#define PP_LGKMCNT0() __builtin_amdgcn_s_waitcnt((15) | (3 << 14) | (7 << 4) | (0 << 8))

template <bool GATED, int FM, int NS>
__global__ __launch_bounds__(PP_WAVES * 64) void gemm_pingpong_kernel(
    const bf16_t* __restrict__ A, int lda, const bf16_t* __restrict__ W, const bf16_t* __restrict__ W2,
    const void* __restrict__ bias, int bias_dtype, void* __restrict__ out, int out_dtype, int ldo, int M, int N, int K,
    int epilogue, float* __restrict__ partial) {
  constexpr int WGM = 2, WGN = 4, FN = 2;
  constexpr int TBM = WGM * FM * 32, TBN = WGN * FN * 32;
  constexpr int STAGE = (TBM + TBN) * PP_ROW_BYTES;
  constexpr int LA = TBM / 16 / PP_WAVES, LB = TBN / 16 / PP_WAVES;  // load instructions per wave and stage
  constexpr int LPW = LA + LB;
  static_assert(LA >= 1 && LB >= 1, "every wave loads rows of both operands");
  extern __shared__ __align__(1024) unsigned char smem[];
  const int tid = threadIdx.x;
  // the wave's number is the same in all its lanes: said so, its group, its part of the tile and the places in LDS it
  // fills stay in scalar registers (no vector arithmetic for them per stage, jumps instead of lane masks)
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
  const int group = wave >> 2;  // waves 0..3 and 4..7: one of each on every SIMD
  const int wm = wave / WGN, wn = wave % WGN;
  const int m0 = blockIdx.y * TBM;
  const int n0 = blockIdx.x * (GATED ? TBN / 2 : TBN);
  const int nk_all = K / PP_BK;
  const int nk_per = (nk_all + gridDim.z - 1) / gridDim.z;
  const int kt0 = blockIdx.z * nk_per;
  const int nk = max(0, min(nk_all, kt0 + nk_per) - kt0);

  // ---- global side of the loads: this lane's piece of each of the wave's 16-row chunks. The address of a load is a
  // scalar base (the operand's start plus the stage's place in K, advanced by scalar arithmetic) plus a 32-bit byte
  // offset per lane that never changes (row and piece), so a stage's loads cost no vector instruction.
  const int lrow = lane >> 2, lslot = lane & 3;
  uint32_t goff[LPW];              // this lane's byte offset from the operand's start (rows x row length < 4 GB: checked on the host)
  const unsigned char* gbase[LPW];  // the operand's start at this workgroup's first K step (the same in all lanes)
  uint32_t ldst[LPW];              // LDS byte address of the chunk inside stage 0 (the same in all lanes)
  const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char*)smem;
#pragma unroll
  for (int c = 0; c < LA; ++c) {
    const int r = (wave * LA + c) * 16 + lrow;
    goff[c] = (uint32_t)min(m0 + r, M - 1) * (uint32_t)lda * 2u + (uint32_t)((lslot ^ pp_swz(r)) * 16);
    gbase[c] = (const unsigned char*)A + (size_t)kt0 * PP_ROW_BYTES;
    ldst[c] = lds0 + (wave * LA + c) * 16 * PP_ROW_BYTES;
  }
#pragma unroll
  for (int c = 0; c < LB; ++c) {
    const int r = (wave * LB + c) * 16 + lrow;
    int wr;
    const bf16_t* wb = W;
    if (GATED) {  // LDS row r: quarter r / 32: even = gate, odd = up of the outputs n0 + (quarter / 2) * 32 ..
      const int quarter = (wave * LB + c) >> 1;  // of the chunk's 16 rows: the same in all lanes
      wr = n0 + (quarter >> 1) * 32 + (r & 31);
      wb = (quarter & 1) ? W2 : W;
    } else {
      wr = n0 + r;
    }
    goff[LA + c] = (uint32_t)min(wr, N - 1) * (uint32_t)K * 2u + (uint32_t)((lslot ^ pp_swz(r)) * 16);
    gbase[LA + c] = (const unsigned char*)wb + (size_t)kt0 * PP_ROW_BYTES;
    ldst[LA + c] = lds0 + TBM * PP_ROW_BYTES + (wave * LB + c) * 16 * PP_ROW_BYTES;
  }
  auto issue = [&](int t) {  // the wave's loads of stage t
    const uint32_t slot = (uint32_t)(t % NS) * STAGE;
    const size_t kbytes = (size_t)t * PP_ROW_BYTES;
#pragma unroll
    for (int c = 0; c < LPW; ++c) {
      // the instruction itself: m0 holds the LDS address of the wave's 1 KB, lane l's 16 bytes land at m0 + 16 l
      asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                   :
                   : "v"(goff[c]), "s"(gbase[c] + kbytes), "s"(ldst[c] + slot)
                   : "memory", "m0");
    }
  };

  // ---- LDS side: fragment (row block i, k16 step ks): row = block * 32 + lane % 32, piece = 2 ks + lane / 32
  const int fr = lane & 31, half = lane >> 5;
  int aoff[2], boff[2];
#pragma unroll
  for (int ks = 0; ks < 2; ++ks) {
    const int ra = wm * FM * 32 + fr, rb = wn * FN * 32 + fr;  // + 32 i leaves pp_swz unchanged
    aoff[ks] = ra * PP_ROW_BYTES + (((2 * ks + half) ^ pp_swz(ra)) * 16);
    boff[ks] = TBM * PP_ROW_BYTES + rb * PP_ROW_BYTES + (((2 * ks + half) ^ pp_swz(rb)) * 16);
  }

  floatx16 acc[FM][FN];
#pragma unroll
  for (int i = 0; i < FM; ++i)
#pragma unroll
    for (int j = 0; j < FN; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

  // ---- prologue: NS - 1 stages on their way, stages 0 and 1 landed
#pragma unroll
  for (int s = 0; s < NS - 1; ++s)
    if (s < nk) issue(s);
  if (nk >= NS - 1) {
    PP_VMCNT((NS - 3) * LPW);
  } else {
    PP_VMCNT(0);
  }
  __builtin_amdgcn_sched_barrier(0);
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_sched_barrier(0);
  // fragments: f0 = the k16 step 0 of the stage being multiplied, f1 = its step 1, fn = step 0 of the next stage (read
  // during the multiplies); the loop is unrolled by two so that f0 and fn swap names instead of being copied
  u32x4 a0[FM], b0[FN], a1[FM], b1[FN], an[FM], bn[FN];
  auto read = [&](int t, int ks, u32x4 (&af)[FM], u32x4 (&bf)[FN]) {
    const unsigned char* st = smem + (t % NS) * STAGE;
#pragma unroll
    for (int i = 0; i < FM; ++i) af[i] = *(const u32x4*)(st + aoff[ks] + i * 32 * PP_ROW_BYTES);
#pragma unroll
    for (int j = 0; j < FN; ++j) bf[j] = *(const u32x4*)(st + boff[ks] + j * 32 * PP_ROW_BYTES);
  };
  // one stage of one group. Memory phase: the second half of the stage's fragments, then the global loads (a compute
  // unit's load pipe takes about 40 cycles per load instruction and a wave waits at the issue while it is busy, so
  // the LDS reads go first). Multiply phase: 16 MFMAs with the reads of the next stage's first fragments between them.
  auto stage = [&](int t, u32x4 (&fa0)[FM], u32x4 (&fb0)[FN], u32x4 (&na0)[FM], u32x4 (&nb0)[FN]) {
    const bool more = t + NS - 1 < nk;
    read(t, 1, a1, b1);
    __builtin_amdgcn_sched_barrier(0);
    if (more) issue(t + NS - 1);
    // own loads of stage t + 1 must have landed before the barrier that lets group 0 read it during its multiplies:
    // group 0 is here (it has issued up to stage t + 3), group 1 at the end of its multiplies of stage t - 1
    if (group == 0) {
      if (more) {
        PP_VMCNT(2 * LPW);
      } else {
        PP_VMCNT(0);
      }
    }
    PP_LGKMCNT0();
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
    read(t + 1, 0, na0, nb0);  // beyond the last stage: some slot's bytes, never multiplied
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
      for (int j = 0; j < FN; ++j) acc[i][j] = mfma32(fb0[j], fa0[i], acc[i][j]);
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
      for (int j = 0; j < FN; ++j) acc[i][j] = mfma32(b1[j], a1[i], acc[i][j]);
    // order of issue: two multiplies, then one LDS read, ...; the rest of the multiplies
#pragma unroll
    for (int r = 0; r < FM + FN; ++r) {
      __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
    }
    __builtin_amdgcn_sched_group_barrier(0x008, 2 * FM * FN - 2 * (FM + FN), 0);
    if (group == 1) {  // has issued up to stage t + 3; stage t + 2 must have landed (group 0 reads it after the next barrier but one)
      if (more) {
        PP_VMCNT(1 * LPW);
      } else {
        PP_VMCNT(0);
      }
    }
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
  };
  if (nk > 0) read(0, 0, a0, b0);
  if (group == 1) {  // half a stage behind
    PP_LGKMCNT0();
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
  }
  for (int t = 0; t < nk; t += 2) {
    stage(t, a0, b0, an, bn);
    if (t + 1 < nk) stage(t + 1, an, bn, a0, b0);
  }
  if (group == 0) {  // as many barriers as the other group
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
  }
  tile_epilogue<GATED, FM, FN, TBM, TBN>(acc, lane, wm, wn, m0, n0, bias, bias_dtype, out, out_dtype, ldo, M, N, epilogue, partial,
                                         (int)blockIdx.z, (int)gridDim.z);
}

template <int FM, int NS>
static int launch_pingpong(const void* A, int lda, const void* W, const void* W2, const void* bias, int bias_dtype,
                           void* out, int out_dtype, int ldo, int M, int N, int K, int epilogue, int splits,
                           float* partial, hipStream_t stream) {
  constexpr int TBM = 2 * FM * 32, TBN = 256;
  const int cols = W2 ? TBN / 2 : TBN;
  dim3 grid((N + cols - 1) / cols, (M + TBM - 1) / TBM, splits);
  if (grid.y > 65535) return 1;
  const size_t smem = (size_t)NS * (TBM + TBN) * PP_ROW_BYTES;
  static bool configured = false;
  if (!configured) {
    hipError_t e1 = hipFuncSetAttribute((const void*)gemm_pingpong_kernel<true, FM, NS>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    hipError_t e2 = hipFuncSetAttribute((const void*)gemm_pingpong_kernel<false, FM, NS>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    if (e1 != hipSuccess || e2 != hipSuccess) JLLM_FAIL("gemm_pingpong: cannot reserve %zu bytes of LDS", smem);
    configured = true;
  }
  if (W2)
    gemm_pingpong_kernel<true, FM, NS><<<grid, PP_WAVES * 64, smem, stream>>>(
        (const bf16_t*)A, lda, (const bf16_t*)W, (const bf16_t*)W2, bias, bias_dtype, out, out_dtype, ldo, M, N, K, epilogue, partial);
  else
    gemm_pingpong_kernel<false, FM, NS><<<grid, PP_WAVES * 64, smem, stream>>>(
        (const bf16_t*)A, lda, (const bf16_t*)W, nullptr, bias, bias_dtype, out, out_dtype, ldo, M, N, K, epilogue, partial);
  return 0;
}

// `tile_rows`: 256 (rows of the output tile; 256 columns, 128 outputs with the gated epilogue).
// `splits` > 1 cuts K over gridDim.z (not with the gated epilogue): `partial` then holds splits * M * N floats, summed
// in ascending order of the split by the other tiled kernel's reduction. Returns 0 when it ran, 1 when the shape is not one it takes, -1 on errors.
extern "C" int jllm_gemm_pingpong_bf16(const void* A, int lda, const void* W, const void* W2, const void* bias,
                                       int bias_dtype, void* out, int out_dtype, int ldo, int M, int N, int K,
                                       int epilogue, int tile_rows, int splits, float* partial, hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (K <= 0 || (K % PP_BK) || (lda & 7)) return 1;
  if (((uintptr_t)A & 15) || ((uintptr_t)W & 15) || (W2 && ((uintptr_t)W2 & 15))) return 1;
  JLLM_TAKE_GATE("gemm_pingpong", epilogue);
  if (epilogue < 0 || epilogue > 2 || (epilogue == 2) != (W2 != nullptr)) JLLM_FAIL("gemm_pingpong: epilogue %d", epilogue);
  if (epilogue == 1 && out_dtype != JLLM_F32) JLLM_FAIL("gemm_pingpong: the accumulate epilogue adds into fp32");
  if (ldo < N) JLLM_FAIL("gemm_pingpong: ldo %d < N %d", ldo, N);
  // a lane's place in an operand is a 32-bit byte offset from the operand's start
  if ((unsigned long long)M * (unsigned)lda * 2ull >= (1ull << 32) || (unsigned long long)N * (unsigned)K * 2ull >= (1ull << 32)) return 1;
  if (splits < 1) splits = 1;
  if (splits > 1 && (W2 || !partial)) JLLM_FAIL("gemm_pingpong: %d K splits are not possible here", splits);
  if (splits > 65535 || (K / PP_BK) / splits < 4) return 1;
  int rc;
  if (tile_rows == 256)
    rc = launch_pingpong<4, 4>(A, lda, W, W2, bias, bias_dtype, out, out_dtype, ldo, M, N, K, epilogue, splits, partial, stream);
  else
    JLLM_FAIL("gemm_pingpong: tile of %d rows (256 is built)", tile_rows);
  if (rc != 0) return rc;
  JLLM_CHECK_LAUNCH("gemm_pingpong");
  if (splits > 1) return jllm_splitk_reduce(partial, splits, bias, bias_dtype, out, out_dtype, ldo, M, N, epilogue, stream);
  return 0;
}
