// Two probes that measure what this GPU delivers, as denominators beside the published peaks: a kernel that only
// streams memory in (read bandwidth of HBM for a buffer far larger than the caches) and a kernel that only issues
// bf16 MFMAs from registers (what the matrix cores reach at the clock they hold under that load). The reference
// states its rooflines against measured ceilings in the same way (docs/11-performance.md:24-35, :68-74).
#include "common.h"
#include "mfma.h"

// every thread reads 16 bytes at a time, a workgroup a contiguous 4 KB per turn; grid-stride over the buffer
__global__ __launch_bounds__(256) void probe_read_kernel(const u32x4* __restrict__ src, size_t n16, unsigned* __restrict__ sink) {
  u32x4 acc = u32x4{0u, 0u, 0u, 0u};
  const size_t stride = (size_t)gridDim.x * 256 * 4;
  size_t i = (size_t)blockIdx.x * 256 * 4 + threadIdx.x;
  for (; i + 768 < n16; i += stride) {  // four loads in flight per thread
    const u32x4 a = src[i], b = src[i + 256], c = src[i + 512], d = src[i + 768];
    acc ^= a ^ b ^ c ^ d;
  }
  for (; i < n16; i += 256) acc ^= src[i];
  if ((acc.x ^ acc.y ^ acc.z ^ acc.w) == 0x9e3779b9u) sink[0] = 1u;  // keeps the loads alive; practically never true
}

__global__ __launch_bounds__(256) void probe_mfma_kernel(float* __restrict__ sink, int iters) {
  u32x4 a = u32x4{0x3f803f80u + threadIdx.x, 0x3f803f80u, 0x3f803f80u, 0x3f803f80u};
  u32x4 b = u32x4{0x3f003f00u, 0x3f003f00u + threadIdx.x, 0x3f003f00u, 0x3f003f00u};
  floatx16 c0 = {}, c1 = {}, c2 = {}, c3 = {};
  for (int it = 0; it < iters; ++it) {
    c0 = mfma32(a, b, c0);
    c1 = mfma32(a, b, c1);
    c2 = mfma32(a, b, c2);
    c3 = mfma32(a, b, c3);
  }
  const float r = c0[0] + c1[1] + c2[2] + c3[3];
  if (r == 12345.678f) sink[0] = r;
}

// reads `bytes` bytes of src once; the caller times it
extern "C" int jllm_probe_read(const void* src, long long bytes, void* sink, hipStream_t stream) {
  if (bytes < 16 || ((uintptr_t)src & 15)) JLLM_FAIL("probe_read: needs a 16-byte aligned buffer of at least 16 bytes");
  const int cus = jllm_compute_units();
  if (cus <= 0) JLLM_FAIL("probe_read: the GPU's compute units could not be read");
  probe_read_kernel<<<cus * 8, 256, 0, stream>>>((const u32x4*)src, (size_t)bytes / 16, (unsigned*)sink);
  JLLM_CHECK_LAUNCH("probe_read");
  return 0;
}

// issues iters * 4 MFMAs (32x32x16 bf16: 32,768 flop each) per wave on workgroups * 4 waves; returns the flop count
// through `flops`
extern "C" int jllm_probe_mfma(int iters, void* sink, double* flops, hipStream_t stream) {
  const int cus = jllm_compute_units();
  if (cus <= 0 || iters <= 0) JLLM_FAIL("probe_mfma: %d iterations on %d compute units", iters, cus);
  const int groups = cus * 2;  // two workgroups of four waves per compute unit: two waves on every SIMD
  probe_mfma_kernel<<<groups, 256, 0, stream>>>((float*)sink, iters);
  JLLM_CHECK_LAUNCH("probe_mfma");
  if (flops) *flops = (double)groups * 4.0 * (double)iters * 4.0 * 32768.0;
  return 0;
}
