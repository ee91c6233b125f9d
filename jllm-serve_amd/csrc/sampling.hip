// Token selection on the device.
//
// argmax: the lowest index among equal maxima (sampling/Sampler.java:458-466 scans with `>` from 0).
#include <math.h>

#include "common.h"

__global__ __launch_bounds__(256) void argmax_kernel(const float* __restrict__ logits, int ld, int vocab,
                                                     int* __restrict__ out) {
  __shared__ float bv[256];
  __shared__ int bi[256];
  const float* z = logits + (size_t)blockIdx.x * ld;
  float best = -INFINITY;
  int idx = 0x7fffffff;
  for (int i = threadIdx.x; i < vocab; i += 256) {
    const float v = z[i];
    if (v > best || idx == 0x7fffffff) {  // ascending i per thread: ties keep the lower index
      if (v > best || idx == 0x7fffffff) {
        best = v;
        idx = i;
      }
    }
  }
  bv[threadIdx.x] = best;
  bi[threadIdx.x] = idx;
  __syncthreads();
  for (int s = 128; s > 0; s >>= 1) {
    if (threadIdx.x < s) {
      const float ov = bv[threadIdx.x + s];
      const int oi = bi[threadIdx.x + s];
      if (oi != 0x7fffffff && (bi[threadIdx.x] == 0x7fffffff || ov > bv[threadIdx.x] ||
                               (ov == bv[threadIdx.x] && oi < bi[threadIdx.x]))) {
        bv[threadIdx.x] = ov;
        bi[threadIdx.x] = oi;
      }
    }
    __syncthreads();
  }
  if (threadIdx.x == 0) out[blockIdx.x] = bi[0] == 0x7fffffff ? 0 : bi[0];
}

extern "C" int jllm_argmax(const float* logits, int ld, int n_rows, int vocab, int* out, hipStream_t stream) {
  if (n_rows <= 0) return 0;
  if (vocab <= 0 || ld < vocab) JLLM_FAIL("argmax: vocab %d stride %d", vocab, ld);
  argmax_kernel<<<n_rows, 256, 0, stream>>>(logits, ld, vocab, out);
  JLLM_CHECK_LAUNCH("argmax");
  return 0;
}
