// Token choice from 32-bit logits: greedy argmax.
//
// Reference: crates/prelude-cuda/src/kernels/kernels_src/sample/fast_argmax_vocab.cu:38-47,
// :76-188 (ties go to the smaller index).
#include "common.h"
#include "api.h"

namespace pa {

struct MaxIdx {
  float v;
  int i;
};
__device__ __forceinline__ MaxIdx better(MaxIdx a, MaxIdx b) {
  if (b.v > a.v || (b.v == a.v && b.i < a.i)) return b;
  return a;
}

// One block per row.
__global__ __launch_bounds__(1024) void argmax_kernel(const float* __restrict__ logits, int* __restrict__ out,
                                                       int vocab) {
  __shared__ float sv[16];
  __shared__ int si[16];
  const float* row = logits + (size_t)blockIdx.x * vocab;
  MaxIdx best{-INFINITY, 0x7fffffff};
  for (int i = threadIdx.x; i < vocab; i += blockDim.x) {
    const float v = row[i];
    // NaN never wins; a row of only NaN or -inf yields index 0 below
    if (v > best.v || (v == best.v && i < best.i)) best = MaxIdx{v, i};
  }
#pragma unroll
  for (int m = kWave / 2; m > 0; m >>= 1) {
    MaxIdx o{__shfl_xor(best.v, m, kWave), __shfl_xor(best.i, m, kWave)};
    best = better(best, o);
  }
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  if (lane == 0) {
    sv[wave] = best.v;
    si[wave] = best.i;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    const int nw = (blockDim.x + kWave - 1) / kWave;
    for (int w = 1; w < nw; ++w) best = better(best, MaxIdx{sv[w], si[w]});
    out[blockIdx.x] = best.i == 0x7fffffff ? 0 : best.i;
  }
}

}  // namespace pa

using namespace pa;

extern "C" int pa_argmax(void* stream, const float* logits, int* out, int rows, int vocab) {
  if (rows == 0) return 0;
  PA_REQUIRE(rows > 0 && vocab > 0, "argmax: bad sizes rows=%d vocab=%d", rows, vocab);
  hipLaunchKernelGGL(argmax_kernel, dim3(rows), dim3(1024), 0, (hipStream_t)stream, logits, out, vocab);
  return check_launch("argmax");
}
