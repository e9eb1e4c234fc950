// A measurement, not an op: do a SIMD's matrix products and its vector instructions run at the same time?
//
// A workgroup of eight wavefronts (two a SIMD) repeats a phase of 34 MFMAs 16x16x32 (eight accumulators, four
// products deep each, and two more: what an attention step of two heads and 32 keys issues) and a phase of 64
// vector instructions, 16 of them exponentials (that step's softmax).  What the phases take alone and together,
// with the two wavefronts of a SIMD in the same order or held in opposite phases by barriers, says how much of the
// vector work can hide behind the products: `python -m prelude_amd.bench_kernels overlap`.
#include "common.h"
#include "api.h"

namespace pa {

// order 0: every wavefront products then vector work, no barrier; 1: the same with a barrier after each phase;
// 2: the wavefronts 4..7 start with the vector work, so that a SIMD's two wavefronts are in opposite phases, a
// barrier after each phase; 3: as 2, the products at raised priority; 4: products only; 5: vector work only.
// ACC: the products' accumulators in the accumulation registers (only the matrix instructions touch them then).
template <int ORDER, bool ACC>
__global__ __launch_bounds__(512, 2) void overlap_probe_kernel(float* out, int iters, float seed) {
  const bool second = threadIdx.x / kWave >= 4;
  bf16x8 a, b;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    a[i] = from_f32<bf16>(seed + (float)i);
    b[i] = from_f32<bf16>(seed * 0.5f + (float)threadIdx.x);
  }
  f32x4 acc[9];
#pragma unroll
  for (int i = 0; i < 9; ++i) acc[i] = f32x4{0.f, 0.f, 0.f, 0.f};
  float s[16];
#pragma unroll
  for (int i = 0; i < 16; ++i) s[i] = seed * (float)i;
  float mx = 0.f;
  auto product = [&](f32x4& c, const bf16x8& x, const bf16x8& y) {
    if (ACC) {
      asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(c) : "v"(x), "v"(y));
    } else {
      c = __builtin_amdgcn_mfma_f32_16x16x32_bf16(x, y, c, 0, 0, 0);
    }
  };
  auto products = [&]() {
    if (ORDER == 3) __builtin_amdgcn_s_setprio(1);
#pragma unroll
    for (int r = 0; r < 4; ++r)
#pragma unroll
      for (int t = 0; t < 8; ++t) product(acc[t], a, b);
    product(acc[8], a, b);
    product(acc[8], b, a);
    if (ORDER == 3) __builtin_amdgcn_s_setprio(0);
  };
  auto vector_work = [&]() {
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      mx = fmaxf(mx, s[i]);
      s[i] = __builtin_amdgcn_exp2f(s[i] * 0.99f - mx);
      s[i] = s[i] * 1.0001f;
    }
  };
  for (int it = 0; it < iters; ++it) {
    if (ORDER == 4) {
      products();
    } else if (ORDER == 5) {
      vector_work();
    } else if (ORDER <= 1) {
      products();
      if (ORDER == 1) __builtin_amdgcn_s_barrier();
      vector_work();
      if (ORDER == 1) __builtin_amdgcn_s_barrier();
    } else {
      if (!second) products(); else vector_work();
      __builtin_amdgcn_s_barrier();
      if (!second) vector_work(); else products();
      __builtin_amdgcn_s_barrier();
    }
  }
  if (ACC) asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");   // the last product's result, before anything reads it
  float r = mx;
#pragma unroll
  for (int i = 0; i < 16; ++i) r += s[i];
#pragma unroll
  for (int i = 0; i < 9; ++i) r += acc[i][0] + acc[i][3];
  if (r == 12345.678f) out[threadIdx.x] = r;   // (almost) never: keeps the work from being dropped
}

}  // namespace pa

using namespace pa;

// Launches the probe on every compute unit (`blocks` workgroups of 512 threads); out: 512 floats.
extern "C" int pa_overlap_probe(void* stream, int order, int accumulators, int iters, int blocks, void* out) {
  PA_REQUIRE(order >= 0 && order <= 5 && iters > 0 && iters <= (1 << 20) && blocks > 0 && blocks <= 4096 && out,
             "overlap_probe: order %d (0..5), %d iterations, %d workgroups", order, iters, blocks);
  hipStream_t st = (hipStream_t)stream;
#define PA_PROBE(O)                                                                                                  \
  case O:                                                                                                            \
    if (accumulators)                                                                                                \
      hipLaunchKernelGGL((overlap_probe_kernel<O, true>), dim3(blocks), dim3(512), 0, st, (float*)out, iters, 1.0f); \
    else                                                                                                             \
      hipLaunchKernelGGL((overlap_probe_kernel<O, false>), dim3(blocks), dim3(512), 0, st, (float*)out, iters, 1.0f); \
    break;
  switch (order) {
    PA_PROBE(0)
    PA_PROBE(1)
    PA_PROBE(2)
    PA_PROBE(3)
    PA_PROBE(4)
    PA_PROBE(5)
  }
#undef PA_PROBE
  return check_launch("overlap_probe");
}
