// Shared device helpers for the gfx950 kernels: element types, conversions,
// wavefront (64 lanes) and block reductions, and the host-side error channel.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace pa {

constexpr int kWave = 64;

typedef __bf16 bf16;
typedef bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

// Element type codes shared with the Python side.
enum DType : int { kF32 = 0, kBF16 = 1 };

// The activation of a gated feed-forward act(gate) * up, by a code shared with the Python side: SiLU
// x / (1 + e^-x) (crates/prelude-cuda/src/kernels/kernels_src/common/common.cuh:78-80, what the reference's Qwen3
// is wired to, qwen3.rs:429-447) or GELU in its tanh form 0.5 x (1 + tanh(sqrt(2 / pi) (x + 0.044715 x^3))) (the
// reference's Activation::GeluPytorchTanh, crates/prelude-core/src/models/commons/activation.rs:3-25).  The code
// is the same in every lane, so the choice is a branch, and SiLU's arithmetic is what it was without it.
enum GateActivation : int { kActSilu = 0, kActGeluTanh = 1, kActCount = 2 };
__device__ __forceinline__ float gate_activation(float x, int act) {
  if (act == kActGeluTanh) return 0.5f * x * (1.0f + tanhf(0.7978845608028654f * (x + 0.044715f * x * x * x)));
  return x / (1.0f + expf(-x));
}

__device__ __forceinline__ float to_f32(float v) { return v; }
__device__ __forceinline__ float to_f32(bf16 v) { return static_cast<float>(v); }
template <typename T> __device__ __forceinline__ T from_f32(float v);
template <> __device__ __forceinline__ float from_f32<float>(float v) { return v; }
template <> __device__ __forceinline__ bf16 from_f32<bf16>(float v) { return static_cast<bf16>(v); }  // round to nearest even

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int m = kWave / 2; m > 0; m >>= 1) v += __shfl_xor(v, m, kWave);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int m = kWave / 2; m > 0; m >>= 1) v = fmaxf(v, __shfl_xor(v, m, kWave));
  return v;
}

// Sum over a block of up to 1024 threads; every thread gets the result.
// `scratch` is LDS for at least 16 floats.  The order of the additions is
// fixed by the thread layout alone, so a row's result never depends on what
// else the launch holds.
__device__ __forceinline__ float block_sum(float v, float* scratch) {
  v = wave_sum(v);
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const int nwaves = (blockDim.x + kWave - 1) / kWave;
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  float t = 0.f;
  for (int i = 0; i < nwaves; ++i) t += scratch[i];
  return t;
}

}  // namespace pa

// ---- host side -----------------------------------------------------------
// Every entry point returns 0 on success.  On a refusal (a size the kernel
// does not take, a launch error) it returns nonzero and leaves a message for
// pa_last_error().
extern "C" const char* pa_last_error();
namespace pa {
int fail(const char* fmt, ...);
int check_launch(const char* what);
}  // namespace pa

#define PA_REQUIRE(cond, ...)                  \
  do {                                         \
    if (!(cond)) return pa::fail(__VA_ARGS__); \
  } while (0)
