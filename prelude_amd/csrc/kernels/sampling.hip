// Token choice from 32-bit logits: greedy argmax, and a seeded draw from
// softmax(logits / T) restricted by top-k and top-p.
//
// Reference: crates/prelude-cuda/src/kernels/kernels_src/sample/fast_argmax_vocab.cu:38-47,
// :76-188 (ties go to the smaller index); the draw follows
// crates/prelude-core/src/engine/sampling/logits_processor.rs:51-136: softmax
// over the whole vocabulary in 32-bit, keep the k largest, then keep the
// shortest descending prefix whose mass reaches p, draw from what is left in
// proportion to its weight.  The reference does this on the host with a
// sorted copy; here one block per row finds the two thresholds by a bitwise
// search over the order-preserving integer image of the floats (32 counting
// passes each, all in cache), so nothing is sorted and nothing leaves the
// device.  Entries equal to a threshold are all kept (a sort would keep some).
// The draw is the inverse CDF in index order at a uniform number the host
// supplies per row, which makes it reproducible and testable.
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

// Wide rows: grid (rows, chunks) writes one candidate per chunk, a second launch picks among them.
__global__ __launch_bounds__(256) void argmax_chunks_kernel(const float* __restrict__ logits, float* __restrict__ cand_v,
                                                          int* __restrict__ cand_i, int vocab, int chunk) {
  __shared__ float sv[4];
  __shared__ int si[4];
  const float* row = logits + (size_t)blockIdx.x * vocab;
  const int begin = blockIdx.y * chunk;
  const int end = begin + chunk < vocab ? begin + chunk : vocab;
  MaxIdx best{-INFINITY, 0x7fffffff};
  for (int i = begin + threadIdx.x; i < end; i += blockDim.x) {
    const float v = row[i];
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
    for (int w = 1; w < 4; ++w) best = better(best, MaxIdx{sv[w], si[w]});
    cand_v[blockIdx.x * gridDim.y + blockIdx.y] = best.v;
    cand_i[blockIdx.x * gridDim.y + blockIdx.y] = best.i;
  }
}

__global__ __launch_bounds__(kWave) void argmax_pick_kernel(const float* __restrict__ cand_v,
                                                            const int* __restrict__ cand_i, int* __restrict__ out,
                                                            int chunks) {
  MaxIdx best{-INFINITY, 0x7fffffff};
  for (int c = threadIdx.x; c < chunks; c += kWave)
    best = better(best, MaxIdx{cand_v[blockIdx.x * chunks + c], cand_i[blockIdx.x * chunks + c]});
#pragma unroll
  for (int m = kWave / 2; m > 0; m >>= 1) {
    MaxIdx o{__shfl_xor(best.v, m, kWave), __shfl_xor(best.i, m, kWave)};
    best = better(best, o);
  }
  if (threadIdx.x == 0) out[blockIdx.x] = best.i == 0x7fffffff ? 0 : best.i;
}

__device__ __forceinline__ unsigned order_key(float v) {
  const unsigned u = __float_as_uint(v);
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

constexpr int kSampleThreads = 1024;

// Largest key t such that measure{ i : key_i >= t and key_i >= floor_key } >= target,
// where measure counts entries (weights == false) or sums exp((x - mx) * inv_t).
template <bool kWeights>
__device__ unsigned threshold_search(const float* row, int vocab, unsigned floor_key, float target, float mx,
                                     float inv_t, float* scratch) {
  unsigned t = 0;
  for (int bit = 31; bit >= 0; --bit) {
    const unsigned cand = t | (1u << bit);
    float acc = 0.f;
    for (int i = threadIdx.x; i < vocab; i += blockDim.x) {
      const float x = row[i];
      const unsigned k = order_key(x);
      if (k >= cand && k >= floor_key) acc += kWeights ? expf((x - mx) * inv_t) : 1.0f;
    }
    acc = block_sum(acc, scratch);
    if (acc >= target) t = cand;
  }
  return t;
}

__global__ __launch_bounds__(kSampleThreads) void sample_kernel(const float* __restrict__ logits, int vocab,
                                                                const float* __restrict__ temperature,
                                                                const int* __restrict__ top_k,
                                                                const float* __restrict__ top_p,
                                                                const float* __restrict__ uniform,
                                                                int* __restrict__ out) {
  __shared__ float scratch[16];
  __shared__ float sv[16];
  __shared__ int si[16];
  __shared__ float partial[kSampleThreads];
  __shared__ int pick_thread;
  __shared__ float pick_before;
  const int r = blockIdx.x;
  const float* row = logits + (size_t)r * vocab;
  const float temp = temperature[r];

  // maximum and its first index
  MaxIdx best{-INFINITY, 0x7fffffff};
  for (int i = threadIdx.x; i < vocab; i += blockDim.x) {
    const float v = row[i];
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
  best = MaxIdx{sv[0], si[0]};
  for (int w = 1; w < kSampleThreads / kWave; ++w) best = better(best, MaxIdx{sv[w], si[w]});
  const int arg = best.i == 0x7fffffff ? 0 : best.i;
  if (!(temp >= 1e-7f)) {  // greedy (crates/prelude-core/src/engine/model_runner/postprocess.rs:18-37)
    if (threadIdx.x == 0) out[r] = arg;
    return;
  }
  const float mx = best.v, inv_t = 1.0f / temp;

  unsigned floor_key = 0;
  const int k = top_k[r];
  if (k > 0 && k < vocab) floor_key = threshold_search<false>(row, vocab, 0u, (float)k, mx, inv_t, scratch);

  const float p = top_p[r];
  if (p > 0.f && p < 1.f) {
    float z = 0.f;
    for (int i = threadIdx.x; i < vocab; i += blockDim.x) z += expf((row[i] - mx) * inv_t);
    z = block_sum(z, scratch);
    const unsigned t = threshold_search<true>(row, vocab, floor_key, p * z, mx, inv_t, scratch);
    // t == 0 means even everything kept so far weighs less than p: keep it all
    if (t > floor_key) floor_key = t;
  }

  // inverse CDF over the kept entries in index order; each thread owns a contiguous run
  const int chunk = (vocab + kSampleThreads - 1) / kSampleThreads;
  const int begin = threadIdx.x * chunk;
  const int end = begin + chunk < vocab ? begin + chunk : vocab;
  float mine = 0.f;
  for (int i = begin; i < end; ++i) {
    const float x = row[i];
    if (order_key(x) >= floor_key) mine += expf((x - mx) * inv_t);
  }
  partial[threadIdx.x] = mine;
  __syncthreads();
  if (threadIdx.x == 0) {
    float total = 0.f;
    for (int t = 0; t < kSampleThreads; ++t) total += partial[t];
    const float target = uniform[r] * total;
    float before = 0.f;
    int who = -1, last_nonzero = 0;
    for (int t = 0; t < kSampleThreads; ++t) {
      if (partial[t] > 0.f) last_nonzero = t;
      if (who < 0 && before + partial[t] > target) {
        who = t;
        pick_before = before;
      }
      if (who < 0) before += partial[t];
    }
    if (who < 0) {  // rounding left the target at or past the total: the last kept entry
      who = last_nonzero;
      pick_before = -1.f;
    }
    pick_thread = who;
    scratch[0] = target;
  }
  __syncthreads();
  if ((int)threadIdx.x == pick_thread) {
    const float target = scratch[0];
    float cum = pick_before;
    int chosen = -1, last_kept = arg;
    for (int i = begin; i < end; ++i) {
      const float x = row[i];
      if (order_key(x) < floor_key) continue;
      last_kept = i;
      if (pick_before < 0.f) continue;
      cum += expf((x - mx) * inv_t);
      if (cum > target) {
        chosen = i;
        break;
      }
    }
    out[r] = chosen >= 0 ? chosen : last_kept;
  }
}

}  // namespace pa

using namespace pa;

extern "C" int pa_sample(void* stream, const float* logits, const float* temperature, const int* top_k,
                         const float* top_p, const float* uniform, int* out, int rows, int vocab) {
  if (rows == 0) return 0;
  PA_REQUIRE(rows > 0 && vocab > 0, "sample: bad sizes rows=%d vocab=%d", rows, vocab);
  hipLaunchKernelGGL(sample_kernel, dim3(rows), dim3(kSampleThreads), 0, (hipStream_t)stream, logits, vocab,
                     temperature, top_k, top_p, uniform, out);
  return check_launch("sample");
}

// Floats of scratch pa_argmax needs for rows of this width (0: none).
extern "C" int pa_argmax_scratch(int rows, int vocab) {
  return vocab <= 8192 ? 0 : rows * ((vocab + 2047) / 2048) * 2;
}

extern "C" int pa_argmax(void* stream, const float* logits, int* out, float* scratch, int rows, int vocab) {
  if (rows == 0) return 0;
  PA_REQUIRE(rows > 0 && vocab > 0, "argmax: bad sizes rows=%d vocab=%d", rows, vocab);
  if (vocab <= 8192) {
    hipLaunchKernelGGL(argmax_kernel, dim3(rows), dim3(1024), 0, (hipStream_t)stream, logits, out, vocab);
    return check_launch("argmax");
  }
  PA_REQUIRE(scratch, "argmax: rows of %d need scratch", vocab);
  const int chunks = (vocab + 2047) / 2048;
  PA_REQUIRE(chunks <= 65535, "argmax: %d columns exceed the grid", vocab);
  float* cand_v = scratch;
  int* cand_i = reinterpret_cast<int*>(scratch + (size_t)rows * chunks);
  hipLaunchKernelGGL(argmax_chunks_kernel, dim3(rows, chunks), dim3(256), 0, (hipStream_t)stream, logits, cand_v, cand_i,
                     vocab, 2048);
  if (int rc = check_launch("argmax")) return rc;
  hipLaunchKernelGGL(argmax_pick_kernel, dim3(rows), dim3(kWave), 0, (hipStream_t)stream, cand_v, cand_i, out, chunks);
  return check_launch("argmax");
}
