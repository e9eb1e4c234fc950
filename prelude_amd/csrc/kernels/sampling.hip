// Token choice from 32-bit logits: greedy argmax, and a seeded draw from
// softmax(logits / T) restricted by top-k and top-p.
//
// Reference: crates/prelude-cuda/src/kernels/kernels_src/sample/fast_argmax_vocab.cu:38-47,
// :76-188 (ties go to the smaller index); the draw follows
// crates/prelude-core/src/engine/sampling/logits_processor.rs:51-136: softmax
// over the whole vocabulary in 32-bit, keep the k largest, then keep the
// shortest descending prefix whose mass reaches p, draw from what is left in
// proportion to its weight.  The reference does this on the host with a
// sorted copy; here one block per row finds the two thresholds by a search
// over the order-preserving integer image of the floats, four bits a pass
// (eight passes each over a row that stays in cache), so nothing is sorted
// and nothing leaves the device.  Entries equal to a threshold are all kept (a sort would keep some).
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

// exp((x - mx) / T) as one hardware exponential: inv_t holds log2(e) / T.  (The library's expf is thirty
// instructions; a pass over a row is bound by the vector units of the one compute unit that works on it.)
__device__ __forceinline__ float weight_of(float x, float mx, float inv_t) {
  return __builtin_amdgcn_exp2f((x - mx) * inv_t);
}

constexpr int kSampleThreads = 1024;
constexpr int kSampleWaves = kSampleThreads / kWave;
constexpr int kDigitBits = 4, kBuckets = 1 << kDigitBits;

// What the block of a row shares.  `bins` gives every thread a column of its own per bucket, so the sums a
// search pass takes are formed without atomics and in the same order whenever the row is the same.
struct SampleLds {
  float bins[kBuckets][kSampleThreads];
  float red[kSampleWaves][kBuckets];
  float wave_v[kSampleWaves];
  int wave_i[kSampleWaves];
  float scratch[16];
  float pick_before;
  int pick_range;
};

// f(value, index) for the entries begin + first, begin + first + stride, ... below end, `first` counted in
// vectors of four when the stretch allows 16-byte loads (begin and the row 16-byte aligned) and in single
// entries otherwise; eight loads are on their way before the first value is used.  One load in flight per
// thread would make a pass over a 600 KB row 150 round trips to L2.
template <typename F>
__device__ __forceinline__ void walk(const float* row, int begin, int end, int first, int stride, F f) {
  constexpr int U = 8;
  const bool wide = (reinterpret_cast<size_t>(row + begin) & 15) == 0;
  if (wide) {
    const f32x4* r4 = reinterpret_cast<const f32x4*>(row + begin);
    const int n4 = (end - begin) / 4;
    for (int b = first; b < n4; b += stride * U) {
      f32x4 v[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int idx = b + u * stride;
        v[u] = idx < n4 ? r4[idx] : f32x4{0.f, 0.f, 0.f, 0.f};
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int idx = b + u * stride;
        if (idx < n4) {
#pragma unroll
          for (int e = 0; e < 4; ++e) f(v[u][e], begin + 4 * idx + e);
        }
      }
    }
    begin += 4 * n4;   // up to three entries are left
  }
  for (int b = begin + first; b < end; b += stride * U) {
    float v[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int idx = b + u * stride;
      v[u] = idx < end ? row[idx] : 0.f;
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int idx = b + u * stride;
      if (idx < end) f(v[u], idx);
    }
  }
}

// Largest key t such that measure{ i : key_i >= t and key_i >= floor_key } >= target, where measure counts
// entries (kWeights false) or sums the weights exp((x - mx) / T); 0 if even all entries measure less.  The key is
// settled four bits at a time from the top: a pass over the row sorts the entries that agree with the bits
// settled so far into the sixteen values of the next digit, and the largest digit whose entries, with all
// above them, reach the target is taken.  Eight passes instead of one per bit.
template <bool kWeights>
__device__ unsigned threshold_search(const float* row, int vocab, unsigned floor_key, float target, float mx,
                                     float inv_t, SampleLds& lds) {
  const int tid = threadIdx.x, lane = tid % kWave, wave = tid / kWave;
  unsigned prefix = 0;
  float above = 0.f;   // measure of the entries whose settled bits are greater than the prefix's
  for (int shift = 32 - kDigitBits; shift >= 0; shift -= kDigitBits) {
#pragma unroll
    for (int b = 0; b < kBuckets; ++b) lds.bins[b][tid] = 0.f;
    const unsigned settled = shift + kDigitBits >= 32 ? 0u : ~0u << (shift + kDigitBits);
    walk(row, 0, vocab, tid, kSampleThreads, [&](float x, int) {
      const unsigned k = order_key(x);
      if (k >= floor_key && (k & settled) == prefix)
        lds.bins[(k >> shift) & (kBuckets - 1)][tid] += kWeights ? weight_of(x, mx, inv_t) : 1.0f;
    });
#pragma unroll
    for (int b = 0; b < kBuckets; ++b) {
      const float v = wave_sum(lds.bins[b][tid]);
      if (lane == 0) lds.red[wave][b] = v;
    }
    __syncthreads();
    float run = above;
    int digit = -1;
    for (int b = kBuckets - 1; b >= 0; --b) {   // the same in every thread
      float sb = 0.f;
#pragma unroll
      for (int w = 0; w < kSampleWaves; ++w) sb += lds.red[w][b];
      if (digit < 0) {
        if (run + sb >= target) {
          digit = b;
        } else {
          run += sb;
        }
      }
    }
    __syncthreads();   // red is written again in the next pass
    if (digit < 0) return 0u;
    above = run;
    prefix |= (unsigned)digit << shift;
  }
  return prefix;
}

__device__ __forceinline__ float wave_scan_inclusive(float v, int lane) {
#pragma unroll
  for (int off = 1; off < kWave; off <<= 1) {
    const float o = __shfl_up(v, off, kWave);
    if (lane >= off) v += o;
  }
  return v;
}

__global__ __launch_bounds__(kSampleThreads) void sample_kernel(const float* __restrict__ logits, int vocab,
                                                                const float* __restrict__ temperature,
                                                                const int* __restrict__ top_k,
                                                                const float* __restrict__ top_p,
                                                                const float* __restrict__ uniform,
                                                                int* __restrict__ out) {
  extern __shared__ __align__(16) unsigned char lds_raw[];
  SampleLds& lds = *reinterpret_cast<SampleLds*>(lds_raw);
  const int r = blockIdx.x;
  const float* row = logits + (size_t)r * vocab;
  const float temp = temperature[r];
  const int tid = threadIdx.x, lane = tid % kWave, wave = tid / kWave;

  // maximum and its first index
  MaxIdx best{-INFINITY, 0x7fffffff};
  walk(row, 0, vocab, tid, kSampleThreads, [&](float v, int i) {
    if (v > best.v || (v == best.v && i < best.i)) best = MaxIdx{v, i};
  });
#pragma unroll
  for (int m = kWave / 2; m > 0; m >>= 1) {
    MaxIdx o{__shfl_xor(best.v, m, kWave), __shfl_xor(best.i, m, kWave)};
    best = better(best, o);
  }
  if (lane == 0) {
    lds.wave_v[wave] = best.v;
    lds.wave_i[wave] = best.i;
  }
  __syncthreads();
  best = MaxIdx{lds.wave_v[0], lds.wave_i[0]};
  for (int w = 1; w < kSampleWaves; ++w) best = better(best, MaxIdx{lds.wave_v[w], lds.wave_i[w]});
  const int arg = best.i == 0x7fffffff ? 0 : best.i;
  if (!(temp >= 1e-7f)) {  // greedy (crates/prelude-core/src/engine/model_runner/postprocess.rs:18-37)
    if (tid == 0) out[r] = arg;
    return;
  }
  const float mx = best.v, inv_t = 1.4426950408889634f / temp;
  __syncthreads();   // wave_v and wave_i are used again below

  unsigned floor_key = 0;
  const int k = top_k[r];
  if (k > 0 && k < vocab) floor_key = threshold_search<false>(row, vocab, 0u, (float)k, mx, inv_t, lds);

  const float p = top_p[r];
  if (p > 0.f && p < 1.f) {
    float z = 0.f;
    walk(row, 0, vocab, tid, kSampleThreads, [&](float x, int) { z += weight_of(x, mx, inv_t); });
    z = block_sum(z, lds.scratch);
    const unsigned t = threshold_search<true>(row, vocab, floor_key, p * z, mx, inv_t, lds);
    // t == 0 means even everything kept so far weighs less than p: keep it all
    if (t > floor_key) floor_key = t;
  }

  // The draw: the first index, in index order, at which the running weight of the kept entries passes
  // uniform * total.  The row is cut into a stretch per wavefront, then the stretch that holds the target
  // into a stretch per wavefront again, and the last one is walked 64 entries at a time with a prefix sum.
  auto weight = [&](float x) { return order_key(x) >= floor_key ? weight_of(x, mx, inv_t) : 0.f; };
  constexpr int kLast = 16 * kWave;   // a stretch this short is walked by one wavefront
  int begin = 0, end = vocab;
  float before = 0.f, target = 0.f;
  int fallback = arg;   // the last kept entry of the stretch in hand, for a target that rounding puts past it
  for (int level = 0; level == 0 || end - begin > kLast; ++level) {
    const int span = ((end - begin + kSampleWaves * kWave - 1) / (kSampleWaves * kWave)) * kWave;   // per wavefront
    const int wb = begin + wave * span < end ? begin + wave * span : end;
    const int we = wb + span < end ? wb + span : end;
    float sum = 0.f;
    int last = -1;
    walk(row, wb, we, lane, kWave, [&](float x, int i) {
      const float wgt = weight(x);
      sum += wgt;
      if (wgt > 0.f && i > last) last = i;
    });
    sum = wave_sum(sum);
#pragma unroll
    for (int m = kWave / 2; m > 0; m >>= 1) {
      const int o = __shfl_xor(last, m, kWave);
      last = o > last ? o : last;
    }
    if (lane == 0) {
      lds.wave_v[wave] = sum;
      lds.wave_i[wave] = last;
    }
    __syncthreads();
    if (level == 0) {
      float total = 0.f;
      for (int w = 0; w < kSampleWaves; ++w) total += lds.wave_v[w];
      target = uniform[r] * total;
    }
    int pick = -1;
    float run = before;
    int last_kept = -1;
    for (int w = 0; w < kSampleWaves; ++w) {   // the same in every thread
      if (lds.wave_i[w] > last_kept) last_kept = lds.wave_i[w];
      if (pick < 0) {
        if (run + lds.wave_v[w] > target) {
          pick = w;
        } else {
          run += lds.wave_v[w];
        }
      }
    }
    if (last_kept < 0) last_kept = fallback;
    const int pick_last = pick >= 0 ? lds.wave_i[pick] : -1;
    __syncthreads();   // wave_v and wave_i are written again at the next level
    if (pick < 0) {   // rounding left the target at or past the total: the last kept entry
      if (tid == 0) out[r] = last_kept;
      return;
    }
    before = run;
    fallback = pick_last >= 0 ? pick_last : fallback;
    begin = begin + pick * span;
    end = begin + span < end ? begin + span : end;
  }
  if (wave != 0) return;
  // at most sixteen groups of 64 entries, all asked for at once, then a prefix sum per group
  float wgt[kLast / kWave];
#pragma unroll
  for (int j = 0; j < kLast / kWave; ++j) {
    const int i = begin + j * kWave + lane;
    wgt[j] = i < end ? row[i] : -INFINITY;
  }
  float cum = before;
#pragma unroll
  for (int j = 0; j < kLast / kWave; ++j) {
    if (begin + j * kWave >= end) break;
    const float c = cum + wave_scan_inclusive(wgt[j] == -INFINITY ? 0.f : weight(wgt[j]), lane);
    const unsigned long long hit = __ballot(c > target);
    if (hit) {
      if (lane == 0) out[r] = begin + j * kWave + __builtin_ctzll(hit);
      return;
    }
    cum = __shfl(c, kWave - 1, kWave);
  }
  if (lane == 0) out[r] = fallback;
}

}  // namespace pa

using namespace pa;

extern "C" int pa_sample(void* stream, const float* logits, const float* temperature, const int* top_k,
                         const float* top_p, const float* uniform, int* out, int rows, int vocab) {
  if (rows == 0) return 0;
  PA_REQUIRE(rows > 0 && vocab > 0, "sample: bad sizes rows=%d vocab=%d", rows, vocab);
  // the per-thread bins are more than the 64 KB a kernel may declare: asked for at launch, allowed once
  static const hipError_t allowed = hipFuncSetAttribute(reinterpret_cast<const void*>(&sample_kernel),
                                                        hipFuncAttributeMaxDynamicSharedMemorySize,
                                                        (int)sizeof(SampleLds));
  if (allowed != hipSuccess)
    return pa::fail("sample: %zu bytes of LDS refused: %s", sizeof(SampleLds), hipGetErrorString(allowed));
  hipLaunchKernelGGL(sample_kernel, dim3(rows), dim3(kSampleThreads), sizeof(SampleLds), (hipStream_t)stream, logits,
                     vocab, temperature, top_k, top_p, uniform, out);
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
