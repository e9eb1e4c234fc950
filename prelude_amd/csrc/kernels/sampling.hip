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

#include <mutex>

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
    // bucket b is added up by wavefront b: sixteen columns a lane, then one sum over the wavefront (sixteen
    // wavefront-wide sums in a row would each wait for six exchanges)
    __syncthreads();
    {
      static_assert(kSampleWaves == kBuckets, "a wavefront a bucket");
      float v = 0.f;
#pragma unroll
      for (int j = 0; j < kSampleThreads / kWave; ++j) v += lds.bins[wave][lane * (kSampleThreads / kWave) + j];
      v = wave_sum(v);
      if (lane == 0) lds.red[0][wave] = v;
    }
    __syncthreads();
    float run = above;
    int digit = -1;
    for (int b = kBuckets - 1; b >= 0; --b) {   // the same in every thread
      const float sb = lds.red[0][b];
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

// The draw: the first index, in index order, at which the running weight of the kept entries passes the target.
// The stretch [begin, end) is cut into a stretch per wavefront, the one that holds the target into a stretch per
// wavefront again, until one is short enough to be walked 64 entries at a time with a prefix sum.
// `fresh`: the target is uniform * (the stretch's total), found at the first level; else `target` is given and
// `before` is the weight that lies before the stretch.  `fallback` is the last kept entry of the stretch (any
// kept entry at the start), taken when rounding puts the target at or past the total.
// Every thread of the WAVES wavefronts calls this; wave_v / wave_i are LDS arrays of WAVES entries.
template <int WAVES>
__device__ void draw_from(const float* row, int begin, int end, float before, float target, bool fresh, int fallback,
                          unsigned floor_key, float mx, float inv_t, float* wave_v, int* wave_i, int* out) {
  const int tid = threadIdx.x, lane = tid % kWave, wave = tid / kWave;
  auto weight = [&](float x) { return order_key(x) >= floor_key ? weight_of(x, mx, inv_t) : 0.f; };
  constexpr int kLast = 16 * kWave;   // a stretch this short is walked by one wavefront
  for (int level = 0; (level == 0 && fresh) || end - begin > kLast; ++level) {
    const int span = ((end - begin + WAVES * kWave - 1) / (WAVES * kWave)) * kWave;   // per wavefront
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
      wave_v[wave] = sum;
      wave_i[wave] = last;
    }
    __syncthreads();
    if (level == 0 && fresh) {
      float total = 0.f;
      for (int w = 0; w < WAVES; ++w) total += wave_v[w];
      target *= total;
    }
    int pick = -1;
    float run = before;
    int last_kept = -1;
    for (int w = 0; w < WAVES; ++w) {   // the same in every thread
      if (wave_i[w] > last_kept) last_kept = wave_i[w];
      if (pick < 0) {
        if (run + wave_v[w] > target) {
          pick = w;
        } else {
          run += wave_v[w];
        }
      }
    }
    if (last_kept < 0) last_kept = fallback;
    const int pick_last = pick >= 0 ? wave_i[pick] : -1;
    __syncthreads();   // wave_v and wave_i are written again at the next level
    if (pick < 0) {   // rounding left the target at or past the total: the last kept entry
      if (tid == 0) *out = last_kept;
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
      if (lane == 0) *out = begin + j * kWave + __builtin_ctzll(hit);
      return;
    }
    cum = __shfl(c, kWave - 1, kWave);
  }
  if (lane == 0) *out = fallback;
}

// Log-probabilities: lp[r] = logits[r, ids[r]] - logsumexp(logits[r]) (nothing the size of the row is written:
// crates/prelude-cuda/src/kernels/kernels_src/logprobs/gather_log_softmax.cu), and, for k > 0, the entries among
// the k largest of the row with their log-probabilities, ties at the k-th value included, unsorted, at most `cap`
// of them (crates/prelude-core/src/engine/model_runner/postprocess.rs:88-155 sorts a copy of the row on the host).
// ids[r] < 0: no target, lp[r] = 0.  One workgroup a row.
__global__ __launch_bounds__(kSampleThreads) void logprob_kernel(const float* __restrict__ logits, int vocab,
                                                                 const int* __restrict__ ids, int k, int cap,
                                                                 float* __restrict__ lp, float* __restrict__ top_v,
                                                                 int* __restrict__ top_i, int* __restrict__ count) {
  extern __shared__ __align__(16) unsigned char lds_raw[];
  SampleLds& lds = *reinterpret_cast<SampleLds*>(lds_raw);
  const int r = blockIdx.x;
  const float* row = logits + (size_t)r * vocab;
  const int tid = threadIdx.x;
  float mx = -INFINITY;
  walk(row, 0, vocab, tid, kSampleThreads, [&](float v, int) { mx = fmaxf(mx, v); });
  mx = wave_max(mx);
  if (tid % kWave == 0) lds.wave_v[tid / kWave] = mx;
  __syncthreads();
  mx = lds.wave_v[0];
  for (int w = 1; w < kSampleWaves; ++w) mx = fmaxf(mx, lds.wave_v[w]);
  __syncthreads();
  float z = 0.f;
  walk(row, 0, vocab, tid, kSampleThreads, [&](float x, int) { z += expf(x - mx); });
  z = block_sum(z, lds.scratch);
  const float lse = mx + logf(z);
  if (tid == 0) {
    const int id = ids[r];
    lp[r] = id >= 0 && id < vocab ? row[id] - lse : 0.f;
  }
  if (k <= 0) return;
  const unsigned floor_key = k < vocab ? threshold_search<false>(row, vocab, 0u, (float)k, mx, 1.0f, lds) : 0u;
  if (tid == 0) lds.pick_range = 0;
  __syncthreads();
  walk(row, 0, vocab, tid, kSampleThreads, [&](float x, int i) {
    if (order_key(x) >= floor_key) {
      const int at = atomicAdd(&lds.pick_range, 1);
      if (at < cap) {
        top_v[(size_t)r * cap + at] = x - lse;
        top_i[(size_t)r * cap + at] = i;
      }
    }
  });
  __syncthreads();
  if (tid == 0) count[r] = lds.pick_range < cap ? lds.pick_range : cap;
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

  draw_from<kSampleWaves>(row, 0, vocab, 0.f, uniform[r], true, arg, floor_key, mx, inv_t, lds.wave_v, lds.wave_i,
                          out + r);
}


// ---------------------------------------------------------------------------
// The same choice for long rows, spread over the chip.  One compute unit reads a 600 KB row in about 20 us
// however it is programmed (its outstanding misses bound it), and a draw with top-k and top-p needs some
// twenty passes.  Here every pass is a launch of rows x slices workgroups, each reading a slice of a row and
// leaving partial results; the next launch begins by adding the partials up, slice by slice in order, so every
// workgroup of a row reaches the same decision and the result does not depend on the launch shape's timing.
// What a row has settled so far travels in WideState; it and the partial results are read from one copy and
// written to the other, so no workgroup reads what another is writing.
// ---------------------------------------------------------------------------
constexpr int kWideThreads = 256;
constexpr int kWideWaves = kWideThreads / kWave;

struct WideState {
  float mx;            // the row's maximum
  int arg;             // its first index
  unsigned floor_key;  // entries below this key are dropped
  unsigned prefix;     // the threshold search in hand: bits settled so far
  float above;         //   measure of the entries above them
  float target;        //   measure to reach
  float z;             // sum of all weights
  int dead;            // the search in hand cannot reach its target: its threshold is 0
};

enum WidePhase : int { kWideMax = 0, kWideDigit = 1, kWideZ = 2, kWideDraw = 3, kWideFinal = 4 };
enum WidePrev : int { kPrevNone = 0, kPrevMax = 1, kPrevDigit = 2, kPrevZ = 3, kPrevDraw = 4 };

struct WideArgs {
  const float* logits;
  const float* temperature;
  const int* top_k;
  const float* top_p;
  const float* uniform;
  int* out;
  const WideState* state_in;
  WideState* state_out;
  const float* part_in;   // [rows, slices, 16]: what the launch before left
  const int* parti_in;    // [rows, slices]
  float* part_out;        // this launch's
  int* parti_out;
  int vocab, slices, slice_len;
  int phase;       // what this launch computes
  int weights;     //   digit passes: 0 counts (top-k), 1 weights (top-p)
  int shift;       //   digit passes: the digit's lowest bit
  int prev;        // what the launch before it left in part / parti
  int prev_weights, prev_shift;
};

__device__ __forceinline__ bool wide_row_active(int phase, int weights, float temp, int k, float p, int vocab) {
  if (phase == kWideMax) return true;
  if (!(temp >= 1e-7f)) return false;   // greedy rows are done once their maximum is known
  if (phase == kWideDigit && !weights) return k > 0 && k < vocab;
  if (phase == kWideZ || (phase == kWideDigit && weights)) return p > 0.f && p < 1.f;
  return true;
}

// A workgroup's slice of a row, asked for before anything else so that it arrives while the partial results of
// the launch before are being added up: up to kSliceVecs 16-byte loads a thread.  A slice that does not allow
// them (a row that is not 16-byte aligned) is walked afterwards instead.
constexpr int kSliceVecs = 12;
constexpr int kSliceMax = kSliceVecs * 4 * kWideThreads;

struct SliceRegs {
  f32x4 v[kSliceVecs];
  bool held;

  __device__ __forceinline__ void load(const float* row, int begin, int end, int tid) {
    held = (reinterpret_cast<size_t>(row + begin) & 15) == 0 && (end - begin) % 4 == 0 && end - begin <= kSliceMax;
    if (!held) return;
    const f32x4* r4 = reinterpret_cast<const f32x4*>(row + begin);
    const int n4 = (end - begin) / 4;
#pragma unroll
    for (int j = 0; j < kSliceVecs; ++j) {
      const int idx = tid + j * kWideThreads;
      v[j] = idx < n4 ? r4[idx] : f32x4{0.f, 0.f, 0.f, 0.f};
    }
  }

  template <typename F>
  __device__ __forceinline__ void for_each(const float* row, int begin, int end, int tid, F f) const {
    if (!held) {
      walk(row, begin, end, tid, kWideThreads, f);
      return;
    }
    const int n4 = (end - begin) / 4;
#pragma unroll
    for (int j = 0; j < kSliceVecs; ++j) {
      const int idx = tid + j * kWideThreads;
      if (idx < n4) {
#pragma unroll
        for (int e = 0; e < 4; ++e) f(v[j][e], begin + 4 * idx + e);
      }
    }
  }
};

__global__ __launch_bounds__(kWideThreads) void sample_wide_kernel(WideArgs a) {
  __shared__ float bins[kBuckets][kWideThreads];
  __shared__ float segs[kBuckets][kBuckets + 1];
  __shared__ float wave_v[kWideWaves];
  __shared__ int wave_i[kWideWaves];
  __shared__ float scratch[16];
  static_assert(kWideWaves >= 3 && kWideThreads == kBuckets * kBuckets, "the shared arrays double as scratch");
  const int r = blockIdx.y, slice = blockIdx.x;
  const int tid = threadIdx.x, lane = tid % kWave, wave = tid / kWave;
  const float* row = a.logits + (size_t)r * a.vocab;
  const float temp = a.temperature[r];
  const int k = a.top_k[r];
  const float p = a.top_p[r];
  const float* part = a.part_in + (size_t)r * a.slices * kBuckets;
  const int* parti = a.parti_in + (size_t)r * a.slices;
  const int begin = slice * a.slice_len < a.vocab ? slice * a.slice_len : a.vocab;
  const int end = begin + a.slice_len < a.vocab ? begin + a.slice_len : a.vocab;
  SliceRegs mine;
  mine.held = false;
  if (a.phase != kWideFinal && wide_row_active(a.phase, a.weights, temp, k, p, a.vocab)) mine.load(row, begin, end, tid);

  // ---- what the launch before this one found: the slices' partial results, fetched by a thread each (all on
  // their way at once) and combined in a fixed order, the same in every workgroup of the row ----
  WideState st = a.prev == kPrevNone ? WideState{} : a.state_in[r];
  if (a.prev == kPrevMax) {
    if (wave == 0) {
      MaxIdx best = lane < a.slices ? MaxIdx{part[(size_t)lane * kBuckets], parti[lane]} : MaxIdx{-INFINITY, 0x7fffffff};
#pragma unroll
      for (int m = kWave / 2; m > 0; m >>= 1) {
        MaxIdx o{__shfl_xor(best.v, m, kWave), __shfl_xor(best.i, m, kWave)};
        best = better(best, o);
      }
      if (lane == 0) {
        wave_v[0] = best.v;
        wave_i[0] = best.i;
      }
    }
    __syncthreads();
    st.mx = wave_v[0];
    st.arg = wave_i[0] == 0x7fffffff ? 0 : wave_i[0];
    st.floor_key = 0;
    __syncthreads();
    if (!(temp >= 1e-7f) && slice == 0 && tid == 0) a.out[r] = st.arg;   // greedy
  } else if (a.prev == kPrevZ && wide_row_active(kWideZ, 0, temp, k, p, a.vocab)) {
    if (wave == 0) {
      const float z = wave_sum(lane < a.slices ? part[(size_t)lane * kBuckets] : 0.f);
      if (lane == 0) wave_v[0] = z;
    }
    __syncthreads();
    st.z = wave_v[0];
    __syncthreads();
  } else if (a.prev == kPrevDigit && wide_row_active(kWideDigit, a.prev_weights, temp, k, p, a.vocab)) {
    if (!st.dead) {
      // thread (chunk, bucket) adds up every sixteenth slice of its bucket; the chunks are added in order below
      {
        const int b = tid % kBuckets, ch = tid / kBuckets;
        float v = 0.f;
        for (int s = ch; s < a.slices; s += kWideThreads / kBuckets) v += part[(size_t)s * kBuckets + b];
        bins[ch][b] = v;   // bins is free until the pass below
      }
      __syncthreads();
      float run = st.above;
      int digit = -1;
      for (int b = kBuckets - 1; b >= 0; --b) {
        float sb = 0.f;
#pragma unroll
        for (int ch = 0; ch < kWideThreads / kBuckets; ++ch) sb += bins[ch][b];
        if (digit < 0) {
          if (run + sb >= st.target) {
            digit = b;
          } else {
            run += sb;
          }
        }
      }
      __syncthreads();
      if (digit < 0) {
        st.dead = 1;
      } else {
        st.above = run;
        st.prefix |= (unsigned)digit << a.prev_shift;
      }
    }
    if (a.prev_shift == 0) {   // the search is over
      const unsigned t = st.dead ? 0u : st.prefix;
      // top-k: the threshold; top-p: t == 0 means even everything kept so far weighs less than p: keep it all
      if (!a.prev_weights || t > st.floor_key) st.floor_key = t;
    }
  }
  const bool active = wide_row_active(a.phase, a.weights, temp, k, p, a.vocab);
  if (a.phase == kWideDigit && active && a.shift == 32 - kDigitBits) {   // a search begins
    st.prefix = 0;
    st.above = 0.f;
    st.dead = 0;
    st.target = a.weights ? p * st.z : (float)k;
  }
  if (slice == 0 && tid == 0 && a.phase != kWideFinal) a.state_out[r] = st;
  if (!active) return;

  float* my_part = a.part_out + ((size_t)r * a.slices + slice) * kBuckets;
  const float inv_t = 1.4426950408889634f / temp;

  if (a.phase == kWideMax) {
    MaxIdx best{-INFINITY, 0x7fffffff};
    mine.for_each(row, begin, end, tid, [&](float v, int i) {
      if (v > best.v || (v == best.v && i < best.i)) best = MaxIdx{v, i};
    });
#pragma unroll
    for (int m = kWave / 2; m > 0; m >>= 1) {
      MaxIdx o{__shfl_xor(best.v, m, kWave), __shfl_xor(best.i, m, kWave)};
      best = better(best, o);
    }
    if (lane == 0) {
      wave_v[wave] = best.v;
      wave_i[wave] = best.i;
    }
    __syncthreads();
    if (tid == 0) {
      best = MaxIdx{wave_v[0], wave_i[0]};
      for (int w = 1; w < kWideWaves; ++w) best = better(best, MaxIdx{wave_v[w], wave_i[w]});
      my_part[0] = best.v;
      a.parti_out[(size_t)r * a.slices + slice] = best.i;
    }
  } else if (a.phase == kWideDigit) {
    if (st.dead) {   // nothing can change any more; leave zeros so that the next launch adds up nothing new
      if (tid < kBuckets) my_part[tid] = 0.f;
      return;
    }
#pragma unroll
    for (int b = 0; b < kBuckets; ++b) bins[b][tid] = 0.f;
    const unsigned settled = a.shift + kDigitBits >= 32 ? 0u : ~0u << (a.shift + kDigitBits);
    const unsigned prefix = st.prefix, floor_key = st.floor_key;
    const float mx = st.mx;
    const bool weights = a.weights != 0;
    const int shift = a.shift;
    mine.for_each(row, begin, end, tid, [&](float x, int) {
      const unsigned key = order_key(x);
      if (key >= floor_key && (key & settled) == prefix)
        bins[(key >> shift) & (kBuckets - 1)][tid] += weights ? weight_of(x, mx, inv_t) : 1.0f;
    });
    // the bucket sums through LDS in two steps of sixteen (sixteen wavefront-wide sums in a row would each wait
    // for six exchanges)
    __syncthreads();
    {
      const int b = tid / kBuckets, seg = tid % kBuckets;
      float v = 0.f;
#pragma unroll
      for (int j = 0; j < kWideThreads / kBuckets; ++j) v += bins[b][seg * (kWideThreads / kBuckets) + j];
      segs[b][seg] = v;
    }
    __syncthreads();
    if (tid < kBuckets) {
      float v = 0.f;
#pragma unroll
      for (int seg = 0; seg < kBuckets; ++seg) v += segs[tid][seg];
      my_part[tid] = v;
    }
  } else if (a.phase == kWideZ) {
    float z = 0.f;
    const float mx = st.mx;
    mine.for_each(row, begin, end, tid, [&](float x, int) { z += weight_of(x, mx, inv_t); });
    z = block_sum(z, scratch);
    if (tid == 0) my_part[0] = z;
  } else if (a.phase == kWideDraw) {
    float sum = 0.f;
    int last = -1;
    const unsigned floor_key = st.floor_key;
    const float mx = st.mx;
    mine.for_each(row, begin, end, tid, [&](float x, int i) {
      const float wgt = order_key(x) >= floor_key ? weight_of(x, mx, inv_t) : 0.f;
      sum += wgt;
      if (wgt > 0.f && i > last) last = i;
    });
    sum = block_sum(sum, scratch);
#pragma unroll
    for (int m = kWave / 2; m > 0; m >>= 1) {
      const int o = __shfl_xor(last, m, kWave);
      last = o > last ? o : last;
    }
    if (lane == 0) wave_i[wave] = last;
    __syncthreads();
    if (tid == 0) {
      for (int w = 1; w < kWideWaves; ++w) last = wave_i[w] > last ? wave_i[w] : last;
      my_part[0] = sum;
      a.parti_out[(size_t)r * a.slices + slice] = last;
    }
  } else {   // kWideFinal: one workgroup a row (slice 0) picks the slice and walks it
    if (wave == 0) {   // a slice a lane: total, then the first slice at which the running weight passes the target
      const float mine = lane < a.slices ? part[(size_t)lane * kBuckets] : 0.f;
      int last = lane < a.slices ? parti[lane] : -1;
      const float incl = wave_scan_inclusive(mine, lane);
      const float total = __shfl(incl, kWave - 1, kWave);
      const float target = a.uniform[r] * total;
      const unsigned long long hit = __ballot(incl > target && lane < a.slices);
#pragma unroll
      for (int m = kWave / 2; m > 0; m >>= 1) {
        const int o = __shfl_xor(last, m, kWave);
        last = o > last ? o : last;
      }
      const int pick = hit ? __builtin_ctzll(hit) : -1;
      const float before = pick > 0 ? __shfl(incl, pick - 1, kWave) : 0.f;
      const int pick_last = pick >= 0 ? __shfl(lane < a.slices ? parti[lane] : -1, pick, kWave) : -1;
      if (lane == 0) {
        wave_v[0] = target;
        wave_v[1] = before;
        wave_i[0] = pick;
        wave_i[1] = last;
        wave_i[2] = pick_last;
      }
    }
    __syncthreads();
    const float target = wave_v[0], run = wave_v[1];
    const int pick = wave_i[0];
    const int last_kept = wave_i[1] >= 0 ? wave_i[1] : st.arg;   // the maximum is always kept
    const int pick_last = wave_i[2];
    __syncthreads();
    if (pick < 0) {   // rounding left the target at or past the total: the last kept entry
      if (tid == 0) a.out[r] = last_kept;
      return;
    }
    const int pb = pick * a.slice_len;
    const int pe = pb + a.slice_len < a.vocab ? pb + a.slice_len : a.vocab;
    draw_from<kWideWaves>(row, pb, pe, run, target, false, pick_last >= 0 ? pick_last : last_kept, st.floor_key,
                          st.mx, inv_t, wave_v, wave_i, a.out + r);
  }
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

// Slices a row of `vocab` entries is cut into when `rows` rows are sampled by pa_sample_wide, and their length.
static void wide_shape(int rows, int vocab, int* slices, int* slice_len) {
  int want = 1024 / rows;
  want = want < 1 ? 1 : (want > 64 ? 64 : want);
  int len = (vocab + want - 1) / want;
  len = (len + 255) / 256 * 256;   // whole 64-entry groups and 16-byte loads in every slice
  if (len > kSliceMax && (vocab + kSliceMax - 1) / kSliceMax <= 64) len = kSliceMax;   // what a workgroup's registers hold
  *slice_len = len;
  *slices = (vocab + len - 1) / len;
}

// Bytes of workspace pa_sample_wide needs for `rows` rows of `vocab` entries.
extern "C" long pa_sample_wide_workspace(int rows, int vocab) {
  if (rows <= 0 || vocab <= 0) return 0;
  int slices, len;
  wide_shape(rows, vocab, &slices, &len);
  return (long)rows * 2 * (sizeof(WideState) + (size_t)slices * (kBuckets * sizeof(float) + sizeof(int)));
}

// pa_sample for long rows: the same choice (to rounding of the sums), every pass spread over rows x slices
// workgroups.  modes: bit 0 set if some row may have a top-k, bit 1 if some row may have a top-p (the searches
// no row needs are not launched); workspace: pa_sample_wide_workspace bytes, 16-byte aligned.
extern "C" int pa_sample_wide(void* stream, const float* logits, const float* temperature, const int* top_k,
                              const float* top_p, const float* uniform, int* out, void* workspace, int rows,
                              int vocab, int modes) {
  if (rows == 0) return 0;
  PA_REQUIRE(rows > 0 && vocab > 0 && rows <= 65535, "sample_wide: bad sizes rows=%d vocab=%d", rows, vocab);
  PA_REQUIRE(workspace && (reinterpret_cast<size_t>(workspace) & 15) == 0, "sample_wide: no aligned workspace");
  WideArgs a{};
  wide_shape(rows, vocab, &a.slices, &a.slice_len);
  WideState* states = reinterpret_cast<WideState*>(workspace);
  float* parts = reinterpret_cast<float*>(states + 2 * (size_t)rows);
  const size_t part_words = (size_t)rows * a.slices * kBuckets, parti_words = (size_t)rows * a.slices;
  int* partis = reinterpret_cast<int*>(parts + 2 * part_words);
  a.logits = logits, a.temperature = temperature, a.top_k = top_k, a.top_p = top_p, a.uniform = uniform, a.out = out;
  a.vocab = vocab;
  int flip = 0;
  hipStream_t st = (hipStream_t)stream;
  auto launch = [&](int phase, int weights, int shift) {
    a.phase = phase, a.weights = weights, a.shift = shift;
    a.state_in = states + (size_t)flip * rows;
    a.state_out = states + (size_t)(flip ^ 1) * rows;
    a.part_in = parts + flip * part_words, a.part_out = parts + (flip ^ 1) * part_words;
    a.parti_in = partis + flip * parti_words, a.parti_out = partis + (flip ^ 1) * parti_words;
    const dim3 grid(phase == kWideFinal ? 1 : a.slices, rows);
    hipLaunchKernelGGL(sample_wide_kernel, grid, dim3(kWideThreads), 0, st, a);
    if (phase != kWideFinal) flip ^= 1;
    a.prev = phase == kWideMax ? kPrevMax : phase == kWideDigit ? kPrevDigit : phase == kWideZ ? kPrevZ : kPrevDraw;
    a.prev_weights = weights, a.prev_shift = shift;
  };
  a.prev = kPrevNone;
  launch(kWideMax, 0, 0);
  if (modes & 1)
    for (int shift = 32 - kDigitBits; shift >= 0; shift -= kDigitBits) launch(kWideDigit, 0, shift);
  if (modes & 2) {
    launch(kWideZ, 0, 0);
    for (int shift = 32 - kDigitBits; shift >= 0; shift -= kDigitBits) launch(kWideDigit, 1, shift);
  }
  launch(kWideDraw, 0, 0);
  launch(kWideFinal, 0, 0);
  return check_launch("sample_wide");
}

// lp[r] = log-probability of ids[r] in softmax(logits[r]); for k > 0 also the entries among the row's k largest
// (ties included, unsorted, at most cap): top_v / top_i [rows, cap] and count[rows].
extern "C" int pa_logprobs(void* stream, const float* logits, const int* ids, float* lp, float* top_v, int* top_i,
                           int* count, int rows, int vocab, int k, int cap) {
  if (rows == 0) return 0;
  PA_REQUIRE(rows > 0 && vocab > 0 && k >= 0, "logprobs: bad sizes rows=%d vocab=%d k=%d", rows, vocab, k);
  PA_REQUIRE(k == 0 || (top_v && top_i && count && cap >= k), "logprobs: no room for the %d largest (cap %d)", k, cap);
  static const hipError_t allowed = hipFuncSetAttribute(reinterpret_cast<const void*>(&logprob_kernel),
                                                        hipFuncAttributeMaxDynamicSharedMemorySize,
                                                        (int)sizeof(SampleLds));
  if (allowed != hipSuccess)
    return pa::fail("logprobs: %zu bytes of LDS refused: %s", sizeof(SampleLds), hipGetErrorString(allowed));
  hipLaunchKernelGGL(logprob_kernel, dim3(rows), dim3(kSampleThreads), sizeof(SampleLds), (hipStream_t)stream, logits,
                     vocab, ids, k, cap, lp, top_v, top_i, count);
  return check_launch("logprobs");
}

// Floats of scratch pa_argmax needs for rows of this width (0: none).
extern "C" int pa_argmax_scratch(int rows, int vocab) {
  return vocab <= 8192 ? 0 : rows * ((vocab + 2047) / 2048) * 2;
}

// The launches of an argmax: a workgroup a row for narrow rows; for wide ones a candidate per 2,048-entry chunk
// into `scratch` (values, then indices), and a second launch that picks among them.  Every word of `scratch`
// the second launch reads has been written by the first, so it need not start at any value.
static int argmax_launch(hipStream_t st, const float* logits, int* out, float* scratch, int rows, int vocab) {
  if (vocab <= 8192) {
    hipLaunchKernelGGL(argmax_kernel, dim3(rows), dim3(1024), 0, st, logits, out, vocab);
    return check_launch("argmax");
  }
  PA_REQUIRE(scratch, "argmax: rows of %d need scratch", vocab);
  const int chunks = (vocab + 2047) / 2048;
  PA_REQUIRE(chunks <= 65535, "argmax: %d columns exceed the grid", vocab);
  float* cand_v = scratch;
  int* cand_i = reinterpret_cast<int*>(scratch + (size_t)rows * chunks);
  hipLaunchKernelGGL(argmax_chunks_kernel, dim3(rows, chunks), dim3(256), 0, st, logits, cand_v, cand_i, vocab, 2048);
  if (int rc = check_launch("argmax")) return rc;
  hipLaunchKernelGGL(argmax_pick_kernel, dim3(rows), dim3(kWave), 0, st, cand_v, cand_i, out, chunks);
  return check_launch("argmax");
}

extern "C" int pa_argmax(void* stream, const float* logits, int* out, float* scratch, int rows, int vocab) {
  if (rows == 0) return 0;
  PA_REQUIRE(rows > 0 && vocab > 0, "argmax: bad sizes rows=%d vocab=%d", rows, vocab);
  return argmax_launch((hipStream_t)stream, logits, out, scratch, rows, vocab);
}

// ---------------------------------------------------------------------------
// pa_argmax for callers that cannot allocate: the candidates of wide rows go to an array that is part of the
// library's image on every GPU.  In host code the array's name is only a stand-in for the symbol; the address
// of a GPU's copy comes from hipGetSymbolAddress with that GPU current, once per GPU, and only that address is
// ever handed to a kernel.
// ---------------------------------------------------------------------------
constexpr int kStaticArgmaxWords = 1 << 16;   // 256 KB a GPU
static __device__ __align__(256) float scratch[kStaticArgmaxWords];

constexpr int kStaticMaxDevices = 64;
static float* g_static_scratch[kStaticMaxDevices];   // per GPU: where its copy of `scratch` lies
static std::mutex g_static_lock;

static int static_scratch(float** out) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return pa::fail("argmax_static: hipGetDevice: %s", hipGetErrorString(e));
  PA_REQUIRE(dev >= 0 && dev < kStaticMaxDevices, "argmax_static: device %d is beyond the %d this library keeps track of",
             dev, kStaticMaxDevices);
  std::lock_guard<std::mutex> hold(g_static_lock);
  if (!g_static_scratch[dev]) {
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !p)
      return pa::fail("argmax_static: hipGetSymbolAddress on device %d: %s", dev, hipGetErrorString(e));
    g_static_scratch[dev] = static_cast<float*>(p);
  }
  *out = g_static_scratch[dev];
  return 0;
}

extern "C" int pa_argmax_static_capacity() { return kStaticArgmaxWords; }

extern "C" int pa_argmax_static(void* stream, const float* logits, int* out, int rows, int vocab) {
  if (rows == 0) return 0;
  PA_REQUIRE(rows > 0 && vocab > 0, "argmax_static: bad sizes rows=%d vocab=%d", rows, vocab);
  const long words = (long)rows * ((vocab + 2047) / 2048) * 2;
  PA_REQUIRE(vocab <= 8192 || words <= kStaticArgmaxWords,
             "argmax_static: %d rows of %d entries need %ld words of scratch, the built-in array holds %d "
             "(use pa_argmax with a workspace of the caller's)", rows, vocab, words, kStaticArgmaxWords);
  float* ptr = nullptr;
  if (int rc = static_scratch(&ptr)) return rc;
  return argmax_launch((hipStream_t)stream, logits, out, ptr, rows, vocab);
}
