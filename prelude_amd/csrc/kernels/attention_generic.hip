// Paged causal attention for any mix of prompt portions and decode tokens,
// any head_dim up to 256, any page size, with or without a window, in 32-bit
// or bfloat16 storage.  All arithmetic is 32-bit on the vector ALU.  It is the
// attention of the true 32-bit path and the one that takes the sizes the MFMA
// kernels refuse.
//
// One wavefront per (query token, query head).  Keys are walked in chunks of
// 64 anchored at absolute key positions that are multiples of 64, so the
// order of every sum depends only on the query's position and window: the
// result for a token is bit-identical whether it arrives in a whole prompt,
// in a portion, or as a single decode token, and whatever pages hold its keys.
//
// K pages are [page, kv_head, offset, head_dim], V pages [page, kv_head, head_dim, offset].
//
// Formula: crates/prelude-core/src/models/qwen3.rs:276-370 and
// crates/prelude-core/src/ops/traits/attention.rs:10-99 (scores q.k * scale,
// key c visible to the query at position p when c <= p and, with a window of
// W keys, c > p - W; softmax in 32-bit; query head h reads KV head h / (nh/nkv)).  The reference's attention has
// no score cap (qwen3.rs:204); `softcap` > 0 bends the scaled scores to cap * tanh(s / cap) for mixers that want one.
#include "common.h"
#include "api.h"

namespace pa {

constexpr int kAttnWaves = 4;
constexpr int kAttnMaxHd = 256;

template <typename T>
__global__ __launch_bounds__(kAttnWaves* kWave) void attn_generic_kernel(
    const T* __restrict__ q, const T* __restrict__ k_cache, const T* __restrict__ v_cache,
    const int* __restrict__ block_table, int table_stride, const int* __restrict__ seq_of_token,
    const int* __restrict__ positions, T* __restrict__ out, int nh, int nkv, int hd, int page_size, int window,
    float scale, float softcap) {
  __shared__ float qs[kAttnWaves][kAttnMaxHd];
  __shared__ float ps[kAttnWaves][kWave];
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
  const int t = blockIdx.x;
  const int h = blockIdx.y * kAttnWaves + wave;
  const bool active = h < nh;  // every wave of the block shares the token, hence the trip count below
  const int pos = positions[t];
  const int seq = seq_of_token[t];
  const int hi = pos;
  const int lo = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
  const int kvh = active ? h / (nh / nkv) : 0;
  const int* table = block_table + (size_t)seq * table_stride;

  if (active) {
    const T* qr = q + ((size_t)t * nh + h) * hd;
    for (int d = lane; d < hd; d += kWave) qs[wave][d] = to_f32(qr[d]);
  }
  __syncthreads();

  float m = -INFINITY, l = 0.f;
  float o[kAttnMaxHd / kWave] = {};
  for (int c0 = (lo / kWave) * kWave; c0 <= hi; c0 += kWave) {
    const int c = c0 + lane;
    const bool valid = active && c >= lo && c <= hi;
    float s = -INFINITY;
    if (valid) {
      const int page = table[c / page_size];
      const T* kr = k_cache + (((size_t)page * nkv + kvh) * page_size + (c % page_size)) * hd;
      float dot = 0.f;
      for (int d = 0; d < hd; ++d) dot = fmaf(qs[wave][d], to_f32(kr[d]), dot);
      s = dot * scale;
      if (softcap != 0.f) s = softcap * tanhf(s / softcap);   // scores bent into (-cap, cap); off: the same bits as ever
    }
    const float m_new = fmaxf(m, wave_max(s));
    const float p = valid ? expf(s - m_new) : 0.f;
    const float alpha = active ? expf(m - m_new) : 0.f;  // exp(-inf) = 0 on the first chunk
    l = l * alpha + wave_sum(p);
    ps[wave][lane] = p;
    __syncthreads();
#pragma unroll
    for (int e = 0; e < kAttnMaxHd / kWave; ++e) o[e] *= alpha;
    if (active) {
      const int j_lo = lo > c0 ? lo - c0 : 0;
      const int j_hi = hi - c0 < kWave - 1 ? hi - c0 : kWave - 1;
      for (int j = j_lo; j <= j_hi; ++j) {
        const int cj = c0 + j;
        const int page = table[cj / page_size];
        const T* vr = v_cache + ((size_t)page * nkv + kvh) * hd * page_size + (cj % page_size);
        const float pj = ps[wave][j];
#pragma unroll
        for (int e = 0; e < kAttnMaxHd / kWave; ++e) {
          const int d = lane + e * kWave;
          if (d < hd) o[e] = fmaf(pj, to_f32(vr[(size_t)d * page_size]), o[e]);
        }
      }
    }
    __syncthreads();
    m = m_new;
  }
  if (active) {
    T* orow = out + ((size_t)t * nh + h) * hd;
    const float inv = 1.0f / l;
#pragma unroll
    for (int e = 0; e < kAttnMaxHd / kWave; ++e) {
      const int d = lane + e * kWave;
      if (d < hd) orow[d] = from_f32<T>(o[e] * inv);
    }
  }
}

}  // namespace pa

using namespace pa;

extern "C" int pa_attn_generic(void* stream, int dtype, const void* q, const void* k_cache, const void* v_cache,
                               const int* block_table, int table_stride, const int* seq_of_token,
                               const int* positions, void* out, int tokens, int nh, int nkv, int hd, int page_size,
                               int window, float scale, float softcap) {
  if (tokens == 0) return 0;
  PA_REQUIRE(tokens > 0 && nh > 0 && nkv > 0 && page_size > 0 && table_stride > 0,
             "attn_generic: bad sizes tokens=%d nh=%d nkv=%d page=%d table_stride=%d", tokens, nh, nkv, page_size,
             table_stride);
  PA_REQUIRE(nh % nkv == 0, "attn_generic: %d query heads are not a multiple of %d KV heads", nh, nkv);
  PA_REQUIRE(hd > 0 && hd <= kAttnMaxHd, "attn_generic: head_dim %d is outside 1..%d", hd, kAttnMaxHd);
  PA_REQUIRE(window >= 0, "attn_generic: window %d is negative (0 means none)", window);
  PA_REQUIRE(softcap >= 0.f, "attn_generic: a score cap of %g is negative (0 means none)", (double)softcap);
  dim3 grid(tokens, (nh + kAttnWaves - 1) / kAttnWaves);
  hipStream_t st = (hipStream_t)stream;
  if (dtype == kF32) {
    hipLaunchKernelGGL(attn_generic_kernel<float>, grid, dim3(kAttnWaves * kWave), 0, st, (const float*)q,
                       (const float*)k_cache, (const float*)v_cache, block_table, table_stride, seq_of_token, positions,
                       (float*)out, nh, nkv, hd, page_size, window, scale, softcap);
  } else if (dtype == kBF16) {
    hipLaunchKernelGGL(attn_generic_kernel<bf16>, grid, dim3(kAttnWaves * kWave), 0, st, (const bf16*)q,
                       (const bf16*)k_cache, (const bf16*)v_cache, block_table, table_stride, seq_of_token, positions,
                       (bf16*)out, nh, nkv, hd, page_size, window, scale, softcap);
  } else {
    return pa::fail("attn_generic: unknown element type code %d", dtype);
  }
  return check_launch("attn_generic");
}
