// Per-head RMSNorm of Q and K, rotary position encoding, and the write of K
// and V into the paged cache, in one launch over a merged QKV activation.
//
// Formula: crates/prelude-cuda/src/kernels/kernels_src/rope/qknorm_rope.cu:20-91
// (norm over head_dim in 32-bit, then rotate-half, one rounding at the end) and
// crates/prelude-cuda/src/kernels/kernels_src/kvcache/scatter_kv_cache.cu:19-81,
// knorm_rope_kv_write.cu:17-113 (K is normed and rotated on its way into the
// cache; V is copied).  Differences that are ours: the norm weights and the
// cos/sin tables are 32-bit in every mode, the rotary width may be smaller
// than the head (the rest passes through after the norm), the norm may be
// absent, and the caches are laid out K [page, kv_head, offset, head_dim] and
// V [page, kv_head, head_dim, offset]: V transposed, so that the attention
// kernels can feed both straight from memory into the matrix cores (keys are
// the contraction index of P.V, and an MFMA operand wants it contiguous).
#include "common.h"
#include "api.h"

namespace pa {

constexpr int kQkWaves = 4;
constexpr int kQkGroup = 4;   // heads a wavefront of the wide kernel takes
constexpr int kMaxHeadDim = 256;

// One wavefront per (token, head) over the nh + 2*nkv heads of a token's row.
template <typename T>
__global__ void qknorm_rope_kv_kernel(const T* __restrict__ qkv, const float* __restrict__ q_weight,
                                      const float* __restrict__ k_weight, const float* __restrict__ cos_table,
                                      const float* __restrict__ sin_table, const int* __restrict__ positions,
                                      const int* __restrict__ slots, T* __restrict__ q_out,
                                      T* __restrict__ k_cache, T* __restrict__ v_cache, int tokens, int nh, int nkv,
                                      int hd, int rot, int page_size, float eps) {
  __shared__ float normed[kQkWaves][kMaxHeadDim];
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
  const int heads = nh + 2 * nkv;
  const long long unit = (long long)blockIdx.x * kQkWaves + wave;
  const bool active = unit < (long long)tokens * heads;
  const int t = active ? (int)(unit / heads) : 0;
  const int h = active ? (int)(unit % heads) : 0;
  const T* src = qkv + ((size_t)t * heads + h) * hd;

  // Where this head goes.
  T* dst = nullptr;
  long dst_stride = 1;  // distance between consecutive head_dim elements at the destination
  const float* weight = nullptr;
  bool rotate = false;
  if (active) {
    if (h < nh) {
      dst = q_out + ((size_t)t * nh + h) * hd;
      weight = q_weight;
      rotate = true;
    } else {
      const long long slot = slots ? (long long)slots[t] : -1;
      if (slot >= 0) {
        const long long page = slot / page_size, off = slot % page_size;
        const bool is_k = h < nh + nkv;
        const int kvh = is_k ? h - nh : h - nh - nkv;
        if (is_k) {
          dst = k_cache + (((size_t)page * nkv + kvh) * page_size + off) * hd;
        } else {
          dst = v_cache + ((size_t)page * nkv + kvh) * hd * page_size + off;
          dst_stride = page_size;
        }
        weight = is_k ? k_weight : nullptr;
        rotate = is_k;
      }
    }
  }
  const bool is_v = active && h >= nh + nkv;

  float x[kMaxHeadDim / kWave];
  float ss = 0.f;
#pragma unroll
  for (int e = 0; e < kMaxHeadDim / kWave; ++e) {
    const int i = lane + e * kWave;
    x[e] = (active && i < hd) ? to_f32(src[i]) : 0.f;
    ss += x[e] * x[e];
  }
  if (is_v) {  // plain copy
    if (dst) {
#pragma unroll
      for (int e = 0; e < kMaxHeadDim / kWave; ++e) {
        const int i = lane + e * kWave;
        if (i < hd) dst[(size_t)i * dst_stride] = src[i];
      }
    }
  }
  ss = wave_sum(ss);
  const float inv = rsqrtf(ss / (float)hd + eps);
#pragma unroll
  for (int e = 0; e < kMaxHeadDim / kWave; ++e) {
    const int i = lane + e * kWave;
    if (i < hd) {
      if (!is_v && weight) x[e] = x[e] * inv * weight[i];
      normed[wave][i] = x[e];
    }
  }
  __syncthreads();
  if (!active || is_v || !dst) return;
  const int half = rot / 2;
  const int pos = rot > 0 ? positions[t] : 0;
  const float* c = cos_table + (size_t)pos * half;
  const float* s = sin_table + (size_t)pos * half;
#pragma unroll
  for (int e = 0; e < kMaxHeadDim / kWave; ++e) {
    const int i = lane + e * kWave;
    if (i >= hd) continue;
    float r = x[e];
    if (rotate && i < rot) {
      if (i < half) {
        r = x[e] * c[i] - normed[wave][i + half] * s[i];
      } else {
        const int j = i - half;
        r = normed[wave][j] * s[j] + x[e] * c[j];
      }
    }
    dst[i] = from_f32<T>(r);
  }
}

// The same for head_dim 64, 128 or 256 rotated over its whole width: a lane owns EPL = head_dim / 64
// contiguous elements, read and written as one vector; its rotation partner (element + head_dim / 2)
// sits in lane ^ 32, so nothing goes through LDS.
//
// Units (one wavefront each): ceil(tokens / vgroup) x nkv groups of vgroup (1 or 8) tokens of one value head, then
// tokens x groups of kQkGroup query and key heads.  In the transposed value page a token's elements lie
// page_size apart, but eight tokens whose slots are consecutive and start at a multiple of eight (a run: the usual
// case inside a prompt portion) lie side by side for every element, so a run is written with one vector store
// per element by the wavefront in whose group the run starts; tokens outside runs are written one by one.
template <typename T, int EPL>
__global__ __launch_bounds__(kQkWaves* kWave) void qknorm_rope_kv_wide_kernel(
    const T* __restrict__ qkv, const float* __restrict__ q_weight, const float* __restrict__ k_weight,
    const float* __restrict__ cos_table, const float* __restrict__ sin_table, const int* __restrict__ positions,
    const int* __restrict__ slots, T* __restrict__ q_out, T* __restrict__ k_cache, T* __restrict__ v_cache, int tokens,
    int nh, int nkv, int page_size, float eps, int vgroup) {
  typedef T vec_t __attribute__((ext_vector_type(EPL)));
  typedef T run_t __attribute__((ext_vector_type(8)));
  constexpr int hd = EPL * kWave;
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
  const int heads = nh + 2 * nkv;
  const int qk_heads = nh + nkv;
  const int head_groups = (qk_heads + kQkGroup - 1) / kQkGroup;
  const long long qk_units = (long long)tokens * head_groups;
  const long long v_units = (slots && nkv > 0) ? (long long)((tokens + vgroup - 1) / vgroup) * nkv : 0;
  long long unit = (long long)blockIdx.x * kQkWaves + wave;
  if (unit < v_units && vgroup == 1) {  // few tokens (decode steps): a wavefront per token and value head
    const int x = (int)(unit / nkv), kvh = (int)(unit % nkv);
    const int slot = slots[x];
    if (slot < 0) return;
    const vec_t xv = *reinterpret_cast<const vec_t*>(qkv + ((size_t)x * heads + qk_heads + kvh) * hd + lane * EPL);
    T* dst = v_cache + ((size_t)(slot / page_size) * nkv + kvh) * hd * page_size + slot % page_size;
#pragma unroll
    for (int e = 0; e < EPL; ++e) dst[(size_t)(lane * EPL + e) * page_size] = xv[e];
    return;
  }
  if (unit < v_units) {  // V first (the longer units): copies into the transposed pages
    const int group = (int)(unit / nkv), kvh = (int)(unit % nkv);
    const int t0 = group * 8;
    // slots of the tokens from seven before the group to seven behind it (the same in every lane: scalar loads)
    int sl[22];
#pragma unroll
    for (int i = 0; i < 22; ++i) {
      const int x = t0 - 7 + i;
      sl[i] = (x >= 0 && x < tokens) ? slots[x] : -2;
    }
    // bit i: a run starts at token t0 - 7 + i
    unsigned starts = 0;
    if (page_size % 8 == 0) {
#pragma unroll
      for (int i = 0; i < 15; ++i) {
        bool ok = sl[i] >= 0 && (sl[i] & 7) == 0;
#pragma unroll
        for (int k = 1; k < 8; ++k) ok = ok && sl[i + k] == sl[i] + k;
        starts |= (ok ? 1u : 0u) << i;
      }
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int x = t0 + j;
      const int slot = sl[7 + j];
      if (slot < 0) continue;   // not cached, or beyond the batch
      const int head = 7 + j - (slot & 7);   // where this token's run would start
      const bool in_run = (starts >> head) & 1u;
      if (in_run && (slot & 7)) continue;    // written with its run (by this group or the one before)
      const size_t page = (size_t)(slot / page_size);
      const int off = slot % page_size;
      T* dst = v_cache + (page * nkv + kvh) * hd * page_size + off;
      if (in_run) {
        vec_t v[8];
#pragma unroll
        for (int i = 0; i < 8; ++i)
          v[i] = *reinterpret_cast<const vec_t*>(qkv + ((size_t)(x + i) * heads + qk_heads + kvh) * hd + lane * EPL);
#pragma unroll
        for (int e = 0; e < EPL; ++e) {
          run_t r;
#pragma unroll
          for (int i = 0; i < 8; ++i) r[i] = v[i][e];
          *reinterpret_cast<run_t*>(dst + (size_t)(lane * EPL + e) * page_size) = r;
        }
      } else {
        const vec_t xv = *reinterpret_cast<const vec_t*>(qkv + ((size_t)x * heads + qk_heads + kvh) * hd + lane * EPL);
#pragma unroll
        for (int e = 0; e < EPL; ++e) dst[(size_t)(lane * EPL + e) * page_size] = xv[e];
      }
    }
    return;
  }
  unit -= v_units;
  if (unit >= qk_units) return;
  // queries and keys: kQkGroup heads of one token, loaded together so one memory round trip serves them all
  const int t = (int)(unit / head_groups), h0 = (int)(unit % head_groups) * kQkGroup;
  const long long slot = slots ? (long long)slots[t] : -1;
  const int pos = positions[t];
  const int j0 = (lane % 32) * EPL;  // index into the cos/sin row
  typedef float rot_t __attribute__((ext_vector_type(EPL)));
  const rot_t c = *reinterpret_cast<const rot_t*>(cos_table + (size_t)pos * (hd / 2) + j0);
  const rot_t sn = *reinterpret_cast<const rot_t*>(sin_table + (size_t)pos * (hd / 2) + j0);
  vec_t xv[kQkGroup];
#pragma unroll
  for (int i = 0; i < kQkGroup; ++i)
    if (h0 + i < qk_heads) xv[i] = *reinterpret_cast<const vec_t*>(qkv + ((size_t)t * heads + h0 + i) * hd + lane * EPL);
  rot_t qw, kw;
#pragma unroll
  for (int e = 0; e < EPL; ++e) {
    qw[e] = q_weight ? q_weight[lane * EPL + e] : 1.0f;
    kw[e] = k_weight ? k_weight[lane * EPL + e] : 1.0f;
  }
#pragma unroll
  for (int i = 0; i < kQkGroup; ++i) {
    const int h = h0 + i;
    if (h >= qk_heads) break;
    T* dst;
    const bool is_q = h < nh;
    if (is_q) {
      dst = q_out + ((size_t)t * nh + h) * hd;
    } else {
      if (slot < 0) continue;
      const long long page = slot / page_size, off = slot % page_size;
      dst = k_cache + (((size_t)page * nkv + (h - nh)) * page_size + off) * hd;
    }
    const bool normed = is_q ? q_weight != nullptr : k_weight != nullptr;
    float x[EPL];
    float ss = 0.f;
#pragma unroll
    for (int e = 0; e < EPL; ++e) {
      x[e] = to_f32(xv[i][e]);
      ss += x[e] * x[e];
    }
    ss = wave_sum(ss);
    const float inv = rsqrtf(ss / (float)hd + eps);
    vec_t ov;
#pragma unroll
    for (int e = 0; e < EPL; ++e) {
      if (normed) x[e] = x[e] * inv * (is_q ? qw[e] : kw[e]);
      const float partner = __shfl_xor(x[e], 32, kWave);
      const float r = lane < 32 ? x[e] * c[e] - partner * sn[e] : partner * sn[e] + x[e] * c[e];
      ov[e] = from_f32<T>(r);
    }
    *reinterpret_cast<vec_t*>(dst + lane * EPL) = ov;
  }
}

}  // namespace pa

using namespace pa;

extern "C" int pa_qknorm_rope_kv(void* stream, int dtype, const void* qkv, const float* q_weight,
                                 const float* k_weight, const float* cos_table, const float* sin_table,
                                 const int* positions, const int* slots, void* q_out, void* k_cache,
                                 void* v_cache, int tokens, int nh, int nkv, int hd, int rot, int page_size,
                                 float eps) {
  if (tokens == 0) return 0;
  PA_REQUIRE(tokens > 0 && nh > 0 && nkv >= 0 && page_size > 0, "qknorm_rope_kv: bad sizes tokens=%d nh=%d nkv=%d page=%d",
             tokens, nh, nkv, page_size);
  PA_REQUIRE(hd > 0 && hd <= kMaxHeadDim, "qknorm_rope_kv: head_dim %d is outside 1..%d", hd, kMaxHeadDim);
  PA_REQUIRE(rot >= 0 && rot <= hd && rot % 2 == 0, "qknorm_rope_kv: rotary width %d must be even and at most head_dim %d",
             rot, hd);
  PA_REQUIRE(rot == 0 || (cos_table && sin_table && positions), "qknorm_rope_kv: rotary tables or positions missing");
  const long long units = (long long)tokens * (nh + 2 * nkv);
  const unsigned blocks = (unsigned)((units + kQkWaves - 1) / kQkWaves);
  hipStream_t st = (hipStream_t)stream;
  if (rot == hd && rot > 0 && (hd == 64 || hd == 128 || hd == 256) && (dtype == kF32 || dtype == kBF16)) {
    const int vgroup = tokens >= 64 ? 8 : 1;   // runs of eight tokens pay only in prompt portions
    const long long wide_units =
        (long long)tokens * ((nh + nkv + kQkGroup - 1) / kQkGroup) + (long long)((tokens + vgroup - 1) / vgroup) * nkv;
    const unsigned wide_blocks = (unsigned)((wide_units + kQkWaves - 1) / kQkWaves);
#define PA_WIDE(T, EPL)                                                                                             \
  hipLaunchKernelGGL((qknorm_rope_kv_wide_kernel<T, EPL>), dim3(wide_blocks), dim3(kQkWaves * kWave), 0, st, (const T*)qkv, \
                     q_weight, k_weight, cos_table, sin_table, positions, slots, (T*)q_out, (T*)k_cache, (T*)v_cache, \
                     tokens, nh, nkv, page_size, eps, vgroup)
    if (dtype == kF32) {
      if (hd == 64) PA_WIDE(float, 1);
      else if (hd == 128) PA_WIDE(float, 2);
      else PA_WIDE(float, 4);
    } else {
      if (hd == 64) PA_WIDE(bf16, 1);
      else if (hd == 128) PA_WIDE(bf16, 2);
      else PA_WIDE(bf16, 4);
    }
#undef PA_WIDE
    return check_launch("qknorm_rope_kv");
  }
  if (dtype == kF32) {
    hipLaunchKernelGGL(qknorm_rope_kv_kernel<float>, dim3(blocks), dim3(kQkWaves * kWave), 0, st, (const float*)qkv,
                       q_weight, k_weight, cos_table, sin_table, positions, slots, (float*)q_out, (float*)k_cache,
                       (float*)v_cache, tokens, nh, nkv, hd, rot, page_size, eps);
  } else if (dtype == kBF16) {
    hipLaunchKernelGGL(qknorm_rope_kv_kernel<bf16>, dim3(blocks), dim3(kQkWaves * kWave), 0, st, (const bf16*)qkv,
                       q_weight, k_weight, cos_table, sin_table, positions, slots, (bf16*)q_out, (bf16*)k_cache,
                       (bf16*)v_cache, tokens, nh, nkv, hd, rot, page_size, eps);
  } else {
    return pa::fail("qknorm_rope_kv: unknown element type code %d", dtype);
  }
  return check_launch("qknorm_rope_kv");
}
