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

// Query and key heads a wavefront of the wide kernel takes: U loads of 64 lanes x 16 bytes.
template <typename T, int EPL, int U>
__host__ __device__ constexpr int wide_heads() {
  return U * kWave / (EPL * kWave / (16 / (int)sizeof(T)));
}

// The same for head_dim 64, 128 or 256 rotated over its whole width: a lane owns EPL = head_dim / 64
// contiguous elements, read and written as one vector; its rotation partner (element + head_dim / 2)
// sits in lane ^ 32, so nothing goes through LDS.
//
// Units (one wavefront each): ceil(tokens / vgroup) x nkv groups of vgroup (1 or 8) tokens of one value head, then
// tokens x groups of query and key heads (see below).  In the transposed value page a token's elements lie
// page_size apart, but eight tokens whose slots are consecutive and start at a multiple of eight (a run: the usual
// case inside a prompt portion) lie side by side for every element, so a run is written with one vector store
// per element by the wavefront in whose group the run starts; tokens outside runs are written one by one.
template <typename T, int EPL, int U>
__global__ __launch_bounds__(kQkWaves* kWave) void qknorm_rope_kv_wide_kernel(
    const T* __restrict__ qkv, const float* __restrict__ q_weight, const float* __restrict__ k_weight,
    const float* __restrict__ cos_table, const float* __restrict__ sin_table, const int* __restrict__ positions,
    const int* __restrict__ slots, T* __restrict__ q_out, T* __restrict__ k_cache, T* __restrict__ v_cache, int tokens,
    int nh, int nkv, int page_size, float eps, int vgroup) {
  typedef T vec_t __attribute__((ext_vector_type(EPL)));
  typedef T run_t __attribute__((ext_vector_type(8)));
  constexpr int hd = EPL * kWave;
  __shared__ __align__(16) T turn[kQkWaves][8][hd];   // a run of eight value rows on its way to being columns
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
  const int heads = nh + 2 * nkv;
  const int qk_heads = nh + nkv;
  const int head_groups = (qk_heads + wide_heads<T, EPL, U>() - 1) / wide_heads<T, EPL, U>();
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
        // the eight rows come in with 16 bytes a lane and are turned through LDS (the wavefront's own
        // stretch of it: LDS operations of one wavefront keep their order)
        constexpr int VEC = 16 / (int)sizeof(T);
        constexpr int LPH = hd / VEC, TPL = kWave / LPH;   // lanes a row, rows a load
        typedef T row_t __attribute__((ext_vector_type(VEC)));
        const int c = lane % LPH;
#pragma unroll
        for (int l = 0; l < 8 / TPL; ++l) {
          const int tok = l * TPL + lane / LPH;
          const row_t v =
              *reinterpret_cast<const row_t*>(qkv + ((size_t)(x + tok) * heads + qk_heads + kvh) * hd + c * VEC);
          *reinterpret_cast<row_t*>(&turn[wave][tok][c * VEC]) = v;
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int e = 0; e < EPL; ++e) {
          const int d = e * kWave + lane;
          run_t r;
#pragma unroll
          for (int i = 0; i < 8; ++i) r[i] = turn[wave][i][d];
          *reinterpret_cast<run_t*>(dst + (size_t)d * page_size) = r;
        }
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        __builtin_amdgcn_wave_barrier();
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
  // Queries and keys: a lane owns 16 bytes of a head, LPH lanes a head, so one load of the wavefront brings
  // 64 / LPH heads that lie side by side (1 KB), and U such loads are in flight before anything is computed.
  // A lane's rotation partner (element + head_dim / 2) sits LPH / 2 lanes away.  Heads past the last one, and
  // keys of tokens that are not cached, are computed on zeros and not stored, so every lane takes every shuffle.
  constexpr int VEC = 16 / (int)sizeof(T);
  constexpr int LPH = hd / VEC, HPL = kWave / LPH;
  typedef T row_t __attribute__((ext_vector_type(VEC)));
  const int t = (int)(unit / head_groups), h0 = (int)(unit % head_groups) * HPL * U;
  const int sub = lane / LPH, c = lane % LPH;
  const long long slot = slots ? (long long)slots[t] : -1;
  const int pos = positions[t];
  const int j0 = (c % (LPH / 2)) * VEC;  // index into the cos/sin row
  float cs[VEC], sn[VEC], qw[VEC], kw[VEC];
#pragma unroll
  for (int e = 0; e < VEC; e += 4) {
    const f32x4 cv = *reinterpret_cast<const f32x4*>(cos_table + (size_t)pos * (hd / 2) + j0 + e);
    const f32x4 sv = *reinterpret_cast<const f32x4*>(sin_table + (size_t)pos * (hd / 2) + j0 + e);
    const f32x4 one = {1.f, 1.f, 1.f, 1.f};
    const f32x4 qv = q_weight ? *reinterpret_cast<const f32x4*>(q_weight + c * VEC + e) : one;
    const f32x4 kv = k_weight ? *reinterpret_cast<const f32x4*>(k_weight + c * VEC + e) : one;
#pragma unroll
    for (int i = 0; i < 4; ++i) cs[e + i] = cv[i], sn[e + i] = sv[i], qw[e + i] = qv[i], kw[e + i] = kv[i];
  }
  row_t xv[U];
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const int h = h0 + u * HPL + sub;
    if (h < qk_heads) {
      xv[u] = *reinterpret_cast<const row_t*>(qkv + ((size_t)t * heads + h) * hd + c * VEC);
    } else {
#pragma unroll
      for (int e = 0; e < VEC; ++e) xv[u][e] = from_f32<T>(0.f);
    }
  }
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const int h = h0 + u * HPL + sub;
    const bool is_q = h < nh;
    const bool normed = is_q ? q_weight != nullptr : k_weight != nullptr;
    float x[VEC];
    float ss = 0.f;
#pragma unroll
    for (int e = 0; e < VEC; ++e) {
      x[e] = to_f32(xv[u][e]);
      ss += x[e] * x[e];
    }
#pragma unroll
    for (int off = LPH / 2; off >= 1; off >>= 1) ss += __shfl_xor(ss, off, kWave);
    const float inv = rsqrtf(ss / (float)hd + eps);
    row_t ov;
#pragma unroll
    for (int e = 0; e < VEC; ++e) {
      if (normed) x[e] = x[e] * inv * (is_q ? qw[e] : kw[e]);
      const float partner = __shfl_xor(x[e], LPH / 2, kWave);
      const float r = c < LPH / 2 ? x[e] * cs[e] - partner * sn[e] : partner * sn[e] + x[e] * cs[e];
      ov[e] = from_f32<T>(r);
    }
    if (h >= qk_heads || (!is_q && slot < 0)) continue;
    T* dst;
    if (is_q) {
      dst = q_out + ((size_t)t * nh + h) * hd;
    } else {
      const long long page = slot / page_size, off = slot % page_size;
      dst = k_cache + (((size_t)page * nkv + (h - nh)) * page_size + off) * hd;
    }
    *reinterpret_cast<row_t*>(dst + c * VEC) = ov;
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
    const long long v_units = (long long)((tokens + vgroup - 1) / vgroup) * nkv;
    // many tokens: five loads in flight per wavefront; few: one, so that there are wavefronts enough
#define PA_WIDE_U(T, EPL, U)                                                                                          \
  {                                                                                                                   \
    const int per = wide_heads<T, EPL, U>();                                                                          \
    const long long wide_units = (long long)tokens * ((nh + nkv + per - 1) / per) + v_units;                          \
    const unsigned wide_blocks = (unsigned)((wide_units + kQkWaves - 1) / kQkWaves);                                  \
    hipLaunchKernelGGL((qknorm_rope_kv_wide_kernel<T, EPL, U>), dim3(wide_blocks), dim3(kQkWaves * kWave), 0, st,      \
                       (const T*)qkv, q_weight, k_weight, cos_table, sin_table, positions, slots, (T*)q_out,          \
                       (T*)k_cache, (T*)v_cache, tokens, nh, nkv, page_size, eps, vgroup);                            \
  }
#define PA_WIDE(T, EPL)          \
  do {                           \
    if (tokens >= 64) {          \
      PA_WIDE_U(T, EPL, 5)       \
    } else {                     \
      PA_WIDE_U(T, EPL, 1)       \
    }                            \
  } while (0)
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
#undef PA_WIDE_U
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
