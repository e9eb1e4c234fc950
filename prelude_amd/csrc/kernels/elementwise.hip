// Row-wise kernels: embedding gather, RMSNorm with and without the residual
// add, SiLU*mul, row gather, bias add and the cast to 32-bit logits.
//
// Counterparts in the reference (formulas only; the launch shapes are ours):
//   rmsnorm / add_rmsnorm  crates/prelude-cuda/src/kernels/kernels_src/normalization/rmsnorm.cu:12-355
//   silu_mul               crates/prelude-cuda/src/kernels/kernels_src/elementwise/silu_mul.cu:7-43
//   embedding, row gather  crates/prelude-core/src/models/commons/embedding.rs:29-36,
//                          crates/prelude-core/src/models/commons/mod.rs:227-243
#include "common.h"
#include "api.h"

namespace pa {

// ---- embedding gather ------------------------------------------------------
// One block per token; 16-byte copies when the row width allows.
template <typename T>
__global__ void embed_gather_kernel(const int* __restrict__ ids, const T* __restrict__ table,
                                    T* __restrict__ out, int hidden, int vocab) {
  const int t = blockIdx.x;
  int id = ids[t];
  // The host refuses ids outside the vocabulary before any launch; the clamp
  // only keeps a stray id from reading outside the table.
  id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);
  const T* src = table + (size_t)id * hidden;
  T* dst = out + (size_t)t * hidden;
  constexpr int kVec = 16 / sizeof(T);
  if (hidden % kVec == 0) {
    const uint4* s4 = reinterpret_cast<const uint4*>(src);
    uint4* d4 = reinterpret_cast<uint4*>(dst);
    for (int i = threadIdx.x; i < hidden / kVec; i += blockDim.x) d4[i] = s4[i];
  } else {
    for (int i = threadIdx.x; i < hidden; i += blockDim.x) dst[i] = src[i];
  }
}

// ---- token ids that never left the device ------------------------------
// ids[dst[i]] = sampled[src[i]] for every i with src[i] >= 0: a step that is
// launched before the host has read the previous step's tokens takes them here.
__global__ void carry_tokens_kernel(const int* __restrict__ sampled, const int* __restrict__ src,
                                    const int* __restrict__ dst, int* __restrict__ ids, int n, int sampled_rows,
                                    int tokens) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const int s = src[i], d = dst[i];
  if (s < 0 || s >= sampled_rows || d < 0 || d >= tokens) return;
  ids[d] = sampled[s];
}

// ---- state of fixed size per request, started from zero ------------------
// Row slots[i] of `data` (rows of `row_words` 32-bit words) is cleared for every sequence i of the step that
// starts its request (fresh[i] != 0) and has a slot.  Grid (sequences, pieces of a row).
__global__ void zero_fresh_rows_kernel(uint32_t* __restrict__ data, long row_words, const int* __restrict__ slots,
                                       const int* __restrict__ fresh, int num_rows) {
  const int i = blockIdx.x;
  const int slot = slots[i];
  if (!fresh[i] || slot < 0 || slot >= num_rows) return;
  uint32_t* row = data + (size_t)slot * row_words;
  for (long w = (long)blockIdx.y * blockDim.x + threadIdx.x; w < row_words; w += (long)gridDim.y * blockDim.x) row[w] = 0u;
}

// ---- how fast memory can be read at all ------------------------------------
// Every thread reads 16-byte pieces a whole grid apart, eight in flight, and folds them into one word; a block
// writes one word.  Nothing else happens: the rate this reaches is what a kernel that streams memory can be held to.
__global__ __launch_bounds__(256) void stream_read_kernel(const uint4* __restrict__ src, size_t pieces,
                                                         unsigned* __restrict__ out) {
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  unsigned acc = 0;
  for (; i + 7 * stride < pieces; i += 8 * stride) {
    uint4 v[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) v[j] = src[i + j * stride];
#pragma unroll
    for (int j = 0; j < 8; ++j) acc ^= v[j].x ^ v[j].y ^ v[j].z ^ v[j].w;
  }
  for (; i < pieces; i += stride) {
    const uint4 v = src[i];
    acc ^= v.x ^ v.y ^ v.z ^ v.w;
  }
  if (acc == 0x9e3779b9u) out[blockIdx.x] = acc;   // (almost) never: keeps the loads from being dropped
}

// ---- RMSNorm, optionally fused with the residual add --------------------
//   s = x (+ residual)                         in 32-bit
//   residual <- round(s)                       (only when `residual` is given and `rows` is not)
//   out = round(s * rsqrt(mean(s^2) + eps) * w)   from the unrounded s
// With `rows`, output row r is computed from input row rows[r] and nothing
// is written back to the residual: the final norm of only the wanted rows.
// x may come as `slices` 32-bit partial sums instead ([slices, rows, hidden], `slice_stride` elements apart, as a
// product cut along its inner size leaves them): they are added in order, in place of the load of x.
template <typename T>
__global__ void rmsnorm_kernel(const T* __restrict__ x, const float* __restrict__ parts, int slices, size_t slice_stride,
                               T* residual, const float* __restrict__ w, T* __restrict__ out,
                               const int* __restrict__ rows, int hidden, float eps) {
  __shared__ float scratch[16];
  const int r = blockIdx.x;
  const size_t src = rows ? (size_t)rows[r] : (size_t)r;
  const T* xr = x ? x + src * hidden : nullptr;
  const float* pr = parts ? parts + src * hidden : nullptr;
  T* rr = residual ? residual + src * hidden : nullptr;
  T* orow = out + (size_t)r * hidden;
  auto value = [&](int i) {
    if (!pr) return to_f32(xr[i]);
    float v = pr[i];
    for (int p = 1; p < slices; ++p) v += pr[(size_t)p * slice_stride + i];
    return v;
  };
  float ss = 0.f;
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
    float s = value(i);
    if (rr) s += to_f32(rr[i]);
    ss += s * s;
  }
  ss = block_sum(ss, scratch);
  const float inv = rsqrtf(ss / (float)hidden + eps);
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
    float s = value(i);
    if (rr) s += to_f32(rr[i]);
    if (rr && !rows) rr[i] = from_f32<T>(s);
    orow[i] = from_f32<T>(s * inv * w[i]);
  }
}

// The same with 16-byte loads and every element held in registers between the
// two passes: one read of x and the residual, one write of each output.
// NV vectors per thread; the block has ceil(hidden / VEC / NV) threads rounded up to a wavefront.
constexpr int kSlicesAtOnce = 8;

template <typename T, int NV>
__global__ void rmsnorm_vec_kernel(const T* __restrict__ x, const float* __restrict__ parts, int slices,
                                   size_t slice_stride, T* residual, const float* __restrict__ w,
                                   T* __restrict__ out, const int* __restrict__ rows, int hidden, float eps) {
  constexpr int VEC = 16 / sizeof(T);
  typedef T vec_t __attribute__((ext_vector_type(VEC)));
  __shared__ float scratch[16];
  const int r = blockIdx.x;
  const size_t src = rows ? (size_t)rows[r] : (size_t)r;
  const vec_t* xr = reinterpret_cast<const vec_t*>(x + src * hidden);
  const float* pr = parts ? parts + src * hidden : nullptr;
  vec_t* rr = residual ? reinterpret_cast<vec_t*>(residual + src * hidden) : nullptr;
  vec_t* orow = reinterpret_cast<vec_t*>(out + (size_t)r * hidden);
  const int nvec = hidden / VEC;
  float s[NV][VEC];
  float wv[NV][VEC];   // the scale, asked for with the row: its way from memory is not waited for after the sum
  float ss = 0.f;
#pragma unroll
  for (int j = 0; j < NV; ++j) {
    const int v = threadIdx.x + j * blockDim.x;
    if (v < nvec) {
      if (pr) {   // the slices of a product, added in their order
#pragma unroll
        for (int e = 0; e < VEC; e += 4) {
          float4 a = *reinterpret_cast<const float4*>(pr + (size_t)v * VEC + e);
          // up to eight slices are asked for together and then added (one trip to memory instead of one a slice)
          float4 b[kSlicesAtOnce - 1];
#pragma unroll
          for (int p = 1; p < kSlicesAtOnce; ++p)
            if (p < slices) b[p - 1] = *reinterpret_cast<const float4*>(pr + (size_t)p * slice_stride + (size_t)v * VEC + e);
#pragma unroll
          for (int p = 1; p < kSlicesAtOnce; ++p)
            if (p < slices) a.x += b[p - 1].x, a.y += b[p - 1].y, a.z += b[p - 1].z, a.w += b[p - 1].w;
          for (int p = kSlicesAtOnce; p < slices; ++p) {
            const float4 c = *reinterpret_cast<const float4*>(pr + (size_t)p * slice_stride + (size_t)v * VEC + e);
            a.x += c.x, a.y += c.y, a.z += c.z, a.w += c.w;
          }
          s[j][e] = a.x, s[j][e + 1] = a.y, s[j][e + 2] = a.z, s[j][e + 3] = a.w;
        }
      } else {
        const vec_t xv = xr[v];
#pragma unroll
        for (int e = 0; e < VEC; ++e) s[j][e] = to_f32(xv[e]);
      }
#pragma unroll
      for (int e = 0; e < VEC; e += 4) {
        const float4 w4 = *reinterpret_cast<const float4*>(w + (size_t)v * VEC + e);
        wv[j][e] = w4.x, wv[j][e + 1] = w4.y, wv[j][e + 2] = w4.z, wv[j][e + 3] = w4.w;
      }
      if (rr) {
        const vec_t rv = rr[v];
#pragma unroll
        for (int e = 0; e < VEC; ++e) s[j][e] += to_f32(rv[e]);
      }
#pragma unroll
      for (int e = 0; e < VEC; ++e) ss += s[j][e] * s[j][e];
    }
  }
  ss = block_sum(ss, scratch);
  const float inv = rsqrtf(ss / (float)hidden + eps);
#pragma unroll
  for (int j = 0; j < NV; ++j) {
    const int v = threadIdx.x + j * blockDim.x;
    if (v < nvec) {
      vec_t ov, sv;
#pragma unroll
      for (int e = 0; e < VEC; ++e) {
        sv[e] = from_f32<T>(s[j][e]);
        ov[e] = from_f32<T>(s[j][e] * inv * wv[j][e]);
      }
      if (rr && !rows) rr[v] = sv;
      orow[v] = ov;
    }
  }
}

// ---- SiLU(gate) * up over a merged [T, 2I] input whose columns alternate gate_j, up_j ----
template <typename T>
__global__ void silu_mul_kernel(const T* __restrict__ gate_up, T* __restrict__ out, int inter, size_t total, int act) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total) return;
  const float g = to_f32(gate_up[2 * i]);
  const float u = to_f32(gate_up[2 * i + 1]);
  out[i] = from_f32<T>(gate_activation(g, act) * u);
}

// Eight outputs a thread: two 16-byte loads (eight gate/up pairs), one 16-byte store.
__global__ void silu_mul_vec_kernel(const bf16* __restrict__ gate_up, bf16* __restrict__ out, size_t groups, int act) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= groups) return;
  const uint4* src = reinterpret_cast<const uint4*>(gate_up) + 2 * i;
  union { uint4 v; bf16 h[8]; } a, b, o;
  a.v = src[0];
  b.v = src[1];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const float g0 = (float)a.h[2 * j], u0 = (float)a.h[2 * j + 1];
    const float g1 = (float)b.h[2 * j], u1 = (float)b.h[2 * j + 1];
    o.h[j] = (bf16)(gate_activation(g0, act) * u0);
    o.h[4 + j] = (bf16)(gate_activation(g1, act) * u1);
  }
  reinterpret_cast<uint4*>(out)[i] = o.v;
}

// ---- row gather ------------------------------------------------------------
template <typename T>
__global__ void gather_rows_kernel(const T* __restrict__ x, const int* __restrict__ rows, T* __restrict__ out,
                                   int width) {
  const T* src = x + (size_t)rows[blockIdx.x] * width;
  T* dst = out + (size_t)blockIdx.x * width;
  for (int i = threadIdx.x; i < width; i += blockDim.x) dst[i] = src[i];
}

// ---- y[t, n] += b[n] -------------------------------------------------------
template <typename T>
__global__ void add_bias_kernel(T* __restrict__ y, const float* __restrict__ b, int width, size_t total) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total) return;
  y[i] = from_f32<T>(to_f32(y[i]) + b[i % width]);
}

template <typename T>
__global__ void to_f32_kernel(const T* __restrict__ x, float* __restrict__ out, size_t total) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < total) out[i] = to_f32(x[i]);
}

}  // namespace pa

using namespace pa;

#define PA_DISPATCH(dtype, ...)                                      \
  do {                                                               \
    if ((dtype) == kF32) {                                           \
      using T = float;                                               \
      __VA_ARGS__;                                                   \
    } else if ((dtype) == kBF16) {                                   \
      using T = bf16;                                                \
      __VA_ARGS__;                                                   \
    } else {                                                         \
      return pa::fail("unknown element type code %d", (int)(dtype)); \
    }                                                                \
  } while (0)

extern "C" int pa_embed_gather(void* stream, int dtype, const int* ids, const void* table, void* out, int tokens,
                               int hidden, int vocab) {
  if (tokens == 0) return 0;
  PA_REQUIRE(tokens > 0 && hidden > 0 && vocab > 0, "embed_gather: bad sizes tokens=%d hidden=%d vocab=%d", tokens,
             hidden, vocab);
  PA_DISPATCH(dtype, hipLaunchKernelGGL(embed_gather_kernel<T>, dim3(tokens), dim3(256), 0, (hipStream_t)stream, ids,
                                        (const T*)table, (T*)out, hidden, vocab));
  return check_launch("embed_gather");
}

extern "C" int pa_carry_tokens(void* stream, const int* sampled, const int* src, const int* dst, int* ids, int n,
                               int sampled_rows, int tokens) {
  if (n == 0) return 0;
  PA_REQUIRE(n > 0 && sampled_rows > 0 && tokens > 0, "carry_tokens: bad sizes n=%d sampled=%d tokens=%d", n,
             sampled_rows, tokens);
  hipLaunchKernelGGL(carry_tokens_kernel, dim3((n + 255) / 256), dim3(256), 0, (hipStream_t)stream, sampled, src, dst,
                     ids, n, sampled_rows, tokens);
  return check_launch("carry_tokens");
}

// Reads `bytes` (a multiple of 16) from src with `blocks` workgroups of 256 threads; out: one word a workgroup.
extern "C" int pa_stream_read(void* stream, const void* src, long bytes, void* out, int blocks) {
  PA_REQUIRE(src && out && bytes > 0 && bytes % 16 == 0 && blocks > 0, "stream_read: bad operands");
  hipLaunchKernelGGL(stream_read_kernel, dim3(blocks), dim3(256), 0, (hipStream_t)stream, (const uint4*)src,
                     (size_t)(bytes / 16), (unsigned*)out);
  return check_launch("stream_read");
}

extern "C" int pa_zero_fresh_rows(void* stream, void* data, long row_bytes, const int* slots, const int* fresh, int nseq,
                                  int num_rows) {
  if (nseq == 0 || row_bytes == 0) return 0;
  PA_REQUIRE(nseq > 0 && num_rows > 0 && row_bytes > 0 && row_bytes % 4 == 0,
             "zero_fresh_rows: bad sizes sequences=%d rows=%d row_bytes=%ld (a multiple of 4)", nseq, num_rows, row_bytes);
  PA_REQUIRE(data && slots && fresh, "zero_fresh_rows: a null operand");
  const long words = row_bytes / 4;
  const int pieces = (int)((words + 4095) / 4096 < 64 ? (words + 4095) / 4096 : 64);
  hipLaunchKernelGGL(zero_fresh_rows_kernel, dim3(nseq, pieces), dim3(256), 0, (hipStream_t)stream, (uint32_t*)data, words,
                     slots, fresh, num_rows);
  return check_launch("zero_fresh_rows");
}

static int rmsnorm_launch(void* stream, int dtype, const void* x, const float* parts, int slices, long slice_stride,
                          void* residual, const float* w, void* out, const int* rows, int nrows, int hidden, float eps) {
  const int vec = dtype == kF32 ? 4 : 8;
  if (hidden % vec == 0 && hidden / vec <= 4 * 1024) {
    const int nvec = hidden / vec;
    const int nv = (nvec + 1023) / 1024;   // vectors per thread: 1, 2 or 4
    const int per = nv == 3 ? 4 : nv;
    const int threads = (((nvec + per - 1) / per) + 63) / 64 * 64;
#define PA_RMS(NV)                                                                                                   \
  PA_DISPATCH(dtype, hipLaunchKernelGGL((rmsnorm_vec_kernel<T, NV>), dim3(nrows), dim3(threads), 0, (hipStream_t)stream, \
                                        (const T*)x, parts, slices, (size_t)slice_stride, (T*)residual, w, (T*)out, rows, \
                                        hidden, eps))
    if (per == 1) {
      PA_RMS(1);
    } else if (per == 2) {
      PA_RMS(2);
    } else {
      PA_RMS(4);
    }
#undef PA_RMS
    return check_launch("rmsnorm");
  }
  const int threads = hidden >= 2048 ? 512 : (hidden >= 512 ? 256 : 64);
  PA_DISPATCH(dtype, hipLaunchKernelGGL(rmsnorm_kernel<T>, dim3(nrows), dim3(threads), 0, (hipStream_t)stream,
                                        (const T*)x, parts, slices, (size_t)slice_stride, (T*)residual, w, (T*)out, rows,
                                        hidden, eps));
  return check_launch("rmsnorm");
}

extern "C" int pa_rmsnorm(void* stream, int dtype, const void* x, void* residual, const float* w, void* out,
                          const int* rows, int nrows, int hidden, float eps) {
  if (nrows == 0) return 0;
  PA_REQUIRE(nrows > 0 && hidden > 0, "rmsnorm: bad sizes rows=%d hidden=%d", nrows, hidden);
  return rmsnorm_launch(stream, dtype, x, nullptr, 0, 0, residual, w, out, rows, nrows, hidden, eps);
}

extern "C" int pa_rmsnorm_slices(void* stream, int dtype, const float* parts, int slices, long slice_stride,
                                 void* residual, const float* w, void* out, const int* rows, int nrows, int hidden,
                                 float eps) {
  if (nrows == 0) return 0;
  PA_REQUIRE(nrows > 0 && hidden > 0, "rmsnorm: bad sizes rows=%d hidden=%d", nrows, hidden);
  PA_REQUIRE(parts && slices >= 1 && slice_stride >= 0 && hidden % 4 == 0,
             "rmsnorm: %d slices %ld apart of rows of %d (a multiple of 4)", slices, slice_stride, hidden);
  return rmsnorm_launch(stream, dtype, nullptr, parts, slices, slice_stride, residual, w, out, rows, nrows, hidden, eps);
}

extern "C" int pa_silu_mul(void* stream, int dtype, const void* gate_up, void* out, int tokens, int inter, int act) {
  if (tokens == 0) return 0;
  PA_REQUIRE(tokens > 0 && inter > 0, "silu_mul: bad sizes tokens=%d inter=%d", tokens, inter);
  PA_REQUIRE(act >= 0 && act < kActCount, "silu_mul: unknown activation code %d", act);
  const size_t total = (size_t)tokens * inter;
  if (dtype == kBF16 && inter % 8 == 0) {
    const size_t groups = total / 8;
    hipLaunchKernelGGL(silu_mul_vec_kernel, dim3((unsigned)((groups + 255) / 256)), dim3(256), 0, (hipStream_t)stream,
                       (const bf16*)gate_up, (bf16*)out, groups, act);
    return check_launch("silu_mul");
  }
  const unsigned blocks = (unsigned)((total + 255) / 256);
  PA_DISPATCH(dtype, hipLaunchKernelGGL(silu_mul_kernel<T>, dim3(blocks), dim3(256), 0, (hipStream_t)stream,
                                        (const T*)gate_up, (T*)out, inter, total, act));
  return check_launch("silu_mul");
}

extern "C" int pa_gather_rows(void* stream, int dtype, const void* x, const int* rows, void* out, int nrows,
                              int width) {
  if (nrows == 0) return 0;
  PA_REQUIRE(nrows > 0 && width > 0, "gather_rows: bad sizes rows=%d width=%d", nrows, width);
  PA_DISPATCH(dtype, hipLaunchKernelGGL(gather_rows_kernel<T>, dim3(nrows), dim3(256), 0, (hipStream_t)stream,
                                        (const T*)x, rows, (T*)out, width));
  return check_launch("gather_rows");
}

extern "C" int pa_add_bias(void* stream, int dtype, void* y, const float* b, int tokens, int width) {
  if (tokens == 0) return 0;
  PA_REQUIRE(tokens > 0 && width > 0, "add_bias: bad sizes tokens=%d width=%d", tokens, width);
  const size_t total = (size_t)tokens * width;
  const unsigned blocks = (unsigned)((total + 255) / 256);
  PA_DISPATCH(dtype, hipLaunchKernelGGL(add_bias_kernel<T>, dim3(blocks), dim3(256), 0, (hipStream_t)stream, (T*)y, b,
                                        width, total));
  return check_launch("add_bias");
}

extern "C" int pa_to_f32(void* stream, int dtype, const void* x, float* out, long total) {
  if (total == 0) return 0;
  PA_REQUIRE(total > 0, "to_f32: bad size %ld", total);
  const unsigned blocks = (unsigned)(((size_t)total + 255) / 256);
  PA_DISPATCH(dtype, hipLaunchKernelGGL(to_f32_kernel<T>, dim3(blocks), dim3(256), 0, (hipStream_t)stream,
                                        (const T*)x, out, (size_t)total));
  return check_launch("to_f32");
}
