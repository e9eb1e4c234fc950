// C[M,N] = A[M,K] * W[N,K]^T (+ bias[N]) with true 32-bit arithmetic: every
// product and every sum is an IEEE float FMA on the vector ALU, no matrix-core
// mode of reduced precision.  It is the matrix product of the 32-bit path and
// the slow, safe product for sizes the MFMA kernels refuse.
//
// Each output element sums its K products in ascending k, sixteen at a time with
// one FMA each, and adds the sixteens up with a compensated sum (the rounding
// error of every addition is carried along and taken off the next term), so
// that long rows round no worse than short ones: a 9,728-term row is off by
// 3e-7 of the largest output instead of 4e-6.  The order is fixed, so a row's
// result does not depend on the number of rows, on the tile it falls in, or
// on what else is in the batch.
//
// Reference counterpart: y = x W^T (+b), W [out, in]
// (crates/prelude-core/src/models/commons/linear.rs:30-98; f32 GEMM with
// 32-bit compute, crates/prelude-cuda/src/ops/gemm.rs:359-365).
#include "common.h"
#include "api.h"

namespace pa {

constexpr int kTileM = 64, kTileN = 64, kTileK = 16;

template <typename TA, typename TW, typename TC>
__global__ __launch_bounds__(256) void gemm_plain_kernel(const TA* __restrict__ a, const TW* __restrict__ w,
                                                         const float* __restrict__ bias, TC* __restrict__ c, int m,
                                                         int n, int k, long lda, long ldw, long ldc) {
  __shared__ float as[kTileK][kTileM + 4];
  __shared__ float ws[kTileK][kTileN + 4];
  const int tx = threadIdx.x % 16, ty = threadIdx.x / 16;
  const int m0 = blockIdx.y * kTileM, n0 = blockIdx.x * kTileN;
  float acc[4][4] = {};
  float lost[4][4] = {};   // what the additions into acc have rounded away so far
  for (int k0 = 0; k0 < k; k0 += kTileK) {
    // 64 x 16 elements of each operand, four per thread.
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int e = threadIdx.x + i * 256;
      const int row = e / kTileK, kk = e % kTileK;
      const int gk = k0 + kk;
      const int gm = m0 + row, gn = n0 + row;
      as[kk][row] = (gm < m && gk < k) ? to_f32(a[(size_t)gm * lda + gk]) : 0.f;
      ws[kk][row] = (gn < n && gk < k) ? to_f32(w[(size_t)gn * ldw + gk]) : 0.f;
    }
    __syncthreads();
    float part[4][4] = {};
#pragma unroll
    for (int kk = 0; kk < kTileK; ++kk) {
      float av[4], wv[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) av[i] = as[kk][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) wv[j] = ws[kk][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) part[i][j] = fmaf(av[i], wv[j], part[i][j]);
    }
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float y = part[i][j] - lost[i][j];
        const float t = acc[i][j] + y;
        lost[i][j] = (t - acc[i][j]) - y;
        acc[i][j] = t;
      }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int gm = m0 + ty * 4 + i;
    if (gm >= m) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int gn = n0 + tx * 4 + j;
      if (gn >= n) continue;
      float v = acc[i][j];
      if (bias) v += bias[gn];
      c[(size_t)gm * ldc + gn] = from_f32<TC>(v);
    }
  }
}

template <typename TA, typename TW, typename TC>
int launch_plain(hipStream_t st, const void* a, const void* w, const float* bias, void* c, int m, int n, int k, long lda,
                 long ldw, long ldc) {
  dim3 grid((n + kTileN - 1) / kTileN, (m + kTileM - 1) / kTileM);
  hipLaunchKernelGGL((gemm_plain_kernel<TA, TW, TC>), grid, dim3(256), 0, st, (const TA*)a, (const TW*)w, bias, (TC*)c,
                     m, n, k, lda, ldw, ldc);
  return check_launch("gemm_plain");
}

}  // namespace pa

using namespace pa;

// in_dtype: element type of A and W; out_dtype: element type of C.
extern "C" int pa_gemm_plain(void* stream, int in_dtype, int out_dtype, const void* a, const void* w,
                             const float* bias, void* c, int m, int n, int k, long lda, long ldw, long ldc) {
  if (m == 0 || n == 0) return 0;
  PA_REQUIRE(m > 0 && n > 0 && k > 0, "gemm_plain: bad sizes m=%d n=%d k=%d", m, n, k);
  PA_REQUIRE(lda >= k && ldw >= k && ldc >= n, "gemm_plain: a row stride is smaller than the row (lda=%ld ldw=%ld ldc=%ld)",
             lda, ldw, ldc);
  PA_REQUIRE((m + kTileM - 1) / kTileM <= 65535, "gemm_plain: m=%d needs more than 65535 row tiles", m);
  hipStream_t st = (hipStream_t)stream;
  if (in_dtype == kF32 && out_dtype == kF32) return launch_plain<float, float, float>(st, a, w, bias, c, m, n, k, lda, ldw, ldc);
  if (in_dtype == kBF16 && out_dtype == kBF16) return launch_plain<bf16, bf16, bf16>(st, a, w, bias, c, m, n, k, lda, ldw, ldc);
  if (in_dtype == kBF16 && out_dtype == kF32) return launch_plain<bf16, bf16, float>(st, a, w, bias, c, m, n, k, lda, ldw, ldc);
  return pa::fail("gemm_plain: unsupported element types in=%d out=%d", in_dtype, out_dtype);
}
