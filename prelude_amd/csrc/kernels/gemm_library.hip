// C[M,N] = X[M,K] * W[N,K]^T in bfloat16 with 32-bit accumulation through hipBLASLt: the matrix product of
// steps with many rows (prompt portions, large decode batches), where a library product stands as it does in the
// reference (crates/prelude-cuda/src/ops/gemm.rs:35-137 hands these to cuBLAS / CUTLASS).
//
// The library is called directly: the operation descriptor, the three layouts and the algorithm its heuristic
// names first are made once per shape and kept, so a later call is a map lookup and the library's launch: 14 us
// of host time a call against 20 through a tensor library's matmul (same kernel, same bits), which is what a
// small model's prefill step waits for.
//
// hipBLASLt counts in column-major terms.  W [N,K] in rows is a K x N matrix there (leading dimension K), taken
// transposed; X [M,K] is K x M; the result is N x M with leading dimension ldc, which is C [M,N] in rows.
#include "common.h"
#include "api.h"

#include <hipblaslt/hipblaslt.h>

#include <map>
#include <mutex>
#include <tuple>

namespace {

struct Plan {
  hipblasLtMatmulDesc_t op = nullptr;
  hipblasLtMatrixLayout_t w = nullptr, x = nullptr, c = nullptr;
  hipblasLtMatmulAlgo_t algo;
  size_t workspace = 0;
};

struct Library {
  hipblasLtHandle_t handle = nullptr;
  std::map<std::tuple<int, int, int, long, long, long>, Plan> plans;   // m, n, k, ldx, ldc, workspace allowed
};

std::mutex g_mutex;
std::map<int, Library> g_libraries;   // by device

#define PA_LT(call, what)                                                                   \
  do {                                                                                      \
    hipblasStatus_t s_ = (call);                                                            \
    if (s_ != HIPBLAS_STATUS_SUCCESS) return pa::fail("gemm_library: %s failed with status %d", what, (int)s_); \
  } while (0)

int make_plan(Library& lib, Plan& p, int m, int n, int k, long ldx, long ldc, long workspace_bytes) {
  PA_LT(hipblasLtMatmulDescCreate(&p.op, HIPBLAS_COMPUTE_32F, HIP_R_32F), "hipblasLtMatmulDescCreate");
  const int32_t trans = HIPBLAS_OP_T, plain = HIPBLAS_OP_N;
  PA_LT(hipblasLtMatmulDescSetAttribute(p.op, HIPBLASLT_MATMUL_DESC_TRANSA, &trans, sizeof(trans)), "setting TRANSA");
  PA_LT(hipblasLtMatmulDescSetAttribute(p.op, HIPBLASLT_MATMUL_DESC_TRANSB, &plain, sizeof(plain)), "setting TRANSB");
  PA_LT(hipblasLtMatrixLayoutCreate(&p.w, HIP_R_16BF, k, n, k), "layout of W");
  PA_LT(hipblasLtMatrixLayoutCreate(&p.x, HIP_R_16BF, k, m, ldx), "layout of X");
  PA_LT(hipblasLtMatrixLayoutCreate(&p.c, HIP_R_16BF, n, m, ldc), "layout of C");
  hipblasLtMatmulPreference_t pref = nullptr;
  PA_LT(hipblasLtMatmulPreferenceCreate(&pref), "hipblasLtMatmulPreferenceCreate");
  const uint64_t allowed = (uint64_t)workspace_bytes;
  hipblasStatus_t s = hipblasLtMatmulPreferenceSetAttribute(pref, HIPBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES, &allowed,
                                                            sizeof(allowed));
  hipblasLtMatmulHeuristicResult_t found[1];
  int count = 0;
  if (s == HIPBLAS_STATUS_SUCCESS)
    s = hipblasLtMatmulAlgoGetHeuristic(lib.handle, p.op, p.w, p.x, p.c, p.c, pref, 1, found, &count);
  hipblasLtMatmulPreferenceDestroy(pref);
  if (s != HIPBLAS_STATUS_SUCCESS) return pa::fail("gemm_library: the heuristic failed with status %d", (int)s);
  if (count < 1 || found[0].state != HIPBLAS_STATUS_SUCCESS)
    return pa::fail("gemm_library: no algorithm for m=%d n=%d k=%d (bfloat16, 32-bit accumulation)", m, n, k);
  if (found[0].workspaceSize > (size_t)workspace_bytes)
    return pa::fail("gemm_library: the algorithm wants %zu bytes of workspace, %ld are there", found[0].workspaceSize,
                    workspace_bytes);
  p.algo = found[0].algo;
  p.workspace = found[0].workspaceSize;
  return 0;
}

void drop_plan(Plan& p) {
  if (p.w) hipblasLtMatrixLayoutDestroy(p.w);
  if (p.x) hipblasLtMatrixLayoutDestroy(p.x);
  if (p.c) hipblasLtMatrixLayoutDestroy(p.c);
  if (p.op) hipblasLtMatmulDescDestroy(p.op);
  p = Plan();
}

}  // namespace

// workspace: device memory of workspace_bytes the library's kernels may use (stream-K partial sums); the same
// buffer for every call on a stream.  The first call with a shape makes and keeps its plan (host memory).
extern "C" int pa_gemm_library(void* stream, const void* x, const void* w, void* c, int m, int n, int k, long ldx,
                               long ldc, void* workspace, long workspace_bytes) {
  if (m == 0 || n == 0) return 0;
  PA_REQUIRE(m > 0 && n > 0 && k > 0, "gemm_library: bad sizes m=%d n=%d k=%d", m, n, k);
  PA_REQUIRE(ldx >= k && ldc >= n, "gemm_library: row strides %ld, %ld are smaller than k=%d, n=%d", ldx, ldc, k, n);
  PA_REQUIRE(workspace_bytes >= 0 && (workspace != nullptr || workspace_bytes == 0), "gemm_library: bad workspace");
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return pa::fail("gemm_library: hipGetDevice: %s", hipGetErrorString(e));

  std::lock_guard<std::mutex> hold(g_mutex);
  Library& lib = g_libraries[dev];
  if (!lib.handle) PA_LT(hipblasLtCreate(&lib.handle), "hipblasLtCreate");
  const auto key = std::make_tuple(m, n, k, ldx, ldc, workspace_bytes);
  auto it = lib.plans.find(key);
  if (it == lib.plans.end()) {
    if (lib.plans.size() >= 4096) {   // every row count a server ever saw: start over rather than grow for ever
      for (auto& kv : lib.plans) drop_plan(kv.second);
      lib.plans.clear();
    }
    Plan p;
    if (int rc = make_plan(lib, p, m, n, k, ldx, ldc, workspace_bytes)) {
      drop_plan(p);
      return rc;
    }
    it = lib.plans.emplace(key, p).first;
  }
  const Plan& p = it->second;
  const float one = 1.f, zero = 0.f;
  PA_LT(hipblasLtMatmul(lib.handle, p.op, &one, w, p.w, x, p.x, &zero, c, p.c, c, p.c, &p.algo, workspace,
                        (size_t)workspace_bytes, (hipStream_t)stream),
        "hipblasLtMatmul");
  return 0;
}
