// C[M,N] = X[M,K] . W[N,K]^T (+ R[M,N]) in bfloat16 through hipBLASLt: the matrix product of many rows, where
// the reference's engine uses a library too (x @ W, main_models_new.py:19-20).
//
// The library is called directly, not through the tensor framework, because of what a call costs on the host:
// choosing an algorithm for a shape takes as long as launching it, and the framework's path asks again on every
// call (18 us a product measured on MI355X's host; a prompt step of 32 blocks issues 128 of them). Here the
// descriptors and the algorithm of a shape are made once and kept, which leaves the launch itself (9.5 us).
// The kernels that run, and so the results, are the library's own choice for the shape, as before.
//
// Row-major operands are handed over as their column-major transposes: D^T [N x M] = W [N x K] . X^T [K x M], with W
// as stored ([N, K] row-major = K x N column-major) under a transpose flag.
#include <hipblaslt/hipblaslt.h>

#include <cstdio>
#include <cstdlib>
#include <map>
#include <mutex>
#include <tuple>

#include "common.h"

TIS_DEFINE_LAST_ERROR(tis_gemm_library)

namespace {

struct Plan {
  hipblasLtMatmulDesc_t desc;
  hipblasLtMatrixLayout_t w, x, r, c;
  hipblasLtMatmulAlgo_t algo;
};

struct DeviceState {
  hipblasLtHandle_t handle = nullptr;
  void* workspace = nullptr;
  // (M, N, K, x_ld, r_ld or 0, c_ld, 32-bit output)
  std::map<std::tuple<int, int, int, long, long, long, int>, Plan> plans;
};

constexpr size_t kWorkspaceBytes = 32u << 20;   // what the library may use for split reductions
// The library's kernels for these shapes split tiles over workgroups and keep partial tiles and arrival flags in the
// workspace; by tile size times workgroups that can come to 64 MiB, and for such shapes the heuristic reports a need
// of 0 under the 32 MiB limit. The allocation is therefore longer than the size the library is told, and starts
// zeroed: both cost nothing, change no choice the library makes, and keep a kernel that overran what it was told,
// or that met stale flags, inside memory that is the wrapper's own.
constexpr size_t kWorkspaceAllocated = 160u << 20;
std::mutex g_mutex;
std::map<int, DeviceState> g_devices;

int device_state(DeviceState** out) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return tis_fail("gemm_library: no current device");
  DeviceState& st = g_devices[dev];
  if (!st.handle) {
    if (hipblasLtCreate(&st.handle) != HIPBLAS_STATUS_SUCCESS) return tis_fail("gemm_library: hipblasLtCreate failed");
    if (hipMalloc(&st.workspace, kWorkspaceAllocated) != hipSuccess) {
      st.handle = nullptr;
      return tis_fail("gemm_library: no memory for the library's %zu-byte workspace", kWorkspaceAllocated);
    }
    if (hipMemset(st.workspace, 0, kWorkspaceAllocated) != hipSuccess || hipDeviceSynchronize() != hipSuccess) {
      st.handle = nullptr;
      return tis_fail("gemm_library: the workspace could not be cleared");
    }
  }
  *out = &st;
  return 0;
}

}  // namespace

// Creates the device's handle and workspace. Call once before any stream capture: both allocate.
TIS_EXPORT int tis_gemm_library_init() {
  std::lock_guard<std::mutex> lock(g_mutex);
  DeviceState* st;
  return device_state(&st);
}

// R: null, or the residual added to the product (it may be C itself). A shape's first call asks the library for
// an algorithm and must not happen under stream capture; later calls only launch.
// out_f32: C holds 32-bit floats (the output table's logits); no residual then.
TIS_EXPORT int tis_gemm_library(const void* X, long x_ld, const void* W, const void* R, long r_ld, void* C, long c_ld,
                                int M, int N, int K, int out_f32, hipStream_t stream) {
  if (M == 0 || N == 0) return 0;
  if (M < 0 || N < 0 || K < 1) return tis_fail("gemm_library: bad size M=%d N=%d K=%d", M, N, K);
  if (x_ld < K || c_ld < N || (R && r_ld < N)) return tis_fail("gemm_library: a row stride is shorter than its row");
  if (out_f32 && R) return tis_fail("gemm_library: a 32-bit result takes no residual");
  const hipDataType out_type = out_f32 ? HIP_R_32F : HIP_R_16BF;
  std::lock_guard<std::mutex> lock(g_mutex);
  DeviceState* st;
  if (device_state(&st)) return -1;
  const auto key = std::make_tuple(M, N, K, x_ld, R ? r_ld : 0L, c_ld, out_f32 ? 1 : 0);
  auto it = st->plans.find(key);
  if (it == st->plans.end()) {
    Plan p;
    const hipblasOperation_t transposed = HIPBLAS_OP_T, plain = HIPBLAS_OP_N;
    bool ok = hipblasLtMatmulDescCreate(&p.desc, HIPBLAS_COMPUTE_32F, HIP_R_32F) == HIPBLAS_STATUS_SUCCESS;
    ok = ok && hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_TRANSA, &transposed, sizeof(transposed)) == HIPBLAS_STATUS_SUCCESS;
    ok = ok && hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_TRANSB, &plain, sizeof(plain)) == HIPBLAS_STATUS_SUCCESS;
    ok = ok && hipblasLtMatrixLayoutCreate(&p.w, HIP_R_16BF, K, N, K) == HIPBLAS_STATUS_SUCCESS;
    ok = ok && hipblasLtMatrixLayoutCreate(&p.x, HIP_R_16BF, K, M, x_ld) == HIPBLAS_STATUS_SUCCESS;
    ok = ok && hipblasLtMatrixLayoutCreate(&p.r, out_type, N, M, R ? r_ld : c_ld) == HIPBLAS_STATUS_SUCCESS;
    ok = ok && hipblasLtMatrixLayoutCreate(&p.c, out_type, N, M, c_ld) == HIPBLAS_STATUS_SUCCESS;
    if (!ok) return tis_fail("gemm_library: the library refused the descriptors of M=%d N=%d K=%d", M, N, K);
    hipblasLtMatmulPreference_t pref;
    if (hipblasLtMatmulPreferenceCreate(&pref) != HIPBLAS_STATUS_SUCCESS) return tis_fail("gemm_library: no preference object");
    size_t ws = kWorkspaceBytes;
    hipblasLtMatmulPreferenceSetAttribute(pref, HIPBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES, &ws, sizeof(ws));
    hipblasLtMatmulHeuristicResult_t found[1];
    int n_found = 0;
    const hipblasStatus_t hs =
        hipblasLtMatmulAlgoGetHeuristic(st->handle, p.desc, p.w, p.x, p.r, p.c, pref, 1, found, &n_found);
    hipblasLtMatmulPreferenceDestroy(pref);
    if (hs != HIPBLAS_STATUS_SUCCESS || n_found < 1)
      return tis_fail("gemm_library: the library has no algorithm for M=%d N=%d K=%d (status %d)", M, N, K, (int)hs);
    p.algo = found[0].algo;
    it = st->plans.emplace(key, p).first;
    // TIS_TRACE_SHAPES=1: a line on standard error before the first launch of every new shape, flushed, so that a
    // run that ends badly has named the last kernel of the library's that was new to it
    static const bool trace = [] { const char* e = getenv("TIS_TRACE_SHAPES"); return e && e[0] == '1'; }();
    if (trace) {
      fprintf(stderr, "[tis-amd] library product, new shape: rows %d, out %d, in %d, residual %d, 32-bit out %d; workspace asked %zu\n",
              M, N, K, R ? 1 : 0, out_f32 ? 1 : 0, found[0].workspaceSize);
      fflush(stderr);
    }
  }
  const Plan& p = it->second;
  const float alpha = 1.f, beta = R ? 1.f : 0.f;
  const hipblasStatus_t ms = hipblasLtMatmul(st->handle, p.desc, &alpha, W, p.w, X, p.x, &beta, R ? R : C, p.r, C, p.c,
                                             &p.algo, st->workspace, kWorkspaceBytes, stream);
  if (ms != HIPBLAS_STATUS_SUCCESS) return tis_fail("gemm_library: hipblasLtMatmul failed for M=%d N=%d K=%d (status %d)", M, N, K, (int)ms);
  return 0;
}
