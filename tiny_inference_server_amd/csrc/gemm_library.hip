// C[M,N] = X[M,K] . W[N,K]^T (+ R[M,N]) in bfloat16 through hipBLASLt: the matrix product of many rows, where
// the reference's engine uses a library too (x @ W, main_models_new.py:19-20).
//
// The library is called directly, not through the tensor framework, because of what a call costs on the host:
// choosing an algorithm for a shape takes as long as launching it, and the framework's path asks again on every
// call (18 us a product measured on MI355X's host; a prompt step of 32 blocks issues 128 of them). Here the
// descriptors and the algorithm of a shape are made once and kept, which leaves the launch itself (9.5 us).
// The kernel that runs is the library's own first choice for the shape.
//
// What the caller must keep to, checked here: every operand 16-byte aligned with row strides in steps of 8
// elements (so one plan serves every call of a shape: nothing about a kernel's choice depends on where the operands
// lie), and an output that is not the residual (a kernel that cuts tiles over workgroups reads the residual's tile
// when it finishes the tile; with an output of its own, no order of its workgroups can read a tile that was already
// written). Which shapes may come here at all is the caller's business (ops/hip_ops.py keeps the list of widths).
//
// Row-major operands are handed over as their column-major transposes: D^T [N x M] = W [N x K] . X^T [K x M], with W
// as stored ([N, K] row-major = K x N column-major) under a transpose flag.
#include <hipblaslt/hipblaslt-ext.hpp>
#include <hipblaslt/hipblaslt.h>

#include <cstdio>
#include <cstdlib>
#include <list>
#include <map>
#include <mutex>
#include <string>
#include <tuple>

#include "common.h"

TIS_DEFINE_LAST_ERROR(tis_gemm_library)

namespace {

using Key = std::tuple<int, int, int, long, long, long, int>;   // (M, N, K, x_ld, r_ld or 0, c_ld, 32-bit output)

struct Plan {
  hipblasLtMatmulDesc_t desc = nullptr;
  hipblasLtMatrixLayout_t w = nullptr, x = nullptr, r = nullptr, c = nullptr;
  hipblasLtMatmulAlgo_t algo;
  size_t workspace_asked = 0;
  std::string kernel;
  std::list<Key>::iterator used;      // its place in the order of use

  void destroy() {
    if (desc) hipblasLtMatmulDescDestroy(desc);
    for (hipblasLtMatrixLayout_t l : {w, x, r, c})
      if (l) hipblasLtMatrixLayoutDestroy(l);
    desc = nullptr;
    w = x = r = c = nullptr;
  }
};

struct DeviceState {
  hipblasLtHandle_t handle = nullptr;
  void* workspace = nullptr;
  std::map<Key, Plan> plans;
  std::list<Key> order;               // least recently used first
};

// A serving run meets a shape per row count; rows come rounded (see the caller), so a few dozen shapes are all there
// are. Beyond this many the least recently used plan's descriptors are destroyed.
constexpr size_t kMaxPlans = 256;
constexpr size_t kWorkspaceBytes = 32u << 20;   // what the library is told it may use for split reductions
// Kernels that cut tiles over workgroups keep partial tiles and arrival flags in the workspace: tile size x 4 bytes x
// workgroups, which comes to 64 MiB for 256 x 256 tiles on 256 compute units, while the heuristic reports a need of 0
// for such shapes under the 32 MiB it is told. What is allocated is therefore more than either figure, and starts
// zeroed.
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

// The plan of a shape: found, or made (descriptors, the heuristic's first choice, its kernel's name).
int plan_of(DeviceState* st, const Key& key, bool has_residual, Plan** out) {
  auto it = st->plans.find(key);
  if (it != st->plans.end()) {
    st->order.splice(st->order.end(), st->order, it->second.used);
    *out = &it->second;
    return 0;
  }
  const int M = std::get<0>(key), N = std::get<1>(key), K = std::get<2>(key);
  const long x_ld = std::get<3>(key), r_ld = std::get<4>(key), c_ld = std::get<5>(key);
  const hipDataType out_type = std::get<6>(key) ? HIP_R_32F : HIP_R_16BF;
  Plan p;
  const hipblasOperation_t transposed = HIPBLAS_OP_T, plain = HIPBLAS_OP_N;
  bool ok = hipblasLtMatmulDescCreate(&p.desc, HIPBLAS_COMPUTE_32F, HIP_R_32F) == HIPBLAS_STATUS_SUCCESS;
  ok = ok && hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_TRANSA, &transposed, sizeof(transposed)) == HIPBLAS_STATUS_SUCCESS;
  ok = ok && hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_TRANSB, &plain, sizeof(plain)) == HIPBLAS_STATUS_SUCCESS;
  ok = ok && hipblasLtMatrixLayoutCreate(&p.w, HIP_R_16BF, K, N, K) == HIPBLAS_STATUS_SUCCESS;
  ok = ok && hipblasLtMatrixLayoutCreate(&p.x, HIP_R_16BF, K, M, x_ld) == HIPBLAS_STATUS_SUCCESS;
  ok = ok && hipblasLtMatrixLayoutCreate(&p.r, out_type, N, M, has_residual ? r_ld : c_ld) == HIPBLAS_STATUS_SUCCESS;
  ok = ok && hipblasLtMatrixLayoutCreate(&p.c, out_type, N, M, c_ld) == HIPBLAS_STATUS_SUCCESS;
  if (!ok) {
    p.destroy();
    return tis_fail("gemm_library: the library refused the descriptors of M=%d N=%d K=%d", M, N, K);
  }
  hipblasLtMatmulPreference_t pref;
  if (hipblasLtMatmulPreferenceCreate(&pref) != HIPBLAS_STATUS_SUCCESS) {
    p.destroy();
    return tis_fail("gemm_library: no preference object");
  }
  size_t ws = kWorkspaceBytes;
  hipblasLtMatmulPreferenceSetAttribute(pref, HIPBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES, &ws, sizeof(ws));
  hipblasLtMatmulHeuristicResult_t found[1];
  int n_found = 0;
  const hipblasStatus_t hs =
      hipblasLtMatmulAlgoGetHeuristic(st->handle, p.desc, p.w, p.x, p.r, p.c, pref, 1, found, &n_found);
  hipblasLtMatmulPreferenceDestroy(pref);
  if (hs != HIPBLAS_STATUS_SUCCESS || n_found < 1) {
    p.destroy();
    return tis_fail("gemm_library: the library has no algorithm for M=%d N=%d K=%d (status %d)", M, N, K, (int)hs);
  }
  p.algo = found[0].algo;
  p.workspace_asked = found[0].workspaceSize;
  p.kernel = hipblaslt_ext::getKernelNameFromAlgo(st->handle, p.algo);
  while (st->plans.size() >= kMaxPlans) {
    auto oldest = st->plans.find(st->order.front());
    oldest->second.destroy();
    st->plans.erase(oldest);
    st->order.pop_front();
  }
  st->order.push_back(key);
  p.used = std::prev(st->order.end());
  it = st->plans.emplace(key, p).first;
  *out = &it->second;
  // TIS_TRACE_SHAPES=1: a line on standard error before the first launch of every new shape, flushed, so that a
  // run that ends badly has named the last kernel of the library's that was new to it
  static const bool trace = [] { const char* e = getenv("TIS_TRACE_SHAPES"); return e && e[0] == '1'; }();
  if (trace) {
    fprintf(stderr, "[tis-amd] library product, new shape: rows %d, out %d, in %d, residual %d, 32-bit out %d; "
            "workspace asked %zu; kernel %s\n", M, N, K, has_residual ? 1 : 0, std::get<6>(key), p.workspace_asked,
            p.kernel.c_str());
    fflush(stderr);
  }
  return 0;
}

int check_operands(const void* X, long x_ld, const void* W, const void* R, long r_ld, const void* C, long c_ld, int M,
                   int N, int K, int out_f32) {
  if (M < 0 || N < 0 || K < 1) return tis_fail("gemm_library: bad size M=%d N=%d K=%d", M, N, K);
  if (x_ld < K || c_ld < N || (R && r_ld < N)) return tis_fail("gemm_library: a row stride is shorter than its row");
  if (out_f32 && R) return tis_fail("gemm_library: a 32-bit result takes no residual");
  if (R && R == C) return tis_fail("gemm_library: the output must not be the residual");
  if (K % 8 || x_ld % 8 || c_ld % 8 || (R && r_ld % 8))
    return tis_fail("gemm_library: K=%d and the row strides (%ld, %ld, %ld) must be multiples of 8", K, x_ld, r_ld, c_ld);
  if (((uintptr_t)X | (uintptr_t)W | (uintptr_t)R | (uintptr_t)C) % 16)
    return tis_fail("gemm_library: operands must be 16-byte aligned");
  return 0;
}

}  // namespace

// Creates the device's handle and workspace. Call once before any stream capture: both allocate.
TIS_EXPORT int tis_gemm_library_init() {
  std::lock_guard<std::mutex> lock(g_mutex);
  DeviceState* st;
  return device_state(&st);
}

// R: null, or the residual added to the product (never C itself). A shape's first call asks the library for
// an algorithm and must not happen under stream capture; later calls only launch.
// out_f32: C holds 32-bit floats; no residual then.
TIS_EXPORT int tis_gemm_library(const void* X, long x_ld, const void* W, const void* R, long r_ld, void* C, long c_ld,
                                int M, int N, int K, int out_f32, hipStream_t stream) {
  if (M == 0 || N == 0) return 0;
  if (check_operands(X, x_ld, W, R, r_ld, C, c_ld, M, N, K, out_f32)) return -1;
  std::lock_guard<std::mutex> lock(g_mutex);
  DeviceState* st;
  if (device_state(&st)) return -1;
  Plan* p;
  if (plan_of(st, std::make_tuple(M, N, K, x_ld, R ? r_ld : 0L, c_ld, out_f32 ? 1 : 0), R != nullptr, &p)) return -1;
  const float alpha = 1.f, beta = R ? 1.f : 0.f;
  const hipblasStatus_t ms = hipblasLtMatmul(st->handle, p->desc, &alpha, W, p->w, X, p->x, &beta, R ? R : C, p->r, C,
                                             p->c, &p->algo, st->workspace, kWorkspaceBytes, stream);
  if (ms != HIPBLAS_STATUS_SUCCESS) return tis_fail("gemm_library: hipblasLtMatmul failed for M=%d N=%d K=%d (status %d)", M, N, K, (int)ms);
  return 0;
}

// What the library would run for a shape, without running it: the kernel's name goes into `name` (at most `name_len`
// bytes with the closing zero), the workspace it reports into *workspace. Host calls only; the plan is kept.
TIS_EXPORT int tis_gemm_library_describe(int M, int N, int K, long x_ld, long r_ld, long c_ld, int out_f32, char* name,
                                         int name_len, long* workspace) {
  if (M < 1 || N < 1 || K < 1) return tis_fail("gemm_library: bad size M=%d N=%d K=%d", M, N, K);
  std::lock_guard<std::mutex> lock(g_mutex);
  DeviceState* st;
  if (device_state(&st)) return -1;
  Plan* p;
  if (plan_of(st, std::make_tuple(M, N, K, x_ld, r_ld, c_ld, out_f32 ? 1 : 0), r_ld != 0, &p)) return -1;
  if (name && name_len > 0) snprintf(name, name_len, "%s", p->kernel.c_str());
  if (workspace) *workspace = (long)p->workspace_asked;
  return 0;
}

// Plans held for the current device (a bounded number: see kMaxPlans).
TIS_EXPORT int tis_gemm_library_plans() {
  std::lock_guard<std::mutex> lock(g_mutex);
  DeviceState* st;
  if (device_state(&st)) return -1;
  return (int)st->plans.size();
}
