// Dense fp16 GEMM of the two-pass prefill path through the vendor library:
//   C[M,N] = A[M,K] . Wd[N,K]^T,  Wd = the weights dequantized to fp16 by dequant_kernel.
// Once the weights are plain fp16 the multiplication is an ordinary library
// GEMM, and hipBLASLt's kernels for gfx950 run it faster than gemm_dense_kernel
// (dequantize + GEMM at M = 2048, N = 14336, K = 4096: 222 us against 340 us).
// The library is opened at run time (dlopen), never linked: a process that
// already holds a copy (PyTorch ships one with the same soname) shares it, and
// a machine without it simply keeps the hand-written GEMM.
// It is opt-in: the library's own choice by shape never takes this path; only
// an explicit variant index (5), or a tuning rule that names it, does.  The
// library is opened, and its handle created
// for the device current then, by the first cuthip_variant_available(MATMUL_GGUF,
// 5) or the first use; a caller that captures streams does one of these before it
// captures.
#include <dlfcn.h>
#include <hipblaslt/hipblaslt.h>

#include <cstdlib>
#include <map>
#include <mutex>
#include <tuple>

#include "common.hpp"

namespace cuthip {

namespace {

struct BlasLtApi {
  decltype(&hipblasLtCreate) create = nullptr;
  decltype(&hipblasLtMatrixLayoutCreate) layout_create = nullptr;
  decltype(&hipblasLtMatmulDescCreate) desc_create = nullptr;
  decltype(&hipblasLtMatmulDescSetAttribute) desc_set = nullptr;
  decltype(&hipblasLtMatmulPreferenceCreate) pref_create = nullptr;
  decltype(&hipblasLtMatmulPreferenceSetAttribute) pref_set = nullptr;
  decltype(&hipblasLtMatmulPreferenceDestroy) pref_destroy = nullptr;
  decltype(&hipblasLtMatmulAlgoGetHeuristic) heuristic = nullptr;
  decltype(&hipblasLtMatmul) matmul = nullptr;
  decltype(&hipblasLtMatmulDescDestroy) desc_destroy = nullptr;
  decltype(&hipblasLtMatrixLayoutDestroy) layout_destroy = nullptr;
  hipblasLtHandle_t handle = nullptr;
  int device = -1;   // the device that was current when the handle was created
  bool ok = false;
};

// one prepared problem: descriptors and the algorithm the heuristic picked
struct BlasLtPlan {
  hipblasLtMatmulDesc_t desc = nullptr;
  hipblasLtMatrixLayout_t a = nullptr, b = nullptr, c = nullptr;
  hipblasLtMatmulAlgo_t algo;
  size_t workspace = 0;
  bool tried = false, ok = false;
  uint64_t last_use = 0;
};
constexpr size_t kMaxPlans = 64;   // prepared problems kept; the least recently used one makes room for a new shape

std::mutex g_mu;
BlasLtApi g_api;
bool g_tried = false;
typedef std::tuple<uint32_t, uint32_t, uint32_t, uint32_t, uint32_t, int, size_t> PlanKey;
std::map<PlanKey, BlasLtPlan> g_plans;
uint64_t g_use_counter = 0;

template <typename F> bool sym(void *dl, const char *name, F &fn) {
  fn = reinterpret_cast<F>(dlsym(dl, name));
  return fn != nullptr;
}

// caller holds g_mu
BlasLtApi &api() {
  if (g_tried) return g_api;
  g_tried = true;
  if (const char *off = std::getenv("CUT_HIP_NO_BLASLT")) {
    if (off[0] && off[0] != '0') return g_api;
  }
  int ndev = 0, dev = -1;
  if (hipGetDeviceCount(&ndev) != hipSuccess || ndev <= 0 || hipGetDevice(&dev) != hipSuccess) {
    (void)hipGetLastError();
    g_tried = false;   // no device yet: ask again later
    return g_api;
  }
  void *dl = dlopen("libhipblaslt.so.1", RTLD_NOW | RTLD_LOCAL);
  if (!dl) dl = dlopen("/opt/rocm/lib/libhipblaslt.so.1", RTLD_NOW | RTLD_LOCAL);
  if (!dl) return g_api;
  BlasLtApi a;
  bool all = sym(dl, "hipblasLtCreate", a.create) && sym(dl, "hipblasLtMatrixLayoutCreate", a.layout_create) &&
             sym(dl, "hipblasLtMatmulDescCreate", a.desc_create) && sym(dl, "hipblasLtMatmulDescSetAttribute", a.desc_set) &&
             sym(dl, "hipblasLtMatmulPreferenceCreate", a.pref_create) &&
             sym(dl, "hipblasLtMatmulPreferenceSetAttribute", a.pref_set) &&
             sym(dl, "hipblasLtMatmulPreferenceDestroy", a.pref_destroy) &&
             sym(dl, "hipblasLtMatmulAlgoGetHeuristic", a.heuristic) && sym(dl, "hipblasLtMatmul", a.matmul) &&
             sym(dl, "hipblasLtMatmulDescDestroy", a.desc_destroy) && sym(dl, "hipblasLtMatrixLayoutDestroy", a.layout_destroy);
  if (!all) return g_api;
  if (a.create(&a.handle) != HIPBLAS_STATUS_SUCCESS) return g_api;
  a.device = dev;
  a.ok = true;
  g_api = a;
  return g_api;
}

}  // namespace

bool blaslt_available() {
  std::lock_guard<std::mutex> lock(g_mu);
  const BlasLtApi &lt = api();
  if (!lt.ok) return false;
  int dev = -1;
  return hipGetDevice(&dev) == hipSuccess && dev == lt.device;   // the handle belongs to one device
}

// Row-major C = A . Wd^T is, column-major, C^T (N x M) = op_T(Wd as K x N) . (A as K x M).
// Returns CUTHIP_OK, or CUTHIP_ERR_INVALID with the error set when the library has no kernel for the problem.
int launch_blaslt_gemm(const void *Wd, const void *A16, void *C, int c_f16, uint32_t M, uint32_t K, uint32_t N, uint32_t strideA,
                       uint32_t strideC, void *workspace, size_t workspace_bytes, hipStream_t stream) {
  std::unique_lock<std::mutex> lock(g_mu);
  BlasLtApi &lt = api();
  int dev = -1;
  if (!lt.ok || hipGetDevice(&dev) != hipSuccess || dev != lt.device) {
    set_error("variant 5 needs hipBLASLt (libhipblaslt.so.1 was not found, CUT_HIP_NO_BLASLT is set, or its handle belongs "
              "to device %d and the current device is %d)", lt.device, dev);
    return CUTHIP_ERR_INVALID;
  }
  const PlanKey key{M, K, N, strideA, strideC, c_f16, workspace_bytes};
  if (g_plans.find(key) == g_plans.end() && g_plans.size() >= kMaxPlans) {   // make room: drop the least recently used
    auto victim = g_plans.begin();
    for (auto it = g_plans.begin(); it != g_plans.end(); ++it)
      if (it->second.last_use < victim->second.last_use) victim = it;
    BlasLtPlan &v = victim->second;
    if (v.desc) lt.desc_destroy(v.desc);
    if (v.a) lt.layout_destroy(v.a);
    if (v.b) lt.layout_destroy(v.b);
    if (v.c) lt.layout_destroy(v.c);
    g_plans.erase(victim);
  }
  BlasLtPlan &plan = g_plans[key];
  plan.last_use = ++g_use_counter;
  if (!plan.tried) {
    plan.tried = true;
    const hipblasOperation_t opT = HIPBLAS_OP_T, opN = HIPBLAS_OP_N;
    const hipDataType ctype = c_f16 ? HIP_R_16F : HIP_R_32F;
    bool ok = lt.desc_create(&plan.desc, HIPBLAS_COMPUTE_32F, HIP_R_32F) == HIPBLAS_STATUS_SUCCESS &&
              lt.desc_set(plan.desc, HIPBLASLT_MATMUL_DESC_TRANSA, &opT, sizeof(opT)) == HIPBLAS_STATUS_SUCCESS &&
              lt.desc_set(plan.desc, HIPBLASLT_MATMUL_DESC_TRANSB, &opN, sizeof(opN)) == HIPBLAS_STATUS_SUCCESS &&
              lt.layout_create(&plan.a, HIP_R_16F, K, N, K) == HIPBLAS_STATUS_SUCCESS &&
              lt.layout_create(&plan.b, HIP_R_16F, K, M, strideA) == HIPBLAS_STATUS_SUCCESS &&
              lt.layout_create(&plan.c, ctype, N, M, strideC) == HIPBLAS_STATUS_SUCCESS;
    hipblasLtMatmulPreference_t pref = nullptr;
    ok = ok && lt.pref_create(&pref) == HIPBLAS_STATUS_SUCCESS;
    if (ok) {
      const uint64_t max_ws = workspace_bytes;
      ok = lt.pref_set(pref, HIPBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES, &max_ws, sizeof(max_ws)) == HIPBLAS_STATUS_SUCCESS;
    }
    if (ok) {
      hipblasLtMatmulHeuristicResult_t res[1];
      int found = 0;
      ok = lt.heuristic(lt.handle, plan.desc, plan.a, plan.b, plan.c, plan.c, pref, 1, res, &found) == HIPBLAS_STATUS_SUCCESS &&
           found > 0 && res[0].workspaceSize <= workspace_bytes;
      if (ok) {
        plan.algo = res[0].algo;
        plan.workspace = res[0].workspaceSize;
      }
    }
    if (pref) lt.pref_destroy(pref);
    plan.ok = ok;
  }
  if (!plan.ok) {
    set_error("hipBLASLt has no kernel for M = %u, N = %u, K = %u (fp16 in, %s out)", M, N, K, c_f16 ? "fp16" : "fp32");
    return CUTHIP_ERR_INVALID;
  }
  // the enqueue itself runs under the lock too: an eviction by another thread must not destroy these descriptors
  // while the library reads them (the call only enqueues; it does not wait for the GPU)
  const float alpha = 1.0f, beta = 0.0f;
  hipblasStatus_t st = lt.matmul(lt.handle, plan.desc, &alpha, Wd, plan.a, A16, plan.b, &beta, C, plan.c, C, plan.c, &plan.algo,
                                 plan.workspace ? workspace : nullptr, plan.workspace, stream);
  if (st != HIPBLAS_STATUS_SUCCESS) {
    set_error("hipblasLtMatmul failed with status %d", (int)st);
    return CUTHIP_ERR_HIP;
  }
  return CUTHIP_OK;
}

}  // namespace cuthip
