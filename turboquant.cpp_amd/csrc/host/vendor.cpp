// Plain bfloat16 products of many rows through the vendor's matrix library (hipBLASLt), called from C.
//
// The reference hands its plain products to a BLAS where it has one (tq_matmul calls cblas_sgemv,
// /root/reference/src/engine/tq_ops.c:296-305); the step executor does the same for products of many rows without
// bias.  The library is not linked: its symbols are looked up at the first call in whatever copy the process has
// loaded already (the Python package's process holds one) or, failing that, in the system's, so that this library
// loads where hipBLASLt is absent and then simply never takes this path (tq_vendor_available() says which).
#include <dlfcn.h>
#include <hipblaslt/hipblaslt.h>

#include <map>
#include <mutex>
#include <tuple>

#include "host_common.h"
#include "vendor.h"

namespace {

struct Api {
  decltype(&hipblasLtCreate) create = nullptr;
  decltype(&hipblasLtMatmulDescCreate) desc_create = nullptr;
  decltype(&hipblasLtMatmulDescSetAttribute) desc_set = nullptr;
  decltype(&hipblasLtMatrixLayoutCreate) layout_create = nullptr;
  decltype(&hipblasLtMatmulPreferenceCreate) pref_create = nullptr;
  decltype(&hipblasLtMatmulPreferenceSetAttribute) pref_set = nullptr;
  decltype(&hipblasLtMatmulPreferenceDestroy) pref_destroy = nullptr;
  decltype(&hipblasLtMatmulDescDestroy) desc_destroy = nullptr;
  decltype(&hipblasLtMatrixLayoutDestroy) layout_destroy = nullptr;
  decltype(&hipblasLtMatmulAlgoGetHeuristic) heuristic = nullptr;
  decltype(&hipblasLtMatmul) matmul = nullptr;
  bool ok = false;
};

struct Problem {        // what the library was asked once for a shape, kept for the process's life
  hipblasLtMatmulDesc_t desc;
  hipblasLtMatrixLayout_t a, b, d;
  hipblasLtMatmulAlgo_t algo;
  size_t workspace;
  bool usable;
};

std::mutex g_lock;
Api g_api;
bool g_tried = false;
std::map<int, hipblasLtHandle_t> g_handles;                                   // by device
std::map<std::tuple<int, int, int, int, int64_t, int>, Problem> g_problems;  // device, M, N, K, lda, out type
constexpr size_t kMostProblems = 2048;     // shapes kept; a host that brings ever new row counts starts over beyond that

void forget(Problem& p) {
  if (p.desc) g_api.desc_destroy(p.desc);
  for (hipblasLtMatrixLayout_t l : {p.a, p.b, p.d})
    if (l) g_api.layout_destroy(l);
  p = Problem{};
}

template <class F>
bool sym(void* lib, const char* name, F& fn) {
  fn = reinterpret_cast<F>(dlsym(lib, name));
  return fn != nullptr;
}

void load_api() {
  if (g_tried) return;
  g_tried = true;
  void* lib = nullptr;
  // a copy that the process has loaded already comes first: two copies of the library in one process would each
  // keep device state of their own
  for (const char* name : {"libhipblaslt.so", "libhipblaslt.so.1", "libhipblaslt.so.0"}) {
    lib = dlopen(name, RTLD_NOW | RTLD_NOLOAD);
    if (lib) break;
  }
  if (!lib) {
    for (const char* name : {"libhipblaslt.so.1", "libhipblaslt.so", "/opt/rocm/lib/libhipblaslt.so"}) {
      lib = dlopen(name, RTLD_NOW | RTLD_LOCAL);
      if (lib) break;
    }
  }
  if (!lib) return;
  Api& a = g_api;
  a.ok = sym(lib, "hipblasLtCreate", a.create) && sym(lib, "hipblasLtMatmulDescCreate", a.desc_create) &&
         sym(lib, "hipblasLtMatmulDescSetAttribute", a.desc_set) && sym(lib, "hipblasLtMatrixLayoutCreate", a.layout_create) &&
         sym(lib, "hipblasLtMatmulPreferenceCreate", a.pref_create) &&
         sym(lib, "hipblasLtMatmulPreferenceSetAttribute", a.pref_set) &&
         sym(lib, "hipblasLtMatmulPreferenceDestroy", a.pref_destroy) && sym(lib, "hipblasLtMatmulDescDestroy", a.desc_destroy) &&
         sym(lib, "hipblasLtMatrixLayoutDestroy", a.layout_destroy) &&
         sym(lib, "hipblasLtMatmulAlgoGetHeuristic", a.heuristic) && sym(lib, "hipblasLtMatmul", a.matmul);
}

}  // namespace

extern "C" int tq_vendor_available(void) {
  std::lock_guard<std::mutex> hold(g_lock);
  load_api();
  return g_api.ok ? 1 : 0;
}

namespace {

// The library's plan for a shape (kept once made), or null: the library is absent or has no kernel for it.
// code: 0, TQ_ERR_UNSUPPORTED or 1000 + the library's status.
const Problem* problem_for(int M, int N, int K, int64_t lda, int out_is_bf16, hipblasLtHandle_t* handle, int* code) {
  *code = TQ_ERR_UNSUPPORTED;
  load_api();
  if (!g_api.ok) return nullptr;
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return nullptr;
  auto h = g_handles.find(dev);
  if (h == g_handles.end()) {
    hipblasLtHandle_t made = nullptr;
    if (g_api.create(&made) != HIPBLAS_STATUS_SUCCESS) return nullptr;
    h = g_handles.emplace(dev, made).first;
  }
  *handle = h->second;
  const auto key = std::make_tuple(dev, M, N, K, lda, out_is_bf16);
  auto p = g_problems.find(key);
  if (p == g_problems.end()) {
    if (g_problems.size() >= kMostProblems) {
      for (auto& kept : g_problems) forget(kept.second);
      g_problems.clear();
    }
    // Column-major as the library counts: out^T [N][M] = w [N][K] a^T, that is op(A) = A^T with A = w seen as
    // [K][N] with leading size K, and B = a seen as [K][M] with leading size lda.
    Problem pr{};
    hipblasStatus_t s = g_api.desc_create(&pr.desc, HIPBLAS_COMPUTE_32F, HIP_R_32F);
    if (s != HIPBLAS_STATUS_SUCCESS) {
      *code = 1000 + (int)s;
      return nullptr;
    }
    const int32_t ta = HIPBLAS_OP_T, tb = HIPBLAS_OP_N;
    g_api.desc_set(pr.desc, HIPBLASLT_MATMUL_DESC_TRANSA, &ta, sizeof(ta));
    g_api.desc_set(pr.desc, HIPBLASLT_MATMUL_DESC_TRANSB, &tb, sizeof(tb));
    const hipDataType out_type = out_is_bf16 ? HIP_R_16BF : HIP_R_32F;
    hipblasLtMatmulPreference_t pref = nullptr;
    if ((s = g_api.layout_create(&pr.a, HIP_R_16BF, K, N, K)) != HIPBLAS_STATUS_SUCCESS ||
        (s = g_api.layout_create(&pr.b, HIP_R_16BF, K, M, lda)) != HIPBLAS_STATUS_SUCCESS ||
        (s = g_api.layout_create(&pr.d, out_type, N, M, N)) != HIPBLAS_STATUS_SUCCESS ||
        (s = g_api.pref_create(&pref)) != HIPBLAS_STATUS_SUCCESS) {
      forget(pr);
      *code = 1000 + (int)s;
      return nullptr;
    }
    const uint64_t max_ws = TQ_VENDOR_WORKSPACE;
    g_api.pref_set(pref, HIPBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES, &max_ws, sizeof(max_ws));
    hipblasLtMatmulHeuristicResult_t found[1];
    int n_found = 0;
    s = g_api.heuristic(h->second, pr.desc, pr.a, pr.b, pr.d, pr.d, pref, 1, found, &n_found);
    g_api.pref_destroy(pref);
    pr.usable = s == HIPBLAS_STATUS_SUCCESS && n_found >= 1 && found[0].workspaceSize <= TQ_VENDOR_WORKSPACE;
    if (pr.usable) {
      pr.algo = found[0].algo;
      pr.workspace = found[0].workspaceSize;
    } else {
      forget(pr);          // what is kept says only that the library has nothing for this shape
    }
    p = g_problems.emplace(key, pr).first;
  }
  if (!p->second.usable) return nullptr;
  *code = 0;
  return &p->second;
}

}  // namespace

// Whether tq_vendor_product would take this product (asked once per shape of the library, then remembered); a
// caller decides with it before it plans its memory.
extern "C" int tq_vendor_takes(int M, int N, int K, int64_t lda, int out_is_bf16) {
  if (M <= 0 || N <= 0 || K <= 0) return 0;
  std::lock_guard<std::mutex> hold(g_lock);
  hipblasLtHandle_t handle = nullptr;
  int code = 0;
  return problem_for(M, N, K, lda, out_is_bf16, &handle, &code) != nullptr;
}

// out[m][n] = sum_k a[m][k] * w[n][k]: a bfloat16 [M][K] with row stride lda, w bfloat16 [N][K], out [M][N] in float
// (out_is_bf16 0) or bfloat16, sums in float.  workspace: TQ_VENDOR_WORKSPACE bytes that no other stream uses
// meanwhile.  Returns 0, TQ_ERR_UNSUPPORTED (the library is absent or has no kernel for the shape: nothing was
// launched) or 1000 + the library's status.
extern "C" int tq_vendor_product(const void* a, int64_t lda, const void* w, void* out, int out_is_bf16, int M, int N,
                                 int K, void* workspace, hipStream_t st) {
  if (M <= 0 || N <= 0) return 0;
  std::lock_guard<std::mutex> hold(g_lock);
  hipblasLtHandle_t handle = nullptr;
  int code = 0;
  const Problem* pr = problem_for(M, N, K, lda, out_is_bf16, &handle, &code);
  if (!pr) return code;
  const float one = 1.0f, zero = 0.0f;
  hipblasStatus_t s = g_api.matmul(handle, pr->desc, &one, w, pr->a, a, pr->b, &zero, out, pr->d, out, pr->d, &pr->algo,
                                   workspace, pr->workspace ? TQ_VENDOR_WORKSPACE : 0, st);
  return s == HIPBLAS_STATUS_SUCCESS ? 0 : 1000 + (int)s;
}
