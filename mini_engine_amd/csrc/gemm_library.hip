// The library matrix product, called without a framework in between.
//
// y[M, N] = x[M, K] . w[N, K]^T for bfloat16 operands through hipBLASLt (reference
// layers/linear.py:25-26 hands the same product to its library). The process already holds one copy
// of hipBLASLt, the one that PyTorch loaded; this file looks that copy up by its soname and never
// loads another, so nothing is linked against it and the core library loads where hipBLASLt is
// absent (the entry point then says so and the caller takes its other path).
//
// Going through the library's own entry point matters for host time: a product's descriptors,
// layouts and the algorithm that the heuristic picks are made once per shape and kept, so a call is
// one hipblasLtMatmul, a few microseconds of host work, where a framework's dispatch, descriptor
// set-up and heuristic query for every call take several times that. Steps that are not replayed
// from a graph (prompt portions, mixed batches) are bound by exactly this host time at small widths.
#include "common.h"
#include <hipblaslt/hipblaslt.h>
#include <dlfcn.h>
#include <map>
#include <mutex>
#include <tuple>

namespace {

struct Api {
  decltype(&hipblasLtCreate) create = nullptr;
  decltype(&hipblasLtMatmulDescCreate) desc_create = nullptr;
  decltype(&hipblasLtMatmulDescSetAttribute) desc_set = nullptr;
  decltype(&hipblasLtMatmulDescDestroy) desc_destroy = nullptr;
  decltype(&hipblasLtMatrixLayoutCreate) layout_create = nullptr;
  decltype(&hipblasLtMatrixLayoutSetAttribute) layout_set = nullptr;
  decltype(&hipblasLtMatrixLayoutDestroy) layout_destroy = nullptr;
  decltype(&hipblasLtMatmulPreferenceCreate) pref_create = nullptr;
  decltype(&hipblasLtMatmulPreferenceSetAttribute) pref_set = nullptr;
  decltype(&hipblasLtMatmulPreferenceDestroy) pref_destroy = nullptr;
  decltype(&hipblasLtMatmulAlgoGetHeuristic) heuristic = nullptr;
  decltype(&hipblasLtMatmul) matmul = nullptr;
  bool looked = false, ok = false;
};

// A product of one shape: everything hipblasLtMatmul needs beside the pointers.
struct Plan {
  hipblasLtMatmulDesc_t desc = nullptr;
  hipblasLtMatrixLayout_t a = nullptr, b = nullptr, c = nullptr;
  hipblasLtMatmulAlgo_t algo;
  size_t workspace = 0;
  bool ok = false;
};

using PlanKey = std::tuple<int, int, int, int, int64_t, int64_t, int64_t, int, size_t, int>;

std::mutex g_mutex;
Api g_api;
std::map<int, hipblasLtHandle_t> g_handles;  // one per device
std::map<PlanKey, Plan> g_plans;

template <typename F> bool bind(void* lib, const char* name, F& fn) {
  fn = reinterpret_cast<F>(dlsym(lib, name));
  return fn != nullptr;
}

// Finds the copy of hipBLASLt that is loaded already. RTLD_NOLOAD: a second copy is never loaded.
bool look_up_api() {
  if (g_api.looked) return g_api.ok;
  g_api.looked = true;
  void* lib = dlopen("libhipblaslt.so.1", RTLD_NOLOAD | RTLD_NOW);
  if (lib == nullptr) lib = dlopen("libhipblaslt.so", RTLD_NOLOAD | RTLD_NOW);
  if (lib == nullptr) return false;
  g_api.ok = bind(lib, "hipblasLtCreate", g_api.create) &&
             bind(lib, "hipblasLtMatmulDescCreate", g_api.desc_create) &&
             bind(lib, "hipblasLtMatmulDescSetAttribute", g_api.desc_set) &&
             bind(lib, "hipblasLtMatmulDescDestroy", g_api.desc_destroy) &&
             bind(lib, "hipblasLtMatrixLayoutCreate", g_api.layout_create) &&
             bind(lib, "hipblasLtMatrixLayoutSetAttribute", g_api.layout_set) &&
             bind(lib, "hipblasLtMatrixLayoutDestroy", g_api.layout_destroy) &&
             bind(lib, "hipblasLtMatmulPreferenceCreate", g_api.pref_create) &&
             bind(lib, "hipblasLtMatmulPreferenceSetAttribute", g_api.pref_set) &&
             bind(lib, "hipblasLtMatmulPreferenceDestroy", g_api.pref_destroy) &&
             bind(lib, "hipblasLtMatmulAlgoGetHeuristic", g_api.heuristic) &&
             bind(lib, "hipblasLtMatmul", g_api.matmul);
  return g_api.ok;
}

// Row-major y = x . w^T is, in the library's column-major terms, D[N, M] = op_T(A)[N, K] . B[K, M]
// with A = w seen as [K, N] (leading dimension ldw) and B = x seen as [K, M] (leading dimension ldx).
// With splits > 1 the product is a strided batch over slices of K: slice s reads k in [s K/splits,
// (s+1) K/splits) of both operands (the slices of one operand interleave in memory, which read-only
// operands may) and writes its own [M, N] of partial sums.
bool set_batch(hipblasLtMatrixLayout_t layout, int32_t count, int64_t stride) {
  return g_api.layout_set(layout, HIPBLASLT_MATRIX_LAYOUT_BATCH_COUNT, &count, sizeof(count)) == HIPBLAS_STATUS_SUCCESS &&
         g_api.layout_set(layout, HIPBLASLT_MATRIX_LAYOUT_STRIDED_BATCH_OFFSET, &stride, sizeof(stride)) ==
             HIPBLAS_STATUS_SUCCESS;
}

bool fill_plan(hipblasLtHandle_t handle, Plan& p, int M, int N, int K, int64_t ldx, int64_t ldw, int64_t ldy,
               int out_dtype, size_t workspace_bytes, int splits) {
  const hipDataType out_type = out_dtype == ME_F32 ? HIP_R_32F : HIP_R_16BF;
  if (g_api.desc_create(&p.desc, HIPBLAS_COMPUTE_32F, HIP_R_32F) != HIPBLAS_STATUS_SUCCESS) return false;
  const int32_t ta = HIPBLAS_OP_T, tb = HIPBLAS_OP_N;
  if (g_api.desc_set(p.desc, HIPBLASLT_MATMUL_DESC_TRANSA, &ta, sizeof(ta)) != HIPBLAS_STATUS_SUCCESS) return false;
  if (g_api.desc_set(p.desc, HIPBLASLT_MATMUL_DESC_TRANSB, &tb, sizeof(tb)) != HIPBLAS_STATUS_SUCCESS) return false;
  if (g_api.layout_create(&p.a, HIP_R_16BF, K, N, ldw) != HIPBLAS_STATUS_SUCCESS) return false;
  if (g_api.layout_create(&p.b, HIP_R_16BF, K, M, ldx) != HIPBLAS_STATUS_SUCCESS) return false;
  if (g_api.layout_create(&p.c, out_type, N, M, ldy) != HIPBLAS_STATUS_SUCCESS) return false;
  if (splits > 1 && !(set_batch(p.a, splits, K) && set_batch(p.b, splits, K) && set_batch(p.c, splits, (int64_t)M * ldy)))
    return false;
  hipblasLtMatmulPreference_t pref = nullptr;
  if (g_api.pref_create(&pref) != HIPBLAS_STATUS_SUCCESS) return false;
  const uint64_t max_ws = workspace_bytes;
  bool ok = g_api.pref_set(pref, HIPBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES, &max_ws, sizeof(max_ws)) ==
            HIPBLAS_STATUS_SUCCESS;
  hipblasLtMatmulHeuristicResult_t found;
  int count = 0;
  ok = ok && g_api.heuristic(handle, p.desc, p.a, p.b, p.c, p.c, pref, 1, &found, &count) == HIPBLAS_STATUS_SUCCESS &&
       count >= 1 && found.state == HIPBLAS_STATUS_SUCCESS && found.workspaceSize <= workspace_bytes;
  g_api.pref_destroy(pref);
  if (!ok) return false;
  p.algo = found.algo;
  p.workspace = found.workspaceSize;
  return true;
}

// A plan that could not be completed gives back what it had made; the shape is remembered as refused.
bool make_plan(hipblasLtHandle_t handle, Plan& p, int M, int N, int K, int64_t ldx, int64_t ldw, int64_t ldy,
               int out_dtype, size_t workspace_bytes, int splits) {
  if (fill_plan(handle, p, M, N, K, ldx, ldw, ldy, out_dtype, workspace_bytes, splits)) return true;
  if (p.desc) g_api.desc_destroy(p.desc);
  for (hipblasLtMatrixLayout_t layout : {p.a, p.b, p.c})
    if (layout) g_api.layout_destroy(layout);
  p = Plan{};
  return false;
}

}  // namespace

// 1 if the process holds a hipBLASLt that this file can call, else 0.
extern "C" int me_gemm_library_available() {
  std::lock_guard<std::mutex> lock(g_mutex);
  return look_up_api() ? 1 : 0;
}

// y[M, N] (bfloat16 or float32, row stride ldy) = x[M, K] (bfloat16, row stride ldx) . w[N, K]^T
// (bfloat16, row stride ldw), float32 accumulation, on `stream`. `workspace` is device memory of
// `workspace_bytes` that the caller owns and that every call on one stream may share. Allocates no
// device memory. Returns 0; -3 if no hipBLASLt is loaded in the process or it offers no algorithm for
// the shape within the workspace (the caller takes another path); -1/-2 on other failures.
// splits > 1: K is cut in that many equal slices and y is float32 [splits, M, ldy], the partial sums
// of the slices, for a consumer that adds them; this is how a product with few output tiles and a long
// K fills the GPU with the library's kernels.
extern "C" int me_gemm_library_bf16(const void* x, int64_t ldx, const void* w, int64_t ldw, void* y, int64_t ldy,
                                    int out_dtype, void* workspace, size_t workspace_bytes, int M, int N, int K,
                                    int splits, hipStream_t stream) {
  ME_CHECK(M >= 1 && N >= 1 && K >= 1, "gemm_library: empty product %d x %d x %d", M, N, K);
  ME_CHECK(ldx >= K && ldw >= K && ldy >= N, "gemm_library: a row stride is shorter than its row");
  ME_CHECK(out_dtype == ME_BF16 || out_dtype == ME_F32, "gemm_library: unknown output dtype %d", out_dtype);
  ME_CHECK(x != nullptr && w != nullptr && y != nullptr, "gemm_library: null operand");
  ME_CHECK(splits >= 1 && K % splits == 0 && (splits == 1 || ((K / splits) % 8 == 0 && out_dtype == ME_F32)),
           "gemm_library: %d splits of K=%d need equal slices of a multiple of 8 and float32 partial sums", splits, K);
  const int Ks = K / splits;
  int device = 0;
  ME_CHECK(hipGetDevice(&device) == hipSuccess, "gemm_library: no current device");
  const Plan* plan = nullptr;
  hipblasLtHandle_t handle = nullptr;
  {
    std::lock_guard<std::mutex> lock(g_mutex);
    if (!look_up_api()) {
      me_set_error("gemm_library: no hipBLASLt is loaded in this process");
      return -3;
    }
    auto h = g_handles.find(device);
    if (h == g_handles.end()) {
      hipblasLtHandle_t made = nullptr;
      if (g_api.create(&made) != HIPBLAS_STATUS_SUCCESS) {
        me_set_error("gemm_library: hipblasLtCreate failed");
        return -3;
      }
      h = g_handles.emplace(device, made).first;
    }
    handle = h->second;
    const PlanKey key{device, M, N, K, ldx, ldw, ldy, out_dtype, workspace_bytes, splits};
    auto it = g_plans.find(key);
    if (it == g_plans.end()) {
      Plan made;
      made.ok = make_plan(handle, made, M, N, Ks, ldx, ldw, ldy, out_dtype, workspace == nullptr ? 0 : workspace_bytes, splits);
      it = g_plans.emplace(key, made).first;
    }
    if (!it->second.ok) {
      me_set_error("gemm_library: hipBLASLt offers no algorithm for %d x %d x %d", M, N, K);
      return -3;
    }
    plan = &it->second;  // std::map keeps the address
  }
  const float one = 1.f, zero = 0.f;
  const hipblasStatus_t status = g_api.matmul(handle, plan->desc, &one, w, plan->a, x, plan->b, &zero, y, plan->c, y,
                                              plan->c, &plan->algo, workspace, workspace_bytes, stream);
  if (status != HIPBLAS_STATUS_SUCCESS) {
    me_set_error("gemm_library: hipblasLtMatmul failed with status %d for %d x %d x %d", (int)status, M, N, K);
    return -2;
  }
  return 0;
}
