// bfloat16 products of many rows through the vendor library (hipBLASLt), called directly:
//   out[r][f] = sum_k x[r][k] * w[f][k] (+ bias[f]),  32-bit accumulation, bfloat16 result
//   (or the 32-bit sums themselves: the logits of many rows).
// The reference's engine uses a library product here as well (F.linear, src/dli/model/llama.py:
// 72-74,95,190,305). What this file adds to the library call is a cache: the operation and layout
// descriptors and the kernel that the library's heuristic picks are looked up once per shape, so
// that a call costs a few microseconds on the host instead of the tens that a framework's
// dispatch takes: an eager step of a few hundred tokens issues 65 products and is bound by the
// host otherwise. The bias is added inside the product (one rounding, as in the reference).
#include <hipblaslt/hipblaslt.h>

#include <map>
#include <mutex>
#include <tuple>

#include "common.h"

namespace {

struct Plan {
  hipblasLtMatmulDesc_t op = nullptr;
  hipblasLtMatrixLayout_t a = nullptr, b = nullptr, d = nullptr;
  hipblasLtMatmulAlgo_t algo;
  size_t workspace = 0;
  bool usable = false;
};

using Key = std::tuple<int, int64_t, int64_t, int64_t, int64_t, int64_t, int64_t, int, int64_t, int>;

std::mutex g_mutex;
std::map<int, hipblasLtHandle_t> g_handles;  // per device
std::map<Key, Plan> g_plans;

hipblasLtHandle_t handle_for(int device) {
  auto it = g_handles.find(device);
  if (it != g_handles.end()) return it->second;
  hipblasLtHandle_t h = nullptr;
  if (hipblasLtCreate(&h) != HIPBLAS_STATUS_SUCCESS) return nullptr;
  g_handles[device] = h;
  return h;
}

// Column-major reading of the row-major operands: out^T [f x r] = (w^T)^T [f x k] * x^T [k x r].
Plan make_plan(hipblasLtHandle_t handle, int64_t rows, int64_t feats, int64_t k, int64_t ldx,
               int64_t ldw, int64_t ldo, bool bias, size_t workspace_limit, bool out_f32) {
  Plan p;
  if (hipblasLtMatmulDescCreate(&p.op, HIPBLAS_COMPUTE_32F, HIP_R_32F) != HIPBLAS_STATUS_SUCCESS) return p;
  const int32_t trans = HIPBLAS_OP_T, none = HIPBLAS_OP_N;
  bool ok = hipblasLtMatmulDescSetAttribute(p.op, HIPBLASLT_MATMUL_DESC_TRANSA, &trans, sizeof(trans)) == HIPBLAS_STATUS_SUCCESS &&
            hipblasLtMatmulDescSetAttribute(p.op, HIPBLASLT_MATMUL_DESC_TRANSB, &none, sizeof(none)) == HIPBLAS_STATUS_SUCCESS;
  if (bias) {
    const uint32_t epilogue = HIPBLASLT_EPILOGUE_BIAS;
    const int32_t bias_type = HIP_R_16BF;
    ok = ok &&
         hipblasLtMatmulDescSetAttribute(p.op, HIPBLASLT_MATMUL_DESC_EPILOGUE, &epilogue, sizeof(epilogue)) == HIPBLAS_STATUS_SUCCESS &&
         hipblasLtMatmulDescSetAttribute(p.op, HIPBLASLT_MATMUL_DESC_BIAS_DATA_TYPE, &bias_type, sizeof(bias_type)) == HIPBLAS_STATUS_SUCCESS;
  }
  ok = ok && hipblasLtMatrixLayoutCreate(&p.a, HIP_R_16BF, k, feats, ldw) == HIPBLAS_STATUS_SUCCESS &&
       hipblasLtMatrixLayoutCreate(&p.b, HIP_R_16BF, k, rows, ldx) == HIPBLAS_STATUS_SUCCESS &&
       hipblasLtMatrixLayoutCreate(&p.d, out_f32 ? HIP_R_32F : HIP_R_16BF, feats, rows, ldo) == HIPBLAS_STATUS_SUCCESS;
  if (!ok) return p;
  hipblasLtMatmulPreference_t pref = nullptr;
  if (hipblasLtMatmulPreferenceCreate(&pref) != HIPBLAS_STATUS_SUCCESS) return p;
  const uint64_t limit = workspace_limit;
  hipblasLtMatmulPreferenceSetAttribute(pref, HIPBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES, &limit, sizeof(limit));
  hipblasLtMatmulHeuristicResult_t found[1];
  int n_found = 0;
  const hipblasStatus_t st =
      hipblasLtMatmulAlgoGetHeuristic(handle, p.op, p.a, p.b, p.d, p.d, pref, 1, found, &n_found);
  hipblasLtMatmulPreferenceDestroy(pref);
  if (st != HIPBLAS_STATUS_SUCCESS || n_found < 1 || found[0].state != HIPBLAS_STATUS_SUCCESS) return p;
  p.algo = found[0].algo;
  p.workspace = found[0].workspaceSize;
  p.usable = p.workspace <= workspace_limit;
  return p;
}

}  // namespace

namespace {

int gemm(const void* x, int64_t ldx, const void* w, int64_t ldw, const void* bias, void* out, int64_t ldo,
         int64_t rows, int64_t feats, int64_t k, void* workspace, int64_t workspace_bytes, int device,
         bool out_f32, hipStream_t stream) {
  if (rows <= 0 || feats <= 0) return DLI_OK;
  if (k <= 0 || ldx < k || ldw < k || ldo < feats || workspace_bytes < 0) return DLI_ERR_ARGUMENT;
  std::lock_guard<std::mutex> lock(g_mutex);
  hipblasLtHandle_t handle = handle_for(device);
  if (handle == nullptr) return DLI_ERR_LAUNCH;
  const Key key{device, rows, feats, k, ldx, ldw, ldo, bias != nullptr ? 1 : 0, workspace_bytes, out_f32 ? 1 : 0};
  auto it = g_plans.find(key);
  if (it == g_plans.end())
    it = g_plans.emplace(key, make_plan(handle, rows, feats, k, ldx, ldw, ldo, bias != nullptr,
                                        (size_t)workspace_bytes, out_f32)).first;
  Plan& p = it->second;
  if (!p.usable) return DLI_ERR_ARGUMENT;
  if (bias != nullptr &&
      hipblasLtMatmulDescSetAttribute(p.op, HIPBLASLT_MATMUL_DESC_BIAS_POINTER, &bias, sizeof(bias)) != HIPBLAS_STATUS_SUCCESS)
    return DLI_ERR_LAUNCH;
  const float one = 1.f, zero = 0.f;
  const hipblasStatus_t st = hipblasLtMatmul(handle, p.op, &one, w, p.a, x, p.b, &zero, out, p.d, out, p.d,
                                             &p.algo, workspace, (size_t)workspace_bytes, stream);
  return st == HIPBLAS_STATUS_SUCCESS ? DLI_OK : DLI_ERR_LAUNCH;
}

}  // namespace

// x [rows, k] (row stride ldx), w [feats, k] (row stride ldw), out [rows, feats] (row stride ldo),
// all bfloat16 on `device`; bias [feats] bfloat16 or null; workspace: device memory that the
// library may use during the call. Returns DLI_ERR_ARGUMENT where the library offers no kernel
// for the shape (the caller then takes another road), DLI_ERR_LAUNCH where a call fails.
extern "C" int dli_gemm_bf16(const void* x, int64_t ldx, const void* w, int64_t ldw, const void* bias,
                             void* out, int64_t ldo, int64_t rows, int64_t feats, int64_t k,
                             void* workspace, int64_t workspace_bytes, int device,
                             hipStream_t stream) {
  return gemm(x, ldx, w, ldw, bias, out, ldo, rows, feats, k, workspace, workspace_bytes, device, false, stream);
}

// The same with `out` float32: the sums as accumulated, not rounded to bfloat16.
extern "C" int dli_gemm_bf16_f32(const void* x, int64_t ldx, const void* w, int64_t ldw, const void* bias,
                                 void* out, int64_t ldo, int64_t rows, int64_t feats, int64_t k,
                                 void* workspace, int64_t workspace_bytes, int device,
                                 hipStream_t stream) {
  return gemm(x, ldx, w, ldw, bias, out, ldo, rows, feats, k, workspace, workspace_bytes, device, true, stream);
}

// Whether the library has a kernel for this product (the plan is made and cached as for a call).
extern "C" int dli_gemm_bf16_usable(int64_t rows, int64_t feats, int64_t k, int64_t ldx, int64_t ldw, int64_t ldo,
                                    int bias, int64_t workspace_bytes, int device) {
  if (rows <= 0 || feats <= 0 || k <= 0 || ldx < k || ldw < k || ldo < feats || workspace_bytes < 0) return 0;
  std::lock_guard<std::mutex> lock(g_mutex);
  hipblasLtHandle_t handle = handle_for(device);
  if (handle == nullptr) return 0;
  const Key key{device, rows, feats, k, ldx, ldw, ldo, bias ? 1 : 0, workspace_bytes, 0};
  auto it = g_plans.find(key);
  if (it == g_plans.end())
    it = g_plans.emplace(key, make_plan(handle, rows, feats, k, ldx, ldw, ldo, bias != 0, (size_t)workspace_bytes, false)).first;
  return it->second.usable ? 1 : 0;
}
