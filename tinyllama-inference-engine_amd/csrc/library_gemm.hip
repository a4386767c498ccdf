// y = x . W^T for many rows through the vendor's matrix-product library, called directly.
//
// reference: every product of the reference's device path is a library call (cublasGemmEx,
// src/cuda/kernels.cu:342-368).  Steps of more than 64 rows take hipBLASLt here.  Through
// torch.mm that costs the host 19 us a call, and a step of prompt portions makes four of them a
// layer; this file calls the same library function itself, with the matrix layouts and the
// algorithm it chose kept per shape, for 10 us.  The library is the copy that torch has loaded
// (its functions are looked up in that file at run time, so nothing here links against a second
// copy); the algorithm is the library's own first choice among those that fit the workspace.
#include "common.h"

#include <dlfcn.h>

#include <map>
#include <mutex>
#include <tuple>

#if __has_include(<hipblaslt/hipblaslt.h>)
#include <hipblaslt/hipblaslt.h>
#define TLIE_HAVE_HIPBLASLT 1
#endif

namespace {

constexpr int kUnavailable = -3;      // the library (or its header, at build time) is not there: the caller takes another route

#ifdef TLIE_HAVE_HIPBLASLT
struct Api {
  decltype(&hipblasLtCreate) create = nullptr;
  decltype(&hipblasLtMatrixLayoutCreate) layout_create = nullptr;
  decltype(&hipblasLtMatmulDescCreate) desc_create = nullptr;
  decltype(&hipblasLtMatmulDescSetAttribute) desc_set = nullptr;
  decltype(&hipblasLtMatmulPreferenceCreate) preference_create = nullptr;
  decltype(&hipblasLtMatmulPreferenceSetAttribute) preference_set = nullptr;
  decltype(&hipblasLtMatmulPreferenceDestroy) preference_destroy = nullptr;
  decltype(&hipblasLtMatmulAlgoGetHeuristic) heuristic = nullptr;
  decltype(&hipblasLtMatmul) matmul = nullptr;
  bool ready = false;
};

struct Plan {
  hipblasLtMatmulDesc_t desc = nullptr;
  hipblasLtMatrixLayout_t w = nullptr, x = nullptr, y = nullptr;
  hipblasLtMatmulAlgo_t algo;
  bool usable = false;               // false: the library offers nothing for this shape
};

Api api;
std::mutex guard;
std::map<int, hipblasLtHandle_t> handles;                              // by device
std::map<std::tuple<int, int, int, int, int, size_t>, Plan> plans;    // by (device, M, N, K, type of y, workspace)
#endif

}  // namespace

// path: the file of the hipBLASLt library that the process has loaded.  0 on success.
extern "C" int tlie_library_gemm_init(const char* path) {
#ifdef TLIE_HAVE_HIPBLASLT
  std::lock_guard<std::mutex> lock(guard);
  if (api.ready) return tlie::kOk;
  void* library = dlopen(path, RTLD_NOW | RTLD_NOLOAD);
  if (library == nullptr) library = dlopen(path, RTLD_NOW);
  if (library == nullptr) return kUnavailable;
#define TLIE_SYMBOL(field, name)                                    \
  api.field = reinterpret_cast<decltype(api.field)>(dlsym(library, #name)); \
  if (api.field == nullptr) return kUnavailable;
  TLIE_SYMBOL(create, hipblasLtCreate)
  TLIE_SYMBOL(layout_create, hipblasLtMatrixLayoutCreate)
  TLIE_SYMBOL(desc_create, hipblasLtMatmulDescCreate)
  TLIE_SYMBOL(desc_set, hipblasLtMatmulDescSetAttribute)
  TLIE_SYMBOL(preference_create, hipblasLtMatmulPreferenceCreate)
  TLIE_SYMBOL(preference_set, hipblasLtMatmulPreferenceSetAttribute)
  TLIE_SYMBOL(preference_destroy, hipblasLtMatmulPreferenceDestroy)
  TLIE_SYMBOL(heuristic, hipblasLtMatmulAlgoGetHeuristic)
  TLIE_SYMBOL(matmul, hipblasLtMatmul)
#undef TLIE_SYMBOL
  api.ready = true;
  return tlie::kOk;
#else
  (void)path;
  return kUnavailable;
#endif
}

// x [M, K], w [N, K]: bfloat16; y [M, N]: bfloat16, or float when y_float != 0 (the sums are float either way);
// row-major, dense.  workspace: device memory the library may use.
// Returns 0, or -3 when the library has no algorithm for the shape (or is not there): nothing was launched then.
extern "C" int tlie_library_gemm(const void* x, const void* w, void* y, int y_float, int M, int N, int K, void* workspace,
                                 size_t workspace_bytes, void* stream) {
#ifdef TLIE_HAVE_HIPBLASLT
  if (M <= 0 || N <= 0 || K <= 0) return tlie::kBadArgument;
  if (!api.ready) return kUnavailable;
  int device = 0;
  if (hipGetDevice(&device) != hipSuccess) return tlie::kLaunchFailed;
  std::lock_guard<std::mutex> lock(guard);
  auto handle = handles.find(device);
  if (handle == handles.end()) {
    hipblasLtHandle_t made = nullptr;
    if (api.create(&made) != HIPBLAS_STATUS_SUCCESS) return kUnavailable;
    handle = handles.emplace(device, made).first;
  }
  const auto key = std::make_tuple(device, M, N, K, y_float != 0 ? 1 : 0, workspace_bytes);
  auto found = plans.find(key);
  if (found == plans.end()) {
    // In the library's column-major terms: y^T [N x M] = op_T(W as K x N) . (x as K x M)
    Plan plan;
    const hipblasOperation_t transposed = HIPBLAS_OP_T, plain = HIPBLAS_OP_N;
    hipblasLtMatmulPreference_t preference = nullptr;
    bool made = api.desc_create(&plan.desc, HIPBLAS_COMPUTE_32F, HIP_R_32F) == HIPBLAS_STATUS_SUCCESS &&
                api.desc_set(plan.desc, HIPBLASLT_MATMUL_DESC_TRANSA, &transposed, sizeof(transposed)) == HIPBLAS_STATUS_SUCCESS &&
                api.desc_set(plan.desc, HIPBLASLT_MATMUL_DESC_TRANSB, &plain, sizeof(plain)) == HIPBLAS_STATUS_SUCCESS &&
                api.layout_create(&plan.w, HIP_R_16BF, K, N, K) == HIPBLAS_STATUS_SUCCESS &&
                api.layout_create(&plan.x, HIP_R_16BF, K, M, K) == HIPBLAS_STATUS_SUCCESS &&
                api.layout_create(&plan.y, y_float != 0 ? HIP_R_32F : HIP_R_16BF, N, M, N) == HIPBLAS_STATUS_SUCCESS &&
                api.preference_create(&preference) == HIPBLAS_STATUS_SUCCESS &&
                api.preference_set(preference, HIPBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES, &workspace_bytes,
                                   sizeof(workspace_bytes)) == HIPBLAS_STATUS_SUCCESS;
    if (made) {
      // the library's candidates come best first by its own estimate; the first one that works
      // within the caller's workspace is taken (for some shapes of very many rows its first
      // choice wants more than any fixed workspace holds)
      constexpr int kCandidates = 16;
      hipblasLtMatmulHeuristicResult_t result[kCandidates];
      int returned = 0, chosen = -1;
      made = api.heuristic(handle->second, plan.desc, plan.w, plan.x, plan.y, plan.y, preference, kCandidates, result,
                           &returned) == HIPBLAS_STATUS_SUCCESS;
      for (int i = 0; made && chosen < 0 && i < returned; ++i)
        if (result[i].state == HIPBLAS_STATUS_SUCCESS && result[i].workspaceSize <= workspace_bytes) chosen = i;
      made = made && chosen >= 0;
      if (made) plan.algo = result[chosen].algo;
    }
    if (preference != nullptr) api.preference_destroy(preference);
    plan.usable = made;                 // (a shape without an algorithm is remembered too, and not asked for again)
    found = plans.emplace(key, plan).first;
  }
  const Plan& plan = found->second;
  if (!plan.usable) return kUnavailable;
  const float one = 1.f, zero = 0.f;
  const hipblasStatus_t status = api.matmul(handle->second, plan.desc, &one, w, plan.w, x, plan.x, &zero, y, plan.y, y, plan.y,
                                            &plan.algo, workspace, workspace_bytes, (hipStream_t)stream);
  return status == HIPBLAS_STATUS_SUCCESS ? tlie::kOk : tlie::kLaunchFailed;
#else
  (void)x, (void)w, (void)y, (void)y_float, (void)M, (void)N, (void)K, (void)workspace, (void)workspace_bytes, (void)stream;
  return kUnavailable;
#endif
}
