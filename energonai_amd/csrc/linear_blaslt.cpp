// y = act(x W^T + bias): the projection GEMMs either side of the padding-removal path, on
// hipBLASLt with its fused bias / ReLU / GELU epilogues.  Host code only; built into its own
// shared object (libenergon_linear.so) so that the kernel library keeps depending on nothing
// but the HIP runtime.
//
// The reference's mlp_gemm (energonai/kernel/cuda_native/csrc/linear_wrapper.cpp:82-111)
// calls cublasGemmEx with a caller-chosen algorithm id that find_algo() obtains by timing
// every id (cuda_native/linear_func.py:35-92).  hipBLASLt has no fixed id table: it returns
// a ranked list of candidate solutions per problem, so `algo` here is an index into that
// list (-1 or 0 = the library's first choice) and en_linear_algo_count() says how long the
// list is for a given problem.
#include <hip/hip_runtime.h>
#include <hipblaslt/hipblaslt.h>

#include <cstdint>
#include <map>
#include <mutex>
#include <tuple>
#include <vector>

#include "energon_linear.h"

namespace {

constexpr int kMaxDevices = 64;
constexpr int kMaxCandidates = 64;

hipblasLtHandle_t g_handle[kMaxDevices];
std::once_flag g_once[kMaxDevices];
int g_create_status[kMaxDevices];

// One handle per device, made on first use with that device current and kept until exit.
hipblasLtHandle_t handle_for_current_device(int *status) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) {
    *status = EN_LINEAR_ERR_HIP;
    return nullptr;
  }
  std::call_once(g_once[dev], [dev]() {
    g_create_status[dev] = (hipblasLtCreate(&g_handle[dev]) == HIPBLAS_STATUS_SUCCESS) ? 0 : EN_LINEAR_ERR_BLAS;
  });
  *status = g_create_status[dev];
  return g_handle[dev];
}

bool to_hip_type(int dtype, hipDataType *t) {
  switch (dtype) {
    case 0: *t = HIP_R_32F; return true;
    case 1: *t = HIP_R_16F; return true;
    case 2: *t = HIP_R_16BF; return true;
    default: return false;
  }
}

struct Problem {
  hipblasLtMatmulDesc_t desc = nullptr;
  hipblasLtMatrixLayout_t a = nullptr, b = nullptr, c = nullptr;
  hipblasLtMatmulPreference_t pref = nullptr;
  ~Problem() {
    if (pref) hipblasLtMatmulPreferenceDestroy(pref);
    if (c) hipblasLtMatrixLayoutDestroy(c);
    if (b) hipblasLtMatrixLayoutDestroy(b);
    if (a) hipblasLtMatrixLayoutDestroy(a);
    if (desc) hipblasLtMatmulDescDestroy(desc);
  }
};

// Column-major view of the row-major tensors, as in the reference call
// (linear_wrapper.cpp:98-108): D[dout, rows] = W[din, dout]^T * X[din, rows].
int describe(Problem &p, int64_t rows, int64_t din, int64_t dout, const void *bias, int activation, int dtype,
             uint64_t workspace_bytes) {
  hipDataType t;
  if (!to_hip_type(dtype, &t)) return EN_LINEAR_ERR_DTYPE;
  if (hipblasLtMatmulDescCreate(&p.desc, HIPBLAS_COMPUTE_32F, HIP_R_32F) != HIPBLAS_STATUS_SUCCESS) return EN_LINEAR_ERR_BLAS;
  const int32_t op_t = HIPBLAS_OP_T, op_n = HIPBLAS_OP_N;
  if (hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_TRANSA, &op_t, sizeof(op_t)) != HIPBLAS_STATUS_SUCCESS ||
      hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_TRANSB, &op_n, sizeof(op_n)) != HIPBLAS_STATUS_SUCCESS)
    return EN_LINEAR_ERR_BLAS;
  uint32_t epi;
  switch (activation) {
    case EN_LINEAR_ACT_NONE: epi = bias ? HIPBLASLT_EPILOGUE_BIAS : HIPBLASLT_EPILOGUE_DEFAULT; break;
    case EN_LINEAR_ACT_RELU: epi = bias ? HIPBLASLT_EPILOGUE_RELU_BIAS : HIPBLASLT_EPILOGUE_RELU; break;
    case EN_LINEAR_ACT_GELU_TANH: epi = bias ? HIPBLASLT_EPILOGUE_GELU_BIAS : HIPBLASLT_EPILOGUE_GELU; break;
    default: return EN_LINEAR_ERR_ARG;
  }
  if (hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_EPILOGUE, &epi, sizeof(epi)) != HIPBLAS_STATUS_SUCCESS)
    return EN_LINEAR_ERR_BLAS;
  if (bias) {
    const int32_t bt = (int32_t)t;
    if (hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_BIAS_POINTER, &bias, sizeof(bias)) != HIPBLAS_STATUS_SUCCESS ||
        hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_BIAS_DATA_TYPE, &bt, sizeof(bt)) != HIPBLAS_STATUS_SUCCESS)
      return EN_LINEAR_ERR_BLAS;
  }
  if (hipblasLtMatrixLayoutCreate(&p.a, t, (uint64_t)din, (uint64_t)dout, din) != HIPBLAS_STATUS_SUCCESS ||
      hipblasLtMatrixLayoutCreate(&p.b, t, (uint64_t)din, (uint64_t)rows, din) != HIPBLAS_STATUS_SUCCESS ||
      hipblasLtMatrixLayoutCreate(&p.c, t, (uint64_t)dout, (uint64_t)rows, dout) != HIPBLAS_STATUS_SUCCESS)
    return EN_LINEAR_ERR_BLAS;
  if (hipblasLtMatmulPreferenceCreate(&p.pref) != HIPBLAS_STATUS_SUCCESS ||
      hipblasLtMatmulPreferenceSetAttribute(p.pref, HIPBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES, &workspace_bytes,
                                            sizeof(workspace_bytes)) != HIPBLAS_STATUS_SUCCESS)
    return EN_LINEAR_ERR_BLAS;
  return 0;
}

// The heuristic query is the slow part of a call (tens of microseconds of host time), so the
// ranked list is kept per device and problem.
typedef std::tuple<int, int64_t, int64_t, int64_t, int, int, int, uint64_t> ProblemKey;
std::mutex g_cache_mutex;
std::map<ProblemKey, std::vector<hipblasLtMatmulHeuristicResult_t>> g_cache;

int query(hipblasLtHandle_t h, Problem &p, std::vector<hipblasLtMatmulHeuristicResult_t> &out);

int candidates(hipblasLtHandle_t h, Problem &p, const ProblemKey &key,
               std::vector<hipblasLtMatmulHeuristicResult_t> &out) {
  {
    std::lock_guard<std::mutex> lock(g_cache_mutex);
    auto it = g_cache.find(key);
    if (it != g_cache.end()) {
      out = it->second;
      return 0;
    }
  }
  const int st = query(h, p, out);
  if (st) return st;
  std::lock_guard<std::mutex> lock(g_cache_mutex);
  g_cache[key] = out;
  return 0;
}

int query(hipblasLtHandle_t h, Problem &p, std::vector<hipblasLtMatmulHeuristicResult_t> &out) {
  out.resize(kMaxCandidates);
  int n = 0;
  if (hipblasLtMatmulAlgoGetHeuristic(h, p.desc, p.a, p.b, p.c, p.c, p.pref, kMaxCandidates, out.data(), &n) != HIPBLAS_STATUS_SUCCESS)
    return EN_LINEAR_ERR_BLAS;
  int kept = 0;
  for (int i = 0; i < n; ++i)
    if (out[i].state == HIPBLAS_STATUS_SUCCESS) out[kept++] = out[i];
  out.resize(kept);
  return 0;
}

ProblemKey key_of(int64_t rows, int64_t din, int64_t dout, bool has_bias, int activation, int dtype, int64_t ws) {
  int dev = 0;
  (void)hipGetDevice(&dev);
  return ProblemKey(dev, rows, din, dout, has_bias ? 1 : 0, activation, dtype, (uint64_t)ws);
}

bool bad_shape(int64_t rows, int64_t din, int64_t dout) {
  return rows < 1 || din < 1 || dout < 1 || rows > INT32_MAX || din > INT32_MAX || dout > INT32_MAX;
}

}  // namespace

extern "C" {

int en_linear_algo_count(int64_t rows, int64_t din, int64_t dout, int has_bias, int activation, int dtype,
                         int64_t workspace_bytes) {
  if (bad_shape(rows, din, dout) || workspace_bytes < 0) return EN_LINEAR_ERR_ARG;
  int st = 0;
  hipblasLtHandle_t h = handle_for_current_device(&st);
  if (st) return st;
  Problem p;
  static const char dummy_bias = 0;   // only its presence matters for the candidate list
  st = describe(p, rows, din, dout, has_bias ? &dummy_bias : nullptr, activation, dtype, (uint64_t)workspace_bytes);
  if (st) return st;
  std::vector<hipblasLtMatmulHeuristicResult_t> res;
  st = candidates(h, p, key_of(rows, din, dout, has_bias != 0, activation, dtype, workspace_bytes), res);
  return st ? st : (int)res.size();
}

int en_linear(const void *x, const void *w, const void *bias, void *y, int64_t rows, int64_t din, int64_t dout,
              int activation, int dtype, int algo, void *workspace, int64_t workspace_bytes, void *stream) {
  if (!x || !w || !y) return EN_LINEAR_ERR_ARG;
  if (bad_shape(rows, din, dout) || workspace_bytes < 0 || (workspace_bytes > 0 && !workspace)) return EN_LINEAR_ERR_ARG;
  int st = 0;
  hipblasLtHandle_t h = handle_for_current_device(&st);
  if (st) return st;
  Problem p;
  st = describe(p, rows, din, dout, bias, activation, dtype, (uint64_t)workspace_bytes);
  if (st) return st;
  std::vector<hipblasLtMatmulHeuristicResult_t> res;
  st = candidates(h, p, key_of(rows, din, dout, bias != nullptr, activation, dtype, workspace_bytes), res);
  if (st) return st;
  if (res.empty()) return EN_LINEAR_ERR_NO_ALGO;
  const int pick = algo < 0 ? 0 : algo;
  if (pick >= (int)res.size()) return EN_LINEAR_ERR_NO_ALGO;
  if (res[pick].workspaceSize > (size_t)workspace_bytes) return EN_LINEAR_ERR_NO_ALGO;
  const float alpha = 1.f, beta = 0.f;
  if (hipblasLtMatmul(h, p.desc, &alpha, w, p.a, x, p.b, &beta, y, p.c, y, p.c, &res[pick].algo, workspace,
                      (size_t)workspace_bytes, (hipStream_t)stream) != HIPBLAS_STATUS_SUCCESS)
    return EN_LINEAR_ERR_BLAS;
  return 0;
}

const char *en_linear_status_string(int status) {
  switch (status) {
    case 0: return "ok";
    case EN_LINEAR_ERR_ARG: return "bad argument (null pointer, shape, activation or workspace)";
    case EN_LINEAR_ERR_DTYPE: return "unsupported dtype";
    case EN_LINEAR_ERR_HIP: return "HIP runtime error";
    case EN_LINEAR_ERR_BLAS: return "hipBLASLt error";
    case EN_LINEAR_ERR_NO_ALGO: return "no hipBLASLt solution with that index fits the workspace";
    default: return "unknown status";
  }
}

#ifndef EN_SOURCE_HASH
#define EN_SOURCE_HASH "unknown"
#endif
const char *en_linear_source_hash(void) { return EN_SOURCE_HASH; }

}  // extern "C"
