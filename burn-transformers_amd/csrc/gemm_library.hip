// Matrix products of steps with many rows (prompts) through hipBLASLt, the vendor's GEMM library.
//
// C[M, N] = A[M, K] . W[N, K]^T with both operands K-contiguous in bfloat16 and 32-bit accumulation,
// finished by the library's own epilogues so that no extra pass over the result is needed:
//   EPI_STORE     bfloat16 out = acc + bias                      (bias stays float32)
//   EPI_ACT       bfloat16 out = gelu_tanh(acc + bias)           (the library's GELU is the tanh form)
//   EPI_RESIDUAL  float32 out += acc + bias, in place            (C = D = the residual stream, beta = 1)
//   EPI_F32       float32 out = acc + bias                       (one split only: logits of many rows)
// Other epilogues (erf GELU, split partial sums, the scatter into the paged cache) are refused
// here; callers keep the hand-written kernels for them.
//
// The library is opened at run time from the path the caller gives (the copy that came with the
// process's HIP runtime), not linked: a process has one HIP runtime, and a second copy of the
// library's own dependencies pulled in by the linker does not load beside it.  Nothing here
// allocates device memory: algorithms that need a workspace are not asked for.
//
// Row-major C[M, N] is column-major C^T[N, M] = W . A^T, so the library sees W as its
// (transposed) first operand and A as its second; the bias vector runs along its rows (N).
#include <dlfcn.h>
#include <hipblaslt/hipblaslt.h>

#include <map>
#include <tuple>

#include "epilogue.h"
#include "host.h"
#include "calls.h"

namespace {

#define BT_LT_FUNCTIONS(X)                                                                            \
  X(hipblasLtCreate) X(hipblasLtMatmulDescCreate) X(hipblasLtMatmulDescSetAttribute)                  \
  X(hipblasLtMatrixLayoutCreate) X(hipblasLtMatmulPreferenceCreate)                                   \
  X(hipblasLtMatmulPreferenceSetAttribute) X(hipblasLtMatmulPreferenceDestroy)                        \
  X(hipblasLtMatmulAlgoGetHeuristic) X(hipblasLtMatmul) X(hipblasLtGetVersion)

#define BT_LT_DECLARE(name) decltype(&name) fn_##name = nullptr;
BT_LT_FUNCTIONS(BT_LT_DECLARE)
#undef BT_LT_DECLARE

void* library = nullptr;
hipblasLtHandle_t handle = nullptr;
int library_version = 0;

struct Plan {
  hipblasLtMatmulDesc_t desc = nullptr;
  hipblasLtMatrixLayout_t w = nullptr, a = nullptr, c = nullptr;
  hipblasLtMatmulAlgo_t algo;
  float beta = 0.f;
};
// (M, N, K, lda, ldo, mode, bias present)
typedef std::tuple<int, int, int, int64_t, int64_t, int, bool> PlanKey;
std::map<PlanKey, Plan> plans;

const char* status_name(hipblasStatus_t s) {
  switch (s) {
    case HIPBLAS_STATUS_SUCCESS: return "success";
    case HIPBLAS_STATUS_NOT_INITIALIZED: return "not initialized";
    case HIPBLAS_STATUS_ALLOC_FAILED: return "allocation failed";
    case HIPBLAS_STATUS_INVALID_VALUE: return "invalid value";
    case HIPBLAS_STATUS_ARCH_MISMATCH: return "architecture mismatch";
    case HIPBLAS_STATUS_EXECUTION_FAILED: return "execution failed";
    case HIPBLAS_STATUS_NOT_SUPPORTED: return "not supported";
    default: return "error";
  }
}

#define BT_LT_CALL(what, expr)                                                          \
  do {                                                                                  \
    hipblasStatus_t st_ = (expr);                                                       \
    if (st_ != HIPBLAS_STATUS_SUCCESS) {                                                \
      bt_set_error("gemm_library: %s: %s (%d)", what, status_name(st_), (int)st_);      \
      return BT_REFUSED;                                                                \
    }                                                                                   \
  } while (0)

int make_plan(const PlanKey& key, Plan& p) {
  const int M = std::get<0>(key), N = std::get<1>(key), K = std::get<2>(key), mode = std::get<5>(key);
  const int64_t lda = std::get<3>(key), ldo = std::get<4>(key);
  const bool with_bias = std::get<6>(key);
  BT_LT_CALL("descriptor", fn_hipblasLtMatmulDescCreate(&p.desc, HIPBLAS_COMPUTE_32F, HIP_R_32F));
  int32_t transposed = HIPBLAS_OP_T, plain = HIPBLAS_OP_N;
  BT_LT_CALL("transa", fn_hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_TRANSA, &transposed, sizeof(int32_t)));
  BT_LT_CALL("transb", fn_hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_TRANSB, &plain, sizeof(int32_t)));
  uint32_t epilogue = mode == EPI_ACT ? (with_bias ? HIPBLASLT_EPILOGUE_GELU_BIAS : HIPBLASLT_EPILOGUE_GELU)
                                      : (with_bias ? HIPBLASLT_EPILOGUE_BIAS : HIPBLASLT_EPILOGUE_DEFAULT);
  BT_LT_CALL("epilogue", fn_hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_EPILOGUE, &epilogue, sizeof(epilogue)));
  if (with_bias) {
    int32_t bias_type = HIP_R_32F;
    BT_LT_CALL("bias type", fn_hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_BIAS_DATA_TYPE, &bias_type, sizeof(bias_type)));
    // the heuristic wants to see that a bias will come; the real pointer is set for each call
    const void* placeholder = &plans;
    BT_LT_CALL("bias", fn_hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_BIAS_POINTER, &placeholder, sizeof(placeholder)));
  }
  const hipDataType out_type = (mode == EPI_RESIDUAL || mode == EPI_F32) ? HIP_R_32F : HIP_R_16BF;
  BT_LT_CALL("layout of W", fn_hipblasLtMatrixLayoutCreate(&p.w, HIP_R_16BF, K, N, K));
  BT_LT_CALL("layout of A", fn_hipblasLtMatrixLayoutCreate(&p.a, HIP_R_16BF, K, M, lda));
  BT_LT_CALL("layout of C", fn_hipblasLtMatrixLayoutCreate(&p.c, out_type, N, M, ldo));
  hipblasLtMatmulPreference_t preference = nullptr;
  BT_LT_CALL("preference", fn_hipblasLtMatmulPreferenceCreate(&preference));
  uint64_t no_workspace = 0;
  fn_hipblasLtMatmulPreferenceSetAttribute(preference, HIPBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES, &no_workspace, sizeof(no_workspace));
  hipblasLtMatmulHeuristicResult_t found[1];
  int count = 0;
  hipblasStatus_t st = fn_hipblasLtMatmulAlgoGetHeuristic(handle, p.desc, p.w, p.a, p.c, p.c, preference, 1, found, &count);
  fn_hipblasLtMatmulPreferenceDestroy(preference);
  if (st != HIPBLAS_STATUS_SUCCESS || count < 1 || found[0].workspaceSize != 0) {
    bt_set_error("gemm_library: no algorithm without workspace for [%d x %d] . [%d x %d]^T, epilogue %d (%s)", M, K, N, K, mode,
                 status_name(st));
    return BT_REFUSED;
  }
  p.algo = found[0].algo;
  p.beta = mode == EPI_RESIDUAL ? 1.f : 0.f;
  return BT_OK;
}

}  // namespace

// Opens the library at `path` and creates its handle.  Returns the library's version through
// `version`.  Safe to call again: the first success stands.
BT_EXPORT int bt_gemm_library_open(const char* path, int* version) {
  if (handle != nullptr) {
    if (version) *version = library_version;
    return BT_OK;
  }
  library = dlopen(path, RTLD_NOW | RTLD_LOCAL);
  if (library == nullptr) {
    bt_set_error("gemm_library: cannot open %s: %s", path, dlerror());
    return BT_REFUSED;
  }
#define BT_LT_LOAD(name)                                                        \
  fn_##name = reinterpret_cast<decltype(fn_##name)>(dlsym(library, #name));     \
  if (fn_##name == nullptr) {                                                   \
    bt_set_error("gemm_library: %s has no %s", path, #name);                    \
    return BT_REFUSED;                                                          \
  }
  BT_LT_FUNCTIONS(BT_LT_LOAD)
#undef BT_LT_LOAD
  hipblasLtHandle_t created = nullptr;
  BT_LT_CALL("create", fn_hipblasLtCreate(&created));
  fn_hipblasLtGetVersion(created, &library_version);
  handle = created;
  if (version) *version = library_version;
  return BT_OK;
}

// Rows a single library call takes: the heuristic finds no algorithm without a workspace for
// very tall products (32,768 rows were refused), and rows are independent, so taller ones go in
// runs of this many.
constexpr int ROWS_PER_CALL = 4096;

namespace {

// The plan for a run of `M` rows, made at first use; nullptr (with the error set) if there is none.
Plan* plan_for(int M, int N, int K, int64_t lda, const Epilogue* epi) {
  PlanKey key(M, N, K, lda, epi->ldo, epi->mode, epi->bias != nullptr);
  auto it = plans.find(key);
  if (it == plans.end()) {
    Plan fresh;
    if (make_plan(key, fresh)) return nullptr;
    it = plans.emplace(key, fresh).first;
  }
  return &it->second;
}

int run_rows(hipStream_t stream, Plan& p, const char* A, const void* W, const Epilogue* epi, char* out) {
  if (epi->bias != nullptr) {
    const void* bias = epi->bias;
    BT_LT_CALL("bias", fn_hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_BIAS_POINTER, &bias, sizeof(bias)));
  }
  const float alpha = 1.f;
  BT_LT_CALL("matmul", fn_hipblasLtMatmul(handle, p.desc, &alpha, W, p.w, A, p.a, &p.beta, out, p.c, out, p.c, &p.algo,
                                          nullptr, 0, stream));
  return BT_OK;
}

}  // namespace

// Not safe for concurrent calls (plans are shared and carry the bias pointer of the last call);
// the engine issues its kernels from one thread.
BT_EXPORT int bt_gemm_library_bf16(void* stream, const void* A, int64_t lda, const void* W, int M, int N, int K,
                                   const Epilogue* epi) {
  if (M <= 0) return BT_OK;
  if (handle == nullptr) BT_REFUSE("gemm_library: the library has not been opened");
  if (N <= 0 || K <= 0 || lda < K || epi->ldo < N) BT_REFUSE("gemm_library: sizes M %d N %d K %d do not fit the pitches", M, N, K);
  if (epi->out == nullptr) BT_REFUSE("gemm_library: no output");
  if (epi->mode != EPI_STORE && epi->mode != EPI_RESIDUAL && epi->mode != EPI_F32 &&
      !(epi->mode == EPI_ACT && epi->act == ACT_GELU_TANH))
    BT_REFUSE("gemm_library: epilogue %d (activation %d) is not one the library has", epi->mode, epi->act);
  // both plans (full runs and the shorter last one) before anything runs, so that a refusal
  // leaves the output untouched
  Plan* full = plan_for(M < ROWS_PER_CALL ? M : ROWS_PER_CALL, N, K, lda, epi);
  if (full == nullptr) return BT_REFUSED;
  Plan* last = full;
  if (M > ROWS_PER_CALL && M % ROWS_PER_CALL != 0) {
    last = plan_for(M % ROWS_PER_CALL, N, K, lda, epi);
    if (last == nullptr) return BT_REFUSED;      // (entries of a std::map stay where they are: `full` is still good)
  }
  const int64_t out_bytes = (epi->mode == EPI_RESIDUAL || epi->mode == EPI_F32) ? 4 : 2;
  for (int m0 = 0; m0 < M; m0 += ROWS_PER_CALL) {
    bool whole = M - m0 >= ROWS_PER_CALL;
    int rc = run_rows((hipStream_t)stream, whole ? *full : *last, (const char*)A + (int64_t)m0 * lda * 2, W, epi,
                      (char*)epi->out + (int64_t)m0 * epi->ldo * out_bytes);
    if (rc) return rc;
  }
  return BT_OK;
}

// Whether the library has an algorithm for this product, found (and kept) without running anything:
// what a launch list asks before it names the library for a product.
BT_EXPORT int bt_gemm_library_plan(int64_t lda, int M, int N, int K, const Epilogue* epi) {
  if (M <= 0) return BT_OK;
  if (handle == nullptr) BT_REFUSE("gemm_library: the library has not been opened");
  if (N <= 0 || K <= 0 || lda < K || epi->ldo < N) BT_REFUSE("gemm_library: sizes M %d N %d K %d do not fit the pitches", M, N, K);
  if (epi->mode != EPI_STORE && epi->mode != EPI_RESIDUAL && epi->mode != EPI_F32 &&
      !(epi->mode == EPI_ACT && epi->act == ACT_GELU_TANH))
    BT_REFUSE("gemm_library: epilogue %d (activation %d) is not one the library has", epi->mode, epi->act);
  if (plan_for(M < ROWS_PER_CALL ? M : ROWS_PER_CALL, N, K, lda, epi) == nullptr) return BT_REFUSED;
  if (M > ROWS_PER_CALL && M % ROWS_PER_CALL != 0 && plan_for(M % ROWS_PER_CALL, N, K, lda, epi) == nullptr) return BT_REFUSED;
  return BT_OK;
}

// The product with its arguments as one structure (calls.h), for launch lists.
BT_EXPORT int bt_gemm_library_call(void* stream, const GemmCall* c) {
  if (c->dtype != 1 || c->splits != 1 || c->has_norm || c->a_rows || c->packed_columns || c->epi.out_rows)
    BT_REFUSE("gemm_library: bfloat16 row-major operands only, no split of K");
  return bt_gemm_library_bf16(stream, c->A, c->lda, c->W, c->M, c->N, c->K, &c->epi);
}
