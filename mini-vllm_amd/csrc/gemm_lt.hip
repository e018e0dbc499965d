// The library's matrix product for many rows (prompt portions, decode steps of more than 64
// sequences), called directly:
//     C[M, N] = A[M, K] * W[N, K]^T (+ bias),   bf16 in, bf16 or float out, float accumulation
//     (hipBLASLt).
// Going through a tensor library's dispatcher costs about 18 us of host time per product on this
// machine, a direct call about 5: a prompt step of a small model has four products per layer that
// take 15 to 30 us each on the device, so the host would be the slower side.
//
// hipBLASLt is column-major. The row-major operands are read as their transposes: W[N, K] is a
// column-major [K, N] (leading dimension K), A[M, K] a column-major [K, M], C[M, N] a column-major
// [N, M]. In its terms the product is D[N, M] = op(W)[N, K] * A[K, M] with op = transpose, i.e.
// transa = T, transb = N. The bias then runs along the rows of D, which is what its bias epilogue
// adds.
//
// One plan (descriptor, layouts, the first algorithm of the heuristic's list that fits the
// workspace) is kept per shape. The caller brings the workspace; nothing is allocated here after a
// shape's first call. A shape the library has no algorithm for is declined with return code 2
// (nothing done), every time it comes.
#include "common.h"

#include <hipblaslt/hipblaslt.h>

#include <map>
#include <mutex>
#include <tuple>

namespace {

struct LtPlan {
    hipblasLtMatmulDesc_t desc = nullptr;
    hipblasLtMatrixLayout_t w = nullptr, a = nullptr, c = nullptr;
    hipblasLtMatmulAlgo_t algo;
    size_t workspace = 0;
    bool served = false;            // the library has an algorithm for the shape that fits the workspace
};

std::mutex g_lock;
hipblasLtHandle_t g_handle = nullptr;
std::map<std::tuple<int, int, int, long, long, int, int>, LtPlan> g_plans;

const char* lt_status(hipblasStatus_t s) {
    switch (s) {
        case HIPBLAS_STATUS_SUCCESS: return "success";
        case HIPBLAS_STATUS_NOT_INITIALIZED: return "not initialised";
        case HIPBLAS_STATUS_ALLOC_FAILED: return "allocation failed";
        case HIPBLAS_STATUS_INVALID_VALUE: return "invalid value";
        case HIPBLAS_STATUS_NOT_SUPPORTED: return "not supported";
        case HIPBLAS_STATUS_EXECUTION_FAILED: return "execution failed";
        case HIPBLAS_STATUS_INTERNAL_ERROR: return "internal error";
        default: return "error";
    }
}

#define LT_CHECK(call)                                                                        \
    do {                                                                                      \
        const hipblasStatus_t st_ = (call);                                                   \
        if (st_ != HIPBLAS_STATUS_SUCCESS) return mv_fail("gemm_lt: %s: %s", #call, lt_status(st_)); \
    } while (0)

void drop_plan(LtPlan& p) {
    if (p.desc) hipblasLtMatmulDescDestroy(p.desc);
    if (p.w) hipblasLtMatrixLayoutDestroy(p.w);
    if (p.a) hipblasLtMatrixLayoutDestroy(p.a);
    if (p.c) hipblasLtMatrixLayoutDestroy(p.c);
    p = LtPlan{};
}

int make_plan(LtPlan& p, int M, int N, int K, long lda, long ldc, bool with_bias, bool float_out,
              size_t workspace_bytes) {
    LT_CHECK(hipblasLtMatmulDescCreate(&p.desc, HIPBLAS_COMPUTE_32F, HIP_R_32F));
    const hipblasOperation_t ta = HIPBLAS_OP_T, tb = HIPBLAS_OP_N;
    LT_CHECK(hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_TRANSA, &ta, sizeof(ta)));
    LT_CHECK(hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_TRANSB, &tb, sizeof(tb)));
    if (with_bias) {
        const hipblasLtEpilogue_t ep = HIPBLASLT_EPILOGUE_BIAS;
        const hipDataType bt = HIP_R_16BF;
        LT_CHECK(hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_EPILOGUE, &ep, sizeof(ep)));
        LT_CHECK(hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_BIAS_DATA_TYPE, &bt, sizeof(bt)));
    }
    LT_CHECK(hipblasLtMatrixLayoutCreate(&p.w, HIP_R_16BF, K, N, K));
    LT_CHECK(hipblasLtMatrixLayoutCreate(&p.a, HIP_R_16BF, K, M, lda));
    LT_CHECK(hipblasLtMatrixLayoutCreate(&p.c, float_out ? HIP_R_32F : HIP_R_16BF, N, M, ldc));
    hipblasLtMatmulPreference_t pref = nullptr;
    LT_CHECK(hipblasLtMatmulPreferenceCreate(&pref));
    LT_CHECK(hipblasLtMatmulPreferenceSetAttribute(pref, HIPBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES, &workspace_bytes,
                                                   sizeof(workspace_bytes)));
    // The heuristic's list is in its order of preference; it may hold algorithms that want more
    // workspace than the preference names, so the first that fits is taken.
    constexpr int kAsk = 8;
    hipblasLtMatmulHeuristicResult_t found[kAsk];
    int n_found = 0;
    const hipblasStatus_t st = hipblasLtMatmulAlgoGetHeuristic(g_handle, p.desc, p.w, p.a, p.c, p.c, pref, kAsk, found,
                                                               &n_found);
    hipblasLtMatmulPreferenceDestroy(pref);
    if (st != HIPBLAS_STATUS_SUCCESS || n_found < 1) return 0;      // no algorithm: the plan stays without one
    for (int i = 0; i < n_found; ++i) {
        if (found[i].workspaceSize > workspace_bytes) continue;
        p.algo = found[i].algo;
        p.workspace = found[i].workspaceSize;
        p.served = true;
        return 0;
    }
    return 0;                                                        // none fits the workspace brought
}

}  // namespace

// Bytes of workspace the caller should bring (plans are made for at most this much).
extern "C" long mv_gemm_lt_workspace() { return 128L << 20; }

extern "C" int mv_gemm_lt(const void* A, long lda, const void* W, const void* bias, void* C, long ldc, int c_dtype, int M,
                          int N, int K, void* workspace, long workspace_bytes, hipStream_t stream) {
    MV_REQUIRE(c_dtype == MV_BF16 || c_dtype == MV_F32, "gemm_lt: output type %d is neither bf16 nor float",
               c_dtype);
    const bool float_out = c_dtype == MV_F32;
    MV_REQUIRE(M > 0 && N > 0 && K > 0, "gemm_lt: bad sizes M=%d N=%d K=%d", M, N, K);
    MV_REQUIRE(lda >= K && ldc >= N, "gemm_lt: lda=%ld / ldc=%ld too small for K=%d / N=%d", lda, ldc, K, N);
    MV_REQUIRE(((uintptr_t)A % 16) == 0 && ((uintptr_t)W % 16) == 0 && ((uintptr_t)C % 16) == 0,
               "gemm_lt: operands must be 16-byte aligned");
    MV_REQUIRE(workspace_bytes >= 0 && (workspace != nullptr || workspace_bytes == 0), "gemm_lt: bad workspace");
    std::lock_guard<std::mutex> guard(g_lock);
    if (g_handle == nullptr) LT_CHECK(hipblasLtCreate(&g_handle));
    const auto key = std::make_tuple(M, N, K, lda, ldc, bias != nullptr ? 1 : 0, float_out ? 1 : 0);
    auto it = g_plans.find(key);
    if (it == g_plans.end()) {
        LtPlan p;
        if (int rc = make_plan(p, M, N, K, lda, ldc, bias != nullptr, float_out, (size_t)workspace_bytes)) {
            drop_plan(p);
            return rc;
        }
        it = g_plans.emplace(key, p).first;
    }
    LtPlan& p = it->second;
    if (!p.served) {
        mv_fail("gemm_lt: the library has no algorithm for M=%d N=%d K=%d (lda %ld, ldc %ld) within %ld bytes of workspace",
                M, N, K, lda, ldc, workspace_bytes);
        return 2;
    }
    MV_REQUIRE((long)p.workspace <= workspace_bytes, "gemm_lt: the plan needs %zu bytes of workspace, %ld were brought",
               p.workspace, workspace_bytes);
    if (bias != nullptr)
        LT_CHECK(hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_BIAS_POINTER, &bias, sizeof(bias)));
    const float alpha = 1.f, beta = 0.f;
    LT_CHECK(hipblasLtMatmul(g_handle, p.desc, &alpha, W, p.w, A, p.a, &beta, C, p.c, C, p.c, &p.algo, workspace,
                             (size_t)workspace_bytes, stream));
    return 0;
}
