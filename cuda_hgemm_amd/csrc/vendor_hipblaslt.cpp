// Vendor-library comparator (libhgemm_hipblaslt.so), the counterpart of the reference's
// cublasTensorOp (reference src/cublas_tensor_op.cu:17-25): process-lifetime handle, the
// same operand view of the row-major / column-major buffers, alpha = 1, beta = 0.
// hipBLASLt offers no fp16-accumulate compute type, so the product is computed in fp32,
// which is also what the hand-written kernels do.
#include <hipblaslt/hipblaslt.h>

#include <map>
#include <tuple>

#include "../../include/hgemm_hipblaslt.h"
#include "common.h"

#define HGEMM_CHECK_HIPBLASLT_ERROR(_expr_)                                          \
    do {                                                                             \
        hipblasStatus_t _ret_ = (_expr_);                                            \
        if (__builtin_expect(_ret_ != HIPBLAS_STATUS_SUCCESS, 0)) {                  \
            HLOG("hipBLASLt API error = %04d (%s)", (int)_ret_, #_expr_);            \
            exit(EXIT_FAILURE);                                                      \
        }                                                                            \
    } while (0)

namespace {

constexpr size_t kWorkspaceBytes = 128ull << 20;

struct Plan {
    hipblasLtMatmulDesc_t desc = nullptr;
    hipblasLtMatrixLayout_t layout_b = nullptr, layout_a = nullptr, layout_c = nullptr;
    hipblasLtMatmulAlgo_t algo;
    size_t workspace = 0;
};

struct Context {
    hipblasLtHandle_t handle = nullptr;
    void *workspace = nullptr;
    std::map<std::tuple<size_t, size_t, size_t>, Plan> plans;

    Context() {
        HGEMM_CHECK_HIPBLASLT_ERROR(hipblasLtCreate(&handle));
        HGEMM_CHECK_HIP_ERROR(hipMalloc(&workspace, kWorkspaceBytes));
    }

    // Column-major view: C^T (N x M, ld N) = op_T(B as K x N, ld K) * (A as K x M, ld K).
    const Plan &plan_for(size_t M, size_t N, size_t K) {
        auto key = std::make_tuple(M, N, K);
        auto it = plans.find(key);
        if (it != plans.end()) return it->second;
        Plan p;
        HGEMM_CHECK_HIPBLASLT_ERROR(hipblasLtMatmulDescCreate(&p.desc, HIPBLAS_COMPUTE_32F, HIP_R_32F));
        hipblasOperation_t op_t = HIPBLAS_OP_T, op_n = HIPBLAS_OP_N;
        HGEMM_CHECK_HIPBLASLT_ERROR(
            hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_TRANSA, &op_t, sizeof(op_t)));
        HGEMM_CHECK_HIPBLASLT_ERROR(
            hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_TRANSB, &op_n, sizeof(op_n)));
        HGEMM_CHECK_HIPBLASLT_ERROR(hipblasLtMatrixLayoutCreate(&p.layout_b, HIP_R_16F, K, N, K));
        HGEMM_CHECK_HIPBLASLT_ERROR(hipblasLtMatrixLayoutCreate(&p.layout_a, HIP_R_16F, K, M, K));
        HGEMM_CHECK_HIPBLASLT_ERROR(hipblasLtMatrixLayoutCreate(&p.layout_c, HIP_R_16F, N, M, N));
        hipblasLtMatmulPreference_t pref = nullptr;
        HGEMM_CHECK_HIPBLASLT_ERROR(hipblasLtMatmulPreferenceCreate(&pref));
        size_t ws = kWorkspaceBytes;
        HGEMM_CHECK_HIPBLASLT_ERROR(hipblasLtMatmulPreferenceSetAttribute(
            pref, HIPBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES, &ws, sizeof(ws)));
        hipblasLtMatmulHeuristicResult_t result[1];
        int found = 0;
        HGEMM_CHECK_HIPBLASLT_ERROR(hipblasLtMatmulAlgoGetHeuristic(handle, p.desc, p.layout_b, p.layout_a, p.layout_c,
                                                                    p.layout_c, pref, 1, result, &found));
        HGEMM_CHECK_MSG(found > 0, "hipBLASLt has no algorithm for M=%zu N=%zu K=%zu", M, N, K);
        p.algo = result[0].algo;
        p.workspace = result[0].workspaceSize;
        HGEMM_CHECK_HIPBLASLT_ERROR(hipblasLtMatmulPreferenceDestroy(pref));
        return plans.emplace(key, p).first->second;
    }
};

}  // namespace

extern "C" void hgemm_hipblaslt(const hgemm_half *A, const hgemm_half *B, hgemm_half *C, size_t M, size_t N,
                                size_t K) {
    hgemm::check_operands(A, B, C, M, N, K);
    static Context ctx;
    static const float alpha = 1.0f, beta = 0.0f;
    const Plan &p = ctx.plan_for(M, N, K);
    HGEMM_CHECK_HIPBLASLT_ERROR(hipblasLtMatmul(ctx.handle, p.desc, &alpha, B, p.layout_b, A, p.layout_a, &beta, C,
                                                p.layout_c, C, p.layout_c, &p.algo, ctx.workspace, kWorkspaceBytes,
                                                nullptr));
}
