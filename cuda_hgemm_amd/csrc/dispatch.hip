// hgemm_skinny and hgemm_auto: shape-driven choice among the tuned kernels.
#include "../../include/hgemm.h"
#include "mfma_pipelined.h"
#include "mfma_skinny.h"
#include "plan.h"

namespace hgemm {

namespace {

// Process-lifetime fp32 workspace for split-K partial sums; grows on demand, never freed
// (the reference keeps its vendor handle the same way, src/cublas_tensor_op.cu:18).
float *splitk_workspace(size_t bytes) {
    static float *ptr = nullptr;
    static size_t capacity = 0;
    if (bytes > capacity) {
        if (ptr) {
            HGEMM_CHECK_HIP_ERROR(hipDeviceSynchronize());  // earlier launches may still use it
            HGEMM_CHECK_HIP_ERROR(hipFree(ptr));
        }
        size_t want = bytes < (64ull << 20) ? (64ull << 20) : bytes;
        HGEMM_CHECK_HIP_ERROR(hipMalloc(reinterpret_cast<void **>(&ptr), want));
        capacity = want;
    }
    return ptr;
}

int compute_units() {
    static int cus = [] {
        // A planning query must also work where no GPU is visible: assume one MI355X.
        int dev = 0, n = 0;
        if (hipGetDevice(&dev) != hipSuccess) return 256;
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) return 256;
        return n > 0 ? n : 256;
    }();
    return cus;
}

template <class Cfg>
void launch_splitk(const void *A, const void *B, void *C, size_t M, size_t N, size_t K, int splits) {
    static bool configured = [] {
        HGEMM_CHECK_HIP_ERROR(hipFuncSetAttribute(reinterpret_cast<const void *>(&hgemm_skinny_kernel<Cfg>),
                                                  hipFuncAttributeMaxDynamicSharedMemorySize, Cfg::LDS_BYTES));
        return true;
    }();
    (void)configured;
    HGEMM_CHECK(N % Cfg::BN == 0);
    HGEMM_CHECK(splits >= 1 && K % ((size_t)splits * Cfg::BK) == 0);
    const dim3 grid((unsigned)(N / Cfg::BN), (unsigned)div_ceil(M, Cfg::BM), (unsigned)splits);
    float *partial = splits > 1 ? splitk_workspace((size_t)splits * M * N * sizeof(float)) : nullptr;
    hgemm_skinny_kernel<Cfg><<<grid, dim3(Cfg::THREADS), Cfg::LDS_BYTES, nullptr>>>(
        reinterpret_cast<const half_t *>(A), reinterpret_cast<const half_t *>(B), reinterpret_cast<half_t *>(C),
        partial, (int)M, (int)N, (int)K, (int)(K / splits));
    HGEMM_CHECK_HIP_ERROR(hipGetLastError());
    if (splits > 1) {
        const size_t elems = M * N;
        const unsigned blocks = (unsigned)div_ceil(elems / 8, 256);
        splitk_reduce_kernel<<<dim3(blocks), dim3(256), 0, nullptr>>>(partial, reinterpret_cast<half_t *>(C), elems,
                                                                      splits);
        HGEMM_CHECK_HIP_ERROR(hipGetLastError());
    }
}

//                         BM   BN  WM WN stages
using Skinny32 = SkinnyConfig<32, 128, 1, 4, 4>;
using Skinny64 = SkinnyConfig<64, 128, 2, 2, 4>;
using Skinny128 = SkinnyConfig<128, 128, 2, 2, 4>;
using Split64 = SkinnyConfig<64, 64, 2, 2, 4>;

// 256x256x64 tile on v_mfma_f32_16x16x32_f16, two B buffers and three A buffers (all 160 KB of LDS)
using Big256 = PipeConfig<256, 256, 64, 2, 2, 2, 16, 8, 0, 1>;
using Mid128 = PipeConfig<128, 128, 64, 2, 2, 3, 16>;

// Number of K slices for a launch of `tiles` workgroups when `slots` can be resident at
// once: the power of two (<= 16) that fills the most slots per round; fewer slices win
// ties.  Each slice must be a whole number of 64-wide chunks and at least two of them.
int choose_splits(size_t tiles, size_t slots, size_t K) {
    int best = 1;
    double best_fill = 0.0;
    for (int s = 1; s <= 16; s *= 2) {
        if (K % ((size_t)s * 64) != 0 || K / s < 128) break;
        const size_t wgs = tiles * s;
        const size_t rounds = div_ceil(wgs, slots);
        const double fill = (double)wgs / (double)(rounds * slots);
        if (fill > best_fill + 0.02) {
            best_fill = fill;
            best = s;
        }
    }
    return best;
}

}  // namespace

bool skinny_supports(size_t M, size_t N, size_t K) {
    return M >= 1 && M <= 128 && N % 128 == 0 && K % 64 == 0 && N > 0 && K > 0;
}

Plan plan_for(size_t M, size_t N, size_t K) {
    Plan p;
    if (M == 0 || N == 0 || K == 0) return p;
    const size_t cus = (size_t)compute_units();
    if (skinny_supports(M, N, K)) {
        p.kernel = M <= 32 ? KERNEL_SKINNY32 : (M <= 64 ? KERNEL_SKINNY64 : KERNEL_SKINNY128);
        const size_t per_cu = M <= 32 ? 2 : 1;  // ring of 80 KB fits twice in 160 KB of LDS
        p.splits = choose_splits(N / 128, cus * per_cu, K);
        return p;
    }
    if (Big256::supports(M, N, K) && (M / 256) * (N / 256) >= cus * 3 / 4) {
        p.kernel = KERNEL_BIG256;
        return p;
    }
    if (Mid128::supports(M, N, K) && (M / 128) * (N / 128) >= cus * 3 / 4) {
        p.kernel = KERNEL_MID128;
        return p;
    }
    if (N % 128 == 0 && K % 64 == 0 && (div_ceil(M, 128) * (N / 128)) >= cus / 8) {
        p.kernel = KERNEL_SPLIT128;
        p.splits = choose_splits(div_ceil(M, 128) * (N / 128), cus, K);
        return p;
    }
    if (N % 64 == 0 && K % 64 == 0) {
        p.kernel = KERNEL_SPLIT64;
        p.splits = choose_splits(div_ceil(M, 64) * (N / 64), cus * 2, K);
        return p;
    }
    p.kernel = KERNEL_SIMT;
    return p;
}

void run_plan(const Plan &p, const void *A, const void *B, void *C, size_t M, size_t N, size_t K) {
    switch (p.kernel) {
        case KERNEL_BIG256: launch_pipelined<Big256>(A, B, C, M, N, K, "hgemm_auto"); break;
        case KERNEL_MID128: launch_pipelined<Mid128>(A, B, C, M, N, K, "hgemm_auto"); break;
        case KERNEL_SKINNY32: launch_splitk<Skinny32>(A, B, C, M, N, K, p.splits); break;
        case KERNEL_SKINNY64: launch_splitk<Skinny64>(A, B, C, M, N, K, p.splits); break;
        case KERNEL_SKINNY128:
        case KERNEL_SPLIT128: launch_splitk<Skinny128>(A, B, C, M, N, K, p.splits); break;
        case KERNEL_SPLIT64: launch_splitk<Split64>(A, B, C, M, N, K, p.splits); break;
        case KERNEL_SIMT:
            hgemm_simt_naive(reinterpret_cast<const hgemm_half *>(A), reinterpret_cast<const hgemm_half *>(B),
                             reinterpret_cast<hgemm_half *>(C), M, N, K);
            break;
        default: HGEMM_CHECK_MSG(false, "no kernel for M=%zu N=%zu K=%zu", M, N, K);
    }
}

}  // namespace hgemm

using namespace hgemm;

extern "C" void hgemm_skinny(const hgemm_half *A, const hgemm_half *B, hgemm_half *C, size_t M, size_t N, size_t K) {
    check_operands(A, B, C, M, N, K);
    HGEMM_CHECK_MSG(skinny_supports(M, N, K),
                    "hgemm_skinny needs M <= 128, N %% 128 == 0, K %% 64 == 0 (got M=%zu N=%zu K=%zu)", M, N, K);
    run_plan(plan_for(M, N, K), A, B, C, M, N, K);
}
extern "C" int hgemm_skinny_supports(size_t M, size_t N, size_t K) { return skinny_supports(M, N, K) ? 1 : 0; }

extern "C" void hgemm_auto(const hgemm_half *A, const hgemm_half *B, hgemm_half *C, size_t M, size_t N, size_t K) {
    check_operands(A, B, C, M, N, K);
    run_plan(plan_for(M, N, K), A, B, C, M, N, K);
}
extern "C" int hgemm_auto_supports(size_t M, size_t N, size_t K) { return M > 0 && N > 0 && K > 0; }

// Which kernel and how many K slices hgemm_auto uses for a shape (for reports and tests).
extern "C" int hgemm_auto_plan(size_t M, size_t N, size_t K, int *splits) {
    const Plan p = plan_for(M, N, K);
    if (splits) *splits = p.splits;
    return p.kernel;
}
extern "C" const char *hgemm_kernel_name(int kernel) {
    switch (kernel) {
        case KERNEL_BIG256: return "pipelined 256x256x64, 4 waves, LDS ring 3 (A) + 2 (B)";
        case KERNEL_MID128: return "pipelined 128x128x64, 4 waves, 3-stage ring";
        case KERNEL_SKINNY32: return "split-K 32x128x64, 4-stage ring";
        case KERNEL_SKINNY64: return "split-K 64x128x64, 4-stage ring";
        case KERNEL_SKINNY128: return "split-K 128x128x64, 4-stage ring";
        case KERNEL_SPLIT128: return "split-K 128x128x64, 4-stage ring";
        case KERNEL_SPLIT64: return "split-K 64x64x64, 4-stage ring";
        case KERNEL_SIMT: return "scalar fallback";
        default: return "none";
    }
}
