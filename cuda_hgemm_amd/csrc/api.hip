// Variant registry, dispatcher and harness helpers of the C ABI (include/hgemm.h).
#include "../../include/hgemm.h"
#include "common.h"
#include "variant_def.h"

#include <mutex>

HGEMM_DECLARE_SUPPORTS(hgemm_mfma_base);
HGEMM_DECLARE_SUPPORTS(hgemm_mfma_padding);
HGEMM_DECLARE_SUPPORTS(hgemm_mfma_swizzle);
HGEMM_DECLARE_SUPPORTS(hgemm_mfma_async);
HGEMM_DECLARE_SUPPORTS(hgemm_mfma_async_pg2s);
HGEMM_DECLARE_SUPPORTS(hgemm_mfma_async_pg2s_ps2r);
HGEMM_DECLARE_SUPPORTS(hgemm_mfma_async_stage2);
HGEMM_DECLARE_SUPPORTS(hgemm_mfma_async_stage3);
HGEMM_DECLARE_SUPPORTS(hgemm_mfma_async_stage4);
HGEMM_DECLARE_SUPPORTS(hgemm_mfma_tiled_64x64);
HGEMM_DECLARE_SUPPORTS(hgemm_mfma_pipelined_64x64);
HGEMM_DECLARE_SUPPORTS(hgemm_mfma_pipelined_128x128);
HGEMM_DECLARE_SUPPORTS(hgemm_mfma_pipelined_192x192);
HGEMM_DECLARE_SUPPORTS(hgemm_mfma_pipelined_256x128);
HGEMM_DECLARE_SUPPORTS(hgemm_mfma_pipelined_256x256);
HGEMM_DECLARE_SUPPORTS(hgemm_mfma_chained_192x192);
HGEMM_DECLARE_SUPPORTS(hgemm_mfma_chained_256x128);
HGEMM_DECLARE_SUPPORTS(hgemm_mfma_chained_256x256);
HGEMM_DECLARE_SUPPORTS(hgemm_skinny);
HGEMM_DECLARE_SUPPORTS(hgemm_auto);

namespace {

int any_shape(size_t M, size_t N, size_t K) { return M > 0 && N > 0 && K > 0; }
int naive_mfma_shape(size_t M, size_t N, size_t K) {
    return M > 0 && N > 0 && K > 0 && M % 32 == 0 && N % 32 == 0 && K % 16 == 0;
}

struct Variant {
    const char *name;    // display name, as in the reference's evaluate() calls (src/main.cu:100-123)
    const char *symbol;  // exported function
    hgemm_fn fn;
    int (*supports)(size_t, size_t, size_t);
    int in_default_run;  // the reference comments the naive / base kernels out of its run
};

const Variant kVariants[] = {
    {"Simt-Naive", "hgemm_simt_naive", hgemm_simt_naive, any_shape, 0},
    {"Mfma-Naive", "hgemm_mfma_naive", hgemm_mfma_naive, naive_mfma_shape, 0},
    {"Mfma-Base", "hgemm_mfma_base", hgemm_mfma_base, hgemm_mfma_base_supports, 0},
    {"Mfma-Padding", "hgemm_mfma_padding", hgemm_mfma_padding, hgemm_mfma_padding_supports, 1},
    {"Mfma-Swizzle", "hgemm_mfma_swizzle", hgemm_mfma_swizzle, hgemm_mfma_swizzle_supports, 1},
    {"Mfma-Async", "hgemm_mfma_async", hgemm_mfma_async, hgemm_mfma_async_supports, 1},
    {"Mfma-Async-Pg2s", "hgemm_mfma_async_pg2s", hgemm_mfma_async_pg2s, hgemm_mfma_async_pg2s_supports, 1},
    {"Mfma-Async-Pg2s-Ps2r", "hgemm_mfma_async_pg2s_ps2r", hgemm_mfma_async_pg2s_ps2r,
     hgemm_mfma_async_pg2s_ps2r_supports, 1},
    {"Mfma-Async-Stage2", "hgemm_mfma_async_stage2", hgemm_mfma_async_stage2, hgemm_mfma_async_stage2_supports, 1},
    {"Mfma-Async-Stage3", "hgemm_mfma_async_stage3", hgemm_mfma_async_stage3, hgemm_mfma_async_stage3_supports, 1},
    {"Mfma-Async-Stage4", "hgemm_mfma_async_stage4", hgemm_mfma_async_stage4, hgemm_mfma_async_stage4_supports, 1},
    // the ladder's kernel on the small tile hgemm_auto uses for small grids
    {"Mfma-Tiled-64x64", "hgemm_mfma_tiled_64x64", hgemm_mfma_tiled_64x64, hgemm_mfma_tiled_64x64_supports, 1},
    // the tuned kernel, one entry per tile, smallest first: the ladder ends at its fastest rung,
    // as the reference's run ends at mmaAsyncStage4 (src/main.cu:123)
    {"Mfma-Pipelined-64x64", "hgemm_mfma_pipelined_64x64", hgemm_mfma_pipelined_64x64,
     hgemm_mfma_pipelined_64x64_supports, 1},
    {"Mfma-Pipelined-128x128", "hgemm_mfma_pipelined_128x128", hgemm_mfma_pipelined_128x128,
     hgemm_mfma_pipelined_128x128_supports, 1},
    {"Mfma-Pipelined-192x192", "hgemm_mfma_pipelined_192x192", hgemm_mfma_pipelined_192x192,
     hgemm_mfma_pipelined_192x192_supports, 1},
    {"Mfma-Pipelined-256x128", "hgemm_mfma_pipelined_256x128", hgemm_mfma_pipelined_256x128,
     hgemm_mfma_pipelined_256x128_supports, 1},
    {"Mfma-Pipelined-256x256", "hgemm_mfma_pipelined_256x256", hgemm_mfma_pipelined_256x256,
     hgemm_mfma_pipelined_256x256_supports, 1},
    // the last rung: each accumulator's MFMAs back to back
    {"Mfma-Chained-192x192", "hgemm_mfma_chained_192x192", hgemm_mfma_chained_192x192,
     hgemm_mfma_chained_192x192_supports, 1},
    {"Mfma-Chained-256x128", "hgemm_mfma_chained_256x128", hgemm_mfma_chained_256x128,
     hgemm_mfma_chained_256x128_supports, 1},
    {"Mfma-Chained-256x256", "hgemm_mfma_chained_256x256", hgemm_mfma_chained_256x256,
     hgemm_mfma_chained_256x256_supports, 1},
    {"Skinny", "hgemm_skinny", hgemm_skinny, hgemm_skinny_supports, 1},
    {"Auto", "hgemm_auto", hgemm_auto, hgemm_auto_supports, 1},
};
constexpr int kVariantCount = (int)(sizeof(kVariants) / sizeof(kVariants[0]));

const Variant *variant_at(int index) {
    HGEMM_CHECK_MSG(index >= 0 && index < kVariantCount, "variant index %d out of range [0, %d)", index,
                    kVariantCount);
    return &kVariants[index];
}

}  // namespace

extern "C" int hgemm_variant_count(void) { return kVariantCount; }
extern "C" const char *hgemm_variant_name(int index) { return variant_at(index)->name; }
extern "C" const char *hgemm_variant_symbol(int index) { return variant_at(index)->symbol; }
extern "C" hgemm_fn hgemm_variant_fn(int index) { return variant_at(index)->fn; }
extern "C" int hgemm_variant_in_default_run(int index) { return variant_at(index)->in_default_run; }

extern "C" int hgemm_variant_find(const char *name) {
    if (!name) return -1;
    for (int i = 0; i < kVariantCount; ++i)
        if (strcmp(name, kVariants[i].name) == 0 || strcmp(name, kVariants[i].symbol) == 0) return i;
    return -1;
}

extern "C" int hgemm_variant_supports(int index, size_t M, size_t N, size_t K) {
    if (M == 0 || N == 0 || K == 0) return 0;
    if (M * K >= (1ull << 31) || N * K >= (1ull << 31) || M * N >= (1ull << 31)) return 0;
    return variant_at(index)->supports(M, N, K);
}

// Timing loop of Tester::profile (reference src/common/tester.h:89-97) with the event
// handling of CudaTimer (reference src/common/cuda_timer.h:32-42): events on the null
// stream, no synchronisation between the timed calls.
extern "C" double hgemm_profile_ms(hgemm_fn fn, const hgemm_half *A, const hgemm_half *B, hgemm_half *C, size_t M,
                                   size_t N, size_t K, size_t warmup, size_t iterations) {
    const hgemm_half *As[1] = {A};
    const hgemm_half *Bs[1] = {B};
    hgemm_half *Cs[1] = {C};
    return hgemm_profile_rotating_ms(fn, As, Bs, Cs, 1, M, N, K, warmup, iterations);
}

extern "C" double hgemm_profile_rotating_ms(hgemm_fn fn, const hgemm_half *const *A, const hgemm_half *const *B,
                                            hgemm_half *const *C, size_t n_sets, size_t M, size_t N, size_t K,
                                            size_t warmup, size_t iterations) {
    HGEMM_CHECK(fn != nullptr);
    HGEMM_CHECK_GT(n_sets, 0u);
    HGEMM_CHECK_GT(iterations, 0u);
    hipEvent_t start = nullptr, stop = nullptr;
    HGEMM_CHECK_HIP_ERROR(hipEventCreate(&start));
    HGEMM_CHECK_HIP_ERROR(hipEventCreate(&stop));
    for (size_t i = 0; i < warmup; ++i) fn(A[i % n_sets], B[i % n_sets], C[i % n_sets], M, N, K);
    HGEMM_CHECK_HIP_ERROR(hipEventRecord(start, nullptr));
    for (size_t i = 0; i < iterations; ++i) fn(A[i % n_sets], B[i % n_sets], C[i % n_sets], M, N, K);
    HGEMM_CHECK_HIP_ERROR(hipEventRecord(stop, nullptr));
    HGEMM_CHECK_HIP_ERROR(hipEventSynchronize(stop));
    float ms = 0.0f;
    HGEMM_CHECK_HIP_ERROR(hipEventElapsedTime(&ms, start, stop));
    HGEMM_CHECK_HIP_ERROR(hipEventDestroy(start));
    HGEMM_CHECK_HIP_ERROR(hipEventDestroy(stop));
    return (double)ms / (double)iterations;
}

// ---- shader clock between two points of the null stream.  A power-managed part runs matrix
// work well below its nominal clock, by an amount that differs from board to board, so a
// throughput figure is only comparable across boards together with the clock it was reached
// at.  s_memtime counts shader cycles, s_memrealtime counts at a constant rate
// (hipDeviceAttributeWallClockRate).  The cycle counters of different SIMDs do not share a
// starting point (measured: tens of millions of cycles apart), so a pair of samples is only
// meaningful when both were taken on the same SIMD of the same CU: a mark is a launch of many
// small workgroups in which every wave files its sample under its hardware position, and the
// clock is taken from the positions that were sampled at both marks.
namespace {

// position = XCC_ID (4 bits) | SE_ID (3) | SH_ID (1) | CU_ID (4) | SIMD_ID (2)
constexpr int CLOCK_POSITIONS = 1 << 14, CLOCK_XCDS = 16;
struct ClockSample {
    unsigned long long shader, constant_rate;
};
std::mutex g_clock_mutex;
ClockSample *g_clock_samples[64];  // per device: [2][CLOCK_POSITIONS], allocated by the first mark

__global__ void __launch_bounds__(256) clock_clear_kernel(ClockSample *all) {
    typedef unsigned long long u64x2 __attribute__((ext_vector_type(2)));
    u64x2 zero = {0ull, 0ull};
    *reinterpret_cast<u64x2 *>(&all[(size_t)blockIdx.x * blockDim.x + threadIdx.x]) = zero;
}

__global__ void __launch_bounds__(256) clock_mark_kernel(ClockSample *out) {
    if ((threadIdx.x & 63) != 0) return;
    const unsigned hw = __builtin_amdgcn_s_getreg((31 << 11) | 4);    // HW_ID: simd [5:4], cu [11:8], sh [12], se [15:13]
    const unsigned xcc = __builtin_amdgcn_s_getreg((31 << 11) | 20);  // XCC_ID [3:0]
    const unsigned position = ((xcc & 15) << 10) | (((hw >> 13) & 7) << 7) | (((hw >> 12) & 1) << 6) |
                              (((hw >> 8) & 15) << 2) | ((hw >> 4) & 3);
    typedef unsigned long long u64x2 __attribute__((ext_vector_type(2)));
    u64x2 v;
    v[0] = (unsigned long long)clock64();       // s_memtime
    v[1] = (unsigned long long)wall_clock64();  // s_memrealtime
    *reinterpret_cast<u64x2 *>(&out[position]) = v;  // one 16-byte store: a slot never mixes two waves' samples
}

ClockSample *clock_buffer() {
    int dev = 0;
    HGEMM_CHECK_HIP_ERROR(hipGetDevice(&dev));
    HGEMM_CHECK(dev >= 0 && dev < 64);
    std::lock_guard<std::mutex> lock(g_clock_mutex);
    if (!g_clock_samples[dev])
        HGEMM_CHECK_HIP_ERROR(hipMalloc(reinterpret_cast<void **>(&g_clock_samples[dev]),
                                        sizeof(ClockSample) * 2 * CLOCK_POSITIONS));
    return g_clock_samples[dev];
}

}  // namespace

extern "C" void hgemm_clock_mark(int which) {
    HGEMM_CHECK_MSG(which == 0 || which == 1, "mark %d: there are marks 0 and 1", which);
    ClockSample *base = clock_buffer();
    if (which == 0)  // a position that mark 1 does not reach must not pair with a stale sample
        clock_clear_kernel<<<dim3(2 * CLOCK_POSITIONS / 256), dim3(256), 0, nullptr>>>(base);
    // four waves per workgroup, one per SIMD; 4096 workgroups reach every SIMD of the chip several times over
    clock_mark_kernel<<<dim3(4096), dim3(256), 0, nullptr>>>(base + which * CLOCK_POSITIONS);
    HGEMM_CHECK_HIP_ERROR(hipGetLastError());
}

extern "C" double hgemm_clock_between_marks_mhz(double *per_xcd_mhz, int xcds, double *elapsed_ms, double *detail) {
    static ClockSample h[2][CLOCK_POSITIONS];
    static std::mutex host_mutex;
    std::lock_guard<std::mutex> host_lock(host_mutex);
    HGEMM_CHECK_HIP_ERROR(hipMemcpy(h, clock_buffer(), sizeof(h), hipMemcpyDeviceToHost));  // waits for the null stream
    int dev = 0, wall_khz = 0;
    HGEMM_CHECK_HIP_ERROR(hipGetDevice(&dev));
    HGEMM_CHECK_HIP_ERROR(hipDeviceGetAttribute(&wall_khz, hipDeviceAttributeWallClockRate, dev));
    HGEMM_CHECK_GT(wall_khz, 0);
    double sum_mhz = 0.0, sum_ms = 0.0, lo = 0.0, hi = 0.0, xcd_sum[CLOCK_XCDS] = {};
    int pairs = 0, xcd_pairs[CLOCK_XCDS] = {};
    for (int p = 0; p < CLOCK_POSITIONS; ++p) {
        if (h[0][p].constant_rate == 0 || h[1][p].constant_rate <= h[0][p].constant_rate) continue;
        const double ticks = (double)(h[1][p].constant_rate - h[0][p].constant_rate);
        const double mhz = (double)(h[1][p].shader - h[0][p].shader) / ticks * (double)wall_khz * 1e-3;
        sum_mhz += mhz;
        sum_ms += ticks / (double)wall_khz;
        lo = (pairs == 0 || mhz < lo) ? mhz : lo;
        hi = (pairs == 0 || mhz > hi) ? mhz : hi;
        xcd_sum[p >> 10] += mhz;
        ++xcd_pairs[p >> 10];
        ++pairs;
    }
    HGEMM_CHECK_MSG(pairs > 0, "no SIMD was sampled at both marks: call hgemm_clock_mark(0), then (1), first");
    for (int x = 0; per_xcd_mhz && x < xcds; ++x)
        per_xcd_mhz[x] = (x < CLOCK_XCDS && xcd_pairs[x]) ? xcd_sum[x] / xcd_pairs[x] : 0.0;
    if (elapsed_ms) *elapsed_ms = sum_ms / pairs;
    if (detail) detail[0] = lo, detail[1] = hi, detail[2] = (double)pairs;
    return sum_mhz / pairs;
}

extern "C" double hgemm_tflops(size_t M, size_t N, size_t K, double ms) {
    return (double)(M * N * K * 2) * 1e-12 / (ms * 1e-3);
}

extern "C" double hgemm_bytes(size_t M, size_t N, size_t K) { return 2.0 * ((double)M * K + (double)K * N + (double)M * N); }

extern "C" const char *hgemm_version(void) { return "hgemm-gfx950 0.1"; }
