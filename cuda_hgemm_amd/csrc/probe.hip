// hgemm_probe_loop: where the time of the tuned 256x256x64 kernel goes, measured inside
// the kernel.  The kernel is launched `launches` times back to back (the part settles on
// its power-limited clock only after some tens of launches); in the last launch one thread
// per workgroup records wall-clock and shader-clock timestamps around its K loop.  Three
// builds of the same kernel are available: the real one, one whose loop issues no
// global -> LDS copies, and one that issues neither copies nor operand reads (their
// results are meaningless; they exist to price the copies and the reads in issue slots and
// in clock).
#include <vector>

#include "../../include/hgemm.h"
#include "mfma_pipelined.h"

namespace hgemm {
namespace {

template <int DBG>
using ProbeConfig = PipeConfig<256, 256, 64, 2, 2, 2, 16, 8, DBG, 1>;

template <int DBG>
void run_probe(const void *A, const void *B, void *C, size_t M, size_t N, size_t K, size_t launches, double *out) {
    using Cfg = ProbeConfig<DBG>;
    HGEMM_CHECK_MSG(Cfg::supports(M, N, K), "the probe needs M %% 256 == 0, N %% 256 == 0, K %% 64 == 0, K >= 128");
    HGEMM_CHECK(launches >= 1);
    const size_t workgroups = (M / Cfg::BM) * (N / Cfg::BN);
    long long *trace = nullptr;
    HGEMM_CHECK_HIP_ERROR(hipMalloc(reinterpret_cast<void **>(&trace), workgroups * 8 * sizeof(long long)));
    hipEvent_t begin, last, end;
    HGEMM_CHECK_HIP_ERROR(hipEventCreate(&begin));
    HGEMM_CHECK_HIP_ERROR(hipEventCreate(&last));
    HGEMM_CHECK_HIP_ERROR(hipEventCreate(&end));
    HGEMM_CHECK_HIP_ERROR(hipEventRecord(begin, nullptr));
    for (size_t i = 0; i < launches; ++i) {
        if (i + 1 == launches) HGEMM_CHECK_HIP_ERROR(hipEventRecord(last, nullptr));
        launch_pipelined<Cfg>(A, B, C, M, N, K, "hgemm_probe_loop", i + 1 == launches ? trace : nullptr);
    }
    HGEMM_CHECK_HIP_ERROR(hipEventRecord(end, nullptr));
    HGEMM_CHECK_HIP_ERROR(hipEventSynchronize(end));
    float ms_all = 0.f, ms_last = 0.f;
    HGEMM_CHECK_HIP_ERROR(hipEventElapsedTime(&ms_all, begin, end));
    HGEMM_CHECK_HIP_ERROR(hipEventElapsedTime(&ms_last, last, end));
    std::vector<long long> h(workgroups * 8);
    HGEMM_CHECK_HIP_ERROR(hipMemcpy(h.data(), trace, h.size() * sizeof(long long), hipMemcpyDeviceToHost));
    HGEMM_CHECK_HIP_ERROR(hipFree(trace));
    HGEMM_CHECK_HIP_ERROR(hipEventDestroy(begin));
    HGEMM_CHECK_HIP_ERROR(hipEventDestroy(last));
    HGEMM_CHECK_HIP_ERROR(hipEventDestroy(end));

    int wall_khz = 100000;  // s_memrealtime ticks
    (void)hipDeviceGetAttribute(&wall_khz, hipDeviceAttributeWallClockRate, 0);
    const double us_per_tick = 1e3 / (double)wall_khz;
    double prologue = 0, loop = 0, epilogue = 0, cycles = 0;
    for (size_t w = 0; w < workgroups; ++w) {
        const long long *t = &h[w * 8];  // begin, loop start, loop end, end, hw id, xcc id, loop shader cycles
        prologue += (double)(t[1] - t[0]) * us_per_tick;
        loop += (double)(t[2] - t[1]) * us_per_tick;
        epilogue += (double)(t[3] - t[2]) * us_per_tick;
        cycles += (double)t[6];
    }
    prologue /= workgroups, loop /= workgroups, epilogue /= workgroups, cycles /= workgroups;
    // MFMAs a wave issues in the loop, 16 cycles of the matrix pipe each
    const double mfma_cycles = (double)(K / Cfg::BK) * Cfg::PKSTEPS * Cfg::PTM * Cfg::PTN * 16.0;
    out[0] = ms_all / (double)launches;  // average over all launches, ms
    out[1] = ms_last;                    // the traced launch, ms
    out[2] = prologue;                   // per workgroup, us
    out[3] = loop;
    out[4] = epilogue;
    out[5] = cycles;                     // shader cycles inside the loop
    out[6] = cycles / loop * 1e-3;       // shader clock during the loop, GHz
    out[7] = mfma_cycles / cycles;       // fraction of loop cycles in which the wave's SIMD has an MFMA issued
}

}  // namespace
}  // namespace hgemm

extern "C" void hgemm_probe_loop(const hgemm_half *A, const hgemm_half *B, hgemm_half *C, size_t M, size_t N, size_t K,
                                 int mode, size_t launches, double *out8) {
    using namespace hgemm;
    HGEMM_CHECK(out8 != nullptr);
    switch (mode) {
        case 0: run_probe<0>(A, B, C, M, N, K, launches, out8); break;
        case 1: run_probe<1>(A, B, C, M, N, K, launches, out8); break;
        case 2: run_probe<4>(A, B, C, M, N, K, launches, out8); break;
        default: HGEMM_CHECK_MSG(false, "probe mode %d (0: real kernel, 1: no copies, 2: no copies, no operand reads)", mode);
    }
}
