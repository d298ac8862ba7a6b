// hgemm_probe: where the time of the tuned 256x256x64 kernels (interleaved and chained) goes,
// measured inside the kernel.  A program of its own (bin/hgemm_probe), not part of libhgemm.so: the builds of
// the kernel it runs carry timestamp code, and three of them compute nothing meaningful.  The kernel is launched `launches` times back to back (the part settles on
// its power-limited clock only after some tens of launches); in the last launch one thread
// per workgroup records wall-clock and shader-clock timestamps around its K loop.  Four
// builds of the same kernel are run: the real one, one whose copies always fetch the same
// two K chunks (every copy hits L2: prices the traffic between L2 and the memory fabric),
// one whose loop issues no global -> LDS copies, and one that issues neither copies nor
// operand reads (the results of the last three are meaningless; they exist to price the
// traffic, the copies and the reads in issue slots and in clock).
//
//     bin/hgemm_probe -M=8192 -N=8192 -K=8192 -launches=150
#include <vector>

#include "../driver/flags.h"
#include "../driver/matrix.h"
#include "../mfma_pipelined.h"

namespace hgemm {
namespace {

// DBG 8: timestamps only; + 1: no copies; + 2: copies from a fixed K offset; + 4: no operand reads;
// + 16 / + 32: tiles in the strip / block order whatever the size of B
template <int DBG>
using ProbeConfig = PipeConfig<256, 256, 64, 2, 2, 2, 16, DBG, 1>;

template <int DBG, PipeKernel WHICH = PipeKernel::Interleaved>
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
        launch_pipelined<Cfg>(A, B, C, M, N, K, "hgemm_probe", i + 1 == launches ? trace : nullptr, WHICH);
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

int main(int argc, char *argv[]) {
    using namespace hgemm;
    Flags flags;
    flags.define("M", "8192", "M (a multiple of 256)");
    flags.define("N", "8192", "N (a multiple of 256)");
    flags.define("K", "8192", "K (a multiple of 64, at least 128)");
    flags.define("launches", "150", "back-to-back launches per build; the last one is traced");
    flags.define("seed", "20230212", "seed of the input matrices");
    flags.parse(argc, argv);
    const size_t M = flags.u64("M"), N = flags.u64("N"), K = flags.u64("K"), launches = flags.u64("launches");
    const FillSpec uniform;
    Matrix A(M, K, "Matrix A", flags.u64("seed"), 1, uniform), B(K, N, "Matrix B", flags.u64("seed"), 2, uniform);
    Matrix C(M, N, "Matrix C", flags.u64("seed"), 3, FillSpec{Fill::Zero, 0.f, 0.f});
    static const char *names[10] = {"interleaved kernel", "interleaved, copies always from the same two chunks (all L2 hits)",
                                   "interleaved, loop without copies", "interleaved, loop without copies and operand reads",
                                   "chained kernel", "chained, copies always from the same two chunks (all L2 hits)",
                                   "chained, loop without copies", "chained, loop without copies and operand reads",
                                   "chained, tiles in strips (the order for a B of at most 144 MiB)",
                                   "chained, tiles in 16 x 16 blocks per round (the order for a larger B)"};
    constexpr PipeKernel CH = PipeKernel::Chained;
    for (int mode = 0; mode < 10; ++mode) {
        double r[8];
        const uint16_t *a = A.getDevPtr(), *b = B.getDevPtr();
        uint16_t *c = C.getDevPtr();
        switch (mode) {
            case 0: run_probe<8>(a, b, c, M, N, K, launches, r); break;
            case 1: run_probe<8 + 2>(a, b, c, M, N, K, launches, r); break;
            case 2: run_probe<8 + 1>(a, b, c, M, N, K, launches, r); break;
            case 3: run_probe<8 + 4>(a, b, c, M, N, K, launches, r); break;
            case 4: run_probe<8, CH>(a, b, c, M, N, K, launches, r); break;
            case 5: run_probe<8 + 2, CH>(a, b, c, M, N, K, launches, r); break;
            case 6: run_probe<8 + 1, CH>(a, b, c, M, N, K, launches, r); break;
            case 7: run_probe<8 + 4, CH>(a, b, c, M, N, K, launches, r); break;
            case 8: run_probe<8 + 16, CH>(a, b, c, M, N, K, launches, r); break;
            default: run_probe<8 + 32, CH>(a, b, c, M, N, K, launches, r); break;
        }
        HLOG("Probe %s: %zu launches avg %.4f ms, traced launch %.4f ms (%.1f TFLOPS); per workgroup: prologue "
             "%.2f us, loop %.2f us, epilogue %.2f us; loop %.0f shader cycles at %.3f GHz, MFMA issue %.1f%%",
             names[mode], launches, r[0], r[1], 2.0 * M * N * K * 1e-12 / (r[1] * 1e-3), r[2], r[3], r[4], r[5], r[6],
             100.0 * r[7]);
    }
    return 0;
}
