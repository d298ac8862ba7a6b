// Benchmark / check harness around one (M, N, K) problem.  Counterpart of the reference's
// Tester (src/common/tester.h:14-131): owns A, B, C and the vendor result `base`, runs
// warm-up and timed iterations of a kernel entry point, logs time, TFLOPS and the ratio to
// the first variant evaluated (the vendor library), and optionally checks the result.
// Differences: inputs are seeded; C starts from a NaN pattern so unwritten outputs are
// caught; the check has a threshold (max |diff| <= 1e-2 * sqrt(K/256) * rms(base)) and
// failures are counted; small problems can rotate over several operand sets so repeated
// calls read HBM rather than the on-chip caches.
#pragma once

#include <math.h>
#include <unistd.h>

#include <memory>
#include <string>
#include <vector>

#include "../../../include/hgemm.h"
#include "../../../include/hgemm_hipblaslt.h"
#include "hip_timer.h"
#include "matrix.h"

namespace hgemm {

struct EvalRecord {
    std::string name;
    double warmup_ms = 0.0, ms = 0.0, tflops = 0.0, gbps = 0.0, pct_of_base = 0.0;
    double shader_mhz = 0.0;  // average shader clock over the timed calls
    bool checked = false, pass = true;
    double max_diff = 0.0, avg_diff = 0.0, rel_err = 0.0;
};

class Tester {
public:
    Tester(size_t M, size_t N, size_t K, size_t warmup_iterations, size_t profiling_iterations, size_t sleep_duration,
           bool enable_check, uint64_t seed, const FillSpec &fill_a, const FillSpec &fill_b, size_t rotate_mb)
        : m_M(M),
          m_N(N),
          m_K(K),
          m_warmup_iterations(warmup_iterations),
          m_profiling_iterations(profiling_iterations),
          m_sleep_duration(sleep_duration),
          m_enable_check(enable_check) {
        HGEMM_CHECK_GT(m_M, 0u);
        HGEMM_CHECK_GT(m_N, 0u);
        HGEMM_CHECK_GT(m_K, 0u);
        HGEMM_CHECK_GT(m_warmup_iterations, 0u);
        HGEMM_CHECK_GT(m_profiling_iterations, 0u);
        HGEMM_CHECK_GT(m_sleep_duration, 0u);
        int dev = 0;
        HGEMM_CHECK_HIP_ERROR(hipGetDevice(&dev));
        HGEMM_CHECK_HIP_ERROR(hipDeviceGetAttribute(&m_compute_units, hipDeviceAttributeMultiprocessorCount, dev));
        HGEMM_CHECK_GT(m_compute_units, 0);

        m_A = std::make_shared<Matrix>(m_M, m_K, "Matrix A", seed, 1, fill_a);
        m_B = std::make_shared<Matrix>(m_K, m_N, "Matrix B", seed, 2, fill_b);  // stored as N rows of K
        m_C = std::make_shared<Matrix>(m_M, m_N, "Matrix C", seed, 3, FillSpec{Fill::Zero, 0.f, 0.f});
        m_base = std::make_shared<Matrix>(m_M, m_N, "Matrix Base", seed, 4, FillSpec{Fill::Zero, 0.f, 0.f});

        if (m_enable_check) {
            m_timer.start();
            hgemm_hipblaslt(m_A->getDevPtr(), m_B->getDevPtr(), m_base->getDevPtr(), m_M, m_N, m_K);
            HLOG("Hipblaslt-Gemm use: %.3f ms", m_timer.end());
            m_base->moveToHost();
        }
        m_base->memSetDevice(0xff);  // C is reset to NaNs before every variant

        // Extra operand sets for rotation: device-only copies of A, B and C.
        const size_t set_bytes = (m_M * m_K + m_K * m_N + m_M * m_N) * sizeof(uint16_t);
        size_t sets = rotate_mb ? (rotate_mb * (1ull << 20) + set_bytes - 1) / set_bytes : 1;
        sets = sets < 1 ? 1 : (sets > 64 ? 64 : sets);
        m_As.push_back(m_A->getDevPtr());
        m_Bs.push_back(m_B->getDevPtr());
        m_Cs.push_back(m_C->getDevPtr());
        for (size_t s = 1; s < sets; ++s) {
            uint16_t *a = nullptr, *b = nullptr, *c = nullptr;
            HGEMM_CHECK_HIP_ERROR(hipMalloc(reinterpret_cast<void **>(&a), m_M * m_K * 2));
            HGEMM_CHECK_HIP_ERROR(hipMalloc(reinterpret_cast<void **>(&b), m_K * m_N * 2));
            HGEMM_CHECK_HIP_ERROR(hipMalloc(reinterpret_cast<void **>(&c), m_M * m_N * 2));
            HGEMM_CHECK_HIP_ERROR(hipMemcpy(a, m_A->getDevPtr(), m_M * m_K * 2, hipMemcpyDeviceToDevice));
            HGEMM_CHECK_HIP_ERROR(hipMemcpy(b, m_B->getDevPtr(), m_K * m_N * 2, hipMemcpyDeviceToDevice));
            m_As.push_back(a);
            m_Bs.push_back(b);
            m_Cs.push_back(c);
            m_owned.push_back(a);
            m_owned.push_back(b);
            m_owned.push_back(c);
        }
        if (sets > 1) HLOG("Rotating over %zu operand sets (%.1f MB each)", sets, (double)set_bytes / (1 << 20));
    }

    ~Tester() {
        for (void *p : m_owned) (void)hipFree(p);
    }

    template <typename Func>
    void evaluate(Func &&hgemm, const std::string &name) {
        HLOG("----------------- Evaluating %s -----------------", name.c_str());
        usleep(m_sleep_duration * 1000);
        m_C->tearUp(m_base.get());

        EvalRecord rec;
        rec.name = name;

        // warm up
        m_timer.start();
        for (size_t i = 0; i < m_warmup_iterations; ++i) {
            const size_t s = i % m_As.size();
            hgemm(m_As[s], m_Bs[s], m_Cs[s], m_M, m_N, m_K);
        }
        rec.warmup_ms = static_cast<double>(m_timer.end()) / static_cast<double>(m_warmup_iterations);
        HLOG("Warm up time: %.3f ms", rec.warmup_ms);

        if (m_enable_check) {
            m_C->moveToHost();
            m_C->checkValue(m_base.get());
            rec.checked = true;
            rec.max_diff = m_C->maxDiff();
            rec.avg_diff = m_C->avgDiff();
            const double scale = m_C->baseRms() > 0.0009765625 ? m_C->baseRms() : 0.0009765625;
            rec.rel_err = rec.max_diff / scale;
            const double tol = 1e-2 * sqrt((double)m_K / 256.0);
            rec.pass = m_C->nonFinite() == 0 && rec.rel_err <= tol;
            HLOG("Check %s: max diff / rms(base) = %.3e (tolerance %.3e), non-finite outputs: %zu",
                 rec.pass ? "passed" : "FAILED", rec.rel_err, tol, m_C->nonFinite());
            if (!rec.pass) ++m_failures;
        }

        profile(std::forward<Func>(hgemm), rec);
        m_records.push_back(rec);
    }

    size_t failures() const { return m_failures; }
    uint64_t checksumA() const { return m_A->fillChecksum(); }
    uint64_t checksumB() const { return m_B->fillChecksum(); }
    const std::vector<EvalRecord> &records() const { return m_records; }

private:
    template <typename Func>
    void profile(Func &&hgemm, EvalRecord &rec) {
        hgemm_clock_mark(0);  // the shader clock the part sustains over the timed calls (it is power-managed)
        m_timer.start();
        for (size_t i = 0; i < m_profiling_iterations; ++i) {
            const size_t s = i % m_As.size();
            hgemm(m_As[s], m_Bs[s], m_Cs[s], m_M, m_N, m_K);
        }
        rec.ms = static_cast<double>(m_timer.end()) / static_cast<double>(m_profiling_iterations);
        hgemm_clock_mark(1);
        rec.shader_mhz = hgemm_clock_between_marks_mhz(nullptr, 0, nullptr, nullptr);
        rec.tflops = hgemm_tflops(m_M, m_N, m_K, rec.ms);
        rec.gbps = hgemm_bytes(m_M, m_N, m_K) / (rec.ms * 1e-3) * 1e-9;

        if ((fabs(m_base_time) <= 1e-9) && (fabs(m_base_throughput) <= 1e-9)) {
            m_base_time = rec.ms;
            m_base_throughput = rec.tflops;
        }
        rec.pct_of_base = rec.tflops / m_base_throughput * 100;

        HLOG("%s exit, profiling time: %.3f ms (%.2f%%), throughput: %.3f TFLOPS (%.2f%%)", rec.name.c_str(), rec.ms,
             rec.ms / m_base_time * 100, rec.tflops, rec.pct_of_base);
        HLOG("%s roofline: %.2f%% of 2500 TFLOPS dense FP16, %.1f GB/s algorithmic (%.2f%% of 8000 GB/s), shader clock "
             "%.0f MHz: %.0f flop per cycle and CU of 4096",
             rec.name.c_str(), rec.tflops / 2500.0 * 100, rec.gbps, rec.gbps / 8000.0 * 100, rec.shader_mhz,
             rec.tflops * 1e12 / (rec.shader_mhz * 1e6) / (double)m_compute_units);
    }

    const size_t m_M, m_N, m_K;
    const size_t m_warmup_iterations, m_profiling_iterations, m_sleep_duration;
    const bool m_enable_check;
    int m_compute_units = 0;

    std::shared_ptr<Matrix> m_A;     // row major, M * K
    std::shared_ptr<Matrix> m_B;     // col major, K * N
    std::shared_ptr<Matrix> m_C;     // row major, M * N
    std::shared_ptr<Matrix> m_base;  // row major, M * N: vendor result on the host, NaN pattern on the device

    std::vector<uint16_t *> m_As, m_Bs, m_Cs;  // operand sets cycled through by the loops
    std::vector<void *> m_owned;

    HipTimer m_timer;
    double m_base_time = 0.0;        // first variant evaluated (the vendor library by default)
    double m_base_throughput = 0.0;
    size_t m_failures = 0;
    std::vector<EvalRecord> m_records;

    HGEMM_DISALLOW_COPY_AND_ASSIGN(Tester);
};

}  // namespace hgemm
