// Event-pair timer on one stream: start() records, end() records, waits and returns the
// elapsed milliseconds.  Counterpart of the reference's CudaTimer
// (src/common/cuda_timer.h:11-52).
#pragma once

#include "../common.h"

namespace hgemm {

class HipTimer {
public:
    explicit HipTimer(hipStream_t stream = nullptr) : m_stream(stream) {
        HGEMM_CHECK_HIP_ERROR(hipEventCreate(&m_start));
        HGEMM_CHECK_HIP_ERROR(hipEventCreate(&m_end));
    }
    ~HipTimer() {
        if (m_start) (void)hipEventDestroy(m_start);
        if (m_end) (void)hipEventDestroy(m_end);
    }

    void start() { HGEMM_CHECK_HIP_ERROR(hipEventRecord(m_start, m_stream)); }

    float end() {
        HGEMM_CHECK_HIP_ERROR(hipEventRecord(m_end, m_stream));
        HGEMM_CHECK_HIP_ERROR(hipEventSynchronize(m_end));
        float ms = 0.0f;
        HGEMM_CHECK_HIP_ERROR(hipEventElapsedTime(&ms, m_start, m_end));
        return ms;
    }

private:
    hipStream_t m_stream = nullptr;
    hipEvent_t m_start = nullptr;
    hipEvent_t m_end = nullptr;

    HGEMM_DISALLOW_COPY_AND_ASSIGN(HipTimer);
};

}  // namespace hgemm
