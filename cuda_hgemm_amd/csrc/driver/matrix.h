// Host + device copy of one fp16 matrix with seeded fills, device <-> host moves and the
// max / average absolute difference against another matrix.  Counterpart of the
// reference's Matrix (src/common/matrix.h:13-132); unlike it the fill is seeded and
// counter-based, so a run is reproducible and does not depend on the thread count.
#pragma once

#include <math.h>

#include <string>
#include <vector>

#include "../common.h"

namespace hgemm {

enum class Fill { Uniform, Normal, Zero };

struct FillSpec {
    Fill kind = Fill::Uniform;
    float p0 = -1.0f;  // uniform: low   | normal: mean
    float p1 = 1.0f;   // uniform: high  | normal: sigma
};

// "uniform", "uniform:lo:hi", "normal", "normal:sigma", "normal:mean:sigma", "zero"
inline FillSpec parse_fill(const std::string &text) {
    FillSpec spec;
    std::vector<std::string> parts;
    size_t pos = 0;
    while (true) {
        const size_t next = text.find(':', pos);
        parts.push_back(text.substr(pos, next == std::string::npos ? std::string::npos : next - pos));
        if (next == std::string::npos) break;
        pos = next + 1;
    }
    if (parts[0] == "uniform") {
        spec.kind = Fill::Uniform;
        if (parts.size() == 3) {
            spec.p0 = strtof(parts[1].c_str(), nullptr);
            spec.p1 = strtof(parts[2].c_str(), nullptr);
        }
    } else if (parts[0] == "normal") {
        spec.kind = Fill::Normal;
        spec.p0 = 0.0f;
        spec.p1 = 1.0f;
        if (parts.size() == 2) spec.p1 = strtof(parts[1].c_str(), nullptr);
        if (parts.size() == 3) {
            spec.p0 = strtof(parts[1].c_str(), nullptr);
            spec.p1 = strtof(parts[2].c_str(), nullptr);
        }
    } else if (parts[0] == "zero") {
        spec.kind = Fill::Zero;
    } else {
        HGEMM_CHECK_MSG(false, "unknown distribution '%s'", text.c_str());
    }
    return spec;
}

inline uint64_t mix64(uint64_t z) {
    z += 0x9e3779b97f4a7c15ull;
    z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ull;
    z = (z ^ (z >> 27)) * 0x94d049bb133111ebull;
    return z ^ (z >> 31);
}

// Element i of matrix `stream` under `seed`: a counter-based generator, so a fill does not
// depend on the thread count or on the order of evaluation.  Host code only.
inline void fill_host(_Float16 *dst, size_t elems, uint64_t seed, uint64_t stream, const FillSpec &fill) {
    const uint64_t key = mix64(seed ^ (stream * 0xd1342543de82ef95ull));
    const long n = (long)elems;
#pragma omp parallel for schedule(static)
    for (long i = 0; i < n; ++i) {
        const uint64_t r = mix64(key + (uint64_t)i * 0x9e3779b97f4a7c15ull);
        float v = 0.0f;
        if (fill.kind == Fill::Uniform) {
            v = fill.p0 + (fill.p1 - fill.p0) * ((float)(r >> 40) * (1.0f / 16777216.0f));
        } else if (fill.kind == Fill::Normal) {
            const double u1 = ((double)(uint32_t)(r >> 32) + 1.0) * (1.0 / 4294967296.0);
            const double u2 = (double)(uint32_t)r * (1.0 / 4294967296.0);
            v = (float)(fill.p0 + fill.p1 * sqrt(-2.0 * log(u1)) * cos(6.283185307179586476925 * u2));
        }
        dst[i] = (_Float16)v;  // round-to-nearest-even, as __float2half
    }
}

// Position-dependent 64-bit checksum of fp16 bit patterns: sum of (bits + 1) * odd(i) mod
// 2^64 with odd(i) = (i * 0x9e3779b97f4a7c15) | 1.  Goes into the JSON report so that a run's
// inputs can be compared with another generator's for the same seed.
inline uint64_t checksum64(const _Float16 *data, size_t elems) {
    uint64_t sum = 0;
    const long n = (long)elems;
#pragma omp parallel for schedule(static) reduction(+ : sum)
    for (long i = 0; i < n; ++i) {
        uint16_t bits;
        memcpy(&bits, &data[i], sizeof(bits));
        sum += ((uint64_t)bits + 1u) * (((uint64_t)i * 0x9e3779b97f4a7c15ull) | 1u);
    }
    return sum;
}

class Matrix {
public:
    Matrix(size_t row, size_t col, const std::string &name, uint64_t seed, uint64_t stream, const FillSpec &fill)
        : m_row(row), m_col(col), m_name(name) {
        HGEMM_CHECK_GT(m_row, 0u);
        HGEMM_CHECK_GT(m_col, 0u);
        m_elem_num = m_row * m_col;
        m_host.resize(m_elem_num);
        HGEMM_CHECK_HIP_ERROR(hipMalloc(reinterpret_cast<void **>(&m_dev_ptr), m_elem_num * sizeof(_Float16)));
        fill_host(m_host.data(), m_elem_num, seed, stream, fill);
        m_fill_checksum = checksum64(m_host.data(), m_elem_num);
        moveToDevice();
        HLOG("%s: %zu * %zu, cpu: %p, gpu: %p", m_name.c_str(), m_row, m_col, (void *)m_host.data(), (void *)m_dev_ptr);
    }

    ~Matrix() {
        if (m_dev_ptr) (void)hipFree(m_dev_ptr);
    }

    size_t getRow() const { return m_row; }
    size_t getCol() const { return m_col; }
    size_t getElemNum() const { return m_elem_num; }
    _Float16 *getHostPtr() { return m_host.data(); }
    uint16_t *getDevPtr() const { return m_dev_ptr; }

    // Device-to-device copy of `base` into this matrix: every evaluation starts from the
    // same C contents (reference src/common/matrix.h:72-79).
    void tearUp(const Matrix *base) {
        HGEMM_CHECK(base);
        HGEMM_CHECK_EQ(m_row, base->getRow());
        HGEMM_CHECK_EQ(m_col, base->getCol());
        HGEMM_CHECK_HIP_ERROR(
            hipMemcpy(m_dev_ptr, base->getDevPtr(), m_elem_num * sizeof(_Float16), hipMemcpyDeviceToDevice));
    }
    void moveToHost() {
        HGEMM_CHECK_HIP_ERROR(hipMemcpy(m_host.data(), m_dev_ptr, m_elem_num * sizeof(_Float16), hipMemcpyDeviceToHost));
    }
    void moveToDevice() {
        HGEMM_CHECK_HIP_ERROR(hipMemcpy(m_dev_ptr, m_host.data(), m_elem_num * sizeof(_Float16), hipMemcpyHostToDevice));
    }
    void memSetHost() { memset(m_host.data(), 0, m_elem_num * sizeof(_Float16)); }
    // Byte pattern fill of the device copy; 0xff.. is an fp16 NaN, which exposes any output
    // element a kernel fails to write.
    void memSetDevice(int byte = 0) { HGEMM_CHECK_HIP_ERROR(hipMemset(m_dev_ptr, byte, m_elem_num * sizeof(_Float16))); }

    // max / mean |this - base| and the rms of base (reference src/common/matrix.h:97-114
    // logs the first two; the rms turns the max into a relative error).
    void checkValue(Matrix *base) {
        HGEMM_CHECK(base);
        HGEMM_CHECK_EQ(m_row, base->getRow());
        HGEMM_CHECK_EQ(m_col, base->getCol());
        double max_diff = 0.0, sum = 0.0, sq = 0.0;
        size_t non_finite = 0;
        const _Float16 *a = m_host.data(), *b = base->getHostPtr();
        for (size_t i = 0; i < m_elem_num; ++i) {
            const double x = (double)(float)a[i], y = (double)(float)b[i];
            if (!std::isfinite(x)) {
                ++non_finite;
                continue;
            }
            const double d = fabs(x - y);
            max_diff = d > max_diff ? d : max_diff;
            sum += d;
            sq += y * y;
        }
        m_max_diff = max_diff;
        m_avg_diff = sum / (double)m_elem_num;
        m_base_rms = sqrt(sq / (double)m_elem_num);
        m_non_finite = non_finite;
        HLOG("Max diff: %f, avg diff: %f", m_max_diff, m_avg_diff);
    }
    double maxDiff() const { return m_max_diff; }
    double avgDiff() const { return m_avg_diff; }
    double baseRms() const { return m_base_rms; }
    size_t nonFinite() const { return m_non_finite; }
    // checksum64 of the values the constructor generated (not of later host contents)
    uint64_t fillChecksum() const { return m_fill_checksum; }

private:
    const size_t m_row = 0;
    const size_t m_col = 0;
    const std::string m_name = "Matrix";
    size_t m_elem_num = 0;
    std::vector<_Float16> m_host;
    uint16_t *m_dev_ptr = nullptr;
    double m_max_diff = 0.0, m_avg_diff = 0.0, m_base_rms = 0.0;
    size_t m_non_finite = 0;
    uint64_t m_fill_checksum = 0;

    HGEMM_DISALLOW_COPY_AND_ASSIGN(Matrix);
};

}  // namespace hgemm
