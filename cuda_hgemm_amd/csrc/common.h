// Shared host-side support for the library and its driver: log line, check macros, HIP
// status checks.  Behaviour follows the reference's conventions (log to stderr, then
// exit(EXIT_FAILURE): reference src/common/common.h:23-55, src/common/logging.h:38-42).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <sys/syscall.h>
#include <time.h>
#include <unistd.h>

namespace hgemm {

inline const char *log_basename(const char *path) {
    const char *slash = strrchr(path, '/');
    return slash ? slash + 1 : path;
}

inline void log_prefix(const char *file, int line, const char *func) {
    char stamp[32];
    time_t now = time(nullptr);
    struct tm tm_now;
    localtime_r(&now, &tm_now);
    strftime(stamp, sizeof(stamp), "%Y-%m-%d %H:%M:%S", &tm_now);
    fprintf(stderr, "[HGEMM %s %d:%ld %s:%d %s] ", stamp, (int)getpid(), (long)syscall(SYS_gettid),
            log_basename(file), line, func);
}

}  // namespace hgemm

// Same field order as the reference's log line, which its plotting script indexes by token.
#define HLOG(format, ...)                                        \
    do {                                                         \
        hgemm::log_prefix(__FILE__, __LINE__, __FUNCTION__);     \
        fprintf(stderr, format "\n", ##__VA_ARGS__);             \
    } while (0)

#define HGEMM_CHECK(x)                        \
    do {                                      \
        if (__builtin_expect(!(x), 0)) {      \
            HLOG("Check failed: %s", #x);     \
            exit(EXIT_FAILURE);               \
        }                                     \
    } while (0)

#define HGEMM_CHECK_MSG(x, format, ...)                              \
    do {                                                             \
        if (__builtin_expect(!(x), 0)) {                             \
            HLOG("Check failed: %s: " format, #x, ##__VA_ARGS__);    \
            exit(EXIT_FAILURE);                                      \
        }                                                            \
    } while (0)

#define HGEMM_CHECK_EQ(x, y) HGEMM_CHECK((x) == (y))
#define HGEMM_CHECK_NE(x, y) HGEMM_CHECK((x) != (y))
#define HGEMM_CHECK_LE(x, y) HGEMM_CHECK((x) <= (y))
#define HGEMM_CHECK_LT(x, y) HGEMM_CHECK((x) < (y))
#define HGEMM_CHECK_GE(x, y) HGEMM_CHECK((x) >= (y))
#define HGEMM_CHECK_GT(x, y) HGEMM_CHECK((x) > (y))

#define HGEMM_CHECK_HIP_ERROR(_expr_)                                                                     \
    do {                                                                                                  \
        hipError_t _ret_ = (_expr_);                                                                      \
        if (__builtin_expect(_ret_ != hipSuccess, 0)) {                                                   \
            int _rt_ = 0, _drv_ = 0;                                                                      \
            (void)hipRuntimeGetVersion(&_rt_);                                                            \
            (void)hipDriverGetVersion(&_drv_);                                                            \
            HLOG("HIP Runtime API error = %04d \"%s\" (%s), runtime version: %d, driver version: %d",     \
                 (int)_ret_, hipGetErrorName(_ret_), #_expr_, _rt_, _drv_);                               \
            exit(EXIT_FAILURE);                                                                           \
        }                                                                                                 \
    } while (0)

#define HGEMM_DISALLOW_COPY_AND_ASSIGN(TypeName) \
    TypeName(const TypeName &) = delete;         \
    void operator=(const TypeName &) = delete

namespace hgemm {

inline size_t div_ceil(size_t a, size_t b) { return (a + b - 1) / b; }

// Operand checks common to every entry point: the reference forms pointers unguarded
// (src/mma/mma_async_stage4.cu:79-80,93-94); here a bad call is diagnosed.
inline void check_operands(const void *A, const void *B, const void *C, size_t M, size_t N, size_t K) {
    HGEMM_CHECK(A != nullptr);
    HGEMM_CHECK(B != nullptr);
    HGEMM_CHECK(C != nullptr);
    HGEMM_CHECK_GT(M, 0u);
    HGEMM_CHECK_GT(N, 0u);
    HGEMM_CHECK_GT(K, 0u);
    // 16-byte vector accesses start at the operand bases (hipMalloc returns 256-byte alignment).
    HGEMM_CHECK_MSG((((uintptr_t)A | (uintptr_t)B | (uintptr_t)C) & 15u) == 0,
                    "A, B and C must be 16-byte aligned (got %p %p %p)", A, B, C);
    // Kernels index with 32-bit element offsets inside one operand.
    HGEMM_CHECK_MSG(M * K < (1ull << 31) && N * K < (1ull << 31) && M * N < (1ull << 31),
                    "operand with more than 2^31 elements (M=%zu N=%zu K=%zu)", M, N, K);
}

}  // namespace hgemm
