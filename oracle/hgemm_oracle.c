/*
 * hgemm_oracle.c -- CPU restatement of the HGEMM hot path.  TEST INFRASTRUCTURE ONLY.
 *
 * This file is the checker, not the product: only tests/, the smoke check and the
 * CPU-baseline leg of the benchmark may load it.  The shipped library never links it.
 *
 * What it restates (reference file:line):
 *   - GEMM semantics  C[m*N+n] = sum_k A[m*K+k] * B[n*K+k]      src/simt_naive.cu:18-24
 *   - operand layouts: A row-major MxK, B column-major KxN (stored as N rows of K),
 *     C row-major MxN                                            src/common/tester.h:117-120
 *   - the vendor call's view of the same layouts (OP_T on B, ldb=K, ldc=N, alpha=1, beta=0)
 *                                                                src/cublas_tensor_op.cu:22-24
 *   - uniform[-1,1] inputs rounded to fp16                       src/common/matrix.h:15,30-33
 *   - max / average absolute difference of two fp16 matrices     src/common/matrix.h:102-111
 *   - throughput = 2*M*N*K*1e-12 / (ms*1e-3) TFLOPS              src/common/tester.h:96-97
 *
 * Deliberate divergence from the reference: products are accumulated in fp32 and rounded
 * to fp16 once at the end (the reference accumulates in fp16, src/simt_naive.cu:18).
 *
 * How each function is pinned (see tests/test_oracle.py):
 *   - oracle_f16_to_f32 / oracle_f32_to_f16: exhaustive 65536-value comparison with the
 *     host's F16C hardware conversion and with numpy.float16, plus a tie/overflow table.
 *   - oracle_hgemm (blocked, threaded): exact-integer inputs (any summation order is
 *     exact), all-ones (C == K), identity operands (pins the N-rows-of-K layout of B and
 *     catches transposition), brute-force double-precision triple loop on small shapes,
 *     numpy float64 golden vectors under tests/golden/, linearity and row-permutation
 *     invariants.
 *   - oracle_fill (counter-based RNG): committed first-values fixtures per seed and
 *     distribution, range and moment checks.
 *   - oracle_diff / oracle_tflops: closed forms.
 * The reference holds no golden vectors and its own check is a log line against a closed
 * vendor library without a threshold (src/common/matrix.h:113), so nothing there can pin
 * numeric values; every function above is pinned by the mathematics instead.
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#include <time.h>
#ifdef _OPENMP
#include <omp.h>
#endif
#if defined(__F16C__)
#include <immintrin.h>
#endif

/* ------------------------------------------------------------------ fp16 <-> fp32 */

/* IEEE binary16 -> binary32, exact (every half is representable). */
float oracle_f16_to_f32(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1fu;
    uint32_t man = h & 0x3ffu;
    uint32_t bits;
    if (exp == 0) {
        if (man == 0) {
            bits = sign;
        } else { /* subnormal: value = man * 2^-24, normalise */
            int shift = 0;
            while (!(man & 0x400u)) {
                man <<= 1;
                ++shift;
            }
            man &= 0x3ffu;
            bits = sign | ((uint32_t)(127 - 15 - shift + 1) << 23) | (man << 13);
        }
    } else if (exp == 31) {
        bits = sign | 0x7f800000u | (man << 13); /* inf / nan (payload kept) */
    } else {
        bits = sign | ((exp + 127 - 15) << 23) | (man << 13);
    }
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

/* IEEE binary32 -> binary16, round-to-nearest-even, overflow to inf, gradual underflow. */
uint16_t oracle_f32_to_f16(float f) {
    uint32_t x;
    memcpy(&x, &f, 4);
    uint16_t sign = (uint16_t)((x >> 16) & 0x8000u);
    uint32_t absx = x & 0x7fffffffu;
    if (absx >= 0x7f800000u) { /* inf or nan */
        if (absx == 0x7f800000u) return (uint16_t)(sign | 0x7c00u);
        uint16_t payload = (uint16_t)((absx >> 13) & 0x3ffu);
        return (uint16_t)(sign | 0x7c00u | 0x200u | payload); /* quiet the nan */
    }
    if (absx >= 0x477ff000u) return (uint16_t)(sign | 0x7c00u); /* >= 65520 rounds to inf */
    if (absx < 0x33000001u) return sign;                         /* <= 2^-25 rounds to zero */
    int32_t e = (int32_t)(absx >> 23) - 127;                     /* unbiased exponent */
    uint32_t m = (absx & 0x7fffffu) | 0x800000u;                 /* 24-bit significand */
    int shift;                                                   /* bits dropped from m */
    uint32_t base;
    if (e >= -14) { /* normal half: keep 11 bits (1 implicit + 10) */
        shift = 13;
        base = (uint32_t)(e + 15) << 10;
        m &= 0x7fffffu; /* implicit bit is carried by the exponent field */
    } else {        /* subnormal half: value = q * 2^-24, q = m * 2^(e+1) */
        shift = -e - 1;
        base = 0;
    }
    uint32_t q = m >> shift;
    uint32_t rem = m & ((1u << shift) - 1u);
    uint32_t half_ulp = 1u << (shift - 1);
    if (rem > half_ulp || (rem == half_ulp && (q & 1u))) ++q; /* carries propagate into exp */
    return (uint16_t)(sign | (uint16_t)(base + q));
}

/* Hardware conversions (F16C); present only so the tests can pin the software ones. */
int oracle_has_f16c(void) {
#if defined(__F16C__)
    return 1;
#else
    return 0;
#endif
}
float oracle_hw_f16_to_f32(uint16_t h) {
#if defined(__F16C__)
    return _cvtsh_ss(h);
#else
    return oracle_f16_to_f32(h);
#endif
}
uint16_t oracle_hw_f32_to_f16(float f) {
#if defined(__F16C__)
    return _cvtss_sh(f, _MM_FROUND_TO_NEAREST_INT | _MM_FROUND_NO_EXC);
#else
    return oracle_f32_to_f16(f);
#endif
}

void oracle_f16_to_f32_array(const uint16_t *src, float *dst, size_t n) {
    static float lut[65536];
    static int ready = 0;
#pragma omp critical(oracle_lut)
    {
        if (!ready) {
            for (uint32_t i = 0; i < 65536u; ++i) lut[i] = oracle_f16_to_f32((uint16_t)i);
            ready = 1;
        }
    }
#pragma omp parallel for schedule(static)
    for (size_t i = 0; i < n; ++i) dst[i] = lut[src[i]];
}

void oracle_f32_to_f16_array(const float *src, uint16_t *dst, size_t n) {
#pragma omp parallel for schedule(static)
    for (size_t i = 0; i < n; ++i) dst[i] = oracle_f32_to_f16(src[i]);
}

/* ------------------------------------------------------------------ seeded inputs */

/* Counter-based generator: element i of matrix `stream` under `seed` depends on nothing
 * else, so fills are order independent and identical on every host.  The reference seeds
 * from std::random_device (src/common/matrix.h:28-29) and therefore pins no values. */
static inline uint64_t splitmix64(uint64_t z) {
    z += 0x9e3779b97f4a7c15ull;
    z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ull;
    z = (z ^ (z >> 27)) * 0x94d049bb133111ebull;
    return z ^ (z >> 31);
}

uint64_t oracle_rng_u64(uint64_t seed, uint64_t stream, uint64_t index) {
    uint64_t key = splitmix64(seed ^ (stream * 0xd1342543de82ef95ull));
    return splitmix64(key + index * 0x9e3779b97f4a7c15ull);
}

/* 24 random bits -> [0,1) exactly representable in fp32. */
static inline float u24_to_unit(uint64_t r) { return (float)(r >> 40) * (1.0f / 16777216.0f); }

enum { ORACLE_DIST_UNIFORM = 0, ORACLE_DIST_NORMAL = 1, ORACLE_DIST_TERNARY = 2 };

/* dist 0: uniform [p0, p1)      (src/common/matrix.h:30-32 uses [-1, 1])
 * dist 1: normal(mean p0, sigma p1), Box-Muller in double on two independent 32-bit fields
 * dist 2: integers drawn uniformly from {-r..r}, r = (int)p1 (exact-arithmetic test inputs)
 * Values are rounded to fp16 round-to-nearest-even, as __float2half does. */
void oracle_fill(uint16_t *dst, size_t n, uint64_t seed, uint64_t stream, int dist, float p0, float p1) {
#pragma omp parallel for schedule(static)
    for (size_t i = 0; i < n; ++i) {
        uint64_t r = oracle_rng_u64(seed, stream, (uint64_t)i);
        float v;
        if (dist == ORACLE_DIST_UNIFORM) {
            v = p0 + (p1 - p0) * u24_to_unit(r);
        } else if (dist == ORACLE_DIST_NORMAL) {
            double u1 = ((double)(uint32_t)(r >> 32) + 1.0) * (1.0 / 4294967296.0); /* (0,1] */
            double u2 = (double)(uint32_t)r * (1.0 / 4294967296.0);                 /* [0,1) */
            double z = sqrt(-2.0 * log(u1)) * cos(6.283185307179586476925 * u2);
            v = (float)((double)p0 + (double)p1 * z);
        } else {
            int range = (int)p1;
            v = (float)((int)((r >> 33) % (uint64_t)(2 * range + 1)) - range);
        }
        dst[i] = oracle_f32_to_f16(v);
    }
}

/* ------------------------------------------------------------------ GEMM */

/* Plainest statement of the path: one dot product per output in double precision.
 * Follows src/simt_naive.cu:18-24 index for index; used on small shapes to pin the
 * blocked routine below.  Cd (optional) receives the unrounded double results. */
void oracle_hgemm_naive_f64(const uint16_t *A, const uint16_t *B, uint16_t *C, double *Cd, size_t M, size_t N,
                            size_t K) {
    for (size_t row = 0; row < M; ++row) {
        for (size_t col = 0; col < N; ++col) {
            double tmp = 0.0;
            for (size_t i = 0; i < K; ++i) {
                tmp += (double)oracle_f16_to_f32(A[row * K + i]) * (double)oracle_f16_to_f32(B[i + col * K]);
            }
            if (Cd) Cd[row * N + col] = tmp;
            if (C) C[row * N + col] = oracle_f32_to_f16((float)tmp);
        }
    }
}

/* Same loop with an fp32 accumulator in plain k order: the literal fp32-accumulate form of
 * src/simt_naive.cu:18-24. */
void oracle_hgemm_naive_f32(const uint16_t *A, const uint16_t *B, uint16_t *C, size_t M, size_t N, size_t K) {
    for (size_t row = 0; row < M; ++row) {
        for (size_t col = 0; col < N; ++col) {
            float tmp = 0.0f;
            for (size_t i = 0; i < K; ++i) {
                float p = oracle_f16_to_f32(A[row * K + i]) * oracle_f16_to_f32(B[i + col * K]);
                tmp += p;
            }
            C[row * N + col] = oracle_f32_to_f16(tmp);
        }
    }
}

/* Blocked, threaded fp32-accumulate GEMM on pre-converted fp32 operands.
 * Af: M x K row-major, Bf: N x K row-major (= the reference's column-major K x N),
 * Cf: M x N row-major fp32 results (not yet rounded to fp16).
 * Work is split over (MB x NB) blocks of C; inside a block K is walked in KC chunks and a
 * 4 x 4 register tile of 8-lane partial dot products does the arithmetic. */
typedef float v8f __attribute__((vector_size(32), aligned(4)));

#define OR_MB 64
#define OR_NB 64
#define OR_KC 512

static inline float hsum8(v8f v) { return ((v[0] + v[4]) + (v[1] + v[5])) + ((v[2] + v[6]) + (v[3] + v[7])); }

static void block_kernel(const float *Af, const float *Bf, float *acc /* OR_MB x OR_NB */, size_t m0, size_t mc,
                         size_t n0, size_t nc, size_t k0, size_t kc, size_t K) {
    size_t kv = kc & ~(size_t)7;
    for (size_t i = 0; i < mc; i += 4) {
        size_t ic = mc - i < 4 ? mc - i : 4;
        for (size_t j = 0; j < nc; j += 4) {
            size_t jc = nc - j < 4 ? nc - j : 4;
            if (ic == 4 && jc == 4) {
                const float *a0 = Af + (m0 + i) * K + k0, *a1 = a0 + K, *a2 = a1 + K, *a3 = a2 + K;
                const float *b0 = Bf + (n0 + j) * K + k0, *b1 = b0 + K, *b2 = b1 + K, *b3 = b2 + K;
                v8f c00 = {0}, c01 = {0}, c02 = {0}, c03 = {0}, c10 = {0}, c11 = {0}, c12 = {0}, c13 = {0};
                v8f c20 = {0}, c21 = {0}, c22 = {0}, c23 = {0}, c30 = {0}, c31 = {0}, c32 = {0}, c33 = {0};
                for (size_t k = 0; k < kv; k += 8) {
                    v8f x0 = *(const v8f *)(a0 + k), x1 = *(const v8f *)(a1 + k);
                    v8f x2 = *(const v8f *)(a2 + k), x3 = *(const v8f *)(a3 + k);
                    v8f y0 = *(const v8f *)(b0 + k), y1 = *(const v8f *)(b1 + k);
                    v8f y2 = *(const v8f *)(b2 + k), y3 = *(const v8f *)(b3 + k);
                    c00 += x0 * y0; c01 += x0 * y1; c02 += x0 * y2; c03 += x0 * y3;
                    c10 += x1 * y0; c11 += x1 * y1; c12 += x1 * y2; c13 += x1 * y3;
                    c20 += x2 * y0; c21 += x2 * y1; c22 += x2 * y2; c23 += x2 * y3;
                    c30 += x3 * y0; c31 += x3 * y1; c32 += x3 * y2; c33 += x3 * y3;
                }
                float *r0 = acc + (i + 0) * OR_NB + j, *r1 = r0 + OR_NB, *r2 = r1 + OR_NB, *r3 = r2 + OR_NB;
                r0[0] += hsum8(c00); r0[1] += hsum8(c01); r0[2] += hsum8(c02); r0[3] += hsum8(c03);
                r1[0] += hsum8(c10); r1[1] += hsum8(c11); r1[2] += hsum8(c12); r1[3] += hsum8(c13);
                r2[0] += hsum8(c20); r2[1] += hsum8(c21); r2[2] += hsum8(c22); r2[3] += hsum8(c23);
                r3[0] += hsum8(c30); r3[1] += hsum8(c31); r3[2] += hsum8(c32); r3[3] += hsum8(c33);
                for (size_t k = kv; k < kc; ++k) { /* K tail */
                    const float *ar[4] = {a0, a1, a2, a3};
                    const float *br[4] = {b0, b1, b2, b3};
                    for (int ii = 0; ii < 4; ++ii)
                        for (int jj = 0; jj < 4; ++jj) acc[(i + ii) * OR_NB + j + jj] += ar[ii][k] * br[jj][k];
                }
            } else { /* ragged edge of the block */
                for (size_t ii = 0; ii < ic; ++ii) {
                    for (size_t jj = 0; jj < jc; ++jj) {
                        const float *a = Af + (m0 + i + ii) * K + k0;
                        const float *b = Bf + (n0 + j + jj) * K + k0;
                        float s = 0.0f;
                        for (size_t k = 0; k < kc; ++k) s += a[k] * b[k];
                        acc[(i + ii) * OR_NB + j + jj] += s;
                    }
                }
            }
        }
    }
}

void oracle_sgemm_nt(const float *Af, const float *Bf, float *Cf, size_t M, size_t N, size_t K) {
    size_t mb = (M + OR_MB - 1) / OR_MB, nb = (N + OR_NB - 1) / OR_NB;
#pragma omp parallel
    {
        float *acc = (float *)malloc(sizeof(float) * OR_MB * OR_NB);
#pragma omp for schedule(dynamic, 1) collapse(2)
        for (size_t bi = 0; bi < mb; ++bi) {
            for (size_t bj = 0; bj < nb; ++bj) {
                size_t m0 = bi * OR_MB, n0 = bj * OR_NB;
                size_t mc = M - m0 < OR_MB ? M - m0 : OR_MB;
                size_t nc = N - n0 < OR_NB ? N - n0 : OR_NB;
                memset(acc, 0, sizeof(float) * OR_MB * OR_NB);
                for (size_t k0 = 0; k0 < K; k0 += OR_KC) {
                    size_t kc = K - k0 < OR_KC ? K - k0 : OR_KC;
                    block_kernel(Af, Bf, acc, m0, mc, n0, nc, k0, kc, K);
                }
                for (size_t i = 0; i < mc; ++i)
                    memcpy(Cf + (m0 + i) * N + n0, acc + i * OR_NB, sizeof(float) * nc);
            }
        }
        free(acc);
    }
}

/* The oracle proper: fp16 operands in the reference's layouts, fp32 accumulation, one
 * rounding to fp16.  Cf (optional, M*N floats) receives the unrounded fp32 results so a
 * caller can measure the error of another implementation against the pre-rounding value.
 * Returns 0, or -1 if scratch memory could not be allocated. */
int oracle_hgemm(const uint16_t *A, const uint16_t *B, uint16_t *C, float *Cf, size_t M, size_t N, size_t K) {
    float *Af = (float *)malloc(sizeof(float) * M * K);
    float *Bf = (float *)malloc(sizeof(float) * N * K);
    float *Ct = Cf ? Cf : (float *)malloc(sizeof(float) * M * N);
    if (!Af || !Bf || !Ct) {
        free(Af);
        free(Bf);
        if (!Cf) free(Ct);
        return -1;
    }
    oracle_f16_to_f32_array(A, Af, M * K);
    oracle_f16_to_f32_array(B, Bf, N * K);
    oracle_sgemm_nt(Af, Bf, Ct, M, N, K);
    if (C) oracle_f32_to_f16_array(Ct, C, M * N);
    free(Af);
    free(Bf);
    if (!Cf) free(Ct);
    return 0;
}

/* Rows [m0, m0+mc) of the product only (full N, full K): the sampled form used to check
 * and to time large shapes within a bounded CPU budget.  C_rows / Cf_rows are mc x N. */
int oracle_hgemm_rows(const uint16_t *A, const uint16_t *B, uint16_t *C_rows, float *Cf_rows, size_t m0, size_t mc,
                      size_t N, size_t K) {
    return oracle_hgemm(A + m0 * K, B, C_rows, Cf_rows, mc, N, K);
}

/* ------------------------------------------------------------------ checks and metrics */

/* Max and mean absolute difference of two fp16 arrays (src/common/matrix.h:102-111).
 * out[0]=max diff, out[1]=avg diff, out[2]=rms of `ref`, out[3]=count of non-finite
 * values in `got`, out[4]=index of the max diff. */
void oracle_diff(const uint16_t *got, const uint16_t *ref, size_t n, double *out) {
    double max_diff = 0.0, sum = 0.0, sq = 0.0, bad = 0.0;
    size_t arg = 0;
    for (size_t i = 0; i < n; ++i) {
        float g = oracle_f16_to_f32(got[i]), r = oracle_f16_to_f32(ref[i]);
        if (!isfinite(g)) {
            bad += 1.0;
            continue;
        }
        double d = fabs((double)g - (double)r);
        if (d > max_diff) {
            max_diff = d;
            arg = i;
        }
        sum += d;
        sq += (double)r * (double)r;
    }
    out[0] = max_diff;
    out[1] = n ? sum / (double)n : 0.0;
    out[2] = n ? sqrt(sq / (double)n) : 0.0;
    out[3] = bad;
    out[4] = (double)arg;
}

/* src/common/tester.h:96-97 */
double oracle_tflops(size_t M, size_t N, size_t K, double ms) {
    return (double)(M * N * K * 2) * 1e-12 / (ms * 1e-3);
}

int oracle_num_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

/* Wall-clock seconds of one oracle_sgemm_nt on already-converted operands (the CPU
 * baseline: conversion and allocation stay outside the timed region, as the GPU side keeps
 * its operands resident). */
double oracle_time_sgemm_nt(const float *Af, const float *Bf, float *Cf, size_t M, size_t N, size_t K) {
    struct timespec t0, t1;
    clock_gettime(CLOCK_MONOTONIC, &t0);
    oracle_sgemm_nt(Af, Bf, Cf, M, N, K);
    clock_gettime(CLOCK_MONOTONIC, &t1);
    return (double)(t1.tv_sec - t0.tv_sec) + 1e-9 * (double)(t1.tv_nsec - t0.tv_nsec);
}
