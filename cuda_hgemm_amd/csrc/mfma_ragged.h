// MFMA kernel for shapes nothing else tiles: any M, N, K >= 1.
//
// 128x128x32 tile, 4 waves (2x2), 64x64 wave tiles on v_mfma_f32_32x32x16_f16, operands
// staged global -> registers -> LDS so that every element can be guarded: rows beyond the
// matrix and k beyond K are written to LDS as zeros, outputs beyond the matrix are not
// stored.  When K is a multiple of 8 the rows of A and B are 16-byte aligned and a thread
// moves 16 bytes at a time; otherwise it gathers the eight halves one by one.  Two LDS
// buffers: the registers hold chunk kt+1 while chunk kt is multiplied.
//
// The reference has no such path: its kernels read and write out of bounds unless
// M % 256 == 0, N % 128 == 0, K % 32 == 0 (src/mma/mma_async_stage4.cu:64-66,93-94,612-616).
#pragma once

#include "mfma_tiled.h"

namespace hgemm {

struct RaggedConfig {
    static constexpr int BM = 128, BN = 128, BK = 32, THREADS = 256;
    static constexpr int ROW_BYTES = BK * 2 + 16;  // 16 bytes of padding against bank conflicts
    static constexpr int A_BYTES = BM * ROW_BYTES, STAGE_BYTES = 2 * A_BYTES, LDS_BYTES = 2 * STAGE_BYTES;
    static constexpr int CHUNKS = BM * (BK / 8);   // 16-byte chunks per operand tile
    static constexpr int ITERS = CHUNKS / THREADS;
};

template <bool ALIGNED>
__global__ void __launch_bounds__(RaggedConfig::THREADS)
    hgemm_ragged_kernel(const half_t *__restrict__ A, const half_t *__restrict__ B, half_t *__restrict__ C, int M,
                        int N, int K) {
    using Cfg = RaggedConfig;
    constexpr int BK = Cfg::BK, ROW_BYTES = Cfg::ROW_BYTES, ITERS = Cfg::ITERS;
    __shared__ __attribute__((aligned(16))) unsigned char lds[Cfg::LDS_BYTES];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    // one-dimensional grid, row-major over the tiles of C: no 65535 limit on either dimension
    const int tiles_n = (N + Cfg::BN - 1) / Cfg::BN;
    const int m0 = (int)(blockIdx.x / tiles_n) * Cfg::BM, n0 = (int)(blockIdx.x % tiles_n) * Cfg::BN;
    const int num_k = (K + BK - 1) / BK;

    // eight consecutive k of one row, zero where the row or k is outside the matrix
    auto fetch = [&](const half_t *__restrict__ base, int row, int rows, int k) -> half8 {
        half8 v;
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] = (half_t)0.0f;
        if (row >= rows || k >= K) return v;
        const half_t *src = base + (size_t)row * K + k;
        if constexpr (ALIGNED) {
            v = *reinterpret_cast<const half8 *>(src);  // K % 8 == 0: the chunk is whole and aligned
        } else {
#pragma unroll
            for (int e = 0; e < 8; ++e)
                if (k + e < K) v[e] = src[e];
        }
        return v;
    };

    half8 ra[ITERS], rb[ITERS];
    auto global_fetch = [&](int kt) {
#pragma unroll
        for (int it = 0; it < ITERS; ++it) {
            const int c = tid + it * Cfg::THREADS, row = c >> 2, k = kt * BK + (c & 3) * 8;
            ra[it] = fetch(A, m0 + row, M, k);
            rb[it] = fetch(B, n0 + row, N, k);
        }
    };
    auto lds_commit = [&](int stage) {
        unsigned char *sa = lds + stage * Cfg::STAGE_BYTES;
#pragma unroll
        for (int it = 0; it < ITERS; ++it) {
            const int c = tid + it * Cfg::THREADS;
            const int off = (c >> 2) * ROW_BYTES + (c & 3) * 16;
            *reinterpret_cast<half8 *>(sa + off) = ra[it];
            *reinterpret_cast<half8 *>(sa + Cfg::A_BYTES + off) = rb[it];
        }
    };

    floatx16 acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

    // lane l supplies row l % 32, k chunk l / 32 of each 16-wide MFMA step
    const int frag_off = (lane & 31) * ROW_BYTES + (lane >> 5) * 16;
    auto compute = [&](int stage) {
        const unsigned char *sa = lds + stage * Cfg::STAGE_BYTES + wm * 64 * ROW_BYTES + frag_off;
        const unsigned char *sb = lds + stage * Cfg::STAGE_BYTES + Cfg::A_BYTES + wn * 64 * ROW_BYTES + frag_off;
#pragma unroll
        for (int kk = 0; kk < BK / 16; ++kk) {
            half8 af[2], bf[2];
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                af[i] = *reinterpret_cast<const half8 *>(sa + i * 32 * ROW_BYTES + kk * 32);
                bf[i] = *reinterpret_cast<const half8 *>(sb + i * 32 * ROW_BYTES + kk * 32);
            }
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(bf[j], af[i], acc[i][j], 0, 0, 0);
        }
    };

    global_fetch(0);
    lds_commit(0);
    __syncthreads();
    for (int kt = 0; kt < num_k; ++kt) {
        const int cur = kt & 1;
        if (kt + 1 < num_k) global_fetch(kt + 1);
        compute(cur);
        if (kt + 1 < num_k) lds_commit(cur ^ 1);  // last read of that buffer was before the previous barrier
        __syncthreads();
    }

    // Operands were swapped in the MFMA: a lane holds, for row l % 32 of a 32x32 tile,
    // groups of four consecutive n at 8*g + 4*(l / 32).
    const bool packed = (N & 3) == 0;  // then a group is wholly inside or outside and 8-byte aligned
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int m = m0 + wm * 64 + i * 32 + (lane & 31);
        if (m >= M) continue;
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int n = n0 + wn * 64 + j * 32 + g * 8 + (lane >> 5) * 4;
                half_t *dst = C + (size_t)m * N + n;
                if (packed) {
                    if (n < N) {
                        half4 v;
#pragma unroll
                        for (int r = 0; r < 4; ++r) v[r] = (half_t)acc[i][j][g * 4 + r];
                        *reinterpret_cast<half4 *>(dst) = v;
                    }
                } else {
#pragma unroll
                    for (int r = 0; r < 4; ++r)
                        if (n + r < N) dst[r] = (half_t)acc[i][j][g * 4 + r];
                }
            }
    }
}

inline void launch_ragged(const void *A, const void *B, void *C, size_t M, size_t N, size_t K) {
    check_operands(A, B, C, M, N, K);
    const dim3 grid((unsigned)(div_ceil(N, (size_t)RaggedConfig::BN) * div_ceil(M, (size_t)RaggedConfig::BM)));
    const half_t *a = reinterpret_cast<const half_t *>(A), *b = reinterpret_cast<const half_t *>(B);
    half_t *c = reinterpret_cast<half_t *>(C);
    if (K % 8 == 0)
        hgemm_ragged_kernel<true><<<grid, dim3(RaggedConfig::THREADS), 0, nullptr>>>(a, b, c, (int)M, (int)N, (int)K);
    else
        hgemm_ragged_kernel<false><<<grid, dim3(RaggedConfig::THREADS), 0, nullptr>>>(a, b, c, (int)M, (int)N, (int)K);
    HGEMM_CHECK_HIP_ERROR(hipGetLastError());
}

}  // namespace hgemm
