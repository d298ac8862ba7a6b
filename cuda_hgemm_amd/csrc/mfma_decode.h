// Decode-shaped product, M <= 32: a handful of rows of A against all of B.
//
// The work is reading B (N x K halves) from HBM once, so the kernel is built like a
// streaming read, not like a GEMM: no LDS staging, no barrier in the loop.  A workgroup
// owns BN rows of B (BN columns of C); each of its waves owns one slice of K and loads MFMA
// operands straight from global memory in the operand layout (lane l: row l % 16, eight
// consecutive k at chunk l / 16 of the 32-wide step -- 64 contiguous bytes per row and
// instruction), a group of steps ahead of the MFMAs that consume them.  The rows of A are
// few and hot in L1/L2; rows beyond M are redirected to row M-1 and never stored.  At the
// end the waves add their fp32 partial sums through LDS in wave order, so the result does
// not depend on scheduling and is bit-identical from run to run, and one kernel does the
// whole product (the split-K kernel needs a second launch for its reduction).
//
// The reference has no kernel for these shapes: its tiled kernels need M % 256 == 0
// (src/mma/mma_async_stage4.cu:64-66,93-94).
#pragma once

#include "mfma_tiled.h"

namespace hgemm {

constexpr int DECODE_MAX_WAVES = 8;   // K slices per workgroup

template <int BM, int BN>
__global__ void __launch_bounds__(DECODE_MAX_WAVES * 64)
    hgemm_decode_kernel(const half_t *__restrict__ A, const half_t *__restrict__ B, half_t *__restrict__ C, int M,
                        int N, int K, int k_per_wave) {
    constexpr int TM = BM / 16, TN = BN / 16;
    // 32-wide k steps whose loads are issued together: two buffers of G * (TM + TN) operand
    // fragments stay within 128 VGPRs
    constexpr int G = 16 / (TM + TN) >= 8 ? 8 : (16 / (TM + TN) >= 4 ? 4 : 16 / (TM + TN));
    __shared__ __attribute__((aligned(16))) float partial[DECODE_MAX_WAVES][BM][BN];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), waves = blockDim.x >> 6;
    const int n0 = blockIdx.x * BN;
    const int row = lane & 15, kchunk = (lane >> 4) * 8;
    const int k_begin = wave * k_per_wave;

    const half_t *a_ptr[TM];
    const half_t *b_ptr[TN];
#pragma unroll
    for (int i = 0; i < TM; ++i) {
        int m = i * 16 + row;
        m = m < M ? m : M - 1;
        a_ptr[i] = A + (size_t)m * K + k_begin + kchunk;
    }
#pragma unroll
    for (int j = 0; j < TN; ++j) b_ptr[j] = B + (size_t)(n0 + j * 16 + row) * K + k_begin + kchunk;

    floatx4 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int r = 0; r < 4; ++r) acc[i][j][r] = 0.0f;

    half8 af[2][G][TM], bf[2][G][TN];
    auto fetch = [&](int buf, int k) {
#pragma unroll
        for (int g = 0; g < G; ++g) {
#pragma unroll
            for (int j = 0; j < TN; ++j) bf[buf][g][j] = *reinterpret_cast<const half8 *>(b_ptr[j] + k + g * 32);
#pragma unroll
            for (int i = 0; i < TM; ++i) af[buf][g][i] = *reinterpret_cast<const half8 *>(a_ptr[i] + k + g * 32);
        }
    };
    auto multiply = [&](int buf) {
#pragma unroll
        for (int g = 0; g < G; ++g)
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(bf[buf][g][j], af[buf][g][i], acc[i][j], 0, 0, 0);
    };

    // groups of G steps, the next group's loads in flight while this one is multiplied
    const int groups = k_per_wave / (32 * G);
    if (groups > 0) fetch(0, 0);
    for (int grp = 0; grp < groups; grp += 2) {
        if (grp + 1 < groups) fetch(1, (grp + 1) * 32 * G);
        multiply(0);
        if (grp + 1 < groups) {
            if (grp + 2 < groups) fetch(0, (grp + 2) * 32 * G);
            multiply(1);
        }
    }
    // steps left over when the slice is not a whole number of groups
    for (int k = groups * 32 * G; k < k_per_wave; k += 32) {
        half8 a1[TM], b1[TN];
#pragma unroll
        for (int j = 0; j < TN; ++j) b1[j] = *reinterpret_cast<const half8 *>(b_ptr[j] + k);
#pragma unroll
        for (int i = 0; i < TM; ++i) a1[i] = *reinterpret_cast<const half8 *>(a_ptr[i] + k);
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
                acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(b1[j], a1[i], acc[i][j], 0, 0, 0);
    }

    // Operands were swapped in the MFMA: a lane holds four consecutive n (at 4 * (lane / 16))
    // of row lane % 16 of each 16x16 tile.
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
            *reinterpret_cast<floatx4 *>(&partial[wave][i * 16 + row][j * 16 + (lane >> 4) * 4]) = acc[i][j];
    __syncthreads();
    // slices are added in wave order by whichever thread owns the four outputs
    for (int q = tid; q < BM * BN / 4; q += blockDim.x) {
        const int m = q / (BN / 4), c = (q % (BN / 4)) * 4;
        if (m >= M) continue;
        floatx4 s = *reinterpret_cast<const floatx4 *>(&partial[0][m][c]);
        for (int w = 1; w < waves; ++w) s += *reinterpret_cast<const floatx4 *>(&partial[w][m][c]);
        half4 v;
#pragma unroll
        for (int r = 0; r < 4; ++r) v[r] = (half_t)s[r];
        *reinterpret_cast<half4 *>(C + (size_t)m * N + n0 + c) = v;
    }
}

// M <= 32, N a multiple of 32, K a multiple of 256 (every wave gets whole 32-wide steps for
// any of the slice counts below).
inline bool decode_supports(size_t M, size_t N, size_t K) {
    return M >= 1 && M <= 32 && N > 0 && N % 32 == 0 && K > 0 && K % 256 == 0;
}

// Column tile and K slices per workgroup, from timing the candidates on N = 4096 and 28672
// (K = 4096, operands rotated so they stream from HBM): a wave should own about 1024 of K,
// less when N alone gives too few workgroups to keep every CU streaming; 32-column tiles
// (A is re-read per column tile) only pay once M > 4 and N provides plenty of them.
inline void decode_plan(size_t M, size_t N, size_t K, size_t cus, int *bn, int *waves) {
    *bn = (M > 4 && N / 32 >= 2 * cus) ? 32 : 16;
    const size_t tiles = N / (size_t)*bn;
    int w = 1;
    auto can_double = [&] { return w < DECODE_MAX_WAVES && K % ((size_t)w * 2 * 32) == 0 && K / (w * 2) >= 256; };
    while (K / w > 1024 && can_double()) w *= 2;
    while (tiles * w < 8 * cus && can_double()) w *= 2;
    *waves = w;
}

template <int BM, int BN>
void launch_decode_tile(const void *A, const void *B, void *C, size_t M, size_t N, size_t K, int waves) {
    hgemm_decode_kernel<BM, BN><<<dim3((unsigned)(N / BN)), dim3(waves * 64), 0, nullptr>>>(
        reinterpret_cast<const half_t *>(A), reinterpret_cast<const half_t *>(B), reinterpret_cast<half_t *>(C), (int)M,
        (int)N, (int)K, (int)(K / (size_t)waves));
    HGEMM_CHECK_HIP_ERROR(hipGetLastError());
}

inline void launch_decode(const void *A, const void *B, void *C, size_t M, size_t N, size_t K, int bn, int waves) {
    check_operands(A, B, C, M, N, K);
    HGEMM_CHECK_MSG(decode_supports(M, N, K), "decode kernel needs M <= 32, N %% 32 == 0, K %% 256 == 0 (got M=%zu N=%zu K=%zu)",
                    M, N, K);
    HGEMM_CHECK(waves >= 1 && waves <= DECODE_MAX_WAVES && K % ((size_t)waves * 32) == 0 &&
                (bn == 16 || bn == 32 || bn == 64) && N % (size_t)bn == 0);
    if (M <= 16) {
        if (bn == 16)
            launch_decode_tile<16, 16>(A, B, C, M, N, K, waves);
        else if (bn == 32)
            launch_decode_tile<16, 32>(A, B, C, M, N, K, waves);
        else
            launch_decode_tile<16, 64>(A, B, C, M, N, K, waves);
    } else {
        if (bn == 16)
            launch_decode_tile<32, 16>(A, B, C, M, N, K, waves);
        else if (bn == 32)
            launch_decode_tile<32, 32>(A, B, C, M, N, K, waves);
        else
            launch_decode_tile<32, 64>(A, B, C, M, N, K, waves);
    }
}

}  // namespace hgemm
