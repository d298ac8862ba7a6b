// Decode-shaped product, M <= 128, through per-wave LDS rings.
//
// Like the streaming decode kernel, a workgroup owns 16 rows of B (16 columns of C), each of
// its waves owns one slice of K, there is no barrier in the loop and the waves add their fp32
// partial sums through LDS in wave order (one launch, bit-identical from run to run).  What
// differs is how operands travel.  Loading MFMA operands straight from global memory makes
// every 16-lane quarter of a load touch 16 different rows, 16 bytes of each; the vector
// memory path then handles one 16-byte piece per cache-line look-up and a CU streams at a
// quarter of its rate, which is what the rows of A (re-read by every workgroup through L2)
// cost: 8.0 us at M = 1 but 10.3 us at M = 16 for N = K = 4096.  Here a wave copies
// 64-wide K chunks of its 16 rows of A and 16 rows of B with direct-to-LDS loads whose lanes
// cover eight rows x 128 contiguous bytes per instruction, into a ring of its own, and reads
// the operands back with ds_read_b128.  The ring belongs to one wave, so the only
// synchronisation is the wave's own vmcnt wait (copies complete in order) and an lgkmcnt(0)
// before a slot is refilled.  N = K = 4096: 7.6 / 8.0 / 8.3 us for M = 1 / 8 / 16.  With two,
// four or eight 16-row tiles of A per wave (M <= 32, 64, 128) the kernel still saves the
// split-K kernel's second launch, which pays while K is short (K = 1024, N = 4096, M = 32:
// 6.5 -> 4.8 us; K = 512, N = 4096, M = 128: 11.0 -> 6.1 us).
//
// LDS layout of one chunk: 16 TM rows x 128 bytes of A, then 16 rows of B.  A direct-to-LDS
// load writes lane l's 16 bytes at byte 16 * l of a 1 KB block, so block h holds rows
// 8h ... 8h+7 and the 16-byte piece c of row r is stored at position c ^ ((r >> 1) & 7) of
// its row (the swizzle is applied to the global address a lane reads): the 16 lanes of one
// ds_read_b128 quarter (rows 0 ... 15, same c) then hit 16 different 16-byte bank groups.
//
// The reference has no kernel for these shapes: its tiled kernels need M % 256 == 0
// (src/mma/mma_async_stage4.cu:64-66,93-94).
#pragma once

#include "mfma_tiled.h"

namespace hgemm {

constexpr int RING_MAX_WAVES = 8;  // K slices per workgroup

// TM: 16-row tiles of A per wave; STAGES: chunks in a wave's ring, STAGES - 1 in flight and one being read
template <int TM, int STAGES>
struct RingConfig {
    static constexpr int A_BYTES = TM * 2048;                   // 16 TM rows of 64 halves
    static constexpr int CHUNK_BYTES = A_BYTES + 2048;          // + 16 rows of B
    static constexpr int RING_BYTES = STAGES * CHUNK_BYTES;     // per wave
    static constexpr int COPIES = 2 * TM + 2;                   // per chunk and wave
    static_assert((STAGES - 2) * COPIES <= 63 && RING_BYTES >= TM * 1024,
                  "wait count range; the ring takes the wave's partial sums");
};

// STREAM_B: B's copies carry the non-temporal hint (every byte of B is read once; the launcher sets it from 48 MB of B on,
// the threshold the split-K kernel uses for the same hint).
template <int TM, int STAGES, bool STREAM_B = false>
__global__ void __launch_bounds__(RING_MAX_WAVES * 64)
    hgemm_decode_ring_kernel(const half_t *__restrict__ A, const half_t *__restrict__ B, half_t *__restrict__ C, int M,
                             int N, int K, int k_per_wave) {
    using Cfg = RingConfig<TM, STAGES>;
    constexpr int L = Cfg::COPIES, A_BYTES = Cfg::A_BYTES, RING_CHUNK_BYTES = Cfg::CHUNK_BYTES, RING_BYTES = Cfg::RING_BYTES;
    extern __shared__ __attribute__((aligned(1024))) unsigned char lds[];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), waves = blockDim.x >> 6;
    const int n0 = blockIdx.x * 16;
    const int k_begin = wave * k_per_wave;

    // ---- copies: lane l of instruction h fetches piece (l % 8) ^ swizzle of row 8h + l / 8; rows of A beyond M are
    // redirected to row M-1 and never stored
    const int copy_row = lane >> 3, copy_pos = lane & 7;
    const half_t *a_src[2 * TM], *b_src[2];
#pragma unroll
    for (int h = 0; h < 2 * TM; ++h) {
        const int r = copy_row + 8 * h;
        const int piece = copy_pos ^ ((r >> 1) & 7);
        const int m = r < M ? r : M - 1;
        a_src[h] = A + (size_t)m * K + k_begin + piece * 8;
        if (h < 2) b_src[h] = B + (size_t)(n0 + r) * K + k_begin + piece * 8;
    }
    const uint32_t ring_addr = (uint32_t)(uintptr_t)lds + wave * RING_BYTES;
    auto fetch = [&](int kt, int slot) {
        const uint32_t base = ring_addr + slot * RING_CHUNK_BYTES;
#pragma unroll
        for (int h = 0; h < 2 * TM; ++h) dma_load16(a_src[h] + kt * 64, base + h * 1024);
        if constexpr (STREAM_B) {
            dma_load16_streaming(b_src[0] + kt * 64, base + A_BYTES);
            dma_load16_streaming(b_src[1] + kt * 64, base + A_BYTES + 1024);
        } else {
            dma_load16(b_src[0] + kt * 64, base + A_BYTES);
            dma_load16(b_src[1] + kt * 64, base + A_BYTES + 1024);
        }
    };

    // ---- operands of the two 32-wide steps of a chunk: lane l holds row l % 16 (of each 16-row tile), pieces l / 16
    // and 4 + l / 16
    const int row = lane & 15, quarter = lane >> 4;
    const uint32_t step0 = row * 128 + ((quarter ^ ((row >> 1) & 7)) << 4);
    const uint32_t step1 = row * 128 + (((4 + quarter) ^ ((row >> 1) & 7)) << 4);

    floatx4 acc[TM];
#pragma unroll
    for (int i = 0; i < TM; ++i) acc[i] = floatx4{0.0f, 0.0f, 0.0f, 0.0f};
    const int num_k = k_per_wave / 64;
#pragma unroll
    for (int s = 0; s < STAGES - 1; ++s)
        if (s < num_k) fetch(s, s);
    int cur = 0, fill = STAGES - 1;
    for (int kt = 0; kt < num_k; ++kt) {
        if (num_k - 1 - kt >= STAGES - 2)
            wait_vmcnt<(STAGES - 2) * L>();
        else
            wait_vmcnt<0>();
        wave_lds_exchange_point();  // the reads below stay behind the wait
        const unsigned char *chunk = lds + wave * RING_BYTES + cur * RING_CHUNK_BYTES;
        half8 a0[TM], a1[TM];
#pragma unroll
        for (int i = 0; i < TM; ++i) {
            a0[i] = *reinterpret_cast<const half8 *>(chunk + i * 2048 + step0);
            a1[i] = *reinterpret_cast<const half8 *>(chunk + i * 2048 + step1);
        }
        const half8 b0 = *reinterpret_cast<const half8 *>(chunk + A_BYTES + step0);
        const half8 b1 = *reinterpret_cast<const half8 *>(chunk + A_BYTES + step1);
        // the slot refilled next is the one read in the previous iteration; with this iteration's reads returned too,
        // no read of this wave is outstanding when the copy is issued
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        if (kt + STAGES - 1 < num_k) fetch(kt + STAGES - 1, fill);
#pragma unroll
        for (int i = 0; i < TM; ++i) {
            acc[i] = __builtin_amdgcn_mfma_f32_16x16x32_f16(b0, a0[i], acc[i], 0, 0, 0);
            acc[i] = __builtin_amdgcn_mfma_f32_16x16x32_f16(b1, a1[i], acc[i], 0, 0, 0);
        }
        cur = (cur + 1 == STAGES) ? 0 : cur + 1;
        fill = (fill + 1 == STAGES) ? 0 : fill + 1;
    }

    // Operands were swapped in the MFMA: a lane holds four consecutive n (at 4 * (lane / 16)) of row lane % 16.  The
    // wave's ring is free (every copy has landed, every read has returned) and takes its 16 TM x 16 partial sums.
    float *partial = reinterpret_cast<float *>(lds + wave * RING_BYTES);
#pragma unroll
    for (int i = 0; i < TM; ++i) *reinterpret_cast<floatx4 *>(partial + (i * 16 + row) * 16 + quarter * 4) = acc[i];
    __syncthreads();
    // slices are added in wave order by whichever thread owns the four outputs
    for (int t = tid; t < TM * 64; t += blockDim.x) {
        const int m = t >> 2, c = (t & 3) * 4;
        if (m >= M) continue;
        floatx4 s = *reinterpret_cast<const floatx4 *>(reinterpret_cast<const float *>(lds) + m * 16 + c);
        for (int w = 1; w < waves; ++w)
            s += *reinterpret_cast<const floatx4 *>(reinterpret_cast<const float *>(lds + w * RING_BYTES) + m * 16 + c);
        half4 v;
#pragma unroll
        for (int r = 0; r < 4; ++r) v[r] = (half_t)s[r];
        *reinterpret_cast<half4 *>(C + (size_t)m * N + n0 + c) = v;
    }
}

// M <= 128, N a multiple of 16, K a multiple of 128 (two waves get whole 64-wide chunks).
inline bool decode_ring_supports(size_t M, size_t N, size_t K) {
    return M >= 1 && M <= 128 && N > 0 && N % 16 == 0 && K > 0 && K % 128 == 0 && N <= ((size_t)1 << 31) / 16;
}

inline int decode_ring_max_waves(size_t M);

// K slices per workgroup, from timing 2, 4 and 8 on K = 1024 ... 8192 against N = 1024 ... 14336 (operands rotated
// so they stream from HBM): a wave should own 640 ... 1280 of K (eight waves' rings leave room for one workgroup per
// CU, four waves' for two), but there should be four waves unless N alone provides two or more workgroups per CU.
inline int decode_ring_waves(size_t M, size_t N, size_t K, size_t cus) {
    if (M > 64) return N / 16 <= cus ? 2 : 1;  // eight row tiles of A: two waves only while N gives one workgroup per CU
    int w = 2;
    while (w < decode_ring_max_waves(M) && K / (size_t)w > 1280) w *= 2;
    if (w < 4 && N / 16 < 2 * cus) w = 4;
    while (w > 2 && K % ((size_t)w * 64) != 0) w /= 2;
    return w;
}

template <int TM, int STAGES>
void launch_decode_ring_tile(const void *A, const void *B, void *C, size_t M, size_t N, size_t K, int waves) {
    using Cfg = RingConfig<TM, STAGES>;
    HGEMM_CHECK((size_t)waves * Cfg::RING_BYTES <= 160 * 1024);
    static bool configured = [] {
        HGEMM_CHECK_HIP_ERROR(hipFuncSetAttribute(reinterpret_cast<const void *>(&hgemm_decode_ring_kernel<TM, STAGES, false>),
                                                  hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
        HGEMM_CHECK_HIP_ERROR(hipFuncSetAttribute(reinterpret_cast<const void *>(&hgemm_decode_ring_kernel<TM, STAGES, true>),
                                                  hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
        return true;
    }();
    (void)configured;
    auto kernel = N * K >= ((size_t)24 << 20) ? &hgemm_decode_ring_kernel<TM, STAGES, true>
                                              : &hgemm_decode_ring_kernel<TM, STAGES, false>;
    kernel<<<dim3((unsigned)(N / 16)), dim3(waves * 64), (size_t)waves * Cfg::RING_BYTES, nullptr>>>(
        reinterpret_cast<const half_t *>(A), reinterpret_cast<const half_t *>(B), reinterpret_cast<half_t *>(C), (int)M,
        (int)N, (int)K, (int)(K / (size_t)waves));
    HGEMM_CHECK_HIP_ERROR(hipGetLastError());
}

// Rings of four chunks for one or two row tiles of A (16 and 24 KB per wave), of three for four and eight (30 and
// 54 KB): up to eight, four, four and two waves fit the 160 KB of a CU.
inline int decode_ring_max_waves(size_t M) { return M <= 16 ? RING_MAX_WAVES : M <= 64 ? 4 : 2; }

inline void launch_decode_ring(const void *A, const void *B, void *C, size_t M, size_t N, size_t K, int waves) {
    check_operands(A, B, C, M, N, K);
    HGEMM_CHECK_MSG(decode_ring_supports(M, N, K), "ring decode kernel needs M <= 128, N %% 16 == 0, K %% 128 == 0 (got M=%zu N=%zu K=%zu)",
                    M, N, K);
    HGEMM_CHECK(waves >= 1 && waves <= decode_ring_max_waves(M) && K % ((size_t)waves * 64) == 0);
    if (M <= 16)
        launch_decode_ring_tile<1, 4>(A, B, C, M, N, K, waves);
    else if (M <= 32)
        launch_decode_ring_tile<2, 4>(A, B, C, M, N, K, waves);
    else if (M <= 64)
        launch_decode_ring_tile<4, 3>(A, B, C, M, N, K, waves);
    else
        launch_decode_ring_tile<8, 3>(A, B, C, M, N, K, waves);
}

}  // namespace hgemm
