// Decode-shaped product, M <= 32, against a B with many more 16-column tiles than the chip has CUs: the rows of A stay in
// registers.
//
// The ring decode kernel copies a wave's share of A anew for every 16 columns of C.  The copies hit L2, but from nine
// rows of A on they are as many bytes into the CU as B's (M = 16, N = 28672, K = 4096: 39.6 us where M = 8, whose
// duplicate rows cost nothing, takes 35.8).  Here a workgroup is persistent: it loads its waves' K slices of A once, in
// MFMA operand layout, straight into registers (4 VGPRs per 32 of K and 16-row tile), and then walks over column tiles
// blockIdx.x, blockIdx.x + gridDim.x, ...  Only B moves in the loop: 64-wide chunks of the tile's 16 rows of B,
// direct-to-LDS into a ring per wave that never drains at a tile boundary (the copies of the next tile's first chunks
// are issued during the current tile's last), read back with ds_read_b128.  As in the ring kernel a wave owns a K slice,
// there is no barrier inside a tile, and the waves' fp32 partial sums are added through LDS in wave order: one launch,
// bit-identical from run to run.
//
// The reference has no kernel for these shapes: its tiled kernels need M % 256 == 0
// (src/mma/mma_async_stage4.cu:64-66,93-94).
#pragma once

#include "mfma_pipelined.h"

namespace hgemm {

constexpr int RESIDENT_STAGES = 4;        // chunks in a wave's ring: three in flight, one being read
constexpr int RESIDENT_SLOT_BYTES = 2048;  // 16 rows of B x 64 halves
constexpr int RESIDENT_RING_BYTES = RESIDENT_STAGES * RESIDENT_SLOT_BYTES;

constexpr size_t resident_lds_bytes(int tm, int waves) {
    return (size_t)waves * RESIDENT_RING_BYTES + 2 * (size_t)waves * tm * 1024;  // rings, two sets of partial sums
}

// TM: 16-row tiles of A; CHUNKS: 64-wide chunks of K per wave (K = waves x CHUNKS x 64), a multiple of the ring's
// length so that a chunk's slot does not depend on the tile; STREAM_B: B's copies carry the non-temporal hint.
template <int TM, int CHUNKS, bool STREAM_B>
__global__ void __launch_bounds__(512)
    hgemm_decode_resident_kernel(const half_t *__restrict__ A, const half_t *__restrict__ B, half_t *__restrict__ C, int M,
                                 int N, int K, int tiles) {
    constexpr int STAGES = RESIDENT_STAGES, SLOT = RESIDENT_SLOT_BYTES, RING = RESIDENT_RING_BYTES;
    static_assert(CHUNKS % STAGES == 0 && CHUNKS >= STAGES, "a chunk's ring slot must not depend on the tile");
    static_assert(TM * CHUNKS * 8 <= 192, "A's registers");
    extern __shared__ __attribute__((aligned(1024))) unsigned char lds[];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), waves = blockDim.x >> 6;
    const int k_begin = wave * (CHUNKS * 64);

    // ---- B's copies: lane l of instruction h fetches piece (l % 8) ^ swizzle of row 8h + l / 8 of the tile
    const int copy_row = lane >> 3, copy_pos = lane & 7;
    size_t b_off[2];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        const int r = copy_row + 8 * h;
        b_off[h] = (size_t)r * K + k_begin + ((copy_pos ^ ((r >> 1) & 7)) << 3);
    }
    const uint32_t ring_addr = (uint32_t)(uintptr_t)lds + wave * RING;
    auto fetch = [&](const half_t *tile_rows, int kt, int slot) {
        const uint32_t base = ring_addr + slot * SLOT;
        if constexpr (STREAM_B) {
            dma_load16_streaming(tile_rows + b_off[0] + kt * 64, base);
            dma_load16_streaming(tile_rows + b_off[1] + kt * 64, base + 1024);
        } else {
            dma_load16(tile_rows + b_off[0] + kt * 64, base);
            dma_load16(tile_rows + b_off[1] + kt * 64, base + 1024);
        }
    };

    int tile = blockIdx.x;  // the launcher starts no workgroup without a tile
    const half_t *rows = B + (size_t)tile * 16 * K;
#pragma unroll
    for (int s = 0; s < STAGES - 1; ++s) fetch(rows, s, s);

    // ---- A, once: lane l holds row l % 16 of each 16-row tile and, of every 32 of K, the eight halves at 8 (l / 16);
    // rows beyond M repeat row M-1 and are never stored
    const int row = lane & 15, quarter = lane >> 4;
    half8 a[TM][CHUNKS][2];
#pragma unroll
    for (int i = 0; i < TM; ++i) {
        const int m = i * 16 + row < M ? i * 16 + row : M - 1;
        const half_t *src = A + (size_t)m * K + k_begin + quarter * 8;
#pragma unroll
        for (int kt = 0; kt < CHUNKS; ++kt) {
            a[i][kt][0] = *reinterpret_cast<const half8 *>(src + kt * 64);
            a[i][kt][1] = *reinterpret_cast<const half8 *>(src + kt * 64 + 32);
        }
    }

    const uint32_t step0 = row * 128 + ((quarter ^ ((row >> 1) & 7)) << 4);
    const uint32_t step1 = row * 128 + (((4 + quarter) ^ ((row >> 1) & 7)) << 4);
    const unsigned char *ring = lds + wave * RING;
    float *sums = reinterpret_cast<float *>(lds + waves * RING);  // [2][waves][16 TM][16]
    int parity = 0;

    for (;;) {
        const int next = tile + (int)gridDim.x;
        const bool has_next = next < tiles;
        const half_t *next_rows = B + (size_t)(has_next ? next : tile) * 16 * K;
        floatx4 acc[TM];
#pragma unroll
        for (int i = 0; i < TM; ++i) acc[i] = floatx4{0.0f, 0.0f, 0.0f, 0.0f};

        static_for<CHUNKS>([&](auto kt_c) {
            constexpr int kt = decltype(kt_c)::value;
            // younger than chunk kt's two copies are those of the chunks after it that have been issued: two chunks,
            // fewer at the end of the last tile
            if (kt + 2 < CHUNKS || has_next)
                wait_vmcnt<4>();
            else if (kt + 1 < CHUNKS)
                wait_vmcnt<2>();
            else
                wait_vmcnt<0>();
            wave_lds_exchange_point();  // the reads below stay behind the wait
            const unsigned char *chunk = ring + (kt % STAGES) * SLOT;
            const half8 b0 = *reinterpret_cast<const half8 *>(chunk + step0);
            const half8 b1 = *reinterpret_cast<const half8 *>(chunk + step1);
            // the slot refilled next is the one read in the previous iteration; with this iteration's reads returned
            // too, no read of this wave is outstanding when the copy is issued
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            if constexpr (kt + STAGES - 1 < CHUNKS) {
                fetch(rows, kt + STAGES - 1, (kt + STAGES - 1) % STAGES);
            } else {
                if (has_next) fetch(next_rows, kt + STAGES - 1 - CHUNKS, (kt + STAGES - 1) % STAGES);
            }
#pragma unroll
            for (int i = 0; i < TM; ++i) {
                acc[i] = __builtin_amdgcn_mfma_f32_16x16x32_f16(b0, a[i][kt][0], acc[i], 0, 0, 0);
                acc[i] = __builtin_amdgcn_mfma_f32_16x16x32_f16(b1, a[i][kt][1], acc[i], 0, 0, 0);
            }
        });

        // Operands were swapped in the MFMA: a lane holds four consecutive n (at 4 * (lane / 16)) of row lane % 16.
        // Two sets of partial sums alternate: a wave that writes the set of tile j + 2 has passed the barrier of tile
        // j + 1, which every wave reaches only after it has read the set of tile j.
        float *mine = sums + (parity * waves + wave) * (TM * 256);
#pragma unroll
        for (int i = 0; i < TM; ++i) *reinterpret_cast<floatx4 *>(mine + (i * 16 + row) * 16 + quarter * 4) = acc[i];
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");  // not __syncthreads: B's copies stay in flight
        const float *set = sums + parity * waves * (TM * 256);
        for (int t = tid; t < TM * 64; t += (int)blockDim.x) {
            const int m = t >> 2, c = (t & 3) * 4;
            if (m >= M) continue;
            floatx4 s = *reinterpret_cast<const floatx4 *>(set + m * 16 + c);
            for (int w = 1; w < waves; ++w) s += *reinterpret_cast<const floatx4 *>(set + w * (TM * 256) + m * 16 + c);
            half4 v;
#pragma unroll
            for (int r = 0; r < 4; ++r) v[r] = (half_t)s[r];
            *reinterpret_cast<half4 *>(C + (size_t)m * N + (size_t)tile * 16 + c) = v;
        }
        if (!has_next) break;
        parity ^= 1;
        tile = next;
        rows = next_rows;
    }
}

// K slices per workgroup and chunks per slice for which the kernel is instantiated: K = waves x chunks x 64 with 8, 12,
// 16, 20 or 24 chunks (one row tile of A) or 8 (two) and 2, 4 or 8 waves, the most waves first.  Returns 0 when K has
// no such factorisation.
inline int decode_resident_waves(size_t M, size_t K, int *chunks) {
    if (K % 64 != 0) return 0;
    const size_t k_chunks = K / 64;
    const int options[] = {24, 20, 16, 12, 8};
    for (int waves = 8; waves >= 2; waves /= 2)
        for (int c : options) {
            if (M > 16 && c != 8) continue;
            if (k_chunks == (size_t)waves * c) {
                *chunks = c;
                return waves;
            }
        }
    return 0;
}

inline bool decode_resident_supports(size_t M, size_t N, size_t K) {
    int chunks = 0;
    return M >= 1 && M <= 32 && N > 0 && N % 16 == 0 && N <= ((size_t)1 << 31) / 16 && decode_resident_waves(M, K, &chunks) > 0;
}

template <int TM, int CHUNKS>
void launch_decode_resident_tile(const void *A, const void *B, void *C, size_t M, size_t N, size_t K, int waves,
                                 int workgroups) {
    const size_t lds_bytes = resident_lds_bytes(TM, waves);
    HGEMM_CHECK(lds_bytes <= 160 * 1024 && K == (size_t)waves * CHUNKS * 64 && workgroups >= 1 &&
                (size_t)workgroups <= N / 16);
    static bool configured = [] {
        HGEMM_CHECK_HIP_ERROR(hipFuncSetAttribute(reinterpret_cast<const void *>(&hgemm_decode_resident_kernel<TM, CHUNKS, false>),
                                                  hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
        HGEMM_CHECK_HIP_ERROR(hipFuncSetAttribute(reinterpret_cast<const void *>(&hgemm_decode_resident_kernel<TM, CHUNKS, true>),
                                                  hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
        return true;
    }();
    (void)configured;
    auto kernel = N * K >= ((size_t)24 << 20) ? &hgemm_decode_resident_kernel<TM, CHUNKS, true>
                                              : &hgemm_decode_resident_kernel<TM, CHUNKS, false>;
    kernel<<<dim3((unsigned)workgroups), dim3(waves * 64), lds_bytes, nullptr>>>(
        reinterpret_cast<const half_t *>(A), reinterpret_cast<const half_t *>(B), reinterpret_cast<half_t *>(C), (int)M,
        (int)N, (int)K, (int)(N / 16));
    HGEMM_CHECK_HIP_ERROR(hipGetLastError());
}

// cus: compute units of the device.  Two persistent workgroups per CU share the N / 16 column tiles while A's
// registers leave room for both (M = 16, N = 28672, K = 4096: 38.5 us with one, 37.9 with two; M = 24 ... 32, whose
// two row tiles take twice the registers: 41.5 ... 43.7 us with one, 45.4 ... 48.6 with two).
inline void launch_decode_resident(const void *A, const void *B, void *C, size_t M, size_t N, size_t K, int cus) {
    check_operands(A, B, C, M, N, K);
    HGEMM_CHECK_MSG(decode_resident_supports(M, N, K),
                    "resident decode kernel needs M <= 32, N %% 16 == 0 and K = 64 x {2, 4, 8} x {8, 12, 16, 20, 24} (got M=%zu N=%zu K=%zu)",
                    M, N, K);
    int chunks = 0;
    const int waves = decode_resident_waves(M, K, &chunks);
    HGEMM_CHECK(cus >= 1);
    int workgroups = cus * ((M <= 16 && chunks <= 12) ? 2 : 1);
    if ((size_t)workgroups > N / 16) workgroups = (int)(N / 16);
    if (M > 16)
        launch_decode_resident_tile<2, 8>(A, B, C, M, N, K, waves, workgroups);
    else if (chunks == 24)
        launch_decode_resident_tile<1, 24>(A, B, C, M, N, K, waves, workgroups);
    else if (chunks == 20)
        launch_decode_resident_tile<1, 20>(A, B, C, M, N, K, waves, workgroups);
    else if (chunks == 16)
        launch_decode_resident_tile<1, 16>(A, B, C, M, N, K, waves, workgroups);
    else if (chunks == 12)
        launch_decode_resident_tile<1, 12>(A, B, C, M, N, K, waves, workgroups);
    else
        launch_decode_resident_tile<1, 8>(A, B, C, M, N, K, waves, workgroups);
}

}  // namespace hgemm
