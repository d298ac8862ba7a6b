// The tuned block-tiled kernel behind hgemm_auto: same tiling, LDS layout and MFMA
// operand scheme as mfma_tiled.h, with a software pipeline laid out by hand.
//
//  * K chunks live in a ring of STAGES LDS buffers filled by direct-to-LDS copies.
//  * The loop is rotated: the one barrier of an iteration sits in front of its LAST
//    MFMA step.  By then every wave has already read the whole current chunk into
//    registers, so the barrier only has to confirm that the next chunk has landed; after
//    it the wave prefetches the first operands of the next chunk and starts the copy that
//    refills the buffer just released -- all of it underneath the last step's MFMAs.
//  * Inside a step the operand reads for the following step are issued one at a time
//    between MFMAs, with scheduling fences so the compiler keeps that order: the matrix
//    pipe never waits for LDS.
// (The corresponding steps of the reference are its pg2s / ps2r / K_STAGE kernels,
//  src/mma/mma_async_pg2s_ps2r.cu:215-269 and src/mma/mma_async_stage4.cu:234-426.)
#pragma once

#include <type_traits>

#include "mfma_tiled.h"

namespace hgemm {

template <int BM_, int BN_, int BK_, int WAVES_M_, int WAVES_N_, int STAGES_, int GROUP_N_ = 8>
struct PipeConfig : TileConfig<BM_, BN_, BK_, WAVES_M_, WAVES_N_, STAGES_, LOAD_DMA, LDS_SWIZZLE, true, GROUP_N_> {
    using Base = TileConfig<BM_, BN_, BK_, WAVES_M_, WAVES_N_, STAGES_, LOAD_DMA, LDS_SWIZZLE, true, GROUP_N_>;
    static_assert(STAGES_ >= 2, "the rotated pipeline needs at least two LDS buffers");
    static bool supports(size_t M, size_t N, size_t K) {
        return M % BM_ == 0 && N % BN_ == 0 && K % BK_ == 0 && K >= (size_t)BK_ * STAGES_;
    }
};

// Direct-to-LDS copy, scalar base + 32-bit per-lane byte offset.
__device__ __forceinline__ void dma_load16_sv(const void *sbase, uint32_t voff, uint32_t lds_addr) {
    asm volatile(
        "s_mov_b32 m0, %0\n\t"
        "s_nop 0\n\t"
        "global_load_lds_dwordx4 %1, %2"
        :
        : "s"(lds_addr), "v"(voff), "s"(sbase)
        : "memory");
}

template <class Cfg>
__global__ void __launch_bounds__(Cfg::THREADS)
    hgemm_pipelined_kernel(const half_t *__restrict__ A, const half_t *__restrict__ B, half_t *__restrict__ C, int M,
                           int N, int K, int tiles_m, int tiles_n) {
    constexpr int BM = Cfg::BM, BN = Cfg::BN, BK = Cfg::BK;
    constexpr int TM = Cfg::TM, TN = Cfg::TN, KSTEPS = Cfg::KSTEPS, CPR = Cfg::CPR;
    constexpr int ROW_BYTES = Cfg::ROW_BYTES, STAGES = Cfg::STAGES;
    constexpr int A_DMA = Cfg::A_DMA, B_DMA = Cfg::B_DMA, L = A_DMA + B_DMA;
    constexpr int NFRAG = TM + TN, NMMA = TM * TN;
    static_assert(NFRAG <= NMMA, "one operand read is issued per MFMA slot");
    static_assert(KSTEPS % 2 == 0, "operand double buffer assumes an even number of steps");
    (void)M;

    extern __shared__ __attribute__((aligned(1024))) unsigned char lds[];
    const uint32_t lds_base = (uint32_t)(uintptr_t)lds;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / Cfg::WAVES_N, wn = wave % Cfg::WAVES_N;

    int tile_m, tile_n;
    tile_of_block<Cfg>(blockIdx.x, tiles_m, tiles_n, tile_m, tile_n);
    const int num_k = K / BK;

    // ---- copy set-up: wave w, instruction i fills LDS rows [(i*WAVES + w)*ROWS_PER_DMA, +ROWS_PER_DMA)
    const unsigned char *a_base = reinterpret_cast<const unsigned char *>(A + (size_t)tile_m * BM * K);
    const unsigned char *b_base = reinterpret_cast<const unsigned char *>(B + (size_t)tile_n * BN * K);
    constexpr int DMA_ROW_STEP = Cfg::WAVES * Cfg::ROWS_PER_DMA;
    uint32_t voff[L];
    {
        const int row = wave * Cfg::ROWS_PER_DMA + lane / CPR;
        const int ch = (lane % CPR) ^ swizzle_of_row<Cfg>(row);
#pragma unroll
        for (int it = 0; it < A_DMA; ++it) voff[it] = ((uint32_t)(row + it * DMA_ROW_STEP) * (uint32_t)K + (uint32_t)(ch * 8)) * 2u;
#pragma unroll
        for (int it = 0; it < B_DMA; ++it)
            voff[A_DMA + it] = ((uint32_t)(row + it * DMA_ROW_STEP) * (uint32_t)K + (uint32_t)(ch * 8)) * 2u;
    }
    const uint32_t cp_lds = lds_base + wave * 1024;
    // copy instruction `idx` (0..L-1) of chunk at byte offset kbyte into ring buffer `stage`
    auto dma_one = [&](int idx, int kbyte, int stage) {
        const uint32_t dst = cp_lds + stage * Cfg::STAGE_BYTES;
        if (idx < A_DMA)
            dma_load16_sv(a_base + kbyte, voff[idx], dst + idx * Cfg::WAVES * 1024);
        else
            dma_load16_sv(b_base + kbyte, voff[idx], dst + Cfg::A_BYTES + (idx - A_DMA) * Cfg::WAVES * 1024);
    };

    // ---- operand fragment set-up
    const int frag_row = lane & 31;
    const int frag_x = (lane >> 5) ^ swizzle_of_row<Cfg>(frag_row);
    const uint32_t a_frag_off = (wm * Cfg::WM + frag_row) * ROW_BYTES;
    const uint32_t b_frag_off = Cfg::A_BYTES + (wn * Cfg::WN + frag_row) * ROW_BYTES;
    uint32_t chunk_off[KSTEPS];
#pragma unroll
    for (int kk = 0; kk < KSTEPS; ++kk) chunk_off[kk] = (uint32_t)((kk * 2) ^ frag_x) << 4;

    half8 frag[2][NFRAG];  // [buffer][A fragments 0..TM-1, then B fragments]
    // fragment read number `idx` (0..NFRAG-1) of step kk of ring buffer `stage`
    auto read_one = [&](int idx, int stage, int kk, half8 (&dst)[NFRAG]) {
        const unsigned char *s = lds + stage * Cfg::STAGE_BYTES + chunk_off[kk];
        if (idx < TM)
            dst[idx] = *reinterpret_cast<const half8 *>(s + a_frag_off + idx * 32 * ROW_BYTES);
        else
            dst[idx] = *reinterpret_cast<const half8 *>(s + b_frag_off + (idx - TM) * 32 * ROW_BYTES);
    };

    floatx16 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

    auto mma_one = [&](int idx, const half8 (&src)[NFRAG]) {
        const int i = idx / TN;
        const int j = (i & 1) ? (TN - 1 - idx % TN) : (idx % TN);  // serpentine
        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(src[TM + j], src[i], acc[i][j], 0, 0, 0);
    };

    // ---- prologue: fill the whole ring, wait for chunk 0, read its first operands
#pragma unroll
    for (int s = 0; s < STAGES; ++s)
#pragma unroll
        for (int idx = 0; idx < L; ++idx) dma_one(idx, s * BK * 2, s);
    wait_vmcnt<(STAGES - 1) * L>();
    __syncthreads();
#pragma unroll
    for (int idx = 0; idx < NFRAG; ++idx) read_one(idx, 0, 0, frag[0]);

    // One iteration = one K chunk.  ISSUE: a chunk remains to be copied into the buffer this
    // iteration releases.  NEXT: another chunk follows (its operands are prefetched).
    // STEADY: the full complement of later chunks is in flight at the barrier.
    auto iteration = [&](int kt, int cur, auto issue_tag, auto next_tag, auto steady_tag) {
        constexpr bool ISSUE = decltype(issue_tag)::value, NEXT = decltype(next_tag)::value;
        constexpr bool STEADY = decltype(steady_tag)::value;
        const int nxt = (cur + 1 == STAGES) ? 0 : cur + 1;
#pragma unroll
        for (int kk = 0; kk < KSTEPS; ++kk) {
            const int fb = (kk & 1), nb = fb ^ 1;  // KSTEPS is even: step 0 always uses frag[0]
            if (kk + 1 < KSTEPS) {
#pragma unroll
                for (int idx = 0; idx < NMMA; ++idx) {
                    mma_one(idx, frag[fb]);
                    if (idx < NFRAG) read_one(idx, cur, kk + 1, frag[nb]);
                    __builtin_amdgcn_sched_barrier(0);
                }
            } else {
                if (NEXT) {
                    if (STEADY)
                        wait_vmcnt<(STAGES - 2) * L>();
                    else
                        wait_vmcnt<0>();
                    __syncthreads();
                }
                __builtin_amdgcn_sched_barrier(0);
                constexpr int DMA_PER_SLOT = (L + NMMA - 1) / NMMA;
#pragma unroll
                for (int idx = 0; idx < NMMA; ++idx) {
                    mma_one(idx, frag[fb]);
                    if (NEXT && idx < NFRAG) read_one(idx, nxt, 0, frag[nb]);
                    if (ISSUE) {
#pragma unroll
                        for (int d = 0; d < DMA_PER_SLOT; ++d)
                            if (idx * DMA_PER_SLOT + d < L)
                                dma_one(idx * DMA_PER_SLOT + d, (kt + STAGES) * BK * 2, cur);
                    }
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
        }
    };
    using T = std::true_type;
    using F = std::false_type;

    int kt = 0, cur = 0;
    for (; kt < num_k - STAGES; ++kt) {  // chunks kt+STAGES exist
        iteration(kt, cur, T{}, T{}, T{});
        cur = (cur + 1 == STAGES) ? 0 : cur + 1;
    }
    for (; kt < num_k - 1; ++kt) {  // drain: nothing left to copy
        iteration(kt, cur, F{}, T{}, F{});
        cur = (cur + 1 == STAGES) ? 0 : cur + 1;
    }
    iteration(kt, cur, F{}, F{}, F{});

    // ---- epilogue: accumulators -> fp16 -> C
    half_t *Cw = C + (size_t)(tile_m * BM + wm * Cfg::WM + (lane & 31)) * N + tile_n * BN + wn * Cfg::WN +
                 ((lane >> 5) << 2);
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                half4 v;
#pragma unroll
                for (int r = 0; r < 4; ++r) v[r] = (half_t)acc[i][j][g * 4 + r];
                *reinterpret_cast<half4 *>(Cw + (size_t)i * 32 * N + j * 32 + g * 8) = v;
            }
}

template <class Cfg>
void launch_pipelined(const void *A, const void *B, void *C, size_t M, size_t N, size_t K, const char *name) {
    check_operands(A, B, C, M, N, K);
    HGEMM_CHECK_MSG(Cfg::supports(M, N, K),
                    "%s needs M %% %d == 0, N %% %d == 0, K %% %d == 0, K >= %d (got M=%zu N=%zu K=%zu)", name,
                    Cfg::BM, Cfg::BN, Cfg::BK, Cfg::BK * Cfg::STAGES, M, N, K);
    static bool configured = [] {
        HGEMM_CHECK_HIP_ERROR(hipFuncSetAttribute(reinterpret_cast<const void *>(&hgemm_pipelined_kernel<Cfg>),
                                                  hipFuncAttributeMaxDynamicSharedMemorySize, Cfg::LDS_BYTES));
        return true;
    }();
    (void)configured;
    const int tiles_m = (int)(M / Cfg::BM), tiles_n = (int)(N / Cfg::BN);
    hgemm_pipelined_kernel<Cfg><<<dim3(tiles_m * tiles_n), dim3(Cfg::THREADS), Cfg::LDS_BYTES, nullptr>>>(
        reinterpret_cast<const half_t *>(A), reinterpret_cast<const half_t *>(B), reinterpret_cast<half_t *>(C),
        (int)M, (int)N, (int)K, tiles_m, tiles_n);
    HGEMM_CHECK_HIP_ERROR(hipGetLastError());
}

}  // namespace hgemm
