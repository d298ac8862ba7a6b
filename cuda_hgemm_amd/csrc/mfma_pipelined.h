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

template <int BM_, int BN_, int BK_, int WAVES_M_, int WAVES_N_, int STAGES_, int GROUP_N_ = 8, int DBG_ = 0>
struct PipeConfig : TileConfig<BM_, BN_, BK_, WAVES_M_, WAVES_N_, STAGES_, LOAD_DMA, LDS_SWIZZLE, true, GROUP_N_> {
    using Base = TileConfig<BM_, BN_, BK_, WAVES_M_, WAVES_N_, STAGES_, LOAD_DMA, LDS_SWIZZLE, true, GROUP_N_>;
    static constexpr int DBG = DBG_;  // timing experiments only: 1 = no copies in the loop, 2 = copies from a fixed K offset,
                                      // 3 = 1 + no barrier, 4 = 3 + no operand reads
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
                           int N, int K, int tiles_m, int tiles_n, long long *trace) {
    constexpr int BM = Cfg::BM, BN = Cfg::BN, BK = Cfg::BK;
    constexpr int TM = Cfg::TM, TN = Cfg::TN, KSTEPS = Cfg::KSTEPS, CPR = Cfg::CPR;
    constexpr int ROW_BYTES = Cfg::ROW_BYTES, STAGES = Cfg::STAGES;
    constexpr int A_DMA = Cfg::A_DMA, B_DMA = Cfg::B_DMA, L = A_DMA + B_DMA;
    constexpr int NFRAG = TM + TN, NMMA = TM * TN;
    static_assert(NFRAG <= NMMA, "one operand read is issued per MFMA slot");
    static_assert(KSTEPS % 2 == 0, "operand double buffer assumes an even number of steps");
    (void)M;
    long long t_begin = 0, t_loop = 0, t_epi = 0, c_loop = 0, c_epi = 0;
    if (Cfg::DBG == 7) t_begin = wall_clock64();

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

    // ---- pipeline.  Chunk c lives in ring buffer c % STAGES.
    // SPREAD (three or more buffers): the copy of chunk kt+STAGES-1 goes into the buffer
    // that the barrier of iteration kt-1 released and is issued one instruction at a time
    // across all MFMA slots of iteration kt, so the texture path sees an even stream.
    // Otherwise (two buffers): the buffer is only released by this iteration's barrier,
    // so the copy of chunk kt+STAGES is issued across the slots of the last step.
    constexpr bool SPREAD = STAGES >= 3;
    constexpr int AHEAD = SPREAD ? STAGES - 1 : STAGES;      // chunk kt+AHEAD is copied in iteration kt
    constexpr int SLOTS = SPREAD ? KSTEPS * NMMA : NMMA;     // MFMA slots the copy is spread over
    constexpr int FIRST_SLOT = SPREAD ? 0 : (KSTEPS - 1) * NMMA;
    // copy instructions of the current iteration already issued when its barrier is reached
    constexpr int D_BEFORE = SPREAD ? ((KSTEPS - 1) * NMMA * L + SLOTS - 1) / SLOTS : 0;
    // copies allowed to be still in flight at the barrier while chunk kt+1 must have landed
    constexpr int STEADY_VMCNT = SPREAD ? (STAGES - 3) * L + D_BEFORE : (STAGES - 2) * L;
    static_assert(STEADY_VMCNT <= 63, "vmcnt is a 6-bit counter");

#pragma unroll
    for (int s = 0; s < AHEAD; ++s)
#pragma unroll
        for (int idx = 0; idx < L; ++idx) dma_one(idx, s * BK * 2, s);
    wait_vmcnt<(AHEAD - 1) * L>();
    __syncthreads();
#pragma unroll
    for (int idx = 0; idx < NFRAG; ++idx) read_one(idx, 0, 0, frag[0]);

    // One iteration = one K chunk.  ISSUE: chunk kt+AHEAD exists and is copied now.
    // NEXT: chunk kt+1 exists (the barrier is needed and its operands are prefetched).
    auto iteration = [&](int kt, int cur, int fill, auto issue_tag, auto next_tag) {
        constexpr bool ISSUE = decltype(issue_tag)::value, NEXT = decltype(next_tag)::value;
        const int nxt = (cur + 1 == STAGES) ? 0 : cur + 1;
        const int kbyte = (Cfg::DBG == 2 ? (kt & 1) : (kt + AHEAD)) * BK * 2;
#pragma unroll
        for (int kk = 0; kk < KSTEPS; ++kk) {
            const int fb = (kk & 1), nb = fb ^ 1;  // KSTEPS is even: step 0 always uses frag[0]
            const bool last = (kk + 1 == KSTEPS);
            if (last && NEXT) {
                if (ISSUE)
                    wait_vmcnt<STEADY_VMCNT>();
                else
                    wait_vmcnt<0>();
                if (Cfg::DBG < 3) __syncthreads();
                __builtin_amdgcn_sched_barrier(0);
            }
#pragma unroll
            for (int idx = 0; idx < NMMA; ++idx) {
                mma_one(idx, frag[fb]);
                if (idx < NFRAG && Cfg::DBG < 4) {
                    if (!last)
                        read_one(idx, cur, kk + 1, frag[nb]);
                    else if (NEXT)
                        read_one(idx, nxt, 0, frag[nb]);
                }
                if (ISSUE && (Cfg::DBG == 0 || Cfg::DBG == 2 || Cfg::DBG == 7)) {
                    const int slot = kk * NMMA + idx - FIRST_SLOT;  // slot of this MFMA in the copy window
#pragma unroll
                    for (int d = 0; d < L; ++d)
                        if (slot >= 0 && d * SLOTS / L == slot) dma_one(d, kbyte, fill);
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        }
    };
    if (Cfg::DBG == 7) {
        t_loop = wall_clock64();
        c_loop = clock64();
    }
    using T = std::true_type;
    using F = std::false_type;

    int kt = 0, cur = 0, fill = SPREAD ? STAGES - 1 : 0;
    auto advance = [&] {
        cur = (cur + 1 == STAGES) ? 0 : cur + 1;
        fill = (fill + 1 == STAGES) ? 0 : fill + 1;
    };
    for (; kt < num_k - AHEAD; ++kt) {  // chunk kt+AHEAD exists
        iteration(kt, cur, fill, T{}, T{});
        advance();
    }
    for (; kt < num_k - 1; ++kt) {  // drain: nothing left to copy
        iteration(kt, cur, fill, F{}, T{});
        advance();
    }
    iteration(kt, cur, fill, F{}, F{});

    // ---- epilogue: accumulators -> fp16 -> C (through LDS, whole lines per store)
    if (Cfg::DBG == 7) {
        t_epi = wall_clock64();
        c_epi = clock64();
    }
    __syncthreads();
    store_tile_via_lds<Cfg>(acc, lds, C, N, tile_m * BM + wm * Cfg::WM, tile_n * BN + wn * Cfg::WN, wave, lane);
    if (Cfg::DBG == 7 && trace && tid == 0) {
        __builtin_amdgcn_s_waitcnt(0);
        long long *t = trace + (size_t)blockIdx.x * 8;
        t[0] = t_begin;
        t[1] = t_loop;
        t[2] = t_epi;
        t[3] = wall_clock64();
        t[4] = __builtin_amdgcn_s_getreg((31 << 11) | 4);   // HW_ID: wave / simd / cu / sh / se
        t[5] = __builtin_amdgcn_s_getreg((31 << 11) | 20);  // XCC_ID
        t[6] = c_epi - c_loop;
    }
}

template <class Cfg>
void launch_pipelined(const void *A, const void *B, void *C, size_t M, size_t N, size_t K, const char *name,
                      long long *trace = nullptr) {
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
        (int)M, (int)N, (int)K, tiles_m, tiles_n, trace);
    HGEMM_CHECK_HIP_ERROR(hipGetLastError());
}

}  // namespace hgemm
