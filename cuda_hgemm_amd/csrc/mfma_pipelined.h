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
#include <utility>

#include "mfma_tiled.h"

namespace hgemm {

template <int BM_, int BN_, int BK_, int WAVES_M_, int WAVES_N_, int STAGES_, int MI_ = 16, int EXTRA_A_ = 0>
struct PipeConfig : TileConfig<BM_, BN_, BK_, WAVES_M_, WAVES_N_, STAGES_, LOAD_DMA, LDS_SWIZZLE, true> {
    using Base = TileConfig<BM_, BN_, BK_, WAVES_M_, WAVES_N_, STAGES_, LOAD_DMA, LDS_SWIZZLE, true>;
    // MFMA shape: 32 -> v_mfma_f32_32x32x16_f16, 16 -> v_mfma_f32_16x16x32_f16.  Both move
    // the same bytes from LDS per flop (that depends on the wave tile only); the 16x16x32
    // form reads and writes half as many accumulator registers per flop and sustains a
    // higher clock under the board's power limit.
    static constexpr int MI = MI_;
    static constexpr int PTM = Base::WM / MI, PTN = Base::WN / MI;  // MFMA tiles per wave
    static constexpr int PKSTEP = MI == 32 ? 16 : 32;               // k covered by one MFMA
    static constexpr int PKSTEPS = BK_ / PKSTEP;
    static constexpr int CPS = PKSTEP / 8;                          // 16-byte chunks per row per step
    // Ring depths.  The B ring has STAGES buffers, the A ring STAGES + EXTRA_A: 256x256x64
    // tiles are 32 KB per operand and chunk, so the 160 KB of LDS hold two full stages plus
    // one more A buffer -- the A copies then run two chunks ahead and only the B copies
    // are on the critical path of the barrier.
    static constexpr int SA = STAGES_ + EXTRA_A_, SB = STAGES_;
    static constexpr int RING_BYTES = SA * Base::A_BYTES + SB * Base::B_BYTES;
    static constexpr int LDS_BYTES =
        RING_BYTES > Base::WAVES * Base::C_STRIP_BYTES ? RING_BYTES : Base::WAVES * Base::C_STRIP_BYTES;
    static_assert(EXTRA_A_ == 0 || (EXTRA_A_ == 1 && STAGES_ == 2), "the deeper A ring is defined for two B buffers");
    static_assert(LDS_BYTES <= 160 * 1024, "exceeds the 160 KB LDS of a gfx950 CU");
    static_assert(MI == 16 || MI == 32, "MFMA tile is 16x16x32 or 32x32x16");
    static_assert(STAGES_ >= 2, "the rotated pipeline needs at least two LDS buffers");
    static_assert(Base::WM % MI == 0 && Base::WN % MI == 0, "wave tile must be a multiple of the MFMA tile");
    static_assert(PKSTEPS % 2 == 0, "the operand double buffer needs an even number of MFMA steps per chunk");
    static bool supports(size_t M, size_t N, size_t K) {
        return M % BM_ == 0 && N % BN_ == 0 && K % BK_ == 0 && K >= (size_t)BK_ * STAGES_;
    }
};

// XOR applied to the 16-byte chunk index of LDS row `row`.  A ds_read_b128 serves its 64
// lanes in four cycles of 16 lanes over 64 banks, and (measured with the LDS bank-conflict
// counter) the 16 lanes of one cycle are lanes [8g, 8g+8) together with [32+8g, 32+8g+8).
// With 16x16x32 operands (lane l reads row l % 16, chunk l / 16 of the step) and 128-byte
// rows, one cycle therefore touches 8 rows at chunk c and the same 8 rows at chunk c ^ 2:
// the four rows of equal parity must get XOR values from four different cosets of {0, 2},
// which the row-number swizzle of the other kernels does not give (half of all LDS cycles
// were conflicts).  Rows 8-15 use the complementary values, so 16 consecutive rows at one
// chunk are conflict-free as well.
template <class Cfg>
__device__ __forceinline__ int pipe_swizzle(int row) {
    if constexpr (Cfg::MI == 16 && Cfg::BK == 64) {
        const int x = (row >> 1) & 3;
        return ((x & 1) | ((x & 2) << 1)) ^ (((row >> 3) & 1) << 1);
    }
    return swizzle_of_row<Cfg>(row);
}

template <class T, T V>
constexpr int ring_index(std::integral_constant<T, V>) {
    return (int)V;
}
constexpr int ring_index(int v) { return v; }
constexpr int gcd_of(int a, int b) { return b == 0 ? a : gcd_of(b, a % b); }

// Compile-time loop: f(integral_constant<int, 0>) ... f(integral_constant<int, N-1>).  The
// pipeline body is laid out slot by slot with every index a constant; this does not lean
// on the loop unroller, whose failure would turn the accumulators into scratch memory.
template <class F, int... I>
__device__ __forceinline__ void static_for_impl(F &&f, std::integer_sequence<int, I...>) {
    (f(std::integral_constant<int, I>{}), ...);
}
template <int N, class F>
__device__ __forceinline__ void static_for(F &&f) {
    static_for_impl(static_cast<F &&>(f), std::make_integer_sequence<int, N>{});
}

// LDS operand read and its wait, written as assembly: the optimiser moves ordinary LDS loads
// freely (it batched them at the top of the loop, which both breaks the interleave with
// the MFMAs and blows the register budget), so the reads are pinned here and the kernel
// does its own lgkmcnt accounting.
template <int OFFSET>
__device__ __forceinline__ half8 lds_read16(uint32_t addr) {
    half8 v;
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "i"(OFFSET));
    return v;
}
__device__ __forceinline__ void lds_wait_all() { asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); }
// Ordered no-op that "modifies" a fragment: placed after lds_wait_all, it keeps every later
// use of the fragment (the MFMAs, or a register copy the compiler makes) behind the wait
// without spending an instruction per fragment.
__device__ __forceinline__ void lds_landed(half8 &a) { asm volatile("" : "+v"(a)); }

// The MFMA itself is issued from assembly too, with the accumulator pinned to AGPRs: that
// fixes the order of MFMAs, operand reads and copies exactly as written (volatile
// statements are never reordered against each other) and keeps the register allocator from
// shuttling accumulators between the two register files.  The kernel guarantees what the
// compiler no longer checks: an accumulator is reused only a full step (>= 16 MFMAs) later,
// and operands are covered by lds_wait_all.
template <int MI>
struct MfmaOp;
template <>
struct MfmaOp<32> {
    typedef floatx16 Acc;
    static constexpr int REGS = 16;
    static __device__ __forceinline__ void run(half8 a, half8 b, Acc &c) {
        asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
    }
};
template <>
struct MfmaOp<16> {
    typedef floatx4 Acc;
    static constexpr int REGS = 4;
    static __device__ __forceinline__ void run(half8 a, half8 b, Acc &c) {
        asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
    }
};

// One MFMA slot that also starts a direct-to-LDS copy: M0 (the LDS destination) is set
// before the MFMA, which doubles as the wait state the hardware wants between a write of
// M0 and the copy that reads it, so the slot costs three instructions.
template <int MI, int LDS_IMM, bool NT = false>
__device__ __forceinline__ void mfma_and_dma(half8 a, half8 b, typename MfmaOp<MI>::Acc &c, const void *sbase,
                                             uint32_t voff, uint32_t lds_base) {
    // NT: the copy carries the non-temporal hint (an operand that is read once and should not displace the other's
    // panels from L2 and the Infinity Cache)
    if constexpr (MI == 16 && NT)
        asm volatile(
            "s_add_u32 m0, %3, %6\n\t"
            "v_mfma_f32_16x16x32_f16 %0, %1, %2, %0\n\t"
            "global_load_lds_dwordx4 %4, %5 nt"
            : "+a"(c)
            : "v"(a), "v"(b), "s"(lds_base), "v"(voff), "s"(sbase), "i"(LDS_IMM)
            : "memory", "scc");
    else if constexpr (MI == 16)
        asm volatile(
            "s_add_u32 m0, %3, %6\n\t"
            "v_mfma_f32_16x16x32_f16 %0, %1, %2, %0\n\t"
            "global_load_lds_dwordx4 %4, %5"
            : "+a"(c)
            : "v"(a), "v"(b), "s"(lds_base), "v"(voff), "s"(sbase), "i"(LDS_IMM)
            : "memory", "scc");
    else
        asm volatile(
            "s_add_u32 m0, %3, %6\n\t"
            "v_mfma_f32_32x32x16_f16 %0, %1, %2, %0\n\t"
            "global_load_lds_dwordx4 %4, %5"
            : "+a"(c)
            : "v"(a), "v"(b), "s"(lds_base), "v"(voff), "s"(sbase), "i"(LDS_IMM)
            : "memory", "scc");
    static_assert(!NT || MI == 16, "the non-temporal copy is written for the 16x16x32 kernels");
}

// Ordered no-op that "modifies" an accumulator: later reads of it stay behind this point.
template <class Acc>
__device__ __forceinline__ void pin_accumulator(Acc &c) {
    asm volatile("" : "+a"(c));
}

// Direct-to-LDS copy: global address = scalar base + 32-bit per-lane byte offset, LDS
// destination (wave-uniform, goes through M0) = lds_base + LDS_IMM.
template <int LDS_IMM, bool NT = false>
__device__ __forceinline__ void dma_load16_sv(const void *sbase, uint32_t voff, uint32_t lds_base) {
    if constexpr (NT)
        asm volatile(
            "s_add_u32 m0, %0, %3\n\t"
            "s_nop 0\n\t"
            "global_load_lds_dwordx4 %1, %2 nt"
            :
            : "s"(lds_base), "v"(voff), "s"(sbase), "i"(LDS_IMM)
            : "memory", "scc");
    else
        asm volatile(
            "s_add_u32 m0, %0, %3\n\t"
            "s_nop 0\n\t"
            "global_load_lds_dwordx4 %1, %2"
            :
            : "s"(lds_base), "v"(voff), "s"(sbase), "i"(LDS_IMM)
            : "memory", "scc");
}

// Accumulators -> fp16 -> C through LDS for either MFMA shape (operands swapped, so a lane
// holds groups of four consecutive n of one row m = lane % MI): each wave parks MI rows of
// its tile in a private strip and reads them back row-contiguous, 16 bytes per lane, so a
// global store instruction writes whole 128-byte lines.
// EDGE: rows >= M and 8-column pieces at or beyond N (N % 8 == 0) are not stored.
template <class Cfg, class Acc, bool EDGE = false>
__device__ __forceinline__ void store_wave_tile(const Acc (&acc)[Cfg::PTM][Cfg::PTN], unsigned char *lds,
                                                half_t *__restrict__ C, int M, int N, int row0, int col0, int wave,
                                                int lane) {
    constexpr int MI = Cfg::MI, TM = Cfg::PTM, TN = Cfg::PTN, WN = Cfg::WN;
    constexpr int GROUPS = MI == 32 ? 4 : 1;          // register groups of four n per accumulator
    constexpr int STRIP_ROW_BYTES = WN * 2 + 16;
    constexpr int STRIP_BYTES = 32 * STRIP_ROW_BYTES;  // sized for the 32-row case
    constexpr int LANES_PER_ROW = WN / 8;
    constexpr int ROWS_PER_READ = 64 / LANES_PER_ROW;                   // lanes beyond that many rows idle
    constexpr int READS = (MI + ROWS_PER_READ - 1) / ROWS_PER_READ;
    constexpr bool EXACT = (64 % LANES_PER_ROW == 0) && (MI % ROWS_PER_READ == 0);
    static_assert(STRIP_BYTES == Cfg::C_STRIP_BYTES, "strip size");
    unsigned char *strip = lds + wave * STRIP_BYTES;
    unsigned char *wr = strip + (lane % MI) * STRIP_ROW_BYTES + ((lane / MI) << 3);
    const int rd_row = lane / LANES_PER_ROW, rd_col = lane % LANES_PER_ROW;
    const unsigned char *rd = strip + rd_row * STRIP_ROW_BYTES + rd_col * 16;
    half_t *cp = C + (size_t)(row0 + rd_row) * N + col0 + rd_col * 8;
#pragma unroll
    for (int i = 0; i < TM; ++i) {
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int g = 0; g < GROUPS; ++g) {
                half4 v;
#pragma unroll
                for (int r = 0; r < 4; ++r) v[r] = (half_t)acc[i][j][g * 4 + r];
                *reinterpret_cast<half4 *>(wr + (j * MI + g * 8) * 2) = v;
            }
        wave_lds_exchange_point();
#pragma unroll
        for (int it = 0; it < READS; ++it) {
            if (EXACT || (rd_row < ROWS_PER_READ && it * ROWS_PER_READ + rd_row < MI)) {
                const u32x4 v = *reinterpret_cast<const u32x4 *>(rd + it * ROWS_PER_READ * STRIP_ROW_BYTES);
                if (!EDGE || (row0 + rd_row + i * MI + it * ROWS_PER_READ < M && col0 + rd_col * 8 < N))
                    store_streaming(reinterpret_cast<u32x4 *>(cp + (size_t)(i * MI + it * ROWS_PER_READ) * N), v);
            }
        }
        wave_lds_exchange_point();
    }
}

// fp32 partial sums of a wave tile (16x16x32 accumulators: a lane holds four consecutive n of row m = lane % 16 of
// each tile) -> memory, through LDS like the fp16 tile above: stored straight from that layout an instruction writes
// sixteen 16-byte pieces of sixteen different rows; parked in the wave's strip 16 rows at a time and read back
// row-contiguous, it writes whole 128-byte lines.  `get(i, j)` returns accumulator tile (i, j); `dst` is element (0, 0)
// of the wave tile in a matrix with `ld` floats per row; rows >= rows_valid and 4-column pieces at or beyond
// cols_valid (both relative to the wave tile) are not stored when EDGE.
template <class Cfg, bool EDGE, class Get>
__device__ __forceinline__ void store_wave_tile_f32(Get get, unsigned char *lds, float *__restrict__ dst, size_t ld,
                                                    int rows_valid, int cols_valid, int wave, int lane) {
    constexpr int MI = 16, TM = Cfg::PTM, TN = Cfg::PTN, WN = Cfg::WN;
    static_assert(Cfg::MI == 16, "written for the 16x16x32 accumulator layout");
    constexpr int STRIP_ROW_BYTES = WN * 4 + 16;
    static_assert(MI * STRIP_ROW_BYTES <= Cfg::C_STRIP_BYTES, "the fp16 strip of a wave holds 16 rows of fp32");
    constexpr int LANES_PER_ROW = WN / 4;                               // 16-byte pieces per row
    constexpr int ROWS_PER_READ = 64 / LANES_PER_ROW;                   // lanes beyond that many rows idle
    constexpr int READS = (MI + ROWS_PER_READ - 1) / ROWS_PER_READ;
    constexpr bool EXACT = (64 % LANES_PER_ROW == 0) && (MI % ROWS_PER_READ == 0);
    unsigned char *strip = lds + wave * Cfg::C_STRIP_BYTES;
    unsigned char *wr = strip + (lane % MI) * STRIP_ROW_BYTES + ((lane / MI) << 4);
    const int rd_row = lane / LANES_PER_ROW, rd_col = lane % LANES_PER_ROW;
    const unsigned char *rd = strip + rd_row * STRIP_ROW_BYTES + rd_col * 16;
    float *out = dst + (size_t)rd_row * ld + rd_col * 4;
    static_for<TM>([&](auto i_c) {
        constexpr int i = decltype(i_c)::value;
        static_for<TN>([&](auto j_c) {
            constexpr int j = decltype(j_c)::value;
            *reinterpret_cast<floatx4 *>(wr + j * MI * 4) = get(i_c, j_c);
        });
        wave_lds_exchange_point();
#pragma unroll
        for (int it = 0; it < READS; ++it) {
            if (EXACT || (rd_row < ROWS_PER_READ && it * ROWS_PER_READ + rd_row < MI)) {
                const floatx4 v = *reinterpret_cast<const floatx4 *>(rd + it * ROWS_PER_READ * STRIP_ROW_BYTES);
                if (!EDGE || (i * MI + it * ROWS_PER_READ + rd_row < rows_valid && rd_col * 4 < cols_valid))
                    *reinterpret_cast<floatx4 *>(out + (size_t)(i * MI + it * ROWS_PER_READ) * ld) = v;
            }
        }
        wave_lds_exchange_point();
    });
}

// What both tuned kernels (interleaved below, chained in mfma_chained.h) set up before their loops: which tile
// and K slice the workgroup computes, the per-lane global offsets of its direct-to-LDS copies, and the LDS
// addresses its lanes read MFMA operands from.
// EDGE: M and N need not be multiples of the tile (N % 8 == 0 still, for aligned rows of
// C).  Copies of rows beyond the matrix are redirected to its last row -- valid memory,
// products never stored -- which costs nothing inside the loop; only the stores are guarded.
template <class Cfg, bool SPLIT, bool EDGE>
struct PipeFrame {
    static constexpr int BM = Cfg::BM, BN = Cfg::BN, BK = Cfg::BK, MI = Cfg::MI;
    static constexpr int KSTEPS = Cfg::PKSTEPS, CPR = Cfg::CPR, CPS = Cfg::CPS, ROW_BYTES = Cfg::ROW_BYTES;
    static constexpr int A_DMA = Cfg::A_DMA, B_DMA = Cfg::B_DMA, L = A_DMA + B_DMA;
    static constexpr int B_REGION = Cfg::SA * Cfg::A_BYTES;  // LDS: the A ring (SA buffers), then the B ring (SB buffers)
    // Fragment idx sits idx * MI rows further down.  That never changes bits 0-2 of the
    // row's bank-line index, and changes bit 3 (which the swizzle folds into bit 0) only
    // when MI rows are 8 lines: then odd fragments use the chunk index XOR 1.
    static constexpr int ODD_FLIP = ((MI * BK * 2 / 128) % 16 == 8) ? 16 : 0;
    static constexpr int NF = ODD_FLIP ? 2 : 1;
    static_assert((Cfg::PTN - 1) * MI * ROW_BYTES < 65536 && (Cfg::PTM - 1) * MI * ROW_BYTES < 65536,
                  "fragment offsets must fit the 16-bit ds_read offset field");

    int lane, wave, wm, wn;
    int tile_m, tile_n;      // the workgroup's tile (wave-uniform)
    int slot, slice;         // its position among the launch's tiles and, in a K-sliced launch, its slice
    int num_k;               // chunks it walks
    const unsigned char *a_base, *b_base;  // first chunk of the tile's rows of A and of B
    uint32_t voff[L];        // per-lane byte offset of copy instruction i from a_base (i < A_DMA) or b_base
    uint32_t cp_lds;         // LDS address the wave's copy instruction 0 fills, without the ring-buffer offset
    // Byte address (32-bit LDS offset) of this lane's fragment of A tile 0 / B tile 0 for
    // step kk, without the ring-buffer base; tile t adds the constant t * MI * ROW_BYTES.
    uint32_t a_addr[KSTEPS][NF], b_addr[KSTEPS][NF];

    // false: this workgroup has no tile (a part of a subdivided tile that lies wholly outside the matrix)
    __device__ __forceinline__ bool init(const half_t *A, const half_t *B, int M, int N, int K, int slices, int tiles_m,
                                         int tiles_n, int first_block, int subdiv, uint32_t lds_base) {
        const int tid = threadIdx.x;
        lane = tid & 63;
        wave = __builtin_amdgcn_readfirstlane(tid >> 6);
        wm = wave / Cfg::WAVES_N, wn = wave % Cfg::WAVES_N;
        const bool blocked = blocked_order(N, K);  // the same in every launch that works on this problem
        // this workgroup's slot among the launch's positions: slots are dealt so that the workgroups an XCD runs
        // together are neighbours in the tile order.  A K-sliced launch is one-dimensional as well, slice-major, so
        // that those neighbours also work on the same slice of K.
        slice = 0;
        if constexpr (SPLIT) {
            slice_and_slot_of_workgroup((int)blockIdx.x, (int)gridDim.x / slices, slices, slice, slot);
            slice = __builtin_amdgcn_readfirstlane(slice);
        } else {
            slot = slot_of_workgroup(blocked, (int)blockIdx.x, (int)gridDim.x);
        }
        if (subdiv == 0) {
            // the launch covers positions [first_block, first_block + gridDim.x) of the tile order
            tile_of_position(blocked, first_block + slot, tiles_m, tiles_n, tile_m, tile_n);
        } else {
            // tiles_m x tiles_n is the grid of a larger tile that this one divides sub_m x sub_n times;
            // consecutive slots take the parts of the tile at position first_block + slot / parts
            const int sub_m = subdiv >> 8, sub_n = subdiv & 255, parts = sub_m * sub_n;
            const int part = slot % parts;
            int parent_m, parent_n;
            tile_of_position(blocked, first_block + slot / parts, tiles_m, tiles_n, parent_m, parent_n);
            tile_m = parent_m * sub_m + part / sub_n;
            tile_n = parent_n * sub_n + part % sub_n;
            if (tile_m * BM >= M || tile_n * BN >= N) return false;  // the whole workgroup
        }
        tile_m = __builtin_amdgcn_readfirstlane(tile_m);  // wave-uniform by construction: keep them in SGPRs
        tile_n = __builtin_amdgcn_readfirstlane(tile_n);
        int first_chunk;
        slice_of_k(K / BK, slices, slice, first_chunk, num_k);
        const int k_begin = first_chunk * BK;

        // ---- copies: wave w, instruction i fills LDS rows [(i*WAVES + w)*ROWS_PER_DMA, +ROWS_PER_DMA)
        a_base = reinterpret_cast<const unsigned char *>(A + (size_t)tile_m * BM * K + k_begin);
        b_base = reinterpret_cast<const unsigned char *>(B + (size_t)tile_n * BN * K + k_begin);
        constexpr int DMA_ROW_STEP = Cfg::WAVES * Cfg::ROWS_PER_DMA;
        {
            // lane l of instruction `it` lands on physical chunk l % CPR of LDS row
            // row0 + it * DMA_ROW_STEP, so it fetches the logical chunk the swizzle maps there
            const int row0 = wave * Cfg::ROWS_PER_DMA + lane / CPR;
            const int last_a = M - 1 - tile_m * BM, last_b = N - 1 - tile_n * BN;  // last valid row of the tile
#pragma unroll
            for (int it = 0; it < A_DMA; ++it) {
                const int row = row0 + it * DMA_ROW_STEP;
                const int ch = (lane % CPR) ^ pipe_swizzle<Cfg>(row);
                const int src = (EDGE && row > last_a) ? last_a : row;
                voff[it] = ((uint32_t)src * (uint32_t)K + (uint32_t)(ch * 8)) * 2u;
            }
#pragma unroll
            for (int it = 0; it < B_DMA; ++it) {
                const int row = row0 + it * DMA_ROW_STEP;
                const int ch = (lane % CPR) ^ pipe_swizzle<Cfg>(row);
                const int src = (EDGE && row > last_b) ? last_b : row;
                voff[A_DMA + it] = ((uint32_t)src * (uint32_t)K + (uint32_t)(ch * 8)) * 2u;
            }
        }
        cp_lds = lds_base + wave * 1024;

        // ---- operand fragments: lane l supplies 8 consecutive k (chunk l / MI of the
        // step) of row l % MI, for both operands.
        const int frag_row = lane % MI;
        const int frag_x = (lane / MI) ^ pipe_swizzle<Cfg>(frag_row);
        const uint32_t a_frag_off = (wm * Cfg::WM + frag_row) * ROW_BYTES;
        const uint32_t b_frag_off = B_REGION + (wn * Cfg::WN + frag_row) * ROW_BYTES;
#pragma unroll
        for (int kk = 0; kk < KSTEPS; ++kk)
#pragma unroll
            for (int f = 0; f < NF; ++f) {
                const uint32_t chunk_off = ((uint32_t)((kk * CPS) ^ frag_x) << 4) ^ (uint32_t)(f * ODD_FLIP);
                a_addr[kk][f] = lds_base + a_frag_off + chunk_off;
                b_addr[kk][f] = lds_base + b_frag_off + chunk_off;
            }
        return true;
    }

    // operand fragment of A / B tile t for MFMA step kk of the chunk in the ring buffer at byte offset stage_bytes
    template <class TC, class KC>
    __device__ __forceinline__ half8 read_a(TC, uint32_t stage_bytes, KC) const {
        constexpr int t = TC::value, kk = KC::value;
        return lds_read16<t * MI * ROW_BYTES>(a_addr[kk][ODD_FLIP ? (t & 1) : 0] + stage_bytes);
    }
    template <class TC, class KC>
    __device__ __forceinline__ half8 read_b(TC, uint32_t stage_bytes, KC) const {
        constexpr int t = TC::value, kk = KC::value;
        return lds_read16<t * MI * ROW_BYTES>(b_addr[kk][ODD_FLIP ? (t & 1) : 0] + stage_bytes);
    }
};

// STREAM_B: B's copies carry the non-temporal hint.  For one row of tiles against a B that outgrows the Infinity
// Cache: every byte of B is read once, and as an ordinary read it pushes the A panel every workgroup shares out of
// L2 and the Infinity Cache.
template <class Cfg, bool SPLIT = false, bool EDGE = false, bool STREAM_B = false>
__global__ void __launch_bounds__(Cfg::THREADS)
    hgemm_pipelined_kernel(const half_t *__restrict__ A, const half_t *__restrict__ B, half_t *__restrict__ C,
                           float *__restrict__ partial, int M, int N, int K, int slices, int tiles_m, int tiles_n,
                           int first_block, int tail_tiles, int subdiv) {
    constexpr int BM = Cfg::BM, BN = Cfg::BN, BK = Cfg::BK, MI = Cfg::MI;
    constexpr int TM = Cfg::PTM, TN = Cfg::PTN, KSTEPS = Cfg::PKSTEPS;
    constexpr int STAGES = Cfg::STAGES, SA = Cfg::SA, SB = Cfg::SB;
    constexpr int A_BYTES = Cfg::A_BYTES, B_BYTES = Cfg::B_BYTES, B_REGION = SA * A_BYTES;
    constexpr int A_DMA = Cfg::A_DMA, B_DMA = Cfg::B_DMA, L = A_DMA + B_DMA;
    constexpr int NFRAG = TM + TN, NMMA = TM * TN;
    typedef typename MfmaOp<MI>::Acc Acc;
    static_assert(NFRAG <= NMMA, "at most one operand read is issued per MFMA slot");
    static_assert(!SPLIT || MI == 16, "fp32 partial stores are written for the 16x16x32 accumulator layout");

    extern __shared__ __attribute__((aligned(1024))) unsigned char lds[];
    const uint32_t lds_base = (uint32_t)(uintptr_t)lds;
    PipeFrame<Cfg, SPLIT, EDGE> frame;
    if (!frame.init(A, B, M, N, K, slices, tiles_m, tiles_n, first_block, subdiv, lds_base)) return;
    const int lane = frame.lane, wave = frame.wave, wm = frame.wm, wn = frame.wn;
    const int tile_m = frame.tile_m, tile_n = frame.tile_n, slot = frame.slot, slice = frame.slice;
    const int num_k = frame.num_k;
    const unsigned char *const a_base = frame.a_base, *const b_base = frame.b_base;
    const uint32_t(&voff)[L] = frame.voff;
    const uint32_t cp_lds = frame.cp_lds;
    // copy instruction `idx` (0..L-1) of a chunk: `a_src` / `b_src` already point at the chunk; `dst_a` / `dst_b`
    // are cp_lds plus the byte offset of the ring buffer to fill.
    auto dma_one = [&](auto idx_c, const unsigned char *a_src, const unsigned char *b_src, uint32_t dst_a,
                       uint32_t dst_b) {
        constexpr int idx = decltype(idx_c)::value;
        if constexpr (idx < A_DMA)
            dma_load16_sv<idx * Cfg::WAVES * 1024>(a_src, voff[idx], dst_a);
        else
            dma_load16_sv<(idx - A_DMA) * Cfg::WAVES * 1024, STREAM_B>(b_src, voff[idx], dst_b);
    };

    // Operand registers.  MFMAs run B-major (all A tiles against B tile 0, then B tile 1,
    // ...): a B fragment is dead after TM MFMAs and is reloaded in place for the next step
    // right away, so only the A fragments (needed for the whole step) and the last B
    // fragment are double buffered.  This keeps the kernel well inside the register file
    // next to 256 accumulator registers.
    half8 a_frag[2][TM];
    constexpr int NDB = 2;                 // trailing B tiles that are double buffered
    constexpr int NSB = TN - NDB;          // leading B tiles reloaded in place
    half8 b_frag[NSB > 0 ? NSB : 1];
    half8 b_last[2][NDB];
    auto read_a = [&](auto t_c, uint32_t stage_bytes, auto kk_c) -> half8 { return frame.read_a(t_c, stage_bytes, kk_c); };
    auto read_b = [&](auto t_c, uint32_t stage_bytes, auto kk_c) -> half8 { return frame.read_b(t_c, stage_bytes, kk_c); };
    // every outstanding operand read has landed; ties all fragments of buffer `buf`
    auto wait_operands = [&](auto buf_c) {
        constexpr int buf = decltype(buf_c)::value;
        lds_wait_all();
        static_for<TM>([&](auto t) { lds_landed(a_frag[buf][decltype(t)::value]); });
        static_for<NSB>([&](auto t) { lds_landed(b_frag[decltype(t)::value]); });
        static_for<NDB>([&](auto t) { lds_landed(b_last[buf][decltype(t)::value]); });
    };

    Acc acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int r = 0; r < MfmaOp<MI>::REGS; ++r) acc[i][j][r] = 0.0f;

    // MFMA slot idx of a step: B tile idx / TM against A tile idx % TM, from buffer fb.
    auto mma_one = [&](auto idx_c, auto fb_c) {
        constexpr int idx = decltype(idx_c)::value, fb = decltype(fb_c)::value;
        constexpr int j = idx / TM, i = idx % TM;
        if constexpr (j >= NSB)
            MfmaOp<MI>::run(b_last[fb][j - NSB], a_frag[fb][i], acc[i][j]);
        else
            MfmaOp<MI>::run(b_frag[j], a_frag[fb][i], acc[i][j]);
    };
    // the same slot, also issuing copy instruction d of the chunk being fetched
    auto mma_and_copy = [&](auto idx_c, auto fb_c, auto d_c, const unsigned char *a_src, const unsigned char *b_src,
                            uint32_t dst_a, uint32_t dst_b) {
        constexpr int idx = decltype(idx_c)::value, fb = decltype(fb_c)::value, d = decltype(d_c)::value;
        constexpr int j = idx / TM, i = idx % TM;
        constexpr int imm = (d < A_DMA ? d : d - A_DMA) * Cfg::WAVES * 1024;
        const unsigned char *src = d < A_DMA ? a_src : b_src;
        const uint32_t dst = d < A_DMA ? dst_a : dst_b;
        constexpr bool nt = STREAM_B && d >= A_DMA;
        if constexpr (j >= NSB)
            mfma_and_dma<MI, imm, nt>(b_last[fb][j - NSB], a_frag[fb][i], acc[i][j], src, voff[d], dst);
        else
            mfma_and_dma<MI, imm, nt>(b_frag[j], a_frag[fb][i], acc[i][j], src, voff[d], dst);
    };

    // ---- pipeline.  Chunk c of A lives in A-ring buffer c % SA, of B in B-ring buffer c % SB.
    // Where the copies of an iteration go (one MFMA "slot" = one MFMA issue):
    //  SPREAD (three or more buffers each): chunk kt+STAGES-1 goes into the buffers that the
    //    barrier of iteration kt-1 released, one instruction at a time across all slots.
    //  DEEP_A (two B buffers, three A buffers): A of chunk kt+2 goes into the A buffer the
    //    previous barrier released, across the slots of the steps before the last one; B of
    //    chunk kt+2 goes into the B buffer this iteration's barrier releases, across the
    //    slots of the last step.  At the next barrier only the B copies are recent.
    //  otherwise (two buffers each): both operands of chunk kt+2 follow this iteration's
    //    barrier, across the slots of the last step.
    constexpr bool SPREAD = STAGES >= 3;
    constexpr bool DEEP_A = (SA == 3 && SB == 2);
    constexpr int AHEAD = SPREAD ? STAGES - 1 : 2;  // chunk kt+AHEAD is copied in iteration kt
    constexpr int LAST0 = (KSTEPS - 1) * NMMA;      // first slot of the last step
    static_assert(TM >= 4 && TN >= 2, "the operand schedule needs at least 4 x 2 MFMA tiles per wave");
    // Slot (0 .. KSTEPS*NMMA-1) in which copy instruction d is issued.  Copies are spread
    // evenly and sit in odd slots (operand reads use even ones): issuing them closer
    // together is slower, and staggering the waves of a workgroup against each other was
    // measured and makes no difference.
    auto copy_slot = [](int d) constexpr -> int {
        if (SPREAD) return d * (KSTEPS * NMMA) / L;
        if (DEEP_A)
            return d < A_DMA ? d * LAST0 / A_DMA + 5 : LAST0 + (d - A_DMA) * NMMA / B_DMA + 3;
        return LAST0 + d * NMMA / L;
    };
    // copy instruction issued in slot `slot`, or -1 (no two copies share a slot)
    auto copy_in_slot = [copy_slot](int slot) constexpr -> int {
        for (int d = 0; d < L; ++d)
            if (copy_slot(d) == slot) return d;
        return -1;
    };
    // copies of this iteration issued before its barrier (the barrier opens the last step)
    constexpr int D_BEFORE = SPREAD ? (LAST0 * L + KSTEPS * NMMA - 1) / (KSTEPS * NMMA) : (DEEP_A ? A_DMA : 0);
    // copies allowed to be still in flight at the barrier while chunk kt+1 must have landed
    constexpr int STEADY_VMCNT = SPREAD ? (STAGES - 3) * L + D_BEFORE : D_BEFORE;
    static_assert(STEADY_VMCNT <= 63, "vmcnt is a 6-bit counter");
    // ring buffer (relative to the current one) that this iteration's copies fill
    constexpr int FILL_OFF_A = SPREAD ? SA - 1 : (DEEP_A ? 2 : 0);
    constexpr int FILL_OFF_B = SPREAD ? SB - 1 : 0;

    static_for<AHEAD>([&](auto s_c) {
        constexpr int st = decltype(s_c)::value;
        static_for<L>([&](auto idx_c) {
            dma_one(idx_c, a_base + st * BK * 2, b_base + st * BK * 2, cp_lds + st * A_BYTES,
                    cp_lds + B_REGION + st * B_BYTES);
        });
    });
    wait_vmcnt<(AHEAD - 1) * L>();
    __syncthreads();
    using K0 = std::integral_constant<int, 0>;
    static_for<TM>([&](auto t) { a_frag[0][decltype(t)::value] = read_a(t, 0u, K0{}); });
    static_for<NSB>([&](auto t) { b_frag[decltype(t)::value] = read_b(t, 0u, K0{}); });
    static_for<NDB>([&](auto t) {
        b_last[0][decltype(t)::value] = read_b(std::integral_constant<int, NSB + decltype(t)::value>{}, 0u, K0{});
    });
    wait_operands(std::integral_constant<int, 0>{});

    const unsigned char *a_next = a_base + AHEAD * BK * 2, *b_next = b_base + AHEAD * BK * 2;
    // One iteration = one K chunk.  ISSUE: chunk kt+AHEAD exists and is copied now.
    // NEXT: chunk kt+1 exists (the barrier is needed and its operands are prefetched).
    // cur_a / cur_b (ring buffers holding chunk kt) are plain ints or, in the unrolled steady
    // state, compile-time constants: then every LDS address below is a constant offset.
    auto iteration = [&](auto cur_a_arg, auto cur_b_arg, auto issue_tag, auto next_tag) {
        constexpr bool ISSUE = decltype(issue_tag)::value, NEXT = decltype(next_tag)::value;
        const int cur_a = ring_index(cur_a_arg), cur_b = ring_index(cur_b_arg);
        const int nxt_a = (cur_a + 1 == SA) ? 0 : cur_a + 1;
        const int nxt_b = (cur_b + 1 == SB) ? 0 : cur_b + 1;
        const int fill_a = (cur_a + FILL_OFF_A) % SA, fill_b = (cur_b + FILL_OFF_B) % SB;
        const unsigned char *a_src = a_next, *b_src = b_next;  // chunk kt + AHEAD
        if constexpr (ISSUE) {
            a_next += BK * 2;
            b_next += BK * 2;
        }
        const uint32_t dst_a = cp_lds + fill_a * A_BYTES, dst_b = cp_lds + B_REGION + fill_b * B_BYTES;
        static_for<KSTEPS>([&](auto kk_c) {
            constexpr int kk = decltype(kk_c)::value;
            constexpr int fb = kk & 1, nb = fb ^ 1;  // an even number of steps: step 0 always uses buffer 0
            constexpr bool last = (kk + 1 == KSTEPS);
            if constexpr (last && NEXT) {
                if constexpr (ISSUE)
                    wait_vmcnt<STEADY_VMCNT>();
                else
                    wait_vmcnt<0>();
                __builtin_amdgcn_s_barrier();
            }
            __builtin_amdgcn_sched_barrier(0);
            // Where the operands of the following step come from: the next step of this
            // chunk, or step 0 of the next chunk (none after the final chunk).
            constexpr bool prefetch = !last || NEXT;
            const uint32_t src_a = (uint32_t)((last ? nxt_a : cur_a) * A_BYTES);
            const uint32_t src_b = (uint32_t)((last ? nxt_b : cur_b) * B_BYTES);
            using SrcKK = std::integral_constant<int, (last ? 0 : kk + 1)>;
            static_for<NMMA>([&](auto idx_c) {
                constexpr int idx = decltype(idx_c)::value;
                constexpr int copy = ISSUE ? copy_in_slot(kk * NMMA + idx) : -1;
                if constexpr (copy >= 0)
                    mma_and_copy(idx_c, std::integral_constant<int, fb>{}, std::integral_constant<int, copy>{}, a_src,
                                 b_src, dst_a, dst_b);
                else
                    mma_one(idx_c, std::integral_constant<int, fb>{});
                if constexpr (prefetch) {
                    // One operand read per slot at most, spread out (an LDS read in the slot
                    // right after another one stalls MFMA issue): A tile t for the next step
                    // at slot RS*t + 2, the double-buffered trailing B tiles at slots 0 and
                    // RS, leading B tile j in place RS slots after its last use (TM*j + TM - 1).
                    constexpr int RS = (NMMA / 2) / TM >= 2 ? (NMMA / 2) / TM : 1;  // 4 for 64 MFMAs, 8 A tiles
                    if constexpr (idx >= 2 && (idx - 2) % RS == 0 && (idx - 2) / RS < TM)
                        a_frag[nb][(idx - 2) / RS] =
                            read_a(std::integral_constant<int, (idx - 2) / RS>{}, src_a, SrcKK{});
                    if constexpr (idx % RS == 0 && idx / RS < NDB)
                        b_last[nb][idx / RS] = read_b(std::integral_constant<int, NSB + idx / RS>{}, src_b, SrcKK{});
                    if constexpr (idx >= TM + RS && (idx - RS) % TM == 0 && (idx - RS) / TM - 1 < NSB)
                        b_frag[(idx - RS) / TM - 1] =
                            read_b(std::integral_constant<int, (idx - RS) / TM - 1>{}, src_b, SrcKK{});
                }
                __builtin_amdgcn_sched_barrier(0);
            });
            // Every operand read issued during this step has landed before control leaves
            // it.  The wait sits here, not at the top of the next step, so that no register
            // copy the compiler may place on a loop edge can see a fragment in flight.
            if constexpr (prefetch) wait_operands(std::integral_constant<int, nb>{});
        });
    };
    using T = std::true_type;
    using F = std::false_type;

    // Steady state, unrolled over one period of the two rings so that the ring indices are
    // constants: no index arithmetic or address computation is left inside the loop.
    constexpr int PERIOD = SA * SB / gcd_of(SA, SB);
    int kt = 0;
    for (; kt + PERIOD <= num_k - AHEAD; kt += PERIOD)
        static_for<PERIOD>([&](auto u_c) {
            constexpr int u = decltype(u_c)::value;
            iteration(std::integral_constant<int, u % SA>{}, std::integral_constant<int, u % SB>{}, T{}, T{});
        });
    int cur_a = 0, cur_b = 0;  // kt is a multiple of the period here
    auto advance = [&] {
        cur_a = (cur_a + 1 == SA) ? 0 : cur_a + 1;
        cur_b = (cur_b + 1 == SB) ? 0 : cur_b + 1;
    };
    for (; kt < num_k - AHEAD; ++kt) {  // chunk kt+AHEAD exists
        iteration(cur_a, cur_b, T{}, T{});
        advance();
    }
    for (; kt < num_k - 1; ++kt) {  // drain: nothing left to copy
        iteration(cur_a, cur_b, F{}, T{});
        advance();
    }
    iteration(cur_a, cur_b, F{}, F{});

    // The MFMAs were issued from assembly, so the compiler neither knows their latency nor
    // sees any reason to keep its own accumulator reads behind them.  Let the last results
    // land, then pass every accumulator through an (empty) ordered statement: reads of the
    // accumulators cannot be scheduled above it.
    asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
    static_for<TM>([&](auto i_c) {
        static_for<TN>([&](auto j_c) { pin_accumulator(acc[decltype(i_c)::value][decltype(j_c)::value]); });
    });
    // ---- epilogue: accumulators -> fp16 -> C (through LDS, whole lines per store)
    if constexpr (SPLIT) {
        __syncthreads();  // every wave has read its last operands: the strips reuse the ring
        auto get = [&](auto i_c, auto j_c) -> floatx4 { return acc[decltype(i_c)::value][decltype(j_c)::value]; };
        const int row0 = tile_m * BM + wm * Cfg::WM, col0 = tile_n * BN + wn * Cfg::WN;
        if (tail_tiles > 0)  // compact: whole tiles [slice][slot][BM][BN], nothing to guard
            store_wave_tile_f32<Cfg, false>(get, lds, partial + ((size_t)slice * tail_tiles + slot) * (BM * BN) +
                                                          (size_t)(wm * Cfg::WM) * BN + wn * Cfg::WN,
                                            BN, BM, BN, wave, lane);
        else
            store_wave_tile_f32<Cfg, EDGE>(get, lds, partial + ((size_t)slice * M + row0) * N + col0, N, M - row0,
                                           N - col0, wave, lane);
    } else {
        (void)partial;
        __syncthreads();
        store_wave_tile<Cfg, Acc, EDGE>(acc, lds, C, M, N, tile_m * BM + wm * Cfg::WM, tile_n * BN + wn * Cfg::WN,
                                        wave, lane);
    }
}

// Shapes a pipelined kernel accepts with guarded edges: any M, N a multiple of 8 (rows of C
// stay 16-byte aligned), K a whole number of chunks and at least the ring depth.
template <class Cfg>
bool pipelined_supports_edges(size_t M, size_t N, size_t K) {
    return M > 0 && N > 0 && N % 8 == 0 && K % Cfg::BK == 0 && K >= (size_t)Cfg::BK * Cfg::STAGES;
}

// C[tile of workgroup id first_block + t] = fp16(sum over slices of partial[slice][t][BM][BN]),
// slices added in order; rows and 8-column pieces outside the matrix are skipped.
template <class Cfg>
__global__ void __launch_bounds__(256)
    tail_reduce_kernel(const float *__restrict__ partial, half_t *__restrict__ C, int M, int N, int K, int tiles_m,
                       int tiles_n, int first_block, int tail_tiles, int splits) {
    constexpr int BM = Cfg::BM, BN = Cfg::BN, PIECES = BM * BN / 8;
    const int t = blockIdx.y;
    int tile_m, tile_n;
    tile_of_position(blocked_order(N, K), first_block + t, tiles_m, tiles_n, tile_m, tile_n);
    const size_t slice_stride = (size_t)tail_tiles * (BM * BN);
    for (int piece = blockIdx.x * blockDim.x + threadIdx.x; piece < PIECES; piece += gridDim.x * blockDim.x) {
        const int r = piece / (BN / 8), c = (piece % (BN / 8)) * 8;
        const int row = tile_m * BM + r, col = tile_n * BN + c;
        if (row >= M || col >= N) continue;
        const float *src = partial + (size_t)t * (BM * BN) + r * BN + c;
        floatx4 s0 = *reinterpret_cast<const floatx4 *>(src);
        floatx4 s1 = *reinterpret_cast<const floatx4 *>(src + 4);
        for (int sl = 1; sl < splits; ++sl) {
            s0 += *reinterpret_cast<const floatx4 *>(src + sl * slice_stride);
            s1 += *reinterpret_cast<const floatx4 *>(src + sl * slice_stride + 4);
        }
        half8 v;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            v[e] = (half_t)s0[e];
            v[4 + e] = (half_t)s1[e];
        }
        store_streaming(reinterpret_cast<half8 *>(C + (size_t)row * N + col), v);
    }
}

}  // namespace hgemm

#include "mfma_chained.h"

namespace hgemm {

// Which of the two kernels runs a tile: the chained one needs a wave tile large enough that
// one wave owns a SIMD (with two or three waves per SIMD their MFMAs interleave and nothing
// is chained), enough workgroups that the chip runs at its power limit (chaining saves power,
// not issue slots) and a K long enough to pay for its longer prologue.  Measured on an MI355X
// against the interleaved kernel, tile by tile, over grids of 64 to 1024 tiles and K from 512
// to 8192: 256x256 ahead (1-4 %) from K = 1536 on once most CUs have a tile, 256x128 and
// 192x192 from K = 4096 on, 128x128 and 64x64 behind everywhere.
enum class PipeKernel { Auto, Interleaved, Chained };
template <class Cfg>
constexpr bool chained_available() {
    return Cfg::MI == 16 && Cfg::PTM * Cfg::PTN >= 32 && Cfg::PTN % 2 == 0 && Cfg::SA >= 3;
}
inline bool chained_pays(int bm, int bn, size_t workgroups, size_t k_len) {
    if (bm == 256 && bn == 256) return (workgroups >= 192 && k_len >= 1536) || k_len >= 8192;
    return k_len >= 4096;
}
template <class Cfg>
bool use_chained(PipeKernel which, size_t workgroups, size_t k_len) {
    if (!chained_available<Cfg>() || which == PipeKernel::Interleaved) return false;
    return which == PipeKernel::Chained || chained_pays(Cfg::BM, Cfg::BN, workgroups, k_len);
}

// B copied with the non-temporal hint (the interleaved kernel's STREAM_B form): for one row of tiles against a
// large B.  There every byte of B is read exactly once and A is one panel that every workgroup shares; B read the
// ordinary way pushes that panel out of L2 and the Infinity Cache (128x128 tile, M = 128, N = 28672, K = 4096:
// 52.8 -> 49.4 us).  From 48 MB of B on, the threshold the small-M split-K kernel uses for the same hint.  With two or
// more rows of tiles B's panels are re-read by the rows below and the hint costs more than it returns, and on the
// 256x128 and 256x256 tiles it is worth 2 % or less against their chained kernels (M = 256, N = 28672: 68.6 -> 67.3 us),
// so only the tiles that run one row against many columns (128x128, 64x128; five stages) carry the second instantiation.
template <class Cfg>
constexpr bool stream_b_available() {
    return Cfg::MI == 16 && Cfg::BN == 128 && (((Cfg::BM == 128 || Cfg::BM == 64) && Cfg::STAGES == 5) || (Cfg::BM == 192 && Cfg::STAGES == 4));
}
inline bool stream_b_pays(int tiles_m, size_t N, size_t K) { return tiles_m == 1 && N * K >= ((size_t)24 << 20); }

// Launches workgroup ids [first_block, first_block + blocks) of the tile grid; tail_tiles
// as in the kernel.
template <class Cfg, bool SPLIT, bool EDGE>
void launch_pipelined_impl(const void *A, const void *B, void *C, float *partial, size_t M, size_t N, size_t K,
                           int splits, int first_block = 0, int blocks = -1, int tail_tiles = 0,
                           PipeKernel which = PipeKernel::Auto) {
    constexpr int subdiv = 0;
    static bool configured = [] {
        HGEMM_CHECK_HIP_ERROR(
            hipFuncSetAttribute(reinterpret_cast<const void *>(&hgemm_pipelined_kernel<Cfg, SPLIT, EDGE>),
                                hipFuncAttributeMaxDynamicSharedMemorySize, Cfg::LDS_BYTES));
        if constexpr (chained_available<Cfg>())
            HGEMM_CHECK_HIP_ERROR(
                hipFuncSetAttribute(reinterpret_cast<const void *>(&hgemm_chained_kernel<Cfg, SPLIT, EDGE>),
                                    hipFuncAttributeMaxDynamicSharedMemorySize, Cfg::LDS_BYTES));
        if constexpr (stream_b_available<Cfg>())
            HGEMM_CHECK_HIP_ERROR(
                hipFuncSetAttribute(reinterpret_cast<const void *>(&hgemm_pipelined_kernel<Cfg, SPLIT, EDGE, true>),
                                    hipFuncAttributeMaxDynamicSharedMemorySize, Cfg::LDS_BYTES));
        return true;
    }();
    (void)configured;
    const int tiles_m = (int)div_ceil(M, (size_t)Cfg::BM), tiles_n = (int)div_ceil(N, (size_t)Cfg::BN);
    if (blocks < 0) blocks = tiles_m * tiles_n - first_block;
    HGEMM_CHECK(first_block >= 0 && blocks >= 1 && first_block + blocks <= tiles_m * tiles_n);
    HGEMM_CHECK(splits >= 1 && (SPLIT || splits == 1) && (size_t)blocks * (size_t)splits < ((size_t)1 << 31));
    if constexpr (stream_b_available<Cfg>()) {
        if (which != PipeKernel::Chained && stream_b_pays(tiles_m, N, K)) {
            hgemm_pipelined_kernel<Cfg, SPLIT, EDGE, true><<<dim3(blocks * splits), dim3(Cfg::THREADS), Cfg::LDS_BYTES, nullptr>>>(
                reinterpret_cast<const half_t *>(A), reinterpret_cast<const half_t *>(B), reinterpret_cast<half_t *>(C),
                partial, (int)M, (int)N, (int)K, splits, tiles_m, tiles_n, first_block, tail_tiles, subdiv);
            HGEMM_CHECK_HIP_ERROR(hipGetLastError());
            return;
        }
    }
    if constexpr (chained_available<Cfg>()) {
        if (use_chained<Cfg>(which, (size_t)blocks * (size_t)splits, shortest_slice(K, Cfg::BK, splits))) {
            hgemm_chained_kernel<Cfg, SPLIT, EDGE><<<dim3(blocks * splits), dim3(Cfg::THREADS), Cfg::LDS_BYTES, nullptr>>>(
                reinterpret_cast<const half_t *>(A), reinterpret_cast<const half_t *>(B), reinterpret_cast<half_t *>(C),
                partial, (int)M, (int)N, (int)K, splits, tiles_m, tiles_n, first_block, tail_tiles, subdiv);
            HGEMM_CHECK_HIP_ERROR(hipGetLastError());
            return;
        }
    }
    HGEMM_CHECK_MSG(which != PipeKernel::Chained, "this tile has no chained kernel");
    hgemm_pipelined_kernel<Cfg, SPLIT, EDGE><<<dim3(blocks * splits), dim3(Cfg::THREADS), Cfg::LDS_BYTES, nullptr>>>(
        reinterpret_cast<const half_t *>(A), reinterpret_cast<const half_t *>(B), reinterpret_cast<half_t *>(C), partial,
        (int)M, (int)N, (int)K, splits, tiles_m, tiles_n, first_block, tail_tiles, subdiv);
    HGEMM_CHECK_HIP_ERROR(hipGetLastError());
}

// Whole rounds of workgroups computed tile by tile, the last `tail_tiles` workgroup ids in
// `tail_splits` K slices (so that they fill the chip as well) with an ordered reduction:
// for grids that end in a nearly empty round.  `partial` holds
// tail_splits * tail_tiles * BM * BN floats.
template <class Cfg>
void launch_pipelined_with_tail(const void *A, const void *B, void *C, float *partial, size_t M, size_t N, size_t K,
                                int tail_tiles, int tail_splits, const char *name) {
    check_operands(A, B, C, M, N, K);
    const int tiles_m = (int)div_ceil(M, (size_t)Cfg::BM), tiles_n = (int)div_ceil(N, (size_t)Cfg::BN);
    const int total = tiles_m * tiles_n, head = total - tail_tiles;
    HGEMM_CHECK(partial != nullptr && tail_tiles >= 1 && head >= 1 && tail_splits >= 2 && K % (size_t)Cfg::BK == 0);
    HGEMM_CHECK_MSG(pipelined_supports_edges<Cfg>(M, N, shortest_slice(K, Cfg::BK, tail_splits)),
                    "%s (tail in %d K slices) needs N %% 8 == 0, K %% %d == 0, shortest slice >= %d (got M=%zu N=%zu K=%zu)",
                    name, tail_splits, Cfg::BK, Cfg::BK * Cfg::STAGES, M, N, K);
    if (Cfg::supports(M, N, K)) {
        launch_pipelined_impl<Cfg, false, false>(A, B, C, nullptr, M, N, K, 1, 0, head);
        launch_pipelined_impl<Cfg, true, false>(A, B, nullptr, partial, M, N, K, tail_splits, head, tail_tiles,
                                                tail_tiles);
    } else {
        launch_pipelined_impl<Cfg, false, true>(A, B, C, nullptr, M, N, K, 1, 0, head);
        launch_pipelined_impl<Cfg, true, true>(A, B, nullptr, partial, M, N, K, tail_splits, head, tail_tiles,
                                               tail_tiles);
    }
    constexpr int PIECES = Cfg::BM * Cfg::BN / 8;
    tail_reduce_kernel<Cfg><<<dim3(PIECES / 256 > 8 ? 8 : (PIECES + 255) / 256, tail_tiles), dim3(256), 0, nullptr>>>(
        partial, reinterpret_cast<half_t *>(C), (int)M, (int)N, (int)K, tiles_m, tiles_n, head, tail_tiles, tail_splits);
    HGEMM_CHECK_HIP_ERROR(hipGetLastError());
}

template <class Cfg>
void launch_pipelined(const void *A, const void *B, void *C, size_t M, size_t N, size_t K, const char *name,
                      PipeKernel which = PipeKernel::Auto) {
    check_operands(A, B, C, M, N, K);
    if (Cfg::supports(M, N, K)) {
        launch_pipelined_impl<Cfg, false, false>(A, B, C, nullptr, M, N, K, 1, 0, -1, 0, which);
        return;
    }
    HGEMM_CHECK_MSG(pipelined_supports_edges<Cfg>(M, N, K),
                    "%s needs N %% 8 == 0, K %% %d == 0, K >= %d (got M=%zu N=%zu K=%zu)", name, Cfg::BK,
                    Cfg::BK * Cfg::STAGES, M, N, K);
    launch_pipelined_impl<Cfg, false, true>(A, B, C, nullptr, M, N, K, 1, 0, -1, 0, which);
}

// K split into `splits` slices: fp32 partial sums of slice s go to partial[s][M][N] (the
// caller provides splits * M * N floats and runs the reduction afterwards).
template <class Cfg>
void launch_pipelined_split(const void *A, const void *B, float *partial, size_t M, size_t N, size_t K, int splits,
                            const char *name) {
    HGEMM_CHECK(splits >= 1 && K % (size_t)Cfg::BK == 0 && partial != nullptr);
    const size_t k_len = shortest_slice(K, Cfg::BK, splits);
    if (k_len > 0 && Cfg::supports(M, N, k_len)) {
        launch_pipelined_impl<Cfg, true, false>(A, B, nullptr, partial, M, N, K, splits);
        return;
    }
    HGEMM_CHECK_MSG(k_len > 0 && pipelined_supports_edges<Cfg>(M, N, k_len),
                    "%s (K in %d slices) needs N %% 8 == 0, K %% %d == 0, shortest slice >= %d (got M=%zu N=%zu K=%zu)",
                    name, splits, Cfg::BK, Cfg::BK * Cfg::STAGES, M, N, K);
    launch_pipelined_impl<Cfg, true, true>(A, B, nullptr, partial, M, N, K, splits);
}

// Whole rounds of workgroups on the Parent tile, the last `tail_tiles` workgroup ids of its
// grid on the smaller Child tile (Parent::BM % Child::BM == 0, likewise BN), each parent tile
// divided among (Parent::BM / Child::BM) * (Parent::BN / Child::BN) workgroups: no partial
// sums, no reduction, one more launch.
template <class Parent, class Child>
void launch_pipelined_with_subtiles(const void *A, const void *B, void *C, size_t M, size_t N, size_t K, int tail_tiles,
                                    const char *name) {
    static_assert(Parent::BM % Child::BM == 0 && Parent::BN % Child::BN == 0,
                  "the child tile must divide the parent tile");
    check_operands(A, B, C, M, N, K);
    constexpr int sub_m = Parent::BM / Child::BM, sub_n = Parent::BN / Child::BN;
    const int tiles_m = (int)div_ceil(M, (size_t)Parent::BM), tiles_n = (int)div_ceil(N, (size_t)Parent::BN);
    const int head = tiles_m * tiles_n - tail_tiles;
    HGEMM_CHECK(tail_tiles >= 1 && head >= 1);
    HGEMM_CHECK_MSG(pipelined_supports_edges<Parent>(M, N, K) && pipelined_supports_edges<Child>(M, N, K),
                    "%s needs N %% 8 == 0, K %% 64 == 0, K >= %d (got M=%zu N=%zu K=%zu)", name,
                    64 * (Parent::STAGES > Child::STAGES ? Parent::STAGES : Child::STAGES), M, N, K);
    if (Parent::supports(M, N, K))
        launch_pipelined_impl<Parent, false, false>(A, B, C, nullptr, M, N, K, 1, 0, head);
    else
        launch_pipelined_impl<Parent, false, true>(A, B, C, nullptr, M, N, K, 1, 0, head);
    const bool edge = !Child::supports(M, N, K);
    auto kernel = edge ? &hgemm_pipelined_kernel<Child, false, true> : &hgemm_pipelined_kernel<Child, false, false>;
    static bool configured = [] {
        HGEMM_CHECK_HIP_ERROR(hipFuncSetAttribute(reinterpret_cast<const void *>(&hgemm_pipelined_kernel<Child, false, true>),
                                                  hipFuncAttributeMaxDynamicSharedMemorySize, Child::LDS_BYTES));
        HGEMM_CHECK_HIP_ERROR(hipFuncSetAttribute(reinterpret_cast<const void *>(&hgemm_pipelined_kernel<Child, false, false>),
                                                  hipFuncAttributeMaxDynamicSharedMemorySize, Child::LDS_BYTES));
        return true;
    }();
    (void)configured;
    kernel<<<dim3(tail_tiles * sub_m * sub_n), dim3(Child::THREADS), Child::LDS_BYTES, nullptr>>>(
        reinterpret_cast<const half_t *>(A), reinterpret_cast<const half_t *>(B), reinterpret_cast<half_t *>(C), nullptr,
        (int)M, (int)N, (int)K, 1, tiles_m, tiles_n, head, 0, (sub_m << 8) | sub_n);
    HGEMM_CHECK_HIP_ERROR(hipGetLastError());
}

}  // namespace hgemm
