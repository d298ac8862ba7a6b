// Block-tiled HGEMM for gfx950 on v_mfma_f32_32x32x16_f16, fp32 accumulate.
//
// One workgroup computes a BM x BN tile of C.  Both operands are K-contiguous
// (A[m][k], B[n][k]), so A and B tiles are staged the same way: rows of BK halves in LDS,
// read back as 16-byte fragments (8 consecutive k of one row per lane) which is exactly
// the MFMA operand layout -- no transpose anywhere.
//
// The MFMA is issued with swapped operands (B fragment as the first operand): lane l of
// the accumulator then holds, for row m = l%32 of the 32x32 tile, four consecutive n
// (8*(r/4) + 4*(l/32) + r%4), so C is written with packed 8-byte stores.
//
// Compile-time knobs mirror the steps of the reference's kernel ladder
// (reference src/mma/mma_base.cu .. src/mma/mma_async_stage4.cu):
//   LOADER  REG  global -> VGPR -> LDS            (int4 copies, reference mma_base.cu:96-119)
//           DMA  global -> LDS, bypassing VGPRs   (cp.async, reference mma_async.cu:105-111)
//   LAYOUT  LINEAR / PADDED (reference wmma_padding.cu:38-42) /
//           SWIZZLE (XOR of the 16-byte chunk index with the row, reference mma_permuted.cu:105-108)
//   STAGES  LDS ring depth (reference mma_async_stage4.cu:52 K_STAGE)
//   FRAG_PREFETCH  double-buffered operand registers (reference mma_async_pg2s_ps2r.cu:184-185)
//   LOOKAHEAD  (no counterpart in the reference) the barrier of an iteration confirms the *next* chunk, whose
//           operands are all read into a second set of registers while the MFMAs of the current chunk run: for wave
//           tiles of one or two MFMAs per k-step, where a read issued one step ahead is still in flight when needed
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

#include "common.h"
#include "tile_order.h"

namespace hgemm {

typedef _Float16 half_t;
typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half4 __attribute__((ext_vector_type(4)));
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

enum { LOAD_REG = 0, LOAD_DMA = 1 };
enum { LDS_LINEAR = 0, LDS_PADDED = 1, LDS_SWIZZLE = 2 };

template <int BM_, int BN_, int BK_, int WAVES_M_, int WAVES_N_, int STAGES_, int LOADER_, int LAYOUT_,
          bool FRAG_PREFETCH_, bool LOOKAHEAD_ = false>
struct TileConfig {
    static constexpr int BM = BM_, BN = BN_, BK = BK_;
    static constexpr int WAVES_M = WAVES_M_, WAVES_N = WAVES_N_;
    static constexpr int STAGES = STAGES_, LOADER = LOADER_, LAYOUT = LAYOUT_;
    static constexpr bool FRAG_PREFETCH = FRAG_PREFETCH_, LOOKAHEAD = LOOKAHEAD_;

    static constexpr int WAVES = WAVES_M * WAVES_N;
    static constexpr int THREADS = WAVES * 64;
    static constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;  // wave tile
    static constexpr int TM = WM / 32, TN = WN / 32;            // 32x32 MFMA tiles per wave
    static constexpr int KSTEPS = BK / 16;                      // MFMA k-steps per chunk
    static constexpr int CPR = BK / 8;                          // 16-byte chunks per row
    static constexpr int ROW_BYTES = BK * 2 + (LAYOUT == LDS_PADDED ? 16 : 0);
    static constexpr int A_BYTES = BM * ROW_BYTES, B_BYTES = BN * ROW_BYTES;
    static constexpr int STAGE_BYTES = A_BYTES + B_BYTES;
    static constexpr int RING_BYTES = STAGES * STAGE_BYTES;
    // the C tile is staged through LDS on its way out: one 32-row strip per wave
    static constexpr int C_STRIP_BYTES = 32 * (WN * 2 + 16);
    static constexpr int LDS_BYTES = RING_BYTES > WAVES * C_STRIP_BYTES ? RING_BYTES : WAVES * C_STRIP_BYTES;
    // register-staged copy: each thread moves this many 16-byte chunks per tile
    static constexpr int A_ITERS = BM * CPR / THREADS, B_ITERS = BN * CPR / THREADS;
    // direct-to-LDS copy: one wave instruction fills 1024 contiguous LDS bytes
    static constexpr int ROWS_PER_DMA = 1024 / (BK * 2);
    static constexpr int A_DMA = A_BYTES / 1024 / WAVES, B_DMA = B_BYTES / 1024 / WAVES;
    static constexpr int LOADS_PER_STAGE = (LOADER == LOAD_DMA) ? (A_DMA + B_DMA) : (A_ITERS + B_ITERS);

    static_assert(BK == 32 || BK == 64, "K chunk must be 32 or 64 halves");
    static_assert(WM % 32 == 0 && WN % 32 == 0, "wave tile must be a multiple of the 32x32 MFMA tile");
    static_assert((BM * CPR) % THREADS == 0 && (BN * CPR) % THREADS == 0, "tile copy must divide evenly");
    static_assert(LOADER == LOAD_REG || LAYOUT != LDS_PADDED, "direct-to-LDS rows are contiguous: no padding");
    static_assert(LOADER == LOAD_REG || (A_BYTES % (1024 * WAVES) == 0 && B_BYTES % (1024 * WAVES) == 0),
                  "direct-to-LDS copy must divide evenly over the waves");
    static_assert(STAGES >= 1 && STAGES <= 10, "1..10 LDS stages");
    static_assert(LDS_BYTES <= 160 * 1024, "exceeds the 160 KB LDS of a gfx950 CU");
    static_assert((STAGES - 1) * LOADS_PER_STAGE <= 63, "vmcnt is a 6-bit counter");
    static_assert(!LOOKAHEAD || (LOADER == LOAD_DMA && FRAG_PREFETCH && STAGES >= 3 && KSTEPS % 2 == 0),
                  "the look-ahead loop is written for the direct-to-LDS ring with double-buffered operands");

    static bool supports(size_t M, size_t N, size_t K) {
        return M % BM == 0 && N % BN == 0 && K % BK == 0 && K >= (size_t)BK * (STAGES > 1 ? STAGES - 1 : 1);
    }
};

// K in slices of whole chunks, as even as that allows: the first `chunks % slices` slices walk one chunk more.
// Slice `slice` starts at chunk `first` and walks `count`.
__host__ __device__ __forceinline__ void slice_of_k(int chunks, int slices, int slice, int &first, int &count) {
    const int base = chunks / slices, longer = chunks % slices;
    first = slice * base + (slice < longer ? slice : longer);
    count = base + (slice < longer ? 1 : 0);
}
// the length of the shortest of `splits` such slices of K (chunks of `bk`), which is what a kernel's minimum K applies to
inline size_t shortest_slice(size_t K, int bk, int splits) { return K / (size_t)bk / (size_t)splits * (size_t)bk; }

// s_waitcnt vmcnt(n) only (expcnt / lgkmcnt left at "do not wait"); gfx9 encoding.
template <int N>
__device__ __forceinline__ void wait_vmcnt() {
    static_assert(N >= 0 && N <= 63, "vmcnt range");
    __builtin_amdgcn_s_waitcnt((N & 0xf) | ((N >> 4) << 14) | (0x7 << 4) | (0xf << 8));
}

// 16 bytes per lane from global memory straight into LDS.  The wave's 64 lanes land in
// 1024 consecutive LDS bytes starting at the (wave-uniform) address in M0.  Written as
// inline assembly so the compiler's wait-count insertion does not serialise LDS reads of
// one stage behind copies into another; the kernel places its own s_waitcnt vmcnt(n).
// M0 is written here without the compiler's knowledge (it is a reserved register: hipcc
// warns that a clobber of it is not honoured).  gfx9 LDS instructions do not read M0 and
// these kernels contain nothing else the compiler lowers through it (no indirect register
// indexing, no compiler-generated LDS-DMA, no GWS), so nothing else depends on its value.
__device__ __forceinline__ void dma_load16(const void *gptr, uint32_t lds_addr) {
    asm volatile(
        "s_mov_b32 m0, %0\n\t"
        "s_nop 0\n\t"
        "global_load_lds_dwordx4 %1, off"
        :
        : "s"(lds_addr), "v"(gptr)
        : "memory");
}

// The same copy with the non-temporal hint, for operands that are read once (B of the small-M kernels).
__device__ __forceinline__ void dma_load16_streaming(const void *gptr, uint32_t lds_addr) {
    asm volatile(
        "s_mov_b32 m0, %0\n\t"
        "s_nop 0\n\t"
        "global_load_lds_dwordx4 %1, off nt"
        :
        : "s"(lds_addr), "v"(gptr)
        : "memory");
}

// XOR applied to the 16-byte chunk index of LDS row `row` (rows are BK*2 bytes).
// One 128-byte bank line holds 128/(BK*2) rows; consecutive bank lines get consecutive
// XOR values, and bit 3 of the line index is folded in so that 16 consecutive lines
// still map to 16 distinct (line parity, chunk) pairs.
template <class Cfg>
__device__ __forceinline__ int swizzle_of_row(int row) {
    if (Cfg::LAYOUT != LDS_SWIZZLE) return 0;
    constexpr int ROWS_PER_LINE = 128 / (Cfg::BK * 2);
    const int line = row / ROWS_PER_LINE;
    return ((line & 7) ^ ((line >> 3) & 1)) & (Cfg::CPR - 1);
}

// Lanes of one wave exchange data through LDS in the epilogues below.  The hardware executes a wave's LDS
// instructions in order, so no wait is needed between a store and the load that picks the data up in another lane;
// but the compiler reasons lane by lane: where it can prove that the bytes a lane stores and the bytes the same lane
// loads never coincide, it is free to issue the load first (it did, for some tile shapes: stale strip contents in
// the output).  What the exchange needs is what the language calls it: the stores released and the loads acquired
// at wavefront scope, around a wave barrier.  None of the three emits an instruction; they keep the stores and the
// loads on their own sides.
__device__ __forceinline__ void wave_lds_exchange_point() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// C is written once and never read back by these kernels: stored with the non-temporal hint its lines do not
// displace the A and B panels that other workgroups are about to read from L2 and the Infinity Cache (measured on
// the tuned kernels: 2 % at 8192^3, 9-12 % on 8192^2 ... 16384^2 x 512, where C is most of the traffic).
template <class T>
__device__ __forceinline__ void store_streaming(T *dst, const T &value) {
    __builtin_nontemporal_store(value, dst);
}

// Epilogue shared by the tiled kernels: accumulators -> fp16 -> C, staged through LDS.
// A lane of the (operand-swapped) accumulator holds four consecutive n of one row; stored
// straight to global memory that is 16 useful bytes per 32 rows per instruction, i.e. a
// flood of partial-line write requests.  Instead each wave parks 32 rows of its tile in a
// private LDS strip (row stride WN*2 + 16 bytes) and reads them back row-contiguous, so
// every global store instruction writes whole 128-byte lines, 16 bytes per lane.
// The caller must have passed a workgroup barrier after the last operand read, because
// the strips reuse the operand buffers.
template <class Cfg>
__device__ __forceinline__ void store_tile_via_lds(const floatx16 (&acc)[Cfg::TM][Cfg::TN], unsigned char *lds,
                                                   half_t *__restrict__ C, int N, int row0, int col0, int wave,
                                                   int lane) {
    constexpr int TM = Cfg::TM, TN = Cfg::TN, WN = Cfg::WN;
    constexpr int STRIP_ROW_BYTES = WN * 2 + 16;
    constexpr int STRIP_BYTES = 32 * STRIP_ROW_BYTES;
    constexpr int LANES_PER_ROW = WN / 8;            // 16-byte pieces per row
    constexpr int ROWS_PER_READ = 64 / LANES_PER_ROW;
    constexpr int READS = 32 / ROWS_PER_READ;
    static_assert(STRIP_BYTES == Cfg::C_STRIP_BYTES, "strip size");
    unsigned char *strip = lds + wave * STRIP_BYTES;
    unsigned char *wr = strip + (lane & 31) * STRIP_ROW_BYTES + ((lane >> 5) << 3);
    const int rd_row = lane / LANES_PER_ROW, rd_col = lane % LANES_PER_ROW;
    const unsigned char *rd = strip + rd_row * STRIP_ROW_BYTES + rd_col * 16;
    half_t *cp = C + (size_t)(row0 + rd_row) * N + col0 + rd_col * 8;
#pragma unroll
    for (int i = 0; i < TM; ++i) {
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                half4 v;
#pragma unroll
                for (int r = 0; r < 4; ++r) v[r] = (half_t)acc[i][j][g * 4 + r];
                *reinterpret_cast<half4 *>(wr + (j * 32 + g * 8) * 2) = v;
            }
        wave_lds_exchange_point();
#pragma unroll
        for (int it = 0; it < READS; ++it) {
            const u32x4 v = *reinterpret_cast<const u32x4 *>(rd + it * ROWS_PER_READ * STRIP_ROW_BYTES);
            store_streaming(reinterpret_cast<u32x4 *>(cp + (size_t)(i * 32 + it * ROWS_PER_READ) * N), v);
        }
        wave_lds_exchange_point();
    }
}

// SPLIT: a one-dimensional launch of tiles x slices workgroups; each computes one K slice of one tile and leaves
// fp32 partial sums in partial[slice][M][N] for the ordered reduction; otherwise slices == 1 and C is written.
// The K / BK chunks are dealt to the slices as evenly as whole chunks allow (`slice_of_k`).
template <class Cfg, bool SPLIT = false>
__global__ void __launch_bounds__(Cfg::THREADS)
    hgemm_tiled_kernel(const half_t *__restrict__ A, const half_t *__restrict__ B, half_t *__restrict__ C,
                       float *__restrict__ partial, int M, int N, int K, int slices, int tiles_m, int tiles_n) {
    constexpr int BM = Cfg::BM, BN = Cfg::BN, BK = Cfg::BK;
    constexpr int TM = Cfg::TM, TN = Cfg::TN, KSTEPS = Cfg::KSTEPS, CPR = Cfg::CPR;
    constexpr int ROW_BYTES = Cfg::ROW_BYTES, STAGES = Cfg::STAGES, THREADS = Cfg::THREADS;
    (void)M;

    extern __shared__ __attribute__((aligned(1024))) unsigned char lds[];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / Cfg::WAVES_N, wn = wave % Cfg::WAVES_N;

    int tile_m, tile_n, slice = 0;
    if constexpr (SPLIT) {
        int slot;
        slice_and_slot_of_workgroup((int)blockIdx.x, tiles_m * tiles_n, slices, slice, slot);
        tile_of_position(blocked_order(N, K), slot, tiles_m, tiles_n, tile_m, tile_n);
        slice = __builtin_amdgcn_readfirstlane(slice);
    } else {
        tile_of_workgroup(blocked_order(N, K), 0, (int)blockIdx.x, (int)gridDim.x, tiles_m, tiles_n, tile_m, tile_n);
    }

    int first_chunk, num_k;
    slice_of_k(K / BK, slices, slice, first_chunk, num_k);
    const int k_begin = first_chunk * BK;
    const half_t *Ag = A + (size_t)tile_m * BM * K + k_begin;
    const half_t *Bg = B + (size_t)tile_n * BN * K + k_begin;

    // ---------------- global -> LDS copy set-up ----------------
    // REG: thread t moves chunk (row = t / CPR + it * THREADS/CPR, ch = t % CPR).
    // DMA: wave w, instruction i fills LDS rows [(i*WAVES + w) * ROWS_PER_DMA, +ROWS_PER_DMA);
    //      lane l lands on physical chunk l % CPR of row l / CPR, so it fetches the logical
    //      chunk that the swizzle maps there.
    const half_t *a_src;
    const half_t *b_src;
    uint32_t cp_lds_off;  // byte offset inside the A (or B) tile of this thread's first chunk
    if constexpr (Cfg::LOADER == LOAD_REG) {
        const int row = tid / CPR, ch = tid % CPR;
        a_src = Ag + (size_t)row * K + ch * 8;
        b_src = Bg + (size_t)row * K + ch * 8;
        cp_lds_off = row * ROW_BYTES + ((ch ^ swizzle_of_row<Cfg>(row)) << 4);
    } else {
        const int row = wave * Cfg::ROWS_PER_DMA + lane / CPR;
        const int ch = (lane % CPR) ^ swizzle_of_row<Cfg>(row);
        a_src = Ag + (size_t)row * K + ch * 8;
        b_src = Bg + (size_t)row * K + ch * 8;
        cp_lds_off = wave * 1024;  // wave-uniform base; lanes are placed by the hardware
    }
    constexpr int REG_ROW_STEP = THREADS / CPR;                    // rows between a thread's REG chunks
    constexpr int DMA_ROW_STEP = Cfg::WAVES * Cfg::ROWS_PER_DMA;   // rows between a wave's DMA instructions

    u32x4 ra[Cfg::LOADER == LOAD_REG ? Cfg::A_ITERS : 1];
    u32x4 rb[Cfg::LOADER == LOAD_REG ? Cfg::B_ITERS : 1];

    auto global_fetch = [&](int kt) {  // REG loader: global -> VGPR
        const int koff = kt * BK;
#pragma unroll
        for (int it = 0; it < Cfg::A_ITERS; ++it)
            ra[it] = *reinterpret_cast<const u32x4 *>(a_src + (size_t)it * REG_ROW_STEP * K + koff);
#pragma unroll
        for (int it = 0; it < Cfg::B_ITERS; ++it)
            rb[it] = *reinterpret_cast<const u32x4 *>(b_src + (size_t)it * REG_ROW_STEP * K + koff);
    };
    auto lds_commit = [&](int stage) {  // REG loader: VGPR -> LDS
        unsigned char *sa = lds + stage * Cfg::STAGE_BYTES + cp_lds_off;
        unsigned char *sb = sa + Cfg::A_BYTES;
#pragma unroll
        for (int it = 0; it < Cfg::A_ITERS; ++it)
            *reinterpret_cast<u32x4 *>(sa + it * REG_ROW_STEP * ROW_BYTES) = ra[it];
#pragma unroll
        for (int it = 0; it < Cfg::B_ITERS; ++it)
            *reinterpret_cast<u32x4 *>(sb + it * REG_ROW_STEP * ROW_BYTES) = rb[it];
    };
    auto dma_fetch = [&](int kt, int stage) {  // DMA loader: global -> LDS
        const int koff = kt * BK;
        const uint32_t base =
            (uint32_t)(uintptr_t)(lds) + (uint32_t)(stage * Cfg::STAGE_BYTES) + cp_lds_off;
#pragma unroll
        for (int it = 0; it < Cfg::A_DMA; ++it)
            dma_load16(a_src + (size_t)it * DMA_ROW_STEP * K + koff, base + it * Cfg::WAVES * 1024);
#pragma unroll
        for (int it = 0; it < Cfg::B_DMA; ++it)
            dma_load16(b_src + (size_t)it * DMA_ROW_STEP * K + koff,
                       base + Cfg::A_BYTES + it * Cfg::WAVES * 1024);
    };

    // ---------------- LDS -> MFMA operand set-up ----------------
    const int frag_row = lane & 31;
    const int frag_x = (lane >> 5) ^ swizzle_of_row<Cfg>(frag_row);  // chunk index XOR term
    const uint32_t a_frag_off = (wm * Cfg::WM + frag_row) * ROW_BYTES;
    const uint32_t b_frag_off = Cfg::A_BYTES + (wn * Cfg::WN + frag_row) * ROW_BYTES;

    floatx16 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

    auto load_frags = [&](int stage, int kk, half8 (&af)[TM], half8 (&bf)[TN]) {
        const unsigned char *s = lds + stage * Cfg::STAGE_BYTES;
        const uint32_t chunk = (uint32_t)((kk * 2) ^ frag_x) << 4;
#pragma unroll
        for (int i = 0; i < TM; ++i)
            af[i] = *reinterpret_cast<const half8 *>(s + a_frag_off + i * 32 * ROW_BYTES + chunk);
#pragma unroll
        for (int j = 0; j < TN; ++j)
            bf[j] = *reinterpret_cast<const half8 *>(s + b_frag_off + j * 32 * ROW_BYTES + chunk);
    };
    auto mma_step = [&](const half8 (&af)[TM], const half8 (&bf)[TN]) {
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j) {
                const int jj = (i & 1) ? (TN - 1 - j) : j;  // serpentine over the wave tile
                acc[i][jj] = __builtin_amdgcn_mfma_f32_32x32x16_f16(bf[jj], af[i], acc[i][jj], 0, 0, 0);
            }
    };
    auto compute_stage = [&](int stage) {
        if constexpr (Cfg::FRAG_PREFETCH) {
            half8 af[2][TM], bf[2][TN];
            load_frags(stage, 0, af[0], bf[0]);
#pragma unroll
            for (int kk = 0; kk < KSTEPS; ++kk) {
                if (kk + 1 < KSTEPS) load_frags(stage, kk + 1, af[(kk + 1) & 1], bf[(kk + 1) & 1]);
                mma_step(af[kk & 1], bf[kk & 1]);
            }
        } else {
            half8 af[TM], bf[TN];
#pragma unroll
            for (int kk = 0; kk < KSTEPS; ++kk) {
                load_frags(stage, kk, af, bf);
                mma_step(af, bf);
            }
        }
    };

    // ---------------- main loop ----------------
    if constexpr (Cfg::LOADER == LOAD_REG) {
        if constexpr (STAGES == 1) {
            // fetch, commit, multiply, one chunk at a time
            for (int kt = 0; kt < num_k; ++kt) {
                global_fetch(kt);
                lds_commit(0);
                __syncthreads();
                compute_stage(0);
                __syncthreads();
            }
        } else {
            // two or more LDS buffers: registers hold chunk kt+1 while chunk kt is multiplied
            global_fetch(0);
            lds_commit(0);
            __syncthreads();
            for (int kt = 0; kt < num_k; ++kt) {
                const int cur = kt % STAGES, nxt = (kt + 1) % STAGES;
                if (kt + 1 < num_k) global_fetch(kt + 1);
                compute_stage(cur);
                if (kt + 1 < num_k) lds_commit(nxt);
                __syncthreads();
            }
        }
    } else {
        constexpr int L = Cfg::LOADS_PER_STAGE;
        if constexpr (STAGES == 1) {
            for (int kt = 0; kt < num_k; ++kt) {
                dma_fetch(kt, 0);
                wait_vmcnt<0>();
                __syncthreads();
                compute_stage(0);
                __syncthreads();
            }
        } else if constexpr (Cfg::LOOKAHEAD) {
            // Ring of STAGES buffers, barrier one chunk ahead, whole chunks of operands in registers.  At the top
            // of iteration kt every operand of chunk kt is already on its way into registers; the wait and the
            // barrier confirm chunk kt+1 (and retire every wave's reads of chunk kt-1, whose buffer the new copy
            // refills), then the wave issues all operand reads of chunk kt+1, the copy of chunk kt+STAGES-1, and
            // only then the MFMAs of chunk kt.  With one or two MFMAs per k-step (small wave tiles) a read issued one
            // step ahead is still in flight when its MFMA comes up; a chunk ahead, LDS latency is off the chain.
#pragma unroll
            for (int s = 0; s < STAGES - 1; ++s) dma_fetch(s, s);  // supports() guarantees num_k >= STAGES-1
            wait_vmcnt<(STAGES - 2) * L>();
            __syncthreads();
            half8 af[2][KSTEPS][TM], bf[2][KSTEPS][TN];
            auto load_chunk = [&](int stage, half8 (&a)[KSTEPS][TM], half8 (&b)[KSTEPS][TN]) {
#pragma unroll
                for (int kk = 0; kk < KSTEPS; ++kk) load_frags(stage, kk, a[kk], b[kk]);
            };
            load_chunk(0, af[0], bf[0]);
            int cur = 0, fill = STAGES - 1;
            // STEADY: the copy of chunk kt+STAGES-1 exists (so does chunk kt+1, and the wait count is the full one);
            // the last iterations (the odd one left by the unrolled pairs and those after the last copy) take their
            // decisions at run time.
            auto iteration = [&](auto steady, int kt, half8 (&ca)[KSTEPS][TM], half8 (&cb)[KSTEPS][TN],
                                 half8 (&na)[KSTEPS][TM], half8 (&nb)[KSTEPS][TN]) {
                constexpr bool STEADY = decltype(steady)::value;
                const int nxt = (cur + 1 == STAGES) ? 0 : cur + 1;
                if (STEADY || kt + 1 < num_k) {
                    // copies issued so far: chunks up to min(kt+STAGES-2, num_k-1); all but those beyond kt+1 must land
                    if (STEADY || num_k - 1 - (kt + 1) >= STAGES - 3) {
                        wait_vmcnt<(STAGES - 3) * L>();
                    } else {
                        wait_vmcnt<0>();
                    }
                    // a bare barrier: the fence of __syncthreads() would wait for this wave's own operand reads of
                    // chunk kt, which nothing behind the barrier overwrites (the refilled buffer held chunk kt-1,
                    // consumed by MFMAs already issued)
                    __builtin_amdgcn_sched_barrier(0);  // the MFMAs of chunk kt-1 (and their waits) stay in front
                    asm volatile("s_barrier" ::: "memory");
                    load_chunk(nxt, na, nb);
                }
                if (STEADY || kt + STAGES - 1 < num_k) dma_fetch(kt + STAGES - 1, fill);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int kk = 0; kk < KSTEPS; ++kk) mma_step(ca[kk], cb[kk]);
                cur = nxt;
                fill = (fill + 1 == STAGES) ? 0 : fill + 1;
            };
            const int steady_end = num_k - (STAGES - 1);
            int kt = 0;
            for (; kt + 2 <= steady_end; kt += 2) {
                iteration(std::true_type{}, kt, af[0], bf[0], af[1], bf[1]);
                iteration(std::true_type{}, kt + 1, af[1], bf[1], af[0], bf[0]);
            }
            for (; kt < num_k; kt += 2) {
                iteration(std::false_type{}, kt, af[0], bf[0], af[1], bf[1]);
                if (kt + 1 < num_k) iteration(std::false_type{}, kt + 1, af[1], bf[1], af[0], bf[0]);
            }
        } else {
            // Ring of STAGES buffers.  At the top of iteration kt the copies of chunks
            // kt .. kt+STAGES-2 are in flight; wait for the oldest, meet at the barrier
            // (which also retires every wave's reads of the buffer about to be refilled),
            // start the copy of chunk kt+STAGES-1, multiply chunk kt.
#pragma unroll
            for (int s = 0; s < STAGES - 1; ++s) dma_fetch(s, s);  // supports() guarantees num_k >= STAGES-1
            int cur = 0, fill = STAGES - 1;
            for (int kt = 0; kt < num_k; ++kt) {
                const int in_flight_after = num_k - 1 - kt;  // chunks issued beyond kt
                if (in_flight_after >= STAGES - 2) {
                    wait_vmcnt<(STAGES - 2) * L>();
                } else {
                    wait_vmcnt<0>();
                }
                __syncthreads();
                if (kt + STAGES - 1 < num_k) dma_fetch(kt + STAGES - 1, fill);
                compute_stage(cur);
                cur = (cur + 1 == STAGES) ? 0 : cur + 1;
                fill = (fill + 1 == STAGES) ? 0 : fill + 1;
            }
        }
    }

    if constexpr (SPLIT) {
        // Lane l holds row l % 32 of each 32x32 tile and, per register group g, four consecutive n at
        // 8 g + 4 (l / 32): 16 bytes of an fp32 partial sum.
        float *dst = partial + ((size_t)slice * M + tile_m * BM + wm * Cfg::WM + (lane & 31)) * N + tile_n * BN +
                     wn * Cfg::WN + ((lane >> 5) << 2);
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    floatx4 v;
#pragma unroll
                    for (int r = 0; r < 4; ++r) v[r] = acc[i][j][g * 4 + r];
                    *reinterpret_cast<floatx4 *>(dst + (size_t)(i * 32) * N + j * 32 + g * 8) = v;
                }
        return;
    }
    // ---------------- epilogue: accumulators -> fp16 -> C ----------------
    __syncthreads();
    store_tile_via_lds<Cfg>(acc, lds, C, N, tile_m * BM + wm * Cfg::WM, tile_n * BN + wn * Cfg::WN, wave, lane);
}

// Host launcher shared by every tiled entry point.  Sets the dynamic-LDS limit once per
// instantiation (counterpart of the reference's one-time cudaFuncSetAttribute,
// src/mma/mma_async_stage4.cu:619-635), checks the launch, does not synchronise.
template <class Cfg>
void launch_tiled(const void *A, const void *B, void *C, size_t M, size_t N, size_t K, const char *name) {
    check_operands(A, B, C, M, N, K);
    HGEMM_CHECK_MSG(Cfg::supports(M, N, K),
                    "%s needs M %% %d == 0, N %% %d == 0, K %% %d == 0, K >= %d (got M=%zu N=%zu K=%zu)", name,
                    Cfg::BM, Cfg::BN, Cfg::BK, Cfg::BK * (Cfg::STAGES > 1 ? Cfg::STAGES - 1 : 1), M, N, K);
    static bool configured = [] {
        HGEMM_CHECK_HIP_ERROR(hipFuncSetAttribute(reinterpret_cast<const void *>(&hgemm_tiled_kernel<Cfg>),
                                                  hipFuncAttributeMaxDynamicSharedMemorySize, Cfg::LDS_BYTES));
        return true;
    }();
    (void)configured;
    const int tiles_m = (int)(M / Cfg::BM), tiles_n = (int)(N / Cfg::BN);
    hgemm_tiled_kernel<Cfg><<<dim3(tiles_m * tiles_n), dim3(Cfg::THREADS), Cfg::LDS_BYTES, nullptr>>>(
        reinterpret_cast<const half_t *>(A), reinterpret_cast<const half_t *>(B), reinterpret_cast<half_t *>(C), nullptr,
        (int)M, (int)N, (int)K, 1, tiles_m, tiles_n);
    HGEMM_CHECK_HIP_ERROR(hipGetLastError());
}

// K in `splits` slices: fp32 partial sums of slice s go to partial[s][M][N]; the caller runs the ordered reduction.
template <class Cfg>
void launch_tiled_split(const void *A, const void *B, float *partial, size_t M, size_t N, size_t K, int splits,
                        const char *name) {
    HGEMM_CHECK(splits >= 1 && K % (size_t)Cfg::BK == 0 && partial != nullptr && splits <= 65535);
    const size_t k_len = shortest_slice(K, Cfg::BK, splits);
    HGEMM_CHECK_MSG(k_len > 0 && Cfg::supports(M, N, k_len),
                    "%s (K in %d slices) needs M %% %d == 0, N %% %d == 0, K %% %d == 0, shortest slice >= %d (got M=%zu N=%zu K=%zu)",
                    name, splits, Cfg::BM, Cfg::BN, Cfg::BK, Cfg::BK * (Cfg::STAGES > 1 ? Cfg::STAGES - 1 : 1), M, N, K);
    static bool configured = [] {
        HGEMM_CHECK_HIP_ERROR(hipFuncSetAttribute(reinterpret_cast<const void *>(&hgemm_tiled_kernel<Cfg, true>),
                                                  hipFuncAttributeMaxDynamicSharedMemorySize, Cfg::LDS_BYTES));
        return true;
    }();
    (void)configured;
    const int tiles_m = (int)(M / Cfg::BM), tiles_n = (int)(N / Cfg::BN);
    HGEMM_CHECK((size_t)tiles_m * tiles_n * (size_t)splits < ((size_t)1 << 31));
    hgemm_tiled_kernel<Cfg, true><<<dim3(tiles_m * tiles_n * splits), dim3(Cfg::THREADS), Cfg::LDS_BYTES, nullptr>>>(
        reinterpret_cast<const half_t *>(A), reinterpret_cast<const half_t *>(B), nullptr, partial, (int)M, (int)N, (int)K,
        splits, tiles_m, tiles_n);
    HGEMM_CHECK_HIP_ERROR(hipGetLastError());
}

}  // namespace hgemm
