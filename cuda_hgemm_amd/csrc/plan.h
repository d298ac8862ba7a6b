// Kernel selection record shared by the dispatcher and its reporting helpers.
#pragma once

#include <stddef.h>

namespace hgemm {

enum KernelId {
    KERNEL_NONE = 0,
    KERNEL_BIG256,      // pipelined 256x256x64, 4 waves
    KERNEL_MID128,      // pipelined 128x128x64, 4 waves, 5-stage ring
    KERNEL_SMALL64,     // pipelined 64x64x64, 1 wave, 3-stage ring
    KERNEL_SPLIT_32x64,   // split-K family: BM x BN tile, 4-stage ring, M guarded
    KERNEL_SPLIT_64x64,
    KERNEL_SPLIT_64x128,
    KERNEL_SPLIT_128x64,
    KERNEL_SPLIT_128x128,
    KERNEL_SIMT,        // scalar fallback for shapes no MFMA kernel tiles
    KERNEL_T192,        // pipelined 192x192x64, 4 waves, 3-stage ring
    KERNEL_R256x128,    // pipelined 256x128x64, 4 waves, 3-stage ring
    KERNEL_RAGGED,      // guarded 128x128x32 MFMA kernel: any shape
    KERNEL_DECODE_BN16, // streaming kernel for M <= 8: 16 or 32 columns per workgroup, `splits` waves over K
    KERNEL_DECODE_BN32,
    KERNEL_SMALL64_W4,  // 64x64x64 tile on four waves of 32x32 (the ladder's kernel): grids of at most one tile per CU
    KERNEL_MID128_S2,   // pipelined 128x128x64, 4 waves, 2-stage ring: two workgroups per CU, for K of at most four chunks
    KERNEL_DECODE_RING, // decode kernel for M <= 128 whose waves stage operands through LDS rings of their own; `splits` waves over K
    KERNEL_PADDED,      // operands copied zero-padded to N % 8 == 0, K % 64 == 0, then the plan for that shape
    KERNEL_ROW64x128,   // pipelined 64x128x64, 4 waves side by side, 5-stage ring: one row of tiles for M <= 64 against many columns
    KERNEL_DECODE_RESIDENT,  // decode kernel for M <= 32 with A in registers: persistent workgroups walk over 16-column tiles; `splits` waves over K
    KERNEL_ROW192x128,  // pipelined 192x128x64, 4 waves, 4-stage ring: one row of tiles for M = 129 ... 192 against many columns
};

struct Plan {
    int kernel = KERNEL_NONE;
    int splits = 1;
    double est_us = 0.0;  // the cost model's estimate where it was used, else 0
    // device memory the plan needs beyond A, B and C: fp32 partial sums of K slices, and
    // zero-padded copies of unaligned operands (KERNEL_PADDED)
    size_t partial_bytes = 0, operand_bytes = 0;
    // pipelined kernels only: the last tail_tiles workgroup ids of the grid run in tail_splits K slices, or
    // (tail_kernel != KERNEL_NONE, 256x256 tiles only) divided among workgroups of that smaller tile
    int tail_tiles = 0, tail_splits = 1, tail_kernel = KERNEL_NONE;
};

// Device memory handed to run_plan; a plan is only run with at least what it asks for.
struct Workspace {
    float *partial = nullptr;
    size_t partial_bytes = 0;
    unsigned char *operands = nullptr;
    size_t operand_bytes = 0;
};

// Upper bounds on what a plan may ask for (0: plans that need no such memory only).
struct PlanLimits {
    size_t partial_bytes = 512ull << 20;
    size_t operand_bytes = 1024ull << 20;
    // For the tuner, which asks for the best plan, then the best plan that is none of those it already has, and so
    // on: plans to leave out (compared by kernel, K slices and the treatment of the last round), and whether the
    // small-M table's rows apply to every shape their kernel can run rather than to their boxes only.
    const Plan *excluded = nullptr;
    int excluded_count = 0;
    bool every_small_m_kernel = false;
};

bool skinny_supports(size_t M, size_t N, size_t K);
Plan plan_for(size_t M, size_t N, size_t K, const PlanLimits &limits = PlanLimits());
void run_plan(const Plan &p, const Workspace &ws, const void *A, const void *B, void *C, size_t M, size_t N, size_t K);

}  // namespace hgemm
