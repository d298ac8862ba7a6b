// Kernel selection record shared by the dispatcher and its reporting helpers.
#pragma once

#include <stddef.h>

namespace hgemm {

enum KernelId {
    KERNEL_NONE = 0,
    KERNEL_BIG256,     // pipelined 256x256x64
    KERNEL_MID128,     // pipelined 128x128x64
    KERNEL_SKINNY32,   // M <= 32
    KERNEL_SKINNY64,   // M <= 64
    KERNEL_SKINNY128,  // M <= 128
    KERNEL_SPLIT128,   // 128x128 tiles with K slices (few tiles, long K)
    KERNEL_SPLIT64,    // 64x64 tiles with K slices
    KERNEL_SIMT,       // scalar fallback for shapes no MFMA kernel tiles
};

struct Plan {
    int kernel = KERNEL_NONE;
    int splits = 1;
};

bool skinny_supports(size_t M, size_t N, size_t K);
Plan plan_for(size_t M, size_t N, size_t K);
void run_plan(const Plan &p, const void *A, const void *B, void *C, size_t M, size_t N, size_t K);

}  // namespace hgemm
