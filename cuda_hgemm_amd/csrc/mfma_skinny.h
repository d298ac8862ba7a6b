// Small-M ("decode shaped") product: M <= 128 rows of A against a large B.
//
// The work is streaming B (N x K halves) from HBM exactly once; MFMA throughput is
// irrelevant.  A workgroup owns BN rows of B and one slice of K, keeps a deep ring of
// direct-to-LDS copies in flight, and multiplies against the (L2-resident) A rows with the
// same LDS layout and fragment scheme as the big-tile kernels.  Rows of the tile beyond M
// are loaded from row M-1 (valid memory) and never stored.
//
// When N alone does not give enough workgroups to fill 256 CUs, K is split: each slice
// writes fp32 partial sums to a workspace and a second kernel adds the slices in index
// order and rounds to fp16, so the result does not depend on scheduling (no float
// atomics) and is bit-identical from run to run.
//
// The reference has no kernel for these shapes: its tiled kernels need M % 256 == 0
// (src/mma/mma_async_stage4.cu:64-66,93-94).
#pragma once

#include "mfma_tiled.h"

namespace hgemm {

template <int BM_, int BN_, int WAVES_M_, int WAVES_N_, int STAGES_>
struct SkinnyConfig : TileConfig<BM_, BN_, 64, WAVES_M_, WAVES_N_, STAGES_, LOAD_DMA, LDS_SWIZZLE, true> {};

// STREAM_B: B is copied with the non-temporal hint.  Every byte of B is read once; when B is larger than the
// Infinity Cache keeps (N = 28672, K = 4096: 235 MB) the hint is worth 11-12 % (M = 16 ... 64: 64.5 -> 72.6 %, 63.6 ->
// 70.5 %, 57.6 -> 64.7 % of 8 TB/s), when B fits (N = K = 4096) it costs up to 7 %, so the launcher decides by size.
template <class Cfg, bool STREAM_B = false>
__global__ void __launch_bounds__(Cfg::THREADS)
    hgemm_skinny_kernel(const half_t *__restrict__ A, const half_t *__restrict__ B, half_t *__restrict__ C,
                        float *__restrict__ partial, int M, int N, int K, int splits, int tiles_n) {
    constexpr int BM = Cfg::BM, BN = Cfg::BN, BK = Cfg::BK;
    constexpr int TM = Cfg::TM, TN = Cfg::TN, KSTEPS = Cfg::KSTEPS, CPR = Cfg::CPR;
    constexpr int ROW_BYTES = Cfg::ROW_BYTES, STAGES = Cfg::STAGES;
    constexpr int L = Cfg::A_DMA + Cfg::B_DMA;

    extern __shared__ __attribute__((aligned(1024))) unsigned char lds[];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / Cfg::WAVES_N, wn = wave % Cfg::WAVES_N;

    // grid: x = tiles of C, row-major (no 65535 limit on the number of row or column tiles), y = K slice
    const int tile_n = (int)blockIdx.x % tiles_n, tile_m = (int)blockIdx.x / tiles_n, split = blockIdx.y;
    const int m0 = tile_m * BM;
    int first_chunk, num_k;  // K's chunks are dealt to the slices as evenly as whole chunks allow
    slice_of_k(K / BK, splits, split, first_chunk, num_k);
    const int k_begin = first_chunk * BK;

    // ---- copy set-up (rows of A clamped to the last valid row)
    constexpr int DMA_ROW_STEP = Cfg::WAVES * Cfg::ROWS_PER_DMA;
    const int cp_row = wave * Cfg::ROWS_PER_DMA + lane / CPR;
    const int cp_ch = (lane % CPR) ^ swizzle_of_row<Cfg>(cp_row);
    const half_t *a_src[Cfg::A_DMA];
    const half_t *b_src[Cfg::B_DMA];
#pragma unroll
    for (int it = 0; it < Cfg::A_DMA; ++it) {
        int r = m0 + cp_row + it * DMA_ROW_STEP;
        r = r < M ? r : M - 1;
        a_src[it] = A + (size_t)r * K + k_begin + cp_ch * 8;
    }
#pragma unroll
    for (int it = 0; it < Cfg::B_DMA; ++it)
        b_src[it] = B + (size_t)(tile_n * BN + cp_row + it * DMA_ROW_STEP) * K + k_begin + cp_ch * 8;
    const uint32_t cp_lds = (uint32_t)(uintptr_t)lds + wave * 1024;

    auto dma_fetch = [&](int kt, int stage) {
        const int koff = kt * BK;
        const uint32_t base = cp_lds + stage * Cfg::STAGE_BYTES;
#pragma unroll
        for (int it = 0; it < Cfg::A_DMA; ++it) dma_load16(a_src[it] + koff, base + it * Cfg::WAVES * 1024);
#pragma unroll
        for (int it = 0; it < Cfg::B_DMA; ++it)
            if constexpr (STREAM_B)
                dma_load16_streaming(b_src[it] + koff, base + Cfg::A_BYTES + it * Cfg::WAVES * 1024);
            else
                dma_load16(b_src[it] + koff, base + Cfg::A_BYTES + it * Cfg::WAVES * 1024);
    };

    // ---- fragments
    const int frag_row = lane & 31;
    const int frag_x = (lane >> 5) ^ swizzle_of_row<Cfg>(frag_row);
    const uint32_t a_frag_off = (wm * Cfg::WM + frag_row) * ROW_BYTES;
    const uint32_t b_frag_off = Cfg::A_BYTES + (wn * Cfg::WN + frag_row) * ROW_BYTES;

    floatx16 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

    auto compute_stage = [&](int stage) {
        const unsigned char *s = lds + stage * Cfg::STAGE_BYTES;
#pragma unroll
        for (int kk = 0; kk < KSTEPS; ++kk) {
            const uint32_t chunk = (uint32_t)((kk * 2) ^ frag_x) << 4;
            half8 af[TM], bf[TN];
#pragma unroll
            for (int i = 0; i < TM; ++i)
                af[i] = *reinterpret_cast<const half8 *>(s + a_frag_off + i * 32 * ROW_BYTES + chunk);
#pragma unroll
            for (int j = 0; j < TN; ++j)
                bf[j] = *reinterpret_cast<const half8 *>(s + b_frag_off + j * 32 * ROW_BYTES + chunk);
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(bf[j], af[i], acc[i][j], 0, 0, 0);
        }
    };

    // ---- ring of STAGES buffers, STAGES-1 chunks in flight
#pragma unroll
    for (int s = 0; s < STAGES - 1; ++s)
        if (s < num_k) dma_fetch(s, s);
    int cur = 0, fill = STAGES - 1;
    for (int kt = 0; kt < num_k; ++kt) {
        if (num_k - 1 - kt >= STAGES - 2)
            wait_vmcnt<(STAGES - 2) * L>();
        else
            wait_vmcnt<0>();
        __syncthreads();
        if (kt + STAGES - 1 < num_k) dma_fetch(kt + STAGES - 1, fill);
        compute_stage(cur);
        cur = (cur + 1 == STAGES) ? 0 : cur + 1;
        fill = (fill + 1 == STAGES) ? 0 : fill + 1;
    }

    // ---- epilogue.  Lane l holds row l%32 of each 32x32 tile and four consecutive n per
    // register group: 8 bytes of fp16, or 16 bytes of an fp32 partial sum.
    const int row_in_wave = lane & 31;
    const int col_in_tile = (lane >> 5) << 2;
#pragma unroll
    for (int i = 0; i < TM; ++i) {
        const int m = m0 + wm * Cfg::WM + i * 32 + row_in_wave;
        if (m >= M) continue;
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            const int n = tile_n * BN + wn * Cfg::WN + j * 32 + col_in_tile;
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                if (partial) {
                    floatx4 v;
#pragma unroll
                    for (int r = 0; r < 4; ++r) v[r] = acc[i][j][g * 4 + r];
                    *reinterpret_cast<floatx4 *>(partial + ((size_t)split * M + m) * N + n + g * 8) = v;
                } else {
                    half4 v;
#pragma unroll
                    for (int r = 0; r < 4; ++r) v[r] = (half_t)acc[i][j][g * 4 + r];
                    *reinterpret_cast<half4 *>(C + (size_t)m * N + n + g * 8) = v;
                }
            }
        }
    }
}

// C[i] = fp16( partial[0][i] + partial[1][i] + ... ), always added in slice order, VEC
// outputs per thread.  The loads of four slices are issued together before their adds, so
// the kernel is not one memory round trip per slice; small outputs use a small VEC so the
// reduction still spreads over the chip.
template <int VEC>
__global__ void __launch_bounds__(256)
    splitk_reduce_kernel(const float *__restrict__ partial, half_t *__restrict__ C, size_t elems, int splits) {
    typedef float vec_t __attribute__((ext_vector_type(VEC)));
    typedef half_t hvec_t __attribute__((ext_vector_type(VEC)));
    const size_t i = ((size_t)blockIdx.x * blockDim.x + threadIdx.x) * VEC;
    if (i >= elems) return;
    const float *src = partial + i;
    vec_t acc = *reinterpret_cast<const vec_t *>(src);
    int s = 1;
    for (; s + 4 <= splits; s += 4) {
        const vec_t v0 = *reinterpret_cast<const vec_t *>(src + (size_t)s * elems);
        const vec_t v1 = *reinterpret_cast<const vec_t *>(src + (size_t)(s + 1) * elems);
        const vec_t v2 = *reinterpret_cast<const vec_t *>(src + (size_t)(s + 2) * elems);
        const vec_t v3 = *reinterpret_cast<const vec_t *>(src + (size_t)(s + 3) * elems);
        acc += v0;
        acc += v1;
        acc += v2;
        acc += v3;
    }
    for (; s < splits; ++s) acc += *reinterpret_cast<const vec_t *>(src + (size_t)s * elems);
    hvec_t out;
#pragma unroll
    for (int r = 0; r < VEC; ++r) out[r] = (half_t)acc[r];
    store_streaming(reinterpret_cast<hvec_t *>(C + i), out);
}

// elems must be a multiple of 8 (every tile dimension is).
inline void launch_splitk_reduce(const float *partial, half_t *C, size_t elems, int splits) {
    if (elems >= (size_t)2 << 20)
        splitk_reduce_kernel<8><<<dim3((unsigned)div_ceil(elems / 8, 256)), dim3(256), 0, nullptr>>>(partial, C, elems,
                                                                                                    splits);
    else if (elems >= (size_t)512 << 10)
        splitk_reduce_kernel<4><<<dim3((unsigned)div_ceil(elems / 4, 256)), dim3(256), 0, nullptr>>>(partial, C, elems,
                                                                                                    splits);
    else
        splitk_reduce_kernel<2><<<dim3((unsigned)div_ceil(elems / 2, 256)), dim3(256), 0, nullptr>>>(partial, C, elems,
                                                                                                    splits);
    HGEMM_CHECK_HIP_ERROR(hipGetLastError());
}

}  // namespace hgemm
