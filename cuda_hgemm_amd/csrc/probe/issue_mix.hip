// hgemm_mix_probe: what the pieces of the 256x256x64 loop cost under the board's power limit,
// one lever at a time.  A program of its own (bin/hgemm_mix_probe), not part of libhgemm.so.
//
// Part 1 runs the loop's instruction mix with the MFMAs on fixed random registers and the
// memory instructions moving the real kernel's bytes from the real kernel's addresses into
// sinks (nothing depends on what they fetch, so every variant is "perfectly scheduled"):
//   1  A and B through LDS: 32 ds_read_b128 + 16 direct-to-LDS copies per wave and chunk
//   5  the same, persistent: 256 workgroups walk 4 tiles each, no gaps between workgroups
//   6  the same, each accumulator's two k-steps back to back (the chained kernel's order)
//   7  the same, four k-steps back to back
//   2  A through LDS, B fragments loaded straight from global memory in operand layout
//      (16 ds_read_b128 + 8 copies + 16 global_load_dwordx4)
//   3  as 2, the B loads always hitting the same lines (resident in L1)
//   4  A through LDS, no B traffic at all
//   0  MFMAs only
// Part 2 is an MFMA-only loop under different accumulator orders, for both MFMA shapes.
// Part 3 gives the floors the small-M (decode) shapes are measured against: the time of an
// empty launch and of a plain streaming read of 32 MB and 224 MB (B of N = 4096 and 28672 at
// K = 4096), back to back and rotating over 800 MB so that every read comes from HBM.
// Results are throughput only; the outputs are meaningless.
//
//     bin/hgemm_mix_probe
#include <stdio.h>

#include <vector>

#include "../mfma_pipelined.h"

using namespace hgemm;
#define CK(x) HGEMM_CHECK_HIP_ERROR(x)

__device__ inline half8 rnd8(uint32_t &s) {
    half8 v;
    for (int i = 0; i < 8; ++i) { s = s * 1664525u + 1013904223u; v[i] = (_Float16)(((int)(s >> 8) % 2001 - 1000) * 0.001f); }
    return v;
}

// ---- part 1: the loop's instruction mix (modes in the header of this file)
template <int MODE_>
__global__ void __launch_bounds__(256) mix(const half_t *A, const half_t *B, float *out, int K, int tiles_m, int tiles_n) {
    extern __shared__ __attribute__((aligned(1024))) unsigned char lds[];
    const uint32_t lds_base = (uint32_t)(uintptr_t)lds;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave >> 1, wn = wave & 1;
    int tile_m, tile_n;
    constexpr int MODE = (MODE_ >= 5) ? 1 : MODE_;
    constexpr int CHAIN = MODE_ == 6 ? 2 : (MODE_ == 7 ? 4 : 1);
    for (int bid = blockIdx.x; bid < tiles_m * tiles_n; bid += gridDim.x) {
    tile_of_workgroup(false, 0, bid, tiles_m * tiles_n, tiles_m, tiles_n, tile_m, tile_n);
    tile_m = __builtin_amdgcn_readfirstlane(tile_m); tile_n = __builtin_amdgcn_readfirstlane(tile_n);
    uint32_t s = tid * 7919u + blockIdx.x * 104729u + 1;
    half8 a[8], b[8];
    for (int i = 0; i < 8; ++i) { a[i] = rnd8(s); b[i] = rnd8(s); }
    floatx4 acc[8][8];
    for (int i = 0; i < 8; ++i) for (int j = 0; j < 8; ++j) for (int r = 0; r < 4; ++r) acc[i][j][r] = 0.f;

    // copies: wave w instruction it covers rows (it*4 + w)*8 + lane/8, chunk lane%8
    const unsigned char *a_base = (const unsigned char *)(A + (size_t)tile_m * 256 * K);
    const unsigned char *b_base = (const unsigned char *)(B + (size_t)tile_n * 256 * K);
    uint32_t voff[8];
    for (int it = 0; it < 8; ++it) voff[it] = ((uint32_t)((it * 4 + wave) * 8 + lane / 8) * (uint32_t)K + (lane % 8) * 8) * 2u;
    // direct B fragments: tile t row wn*128 + t*16 + lane%16, 16 bytes at (lane/16)*16 (+ 64 for the second step)
    uint32_t boff[8];
    for (int t = 0; t < 8; ++t) boff[t] = ((uint32_t)(wn * 128 + t * 16 + lane % 16) * (uint32_t)K + (lane / 16) * 8) * 2u;
    const uint32_t cp_lds = lds_base + wave * 1024;
    // LDS fragment addresses (conflict-free pattern of the tuned kernel)
    const int frag_row = lane % 16;
    const int x = (frag_row >> 1) & 3;
    const int swz = ((x & 1) | ((x & 2) << 1)) ^ (((frag_row >> 3) & 1) << 1);
    uint32_t faddr[2];
    for (int kk = 0; kk < 2; ++kk) faddr[kk] = lds_base + (wm * 128 + frag_row) * 128 + ((((lane / 16) + 4 * kk) ^ swz) << 4);
    uint32_t gaddr[2];
    for (int kk = 0; kk < 2; ++kk) gaddr[kk] = lds_base + 3 * 32768 + (wn * 128 + frag_row) * 128 + ((((lane / 16) + 4 * kk) ^ swz) << 4);

    half8 sink_a[8], sink_b[8], sink_g[16];
    const int num_k = K / 64;
    for (int kt = 0; kt < num_k; ++kt) {
        const unsigned char *a_src = a_base + (size_t)kt * 128, *b_src = b_base + (size_t)(MODE == 3 ? (kt & 1) : kt) * 128;
        const uint32_t dst_a = cp_lds + (kt % 3) * 32768, dst_b = cp_lds + 3 * 32768 + (kt & 1) * 32768;
        const uint32_t ra = (kt % 3) * 32768, rb = (kt & 1) * 32768;
        static_for<2>([&](auto kk_c) {
            constexpr int kk = decltype(kk_c)::value;
            if constexpr (kk == 1 && MODE != 0) {
                if constexpr (MODE == 1) wait_vmcnt<8>();
                else if constexpr (MODE == 4) wait_vmcnt<8>();
                else wait_vmcnt<24>();
                __builtin_amdgcn_s_barrier();
            }
            __builtin_amdgcn_sched_barrier(0);
            static_for<64>([&](auto idx_c) {
                constexpr int idx = decltype(idx_c)::value;
                constexpr int slot = kk * 64 + idx;
                constexpr int j = CHAIN == 1 ? idx / 8 : (slot / CHAIN) / 8, i = CHAIN == 1 ? idx % 8 : (slot / CHAIN) % 8;
                // copies: A in step 0 at slots 5, 13, ...; B (MODE 1) in step 1 at slots 3, 11, ...
                if constexpr (MODE != 0 && kk == 0 && idx % 8 == 5)
                    mfma_and_dma<16, (idx / 8) * 4096>(b[j], a[i], acc[i][j], a_src, voff[idx / 8], dst_a);
                else if constexpr (MODE == 1 && kk == 1 && idx % 8 == 3)
                    mfma_and_dma<16, (idx / 8) * 4096>(b[j], a[i], acc[i][j], b_src, voff[idx / 8], dst_b);
                else
                    MfmaOp<16>::run(b[j], a[i], acc[i][j]);
                if constexpr (MODE != 0) {
                    // operand reads: A tile t at slot 4t + 2; B tile t at slot 4t (first half of the step)
                    if constexpr (idx >= 2 && (idx - 2) % 4 == 0 && (idx - 2) / 4 < 8)
                        sink_a[(idx - 2) / 4] = lds_read16<((idx - 2) / 4) * 16 * 128>(faddr[kk] + ra);
                    if constexpr (MODE == 1 && idx % 4 == 0 && idx / 4 < 8)
                        sink_b[idx / 4] = lds_read16<(idx / 4) * 16 * 128>(gaddr[kk] + rb);
                    // direct B fragments of the next chunk: 8 per step, one per 8 slots (slot 8t + 7)
                    if constexpr ((MODE == 2 || MODE == 3) && idx % 8 == 7) {
                        constexpr int t = idx / 8;
                        asm volatile("global_load_dwordx4 %0, %1, %2 offset:%3" : "=v"(sink_g[kk * 8 + t]) : "v"(boff[t]), "s"(b_src + 128), "i"(kk * 64) : "memory");
                    }
                }
                __builtin_amdgcn_sched_barrier(0);
            });
            if constexpr (MODE != 0) {
                lds_wait_all();
                static_for<8>([&](auto t) { lds_landed(sink_a[decltype(t)::value]); });
                if constexpr (MODE == 1) static_for<8>([&](auto t) { lds_landed(sink_b[decltype(t)::value]); });
            }
        });
    }
    asm volatile("s_waitcnt vmcnt(0)\n\ts_nop 15\n\ts_nop 15" ::: "memory");
    __builtin_amdgcn_s_barrier();
    static_for<8>([&](auto i_c) { static_for<8>([&](auto j_c) { pin_accumulator(acc[decltype(i_c)::value][decltype(j_c)::value]); }); });
    if constexpr (MODE == 2 || MODE == 3) static_for<16>([&](auto t) { lds_landed(sink_g[decltype(t)::value]); });
    float t = 0;
    for (int i = 0; i < 8; ++i) for (int j = 0; j < 8; ++j) for (int r = 0; r < 4; ++r) t += acc[i][j][r];
    if (MODE == 2 || MODE == 3) for (int q = 0; q < 16; ++q) t += (float)sink_g[q][0];
    if (MODE != 0) for (int q = 0; q < 8; ++q) t += (float)sink_a[q][0];
    out[(size_t)bid * 256 + tid] = t;
    }
}

template <int MODE>
void run_mix(const half_t *A, const half_t *B, float *out, int n, const char *name) {
    CK(hipFuncSetAttribute((const void *)&mix<MODE>, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
    hipEvent_t e0, e1; CK(hipEventCreate(&e0)); CK(hipEventCreate(&e1));
    const int tiles = n / 256;
    for (int phase = 0; phase < 3; ++phase) {
        const int launches = 80; float ms;
        CK(hipEventRecord(e0));
        for (int l = 0; l < launches; ++l) mix<MODE><<<MODE == 5 ? 256 : tiles * tiles, 256, 160 * 1024>>>(A, B, out, n, tiles, tiles);
        CK(hipEventRecord(e1)); CK(hipEventSynchronize(e1)); CK(hipEventElapsedTime(&ms, e0, e1));
        CK(hipGetLastError());
        printf("%-58s phase %d: %.4f ms per launch, %.1f TFLOPS\n", name, phase, ms / launches, 2.0 * n * n * n * 1e-12 / (ms / launches * 1e-3));
    }
    fflush(stdout);
}

// ---- part 2: MFMA-only loop, accumulator orders
// ORDER 0: 64 distinct accumulators per step, B-major (the tuned kernel); two steps with different operands
// ORDER 1: each accumulator gets its two k-steps back to back (dependent pair)
// ORDER 2: four k-steps back to back on each accumulator
// ORDER 3: as 0 but A-major
template <int ORDER>
__global__ void __launch_bounds__(256) mfma_only_16(float *out, int iters) {
    uint32_t s = threadIdx.x * 7919u + blockIdx.x * 104729u + 1;
    half8 a[2][8], b[2][8];
    static_for<2>([&](auto q_c) { static_for<8>([&](auto i_c) { a[decltype(q_c)::value][decltype(i_c)::value] = rnd8(s); b[decltype(q_c)::value][decltype(i_c)::value] = rnd8(s); }); });
    floatx4 acc[8][8];
    for (int i = 0; i < 8; ++i) for (int j = 0; j < 8; ++j) for (int r = 0; r < 4; ++r) acc[i][j][r] = 0.f;
    for (int it = 0; it < iters; ++it) {   // one iteration = 256 MFMAs = 4 k-steps over the 8x8 tile
        if constexpr (ORDER == 0 || ORDER == 3) {
            static_for<4>([&](auto q_c) {
                constexpr int q = decltype(q_c)::value;
                static_for<64>([&](auto idx_c) {
                    constexpr int idx = decltype(idx_c)::value;
                    constexpr int j = ORDER == 0 ? idx / 8 : idx % 8, i = ORDER == 0 ? idx % 8 : idx / 8;
                    MfmaOp<16>::run(b[q % 2][j], a[q % 2][i], acc[i][j]);
                });
            });
        } else if constexpr (ORDER == 1) {
            static_for<2>([&](auto h_c) {
                constexpr int h = decltype(h_c)::value;
                static_for<64>([&](auto idx_c) {
                    constexpr int idx = decltype(idx_c)::value;
                    constexpr int j = idx / 8, i = idx % 8;
                    MfmaOp<16>::run(b[0][j], a[0][i], acc[i][j]);
                    MfmaOp<16>::run(b[1][j], a[1][i], acc[i][j]);
                });
            });
        } else {
            static_for<64>([&](auto idx_c) {
                constexpr int idx = decltype(idx_c)::value;
                constexpr int j = idx / 8, i = idx % 8;
                static_for<4>([&](auto q_c) { constexpr int q = decltype(q_c)::value; MfmaOp<16>::run(b[q % 2][j], a[q % 2][i], acc[i][j]); });
            });
        }
    }
    asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
    static_for<8>([&](auto i_c) { static_for<8>([&](auto j_c) { pin_accumulator(acc[decltype(i_c)::value][decltype(j_c)::value]); }); });
    float t = 0;
    for (int i = 0; i < 8; ++i) for (int j = 0; j < 8; ++j) for (int r = 0; r < 4; ++r) t += acc[i][j][r];
    out[(size_t)blockIdx.x * 256 + threadIdx.x] = t;
}
// 32x32x16: 4 x 4 accumulators of 16 registers; CHAIN k-steps back to back on each (1: 16 accumulators in turn)
template <int CHAIN>
__global__ void __launch_bounds__(256) mfma_only_32(float *out, int iters) {
    uint32_t s = threadIdx.x * 7919u + blockIdx.x * 104729u + 1;
    half8 a[4][4], b[4][4];
    static_for<4>([&](auto q_c) { static_for<4>([&](auto i_c) { a[decltype(q_c)::value][decltype(i_c)::value] = rnd8(s); b[decltype(q_c)::value][decltype(i_c)::value] = rnd8(s); }); });
    floatx16 acc[4][4];
    for (int i = 0; i < 4; ++i) for (int j = 0; j < 4; ++j) for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;
    for (int it = 0; it < iters; ++it) {   // one iteration = 128 MFMAs = 8 k-steps of 16 over the 4x4 tile (same flops as 256 16x16x32)
        static_for<2>([&](auto h_c) {
            static_for<4 / CHAIN>([&](auto g_c) {
                constexpr int g = decltype(g_c)::value;
                static_for<16>([&](auto idx_c) {
                    constexpr int idx = decltype(idx_c)::value;
                    constexpr int j = idx / 4, i = idx % 4;
                    static_for<CHAIN>([&](auto q_c) {
                        constexpr int q = g * CHAIN + decltype(q_c)::value;
                        MfmaOp<32>::run(b[q][j], a[q][i], acc[i][j]);
                    });
                });
            });
        });
    }
    asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
    static_for<4>([&](auto i_c) { static_for<4>([&](auto j_c) { pin_accumulator(acc[decltype(i_c)::value][decltype(j_c)::value]); }); });
    float t = 0;
    for (int i = 0; i < 4; ++i) for (int j = 0; j < 4; ++j) for (int r = 0; r < 16; ++r) t += acc[i][j][r];
    out[(size_t)blockIdx.x * 256 + threadIdx.x] = t;
}
template <int CHAIN>
void run32(float *out, const char *name) {
    hipEvent_t e0, e1; CK(hipEventCreate(&e0)); CK(hipEventCreate(&e1));
    const int iters = 2048;
    const double flop = 1024.0 * iters * 128 * 32768.0;
    for (int phase = 0; phase < 3; ++phase) {
        const int launches = 20; float ms;
        CK(hipEventRecord(e0));
        for (int l = 0; l < launches; ++l) mfma_only_32<CHAIN><<<256, 256>>>(out, iters);
        CK(hipEventRecord(e1)); CK(hipEventSynchronize(e1)); CK(hipEventElapsedTime(&ms, e0, e1));
        printf("%-60s phase %d: %.3f ms per launch, %.1f TFLOPS\n", name, phase, ms / launches, flop * launches / ms * 1e-9);
    }
    fflush(stdout);
}
template <int ORDER>
void run_order(float *out, const char *name) {
    hipEvent_t e0, e1; CK(hipEventCreate(&e0)); CK(hipEventCreate(&e1));
    const int iters = 2048;  // x 256 MFMAs x 16384 flop x 1024 waves = 8.8e12 ... scaled to ~4 ms
    const double flop = 1024.0 * iters * 256 * 16384.0;
    for (int phase = 0; phase < 3; ++phase) {
        const int launches = 20; float ms;
        CK(hipEventRecord(e0));
        for (int l = 0; l < launches; ++l) mfma_only_16<ORDER><<<256, 256>>>(out, iters);
        CK(hipEventRecord(e1)); CK(hipEventSynchronize(e1)); CK(hipEventElapsedTime(&ms, e0, e1));
        printf("%-60s phase %d: %.3f ms per launch, %.1f TFLOPS\n", name, phase, ms / launches, flop * launches / ms * 1e-9);
    }
    fflush(stdout);
}
// ---- part 3: launch and streaming floors
typedef unsigned int probe_u32x4 __attribute__((ext_vector_type(4)));
__global__ void __launch_bounds__(256) stream_read(const probe_u32x4 *p, size_t n16, unsigned *out) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    probe_u32x4 v = {0, 0, 0, 0};
    if (i < n16) v = p[i];
    if ((v.x ^ v.y ^ v.z ^ v.w) == 0x12345678u) out[0] = 1;  // never true for the fill pattern: keeps the load
}
__global__ void empty_kernel(unsigned *out) {
    if (threadIdx.x == 1234567) out[0] = 1;
}
void run_floors() {
    unsigned *out;
    CK(hipMalloc(&out, 4));
    hipEvent_t e0, e1;
    CK(hipEventCreate(&e0));
    CK(hipEventCreate(&e1));
    float ms;
    for (int i = 0; i < 50; ++i) empty_kernel<<<256, 256>>>(out);
    CK(hipEventRecord(e0));
    for (int i = 0; i < 500; ++i) empty_kernel<<<256, 256>>>(out);
    CK(hipEventRecord(e1));
    CK(hipEventSynchronize(e1));
    CK(hipEventElapsedTime(&ms, e0, e1));
    printf("empty kernel, back to back: %.2f us per launch\n", ms * 1e3 / 500);
    for (size_t bytes : {(size_t)4096 * 4096 * 2, (size_t)28672 * 4096 * 2}) {
        const int sets = (int)((800ull << 20) / bytes + 1);
        std::vector<probe_u32x4 *> bufs(sets);
        for (auto &b : bufs) {
            CK(hipMalloc(&b, bytes));
            CK(hipMemset(b, 0x11, bytes));
        }
        const size_t n16 = bytes / 16;
        const unsigned grid = (unsigned)((n16 + 255) / 256);
        for (int i = 0; i < 20; ++i) stream_read<<<grid, 256>>>(bufs[i % sets], n16, out);
        CK(hipEventRecord(e0));
        for (int i = 0; i < 200; ++i) stream_read<<<grid, 256>>>(bufs[i % sets], n16, out);
        CK(hipEventRecord(e1));
        CK(hipEventSynchronize(e1));
        CK(hipEventElapsedTime(&ms, e0, e1));
        const double us = ms * 1e3 / 200;
        printf("plain read of %zu MB, 16 bytes per thread, rotating over %d buffers: %.2f us per launch, %.0f GB/s\n",
               bytes >> 20, sets, us, bytes / us * 1e-3);
        for (auto &b : bufs) CK(hipFree(b));
    }
    fflush(stdout);
}

int main() {
    run_floors();
    const int n = 8192;
    half_t *A, *B;
    float *out;
    CK(hipMalloc(&A, (size_t)n * n * 2 + 4096));
    CK(hipMalloc(&B, (size_t)n * n * 2 + 4096));
    CK(hipMalloc(&out, 1024 * 256 * 4));
    std::vector<uint16_t> h((size_t)n * n);
    uint32_t s = 12345;
    for (auto &v : h) {
        s = s * 1664525u + 1013904223u;
        _Float16 f = (_Float16)(((int)(s >> 8) % 2001 - 1000) * 0.001f);
        memcpy(&v, &f, 2);
    }
    CK(hipMemcpy(A, h.data(), h.size() * 2, hipMemcpyHostToDevice));
    CK(hipMemcpy(B, h.data(), h.size() * 2, hipMemcpyHostToDevice));
    for (int rep = 0; rep < 2; ++rep) {
        run_mix<1>(A, B, out, n, "1: A and B through LDS (the tuned kernels' mix)");
        run_mix<5>(A, B, out, n, "5: as 1, persistent: 256 workgroups x 4 tiles, no gaps");
        run_mix<6>(A, B, out, n, "6: as 1, two k-steps back to back on each accumulator");
        run_mix<7>(A, B, out, n, "7: as 1, four k-steps back to back (half the accumulators)");
        run_mix<2>(A, B, out, n, "2: A through LDS, B fragments straight from global");
        run_mix<3>(A, B, out, n, "3: as 2, B loads always from the same lines (L1 hits)");
        run_mix<4>(A, B, out, n, "4: A through LDS, no B traffic at all");
        run_mix<0>(A, B, out, n, "0: MFMA only");
    }
    for (int rep = 0; rep < 2; ++rep) {
        run_order<0>(out, "16x16x32: 64 accumulators in turn, B-major (interleaved kernel)");
        run_order<3>(out, "16x16x32: 64 accumulators in turn, A-major");
        run_order<1>(out, "16x16x32: two k-steps back to back on each accumulator");
        run_order<2>(out, "16x16x32: four k-steps back to back on each accumulator");
        run32<1>(out, "32x32x16: 16 accumulators in turn");
        run32<2>(out, "32x32x16: two k-steps back to back");
        run32<4>(out, "32x32x16: four k-steps back to back");
    }
    return 0;
}
