// The two un-tiled kernels: the scalar definition of the product and the smallest MFMA
// kernel (one wavefront per 32x32 tile), which pins the MFMA operand / accumulator lane
// layout that every tiled kernel relies on.
#include "../../include/hgemm.h"
#include "mfma_tiled.h"

namespace hgemm {

// C[row*N+col] = sum_i A[row*K+i] * B[i+col*K]   (reference src/simt_naive.cu:18-24), with
// an fp32 accumulator and a guard that holds for ragged shapes (the reference's guard
// uses && and lets edge threads run out of bounds, src/simt_naive.cu:14).
__global__ void __launch_bounds__(256)
    simt_naive_kernel(const half_t *__restrict__ A, const half_t *__restrict__ B, half_t *__restrict__ C, size_t M,
                      size_t N, size_t K, unsigned blocks_n) {
    // one-dimensional grid (row-major over 16x16 blocks of C): no 65535 limit on either dimension
    const size_t row = threadIdx.y + (size_t)blockDim.y * (blockIdx.x / blocks_n);
    const size_t col = threadIdx.x + (size_t)blockDim.x * (blockIdx.x % blocks_n);
    if (row >= M || col >= N) return;
    float tmp = 0.0f;
    for (size_t i = 0; i < K; ++i) tmp += (float)A[row * K + i] * (float)B[i + col * K];
    C[row * N + col] = (half_t)tmp;
}

// One wavefront per 32x32 tile, operands straight from global memory.
// Operand layout of v_mfma_f32_32x32x16_f16: lane l supplies 8 consecutive k
// (8*(l/32) .. +7) of row l%32 for both operands; with the B fragment passed first the
// accumulator register r of lane l is C[m = l%32][n = 8*(r/4) + 4*(l/32) + r%4].
__global__ void __launch_bounds__(64)
    mfma_naive_kernel(const half_t *__restrict__ A, const half_t *__restrict__ B, half_t *__restrict__ C, int N,
                      int K) {
    const int lane = threadIdx.x;
    const int tiles_n = N / 32;  // one-dimensional grid, row-major over the 32x32 tiles of C
    const int m0 = (int)(blockIdx.x / tiles_n) * 32, n0 = (int)(blockIdx.x % tiles_n) * 32;
    const half_t *a = A + (size_t)(m0 + (lane & 31)) * K + (lane >> 5) * 8;
    const half_t *b = B + (size_t)(n0 + (lane & 31)) * K + (lane >> 5) * 8;
    floatx16 acc;
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[r] = 0.0f;
    for (int k = 0; k < K; k += 16) {
        const half8 af = *reinterpret_cast<const half8 *>(a + k);
        const half8 bf = *reinterpret_cast<const half8 *>(b + k);
        acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(bf, af, acc, 0, 0, 0);
    }
    half_t *c = C + (size_t)(m0 + (lane & 31)) * N + n0 + ((lane >> 5) << 2);
#pragma unroll
    for (int g = 0; g < 4; ++g) {
        half4 v;
#pragma unroll
        for (int r = 0; r < 4; ++r) v[r] = (half_t)acc[g * 4 + r];
        *reinterpret_cast<half4 *>(c + g * 8) = v;
    }
}

}  // namespace hgemm

using namespace hgemm;

extern "C" void hgemm_simt_naive(const hgemm_half *A, const hgemm_half *B, hgemm_half *C, size_t M, size_t N,
                                 size_t K) {
    check_operands(A, B, C, M, N, K);
    dim3 block(16, 16);
    const unsigned blocks_n = (unsigned)div_ceil(N, block.x);
    dim3 grid(blocks_n * (unsigned)div_ceil(M, block.y));
    simt_naive_kernel<<<grid, block, 0, nullptr>>>(reinterpret_cast<const half_t *>(A),
                                                   reinterpret_cast<const half_t *>(B),
                                                   reinterpret_cast<half_t *>(C), M, N, K, blocks_n);
    HGEMM_CHECK_HIP_ERROR(hipGetLastError());
}

extern "C" void hgemm_mfma_naive(const hgemm_half *A, const hgemm_half *B, hgemm_half *C, size_t M, size_t N,
                                 size_t K) {
    check_operands(A, B, C, M, N, K);
    HGEMM_CHECK_MSG(M % 32 == 0 && N % 32 == 0 && K % 16 == 0,
                    "hgemm_mfma_naive needs M %% 32 == 0, N %% 32 == 0, K %% 16 == 0 (got M=%zu N=%zu K=%zu)", M, N, K);
    dim3 grid((unsigned)((N / 32) * (M / 32)));
    mfma_naive_kernel<<<grid, dim3(64), 0, nullptr>>>(reinterpret_cast<const half_t *>(A),
                                                      reinterpret_cast<const half_t *>(B),
                                                      reinterpret_cast<half_t *>(C), (int)N, (int)K);
    HGEMM_CHECK_HIP_ERROR(hipGetLastError());
}
