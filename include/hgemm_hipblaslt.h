/*
 * hgemm_hipblaslt.h -- vendor-library comparator, shipped as its own shared object
 * (libhgemm_hipblaslt.so) so that the measured library carries no BLAS dependency.
 *
 * Replaces cublasTensorOp (reference src/cublas_tensor_op.cu:17-25): the same operand
 * view (op(B)=T with ldb=K, op(A)=N with lda=K, ldc=N, alpha=1, beta=0, m=N, n=M, k=K) on
 * hipBLASLt with fp32 compute.  It is timed beside the hand-written kernels as the 100 %
 * line (reference src/common/tester.h:99-102) and is never part of the measured path.
 */
#ifndef HGEMM_HIPBLASLT_H_
#define HGEMM_HIPBLASLT_H_

#include "hgemm.h"

#ifdef __cplusplus
extern "C" {
#endif

HGEMM_FUNC(hgemm_hipblaslt);

#ifdef __cplusplus
}
#endif

#endif /* HGEMM_HIPBLASLT_H_ */
