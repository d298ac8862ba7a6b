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

/* The first call for a shape asks hipBLASLt's heuristic for up to 16 kernels, times each on
 * the caller's operands (one warm-up and three timed calls: C is overwritten) and keeps the
 * fastest, so that the 100 % line is the library's best kernel and not merely its first guess;
 * later calls of that shape go straight to the kept kernel. */
HGEMM_FUNC(hgemm_hipblaslt);

/* What that first call found for a shape: the number of kernels the heuristic offered (0 if
 * the shape has not been called yet) and, through the pointers that are not NULL, the index
 * of the fastest, its time and the time of the heuristic's first entry (ms per call). */
int hgemm_hipblaslt_candidates(size_t M, size_t N, size_t K, int *chosen, float *chosen_ms, float *first_ms);

/* Path of the hipBLASLt shared object this comparator is bound to in this process. */
const char *hgemm_hipblaslt_loaded_from(void);

#ifdef __cplusplus
}
#endif

#endif /* HGEMM_HIPBLASLT_H_ */
