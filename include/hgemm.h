/*
 * hgemm.h -- C ABI of the MI355X (gfx950) half-precision GEMM library.
 *
 * Every kernel entry point has the shape of the reference's HGEMM_FUNC
 * (reference src/main.cu:11):
 *
 *     void name(half *A, half *B, half *C, size_t M, size_t N, size_t K)
 *
 * and computes  C[m*N + n] = sum_k A[m*K + k] * B[n*K + k]  (reference
 * src/simt_naive.cu:18-24) on DEVICE pointers the caller owns:
 *     A  row-major   M x K                      (reference src/common/tester.h:117)
 *     B  column-major K x N, i.e. N rows of K    (reference src/common/tester.h:118)
 *     C  row-major   M x N, fully overwritten    (reference src/common/tester.h:119)
 * Elements are IEEE binary16 (2 bytes); A, B and C start on 16-byte boundaries (hipMalloc
 * gives 256).  Products are accumulated in fp32 and rounded to
 * fp16 once (the reference accumulates in fp16; this is the one deliberate difference).
 *
 * Calling convention, as in the reference (src/mma/mma_async_stage4.cu:637-644,
 * src/common/tester.h:59-62,91-94): launched asynchronously on the null stream, the caller
 * synchronises.  Nothing is allocated per call; hgemm_auto and hgemm_skinny allocate a
 * process-lifetime workspace the first time a plan needs one (see "workspace" below).  A contract violation (null pointer, zero
 * dimension, a shape the variant cannot tile) is reported on stderr and ends the process
 * with EXIT_FAILURE, the convention of the reference's HGEMM_CHECK macros
 * (src/common/common.h:23-29); unlike the reference, unsupported shapes are diagnosed
 * instead of being read out of bounds.  hgemm_variant_supports() lets a caller ask first.
 */
#ifndef HGEMM_H_
#define HGEMM_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* 16-bit storage type of one element; bit-compatible with _Float16 / __half. */
typedef uint16_t hgemm_half;

typedef void (*hgemm_fn)(const hgemm_half *A, const hgemm_half *B, hgemm_half *C, size_t M, size_t N, size_t K);

#define HGEMM_FUNC(name) \
    void name(const hgemm_half *A, const hgemm_half *B, hgemm_half *C, size_t M, size_t N, size_t K)

/* One thread per output element, fp32 accumulate; any shape.
 * Replaces simtNaive (reference src/simt_naive.cu:27). */
HGEMM_FUNC(hgemm_simt_naive);

/* One wavefront per 32x32 tile of C straight from global memory on
 * v_mfma_f32_32x32x16_f16; needs M%32 == N%32 == 0, K%16 == 0.
 * Replaces wmmaNaive / mmaNaive (reference src/wmma/wmma_naive.cu:46, src/mma/mma_naive.cu:70). */
HGEMM_FUNC(hgemm_mfma_naive);

/* Block-tiled ladder.  Each step adds one technique to the previous one, the way the
 * reference's files do.  Shape needs are those of the tile (see hgemm_variant_supports). */
/* LDS-staged 256x128x32 tile, plain row-major LDS rows.
 * Replaces wmmaBase / mmaBase (reference src/wmma/wmma_base.cu:194, src/mma/mma_base.cu:200). */
HGEMM_FUNC(hgemm_mfma_base);
/* + 16-byte row padding against LDS bank conflicts.
 * Replaces wmmaPadding (reference src/wmma/wmma_padding.cu:196). */
HGEMM_FUNC(hgemm_mfma_padding);
/* + XOR-swizzled LDS rows instead of padding.
 * Replaces mmaPermuted (reference src/mma/mma_permuted.cu:224). */
HGEMM_FUNC(hgemm_mfma_swizzle);
/* + global -> LDS copies that bypass registers (global_load_lds_dwordx4).
 * Replaces wmmaAsync / mmaAsync (reference src/wmma/wmma_async.cu:207, src/mma/mma_async.cu:233). */
HGEMM_FUNC(hgemm_mfma_async);
/* + two LDS buffers: the next K chunk is fetched while the current one is multiplied.
 * Replaces wmmaAsyncPg2s / mmaAsyncPg2s (reference src/wmma/wmma_async_pg2s.cu:282,
 * src/mma/mma_async_pg2s.cu:323). */
HGEMM_FUNC(hgemm_mfma_async_pg2s);
/* + double-buffered MFMA operand registers (LDS -> register prefetch).
 * Replaces wmmaAsyncPg2sPs2r / mmaAsyncPg2sPs2r (reference src/wmma/wmma_async_pg2s_ps2r.cu:346,
 * src/mma/mma_async_pg2s_ps2r.cu:412). */
HGEMM_FUNC(hgemm_mfma_async_pg2s_ps2r);
/* K_STAGE-deep LDS ring, s_waitcnt vmcnt(n) in place of cp.async.wait_group.
 * Replace wmmaAsyncStage2/3 and mmaAsyncStage2/3/4 (reference src/wmma/wmma_async_stage2.cu:375,
 * src/wmma/wmma_async_stage3.cu:453, src/mma/mma_async_stage2.cu:447,
 * src/mma/mma_async_stage3.cu:542, src/mma/mma_async_stage4.cu:637). */
HGEMM_FUNC(hgemm_mfma_async_stage2);
HGEMM_FUNC(hgemm_mfma_async_stage3);
HGEMM_FUNC(hgemm_mfma_async_stage4);
/* The ladder's kernel on a small tile: 64x64x64, four waves of one 32x32 MFMA tile each, 5-stage
 * direct-to-LDS ring whose barrier confirms the chunk after the one being multiplied, so a whole
 * chunk of operands is in registers before its MFMAs start.  hgemm_auto runs it on grids of at
 * most one whole tile per CU (the small squares of the sweep), where a launch is all latency.
 * Needs M % 64 == 0, N % 64 == 0, K % 64 == 0, K >= 256.  No counterpart in the reference, whose
 * tiles are all 256x128. */
HGEMM_FUNC(hgemm_mfma_tiled_64x64);

/* The tuned CDNA4 kernel, one entry point per tile: K chunks of 64 in a ring of LDS buffers
 * filled by direct-to-LDS copies, v_mfma_f32_16x16x32_f16 with a hand-laid issue order,
 * XCD-aware tile order.  256x256 is the kernel hgemm_auto runs on large shapes and the top
 * of the ladder, where the reference's run ends at mmaAsyncStage4 (reference
 * src/main.cu:123, src/mma/mma_async_stage4.cu:637).  Need N % 8 == 0, K % 64 == 0 and
 * K >= 64 * ring depth (128 / 192 / 192 / 320 / 192 in the order below); M and N may end
 * inside a tile. */
HGEMM_FUNC(hgemm_mfma_pipelined_256x256);
HGEMM_FUNC(hgemm_mfma_pipelined_256x128);
HGEMM_FUNC(hgemm_mfma_pipelined_192x192);
HGEMM_FUNC(hgemm_mfma_pipelined_128x128);
HGEMM_FUNC(hgemm_mfma_pipelined_64x64);
/* The same tiles with the work inside a K chunk reordered so that every accumulator receives
 * its two MFMAs back to back (the matrix pipe forwards the running sum instead of going
 * through the register file: less power, hence more clock) and with the accumulators in
 * registers the compiler never sees.  The top of the ladder; hgemm_auto runs these on large
 * grids with long K (256x256: from K = 1536 once most CUs have a tile; the others from 4096).  Same shape needs as the pipelined entry points above. */
HGEMM_FUNC(hgemm_mfma_chained_256x256);
HGEMM_FUNC(hgemm_mfma_chained_256x128);
HGEMM_FUNC(hgemm_mfma_chained_192x192);

/* Small-M (decode-shaped) product: streams B once, bound by HBM bandwidth, M <= 128.
 * No counterpart in the reference, whose tiled kernels cannot run M < 256
 * (reference src/mma/mma_async_stage4.cu:64-66,93-94). */
HGEMM_FUNC(hgemm_skinny);

/* Dispatcher: picks tile, kernel and number of K slices for the shape from a cost model
 * fitted to measurements; accepts every shape.  N % 8 == 0 and K % 64 == 0 run on the
 * pipelined kernels (M and N may end inside a tile: edges are guarded), anything else on a
 * fully guarded MFMA kernel.  This is the entry point the benchmark measures. */
HGEMM_FUNC(hgemm_auto);

/* Kernel hgemm_auto would pick for a shape (an id for hgemm_kernel_name) and, through
 * `splits` if not NULL, the number of K slices; no launch happens. */
int hgemm_auto_plan(size_t M, size_t N, size_t K, int *splits);
/* For grids of whole rounds of workgroups plus a few: how many workgroups of the last round
 * hgemm_auto runs in K slices so that they fill the chip too (0: none) and, through
 * `splits` if not NULL, in how many slices. */
int hgemm_auto_plan_tail(size_t M, size_t N, size_t K, int *splits);
/* The other treatment of such a last round: its workgroups' tiles are divided among
 * workgroups of a smaller tile.  Returns that kernel's id (for hgemm_kernel_name), 0 if
 * the plan does not do this; hgemm_auto_plan_tail still gives the number of tiles. */
int hgemm_auto_plan_tail_kernel(size_t M, size_t N, size_t K);
/* 1 if the plan's main launch runs its tile's chained kernel (hgemm_mfma_chained_*), 0 if the
 * interleaved one (hgemm_mfma_pipelined_*) or a kernel of another family. */
int hgemm_auto_plan_chained(size_t M, size_t N, size_t K);
const char *hgemm_kernel_name(int kernel);
/* Tuning on the caller's operands, for callers who run a shape many times: times up to max_plans (at most 12)
 * plans for the shape -- the one hgemm_auto would run, then the cost model's next best, each different in tile,
 * K slices or, for M <= 128, kernel -- with three untimed and 5 ... 40 timed launches each (`flags`: 0 or
 * HGEMM_TUNE_COLD), and keeps the fastest (the model's own plan unless another is more than 3 % faster) for
 * every later hgemm_auto call of this shape in this process, from any thread; the hgemm_auto_plan* queries then
 * report the kept plan.  Blocks until the device is idle; C holds the product as the kept plan computes it (every
 * plan computes the same product; plans that slice K differently differ in the last bit of some outputs).  May
 * allocate the workspace.  Returns the number of plans timed.  The vendor comparator is tuned the same way at its
 * first call of a shape (include/hgemm_hipblaslt.h).  No counterpart in the reference, whose kernels are one per
 * entry point. */
#define HGEMM_TUNE_COLD 1 /* flags: read 512 MiB through the device before every timed launch, so that A and B come
                           * from HBM -- for callers whose operands (weights) do not stay cached between calls */
int hgemm_auto_tune(const hgemm_half *A, const hgemm_half *B, hgemm_half *C, size_t M, size_t N, size_t K,
                    int max_plans, int flags);
/* The plans hgemm_auto_tune would time, best first by the model, without a launch: kernel ids (for
 * hgemm_kernel_name) and K slices into arrays of max_plans entries (either may be NULL); returns their number. */
int hgemm_auto_tune_plans(size_t M, size_t N, size_t K, int max_plans, int *kernels, int *splits);
/* What the calling thread's last hgemm_auto_tune measured, plan by plan in the order they were timed: kernel id,
 * K slices, milliseconds per launch, and whether that plan was the one kept.  Returns 0 past the last plan, else 1. */
int hgemm_auto_tune_result(int index, int *kernel, int *splits, float *ms, int *kept);
/* Forgets every kept plan; 1 if the shape has one. */
void hgemm_auto_forget_tuning(void);
int hgemm_auto_plan_is_tuned(size_t M, size_t N, size_t K);
/* The table behind hgemm_auto's choice for M <= 128 (decode-shaped products), row by row: the
 * first row that covers a shape, and whose kernel can run it, decides.  bounds receives
 * {m_lo, m_hi, n_lo, n_hi, k_lo, k_hi, b_lo, b_hi}, all inclusive, b = N * K (elements of B);
 * flags bit 0: the row holds only where K < 4 N, bit 1: not where K is a multiple of 16384.
 * Returns the row's kernel id (for hgemm_kernel_name; the streaming decode kernel's rows
 * name its 16-column form and stand for both widths), or -1 past the last row.  No
 * counterpart in the reference, which has no kernel for M < 256. */
int hgemm_small_m_rule(int index, size_t *bounds, int *flags);

/* ---- workspace of hgemm_auto / hgemm_skinny.  Plans that cut K into slices keep fp32
 * partial sums in device memory, and large shapes with N % 8 != 0 or K % 64 != 0 run on
 * zero-padded copies of A and B.  Both buffers belong to the library, one pair per device,
 * and live until hgemm_release_workspace or the end of the process (the reference keeps its
 * vendor handle the same way, src/cublas_tensor_op.cu:18).  Each is allocated ONCE, at its
 * cap (512 MiB of partial sums, 1 GiB of operand copies), by the first call that needs it:
 * that one call contains a hipMalloc; no later call frees or synchronises, and none
 * allocates unless that first hipMalloc was refused (then the size the plan needs is tried
 * once; refused sizes are remembered and not asked for again).  Callers that cannot have
 * even that (a timed loop) reserve beforehand.  If the memory cannot be had, hgemm_auto
 * runs the best plan that needs none.
 * Entry points may be called from several host threads.  The workspaces are shared: the
 * library enqueues the launches of a plan that uses one under a lock, and since every
 * launch goes to the null stream, which runs launches in the order they were enqueued, one
 * call's partial sums are consumed before the next call's overwrite them.
 * hgemm_reserve_workspace and hgemm_release_workspace wait for the device before they free
 * anything and take the same lock. */
/* Allocates the current device's workspaces now: each at least as large as asked, and at
 * least its cap, unless 0 is asked (that buffer is then left alone).  Returns 0, or 1 if
 * device memory ran out. */
int hgemm_reserve_workspace(size_t partial_bytes, size_t operand_bytes);
/* Waits for the device and frees its workspaces. */
void hgemm_release_workspace(void);
/* Bytes of partial sums (return value) and of operand copies (*operand_bytes, if not NULL)
 * that hgemm_auto's plan for the shape uses. */
size_t hgemm_auto_workspace_bytes(size_t M, size_t N, size_t K, size_t *operand_bytes);

/* hgemm_auto for callers that cannot allocate device memory (serving loops, harnesses that
 * forbid hipMalloc).  No counterpart in the reference.  Like every entry point it launches
 * on the null stream, which cannot be captured into a HIP graph; what it guarantees is that
 * no call performs a hipMalloc or hipFree (its first call on a device looks up the array's
 * address and sets kernel attributes, which allocate nothing).  Runs
 * the same plan as hgemm_auto, hence the same result bit for bit, but keeps partial sums and
 * padded operand copies in a fixed array of HGEMM_STATIC_WORKSPACE_BYTES inside the library's
 * code object (every GPU the library runs on holds one copy until the process ends) and
 * calls no hipMalloc, hipFree or other allocating routine.  Returns 0, or 1 -- with a
 * message on stderr and nothing launched -- when the plan needs more than the array holds
 * (hgemm_auto_workspace_bytes tells beforehand).  Other contract violations end the process
 * as everywhere.  All calls on one GPU share that GPU's array, which keeps the last call's
 * contents (nothing in it has to start at zero: every kernel reads only what an earlier
 * kernel of the same call wrote in full).  Calls from several host threads are enqueued one
 * plan at a time and the null stream orders them; work a caller moves to other streams so
 * that two calls overlap on one GPU would race on the array. */
#define HGEMM_STATIC_WORKSPACE_BYTES ((size_t)64 << 20)
int hgemm_auto_static_workspace(const hgemm_half *A, const hgemm_half *B, hgemm_half *C, size_t M, size_t N,
                                size_t K);
size_t hgemm_static_workspace_bytes(void);

/* ---- registry, so a driver can enumerate variants the way the reference's main lists
 * them (reference src/main.cu:100-123) without an edit per variant. ---- */
int hgemm_variant_count(void);
/* Display name used in the log line, e.g. "Mfma-Async-Stage4" (reference src/main.cu:120). */
const char *hgemm_variant_name(int index);
/* Exported symbol name, e.g. "hgemm_mfma_async_stage4". */
const char *hgemm_variant_symbol(int index);
hgemm_fn hgemm_variant_fn(int index);
/* Index of a variant by display or symbol name, -1 if unknown. */
int hgemm_variant_find(const char *name);
/* 1 if variant `index` can run the shape, 0 otherwise (no side effects). */
int hgemm_variant_supports(int index, size_t M, size_t N, size_t K);
/* 1 if the variant belongs to the default run (reference src/main.cu:100-123 comments the
 * slow ones out), 0 otherwise. */
int hgemm_variant_in_default_run(int index);

/* ---- harness helpers: the timing loop of Tester::profile with CudaTimer semantics
 * (reference src/common/tester.h:89-97, src/common/cuda_timer.h:32-42). ---- */
/* Runs `warmup` untimed calls, then `iterations` back-to-back calls bracketed by a pair of
 * HIP events on the null stream; returns the average milliseconds per call. */
double hgemm_profile_ms(hgemm_fn fn, const hgemm_half *A, const hgemm_half *B, hgemm_half *C, size_t M, size_t N,
                        size_t K, size_t warmup, size_t iterations);
/* As above, but call i uses operand set i % n_sets (A[i], B[i], C[i]) so that repeated
 * calls on small operands stream from HBM instead of the on-chip caches. */
double hgemm_profile_rotating_ms(hgemm_fn fn, const hgemm_half *const *A, const hgemm_half *const *B,
                                 hgemm_half *const *C, size_t n_sets, size_t M, size_t N, size_t K, size_t warmup,
                                 size_t iterations);
/* Shader clock sustained between two points of the null stream (no counterpart in the
 * reference, whose hardware held its clock: on a power-managed part the clock under matrix
 * load differs from board to board, and throughput is only comparable together with it).
 * hgemm_clock_mark(0) and hgemm_clock_mark(1) each enqueue a small kernel whose waves sample
 * the shader-cycle counter and the constant-rate counter and file the pair under the SIMD
 * they run on (the first mark on a device allocates the 512 KB the samples live in).
 * hgemm_clock_between_marks_mhz waits for the device and returns the average shader clock in
 * MHz between the marks, taken over the SIMDs that were sampled at both; per XCD into
 * per_xcd_mhz[0 .. xcds) if not NULL (0 for an XCD without such a SIMD); through elapsed_ms
 * if not NULL the time between the marks by the constant-rate counter; through detail if not
 * NULL three numbers: the lowest and the highest clock of a single SIMD, and how many SIMDs
 * were used. */
void hgemm_clock_mark(int which);
double hgemm_clock_between_marks_mhz(double *per_xcd_mhz, int xcds, double *elapsed_ms, double *detail);
/* 2*M*N*K*1e-12 / (ms*1e-3)  (reference src/common/tester.h:96-97). */
double hgemm_tflops(size_t M, size_t N, size_t K, double ms);
/* Algorithmic bytes of one call: 2*(M*K + K*N + M*N). */
double hgemm_bytes(size_t M, size_t N, size_t K);

/* Library version string. */
const char *hgemm_version(void);

#ifdef __cplusplus
}
#endif

#endif /* HGEMM_H_ */
