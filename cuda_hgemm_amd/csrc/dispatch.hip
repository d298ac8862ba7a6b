// hgemm_skinny and hgemm_auto: shape-driven choice among the tuned kernels.
#include "../../include/hgemm.h"
#include "mfma_decode.h"
#include "mfma_decode_ring.h"
#include "mfma_decode_resident.h"
#include "mfma_pipelined.h"
#include "mfma_ragged.h"
#include "mfma_skinny.h"
#include "plan.h"

#include <atomic>
#include <map>
#include <mutex>

namespace hgemm {

namespace {

constexpr size_t MAX_PARTIAL_BYTES = PlanLimits().partial_bytes;
constexpr size_t MAX_PADDED_BYTES = PlanLimits().operand_bytes;
constexpr int MAX_DEVICES = 64;

int current_device() {
    int dev = 0;
    HGEMM_CHECK_HIP_ERROR(hipGetDevice(&dev));
    HGEMM_CHECK_MSG(dev >= 0 && dev < MAX_DEVICES, "device %d beyond the %d this library keeps state for", dev, MAX_DEVICES);
    return dev;
}

// Heap workspaces of hgemm_auto / hgemm_skinny, one pair per device, kept for the life of
// the process (the reference keeps its vendor handle the same way,
// src/cublas_tensor_op.cu:18).  Each is allocated once, at its cap, the first time a plan
// needs it (or by hgemm_reserve_workspace).  If the cap cannot be had, the size asked for is
// tried, and sizes hipMalloc has refused are remembered so that no later call asks again.
// An entry point never frees or replaces a buffer: a plan that needs more than the buffer
// holds (possible only after such a refusal) is not run, the caller plans again without a
// workspace.  Only hgemm_reserve_workspace and hgemm_release_workspace replace or free, after
// waiting for the device.
//
// g_heap_mutex guards the table AND is held while the launches of a plan that uses a
// workspace are enqueued: every launch goes to the null stream, which runs them in the order
// they were enqueued, so with the lock held two host threads cannot interleave one plan's
// partial-sum kernel with the other's reduction, and no thread holds a workspace pointer
// while another frees it.
struct HeapState {
    Workspace ws;
    size_t partial_refused = SIZE_MAX, operand_refused = SIZE_MAX;  // smallest size hipMalloc has refused
};
std::mutex g_heap_mutex;
HeapState g_heap[MAX_DEVICES];

// Caller holds g_heap_mutex.  `may_replace`: an existing, smaller buffer may be freed (after a device synchronisation).
bool grow(void **ptr, size_t *have, size_t need, size_t cap, size_t *refused, bool may_replace) {
    if (need <= *have) return true;
    if (need >= *refused) return false;
    if (*ptr) {
        if (!may_replace) return false;
        HGEMM_CHECK_HIP_ERROR(hipDeviceSynchronize());
        HGEMM_CHECK_HIP_ERROR(hipFree(*ptr));
        *ptr = nullptr;
        *have = 0;
    }
    for (size_t want : {need > cap ? need : cap, need}) {
        if (want >= *refused) continue;
        if (hipMalloc(ptr, want) == hipSuccess) {
            *have = want;
            return true;
        }
        (void)hipGetLastError();  // clear the allocation failure
        *ptr = nullptr;
        *refused = want;
    }
    return false;
}

// The device's heap workspace with at least the given sizes; false if it does not hold them and
// cannot be made to.  Caller holds g_heap_mutex.
bool heap_workspace(size_t partial_bytes, size_t operand_bytes, Workspace *out, bool may_replace) {
    HeapState &h = g_heap[current_device()];
    Workspace &w = h.ws;
    bool ok = true;
    if (partial_bytes > w.partial_bytes)
        ok = grow(reinterpret_cast<void **>(&w.partial), &w.partial_bytes, partial_bytes, MAX_PARTIAL_BYTES,
                  &h.partial_refused, may_replace) && ok;
    if (operand_bytes > w.operand_bytes)
        ok = grow(reinterpret_cast<void **>(&w.operands), &w.operand_bytes, operand_bytes, MAX_PADDED_BYTES,
                  &h.operand_refused, may_replace) && ok;
    *out = w;
    return ok;
}

// Scratch of the entry point that allocates nothing: a fixed array in the code object, one
// copy per device, partial sums first and padded operands behind them.  In host code the
// array's name is only a handle for hipGetSymbolAddress; kernels get the device address.
constexpr size_t STATIC_WORKSPACE_BYTES = HGEMM_STATIC_WORKSPACE_BYTES;
static __device__ __align__(256) unsigned char scratch[STATIC_WORKSPACE_BYTES];
std::mutex g_scratch_mutex;
unsigned char *g_scratch_ptr[MAX_DEVICES];

unsigned char *static_scratch() {
    const int dev = current_device();
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void *ptr = nullptr;
        HGEMM_CHECK_HIP_ERROR(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
        HGEMM_CHECK(ptr != nullptr);
        g_scratch_ptr[dev] = reinterpret_cast<unsigned char *>(ptr);
    }
    return g_scratch_ptr[dev];
}

int compute_units() {
    static int cus = [] {
        // A planning query must also work where no GPU is visible: assume one MI355X.
        int dev = 0, n = 0;
        if (hipGetDevice(&dev) != hipSuccess) return 256;
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) return 256;
        return n > 0 ? n : 256;
    }();
    return cus;
}

template <class Cfg>
void launch_splitk(const void *A, const void *B, void *C, size_t M, size_t N, size_t K, int splits,
                   const Workspace &ws) {
    static bool configured = [] {
        HGEMM_CHECK_HIP_ERROR(hipFuncSetAttribute(reinterpret_cast<const void *>(&hgemm_skinny_kernel<Cfg, false>),
                                                  hipFuncAttributeMaxDynamicSharedMemorySize, Cfg::LDS_BYTES));
        HGEMM_CHECK_HIP_ERROR(hipFuncSetAttribute(reinterpret_cast<const void *>(&hgemm_skinny_kernel<Cfg, true>),
                                                  hipFuncAttributeMaxDynamicSharedMemorySize, Cfg::LDS_BYTES));
        return true;
    }();
    (void)configured;
    HGEMM_CHECK(N % Cfg::BN == 0);
    HGEMM_CHECK(splits >= 1 && K % (size_t)Cfg::BK == 0 && K / (size_t)Cfg::BK >= (size_t)splits);
    const size_t tiles_n = N / Cfg::BN, tiles = tiles_n * div_ceil(M, Cfg::BM);  // < 2^31 / (BM * BN)
    const dim3 grid((unsigned)tiles, (unsigned)splits);
    HGEMM_CHECK(splits <= 65535);
    float *partial = nullptr;
    if (splits > 1) {
        HGEMM_CHECK(ws.partial != nullptr && ws.partial_bytes >= (size_t)splits * M * N * sizeof(float));
        partial = ws.partial;
    }
    // a B of 48 MB or more is streamed past the caches: +2-12 % from 64 MB up (N = 8192 ... 28672 at K = 4096),
    // 0-7 % slower at 32 MB (N = K = 4096), where the next call finds parts of B in the Infinity Cache otherwise
    const bool stream_b = div_ceil(M, Cfg::BM) == 1 && N * K >= ((size_t)24 << 20);
    auto kernel = stream_b ? &hgemm_skinny_kernel<Cfg, true> : &hgemm_skinny_kernel<Cfg, false>;
    kernel<<<grid, dim3(Cfg::THREADS), Cfg::LDS_BYTES, nullptr>>>(
        reinterpret_cast<const half_t *>(A), reinterpret_cast<const half_t *>(B), reinterpret_cast<half_t *>(C),
        partial, (int)M, (int)N, (int)K, splits, (int)tiles_n);
    HGEMM_CHECK_HIP_ERROR(hipGetLastError());
    if (splits > 1) launch_splitk_reduce(partial, reinterpret_cast<half_t *>(C), M * N, splits);
}

//                             BM   BN  WM WN stages
using Split32x64 = SkinnyConfig<32, 64, 1, 2, 4>;
using Split64x64 = SkinnyConfig<64, 64, 2, 2, 4>;
using Split64x128 = SkinnyConfig<64, 128, 2, 2, 4>;
using Split128x64 = SkinnyConfig<128, 64, 2, 2, 4>;
using Split128x128 = SkinnyConfig<128, 128, 2, 2, 4>;

// 256x256x64 tile on v_mfma_f32_16x16x32_f16, two B buffers and three A buffers (all 160 KB of LDS)
using Big256 = PipeConfig<256, 256, 64, 2, 2, 2, 16, 1>;
using Mid128 = PipeConfig<128, 128, 64, 2, 2, 5, 16>;
// two LDS buffers (64 KB): two workgroups fit a CU, and one's C tile goes out while the other multiplies.  Pays where
// a workgroup's K loop is shorter than its epilogue and C outgrows the Infinity Cache: 16384^2 x 256 201 -> 170 us.
using Mid128S2 = PipeConfig<128, 128, 64, 2, 2, 2, 16>;
using Small64 = PipeConfig<64, 64, 64, 1, 1, 3, 16>;
// one row of tiles for M <= 64: four waves side by side, 64x32 each
using Row64x128 = PipeConfig<64, 128, 64, 1, 4, 5, 16>;
// one row of tiles for M = 129 ... 192: four stages of 24 + 16 KB are the whole LDS
using Row192x128 = PipeConfig<192, 128, 64, 2, 2, 4, 16>;
using Tile192 = PipeConfig<192, 192, 64, 2, 2, 3, 16>;
using Rect256x128 = PipeConfig<256, 128, 64, 2, 2, 3, 16>;
// 64x64x64 on four waves (one 32x32 MFMA tile each) with the ladder's kernel: a small tile whose chunk takes a quarter
// of the one-wave tile's matrix-pipe time; for grids that give a CU at most one tile.  Three forms by the number of
// chunks a workgroup walks: the plain 3-stage ring up to 4 (the look-ahead prologue costs more than it returns),
// the look-ahead loop on 5 stages (also the entry point hgemm_mfma_tiled_64x64; 4 stages are 1-2 % ahead while the
// operands sit in L2 and 15-25 % behind once they do not: 512 x 512 x 4096), and on 6 stages from 40 chunks
// (K >= 2560 per slice), where one more chunk in flight pays.
using Small64W4Short = TileConfig<64, 64, 64, 2, 2, 3, LOAD_DMA, LDS_SWIZZLE, true>;
using Small64W4 = TileConfig<64, 64, 64, 2, 2, 5, LOAD_DMA, LDS_SWIZZLE, true, true>;
using Small64W4Deep = TileConfig<64, 64, 64, 2, 2, 6, LOAD_DMA, LDS_SWIZZLE, true, true>;
// two workgroups per CU (grids of one to two tiles per CU): the 4-stage form, 64 KB each, 0-6 % ahead of 5 stages there
using Small64W4Pair = TileConfig<64, 64, 64, 2, 2, 4, LOAD_DMA, LDS_SWIZZLE, true, true>;
constexpr size_t W4_SHORT_MAX_CHUNKS = 4, W4_DEEP_MIN_CHUNKS = 40;

// Pipelined kernel with K cut into `splits` slices: fp32 partial sums per slice, then the
// ordered reduction (the same one the small-M kernel uses), so the result is bit-identical
// from run to run.
template <class Cfg>
void launch_pipelined_plan(const void *A, const void *B, void *C, size_t M, size_t N, size_t K, const Plan &plan,
                           const Workspace &ws) {
    const int splits = plan.splits;
    if constexpr (Cfg::BM == 256 && Cfg::BN == 256) {
        switch (plan.tail_kernel) {
            case KERNEL_R256x128:
                launch_pipelined_with_subtiles<Cfg, Rect256x128>(A, B, C, M, N, K, plan.tail_tiles, "hgemm_auto");
                return;
            case KERNEL_MID128:
                launch_pipelined_with_subtiles<Cfg, Mid128>(A, B, C, M, N, K, plan.tail_tiles, "hgemm_auto");
                return;
            case KERNEL_SMALL64:
                launch_pipelined_with_subtiles<Cfg, Small64>(A, B, C, M, N, K, plan.tail_tiles, "hgemm_auto");
                return;
            default: break;
        }
    }
    if (plan.tail_splits > 1) {
        HGEMM_CHECK(ws.partial != nullptr &&
                    ws.partial_bytes >= (size_t)plan.tail_splits * plan.tail_tiles * Cfg::BM * Cfg::BN * sizeof(float));
        launch_pipelined_with_tail<Cfg>(A, B, C, ws.partial, M, N, K, plan.tail_tiles, plan.tail_splits, "hgemm_auto");
        return;
    }
    if (splits <= 1) {
        launch_pipelined<Cfg>(A, B, C, M, N, K, "hgemm_auto");
        return;
    }
    HGEMM_CHECK(ws.partial != nullptr && ws.partial_bytes >= (size_t)splits * M * N * sizeof(float));
    launch_pipelined_split<Cfg>(A, B, ws.partial, M, N, K, splits, "hgemm_auto");
    launch_splitk_reduce(ws.partial, reinterpret_cast<half_t *>(C), M * N, splits);
}

// ---- cost model for the tile-aligned shapes.  A candidate is a tile (its kernel), how
// many of its workgroups a CU holds, and three times in microseconds fitted to
// measurements on an MI355X over ~60 shapes (rms error 7 %): `fix` per workgroup
// (prologue, epilogue, scheduling) and the time of one 64-wide K chunk with few (`lo`)
// and with all (`hi`) CUs busy -- the chip is power-limited, so a chunk costs more when
// the whole chip computes.  time = launch + full rounds * (fix + chunks * hi)
//                                 + last partial round * (fix + chunks * between lo and hi)
//                                 + reduction of the fp32 partials when K is split.
struct Candidate {
    int kernel, bm, bn, per_cu, stages;
    double fix, lo, hi;
};
constexpr Candidate CANDIDATES[] = {
    {KERNEL_BIG256, 256, 256, 1, 2, 7.92, 0.841, 1.462},
    {KERNEL_T192, 192, 192, 1, 3, 5.17, 0.495, 0.948},
    {KERNEL_R256x128, 256, 128, 1, 3, 4.25, 0.476, 0.856},
    {KERNEL_MID128, 128, 128, 1, 5, 3.17, 0.266, 0.510},
    {KERNEL_SMALL64, 64, 64, 3, 3, 1.39, 0.294, 0.585},
    // K of at most four chunks only (kept to that below); fitted on 8192^2 ... 16384^2 x 256
    {KERNEL_MID128_S2, 128, 128, 2, 2, 1.77, 0.60, 0.885},
    // whole tiles only, at most one workgroup per CU (larger grids are kept from it below: it is behind there);
    // fitted on 16 to 256 workgroups, K = 256 to 16384, in the forms run_plan picks by the length of a slice
    {KERNEL_SMALL64_W4, 64, 64, 1, 3, 2.40, 0.168, 0.195},
    // the same tile with two workgroups sharing a CU (its 5-stage form takes 80 KB of LDS): grids of one to two
    // tiles per CU, unsliced, fewer than 40 chunks (kept to that below); fitted on 1088^2 ... 1408^2, K = 512 ... 2048,
    // where it is 7-19 % ahead of the 128x128 and one-wave 64x64 tiles; from 2 x CUs + 1 tiles on it is far behind
    {KERNEL_SMALL64_W4, 64, 64, 2, 3, 2.40, 0.10, 0.40},
};
// launch; reduction kernel: fixed + per slice + fp32 partials written and read back.  Partial sums of a few MB
// come back from the L2s: measured 3.0 us behind the same kernel at 2.4 MB against 4.5-5 us at 4.2 MB, and twice
// the slices cost nothing there.  (Refitted with K-sliced launches dealt slice-major: 2.8-7.4 us for 2-17 MB.)
constexpr double LAUNCH_US = 0.16, REDUCE_US = 3.00, REDUCE_SLICE_US = 0.10, REDUCE_BYTES_PER_US = 8700e3;
constexpr double REDUCE_SMALL_US = 2.40, REDUCE_SMALL_SLICE_US = 0.05, REDUCE_SMALL_BYTES = 3e6;
double reduce_us(int slices, double elems) {
    const double bytes = (double)slices * elems * 4.0;
    const bool small = bytes <= REDUCE_SMALL_BYTES;
    return (small ? REDUCE_SMALL_US : REDUCE_US) + (small ? REDUCE_SMALL_SLICE_US : REDUCE_SLICE_US) * slices +
           2.0 * bytes / REDUCE_BYTES_PER_US;
}
// extra cost of finishing a grid with a separate launch for its last round: in K slices / on smaller tiles
constexpr double TAIL_US = 3.6, TAIL_SUB_US = 4.4;
size_t padded_n(size_t N) { return (N + 7) / 8 * 8; }
size_t padded_k(size_t K) { return (K + 63) / 64 * 64; }
// A' (M x K'), B' (N' x K') and, when N grows, C' (M x N')
size_t padded_bytes(size_t M, size_t N, size_t K) {
    const size_t Np = padded_n(N), Kp = padded_k(K);
    return ((M + Np) * Kp + (Np != N ? M * Np : 0)) * sizeof(half_t);
}

double predict_us(const Candidate &c, size_t M, size_t N, size_t K, int splits, size_t cus) {
    const size_t wgs = div_ceil(M, (size_t)c.bm) * div_ceil(N, (size_t)c.bn) * (size_t)splits;
    const size_t slots = cus * (size_t)c.per_cu;
    const double chunks = (double)div_ceil(K / 64, (size_t)splits);  // the longest slice
    const size_t full = wgs / slots, rem = wgs % slots;
    double t = LAUNCH_US + (double)full * (c.fix + chunks * c.hi);
    if (rem) t += c.fix + chunks * (c.lo + (c.hi - c.lo) * (double)rem / (double)slots);
    if (splits > 1) t += reduce_us(splits, (double)M * (double)N);
    return t;
}

// The same grid with its last, partly filled round (`rem` workgroups) run in `ts` K slices
// so that it fills the chip too: whole rounds, then one round of rem * ts shorter
// workgroups, then the reduction of their compact fp32 partial sums.
double predict_tail_us(const Candidate &c, size_t M, size_t N, size_t K, int ts, size_t cus) {
    const size_t wgs = div_ceil(M, (size_t)c.bm) * div_ceil(N, (size_t)c.bn), slots = cus * (size_t)c.per_cu;
    const size_t full = wgs / slots, rem = wgs % slots;
    const double chunks = (double)(K / 64);
    double t = LAUNCH_US + (double)full * (c.fix + chunks * c.hi);
    t += LAUNCH_US + c.fix + (double)div_ceil(K / 64, (size_t)ts) * (c.lo + (c.hi - c.lo) * (double)(rem * ts) / (double)slots);
    t += reduce_us(ts, (double)rem * c.bm * c.bn) + TAIL_US;
    return t;
}

// A grid of 256x256 tiles whose last round (`rem` workgroups) is handed to a smaller tile
// that divides it: whole rounds of the big tile, then rem * parts workgroups of the small
// one.  No partial sums and no reduction.
double predict_subtile_us(const Candidate &big, const Candidate &small, size_t M, size_t N, size_t K, size_t cus) {
    const size_t wgs = div_ceil(M, (size_t)big.bm) * div_ceil(N, (size_t)big.bn), slots = cus * (size_t)big.per_cu;
    const size_t full = wgs / slots, rem = wgs % slots;
    const size_t parts = (size_t)(big.bm / small.bm) * (big.bn / small.bn);
    const size_t small_slots = cus * (size_t)small.per_cu, small_wgs = rem * parts;
    const double chunks = (double)(K / 64);
    double t = LAUNCH_US + (double)full * (big.fix + chunks * big.hi);
    t += LAUNCH_US + (double)(small_wgs / small_slots) * (small.fix + chunks * small.hi);
    if (small_wgs % small_slots)
        t += small.fix + chunks * (small.lo + (small.hi - small.lo) * (double)(small_wgs % small_slots) / (double)small_slots);
    return t + TAIL_SUB_US;
}

// Number of K slices (1 ... 16) for `tiles` output tiles of a split-K kernel, by a model of its time fitted to 91
// shapes (M = 7 ... 128, N = 1408 ... 65536, K = 384 ... 15104, all five tiles) timed at every slice count on an MI355X,
// operands rotated so that B streams from HBM:
//     t(s) = t_B (1 + [s > 1] 8 s M / K) / balance(s) + [s > 1] 1 us,    t_B = 2 N K bytes at 5 TB/s,
// balance(s) = w / (ceil(w / CUs) CUs) for w = tiles x s workgroups: the busiest CU runs ceil(w / CUs) of them, whether
// side by side or one after the other, so 144 tiles run better in three slices (432 workgroups, two on most CUs) than
// in two (288: two on a few CUs, one on the rest) -- M = 48, N = 9216, K = 8192: 43.8 / 45.0 / 35.8 / 41.9 us in 1 ... 4
// slices.  The middle factor is the traffic of the fp32 partial sums (8 M bytes per slice and column of C, out and
// back) against B's (2 K bytes per column), counted twice.  The model's choice is 1.2 % behind the best count on
// average (16 % at worst); the rule it replaces (the smallest power of two that divides K's chunks and gives three
// quarters of the CUs a workgroup) was 22 % behind on average.  A slice is a whole number of 64-wide chunks, at least
// two (`min_chunks`: the pipelined tiles need as many as their ring has stages); slices differ by at most one chunk.
// `slice_bytes`: fp32 partial sums of one slice; the slices together stay within `limit`.
int choose_splits(size_t tiles, size_t M, size_t N, size_t cus, size_t K, size_t slice_bytes, size_t limit,
                  size_t min_chunks = 2) {
    int best = 1;
    double best_us = 0.0;
    const double stream_us = 2.0 * (double)N * (double)K / 5e6;
    for (int s = 1; s <= 16; ++s) {
        if (s > 1 && (K % 64 != 0 || K / 64 / (size_t)s < min_chunks || (size_t)s * slice_bytes > limit)) break;
        const size_t wgs = tiles * (size_t)s;
        const double balance = (double)wgs / (double)(div_ceil(wgs, cus) * cus);
        const double partials = s > 1 ? 8.0 * s * (double)M / (double)K : 0.0;
        const double us = stream_us * (1.0 + partials) / balance + (s > 1 ? 1.0 : 0.0);
        if (s == 1 || us < best_us - 1e-9) {
            best_us = us;
            best = s;
        }
    }
    return best;
}


// ---- kernels for M <= 128 ("decode-shaped": B is streamed once, the bound is HBM bandwidth).  Which kernel runs
// where was settled by timing the candidates against each other on an MI355X, operands rotated so that every call
// reads HBM: library builds with and without a rule, hgemm_auto on both in one process, over K = 256 ... 28672 x
// N = 256 ... 32768 x M = 1 ... 128.  The outcome is this table: the first row that covers a shape, and whose
// kernel can run it (divisibility), decides.  Rows are boxes in (M, N, K, elements of B); the two conditions that
// are not boxes are flags.
enum SmallMFlags {
    RULE_K_BELOW_4N = 1,        // only where K < 4 N (beyond, K slices across workgroups win)
    RULE_K_NOT_16384S = 2,      // not where K is a multiple of 16384 (the ring kernel's 16 rows of B per workgroup then
                                // lie 32 KB apart: 20-28 % behind)
};
struct SmallMRule {
    int m_lo, m_hi;
    size_t n_lo, n_hi, k_lo, k_hi, b_lo, b_hi;  // inclusive bounds; b = N * K, the elements of B
    int flags, kernel;
};
constexpr size_t ANY = ~(size_t)0;
constexpr size_t LARGE_B = (size_t)48 << 20;  // elements: a B of 96 MB
constexpr SmallMRule SMALL_M_RULES[] = {
    // --- M = 1 ... 8.  Below K = 1024 the streaming kernel (as fast or faster, M = 1 by 6-26 %) where it can run,
    // i.e. N % 32 == 0 and K % 256 == 0; else the ring kernel (2.0x median over what ran such shapes before).
    {1, 8, 1, 8192, 256, 1023, 0, ANY, 0, KERNEL_DECODE_BN16},
    // The ring kernel: 0-60 % ahead (median 18 %); not for K < 2048 against N > 8192 (up to 4 % behind at M = 1).  Its
    // copies of B carry the non-temporal hint from 48 MB of B on, and with the hint it is also ahead against a B of
    // 96 MB or more, where the streaming and split-K kernels used to tie with it: K = 1024 ... 12288 x N = 10240 ...
    // 57344, M = 1: 0.97 ... 1.18x (N = 28672, K = 4096: 39.2 -> 35.9 us, 82 % of 8 TB/s; N = 57344: 87 %), M = 8:
    // 0.95 ... 1.31x from K = 2048 (ties at K = 1024).
    {1, 8, 1, 8192, 256, 2047, 0, ANY, 0, KERNEL_DECODE_RING},
    {1, 8, 1, ANY, 2048, 8191, 0, LARGE_B - 1, 0, KERNEL_DECODE_RING},
    {1, 8, 1, ANY, 8192, ANY, 0, LARGE_B - 1, 0, KERNEL_DECODE_RING},
    {1, 8, 1, ANY, 8192, ANY, LARGE_B, ANY, RULE_K_NOT_16384S, KERNEL_DECODE_RING},
    {1, 5, 1, ANY, 1024, 8191, LARGE_B, ANY, 0, KERNEL_DECODE_RING},
    {6, 8, 1, ANY, 2048, 8191, LARGE_B, ANY, 0, KERNEL_DECODE_RING},
    // M = 6 ... 8 against a B of 96 MB or more with K < 2048: the split-K kernel (2-16 % ahead of the streaming
    // kernel); below M = 6 and for smaller B the streaming kernel stays ahead.
    {6, 8, 1, ANY, 1, ANY, LARGE_B, ANY, 0, KERNEL_SPLIT_32x64},
    {1, 8, 1, ANY, 1, ANY, 0, ANY, 0, KERNEL_DECODE_BN16},
    // --- M = 9 ... 24 against N >= 14336: the persistent kernel that keeps A in registers, where every wave can hold
    // its slice of A (K = 512 ... 1536 per wave, eight waves; four waves of 1280 at K = 5120).  Against what ran these
    // shapes before, over N = 14336 ... 57344: K = 6144 (split-K before) 1.06 ... 1.30x, K = 10240 and 12288 1.08 ... 1.40x,
    // K = 5120 1.07 ... 1.31x from N = 18432 (0.96 ... 1.08x at 14336), K = 8192 (ring kernel) 1.03 ... 1.14x, K = 4096
    // 1.04 ... 1.06x at M = 16 from N = 18432 (N = 28672: 40.1 -> 37.8 us) and level at M = 9, so from M = 13; M = 17 ... 24
    // (two row tiles, 64x128 pipelined tile before) 1.09 ... 1.13x at N = 18432 and 57344 and 0.93 ... 1.09x at N = 28672
    // depending on the box; M = 25 ... 32 mixed up to N = 32000 (0.88 ... 1.07x) and 1.07 ... 1.24x against N = 40960 ...
    // 151936 (the 64x128 tile's second and later rounds cost it more), so from N = 32768; K <= 3072 mixed (0.68 ... 1.2x),
    // so not taken.
    {9, 16, 18432, ANY, 5120, 5120, (size_t)24 << 20, ANY, 0, KERNEL_DECODE_RESIDENT},
    {9, 16, 14336, ANY, 10240, 10240, (size_t)24 << 20, ANY, 0, KERNEL_DECODE_RESIDENT},
    {9, 16, 14336, ANY, 12288, 12288, (size_t)24 << 20, ANY, 0, KERNEL_DECODE_RESIDENT},
    {9, 16, 14336, ANY, 6144, 6144, (size_t)24 << 20, ANY, 0, KERNEL_DECODE_RESIDENT},
    {9, 16, 14336, ANY, 8192, 8192, (size_t)24 << 20, ANY, 0, KERNEL_DECODE_RESIDENT},
    {13, 16, 18432, ANY, 4096, 4096, (size_t)24 << 20, ANY, 0, KERNEL_DECODE_RESIDENT},
    {17, 24, 18432, ANY, 4096, 4096, (size_t)24 << 20, ANY, 0, KERNEL_DECODE_RESIDENT},
    {25, 32, 32768, ANY, 4096, 4096, (size_t)24 << 20, ANY, 0, KERNEL_DECODE_RESIDENT},
    // --- M = 9 ... 16: the ring kernel up to N = 8192 while K <= 4096 (K <= 8192 up to N = 4096); beyond, K slices
    // across workgroups are up to 29 % ahead -- except, with the non-temporal copies, against a B of 48 MB or more at
    // K = 2048, 4096 and 8192, where every wave walks 1024 of K (M = 12: 1.05 ... 1.29x, M = 16: 0.97 ... 1.23x over
    // N = 10240 ... 57344); at K = 1024, 3072, 6144 and 12288 the split-K kernel stays ahead (0.84 ... 1.06x).
    {9, 16, 1, 8192, 256, 4096, 0, ANY, RULE_K_BELOW_4N, KERNEL_DECODE_RING},
    {9, 16, 1, 4096, 4097, 8192, 0, ANY, RULE_K_BELOW_4N, KERNEL_DECODE_RING},
    {9, 16, 8193, ANY, 2048, 2048, (size_t)24 << 20, ANY, 0, KERNEL_DECODE_RING},
    {9, 16, 8193, ANY, 4096, 4096, (size_t)24 << 20, ANY, 0, KERNEL_DECODE_RING},
    {9, 16, 8193, ANY, 8192, 8192, (size_t)24 << 20, ANY, 0, KERNEL_DECODE_RING},
    // --- M = 17 ... 64 (two or four row tiles of A per wave): the ring kernel while K is short, where one launch beats
    // the split-K kernel plus the launch that adds its slices: K < 1024 up to N = 8192 (median 1.65x), K <= 2048 up
    // to N = 4096 (median 1.31x); and up to K = 4096 for M <= 24 against N = 3072 ... 4096 (median 1.21x; at
    // N <= 2048 M = 24 is 1-9 % behind).
    {17, 64, 1, 8192, 256, 1023, 0, ANY, RULE_K_BELOW_4N, KERNEL_DECODE_RING},
    {17, 64, 1, 4096, 1024, 2048, 0, ANY, RULE_K_BELOW_4N, KERNEL_DECODE_RING},
    {17, 24, 3072, 4096, 2049, 4096, 0, ANY, RULE_K_BELOW_4N, KERNEL_DECODE_RING},
    // --- M = 65 ... 128 (eight row tiles): the ring kernel for K <= 512 up to N = 8192, K <= 1024 up to N = 4096
    // (median 1.45x).
    {65, 128, 1, 8192, 256, 512, 0, ANY, RULE_K_BELOW_4N, KERNEL_DECODE_RING},
    {65, 128, 1, 4096, 513, 1024, 0, ANY, RULE_K_BELOW_4N, KERNEL_DECODE_RING},
    // Against N >= 18432 (at least 144 column tiles, i.e. more than half the CUs busy without K slices): one launch
    // of the hand-scheduled 128x128 tile, B copied with the non-temporal hint.  K = 2048 ... 8192 x N = 18432 ...
    // 32768, M = 65 and 128: 3-50 % ahead of the split-K kernels (N = 28672, K = 4096, M = 128: 53.1 -> 48.6 us,
    // 62.6 % of 8 TB/s), K = 384 ... 768 x N = 28672, 57344: 1.11 ... 1.24x; at N = 16384 mixed (0.84 ... 1.14), below
    // it behind (0.76 ... 0.90).  From K = 320, the shortest K its five-stage ring takes.
    // N = 32769 ... 49152 are 257 ... 384 column tiles of 128, i.e. a second round of workgroups on a part of the chip, but
    // at most 256 tiles of 192: one row of the 192x192 tile (its rows beyond M idle, which an HBM-bound kernel can
    // afford) is 1.11 ... 1.34x up to K = 4096 over N = 34816 ... 49152 (M = 100, N = 36864, K = 1024: 27.1 -> 22.5 us);
    // at K = 8192, where the 128x128 tile finishes its second round in K slices, 0.94 ... 1.03x.
    {65, 128, 32769, 49152, 192, 6144, 0, ANY, 0, KERNEL_T192},
    {65, 128, 18432, ANY, 320, ANY, 0, ANY, 0, KERNEL_MID128},
    // M = 33 ... 64 there: the same kernel on a 64x128 tile, four waves side by side.  K = 384 ... 8192 x N = 18432 ...
    // 57344: 1-4 % ahead of the split-K 64x128 kernel where that ran unsliced (N = 28672, K = 4096, M = 64: 43.3 ->
    // 42.4 us, 70 % of 8 TB/s), 1.35x where it ran in two slices (N = 18432, 20480).
    // (the 192-wide tile here only while the second round of 64x128 tiles would be almost empty: N = 34816: 0.97 ... 1.27x
    // over K = 512 ... 4096; N = 40960: 0.91 ... 1.10x; N = 49152: 0.88 ... 1.03x)
    {33, 64, 32769, 36864, 192, 6144, 0, ANY, 0, KERNEL_T192},
    {33, 64, 18432, ANY, 320, ANY, 0, ANY, 0, KERNEL_ROW64x128},
    // M = 17 ... 32 take that tile too once K is long (half its rows are idle, which an HBM-bound kernel can afford):
    // K = 4096, 8192 x N = 18432 ... 57344: 0.97 ... 1.27x over the split-K 32x64 kernel; K = 2944 ... 3584: 1.00 ... 1.15x;
    // at K <= 2560 that kernel stays ahead or level against N >= 28672 (0.92 ... 1.05x).
    {17, 32, 18432, ANY, 3072, ANY, 0, ANY, 0, KERNEL_ROW64x128},
    // M = 33 ... 128 against N = 6144 ... 18431 with a long K: the same two tiles with K in slices (their copies of B
    // non-temporal too), the slice count by the split-K family's model: over N = 6144 ... 16384, M = 64 and 128,
    // K = 8192 and 16384: 0.99 ... 1.34x of the split-K kernels at their best slice count (median 1.17x; M = 128,
    // N = 10240, K = 16384: 106.9 -> 79.8 us); at K = 4096 mixed (0.92 ... 1.13x), at K = 2048 behind (0.80 ... 1.07x).
    // M = 65 ... 128 already from K = 6144: 1.01 ... 1.30x over N = 6144 ... 14336 at K = 6144 and 7168 (median 1.12x).
    {65, 128, 6144, ANY, 6144, ANY, 0, ANY, 0, KERNEL_MID128},
    {33, 64, 6144, ANY, 8192, ANY, 0, ANY, 0, KERNEL_ROW64x128},
    // --- everything else with N % 64 == 0 and K % 64 == 0: the split-K family, the tile by M; 128-wide tiles where
    // N gives enough of them and is a multiple of 128 (they stream B better).
    {1, 32, 1, ANY, 1, ANY, 0, ANY, 0, KERNEL_SPLIT_32x64},
    {33, 64, 16384, ANY, 1, ANY, 0, ANY, 0, KERNEL_SPLIT_64x128},
    {33, 64, 1, ANY, 1, ANY, 0, ANY, 0, KERNEL_SPLIT_64x64},
    {65, 128, 16384, ANY, 1, ANY, 0, ANY, 0, KERNEL_SPLIT_128x128},
    {65, 128, 1, ANY, 1, ANY, 0, ANY, 0, KERNEL_SPLIT_128x64},
};
constexpr int SMALL_M_RULE_COUNT = (int)(sizeof(SMALL_M_RULES) / sizeof(SMALL_M_RULES[0]));

bool small_m_rule_covers(const SmallMRule &r, size_t M, size_t N, size_t K) {
    const size_t b = N * K;
    if (M < (size_t)r.m_lo || M > (size_t)r.m_hi || N < r.n_lo || N > r.n_hi || K < r.k_lo || K > r.k_hi || b < r.b_lo ||
        b > r.b_hi)
        return false;
    if ((r.flags & RULE_K_BELOW_4N) && K >= 4 * N) return false;
    if ((r.flags & RULE_K_NOT_16384S) && K % 16384 == 0) return false;
    return true;
}

// shapes the kernel of a row can run at all (the row is skipped otherwise)
bool small_m_kernel_supports(int kernel, size_t M, size_t N, size_t K) {
    switch (kernel) {
        case KERNEL_DECODE_RING: return decode_ring_supports(M, N, K);
        case KERNEL_DECODE_RESIDENT: return decode_resident_supports(M, N, K);
        case KERNEL_DECODE_BN16: return decode_supports(M, N, K);
        case KERNEL_MID128:
        case KERNEL_ROW64x128: return N % 8 == 0 && K % 64 == 0 && K >= 64 * 5;
        case KERNEL_T192: return N % 8 == 0 && K % 64 == 0 && K >= 64 * 3;
        case KERNEL_SPLIT_64x128:
        case KERNEL_SPLIT_128x128: return skinny_supports(M, N, K) && N % 128 == 0;
        default: return skinny_supports(M, N, K);
    }
}

// One row of BM x 128 tiles, one workgroup per CU, with more column tiles than CUs: the tiles beyond the whole rounds
// would run as a round of their own on a few CUs, so they are cut into K slices that fill the chip (M = 103,
// N = 34304, K = 6656: 268 tiles, 133 us as two rounds, 80 us this way; hipBLASLt 89 us).  Worth its extra launch and
// reduction when the round it shortens is long, i.e. from K of about 2500 ... 4000 on (M = 76, N = 39552, K = 640:
// 19.8 us as two rounds, 23.7 with the 53 tiles of the second in two slices; K = 1280 ... 1792 with the tail: 78 ... 81 %
// of hipBLASLt, K = 4352 ... 6656: 86 ... 111 %).
void one_row_tail(Plan &p, size_t bm, size_t stages, size_t N, size_t K, size_t cus, size_t partial_limit) {
    const size_t tiles = div_ceil(N, (size_t)128), rem = tiles % cus;
    const size_t tile_bytes = bm * 128 * sizeof(float);
    if (tiles <= cus || rem == 0) return;
    size_t ts = cus / rem < 16 ? cus / rem : 16;
    while (ts >= 2 && (shortest_slice(K, 64, (int)ts) < 64 * stages || ts * rem * tile_bytes > partial_limit)) --ts;
    if (ts >= 2 && (double)(K / 64) * (1.0 - 1.0 / (double)ts) > 32.0) {
        p.tail_tiles = (int)rem;
        p.tail_splits = (int)ts;
        p.partial_bytes = ts * rem * tile_bytes;
    }
}

}  // namespace

bool skinny_supports(size_t M, size_t N, size_t K) {
    return M >= 1 && M <= 128 && N > 0 && N % 64 == 0 && K > 0 && K % 64 == 0;
}

bool same_choice(const Plan &a, const Plan &b) {
    return a.kernel == b.kernel && a.splits == b.splits && a.tail_tiles == b.tail_tiles && a.tail_splits == b.tail_splits &&
           a.tail_kernel == b.tail_kernel;
}
bool left_out(const PlanLimits &limits, const Plan &p) {
    for (int i = 0; i < limits.excluded_count; ++i)
        if (same_choice(limits.excluded[i], p)) return true;
    return false;
}
bool left_out(const PlanLimits &limits, int kernel, int splits, int tail_tiles = 0, int tail_splits = 1,
              int tail_kernel = KERNEL_NONE) {
    Plan p;
    p.kernel = kernel, p.splits = splits, p.tail_tiles = tail_tiles, p.tail_splits = tail_splits, p.tail_kernel = tail_kernel;
    return left_out(limits, p);
}

// M <= 128: choices come from timing every candidate (tile x slices) on the specification's
// decode shapes on an MI355X, operands rotated so small problems read HBM.  Larger,
// tile-aligned shapes: the cheapest (tile, slices) pair under the cost model above.
Plan plan_for(size_t M, size_t N, size_t K, const PlanLimits &limits) {
    Plan p;
    if (M == 0 || N == 0 || K == 0) return p;
    const size_t cus = (size_t)compute_units();
    const size_t slice_bytes = M * N * sizeof(float);  // fp32 partial sums of one K slice of the whole product
    // M <= 128: the first row of the table above that covers the shape and whose kernel can run it
    for (const SmallMRule &r : SMALL_M_RULES) {
        if (M > 128) break;
        if (limits.every_small_m_kernel ? (M < (size_t)r.m_lo || M > (size_t)r.m_hi) : !small_m_rule_covers(r, M, N, K)) continue;
        if (!small_m_kernel_supports(r.kernel, M, N, K)) continue;
        p = Plan();
        p.kernel = r.kernel;
        switch (r.kernel) {
            case KERNEL_DECODE_RING: p.splits = decode_ring_waves(M, N, K, cus); break;
            case KERNEL_DECODE_RESIDENT: {
                int chunks = 0;
                p.splits = decode_resident_waves(M, K, &chunks);
                break;
            }
            case KERNEL_DECODE_BN16: {  // the streaming kernel: 16 or 32 columns per workgroup
                int bn = 16, waves = 1;
                decode_plan(M, N, K, cus, &bn, &waves);
                p.kernel = bn == 16 ? KERNEL_DECODE_BN16 : KERNEL_DECODE_BN32;
                p.splits = waves;
                break;
            }
            case KERNEL_T192: p.splits = 1; break;
            case KERNEL_MID128:
            case KERNEL_ROW64x128: {
                // up to one workgroup per CU: K slices by the split-K family's model (the same balance against the
                // same partial sums); more tiles than CUs: whole rounds unsliced, the rest in K slices
                const size_t tiles = div_ceil(N, (size_t)128);
                // (from K = 6144: below, slices were measured level or behind -- M = 96, N = 18432, K = 4096: 40.8 us
                // unsliced, 43.6 in three; at K = 6144 and 7168 against N = 18432 1.00 ... 1.04x)
                p.splits = tiles <= cus && K >= 6144 ? choose_splits(tiles, M, N, cus, K, slice_bytes, limits.partial_bytes, 5) : 1;
                if (p.splits > 1) p.partial_bytes = (size_t)p.splits * slice_bytes;
                if (tiles > cus) one_row_tail(p, r.kernel == KERNEL_MID128 ? 128 : 64, 5, N, K, cus, limits.partial_bytes);
                break;
            }
            default: {  // the split-K family: K slices across workgroups, then the ordered reduction
                const size_t bn = (r.kernel == KERNEL_SPLIT_64x128 || r.kernel == KERNEL_SPLIT_128x128) ? 128 : 64;
                p.splits = choose_splits(N / bn, M, N, cus, K, slice_bytes, limits.partial_bytes);
                if (p.splits > 1) p.partial_bytes = (size_t)p.splits * slice_bytes;
            }
        }
        if (left_out(limits, p)) continue;
        return p;
    }
    p = Plan();
    // M = 129 ... 192 against many columns: one row of 192x128 tiles, B copied non-temporally, where the last round of
    // workgroups is at least 55 % full (N = 18432 ... 32768, 50688 ... 65536, ...).  Against the cost model's choice
    // (192x192 tiles, 150 of them at N = 28672): N = 28672, K = 2048 ... 8192: 1.17 ... 1.30x (M = 192, K = 2048:
    // 40.3 -> 31.4 us), K = 14336: 0.97 ... 1.12x; N = 57344: 1.01 ... 1.13x up to K = 8192, 0.96 ... 0.98x at 14336;
    // N = 14336 (112 tiles): 0.81 ... 0.86x, N = 34304 (268 tiles): 0.76x.  The ring of four stages keeps three chunks
    // of B in flight per CU where the 192x192 tile's three stages keep two.
    {
        const size_t tiles = div_ceil(N, (size_t)128), last = tiles % cus;
        if (M > 128 && M <= 192 && N % 8 == 0 && K % 64 == 0 && K >= 2048 && K <= 12288 && tiles >= 144 &&
            (last == 0 || last * 100 >= cus * 55) && !left_out(limits, KERNEL_ROW192x128, 1)) {
            p.kernel = KERNEL_ROW192x128;
            p.splits = 1;
            return p;
        }
    }
    // Pipelined tiles: M and N may end inside a tile (guarded edges; the model charges whole
    // tiles), as long as rows of C stay 16-byte aligned and K is a whole number of chunks.
    double best = 0.0;
    for (const Candidate &c : CANDIDATES) {
        if (N % 8) break;
        const bool whole_tiles_only = c.kernel == KERNEL_SMALL64_W4;
        if (whole_tiles_only && (M % c.bm || N % c.bn)) continue;
        for (int s = 1; s <= 32; ++s) {  // K slices: whole chunks, as even as that allows
            if (whole_tiles_only) {
                const size_t wgs = (M / c.bm) * (N / c.bn) * (size_t)s;
                if (wgs > cus * (size_t)c.per_cu) break;
                if (c.per_cu == 2 && (wgs <= cus || s > 1 || K / 64 >= W4_DEEP_MIN_CHUNKS)) break;
                // most CUs busy and a long walk per workgroup: the 128x128 tile in K slices moves half the bytes per
                // flop into LDS and is ahead (1024^2 x 7168: 25.3 us here, 22.2 us in four slices of 128x128 tiles;
                // level at K = 5120, behind at 4096)
                if (wgs * 4 > cus * 3 && shortest_slice(K, 64, s) >= 64 * 96) continue;
            }
            if (c.kernel == KERNEL_MID128_S2 && (s > 1 || K > 256)) break;
            // whole 64x64 tiles, at most one workgroup per CU: the four-wave tile is ahead of the one-wave tile on
            // every such grid that was measured (the model, fitted on larger grids, flatters the one-wave tile there)
            if (c.kernel == KERNEL_SMALL64 && M % 64 == 0 && N % 64 == 0 && (M / 64) * (N / 64) * (size_t)s <= cus) continue;
            if (K % 64 || shortest_slice(K, 64, s) < (size_t)64 * c.stages) break;
            if (s > 1 && (size_t)s * slice_bytes > limits.partial_bytes) break;
            if (left_out(limits, c.kernel, s)) continue;
            const double t = predict_us(c, M, N, K, s, cus);
            if (p.kernel == KERNEL_NONE || t < best) {
                best = t;
                p.kernel = c.kernel;
                p.splits = s;
                p.est_us = t;
                p.tail_tiles = 0;
                p.tail_splits = 1;
                p.tail_kernel = KERNEL_NONE;
                p.partial_bytes = s > 1 ? (size_t)s * slice_bytes : 0;
            }
        }
        // a grid of whole rounds plus a few workgroups: run those few in K slices
        const size_t wgs = div_ceil(M, (size_t)c.bm) * div_ceil(N, (size_t)c.bn), slots = cus * (size_t)c.per_cu;
        const size_t rem = wgs % slots;
        if (wgs > slots && rem > 0 && !whole_tiles_only && c.kernel != KERNEL_MID128_S2) {
            for (int ts = 2; ts <= 16; ++ts) {
                if (K % 64 || shortest_slice(K, 64, ts) < (size_t)64 * c.stages || rem * ts > slots) break;
                if ((size_t)ts * rem * c.bm * c.bn * sizeof(float) > limits.partial_bytes) break;
                if (left_out(limits, c.kernel, 1, (int)rem, ts)) continue;
                const double t = predict_tail_us(c, M, N, K, ts, cus);
                if (p.kernel != KERNEL_NONE && t < best) {
                    best = t;
                    p.kernel = c.kernel;
                    p.splits = 1;
                    p.est_us = t;
                    p.tail_tiles = (int)rem;
                    p.tail_splits = ts;
                    p.tail_kernel = KERNEL_NONE;
                    p.partial_bytes = (size_t)ts * rem * c.bm * c.bn * sizeof(float);
                }
            }
            if (c.kernel == KERNEL_BIG256) {  // ... or on smaller tiles that divide this one
                for (const Candidate &small : CANDIDATES) {
                    if (small.kernel == KERNEL_BIG256 || small.kernel == KERNEL_SMALL64_W4 || small.kernel == KERNEL_MID128_S2 ||
                        c.bm % small.bm || c.bn % small.bn)
                        continue;
                    if (K < (size_t)64 * small.stages || left_out(limits, c.kernel, 1, (int)rem, 1, small.kernel)) continue;
                    const double t = predict_subtile_us(c, small, M, N, K, cus);
                    if (p.kernel != KERNEL_NONE && t < best) {
                        best = t;
                        p.kernel = c.kernel;
                        p.splits = 1;
                        p.est_us = t;
                        p.tail_tiles = (int)rem;
                        p.tail_splits = 1;
                        p.tail_kernel = small.kernel;
                        p.partial_bytes = 0;
                    }
                }
            }
        }
    }
    if (p.kernel != KERNEL_NONE) return p;
    if (limits.excluded_count > 0) return Plan();  // the tuner's question has no further answer
    if (N % 64 == 0 && K % 64 == 0) {  // any M: rows beyond M are guarded
        p.kernel = KERNEL_SPLIT_64x64;
        p.splits = choose_splits(div_ceil(M, 64) * (N / 64), M, N, cus, K, slice_bytes, limits.partial_bytes);
        if (p.splits > 1) p.partial_bytes = (size_t)p.splits * slice_bytes;
        return p;
    }
    // Rows of C not 16-byte aligned (N % 8) or K not a whole number of chunks.  Large
    // products are worth two extra passes over the operands: copy A and B zero-padded to a
    // shape the pipelined kernels take and run that (same products, same result); the rest
    // goes to the guarded kernel, which sustains about 80 TFLOP/s.
    const size_t Np = padded_n(N), Kp = padded_k(K);
    if (K >= 192 && padded_bytes(M, N, K) <= limits.operand_bytes) {
        const Plan inner = plan_for(M, Np, Kp, limits);
        const double inner_us = inner.est_us > 0.0 ? inner.est_us : 8.0 + (double)(Np * Kp * 2) / 4e6;
        const double copy_us = 6.0 + 4.0 * (double)((M + Np) * Kp + (Np != N ? M * Np : 0)) / 3.5e6;
        const double guarded_us = 5.0 + 2.0 * (double)M * (double)N * (double)K / 80e6;
        if (inner.kernel != KERNEL_RAGGED && inner.kernel != KERNEL_PADDED && copy_us + inner_us < guarded_us) {
            p.kernel = KERNEL_PADDED;
            p.splits = inner.splits;
            p.est_us = copy_us + inner_us;
            p.partial_bytes = inner.partial_bytes;
            p.operand_bytes = padded_bytes(M, N, K);
            return p;
        }
    }
    p.kernel = KERNEL_RAGGED;
    return p;
}

// dst[r][0..cols_dst) = src[r][0..cols_src) followed by zeros, for r < rows_src; rows
// beyond rows_src are all zeros.  One thread per 8 halves of dst.
__global__ void __launch_bounds__(256)
    pad_copy_kernel(const half_t *__restrict__ src, half_t *__restrict__ dst, int rows_src, int cols_src, int rows_dst,
                    int cols_dst) {
    const size_t chunk = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int chunks_per_row = cols_dst / 8;
    const size_t row = chunk / chunks_per_row;
    if (row >= (size_t)rows_dst) return;
    const int col = (int)(chunk % chunks_per_row) * 8;
    half8 v;
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = (half_t)0.0f;
    if (row < (size_t)rows_src && col < cols_src) {
        const half_t *s = src + row * cols_src + col;
        if ((cols_src & 7) == 0) {
            v = *reinterpret_cast<const half8 *>(s);
        } else {
#pragma unroll
            for (int e = 0; e < 8; ++e)
                if (col + e < cols_src) v[e] = s[e];
        }
    }
    *reinterpret_cast<half8 *>(dst + row * cols_dst + col) = v;
}
// dst[r][c] = src[r][c] for c < cols_dst <= cols_src (drops the padding columns of C).
__global__ void __launch_bounds__(256)
    unpad_copy_kernel(const half_t *__restrict__ src, half_t *__restrict__ dst, int rows, int cols_src, int cols_dst) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= (size_t)rows * cols_dst) return;
    const size_t r = i / cols_dst, c = i % cols_dst;
    dst[i] = src[r * cols_src + c];
}

void run_padded(const Plan &p, const Workspace &ws, const void *A, const void *B, void *C, size_t M, size_t N,
                size_t K) {
    const size_t Np = padded_n(N), Kp = padded_k(K);
    HGEMM_CHECK(ws.operands != nullptr && ws.operand_bytes >= padded_bytes(M, N, K));
    half_t *Ap = reinterpret_cast<half_t *>(ws.operands), *Bp = Ap + M * Kp;
    half_t *Cp = Np != N ? Bp + Np * Kp : reinterpret_cast<half_t *>(C);
    pad_copy_kernel<<<dim3((unsigned)div_ceil(M * (Kp / 8), (size_t)256)), dim3(256), 0, nullptr>>>(
        reinterpret_cast<const half_t *>(A), Ap, (int)M, (int)K, (int)M, (int)Kp);
    pad_copy_kernel<<<dim3((unsigned)div_ceil(Np * (Kp / 8), (size_t)256)), dim3(256), 0, nullptr>>>(
        reinterpret_cast<const half_t *>(B), Bp, (int)N, (int)K, (int)Np, (int)Kp);
    HGEMM_CHECK_HIP_ERROR(hipGetLastError());
    // The inner plan that plan_for sized p for: the best plan within a limit is still the best
    // within the smaller limit of what it needs itself.
    PlanLimits inner_limits;
    inner_limits.partial_bytes = p.partial_bytes;
    inner_limits.operand_bytes = 0;
    const Plan inner = plan_for(M, Np, Kp, inner_limits);
    HGEMM_CHECK(inner.kernel != KERNEL_PADDED && inner.kernel != KERNEL_RAGGED && inner.partial_bytes == p.partial_bytes);
    run_plan(inner, ws, Ap, Bp, Cp, M, Np, Kp);
    if (Np != N) {
        unpad_copy_kernel<<<dim3((unsigned)div_ceil(M * N, (size_t)256)), dim3(256), 0, nullptr>>>(
            Cp, reinterpret_cast<half_t *>(C), (int)M, (int)Np, (int)N);
        HGEMM_CHECK_HIP_ERROR(hipGetLastError());
    }
}

void run_plan(const Plan &p, const Workspace &ws, const void *A, const void *B, void *C, size_t M, size_t N,
              size_t K) {
    switch (p.kernel) {
        case KERNEL_BIG256: launch_pipelined_plan<Big256>(A, B, C, M, N, K, p, ws); break;
        case KERNEL_T192: launch_pipelined_plan<Tile192>(A, B, C, M, N, K, p, ws); break;
        case KERNEL_R256x128: launch_pipelined_plan<Rect256x128>(A, B, C, M, N, K, p, ws); break;
        case KERNEL_MID128: launch_pipelined_plan<Mid128>(A, B, C, M, N, K, p, ws); break;
        case KERNEL_MID128_S2: launch_pipelined<Mid128S2>(A, B, C, M, N, K, "hgemm_auto"); break;
        case KERNEL_ROW64x128: launch_pipelined_plan<Row64x128>(A, B, C, M, N, K, p, ws); break;
        case KERNEL_ROW192x128: launch_pipelined_plan<Row192x128>(A, B, C, M, N, K, p, ws); break;
        case KERNEL_SMALL64: launch_pipelined_plan<Small64>(A, B, C, M, N, K, p, ws); break;
        case KERNEL_SMALL64_W4: {
            const size_t chunks = K / 64 / (size_t)(p.splits > 1 ? p.splits : 1);
            if (p.splits <= 1) {
                if (chunks <= W4_SHORT_MAX_CHUNKS)
                    launch_tiled<Small64W4Short>(A, B, C, M, N, K, "hgemm_auto");
                else if ((M / 64) * (N / 64) > (size_t)compute_units())
                    launch_tiled<Small64W4Pair>(A, B, C, M, N, K, "hgemm_auto");
                else if (chunks < W4_DEEP_MIN_CHUNKS)
                    launch_tiled<Small64W4>(A, B, C, M, N, K, "hgemm_auto");
                else
                    launch_tiled<Small64W4Deep>(A, B, C, M, N, K, "hgemm_auto");
            } else {
                check_operands(A, B, C, M, N, K);
                HGEMM_CHECK(ws.partial != nullptr && ws.partial_bytes >= (size_t)p.splits * M * N * sizeof(float));
                if (chunks <= W4_SHORT_MAX_CHUNKS)
                    launch_tiled_split<Small64W4Short>(A, B, ws.partial, M, N, K, p.splits, "hgemm_auto");
                else if (chunks < W4_DEEP_MIN_CHUNKS)
                    launch_tiled_split<Small64W4>(A, B, ws.partial, M, N, K, p.splits, "hgemm_auto");
                else
                    launch_tiled_split<Small64W4Deep>(A, B, ws.partial, M, N, K, p.splits, "hgemm_auto");
                launch_splitk_reduce(ws.partial, reinterpret_cast<half_t *>(C), M * N, p.splits);
            }
            break;
        }
        case KERNEL_SPLIT_32x64: launch_splitk<Split32x64>(A, B, C, M, N, K, p.splits, ws); break;
        case KERNEL_SPLIT_64x64: launch_splitk<Split64x64>(A, B, C, M, N, K, p.splits, ws); break;
        case KERNEL_SPLIT_64x128: launch_splitk<Split64x128>(A, B, C, M, N, K, p.splits, ws); break;
        case KERNEL_SPLIT_128x64: launch_splitk<Split128x64>(A, B, C, M, N, K, p.splits, ws); break;
        case KERNEL_SPLIT_128x128: launch_splitk<Split128x128>(A, B, C, M, N, K, p.splits, ws); break;
        case KERNEL_DECODE_BN16: launch_decode(A, B, C, M, N, K, 16, p.splits); break;
        case KERNEL_DECODE_BN32: launch_decode(A, B, C, M, N, K, 32, p.splits); break;
        case KERNEL_DECODE_RING: launch_decode_ring(A, B, C, M, N, K, p.splits); break;
        case KERNEL_DECODE_RESIDENT: launch_decode_resident(A, B, C, M, N, K, compute_units()); break;
        case KERNEL_RAGGED: launch_ragged(A, B, C, M, N, K); break;
        case KERNEL_PADDED: run_padded(p, ws, A, B, C, M, N, K); break;
        case KERNEL_SIMT:
            hgemm_simt_naive(reinterpret_cast<const hgemm_half *>(A), reinterpret_cast<const hgemm_half *>(B),
                             reinterpret_cast<hgemm_half *>(C), M, N, K);
            break;
        default: HGEMM_CHECK_MSG(false, "no kernel for M=%zu N=%zu K=%zu", M, N, K);
    }
}

}  // namespace hgemm

using namespace hgemm;

namespace {

// Plans of the shapes this thread saw last: a 5 us launch should not re-run the cost model
// (five tiles x K slices x tails, in doubles) on every call.  Direct-mapped, fixed size,
// per thread: no allocation, no lock.  Two tables: the best plan, and the best plan that
// needs no workspace (what runs when device memory for the workspace cannot be had).
struct CachedPlan {
    size_t M = 0, N = 0, K = 0;
    Plan plan;
};
constexpr int PLAN_CACHE_SLOTS = 64;

// Plans that hgemm_auto_tune measured to be the fastest for a shape: process-wide, consulted before the model.  The
// per-thread tables below are thrown away whenever this one changes (`g_tuned_version`).
struct TunedShape {
    size_t M, N, K;
    bool operator<(const TunedShape &o) const { return M != o.M ? M < o.M : N != o.N ? N < o.N : K < o.K; }
};
std::map<TunedShape, Plan> g_tuned;
std::mutex g_tuned_mutex;
std::atomic<unsigned> g_tuned_version{0};

bool tuned_plan(size_t M, size_t N, size_t K, Plan *out) {
    if (g_tuned_version.load(std::memory_order_acquire) == 0) return false;  // nothing was ever tuned: no lock
    std::lock_guard<std::mutex> lock(g_tuned_mutex);
    const auto it = g_tuned.find(TunedShape{M, N, K});
    if (it == g_tuned.end()) return false;
    *out = it->second;
    return true;
}

// the plan hgemm_auto runs and the hgemm_auto_plan* queries report: the tuned one if there is one, else the model's
Plan current_plan(size_t M, size_t N, size_t K) {
    Plan p;
    return tuned_plan(M, N, K, &p) ? p : plan_for(M, N, K);
}

const Plan &cached_plan(size_t M, size_t N, size_t K, bool without_workspace = false) {
    static thread_local CachedPlan cache[2][PLAN_CACHE_SLOTS];
    static thread_local unsigned seen_version = 0;
    const unsigned version = g_tuned_version.load(std::memory_order_acquire);
    if (version != seen_version) {
        for (auto &table : cache)
            for (CachedPlan &slot : table) slot = CachedPlan();
        seen_version = version;
    }
    const size_t h = (M * 0x9e3779b97f4a7c15ull) ^ (N * 0xc2b2ae3d27d4eb4full) ^ (K * 0x165667b19e3779f9ull);
    CachedPlan &slot = cache[without_workspace ? 1 : 0][(h >> 32) % PLAN_CACHE_SLOTS];
    if (slot.M != M || slot.N != N || slot.K != K) {
        PlanLimits limits;
        if (without_workspace) limits.partial_bytes = limits.operand_bytes = 0;
        if (without_workspace || !tuned_plan(M, N, K, &slot.plan)) slot.plan = plan_for(M, N, K, limits);
        slot.M = M, slot.N = N, slot.K = K;
    }
    return slot.plan;
}

// Runs the cached plan of the shape on the heap workspace; when the workspace does not hold
// what the plan needs and device memory for it cannot be had, the best plan that needs none
// (no K slices, the guarded kernel instead of padded copies).
void run_with_heap_workspace(const void *A, const void *B, void *C, size_t M, size_t N, size_t K) {
    const Plan &p = cached_plan(M, N, K);
    if (p.partial_bytes == 0 && p.operand_bytes == 0) {
        run_plan(p, Workspace(), A, B, C, M, N, K);
        return;
    }
    {
        std::lock_guard<std::mutex> lock(g_heap_mutex);  // held while the plan's launches are enqueued
        Workspace ws;
        if (heap_workspace(p.partial_bytes, p.operand_bytes, &ws, false)) {
            run_plan(p, ws, A, B, C, M, N, K);
            return;
        }
    }
    run_plan(cached_plan(M, N, K, true), Workspace(), A, B, C, M, N, K);
}

}  // namespace

extern "C" void hgemm_skinny(const hgemm_half *A, const hgemm_half *B, hgemm_half *C, size_t M, size_t N, size_t K) {
    check_operands(A, B, C, M, N, K);
    HGEMM_CHECK_MSG(skinny_supports(M, N, K),
                    "hgemm_skinny needs M <= 128, N %% 64 == 0, K %% 64 == 0 (got M=%zu N=%zu K=%zu)", M, N, K);
    run_with_heap_workspace(A, B, C, M, N, K);
}
extern "C" int hgemm_skinny_supports(size_t M, size_t N, size_t K) { return skinny_supports(M, N, K) ? 1 : 0; }

extern "C" void hgemm_auto(const hgemm_half *A, const hgemm_half *B, hgemm_half *C, size_t M, size_t N, size_t K) {
    check_operands(A, B, C, M, N, K);
    run_with_heap_workspace(A, B, C, M, N, K);
}

// The plans hgemm_auto_tune times for a shape, best first by the model: the plan hgemm_auto runs anyway, then the
// best that is none of the earlier.
constexpr int TUNE_MOST_PLANS = 12;
int plans_to_time(size_t M, size_t N, size_t K, int max_plans, Plan *plans) {
    if (max_plans < 1) max_plans = 1;
    if (max_plans > TUNE_MOST_PLANS) max_plans = TUNE_MOST_PLANS;
    int count = 0;
    PlanLimits limits;
    limits.excluded = plans;
    while (count < max_plans) {
        limits.excluded_count = count;
        limits.every_small_m_kernel = count > 0;
        const Plan p = plan_for(M, N, K, limits);
        if (p.kernel == KERNEL_NONE) break;
        plans[count++] = p;
        if (p.kernel == KERNEL_PADDED || p.kernel == KERNEL_RAGGED || p.kernel == KERNEL_SIMT) break;  // nothing to choose from
    }
    return count;
}

// What hgemm_auto_tune would time, without launching anything: kernel ids and K slices of up to max_plans plans.
extern "C" int hgemm_auto_tune_plans(size_t M, size_t N, size_t K, int max_plans, int *kernels, int *splits) {
    Plan plans[TUNE_MOST_PLANS];
    const int count = plans_to_time(M, N, K, max_plans, plans);
    for (int i = 0; i < count; ++i) {
        if (kernels) kernels[i] = plans[i].kernel;
        if (splits) splits[i] = plans[i].splits;
    }
    return count;
}

// What the calling thread's last hgemm_auto_tune measured, plan by plan in the order they were timed.
struct TuneRecord {
    Plan plan;
    float ms;
};
thread_local TuneRecord t_tune_records[TUNE_MOST_PLANS];
thread_local int t_tune_record_count = 0, t_tune_kept = -1;

// Reads a buffer larger than the caches hold, so that what was cached before is not afterwards.  Reads, not writes:
// the caches are left full of clean lines, as they are in a caller's loop over read-only weights; after a flush that
// writes, the next kernel's loads must first push out dirty lines, which penalises kernels by how they load (the
// streaming decode kernel read 30 us after a writing flush where it takes 13.5 us between other GEMMs).
// `never` is a value no sum of the zero-filled buffer takes, so nothing is stored.
__global__ void __launch_bounds__(256) cache_flush_kernel(floatx4 *buffer, size_t count, float never) {
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    floatx4 sum = floatx4{0.0f, 0.0f, 0.0f, 0.0f};
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < count; i += stride) sum += buffer[i];
    if (sum[0] + sum[1] + sum[2] + sum[3] == never) buffer[0] = sum;
}

// Times the model's best plans for this shape on the caller's operands and keeps the fastest for every later
// hgemm_auto call of the shape in this process: the first plan is the one hgemm_auto would run anyway, each next
// one the best that is none of the earlier (another tile, another slice count, for M <= 128 another kernel).  Per
// plan three untimed launches, then 5 ... 40 timed ones (about half a millisecond of work) enqueued back to back, each
// between events of its own on the null stream; with HGEMM_TUNE_COLD 512 MiB are read through the device before
// each of them, so that A and B come from HBM as they do for a caller whose weights do not stay cached between
// calls.  About 30 ms of untimed work come first, so that every plan meets a settled clock.  Another plan replaces
// the model's only if it is more than 3 % faster than the better of two timings of the model's.  The call returns when the device is
// idle and C holds the product as the kept plan computes it.
extern "C" int hgemm_auto_tune(const hgemm_half *A, const hgemm_half *B, hgemm_half *C, size_t M, size_t N, size_t K,
                               int max_plans, int flags) {
    check_operands(A, B, C, M, N, K);
    Plan plans[TUNE_MOST_PLANS];
    const int count = plans_to_time(M, N, K, max_plans, plans);
    constexpr size_t FLUSH_BYTES = (size_t)512 << 20;
    floatx4 *flush = nullptr;
    if ((flags & HGEMM_TUNE_COLD) && hipMalloc(reinterpret_cast<void **>(&flush), FLUSH_BYTES) != hipSuccess) {
        (void)hipGetLastError();
        flush = nullptr;  // no memory for it: the plans are timed on whatever the caches hold
    }
    if (flush) HGEMM_CHECK_HIP_ERROR(hipMemsetAsync(flush, 0, FLUSH_BYTES, nullptr));
    constexpr int MOST_LAUNCHES = 40;
    hipEvent_t start[MOST_LAUNCHES], stop[MOST_LAUNCHES];
    for (int i = 0; i < MOST_LAUNCHES; ++i) {
        HGEMM_CHECK_HIP_ERROR(hipEventCreate(&start[i]));
        HGEMM_CHECK_HIP_ERROR(hipEventCreate(&stop[i]));
    }
    auto run = [&](const Plan &p) {  // false: the workspace the plan needs could not be had
        std::lock_guard<std::mutex> lock(g_heap_mutex);
        Workspace ws;
        if ((p.partial_bytes || p.operand_bytes) && !heap_workspace(p.partial_bytes, p.operand_bytes, &ws, false)) return false;
        run_plan(p, ws, A, B, C, M, N, K);
        return true;
    };
    // `launches` launches enqueued back to back (with the flush between them when asked for), each between two events
    // of its own: the device stays busy as in a caller's loop, and the flushes are not in the sum.  Milliseconds per launch.
    auto time_plan = [&](const Plan &p, int launches) {
        for (int i = 0; i < launches; ++i) {
            if (flush) {
                cache_flush_kernel<<<dim3(2048), dim3(256), 0, nullptr>>>(flush, FLUSH_BYTES / sizeof(floatx4), 1.0f);
                HGEMM_CHECK_HIP_ERROR(hipGetLastError());
            }
            HGEMM_CHECK_HIP_ERROR(hipEventRecord(start[i], nullptr));
            run(p);
            HGEMM_CHECK_HIP_ERROR(hipEventRecord(stop[i], nullptr));
        }
        HGEMM_CHECK_HIP_ERROR(hipEventSynchronize(stop[launches - 1]));
        float total = 0.0f;
        for (int i = 0; i < launches; ++i) {
            float ms = 0.0f;
            HGEMM_CHECK_HIP_ERROR(hipEventElapsedTime(&ms, start[i], stop[i]));
            total += ms;
        }
        return total / (float)launches;
    };
    int best = -1, timed = 0;
    float best_ms = 0.0f, first_ms = 0.0f;
    t_tune_record_count = 0;
    // The part is power-managed and takes tens of milliseconds of work to settle from idle: whoever is timed first is
    // timed on a different clock (the model's own plan measured 13-23 % slower than the same kernel a moment later).
    // So the device is kept busy with the first plan for about 30 ms before anything is timed, and that plan is timed
    // once more after all the others; the better of its two timings counts.
    if (count > 0 && run(plans[0])) {
        float spent_ms = 0.0f;
        for (int round = 0; round < 20 && spent_ms < 30.0f; ++round) spent_ms += 5.0f * time_plan(plans[0], 5);
    }
    for (int i = 0; i < count; ++i) {
        if (!run(plans[i])) continue;
        // two untimed launches that also say how many timed ones make about half a millisecond of work (5 ... 40)
        const float rough_ms = time_plan(plans[i], 2);
        int launches = rough_ms > 0.0f ? (int)(0.5f / rough_ms) : MOST_LAUNCHES;
        launches = launches < 5 ? 5 : launches > MOST_LAUNCHES ? MOST_LAUNCHES : launches;
        const float ms = time_plan(plans[i], launches);
        ++timed;
        t_tune_records[t_tune_record_count++] = TuneRecord{plans[i], ms};
        if (i == 0) first_ms = ms;
        // the model's own plan stays unless another is ahead by more than the 3 % that two timings of one plan differ by
        if (best < 0 || ms < (best == 0 ? 0.97f * first_ms : best_ms)) best = i, best_ms = ms, t_tune_kept = t_tune_record_count - 1;
    }
    if (best > 0 && t_tune_record_count > 0 && same_choice(t_tune_records[0].plan, plans[0])) {
        const float rough_ms = time_plan(plans[0], 2);
        int launches = rough_ms > 0.0f ? (int)(0.5f / rough_ms) : MOST_LAUNCHES;
        launches = launches < 5 ? 5 : launches > MOST_LAUNCHES ? MOST_LAUNCHES : launches;
        const float again_ms = time_plan(plans[0], launches);
        if (again_ms < t_tune_records[0].ms) t_tune_records[0].ms = again_ms;
        if (best_ms >= 0.97f * t_tune_records[0].ms) best = 0, best_ms = t_tune_records[0].ms, t_tune_kept = 0;
    }
    for (int i = 0; i < MOST_LAUNCHES; ++i) {
        HGEMM_CHECK_HIP_ERROR(hipEventDestroy(start[i]));
        HGEMM_CHECK_HIP_ERROR(hipEventDestroy(stop[i]));
    }
    HGEMM_CHECK_MSG(best >= 0, "hgemm_auto_tune: no plan for M=%zu N=%zu K=%zu could be run", M, N, K);
    {
        std::lock_guard<std::mutex> lock(g_tuned_mutex);
        g_tuned[TunedShape{M, N, K}] = plans[best];
        g_tuned_version.fetch_add(1, std::memory_order_release);
    }
    run(plans[best]);
    HGEMM_CHECK_HIP_ERROR(hipDeviceSynchronize());
    if (flush) HGEMM_CHECK_HIP_ERROR(hipFree(flush));
    return timed;
}

// The calling thread's last hgemm_auto_tune, plan by plan in the order they were timed: kernel id, K slices,
// milliseconds per launch, whether it is the one that was kept.  Returns 0 past the last plan, else 1.
extern "C" int hgemm_auto_tune_result(int index, int *kernel, int *splits, float *ms, int *kept) {
    if (index < 0 || index >= t_tune_record_count) return 0;
    if (kernel) *kernel = t_tune_records[index].plan.kernel;
    if (splits) *splits = t_tune_records[index].plan.splits;
    if (ms) *ms = t_tune_records[index].ms;
    if (kept) *kept = index == t_tune_kept ? 1 : 0;
    return 1;
}

// Forgets every tuned plan: hgemm_auto goes by the model again.
extern "C" void hgemm_auto_forget_tuning(void) {
    std::lock_guard<std::mutex> lock(g_tuned_mutex);
    g_tuned.clear();
    g_tuned_version.fetch_add(1, std::memory_order_release);
}

// 1 if the shape's plan was set by hgemm_auto_tune.
extern "C" int hgemm_auto_plan_is_tuned(size_t M, size_t N, size_t K) {
    Plan p;
    return tuned_plan(M, N, K, &p) ? 1 : 0;
}

// The tuned kernel by tile, as entry points of their own.  M and N may end inside a tile.
#define HGEMM_DEFINE_PIPELINED_VARIANT(symbol, Cfg, which)                                                   \
    extern "C" void symbol(const hgemm_half *A, const hgemm_half *B, hgemm_half *C, size_t M, size_t N,      \
                           size_t K) {                                                                       \
        launch_pipelined<Cfg>(A, B, C, M, N, K, #symbol, which);                                             \
    }                                                                                                        \
    extern "C" int symbol##_supports(size_t M, size_t N, size_t K) {                                         \
        return pipelined_supports_edges<Cfg>(M, N, K) ? 1 : 0;                                               \
    }
HGEMM_DEFINE_PIPELINED_VARIANT(hgemm_mfma_pipelined_64x64, Small64, PipeKernel::Interleaved)
HGEMM_DEFINE_PIPELINED_VARIANT(hgemm_mfma_pipelined_128x128, Mid128, PipeKernel::Interleaved)
HGEMM_DEFINE_PIPELINED_VARIANT(hgemm_mfma_pipelined_192x192, Tile192, PipeKernel::Interleaved)
HGEMM_DEFINE_PIPELINED_VARIANT(hgemm_mfma_pipelined_256x128, Rect256x128, PipeKernel::Interleaved)
HGEMM_DEFINE_PIPELINED_VARIANT(hgemm_mfma_pipelined_256x256, Big256, PipeKernel::Interleaved)
// ... and with each accumulator's MFMAs chained (the tiles that have that kernel)
HGEMM_DEFINE_PIPELINED_VARIANT(hgemm_mfma_chained_192x192, Tile192, PipeKernel::Chained)
HGEMM_DEFINE_PIPELINED_VARIANT(hgemm_mfma_chained_256x128, Rect256x128, PipeKernel::Chained)
HGEMM_DEFINE_PIPELINED_VARIANT(hgemm_mfma_chained_256x256, Big256, PipeKernel::Chained)

extern "C" int hgemm_reserve_workspace(size_t partial_bytes, size_t operand_bytes) {
    std::lock_guard<std::mutex> lock(g_heap_mutex);
    Workspace ws;
    return heap_workspace(partial_bytes, operand_bytes, &ws, true) ? 0 : 1;
}

extern "C" void hgemm_release_workspace(void) {
    const int dev = current_device();
    std::lock_guard<std::mutex> lock(g_heap_mutex);
    Workspace &w = g_heap[dev].ws;
    if (w.partial || w.operands) HGEMM_CHECK_HIP_ERROR(hipDeviceSynchronize());  // launches may still use them
    if (w.partial) HGEMM_CHECK_HIP_ERROR(hipFree(w.partial));
    if (w.operands) HGEMM_CHECK_HIP_ERROR(hipFree(w.operands));
    g_heap[dev] = HeapState();
}

extern "C" int hgemm_auto_static_workspace(const hgemm_half *A, const hgemm_half *B, hgemm_half *C, size_t M, size_t N,
                                           size_t K) {
    check_operands(A, B, C, M, N, K);
    const Plan &p = cached_plan(M, N, K);  // the plan hgemm_auto runs: same kernels, same order of additions
    const size_t partial_bytes = (p.partial_bytes + 255) / 256 * 256;
    if (partial_bytes + p.operand_bytes > STATIC_WORKSPACE_BYTES) {
        HLOG("hgemm_auto_static_workspace: the plan for M=%zu N=%zu K=%zu keeps %zu bytes of partial sums and %zu bytes "
             "of padded operands, the static workspace holds %zu; nothing was launched (hgemm_auto has no such limit)",
             M, N, K, p.partial_bytes, p.operand_bytes, STATIC_WORKSPACE_BYTES);
        return 1;
    }
    Workspace ws;
    if (partial_bytes + p.operand_bytes > 0) {
        unsigned char *base = static_scratch();
        ws.partial = reinterpret_cast<float *>(base);
        ws.partial_bytes = partial_bytes;
        ws.operands = base + partial_bytes;
        ws.operand_bytes = STATIC_WORKSPACE_BYTES - partial_bytes;
    }
    // Nothing in the array has to start at zero: every kernel that reads partial sums or padded
    // operands reads only what a kernel launched before it in this call has written in full.
    if (partial_bytes + p.operand_bytes > 0) {
        std::lock_guard<std::mutex> lock(g_scratch_mutex);  // one plan's launches at a time into the null stream
        run_plan(p, ws, A, B, C, M, N, K);
    } else {
        run_plan(p, ws, A, B, C, M, N, K);
    }
    return 0;
}

extern "C" size_t hgemm_static_workspace_bytes(void) { return STATIC_WORKSPACE_BYTES; }

extern "C" size_t hgemm_auto_workspace_bytes(size_t M, size_t N, size_t K, size_t *operand_bytes) {
    const Plan p = current_plan(M, N, K);
    if (operand_bytes) *operand_bytes = p.operand_bytes;
    return p.partial_bytes;
}
extern "C" int hgemm_auto_supports(size_t M, size_t N, size_t K) { return M > 0 && N > 0 && K > 0; }

// Which kernel and how many K slices hgemm_auto uses for a shape (for reports and tests).
extern "C" int hgemm_auto_plan(size_t M, size_t N, size_t K, int *splits) {
    const Plan p = current_plan(M, N, K);
    if (splits) *splits = p.splits;
    return p.kernel;
}
// How hgemm_auto treats the last, partly filled round of a large grid: the number of
// workgroups in it that run in K slices (0: none) and, through `splits`, the slice count.
extern "C" int hgemm_auto_plan_tail(size_t M, size_t N, size_t K, int *splits) {
    const Plan p = current_plan(M, N, K);
    if (splits) *splits = p.tail_splits;
    return p.tail_tiles;
}
// Row `index` of the table that decides the kernel for M <= 128 (first covering row whose kernel can run the shape
// wins): bounds = {m_lo, m_hi, n_lo, n_hi, k_lo, k_hi, b_lo, b_hi}, inclusive, b = N * K; flags bit 0: only where
// K < 4 N, bit 1: not where K is a multiple of 16384.  Returns the kernel id, or -1 past the end of the table.
extern "C" int hgemm_small_m_rule(int index, size_t *bounds, int *flags) {
    if (index < 0 || index >= SMALL_M_RULE_COUNT) return -1;
    const SmallMRule &r = SMALL_M_RULES[index];
    if (bounds) {
        const size_t b[8] = {(size_t)r.m_lo, (size_t)r.m_hi, r.n_lo, r.n_hi, r.k_lo, r.k_hi, r.b_lo, r.b_hi};
        for (int i = 0; i < 8; ++i) bounds[i] = b[i];
    }
    if (flags) *flags = r.flags;
    return r.kernel;
}
// Kernel id of the smaller tile that takes over the last round (0: none).
extern "C" int hgemm_auto_plan_tail_kernel(size_t M, size_t N, size_t K) { return current_plan(M, N, K).tail_kernel; }
// 1 if the plan's main launch runs the chained kernel of its tile, 0 for the interleaved one.
extern "C" int hgemm_auto_plan_chained(size_t M, size_t N, size_t K) {
    const Plan p = current_plan(M, N, K);
    if (p.splits < 1) return 0;
    const size_t k_len = shortest_slice(K, 64, p.splits);
    auto workgroups = [&](size_t bm, size_t bn) {  // of the main launch
        return (div_ceil(M, bm) * div_ceil(N, bn) - (size_t)p.tail_tiles) * (size_t)p.splits;
    };
    switch (p.kernel) {
        case KERNEL_BIG256: return use_chained<Big256>(PipeKernel::Auto, workgroups(256, 256), k_len) ? 1 : 0;
        case KERNEL_T192: return use_chained<Tile192>(PipeKernel::Auto, workgroups(192, 192), k_len) ? 1 : 0;
        case KERNEL_R256x128: return use_chained<Rect256x128>(PipeKernel::Auto, workgroups(256, 128), k_len) ? 1 : 0;
        default: return 0;
    }
}
extern "C" const char *hgemm_kernel_name(int kernel) {
    switch (kernel) {
        case KERNEL_BIG256: return "pipelined 256x256x64, 4 waves, LDS ring 3 (A) + 2 (B)";
        case KERNEL_MID128: return "pipelined 128x128x64, 4 waves, 5-stage ring";
        case KERNEL_MID128_S2: return "pipelined 128x128x64, 4 waves, 2-stage ring";
        case KERNEL_ROW64x128: return "pipelined 64x128x64, 4 waves, 5-stage ring";
        case KERNEL_ROW192x128: return "pipelined 192x128x64, 4 waves, 4-stage ring";
        case KERNEL_SMALL64: return "pipelined 64x64x64, 1 wave, 3-stage ring";
        case KERNEL_SMALL64_W4: return "tiled 64x64x64, 4 waves of 32x32, look-ahead ring";
        case KERNEL_T192: return "pipelined 192x192x64, 4 waves, 3-stage ring";
        case KERNEL_R256x128: return "pipelined 256x128x64, 4 waves, 3-stage ring";
        case KERNEL_SPLIT_32x64: return "split-K 32x64x64, 2 waves, 4-stage ring";
        case KERNEL_SPLIT_64x64: return "split-K 64x64x64, 4 waves, 4-stage ring";
        case KERNEL_SPLIT_64x128: return "split-K 64x128x64, 4 waves, 4-stage ring";
        case KERNEL_SPLIT_128x64: return "split-K 128x64x64, 4 waves, 4-stage ring";
        case KERNEL_SPLIT_128x128: return "split-K 128x128x64, 4 waves, 4-stage ring";
        case KERNEL_DECODE_BN16: return "streaming decode, 16 columns per workgroup, one wave per K slice";
        case KERNEL_DECODE_BN32: return "streaming decode, 32 columns per workgroup, one wave per K slice";
        case KERNEL_DECODE_RING: return "streaming decode, 16 columns per workgroup, one wave and one LDS ring per K slice";
        case KERNEL_DECODE_RESIDENT: return "decode with A in registers, persistent workgroups over 16-column tiles, one wave per K slice";
        case KERNEL_RAGGED: return "guarded 128x128x32, 4 waves, any shape";
        case KERNEL_PADDED: return "zero-padded operand copies + pipelined kernel of the padded shape";
        case KERNEL_SIMT: return "scalar fallback";
        default: return "none";
    }
}
