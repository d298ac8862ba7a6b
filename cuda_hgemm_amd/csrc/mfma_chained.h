// The chained variant of the pipelined kernel (included by mfma_pipelined.h, which defines
// the tile configuration and the assembly helpers it uses): same tiles, LDS rings and
// layouts, different order of work inside a K chunk.
//
//  * Every accumulator tile receives the chunk's two MFMAs back to back, a dependent chain.
//    The matrix pipe then keeps the running sum to itself instead of reading and writing the
//    accumulator registers for every instruction; under the board's power limit that is worth
//    6 % in an MFMA-only loop and 3-4 % in the whole kernel at 8192^3.
//  * Tiles are visited column by column, so the A fragments of the whole chunk stay in
//    registers for the iteration (the next chunk's are collected meanwhile) and B needs only
//    the current column's and the next column's fragments.
//  * The accumulators live in named AGPRs that the compiler never sees.
// It pays for the larger tiles when K is long (the prologue fetches one more chunk of A and
// passes one more barrier than the interleaved kernel's); the launcher chooses.
#pragma once

namespace hgemm {

// The accumulators of the chained kernel are not C++ objects.  Tile r of a wave's output
// (a 16x16 MFMA tile, four registers) lives in AGPRs a[4r : 4r+3] by name, touched only by
// the statements below.  With accumulators as variables, every place where two loop bodies
// meet let the register allocator permute or spill them, with copies that read registers
// an MFMA issued from assembly was still writing (the compiler does not know the latency
// of instructions inside an asm statement).  Named registers leave it nothing to move.  The
// statement that zeroes a tile lists its registers as clobbered, which makes the kernel
// reserve them; the MFMA statements do not (the compiler would put a wait state between two
// statements that clobber the same registers).  The rest of the kernel stays below 256 VGPRs
// (the build checks that nothing is spilled), so the compiler never looks for a free AGPR of
// its own.
// An assembler template has to be a literal, hence one specialisation per tile.
#define HGEMM_FOR_EACH_ACC_TILE(X) \
    X(0, 0, 1, 2, 3) X(1, 4, 5, 6, 7) X(2, 8, 9, 10, 11) X(3, 12, 13, 14, 15) X(4, 16, 17, 18, 19) X(5, 20, 21, 22, 23) X(6, 24, 25, 26, 27) X(7, 28, 29, 30, 31) X(8, 32, 33, 34, 35) X(9, 36, 37, 38, 39) X(10, 40, 41, 42, 43) X(11, 44, 45, 46, 47) X(12, 48, 49, 50, 51) X(13, 52, 53, 54, 55) X(14, 56, 57, 58, 59) X(15, 60, 61, 62, 63) X(16, 64, 65, 66, 67) X(17, 68, 69, 70, 71) X(18, 72, 73, 74, 75) X(19, 76, 77, 78, 79) X(20, 80, 81, 82, 83) X(21, 84, 85, 86, 87) X(22, 88, 89, 90, 91) X(23, 92, 93, 94, 95) X(24, 96, 97, 98, 99) X(25, 100, 101, 102, 103) X(26, 104, 105, 106, 107) X(27, 108, 109, 110, 111) X(28, 112, 113, 114, 115) X(29, 116, 117, 118, 119) X(30, 120, 121, 122, 123) X(31, 124, 125, 126, 127) X(32, 128, 129, 130, 131) X(33, 132, 133, 134, 135) X(34, 136, 137, 138, 139) X(35, 140, 141, 142, 143) X(36, 144, 145, 146, 147) X(37, 148, 149, 150, 151) X(38, 152, 153, 154, 155) X(39, 156, 157, 158, 159) X(40, 160, 161, 162, 163) X(41, 164, 165, 166, 167) X(42, 168, 169, 170, 171) X(43, 172, 173, 174, 175) X(44, 176, 177, 178, 179) X(45, 180, 181, 182, 183) X(46, 184, 185, 186, 187) X(47, 188, 189, 190, 191) X(48, 192, 193, 194, 195) X(49, 196, 197, 198, 199) X(50, 200, 201, 202, 203) X(51, 204, 205, 206, 207) X(52, 208, 209, 210, 211) X(53, 212, 213, 214, 215) X(54, 216, 217, 218, 219) X(55, 220, 221, 222, 223) X(56, 224, 225, 226, 227) X(57, 228, 229, 230, 231) X(58, 232, 233, 234, 235) X(59, 236, 237, 238, 239) X(60, 240, 241, 242, 243) X(61, 244, 245, 246, 247) X(62, 248, 249, 250, 251) X(63, 252, 253, 254, 255)

template <int R>
struct AccTile;
#define X(R, A0, A1, A2, A3)                                                                                      \
    template <>                                                                                                   \
    struct AccTile<R> {                                                                                           \
        static __device__ __forceinline__ void zero() {                                                           \
            asm volatile("v_accvgpr_write_b32 a" #A0 ", 0\n\tv_accvgpr_write_b32 a" #A1 ", 0\n\t"                   \
                         "v_accvgpr_write_b32 a" #A2 ", 0\n\tv_accvgpr_write_b32 a" #A3 ", 0" ::                    \
                             : "a" #A0, "a" #A1, "a" #A2, "a" #A3);                                               \
        }                                                                                                         \
        /* tile += a x b (16x16x32); a is the first source operand */                                             \
        static __device__ __forceinline__ void mfma(half8 a, half8 b) {                                           \
            asm volatile("v_mfma_f32_16x16x32_f16 a[" #A0 ":" #A3 "], %0, %1, a[" #A0 ":" #A3 "]" ::"v"(a), "v"(b)); \
        }                                                                                                         \
        /* The same MFMA slot, also starting a direct-to-LDS copy: M0 (the LDS destination) is set before the */ \
        /* MFMA, which doubles as the wait state the hardware wants between a write of M0 and the copy that */   \
        /* reads it, so the slot costs three instructions. */                                                     \
        template <int LDS_IMM>                                                                                    \
        static __device__ __forceinline__ void mfma_and_dma(half8 a, half8 b, const void *sbase, uint32_t voff,   \
                                                            uint32_t lds_base) {                                  \
            asm volatile("s_add_u32 m0, %2, %5\n\t"                                                                \
                         "v_mfma_f32_16x16x32_f16 a[" #A0 ":" #A3 "], %0, %1, a[" #A0 ":" #A3 "]\n\t"              \
                         "global_load_lds_dwordx4 %3, %4" ::"v"(a),                                                \
                         "v"(b), "s"(lds_base), "v"(voff), "s"(sbase), "i"(LDS_IMM)                               \
                         : "memory", "scc");                                                                      \
        }                                                                                                         \
        /* after the last MFMA and enough wait states (the kernel issues s_nop for them) */                       \
        static __device__ __forceinline__ floatx4 read() {                                                        \
            floatx4 v;                                                                                            \
            asm volatile("v_accvgpr_read_b32 %0, a" #A0 "\n\tv_accvgpr_read_b32 %1, a" #A1 "\n\t"                   \
                         "v_accvgpr_read_b32 %2, a" #A2 "\n\tv_accvgpr_read_b32 %3, a" #A3                          \
                         : "=v"(v[0]), "=v"(v[1]), "=v"(v[2]), "=v"(v[3]));                                       \
            return v;                                                                                             \
        }                                                                                                         \
    };
HGEMM_FOR_EACH_ACC_TILE(X)
#undef X


// Accumulators -> fp16 -> C through LDS (operands swapped in the MFMA, so a lane holds four
// consecutive n of one row m = lane % 16 of each tile): each wave parks 16 rows of its tile
// in a private strip and reads them back row-contiguous, 16 bytes per lane, so a global
// store instruction writes whole 128-byte lines.  Tile (i, j) of the wave is AccTile<j * TM + i>.
// EDGE: rows >= M and 8-column pieces at or beyond N (N % 8 == 0) are not stored.
template <class Cfg, bool EDGE = false>
__device__ __forceinline__ void store_chained_tile(unsigned char *lds, half_t *__restrict__ C, int M, int N, int row0,
                                                int col0, int wave, int lane) {
    constexpr int MI = Cfg::MI, TM = Cfg::PTM, TN = Cfg::PTN, WN = Cfg::WN;
    constexpr int STRIP_ROW_BYTES = WN * 2 + 16;
    constexpr int STRIP_BYTES = 32 * STRIP_ROW_BYTES;  // sized for 32 rows
    constexpr int LANES_PER_ROW = WN / 8;
    constexpr int ROWS_PER_READ = 64 / LANES_PER_ROW;                   // lanes beyond that many rows idle
    constexpr int READS = (MI + ROWS_PER_READ - 1) / ROWS_PER_READ;
    constexpr bool EXACT = (64 % LANES_PER_ROW == 0) && (MI % ROWS_PER_READ == 0);
    static_assert(STRIP_BYTES == Cfg::C_STRIP_BYTES, "strip size");
    unsigned char *strip = lds + wave * STRIP_BYTES;
    unsigned char *wr = strip + (lane % MI) * STRIP_ROW_BYTES + ((lane / MI) << 3);
    const int rd_row = lane / LANES_PER_ROW, rd_col = lane % LANES_PER_ROW;
    const unsigned char *rd = strip + rd_row * STRIP_ROW_BYTES + rd_col * 16;
    half_t *cp = C + (size_t)(row0 + rd_row) * N + col0 + rd_col * 8;
    static_for<TM>([&](auto i_c) {
        constexpr int i = decltype(i_c)::value;
        static_for<TN>([&](auto j_c) {
            constexpr int j = decltype(j_c)::value;
            const floatx4 acc = AccTile<j * TM + i>::read();
            half4 v;
#pragma unroll
            for (int r = 0; r < 4; ++r) v[r] = (half_t)acc[r];
            *reinterpret_cast<half4 *>(wr + (j * MI) * 2) = v;
        });
        wave_lds_exchange_point();
#pragma unroll
        for (int it = 0; it < READS; ++it) {
            if (EXACT || (rd_row < ROWS_PER_READ && it * ROWS_PER_READ + rd_row < MI)) {
                const u32x4 v = *reinterpret_cast<const u32x4 *>(rd + it * ROWS_PER_READ * STRIP_ROW_BYTES);
                if (!EDGE || (row0 + rd_row + i * MI + it * ROWS_PER_READ < M && col0 + rd_col * 8 < N))
                    store_streaming(reinterpret_cast<u32x4 *>(cp + (size_t)(i * MI + it * ROWS_PER_READ) * N), v);
            }
        }
        wave_lds_exchange_point();
    });
}

// Tile, K slice, copy offsets and operand addresses come from PipeFrame (mfma_pipelined.h), as in the interleaved
// kernel; EDGE as there.
template <class Cfg, bool SPLIT = false, bool EDGE = false>
__global__ void __launch_bounds__(Cfg::THREADS)
    hgemm_chained_kernel(const half_t *__restrict__ A, const half_t *__restrict__ B, half_t *__restrict__ C,
                           float *__restrict__ partial, int M, int N, int K, int slices, int tiles_m, int tiles_n,
                           int first_block, int tail_tiles, int subdiv) {
    constexpr int BM = Cfg::BM, BN = Cfg::BN, BK = Cfg::BK, MI = Cfg::MI;
    constexpr int TM = Cfg::PTM, TN = Cfg::PTN, KSTEPS = Cfg::PKSTEPS;
    constexpr int SA = Cfg::SA, SB = Cfg::SB;
    constexpr int A_BYTES = Cfg::A_BYTES, B_BYTES = Cfg::B_BYTES, B_REGION = SA * A_BYTES;
    constexpr int A_DMA = Cfg::A_DMA, B_DMA = Cfg::B_DMA, L = A_DMA + B_DMA;
    constexpr int NFRAG = TM + TN, NMMA = TM * TN;
    static_assert(NFRAG <= NMMA, "at most one operand read is issued per MFMA slot");
    static_assert(MI == 16 && TM * TN <= 64, "the schedule and the named accumulator registers are laid out for 16x16x32 tiles");

    extern __shared__ __attribute__((aligned(1024))) unsigned char lds[];
    const uint32_t lds_base = (uint32_t)(uintptr_t)lds;
    PipeFrame<Cfg, SPLIT, EDGE> frame;
    if (!frame.init(A, B, M, N, K, slices, tiles_m, tiles_n, first_block, subdiv, lds_base)) return;
    const int lane = frame.lane, wave = frame.wave, wm = frame.wm, wn = frame.wn;
    int tile_m = frame.tile_m, tile_n = frame.tile_n;
    const int slot = frame.slot, slice = frame.slice, num_k = frame.num_k;
    const unsigned char *const a_base = frame.a_base, *const b_base = frame.b_base;
    const uint32_t(&voff)[L] = frame.voff;
    const uint32_t cp_lds = frame.cp_lds;

    // Operand registers.  Every accumulator receives the chunk's KSTEPS MFMAs back to back
    // (a dependent chain: the matrix pipe then keeps the running sum to itself instead of
    // reading and writing the accumulator registers for every instruction, which is worth
    // about 6 % of throughput under the board's power limit), accumulators are visited
    // column by column (j outer, i inner).  So the A fragments of the whole chunk stay in
    // registers for the whole iteration and the next chunk's are collected meanwhile
    // (double buffer), while B needs only the current column's fragments and the next
    // column's.
    half8 a_frag[2][KSTEPS][TM];
    half8 b_frag[2][KSTEPS];
    static_assert(TN % 2 == 0, "columns alternate between two B fragment buffers");
    auto read_a = [&](auto t_c, uint32_t stage_bytes, auto kk_c) -> half8 { return frame.read_a(t_c, stage_bytes, kk_c); };
    auto read_b = [&](auto t_c, uint32_t stage_bytes, auto kk_c) -> half8 { return frame.read_b(t_c, stage_bytes, kk_c); };

    // ---- pipeline.  Chunk c of A lives in A-ring buffer c % SA, of B in B-ring buffer c % SB.
    //
    // One iteration = one K chunk = NM MFMA "slots" (one MFMA issue each), TN blocks of
    // BS = TM * KSTEPS slots, block j = column j of the wave tile.  During iteration kt a wave
    //   * multiplies chunk kt (A fragments already in registers, B column by column),
    //   * reads chunk kt+1's A fragments from LDS (blocks 0 .. TN-2) and, in block j, column
    //     j+1's B fragments of chunk kt; in the last block column 0 of chunk kt+1,
    //   * passes the one barrier of the iteration in front of its last block.  By then every
    //     wave has read all of A(kt+1) and B(kt) out of LDS, so the barrier releases those two
    //     buffers, and it confirms that A(kt+2) and B(kt+1) have landed.
    // Copies are organised in windows: window kt runs from barrier kt to barrier kt+1 (the
    // last block of iteration kt and blocks 0 .. TN-2 of iteration kt+1) and refills the two
    // released buffers with B(kt+SB), then A(kt+1+SA), one instruction per NM / L slots.
    // A is one chunk further ahead than B because its buffer is released a whole chunk before
    // its successor is read.  Past the end of K the copies fetch the last chunk again, into
    // buffers nobody reads any more: every iteration issues the same instructions, so the
    // wait counts below hold throughout.
    constexpr int NM = KSTEPS * NMMA, BS = TM * KSTEPS, SBAR = NM - BS;
    // slot, relative to its window's barrier, of copy instruction d (B first, then A)
    auto copy_rel_slot = [](int d) constexpr -> int { return d * NM / L + 1; };
    static_assert((L - 1) * NM / L + 1 < NM && NM / L >= 1, "one copy per slot at most");
    // copy instruction of the window issued at relative slot `rel`, or -1
    auto copy_at = [copy_rel_slot](int rel) constexpr -> int {
        for (int d = 0; d < L; ++d)
            if (copy_rel_slot(d) == rel) return d;
        return -1;
    };
    // Copies that may still be in flight at barrier kt, when A up to chunk kt+2 and B up to
    // chunk kt+1 must have landed: walking back from the most recent, window kt-w copied
    // A(kt-w+1+SA) last and B(kt-w+SB) before it.
    auto steady_vmcnt = []() constexpr -> int {
        int n = 0;
        for (int w = 1;; ++w) {
            if (SA > w + 1) n += A_DMA; else break;
            if (SB > w + 1) n += B_DMA; else break;
        }
        return n;
    };
    constexpr int STEADY_VMCNT = steady_vmcnt();
    static_assert(STEADY_VMCNT <= 63, "vmcnt is a 6-bit counter");
    static_assert(SA >= 3 && SB >= 2 && SA >= SB, "ring depths the schedule is written for");
    // Operand reads of block j: first the KSTEPS B fragments of the next column, then this
    // block's share of the next chunk's A fragments (blocks 0 .. TN-2 share KSTEPS * TM reads,
    // the earlier blocks taking the extra ones).  Reads prefer slots 2, 6, 10, ... of the
    // block, then 0, 4, 8, ..., then odd ones (copies sit in odd slots, and two LDS reads in
    // adjacent slots stall MFMA issue).
    // Block TN-2 ends at the barrier and waits for every read of the wave (the barrier hands the
    // buffers just read to the copies), so wide wave tiles keep the A reads out of it.
    constexpr int A_READS = KSTEPS * TM, A_BLOCKS = TN >= 6 ? TN - 2 : TN - 1;
    auto a_reads_in_block = [](int j) constexpr -> int {
        if (j >= A_BLOCKS) return 0;
        return A_READS / A_BLOCKS + (j < A_READS % A_BLOCKS ? 1 : 0);
    };
    auto a_reads_before_block = [a_reads_in_block](int j) constexpr -> int {
        int n = 0;
        for (int b = 0; b < j; ++b) n += a_reads_in_block(b);
        return n;
    };
    // the k-th (ascending) of the m read slots of a block
    auto read_slot = [](int m, int k) constexpr -> int {
        bool used[64] = {};  // BS <= 64
        int taken = 0;
        for (int pass = 0; pass < 3 && taken < m; ++pass)
            for (int sl = 0; sl < BS && taken < m; ++sl) {
                const bool want = pass == 0 ? (sl % 4 == 2) : (pass == 1 ? (sl % 4 == 0) : (sl % 2 == 1));
                if (want && !used[sl]) {
                    used[sl] = true;
                    ++taken;
                }
            }
        int seen = 0;
        for (int sl = 0; sl < BS; ++sl)
            if (used[sl] && seen++ == k) return sl;
        return -1;
    };
    // which read (0 .. m-1) of its block is issued in block slot `sl`, or -1
    auto read_at = [read_slot](int m, int sl) constexpr -> int {
        for (int k = 0; k < m; ++k)
            if (read_slot(m, k) == sl) return k;
        return -1;
    };
    static_assert(BS <= 64, "read_slot's table");
    static_assert(BS >= KSTEPS + (A_READS + A_BLOCKS - 1) / A_BLOCKS, "a block has a slot for each of its operand reads");

    // copy instruction d of a window: source chunk pointers and destination buffers
    auto issue_copy_with_mfma = [&](auto d_c, auto r_c, half8 bf, half8 af, const unsigned char *a_src,
                                    const unsigned char *b_src, uint32_t dst_a, uint32_t dst_b) {
        constexpr int d = decltype(d_c)::value;
        using Tile = AccTile<decltype(r_c)::value>;
        if constexpr (d < B_DMA)
            Tile::template mfma_and_dma<d * Cfg::WAVES * 1024>(bf, af, b_src, voff[A_DMA + d], dst_b);
        else
            Tile::template mfma_and_dma<(d - B_DMA) * Cfg::WAVES * 1024>(bf, af, a_src, voff[d - B_DMA], dst_a);
    };
    auto issue_copy = [&](auto d_c, const unsigned char *a_src, const unsigned char *b_src, uint32_t dst_a,
                          uint32_t dst_b) {
        constexpr int d = decltype(d_c)::value;
        if constexpr (d < B_DMA)
            dma_load16_sv<d * Cfg::WAVES * 1024>(b_src, voff[A_DMA + d], dst_b);
        else
            dma_load16_sv<(d - B_DMA) * Cfg::WAVES * 1024>(a_src, voff[d - B_DMA], dst_a);
    };
    const int last_chunk = num_k - 1;
    auto a_chunk = [&](int c) { return a_base + (c < last_chunk ? c : last_chunk) * (BK * 2); };
    auto b_chunk = [&](int c) { return b_base + (c < last_chunk ? c : last_chunk) * (BK * 2); };

    // ---- prologue: A(0 .. SA-1) and B(0 .. SB-2) in that interleaved order; B(SB-1) and A(SA)
    // belong to the window before iteration 0.
    static_for<SA>([&](auto st_c) {
        constexpr int st = decltype(st_c)::value;
        static_for<A_DMA>([&](auto d_c) {
            issue_copy(std::integral_constant<int, B_DMA + decltype(d_c)::value>{}, a_chunk(st), nullptr,
                       cp_lds + st * A_BYTES, 0u);
        });
        if constexpr (st < SB - 1)
            static_for<B_DMA>([&](auto d_c) { issue_copy(d_c, nullptr, b_chunk(st), 0u, cp_lds + B_REGION + st * B_BYTES); });
    });
    constexpr int PROLOGUE_COPIES = SA * A_DMA + (SB - 1) * B_DMA;
    // the accumulators, while the first copies are under way; tile (i, j) is AccTile<j * TM + i>
    static_for<TM * TN>([&](auto r_c) { AccTile<decltype(r_c)::value>::zero(); });
    wait_vmcnt<PROLOGUE_COPIES - A_DMA - B_DMA>();  // A(0) and B(0) have landed
    __syncthreads();
    using K0 = std::integral_constant<int, 0>;
    static_for<KSTEPS>([&](auto kk_c) {
        constexpr int kk = decltype(kk_c)::value;
        static_for<TM>([&](auto t) { a_frag[0][kk][decltype(t)::value] = read_a(t, 0u, kk_c); });
        b_frag[0][kk] = read_b(K0{}, 0u, kk_c);
    });
    lds_wait_all();
    static_for<KSTEPS>([&](auto kk_c) {
        constexpr int kk = decltype(kk_c)::value;
        static_for<TM>([&](auto t) { lds_landed(a_frag[0][kk][decltype(t)::value]); });
        lds_landed(b_frag[0][kk]);
    });
    // A(1) has landed too (iteration 0 starts reading it at once) and every wave is done with
    // A(0): the barrier "before iteration 0" that opens window -1
    wait_vmcnt<PROLOGUE_COPIES - 2 * A_DMA - (SB > 2 ? 2 : 1) * B_DMA>();
    __syncthreads();
    static_for<L>([&](auto d_c) {
        if constexpr (copy_rel_slot(decltype(d_c)::value) < NM - SBAR)
            issue_copy(d_c, a_chunk(SA), b_chunk(SB - 1), cp_lds, cp_lds + B_REGION + (SB - 1) * B_BYTES);
    });

    // Sources of the copies, kept as byte offsets of K chunks so that "the last chunk again" is
    // one s_min: A(kt+SA) / B(kt-1+SB) finish window kt-1, A(kt+1+SA) / B(kt+SB) start window kt.
    const uint32_t last_off = (uint32_t)last_chunk * (BK * 2);
    auto clamped = [&](int c) { return (uint32_t)(c < last_chunk ? c : last_chunk) * (uint32_t)(BK * 2); };
    uint32_t a_off_far = clamped(SA), b_off_far = clamped(SB - 1);  // furthest chunk with a pointer so far
    const unsigned char *a_pre = a_base + a_off_far, *b_pre = b_base + b_off_far, *a_post = a_pre, *b_post = b_pre;

    // One iteration (chunk kt in ring buffers CUR_A / CUR_B, its A fragments in half AB of
    // a_frag).  Every iteration but the last is the same code.
    auto iteration = [&](auto cur_a_arg, auto cur_b_arg, auto ab_c, auto final_tag) {
        constexpr bool FINAL = decltype(final_tag)::value;  // the last chunk: nothing to fetch, nobody to wait for
        // ring buffers of chunk kt: plain ints or, in the unrolled loop, compile-time constants --
        // then every LDS address below is a constant offset
        const int CUR_A = ring_index(cur_a_arg), CUR_B = ring_index(cur_b_arg);
        constexpr int AB = decltype(ab_c)::value, NB = AB ^ 1;
        const int NXT_A = (CUR_A + 1) % SA, NXT_B = (CUR_B + 1) % SB, PRV_B = (CUR_B + SB - 1) % SB;
        const uint32_t pre_dst_a = cp_lds + CUR_A * A_BYTES, pre_dst_b = cp_lds + B_REGION + PRV_B * B_BYTES;
        const uint32_t post_dst_a = cp_lds + NXT_A * A_BYTES, post_dst_b = cp_lds + B_REGION + CUR_B * B_BYTES;
        const uint32_t src_a_next = NXT_A * A_BYTES, src_b_cur = CUR_B * B_BYTES, src_b_next = NXT_B * B_BYTES;
        static_for<TN>([&](auto j_c) {
            constexpr int j = decltype(j_c)::value;
            constexpr bool last = (j + 1 == TN);
            if constexpr (last && !FINAL) {
                wait_vmcnt<STEADY_VMCNT>();
                __builtin_amdgcn_s_barrier();
            }
            __builtin_amdgcn_sched_barrier(0);
            // operand reads of this block: B fragments of the next column (of the next chunk's
            // column 0 in the last block), then A fragments of the next chunk
            constexpr int n_b = !(FINAL && last) ? KSTEPS : 0;
            constexpr int n_a = !FINAL ? a_reads_in_block(j) : 0;
            constexpr int a_first = a_reads_before_block(j);
            static_for<BS>([&](auto sl_c) {
                constexpr int sl = decltype(sl_c)::value, slot = j * BS + sl;
                constexpr int i = sl / KSTEPS, kk = sl % KSTEPS;
                constexpr int rel = slot >= SBAR ? slot - SBAR : slot + NM - SBAR;
                constexpr int copy = !FINAL ? copy_at(rel) : -1;
                using Tile = std::integral_constant<int, j * TM + i>;
                if constexpr (copy >= 0) {
                    if constexpr (slot >= SBAR)
                        issue_copy_with_mfma(std::integral_constant<int, copy>{}, Tile{}, b_frag[j & 1][kk],
                                             a_frag[AB][kk][i], a_post, b_post, post_dst_a, post_dst_b);
                    else
                        issue_copy_with_mfma(std::integral_constant<int, copy>{}, Tile{}, b_frag[j & 1][kk],
                                             a_frag[AB][kk][i], a_pre, b_pre, pre_dst_a, pre_dst_b);
                } else {
                    AccTile<Tile::value>::mfma(b_frag[j & 1][kk], a_frag[AB][kk][i]);
                }
                constexpr int rd = (n_a + n_b) > 0 ? read_at(n_a + n_b, sl) : -1;
                if constexpr (rd >= 0 && rd < n_b) {
                    using KK = std::integral_constant<int, rd>;
                    if constexpr (last)
                        b_frag[(j + 1) & 1][rd] = read_b(K0{}, src_b_next, KK{});
                    else
                        b_frag[(j + 1) & 1][rd] = read_b(std::integral_constant<int, j + 1>{}, src_b_cur, KK{});
                } else if constexpr (rd >= n_b) {
                    constexpr int q = a_first + (rd - n_b);  // q-th A fragment of the next chunk
                    a_frag[NB][q / TM][q % TM] =
                        read_a(std::integral_constant<int, q % TM>{}, src_a_next, std::integral_constant<int, q / TM>{});
                }
                // The sources of the next window, a few scalar instructions at a time in slots that
                // host nothing else (block 1: no copy of this window's start is issued before the barrier).
                if constexpr (!FINAL && j == 1 && sl == 3) {
                    a_off_far = a_off_far + BK * 2 < last_off ? a_off_far + BK * 2 : last_off;
                    a_post = a_base + a_off_far;
                }
                if constexpr (!FINAL && j == 1 && sl == 5) {
                    b_off_far = b_off_far + BK * 2 < last_off ? b_off_far + BK * 2 : last_off;
                    b_post = b_base + b_off_far;
                }
                __builtin_amdgcn_sched_barrier(0);
            });
            // The next column's B fragments have landed before control leaves the block; the
            // A fragments read after them may still be in flight (LDS reads return in order) and
            // are not touched before the block in front of the barrier, where everything has landed.
            if constexpr (n_b > 0) {
                if constexpr (last || j == TN - 2 || n_a == 0) {
                    lds_wait_all();
                } else {
                    static_assert(n_a <= 15, "lgkmcnt is a 4-bit counter");
                    __builtin_amdgcn_s_waitcnt((0x3f & 0xf) | ((0x3f >> 4) << 14) | (0x7 << 4) | (n_a << 8));
                }
                static_for<KSTEPS>([&](auto kk_c) { lds_landed(b_frag[(j + 1) & 1][decltype(kk_c)::value]); });
            }
            if constexpr (j == TN - 2 && !FINAL) {
                static_for<KSTEPS>([&](auto kk_c) {
                    static_for<TM>([&](auto t) { lds_landed(a_frag[NB][decltype(kk_c)::value][decltype(t)::value]); });
                });
            }
        });
        a_pre = a_post;  // what started as this window's start is the next iteration's "rest of the previous window"
        b_pre = b_post;
    };

    // The loop, unrolled over one period of the two rings and of the A fragment double buffer
    // so that every buffer index is a constant: no index arithmetic or address computation is
    // left inside it.
    constexpr int PERIOD0 = SA * SB / gcd_of(SA, SB);
    constexpr int PERIOD = PERIOD0 % 2 == 0 ? PERIOD0 : 2 * PERIOD0;
    using T = std::true_type;
    using F = std::false_type;
    int kt = 0;
    for (; kt + PERIOD <= last_chunk; kt += PERIOD)
        static_for<PERIOD>([&](auto u_c) {
            constexpr int u = decltype(u_c)::value;
            iteration(std::integral_constant<int, u % SA>{}, std::integral_constant<int, u % SB>{},
                      std::integral_constant<int, u % 2>{}, F{});
        });
    // The chunks left over (at most a period): one body with run-time ring indices, which hands
    // the fragments it collected back to the half of a_frag it started from, so that it can
    // follow itself; then the last chunk.
    int cur_a = 0, cur_b = 0;  // kt is a multiple of the period here
    for (; kt < last_chunk; ++kt) {
        iteration(cur_a, cur_b, std::integral_constant<int, 0>{}, F{});
        static_for<KSTEPS>([&](auto kk_c) {
            static_for<TM>([&](auto t) {
                a_frag[0][decltype(kk_c)::value][decltype(t)::value] = a_frag[1][decltype(kk_c)::value][decltype(t)::value];
            });
        });
        cur_a = (cur_a + 1 == SA) ? 0 : cur_a + 1;
        cur_b = (cur_b + 1 == SB) ? 0 : cur_b + 1;
    }
    iteration(cur_a, cur_b, std::integral_constant<int, 0>{}, T{});

    // The last MFMAs are still writing their accumulators: wait states before the reads below
    // (ordered statements, like the MFMAs themselves).
    asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
    // The epilogue's per-lane addresses depend only on kernel arguments, so the optimiser would
    // compute them ahead of the loop and carry some tens of registers through it, which the
    // loop does not have.  Passing their inputs through an (empty) ordered statement here keeps
    // that arithmetic behind the loop.
    asm volatile("" : "+s"(M), "+s"(N), "+s"(tile_m), "+s"(tile_n), "+s"(C), "+s"(partial));
    int lane_late = lane;
    asm volatile("" : "+v"(lane_late));
    // ---- epilogue: accumulators -> fp16 -> C (through LDS, whole lines per store)
    wait_vmcnt<0>();  // the redundant copies of the last iterations: landed before LDS is reused or the wave ends
    if constexpr (SPLIT) {
        __syncthreads();  // every wave has read its last operands: the strips reuse the ring
        auto get = [&](auto i_c, auto j_c) -> floatx4 { return AccTile<decltype(j_c)::value * TM + decltype(i_c)::value>::read(); };
        const int row0 = tile_m * BM + wm * Cfg::WM, col0 = tile_n * BN + wn * Cfg::WN;
        if (tail_tiles > 0)  // compact: whole tiles [slice][slot][BM][BN], nothing to guard
            store_wave_tile_f32<Cfg, false>(get, lds, partial + ((size_t)slice * tail_tiles + slot) * (BM * BN) +
                                                          (size_t)(wm * Cfg::WM) * BN + wn * Cfg::WN,
                                            BN, BM, BN, wave, lane_late);
        else
            store_wave_tile_f32<Cfg, EDGE>(get, lds, partial + ((size_t)slice * M + row0) * N + col0, N, M - row0,
                                           N - col0, wave, lane_late);
    } else {
        (void)partial;
        __syncthreads();
        store_chained_tile<Cfg, EDGE>(lds, C, M, N, tile_m * BM + wm * Cfg::WM, tile_n * BN + wn * Cfg::WN, wave, lane_late);
    }
}

}  // namespace hgemm
