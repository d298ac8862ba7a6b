// Which tile of C a workgroup computes.  Plain integer functions, usable on the host too
// (without a HIP compiler the qualifiers vanish), so that the orders can be checked
// exhaustively on a CPU.
//
// The chip is 8 XCDs of 32 CUs, each XCD with its own 4 MB L2, all behind one memory-side
// cache (256 MB) in front of HBM.  Workgroup b of a launch runs on XCD b % 8, and an XCD
// starts its workgroups in order of b; with one 256x256 workgroup per CU the chip works
// through "rounds" of 256 workgroups, 32 per XCD.  In both orders below the 32 workgroups
// that share an L2 form a block of 4 x 8 tiles (12 operand panels for 32 tiles).  They
// differ in what the eight XCDs hold between them, i.e. in what reaches HBM:
//   * strips: every XCD walks its own contiguous part of 8-column strips down M.  The
//     XCDs sit in different strips at the same rows: a round touches few A panels and up
//     to 64 B panels.  HBM sees A once and B once as long as B stays in the memory-side
//     cache.  (Counterpart of the reference's 16-tile strips, src/mma/mma_base.cu:51-53.)
//   * blocks: the 8 blocks of a round form one block of 16 x 16 tiles (32 panels for the
//     whole chip), and consecutive rounds walk along M inside a band of 16 columns, so a
//     band's 16 B panels stay cached while A streams past.  For a B too large for the
//     cache this halves what HBM delivers: measured 3-6 % faster from 9216^3 to 16384^3
//     and on 8192 x 28672 x 8192 (the chip is power-limited and HBM traffic costs clock),
//     1-2 % slower than strips when B is at most 128 MiB, equal when A and B both fit.
// Edge blocks are clipped; every order is a bijection for any grid and any launch size.
#pragma once

#ifdef __HIPCC__
#define HGEMM_HOST_DEVICE __host__ __device__ __forceinline__
#else
#define HGEMM_HOST_DEVICE inline
#endif

namespace hgemm {

constexpr int STRIP_TILES_N = 8;
constexpr int XCD_ROUND = 32, CHIP_ROUND = 8 * XCD_ROUND;
constexpr int CHIP_BLOCK = 16, XCD_BLOCK_M = 4, XCD_BLOCK_N = 8;
static_assert(CHIP_BLOCK * CHIP_BLOCK == CHIP_ROUND && XCD_BLOCK_M * XCD_BLOCK_N == XCD_ROUND, "blocks are rounds");
// B (N rows of K halves) above this many elements takes the blocked order: 144 MiB, between
// the largest B measured faster in strips (128 MiB) and the smallest faster in blocks (162 MiB)
constexpr long long BLOCKED_ORDER_MIN_B_ELEMS = 72ll << 20;

HGEMM_HOST_DEVICE bool blocked_order(long long N, long long K) { return N * K > BLOCKED_ORDER_MIN_B_ELEMS; }

// Workgroup b of `count` -> position in [0, count), a bijection: XCD x (= b % 8) walks a
// contiguous range of positions (the first count % 8 XCDs one more than the rest).
HGEMM_HOST_DEVICE int xcd_contiguous(int b, int count) {
    const int x = b & 7, q = count >> 3, r = count & 7;
    return x * q + (x < r ? x : r) + (b >> 3);
}

// Workgroup b of `count` -> position in [0, count), a bijection: whole rounds of 256
// positions, inside a round XCD x takes positions [32 x, 32 x + 32); what is left over after
// the whole rounds is dealt contiguously per XCD.
HGEMM_HOST_DEVICE int xcd_rounds(int b, int count) {
    const int whole = count & ~(CHIP_ROUND - 1);
    if (b >= whole) return whole + xcd_contiguous(b - whole, count - whole);
    const int local = b >> 3;  // index among the XCD's own workgroups
    return (local / XCD_ROUND) * CHIP_ROUND + (b & 7) * XCD_ROUND + local % XCD_ROUND;
}

// Strips: position -> tile, 8-column strips walked down M, row-major inside a strip.
HGEMM_HOST_DEVICE void tile_in_strips(int pos, int tiles_m, int tiles_n, int &tile_m, int &tile_n) {
    const int strip_tiles = STRIP_TILES_N * tiles_m;
    const int strip = pos / strip_tiles;
    const int within = pos - strip * strip_tiles;
    const int n_first = strip * STRIP_TILES_N;
    const int width = (tiles_n - n_first) < STRIP_TILES_N ? (tiles_n - n_first) : STRIP_TILES_N;
    tile_m = within / width;
    tile_n = n_first + within % width;
}

// Blocks: position -> tile.  Bands of 16 columns; in a band, blocks of 16 rows walked down M
// (up in odd bands, so the turn keeps its A panels); in a block, sub-blocks of 4 rows x 8
// columns, the two column halves one after the other; in a sub-block down the rows first.
// Full blocks divide by constants (shifts); only clipped ones pay for real divisions.
HGEMM_HOST_DEVICE void tile_in_blocks(int pos, int tiles_m, int tiles_n, int &tile_m, int &tile_n) {
    const int band = pos / (CHIP_BLOCK * tiles_m);  // every band before the last is full
    int rem = pos - band * (CHIP_BLOCK * tiles_m);
    const int left_n = tiles_n - band * CHIP_BLOCK, wb = left_n < CHIP_BLOCK ? left_n : CHIP_BLOCK;
    const int blk = wb == CHIP_BLOCK ? rem / (CHIP_BLOCK * CHIP_BLOCK) : rem / (wb * CHIP_BLOCK);
    rem -= blk * (wb * CHIP_BLOCK);  // every block of the band before its last is full
    const int left_m = tiles_m - blk * CHIP_BLOCK, hb = left_m < CHIP_BLOCK ? left_m : CHIP_BLOCK;
    const int half = hb == CHIP_BLOCK ? rem / (XCD_BLOCK_N * CHIP_BLOCK) : rem / (XCD_BLOCK_N * hb);
    rem -= half * (XCD_BLOCK_N * hb);
    const int left_w = wb - half * XCD_BLOCK_N, ws = left_w < XCD_BLOCK_N ? left_w : XCD_BLOCK_N;
    const int sub = ws == XCD_BLOCK_N ? rem / (XCD_BLOCK_N * XCD_BLOCK_M) : rem / (ws * XCD_BLOCK_M);
    rem -= sub * (ws * XCD_BLOCK_M);
    const int left_h = hb - sub * XCD_BLOCK_M, hs = left_h < XCD_BLOCK_M ? left_h : XCD_BLOCK_M;
    const int col = hs == XCD_BLOCK_M ? rem / XCD_BLOCK_M : rem / hs;
    const int m = blk * CHIP_BLOCK + sub * XCD_BLOCK_M + (rem - col * hs);
    tile_m = (band & 1) ? tiles_m - 1 - m : m;
    tile_n = band * CHIP_BLOCK + half * XCD_BLOCK_N + col;
}

// Position -> tile in the order chosen for the problem.
HGEMM_HOST_DEVICE void tile_of_position(bool blocked, int pos, int tiles_m, int tiles_n, int &tile_m, int &tile_n) {
    if (blocked)
        tile_in_blocks(pos, tiles_m, tiles_n, tile_m, tile_n);
    else
        tile_in_strips(pos, tiles_m, tiles_n, tile_m, tile_n);
}

// Workgroup b of a launch of `count` workgroups -> its slot in [0, count), dealt as the order wants.
HGEMM_HOST_DEVICE int slot_of_workgroup(bool blocked, int b, int count) {
    return blocked ? xcd_rounds(b, count) : xcd_contiguous(b, count);
}

// Workgroup b of a launch of `count` workgroups that covers positions [first, first + count).
HGEMM_HOST_DEVICE void tile_of_workgroup(bool blocked, int first, int b, int count, int tiles_m, int tiles_n,
                                         int &tile_m, int &tile_n) {
    tile_of_position(blocked, first + slot_of_workgroup(blocked, b, count), tiles_m, tiles_n, tile_m, tile_n);
}

// K-sliced launches are one-dimensional too: `count` positions times `slices`, slice-major, dealt in contiguous
// shares like a strip launch.  An XCD then works on whole slices, or on a run of neighbouring tiles of one slice,
// and the panels it streams are shared by the workgroups it runs together; with the slice as the launch's second
// dimension an XCD would get every slice of a few tiles, whose K ranges share nothing.
HGEMM_HOST_DEVICE void slice_and_slot_of_workgroup(int b, int count, int slices, int &slice, int &slot) {
    const int p = xcd_contiguous(b, count * slices);
    slice = p / count;
    slot = p - slice * count;
}

}  // namespace hgemm
