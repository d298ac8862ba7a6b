"""The workgroup -> tile orders of the tuned kernels (cuda_hgemm_amd/csrc/tile_order.h), checked on the CPU.

The header is plain integer code that g++ compiles as host code.  Every order must be a bijection (a tile nobody
computes, or one computed twice, is a wrong C), for any grid and any launch size, and must keep the locality it is
there for: the 32 workgroups an XCD runs together form a block of few operand panels, and in the blocked order the
256 workgroups of a round form one 16 x 16 block.  (The reference's counterpart is the strip order of
src/mma/mma_base.cu:51-53.)
"""
import os
import subprocess
import textwrap

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "cuda_hgemm_amd", "csrc", "tile_order.h")

PROGRAM = textwrap.dedent(
    r"""
    #include "%s"
    #include <cstdio>
    #include <set>
    #include <vector>
    using namespace hgemm;
    int main() {
        // workgroup -> position, both dealings, every launch size up to 3000
        for (int count = 1; count <= 3000; ++count)
            for (int which = 0; which < 2; ++which) {
                std::vector<int> seen(count, 0);
                for (int b = 0; b < count; ++b) {
                    const int p = which ? xcd_rounds(b, count) : xcd_contiguous(b, count);
                    if (p < 0 || p >= count || seen[p]++) return printf("position: count %%d workgroup %%d\n", count, b), 1;
                }
            }
        // position -> tile, both orders, every grid up to 70 x 70
        for (int blocked = 0; blocked < 2; ++blocked)
            for (int tm = 1; tm <= 70; ++tm)
                for (int tn = 1; tn <= 70; ++tn) {
                    std::vector<int> seen(tm * tn, 0);
                    for (int p = 0; p < tm * tn; ++p) {
                        int m = -1, n = -1;
                        tile_of_position(blocked != 0, p, tm, tn, m, n);
                        if (m < 0 || m >= tm || n < 0 || n >= tn || seen[m * tn + n]++)
                            return printf("tile: order %%d grid %%d x %%d position %%d\n", blocked, tm, tn, p), 1;
                    }
                }
        // K-sliced launches: every (slice, slot) pair exactly once, and the 32 workgroups an XCD runs together in a
        // launch of 64 tiles x 4 slices stay inside one slice
        for (int count = 1; count <= 300; ++count)
            for (int slices = 1; slices <= 32; slices += (slices < 4 ? 1 : 7)) {
                std::vector<int> seen(count * slices, 0);
                for (int b = 0; b < count * slices; ++b) {
                    int slice = -1, slot = -1;
                    slice_and_slot_of_workgroup(b, count, slices, slice, slot);
                    if (slice < 0 || slice >= slices || slot < 0 || slot >= count || seen[slice * count + slot]++)
                        return printf("slices: count %%d slices %%d workgroup %%d\n", count, slices, b), 1;
                }
            }
        for (int x = 0; x < 8; ++x) {
            std::set<int> slices_of_xcd;
            for (int w = 0; w < 32; ++w) {
                int slice, slot;
                slice_and_slot_of_workgroup(w * 8 + x, 64, 4, slice, slot);
                slices_of_xcd.insert(slice);
            }
            if (slices_of_xcd.size() != 1) return printf("slices: XCD %%d works on %%zu slices\n", x, slices_of_xcd.size()), 1;
        }
        // a launch that covers positions [first, first + count): the tiles of head and tail launches are disjoint
        for (int blocked = 0; blocked < 2; ++blocked) {
            const int tm = 17, tn = 23, total = tm * tn, head = 256;
            std::set<int> tiles;
            for (int b = 0; b < head; ++b) {
                int m, n;
                tile_of_workgroup(blocked != 0, 0, b, head, tm, tn, m, n);
                tiles.insert(m * tn + n);
            }
            for (int b = 0; b < total - head; ++b) {
                int m, n;
                tile_of_workgroup(blocked != 0, head, b, total - head, tm, tn, m, n);
                tiles.insert(m * tn + n);
            }
            if ((int)tiles.size() != total) return printf("head + tail: order %%d covers %%zu of %%d\n", blocked, tiles.size(), total), 1;
        }
        // locality on a 64 x 64 grid (16 rounds): panels per XCD and round, panels per round of the whole chip
        for (int blocked = 0; blocked < 2; ++blocked) {
            const int tm = 64, tn = 64, total = tm * tn;
            int worst_xcd = 0, worst_chip = 0;
            for (int round = 0; round < total / 256; ++round) {
                std::set<int> chip;
                for (int x = 0; x < 8; ++x) {
                    std::set<int> panels;
                    for (int w = 0; w < 32; ++w) {
                        int m, n;
                        tile_of_workgroup(blocked != 0, 0, (round * 32 + w) * 8 + x, total, tm, tn, m, n);
                        panels.insert(m), panels.insert(1000 + n);
                        chip.insert(m), chip.insert(1000 + n);
                    }
                    if ((int)panels.size() > worst_xcd) worst_xcd = (int)panels.size();
                }
                if ((int)chip.size() > worst_chip) worst_chip = (int)chip.size();
            }
            printf("order %%d: at most %%d panels per XCD and round, %%d per round of the chip\n", blocked, worst_xcd, worst_chip);
        }
        printf("blocked %%d %%d %%d\n", (int)blocked_order(8192, 8192), (int)blocked_order(9216, 9216), (int)blocked_order(28672, 4096));
        return 0;
    }
    """
)


@pytest.fixture(scope="module")
def order_report(tmp_path_factory):
    work = tmp_path_factory.mktemp("tile_order")
    src = work / "order.cpp"
    src.write_text(PROGRAM % HEADER)
    exe = work / "order"
    subprocess.run(["g++", "-O2", "-std=c++17", "-Wall", "-Werror", "-o", str(exe), str(src)], check=True)
    done = subprocess.run([str(exe)], capture_output=True, text=True, timeout=300)
    assert done.returncode == 0, done.stdout + done.stderr
    return done.stdout


def test_orders_are_bijections(order_report):
    assert "order 0" in order_report and "order 1" in order_report


def test_orders_keep_their_locality(order_report):
    lines = {line.split(":")[0]: line for line in order_report.splitlines() if line.startswith("order")}
    # 4 x 8 tiles per XCD and round: 12 panels; strips: the XCDs share their rows, 4 A + 64 B panels per round;
    # blocks: one 16 x 16 block per round
    assert "at most 12 panels per XCD and round, 68 per round of the chip" in lines["order 0"]
    assert "at most 12 panels per XCD and round, 32 per round of the chip" in lines["order 1"]


def test_blocked_order_threshold(order_report):
    # B = N x K halves: 128 MiB stays in strips, 162 MiB and 224 MiB go to blocks
    assert "blocked 0 1 1" in order_report
