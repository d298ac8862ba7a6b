"""The C-ABI boundary without a GPU: the library loads, exports every symbol the headers
declare, its registry and shape predicates answer, and contract violations end the
process with a message (the convention of the reference's HGEMM_CHECK macros,
src/common/common.h:23-29) before any GPU call."""
import ctypes
import os
import re
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
INCLUDE = os.path.join(ROOT, "include")


def _declared_symbols(header):
    text = open(os.path.join(INCLUDE, header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    names = set(re.findall(r"^HGEMM_FUNC\((\w+)\);", text, flags=re.M))
    names |= set(re.findall(r"^(?:const\s+)?\w[\w\s\*]*?\b(hgemm_\w+)\s*\(", text, flags=re.M))
    names.discard("hgemm_fn")
    return names


def test_library_exports_every_declared_symbol(hgemm_lib):
    declared = _declared_symbols("hgemm.h")
    assert len(declared) >= 25, declared
    for name in sorted(declared):
        assert hasattr(hgemm_lib.dll, name), f"libhgemm.so does not export {name}"
    from cuda_hgemm_amd.binding import HELPER_SYMBOLS, KERNEL_SYMBOLS
    assert declared == set(KERNEL_SYMBOLS) | set(HELPER_SYMBOLS)


def test_vendor_library_exports_its_symbols(vendor_lib):
    from cuda_hgemm_amd.binding import VENDOR_SYMBOLS
    declared = _declared_symbols("hgemm_hipblaslt.h")
    assert declared == set(VENDOR_SYMBOLS) and "hgemm_hipblaslt" in declared
    for name in sorted(declared):
        assert hasattr(vendor_lib.dll, name), f"libhgemm_hipblaslt.so does not export {name}"
    # bound to a hipBLASLt that exists; a shape that has not been called has no candidates yet (no GPU call here)
    assert os.path.exists(vendor_lib.loaded_from()) and "hipblaslt" in vendor_lib.loaded_from().lower()
    assert vendor_lib.candidates(123, 456, 789)["candidates"] == 0


def test_measured_library_has_no_blas_dependency(hgemm_lib):
    out = subprocess.run(["ldd", hgemm_lib.path], capture_output=True, text=True).stdout
    assert "blas" not in out.lower(), out
    assert "libamdhip64" in out


def test_registry(hgemm_lib):
    variants = hgemm_lib.variants()
    names = [v["name"] for v in variants]
    assert names[0] == "Simt-Naive" and "Mfma-Async-Stage4" in names and names[-1] == "Auto"
    # the tuned kernel is selectable by name and closes the ladder (reference src/main.cu:123)
    assert names.index("Mfma-Pipelined-256x256") == names.index("Mfma-Async-Stage4") + 6
    assert names.index("Mfma-Chained-256x256") == names.index("Mfma-Pipelined-256x256") + 3 == len(names) - 3
    assert all(v["default_run"] for v in variants if v["name"].startswith(("Mfma-Pipelined-", "Mfma-Chained-", "Mfma-Tiled-")))
    assert len(set(names)) == len(names)
    for v in variants:
        assert hgemm_lib.find(v["name"]) == v["index"] == hgemm_lib.find(v["symbol"])
        assert hasattr(hgemm_lib.dll, v["symbol"])
    # the naive / base kernels are left out of the default run, as in the reference's main
    assert [v["name"] for v in variants if not v["default_run"]] == ["Simt-Naive", "Mfma-Naive", "Mfma-Base"]
    with pytest.raises(KeyError):
        hgemm_lib.find("no-such-variant")


def test_shape_predicates(hgemm_lib):
    s = hgemm_lib.supports
    assert s("hgemm_simt_naive", 1, 1, 1) and s("hgemm_auto", 100, 100, 100)
    assert s("hgemm_mfma_naive", 32, 64, 16) and not s("hgemm_mfma_naive", 32, 64, 8)
    # 256 x 128 x 32 tiles, as the reference's kernels (src/mma/mma_async_stage4.cu:13-14)
    for name in ("hgemm_mfma_base", "hgemm_mfma_padding", "hgemm_mfma_swizzle", "hgemm_mfma_async",
                 "hgemm_mfma_async_pg2s", "hgemm_mfma_async_pg2s_ps2r", "hgemm_mfma_async_stage3",
                 "hgemm_mfma_async_stage4"):
        assert s(name, 256, 128, 256) and s(name, 512, 2048, 1024)
        assert not s(name, 128, 128, 256) and not s(name, 256, 64, 256) and not s(name, 256, 128, 48)
    assert not s("hgemm_mfma_async_stage4", 256, 128, 64)      # K must cover the 3-chunk prologue
    assert s("hgemm_mfma_async_stage4", 256, 128, 96)
    for name, ring in (("hgemm_mfma_pipelined_256x256", 2), ("hgemm_mfma_pipelined_256x128", 3),
                       ("hgemm_mfma_pipelined_192x192", 3), ("hgemm_mfma_pipelined_128x128", 5),
                       ("hgemm_mfma_pipelined_64x64", 3), ("hgemm_mfma_chained_256x256", 2),
                       ("hgemm_mfma_chained_256x128", 3), ("hgemm_mfma_chained_192x192", 3)):
        assert s(name, 8192, 8192, 8192) and s(name, 1, 8, 64 * ring) and s(name, 1000, 4000, 1024)
        assert not s(name, 256, 256, 64 * (ring - 1)) and not s(name, 256, 100, 1024) and not s(name, 256, 256, 1000)
    # one-dimensional grids: no limit of 65535 row or column tiles
    assert s("hgemm_auto", 4300000, 64, 64) and s("hgemm_simt_naive", 1100000, 16, 16)
    assert s("hgemm_skinny", 1, 4096, 4096) and s("hgemm_skinny", 128, 28672, 4096) and s("hgemm_skinny", 8, 192, 64)
    assert not s("hgemm_skinny", 129, 4096, 4096) and not s("hgemm_skinny", 8, 100, 4096)
    assert not s("hgemm_auto", 0, 8, 8) and not s("hgemm_auto", 1 << 20, 8, 1 << 20)


def test_auto_plan_covers_every_benchmark_config(hgemm_lib):
    plan = hgemm_lib.auto_plan
    for n in (256, 512, 1024, 2048, 4096, 8192, 16384):
        p = plan(n, n, n)
        assert p["kernel"] != "scalar fallback" and p["splits"] >= 1, (n, p)
    assert plan(8192, 8192, 8192)["kernel"].startswith("pipelined 256x256") and plan(8192, 8192, 8192)["chained"]
    assert plan(4096, 4096, 2048)["chained"] and not plan(4096, 4096, 1024)["chained"]       # 256 tiles: from K = 1536
    assert not plan(2048, 2048, 4096)["chained"] and not plan(1024, 1024, 8192)["chained"]   # few tiles; small tile
    assert plan(3072, 3072, 3072)["kernel"].startswith("pipelined 192x192") and not plan(3072, 3072, 3072)["chained"]
    assert plan(3072, 3072, 4096)["kernel"].startswith("pipelined 192x192") and plan(3072, 3072, 4096)["chained"]
    for shape in ((4096, 14336, 4096), (4096, 4096, 14336)):
        assert plan(*shape)["kernel"].startswith("pipelined"), shape
    for m in (1, 8, 16, 64, 128):
        for n in (4096, 28672):
            p = plan(m, n, 4096)
            if m == 16 and n == 28672:   # A in registers, persistent workgroups, eight K slices of 512 per workgroup
                assert p["kernel"].startswith("decode with A in registers") and p["splits"] == 8, (m, n, p)
            elif m <= 16:    # the decode kernel with per-wave LDS rings (B copied non-temporally at N = 28672)
                assert "LDS ring per K slice" in p["kernel"] and p["splits"] == 4, (m, n, p)
            elif n == 28672:                                # one tile row against 224 column tiles: one launch
                assert p["kernel"].startswith("pipelined %dx128x64" % m) and p["splits"] == 1, (m, n, p)
            else:
                assert p["kernel"].startswith("split-K"), (m, n, p)
            assert 4096 % (p["splits"] * 64) == 0
    assert plan(4, 28672, 512)["kernel"].startswith("streaming decode, 16 columns per workgroup, one wave per K slice")
    assert plan(7, 57344, 1024)["kernel"].startswith("split-K 32x64")
    assert plan(100, 100, 100)["kernel"].startswith("guarded 128x128x32")      # no tile divides it
    assert plan(1000, 4000, 4096)["kernel"].startswith("pipelined")            # ragged M, N: guarded edges
    assert plan(4095, 4095, 4095)["kernel"].startswith("zero-padded")          # large and unaligned


def test_small_m_rule_table(hgemm_lib):
    """The table that decides the kernel for M <= 128 is data the library hands out: its rows are well-formed boxes,
    every M in 1 ... 128 ends in a catch-all row of the split-K family, and hgemm_auto's plan is the first covering
    row whose kernel can run the shape -- looked up here independently over a grid of shapes."""
    rules = hgemm_lib.small_m_rules()
    assert 15 <= len(rules) <= 40, len(rules)
    for r in rules:
        assert 1 <= r["m_lo"] <= r["m_hi"] <= 128 and r["n_lo"] <= r["n_hi"] and r["k_lo"] <= r["k_hi"], r
        assert r["b_lo"] <= r["b_hi"] and r["kernel"] != "none", r
    for m in range(1, 129):
        last = [r for r in rules if r["m_lo"] <= m <= r["m_hi"]][-1]
        assert last["kernel"].startswith("split-K") and last["n_lo"] <= 64 and last["k_lo"] <= 64, (m, last)
        assert last["n_hi"] > 1 << 40 and last["k_hi"] > 1 << 40 and not last["k_below_4n"], (m, last)

    def can_run(kernel, M, N, K):
        if kernel.startswith("decode with A in registers"):      # K = waves x chunks x 64, the chunks in registers
            chunk_options = (8,) if M > 16 else (8, 12, 16, 20, 24)
            return M <= 32 and N % 16 == 0 and K % 64 == 0 and any(K // 64 == w * c for w in (2, 4, 8) for c in chunk_options)
        if "LDS ring per K slice" in kernel:
            return N % 16 == 0 and K % 128 == 0
        if kernel.startswith("streaming decode"):
            return M <= 32 and N % 32 == 0 and K % 256 == 0
        if kernel.startswith(("pipelined 128x128", "pipelined 64x128")):
            return N % 8 == 0 and K % 64 == 0 and K >= 320
        if kernel.startswith("pipelined 192x192"):
            return N % 8 == 0 and K % 64 == 0 and K >= 192
        if kernel.startswith("split-K"):
            wide = kernel.split()[1].split("x")[1] == "128"       # "split-K <BM>x<BN>x64, ...": 128-column tiles
            return N % 64 == 0 and K % 64 == 0 and (N % 128 == 0 or not wide)
        raise AssertionError(kernel)

    def lookup(M, N, K):
        for r in rules:
            if not (r["m_lo"] <= M <= r["m_hi"] and r["n_lo"] <= N <= r["n_hi"] and r["k_lo"] <= K <= r["k_hi"]
                    and r["b_lo"] <= N * K <= r["b_hi"]):
                continue
            if (r["k_below_4n"] and K >= 4 * N) or (r["k_not_multiple_of_16384"] and K % 16384 == 0):
                continue
            if can_run(r["kernel"], M, N, K):
                return r["kernel"]
        return None

    family = lambda name: name.split(",")[0].replace("32 columns", "16 columns")   # the streaming kernel's two widths
    checked = 0
    for M in (1, 5, 6, 8, 9, 12, 13, 16, 17, 24, 25, 32, 33, 64, 65, 100, 128):    # both sides of every M class boundary
        for N in (16, 48, 64, 272, 2048, 3072, 4096, 4112, 8192, 8208, 14336, 16384, 18432, 20488, 28672, 40960, 57344):
            for K in (64, 256, 384, 512, 1024, 1152, 2048, 2304, 4096, 4160, 6144, 8192, 12288, 16384, 32768):
                expect = lookup(M, N, K)
                if expect is None:
                    continue
                got = hgemm_lib.auto_plan(M, N, K)["kernel"]
                assert family(got) == family(expect), (M, N, K, got, expect)
                checked += 1
    assert checked > 2000, checked
    # the headline decode shapes, by row
    assert lookup(1, 4096, 4096).endswith("one LDS ring per K slice") and lookup(128, 4096, 4096).startswith("split-K 128x64")
    assert lookup(1, 28672, 4096).endswith("one LDS ring per K slice") and lookup(128, 28672, 4096).startswith("pipelined 128x128")
    assert lookup(64, 28672, 4096).startswith("pipelined 64x128") and lookup(8, 28672, 4096).endswith("one LDS ring per K slice")
    assert lookup(16, 28672, 4096).startswith("decode with A in registers") and lookup(12, 28672, 4096).endswith("one LDS ring per K slice")
    assert lookup(16, 28672, 3072).startswith("split-K 32x64") and lookup(2, 28672, 512).startswith("streaming decode, 16")


def test_auto_plan_invariants_over_many_shapes(hgemm_lib):
    """What run_plan relies on, for every plan the model can come up with (no launch, no GPU): K slices are whole
    numbers of 64-wide chunks (the slices of a launch differ by at most one chunk), each at least as long as the
    shortest K its kernel takes, and fit the workspace cap; the four-wave 64x64 tile only takes grids of whole tiles, at
    most two per CU, and is unsliced and below 40 chunks when two share a CU; the 2-stage 128x128 tile only takes
    K <= 256, unsliced, without a tail."""
    import random
    rng = random.Random(5)
    shapes = [(t, t, k) for t in range(64, 3073, 64) for k in (64, 128, 192, 256, 320, 1024, 2560, 4096, 16384)]
    for _ in range(1500):
        shapes.append((rng.randrange(1, 9000), 8 * rng.randrange(1, 1100), 64 * rng.randrange(1, 260)))
    for _ in range(1500):                                                   # small M: the decode and split-K kernels
        shapes.append((rng.randrange(1, 130), 16 * rng.randrange(1, 2000), 64 * rng.randrange(1, 300)))
    cus = 256
    for (m, n, k) in shapes:
        p = hgemm_lib.auto_plan(m, n, k)
        s = p["splits"]
        assert s >= 1 and p["tail_splits"] >= 1, (m, n, k, p)
        if p["kernel"].startswith(("pipelined", "tiled", "split-K")):
            shortest = {"pipelined 256x256": 2, "pipelined 192x192": 3, "pipelined 192x128": 4, "pipelined 256x128": 3, "pipelined 128x128": 5,
                        "pipelined 64x128": 5, "pipelined 64x64": 3, "tiled 64x64x64": 3, "split-K": 1}
            floor = [v for key, v in shortest.items() if p["kernel"].startswith(key)][0]
            if "2-stage ring" in p["kernel"]:
                floor = 2
            assert k % 64 == 0 and k // 64 // s >= (floor if s > 1 or not p["kernel"].startswith("split-K") else 1), (m, n, k, p)
            assert k // 64 // p["tail_splits"] >= (floor if p["tail_splits"] > 1 else 1), (m, n, k, p)
        need = hgemm_lib.auto_workspace_bytes(m, n, k)
        assert need["partial"] <= 512 << 20 and need["operands"] <= 1024 << 20, (m, n, k, need)
        if p["kernel"].startswith("tiled 64x64x64"):
            assert m % 64 == 0 and n % 64 == 0 and p["tail_tiles"] == 0, (m, n, k, p)
            tiles = (m // 64) * (n // 64)
            assert tiles * s <= 2 * cus and k // 64 // s >= 3, (m, n, k, p)
            if tiles * s > cus:
                assert s == 1 and k // 64 < 40, (m, n, k, p)
        if "2-stage ring" in p["kernel"]:
            assert k <= 256 and s == 1 and p["tail_tiles"] == 0, (m, n, k, p)
        if p["kernel"].startswith("decode with A in registers"):
            # eight (four, two) waves, each with 8 ... 24 chunks of A in registers; rings and partial sums fit a CU
            assert m <= 32 and n % 16 == 0 and s in (2, 4, 8) and k % (64 * s) == 0 and k // (64 * s) in (8, 12, 16, 20, 24), (m, n, k, p)
            assert need == {"partial": 0, "operands": 0} and s * 8192 + 2 * s * (2 if m > 16 else 1) * 1024 <= 160 << 10, (m, n, k, p)
        elif "LDS ring per K slice" in p["kernel"]:
            # whole 64-wide chunks per wave; the waves' rings (16, 24, 30, 54 KB for 1, 2, 4, 8 row tiles of A) fit a CU
            assert m <= 128 and n % 16 == 0 and k % (64 * s) == 0 and need == {"partial": 0, "operands": 0}, (m, n, k, p)
            ring_kb = 16 if m <= 16 else 24 if m <= 32 else 30 if m <= 64 else 54
            assert s * ring_kb <= 160, (m, n, k, p)


def test_workspace_needs_of_auto_plans(hgemm_lib):
    """What hgemm_auto's plan keeps in device memory beyond A, B and C (no launch, no GPU)."""
    need = hgemm_lib.auto_workspace_bytes
    assert need(8192, 8192, 8192) == {"partial": 0, "operands": 0}
    assert need(1, 4096, 4096) == {"partial": 0, "operands": 0}                 # one-launch decode kernel
    p = hgemm_lib.auto_plan(256, 256, 16384)
    assert p["splits"] > 1 and need(256, 256, 16384) == {"partial": p["splits"] * 256 * 256 * 4, "operands": 0}
    p = hgemm_lib.auto_plan(64, 4096, 4096)
    assert need(64, 4096, 4096)["partial"] == (p["splits"] * 64 * 4096 * 4 if p["splits"] > 1 else 0)
    p = hgemm_lib.auto_plan(7168, 7168, 7168)                                    # last round in K slices
    assert need(7168, 7168, 7168)["partial"] == p["tail_splits"] * p["tail_tiles"] * 256 * 256 * 4
    padded = need(4095, 4095, 4095)                                             # A', B' and C' of 4095 x 4096 x 4096
    assert padded["operands"] == 2 * (4095 * 4096 + 4096 * 4096 + 4095 * 4096)
    for shape in ((16384, 16384, 16384), (100, 100, 100), (1 << 15, 1 << 15, 64)):
        n = need(*shape)
        assert n["partial"] <= 512 << 20 and n["operands"] <= 1024 << 20


def test_metrics(hgemm_lib):
    assert abs(hgemm_lib.tflops(8192, 8192, 8192, 1.0) - 1099.511627776) < 1e-9
    assert hgemm_lib.bytes(8192, 8192, 8192) == 2.0 * 3 * 8192 * 8192
    assert hgemm_lib.bytes(1, 4096, 4096) == 2.0 * (4096 + 4096 * 4096 + 4096)
    assert "gfx950" in hgemm_lib.version()


_VIOLATION = r"""
import ctypes, sys
sys.path.insert(0, {root!r})
import cuda_hgemm_amd
L = cuda_hgemm_amd.library()
buf = ctypes.create_string_buffer(64)
p = ctypes.addressof(buf)
{call}
print("returned")
"""


@pytest.mark.parametrize("call,needle", [
    ("L.dll.hgemm_auto(None, p, p, 8, 8, 8)", "Check failed: A != nullptr"),
    ("L.dll.hgemm_auto(p, p, p, 0, 8, 8)", "Check failed: (M) > (0u)"),
    ("L.dll.hgemm_mfma_async_stage4(p, p, p, 100, 128, 256)", "needs M % 256 == 0"),
    ("L.dll.hgemm_mfma_naive(p, p, p, 32, 32, 8)", "K % 16 == 0"),
    ("L.dll.hgemm_skinny(p, p, p, 200, 4096, 4096)", "M <= 128"),
    ("L.dll.hgemm_variant_name(99)", "out of range"),
])
def test_contract_violation_ends_the_process_with_a_message(call, needle):
    """No GPU call is reached: the checks run first, so this is safe on a CPU-only box."""
    code = _VIOLATION.format(root=ROOT, call=call)
    r = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, timeout=120)
    assert r.returncode == 1, (r.returncode, r.stdout, r.stderr)
    assert "returned" not in r.stdout
    assert needle in r.stderr and "[HGEMM " in r.stderr, r.stderr


def test_binding_rejects_bad_tensors(hgemm_lib):
    import torch
    a = torch.zeros((8, 8), dtype=torch.float16)
    with pytest.raises(ValueError, match="must live on the GPU"):
        hgemm_lib.call("hgemm_auto", a, a, a, 8, 8, 8)
    with pytest.raises(TypeError, match="float16"):
        hgemm_lib.call("hgemm_auto", a.float(), a, a, 8, 8, 8)


def test_driver_flag_parser():
    from cuda_hgemm_amd import driver_path
    exe = driver_path()
    assert os.path.exists(exe), "build the driver with `python -m cuda_hgemm_amd.build`"
    r = subprocess.run([exe, "-help"], capture_output=True, text=True, timeout=60)
    assert r.returncode == 0
    for flag in ("-M ", "-N ", "-K ", "-warmup_iterations", "-profiling_iterations", "-sleep_duration", "-enable_check",
                 "-cpu_procs", "-gpu_rank", "-seed", "-dist_a", "-dist_b"):
        assert flag in r.stderr, flag
    r = subprocess.run([exe, "-no_such_flag=1"], capture_output=True, text=True, timeout=60)
    assert r.returncode == 1 and "unknown flag -no_such_flag" in r.stderr
    r = subprocess.run([exe, "-M=abc"], capture_output=True, text=True, timeout=60)
    assert r.returncode == 1 and "is not a count" in r.stderr


def test_plans_the_tuner_would_time(hgemm_lib):
    """hgemm_auto_tune_plans (no launch): the first plan is hgemm_auto's own, no two are the same choice of kernel
    and K slices unless they differ in how the last round of a large grid is run, small-M shapes offer the other
    kernels of the rule table, and a shape with one possible kernel offers one plan."""
    for shape in ((8192, 8192, 8192), (384, 6144, 5120), (64, 4096, 4096), (16, 28672, 4096), (1, 4096, 4096), (2048, 2048, 2048)):
        plans = hgemm_lib.tune_plans(*shape, 8)
        own = hgemm_lib.auto_plan(*shape)
        assert 2 <= len(plans) <= 8 and (plans[0]["kernel_id"], plans[0]["splits"]) == (own["kernel_id"], own["splits"]), (shape, plans)
    small = hgemm_lib.tune_plans(64, 4096, 4096, 8)
    assert len({p["kernel"].split(",")[0] for p in small}) >= 3, small       # other kernels, not only other slice counts
    assert len(hgemm_lib.tune_plans(100, 100, 100, 8)) == 1                  # the guarded kernel only
    assert len(hgemm_lib.tune_plans(4095, 4095, 4095, 8)) == 1               # padded copies: the inner plan is not tuned
    assert len(hgemm_lib.tune_plans(8192, 8192, 8192, 1)) == 1 and len(hgemm_lib.tune_plans(8192, 8192, 8192, 100)) <= 12
    assert not hgemm_lib.plan_is_tuned(8192, 8192, 8192)


def test_slice_counts_of_the_split_k_family_on_timed_shapes(hgemm_lib):
    """The model behind the split-K family's slice count against shapes that were timed at every count from 1 to 16
    on an MI355X (microseconds at the count in brackets): the plan takes the fastest count, or one within 6 % of it."""
    timed = {   # shape: (kernel, {slices: microseconds})
        (96, 5120, 4096): ("split-K 128x64x64", {1: 27.6, 2: 19.6, 3: 16.3, 4: 22.3, 5: 20.4, 6: 19.8, 8: 23.8}),
        (128, 13312, 4096): ("split-K 128x64x64", {1: 32.5, 2: 40.2, 3: 43.9, 4: 47.1, 6: 50.5, 8: 60.2}),
        (48, 3072, 4096): ("split-K 64x64x64", {1: 21.2, 2: 14.5, 3: 12.2, 4: 10.7, 5: 10.3, 6: 12.5, 8: 12.5}),
        (64, 4096, 4096): ("split-K 64x64x64", {1: 22.1, 2: 16.2, 3: 13.6, 4: 12.6, 5: 14.4, 6: 13.8, 8: 14.0}),
        (128, 4096, 4096): ("split-K 128x64x64", {1: 28.8, 2: 20.2, 3: 16.9, 4: 15.9, 5: 21.4, 6: 20.7, 8: 20.8}),
        (32, 4096, 4096): ("split-K 32x64x64", {1: 20.9, 2: 14.2, 3: 12.0, 4: 11.5, 5: 11.9, 6: 11.8, 8: 11.8}),
        (96, 9216, 4096): ("split-K 128x64x64", {1: 29.1, 2: 35.1, 3: 28.2, 4: 33.0, 5: 31.1, 6: 35.0, 8: 38.5}),
        (48, 13312, 2048): ("split-K 64x64x64", {1: 14.0, 2: 17.5, 3: 20.1, 4: 21.7, 5: 23.3, 6: 23.6, 8: 25.1}),
        (22, 11264, 7296): ("split-K 32x64x64", {1: 36.5, 2: 36.5, 3: 36.7, 4: 33.1, 5: 33.8, 6: 35.4, 8: 35.6}),
        (128, 9216, 2048): ("split-K 128x64x64", {1: 18.1, 2: 24.3, 3: 21.7, 4: 27.4, 5: 26.3, 6: 30.2, 8: 34.2}),
    }
    for shape, (kernel, us) in timed.items():
        plan = hgemm_lib.auto_plan(*shape)
        assert plan["kernel"].startswith(kernel) and plan["splits"] in us, (shape, plan)
        assert us[plan["splits"]] <= 1.06 * min(us.values()), (shape, plan["splits"], us)
