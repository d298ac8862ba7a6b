"""Parity of the HIP kernels with the CPU checker, through the C ABI, on a real MI355X.

Bit-exact where the mathematics allows it (integer-valued inputs, identity operands,
one-hot probes, run-to-run), otherwise within the fp16 output tolerance of the benchmark
specification: max |err| <= 1e-2 * sqrt(K / 256) relative to the output scale (rms of the
reference), and additionally within one fp16 ulp of the largest output, which is what an
fp32-accumulate kernel should achieve.
"""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

POISON = 0xFFFF  # an fp16 NaN: any output element a kernel skips stays non-finite


def _to_gpu(bits, gpu):
    import torch
    return torch.from_numpy(np.ascontiguousarray(bits).view(np.int16)).to(gpu).view(torch.float16)


def _to_bits(t):
    import torch
    torch.cuda.synchronize()
    return t.view(torch.int16).cpu().numpy().view(np.uint16)


def _run(lib, variant, A_bits, B_bits, gpu, repeat=1):
    import torch
    M, K = A_bits.shape
    N = B_bits.shape[0]
    A, B = _to_gpu(A_bits, gpu), _to_gpu(B_bits, gpu)
    outs = []
    for _ in range(repeat):
        C = torch.full((M, N), POISON - 65536, dtype=torch.int16, device=gpu).view(torch.float16)
        print(f"[gpu] {variant} M={M} N={N} K={K}", flush=True)
        lib.call(variant, A, B, C, M, N, K)
        outs.append(_to_bits(C))
    return outs if repeat > 1 else outs[0]


def _assert_close(oracle, got, ref_bits, K, ref_f32=None):
    res = oracle.check(got, ref_bits, K)
    assert res["non_finite"] == 0, "outputs left unwritten or non-finite"
    assert res["ok"], res                                   # the specification's tolerance
    peak = float(np.abs(ref_bits.view(np.float16).astype(np.float32)).max())
    one_ulp = float(np.spacing(np.float16(peak))) if peak > 0 else 2.0 ** -24
    assert res["max_diff"] <= one_ulp, (res, one_ulp)       # what fp32 accumulation should give
    assert np.mean(got != ref_bits) < 0.02, np.mean(got != ref_bits)


TILED = ["hgemm_mfma_base", "hgemm_mfma_padding", "hgemm_mfma_swizzle", "hgemm_mfma_async", "hgemm_mfma_async_pg2s",
         "hgemm_mfma_async_pg2s_ps2r", "hgemm_mfma_async_stage2", "hgemm_mfma_async_stage3", "hgemm_mfma_async_stage4",
         "hgemm_mfma_tiled_64x64"]
PIPELINED = ["hgemm_mfma_pipelined_64x64", "hgemm_mfma_pipelined_128x128", "hgemm_mfma_pipelined_192x192",
             "hgemm_mfma_pipelined_256x128", "hgemm_mfma_pipelined_256x256", "hgemm_mfma_chained_192x192",
             "hgemm_mfma_chained_256x128", "hgemm_mfma_chained_256x256"]
ALL_AT_512 = ["hgemm_simt_naive", "hgemm_mfma_naive"] + TILED + ["hgemm_auto"]


# ------------------------------------------------------------------ exact cases
@pytest.mark.parametrize("variant", ALL_AT_512)
@pytest.mark.parametrize("shape", [(256, 128, 256), (512, 2048, 1024)])
def test_integer_inputs_are_bit_identical(oracle, hgemm_lib, gpu, variant, shape):
    """Entries in {-1,0,1}, K <= 2048: exact under any summation order (see tests/test_oracle.py)."""
    M, N, K = shape
    A = oracle.fill((M, K), 101, 1, oracle.TERNARY, 0, 1)
    B = oracle.fill((N, K), 101, 2, oracle.TERNARY, 0, 1)
    ref = A.view(np.float16).astype(np.int64) @ B.view(np.float16).astype(np.int64).T
    got = _run(hgemm_lib, variant, A, B, gpu)
    assert np.array_equal(got.view(np.float16).astype(np.int64), ref)
    assert np.array_equal(got, oracle.hgemm(A, B))


@pytest.mark.parametrize("variant", ["hgemm_mfma_naive", "hgemm_mfma_swizzle", "hgemm_mfma_async_stage4", "hgemm_auto"])
@pytest.mark.parametrize("K", [128, 1024, 32768])
def test_all_ones_gives_K(hgemm_lib, gpu, variant, K):
    ones = lambda r: np.full((r, K), 0x3C00, np.uint16)
    got = _run(hgemm_lib, variant, ones(256), ones(256), gpu)
    assert np.all(got.view(np.float16) == np.float16(K))


@pytest.mark.parametrize("variant", ALL_AT_512)
def test_identity_pins_operand_layouts(oracle, hgemm_lib, gpu, variant):
    """A = I: C[m][n] = B[n*K + m] -- fails if B is read as row-major K x N or if A and B
    are swapped.  B = I: C = A."""
    n = 256
    eye = np.eye(n, dtype=np.float16).view(np.uint16)
    B = oracle.fill((n, n), 7, 2)
    assert np.array_equal(_run(hgemm_lib, variant, eye, B, gpu), B.T)
    A = oracle.fill((n, n), 7, 1)
    assert np.array_equal(_run(hgemm_lib, variant, A, eye, gpu), A)


@pytest.mark.parametrize("variant", ["hgemm_mfma_naive", "hgemm_mfma_async_stage4", "hgemm_auto"])
def test_one_hot_probes_touch_exactly_one_output(hgemm_lib, gpu, variant):
    M, N, K = 512, 512, 256
    for (m, n, k) in [(0, 0, 0), (511, 511, 255), (255, 256, 31), (256, 127, 32), (37, 300, 200), (300, 33, 63)]:
        A = np.zeros((M, K), np.float16)
        B = np.zeros((N, K), np.float16)
        A[m, k], B[n, k] = 2.0, -1.5
        got = _run(hgemm_lib, variant, A.view(np.uint16), B.view(np.uint16), gpu).view(np.float16)
        expect = np.zeros((M, N), np.float16)
        expect[m, n] = -3.0
        assert np.array_equal(got, expect), (m, n, k, np.argwhere(got != expect)[:4])


# ------------------------------------------------------------------ random inputs, every variant
@pytest.mark.parametrize("variant", ALL_AT_512)
@pytest.mark.parametrize("shape", [(256, 256, 256), (512, 2048, 1024)])
def test_random_inputs_within_tolerance_and_deterministic(oracle, hgemm_lib, gpu, variant, shape):
    """(256,256,256) is the CPU-runnable configuration of the specification; (512,2048,1024)
    is the reference's own checked sample run (run_sample.sh:60)."""
    M, N, K = shape
    A, B = oracle.fill((M, K), oracle.DEFAULT_SEED, 1), oracle.fill((N, K), oracle.DEFAULT_SEED, 2)
    ref = oracle.hgemm(A, B)
    first, second = _run(hgemm_lib, variant, A, B, gpu, repeat=2)
    _assert_close(oracle, first, ref, K)
    assert np.array_equal(first, second), "results differ from run to run"


# ------------------------------------------------------------------ the tuned kernel by tile, as named variants
@pytest.mark.parametrize("variant", PIPELINED)
@pytest.mark.parametrize("shape", [(256, 256, 320), (512, 2048, 1024), (300, 136, 384), (1000, 1000, 448),
                                   (768, 512, 3072), (520, 776, 3136)])
def test_pipelined_variants(oracle, hgemm_lib, gpu, variant, shape):
    """Every tile of the tuned kernel through its own entry point, interleaved and chained: the
    reference's checked sample shape (run_sample.sh:60), the shortest K every ring accepts, M and
    N ending inside a tile, K of 5, 6, 7, 16, 48 and 49 chunks (the chained kernel's unrolled loop
    covers six chunks per trip, the rest go through its loop with run-time ring indices).
    Exact on ternary inputs, within tolerance and bit-identical run to run on random ones."""
    M, N, K = shape
    assert hgemm_lib.supports(variant, M, N, K)
    At, Bt = oracle.fill((M, K), 51, 1, oracle.TERNARY, 0, 1), oracle.fill((N, K), 51, 2, oracle.TERNARY, 0, 1)
    assert np.array_equal(_run(hgemm_lib, variant, At, Bt, gpu), oracle.hgemm(At, Bt))
    A, B = oracle.fill((M, K), 52, 1), oracle.fill((N, K), 52, 2)
    first, second = _run(hgemm_lib, variant, A, B, gpu, repeat=2)
    _assert_close(oracle, first, oracle.hgemm(A, B), K)
    assert np.array_equal(first, second)


@pytest.mark.parametrize("variant", PIPELINED)
def test_pipelined_variants_identity_and_min_k(oracle, hgemm_lib, gpu, variant):
    ring = {"64x64": 3, "128x128": 5, "192x192": 3, "256x128": 3, "256x256": 2}[variant.rsplit("_", 1)[1]]
    K = 64 * ring
    assert hgemm_lib.supports(variant, 256, 256, K) and not hgemm_lib.supports(variant, 256, 256, K - 64)
    At, Bt = oracle.fill((256, K), 53, 1, oracle.TERNARY, 0, 1), oracle.fill((256, K), 53, 2, oracle.TERNARY, 0, 1)
    assert np.array_equal(_run(hgemm_lib, variant, At, Bt, gpu), oracle.hgemm(At, Bt))
    n = 384
    eye = np.eye(n, dtype=np.float16).view(np.uint16)
    B = oracle.fill((n, n), 7, 2)
    assert np.array_equal(_run(hgemm_lib, variant, eye, B, gpu), B.T)


def test_flagship_variant_is_the_kernel_auto_runs_at_8192(oracle, hgemm_lib, gpu):
    """The top rung by name; the interleaved kernel on the same tile adds every output's products
    in the same order, so all three agree bit for bit."""
    n = 8192
    assert hgemm_lib.auto_plan(n, n, n)["kernel"].startswith("pipelined 256x256x64")
    A, B = oracle.fill((n, n), oracle.DEFAULT_SEED, 1), oracle.fill((n, n), oracle.DEFAULT_SEED, 2)
    named = _run(hgemm_lib, "hgemm_mfma_chained_256x256", A, B, gpu)
    assert np.array_equal(named, _run(hgemm_lib, "hgemm_auto", A, B, gpu))
    assert np.array_equal(named, _run(hgemm_lib, "hgemm_mfma_pipelined_256x256", A, B, gpu))
    _sampled_check(oracle, named, A, B, n, rows_per_slab=8, slabs=2)


# ------------------------------------------------------------------ the ladder's rings at their shortest K
@pytest.mark.parametrize("variant", TILED)
def test_ladder_rings_at_minimum_k(oracle, hgemm_lib, gpu, variant):
    """The shortest K each variant accepts (its prologue fills STAGES-1 buffers, so the loop
    starts draining at once: the branch that waits for every copy from the first iteration
    on), and one K chunk more."""
    M, N = 512, 256
    kmin = min(k for k in (32, 64, 96, 128, 160, 192, 256) if hgemm_lib.supports(variant, M, N, k))
    expected = {"hgemm_mfma_async_stage2": 64, "hgemm_mfma_async_stage3": 64, "hgemm_mfma_async_stage4": 96,
                "hgemm_mfma_tiled_64x64": 256}.get(variant, 32)
    assert kmin == expected, (variant, kmin)
    step = 64 if variant in ("hgemm_mfma_async_stage2", "hgemm_mfma_tiled_64x64") else 32      # their K chunk is 64 wide
    for K in (kmin, kmin + step):
        At, Bt = oracle.fill((M, K), 61, 1, oracle.TERNARY, 0, 1), oracle.fill((N, K), 61, 2, oracle.TERNARY, 0, 1)
        assert np.array_equal(_run(hgemm_lib, variant, At, Bt, gpu), oracle.hgemm(At, Bt)), K
        A, B = oracle.fill((M, K), 62, 1), oracle.fill((N, K), 62, 2)
        _assert_close(oracle, _run(hgemm_lib, variant, A, B, gpu), oracle.hgemm(A, B), K)


@pytest.mark.parametrize("chunks", [5, 6, 7, 8, 9, 12, 13])
def test_lookahead_ring_every_chunk_count(oracle, hgemm_lib, gpu, chunks):
    """hgemm_mfma_tiled_64x64 walks K in unrolled pairs of iterations while a copy is still to be issued, then one
    iteration at a time: odd and even counts of either kind, exact on ternary inputs."""
    M, N, K = 192, 320, 64 * chunks
    At, Bt = oracle.fill((M, K), 63, 1, oracle.TERNARY, 0, 1), oracle.fill((N, K), 63, 2, oracle.TERNARY, 0, 1)
    assert np.array_equal(_run(hgemm_lib, "hgemm_mfma_tiled_64x64", At, Bt, gpu), oracle.hgemm(At, Bt))
    A, B = oracle.fill((M, K), 64, 1), oracle.fill((N, K), 64, 2)
    _assert_close(oracle, _run(hgemm_lib, "hgemm_mfma_tiled_64x64", A, B, gpu), oracle.hgemm(A, B), K)


def test_vendor_comparator_matches_the_checker(oracle, vendor_lib, gpu):
    """Pins the transposes and leading dimensions of the hipBLASLt call."""
    import torch
    M, N, K = 384, 640, 512
    A, B = oracle.fill((M, K), 5, 1), oracle.fill((N, K), 5, 2)
    C = torch.full((M, N), float("nan"), dtype=torch.float16, device=gpu)
    vendor_lib.call(_to_gpu(A, gpu), _to_gpu(B, gpu), C, M, N, K)
    _assert_close(oracle, _to_bits(C), oracle.hgemm(A, B), K)


# ------------------------------------------------------------------ the dispatcher on the benchmark configurations
@pytest.mark.parametrize("n", [256, 512, 1024, 2048])
def test_auto_squares_full_check(oracle, hgemm_lib, gpu, n):
    A, B = oracle.fill((n, n), oracle.DEFAULT_SEED, 1), oracle.fill((n, n), oracle.DEFAULT_SEED, 2)
    first, second = _run(hgemm_lib, "hgemm_auto", A, B, gpu, repeat=2)
    _assert_close(oracle, first, oracle.hgemm(A, B), n)
    assert np.array_equal(first, second)


def _sampled_check(oracle, got, A, B, K, rows_per_slab=16, slabs=4, seed=0):
    M = A.shape[0]
    rng = np.random.default_rng(seed)
    starts = sorted(set([0, M - rows_per_slab] + [int(x) for x in rng.integers(0, M - rows_per_slab, slabs)]))
    for m0 in starts:
        ref = oracle.hgemm_rows(A, B, m0, rows_per_slab)
        _assert_close(oracle, got[m0:m0 + rows_per_slab], ref, K)
    assert not np.any((got & 0x7C00) == 0x7C00), "non-finite outputs"   # whole matrix, not only the sample


@pytest.mark.parametrize("shape,dist_b", [((4096, 4096, 4096), "uniform"), ((8192, 8192, 8192), "uniform"),
                                          ((4096, 14336, 4096), "weights"), ((4096, 4096, 14336), "weights")])
def test_auto_large_shapes_sampled_rows(oracle, hgemm_lib, gpu, shape, dist_b):
    """Full-size runs; the checker computes slabs of complete output rows (all N, all K)."""
    M, N, K = shape
    A = oracle.fill((M, K), oracle.DEFAULT_SEED, 1)
    B = oracle.fill((N, K), oracle.DEFAULT_SEED, 2) if dist_b == "uniform" else \
        oracle.fill((N, K), oracle.DEFAULT_SEED, 2, oracle.NORMAL, 0.0, 0.02)
    first, second = _run(hgemm_lib, "hgemm_auto", A, B, gpu, repeat=2)
    _sampled_check(oracle, first, A, B, K)
    assert np.array_equal(first, second)


@pytest.mark.parametrize("n", [768, 1536, 3072, 5120, 7168, 15360])
def test_auto_reference_sweep_dimensions(oracle, hgemm_lib, gpu, n):
    """The squares of the reference's sweep (run_sample.sh:30) that are not benchmark
    configurations, against the checker: whole matrix up to 1536, complete rows beyond."""
    A, B = oracle.fill((n, n), oracle.DEFAULT_SEED, 1), oracle.fill((n, n), oracle.DEFAULT_SEED, 2)
    first, second = _run(hgemm_lib, "hgemm_auto", A, B, gpu, repeat=2)
    if n <= 1536:
        _assert_close(oracle, first, oracle.hgemm(A, B), n)
    else:
        _sampled_check(oracle, first, A, B, n, rows_per_slab=8, slabs=4, seed=n)
    assert np.array_equal(first, second)


def test_auto_16384_sampled_rows(oracle, hgemm_lib, gpu):
    n = 16384
    A, B = oracle.fill((n, n), oracle.DEFAULT_SEED, 1), oracle.fill((n, n), oracle.DEFAULT_SEED, 2)
    got = _run(hgemm_lib, "hgemm_auto", A, B, gpu)
    _sampled_check(oracle, got, A, B, n, rows_per_slab=8, slabs=2)


@pytest.mark.parametrize("shape,tile,split", [
    ((3072, 3072, 256), "192x192x64", False), ((2560, 2560, 320), "256x128x64", False),
    ((4096, 4096, 256), "2-stage ring", False), ((4100, 4104, 192), "2-stage ring", False), ((2048, 2048, 128), "2-stage ring", False),
    ((256, 256, 8192), "64x64x64", True), ((1024, 1024, 16384), "128x128x64", True),
    ((1024, 1024, 4096), "tiled 64x64x64", False), ((512, 768, 640), "tiled 64x64x64", False), ((1152, 1280, 1024), "tiled 64x64x64", False), ((1408, 1408, 2048), "tiled 64x64x64", False), ((192, 192, 192), "tiled 64x64x64", False),
    ((512, 512, 4096), "tiled 64x64x64", True), ((256, 256, 16384), "tiled 64x64x64", True),
    ((512, 512, 8192), "64x64x64", True), ((1536, 1536, 16384), "192x192x64", True),
    ((2048, 2048, 16384), "256x256x64", True), ((1536, 1536, 8192), "192x192x64", True),
    ((2048, 2048, 10240), "256x128x64", True)])
def test_auto_every_tile_with_and_without_k_slices(oracle, hgemm_lib, gpu, shape, tile, split):
    """Shapes chosen so the dispatcher's cost model lands on each pipelined tile, alone and
    with K cut into slices (fp32 partial sums + ordered reduction), and on the four-wave 64x64
    tile it runs on small grids of whole tiles."""
    M, N, K = shape
    plan = hgemm_lib.auto_plan(M, N, K)
    assert tile in plan["kernel"] and (plan["splits"] > 1) == split, plan
    A, B = oracle.fill((M, K), 21, 1), oracle.fill((N, K), 21, 2)
    first, second = _run(hgemm_lib, "hgemm_auto", A, B, gpu, repeat=2)
    _assert_close(oracle, first, oracle.hgemm(A, B), K)
    assert np.array_equal(first, second)
    At, Bt = oracle.fill((M, K), 22, 1, oracle.TERNARY, 0, 1), oracle.fill((N, K), 22, 2, oracle.TERNARY, 0, 1)
    ref = oracle.hgemm(At, Bt)
    assert np.abs(ref.view(np.float16).astype(np.float32)).max() <= 2048      # integers exact in fp16
    assert np.array_equal(_run(hgemm_lib, "hgemm_auto", At, Bt, gpu), ref)


@pytest.mark.parametrize("shape,kernel,where", [
    ((227, 128, 1216), "pipelined 64x64x64", "main"), ((2531, 256, 3392), "pipelined 128x128x64", "main"),
    ((131, 4096, 9536), "pipelined 192x192x64", "main"), ((320, 6272, 12352), "pipelined 192x192x64", "main chained"),
    ((2900, 264, 11072), "pipelined 256x128x64", "main"), ((2089, 1024, 12608), "pipelined 256x128x64", "main chained"),
    ((1075, 4120, 5632), "pipelined 256x256x64", "main chained"), ((192, 128, 1408), "tiled 64x64x64", "main"),
    ((256, 256, 16384), "tiled 64x64x64", "main"), ((512, 8280, 4864), "pipelined 128x128x64", "tail"),
    ((1024, 8240, 3264), "pipelined 256x128x64", "tail"), ((1024, 8840, 4288), "pipelined 256x128x64", "tail chained"),
    ((640, 28672, 8192), "pipelined 256x256x64", "tail chained"),
    ((1, 192, 1344), "split-K 32x64x64", "main"), ((63, 64, 1216), "split-K 64x64x64", "main"),
    ((37, 17152, 2176), "split-K 64x128x64", "main"), ((80, 64, 1088), "split-K 128x64x64", "main"),
    ((102, 16384, 1856), "split-K 128x128x64", "main"), ((110, 3072, 10112), "split-K 128x64x64", "main")])
def test_k_slices_that_differ_by_a_chunk(oracle, hgemm_lib, gpu, shape, kernel, where):
    """K is cut into slices of whole 64-wide chunks, as even as that allows: where the slice count does not divide the
    chunk count the first slices walk one chunk more.  Every kernel that takes K slices (each pipelined tile,
    interleaved and chained, the four-wave 64x64 tile, the last round of a large grid, the five split-K tiles), on a
    shape whose plan has such slices."""
    M, N, K = shape
    plan = hgemm_lib.auto_plan(M, N, K)
    slices = plan["tail_splits"] if where.startswith("tail") else plan["splits"]
    assert plan["kernel"].startswith(kernel) and slices > 1 and (K // 64) % slices != 0, plan
    assert bool(plan["chained"]) == where.endswith("chained"), plan
    assert (plan["tail_tiles"] > 0) == where.startswith("tail"), plan
    A, B = oracle.fill((M, K), 81, 1), oracle.fill((N, K), 81, 2)
    first, second = _run(hgemm_lib, "hgemm_auto", A, B, gpu, repeat=2)
    assert np.array_equal(first, second)
    At, Bt = oracle.fill((M, K), 82, 1, oracle.TERNARY, 0, 1), oracle.fill((N, K), 82, 2, oracle.TERNARY, 0, 1)
    exact = _run(hgemm_lib, "hgemm_auto", At, Bt, gpu)
    if M * N * K <= 3e10:
        _assert_close(oracle, first, oracle.hgemm(A, B), K)
        assert np.array_equal(exact, oracle.hgemm(At, Bt))
    else:                                      # complete rows from every row of tiles
        _sampled_check(oracle, first, A, B, K, rows_per_slab=16, slabs=6, seed=5)
        for m0 in list(range(0, M - 16, 131)) + [M - 8]:
            assert np.array_equal(exact[m0:m0 + 8], oracle.hgemm_rows(At, Bt, m0, 8)), m0


@pytest.mark.parametrize("t", [768, 1280, 1536, 1792, 2048, 2304])
@pytest.mark.parametrize("K", [7168, 10240, 13312, 16384])
def test_auto_deep_k_plans(oracle, hgemm_lib, gpu, t, K):
    """Squares of few tiles under a deep K: the dispatcher cuts K into slices on every tile, with either tuned
    kernel (the shapes cover 128x128, 192x192, 256x128 and 256x256, interleaved and chained).  Slabs of 16 complete
    rows are checked, so every row of an MFMA tile and every lane of the wave that stores it is looked at."""
    A, B = oracle.fill((t, K), 71, 1), oracle.fill((t, K), 71, 2)
    got = _run(hgemm_lib, "hgemm_auto", A, B, gpu)
    _sampled_check(oracle, got, A, B, K, rows_per_slab=16, slabs=3, seed=t + K)


@pytest.mark.parametrize("shape,mode", [((7168, 7168, 7168), "k slices"), ((7168, 7168, 2048), "128x128x64"),
                                        ((4352, 4344, 4096), "128x128x64"), ((4352, 4352, 1024), "64x64x64"),
                                        ((4096, 14336, 4096), "256x128x64"), ((4360, 4352, 512), "128x128x64")])
def test_auto_last_round_of_a_large_grid(oracle, hgemm_lib, gpu, shape, mode):
    """Grids of whole rounds of workgroups plus a few: the few run in K slices with compact
    partial sums, or their tiles are divided among workgroups of a smaller tile (also with
    ragged edges).  Complete rows are checked, including rows of the tiles treated that way."""
    M, N, K = shape
    plan = hgemm_lib.auto_plan(M, N, K)
    assert plan["tail_tiles"] > 0, plan
    if mode == "k slices":
        assert plan["tail_splits"] > 1 and plan["tail_kernel"] == "none", plan
    else:
        assert plan["tail_splits"] == 1 and mode in plan["tail_kernel"], plan
    A, B = oracle.fill((M, K), 41, 1), oracle.fill((N, K), 41, 2)
    first, second = _run(hgemm_lib, "hgemm_auto", A, B, gpu, repeat=2)
    _sampled_check(oracle, first, A, B, K, rows_per_slab=16, slabs=12, seed=3)
    assert np.array_equal(first, second)
    At, Bt = oracle.fill((M, K), 42, 1, oracle.TERNARY, 0, 1), oracle.fill((N, K), 42, 2, oracle.TERNARY, 0, 1)
    got = _run(hgemm_lib, "hgemm_auto", At, Bt, gpu)
    for m0 in range(0, M - 64, 509):          # exact, rows spread over every row of tiles
        assert np.array_equal(got[m0:m0 + 8], oracle.hgemm_rows(At, Bt, m0, 8)), m0
    assert np.array_equal(got[M - 8:], oracle.hgemm_rows(At, Bt, M - 8, 8))


@pytest.mark.parametrize("variant,shape", [
    ("hgemm_auto", (520, 9480, 8192)),                    # 3 x 38 tiles of 256: clipped blocks, ragged M and N
    ("hgemm_auto", (4352, 9472, 8192)),                   # 17 x 37 tiles: whole rounds plus a last, separately launched one
    ("hgemm_mfma_chained_256x256", (2304, 9472, 8192)),   # 9 x 37 tiles in one launch
    ("hgemm_mfma_pipelined_256x256", (2304, 9472, 8192)),
    ("hgemm_mfma_pipelined_128x128", (648, 9480, 8192)),  # 6 x 75 tiles of 128, three workgroups per round and XCD
    ("hgemm_mfma_async_stage4", (512, 9472, 8192)),       # the ladder's 256 x 128 tiles: 2 x 74
])
def test_block_tile_order(oracle, hgemm_lib, gpu, variant, shape):
    """A B of more than 144 MiB switches the tuned kernels (and the ladder) to the order that
    deals 16 x 16 blocks of tiles per round: every tile must still be computed exactly once,
    whatever the grid and however the launch is cut.  C starts as NaN, so a tile nobody
    computes shows; ternary inputs make complete rows exact, rows taken from every row of tiles."""
    M, N, K = shape
    assert N * K > 72 << 20
    At, Bt = oracle.fill((M, K), 43, 1, oracle.TERNARY, 0, 1), oracle.fill((N, K), 43, 2, oracle.TERNARY, 0, 1)
    first, second = _run(hgemm_lib, variant, At, Bt, gpu, repeat=2)
    assert not np.any((first & 0x7C00) == 0x7C00), "outputs left unwritten or non-finite"
    assert np.array_equal(first, second)
    rows = np.unique(np.concatenate([np.arange(m0, m0 + 4) for m0 in list(range(0, M - 8, 61)) + [M - 4]]))
    assert np.array_equal(first[rows], oracle.hgemm(np.ascontiguousarray(At[rows]), Bt))


@pytest.mark.parametrize("N", [4096, 28672])
@pytest.mark.parametrize("M", [1, 8, 16, 64, 128])
def test_decode_shapes(oracle, hgemm_lib, gpu, M, N):
    K = 4096
    A = oracle.fill((M, K), oracle.DEFAULT_SEED, 1, oracle.NORMAL, 0.0, 1.0)
    B = oracle.fill((N, K), oracle.DEFAULT_SEED, 2, oracle.NORMAL, 0.0, 0.02)
    ref = oracle.hgemm(A, B)
    for variant in ("hgemm_skinny", "hgemm_auto"):
        first, second = _run(hgemm_lib, variant, A, B, gpu, repeat=2)
        _assert_close(oracle, first, ref, K)
        assert np.array_equal(first, second)


@pytest.mark.parametrize("shape", [(1, 4096, 4096), (2, 32, 256), (3, 96, 512), (5, 4096, 1024), (5, 28672, 2048),
                                   (8, 2048, 8192), (4, 16384, 4096), (8, 32768, 1280), (6, 64, 16384), (3, 64, 768),
                                   (4, 20480, 2816), (7, 8192, 4096)])
def test_streaming_decode_kernel(oracle, hgemm_lib, gpu, shape):
    """M <= 8: both column-tile widths, one to eight K slices per workgroup, slices that are
    and are not a whole number of load groups."""
    M, N, K = shape
    assert hgemm_lib.auto_plan(M, N, K)["kernel"].startswith("streaming decode")
    A = oracle.fill((M, K), 31, 1, oracle.NORMAL, 0.0, 1.0)
    B = oracle.fill((N, K), 31, 2, oracle.NORMAL, 0.0, 0.02)
    first, second = _run(hgemm_lib, "hgemm_auto", A, B, gpu, repeat=2)
    _assert_close(oracle, first, oracle.hgemm(A, B), K)
    assert np.array_equal(first, second)
    At, Bt = oracle.fill((M, K), 32, 1, oracle.TERNARY, 0, 1), oracle.fill((N, K), 32, 2, oracle.TERNARY, 0, 1)
    assert np.array_equal(_run(hgemm_lib, "hgemm_auto", At, Bt, gpu), oracle.hgemm(At, Bt))


@pytest.mark.parametrize("shape", [(1, 4096, 4096), (16, 4096, 4096), (9, 272, 1024), (13, 1040, 1152), (16, 8192, 1024),
                                   (3, 16, 3072), (8, 2048, 8192), (11, 4096, 8192), (16, 336, 1280), (2, 14336, 2048),
                                   (5, 8192, 8192), (7, 4112, 16384 - 128), (17, 4096, 2048), (32, 4096, 1024),
                                   (24, 1040, 1280), (33, 4096, 2048), (64, 4096, 1024), (48, 2064, 1152), (40, 272, 1024),
                                   (16, 4096, 256), (64, 8192, 896), (33, 272, 384), (9, 1040, 640),
                                   (65, 4096, 1024), (128, 8192, 512), (100, 272, 384), (128, 4096, 256), (24, 4096, 4096), (5, 1040, 384), (8, 4096, 640),
                                   # B of 48 MB or more: the copies of B carry the non-temporal hint
                                   (1, 28672, 4096), (8, 28672, 4096), (12, 28672, 4096), (5, 14336, 4096), (12, 12288, 8192),
                                   (3, 57344, 1024), (7, 28672, 2048), (8, 20480, 2816), (6, 14336, 4096), (16, 8192, 4096)])
def test_decode_kernel_with_lds_rings(oracle, hgemm_lib, gpu, shape):
    """M <= 128 through per-wave LDS rings (one, two, four or eight 16-row tiles of A per wave): one, two, four and eight K slices per workgroup, slices of one chunk and of
    many (127 when only two waves divide K), slices shorter than the ring, N of one to 896 column tiles, rows of A
    beyond M."""
    M, N, K = shape
    plan = hgemm_lib.auto_plan(M, N, K)
    assert "LDS ring per K slice" in plan["kernel"] and K % (plan["splits"] * 64) == 0, plan
    A = oracle.fill((M, K), 35, 1, oracle.NORMAL, 0.0, 1.0)
    B = oracle.fill((N, K), 35, 2, oracle.NORMAL, 0.0, 0.02)
    first, second = _run(hgemm_lib, "hgemm_auto", A, B, gpu, repeat=2)
    _assert_close(oracle, first, oracle.hgemm(A, B), K)
    assert np.array_equal(first, second)
    At, Bt = oracle.fill((M, K), 36, 1, oracle.TERNARY, 0, 1), oracle.fill((N, K), 36, 2, oracle.TERNARY, 0, 1)
    assert np.array_equal(_run(hgemm_lib, "hgemm_auto", At, Bt, gpu), oracle.hgemm(At, Bt))


@pytest.mark.parametrize("shape", [(16, 28672, 4096), (13, 18448, 4096), (9, 14336, 6144), (16, 14336, 8192), (11, 14352, 8192),
                                   (17, 18432, 4096), (24, 20496, 4096), (20, 57344, 4096), (14, 16384, 6144), (32, 40976, 4096)])
def test_decode_kernel_with_a_in_registers(oracle, hgemm_lib, gpu, shape):
    """M = 9 ... 24 against N >= 14336 (up to M = 32 from N = 32768): persistent workgroups that load their waves' K slices of A into registers once
    and walk over 16-column tiles of C.  8, 12 and 16 chunks of K per wave, one and two row tiles of A, one and two
    workgroups per CU, tile counts that do and do not divide among the workgroups (some get one tile more; with 897
    tiles and 512 workgroups some get a single tile), rows of A beyond M."""
    M, N, K = shape
    plan = hgemm_lib.auto_plan(M, N, K)
    assert plan["kernel"].startswith("decode with A in registers") and plan["splits"] == 8, plan
    A = oracle.fill((M, K), 37, 1, oracle.NORMAL, 0.0, 1.0)
    B = oracle.fill((N, K), 37, 2, oracle.NORMAL, 0.0, 0.02)
    first, second = _run(hgemm_lib, "hgemm_auto", A, B, gpu, repeat=2)
    _assert_close(oracle, first, oracle.hgemm(A, B), K)
    assert np.array_equal(first, second)
    At, Bt = oracle.fill((M, K), 38, 1, oracle.TERNARY, 0, 1), oracle.fill((N, K), 38, 2, oracle.TERNARY, 0, 1)
    assert np.array_equal(_run(hgemm_lib, "hgemm_auto", At, Bt, gpu), oracle.hgemm(At, Bt))


@pytest.mark.parametrize("shape", [(7, 57344, 1024), (8, 65536, 1536), (12, 28672, 3072), (100, 14336, 4096)])
def test_small_m_against_a_large_b(oracle, hgemm_lib, gpu, shape):
    """B of 96 MB or more where the split-K kernel runs, with B copied past the caches (non-temporal hint): M = 6 ... 8
    while K < 2048, M = 9 ... 16 at the K where it is ahead of the ring kernel, M = 65 ... 128 below 144 column tiles."""
    M, N, K = shape
    assert hgemm_lib.auto_plan(M, N, K)["kernel"].startswith("split-K")
    A = oracle.fill((M, K), 33, 1, oracle.NORMAL, 0.0, 1.0)
    B = oracle.fill((N, K), 33, 2, oracle.NORMAL, 0.0, 0.02)
    first, second = _run(hgemm_lib, "hgemm_auto", A, B, gpu, repeat=2)
    _assert_close(oracle, first, oracle.hgemm(A, B), K)
    assert np.array_equal(first, second)
    At, Bt = oracle.fill((M, K), 34, 1, oracle.TERNARY, 0, 1), oracle.fill((N, K), 34, 2, oracle.TERNARY, 0, 1)
    assert np.array_equal(_run(hgemm_lib, "hgemm_auto", At, Bt, gpu), oracle.hgemm(At, Bt))


@pytest.mark.parametrize("shape", [(128, 28672, 4096), (100, 18440, 1024), (65, 20480, 2048), (128, 18432, 1088),
                                   (97, 24584, 1024), (128, 28672, 320 + 704),
                                   (64, 28672, 4096), (33, 18440, 1024), (50, 20480, 2048), (64, 24584, 1088), (64, 28672, 320),
                                   (128, 28672, 384), (25, 28672, 4096), (32, 18432, 4096)])
def test_one_tile_row_against_many_column_tiles(oracle, hgemm_lib, gpu, shape):
    """M = 33 ... 128 against N >= 18432: one launch of the pipelined kernel on a 128x128 tile (a 64x128 tile up to
    M = 64) whose copies of B carry the non-temporal hint (from 48 MB of B on; the smaller cases run the same rule
    without the hint), rows of the tile beyond M and a last column tile that ends inside the tile included."""
    M, N, K = shape
    plan = hgemm_lib.auto_plan(M, N, K)
    tile = "128x128x64" if M > 64 else "64x128x64"      # M = 25 ... 32 (at K = 8192: 17 ... 32) join the 64x128 tile from K = 4096
    assert plan["kernel"].startswith(f"pipelined {tile}, 4 waves, 5-stage") and plan["splits"] == 1, plan
    A = oracle.fill((M, K), 41, 1, oracle.NORMAL, 0.0, 1.0)
    B = oracle.fill((N, K), 41, 2, oracle.NORMAL, 0.0, 0.02)
    first, second = _run(hgemm_lib, "hgemm_auto", A, B, gpu, repeat=2)
    _assert_close(oracle, first, oracle.hgemm(A, B), K)
    assert np.array_equal(first, second)
    At, Bt = oracle.fill((M, K), 42, 1, oracle.TERNARY, 0, 1), oracle.fill((N, K), 42, 2, oracle.TERNARY, 0, 1)
    assert np.array_equal(_run(hgemm_lib, "hgemm_auto", At, Bt, gpu), oracle.hgemm(At, Bt))


@pytest.mark.parametrize("shape,slices", [((128, 6144, 8192), 5), ((64, 8192, 8192), 4), ((100, 12296, 8256), 5),
                                           ((40, 18432, 12352), 7), ((32, 18432, 8192), 5), ((128, 16384, 8192), 2),
                                           ((100, 10240, 6144), 3), ((65, 6144, 7168), 5)])
def test_one_tile_row_in_k_slices(oracle, hgemm_lib, gpu, shape, slices):
    """M = 17 ... 128 with a long K against fewer column tiles than CUs: the one-row 128x128 / 64x128 tiles with K in
    slices (B copied non-temporally in the sliced launch as well), slice counts that do and do not divide K's chunks,
    a last column tile that ends inside N."""
    M, N, K = shape
    plan = hgemm_lib.auto_plan(M, N, K)
    assert plan["kernel"].startswith("pipelined %s" % ("128x128x64" if M > 64 else "64x128x64")) and plan["splits"] == slices, plan
    A = oracle.fill((M, K), 47, 1, oracle.NORMAL, 0.0, 1.0)
    B = oracle.fill((N, K), 47, 2, oracle.NORMAL, 0.0, 0.02)
    first, second = _run(hgemm_lib, "hgemm_auto", A, B, gpu, repeat=2)
    _assert_close(oracle, first, oracle.hgemm(A, B), K)
    assert np.array_equal(first, second)
    At, Bt = oracle.fill((M, K), 48, 1, oracle.TERNARY, 0, 1), oracle.fill((N, K), 48, 2, oracle.TERNARY, 0, 1)
    assert np.array_equal(_run(hgemm_lib, "hgemm_auto", At, Bt, gpu), oracle.hgemm(At, Bt))


@pytest.mark.parametrize("shape,tail", [((103, 34304, 6656), (12, 16)), ((117, 39936, 6464), (56, 4)), ((50, 33024, 6464), (2, 16)),
                                        ((128, 65792, 4160), (2, 13)), ((64, 32776, 8192), (1, 16)), ((76, 52224, 640), (0, 1)),
                                        ((60, 42496, 1536), (0, 1))])
def test_one_tile_row_with_more_tiles_than_cus(oracle, hgemm_lib, gpu, shape, tail):
    """One row of 128x128 or 64x128 tiles against more column tiles than the chip has CUs: whole rounds in one launch
    (B copied non-temporally), the tiles beyond them in K slices that fill the chip, slices that differ by a chunk
    and a last tile that ends inside N included; with a short K the tiles beyond the whole rounds stay a round of
    their own."""
    M, N, K = shape
    plan = hgemm_lib.auto_plan(M, N, K)
    assert plan["kernel"].startswith("pipelined %s" % ("128x128x64" if M > 64 else "64x128x64")) and plan["splits"] == 1, plan
    assert (plan["tail_tiles"], plan["tail_splits"]) == tail and plan["tail_kernel"] == "none", plan
    A = oracle.fill((M, K), 43, 1, oracle.NORMAL, 0.0, 1.0)
    B = oracle.fill((N, K), 43, 2, oracle.NORMAL, 0.0, 0.02)
    first, second = _run(hgemm_lib, "hgemm_auto", A, B, gpu, repeat=2)
    _assert_close(oracle, first, oracle.hgemm(A, B), K)
    assert np.array_equal(first, second)
    At, Bt = oracle.fill((M, K), 44, 1, oracle.TERNARY, 0, 1), oracle.fill((N, K), 44, 2, oracle.TERNARY, 0, 1)
    assert np.array_equal(_run(hgemm_lib, "hgemm_auto", At, Bt, gpu), oracle.hgemm(At, Bt))


@pytest.mark.parametrize("shape", [(100, 36864, 1024), (65, 34816, 512), (128, 49152, 2048), (96, 40968, 4096),
                                   (64, 34816, 4096), (40, 36864, 512)])
def test_one_row_of_192_wide_tiles(oracle, hgemm_lib, gpu, shape):
    """M = 65 ... 128 against N = 32769 ... 49152 (M = 33 ... 64: up to N = 36864): more than 256 column tiles of 128 but
    at most 256 of 192, so one row of the 192x192 tile; rows of the tile beyond M, a last column tile that ends inside N."""
    M, N, K = shape
    plan = hgemm_lib.auto_plan(M, N, K)
    assert plan["kernel"].startswith("pipelined 192x192x64") and plan["splits"] == 1 and plan["tail_tiles"] == 0, plan
    A = oracle.fill((M, K), 49, 1, oracle.NORMAL, 0.0, 1.0)
    B = oracle.fill((N, K), 49, 2, oracle.NORMAL, 0.0, 0.02)
    first, second = _run(hgemm_lib, "hgemm_auto", A, B, gpu, repeat=2)
    _assert_close(oracle, first, oracle.hgemm(A, B), K)
    assert np.array_equal(first, second)
    At, Bt = oracle.fill((M, K), 50, 1, oracle.TERNARY, 0, 1), oracle.fill((N, K), 50, 2, oracle.TERNARY, 0, 1)
    assert np.array_equal(_run(hgemm_lib, "hgemm_auto", At, Bt, gpu), oracle.hgemm(At, Bt))


@pytest.mark.parametrize("shape", [(192, 28672, 2048), (129, 18440, 4096), (160, 57344, 2112), (177, 20480, 8192)])
def test_one_row_of_192x128_tiles(oracle, hgemm_lib, gpu, shape):
    """M = 129 ... 192 against 144 column tiles or more: one row of 192x128 tiles on a four-stage ring, B copied
    non-temporally; rows of the tile beyond M, a last column tile that ends inside N, more tiles than CUs."""
    M, N, K = shape
    plan = hgemm_lib.auto_plan(M, N, K)
    assert plan["kernel"].startswith("pipelined 192x128x64, 4 waves, 4-stage") and plan["splits"] == 1 and plan["tail_tiles"] == 0, plan
    A = oracle.fill((M, K), 45, 1, oracle.NORMAL, 0.0, 1.0)
    B = oracle.fill((N, K), 45, 2, oracle.NORMAL, 0.0, 0.02)
    first, second = _run(hgemm_lib, "hgemm_auto", A, B, gpu, repeat=2)
    _assert_close(oracle, first, oracle.hgemm(A, B), K)
    assert np.array_equal(first, second)
    At, Bt = oracle.fill((M, K), 46, 1, oracle.TERNARY, 0, 1), oracle.fill((N, K), 46, 2, oracle.TERNARY, 0, 1)
    assert np.array_equal(_run(hgemm_lib, "hgemm_auto", At, Bt, gpu), oracle.hgemm(At, Bt))


@pytest.mark.parametrize("M", [3, 17, 33, 100, 127])
def test_skinny_ragged_M(oracle, hgemm_lib, gpu, M):
    N, K = 1024, 512
    A, B = oracle.fill((M, K), 9, 1), oracle.fill((N, K), 9, 2)
    _assert_close(oracle, _run(hgemm_lib, "hgemm_skinny", A, B, gpu), oracle.hgemm(A, B), K)
    At = oracle.fill((M, K), 9, 1, oracle.TERNARY, 0, 1)
    Bt = oracle.fill((N, K), 9, 2, oracle.TERNARY, 0, 1)
    assert np.array_equal(_run(hgemm_lib, "hgemm_skinny", At, Bt, gpu), oracle.hgemm(At, Bt))


RAGGED = [(100, 100, 100), (1, 7, 5), (3, 17, 33), (257, 129, 33), (640, 384, 192), (192, 320, 4096),
          (300, 304, 64), (130, 250, 1000), (1000, 1000, 1000), (129, 4096, 512), (1000, 4000, 1024),
          (1030, 520, 2048), (70, 72, 8192), (2100, 2056, 384), (515, 1032, 4100), (260, 1288, 6144),
          (2047, 2049, 2051), (2050, 2050, 2048), (64, 1023, 1022),
          # tile-aligned but K shorter than any LDS ring; tall and thin outputs
          (256, 256, 64), (512, 512, 128), (128, 128, 64), (4096, 64, 1024), (8192, 8, 512), (2048, 16, 4096),
          (129, 8, 64), (16, 24, 320), (9, 32, 256), (33, 4096, 256)]


@pytest.mark.parametrize("shape", RAGGED)
def test_auto_handles_shapes_no_tile_divides(oracle, hgemm_lib, gpu, shape):
    """M, N, K that end inside a tile: the pipelined kernels with guarded edges (N % 8 == 0,
    K % 64 == 0, with and without K slices), zero-padded operand copies for large unaligned
    shapes, and the fully guarded kernel for the rest.
    Poisoned C shows any element left unwritten; exact ternary inputs show any element
    taken from a wrong row or from beyond K."""
    M, N, K = shape
    A, B = oracle.fill((M, K), 13, 1), oracle.fill((N, K), 13, 2)
    first, second = _run(hgemm_lib, "hgemm_auto", A, B, gpu, repeat=2)
    _assert_close(oracle, first, oracle.hgemm(A, B), K)
    assert np.array_equal(first, second)
    At, Bt = oracle.fill((M, K), 14, 1, oracle.TERNARY, 0, 1), oracle.fill((N, K), 14, 2, oracle.TERNARY, 0, 1)
    assert np.array_equal(_run(hgemm_lib, "hgemm_auto", At, Bt, gpu), oracle.hgemm(At, Bt))


@pytest.mark.parametrize("variant,shape", [("hgemm_auto", (4300000, 64, 64)), ("hgemm_auto", (70000, 64, 128)),
                                           ("hgemm_auto", (66000 * 128 + 5, 3, 5)), ("hgemm_simt_naive", (1100000, 16, 16)),
                                           ("hgemm_simt_naive", (16, 1100000, 16)), ("hgemm_mfma_naive", (32, 2200000, 16)),
                                           ("hgemm_mfma_naive", (2200000, 32, 16)), ("hgemm_auto", (8, 4300032, 64))])
def test_more_row_or_column_tiles_than_a_grid_dimension_holds(oracle, hgemm_lib, gpu, variant, shape):
    """Very tall or very wide outputs: more than 65535 tiles along M or N.  Every kernel
    indexes its tiles through a one-dimensional grid, so these launch like any other shape."""
    M, N, K = shape
    assert hgemm_lib.supports(variant, M, N, K)
    At, Bt = oracle.fill((M, K), 71, 1, oracle.TERNARY, 0, 1), oracle.fill((N, K), 71, 2, oracle.TERNARY, 0, 1)
    got = _run(hgemm_lib, variant, At, Bt, gpu)
    ref = At.view(np.float16).astype(np.float32) @ Bt.view(np.float16).astype(np.float32).T   # exact: small integers
    assert np.array_equal(got.view(np.float16).astype(np.float32), ref)


def test_workspace_reserve_release_and_shape_changes(oracle, hgemm_lib, gpu):
    """Shapes whose plans need growing amounts of partial sums and padded operand copies, in
    turn, around an explicit reserve and release; results exact on ternary inputs."""
    shapes = [(256, 256, 8192), (2048, 2048, 16384), (512, 512, 8192), (1111, 1111, 1111), (64, 4096, 4096),
              (2047, 2049, 2051), (256, 256, 8192)]
    need = [hgemm_lib.auto_workspace_bytes(*s) for s in shapes]
    assert need[0]["partial"] > 0 and need[1]["partial"] > need[0]["partial"] and need[5]["operands"] > 0
    hgemm_lib.release_workspace()
    for round_ in range(2):
        for (M, N, K) in shapes:
            At, Bt = oracle.fill((M, K), 81, 1, oracle.TERNARY, 0, 1), oracle.fill((N, K), 81, 2, oracle.TERNARY, 0, 1)
            assert np.array_equal(_run(hgemm_lib, "hgemm_auto", At, Bt, gpu), oracle.hgemm(At, Bt)), (M, N, K)
        if round_ == 0:
            hgemm_lib.release_workspace()
            hgemm_lib.reserve_workspace(1 << 20, 1 << 20)


def test_guarded_edges_do_not_write_outside_c(oracle, hgemm_lib, gpu):
    """C sits inside a larger poisoned allocation: nothing before or after it may change."""
    import torch
    for (M, N, K) in [(1000, 1000, 1000), (1000, 4000, 1024), (130, 136, 8192), (100, 100, 100), (1026, 1030, 1100)]:
        A, B = oracle.fill((M, K), 15, 1), oracle.fill((N, K), 15, 2)
        pad = 4096   # elements; keeps C 16-byte aligned
        buf = torch.full((pad + M * N + pad,), POISON - 65536, dtype=torch.int16, device=gpu)
        C = buf[pad:pad + M * N].view(torch.float16).view(M, N)
        print(f"[gpu] hgemm_auto M={M} N={N} K={K} inside a guard band", flush=True)
        hgemm_lib.call("hgemm_auto", _to_gpu(A, gpu), _to_gpu(B, gpu), C, M, N, K)
        torch.cuda.synchronize()
        host = buf.cpu().numpy().view(np.uint16)
        assert np.all(host[:pad] == POISON) and np.all(host[pad + M * N:] == POISON)
        _assert_close(oracle, host[pad:pad + M * N].reshape(M, N), oracle.hgemm(A, B), K)


def test_auto_random_shapes_against_the_vendor_comparator(oracle, hgemm_lib, vendor_lib, gpu):
    """300 seeded shapes over every alignment class the dispatcher distinguishes (tile
    multiples, N % 8, K % 64, K % 8, odd everything; small, tall, wide, deep), each against
    hipBLASLt on the same inputs -- the comparator itself is pinned against the CPU checker
    above.  Both accumulate in fp32 and round once, so they agree to an output ulp; the
    specification's tolerance is asserted, plus bit-identity from run to run."""
    import torch
    rng = np.random.default_rng(20230212)
    grains = [(256, 256, 64), (64, 64, 64), (8, 8, 64), (1, 8, 64), (1, 8, 8), (1, 1, 8), (1, 1, 1)]
    gen = torch.Generator(device=gpu).manual_seed(7)
    checked = 0
    for i in range(300):
        gm, gn, gk = grains[i % len(grains)]
        big = i % 3 == 0
        top = 9000 if (big and gm == 256) else (5000 if big else 700)   # the largest reach grids with a last round
        M = int(rng.integers(1, top // gm + 1)) * gm
        N = int(rng.integers(1, top // gn + 1)) * gn
        K = int(rng.integers(1, (3000 if big else 9000) // gk + 1)) * gk
        if i % 10 == 7:
            M = int(rng.integers(1, 129))                      # decode-like
        A = (torch.rand((M, K), device=gpu, generator=gen) * 2 - 1).half()
        B = (torch.rand((N, K), device=gpu, generator=gen) * 2 - 1).half()
        C = torch.full((M, N), POISON - 65536, dtype=torch.int16, device=gpu).view(torch.float16)
        C2 = torch.full((M, N), POISON - 65536, dtype=torch.int16, device=gpu).view(torch.float16)
        Cv = torch.empty((M, N), dtype=torch.float16, device=gpu)
        plan = hgemm_lib.auto_plan(M, N, K)
        print(f"[gpu] hgemm_auto M={M} N={N} K={K} {plan['kernel']} x{plan['splits']} tail {plan['tail_tiles']}",
              flush=True)
        hgemm_lib.call("hgemm_auto", A, B, C, M, N, K)
        hgemm_lib.call("hgemm_auto", A, B, C2, M, N, K)
        vendor_lib.call(A, B, Cv, M, N, K)
        got, again, ref = _to_bits(C), _to_bits(C2), _to_bits(Cv)
        res = oracle.check(got, ref, K)
        assert res["non_finite"] == 0 and res["ok"], (M, N, K, plan, res)
        assert np.array_equal(got, again), (M, N, K, plan)
        checked += 1
    assert checked == 300


# ------------------------------------------------------------------ size-independent properties at full size
def test_properties_at_8192(oracle, hgemm_lib, gpu):
    import torch
    n = 8192
    A = _to_gpu(oracle.fill((n, n), 77, 1), gpu)
    B = _to_gpu(oracle.fill((n, n), 77, 2), gpu)
    C = torch.empty((n, n), dtype=torch.float16, device=gpu)
    print("[gpu] properties hgemm_auto 8192", flush=True)
    hgemm_lib.call("hgemm_auto", A, B, C, n, n, n)
    base = C.clone()
    # doubling A doubles every product and partial sum exactly (doubling, unlike halving,
    # cannot push an fp16 input or output into the subnormal range and lose a bit)
    hgemm_lib.call("hgemm_auto", A * 2.0, B, C, n, n, n)
    normal = base.abs() >= 2.0 ** -14           # outputs that were rounded on the normal fp16 grid
    assert torch.equal(C[normal], (base * 2.0)[normal])
    # a subnormal output was rounded on a coarser grid than its double: one step of 2^-24 at most
    assert float((C.float() - base.float() * 2.0).abs().max()) <= 2.0 ** -24
    assert int((~normal).sum()) < 1000
    # permuting rows of A permutes rows of C: a row's sum does not depend on where it sits
    perm = torch.randperm(n, device=gpu, generator=torch.Generator(device=gpu).manual_seed(1))
    hgemm_lib.call("hgemm_auto", A[perm].contiguous(), B, C, n, n, n)
    assert torch.equal(C, base[perm])
    # and likewise for rows of B (columns of the K x N operand)
    hgemm_lib.call("hgemm_auto", A, B[perm].contiguous(), C, n, n, n)
    assert torch.equal(C, base[:, perm])
    # swapping the operands transposes the result (A.B^T)^T = B.A^T
    hgemm_lib.call("hgemm_auto", B, A, C, n, n, n)
    assert torch.equal(C, base.t())
    torch.cuda.synchronize()


def test_profile_helper_matches_the_throughput_formula(oracle, hgemm_lib, gpu):
    import torch
    n = 1024
    A = _to_gpu(oracle.fill((n, n), 3, 1), gpu)
    B = _to_gpu(oracle.fill((n, n), 3, 2), gpu)
    C = torch.empty((n, n), dtype=torch.float16, device=gpu)
    ms = hgemm_lib.profile_ms("hgemm_auto", A, B, C, n, n, n, 2, 10)
    assert 0.0 < ms < 50.0
    assert abs(hgemm_lib.tflops(n, n, n, ms) - oracle.tflops(n, n, n, ms)) < 1e-9
    _assert_close(oracle, _to_bits(C), oracle.hgemm(_to_bits(A), _to_bits(B)), n)
