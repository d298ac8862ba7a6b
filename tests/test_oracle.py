"""Pins the CPU checker (oracle/) without a GPU: conversions, seeded inputs, the GEMM and
the metrics, each against something that does not share its code or its formula."""
import json
import os

import numpy as np
import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
GOLDEN = os.path.join(HERE, "golden")


# ------------------------------------------------------------------ fp16 <-> fp32
def test_f16_to_f32_exhaustive_vs_numpy(oracle):
    bits = np.arange(65536, dtype=np.uint16)
    got = oracle.f16_to_f32(bits)
    ref = bits.view(np.float16).astype(np.float32)
    nan = np.isnan(ref)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got.view(np.uint32)[~nan], ref.view(np.uint32)[~nan])


def test_f16_to_f32_exhaustive_vs_hardware(oracle):
    L = oracle.lib()
    if not L.oracle_has_f16c():
        pytest.skip("host has no F16C")
    for b in range(0, 65536):
        sw, hw = L.oracle_f16_to_f32(b), L.oracle_hw_f16_to_f32(b)
        assert (np.isnan(sw) and np.isnan(hw)) or np.float32(sw).view(np.uint32) == np.float32(hw).view(np.uint32), b


def test_f32_to_f16_round_trip_exhaustive(oracle):
    bits = np.arange(65536, dtype=np.uint16)
    f = bits.view(np.float16).astype(np.float32)
    back = oracle.f32_to_f16(f)
    nan = np.isnan(f)
    assert np.array_equal(back[~nan], bits[~nan])
    assert np.all((back[nan] & 0x7C00) == 0x7C00) and np.all((back[nan] & 0x03FF) != 0)


def test_f32_to_f16_ties_and_edges(oracle):
    L = oracle.lib()
    table = [
        (1.0, 0x3C00), (-2.0, 0xC000), (65504.0, 0x7BFF), (65519.996, 0x7BFF), (65520.0, 0x7C00), (1e9, 0x7C00),
        (-1e9, 0xFC00), (2.0 ** -24, 0x0001), (2.0 ** -25, 0x0000),          # tie to even (zero)
        (1.5 * 2.0 ** -24, 0x0002),                                          # tie to even (up)
        (2.0 ** -25 * 1.0000001, 0x0001), (2.0 ** -14, 0x0400), (2.0 ** -14 - 2.0 ** -25, 0x0400),
        (1.0 + 2.0 ** -11, 0x3C00),                                          # tie -> even mantissa
        (1.0 + 3 * 2.0 ** -11, 0x3C02),                                      # tie -> even mantissa (up)
        (1.0 + 2.0 ** -11 + 2.0 ** -20, 0x3C01), (0.0, 0x0000), (-0.0, 0x8000),
        (float("inf"), 0x7C00), (float("-inf"), 0xFC00),
    ]
    for value, bits in table:
        assert L.oracle_f32_to_f16(value) == bits, (value, hex(bits), hex(L.oracle_f32_to_f16(value)))


def test_f32_to_f16_random_vs_numpy_and_hardware(oracle):
    rng = np.random.default_rng(7)
    scale = rng.choice(np.array([1e-8, 1e-5, 1e-3, 1.0, 100.0, 70000.0], np.float32), 400000)
    x = np.concatenate([rng.standard_normal(400000).astype(np.float32) * scale,
                        rng.integers(0, 2 ** 32, 400000, dtype=np.uint64).astype(np.uint32).view(np.float32)])
    x = x[~np.isnan(x)]
    with np.errstate(over="ignore"):
        ref = x.astype(np.float16).view(np.uint16)
    assert np.array_equal(oracle.f32_to_f16(x), ref)
    L = oracle.lib()
    if L.oracle_has_f16c():
        for v in x[:20000]:
            assert L.oracle_f32_to_f16(float(v)) == L.oracle_hw_f32_to_f16(float(v)), v


# ------------------------------------------------------------------ seeded inputs
def test_rng_fixture(oracle):
    fx = json.load(open(os.path.join(GOLDEN, "rng_first_values.json")))
    for case in fx["cases"]:
        got = oracle.fill((16,), fx["seed"], case["stream"], case["dist"], case["p0"], case["p1"])
        assert [int(v) for v in got] == case["first16"], case["name"]


def test_rng_is_counter_based(oracle):
    whole = oracle.fill((4, 100), 5, 1)
    assert np.array_equal(whole.reshape(-1)[:137], oracle.fill((137,), 5, 1))       # prefix independent of size
    assert not np.array_equal(oracle.fill((64,), 5, 1), oracle.fill((64,), 5, 2))   # streams differ
    assert not np.array_equal(oracle.fill((64,), 5, 1), oracle.fill((64,), 6, 1))   # seeds differ


def test_rng_distributions(oracle):
    n = 1 << 20
    u = oracle.fill((n,), 1, 1).view(np.float16).astype(np.float64)
    assert u.min() >= -1.0 and u.max() <= 1.0
    assert abs(u.mean()) < 3e-3 and abs(u.var() - 1.0 / 3.0) < 3e-3
    g = oracle.fill((n,), 1, 2, oracle.NORMAL, 0.0, 1.0).view(np.float16).astype(np.float64)
    assert abs(g.mean()) < 4e-3 and abs(g.std() - 1.0) < 4e-3
    assert abs(np.mean(np.abs(g) < 1.0) - 0.6827) < 3e-3
    w = oracle.fill((n,), 1, 2, oracle.NORMAL, 0.0, 0.02).view(np.float16).astype(np.float64)
    assert abs(w.std() - 0.02) < 2e-4
    t = oracle.fill((n,), 1, 3, oracle.TERNARY, 0.0, 1.0).view(np.float16).astype(np.float64)
    assert set(np.unique(t)) == {-1.0, 0.0, 1.0}
    assert all(abs(np.mean(t == v) - 1 / 3) < 3e-3 for v in (-1.0, 0.0, 1.0))


# ------------------------------------------------------------------ GEMM
def _f16(x):
    return np.asarray(x, np.float16).view(np.uint16)


@pytest.mark.parametrize("shape", [(64, 96, 128), (37, 53, 71), (1, 130, 1000), (130, 1, 515), (128, 128, 2048)])
def test_exact_integer_inputs_any_order_is_exact(oracle, shape):
    """Entries in {-1,0,1} and K <= 2048: every partial sum is an integer below 2^24 and
    the result is at most 2048 in magnitude, so fp32 accumulation in ANY order and the fp16
    rounding are exact -- the blocked routine must equal the integer product bit for bit."""
    M, N, K = shape
    A = oracle.fill((M, K), 11, 1, oracle.TERNARY, 0, 1)
    B = oracle.fill((N, K), 11, 2, oracle.TERNARY, 0, 1)
    ref = A.view(np.float16).astype(np.int64) @ B.view(np.float16).astype(np.int64).T
    C = oracle.hgemm(A, B)
    assert np.array_equal(C.view(np.float16).astype(np.int64), ref)
    assert np.array_equal(oracle.hgemm_naive_f32(A, B), C)
    assert np.array_equal(oracle.hgemm_naive_f64(A, B)[0], C)


@pytest.mark.parametrize("K", [1, 8, 64, 512, 4096, 32768])
def test_all_ones_gives_K(oracle, K):
    A, B = _f16(np.ones((5, K))), _f16(np.ones((7, K)))
    assert np.all(oracle.hgemm(A, B).view(np.float16) == np.float16(K))


def test_identity_pins_the_layout_of_B(oracle):
    """A = I (M = K): C[m][n] = B[n*K + m].  A transposed or row-major-KxN reading of B
    fails this; so does swapping the roles of M and N."""
    K, N = 48, 20
    A = _f16(np.eye(K))
    B = oracle.fill((N, K), 3, 2)
    C = oracle.hgemm(A, B)
    assert np.array_equal(C, B.T)
    # B = I (N = K): C = A
    A2 = oracle.fill((9, K), 3, 1)
    assert np.array_equal(oracle.hgemm(A2, _f16(np.eye(K))), A2)


def test_one_hot_probe_touches_one_output(oracle):
    M, N, K = 19, 23, 40
    A = np.zeros((M, K), np.float16)
    B = np.zeros((N, K), np.float16)
    A[5, 17] = 2.0
    B[11, 17] = 3.0
    C = oracle.hgemm(_f16(A), _f16(B)).view(np.float16)
    expect = np.zeros((M, N), np.float16)
    expect[5, 11] = 6.0
    assert np.array_equal(C, expect)


@pytest.mark.parametrize("shape", [(16, 16, 16), (33, 47, 61), (64, 64, 64), (5, 70, 300), (70, 3, 1025)])
def test_blocked_matches_brute_force_double(oracle, shape):
    M, N, K = shape
    A, B = oracle.fill((M, K), 21, 1), oracle.fill((N, K), 21, 2)
    C, Cf = oracle.hgemm(A, B, want_f32=True)
    Cn, Cd = oracle.hgemm_naive_f64(A, B)
    # fp32 accumulation error bound: K * eps32 * sum|a||b| is far below this
    assert np.max(np.abs(Cf - Cd)) <= 1e-5 * np.sqrt(K) + 1e-6
    # rounded results may differ from the double-rounded ones only by one fp16 ulp, rarely
    diff = oracle.diff(C, Cn)
    assert diff["max_diff"] <= np.spacing(np.float16(np.abs(Cd).max())) and np.mean(C != Cn) < 0.01


@pytest.mark.parametrize("name", ["gemm_32x32x64", "gemm_48x80x96", "gemm_1x128x256", "gemm_64x64x1024"])
def test_numpy_float64_golden_vectors(oracle, name):
    z = np.load(os.path.join(GOLDEN, name + ".npz"))
    C, Cf = oracle.hgemm(z["A"], z["B"], want_f32=True)
    K = z["A"].shape[1]
    assert np.max(np.abs(Cf - z["C_f64"])) <= 1e-5 * np.sqrt(K)
    res = oracle.check(C, z["C"], K)
    assert res["ok"] and res["max_diff"] <= np.spacing(np.float16(np.abs(z["C_f64"]).max()))
    assert np.mean(C != z["C"]) < 0.01


def test_linearity_and_row_permutation(oracle):
    M, N, K = 24, 40, 256
    A, B = oracle.fill((M, K), 31, 1), oracle.fill((N, K), 31, 2)
    # scaling A by a power of two scales C exactly
    A2 = _f16(A.view(np.float16).astype(np.float32) * 0.5)
    C1 = oracle.hgemm(A, B).view(np.float16).astype(np.float32)
    C2 = oracle.hgemm(A2, B).view(np.float16).astype(np.float32)
    assert np.array_equal(C2, C1 * 0.5)
    # permuting the rows of A permutes the rows of C
    perm = np.random.default_rng(0).permutation(M)
    assert np.array_equal(oracle.hgemm(A[perm], B), oracle.hgemm(A, B)[perm])
    # permuting the rows of B (columns of the K x N matrix) permutes the columns of C
    permn = np.random.default_rng(1).permutation(N)
    assert np.array_equal(oracle.hgemm(A, B[permn]), oracle.hgemm(A, B)[:, permn])


def test_rows_sampling_equals_full(oracle):
    A, B = oracle.fill((40, 128), 41, 1), oracle.fill((24, 128), 41, 2)
    full = oracle.hgemm(A, B)
    assert np.array_equal(oracle.hgemm_rows(A, B, 8, 16), full[8:24])


# ------------------------------------------------------------------ metrics
def test_diff_and_tolerance(oracle):
    a = _f16([1.0, 2.0, 3.0, 4.0])
    b = _f16([1.0, 2.5, 3.0, 2.0])
    d = oracle.diff(a, b)
    assert d["max_diff"] == 2.0 and d["avg_diff"] == 2.5 / 4 and d["argmax"] == 3 and d["non_finite"] == 0
    assert abs(d["ref_rms"] - np.sqrt((1 + 6.25 + 9 + 4) / 4)) < 1e-12
    nan = np.array([0x7E00, 0x3C00], np.uint16)
    assert oracle.diff(nan, _f16([1.0, 1.0]))["non_finite"] == 1
    assert oracle.tolerance(256) == 1e-2 and abs(oracle.tolerance(8192) - 1e-2 * np.sqrt(32)) < 1e-15
    assert not oracle.check(nan, _f16([1.0, 1.0]), 256)["ok"]


def test_tflops_formula(oracle):
    # 2*M*N*K*1e-12 / (ms*1e-3): 8192^3 in 0.583 ms is 75 % of 2.5 PFLOPS
    assert abs(oracle.tflops(8192, 8192, 8192, 1.0) - 1099.511627776) < 1e-9
    assert abs(oracle.tflops(8192, 8192, 8192, 0.5831) / 2500 - 0.754) < 2e-3
    assert oracle.tflops(512, 2048, 1024, 2.0) == 2 * 512 * 2048 * 1024 * 1e-12 / 2e-3
