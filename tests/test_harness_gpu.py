"""The parts of the C ABI around the kernels, on a real MI355X: calls from several host threads
that share the K-slice workspace, the shader-clock marks, the vendor comparator's choice among
hipBLASLt's candidate kernels, and device buffers that do not come from PyTorch."""
import threading

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _to_gpu(bits, gpu):
    import torch
    return torch.from_numpy(np.ascontiguousarray(bits).view(np.int16)).to(gpu).view(torch.float16)


def _to_bits(t):
    import torch
    torch.cuda.synchronize()
    return t.view(torch.int16).cpu().numpy().view(np.uint16)


def test_two_host_threads_share_the_workspace(oracle, hgemm_lib, gpu):
    """Both shapes run in K slices, i.e. keep fp32 partial sums in the one workspace the device has.  Two threads
    call hgemm_auto at the same time, 40 calls each into 40 output buffers; every output must equal what the same
    call gives alone, bit for bit (the reference keeps its one cuBLAS handle in a function-local static the same
    way, src/cublas_tensor_op.cu:18, and exercises no concurrency at all)."""
    import torch
    shapes = [(64, 4096, 4096), (512, 512, 8192)]
    calls = 40
    work = []
    for t, (M, N, K) in enumerate(shapes):
        plan = hgemm_lib.auto_plan(M, N, K)
        assert plan["splits"] > 1 and hgemm_lib.auto_workspace_bytes(M, N, K)["partial"] > 0, (M, N, K, plan)
        A = oracle.fill((M, K), 77 + t, 1, oracle.TERNARY, 0, 1)
        B = oracle.fill((N, K), 77 + t, 2, oracle.TERNARY, 0, 1)
        Ad, Bd = _to_gpu(A, gpu), _to_gpu(B, gpu)
        alone = torch.full((M, N), float("nan"), dtype=torch.float16, device=gpu)
        print(f"[gpu] hgemm_auto alone M={M} N={N} K={K}", flush=True)
        hgemm_lib.call("hgemm_auto", Ad, Bd, alone, M, N, K)
        expect = _to_bits(alone)
        assert np.array_equal(expect, oracle.hgemm(A, B))       # ternary inputs: exact under any order
        outs = [torch.full((M, N), float("nan"), dtype=torch.float16, device=gpu) for _ in range(calls)]
        work.append((M, N, K, Ad, Bd, outs, expect))
    torch.cuda.synchronize()
    start = threading.Barrier(len(work))
    errors = []

    def caller(M, N, K, Ad, Bd, outs, _expect):
        try:
            fn = hgemm_lib.fn("hgemm_auto")
            start.wait()
            for out in outs:                                     # ctypes releases the GIL for the call
                fn(Ad.data_ptr(), Bd.data_ptr(), out.data_ptr(), M, N, K)
        except Exception as exc:                                 # pragma: no cover
            errors.append(exc)

    print("[gpu] hgemm_auto from two host threads", flush=True)
    threads = [threading.Thread(target=caller, args=w) for w in work]
    for th in threads:
        th.start()
    for th in threads:
        th.join(timeout=100)
        assert not th.is_alive()
    assert not errors, errors
    torch.cuda.synchronize()
    for (M, N, K, _a, _b, outs, expect) in work:
        for i, out in enumerate(outs):
            assert np.array_equal(_to_bits(out), expect), (M, N, K, i)


def test_shader_clock_between_marks(oracle, hgemm_lib, gpu):
    """Two samples of (shader cycles, constant-rate ticks) per SIMD bracket 30 launches at 4096^3: every XCD is
    sampled, the clock lies in the part's range and the SIMDs agree; the elapsed time by the constant-rate counter
    agrees with the HIP events of the same launches."""
    import torch
    n = 4096
    A, B = _to_gpu(oracle.fill((n, n), 3, 1), gpu), _to_gpu(oracle.fill((n, n), 3, 2), gpu)
    C = torch.empty((n, n), dtype=torch.float16, device=gpu)
    hgemm_lib.profile_ms("hgemm_auto", A, B, C, n, n, n, 5, 5)
    print("[gpu] clock marks around 30 launches of hgemm_auto 4096^3", flush=True)
    hgemm_lib.clock_mark(0)
    ms = hgemm_lib.profile_ms("hgemm_auto", A, B, C, n, n, n, 0, 30) * 30
    hgemm_lib.clock_mark(1)
    clk = hgemm_lib.clock_between_marks()
    sampled = [m for m in clk["per_xcd_mhz"] if m > 0]
    assert len(sampled) == 8, clk
    assert 500.0 < clk["mhz"] < 2600.0, clk
    assert clk["simds"] >= 256, clk
    # every XCD manages its own clock (they differ by several per cent under load); a SIMD whose samples were not a
    # pair from one counter would be off by a multiple of the clock, not by per cents
    assert clk["max_mhz"] - clk["min_mhz"] < 0.25 * clk["mhz"], clk
    assert min(sampled) >= clk["min_mhz"] - 1e-6 and max(sampled) <= clk["max_mhz"] + 1e-6, clk
    assert ms <= clk["elapsed_ms"] < ms + 1.0, (ms, clk)     # the marks sit just outside the event pair
    flops_per_cycle_cu = 2.0 * n ** 3 * 30 / (clk["elapsed_ms"] * 1e-3) / (clk["mhz"] * 1e6) / 256
    assert 0.0 < flops_per_cycle_cu < 4096.0, flops_per_cycle_cu


def test_vendor_comparator_keeps_the_fastest_candidate(oracle, vendor_lib, gpu):
    import torch
    M, N, K = 256, 1024, 1024
    assert vendor_lib.candidates(M, N, K + 64)["candidates"] == 0        # never called
    A, B = oracle.fill((M, K), 5, 1), oracle.fill((N, K), 5, 2)
    C = torch.full((M, N), float("nan"), dtype=torch.float16, device=gpu)
    print(f"[gpu] hgemm_hipblaslt M={M} N={N} K={K}", flush=True)
    vendor_lib.call(_to_gpu(A, gpu), _to_gpu(B, gpu), C, M, N, K)
    res = oracle.check(_to_bits(C), oracle.hgemm(A, B), K)
    assert res["ok"] and res["non_finite"] == 0, res
    pick = vendor_lib.candidates(M, N, K)
    assert 1 <= pick["candidates"] <= 16 and 0 <= pick["chosen"] < pick["candidates"], pick
    assert 0.0 < pick["chosen_ms"] <= pick["first_ms"] or pick["first_ms"] == 0.0, pick
    assert "hipblaslt" in vendor_lib.loaded_from().lower()


def test_device_buffers_without_torch(oracle, hgemm_lib, gpu):
    """hipmem.DeviceArray (what the benchmark allocates with) round-trips bits and is accepted as an operand:
    same result as with torch tensors."""
    import torch
    from cuda_hgemm_amd import hipmem
    M, N, K = 192, 320, 512
    A, B = oracle.fill((M, K), 11, 1), oracle.fill((N, K), 11, 2)
    Ad, Bd = hipmem.DeviceArray.from_host(A), hipmem.DeviceArray.from_host(B)
    assert np.array_equal(Ad.to_host(), A) and np.array_equal(Bd.to_host(), B)
    Cd = hipmem.DeviceArray((M, N)).fill_bytes(0xFF)
    assert np.all(Cd.to_host() == 0xFFFF)
    print(f"[gpu] hgemm_auto on hipmem buffers M={M} N={N} K={K}", flush=True)
    hgemm_lib.call("hgemm_auto", Ad, Bd, Cd, M, N, K)
    Ct = torch.full((M, N), float("nan"), dtype=torch.float16, device=gpu)
    hgemm_lib.call("hgemm_auto", _to_gpu(A, gpu), _to_gpu(B, gpu), Ct, M, N, K)
    got = Cd.to_host()
    assert np.array_equal(got, _to_bits(Ct))
    assert oracle.check(got, oracle.hgemm(A, B), K)["ok"]
    assert hipmem.compute_units() == torch.cuda.get_device_properties(0).multi_processor_count
    with pytest.raises(ValueError):
        hgemm_lib.call("hgemm_auto", Ad, Bd, Cd, M, N + 8, K)
    for buf in (Ad, Bd, Cd):
        buf.free()
    with pytest.raises(ValueError):
        hgemm_lib.call("hgemm_auto", Ad, Bd, Cd, M, N, K)


@pytest.mark.parametrize("shape", [(384, 6144, 5120), (64, 4096, 4096), (16, 28672, 4096), (1000, 4000, 4096),
                                   (100, 100, 100)])
def test_tuning_on_the_callers_operands(oracle, hgemm_lib, gpu, shape):
    """hgemm_auto_tune times the model's best plans for a shape and keeps the fastest: the kept plan is one of those
    hgemm_auto_tune_plans lists, the plan queries report it, C holds its product (within the tolerance of the
    specification: plans that slice K differently differ in the last bit), hgemm_auto then reproduces C bit for bit,
    and forgetting the tuning brings the model's plan back.  A shape with nothing to choose from (no tile divides
    it) times one plan."""
    import torch
    M, N, K = shape
    hgemm_lib.forget_tuning()
    model_plan = hgemm_lib.auto_plan(M, N, K)
    listed = hgemm_lib.tune_plans(M, N, K, 6)
    assert 1 <= len(listed) <= 6 and listed[0]["kernel_id"] == model_plan["kernel_id"] and listed[0]["splits"] == model_plan["splits"]
    A = oracle.fill((M, K), 91, 1, oracle.NORMAL, 0.0, 1.0)
    B = oracle.fill((N, K), 91, 2, oracle.NORMAL, 0.0, 0.02)
    Ad, Bd = _to_gpu(A, gpu), _to_gpu(B, gpu)
    C = torch.full((M, N), float("nan"), dtype=torch.float16, device=gpu)
    try:
        print(f"[gpu] hgemm_auto_tune M={M} N={N} K={K}", flush=True)
        timed = hgemm_lib.tune(Ad, Bd, C, M, N, K, 6, cold=(M % 2 == 0 and N == 4096))
        assert 1 <= timed <= len(listed) and hgemm_lib.plan_is_tuned(M, N, K)
        if shape == (100, 100, 100):
            assert timed == 1
        results = hgemm_lib.tune_results()
        assert len(results) == timed and sum(r["kept"] for r in results) == 1 and all(r["ms"] > 0 for r in results), results
        kept = hgemm_lib.auto_plan(M, N, K)
        assert [r for r in results if r["kept"]][0]["kernel_id"] == kept["kernel_id"]
        assert any(kept["kernel_id"] == p["kernel_id"] and kept["splits"] == p["splits"] for p in listed), (kept, listed)
        tuned_bits = _to_bits(C)
        res = oracle.check(tuned_bits, oracle.hgemm(A, B), K)
        assert res["ok"] and res["non_finite"] == 0, res
        again = torch.full((M, N), float("nan"), dtype=torch.float16, device=gpu)
        print(f"[gpu] hgemm_auto (tuned) M={M} N={N} K={K}", flush=True)
        hgemm_lib.call("hgemm_auto", Ad, Bd, again, M, N, K)
        assert np.array_equal(_to_bits(again), tuned_bits)
    finally:
        hgemm_lib.forget_tuning()
    assert not hgemm_lib.plan_is_tuned(M, N, K) and hgemm_lib.auto_plan(M, N, K) == model_plan
