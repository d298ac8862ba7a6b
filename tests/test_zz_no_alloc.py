"""hgemm_auto_static_workspace: the entry point that allocates nothing.  Called through the C
ABI twice in a row, the second time on a smaller input, and compared bit for bit with
hgemm_auto (which runs the same plan on the heap workspace); both against the CPU checker."""
import ctypes

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

POISON = 0xFFFF


def _to_gpu(bits, gpu):
    import torch
    return torch.from_numpy(np.ascontiguousarray(bits).view(np.int16)).to(gpu).view(torch.float16)


def _bits(t):
    import torch
    torch.cuda.synchronize()
    return t.view(torch.int16).cpu().numpy().view(np.uint16)


def _call(lib, symbol, A, B, M, N, K, gpu):
    import torch
    C = torch.full((M, N), POISON - 65536, dtype=torch.int16, device=gpu).view(torch.float16)
    fn = getattr(lib.dll, symbol)
    print(f"[gpu] {symbol} M={M} N={N} K={K}", flush=True)
    rc = fn(ctypes.c_void_p(A.data_ptr()), ctypes.c_void_p(B.data_ptr()), ctypes.c_void_p(C.data_ptr()), M, N, K)
    return rc, _bits(C)


# each pair: a shape whose plan keeps partial sums or padded operands in the workspace, then a smaller one
PAIRS = [((1024, 1024, 8192), (256, 256, 8192)),          # K slices on 128x128 tiles, then on 64x64 tiles
         ((7168, 7168, 2048), (64, 4096, 4096)),          # (no workspace: last round on smaller tiles), split-K small-M kernel
         ((7168, 7168, 7168), (512, 512, 8192)),          # last round of a large grid in K slices
         ((1111, 1111, 1111), (515, 1032, 1100)),         # zero-padded operand copies
         ((2048, 2048, 16384), (16, 4096, 4096))]         # partial sums that fill the array to its last byte


@pytest.mark.parametrize("first,second", PAIRS)
def test_static_workspace_matches_heap_workspace(oracle, hgemm_lib, gpu, first, second):
    limit = hgemm_lib.static_workspace_bytes()
    used_scratch = False
    for (M, N, K) in (first, second):
        need = hgemm_lib.auto_workspace_bytes(M, N, K)
        assert need["partial"] + need["operands"] <= limit, (M, N, K, need)
        used_scratch |= need["partial"] + need["operands"] > 0
        A = oracle.fill((M, K), 91, 1, oracle.TERNARY, 0, 1)
        B = oracle.fill((N, K), 91, 2, oracle.TERNARY, 0, 1)
        Ad, Bd = _to_gpu(A, gpu), _to_gpu(B, gpu)
        rc, got = _call(hgemm_lib, "hgemm_auto_static_workspace", Ad, Bd, M, N, K, gpu)
        assert rc == 0
        _, ref = _call(hgemm_lib, "hgemm_auto", Ad, Bd, M, N, K, gpu)
        assert np.array_equal(got, ref), (M, N, K)
        if M * N * K <= 2048 * 2048 * 16384:
            exact = oracle.hgemm(A, B)
        else:
            exact = None
            for m0 in (0, M // 2 + 3, M - 8):
                assert np.array_equal(got[m0:m0 + 8], oracle.hgemm_rows(A, B, m0, 8)), (M, N, K, m0)
        if exact is not None:      # integer sums below 2^24 are exact in fp32 under any order, then rounded once
            assert np.array_equal(got, exact), (M, N, K)
        # random inputs: same plan, same order of additions, so bit-identical again
        A = oracle.fill((M, K), 92, 1)
        B = oracle.fill((N, K), 92, 2)
        Ad, Bd = _to_gpu(A, gpu), _to_gpu(B, gpu)
        rc, got = _call(hgemm_lib, "hgemm_auto_static_workspace", Ad, Bd, M, N, K, gpu)
        _, ref = _call(hgemm_lib, "hgemm_auto", Ad, Bd, M, N, K, gpu)
        assert rc == 0 and np.array_equal(got, ref), (M, N, K)
    assert used_scratch


def test_static_workspace_allocates_nothing_and_rejects_what_does_not_fit(oracle, hgemm_lib, gpu):
    import torch
    M, N, K = 1024, 1024, 8192
    assert hgemm_lib.auto_workspace_bytes(M, N, K)["partial"] > 0
    A, B = _to_gpu(oracle.fill((M, K), 93, 1), gpu), _to_gpu(oracle.fill((N, K), 93, 2), gpu)
    _call(hgemm_lib, "hgemm_auto_static_workspace", A, B, M, N, K, gpu)        # code object and scratch are resident now
    hgemm_lib.release_workspace()
    C = torch.empty((M, N), dtype=torch.float16, device=gpu)
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    for _ in range(3):
        rc = hgemm_lib.dll.hgemm_auto_static_workspace(ctypes.c_void_p(A.data_ptr()), ctypes.c_void_p(B.data_ptr()),
                                                       ctypes.c_void_p(C.data_ptr()), M, N, K)
        assert rc == 0
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before, "device memory was allocated"
    # a plan that needs more than the static array holds: refused with a message, nothing launched
    M, N, K = 4095, 4095, 4095
    need = hgemm_lib.auto_workspace_bytes(M, N, K)
    assert need["partial"] + need["operands"] > hgemm_lib.static_workspace_bytes()
    A = torch.zeros((M, K), dtype=torch.float16, device=gpu)
    B = torch.zeros((N, K), dtype=torch.float16, device=gpu)
    rc, got = _call(hgemm_lib, "hgemm_auto_static_workspace", A, B, M, N, K, gpu)
    assert rc == 1 and np.all(got == POISON)
