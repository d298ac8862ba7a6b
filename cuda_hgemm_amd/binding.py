"""ctypes binding of ``include/hgemm.h`` / ``include/hgemm_hipblaslt.h``.

Operand layouts are the reference's (``src/common/tester.h:117-120``): ``A`` is ``(M, K)``
row-major, ``B`` is handed over as its ``(N, K)`` storage (column-major ``K x N``), ``C`` is
``(M, N)`` row-major; all fp16, all on the GPU.  Calls are asynchronous on the null stream,
which is also torch's default stream.  Operands are torch CUDA tensors or
``cuda_hgemm_amd.hipmem.DeviceArray`` buffers (device memory without torch).
"""
from __future__ import annotations

import ctypes as C
import os
import sys
from typing import List, Optional

_HERE = os.path.dirname(os.path.abspath(__file__))


def lib_path() -> str:
    return os.path.join(_HERE, "lib", "libhgemm.so")


def vendor_lib_path() -> str:
    return os.path.join(_HERE, "lib", "libhgemm_hipblaslt.so")


def driver_path() -> str:
    return os.path.join(_HERE, "bin", "hgemm")


_SZ = C.c_size_t
_PTR = C.c_void_p
_HGEMM_ARGS = [_PTR, _PTR, _PTR, _SZ, _SZ, _SZ]
HGEMM_FN = C.CFUNCTYPE(None, *_HGEMM_ARGS)

# every symbol include/hgemm.h declares
KERNEL_SYMBOLS = [
    "hgemm_simt_naive", "hgemm_mfma_naive", "hgemm_mfma_base", "hgemm_mfma_padding", "hgemm_mfma_swizzle",
    "hgemm_mfma_async", "hgemm_mfma_async_pg2s", "hgemm_mfma_async_pg2s_ps2r", "hgemm_mfma_async_stage2",
    "hgemm_mfma_async_stage3", "hgemm_mfma_async_stage4", "hgemm_mfma_tiled_64x64", "hgemm_mfma_pipelined_64x64",
    "hgemm_mfma_pipelined_128x128", "hgemm_mfma_pipelined_192x192", "hgemm_mfma_pipelined_256x128",
    "hgemm_mfma_pipelined_256x256", "hgemm_mfma_chained_192x192", "hgemm_mfma_chained_256x128",
    "hgemm_mfma_chained_256x256", "hgemm_skinny", "hgemm_auto",
]
HELPER_SYMBOLS = [
    "hgemm_auto_plan", "hgemm_auto_plan_tail", "hgemm_auto_plan_tail_kernel", "hgemm_auto_plan_chained", "hgemm_kernel_name",
    "hgemm_small_m_rule", "hgemm_variant_count", "hgemm_variant_name", "hgemm_variant_symbol",
    "hgemm_variant_fn", "hgemm_variant_find", "hgemm_variant_supports", "hgemm_variant_in_default_run",
    "hgemm_profile_ms", "hgemm_profile_rotating_ms", "hgemm_clock_mark", "hgemm_clock_between_marks_mhz",
    "hgemm_tflops", "hgemm_bytes", "hgemm_version",
    "hgemm_reserve_workspace", "hgemm_release_workspace", "hgemm_auto_workspace_bytes",
    "hgemm_auto_static_workspace", "hgemm_static_workspace_bytes",
    "hgemm_auto_tune", "hgemm_auto_tune_plans", "hgemm_auto_tune_result", "hgemm_auto_forget_tuning", "hgemm_auto_plan_is_tuned",
]


VENDOR_SYMBOLS = ["hgemm_hipblaslt", "hgemm_hipblaslt_candidates", "hgemm_hipblaslt_loaded_from"]


def _share_hip_runtime_with_torch() -> None:
    """PyTorch wheels carry their own libamdhip64 (same soname as the system one).  Two HIP
    runtimes in one process do not share devices or memory, so torch must be loaded first:
    the dynamic linker then resolves this library's libamdhip64 dependency to the copy that
    is already mapped, and tensors and kernels live in one runtime."""
    try:
        import torch  # noqa: F401
    except ImportError:
        pass  # a caller without torch brings its own device pointers and the system runtime


def _tensor_ptr(t, rows: int, cols: int, what: str) -> int:
    from .hipmem import DeviceArray
    if isinstance(t, DeviceArray):
        if tuple(t.shape) != (rows, cols):
            raise ValueError(f"{what}: expected shape {(rows, cols)}, got {tuple(t.shape)}")
        if not t.ptr:
            raise ValueError(f"{what}: the buffer has been freed")
        return t.ptr
    import torch
    if not isinstance(t, torch.Tensor):
        raise TypeError(f"{what}: expected a torch.Tensor or a hipmem.DeviceArray, got {type(t).__name__}")
    if t.dtype != torch.float16:
        raise TypeError(f"{what}: expected float16, got {t.dtype}")
    if not t.is_cuda:
        raise ValueError(f"{what}: must live on the GPU")
    if tuple(t.shape) != (rows, cols):
        raise ValueError(f"{what}: expected shape {(rows, cols)}, got {tuple(t.shape)}")
    if not t.is_contiguous():
        raise ValueError(f"{what}: must be contiguous")
    if t.data_ptr() % 16:
        raise ValueError(f"{what}: must start on a 16-byte boundary")
    return t.data_ptr()


class HgemmLibrary:
    """``libhgemm.so`` loaded through ctypes; fails loudly when it has not been built."""

    def __init__(self, path: Optional[str] = None, torch_runtime: bool = True):
        """``torch_runtime=False``: do not import torch first, i.e. run on the system's ROCm
        libraries (operands are then ``hipmem.DeviceArray`` buffers; importing torch later in
        such a process would hand torch a runtime it was not built with)."""
        self.path = path or lib_path()
        if not os.path.exists(self.path):
            raise FileNotFoundError(
                f"{self.path} is missing: build it with `python -m cuda_hgemm_amd.build` (needs hipcc); "
                "there is no non-HIP fallback")
        if torch_runtime:
            _share_hip_runtime_with_torch()
        self.dll = C.CDLL(self.path)
        d = self.dll
        for name in KERNEL_SYMBOLS:
            fn = getattr(d, name)
            fn.argtypes, fn.restype = _HGEMM_ARGS, None
        d.hgemm_auto_plan.argtypes, d.hgemm_auto_plan.restype = [_SZ, _SZ, _SZ, C.POINTER(C.c_int)], C.c_int
        d.hgemm_auto_plan_tail.argtypes, d.hgemm_auto_plan_tail.restype = [_SZ, _SZ, _SZ, C.POINTER(C.c_int)], C.c_int
        d.hgemm_auto_plan_tail_kernel.argtypes, d.hgemm_auto_plan_tail_kernel.restype = [_SZ, _SZ, _SZ], C.c_int
        d.hgemm_auto_plan_chained.argtypes, d.hgemm_auto_plan_chained.restype = [_SZ, _SZ, _SZ], C.c_int
        d.hgemm_kernel_name.argtypes, d.hgemm_kernel_name.restype = [C.c_int], C.c_char_p
        d.hgemm_auto_tune.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, _SZ, _SZ, _SZ, C.c_int, C.c_int]
        d.hgemm_auto_tune.restype = C.c_int
        d.hgemm_auto_tune_plans.argtypes = [_SZ, _SZ, _SZ, C.c_int, C.POINTER(C.c_int), C.POINTER(C.c_int)]
        d.hgemm_auto_tune_plans.restype = C.c_int
        d.hgemm_auto_tune_result.argtypes = [C.c_int, C.POINTER(C.c_int), C.POINTER(C.c_int), C.POINTER(C.c_float), C.POINTER(C.c_int)]
        d.hgemm_auto_tune_result.restype = C.c_int
        d.hgemm_auto_forget_tuning.argtypes, d.hgemm_auto_forget_tuning.restype = [], None
        d.hgemm_auto_plan_is_tuned.argtypes, d.hgemm_auto_plan_is_tuned.restype = [_SZ, _SZ, _SZ], C.c_int
        d.hgemm_small_m_rule.argtypes = [C.c_int, C.POINTER(_SZ), C.POINTER(C.c_int)]
        d.hgemm_small_m_rule.restype = C.c_int
        d.hgemm_variant_count.argtypes, d.hgemm_variant_count.restype = [], C.c_int
        d.hgemm_variant_name.argtypes, d.hgemm_variant_name.restype = [C.c_int], C.c_char_p
        d.hgemm_variant_symbol.argtypes, d.hgemm_variant_symbol.restype = [C.c_int], C.c_char_p
        d.hgemm_variant_fn.argtypes, d.hgemm_variant_fn.restype = [C.c_int], HGEMM_FN
        d.hgemm_variant_find.argtypes, d.hgemm_variant_find.restype = [C.c_char_p], C.c_int
        d.hgemm_variant_supports.argtypes, d.hgemm_variant_supports.restype = [C.c_int, _SZ, _SZ, _SZ], C.c_int
        d.hgemm_variant_in_default_run.argtypes, d.hgemm_variant_in_default_run.restype = [C.c_int], C.c_int
        d.hgemm_profile_ms.argtypes = [HGEMM_FN, _PTR, _PTR, _PTR, _SZ, _SZ, _SZ, _SZ, _SZ]
        d.hgemm_profile_ms.restype = C.c_double
        d.hgemm_profile_rotating_ms.argtypes = [HGEMM_FN, C.POINTER(_PTR), C.POINTER(_PTR), C.POINTER(_PTR), _SZ, _SZ,
                                                _SZ, _SZ, _SZ, _SZ]
        d.hgemm_profile_rotating_ms.restype = C.c_double
        d.hgemm_clock_mark.argtypes, d.hgemm_clock_mark.restype = [C.c_int], None
        d.hgemm_clock_between_marks_mhz.argtypes = [C.POINTER(C.c_double), C.c_int, C.POINTER(C.c_double),
                                                    C.POINTER(C.c_double)]
        d.hgemm_clock_between_marks_mhz.restype = C.c_double
        d.hgemm_tflops.argtypes, d.hgemm_tflops.restype = [_SZ, _SZ, _SZ, C.c_double], C.c_double
        d.hgemm_bytes.argtypes, d.hgemm_bytes.restype = [_SZ, _SZ, _SZ], C.c_double
        d.hgemm_version.argtypes, d.hgemm_version.restype = [], C.c_char_p
        d.hgemm_reserve_workspace.argtypes, d.hgemm_reserve_workspace.restype = [_SZ, _SZ], C.c_int
        d.hgemm_release_workspace.argtypes, d.hgemm_release_workspace.restype = [], None
        d.hgemm_auto_workspace_bytes.argtypes = [_SZ, _SZ, _SZ, C.POINTER(_SZ)]
        d.hgemm_auto_workspace_bytes.restype = _SZ
        d.hgemm_auto_static_workspace.argtypes, d.hgemm_auto_static_workspace.restype = _HGEMM_ARGS, C.c_int
        d.hgemm_static_workspace_bytes.argtypes, d.hgemm_static_workspace_bytes.restype = [], _SZ

    # ---- registry -------------------------------------------------------------------
    def variants(self) -> List[dict]:
        out = []
        for i in range(self.dll.hgemm_variant_count()):
            out.append({"index": i, "name": self.dll.hgemm_variant_name(i).decode(),
                        "symbol": self.dll.hgemm_variant_symbol(i).decode(),
                        "default_run": bool(self.dll.hgemm_variant_in_default_run(i))})
        return out

    def find(self, name: str) -> int:
        idx = self.dll.hgemm_variant_find(name.encode())
        if idx < 0:
            raise KeyError(f"unknown hgemm variant {name!r}")
        return idx

    def supports(self, name: str, M: int, N: int, K: int) -> bool:
        return bool(self.dll.hgemm_variant_supports(self.find(name), M, N, K))

    def auto_plan(self, M: int, N: int, K: int) -> dict:
        splits = C.c_int(0)
        kernel = self.dll.hgemm_auto_plan(M, N, K, C.byref(splits))
        tail_splits = C.c_int(1)
        tail_tiles = self.dll.hgemm_auto_plan_tail(M, N, K, C.byref(tail_splits))
        return {"kernel_id": kernel, "kernel": self.dll.hgemm_kernel_name(kernel).decode(), "splits": splits.value,
                "chained": bool(self.dll.hgemm_auto_plan_chained(M, N, K)),
                "tail_tiles": tail_tiles, "tail_splits": tail_splits.value,
                "tail_kernel": self.dll.hgemm_kernel_name(self.dll.hgemm_auto_plan_tail_kernel(M, N, K)).decode()}

    def tune(self, A, B, C_out, M: int, N: int, K: int, max_plans: int = 6, cold: bool = False) -> int:
        """Times up to ``max_plans`` plans for the shape on these operands and keeps the fastest for every later
        ``hgemm_auto`` call of the shape (``hgemm_auto_tune``); ``cold``: with the caches flushed before every timed
        launch.  Returns how many were timed."""
        return self.dll.hgemm_auto_tune(_tensor_ptr(A, M, K, "A"), _tensor_ptr(B, N, K, "B (stored as N rows of K)"),
                                        _tensor_ptr(C_out, M, N, "C"), M, N, K, max_plans, 1 if cold else 0)

    def tune_plans(self, M: int, N: int, K: int, max_plans: int = 6) -> List[dict]:
        """What ``tune`` would time, best first by the model (no launch)."""
        kernels, splits = (C.c_int * max_plans)(), (C.c_int * max_plans)()
        n = self.dll.hgemm_auto_tune_plans(M, N, K, max_plans, kernels, splits)
        return [{"kernel_id": kernels[i], "kernel": self.dll.hgemm_kernel_name(kernels[i]).decode(), "splits": splits[i]}
                for i in range(n)]

    def tune_results(self) -> List[dict]:
        """What this thread's last ``tune`` measured, plan by plan in the order they were timed."""
        out, i = [], 0
        kernel, splits, ms, kept = C.c_int(0), C.c_int(0), C.c_float(0.0), C.c_int(0)
        while self.dll.hgemm_auto_tune_result(i, C.byref(kernel), C.byref(splits), C.byref(ms), C.byref(kept)):
            out.append({"kernel_id": kernel.value, "kernel": self.dll.hgemm_kernel_name(kernel.value).decode(),
                        "splits": splits.value, "ms": ms.value, "kept": bool(kept.value)})
            i += 1
        return out

    def forget_tuning(self) -> None:
        self.dll.hgemm_auto_forget_tuning()

    def plan_is_tuned(self, M: int, N: int, K: int) -> bool:
        return bool(self.dll.hgemm_auto_plan_is_tuned(M, N, K))

    def small_m_rules(self) -> List[dict]:
        """The table behind hgemm_auto's choice for M <= 128, in order (first covering row wins)."""
        rows, i = [], 0
        while True:
            bounds, flags = (_SZ * 8)(), C.c_int(0)
            kernel = self.dll.hgemm_small_m_rule(i, bounds, C.byref(flags))
            if kernel < 0:
                return rows
            keys = ("m_lo", "m_hi", "n_lo", "n_hi", "k_lo", "k_hi", "b_lo", "b_hi")
            rows.append({**dict(zip(keys, list(bounds))), "k_below_4n": bool(flags.value & 1),
                         "k_not_multiple_of_16384": bool(flags.value & 2), "kernel_id": kernel,
                         "kernel": self.dll.hgemm_kernel_name(kernel).decode()})
            i += 1

    def auto_workspace_bytes(self, M: int, N: int, K: int) -> dict:
        operands = _SZ(0)
        partial = self.dll.hgemm_auto_workspace_bytes(M, N, K, C.byref(operands))
        return {"partial": partial, "operands": operands.value}

    def reserve_workspace(self, partial_bytes: int = 0, operand_bytes: int = 0) -> None:
        if self.dll.hgemm_reserve_workspace(partial_bytes, operand_bytes) != 0:
            raise MemoryError("hgemm_reserve_workspace: device memory ran out")

    def release_workspace(self) -> None:
        self.dll.hgemm_release_workspace()

    def static_workspace_bytes(self) -> int:
        return self.dll.hgemm_static_workspace_bytes()

    def version(self) -> str:
        return self.dll.hgemm_version().decode()

    # ---- calls ----------------------------------------------------------------------
    def fn(self, name: str):
        """The raw entry point ``void f(const half*, const half*, half*, size_t, size_t, size_t)``."""
        return getattr(self.dll, self.dll.hgemm_variant_symbol(self.find(name)).decode())

    def call(self, name: str, A, B, C_out, M: int, N: int, K: int) -> None:
        """Launch variant ``name`` on device tensors; shapes are checked here because the
        library answers a contract violation by ending the process."""
        a = _tensor_ptr(A, M, K, "A")
        b = _tensor_ptr(B, N, K, "B (stored as N rows of K)")
        c = _tensor_ptr(C_out, M, N, "C")
        if not self.supports(name, M, N, K):
            raise ValueError(f"variant {name!r} cannot run M={M} N={N} K={K}")
        self.fn(name)(a, b, c, M, N, K)

    def profile_ms(self, name: str, A, B, C_out, M: int, N: int, K: int, warmup: int, iterations: int) -> float:
        """Average milliseconds per call of ``iterations`` back-to-back calls after ``warmup``
        untimed ones (HIP events on the null stream, the loop of ``Tester::profile``)."""
        a = _tensor_ptr(A, M, K, "A")
        b = _tensor_ptr(B, N, K, "B (stored as N rows of K)")
        c = _tensor_ptr(C_out, M, N, "C")
        if not self.supports(name, M, N, K):
            raise ValueError(f"variant {name!r} cannot run M={M} N={N} K={K}")
        fn = self.dll.hgemm_variant_fn(self.find(name))
        return self.dll.hgemm_profile_ms(fn, a, b, c, M, N, K, warmup, iterations)

    def profile_fn_rotating_ms(self, fn, As, Bs, Cs, M: int, N: int, K: int, warmup: int, iterations: int) -> float:
        """Same loop over a cycle of operand sets; ``fn`` is an ``HGEMM_FN`` (ours or the vendor's)."""
        n = len(As)
        assert n == len(Bs) == len(Cs) and n > 0
        pa = (_PTR * n)(*[_tensor_ptr(t, M, K, "A") for t in As])
        pb = (_PTR * n)(*[_tensor_ptr(t, N, K, "B") for t in Bs])
        pc = (_PTR * n)(*[_tensor_ptr(t, M, N, "C") for t in Cs])
        return self.dll.hgemm_profile_rotating_ms(fn, pa, pb, pc, n, M, N, K, warmup, iterations)

    def variant_fn(self, name: str):
        return self.dll.hgemm_variant_fn(self.find(name))

    def clock_mark(self, which: int) -> None:
        """Enqueue shader-clock sample 0 or 1 on the null stream."""
        self.dll.hgemm_clock_mark(which)

    def clock_between_marks(self, xcds: int = 8) -> dict:
        """Average shader clock between the two marks (waits for the device)."""
        per_xcd = (C.c_double * xcds)()
        detail = (C.c_double * 3)()
        elapsed = C.c_double(0.0)
        mhz = self.dll.hgemm_clock_between_marks_mhz(per_xcd, xcds, C.byref(elapsed), detail)
        return {"mhz": mhz, "per_xcd_mhz": list(per_xcd), "elapsed_ms": elapsed.value, "min_mhz": detail[0],
                "max_mhz": detail[1], "simds": int(detail[2])}

    def tflops(self, M: int, N: int, K: int, ms: float) -> float:
        return self.dll.hgemm_tflops(M, N, K, ms)

    def bytes(self, M: int, N: int, K: int) -> float:
        return self.dll.hgemm_bytes(M, N, K)


class VendorLibrary:
    """``libhgemm_hipblaslt.so``: the hipBLASLt comparator, timed beside the kernels only."""

    def __init__(self, path: Optional[str] = None, torch_runtime: bool = True):
        """``torch_runtime=False``: bind to the system's hipBLASLt instead of the copy a PyTorch
        wheel carries under the same soname (torch must then not have been imported)."""
        self.path = path or vendor_lib_path()
        if not os.path.exists(self.path):
            raise FileNotFoundError(f"{self.path} is missing: build it with `python -m cuda_hgemm_amd.build`")
        if torch_runtime:
            _share_hip_runtime_with_torch()
        elif "torch" in sys.modules:
            raise RuntimeError("torch is already imported: its libhipblaslt answers the comparator's dependency")
        self.dll = C.CDLL(self.path)
        self.dll.hgemm_hipblaslt.argtypes, self.dll.hgemm_hipblaslt.restype = _HGEMM_ARGS, None
        self.dll.hgemm_hipblaslt_candidates.argtypes = [_SZ, _SZ, _SZ, C.POINTER(C.c_int), C.POINTER(C.c_float),
                                                        C.POINTER(C.c_float)]
        self.dll.hgemm_hipblaslt_candidates.restype = C.c_int
        self.dll.hgemm_hipblaslt_loaded_from.argtypes, self.dll.hgemm_hipblaslt_loaded_from.restype = [], C.c_char_p

    def loaded_from(self) -> str:
        """The hipBLASLt shared object this process bound the comparator to."""
        return os.path.realpath(self.dll.hgemm_hipblaslt_loaded_from().decode())

    def candidates(self, M: int, N: int, K: int) -> dict:
        """What the comparator's first call for the shape found (zero candidates: not called yet)."""
        chosen, chosen_ms, first_ms = C.c_int(-1), C.c_float(0.0), C.c_float(0.0)
        n = self.dll.hgemm_hipblaslt_candidates(M, N, K, C.byref(chosen), C.byref(chosen_ms), C.byref(first_ms))
        return {"candidates": n, "chosen": chosen.value, "chosen_ms": chosen_ms.value, "first_ms": first_ms.value}

    def fn(self):
        return C.cast(self.dll.hgemm_hipblaslt, HGEMM_FN)

    def call(self, A, B, C_out, M: int, N: int, K: int) -> None:
        self.dll.hgemm_hipblaslt(_tensor_ptr(A, M, K, "A"), _tensor_ptr(B, N, K, "B"), _tensor_ptr(C_out, M, N, "C"),
                                 M, N, K)


_library: Optional[HgemmLibrary] = None
_vendor: Optional[VendorLibrary] = None


def library(torch_runtime: bool = True) -> HgemmLibrary:
    global _library
    if _library is None:
        _library = HgemmLibrary(torch_runtime=torch_runtime)
    return _library


def vendor_library(torch_runtime: bool = True) -> VendorLibrary:
    global _vendor
    if _vendor is None:
        _vendor = VendorLibrary(torch_runtime=torch_runtime)
    return _vendor


def hgemm(A, B, variant: str = "hgemm_auto", out=None):
    """``C = A @ B.T`` for fp16 GPU tensors ``A (M, K)`` and ``B (N, K)`` through variant ``variant``."""
    import torch
    M, K = A.shape
    N = B.shape[0]
    if out is None:
        out = torch.empty((M, N), dtype=torch.float16, device=A.device)
    library().call(variant, A, B, out, M, N, K)
    return out
