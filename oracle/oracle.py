"""ctypes loader for the CPU checker (``libhgemm_oracle.so``).  TEST INFRASTRUCTURE ONLY.

Only ``tests/``, the smoke check and the CPU-baseline leg of the benchmark import this
module; the shipped package never does.  Arrays of fp16 values travel as ``numpy.uint16``
bit patterns (``.view(numpy.float16)`` gives the values).

Layouts follow the reference (``src/common/tester.h:117-120``): ``A`` is ``(M, K)``
row-major, ``B`` is handed over as its ``(N, K)`` storage (column-major ``K x N``), ``C`` is
``(M, N)`` row-major.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libhgemm_oracle.so")

UNIFORM, NORMAL, TERNARY = 0, 1, 2
DEFAULT_SEED = 20230212
STREAM_A, STREAM_B = 1, 2


def build(force: bool = False) -> str:
    """Compile the checker with the Makefile beside this file."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.run(["make", "-C", _HERE] + (["-B"] if force else []), check=True, capture_output=True)
    return _LIB_PATH


_lib = None


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        build()
        L = C.CDLL(_LIB_PATH)
        u16p, f32p, f64p = C.POINTER(C.c_uint16), C.POINTER(C.c_float), C.POINTER(C.c_double)
        sz = C.c_size_t
        L.oracle_f16_to_f32.argtypes, L.oracle_f16_to_f32.restype = [C.c_uint16], C.c_float
        L.oracle_f32_to_f16.argtypes, L.oracle_f32_to_f16.restype = [C.c_float], C.c_uint16
        L.oracle_hw_f16_to_f32.argtypes, L.oracle_hw_f16_to_f32.restype = [C.c_uint16], C.c_float
        L.oracle_hw_f32_to_f16.argtypes, L.oracle_hw_f32_to_f16.restype = [C.c_float], C.c_uint16
        L.oracle_has_f16c.restype = C.c_int
        L.oracle_f16_to_f32_array.argtypes = [u16p, f32p, sz]
        L.oracle_f32_to_f16_array.argtypes = [f32p, u16p, sz]
        L.oracle_rng_u64.argtypes, L.oracle_rng_u64.restype = [C.c_uint64] * 3, C.c_uint64
        L.oracle_fill.argtypes = [u16p, sz, C.c_uint64, C.c_uint64, C.c_int, C.c_float, C.c_float]
        L.oracle_hgemm_naive_f64.argtypes = [u16p, u16p, u16p, f64p, sz, sz, sz]
        L.oracle_hgemm_naive_f32.argtypes = [u16p, u16p, u16p, sz, sz, sz]
        L.oracle_sgemm_nt.argtypes = [f32p, f32p, f32p, sz, sz, sz]
        L.oracle_hgemm.argtypes, L.oracle_hgemm.restype = [u16p, u16p, u16p, f32p, sz, sz, sz], C.c_int
        L.oracle_diff.argtypes = [u16p, u16p, sz, f64p]
        L.oracle_tflops.argtypes, L.oracle_tflops.restype = [sz, sz, sz, C.c_double], C.c_double
        L.oracle_num_threads.restype = C.c_int
        L.oracle_time_sgemm_nt.argtypes, L.oracle_time_sgemm_nt.restype = [f32p, f32p, f32p, sz, sz, sz], C.c_double
        _lib = L
    return _lib


def _p(a: np.ndarray, ty):
    return a.ctypes.data_as(C.POINTER(ty))


def _u16(a) -> np.ndarray:
    a = np.ascontiguousarray(a)
    if a.dtype == np.float16:
        a = a.view(np.uint16)
    assert a.dtype == np.uint16, a.dtype
    return a


def f16_to_f32(bits) -> np.ndarray:
    bits = _u16(bits)
    out = np.empty(bits.shape, np.float32)
    lib().oracle_f16_to_f32_array(_p(bits, C.c_uint16), _p(out, C.c_float), bits.size)
    return out


def f32_to_f16(vals) -> np.ndarray:
    vals = np.ascontiguousarray(vals, dtype=np.float32)
    out = np.empty(vals.shape, np.uint16)
    lib().oracle_f32_to_f16_array(_p(vals, C.c_float), _p(out, C.c_uint16), vals.size)
    return out


def fill(shape, seed=DEFAULT_SEED, stream=STREAM_A, dist=UNIFORM, p0=-1.0, p1=1.0) -> np.ndarray:
    """Seeded fp16 matrix (uint16 bit patterns) of the given shape."""
    out = np.empty(shape, np.uint16)
    lib().oracle_fill(_p(out, C.c_uint16), out.size, seed, stream, dist, p0, p1)
    return out


def hgemm(A, B, want_f32: bool = False):
    """fp32-accumulate product in the reference's layouts.  A: (M,K), B: (N,K) -> C: (M,N) uint16."""
    A, B = _u16(A), _u16(B)
    M, K = A.shape
    N, K2 = B.shape
    assert K == K2, (A.shape, B.shape)
    Cb = np.empty((M, N), np.uint16)
    Cf = np.empty((M, N), np.float32) if want_f32 else None
    rc = lib().oracle_hgemm(_p(A, C.c_uint16), _p(B, C.c_uint16), _p(Cb, C.c_uint16),
                            _p(Cf, C.c_float) if want_f32 else None, M, N, K)
    if rc != 0:
        raise MemoryError("oracle_hgemm: scratch allocation failed")
    return (Cb, Cf) if want_f32 else Cb


def hgemm_rows(A, B, m0: int, mc: int, want_f32: bool = False):
    """Rows [m0, m0+mc) of the product (sampled check of large shapes)."""
    return hgemm(_u16(A)[m0:m0 + mc], B, want_f32)


def hgemm_naive_f64(A, B):
    """Brute-force double-precision triple loop; returns (C uint16, C double)."""
    A, B = _u16(A), _u16(B)
    M, K = A.shape
    N = B.shape[0]
    Cb = np.empty((M, N), np.uint16)
    Cd = np.empty((M, N), np.float64)
    lib().oracle_hgemm_naive_f64(_p(A, C.c_uint16), _p(B, C.c_uint16), _p(Cb, C.c_uint16), _p(Cd, C.c_double), M, N, K)
    return Cb, Cd


def hgemm_naive_f32(A, B) -> np.ndarray:
    A, B = _u16(A), _u16(B)
    M, K = A.shape
    N = B.shape[0]
    Cb = np.empty((M, N), np.uint16)
    lib().oracle_hgemm_naive_f32(_p(A, C.c_uint16), _p(B, C.c_uint16), _p(Cb, C.c_uint16), M, N, K)
    return Cb


def diff(got, ref) -> dict:
    """max / avg abs diff (``src/common/matrix.h:102-111``) plus the rms of ``ref``."""
    got, ref = _u16(got), _u16(ref)
    assert got.shape == ref.shape
    out = np.zeros(5, np.float64)
    lib().oracle_diff(_p(got, C.c_uint16), _p(ref, C.c_uint16), got.size, _p(out, C.c_double))
    return {"max_diff": out[0], "avg_diff": out[1], "ref_rms": out[2], "non_finite": int(out[3]), "argmax": int(out[4])}


def tolerance(K: int) -> float:
    """Allowed max |err| relative to the output scale: 1e-2 * sqrt(K / 256)."""
    return 1e-2 * float(np.sqrt(K / 256.0))


def check(got, ref, K: int) -> dict:
    """Apply the fp16-output tolerance.  Output scale = rms of the reference result
    (never below one fp16 ulp of 1.0 so an all-zero reference does not divide by zero)."""
    d = diff(got, ref)
    scale = max(d["ref_rms"], 2.0 ** -10)
    d["rel_err"] = d["max_diff"] / scale
    d["tol"] = tolerance(K)
    d["ok"] = bool(d["non_finite"] == 0 and d["rel_err"] <= d["tol"])
    return d


def tflops(M: int, N: int, K: int, ms: float) -> float:
    return lib().oracle_tflops(M, N, K, ms)


def num_threads() -> int:
    return lib().oracle_num_threads()


def time_sgemm_nt(Af: np.ndarray, Bf: np.ndarray) -> tuple[float, np.ndarray]:
    """Seconds for one blocked fp32 GEMM on pre-converted operands; returns (seconds, Cf)."""
    Af = np.ascontiguousarray(Af, np.float32)
    Bf = np.ascontiguousarray(Bf, np.float32)
    M, K = Af.shape
    N = Bf.shape[0]
    Cf = np.empty((M, N), np.float32)
    s = lib().oracle_time_sgemm_nt(_p(Af, C.c_float), _p(Bf, C.c_float), _p(Cf, C.c_float), M, N, K)
    return s, Cf
