"""Device memory without PyTorch: a minimal ctypes view of the HIP runtime.

The benchmark uses this instead of torch tensors so that its process holds exactly one set of
ROCm libraries, the system's: a PyTorch wheel ships its own ``libamdhip64`` and
``libhipblaslt`` under the same sonames, and whichever copy is mapped first answers every
later dependency on that soname -- with torch imported, the vendor comparator would be timed
on the wheel's older hipBLASLt.  Tests keep using torch tensors; both kinds of buffer are
accepted wherever the binding takes an operand.

Only what a benchmark needs: allocate, copy in, copy out, synchronise, device properties.
"""
from __future__ import annotations

import ctypes as C
from typing import Optional, Tuple

import numpy as np

_HIP_MEMCPY_H2D, _HIP_MEMCPY_D2H = 1, 2
_hip: Optional[C.CDLL] = None


class HipError(RuntimeError):
    pass


def runtime() -> C.CDLL:
    """The HIP runtime of this process: the copy already mapped under its soname (load
    ``libhgemm.so`` first and it is the one that library is bound to), else the system's."""
    global _hip
    if _hip is None:
        for name in ("libamdhip64.so.7", "/opt/rocm/lib/libamdhip64.so.7", "/opt/rocm/lib/libamdhip64.so"):
            try:
                _hip = C.CDLL(name)
                break
            except OSError:
                continue
        else:
            raise HipError("libamdhip64 is not loadable: no HIP runtime on this machine")
        _hip.hipGetErrorString.restype = C.c_char_p
        _hip.hipGetErrorString.argtypes = [C.c_int]
        _hip.hipMalloc.argtypes = [C.POINTER(C.c_void_p), C.c_size_t]
        _hip.hipFree.argtypes = [C.c_void_p]
        _hip.hipMemcpy.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_int]
        _hip.hipMemset.argtypes = [C.c_void_p, C.c_int, C.c_size_t]
        _hip.hipDeviceGetAttribute.argtypes = [C.POINTER(C.c_int), C.c_int, C.c_int]
        _hip.hipDeviceGetName.argtypes = [C.c_char_p, C.c_int, C.c_int]
        _hip.hipGetDeviceCount.argtypes = [C.POINTER(C.c_int)]
    return _hip


def _check(status: int, what: str) -> None:
    if status != 0:
        raise HipError(f"{what}: HIP error {status} ({runtime().hipGetErrorString(status).decode()})")


def device_count() -> int:
    n = C.c_int(0)
    status = runtime().hipGetDeviceCount(C.byref(n))
    return n.value if status == 0 else 0


def synchronize() -> None:
    _check(runtime().hipDeviceSynchronize(), "hipDeviceSynchronize")


def device_name(device: int = 0) -> str:
    buf = C.create_string_buffer(256)
    _check(runtime().hipDeviceGetName(buf, 256, device), "hipDeviceGetName")
    return buf.value.decode()


def compute_units(device: int = 0) -> int:
    n = C.c_int(0)
    _check(runtime().hipDeviceGetAttribute(C.byref(n), 63, device),  # hipDeviceAttributeMultiprocessorCount
           "hipDeviceGetAttribute")
    return n.value


class DeviceArray:
    """A ``rows x cols`` matrix of 2-byte elements (fp16 bit patterns) in device memory."""

    dtype_name = "float16"

    def __init__(self, shape: Tuple[int, int]):
        self.shape = (int(shape[0]), int(shape[1]))
        self.nbytes = self.shape[0] * self.shape[1] * 2
        ptr = C.c_void_p()
        _check(runtime().hipMalloc(C.byref(ptr), max(self.nbytes, 16)), f"hipMalloc({self.nbytes})")
        self.ptr = ptr.value

    @classmethod
    def from_host(cls, bits: np.ndarray) -> "DeviceArray":
        """``bits``: a 2-D uint16 or float16 array (the fp16 bit patterns)."""
        host = np.ascontiguousarray(bits)
        if host.ndim != 2 or host.dtype.itemsize != 2:
            raise TypeError(f"expected a 2-D array of 2-byte elements, got {host.dtype} with shape {host.shape}")
        out = cls(host.shape)
        _check(runtime().hipMemcpy(out.ptr, host.ctypes.data, out.nbytes, _HIP_MEMCPY_H2D), "hipMemcpy to device")
        return out

    def to_host(self) -> np.ndarray:
        """The fp16 bit patterns as a uint16 array (waits for the device, like any synchronous copy)."""
        host = np.empty(self.shape, np.uint16)
        _check(runtime().hipMemcpy(host.ctypes.data, self.ptr, self.nbytes, _HIP_MEMCPY_D2H), "hipMemcpy to host")
        return host

    def fill_bytes(self, byte: int) -> "DeviceArray":
        _check(runtime().hipMemset(self.ptr, byte, self.nbytes), "hipMemset")
        return self

    def data_ptr(self) -> int:
        return self.ptr

    def free(self) -> None:
        if self.ptr:
            runtime().hipFree(self.ptr)
            self.ptr = 0

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass
