"""Builds the native pieces in-tree with hipcc for gfx950:

    cuda_hgemm_amd/lib/libhgemm.so            the kernels + C ABI (include/hgemm.h)
    cuda_hgemm_amd/lib/libhgemm_hipblaslt.so  vendor comparator (include/hgemm_hipblaslt.h)
    cuda_hgemm_amd/bin/hgemm                  C++ benchmark / check driver

Run as ``python -m cuda_hgemm_amd.build`` (add ``--force`` to rebuild everything).
hipcc cross-compiles without a GPU, so this works on a CPU-only machine.
"""
from __future__ import annotations

import concurrent.futures as cf
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(HERE, "build")
LIB = os.path.join(HERE, "lib")
BIN = os.path.join(HERE, "bin")
INCLUDE = os.path.join(os.path.dirname(HERE), "include")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
ARCH = "gfx950"
# -packed-fp32-ops is switched off on purpose: the packed FP32 forms the compiler would
# pick by itself are not trusted on this hardware pool.
DEVICE_FLAGS = ["--offload-arch=" + ARCH, "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]
CXXFLAGS = ["-O3", "-std=c++17", "-fPIC", "-Wall", "-Wextra", "-Wno-unused-parameter", "-I" + INCLUDE]

LIB_SOURCES = ["basic_kernels.hip", "ladder_sync.hip", "ladder_async.hip", "ladder_stages.hip", "dispatch.hip",
               "probe.hip", "api.hip"]
VENDOR_SOURCES = ["vendor_hipblaslt.cpp"]
DRIVER_SOURCES = ["driver/main.cpp"]


def _headers():
    out = []
    for root, _, files in os.walk(CSRC):
        out += [os.path.join(root, f) for f in files if f.endswith(".h")]
    out += [os.path.join(INCLUDE, f) for f in os.listdir(INCLUDE)]
    return out


def _stale(target, deps):
    if not os.path.exists(target):
        return True
    t = os.path.getmtime(target)
    return any(os.path.getmtime(d) > t for d in deps)


def _run(cmd):
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    lines = [l for l in r.stdout.splitlines() if "is not a recognized feature for this target" not in l]
    if r.returncode != 0:
        raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), "\n".join(lines)))
    return "\n".join(lines)


def _compile(src, force):
    obj = os.path.join(OBJ, src.replace("/", "_") + ".o")
    path = os.path.join(CSRC, src)
    if force or _stale(obj, [path] + _headers()):
        flags = CXXFLAGS + (DEVICE_FLAGS if src.endswith(".hip") else [])
        if src.startswith("driver/"):
            flags = flags + ["-fopenmp"]
        _run([HIPCC] + flags + ["-c", path, "-o", obj])
    return obj


def build(force: bool = False, verbose: bool = False) -> dict:
    for d in (OBJ, LIB, BIN):
        os.makedirs(d, exist_ok=True)
    sources = LIB_SOURCES + VENDOR_SOURCES + DRIVER_SOURCES
    with cf.ThreadPoolExecutor(max_workers=min(8, len(sources))) as pool:
        objs = dict(zip(sources, pool.map(lambda s: _compile(s, force), sources)))
    libhgemm = os.path.join(LIB, "libhgemm.so")
    vendor = os.path.join(LIB, "libhgemm_hipblaslt.so")
    driver = os.path.join(BIN, "hgemm")
    lib_objs = [objs[s] for s in LIB_SOURCES]
    if force or _stale(libhgemm, lib_objs):
        _run([HIPCC, "-shared", "-o", libhgemm] + lib_objs)
    ven_objs = [objs[s] for s in VENDOR_SOURCES]
    if force or _stale(vendor, ven_objs):
        _run([HIPCC, "-shared", "-o", vendor] + ven_objs + ["-lhipblaslt"])
    drv_objs = [objs[s] for s in DRIVER_SOURCES]
    if force or _stale(driver, drv_objs + [libhgemm, vendor]):
        _run([HIPCC, "-o", driver] + drv_objs + ["-L" + LIB, "-lhgemm", "-lhgemm_hipblaslt", "-fopenmp",
                                                  "-Wl,-rpath,$ORIGIN/../lib"])
    if verbose:
        print("built", libhgemm, vendor, driver)
    return {"libhgemm": libhgemm, "vendor": vendor, "driver": driver}


if __name__ == "__main__":
    build(force="--force" in sys.argv, verbose=True)
