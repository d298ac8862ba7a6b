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
import re
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
               "api.hip"]
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


# Kernels whose operands and accumulators are handled from inline assembly in an order the
# compiler does not know: a register spill between an LDS read and its wait, or of an
# accumulator, would corrupt results silently, so the build fails if one appears.  The chained
# kernel keeps its accumulators in AGPRs a0 ... a(4*TM*TN-1) that only its asm statements name:
# it must use exactly that many AGPRs (one more would be an accumulator register the compiler
# took for itself) and fewer than 256 VGPRs (beyond them the allocator starts looking for AGPRs).
# (the decode kernel that keeps A in registers is here because a spill of those registers would put A in scratch
# memory and silently cost what the kernel exists to save)
NO_SPILL_KERNELS = ("hgemm_pipelined_kernel", "hgemm_chained_kernel", "hgemm_decode_resident_kernel")
# sources that must contain such kernels: a remark format the parser no longer understands
# must not turn the guard into a no-op
MUST_CHECK = {"dispatch.hip": NO_SPILL_KERNELS}


def _chained_accumulator_registers(mangled):
    """4 * PTM * PTN of a hgemm_chained_kernel instantiation, from the PipeConfig arguments in
    its mangled name (BM, BN, BK, WAVES_M, WAVES_N, STAGES, MI, ...): 16x16 tiles, 4 registers each."""
    m = re.search(r"PipeConfigI((?:Li\d+E)+)E", mangled)
    if not m:
        raise RuntimeError(f"cannot read the tile configuration out of {mangled}")
    bm, bn, _bk, waves_m, waves_n, _stages, mi = [int(v) for v in re.findall(r"Li(\d+)E", m.group(1))[:7]]
    return 4 * (bm // waves_m // mi) * (bn // waves_n // mi)


def _check_no_spills(src, remarks):
    """`remarks`: output of -Rpass-analysis=kernel-resource-usage for one source file.
    Returns the names of the guarded kernel templates that were seen and checked."""
    usage = {}  # kernel -> {key: value}
    name = None
    for line in remarks.splitlines():
        if "remark: Function Name:" in line:
            name = line.split("Function Name:")[1].split()[0]
            usage[name] = {}
            continue
        if name is None:
            continue
        for key in ("ScratchSize [bytes/lane]:", "VGPRs Spill:", "VGPRs:", "AGPRs:"):
            if "remark:     " + key in line or "remark: " + key in line:
                usage[name][key] = int(line.split(key)[1].split()[0])
    seen = set()
    for name, u in usage.items():
        kind = next((k for k in NO_SPILL_KERNELS if k in name), None)
        if kind is None:
            continue
        missing = [k for k in ("ScratchSize [bytes/lane]:", "VGPRs Spill:", "VGPRs:", "AGPRs:") if k not in u]
        if missing:
            raise RuntimeError(f"{src}: no {missing} remark for kernel {name}: the resource guard cannot check it")
        for key in ("ScratchSize [bytes/lane]:", "VGPRs Spill:"):
            if u[key] != 0:
                raise RuntimeError(f"{src}: kernel {name} has {key} {u[key]}; its inline-assembly schedule "
                                   "needs every operand and accumulator in registers")
        if kind == "hgemm_chained_kernel":
            want = _chained_accumulator_registers(name)
            if u["AGPRs:"] != want or u["VGPRs:"] >= 256:
                raise RuntimeError(f"{src}: kernel {name} uses {u['AGPRs:']} AGPRs and {u['VGPRs:']} VGPRs; its named "
                                   f"accumulators need exactly {want} AGPRs and fewer than 256 VGPRs")
        seen.add(kind)
    for kind in MUST_CHECK.get(os.path.basename(src), ()):
        if kind not in seen:
            raise RuntimeError(f"{src}: the resource guard found no {kind} in the compiler's remarks")
    return seen


def _compile(src, force):
    obj = os.path.join(OBJ, src.replace("/", "_") + ".o")
    path = os.path.join(CSRC, src)
    if force or _stale(obj, [path] + _headers()):
        flags = CXXFLAGS + (DEVICE_FLAGS if src.endswith(".hip") else [])
        if src.startswith("driver/"):
            flags = flags + ["-fopenmp"]
        if src.endswith(".hip"):
            flags = flags + ["-Rpass-analysis=kernel-resource-usage"]
        out = _run([HIPCC] + flags + ["-c", path, "-o", obj])
        if src.endswith(".hip"):
            with open(obj + ".resources.txt", "w") as f:  # registers, scratch and occupancy per kernel, for inspection
                f.write(out)
            try:
                _check_no_spills(src, out)
            except RuntimeError:
                os.remove(obj)
                raise
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
        _run([HIPCC, "-shared", "-o", vendor] + ven_objs + ["-L/opt/rocm/lib", "-lhipblaslt", "-ldl", "-Wl,-rpath,/opt/rocm/lib"])
    drv_objs = [objs[s] for s in DRIVER_SOURCES]
    if force or _stale(driver, drv_objs + [libhgemm, vendor]):
        _run([HIPCC, "-o", driver] + drv_objs + ["-L" + LIB, "-lhgemm", "-lhgemm_hipblaslt", "-fopenmp",
                                                  "-Wl,-rpath,$ORIGIN/../lib"])
    if verbose:
        print("built", libhgemm, vendor, driver)
    return {"libhgemm": libhgemm, "vendor": vendor, "driver": driver}


if __name__ == "__main__":
    build(force="--force" in sys.argv, verbose=True)
