"""Dimension sweep with the command-line driver: the counterpart of the reference's
``benchmark_hgemm`` (run_sample.sh:29-58).

For every shape the driver ``bin/hgemm`` runs once, hipBLASLt first (the 100 % line) and
then the default variants, and its log goes to ``<out>/hgemm_<M>_<N>_<K>.log`` -- the file
naming the reference uses (run_sample.sh:18), which ``cuda_hgemm_amd.performance`` reads
back into tables and charts.

    python -m cuda_hgemm_amd.benchmark --out log                     # 20 squares 256 ... 16384
    python -m cuda_hgemm_amd.benchmark --sweep wide --out log_wide   # M = N > K
    python -m cuda_hgemm_amd.benchmark --sweep deep --out log_deep   # M = N < K
    python -m cuda_hgemm_amd.benchmark --profile --dims 8192         # under rocprofv3 (the reference: ncu)
    python -m cuda_hgemm_amd.benchmark --pmc mfma --dims 8192        # hardware counters, one named set per run

The driver is started as a child process per shape, like the shell loop of the reference;
this module never touches the GPU itself.
"""
from __future__ import annotations

import argparse
import os
import subprocess
import sys
import time

# the reference's dimension list (run_sample.sh:30)
DIMS = [256, 512, 768, 1024, 1536, 2048, 3072, 4096, 5120, 6144, 7168, 8192, 9216, 10240, 11264, 12288, 13312,
        14336, 15360, 16384]

# Hardware-counter sets for --pmc, each small enough for one pass (rocprofv3 does not split
# counters over passes: at most 8 SQ, 4 TCC -- FETCH_SIZE takes 3 of them, WRITE_SIZE 2 -- and
# 2 GRBM counters per run).  Together they cover what the reference's `ncu --set full` run is
# read for (run_sample.sh:23-27): matrix-pipe occupancy, LDS bank conflicts, bytes moved
# between L2 and the memory fabric.
PMC_SETS = {
    "mfma": ["SQ_VALU_MFMA_BUSY_CYCLES", "SQ_INSTS_VALU_MFMA_MOPS_F16", "SQ_BUSY_CYCLES", "SQ_WAVES", "GRBM_GUI_ACTIVE"],
    "lds": ["SQ_LDS_BANK_CONFLICT", "SQ_LDS_IDX_ACTIVE", "SQ_INSTS_LDS", "SQ_VALU_MFMA_BUSY_CYCLES", "GRBM_GUI_ACTIVE"],
    "fetch": ["FETCH_SIZE"],
    "write": ["WRITE_SIZE"],
}

PACKAGE_DIR = os.path.dirname(os.path.abspath(__file__))
DRIVER = os.path.join(PACKAGE_DIR, "bin", "hgemm")


def shapes(sweep: str, dims: list[int]) -> list[tuple[int, int, int]]:
    """Shapes of one sweep.  ``square``: M = N = K over ``dims`` (run_sample.sh:33-37).
    ``wide``: M = N from the upper half of ``dims``, K from the lower half
    (run_sample.sh:40-47).  ``deep``: M = N from the lower half, K from the upper half
    (run_sample.sh:50-57)."""
    half = len(dims) // 2
    lower, upper = dims[:half], dims[half:half + half]
    if sweep == "square":
        return [(d, d, d) for d in dims]
    if sweep == "wide":
        return [(m, m, k) for m in upper for k in lower]
    if sweep == "deep":
        return [(m, m, k) for m in lower for k in upper]
    raise ValueError(f"unknown sweep '{sweep}' (square, wide, deep)")


def driver_command(m: int, n: int, k: int, args) -> list[str]:
    cmd = [DRIVER, f"-M={m}", f"-N={n}", f"-K={k}", f"-warmup_iterations={args.warmup}",
           f"-profiling_iterations={args.iterations}", f"-sleep_duration={args.sleep_ms}",
           f"-enable_check={'true' if args.check else 'false'}",
           f"-enable_naive={'true' if args.naive else 'false'}"]
    if args.variant:
        cmd.append(f"-variant={args.variant}")
    if args.json:
        cmd.append(f"-json={os.path.join(args.out, f'hgemm_{m}_{n}_{k}.json')}")
    return cmd


def profiler_command(m: int, n: int, k: int, args, pmc: str = "") -> list[str]:
    """rocprofv3 run of one shape with a single timed iteration, in place of the reference's
    ``ncu --set full`` run (run_sample.sh:23-27): a kernel trace with per-kernel statistics,
    or -- ``pmc`` names one of PMC_SETS -- hardware counters per dispatch.  Counters and
    traces never share a run.  The driver binary itself follows ``--``: the profiler must not
    be handed a launcher that re-executes."""
    out_dir = os.path.join(os.path.abspath(args.out), "rocprof" + ("_" + pmc if pmc else ""), f"hgemm_{m}_{n}_{k}")
    saved = (args.warmup, args.iterations)
    args.warmup, args.iterations = 1, 1
    what = ["--pmc"] + PMC_SETS[pmc] if pmc else ["--kernel-trace", "--stats"]
    cmd = ["rocprofv3"] + what + ["--output-format", "csv", "-d", out_dir, "-o", "hgemm", "--"]
    cmd += driver_command(m, n, k, args)
    args.warmup, args.iterations = saved
    return cmd


def run_one(cmd: list[str], log_path: str, timeout_s: float, scratch_dir: str | None = None) -> int:
    """Runs one command with its output in ``log_path``.  ``scratch_dir``: working directory
    and TMPDIR of the child (rocprofv3 writes temporary files next to where it runs)."""
    env = dict(os.environ, TMPDIR=scratch_dir) if scratch_dir else None
    with open(log_path, "w") as log:
        try:
            return subprocess.run(cmd, stdout=log, stderr=subprocess.STDOUT, timeout=timeout_s, cwd=scratch_dir,
                                  env=env).returncode
        except subprocess.TimeoutExpired:
            log.write(f"\nkilled after {timeout_s:.0f} s\n")
            return 124


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--sweep", default="square", choices=["square", "wide", "deep"])
    ap.add_argument("--dims", default="", help="comma-separated dimension list instead of the reference's 20")
    ap.add_argument("--out", default="log", help="directory for the hgemm_<M>_<N>_<K>.log files")
    ap.add_argument("--warmup", type=int, default=10, help="-warmup_iterations of the driver")
    ap.add_argument("--iterations", type=int, default=100, help="-profiling_iterations of the driver")
    ap.add_argument("--sleep-ms", type=int, default=100, help="-sleep_duration of the driver")
    ap.add_argument("--check", action="store_true", help="check every variant against hipBLASLt")
    ap.add_argument("--naive", action="store_true", help="include the variants left out of the default run")
    ap.add_argument("--variant", default="", help="evaluate only this variant next to hipBLASLt")
    ap.add_argument("--json", action="store_true", help="also keep the driver's JSON report per shape")
    ap.add_argument("--profile", action="store_true", help="additionally trace each shape under rocprofv3")
    ap.add_argument("--pmc", default="", help="comma-separated counter sets to collect per shape, one rocprofv3 run "
                    "each: " + ", ".join(f"{k} ({' '.join(v)})" for k, v in PMC_SETS.items()))
    ap.add_argument("--timeout", type=float, default=300.0, help="seconds allowed per driver run")
    ap.add_argument("--pause", type=float, default=0.0, help="seconds between shapes (the reference sleeps 3)")
    args = ap.parse_args(argv)

    if not os.path.exists(DRIVER):
        print(f"{DRIVER} is not built: run python -m cuda_hgemm_amd.build", file=sys.stderr)
        return 2
    dims = [int(d) for d in args.dims.split(",") if d] if args.dims else DIMS
    pmc_sets = [p for p in args.pmc.split(",") if p]
    for p in pmc_sets:
        if p not in PMC_SETS:
            print(f"unknown counter set '{p}' (known: {', '.join(PMC_SETS)})", file=sys.stderr)
            return 2
    args.out = os.path.abspath(args.out)
    os.makedirs(args.out, exist_ok=True)
    failed = 0
    for (m, n, k) in shapes(args.sweep, dims):
        print(f"Evaluating {m} * {n} * {k}", flush=True)
        rc = run_one(driver_command(m, n, k, args), os.path.join(args.out, f"hgemm_{m}_{n}_{k}.log"), args.timeout)
        if rc == 0 and args.profile:
            print(f"rocprofv3 {m} * {n} * {k}", flush=True)
            rc = run_one(profiler_command(m, n, k, args),
                         os.path.join(args.out, f"rocprof_hgemm_{m}_{n}_{k}.log"), args.timeout, scratch_dir="/tmp")
        for p in pmc_sets if rc == 0 else []:
            print(f"rocprofv3 --pmc {p} {m} * {n} * {k}", flush=True)
            rc = run_one(profiler_command(m, n, k, args, pmc=p),
                         os.path.join(args.out, f"rocprof_{p}_hgemm_{m}_{n}_{k}.log"), args.timeout, scratch_dir="/tmp")
            if rc != 0:
                break
        if rc != 0:
            failed += 1
            print(f"  driver exited with {rc}, see {args.out}/", file=sys.stderr, flush=True)
            if rc in (124, 134, 137, 139, -6, -9, -11):
                print("  stopping: a run was killed or crashed", file=sys.stderr, flush=True)
                break
        if args.pause > 0:
            time.sleep(args.pause)
    return 1 if failed else 0


if __name__ == "__main__":
    sys.exit(main())
