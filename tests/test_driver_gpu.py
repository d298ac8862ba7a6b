"""The C++ harness (Tester / Matrix / HipTimer / main) run the way the reference runs its own:
the checked sample of run_sample.sh:60, the result line as tools/performance/performance.py
tokenises it, the JSON report, exit codes, and the sweep runner on real logs."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def checksum64(bits):
    """The driver's checksum64 (csrc/driver/matrix.h) in numpy: sum of (bits + 1) * odd(i) mod 2^64."""
    flat = np.ascontiguousarray(bits).reshape(-1).astype(np.uint64)
    with np.errstate(over="ignore"):
        idx = np.arange(flat.size, dtype=np.uint64) * np.uint64(0x9E3779B97F4A7C15) | np.uint64(1)
        return int(((flat + np.uint64(1)) * idx).sum(dtype=np.uint64))


def _driver():
    from cuda_hgemm_amd import driver_path
    exe = driver_path()
    assert os.path.exists(exe), "build the driver with `python -m cuda_hgemm_amd.build`"
    return exe


def _result_lines(text):
    """As the reference's plotter finds them (performance.py:26-29): lines with 'exit'."""
    return [line for line in text.splitlines() if " exit, " in line]


# ------------------------------------------------------------------ host side only
@pytest.mark.parametrize("dist,odist", [("uniform", (0, -1.0, 1.0)), ("normal:0.02", (1, 0.0, 0.02)),
                                        ("uniform:0:4", (0, 0.0, 4.0)), ("normal:1.5:0.25", (1, 1.5, 0.25))])
@pytest.mark.parametrize("seed", [20230212, 7])
def test_driver_fill_is_the_checkers_fill(oracle, dist, odist, seed):
    """Matrix's generator (a second implementation, in C++) against oracle.fill for the same
    seed and stream, bit for bit through a position-dependent checksum."""
    M, N, K = 96, 160, 224
    r = subprocess.run([_driver(), f"-M={M}", f"-N={N}", f"-K={K}", f"-seed={seed}", f"-dist_a={dist}",
                        f"-dist_b={dist}", "-fill_only"], capture_output=True, text=True, timeout=60)
    assert r.returncode == 0, r.stderr
    rep = json.loads(r.stdout)
    A = oracle.fill((M, K), seed, oracle.STREAM_A, *odist)
    B = oracle.fill((N, K), seed, oracle.STREAM_B, *odist)
    assert int(rep["a_checksum"], 16) == checksum64(A) and int(rep["b_checksum"], 16) == checksum64(B)
    assert checksum64(A) != checksum64(A[::-1].copy())          # the checksum sees positions


# ------------------------------------------------------------------ on the GPU
@pytest.mark.gpu
def test_driver_checked_sample_run(oracle, hgemm_lib, tmp_path):
    """bin/hgemm -M=512 -N=2048 -K=1024 -enable_check=true (reference run_sample.sh:60)."""
    M, N, K = 512, 2048, 1024
    report = tmp_path / "sample.json"
    print("[gpu] bin/hgemm checked sample run", flush=True)
    r = subprocess.run([_driver(), f"-M={M}", f"-N={N}", f"-K={K}", "-enable_check=true", "-enable_naive=true",
                        "-warmup_iterations=1", "-profiling_iterations=10", "-sleep_duration=10", f"-json={report}"],
                       capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    log = r.stderr
    names = [v["name"] for v in hgemm_lib.variants() if hgemm_lib.supports(v["symbol"], M, N, K)]
    assert len(names) == len(hgemm_lib.variants()) - 1 and "Skinny" not in names     # M > 128
    expected = ["Hipblaslt-Gemm"] + names
    assert log.count("Check passed") == len(expected) and "FAILED" not in log
    assert log.rstrip().endswith("Done")
    # the result line, token for token as the reference's plotter indexes it (performance.py:28-29,57-62)
    lines = _result_lines(log)
    assert [line.split(" ")[6] for line in lines] == expected
    for line in lines:
        tok = line.rstrip("\n").split(" ")
        assert tok[0] == "[HGEMM" and tok[5] == "profile]" and tok[7] == "exit," and tok[15] == "TFLOPS"
        ms, tflops = float(tok[10]), float(tok[14])
        pct = float(tok[16].replace("(", "").replace(")", "").replace("%", ""))
        assert ms > 0 and tflops > 0 and pct > 0
        # reference src/common/tester.h:96-97; the time is printed to 1 us, half of that either way
        assert abs(tflops - 2.0 * M * N * K * 1e-12 / (ms * 1e-3)) <= tflops * 0.00051 / (ms - 0.0005) + 0.01
    assert abs(float(lines[0].split(" ")[16].strip("()%\n")) - 100.0) < 1e-9     # the vendor line is the 100 % line
    # our own parser on the same real log
    from cuda_hgemm_amd import performance
    (tmp_path / f"hgemm_{M}_{N}_{K}.log").write_text(log)
    shapes, methods, table = performance.collect(str(tmp_path), include_naive=True)
    assert shapes == [(M, N, K)] and methods == expected
    # the JSON report
    rep = json.loads(report.read_text())
    assert (rep["M"], rep["N"], rep["K"]) == (M, N, K) and abs(rep["flops"] / (2.0 * M * N * K) - 1.0) < 1e-6
    assert [x["name"] for x in rep["results"]] == expected
    for x, line in zip(rep["results"], lines):
        assert x["checked"] and x["pass"] and x["rel_err"] <= 1e-2 * (K / 256) ** 0.5
        assert abs(x["tflops"] - float(line.split(" ")[14])) < 1e-3
        assert abs(x["tflops"] - table[(M, N, K)][x["name"]]["tflops"]) < 1e-3
    # the driver's inputs are the checker's fills for that seed
    assert int(rep["a_checksum"], 16) == checksum64(oracle.fill((M, K), rep["seed"], oracle.STREAM_A))
    assert int(rep["b_checksum"], 16) == checksum64(oracle.fill((N, K), rep["seed"], oracle.STREAM_B))


@pytest.mark.gpu
def test_driver_exit_codes_and_rotation(tmp_path):
    exe = _driver()
    print("[gpu] bin/hgemm unsupported shape", flush=True)
    r = subprocess.run([exe, "-M=100", "-N=128", "-K=256", "-variant=Mfma-Async-Stage4"], capture_output=True,
                       text=True, timeout=120)
    assert r.returncode == 1 and "cannot run M=100 N=128 K=256" in r.stderr and "Done" not in r.stderr
    r = subprocess.run([exe, "-variant=No-Such-Kernel"], capture_output=True, text=True, timeout=120)
    assert r.returncode == 1 and "unknown variant" in r.stderr
    # the default run skips variants that cannot tile the shape and still succeeds
    print("[gpu] bin/hgemm ragged default run", flush=True)
    r = subprocess.run([exe, "-M=100", "-N=136", "-K=192", "-enable_check=true", "-sleep_duration=10"],
                       capture_output=True, text=True, timeout=300)
    assert r.returncode == 0 and "Skipping Mfma-Async-Stage4" in r.stderr and "Auto exit, profiling time" in r.stderr
    # decode shape, HBM-cold: operands rotate, normal-distributed weights, checked
    print("[gpu] bin/hgemm rotating decode shape", flush=True)
    report = tmp_path / "decode.json"
    r = subprocess.run([exe, "-M=16", "-N=4096", "-K=4096", "-variant=Auto", "-enable_check=true", "-rotate_mb=300",
                        "-dist_a=normal", "-dist_b=normal:0.02", "-sleep_duration=10", f"-json={report}"],
                       capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    assert "Rotating over" in r.stderr and r.stderr.count("Check passed") == 2
    rep = json.loads(report.read_text())
    assert [x["name"] for x in rep["results"]] == ["Hipblaslt-Gemm", "Auto"] and rep["results"][1]["gbps"] > 100.0


@pytest.mark.gpu
def test_sweep_runner_on_real_logs(tmp_path):
    """python -m cuda_hgemm_amd.benchmark over three of the reference's dimensions that are
    not benchmark configurations, checked, then the plotter's tables from those logs."""
    from cuda_hgemm_amd import performance
    out = tmp_path / "log"
    print("[gpu] benchmark sweep 768,1536,5120", flush=True)
    r = subprocess.run([sys.executable, "-m", "cuda_hgemm_amd.benchmark", "--dims", "768,1536,5120", "--check",
                        "--variant", "Auto", "--iterations", "20", "--sleep-ms", "10", "--json", "--out", str(out)],
                       capture_output=True, text=True, timeout=600, cwd=ROOT)
    assert r.returncode == 0, (r.stdout, r.stderr)
    shapes, methods, table = performance.collect(str(out))
    assert shapes == [(768, 768, 768), (1536, 1536, 1536), (5120, 5120, 5120)] and methods == ["Hipblaslt-Gemm", "Auto"]
    for shape in shapes:
        assert table[shape]["Auto"]["tflops"] > 1.0 and table[shape]["Hipblaslt-Gemm"]["pct"] == 100.0
        rep = json.loads((out / "hgemm_{}_{}_{}.json".format(*shape)).read_text())
        assert all(x["checked"] and x["pass"] for x in rep["results"])
    assert performance.analyze(str(out)) == 0 and (out / "summary.md").exists()
