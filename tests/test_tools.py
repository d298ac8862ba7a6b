"""Host-side sweep runner and log plotter (counterparts of the reference's run_sample.sh
and tools/performance/performance.py); no GPU involved."""
import os

from cuda_hgemm_amd import benchmark, performance

PREFIX = "[HGEMM][INFO][tester.h:149][profile] "


def _line(name, ms, ms_pct, tflops, pct):
    # format of the driver's result line (reference src/common/tester.h:104-106)
    return PREFIX + "%s exit, profiling time: %.3f ms (%.2f%%), throughput: %.3f TFLOPS (%.2f%%)\n" % (
        name, ms, ms_pct, tflops, pct)


def test_reference_dimension_list():
    assert len(benchmark.DIMS) == 20 and benchmark.DIMS[0] == 256 and benchmark.DIMS[-1] == 16384
    assert benchmark.DIMS == sorted(benchmark.DIMS)
    sq = benchmark.shapes("square", benchmark.DIMS)
    assert sq[0] == (256, 256, 256) and sq[-1] == (16384, 16384, 16384) and len(sq) == 20
    wide = benchmark.shapes("wide", benchmark.DIMS)
    deep = benchmark.shapes("deep", benchmark.DIMS)
    assert len(wide) == len(deep) == 100
    assert all(m == n and m > k for (m, n, k) in wide)
    assert all(m == n and m < k for (m, n, k) in deep)


def test_driver_command_uses_reference_flags():
    class A:
        warmup, iterations, sleep_ms, check, naive, variant, json, out = 10, 100, 100, True, False, "Auto", False, "log"
    cmd = benchmark.driver_command(512, 2048, 1024, A)
    assert cmd[0].endswith("bin/hgemm")
    for flag in ("-M=512", "-N=2048", "-K=1024", "-warmup_iterations=10", "-profiling_iterations=100",
                 "-sleep_duration=100", "-enable_check=true", "-variant=Auto"):
        assert flag in cmd
    prof = benchmark.profiler_command(512, 2048, 1024, A)
    assert prof[0] == "rocprofv3" and prof[prof.index("--") + 1].endswith("bin/hgemm")
    assert "-profiling_iterations=1" in prof and A.iterations == 100
    assert "--kernel-trace" in prof and "--pmc" not in prof


def test_counter_sets_fit_one_pass_and_never_share_a_run_with_a_trace():
    class A:
        warmup, iterations, sleep_ms, check, naive, variant, json, out = 10, 100, 100, False, False, "Auto", False, "log"
    assert set(benchmark.PMC_SETS) >= {"mfma", "lds", "fetch", "write"}
    cost = {"FETCH_SIZE": ("TCC", 3), "WRITE_SIZE": ("TCC", 2)}
    limit = {"SQ": 8, "TCC": 4, "TCP": 4, "TA": 2, "TD": 2, "GRBM": 2}
    for name, counters in benchmark.PMC_SETS.items():
        used = {}
        for c in counters:
            block, n = cost.get(c, (c.split("_")[0], 1))
            used[block] = used.get(block, 0) + n
        assert all(used[b] <= limit[b] for b in used), (name, used)
        cmd = benchmark.profiler_command(8192, 8192, 8192, A, pmc=name)
        body = cmd[:cmd.index("--")]
        assert body[:2] == ["rocprofv3", "--pmc"] and body[2:2 + len(counters)] == counters
        assert not any(flag in body for flag in ("--kernel-trace", "--stats", "--sys-trace", "-s", "--hip-trace",
                                                 "--hsa-trace", "--memory-copy-trace", "--marker-trace", "-r"))
        assert cmd[cmd.index("--") + 1].endswith("bin/hgemm") and f"rocprof_{name}" in " ".join(cmd)
    assert benchmark.main(["--pmc", "nonsense", "--dims", "256"]) == 2


def test_parse_and_tables(tmp_path):
    for d, (v, a, n) in {256: (3.0, 6.0, 1.0), 1024: (200.0, 220.0, 50.0)}.items():
        with open(tmp_path / f"hgemm_{d}_{d}_{d}.log", "w") as fp:
            fp.write(PREFIX + "----------------- Evaluating Hipblaslt-Gemm -----------------\n")
            fp.write(_line("Hipblaslt-Gemm", 1.0, 100.0, v, 100.0))
            fp.write(_line("Mfma-Naive", 1.0 * v / n, 100.0 * v / n, n, 100.0 * n / v))
            fp.write(_line("Auto", 1.0 * v / a, 100.0 * v / a, a, 100.0 * a / v))
    (tmp_path / "other.log").write_text("noise\n")
    shapes, methods, table = performance.collect(str(tmp_path))
    assert shapes == [(256, 256, 256), (1024, 1024, 1024)]
    assert methods == ["Hipblaslt-Gemm", "Auto"]          # *Naive* left out, evaluation order kept
    assert table[(1024, 1024, 1024)]["Auto"]["tflops"] == 220.0
    assert abs(table[(256, 256, 256)]["Auto"]["pct"] - 200.0) < 1e-9
    _, methods_all, _ = performance.collect(str(tmp_path), include_naive=True)
    assert methods_all == ["Hipblaslt-Gemm", "Mfma-Naive", "Auto"]
    assert performance.analyze(str(tmp_path)) == 0
    md = (tmp_path / "summary.md").read_text()
    assert "| 1024 | 1024 | 1024 | 200.0 (100%) | 220.0 (110%) |" in md
    rows = (tmp_path / "summary.csv").read_text().splitlines()
    assert rows[0].startswith("M,N,K,Hipblaslt-Gemm TFLOPS,Auto TFLOPS") and len(rows) == 3
    try:
        import matplotlib  # noqa: F401
    except ImportError:
        return
    assert os.path.getsize(tmp_path / "throughput.png") > 1000
    assert os.path.getsize(tmp_path / "performance.png") > 1000


def test_empty_directory_is_an_error(tmp_path):
    assert performance.analyze(str(tmp_path)) == 1
