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


# ------------------------------------------------------------------ the build's resource guard
def _remarks(kernels):
    lines = []
    for name, (vgprs, agprs, scratch, spill) in kernels.items():
        tag = "x.hip:1:1: remark: "
        lines += [tag + f"Function Name: {name} [-Rpass-analysis=kernel-resource-usage]",
                  tag + "    SGPRs: 40 [-Rpass-analysis=kernel-resource-usage]",
                  tag + f"    VGPRs: {vgprs} [-Rpass-analysis=kernel-resource-usage]",
                  tag + f"    AGPRs: {agprs} [-Rpass-analysis=kernel-resource-usage]",
                  tag + f"    ScratchSize [bytes/lane]: {scratch} [-Rpass-analysis=kernel-resource-usage]",
                  tag + "    SGPRs Spill: 3 [-Rpass-analysis=kernel-resource-usage]",
                  tag + f"    VGPRs Spill: {spill} [-Rpass-analysis=kernel-resource-usage]"]
    return "\n".join(lines)


def test_build_guard_for_the_inline_assembly_kernels():
    """The build must fail when a hand-scheduled kernel (or the decode kernel that keeps A in registers) spills, when
    a chained kernel's AGPR count is not exactly its named accumulators (or its VGPRs reach 256), and when the guard
    finds nothing to check."""
    import pytest
    from cuda_hgemm_amd import build
    chained = "_ZN5hgemm20hgemm_chained_kernelINS_10PipeConfigILi256ELi256ELi64ELi2ELi2ELi2ELi16ELi1EEELb0ELb0EEEvPKDF16_"
    chained192 = "_ZN5hgemm20hgemm_chained_kernelINS_10PipeConfigILi192ELi192ELi64ELi2ELi2ELi3ELi16ELi0EEELb0ELb0EEEvPKDF16_"
    piped = "_ZN5hgemm22hgemm_pipelined_kernelINS_10PipeConfigILi128ELi128ELi64ELi2ELi2ELi5ELi16ELi0EEELb0ELb0EEEvPKDF16_"
    resident = "_ZN5hgemm28hgemm_decode_resident_kernelILi1ELi16ELb1EEEvPKDF16_S2_PDF16_iiii"
    other = "_ZN5hgemm15pad_copy_kernelEPKDF16_PDF16_iiii"
    assert build._chained_accumulator_registers(chained) == 256
    assert build._chained_accumulator_registers(chained192) == 144
    good = {chained: (179, 256, 0, 0), chained192: (139, 144, 0, 0), piped: (88, 64, 0, 0), resident: (160, 0, 0, 0),
            other: (11, 0, 16, 2)}
    assert build._check_no_spills("dispatch.hip", _remarks(good)) == {"hgemm_chained_kernel", "hgemm_pipelined_kernel",
                                                                      "hgemm_decode_resident_kernel"}
    for bad in ({**good, piped: (88, 64, 8, 0)},             # scratch
                {**good, chained: (179, 256, 0, 1)},         # a spilled VGPR
                {**good, chained: (179, 260, 0, 0)},         # the compiler took AGPRs of its own
                {**good, chained192: (139, 128, 0, 0)},      # fewer AGPRs than named accumulators
                {**good, chained: (256, 256, 0, 0)},         # VGPRs exhausted
                {**good, resident: (255, 0, 24, 6)},         # the rows of A it keeps in registers went to scratch
                {other: (11, 0, 0, 0)},                      # nothing to check in a file that must have such kernels
                {piped: (88, 64, 0, 0)}):                    # ... or only one of the kinds
        with pytest.raises(RuntimeError):
            build._check_no_spills("dispatch.hip", _remarks(bad))
    with pytest.raises(RuntimeError):                        # a remark format the parser does not understand
        build._check_no_spills("dispatch.hip", _remarks(good).replace("VGPRs:", "ArchVGPRs:"))
    assert build._check_no_spills("basic_kernels.hip", _remarks({other: (11, 0, 16, 2)})) == set()
