"""Sweep over every configuration of the benchmark specification: the counterpart of the
reference's ``benchmark_hgemm`` loop (run_sample.sh:29-37) plus the rectangular and
decode-shaped cases the reference cannot run.  Used by ``bench.py --sweep``.

Decode shapes are timed twice: on one operand set (whatever fits stays in the 256 MB
Infinity Cache) and rotating over enough copies of B that every call streams from HBM.
"""
from __future__ import annotations

PEAK_TFLOPS = 2500.0
PEAK_GBPS = 8000.0
SQUARES = [256, 512, 1024, 2048, 4096, 8192, 16384]
FFN = [(4096, 14336, 4096), (4096, 4096, 14336)]
DECODE_M = [1, 8, 16, 64, 128]
DECODE_NK = [(4096, 4096), (28672, 4096)]


def _draw(torch, dev, gen, rows, cols, dist):
    if dist == "uniform":
        return (torch.rand((rows, cols), device=dev, generator=gen, dtype=torch.float32) * 2.0 - 1.0).half()
    sigma = {"normal": 1.0, "weights": 0.02}[dist]
    return (torch.randn((rows, cols), device=dev, generator=gen, dtype=torch.float32) * sigma).half()


def _time(torch, lib, fn, As, Bs, Cs, m, n, k, warmup, steps):
    lib.profile_fn_rotating_ms(fn, As, Bs, Cs, m, n, k, 0, warmup)
    torch.cuda.synchronize()
    return lib.profile_fn_rotating_ms(fn, As, Bs, Cs, m, n, k, 0, steps)


def _row(lib, kind, m, n, k, ms, vms, extra=None):
    flops, nbytes = 2.0 * m * n * k, lib.bytes(m, n, k)
    tflops, gbps = flops / (ms * 1e-3) * 1e-12, nbytes / (ms * 1e-3) * 1e-9
    ai = flops / nbytes
    roof = min(PEAK_TFLOPS, ai * PEAK_GBPS * 1e-3)
    row = {"kind": kind, "M": m, "N": n, "K": k, "ms": ms, "tflops": tflops, "gbps": gbps, "pct_mfma_peak":
           100.0 * tflops / PEAK_TFLOPS, "pct_hbm_peak": 100.0 * gbps / PEAK_GBPS, "pct_roofline": 100.0 * tflops / roof,
           "vendor_ms": vms, "vendor_tflops": flops / (vms * 1e-3) * 1e-12, "pct_of_vendor": 100.0 * vms / ms,
           "plan": lib.auto_plan(m, n, k)}
    if extra:
        row.update(extra)
    return row


def run(torch, lib, vendor, warmup=10, steps=100):
    dev = torch.device("cuda:0")
    gen = torch.Generator(device=dev).manual_seed(20230212)
    auto, vfn = lib.variant_fn("hgemm_auto"), vendor.fn()
    rows = []
    for s in SQUARES:
        A, B = _draw(torch, dev, gen, s, s, "uniform"), _draw(torch, dev, gen, s, s, "uniform")
        C = torch.empty((s, s), dtype=torch.float16, device=dev)
        it = steps if s < 16384 else max(10, steps // 5)
        vms = _time(torch, lib, vfn, [A], [B], [C], s, s, s, warmup, it)
        ms = _time(torch, lib, auto, [A], [B], [C], s, s, s, warmup, it)
        rows.append(_row(lib, "square", s, s, s, ms, vms))
        del A, B, C
    for (m, n, k) in FFN:
        A, B = _draw(torch, dev, gen, m, k, "uniform"), _draw(torch, dev, gen, n, k, "weights")
        C = torch.empty((m, n), dtype=torch.float16, device=dev)
        vms = _time(torch, lib, vfn, [A], [B], [C], m, n, k, warmup, steps)
        ms = _time(torch, lib, auto, [A], [B], [C], m, n, k, warmup, steps)
        rows.append(_row(lib, "ffn", m, n, k, ms, vms))
        del A, B, C
    for (n, k) in DECODE_NK:
        copies = max(2, (768 << 20) // (n * k * 2) + 1)   # > 3x the 256 MB Infinity Cache in total
        Bs = [_draw(torch, dev, gen, n, k, "weights") for _ in range(copies)]
        for m in DECODE_M:
            As = [_draw(torch, dev, gen, m, k, "normal") for _ in range(copies)]
            Cs = [torch.empty((m, n), dtype=torch.float16, device=dev) for _ in range(copies)]
            warm_ms = _time(torch, lib, auto, As[:1], Bs[:1], Cs[:1], m, n, k, warmup, steps)
            cold_ms = _time(torch, lib, auto, As, Bs, Cs, m, n, k, warmup, steps)
            vcold_ms = _time(torch, lib, vfn, As, Bs, Cs, m, n, k, warmup, steps)
            rows.append(_row(lib, "decode", m, n, k, cold_ms, vcold_ms,
                             {"cache_warm_ms": warm_ms, "cache_warm_gbps": lib.bytes(m, n, k) / (warm_ms * 1e-3) * 1e-9,
                              "operand_sets": copies}))
        del Bs
    return {"peak_tflops": PEAK_TFLOPS, "peak_gbps": PEAK_GBPS, "warmup": warmup, "steps": steps, "rows": rows}


def print_table(report, file=None):
    import sys
    f = file or sys.stderr
    print("| kind | M | N | K | ms | TFLOPS | % MFMA peak | GB/s | % HBM peak | % roofline | hipBLASLt TFLOPS | % of hipBLASLt | kernel |",
          file=f)
    print("|---|---|---|---|---|---|---|---|---|---|---|---|---|", file=f)
    for r in report["rows"]:
        print(f"| {r['kind']} | {r['M']} | {r['N']} | {r['K']} | {r['ms']:.4f} | {r['tflops']:.1f} | "
              f"{r['pct_mfma_peak']:.1f} | {r['gbps']:.0f} | {r['pct_hbm_peak']:.1f} | {r['pct_roofline']:.1f} | "
              f"{r['vendor_tflops']:.1f} | {r['pct_of_vendor']:.1f} | {r['plan']['kernel']} x{r['plan']['splits']} |",
              file=f)
