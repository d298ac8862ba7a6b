"""Tables and line charts from the driver's logs: the counterpart of the reference's
``tools/performance/performance.py``.

Reads every ``hgemm_<M>_<N>_<K>.log`` in a directory (written by
``cuda_hgemm_amd.benchmark`` or by hand with ``bin/hgemm ... > log/hgemm_M_N_K.log``),
takes the per-variant result line

    <Name> exit, profiling time: <ms> ms (<%>), throughput: <TFLOPS> TFLOPS (<%>)

(format of the reference, src/common/tester.h:104-106) and writes

    summary.md / summary.csv   one row per shape, one column per variant
    throughput.png             TFLOPS per variant over the shapes
    performance.png            % of the first variant evaluated (hipBLASLt), as the
                               reference's chart is % of cuBLAS

    python -m cuda_hgemm_amd.performance --path log/

As in the reference's charts (performance.py:29,58) variants whose name contains "Naive"
are left out unless --naive is given.  Charts need matplotlib; without it only the tables
are written.
"""
from __future__ import annotations

import argparse
import csv
import os
import re
import sys

RESULT = re.compile(r"(\S+) exit, profiling time: ([0-9.]+) ms \(([0-9.]+)%\), "
                    r"throughput: ([0-9.]+) TFLOPS \(([0-9.]+)%\)")
LOG_NAME = re.compile(r"^hgemm_(\d+)_(\d+)_(\d+)\.log$")


def parse_log(path: str) -> list[dict]:
    """Result lines of one log, in evaluation order."""
    rows = []
    with open(path, errors="replace") as fp:
        for line in fp:
            m = RESULT.search(line)
            if m:
                rows.append({"name": m.group(1), "ms": float(m.group(2)), "ms_pct": float(m.group(3)),
                             "tflops": float(m.group(4)), "pct": float(m.group(5))})
    return rows


def collect(path: str, include_naive: bool = False):
    """(shapes, methods, table) with table[shape][method] = result row.  Shapes are sorted
    by (M, N, K); methods keep the order of their first appearance."""
    table, methods = {}, []
    for name in sorted(os.listdir(path)):
        m = LOG_NAME.match(name)
        if not m:
            continue
        shape = tuple(int(x) for x in m.groups())
        rows = parse_log(os.path.join(path, name))
        if not rows:
            continue
        table[shape] = {}
        for r in rows:
            if "Naive" in r["name"] and not include_naive:
                continue
            table[shape][r["name"]] = r
            if r["name"] not in methods:
                methods.append(r["name"])
    return sorted(table), methods, table


def shape_label(shape, all_square: bool) -> str:
    return str(shape[0]) if all_square else "x".join(str(d) for d in shape)


def write_tables(path: str, shapes, methods, table) -> None:
    with open(os.path.join(path, "summary.csv"), "w", newline="") as fp:
        w = csv.writer(fp)
        w.writerow(["M", "N", "K"] + [f"{m} TFLOPS" for m in methods] + [f"{m} %" for m in methods])
        for s in shapes:
            cells = [table[s].get(m) for m in methods]
            w.writerow(list(s) + [f"{c['tflops']:.3f}" if c else "" for c in cells] +
                       [f"{c['pct']:.2f}" if c else "" for c in cells])
    with open(os.path.join(path, "summary.md"), "w") as fp:
        fp.write("TFLOPS (% of the first variant evaluated)\n\n")
        fp.write("| M | N | K | " + " | ".join(methods) + " |\n")
        fp.write("|---|---|---|" + "---|" * len(methods) + "\n")
        for s in shapes:
            cells = [table[s].get(m) for m in methods]
            fp.write(f"| {s[0]} | {s[1]} | {s[2]} | " +
                     " | ".join(f"{c['tflops']:.1f} ({c['pct']:.0f}%)" if c else "-" for c in cells) + " |\n")


def draw(path: str, shapes, methods, table, key: str, file_name: str, y_label: str, title: str) -> bool:
    try:
        import matplotlib
        matplotlib.use("Agg")
        import matplotlib.pyplot as plt
    except ImportError:
        return False
    all_square = all(s[0] == s[1] == s[2] for s in shapes)
    labels = [shape_label(s, all_square) for s in shapes]
    fig, ax = plt.subplots(figsize=(16, 10), dpi=100)
    styles = ["-", "--", "-.", ":"]
    for i, m in enumerate(methods):
        ys = [table[s][m][key] if m in table[s] else float("nan") for s in shapes]
        ax.plot(labels, ys, marker="o", markersize=4, linestyle=styles[(i // 10) % len(styles)], label=m)
    ax.set_ylim(bottom=0)
    ax.grid(True, linestyle="-.")
    ax.set_xlabel("Matrix Dimension / M = N = K" if all_square else "M x N x K")
    ax.set_ylabel(y_label)
    ax.set_title(title)
    if not all_square:
        ax.tick_params(axis="x", labelrotation=60)
    ax.legend(loc="best", fontsize=9)
    fig.tight_layout()
    fig.savefig(os.path.join(path, file_name))
    plt.close(fig)
    return True


def analyze(path: str, include_naive: bool = False) -> int:
    shapes, methods, table = collect(path, include_naive)
    if not shapes:
        print(f"no hgemm_<M>_<N>_<K>.log with result lines under {path}", file=sys.stderr)
        return 1
    write_tables(path, shapes, methods, table)
    ok = draw(path, shapes, methods, table, "tflops", "throughput.png", "Throughput / TFLOPS", "HGEMM Throughput")
    ok = draw(path, shapes, methods, table, "pct", "performance.png", "Performance Compared with hipBLASLt / %",
              "HGEMM Performance") and ok
    if not ok:
        print("matplotlib is not importable: wrote summary.md and summary.csv only", file=sys.stderr)
    print(f"{len(shapes)} shapes x {len(methods)} variants -> {path}")
    return 0


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("-p", "--path", default="log/", help="directory holding the logs")
    ap.add_argument("--naive", action="store_true", help="keep the variants named *Naive*")
    args = ap.parse_args(argv)
    return analyze(args.path, args.naive)


if __name__ == "__main__":
    sys.exit(main())
