"""Writes the committed fixtures of this directory.  Run from the repository root:

    python tests/golden/make_golden.py

* ``rng_first_values.json``: the first 16 values (fp16 bit patterns) of the seeded input
  generator for each distribution / stream / seed used by the tests and the benchmark.
  They pin the generator against accidental change; they were produced by the generator
  itself and checked here against an independent pure-Python restatement of splitmix64.
* ``gemm_*.npz``: small products whose expected outputs come from numpy in float64
  (``A.astype(float64) @ B.T``), rounded once to fp16 by numpy -- an implementation that
  shares no code with the C checker.  The reference project holds no vectors of its own
  (its inputs are seeded from std::random_device, src/common/matrix.h:28-29).
"""
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from oracle import oracle as o  # noqa: E402

MASK = (1 << 64) - 1


def splitmix64(z):
    z = (z + 0x9E3779B97F4A7C15) & MASK
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & MASK
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & MASK
    return z ^ (z >> 31)


def rng_u64(seed, stream, index):
    key = splitmix64(seed ^ ((stream * 0xD1342543DE82EF95) & MASK))
    return splitmix64((key + index * 0x9E3779B97F4A7C15) & MASK)


def uniform_bits(seed, stream, n, lo=-1.0, hi=1.0):
    out = []
    for i in range(n):
        r = rng_u64(seed, stream, i)
        u = np.float32(r >> 40) * np.float32(1.0 / 16777216.0)
        v = np.float32(lo) + (np.float32(hi) - np.float32(lo)) * u
        out.append(int(np.float32(v).astype(np.float16).view(np.uint16)))
    return out


def main():
    fixtures = {"seed": o.DEFAULT_SEED, "cases": []}
    for stream in (1, 2):
        for dist, p0, p1, name in ((o.UNIFORM, -1.0, 1.0, "uniform[-1,1)"), (o.NORMAL, 0.0, 1.0, "normal(0,1)"),
                                   (o.NORMAL, 0.0, 0.02, "normal(0,0.02)"), (o.TERNARY, 0.0, 1.0, "ternary{-1,0,1}")):
            vals = o.fill((16,), o.DEFAULT_SEED, stream, dist, p0, p1)
            fixtures["cases"].append({"stream": stream, "dist": dist, "p0": p0, "p1": p1, "name": name,
                                      "first16": [int(v) for v in vals]})
    # independent restatement of the uniform path must agree before anything is written
    for case in fixtures["cases"]:
        if case["dist"] == o.UNIFORM:
            assert uniform_bits(o.DEFAULT_SEED, case["stream"], 16) == case["first16"], case
    with open(os.path.join(HERE, "rng_first_values.json"), "w") as f:
        json.dump(fixtures, f, indent=1)

    shapes = {"gemm_32x32x64": (32, 32, 64), "gemm_48x80x96": (48, 80, 96), "gemm_1x128x256": (1, 128, 256),
              "gemm_64x64x1024": (64, 64, 1024)}
    for name, (M, N, K) in shapes.items():
        A = o.fill((M, K), o.DEFAULT_SEED, o.STREAM_A)
        B = o.fill((N, K), o.DEFAULT_SEED, o.STREAM_B)
        Cd = A.view(np.float16).astype(np.float64) @ B.view(np.float16).astype(np.float64).T
        C = Cd.astype(np.float16).view(np.uint16)
        np.savez_compressed(os.path.join(HERE, name + ".npz"), A=A, B=B, C=C, C_f64=Cd)
    print("fixtures written to", HERE)


if __name__ == "__main__":
    main()
