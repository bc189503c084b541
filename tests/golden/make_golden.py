"""Writes tests/golden/ref_cpu_kernel.npz: seeded inputs and the outputs of the REFERENCE's CPU kernel
(boilerplate/kernels/csrc/boilerplate_cpu.cpp::ternary_gemm, compiled from its own source into
oracle/_ref by oracle/Makefile). Run in the build container, where /root/reference exists:

    make -C oracle && python tests/golden/make_golden.py

Shapes are the reference's own test shapes (tests/test_ternary_cuda.py:27-38,69-87 and
tests/test_ternary.py:85-98) plus one ragged case per format. The fixture holds data only.
"""

from __future__ import annotations

import sys
from pathlib import Path

import numpy as np

HERE = Path(__file__).resolve().parent
sys.path.insert(0, str(HERE.parent))

from _util import orc, ref_gemm, reference_build  # noqa: E402

CASES = [  # (name, fmt, act, N, K, group, M, terms)
    *[(f"i8_{fmt}_K{K}_g{g}", fmt, "int8", 24, K, g, 5, 1) for fmt in ("tq1", "tq2") for K, g in ((256, 128), (300, 64), (130, 128))],
    *[(f"f32_{fmt}_K{K}_g{g}", fmt, "f32", 37, K, g, 15, 2) for fmt in ("tq1", "tq2")
      for K, g in ((256, 128), (640, 128), (200, 64), (1024, 256))],
    *[(f"i8_{fmt}_K4160_g128", fmt, "int8", 70, 4160, 128, 3, 1) for fmt in ("tq1", "tq2")],
    *[(f"i8_{fmt}_K7_g3", fmt, "int8", 5, 7, 3, 2, 1) for fmt in ("tq1", "tq2")],
]


def main() -> int:
    if reference_build() is None:
        print("oracle/_ref/boilerplate_cpu_ref.so is missing: run `make -C oracle` first", file=sys.stderr)
        return 1
    out = {}
    for idx, (name, fmt, act, N, K, group, M, terms) in enumerate(CASES):
        rng = np.random.default_rng(1000 + idx)
        G = -(-K // group)
        xf = rng.standard_normal((M, K)).astype(np.float32)
        if act == "int8":
            x, xs = orc.quant_act_int8(xf)
        else:
            x, xs = xf, np.ones(M, np.float32)
        y = np.zeros((M, N), np.float32)
        for t in range(terms):
            trits = rng.integers(-1, 2, (N, K)).astype(np.int8)
            scale = ((rng.random((N, G)) + 0.01) * (0.25 ** t)).astype(np.float16)
            packed = orc.pack(trits, fmt)
            y = ref_gemm(x, xs, packed, scale.astype(np.float32), K, group, fmt, out=y)  # accumulates, as stacked terms do
            out[f"{name}.packed{t}"] = packed
            out[f"{name}.scale{t}"] = scale
        out[f"{name}.x"] = x
        out[f"{name}.x_scale"] = xs
        out[f"{name}.meta"] = np.array([N, K, group, M, terms, 1 if fmt == "tq1" else 2, int(act == "int8")], np.int64)
        out[f"{name}.out"] = y
    np.savez_compressed(HERE / "ref_cpu_kernel.npz", **out)
    print(f"wrote {len(CASES)} cases to {HERE / 'ref_cpu_kernel.npz'}")
    return 0


if __name__ == "__main__":
    raise SystemExit(main())
