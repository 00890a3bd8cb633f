#!/usr/bin/env python3
"""Writes tests/golden/mixed_qlinear_golden.npz: seeded inputs and expected outputs for the hot path.

The reference stores no vectors for this path (its tests evaluate formulas at run time:
test/python/test_quant.py, test_matmul.py, test_cuaprseLt.py, test_fused.py), so these are produced by the numpy
oracle (oracle/quik_oracle.py), which tests/test_oracle.py pins against those formulas, closed forms and the
scalar C restatement.  They are regression fixtures: tests/test_golden.py checks that the oracle still
reproduces them and that the HIP path gives the integer fields bit for bit and the fp16 fields within the
tolerance.  Run from the repo root:  python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import quik_oracle as qo  # noqa: E402

OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "mixed_qlinear_golden.npz")


def build():
    rng = np.random.default_rng(20240607)
    g = {}
    # ---- one layer per case: (tokens, out, in, outliers, bits, symmetric)
    cases = [(24, 40, 160, 32, 4, False), (24, 40, 160, 32, 8, False), (40, 72, 288, 32, 4, False),
             (24, 40, 160, 32, 4, True), (9, 33, 96, 0, 4, False)]
    g["cases"] = np.array(cases, dtype=np.int64)
    for i, (M, N, n_in, F, bits, symm) in enumerate(cases):
        fp_idx = rng.permutation(n_in)[:F].astype(np.int64)
        mask = np.ones(n_in, bool)
        mask[fp_idx] = False
        int_idx = np.arange(n_in, dtype=np.int64)[mask]
        x = rng.standard_normal((M, n_in)).astype(np.float32)
        x[:, fp_idx] *= 50
        x = x.astype(np.float16)
        x[0, :] = 1.5                                     # constant row: scale clamps at 1e-6
        x[1, int_idx[:8]] = [0, 0.5, 1.5, 2.5, 3.5, 4.5, 15, 7.5]
        x[2, :] *= np.float16(1e-4)                       # small range
        x[3, int_idx[3]] = 65504.0
        x[3, int_idx[4]] = -65504.0                       # range overflows fp16
        lo, hi = (-8, 8) if bits == 4 else (-127, 128)
        s_w = rng.uniform(0.001, 0.01, (N, 1)).astype(np.float16)
        W = np.zeros((N, n_in), np.float16)
        W[:, int_idx] = (rng.integers(lo, hi, (N, int_idx.size)) * s_w.astype(np.float32)).astype(np.float16)
        W[:, fp_idx] = (0.02 * rng.standard_normal((N, F))).astype(np.float16)
        bias = rng.standard_normal(N).astype(np.float16)
        mod = qo.from_float(W, s_w, fp_idx, bits, symm=bool(symm))
        out, inter = qo.mixed_qlinear_forward(x, mod, bits, bias, symm=bool(symm))
        p = f"c{i}_"
        g[p + "x"], g[p + "W"], g[p + "s_w"], g[p + "bias"], g[p + "fp_idx"] = x, W, s_w, bias, fp_idx
        g[p + "int_weight"] = mod["int_weight"]
        if not symm:
            g[p + "reduced_w"] = mod["reduced_w"]
            g[p + "meta"] = inter["meta"]
        else:
            g[p + "qscale"] = inter["qscale"]
        g[p + "qx"], g[p + "fp_x"], g[p + "acc"] = inter["qx"], inter["fp_x"], inter["acc"]
        g[p + "out"] = out
    return g


if __name__ == "__main__":
    np.savez_compressed(OUT, **build())
    print("wrote", OUT, os.path.getsize(OUT), "bytes")
