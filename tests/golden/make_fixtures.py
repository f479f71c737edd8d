#!/usr/bin/env python3
"""Writes the golden vectors in this directory. Run from the repository root:

    python tests/golden/make_fixtures.py

Route: numpy only. Weights are drawn as int8, packed with numpy packbits (LSB first),
and the expected outputs are exactly rounded sums (math.fsum) of the exact products
scale * weight * activation taken from a dense unpacked matrix. Neither the oracle
nor any reference code takes part, so the files pin the oracle rather than echo it.
"""
import json
import math
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from tests import synth  # noqa: E402


def make(name, seed, rows, cols, batch, group, p_zero, neg_scales):
    rng = np.random.default_rng(seed)
    w = synth.ternary_matrix(rng, rows, cols, p_zero)
    w[0, :] = 0                      # an all-zero row
    w[1, :] = 1                      # all +1
    w[2, :] = -1                     # all -1
    w[3, :] = 0
    w[3, cols - 1] = -1              # single non-zero in the last column
    nz, sg = synth.pack_np(w)
    sg = sg | (rng.integers(0, 2**32, nz.shape, dtype=np.uint64).astype(np.uint32) & ~nz)
    if neg_scales:                   # the reference's own GEMV test draws U(-0.1, 0.1)
        s = rng.uniform(-0.1, 0.1, (rows, cols // group)).astype(np.float16)
    else:
        s = rng.uniform(0.01, 0.03, (rows, cols // group)).astype(np.float16)
    x = rng.standard_normal((batch, cols)).astype(np.float16)
    dense = w.astype(np.float64) * np.repeat(s.astype(np.float64), group, axis=1)
    y = [[math.fsum((dense[r] * x[b].astype(np.float64)).tolist()) for r in range(rows)]
         for b in range(batch)]
    fx = {
        "name": name, "seed": seed, "rows": rows, "cols": cols, "batch": batch, "group": group,
        "nz": [f"{v:08x}" for v in nz.reshape(-1)],
        "sign": [f"{v:08x}" for v in sg.reshape(-1)],
        "scales": [f"{v:04x}" for v in s.view(np.uint16).reshape(-1)],
        "x": [f"{v:04x}" for v in x.view(np.uint16).reshape(-1)],
        "y_f64": [float(v).hex() for row in y for v in row],
    }
    with open(os.path.join(HERE, name + ".json"), "w") as f:
        json.dump(fx, f, separators=(",", ":"))
        f.write("\n")


if __name__ == "__main__":
    make("gemv_8x256_b2", 1001, 8, 256, 2, 128, 0.42, False)
    make("gemv_16x384_b3_negscale", 1002, 16, 384, 3, 128, 0.5, True)
    make("gemv_20x1024_b17", 1003, 20, 1024, 17, 128, 0.42, False)
