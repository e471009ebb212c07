#!/usr/bin/env python3
"""Writes tests/golden/tiny_vectors.npz: for each format (Q4_0, Q8_0) and two small shapes, the
seeded inputs and every intermediate of the activation-quantized route as the CPU oracle computes
them -- quantized activations, their scales and sums, the int32 block dots -- plus the op's f32
outputs (route chosen by the engine's gate; both associations of the scaled accumulate for the
activation-quantized route).  Shapes: rows = 5, in_dim = 256, out_dim = 64 (the op itself takes the
f32 route there: out_dim < 512) and rows = 5, in_dim = 96, out_dim = 512 (activation-quantized).

Run from the repository root:  python tests/golden/make_tiny_vectors.py
The fixture pins the oracle against silent change and gives the GPU tests vectors that do not
depend on the oracle being built."""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from antfly_amd import synth  # noqa: E402
from oracle import oracle as O  # noqa: E402

CASES = [("k256_n64", 5, 256, 64), ("k96_n512", 5, 96, 512)]
FORMATS = [("q4_0", O.FMT_Q4_0), ("q8_0", O.FMT_Q8_0)]


def build():
    out = {}
    for case, rows, in_dim, out_dim in CASES:
        for name, fmt in FORMATS:
            seed = 7000 + in_dim + fmt
            x = synth.activations(seed, rows, in_dim)
            w = synth.weights(fmt, seed + 1, out_dim, in_dim)
            q, s, sums = O.quantize_activation_rows(x, rows, in_dim)
            key = f"{name}_{case}_"
            out[key + "x"] = x
            out[key + "w_raw"] = w
            out[key + "qx"] = q
            out[key + "sx"] = s
            out[key + "sumx"] = sums
            out[key + "block_dots"] = O.block_dots(fmt, x, w, rows, in_dim, out_dim)
            out[key + "y_pair_assoc"] = O.linear_act_assoc(fmt, O.ASSOC_PAIR, x, w, rows, in_dim, out_dim)
            out[key + "y_single_assoc"] = O.linear_act_assoc(fmt, O.ASSOC_SINGLE, x, w, rows, in_dim, out_dim)
            out[key + "y_f32_route"] = O.linear_f32(fmt, x, w, rows, in_dim, out_dim)
            out[key + "y_op"] = O.linear_no_bias(fmt, x, w, rows, in_dim, out_dim, workers=1)
            out[key + "uses_activation_quant"] = np.array([int(O.uses_activation_quant(rows, in_dim, out_dim))])
    return out


if __name__ == "__main__":
    path = os.path.join(ROOT, "tests", "golden", "tiny_vectors.npz")
    np.savez_compressed(path, **build())
    print(path, os.path.getsize(path), "bytes")
