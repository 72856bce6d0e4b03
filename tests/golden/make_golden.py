#!/usr/bin/env python3
"""Writes the golden fixtures of tests/golden/ from the CPU oracle (oracle/awq_oracle.py).

The reference holds no stored vectors for this path (its only test draws unseeded random data on a
GPU), so these are regression vectors of the oracle itself -- the oracle is pinned independently by
tests/test_oracle.py (hand-derived packing words, closed forms, brute force, the plain-C restatement).
The hand-derived known-answer words of the packing rule are kept in kat_words.json.

Run from the repository root:  python tests/golden/make_golden.py
"""
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from oracle import awq_oracle as o  # noqa: E402


def case(dtype, K, N, g, M, seed):
    rng = np.random.default_rng(seed)
    w = (rng.standard_normal((N, K)) * 0.02).astype(np.float32)
    p = o.make_packed(w, g, dtype)
    x = o.to_bits16(rng.standard_normal((M, K)).astype(np.float32), dtype)
    bias = o.to_bits16(np.linspace(-1, 1, N).astype(np.float32), dtype)
    return {
        "w": w, "qweight": p["qweight"], "qzeros": p["qzeros"], "qscales": p["qscales"],
        "x": x, "bias": bias,
        "w_dequant": o.dequant(p["qweight"], p["qzeros"], p["qscales"], dtype),
        "y": o.linear_fp32(x, p["qweight"], p["qzeros"], p["qscales"], dtype),
        "y_bias": o.linear_fp32(x, p["qweight"], p["qzeros"], p["qscales"], dtype, o.from_bits16(bias, dtype)),
        "group_size": np.int64(g),
    }


def main():
    for dtype, K, N, g, M, seed in [("f16", 256, 128, 128, 5, 11), ("bf16", 256, 128, 128, 5, 12),
                                    ("f16", 128, 72, 32, 3, 13)]:
        np.savez_compressed(os.path.join(HERE, f"awq_{dtype}_K{K}_N{N}_g{g}.npz"), **case(dtype, K, N, g, M, seed))
    kat = {
        "order": [0, 2, 4, 6, 1, 3, 5, 7],
        "shifts": [0, 16, 4, 20, 8, 24, 12, 28],
        "words": [
            {"columns": [0, 1, 2, 3, 4, 5, 6, 7], "int32": 1966171168, "hex": "0x75316420"},
            {"columns": [8, 9, 10, 11, 12, 13, 14, 15], "int32": -38146904, "hex": "0xFDB9ECA8"},
            {"columns": [15] * 8, "int32": -1, "hex": "0xFFFFFFFF"},
            {"columns": [0, 1, 0, 0, 0, 0, 0, 0], "int32": 65536, "hex": "0x00010000"},
            {"columns": [0, 0, 0, 0, 0, 0, 0, 1], "int32": 268435456, "hex": "0x10000000"},
        ],
    }
    with open(os.path.join(HERE, "kat_words.json"), "w") as f:
        json.dump(kat, f, indent=1)


if __name__ == "__main__":
    main()
