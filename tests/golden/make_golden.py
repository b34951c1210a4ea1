"""Writes the golden fixtures of the packed GEMV path into this directory.

    python tests/golden/make_golden.py

Two kinds of vector are committed:

* ``known_answers.json`` -- hand-derived inputs and results (weight decode of
  single bytes, activation quantisation incl. a round-half-even case, three tiny
  GEMVs, the reference converter's all-ones fixture).  They are written out here
  literally; nothing computes them.
* ``gemv_*.npz`` -- small seeded problems with the C oracle's outputs (int32 group
  sums, fp32 result, bf16 bits, quantised activations).  The reference holds no
  numerical fixture for this path (its kernels are CUDA only and it ships no
  GEMV test), so these record the oracle after it was pinned by
  tests/test_oracle.py; they guard against later drift of the oracle and serve as
  inputs for the GPU parity test.
"""
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(HERE, "..", ".."))

KNOWN = {
    "t2_decode": [
        {"byte": 0x1B, "weights": [1, 0, -1, -2]},
        {"byte": 0xFF, "weights": [1, 1, 1, 1]},
        {"byte": 0xAA, "weights": [0, 0, 0, 0]},
        {"byte": 0x55, "weights": [-1, -1, -1, -1]},
    ],
    "q1_decode": [
        {"byte": 0xA5, "weights": [1, -1, 1, -1, -1, 1, -1, 1]},
        {"byte": 0x00, "weights": [-1] * 8},
        {"byte": 0xFF, "weights": [1] * 8},
    ],
    "act_quant": [
        {"x_head": [1.0] * 8, "x_fill": 1.0, "K": 128, "s": 127.0, "q_head": [127] * 8},
        {"x_head": [1.984375, 0.0078125, 0.0234375, 0.0390625, -0.0234375, 0.0], "x_fill": 0.0,
         "K": 128, "s": 64.0, "q_head": [127, 0, 2, 2, -2, 0]},
    ],
    # activations all 127 with multiplier s = 127 (x = 1.0 everywhere)
    "gemv": [
        {"bits": 2, "K": 128, "weight_byte": 0xFF, "ws": [0.5], "G": [16256], "y": 64.0},
        {"bits": 2, "K": 128, "weight_byte": 0x77, "ws": [0.5], "G": [0], "y": 0.0},
        {"bits": 2, "K": 256, "weight_byte": 0xFF, "ws": [1.0, 0.25], "G": [16256, 16256], "y": 160.0},
        {"bits": 1, "K": 128, "weight_byte": 0x00, "ws": [0.5], "G": [-16256], "y": -64.0},
    ],
    "converter_all_ones_128x128": {
        "t2": {"shape": [128, 32], "byte": 0xFF, "scale_shape": [128, 1], "scale_bf16_bits": 0x3F80},
        "q1": {"shape": [128, 16], "byte": 0xFF, "scale_shape": [128, 1], "scale_bf16_bits": 0x3F80},
    },
}

CASES = [("t2_m3_n8_k256", 2, 3, 8, 256, 101), ("t2_m2_n6_k2560", 2, 2, 6, 2560, 102),
         ("q1_m3_n8_k256", 1, 3, 8, 256, 103), ("q1_m2_n5_k1280", 1, 2, 5, 1280, 104)]


def main():
    from oracle import oracle as O
    with open(os.path.join(HERE, "known_answers.json"), "w") as f:
        json.dump(KNOWN, f, indent=1)
    for name, bits, M, N, K, seed in CASES:
        p = O.synth_problem(seed, M, N, K, bits)
        G = O.c_group_sums(p["A"], p["B"], bits)
        y32, y16 = O.c_gemv(p["A"], p["B"], p["s"], p["ws"], bits)
        np.savez_compressed(os.path.join(HERE, f"gemv_{name}.npz"), bits=bits, x=p["x"], A=p["A"],
                            s=p["s"], B=p["B"], ws=p["ws"], G=G, y32=y32, y16=y16)
        print("wrote", name)


if __name__ == "__main__":
    main()
