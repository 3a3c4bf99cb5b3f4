"""Writes the golden fixtures in this directory: small seeded inputs (as 16-bit encodings) and the float64
outputs of the C oracle (oracle/swiglu_oracle.c) for them. Nothing from the reference is executed; the reference
ships no fixtures for this path. Run from the repository root:  python tests/golden/gen_golden.py
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "fused-swiglu_amd"))

from oracle import oracle  # noqa: E402
import fsw_weights  # noqa: E402

# name, M, d, ff, dtype, seed, x_scale
CASES = [
    ("tiny_bf16", 5, 16, 8, torch.bfloat16, 101, 1.0),
    ("ragged_fp16", 17, 40, 12, torch.float16, 102, 0.5),
    ("block_bf16", 24, 64, 40, torch.bfloat16, 103, 1.0),
]


def bits(t):
    return t.contiguous().view(torch.int16).numpy().view(np.uint16).copy()


def main():
    for name, M, d, ff, dtype, seed, xs in CASES:
        inp = fsw_weights.make_inputs(M, d, ff, dtype, seed, xs)
        H = oracle.c_gateup(inp["X"], inp["W13"])
        Y = oracle.c_down(H, inp["W2"])
        np.savez_compressed(
            os.path.join(HERE, name + ".npz"),
            dtype=np.array(0 if dtype == torch.bfloat16 else 1),
            X=bits(inp["X"]), W13=bits(inp["W13"]), W2=bits(inp["W2"]),
            H=H.numpy(), Y=Y.numpy())
        print(name, "H", tuple(H.shape), "Y", tuple(Y.shape))


if __name__ == "__main__":
    main()
