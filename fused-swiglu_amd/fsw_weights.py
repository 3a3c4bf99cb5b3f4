"""Weight packing and seeded synthetic inputs for the SwiGLU MLP forward.

Packing follows the reference's layouts: W1W3 [2*ff, d] row-major with row 2j = up (linear) and row 2j+1 =
gate (SiLU) operand of output feature j (swiglu.cu:380-381, numeric_tests.py:41-43) — the memory order is
(up, gate) even though the tensor is named after Llama's w1 = gate, w3 = up — and W2 [d, ff] = Wd^T so that
the down projection is K-contiguous as well.
"""
import math

import torch

# (name, M, d, ff, dtype, seed, x_scale): the five benchmark configurations
CONFIGS = [
    ("C1", 512, 1024, 2816, torch.bfloat16, 0, 1.0),
    ("C2", 4096, 4096, 11008, torch.bfloat16, 1, 1.0),
    ("C3", 8192, 4096, 14336, torch.bfloat16, 2, 1.0),
    ("C4", 16, 4096, 14336, torch.bfloat16, 3, 1.0),
    ("C5", 2048, 8192, 28672, torch.float16, 4, 0.5),
]


def pack_w13(Wg, Wu):
    """Wg, Wu [d, ff] (mathematical orientation: X @ Wg) -> W1W3 [2*ff, d], rows (up_0, gate_0, up_1, gate_1, ...)."""
    assert Wg.shape == Wu.shape and Wg.dim() == 2
    d, ff = Wg.shape
    out = torch.empty((2 * ff, d), dtype=Wg.dtype, device=Wg.device)
    out[0::2] = Wu.T
    out[1::2] = Wg.T
    return out


def unpack_w13(W13):
    """Inverse of pack_w13: returns (Wg, Wu), each [d, ff]."""
    assert W13.dim() == 2 and W13.shape[0] % 2 == 0
    return W13[1::2].T.contiguous(), W13[0::2].T.contiguous()


def pack_wd(Wd):
    """Wd [ff, d] -> W2 [d, ff] (K-contiguous operand of the down projection)."""
    assert Wd.dim() == 2
    return Wd.T.contiguous()


def flops(M, d, ff):
    """Algorithmic FLOPs of one forward: two [M,d]x[d,ff] products and one [M,ff]x[ff,d] product."""
    return 6 * M * d * ff


def gateup_flops(M, d, ff):
    return 4 * M * d * ff


def reference_gateup_flops(M, N, K):
    """FLOP convention of the reference's benchmark for the gate/up kernel alone (bench_swiglu.py:117)."""
    return M * N * (2 * K - 1) + 6 * M * (N // 2)


def hbm_bytes(M, d, ff, elt=2):
    """Algorithmic HBM bytes of one forward: weights + X + Y + one write and one read of H."""
    return (3 * d * ff + 2 * M * d + 2 * M * ff) * elt


def make_inputs(M, d, ff, dtype, seed, x_scale=1.0):
    """Seeded synthetic inputs on the CPU: X ~ x_scale*N(0,1), W ~ N(0,1)/sqrt(fan_in), drawn in fp32 in the
    order X, Wg, Wu, Wd from one torch.Generator, then rounded to `dtype`.
    Returns dict(X, Wg, Wu, Wd, W13, W2) of CPU tensors in `dtype`."""
    g = torch.Generator().manual_seed(seed)
    X = torch.randn((M, d), generator=g, dtype=torch.float32)
    if x_scale != 1.0:
        X *= x_scale
    X = X.to(dtype)
    Wg = (torch.randn((d, ff), generator=g, dtype=torch.float32) / math.sqrt(d)).to(dtype)
    Wu = (torch.randn((d, ff), generator=g, dtype=torch.float32) / math.sqrt(d)).to(dtype)
    Wd = (torch.randn((ff, d), generator=g, dtype=torch.float32) / math.sqrt(ff)).to(dtype)
    return {"X": X, "Wg": Wg, "Wu": Wu, "Wd": Wd, "W13": pack_w13(Wg, Wu), "W2": pack_wd(Wd)}


def make_config(name):
    for cfg in CONFIGS:
        if cfg[0] == name:
            _, M, d, ff, dtype, seed, xs = cfg
            out = make_inputs(M, d, ff, dtype, seed, xs)
            out.update(name=name, M=M, d=d, ff=ff, dtype=dtype, seed=seed)
            return out
    raise KeyError(name)
