"""Pins the CPU oracle (oracle/) without the reference, which ships no golden vectors for this path and cannot
be built here. Each check is chosen so that a plausible mistake fails it: swapped up/gate roles, a transposed
operand, a dropped term, a wrong rounding mode, an off-by-one in the row interleave."""
import math
import os

import numpy as np
import pytest
import torch

from oracle import oracle
import fsw_weights

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def py_silu(x):
    return x / (1.0 + math.exp(-x))


def brute_mlp(X, Wg, Wu, Wd):
    """(silu(X@Wg) * (X@Wu)) @ Wd with Python loops over Python floats (doubles)."""
    M, d = len(X), len(X[0])
    ff = len(Wg[0])
    H = [[0.0] * ff for _ in range(M)]
    for m in range(M):
        for j in range(ff):
            g = sum(X[m][k] * Wg[k][j] for k in range(d))
            u = sum(X[m][k] * Wu[k][j] for k in range(d))
            H[m][j] = py_silu(g) * u
    Y = [[sum(H[m][j] * Wd[j][n] for j in range(ff)) for n in range(len(Wd[0]))] for m in range(M)]
    return H, Y


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_c_oracle_matches_brute_force_loops(dtype):
    inp = fsw_weights.make_inputs(5, 8, 6, dtype, seed=7)
    H_b, Y_b = brute_mlp(inp["X"].double().tolist(), inp["Wg"].double().tolist(), inp["Wu"].double().tolist(),
                         inp["Wd"].double().tolist())
    H_c = oracle.c_gateup(inp["X"], inp["W13"])
    Y_c = oracle.c_down(H_c, inp["W2"])
    assert torch.allclose(H_c, torch.tensor(H_b, dtype=torch.float64), rtol=1e-12, atol=1e-14)
    assert torch.allclose(Y_c, torch.tensor(Y_b, dtype=torch.float64), rtol=1e-12, atol=1e-14)


def test_silu_closed_forms():
    s = oracle.lib().oracle_silu
    assert s(0.0) == 0.0
    for x in (0.1, 0.5, 1.0, 2.5, 7.0, 20.0):
        assert abs((s(x) - s(-x)) - x) < 1e-14 * max(1, x)                 # silu(x) - silu(-x) = x
        assert abs((s(x) + s(-x)) - x * math.tanh(x / 2)) < 1e-14 * max(1, x)
    assert abs(s(40.0) - 40.0) < 1e-12 and abs(s(-40.0)) < 1e-12 and s(-40.0) <= 0.0
    # global minimum of silu: value -0.27846454276107..., at x = -1.27846454276107...
    xs = np.linspace(-2, -0.5, 150001)
    vals = np.array([s(float(x)) for x in xs])
    i = int(vals.argmin())
    assert abs(xs[i] - (-1.2784645427610738)) < 2e-5 and abs(vals[i] - (-0.2784645427610738)) < 1e-9
    # against torch's fp64 silu
    t = torch.linspace(-12, 12, 97, dtype=torch.float64)
    mine = torch.tensor([s(float(v)) for v in t], dtype=torch.float64)
    assert torch.allclose(mine, torch.nn.functional.silu(t), rtol=1e-13, atol=1e-15)


@pytest.mark.parametrize("impl", ["c", "torch"])
def test_even_rows_are_up_and_odd_rows_are_gate(impl):
    """One-hot probes: with X = I, C[m, n] = W13[n, m]. H[m, j] = C[m, 2j] * silu(C[m, 2j+1]) (swiglu.cu:380-381)."""
    K, ff = 8, 4
    X = torch.eye(K, dtype=torch.bfloat16)
    f = (lambda x, w: oracle.c_gateup(x, w)) if impl == "c" else (lambda x, w: oracle.ref_gateup(x, w, torch.float64))
    a, b = 3.0, -1.5
    W = torch.zeros((2 * ff, K), dtype=torch.bfloat16)
    W[2 * 2, 5] = a       # up row of feature 2, column 5
    W[2 * 2 + 1, 5] = b   # gate row of feature 2
    H = f(X, W)
    expect = torch.zeros((K, ff), dtype=torch.float64)
    expect[5, 2] = a * py_silu(b)          # NOT b * silu(a): the roles are asymmetric
    assert torch.allclose(H.double(), expect, atol=1e-12)
    assert abs(a * py_silu(b) - b * py_silu(a)) > 1.0
    # zeroing all odd (gate) rows kills H because silu(0) = 0; zeroing all even (up) rows kills it too
    g = torch.Generator().manual_seed(3)
    Wr = torch.randn((2 * ff, K), generator=g).to(torch.bfloat16)
    W0 = Wr.clone(); W0[1::2] = 0
    assert f(X, W0).abs().max().item() == 0.0
    W1 = Wr.clone(); W1[0::2] = 0
    assert f(X, W1).abs().max().item() == 0.0
    # feature j only depends on rows 2j and 2j+1
    W2 = Wr.clone(); W2[2:4] = 0
    Hr, H2 = f(X, Wr), f(X, W2)
    assert torch.equal(Hr[:, [0, 2, 3]], H2[:, [0, 2, 3]]) and H2[:, 1].abs().max().item() == 0.0


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_c_and_torch_statements_agree_and_match_unpacked_form(dtype):
    inp = fsw_weights.make_inputs(19, 40, 22, dtype, seed=11, x_scale=0.5)
    Y_c = oracle.c_mlp(inp["X"], inp["W13"], inp["W2"])
    Y_t64 = oracle.ref_mlp(inp["X"], inp["W13"], inp["W2"], torch.float64)
    Y_u64 = oracle.ref_mlp_unpacked(inp["X"], inp["Wg"], inp["Wu"], inp["Wd"], torch.float64)
    Y_t32 = oracle.ref_mlp(inp["X"], inp["W13"], inp["W2"], torch.float32)
    assert torch.allclose(Y_c, Y_t64, rtol=1e-11, atol=1e-13)
    assert torch.allclose(Y_c, Y_u64, rtol=1e-11, atol=1e-13)
    assert torch.allclose(Y_c, Y_t32.double(), rtol=2e-5, atol=2e-6)
    # the down projection alone reduces to a library GEMM
    Hh = oracle.ref_gateup(inp["X"], inp["W13"]).to(dtype)
    assert torch.allclose(oracle.c_down(Hh, inp["W2"]), Hh.double() @ inp["W2"].double().T, rtol=1e-12, atol=1e-14)


def test_invariants_of_the_formulation():
    inp = fsw_weights.make_inputs(7, 24, 10, torch.bfloat16, seed=5)
    X, W13, W2 = inp["X"], inp["W13"], inp["W2"]
    Y = oracle.c_mlp(X, W13, W2)
    # permuting ff jointly in W13 row pairs and W2 columns leaves Y unchanged
    perm = torch.randperm(10, generator=torch.Generator().manual_seed(1))
    W13p = W13.view(10, 2, 24)[perm].reshape(20, 24)
    W2p = W2[:, perm]
    assert torch.allclose(oracle.c_mlp(X, W13p, W2p), Y, rtol=1e-12, atol=1e-13)
    # Y is linear in the up rows: scaling them by 2 (exact in bf16) doubles Y; scaling gate rows does not
    W13u = W13.clone(); W13u[0::2] *= 2
    assert torch.allclose(oracle.c_mlp(X, W13u, W2), 2 * Y, rtol=1e-12, atol=1e-13)
    W13g = W13.clone(); W13g[1::2] *= 2
    assert not torch.allclose(oracle.c_mlp(X, W13g, W2), 2 * Y, rtol=1e-3, atol=1e-4)
    # row independence: row m of Y depends on row m of X only
    assert torch.allclose(oracle.c_mlp(X[3:4].contiguous(), W13, W2), Y[3:4], rtol=1e-12, atol=1e-14)


def test_decode_and_rounding_helpers_exhaustive():
    L = oracle.lib()
    codes = torch.arange(0, 65536, dtype=torch.int32).to(torch.int16)
    for tdtype, dec, enc in ((torch.bfloat16, L.oracle_bf16_to_f32, L.oracle_f32_to_bf16),
                             (torch.float16, L.oracle_f16_to_f32, L.oracle_f32_to_f16)):
        ref = codes.view(tdtype).float()
        step = 7  # every 7th code keeps the ctypes loop short and still hits every exponent and both signs
        for c in range(0, 65536, step):
            v = dec(c)
            r = ref[c].item()
            assert (math.isnan(v) and math.isnan(r)) or v == r, (tdtype, c)
            if not math.isnan(r):
                assert enc(r) == c, (tdtype, c)  # decode -> encode round trip is the identity
    # round-to-nearest-even on ties and near ties, against torch's conversion
    g = torch.Generator().manual_seed(9)
    vals = torch.cat([torch.randn(4000, generator=g) * 3, torch.randn(2000, generator=g) * 1e-6,
                      torch.tensor([1.00390625, 1.01171875, 65504.0, 65519.99, 65520.0, 1e-8, 5.96e-8, 3.0e-8,
                                    0.00006103515625, -2.5, 0.0, -0.0, float("inf")])])
    for tdtype, enc in ((torch.bfloat16, L.oracle_f32_to_bf16), (torch.float16, L.oracle_f32_to_f16)):
        want = vals.to(tdtype).view(torch.int16).to(torch.int32) & 0xFFFF
        for v, w in zip(vals.tolist(), want.tolist()):
            assert enc(v) == w, (tdtype, v, enc(v), w)


@pytest.mark.parametrize("name", ["tiny_bf16", "ragged_fp16", "block_bf16"])
def test_oracle_reproduces_committed_fixtures(name):
    z = np.load(os.path.join(GOLDEN, name + ".npz"))
    tdtype = torch.bfloat16 if int(z["dtype"]) == 0 else torch.float16
    as_t = lambda a: torch.from_numpy(a.view(np.int16).copy()).view(tdtype)
    X, W13, W2 = as_t(z["X"]), as_t(z["W13"]), as_t(z["W2"])
    H = oracle.c_gateup(X, W13)
    assert torch.equal(H, torch.from_numpy(z["H"]))
    assert torch.equal(oracle.c_down(H, W2), torch.from_numpy(z["Y"]))
    # and the torch statement agrees with the stored float64 values
    assert torch.allclose(oracle.ref_mlp(X, W13, W2, torch.float64), torch.from_numpy(z["Y"]), rtol=1e-11, atol=1e-13)


def test_error_metrics_and_gates():
    ref = torch.tensor([[1.0, -2.0], [4.0, 0.0]])
    out = ref + torch.tensor([[0.01, 0.0], [0.0, -0.03]])
    m = oracle.error_metrics(out, ref)
    assert abs(m["max_abs"] - 0.03) < 1e-6 and abs(m["mean_abs"] - 0.01) < 1e-6
    assert abs(m["mean_rel"] - 0.01 / 1.75) < 1e-6
    assert abs(m["fro_rel"] - math.sqrt(0.01 ** 2 + 0.03 ** 2) / math.sqrt(21.0)) < 1e-6
    assert not oracle.passes(m)
    assert oracle.passes(oracle.error_metrics(ref + 1e-4, ref))
    with pytest.raises(AssertionError):
        oracle.assert_parity(out, ref, "demo")
