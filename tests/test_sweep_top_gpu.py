"""The top of the reference's sweeps, once: numeric_tests.py:13-14 goes up to M = N = K = 65536 and
bench_swiglu.py:52-60 to 65536 tokens. One case at M = N = K = 32768 through the reference's operator, and one
whose output has more than 2^31 elements, where 32-bit element indices would wrap. Inputs are drawn on the device;
the oracle is evaluated in fp64 on sampled rows and features (the corners and the last elements among them)."""
import math

import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _sampled_gateup_check(H, X, W13, rows, feats, what):
    """H[rows][:, feats] against the fp64 formulation of numeric_tests.py:41-43 on the same rows / feature pairs."""
    Xs = X[rows.to(DEV)].cpu().double()
    idx = torch.stack([2 * feats, 2 * feats + 1], dim=1).flatten()
    Ws = W13[idx.to(DEV)].cpu().double()
    C = Xs @ Ws.T
    ref = C[:, 0::2] * torch.nn.functional.silu(C[:, 1::2])
    got = H[rows.to(DEV)][:, feats.to(DEV)].cpu().double()
    err = (got - ref).abs()
    bound = ref.abs() * 2.0 ** -7 + 1e-3  # one bf16 rounding of a correctly accumulated value
    assert not (err > bound).any(), "%s: worst |d| = %g" % (what, err.max().item())
    return err.max().item(), (err.norm() / ref.norm()).item()


def _sample(n, count, gen):
    """`count` indices of range(n): both ends, the 256-boundaries next to them, and random ones."""
    fixed = torch.tensor([0, 1, 255, 256, n - 257, n - 256, n - 2, n - 1])
    rnd = torch.randint(0, n, (count - len(fixed),), generator=gen)
    return torch.unique(torch.cat([fixed, rnd]).clamp_(0, n - 1))


def test_top_of_the_numeric_sweep_32768(ext):
    mnk = 32768
    g = torch.Generator(device=DEV).manual_seed(7)
    bound = 1.0 / math.sqrt(mnk)  # the law kaiming_uniform_(a=sqrt(5)) leaves (numeric_tests.py:8-10)
    X = torch.empty((mnk, mnk), device=DEV, dtype=torch.float32).uniform_(-bound, bound, generator=g).to(torch.bfloat16)
    W = torch.empty((mnk, mnk), device=DEV, dtype=torch.float32).uniform_(-bound, bound, generator=g).to(torch.bfloat16)
    H = ext.fused_swiglu_bf16(X, W)
    torch.cuda.synchronize()
    assert H.shape == (mnk, mnk // 2) and torch.isfinite(H.float()).all()
    cg = torch.Generator().manual_seed(8)
    mx, rel = _sampled_gateup_check(H, X, W, _sample(mnk, 40, cg), _sample(mnk // 2, 200, cg), "M=N=K=32768")
    print("\nM=N=K=32768 sampled: max |d| %.3e, relative Frobenius %.3e" % (mx, rel))
    # the reference's own statistic on a row block: against torch's bf16 formulation (numeric_tests.py:41-52)
    C = X[:2048] @ W.T
    theirs = C[:, ::2] * torch.nn.functional.silu(C[:, 1::2])
    d = H[:2048].float() - theirs.float()
    assert (d.norm() / theirs.float().norm()).item() < 2e-2


def test_output_beyond_two_to_the_31_elements(capi, ext):
    """M = 66000 tokens (ragged: 257.8 panels), K = 1024, N = 65536: H has 2.16e9 elements (4.3 GB), so element offsets
    of its last rows do not fit 31 bits. Gate/up through the reference's operator (X re-blocked, row-major H), then
    the down projection of that H with its blocked copy in scratch (a 4.3 GB re-block)."""
    M, K, N = 66000, 1024, 65536
    ff = N // 2
    assert M * ff > 2 ** 31
    g = torch.Generator(device=DEV).manual_seed(9)
    X = torch.randn((M, K), device=DEV, generator=g).to(torch.bfloat16)
    W = (torch.randn((N, K), device=DEV, generator=g) / math.sqrt(K)).to(torch.bfloat16)
    H = ext.fused_swiglu_bf16(X, W)
    torch.cuda.synchronize()
    cg = torch.Generator().manual_seed(10)
    rows, feats = _sample(M, 48, cg), _sample(ff, 200, cg)
    assert int(rows[-1]) * ff + int(feats[-1]) >= 2 ** 31
    _sampled_gateup_check(H, X, W, rows, feats, "M=66000 x ff=32768")
    # same bits as the C ABI without scratch (row-major X, another instance of the kernel) on the last panel
    tail = capi.gateup(X[M - 300:], W)
    assert (tail.float() - H[M - 300:].float()).abs().max().item() <= 2.0 ** -7 * H[M - 300:].float().abs().max().item() + 1e-3
    # down projection of the 4.3 GB H: 258 x 2 tiles of 256 x 256, H re-blocked into scratch first
    D = 512
    W2 = (torch.randn((D, ff), device=DEV, generator=g) / math.sqrt(ff)).to(torch.bfloat16)
    assert capi.lib().fsw_down_workspace_bytes(0, M, D, ff) == capi.lib().fsw_blocked_bytes(M, ff) > 2 ** 32
    Y = capi.down(H, W2)
    torch.cuda.synchronize()
    ref = H[rows.to(DEV)].cpu().double() @ W2.cpu().double().T
    err = (Y[rows.to(DEV)].cpu().double() - ref).abs()
    assert not (err > ref.abs() * 2.0 ** -7 + 2e-3).any(), "down projection of the large H: worst |d| = %g" % err.max().item()
