"""The top of the reference's sweeps, once each: numeric_tests.py:13-14 goes up to M = N = K = 65536 and
bench_swiglu.py:52-60 to 65536 tokens at K = 8192, N = 57344 with a [M, N] output buffer (bench_swiglu.py:91,106).
Both top points, a case at M = N = K = 32768, and one whose output has more than 2^31 elements, where 32-bit element
indices would wrap. Inputs are drawn on the device; the oracle is evaluated in fp64 on sampled rows and features
(the corners and the last elements among them)."""
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


def _uniform_bf16(rows, cols, bound, gen, chunk=8192):
    """[rows, cols] bf16 ~ U(-bound, bound), drawn in row chunks (the fp32 draw of 65536 x 65536 at once is 17 GB)."""
    out = torch.empty((rows, cols), device=DEV, dtype=torch.bfloat16)
    for r in range(0, rows, chunk):
        n = min(chunk, rows - r)
        out[r:r + n] = torch.empty((n, cols), device=DEV, dtype=torch.float32).uniform_(-bound, bound, generator=gen).to(torch.bfloat16)
    return out


def test_top_of_the_numeric_sweep_65536(ext):
    """The last point of numeric_tests.py:13 through the operator it calls (numeric_tests.py:46): 8.6 GB per operand,
    weight panels whose rows lie 128 KB apart, row offsets of X and H beyond 2^32 bytes."""
    mnk = 65536
    g = torch.Generator(device=DEV).manual_seed(11)
    bound = 1.0 / math.sqrt(mnk)
    X = _uniform_bf16(mnk, mnk, bound, g)
    W = _uniform_bf16(mnk, mnk, bound, g)
    H = ext.fused_swiglu_bf16(X, W)
    torch.cuda.synchronize()
    assert H.shape == (mnk, mnk // 2)
    cg = torch.Generator().manual_seed(12)
    mx, rel = _sampled_gateup_check(H, X, W, _sample(mnk, 40, cg), _sample(mnk // 2, 200, cg), "M=N=K=65536")
    print("\nM=N=K=65536 sampled: max |d| %.3e, relative Frobenius %.3e" % (mx, rel))
    # every row block was written: column sums of H over all rows against those of the bf16 torch formulation on a
    # block of features (one GEMM of 65536 x 65536 x 512)
    feats = torch.arange(20000, 20256, device=DEV)
    idx = torch.stack([2 * feats, 2 * feats + 1], dim=1).flatten()
    C = (X @ W[idx].T).float()
    theirs = C[:, 0::2] * torch.nn.functional.silu(C[:, 1::2])
    d = H[:, feats].float() - theirs
    assert (d.norm() / theirs.norm()).item() < 2e-2


def test_top_of_the_benchmark_sweep_65536_tokens(ext):
    """The last point of bench_swiglu.py:52-60 the way the benchmark calls the operator (bench_swiglu.py:84-91,106):
    swiglu_fwd_bf16 with a [M, N] output buffer and ldC = N, so H occupies the first half of the buffer as dense rows
    of N / 2 (swiglu.cu:414) and the second half is never written."""
    M, K, N = 65536, 8192, 57344
    g = torch.Generator(device=DEV).manual_seed(13)
    X = torch.randn((M, K), device=DEV, generator=g).to(torch.bfloat16)
    W = (torch.randn((N, K), device=DEV, generator=g) / math.sqrt(K)).to(torch.bfloat16)
    C = torch.full((M, N), float("nan"), device=DEV, dtype=torch.bfloat16)
    ext.swiglu_fwd_bf16(M, N, K, X, K, W, K, C, N)
    torch.cuda.synchronize()
    flat = C.view(-1)
    H = flat[: M * (N // 2)].view(M, N // 2)
    assert torch.isnan(flat[M * (N // 2):]).all(), "the second half of the [M, N] buffer was written"
    nan_rows = torch.isnan(H).any(dim=1)
    assert not nan_rows.any(), "%d rows of H hold unwritten elements" % int(nan_rows.sum())
    cg = torch.Generator().manual_seed(14)
    _sampled_gateup_check(H, X, W, _sample(M, 40, cg), _sample(N // 2, 200, cg), "65536 tokens, K=8192, N=57344")


def test_output_beyond_two_to_the_31_elements(capi, ext):
    """M = 66000 tokens (ragged: 257.8 panels), K = 1024, N = 65536: H has 2.16e9 elements (4.3 GB), so element offsets
    of its last rows do not fit 31 bits. Gate/up through the reference's operator (row-major H), then the down
    projection of that H, then the same two steps with H panel-blocked (the form fsw_mlp keeps it in)."""
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
    # down projection of the 4.3 GB H: 258 x 2 tiles of 256 x 256 on row-major H
    D = 512
    W2 = (torch.randn((D, ff), device=DEV, generator=g) / math.sqrt(ff)).to(torch.bfloat16)
    L = capi.lib()
    assert L.fsw_down_workspace_bytes(0, M, D, ff) == 0 and capi.variant_name(1, 0, M, D, ff) == "pair16_256x256"
    Y = capi.down(H, W2)
    torch.cuda.synchronize()
    ref = H[rows.to(DEV)].cpu().double() @ W2.cpu().double().T
    err = (Y[rows.to(DEV)].cpu().double() - ref).abs()
    assert not (err > ref.abs() * 2.0 ** -7 + 2e-3).any(), "down projection of the large H: worst |d| = %g" % err.max().item()
    # the same forward with H panel-blocked in between (4.3 GB of blocks, byte offsets beyond 2^32): same bits
    assert L.fsw_blocked_bytes(M, ff) > 2 ** 32
    Hb = torch.empty(L.fsw_blocked_bytes(M, ff), dtype=torch.uint8, device=DEV)
    stream = torch.cuda.current_stream().cuda_stream
    capi.check(L.fsw_gateup_hblocked(0, M, N, K, X.data_ptr(), K, W.data_ptr(), K, 0, Hb.data_ptr(), stream))
    Yb = torch.empty_like(Y)
    capi.check(L.fsw_down_blocked(0, M, D, ff, Hb.data_ptr(), W2.data_ptr(), ff, 0, Yb.data_ptr(), D, stream))
    assert torch.equal(Yb, Y)
