"""Edge values of the gating epilogue on the device, kernel family by kernel family: SiLU where 2^x overflows
(the case the comment at swiglu.cu:95 worries about), signed zeros, infinities and NaN in the inputs, 16-bit
denormals, and fp16 results beyond 65504. X is one-hot per row, so every pre-activation is a single weight element
and the expected H is up * silu(gate) of table values, evaluated by the fp64 oracle (numeric_tests.py:41-43)."""
import pytest
import torch

from oracle import oracle

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
# gate/up kernels by fsw_set_variant id: automatic, the six tiled instances, the weight-streaming kernel and the
# persistent streaming kernel (the last two take at most 64 and 16 rows)
GATEUP_VARIANTS = [-1, 0, 1, 2, 3, 4, 5, 100, 102]


def one_hot_problem(dtype, ups, gates, M=16, K=64, ff=72):
    """X[m] = e_m; W13 rows hold table values in their first M columns: H[m, j] = up(j, m) * silu(gate(j, m))."""
    X = torch.zeros((M, K), dtype=dtype)
    X[torch.arange(M), torch.arange(M)] = 1.0
    W13 = torch.zeros((2 * ff, K), dtype=dtype)
    for j in range(ff):
        for k in range(M):
            W13[2 * j, k] = ups[(j + k) % len(ups)]
            W13[2 * j + 1, k] = gates[(j + 3 * k) % len(gates)]
    return X, W13


def run_gateup(capi, variant, X, W13):
    try:
        if variant >= 0:
            capi.set_variant(0, variant)
        return capi.gateup(X.to(DEV), W13.to(DEV)).cpu()
    finally:
        capi.set_variant(0, -1)


@pytest.mark.parametrize("variant", GATEUP_VARIANTS)
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_silu_where_the_exponential_overflows(capi, variant, dtype):
    """gate = +-{0, 0.5, 20, 88, 90, 200}, up = +-3: exp(-gate) overflows fp32 from gate = -88.8 on, where
    x * rcp(1 + inf) must give -0 and never NaN; large positive gates must give up * gate exactly."""
    gates = [0.0, 0.5, -0.5, 20.0, -20.0, 88.0, -88.0, 90.0, -90.0, 200.0, -200.0]
    ups = [3.0, -3.0]
    X, W13 = one_hot_problem(dtype, ups, gates)
    H = run_gateup(capi, variant, X, W13)
    ref = oracle.ref_gateup(X, W13, torch.float64)
    assert torch.isfinite(H.float()).all(), "non-finite H for finite inputs"
    err = (H.double() - ref).abs()
    ulp = 2.0 ** -7 if dtype == torch.bfloat16 else 2.0 ** -10
    # one rounding of the exact value; results below the 16-bit normal range may be flushed (slack 1e-30 covers
    # bf16's, fp16 results below 6e-8 round to zero anyway)
    bound = ref.abs() * ulp + (1e-30 if dtype == torch.bfloat16 else 6e-8)
    assert not (err > bound).any(), "worst |d| = %g at ref %g" % (err.max().item(), ref.flatten()[err.argmax()].item())
    # the sign survives underflow: up * silu(-200) is -0 for up > 0, +0 for up < 0
    nz = ref != 0
    assert torch.equal(torch.signbit(H.float())[nz], (ref < 0)[nz]), "sign lost where the result underflows"
    # exact cases: silu(g) = g in fp32 for g >= 20
    big = (W13[1::2, :16].T.double() >= 20.0)  # [M, ff] gate table per (m, j)
    exact = (W13[0::2, :16].T.double() * W13[1::2, :16].T.double())
    assert torch.equal(H.double()[big], exact[big])


@pytest.mark.parametrize("variant", GATEUP_VARIANTS)
def test_infinities_and_nan_propagate_like_the_formula(capi, variant):
    """+-inf and NaN in X: the result is NaN / +-inf exactly where the fp64 formulation says (silu(-inf) is NaN:
    -inf * 0), and finite rows stay untouched by their neighbours."""
    dtype = torch.bfloat16
    gates = [2.0, -2.0, 0.5, -1.0, 3.0]
    ups = [1.5, -0.75, 2.0]
    X, W13 = one_hot_problem(dtype, ups, gates)
    X[1, 1] = float("inf")
    X[2, 2] = float("-inf")
    X[5, 5] = float("nan")
    X[7, 9] = float("inf")   # a second non-zero in row 7: finite + inf
    H = run_gateup(capi, variant, X, W13)
    ref = oracle.ref_gateup(X, W13, torch.float64)
    assert torch.equal(torch.isnan(H), torch.isnan(ref)), "NaN pattern differs from the formula's"
    assert torch.equal(torch.isinf(H), torch.isinf(ref)), "inf pattern differs from the formula's"
    inf = torch.isinf(ref)
    assert torch.equal(torch.signbit(H.float())[inf], (ref < 0)[inf])
    fin = torch.isfinite(ref)
    assert ((H.double() - ref).abs()[fin] <= ref.abs()[fin] * 2.0 ** -7 + 1e-6).all()
    clean = [m for m in range(16) if m not in (1, 2, 5, 7)]
    assert torch.isfinite(H[clean].float()).all()


@pytest.mark.parametrize("variant", GATEUP_VARIANTS)
def test_fp16_results_beyond_65504_round_to_infinity(capi, variant):
    """up * silu(gate) with exact products around the fp16 overflow boundary: 65504 and 65518.75 stay 65504, 65520
    and above become inf (round to nearest even on ONE rounding of the fp32 value), with the sign of the product."""
    dtype = torch.float16
    pairs = [(2047.0, 32.0), (238.25, 275.0), (1872.0, 35.0), (478.25, 137.0), (2048.0, 32.0), (1130.0, 58.0)]
    M, K, ff = 16, 64, 2 * len(pairs)
    X = torch.zeros((M, K), dtype=dtype)
    X[torch.arange(M), torch.arange(M)] = 1.0
    W13 = torch.zeros((2 * ff, K), dtype=dtype)
    for j in range(ff):
        u, gt = pairs[j % len(pairs)]
        for k in range(M):
            sign = -1.0 if (j >= len(pairs)) ^ (k % 2 == 1) else 1.0
            W13[2 * j, k] = sign * u
            W13[2 * j + 1, k] = gt
    H = run_gateup(capi, variant, X, W13)
    ref = oracle.ref_gateup(X, W13, torch.float64)  # exact: the products are integers or quarters below 2^17
    expect = ref.to(torch.float32).to(torch.float16)
    assert torch.isinf(expect).any() and (expect.abs() == 65504).any()
    assert torch.equal(H, expect)


def test_sixteen_bit_denormals_are_inputs_like_any_other(capi):
    """bf16 denormals (below 1.18e-38) times weights of 2^100: the fp64 formula gives pre-activations of 2^-30 and
    H = 2^-30 * silu(2^-30), about 4.3e-19. The matrix cores honour denormal inputs (they are not flushed to zero), so
    the result is held to one rounding of that value, not only to the contract's absolute gate."""
    dtype = torch.bfloat16
    M, K, ff = 16, 64, 40
    tiny = torch.tensor(2.0 ** -130, dtype=torch.float32).to(dtype)
    assert float(tiny) > 0 and float(tiny) < 1.18e-38
    X = torch.zeros((M, K), dtype=dtype)
    X[torch.arange(M), torch.arange(M)] = tiny
    W13 = torch.zeros((2 * ff, K), dtype=dtype)
    W13[:, :M] = torch.tensor(2.0 ** 100, dtype=torch.float32).to(dtype)
    H = capi.gateup(X.to(DEV), W13.to(DEV)).cpu()
    ref = oracle.ref_gateup(X, W13, torch.float64)
    assert torch.isfinite(H.float()).all()
    assert (H.double() - ref).abs().max().item() <= 2e-2
    assert (ref.abs() > 1e-19).all()
    assert ((H.double() - ref).abs() <= ref.abs() * 2.0 ** -7).all(), "denormal inputs were flushed: H = %g, formula %g" % (
        float(H[0, 0]), float(ref[0, 0]))


@pytest.mark.parametrize("M", [16, 300])
def test_non_finite_h_reaches_y_like_the_formula(capi, M):
    """The whole forward with an infinity and a NaN in X: Y is NaN / inf where (silu(X@Wg) * (X@Wu)) @ Wd is (the
    pattern does not depend on the summation order: inf - inf and anything + NaN are NaN in any order)."""
    dtype = torch.bfloat16
    d, ff = 256, 520
    g = torch.Generator().manual_seed(21)
    X = torch.randn((M, d), generator=g).to(dtype)
    W13 = (torch.randn((2 * ff, d), generator=g) / d ** 0.5).to(dtype)
    W2 = (torch.randn((d, ff), generator=g) / ff ** 0.5).to(dtype)
    X[3, 17] = float("inf")
    X[M - 2, 5] = float("nan")
    Y = capi.mlp(X.to(DEV), W13.to(DEV), W2.to(DEV)).cpu()
    ref = oracle.ref_mlp(X, W13, W2, torch.float64)
    assert torch.equal(torch.isnan(Y), torch.isnan(ref))
    assert torch.equal(torch.isinf(Y), torch.isinf(ref))
    fin = torch.isfinite(ref).all(dim=1)
    oracle.assert_parity(Y[fin], ref[fin], "rows without non-finite inputs, M=%d" % M)
