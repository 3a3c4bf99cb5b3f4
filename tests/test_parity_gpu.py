"""Parity of the HIP path against the CPU oracle on the same seeded inputs, through the C ABI (fsw_capi) and
through the PyTorch operator surface. Gates: max|d| <= 2e-2 and mean-relative error <= 5e-3 against the fp32/fp64
formulation (silu(X@Wg) * (X@Wu)) @ Wd; kernel-level checks are tighter (one rounding of a correctly
accumulated value)."""
import os

import numpy as np
import pytest
import torch

from oracle import oracle
import fsw_weights

pytestmark = pytest.mark.gpu
GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
DEV = "cuda:0"


def ulp_rel(dtype):
    return 2.0 ** -8 if dtype == torch.bfloat16 else 2.0 ** -11  # half an ulp, relative


def assert_one_rounding(out, ref64, dtype, what, slack=1e-3):
    """out must be ref rounded once to `dtype`, up to fp32 accumulation-order noise."""
    out64 = out.detach().cpu().double()
    err = (out64 - ref64).abs()
    bound = ref64.abs() * (2 * ulp_rel(dtype)) + slack
    bad = err > bound
    assert not bad.any(), "%s: %d elements beyond one rounding; worst |d|=%g at ref=%g" % (
        what, int(bad.sum()), err[bad].max().item(), ref64[bad][err[bad].argmax()].item())


def to_dev(inp):
    return {k: (v.to(DEV) if torch.is_tensor(v) else v) for k, v in inp.items()}


# ---------------------------------------------------------------------------------------------------------------
# golden fixtures and small seeded shapes, every kernel variant
# ---------------------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("name", ["tiny_bf16", "ragged_fp16", "block_bf16"])
def test_golden_fixtures(capi, name):
    z = np.load(os.path.join(GOLDEN, name + ".npz"))
    tdtype = torch.bfloat16 if int(z["dtype"]) == 0 else torch.float16
    as_t = lambda a: torch.from_numpy(a.view(np.int16).copy()).view(tdtype).to(DEV)
    X, W13, W2 = as_t(z["X"]), as_t(z["W13"]), as_t(z["W2"])
    H = capi.gateup(X, W13)
    assert_one_rounding(H, torch.from_numpy(z["H"]), tdtype, name + " H")
    if H.shape[1] % 8:
        # the down projection reads H and W2 in 16-byte vectors along ff: ff % 8 != 0 is refused, not mis-computed
        with pytest.raises(capi.FswError) as ei:
            capi.mlp(X, W13, W2)
        assert ei.value.code == capi.E_ALIGN
        return
    Y = capi.mlp(X, W13, W2)
    oracle.assert_parity(Y, torch.from_numpy(z["Y"]), name + " Y")


SMALL_SHAPES = [  # (M, d, ff) with ff % 8 == 0: ragged M and d, K tails, single rows, tile edges
    (1, 8, 8), (1, 64, 8), (3, 24, 16), (16, 64, 16), (17, 72, 40), (31, 136, 136), (33, 200, 120),
    (64, 64, 128), (65, 264, 136), (127, 320, 264), (128, 512, 64), (129, 1000, 136), (255, 128, 248),
    (256, 256, 256), (257, 64, 304), (300, 448, 520), (513, 96, 264),
]
GATEUP_ONLY_SHAPES = [  # any ff (odd, prime, below one vector): exercises the scalar store path and odd ldh
    (1, 8, 1), (3, 24, 5), (17, 72, 33), (33, 200, 127), (65, 264, 129), (129, 64, 131), (255, 128, 255), (70, 32, 3),
]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("shape", SMALL_SHAPES)
def test_small_shapes_auto_dispatch(capi, shape, dtype):
    M, d, ff = shape
    inp = fsw_weights.make_inputs(M, d, ff, dtype, seed=1000 + M + d + ff, x_scale=0.5 if dtype == torch.float16 else 1.0)
    g = to_dev(inp)
    H = capi.gateup(g["X"], g["W13"])
    H64 = oracle.ref_gateup(inp["X"], inp["W13"], torch.float64)
    assert_one_rounding(H, H64, dtype, "H %s" % (shape,))
    # the down kernel on its own: oracle fed with the GPU's H
    Y = capi.down(H, g["W2"])
    assert_one_rounding(Y, oracle.ref_down(H.cpu(), inp["W2"], torch.float64), dtype, "Y|H %s" % (shape,))
    # whole forward against the unrounded formulation in its unpacked form
    Yf = capi.mlp(g["X"], g["W13"], g["W2"])
    assert torch.equal(Yf, Y)
    oracle.assert_parity(Yf, oracle.ref_mlp_unpacked(inp["X"], inp["Wg"], inp["Wu"], inp["Wd"], torch.float64),
                         "mlp %s" % (shape,))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("shape", GATEUP_ONLY_SHAPES)
def test_gateup_any_ff(capi, shape, dtype):
    M, d, ff = shape
    inp = fsw_weights.make_inputs(M, d, ff, dtype, seed=2000 + M + d + ff, x_scale=0.5)
    H = capi.gateup(inp["X"].to(DEV), inp["W13"].to(DEV))
    assert_one_rounding(H, oracle.ref_gateup(inp["X"], inp["W13"], torch.float64), dtype, "H %s" % (shape,))


@pytest.mark.parametrize("variant", list(range(6)))
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_every_tiled_variant(capi, variant, dtype):
    try:
        capi.set_variant(0, variant)
        capi.set_variant(1, variant)
        for (M, d, ff) in [(5, 40, 8), (70, 136, 152), (300, 264, 328), (520, 64, 264)]:
            inp = fsw_weights.make_inputs(M, d, ff, dtype, seed=7 * variant + M, x_scale=0.5)
            g = to_dev(inp)
            H = capi.gateup(g["X"], g["W13"])
            assert_one_rounding(H, oracle.ref_gateup(inp["X"], inp["W13"], torch.float64), dtype,
                                "variant %d H %s" % (variant, (M, d, ff)))
            Y = capi.down(H, g["W2"])
            assert_one_rounding(Y, oracle.ref_down(H.cpu(), inp["W2"], torch.float64), dtype,
                                "variant %d Y %s" % (variant, (M, d, ff)))
    finally:
        capi.set_variant(0, -1)
        capi.set_variant(1, -1)


def _random_shapes(n, seed):
    rng = np.random.default_rng(seed)
    return [(int(rng.integers(65, 700)), int(rng.integers(1, 70)) * 8, int(rng.integers(1, 70)) * 8) for _ in range(n)]


@pytest.mark.parametrize("shape", _random_shapes(10, 20240607))
def test_large_tile_kernel_on_random_ragged_shapes(capi, shape):
    """The 256 x 256 kernel forced onto shapes it is never picked for: every combination of ragged rows, ragged
    features and K that is no multiple of 64 or even of 32 goes through its zero-filling copies, its K-pair loop
    tails (1 .. 9 pairs) and its narrow store paths. Both projections, against the fp64 oracle."""
    M, d, ff = shape
    dtype = torch.bfloat16 if (M + d + ff) % 2 else torch.float16
    inp = fsw_weights.make_inputs(M, d, ff, dtype, seed=M * 7 + d + ff, x_scale=0.5)
    g = to_dev(inp)
    try:
        capi.set_variant(0, 5)
        capi.set_variant(1, 5)
        H = capi.gateup(g["X"], g["W13"])
        assert_one_rounding(H, oracle.ref_gateup(inp["X"], inp["W13"], torch.float64), dtype, "H %s" % (shape,))
        Y = capi.down(H, g["W2"])
        assert_one_rounding(Y, oracle.ref_down(H.cpu(), inp["W2"], torch.float64), dtype, "Y %s" % (shape,))
    finally:
        capi.set_variant(0, -1)
        capi.set_variant(1, -1)


@pytest.mark.parametrize("pad", [0, 8, 4, 1])
def test_large_tile_output_store_paths(capi, pad):
    """The 256 x 256 kernel stores 16 bytes per lane when the output row stride and base allow it (pad 0, 8), 8 bytes
    when only that alignment holds (pad 4) and single elements otherwise (pad 1); feature counts that end inside a
    pair of 16-feature blocks take the narrow path for that pair. Outputs are column slices of wider NaN-filled
    buffers, so a store past a row's end would show."""
    M, d, ff = 300, 136, 200            # gated: 200 features = 6 whole block pairs + 8; plain: 136 = 4 pairs + 8
    dtype = torch.bfloat16
    inp = fsw_weights.make_inputs(M, d, ff, dtype, seed=77 + pad, x_scale=0.5)
    g = to_dev(inp)
    try:
        capi.set_variant(0, 5)
        capi.set_variant(1, 5)
        Hbig = torch.full((M, ff + pad), float("nan"), dtype=dtype, device=DEV)
        H = capi.gateup(g["X"], g["W13"], out=Hbig[:, :ff])
        assert_one_rounding(H, oracle.ref_gateup(inp["X"], inp["W13"], torch.float64), dtype, "H pad %d" % pad)
        assert pad == 0 or torch.isnan(Hbig[:, ff:]).all()
        Ybig = torch.full((M, d + pad), float("nan"), dtype=dtype, device=DEV)
        Hc = H.contiguous()
        Y = capi.down(Hc, g["W2"], out=Ybig[:, :d])
        assert_one_rounding(Y, oracle.ref_down(Hc.cpu(), inp["W2"], torch.float64), dtype, "Y pad %d" % pad)
        assert pad == 0 or torch.isnan(Ybig[:, d:]).all()
    finally:
        capi.set_variant(0, -1)
        capi.set_variant(1, -1)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("M", [1, 7, 16, 17, 33, 48, 64])
def test_skinny_weight_streaming_variant(capi, M, dtype):
    """The decode kernels (forced for every M <= 64 here; picked automatically for M <= 16)."""
    try:
        capi.set_variant(0, 100)
        capi.set_variant(1, 100)
        for (d, ff) in [(8, 8), (136, 40), (1000, 264), (4096, 520), (256, 2056)]:
            inp = fsw_weights.make_inputs(M, d, ff, dtype, seed=31 * M + d, x_scale=0.5)
            g = to_dev(inp)
            assert capi.variant_name(0, 0, M, 2 * ff, d) == "skinny"
            H = capi.gateup(g["X"], g["W13"])
            assert_one_rounding(H, oracle.ref_gateup(inp["X"], inp["W13"], torch.float64), dtype,
                                "skinny H %s" % ((M, d, ff),))
            Y = capi.down(H, g["W2"])
            assert_one_rounding(Y, oracle.ref_down(H.cpu(), inp["W2"], torch.float64), dtype,
                                "skinny Y %s" % ((M, d, ff),))
        # odd ff: scalar stores, odd ldh
        inp = fsw_weights.make_inputs(M, 72, 37, dtype, seed=5, x_scale=0.5)
        H = capi.gateup(inp["X"].to(DEV), inp["W13"].to(DEV))
        assert_one_rounding(H, oracle.ref_gateup(inp["X"], inp["W13"], torch.float64), dtype, "skinny odd ff")
    finally:
        capi.set_variant(0, -1)
        capi.set_variant(1, -1)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("M", [1, 7, 16])
def test_streaming_decode_variant(capi, M, dtype):
    """The persistent streaming kernel for M <= 16, one projection per launch (variant 102; picked automatically
    only for large d * ff): ragged d / ff, more tiles than one pass of accumulators holds (ff = 20000 at 8 features
    per tile on few CUs is covered by d = 40: many tiles per workgroup), K slices longer than the activation
    registers (d = 9000), odd ff with scalar stores."""
    try:
        capi.set_variant(0, 102)
        capi.set_variant(1, 102)
        for (d, ff) in [(8, 8), (136, 40), (1000, 264), (4096, 520), (256, 2056), (40, 20000), (9000, 72)]:
            inp = fsw_weights.make_inputs(M, d, ff, dtype, seed=41 * M + d, x_scale=0.5)
            g = to_dev(inp)
            assert capi.variant_name(0, 0, M, 2 * ff, d) == "decode_stream"
            assert capi.variant_name(1, 0, M, d, ff) == "decode_stream"
            H = capi.gateup(g["X"], g["W13"])
            assert_one_rounding(H, oracle.ref_gateup(inp["X"], inp["W13"], torch.float64), dtype,
                                "stream H %s" % ((M, d, ff),))
            Y = capi.down(H, g["W2"])
            assert_one_rounding(Y, oracle.ref_down(H.cpu(), inp["W2"], torch.float64), dtype,
                                "stream Y %s" % ((M, d, ff),))
        inp = fsw_weights.make_inputs(M, 72, 37, dtype, seed=6, x_scale=0.5)
        H = capi.gateup(inp["X"].to(DEV), inp["W13"].to(DEV))
        assert_one_rounding(H, oracle.ref_gateup(inp["X"], inp["W13"], torch.float64), dtype, "stream odd ff")
        # above 16 rows the override falls back to the dispatcher's choice
        assert capi.variant_name(0, 0, 17, 2 * 264, 1000) == "skinny"
    finally:
        capi.set_variant(0, -1)
        capi.set_variant(1, -1)
    assert capi.variant_name(0, 0, 16, 2 * 28672, 8192) == "decode_stream"
    assert capi.variant_name(0, 0, 16, 2 * 14336, 4096) == "dma_128x64" and capi.variant_name(1, 0, 16, 4096, 14336) == "skinny"


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("M", [1, 5, 16])
def test_single_launch_decode_forward(capi, M, dtype):
    """With variant 101 fsw_mlp runs M <= 16 as one launch (gate/up, device-wide barrier, down projection); it
    must agree with the two-launch path and with the oracle, call after call (the barrier slots restore
    themselves) and for ragged d / ff."""
    for (d, ff) in [(8, 8), (136, 40), (1000, 264), (4096, 1032), (512, 14336), (4096, 14336)]:
        inp = fsw_weights.make_inputs(M, d, ff, dtype, seed=77 * M + d, x_scale=0.5)
        g = to_dev(inp)
        ws = capi.mlp_workspace(g["X"], ff)
        try:
            capi.set_variant(0, 101)
            Y1 = capi.mlp(g["X"], g["W13"], g["W2"], workspace=ws)
            H1 = ws[: M * ff * 2].view(dtype).view(M, ff).clone()
            reps = [capi.mlp(g["X"], g["W13"], g["W2"], workspace=ws) for _ in range(3)]  # barrier slots are reused
            # other activations through the same H scratch: phase 2 must read what THIS call's phase 1 wrote,
            # from whichever XCD wrote it, not lines an L2 kept from the previous call
            inp_b = fsw_weights.make_inputs(M, d, ff, dtype, seed=9000 + 77 * M + d, x_scale=0.5)
            Xb = inp_b["X"].to(DEV)
            Yb = capi.mlp(Xb, g["W13"], g["W2"], workspace=ws)
            Ya = capi.mlp(g["X"], g["W13"], g["W2"], workspace=ws)
        finally:
            capi.set_variant(0, -1)
        Y2 = capi.mlp(g["X"], g["W13"], g["W2"])
        H2 = capi.gateup(g["X"], g["W13"])
        assert_one_rounding(H1, oracle.ref_gateup(inp["X"], inp["W13"], torch.float64), dtype, "fused H %s" % ((M, d, ff),))
        assert_one_rounding(Y1, oracle.ref_down(H1.cpu(), inp["W2"], torch.float64), dtype, "fused Y|H %s" % ((M, d, ff),))
        oracle.assert_parity(Y1, oracle.ref_mlp(inp["X"], inp["W13"], inp["W2"], torch.float64), "fused mlp %s" % ((M, d, ff),))
        # the two paths differ only in fp32 summation order
        assert (H1.float() - H2.float()).abs().max().item() <= 2 * ulp_rel(dtype) * 2 * H2.float().abs().max().item() + 1e-3
        assert (Y1.float() - Y2.float()).abs().max().item() <= 2e-2
        for r in reps:
            assert torch.equal(r, Y1)
        oracle.assert_parity(Yb, oracle.ref_mlp(inp_b["X"], inp["W13"], inp["W2"], torch.float64), "fused mlp, second input %s" % ((M, d, ff),))
        assert torch.equal(Ya, Y1)
    torch.cuda.synchronize()
    assert capi.decode_barrier_failures() == 0


def test_single_launch_decode_reports_a_failed_barrier(capi):
    """Variant 103 is the single-launch forward with a device-wide barrier that waits for one arrival more than the
    grid has and polls 64 times only: every workgroup takes the give-up path. The kernel must end normally, write NO
    Y (the down projection is skipped, not run on a partial H), leave the barrier slot reusable, and the failure must
    be visible through fsw_decode_barrier_failures() exactly once."""
    M, d, ff = 8, 1000, 264
    inp = fsw_weights.make_inputs(M, d, ff, torch.bfloat16, seed=5, x_scale=0.5)
    g = to_dev(inp)
    ws = capi.mlp_workspace(g["X"], ff)
    torch.cuda.synchronize()
    assert capi.decode_barrier_failures() == 0
    Y = torch.full((M, d), 7.0, dtype=torch.bfloat16, device=DEV)
    # the failing barrier is a test hook: refused unless the process asks for test hooks
    os.environ.pop("FSW_TEST_HOOKS", None)
    assert capi.lib().fsw_set_variant(0, 103) == capi.E_VARIANT
    os.environ["FSW_TEST_HOOKS"] = "1"

    def failing_launch():
        Y.fill_(7.0)
        try:
            capi.set_variant(0, 103)
            capi.mlp(g["X"], g["W13"], g["W2"], out=Y, workspace=ws)
            torch.cuda.synchronize()
        finally:
            capi.set_variant(0, -1)
        assert (Y.float() == 7.0).all(), "a failed single launch must not write Y"

    failing_launch()
    assert capi.decode_barrier_failures() == 1
    assert capi.decode_barrier_failures() == 0
    # the mark of a failure belongs to its launch: with nobody asking in between, 70 good launches (they walk over
    # all 64 barrier slots, the failed one included) each write the whole of Y, and the failure is still reported
    failing_launch()
    good = capi.mlp(g["X"], g["W13"], g["W2"])
    try:
        capi.set_variant(0, 101)
        for i in range(70):
            Y.fill_(7.0)
            capi.mlp(g["X"], g["W13"], g["W2"], out=Y, workspace=ws)
            assert (Y.float() - good.float()).abs().max().item() <= 2e-2, "launch %d after an unreported failure" % i
    finally:
        capi.set_variant(0, -1)
    assert capi.decode_barrier_failures() == 1
    assert capi.decode_barrier_failures() == 0
    failing_launch()
    failing_launch()
    assert capi.decode_barrier_failures() == 2
    os.environ.pop("FSW_TEST_HOOKS", None)
    # the gate/up half did run, and the slot works again: 70 good launches walk over all 64 slots
    H = ws[: M * ff * 2].view(torch.bfloat16).view(M, ff)
    assert_one_rounding(H, oracle.ref_gateup(inp["X"], inp["W13"], torch.float64), torch.bfloat16, "H of a failed launch")
    ref = oracle.ref_mlp(inp["X"], inp["W13"], inp["W2"], torch.float64)
    try:
        capi.set_variant(0, 101)
        for _ in range(70):
            Y.fill_(7.0)
            capi.mlp(g["X"], g["W13"], g["W2"], out=Y, workspace=ws)
        torch.cuda.synchronize()
    finally:
        capi.set_variant(0, -1)
    oracle.assert_parity(Y, ref, "single launch after a failed one")
    assert capi.decode_barrier_failures() == 0
    # on a capturing stream the single launch is refused and the two-launch path is recorded instead
    graph = torch.cuda.CUDAGraph()
    Yg = torch.empty_like(Y)
    try:
        capi.set_variant(0, 101)
        with torch.cuda.graph(graph):
            capi.mlp(g["X"], g["W13"], g["W2"], out=Yg, workspace=ws)
    finally:
        capi.set_variant(0, -1)
    for _ in range(2):
        Yg.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(Yg, capi.mlp(g["X"], g["W13"], g["W2"]))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("M", [1, 9, 16, 17, 32])
def test_split_k_streaming_down_inside_mlp(capi, M, dtype):
    """Inside fsw_mlp the down projection of up to 32 rows runs 32-row tiles with K split over two workgroups whose
    partial tiles meet through ticket counters (zeroed by the gate/up kernel before it). Forced (variant 104) on small
    and ragged shapes, automatic at decode size: against the oracle given the GPU's H, against the 16-row kernel, bit
    for bit call after call (the summation order does not depend on which workgroup arrives last), and with a
    workspace full of garbage (nothing but the gate/up kernel initialises the counters)."""
    shapes = [(8, 8), (136, 40), (1000, 264), (520, 1032), (256, 2056), (40, 20000), (4096, 1032)]
    for (d, ff) in shapes:
        inp = fsw_weights.make_inputs(M, d, ff, dtype, seed=53 * M + d, x_scale=0.5)
        g = to_dev(inp)
        try:
            capi.set_variant(1, 104)
            assert capi.variant_name(2, 0, M, d, ff) == "stream_split"
            ws = capi.mlp_workspace(g["X"], ff)
            ws.fill_(0xFF)
            Y = capi.mlp(g["X"], g["W13"], g["W2"], workspace=ws)
            H = ws[: M * ff * 2].view(dtype).view(M, ff).clone()
            reps = [capi.mlp(g["X"], g["W13"], g["W2"], workspace=ws) for _ in range(5)]
        finally:
            capi.set_variant(1, -1)
        assert_one_rounding(Y, oracle.ref_down(H.cpu(), inp["W2"], torch.float64), dtype, "stream-split Y|H %s" % ((M, d, ff),))
        oracle.assert_parity(Y, oracle.ref_mlp(inp["X"], inp["W13"], inp["W2"], torch.float64), "stream-split mlp %s" % ((M, d, ff),))
        for r in reps:
            assert torch.equal(r, Y)
        try:
            capi.set_variant(1, 100)
            assert capi.variant_name(2, 0, M, d, ff) == "skinny"
            Y16 = capi.mlp(g["X"], g["W13"], g["W2"])
        finally:
            capi.set_variant(1, -1)
        assert (Y.float() - Y16.float()).abs().max().item() <= 2e-2
    # automatic at decode size, and only there
    name = lambda m, d_, ff_: capi.variant_name(2, 0, m, d_, ff_)
    assert name(17, 4096, 14336) == "stream_split" and name(32, 4096, 14336) == "stream_split"
    assert name(16, 4096, 14336) == "skinny" and name(24, 512, 1024) == "skinny" and name(33, 4096, 14336) != "stream_split"
    assert name(16, 8192, 28672) == "decode_stream"
    # decode size with a ragged last tile (d % 32 != 0: 129 tiles, the last one 8 rows wide) and a K that the two
    # workgroups of a tile and their waves do not split evenly
    if M in (17, 32):
        d, ff = 4104, 14344
        assert name(M, d, ff) == "stream_split"
        inp = fsw_weights.make_inputs(M, d, ff, dtype, seed=8, x_scale=0.5)
        g = to_dev(inp)
        ws = capi.mlp_workspace(g["X"], ff)
        ws.fill_(0xA5)
        Y = capi.mlp(g["X"], g["W13"], g["W2"], workspace=ws)
        H = ws[: M * ff * 2].view(dtype).view(M, ff).clone()
        assert_one_rounding(Y, oracle.ref_down(H.cpu(), inp["W2"], torch.float64), dtype, "stream-split ragged decode size")
        for _ in range(5):
            assert torch.equal(capi.mlp(g["X"], g["W13"], g["W2"], workspace=ws), Y)
    if M in (17, 32):
        d, ff = 4096, 14336
        inp = fsw_weights.make_inputs(M, d, ff, dtype, seed=7, x_scale=0.5)
        g = to_dev(inp)
        ws = capi.mlp_workspace(g["X"], ff)
        ws.fill_(0x5A)
        Y = capi.mlp(g["X"], g["W13"], g["W2"], workspace=ws)
        H = ws[: M * ff * 2].view(dtype).view(M, ff).clone()
        assert_one_rounding(Y, oracle.ref_down(H.cpu(), inp["W2"], torch.float64), dtype, "stream-split decode size")
        for _ in range(20):
            assert torch.equal(capi.mlp(g["X"], g["W13"], g["W2"], workspace=ws), Y)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_split_k_down_projection(capi, dtype):
    """65 <= M with few output tiles and a deep ff: fsw_down splits K across workgroups (fp32 partials in the
    workspace, then one rounding). Checked against the oracle and, bit for bit up to summation order, against the
    unsplit kernel."""
    L = capi.lib()
    # the last three shapes are planned on 256 x 256 tiles (the last two with a K tail, the last with ragged M and d
    # as well), the others on 128 x 128 or 128 x 256
    for (M, d, ff) in [(200, 512, 4096), (130, 520, 2120), (65, 136, 8192), (256, 1024, 14336), (300, 264, 1032), (1024, 1024, 4096), (700, 2048, 2056), (768, 4096, 8192),
                       (768, 4096, 8200), (1300, 3080, 8200),
                       (160, 4096, 4096), (250, 4096, 4104)]:  # one 128 x 192 / 128 x 256 tile of rows per workgroup
        inp = fsw_weights.make_inputs(M, d, ff, dtype, seed=900 + M, x_scale=0.5)
        g = to_dev(inp)
        H = capi.gateup(g["X"], g["W13"])
        nbytes = L.fsw_down_workspace_bytes(capi.dtype_code(H), M, d, ff)
        assert nbytes > 0 and nbytes % (M * d * 4) == 0
        Y = capi.down(H, g["W2"])
        rows = torch.arange(0, M, 1 if M * d * ff < 2 ** 32 else 5)
        ref = oracle.ref_down(H[rows.to(DEV)].cpu(), inp["W2"], torch.float64)
        assert_one_rounding(Y[rows.to(DEV)], ref, dtype, "split-K Y %s (scratch %d B)" % ((M, d, ff), nbytes))
        try:
            capi.set_variant(1, 0)  # 128 x 128 tiles, no split
            Y1 = capi.down(H, g["W2"])
        finally:
            capi.set_variant(1, -1)
        assert (Y.float() - Y1.float()).abs().max().item() <= 4 * ulp_rel(dtype) * ref.abs().max().item() + 1e-3
        assert torch.equal(capi.mlp(g["X"], g["W13"], g["W2"]), Y)
    assert L.fsw_down_workspace_bytes(0, 200, 512, 4096) > 0 and L.fsw_down_workspace_bytes(0, 300, 264, 1032) > 0
    # a missing or short workspace is refused, not ignored
    inp = fsw_weights.make_inputs(200, 512, 4096, torch.bfloat16, seed=1)
    g = to_dev(inp)
    H = capi.gateup(g["X"], g["W13"])
    Y = torch.empty(200, 512, dtype=torch.bfloat16, device=DEV)
    rc = L.fsw_down(0, 200, 512, 4096, H.data_ptr(), 4096, g["W2"].data_ptr(), 4096, Y.data_ptr(), 512, None, 0, None)
    assert rc == capi.E_WORKSPACE


def test_empty_and_degenerate_problems(capi):
    bf = torch.bfloat16
    X = torch.randn(0, 64, device=DEV).to(bf)
    W13 = torch.randn(16, 64, device=DEV).to(bf)
    W2 = torch.randn(64, 8, device=DEV).to(bf)
    assert capi.gateup(X, W13).shape == (0, 8)
    assert capi.mlp(X, W13, W2).shape == (0, 64)
    # ff = 0: Y = 0
    X1 = torch.randn(4, 64, device=DEV).to(bf)
    Y = capi.mlp(X1, torch.empty(0, 64, device=DEV, dtype=bf), torch.empty(64, 0, device=DEV, dtype=bf),
                 out=torch.full((4, 64), 7.0, device=DEV, dtype=bf))
    assert Y.abs().max().item() == 0.0
    # K = 0: up = gate = 0, H = 0 * silu(0) = 0
    H = capi.gateup(torch.empty(4, 0, device=DEV, dtype=bf), torch.empty(16, 0, device=DEV, dtype=bf),
                    out=torch.full((4, 8), 7.0, device=DEV, dtype=bf))
    assert H.abs().max().item() == 0.0
    # the same through the tiled kernels (M > 64): K = 0 writes zeros, ff = 0 gives Y = 0, D = 0 needs no Y at all
    for M in (70, 300):
        H = capi.gateup(torch.empty(M, 0, device=DEV, dtype=bf), torch.empty(16, 0, device=DEV, dtype=bf),
                        out=torch.full((M, 8), 7.0, device=DEV, dtype=bf))
        assert H.abs().max().item() == 0.0
        Xm = torch.randn(M, 64, device=DEV).to(bf)
        Y = capi.mlp(Xm, torch.empty(0, 64, device=DEV, dtype=bf), torch.empty(64, 0, device=DEV, dtype=bf),
                     out=torch.full((M, 64), 7.0, device=DEV, dtype=bf))
        assert Y.abs().max().item() == 0.0
        L = capi.lib()
        assert L.fsw_mlp(0, M, 0, 8, Xm.data_ptr(), 64, None, 0, None, 8, None, 0, None, 0, None) == capi.OK
    # a forced tiled kernel runs unsplit and asks for no scratch
    try:
        capi.set_variant(1, 0)
        assert capi.lib().fsw_down_workspace_bytes(0, 200, 512, 4096) == 0
        Hh = torch.randn(200, 4096, device=DEV).to(bf)
        W2 = torch.randn(512, 4096, device=DEV).to(bf)
        Yf = torch.empty(200, 512, device=DEV, dtype=bf)
        assert capi.lib().fsw_down(0, 200, 512, 4096, Hh.data_ptr(), 4096, W2.data_ptr(), 4096, Yf.data_ptr(), 512,
                                   None, 0, torch.cuda.current_stream().cuda_stream) == capi.OK
    finally:
        capi.set_variant(1, -1)
    assert_one_rounding(Yf, Hh.cpu().double() @ W2.cpu().double().T, bf, "forced unsplit down", slack=0.25)


def test_even_odd_convention_on_device(capi):
    """One-hot probe through the HIP kernel: H[m,j] = W13[2j,m] * silu(W13[2j+1,m]) for X = I."""
    K, ff = 64, 41
    X = torch.eye(K, dtype=torch.bfloat16, device=DEV)
    g = torch.Generator().manual_seed(12)
    W13 = (torch.randn((2 * ff, K), generator=g) * 2).to(torch.bfloat16)
    H = capi.gateup(X, W13.to(DEV)).cpu()
    up, gate = W13[0::2].double().T, W13[1::2].double().T
    assert_one_rounding(H, up * torch.nn.functional.silu(gate), torch.bfloat16, "one-hot", slack=1e-6)
    swapped = gate * torch.nn.functional.silu(up)
    assert (H.double() - swapped).abs().max().item() > 0.5


def test_exact_small_integer_products_round_once(capi):
    """K <= 32 and small-integer inputs make every fp32 partial sum exact, so the output must equal the
    round-to-nearest-even of the exact value bit for bit (no accumulation-order slack)."""
    for dtype in (torch.bfloat16, torch.float16):
        g = torch.Generator().manual_seed(21)
        X = torch.randint(-3, 4, (37, 32), generator=g).to(dtype)
        W2 = torch.randint(-3, 4, (50, 32), generator=g).to(dtype)
        Y = capi.down(X.to(DEV), W2.to(DEV)).cpu()
        exact = X.double() @ W2.double().T
        assert torch.equal(Y.double(), exact)  # |values| <= 288: exactly representable in both types
        # ties and inexact values: scale by 1/256 + offsets so many products need rounding
        Xs = (X.double() * 1.01).to(dtype)
        Ws = (W2.double() * 0.37).to(dtype)
        Yr = capi.down(Xs.to(DEV), Ws.to(DEV)).cpu()
        want = (Xs.double() @ Ws.double().T)
        want_f32 = want.float()  # K=32 products of 8/11-bit significands: fp32 sums are exact or within 1 fp32 ulp
        ok = (Yr == want_f32.to(dtype))
        assert ok.float().mean().item() > 0.995, ok.float().mean().item()


# ---------------------------------------------------------------------------------------------------------------
# operator surface (PyTorch extension), the ldC/2 rule, error behaviour
# ---------------------------------------------------------------------------------------------------------------
def test_torch_ops_match_c_abi_and_reference_formulation(capi, ext):
    inp = fsw_weights.make_inputs(200, 256, 328, torch.bfloat16, seed=33)
    g = to_dev(inp)
    H_c = capi.gateup(g["X"], g["W13"])
    H_p = ext.fused_swiglu_bf16(g["X"], g["W13"])
    H_o = torch.ops.ASMLLM.fused_swiglu_bf16(g["X"], g["W13"])
    assert H_p.dtype == torch.bfloat16 and H_p.shape == (200, 328) and H_p.device == g["X"].device
    assert torch.equal(H_c, H_p) and torch.equal(H_c, H_o)
    # the reference's own check (numeric_tests.py:41-52): bf16 torch formulation on the GPU
    C = g["X"] @ g["W13"].T
    gated = C[:, ::2] * torch.nn.functional.silu(C[:, 1::2])
    diff = (H_p - gated).float()
    assert diff.abs().max().item() < 0.1 and (diff.norm() / gated.float().norm()).item() < 2e-2
    Y = ext.fused_swiglu_mlp_bf16(g["X"], g["W13"], g["W2"])
    assert torch.equal(Y, capi.mlp(g["X"], g["W13"], g["W2"]))
    assert torch.equal(Y, torch.ops.ASMLLM.swiglu_down_bf16(H_p, g["W2"]))
    oracle.assert_parity(Y, oracle.ref_mlp(inp["X"], inp["W13"], inp["W2"]), "ext mlp")
    # fp16 additions
    i16 = fsw_weights.make_inputs(96, 128, 200, torch.float16, seed=34, x_scale=0.5)
    g16 = to_dev(i16)
    Y16 = ext.fused_swiglu_mlp_fp16(g16["X"], g16["W13"], g16["W2"])
    oracle.assert_parity(Y16, oracle.ref_mlp(i16["X"], i16["W13"], i16["W2"]), "ext mlp fp16")
    with pytest.raises(RuntimeError):
        ext.fused_swiglu_bf16(g16["X"], g16["W13"])  # fp16 into the bf16 op (swiglu.cu:475-480)


def test_swiglu_fwd_bf16_writes_dense_half_width_rows(ext):
    """bench_swiglu.py:91,106 passes C as [M, N] with ldC = N; the op writes a dense [M, N/2] matrix with row
    stride ldC/2 into its first M*N/2 elements (swiglu.cu:353,408,414) and leaves the rest untouched."""
    M, K, ff = 70, 128, 90
    N = 2 * ff
    inp = fsw_weights.make_inputs(M, K, ff, torch.bfloat16, seed=35)
    g = to_dev(inp)
    C = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device=DEV)
    assert ext.swiglu_fwd_bf16(M, N, K, g["X"], K, g["W13"], K, C, N) is None
    flat = C.flatten()
    H = flat[: M * ff].view(M, ff)
    assert torch.equal(H, ext.fused_swiglu_bf16(g["X"], g["W13"]))
    assert torch.isnan(flat[M * ff:]).all()
    # same through the dispatcher, with padded leading dimensions on the inputs
    Xp = torch.zeros((M, K + 16), dtype=torch.bfloat16, device=DEV)
    Xp[:, :K] = g["X"]
    Wp = torch.zeros((N, K + 8), dtype=torch.bfloat16, device=DEV)
    Wp[:, :K] = g["W13"]
    C2 = torch.full((M, N + 20), float("nan"), dtype=torch.bfloat16, device=DEV)
    torch.ops.ASMLLM.swiglu_fwd_bf16(M, N, K, Xp, K + 16, Wp, K + 8, C2, N + 20)
    H2 = C2.flatten()[: M * (ff + 10)].view(M, ff + 10)
    assert torch.equal(H2[:, :ff], H) and torch.isnan(H2[:, ff:]).all()
    with pytest.raises(RuntimeError):
        ext.swiglu_fwd_bf16(M, N, K, g["X"], K, g["W13"], K, torch.empty(4, 4, dtype=torch.bfloat16, device=DEV), N)
    with pytest.raises(RuntimeError):
        ext.swiglu_fwd_bf16(M, N + 1, K, g["X"], K, g["W13"], K, C, N)  # odd N


@pytest.mark.parametrize("shape", [(16, 520, 8200), (64, 136, 11008), (128, 264, 13824), (100, 72, 8192), (40, 64, 10004)])
def test_weight_stream_cut_into_one_piece_per_compute_unit(capi, shape):
    """Gate/up with one tile of activation rows and between 128 and 216 tiles of 128 weight rows: the dispatcher hands
    every workgroup a piece of 64 .. 120 rows instead (as many pieces as compute units), whose tile reads its missing
    rows as zeros and stores only the features it owns. Against the oracle (every feature, so a piece that stored a
    neighbour's features from its zero rows would show as zeros there) and against the kernel on whole 128-row tiles; H
    inside a wider NaN buffer, so a store past the row's end would show."""
    M, d, ff = shape
    dtype = torch.bfloat16 if ff % 16 == 0 else torch.float16
    inp = fsw_weights.make_inputs(M, d, ff, dtype, seed=M + ff, x_scale=0.5)
    g = to_dev(inp)
    want = "dma_128x64" if M <= 64 else "dma_128x128"
    forced = capi.variant_name(0, 0, M, 2 * ff, d) != want  # small K: the weight-streaming kernel would run
    wide = torch.full((M, ff + 8), float("nan"), dtype=dtype, device=DEV)
    try:
        if forced:
            capi.set_variant(0, 4)
        assert capi.variant_name(0, 0, M, 2 * ff, d) == want
        H = capi.gateup(g["X"], g["W13"], out=wide[:, :ff])
    finally:
        capi.set_variant(0, -1)
    assert_one_rounding(H, oracle.ref_gateup(inp["X"], inp["W13"], torch.float64), dtype, "pieces %s" % (shape,))
    assert torch.isnan(wide[:, ff:]).all()
    # the same kernel on whole tiles: a problem of the same rows that the rule leaves alone (more than 128 activation
    # rows cannot be built from these, so force the unsplit 128 x 128 kernel on a row-padded X instead)
    Xp = torch.zeros((129, d), dtype=dtype, device=DEV)
    Xp[:M] = g["X"]
    try:
        capi.set_variant(0, 0)
        Hp = capi.gateup(Xp, g["W13"])
    finally:
        capi.set_variant(0, -1)
    # (not bit for bit: with one tile of activation rows every workgroup starts its K walk at its own K tile)
    assert (Hp[:M].float() - H.float()).abs().max().item() <= 2 * ulp_rel(dtype) * H.float().abs().max().item() + 1e-3


def test_pieces_zero_the_ticket_counters_of_the_down_projection_too(capi):
    """A decode-sized forward whose gate/up stream is cut into pieces (27648 rows: 247 pieces of 112) AND whose down
    projection is the split-K streaming kernel (24 rows): the first workgroup of the gate/up launch still zeroes the
    ticket counters, whatever rows it owns. Workspace full of garbage, repeated calls bit for bit."""
    M, d, ff = 24, 5120, 13824
    assert capi.variant_name(0, 0, M, 2 * ff, d) == "dma_128x64" and capi.variant_name(2, 0, M, d, ff) == "stream_split"
    inp = fsw_weights.make_inputs(M, d, ff, torch.bfloat16, seed=61, x_scale=0.5)
    g = to_dev(inp)
    ws = capi.mlp_workspace(g["X"], ff)
    ws.fill_(0xC3)
    Y = capi.mlp(g["X"], g["W13"], g["W2"], workspace=ws)
    oracle.assert_parity(Y, oracle.ref_mlp(inp["X"], inp["W13"], inp["W2"], torch.float64), "pieces + stream_split")
    for _ in range(5):
        assert torch.equal(capi.mlp(g["X"], g["W13"], g["W2"], workspace=ws), Y)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("M", [1, 16, 64, 65, 300, 1024])
def test_float32_output_is_the_unrounded_gated_value(capi, M, dtype):
    """fsw_gateup_f32out (the reference's build with C_TYPE float, constants.cuh:9-14, swiglu.cu:470-471): H in
    float32 is up * silu(gate) to fp32 accumulation noise, three orders below a 16-bit rounding; rounding it once gives
    the 16-bit kernel's output bit for bit (same kernel, same K order: the 16-bit path rounds exactly this value)."""
    for (d, ff) in [(512, 1032), (1000, 264), (64, 40)]:
        inp = fsw_weights.make_inputs(M, d, ff, dtype, seed=5 * M + d, x_scale=0.5)
        g = to_dev(inp)
        H32 = capi.gateup_f32out(g["X"], g["W13"])
        assert H32.dtype == torch.float32 and tuple(H32.shape) == (M, ff)
        ref = oracle.ref_gateup(inp["X"], inp["W13"], torch.float64)
        err = (H32.cpu().double() - ref).abs()
        assert not (err > 1e-5 * (1.0 + ref.abs())).any(), "fp32 H %s: worst |d| = %g" % ((M, d, ff), err.max().item())
        try:
            capi.set_variant(0, 100 if M <= 64 else 5)  # the kernel the fp32 path runs for this M
            H16 = capi.gateup(g["X"], g["W13"])
        finally:
            capi.set_variant(0, -1)
        assert torch.equal(H16, H32.to(dtype))
    # strided float output inside a wider NaN buffer, odd row stride (scalar stores): neighbours untouched
    d, ff = 512, 1032
    inp = fsw_weights.make_inputs(M, d, ff, dtype, seed=77, x_scale=0.5)
    g = to_dev(inp)
    wide = torch.full((M, ff + 5), float("nan"), dtype=torch.float32, device=DEV)
    capi.gateup_f32out(g["X"], g["W13"], out=wide[:, :ff])
    assert torch.equal(wide[:, :ff], capi.gateup_f32out(g["X"], g["W13"])) and torch.isnan(wide[:, ff:]).all()


def test_float32_output_through_the_operators(ext):
    """fused_swiglu_bf16_f32out, and swiglu_fwd_bf16 with a float C (the reference's operator compiled with C_TYPE
    float): the ldC / 2 rule holds in elements of C's type (swiglu.cu:414); wrong C types still raise."""
    M, K, N = 300, 512, 2064
    g = torch.Generator(device=DEV).manual_seed(31)
    X = (torch.randn((M, K), device=DEV, generator=g) * 0.5).to(torch.bfloat16)
    W = (torch.randn((N, K), device=DEV, generator=g) / K ** 0.5).to(torch.bfloat16)
    H32 = ext.fused_swiglu_bf16_f32out(X, W)
    assert H32.dtype == torch.float32 and tuple(H32.shape) == (M, N // 2)
    ref = oracle.ref_gateup(X.cpu(), W.cpu(), torch.float64)
    assert ((H32.cpu().double() - ref).abs() <= 1e-5 * (1.0 + ref.abs())).all()
    assert torch.equal(torch.ops.ASMLLM.fused_swiglu_bf16_f32out(X, W), H32)
    C = torch.full((M, N), float("nan"), device=DEV, dtype=torch.float32)
    ext.swiglu_fwd_bf16(M, N, K, X, K, W, K, C, N)
    flat = C.view(-1)
    assert torch.equal(flat[: M * (N // 2)].view(M, N // 2), H32) and torch.isnan(flat[M * (N // 2):]).all()
    with pytest.raises(RuntimeError):
        ext.swiglu_fwd_bf16(M, N, K, X, K, W, K, torch.empty((M, N), device=DEV, dtype=torch.float16), N)
    with pytest.raises(RuntimeError):
        ext.swiglu_fwd_bf16(M, N, K, X, K, W, K, torch.empty((M, N), device=DEV, dtype=torch.float64), N)


def test_strided_views_and_row_independence(capi):
    inp = fsw_weights.make_inputs(150, 192, 144, torch.bfloat16, seed=36)
    g = to_dev(inp)
    Y = capi.mlp(g["X"], g["W13"], g["W2"])
    # row m of Y depends on row m of X only: any row subset gives the same rows, bit for bit
    for rows in (slice(0, 1), slice(17, 18), slice(100, 150), slice(3, 70)):
        assert torch.equal(capi.mlp(g["X"][rows], g["W13"], g["W2"]), Y[rows])
    # every second row through a strided view (ldx = 2 * K)
    assert torch.equal(capi.mlp(g["X"][::2], g["W13"], g["W2"]), Y[::2])
    # padding with zero rows/features does not change the live part
    W13z = torch.cat([g["W13"], torch.zeros(32, 192, dtype=torch.bfloat16, device=DEV)])
    W2z = torch.cat([g["W2"], torch.zeros(192, 16, dtype=torch.bfloat16, device=DEV)], dim=1).contiguous()
    assert torch.equal(capi.mlp(g["X"], W13z, W2z), Y)


def test_permutation_and_linearity_properties(capi):
    inp = fsw_weights.make_inputs(90, 128, 96, torch.bfloat16, seed=37)
    g = to_dev(inp)
    H = capi.gateup(g["X"], g["W13"])
    perm = torch.randperm(96, generator=torch.Generator().manual_seed(2)).to(DEV)
    W13p = g["W13"].view(96, 2, 128)[perm].reshape(192, 128).contiguous()
    assert torch.equal(capi.gateup(g["X"], W13p), H[:, perm])  # features are independent of their position
    W13u = g["W13"].clone()
    W13u[0::2] *= 2  # exact in bf16: doubles every H bit-exactly
    assert torch.equal(capi.gateup(g["X"], W13u).float(), 2 * H.float())
    Y = capi.down(H, g["W2"])
    assert torch.equal(capi.down(H, (g["W2"] * 4).contiguous()).float(), 4 * Y.float())


# ---------------------------------------------------------------------------------------------------------------
# the five benchmark configurations at full size
# ---------------------------------------------------------------------------------------------------------------
def _config_case(capi, name, sample_rows):
    inp = fsw_weights.make_config(name)
    g = {k: inp[k].to(DEV) for k in ("X", "W13", "W2")}
    M, dtype = inp["M"], inp["dtype"]
    H = capi.gateup(g["X"], g["W13"])
    Y = capi.mlp(g["X"], g["W13"], g["W2"])
    torch.cuda.synchronize()
    assert torch.isfinite(Y.float()).all()
    gen = torch.Generator().manual_seed(99)
    rows = torch.sort(torch.randperm(M, generator=gen)[: min(M, sample_rows)]).values
    Xs = inp["X"][rows]
    Href = oracle.ref_gateup(Xs, inp["W13"])
    Yref = oracle.ref_down(Href, inp["W2"])
    # H reaches |H| > 8, where half an ulp of bf16 alone is 0.031: the absolute gate is a statement about the
    # forward's output Y; H is held to "one rounding of the fp32 value" and to the relative gates instead.
    assert_one_rounding(H[rows.to(DEV)], Href.double(), dtype, name + " H", slack=2e-3)
    mh = oracle.assert_parity(H[rows.to(DEV)], Href, name + " H", max_abs_tol=float("inf"))
    my = oracle.assert_parity(Y[rows.to(DEV)], Yref, name + " Y")
    print("\n%s rows=%d H %s\n%s rows=%d Y %s" % (name, len(rows), mh, name, len(rows), my))
    # size-independent property on the FULL output: Y is linear in W2, so sum_n Y[m, n] = H[m, :] . colsum(W2),
    # evaluated in fp64 from the GPU's own H for every row
    colsum = inp["W2"].double().sum(dim=0)
    want = H.cpu().double() @ colsum
    got = Y.cpu().double().sum(dim=1)
    scale = (H.cpu().double().abs() @ inp["W2"].double().abs().sum(dim=0)).clamp_min(1e-6)
    assert ((got - want).abs() / scale).max().item() < 2e-3
    return inp, g, H, Y


def test_config_c1(capi):
    inp, g, H, Y = _config_case(capi, "C1", 512)
    oracle.assert_parity(Y, oracle.ref_mlp_unpacked(inp["X"], inp["Wg"], inp["Wu"], inp["Wd"]), "C1 unpacked")


def test_config_c4_decode(capi):
    _config_case(capi, "C4", 16)


def test_config_c2(capi):
    _config_case(capi, "C2", 192)


def test_config_c3_headline(capi):
    _config_case(capi, "C3", 192)


def test_config_c5_fp16(capi):
    _config_case(capi, "C5", 96)


# ---- panel-blocked layout: the transform, the kernels that read / write it, and fsw_mlp's large-tile regime ----------
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_block_rows_layout(capi, dtype):
    """fsw_block_rows / fsw_prepack_*: block (panel, kt) = [256 rows][32 elements], zero padded; W13 panels carry
    their 128 up rows first, then their 128 gate rows. Bit exact against index arithmetic in torch."""
    for (rows, k, ld) in [(1, 8, 8), (300, 72, 72), (256, 32, 40), (513, 1000, 1008), (700, 4096, 4096)]:
        A = (torch.randn(rows, ld) * 3).to(dtype).to(DEV)[:, :k]
        B = capi.block_rows(A)
        assert torch.equal(capi.unblock(B), A)
        # padding is zero: the K loop of the consumer reads it
        panels, nkt = (rows + 255) // 256, (k + 31) // 32
        full = B.buf[: panels * nkt * 256 * 64].view(dtype).view(panels, nkt, 256, 32).permute(0, 2, 1, 3).reshape(panels * 256, nkt * 32)
        assert full[rows:].abs().max().item() == 0 if rows < panels * 256 else True
        assert full[:, k:].abs().max().item() == 0 if k < nkt * 32 else True
    W13 = (torch.randn(600, 64)).to(dtype).to(DEV)
    P = capi.unblock(capi.block_rows(W13, "w13"))  # row r of panel p: up rows then gate rows of that panel
    expect = torch.zeros(768, 64, dtype=dtype, device=DEV)
    src = torch.zeros(768, 64, dtype=dtype, device=DEV)
    src[:600] = W13
    for p in range(3):
        expect[256 * p: 256 * p + 128] = src[256 * p: 256 * p + 256: 2]
        expect[256 * p + 128: 256 * p + 256] = src[256 * p + 1: 256 * p + 256: 2]
    assert torch.equal(P, expect[:600])


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("prepacked", [False, True])
def test_blocked_kernels_against_oracle(capi, dtype, prepacked):
    """fsw_gateup_blocked / fsw_down_blocked on ragged shapes (M, K, ff not multiples of the 256 / 32 blocking),
    with row-major and with prepacked weights: H (unblocked) to one rounding, Y to one rounding given H."""
    for (M, d, ff) in [(300, 1000, 520), (64, 136, 40), (513, 4096, 264), (1024, 512, 1032)]:
        inp = fsw_weights.make_inputs(M, d, ff, dtype, seed=17 * M + ff, x_scale=0.5)
        g = to_dev(inp)
        Xb = capi.block_rows(g["X"])
        W13 = capi.block_rows(g["W13"], "w13") if prepacked else g["W13"]
        W2 = capi.block_rows(g["W2"], "w2") if prepacked else g["W2"]
        Hb = capi.gateup_blocked(Xb, W13)
        H = capi.unblock(Hb)
        assert_one_rounding(H, oracle.ref_gateup(inp["X"], inp["W13"], torch.float64), dtype, "blocked H %s" % ((M, d, ff),))
        Y = capi.down_blocked(Hb, W2)
        assert_one_rounding(Y, oracle.ref_down(H.cpu(), inp["W2"], torch.float64), dtype, "blocked Y %s" % ((M, d, ff),))
        oracle.assert_parity(Y, oracle.ref_mlp(inp["X"], inp["W13"], inp["W2"], torch.float64), "blocked mlp %s" % ((M, d, ff),))
        # row-major H straight from the blocked X: the same bits as the blocked H
        Hrm = capi.gateup_blocked(Xb, W13, row_major_out=True)
        assert torch.equal(Hrm, H)
        # blocked H straight from the row-major X (the form fsw_mlp runs): the same bits again
        Hb2 = capi.gateup_hblocked(g["X"], W13)
        assert torch.equal(capi.unblock(Hb2), H)
        assert torch.equal(capi.down_blocked(Hb2, W2), Y)
        # against the row-major kernels: the same products, summed in the same K order by the same kernel
        H2 = capi.gateup(g["X"], g["W13"])
        assert (H.float() - H2.float()).abs().max().item() <= 2 * ulp_rel(dtype) * 2 * H2.float().abs().max().item() + 1e-3


def test_blocked_kernels_take_strided_row_major_operands(capi):
    """Row strides larger than the row (column slices of wider tensors) for X into fsw_block_rows, for the
    row-major W13 / W2 of the blocked entry points and for Y."""
    M, d, ff = 300, 1096, 520
    dtype = torch.bfloat16
    inp = fsw_weights.make_inputs(M, d, ff, dtype, seed=123, x_scale=0.5)
    wide = lambda t, extra: torch.cat([t, torch.full((t.shape[0], extra), float("nan"), dtype=t.dtype)], dim=1).to(DEV)[:, : t.shape[1]]
    X, W13, W2 = wide(inp["X"], 24), wide(inp["W13"], 8), wide(inp["W2"], 40)
    assert X.stride(0) == d + 24 and W13.stride(0) == d + 8 and W2.stride(0) == ff + 40
    Xb = capi.block_rows(X)
    Hb = capi.gateup_blocked(Xb, W13)
    Ybig = torch.full((M, d + 16), float("nan"), dtype=dtype, device=DEV)
    Y = capi.down_blocked(Hb, W2, out=Ybig[:, :d])
    oracle.assert_parity(Y, oracle.ref_mlp(inp["X"], inp["W13"], inp["W2"], torch.float64), "blocked, strided operands")
    assert torch.isnan(Ybig[:, d:]).all()


def test_mlp_large_tile_regime_uses_blocked_path(capi):
    """For M > 64 with both projections on 256 x 256 tiles fsw_mlp reads X where it lies and keeps H panel-blocked
    between its two kernels; the result equals that of the separate row-major entry points bit for bit (the K order
    is the same) and agrees with the oracle, and the workspace query covers the blocked H and nothing else."""
    M, d, ff = 4096, 4096, 2048
    L = capi.lib()
    assert L.fsw_mlp_workspace_bytes(0, M, d, ff) == L.fsw_blocked_bytes(M, ff)
    assert L.fsw_gateup_workspace_bytes(0, M, 2 * ff, d) == 0 and L.fsw_down_workspace_bytes(0, M, d, ff) == 0
    inp = fsw_weights.make_inputs(M, d, ff, torch.bfloat16, seed=99, x_scale=0.5)
    g = to_dev(inp)
    Y = capi.mlp(g["X"], g["W13"], g["W2"])
    Y2 = capi.down(capi.gateup(g["X"], g["W13"]), g["W2"])
    rows = torch.arange(0, M, 37)
    oracle.assert_parity(Y[rows.to(DEV)], oracle.ref_mlp(inp["X"][rows], inp["W13"], inp["W2"], torch.float64), "mlp blocked regime")
    assert torch.equal(Y, Y2)
    # the two halves through their own entry points: row-major X -> blocked H -> Y
    Hb = torch.empty(L.fsw_blocked_bytes(M, ff), dtype=torch.uint8, device=DEV)
    stream = torch.cuda.current_stream().cuda_stream
    capi.check(L.fsw_gateup_hblocked(0, M, 2 * ff, d, g["X"].data_ptr(), d, g["W13"].data_ptr(), d, 0, Hb.data_ptr(), stream))
    Y3 = torch.empty_like(Y)
    capi.check(L.fsw_down_blocked(0, M, d, ff, Hb.data_ptr(), g["W2"].data_ptr(), ff, 0, Y3.data_ptr(), d, stream))
    assert torch.equal(Y3, Y)
    # a ragged problem with strided X: rows past M and the K tail come out of the bounds check, not of memory
    M2, d2, ff2 = 700, 1064, 520
    inp = fsw_weights.make_inputs(M2, d2, ff2, torch.float16, seed=98, x_scale=0.5)
    g = to_dev(inp)
    Xs = torch.full((M2, d2 + 24), float("nan"), dtype=torch.float16, device=DEV)
    Xs[:, :d2] = g["X"]
    Hb = torch.full((L.fsw_blocked_bytes(M2, ff2),), 0xFF, dtype=torch.uint8, device=DEV)
    capi.check(L.fsw_gateup_hblocked(1, M2, 2 * ff2, d2, Xs.data_ptr(), d2 + 24, g["W13"].data_ptr(), d2, 0, Hb.data_ptr(), stream))
    Y4 = torch.empty((M2, d2), dtype=torch.float16, device=DEV)
    capi.check(L.fsw_down_blocked(1, M2, d2, ff2, Hb.data_ptr(), g["W2"].data_ptr(), ff2, 0, Y4.data_ptr(), d2, stream))
    oracle.assert_parity(Y4, oracle.ref_mlp(inp["X"], inp["W13"], inp["W2"], torch.float64), "hblocked ragged fp16")
    assert torch.equal(Y4, capi.down(capi.gateup(g["X"], g["W13"]), g["W2"]))


@pytest.mark.parametrize("shape", [(16, 512, 1024), (96, 512, 1024), (600, 1024, 520), (2304, 4096, 2048)])
def test_forward_replays_from_a_hip_graph(capi, shape):
    """fsw_mlp enqueues kernels only (no allocation, no synchronisation, no memset), so a caller can capture it into a
    HIP graph. Every replay — with eager work and synchronisations of the program in between, and with new contents
    in the input buffer — must reproduce the eager result bit for bit. Decode, mid and large-tile regimes, the last
    shape with H panel-blocked between the two kernels."""
    M, d, ff = shape
    inp = fsw_weights.make_inputs(M, d, ff, torch.bfloat16, seed=123, x_scale=0.5)
    g = to_dev(inp)
    X = g["X"].clone()
    Y = torch.empty(M, d, dtype=torch.bfloat16, device=DEV)
    ws = capi.mlp_workspace(X, ff)
    capi.mlp(X, g["W13"], g["W2"], out=Y, workspace=ws)  # warm-up outside the capture
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        capi.mlp(X, g["W13"], g["W2"], out=Y, workspace=ws)
    for rep in range(3):
        X.copy_(g["X"] * (1.0 + 0.25 * rep))
        eager = capi.mlp(X, g["W13"], g["W2"])
        torch.cuda.synchronize()
        Y.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(Y, eager), "replay %d differs from the eager forward" % rep
    oracle.assert_parity(Y, oracle.ref_mlp(X.cpu(), inp["W13"], inp["W2"], torch.float64), "graph replay")


def test_large_tiles_on_row_major_activations(capi):
    """256 x 256 tiles with ROW-MAJOR activations (fetched in K pairs of one whole line per row): fsw_gateup for a
    ragged M and a K that is no multiple of 64, fsw_down without any scratch. Both against the oracle, and the down
    projection bit for bit against the blocked form of the same kernel (H re-blocked by fsw_block_rows first)."""
    L = capi.lib()
    M, d, ff = 1000, 520, 12800          # 4 x 100 tiles of 256 x 256, K = 520 is not a multiple of 64
    assert capi.variant_name(0, 0, M, 2 * ff, d) == "pair16_256x256" and L.fsw_gateup_workspace_bytes(0, M, 2 * ff, d) == 0
    inp = fsw_weights.make_inputs(M, d, ff, torch.bfloat16, seed=31, x_scale=0.5)
    g = to_dev(inp)
    H = capi.gateup(g["X"], g["W13"])
    rows = torch.arange(0, M, 7)
    C = inp["X"][rows].double() @ inp["W13"].double().T
    assert_one_rounding(H[rows.to(DEV)], C[:, 0::2] * torch.nn.functional.silu(C[:, 1::2]), torch.bfloat16, "row-major X, 256x256")
    M2, D2, FF2 = 3300, 4096, 264         # 16 x 13 tiles, ragged M, K = 264
    assert capi.variant_name(1, 0, M2, D2, FF2) == "pair16_256x256"
    gen = torch.Generator().manual_seed(32)
    Hh = (torch.randn(M2, FF2, generator=gen) * 0.5).to(torch.float16)
    W2 = (torch.randn(D2, FF2, generator=gen) / FF2 ** 0.5).to(torch.float16)
    Hd, W2d = Hh.to(DEV), W2.to(DEV)
    Y0 = torch.empty(M2, D2, dtype=torch.float16, device=DEV)
    s = torch.cuda.current_stream().cuda_stream
    capi.check(L.fsw_down(1, M2, D2, FF2, Hd.data_ptr(), FF2, W2d.data_ptr(), FF2, Y0.data_ptr(), D2, None, 0, s))
    assert torch.equal(Y0, capi.down(Hd, W2d)) and L.fsw_down_workspace_bytes(1, M2, D2, FF2) == 0
    Y1 = capi.down_blocked(capi.block_rows(Hd), W2d)   # the same products in the same K order from a blocked H
    assert torch.equal(Y0, Y1)
    rows = torch.arange(0, M2, 31)
    assert_one_rounding(Y0[rows.to(DEV)], Hh[rows].double() @ W2.double().T, torch.float16, "row-major H, 256x256")
