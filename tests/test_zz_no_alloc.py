"""fsw_mlp_static — the forward for callers that cannot allocate — against fsw_mlp through the C ABI.

It runs the same kernels on a static scratch array inside the library, so its output must equal fsw_mlp's bit for
bit (which the other tests hold to the oracle's gates), on calls in a row that reuse the array with different
shapes: the second, smaller problem sees the first one's leftovers in its scratch."""
import pytest
import torch

from oracle import oracle
import fsw_weights

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _case(capi, M, d, ff, dtype, seed):
    inp = fsw_weights.make_inputs(M, d, ff, dtype, seed=seed, x_scale=0.5)
    g = {k: inp[k].to(DEV) for k in ("X", "W13", "W2")}
    want = capi.mlp(g["X"], g["W13"], g["W2"])
    torch.cuda.synchronize()
    return inp, g, want


def test_static_scratch_forward_matches_fsw_mlp_call_after_call(capi):
    L = capi.lib()
    limit = L.fsw_mlp_static_max_bytes()
    assert limit == 64 << 20
    # (M, d, ff): split-K partials + H; small; a decode shape; the split-K streaming down projection of 17 .. 32 rows
    # (its ticket counters sit in the array behind another call's leftovers and are zeroed by the gate/up kernel);
    # ragged everything; tiny; H panel-blocked (both projections on 256 x 256 tiles); ragged mid size
    shapes = [(200, 1024, 4096), (48, 512, 1032), (16, 4096, 14336), (24, 4096, 14336), (300, 264, 1032), (4, 136, 40),
              (2304, 4096, 2048), (700, 1024, 2056)]
    assert capi.variant_name(2, 0, 24, 4096, 14336) == "stream_split"
    assert L.fsw_mlp_workspace_bytes(0, 2304, 4096, 2048) == L.fsw_blocked_bytes(2304, 2048)
    cases = [_case(capi, M, d, ff, torch.bfloat16 if i % 2 == 0 else torch.float16, 400 + i)
             for i, (M, d, ff) in enumerate(shapes)]
    for (M, d, ff) in shapes:
        assert 0 < L.fsw_mlp_workspace_bytes(0, M, d, ff) <= limit
    outs = [torch.full_like(want, float("nan")) for inp, g, want in cases]
    # one call first (it looks the array's address up), then the device's free memory must not move: a hipMalloc
    # inside the library would show here, which torch's own allocator statistics cannot see
    capi.mlp_static(cases[0][1]["X"], cases[0][1]["W13"], cases[0][1]["W2"], out=outs[0])
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    mark = torch.cuda.memory_allocated()
    for (inp, g, want), Y in zip(cases, outs):  # back to back on one stream, no synchronisation in between
        capi.mlp_static(g["X"], g["W13"], g["W2"], out=Y)
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before, "device memory was allocated or freed during fsw_mlp_static"
    assert torch.cuda.memory_allocated() == mark  # nothing came from torch's allocator either
    for (inp, g, want), Y, shape in zip(cases, outs, shapes):
        assert torch.equal(Y, want), "fsw_mlp_static differs from fsw_mlp at %s" % (shape,)
    # and against the oracle directly for the first two (the pair "a call, then a smaller one")
    for (inp, g, want), Y in list(zip(cases, outs))[:2]:
        oracle.assert_parity(Y, oracle.ref_mlp(inp["X"], inp["W13"], inp["W2"], torch.float64), "static scratch")
    # a second pass in reverse order: every call starts from another call's leftovers
    for (inp, g, want), Y in reversed(list(zip(cases, outs))):
        Y.fill_(float("nan"))
        capi.mlp_static(g["X"], g["W13"], g["W2"], out=Y)
    torch.cuda.synchronize()
    for (inp, g, want), Y, shape in zip(cases, outs, shapes):
        assert torch.equal(Y, want), "second pass differs at %s" % (shape,)


def test_static_scratch_limit_and_errors(capi):
    L = capi.lib()
    limit = L.fsw_mlp_static_max_bytes()
    M, d, ff = 8192, 4096, 14336
    assert L.fsw_mlp_workspace_bytes(0, M, d, ff) > limit
    # refused before anything is read: the pointers are never dereferenced
    rc = L.fsw_mlp_static(0, M, d, ff, 0x1000, d, 0x2000, d, 0x3000, ff, 0x4000, d, None)
    assert rc == capi.E_STATIC_LIMIT and "64 MiB" in capi.strerror(rc)
    assert L.fsw_mlp_static(3, 4, 16, 8, 0x1000, 16, 0x2000, 16, 0x3000, 8, 0x4000, 16, None) == capi.E_DTYPE
    assert L.fsw_mlp_static(0, 0, 16, 8, None, 16, None, 16, None, 8, None, 16, None) == capi.OK
    X = torch.zeros(4, 16, dtype=torch.bfloat16, device=DEV)
    assert L.fsw_mlp_static(0, 4, 16, 8, X.data_ptr(), 16, None, 16, None, 8, X.data_ptr(), 16, None) == capi.E_NULL
    assert L.fsw_mlp_static(0, 4, 16, 12, X.data_ptr(), 16, X.data_ptr(), 16, X.data_ptr(), 16, X.data_ptr(), 16,
                            None) == capi.E_ALIGN


def test_static_scratch_forward_replays_from_a_hip_graph(capi):
    """The callers it is for: captured once (after a first call outside the capture), replayed with eager work in
    between; every replay equals the eager fsw_mlp result."""
    inp, g, _ = _case(capi, 96, 512, 1024, torch.bfloat16, 77)
    X = g["X"].clone()
    Y = torch.empty(96, 512, dtype=torch.bfloat16, device=DEV)
    capi.mlp_static(X, g["W13"], g["W2"], out=Y)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        capi.mlp_static(X, g["W13"], g["W2"], out=Y)
    for rep in range(3):
        X.copy_(g["X"] * (1.0 + 0.5 * rep))
        eager = capi.mlp(X, g["W13"], g["W2"])
        torch.cuda.synchronize()
        Y.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(Y, eager), "replay %d" % rep
