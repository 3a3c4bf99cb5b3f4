"""Host-side checks that need no GPU: the C-ABI library loads and exports everything include/fsw.h declares,
argument validation returns the documented codes before any HIP call, the packers follow the reference's
row interleave, and the operator surface matches csrc/torch_bindings.cpp:31-50 of the reference."""
import ctypes
import os
import re

import pytest
import torch

import fsw_weights

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "fsw.h")


def declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return re.findall(r"FSW_API\s+[\w\s\*]+?\b(fsw_\w+)\s*\(", text)


def test_library_exports_every_declared_symbol(capi):
    names = declared_symbols()
    assert len(names) >= 12 and len(set(names)) == len(names)
    raw = ctypes.CDLL(capi.LIB_PATH)
    for n in names:
        assert hasattr(raw, n), "libfsw_hip.so does not export %s" % n
    # the ctypes prototypes cover exactly the header
    assert sorted(capi.PROTOTYPES) == sorted(names)
    assert capi.lib().fsw_version() >= 1000


def test_probe_library_is_separate_from_the_product(capi):
    """The benchmark's measurement kernels are not part of the product ABI: their own header, their own library."""
    text = re.sub(r"/\*.*?\*/", "", open(os.path.join(ROOT, "include", "fsw_probe.h")).read(), flags=re.S)
    names = re.findall(r"FSW_PROBE_API\s+[\w\s\*]+?\b(fsw_\w+)\s*\(", text)
    assert sorted(names) == sorted(capi.PROBE_PROTOTYPES) == ["fsw_probe_mfma", "fsw_probe_read"]
    probe = ctypes.CDLL(capi.PROBE_LIB_PATH)
    product = ctypes.CDLL(capi.LIB_PATH)
    for n in names:
        assert hasattr(probe, n) and not hasattr(product, n)
    assert not [n for n in declared_symbols() if n.startswith("fsw_probe")]


def test_strerror_covers_all_codes(capi):
    seen = set()
    for code in range(0, -11, -1):
        s = capi.strerror(code)
        assert s and s not in seen
        seen.add(s)
    assert "unknown" in capi.strerror(-99)


def _v_gateup(capi, dtype=0, M=4, N=8, K=16, X=0x1000, ldx=None, W=0x2000, ldw=None, H=0x3000, ldh=None):
    return capi.lib().fsw_validate_gateup(dtype, M, N, K, X, K if ldx is None else ldx, W, K if ldw is None else ldw,
                                          H, N // 2 if ldh is None else ldh)


def test_validate_gateup_codes(capi):
    assert _v_gateup(capi) == capi.OK
    assert _v_gateup(capi, dtype=1) == capi.OK
    assert _v_gateup(capi, dtype=2) == capi.E_DTYPE
    assert _v_gateup(capi, M=-1) == capi.E_SHAPE
    assert _v_gateup(capi, N=7) == capi.E_SHAPE          # odd N: rows come in (up, gate) pairs
    assert _v_gateup(capi, M=2 ** 31) == capi.E_SHAPE
    assert _v_gateup(capi, K=12) == capi.E_ALIGN         # K % 8
    assert _v_gateup(capi, ldx=8) == capi.E_LD
    assert _v_gateup(capi, ldw=8) == capi.E_LD
    assert _v_gateup(capi, ldh=3) == capi.E_LD
    assert _v_gateup(capi, ldx=20) == capi.E_ALIGN       # ld % 8
    assert _v_gateup(capi, X=0x1008) == capi.E_ALIGN     # 16-byte rule
    assert _v_gateup(capi, W=0x2004) == capi.E_ALIGN
    assert _v_gateup(capi, X=None) == capi.E_NULL
    assert _v_gateup(capi, W=None) == capi.E_NULL
    assert _v_gateup(capi, H=None) == capi.E_NULL
    # empty problems need no pointers at all
    assert _v_gateup(capi, M=0, X=None, W=None, H=None) == capi.OK
    assert _v_gateup(capi, N=0, X=None, W=None, H=None) == capi.OK
    # K = 0 is a valid (all-zero) product
    assert _v_gateup(capi, K=0) == capi.OK


def test_validate_down_codes(capi):
    v = capi.lib().fsw_validate_down
    assert v(0, 4, 8, 16, 0x1000, 16, 0x2000, 16, 0x3000, 8) == capi.OK
    assert v(3, 4, 8, 16, 0x1000, 16, 0x2000, 16, 0x3000, 8) == capi.E_DTYPE
    assert v(0, 4, 8, 12, 0x1000, 16, 0x2000, 16, 0x3000, 8) == capi.E_ALIGN
    assert v(0, 4, 8, 16, 0x1000, 8, 0x2000, 16, 0x3000, 8) == capi.E_LD
    assert v(0, 4, 8, 16, 0x1000, 16, 0x2000, 16, 0x3000, 4) == capi.E_LD
    assert v(0, 4, 8, 16, None, 16, 0x2000, 16, 0x3000, 8) == capi.E_NULL
    assert v(0, 4, -8, 16, 0x1000, 16, 0x2000, 16, 0x3000, 8) == capi.E_SHAPE
    assert v(0, 0, 8, 16, None, 16, None, 16, None, 8) == capi.OK


def test_entry_points_reject_bad_arguments_before_touching_the_gpu(capi):
    L = capi.lib()
    # these return from validation, so they are safe on a machine without a GPU
    assert L.fsw_gateup(0, 4, 7, 16, 0x1000, 16, 0x2000, 16, 0x3000, 4, None) == capi.E_SHAPE
    assert L.fsw_gateup(5, 4, 8, 16, 0x1000, 16, 0x2000, 16, 0x3000, 4, None) == capi.E_DTYPE
    assert L.fsw_gateup(0, 0, 8, 16, None, 16, None, 16, None, 4, None) == capi.OK
    assert L.fsw_down(0, 4, 8, 12, 0x1000, 16, 0x2000, 16, 0x3000, 8, None, 0, None) == capi.E_ALIGN
    assert L.fsw_mlp(0, 4, 16, 8, 0x1000, 16, 0x2000, 16, 0x3000, 8, 0x4000, 16, None, 0, None) == capi.E_WORKSPACE
    assert L.fsw_mlp_workspace_bytes(0, 4, 16, 8) >= 4 * 8 * 2
    assert L.fsw_mlp_workspace_bytes(0, 0, 16, 8) == 0
    assert L.fsw_set_variant(0, 12345) == capi.E_VARIANT
    # the float-output form of the gate/up product: the same rules, plus a 4-byte aligned H
    f32 = L.fsw_gateup_f32out
    assert f32(0, 4, 7, 16, 0x1000, 16, 0x2000, 16, 0x3000, 4, None) == capi.E_SHAPE
    assert f32(2, 4, 8, 16, 0x1000, 16, 0x2000, 16, 0x3000, 4, None) == capi.E_DTYPE
    assert f32(0, 4, 8, 16, 0x1000, 16, 0x2000, 16, 0x3000, 3, None) == capi.E_LD
    assert f32(0, 4, 8, 16, 0x1000, 16, 0x2000, 16, 0x3002, 4, None) == capi.E_ALIGN
    assert f32(0, 4, 8, 16, 0x1000, 16, 0x2000, 16, None, 4, None) == capi.E_NULL
    assert f32(0, 0, 8, 16, None, 16, None, 16, None, 4, None) == capi.OK
    # row-major X -> blocked H: as fsw_gateup, a K of zero has no blocked representation, H 16-byte aligned
    hb = L.fsw_gateup_hblocked
    assert hb(0, 4, 8, 12, 0x1000, 16, 0x2000, 16, 0, 0x3000, None) == capi.E_ALIGN
    assert hb(0, 4, 8, 16, 0x1000, 8, 0x2000, 16, 0, 0x3000, None) == capi.E_LD
    assert hb(0, 4, 8, 0, 0x1000, 16, 0x2000, 16, 0, 0x3000, None) == capi.E_SHAPE
    assert hb(0, 4, 8, 16, 0x1000, 16, 0x2000, 16, 0, 0x3008, None) == capi.E_ALIGN
    assert hb(0, 4, 8, 16, 0x1000, 16, 0x2000, 0, 1, None, None) == capi.E_NULL   # blocked weights carry no ldw
    assert hb(0, 0, 8, 16, None, 16, None, 16, 0, None, None) == capi.OK
    # the failing barrier of the single-launch decode forward is a test hook: refused without FSW_TEST_HOOKS=1
    os.environ.pop("FSW_TEST_HOOKS", None)
    assert L.fsw_set_variant(0, 103) == capi.E_VARIANT and L.fsw_set_variant(0, 101) == capi.OK
    assert L.fsw_set_variant(0, -1) == capi.OK
    assert L.fsw_set_variant(7, 0) == capi.E_VARIANT
    assert L.fsw_set_variant(2, 4) == capi.E_VARIANT and L.fsw_set_variant(0, 6) == capi.E_VARIANT
    assert L.fsw_mlp(7, 4, 16, 8, 0x1000, 16, 0x2000, 16, 0x3000, 8, 0x4000, 16, None, 0, None) == capi.E_DTYPE
    assert L.fsw_mlp(0, 4, 0, 8, 0x1000, 0, None, 0, None, 8, None, 0, None, 0, None) == capi.OK  # D = 0: no Y
    assert L.fsw_set_variant(0, -1) == capi.OK
    with pytest.raises(capi.FswError) as ei:
        capi.check(capi.E_ALIGN)
    assert isinstance(ei.value, RuntimeError) and ei.value.code == capi.E_ALIGN


def test_variant_choice_by_regime(capi):
    name = lambda fam, M, n, k: capi.variant_name(fam, 0, M, n, k)
    assert name(0, 8192, 28672, 4096) == "pair16_256x256"
    assert name(1, 8192, 4096, 14336) == "pair16_256x256"
    assert "256x256" in name(0, 4096, 22016, 4096)
    assert name(0, 512, 5632, 1024) == "dma_128x128"     # small problem: more, smaller tiles
    assert name(0, 8, 28672, 4096) == "skinny" and name(1, 1, 4096, 14336) == "skinny"
    # the weight-streaming kernels take fewer rows the larger the weights: up to 48 / 32 / 16 rows
    assert name(0, 32, 22016, 4096) == "skinny" and name(1, 32, 4096, 14336) == "skinny"
    assert name(0, 33, 28672, 4096) == "dma_128x64" and name(1, 33, 4096, 14336) == "splitk_dma_128x128"
    assert name(0, 48, 2 * 8192, 2048) == "skinny" and name(0, 49, 2 * 8192, 2048) == "dma_128x64"
    # gate/up with 200 .. 256 tiles of 128 weight rows and a dozen rows or more: the 128 x 64 tiled kernel streams faster
    assert name(0, 16, 28672, 4096) == "dma_128x64" and name(0, 11, 28672, 4096) == "skinny"
    assert name(0, 64, 28672, 0) == "skinny"
    assert name(0, 100, 28672, 4096) == "dma_128x128"
    # at most 16 rows and d * ff >= 2^27: the persistent streaming kernel, one projection per launch
    assert name(0, 16, 2 * 28672, 8192) == "decode_stream" and name(1, 16, 8192, 28672) == "decode_stream"
    assert name(0, 17, 2 * 28672, 8192) == "dma_128x64"
    L = capi.lib()
    try:
        assert L.fsw_set_variant(0, 102) == capi.OK and L.fsw_set_variant(1, 100) == capi.OK
        assert name(0, 4, 64, 32) == "decode_stream" and name(0, 17, 64, 32) == "skinny"
        assert name(1, 16, 8192, 28672) == "skinny"          # forced weight-streaming kernel wins over the size rule
        assert L.fsw_set_variant(1, 101) == capi.E_VARIANT   # the single-launch form is a family-0 (fsw_mlp) option
        assert L.fsw_set_variant(1, 103) == capi.E_VARIANT
        assert L.fsw_set_variant(0, 104) == capi.E_VARIANT
        # with the persistent streaming kernel forced for gate/up nothing zeroes the ticket counters: no split-K streaming
        assert L.fsw_set_variant(1, 104) == capi.OK and capi.variant_name(2, 0, 4, 64, 32) == "skinny"
        assert L.fsw_set_variant(0, -1) == capi.OK
        assert capi.variant_name(2, 0, 4, 64, 32) == "stream_split" and name(1, 4, 64, 32) == "skinny"
    finally:
        L.fsw_set_variant(0, -1)
        L.fsw_set_variant(1, -1)
    # the down product with few output tiles and a deep K asks for split-K scratch; large or tiny M does not
    ws = capi.lib().fsw_down_workspace_bytes
    assert ws(0, 256, 4096, 14336) == 8 * 256 * 4096 * 4 and name(1, 256, 4096, 14336) == "splitk_dma_128x256"
    assert name(1, 160, 4096, 14336) == "splitk_dma_128x192" and name(0, 160, 28672, 4096) == "dma_128x192"
    assert name(0, 256, 28672, 4096) == "dma8w_128x256"
    assert name(1, 128, 4096, 14336) == "splitk_dma_128x128" and ws(0, 128, 4096, 14336) == 8 * 128 * 4096 * 4
    # above 256 rows: as many splits as keep all workgroups resident at once, on the tile the time estimate favours
    assert name(1, 257, 4096, 14336) == "splitk_dma_128x128" and ws(0, 257, 4096, 14336) == 5 * 257 * 4096 * 4
    assert name(1, 1024, 4096, 14336) == "splitk_pair16_256x256" and ws(0, 1024, 4096, 14336) == 4 * 1024 * 4096 * 4
    assert name(1, 2048, 4096, 14336) == "splitk_pair16_256x256" and ws(0, 2048, 4096, 14336) == 2 * 2048 * 4096 * 4
    assert name(1, 2304, 4096, 14336) == "pair16_256x256"    # 144 large tiles in one round: no split
    # 288 large tiles of a very deep K: three splits (four rounds of K / 3 instead of two of K), H stays row-major
    assert name(1, 2049, 8192, 28672) == "splitk_pair16_256x256" and ws(0, 2049, 8192, 28672) == 3 * 2049 * 8192 * 4
    # large-tile regime: fsw_down reads row-major H in whole cache lines and needs no scratch; fsw_gateup never does;
    # fsw_mlp keeps H panel-blocked between its two kernels and nothing else
    assert ws(0, 8192, 4096, 14336) == 0 and ws(0, 3000, 4096, 14336) == 0 and ws(0, 16, 4096, 14336) == 0
    assert L.fsw_gateup_workspace_bytes(0, 8192, 28672, 4096) == 0
    assert L.fsw_mlp_workspace_bytes(0, 8192, 4096, 14336) == L.fsw_blocked_bytes(8192, 14336) == 8192 * 14336 * 2
    assert L.fsw_mlp_workspace_bytes(0, 3000, 4096, 14336) == L.fsw_blocked_bytes(3000, 14336)
    assert capi.lib().fsw_mlp_workspace_bytes(0, 256, 4096, 14336) == 256 * 14336 * 2 + ws(0, 256, 4096, 14336)


def test_variant_override_is_per_thread(capi):
    """fsw_set_variant is thread-local: another thread's override neither shows here nor changes what this thread's
    workspace query and launch agree on."""
    import threading
    L = capi.lib()
    name = lambda: capi.variant_name(1, 0, 200, 512, 4096)
    assert name() == "splitk_dma_128x128" and L.fsw_down_workspace_bytes(0, 200, 512, 4096) > 0
    seen = {}

    def other():
        assert L.fsw_set_variant(1, 0) == capi.OK
        seen["name"] = name()
        seen["ws"] = L.fsw_down_workspace_bytes(0, 200, 512, 4096)

    t = threading.Thread(target=other)
    t.start()
    t.join()
    assert seen == {"name": "dma_128x128", "ws": 0}
    assert name() == "splitk_dma_128x128" and L.fsw_down_workspace_bytes(0, 200, 512, 4096) > 0


def test_ctypes_wrappers_refuse_views_the_c_abi_would_misread(capi):
    """The raw C ABI takes pointers and leading dimensions; a transposed view passes its leading-dimension test and
    would be read as if it were row-major. The wrappers apply the guards of the PyTorch operator surface before any
    GPU call (CPU tensors are refused here as well: there is no CPU path)."""
    X = torch.zeros(16, 16, dtype=torch.bfloat16)
    W = torch.zeros(32, 16, dtype=torch.bfloat16)
    with pytest.raises(capi.FswError) as ei:
        capi.gateup(X, W)
    assert ei.value.code == capi.E_DEVICE
    meta = lambda *shape: torch.empty(*shape, dtype=torch.bfloat16, device="meta")
    with pytest.raises(capi.FswError):
        capi._check_operands(meta(16, 16).t())
    Xt = torch.empty(16, 32, dtype=torch.bfloat16).t()   # [32, 16] with strides (1, 32)
    with pytest.raises(capi.FswError) as ei:
        capi._check_operands(Xt)
    assert ei.value.code in (capi.E_LD, capi.E_DEVICE)
    with pytest.raises(capi.FswError):
        capi._check_operands(torch.zeros(4, 4, 4, dtype=torch.bfloat16))


def test_packers_follow_the_reference_interleave():
    d, ff = 6, 4
    Wg = torch.arange(d * ff, dtype=torch.float32).reshape(d, ff)
    Wu = -Wg - 1
    W13 = fsw_weights.pack_w13(Wg, Wu)
    assert W13.shape == (2 * ff, d)
    for j in range(ff):
        assert torch.equal(W13[2 * j], Wu[:, j])       # even row = up (linear) operand
        assert torch.equal(W13[2 * j + 1], Wg[:, j])   # odd row = gate (SiLU) operand
    g2, u2 = fsw_weights.unpack_w13(W13)
    assert torch.equal(g2, Wg) and torch.equal(u2, Wu)
    Wd = torch.randn(ff, d)
    W2 = fsw_weights.pack_wd(Wd)
    assert W2.shape == (d, ff) and W2.is_contiguous() and torch.equal(W2.T, Wd)
    # the packed layout evaluates to the unpacked formulation (numeric_tests.py:41-43)
    X = torch.randn(3, d)
    C = X @ W13.T
    H = C[:, 0::2] * torch.nn.functional.silu(C[:, 1::2])
    assert torch.allclose(H, torch.nn.functional.silu(X @ Wg) * (X @ Wu), atol=1e-5)


def test_work_formulas_match_the_published_tables():
    # FLOPs and bytes of the five configurations
    want = {"C1": (8858370048, 25165824), "C2": (1108101562368, 517996544), "C3": (2886218022912, 956301312),
            "C4": (5637144576, 353501184), "C5": (2886218022912, 1711276032)}
    for name, M, d, ff, dtype, seed, xs in fsw_weights.CONFIGS:
        assert (fsw_weights.flops(M, d, ff), fsw_weights.hbm_bytes(M, d, ff)) == want[name]
    assert fsw_weights.reference_gateup_flops(8192, 28672, 4096) == 1924615110656  # bench_swiglu.py:117


def test_seeded_inputs_are_reproducible_and_scaled():
    a = fsw_weights.make_inputs(64, 256, 512, torch.bfloat16, seed=3)
    b = fsw_weights.make_inputs(64, 256, 512, torch.bfloat16, seed=3)
    for k in ("X", "W13", "W2"):
        assert torch.equal(a[k], b[k])
    assert abs(a["X"].float().std().item() - 1.0) < 0.05
    assert abs(a["Wg"].float().std().item() * 16 - 1.0) < 0.05          # 1/sqrt(256)
    assert abs(a["Wd"].float().std().item() * 512 ** 0.5 - 1.0) < 0.05  # 1/sqrt(512)


def test_operator_surface_matches_the_reference(ext):
    # pybind functions (torch_bindings.cpp:31-36)
    assert callable(ext.fused_swiglu_bf16) and callable(ext.swiglu_fwd_bf16)
    # dispatcher schemas (torch_bindings.cpp:38-43), byte for byte
    s1 = str(torch.ops.ASMLLM.fused_swiglu_bf16.default._schema)
    s2 = str(torch.ops.ASMLLM.swiglu_fwd_bf16.default._schema)
    assert s1 == "ASMLLM::fused_swiglu_bf16(Tensor X, Tensor W1W3) -> Tensor"
    assert s2 == ("ASMLLM::swiglu_fwd_bf16(int m, int n, int k, Tensor A, int ldA, Tensor B, int ldB, Tensor C, "
                  "int ldC) -> ()")
    for extra in ("fused_swiglu_fp16", "swiglu_down_bf16", "swiglu_down_fp16", "fused_swiglu_mlp_bf16",
                  "fused_swiglu_mlp_fp16"):
        assert hasattr(ext, extra) and hasattr(torch.ops.ASMLLM, extra)


def test_wrong_dtype_raises_runtime_error_like_the_reference(ext):
    # swiglu.cu:475-480: TORCH_CHECK on the dtypes -> RuntimeError; fp16/fp32 inputs are rejected by the bf16 op
    X32, W32 = torch.zeros(4, 8), torch.zeros(6, 8)
    with pytest.raises(RuntimeError, match="Expected tensor A to be of type"):
        ext.fused_swiglu_bf16(X32, W32)
    with pytest.raises(RuntimeError, match="Expected tensor A to be of type"):
        ext.fused_swiglu_bf16(X32.half(), W32.half())
    with pytest.raises(RuntimeError, match="Expected tensor B to be of type"):
        ext.swiglu_fwd_bf16(4, 6, 8, X32.bfloat16(), 8, W32, 8, torch.zeros(4, 6, dtype=torch.bfloat16), 6)
    with pytest.raises(RuntimeError, match="Expected tensor C to be of type"):
        # float32 is the reference's other output type (constants.cuh:9-14) and is accepted; float16 is not
        ext.swiglu_fwd_bf16(4, 6, 8, X32.bfloat16(), 8, W32.bfloat16(), 8, torch.zeros(4, 6, dtype=torch.float16), 6)
    # CPU tensors of the right dtype are refused (no CPU fallback exists)
    with pytest.raises(RuntimeError, match="GPU"):
        ext.fused_swiglu_bf16(X32.bfloat16(), W32.bfloat16())
    with pytest.raises(RuntimeError):
        ext.fused_swiglu_bf16(torch.zeros(4, 8, dtype=torch.bfloat16), torch.zeros(6, 16, dtype=torch.bfloat16))


def test_meta_kernels_trace_shapes_without_a_gpu(ext):
    """Shape-only kernels registered under the Meta key: the ops can be traced by FakeTensor / torch.compile
    front ends on a machine with no GPU. The mutation-annotated variant of swiglu_fwd_bf16 declares its write."""
    X = torch.empty(33, 64, dtype=torch.bfloat16, device="meta")
    W = torch.empty(80, 64, dtype=torch.bfloat16, device="meta")
    W2 = torch.empty(64, 40, dtype=torch.bfloat16, device="meta")
    H = torch.ops.ASMLLM.fused_swiglu_bf16(X, W)
    assert H.shape == (33, 40) and H.dtype == torch.bfloat16 and H.device.type == "meta"
    assert torch.ops.ASMLLM.swiglu_down_bf16(H, W2).shape == (33, 64)
    assert torch.ops.ASMLLM.fused_swiglu_mlp_bf16(X, W, W2).shape == (33, 64)
    assert torch.ops.ASMLLM.fused_swiglu_mlp_fp16(X.half(), W.half(), W2.half()).dtype == torch.float16
    with pytest.raises(RuntimeError):
        torch.ops.ASMLLM.fused_swiglu_bf16(X.half(), W.half())
    with pytest.raises(RuntimeError):
        torch.ops.ASMLLM.fused_swiglu_bf16(X, torch.empty(80, 32, dtype=torch.bfloat16, device="meta"))
    schema = torch.ops.ASMLLM.swiglu_fwd_bf16_out.default._schema
    assert schema.arguments[7].name == "C" and schema.arguments[7].alias_info is not None and schema.arguments[7].alias_info.is_write
    assert not torch.ops.ASMLLM.swiglu_fwd_bf16.default._schema.arguments[7].alias_info  # the reference's schema, kept as is
    from torch._subclasses.fake_tensor import FakeTensorMode
    with FakeTensorMode():
        a = torch.empty(5, 16, dtype=torch.bfloat16, device="cuda")
        b = torch.empty(12, 16, dtype=torch.bfloat16, device="cuda")
        assert torch.ops.ASMLLM.fused_swiglu_bf16(a, b).shape == (5, 6)
