"""ctypes binding of the C ABI declared in include/fsw.h (libfsw_hip.so).

This is the foreign-function stub a maintainer of the reference would add to call the MI355X path without the
PyTorch extension; tensors are only used as owners of device memory (data_ptr) and of the current stream.
The library is never built from here: a missing libfsw_hip.so is an error, not a reason to fall back.
"""
import ctypes
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libfsw_hip.so")

BF16, FP16 = 0, 1
OK = 0
E_NULL, E_DTYPE, E_SHAPE, E_LD, E_ALIGN, E_WORKSPACE, E_LAUNCH, E_DEVICE, E_VARIANT, E_STATIC_LIMIT = range(-1, -11, -1)

# name -> (restype, argtypes); the list the loader test checks against include/fsw.h
_i, _i64, _vp, _sz, _cp = ctypes.c_int, ctypes.c_int64, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_char_p
PROTOTYPES = {
    "fsw_validate_gateup": (_i, [_i, _i64, _i64, _i64, _vp, _i64, _vp, _i64, _vp, _i64]),
    "fsw_gateup": (_i, [_i, _i64, _i64, _i64, _vp, _i64, _vp, _i64, _vp, _i64, _vp]),
    "fsw_gateup_f32out": (_i, [_i, _i64, _i64, _i64, _vp, _i64, _vp, _i64, _vp, _i64, _vp]),
    "fsw_validate_down": (_i, [_i, _i64, _i64, _i64, _vp, _i64, _vp, _i64, _vp, _i64]),
    "fsw_down_workspace_bytes": (_sz, [_i, _i64, _i64, _i64]),
    "fsw_down": (_i, [_i, _i64, _i64, _i64, _vp, _i64, _vp, _i64, _vp, _i64, _vp, _sz, _vp]),
    "fsw_mlp_workspace_bytes": (_sz, [_i, _i64, _i64, _i64]),
    "fsw_mlp": (_i, [_i, _i64, _i64, _i64, _vp, _i64, _vp, _i64, _vp, _i64, _vp, _i64, _vp, _sz, _vp]),
    "fsw_mlp_static_max_bytes": (_sz, []),
    "fsw_mlp_static": (_i, [_i, _i64, _i64, _i64, _vp, _i64, _vp, _i64, _vp, _i64, _vp, _i64, _vp]),
    "fsw_blocked_bytes": (_sz, [_i64, _i64]),
    "fsw_block_rows": (_i, [_i, _i64, _i64, _vp, _i64, _vp, _vp]),
    "fsw_prepack_w13": (_i, [_i, _i64, _i64, _vp, _i64, _vp, _vp]),
    "fsw_prepack_w2": (_i, [_i, _i64, _i64, _vp, _i64, _vp, _vp]),
    "fsw_gateup_blocked": (_i, [_i, _i64, _i64, _i64, _vp, _vp, _i64, _i, _vp, _i64, _vp]),
    "fsw_gateup_hblocked": (_i, [_i, _i64, _i64, _i64, _vp, _i64, _vp, _i64, _i, _vp, _vp]),
    "fsw_down_blocked": (_i, [_i, _i64, _i64, _i64, _vp, _vp, _i64, _i, _vp, _i64, _vp]),
    "fsw_gateup_workspace_bytes": (_sz, [_i, _i64, _i64, _i64]),
    "fsw_gateup_ws": (_i, [_i, _i64, _i64, _i64, _vp, _i64, _vp, _i64, _vp, _i64, _vp, _sz, _vp]),
    "fsw_strerror": (_cp, [_i]),
    "fsw_last_hip_error": (_i, []),
    "fsw_decode_barrier_failures": (_i, []),
    "fsw_version": (_i, []),
    "fsw_set_variant": (_i, [_i, _i]),
    "fsw_variant_name": (_cp, [_i, _i, _i64, _i64, _i64]),
}

# the benchmark's measurement kernels live in a library of their own (include/fsw_probe.h)
PROBE_LIB_PATH = os.path.join(HERE, "libfsw_probe.so")
PROBE_PROTOTYPES = {
    "fsw_probe_mfma": (_i, [_i, _i, _vp, _vp, _i, _vp]),
    "fsw_probe_read": (_i, [_vp, _sz, _vp, _i, _vp]),
}

_lib = None
_probe_lib = None


class FswError(RuntimeError):
    """An FSW_E_* code from the library (RuntimeError, the failure mode of the reference's TORCH_CHECKs)."""

    def __init__(self, code, text):
        super().__init__("%s (code %d)" % (text, code))
        self.code = code


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise FileNotFoundError(
                "%s is missing: build it with `python setup.py build_hip` in %s" % (LIB_PATH, HERE))
        # torch ships its own HIP runtime: when it is installed, load it first, so that this process holds one
        # runtime only (loaded the other way round, the library's launches fail with FSW_E_DEVICE)
        try:
            import torch  # noqa: F401
        except ImportError:
            pass
        L = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in PROTOTYPES.items():
            fn = getattr(L, name)
            fn.restype, fn.argtypes = res, args
        _lib = L
    return _lib


def probe_lib():
    """libfsw_probe.so (measurement kernels for bench.py), loaded after the product library."""
    global _probe_lib
    if _probe_lib is None:
        lib()
        if not os.path.exists(PROBE_LIB_PATH):
            raise FileNotFoundError("%s is missing: build it with `python setup.py build_hip` in %s" % (PROBE_LIB_PATH, HERE))
        L = ctypes.CDLL(PROBE_LIB_PATH)
        for name, (res, args) in PROBE_PROTOTYPES.items():
            fn = getattr(L, name)
            fn.restype, fn.argtypes = res, args
        _probe_lib = L
    return _probe_lib


def strerror(code):
    return lib().fsw_strerror(code).decode()


def check(code):
    if code != OK:
        raise FswError(code, strerror(code))


def dtype_code(t):
    import torch
    if t.dtype == torch.bfloat16:
        return BF16
    if t.dtype == torch.float16:
        return FP16
    raise FswError(E_DTYPE, strerror(E_DTYPE))


def _stream(t):
    import torch
    return torch.cuda.current_stream(t.device).cuda_stream


def _ld(t):
    """Row stride in elements; degenerate shapes (one row, empty rows) report the row length."""
    if t.shape[0] > 1 and t.shape[1] > 0:
        return t.stride(0)
    return t.shape[1]


def _check_operands(first, *others, out=None, out_shape=None, workspace=None):
    """The guards of the PyTorch operator surface, for callers of the raw C ABI: 2-D device tensors with a unit
    inner stride, all on one device; `out` of the same type with the expected shape; `workspace` a uint8 device
    tensor. A transposed view passes a leading-dimension test and would be read as if it were row-major."""
    import torch
    for t in (first,) + others + ((out,) if out is not None else ()):
        if t.dim() != 2:
            raise FswError(E_SHAPE, "fsw: operands must be 2-D")
        if not t.is_cuda:
            raise FswError(E_DEVICE, "fsw: operands must be device tensors")
        if t.device != first.device:
            raise FswError(E_DEVICE, "fsw: operands live on different devices")
        if t.shape[1] > 1 and t.stride(1) != 1:
            raise FswError(E_LD, "fsw: operands must be contiguous in their last dimension")
        if t.shape[0] > 1 and t.shape[1] > 0 and t.stride(0) < t.shape[1]:
            raise FswError(E_LD, "fsw: overlapping rows")
    if out is not None:
        if out.dtype != first.dtype or tuple(out.shape) != tuple(out_shape):
            raise FswError(E_SHAPE, "fsw: `out` must be a %s tensor of shape %s" % (first.dtype, tuple(out_shape)))
    if workspace is not None:
        if workspace.dtype != torch.uint8 or not workspace.is_cuda or workspace.device != first.device or \
                not workspace.is_contiguous():
            raise FswError(E_WORKSPACE, "fsw: workspace must be a contiguous uint8 tensor on the operands' device")


def gateup(X, W13, out=None):
    """H[M, ff] = up * silu(gate) through fsw_gateup on the current stream. X [M,K], W13 [2ff,K] device tensors."""
    import torch
    code = dtype_code(X)
    if W13.dtype != X.dtype:
        raise FswError(E_DTYPE, "fsw: X and W13 differ in element type")
    _check_operands(X, W13)
    M, K = X.shape
    N = W13.shape[0]
    if W13.shape[1] != K:
        raise FswError(E_SHAPE, "fsw: X is [M, K] and W13 is [2 ff, K]: K differs")
    if out is None:
        out = torch.empty((M, N // 2), dtype=X.dtype, device=X.device)
    _check_operands(X, out=out, out_shape=(M, N // 2))
    with torch.cuda.device(X.device):
        check(lib().fsw_gateup(code, M, N, K, X.data_ptr(), _ld(X), W13.data_ptr(), _ld(W13), out.data_ptr(),
                               _ld(out), _stream(X)))
    return out


def gateup_f32out(X, W13, out=None):
    """H[M, ff] as float32, the gated fp32 value unrounded, through fsw_gateup_f32out."""
    import torch
    code = dtype_code(X)
    if W13.dtype != X.dtype:
        raise FswError(E_DTYPE, "fsw: X and W13 differ in element type")
    _check_operands(X, W13)
    M, K = X.shape
    N = W13.shape[0]
    if W13.shape[1] != K:
        raise FswError(E_SHAPE, "fsw: X is [M, K] and W13 is [2 ff, K]: K differs")
    if out is None:
        out = torch.empty((M, N // 2), dtype=torch.float32, device=X.device)
    if out.dtype != torch.float32 or tuple(out.shape) != (M, N // 2):
        raise FswError(E_SHAPE, "fsw: `out` must be a float32 tensor of shape %s" % ((M, N // 2),))
    _check_operands(out)
    with torch.cuda.device(X.device):
        check(lib().fsw_gateup_f32out(code, M, N, K, X.data_ptr(), _ld(X), W13.data_ptr(), _ld(W13), out.data_ptr(),
                                      _ld(out), _stream(X)))
    return out


def down(H, W2, out=None):
    """Y[M, D] = H @ W2.T through fsw_down on the current stream. H [M,FF], W2 [D,FF] device tensors."""
    import torch
    code = dtype_code(H)
    if W2.dtype != H.dtype:
        raise FswError(E_DTYPE, "fsw: H and W2 differ in element type")
    _check_operands(H, W2)
    M, FF = H.shape
    D = W2.shape[0]
    if W2.shape[1] != FF:
        raise FswError(E_SHAPE, "fsw: H is [M, FF] and W2 is [D, FF]: FF differs")
    if out is None:
        out = torch.empty((M, D), dtype=H.dtype, device=H.device)
    _check_operands(H, out=out, out_shape=(M, D))
    nbytes = lib().fsw_down_workspace_bytes(code, M, D, FF)
    ws = torch.empty(nbytes, dtype=torch.uint8, device=H.device) if nbytes else None
    with torch.cuda.device(H.device):
        check(lib().fsw_down(code, M, D, FF, H.data_ptr(), _ld(H), W2.data_ptr(), _ld(W2), out.data_ptr(), _ld(out),
                             ws.data_ptr() if ws is not None else None, nbytes, _stream(H)))
    return out


def mlp_workspace(X, FF):
    import torch
    M, D = X.shape
    nbytes = lib().fsw_mlp_workspace_bytes(dtype_code(X), M, D, FF)
    return torch.empty(max(nbytes, 16), dtype=torch.uint8, device=X.device)


def mlp(X, W13, W2, out=None, workspace=None):
    """Y = (silu(X @ Wg) * (X @ Wu)) @ Wd through fsw_mlp. `workspace` (uint8 device tensor) may be reused."""
    import torch
    code = dtype_code(X)
    if W13.dtype != X.dtype or W2.dtype != X.dtype:
        raise FswError(E_DTYPE, "fsw: X, W13 and W2 differ in element type")
    _check_operands(X, W13, W2)
    M, D = X.shape
    FF = W13.shape[0] // 2
    if W13.shape[1] != D or tuple(W2.shape) != (D, FF):
        raise FswError(E_SHAPE, "fsw: X is [M, d], W13 is [2 ff, d] and W2 is [d, ff]")
    if out is None:
        out = torch.empty((M, D), dtype=X.dtype, device=X.device)
    if workspace is None:
        workspace = mlp_workspace(X, FF)
    _check_operands(X, out=out, out_shape=(M, D), workspace=workspace)
    with torch.cuda.device(X.device):
        check(lib().fsw_mlp(code, M, D, FF, X.data_ptr(), _ld(X), W13.data_ptr(), _ld(W13), W2.data_ptr(), _ld(W2),
                            out.data_ptr(), _ld(out), workspace.data_ptr(), workspace.numel(), _stream(X)))
    return out


def mlp_static(X, W13, W2, out):
    """fsw_mlp_static: the forward with the library's own static scratch; `out` is required (nothing is allocated)."""
    import torch
    code = dtype_code(X)
    if W13.dtype != X.dtype or W2.dtype != X.dtype:
        raise FswError(E_DTYPE, "fsw: X, W13 and W2 differ in element type")
    _check_operands(X, W13, W2)
    M, D = X.shape
    FF = W13.shape[0] // 2
    if W13.shape[1] != D or tuple(W2.shape) != (D, FF):
        raise FswError(E_SHAPE, "fsw: X is [M, d], W13 is [2 ff, d] and W2 is [d, ff]")
    _check_operands(X, out=out, out_shape=(M, D))
    with torch.cuda.device(X.device):
        check(lib().fsw_mlp_static(code, M, D, FF, X.data_ptr(), _ld(X), W13.data_ptr(), _ld(W13), W2.data_ptr(),
                                   _ld(W2), out.data_ptr(), _ld(out), _stream(X)))
    return out


class Blocked:
    """A panel-blocked device copy of a row-major [rows, k] matrix (fsw.h: blocks of [256 rows][32 elements])."""

    def __init__(self, buf, rows, k, dtype):
        self.buf, self.rows, self.k, self.dtype = buf, rows, k, dtype

    def data_ptr(self):
        return self.buf.data_ptr()


def _blocked_empty(rows, k, like):
    import torch
    n = lib().fsw_blocked_bytes(rows, k)
    return Blocked(torch.empty(max(n, 16), dtype=torch.uint8, device=like.device), rows, k, like.dtype)


def block_rows(A, kind="rows"):
    """Row-major device matrix -> Blocked. kind: "rows" (X, H, W2) or "w13" (up/gate rows de-interleaved per panel)."""
    import torch
    _check_operands(A)
    rows, k = A.shape
    out = _blocked_empty(rows, k, A)
    fn = {"rows": lib().fsw_block_rows, "w13": lib().fsw_prepack_w13, "w2": lib().fsw_prepack_w2}[kind]
    with torch.cuda.device(A.device):
        check(fn(dtype_code(A), rows, k, A.data_ptr(), _ld(A), out.data_ptr(), _stream(A)))
    return out


def unblock(B):
    """Blocked -> row-major torch tensor (host-side index arithmetic on the device buffer; for tests)."""
    import torch
    panels, nkt = (B.rows + 255) // 256, (B.k + 31) // 32
    t = B.buf[: panels * nkt * 256 * 64].view(B.dtype).view(panels, nkt, 256, 32)
    return t.permute(0, 2, 1, 3).reshape(panels * 256, nkt * 32)[: B.rows, : B.k].contiguous()


def gateup_blocked(Xb, W13, row_major_out=False):
    """Gate/up of a Blocked X: returns a Blocked H, or a row-major tensor with row_major_out. W13: row-major tensor
    or a Blocked from block_rows(W13, "w13")."""
    import torch
    wb = isinstance(W13, Blocked)
    N = W13.rows if wb else W13.shape[0]
    like = Xb.buf
    if row_major_out:
        H = torch.empty((Xb.rows, N // 2), dtype=Xb.dtype, device=like.device)
        ldh = max(N // 2, 1)
    else:
        H = Blocked(torch.empty(max(lib().fsw_blocked_bytes(Xb.rows, N // 2), 16), dtype=torch.uint8,
                                device=like.device), Xb.rows, N // 2, Xb.dtype)
        ldh = 0
    code = BF16 if Xb.dtype == torch.bfloat16 else FP16
    with torch.cuda.device(like.device):
        check(lib().fsw_gateup_blocked(code, Xb.rows, N, Xb.k, Xb.data_ptr(), W13.data_ptr(), 0 if wb else _ld(W13),
                                       1 if wb else 0, H.data_ptr(), ldh, _stream(like)))
    return H


def gateup_hblocked(X, W13):
    """Gate/up of a row-major X written as a Blocked H (what fsw_mlp runs in the large-tile regime). W13: row-major
    tensor or a Blocked from block_rows(W13, "w13")."""
    import torch
    _check_operands(X)
    wb = isinstance(W13, Blocked)
    if not wb:
        _check_operands(X, W13)
    N = W13.rows if wb else W13.shape[0]
    M, K = X.shape
    H = _blocked_empty(M, N // 2, X)
    with torch.cuda.device(X.device):
        check(lib().fsw_gateup_hblocked(dtype_code(X), M, N, K, X.data_ptr(), _ld(X), W13.data_ptr(),
                                        0 if wb else _ld(W13), 1 if wb else 0, H.data_ptr(), _stream(X)))
    return H


def down_blocked(Hb, W2, out=None):
    """Row-major Y = Blocked H @ W2.T. W2: row-major tensor or a Blocked from block_rows(W2, "w2")."""
    import torch
    wb = isinstance(W2, Blocked)
    D = W2.rows if wb else W2.shape[0]
    like = Hb.buf
    if out is None:
        out = torch.empty((Hb.rows, D), dtype=Hb.dtype, device=like.device)
    code = BF16 if Hb.dtype == torch.bfloat16 else FP16
    with torch.cuda.device(like.device):
        check(lib().fsw_down_blocked(code, Hb.rows, D, Hb.k, Hb.data_ptr(), W2.data_ptr(), 0 if wb else _ld(W2),
                                     1 if wb else 0, out.data_ptr(), _ld(out), _stream(like)))
    return out


def set_variant(family, variant):
    check(lib().fsw_set_variant(family, variant))


def decode_barrier_failures():
    """Single-launch decode forwards whose device-wide barrier gave up since the last call (synchronous)."""
    n = lib().fsw_decode_barrier_failures()
    if n < 0:
        check(n)
    return n


def variant_name(family, dtype, M, n, k):
    return lib().fsw_variant_name(family, dtype, M, n, k).decode()
