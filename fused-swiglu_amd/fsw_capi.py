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
E_NULL, E_DTYPE, E_SHAPE, E_LD, E_ALIGN, E_WORKSPACE, E_LAUNCH, E_DEVICE, E_VARIANT = range(-1, -10, -1)

# name -> (restype, argtypes); the list the loader test checks against include/fsw.h
_i, _i64, _vp, _sz, _cp = ctypes.c_int, ctypes.c_int64, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_char_p
PROTOTYPES = {
    "fsw_validate_gateup": (_i, [_i, _i64, _i64, _i64, _vp, _i64, _vp, _i64, _vp, _i64]),
    "fsw_gateup": (_i, [_i, _i64, _i64, _i64, _vp, _i64, _vp, _i64, _vp, _i64, _vp]),
    "fsw_validate_down": (_i, [_i, _i64, _i64, _i64, _vp, _i64, _vp, _i64, _vp, _i64]),
    "fsw_down_workspace_bytes": (_sz, [_i, _i64, _i64, _i64]),
    "fsw_down": (_i, [_i, _i64, _i64, _i64, _vp, _i64, _vp, _i64, _vp, _i64, _vp, _sz, _vp]),
    "fsw_mlp_workspace_bytes": (_sz, [_i, _i64, _i64, _i64]),
    "fsw_mlp": (_i, [_i, _i64, _i64, _i64, _vp, _i64, _vp, _i64, _vp, _i64, _vp, _i64, _vp, _sz, _vp]),
    "fsw_strerror": (_cp, [_i]),
    "fsw_last_hip_error": (_i, []),
    "fsw_version": (_i, []),
    "fsw_set_variant": (_i, [_i, _i]),
    "fsw_variant_name": (_cp, [_i, _i, _i64, _i64, _i64]),
}

_lib = None


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
        L = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in PROTOTYPES.items():
            fn = getattr(L, name)
            fn.restype, fn.argtypes = res, args
        _lib = L
    return _lib


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


def gateup(X, W13, out=None):
    """H[M, ff] = up * silu(gate) through fsw_gateup on the current stream. X [M,K], W13 [2ff,K] device tensors."""
    import torch
    code = dtype_code(X)
    if W13.dtype != X.dtype:
        raise FswError(E_DTYPE, "fsw: X and W13 differ in element type")
    M, K = X.shape
    N = W13.shape[0]
    if out is None:
        out = torch.empty((M, N // 2), dtype=X.dtype, device=X.device)
    with torch.cuda.device(X.device):
        check(lib().fsw_gateup(code, M, N, K, X.data_ptr(), _ld(X), W13.data_ptr(), _ld(W13), out.data_ptr(),
                               _ld(out), _stream(X)))
    return out


def down(H, W2, out=None):
    """Y[M, D] = H @ W2.T through fsw_down on the current stream. H [M,FF], W2 [D,FF] device tensors."""
    import torch
    code = dtype_code(H)
    if W2.dtype != H.dtype:
        raise FswError(E_DTYPE, "fsw: H and W2 differ in element type")
    M, FF = H.shape
    D = W2.shape[0]
    if out is None:
        out = torch.empty((M, D), dtype=H.dtype, device=H.device)
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
    M, D = X.shape
    FF = W13.shape[0] // 2
    if out is None:
        out = torch.empty((M, D), dtype=X.dtype, device=X.device)
    if workspace is None:
        workspace = mlp_workspace(X, FF)
    with torch.cuda.device(X.device):
        check(lib().fsw_mlp(code, M, D, FF, X.data_ptr(), _ld(X), W13.data_ptr(), _ld(W13), W2.data_ptr(), _ld(W2),
                            out.data_ptr(), _ld(out), workspace.data_ptr(), workspace.numel(), _stream(X)))
    return out


def set_variant(family, variant):
    check(lib().fsw_set_variant(family, variant))


def variant_name(family, dtype, M, n, k):
    return lib().fsw_variant_name(family, dtype, M, n, k).decode()
