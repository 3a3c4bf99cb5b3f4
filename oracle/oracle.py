"""CPU oracle for the fused SwiGLU MLP forward. TEST INFRASTRUCTURE ONLY.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg import this module; the shipped library
and its bindings never do. It holds two statements of the same formulation:

  * `c_*`      — thin ctypes wrappers over oracle/swiglu_oracle.c (double accumulation, plain loops), used on
                 small shapes and to pin the fast statement below;
  * `ref_*`    — the reference's own three lines of stock PyTorch (numeric_tests.py:41-43, second statement at
                 bench_swiglu.py:31-32) evaluated on the CPU in fp32 or fp64 on the dtype-rounded inputs:
                     C = X @ W1W3.T ; H = C[:, 0::2] * silu(C[:, 1::2]) ; Y = H @ W2.T
                 plus the unpacked form (silu(X @ Wg) * (X @ Wu)) @ Wd, which never touches the packed layout
                 and therefore also checks the packers.

Parity pinning: the reference holds no golden vectors for this path (numeric_tests.py is unseeded and asserts
nothing) and cannot be built here (nvcc and the CUTLASS submodule are absent), so every function is pinned by
tests/test_oracle.py: brute-force Python loops on tiny shapes, SiLU closed forms, one-hot probes of the
even = up / odd = gate convention (swiglu.cu:380-381), and agreement between the C and torch statements.
"""
import ctypes
import os
import subprocess

import numpy as np
import torch
import torch.nn.functional as F

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "_build", "liboracle.so")

BF16, FP16 = 0, 1
# tolerance gates: max |out - ref| and mean|out - ref| / mean|ref|
MAX_ABS_TOL = 2e-2
MEAN_REL_TOL = 5e-3

_lib = None


def build():
    """Compile oracle/swiglu_oracle.c with gcc (seconds)."""
    subprocess.run(["make", "-C", HERE, "-B"], check=True, stdout=subprocess.DEVNULL)
    return LIB_PATH


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            build()
        L = ctypes.CDLL(LIB_PATH)
        i64, vp = ctypes.c_int64, ctypes.c_void_p
        L.oracle_gateup.argtypes = [ctypes.c_int, i64, i64, i64, vp, i64, vp, i64, vp, i64]
        L.oracle_down.argtypes = [ctypes.c_int, i64, i64, i64, vp, i64, vp, i64, vp, i64]
        L.oracle_down_f64.argtypes = [ctypes.c_int, i64, i64, i64, vp, i64, vp, i64, vp, i64]
        for f in (L.oracle_gateup, L.oracle_down, L.oracle_down_f64):
            f.restype = ctypes.c_int
        L.oracle_silu.argtypes = [ctypes.c_double]
        L.oracle_silu.restype = ctypes.c_double
        L.oracle_bf16_to_f32.argtypes = [ctypes.c_uint16]
        L.oracle_bf16_to_f32.restype = ctypes.c_float
        L.oracle_f16_to_f32.argtypes = [ctypes.c_uint16]
        L.oracle_f16_to_f32.restype = ctypes.c_float
        L.oracle_f32_to_bf16.argtypes = [ctypes.c_float]
        L.oracle_f32_to_bf16.restype = ctypes.c_uint16
        L.oracle_f32_to_f16.argtypes = [ctypes.c_float]
        L.oracle_f32_to_f16.restype = ctypes.c_uint16
        _lib = L
    return _lib


def dtype_code(t):
    if t.dtype == torch.bfloat16:
        return BF16
    if t.dtype == torch.float16:
        return FP16
    raise TypeError("oracle: expected a bf16 or fp16 tensor, got %s" % t.dtype)


def _bits(t):
    """16-bit encodings of a 2-D CPU half tensor as a C-contiguous uint16 array."""
    assert t.dim() == 2 and t.device.type == "cpu"
    return np.ascontiguousarray(t.contiguous().view(torch.int16).numpy().view(np.uint16))


def c_gateup(X, W13):
    """H (float64, unrounded) from oracle_gateup. X [M,K], W13 [2ff,K], both bf16 or both fp16, on the CPU."""
    code = dtype_code(X)
    assert dtype_code(W13) == code and X.shape[1] == W13.shape[1] and W13.shape[0] % 2 == 0
    M, K = X.shape
    N = W13.shape[0]
    xb, wb = _bits(X), _bits(W13)
    H = np.zeros((M, N // 2), dtype=np.float64)
    rc = lib().oracle_gateup(code, M, N, K, xb.ctypes.data, K, wb.ctypes.data, K, H.ctypes.data, N // 2)
    assert rc == 0
    return torch.from_numpy(H)


def c_down(H, W2):
    """Y (float64) = H @ W2.T from the C loops; H is a half tensor [M,FF] or a float64 tensor, W2 [D,FF] half."""
    code = dtype_code(W2)
    M, FF = H.shape
    D = W2.shape[0]
    assert W2.shape[1] == FF
    wb = _bits(W2)
    Y = np.zeros((M, D), dtype=np.float64)
    if H.dtype == torch.float64:
        hb = np.ascontiguousarray(H.numpy())
        rc = lib().oracle_down_f64(code, M, D, FF, hb.ctypes.data, FF, wb.ctypes.data, FF, Y.ctypes.data, D)
    else:
        assert dtype_code(H) == code
        hb = _bits(H)
        rc = lib().oracle_down(code, M, D, FF, hb.ctypes.data, FF, wb.ctypes.data, FF, Y.ctypes.data, D)
    assert rc == 0
    return torch.from_numpy(Y)


def c_mlp(X, W13, W2):
    """Y (float64) of the whole forward from the C loops, H kept unrounded."""
    return c_down(c_gateup(X, W13), W2)


def ref_gateup(X, W13, dtype=torch.float32):
    """numeric_tests.py:41-43 on the CPU at `dtype` precision, from the rounded 16-bit inputs."""
    C = X.to(dtype) @ W13.to(dtype).T
    return C[:, 0::2] * F.silu(C[:, 1::2])


def ref_down(H, W2, dtype=torch.float32):
    return H.to(dtype) @ W2.to(dtype).T


def ref_mlp(X, W13, W2, dtype=torch.float32):
    """Whole forward at `dtype` precision with no intermediate rounding of H."""
    return ref_down(ref_gateup(X, W13, dtype), W2, dtype)


def ref_mlp_unpacked(X, Wg, Wu, Wd, dtype=torch.float32):
    """(silu(X @ Wg) * (X @ Wu)) @ Wd with Wg, Wu [d, ff] and Wd [ff, d] in their mathematical orientation."""
    Xd = X.to(dtype)
    return (F.silu(Xd @ Wg.to(dtype)) * (Xd @ Wu.to(dtype))) @ Wd.to(dtype)


def error_metrics(out, ref):
    """max|d|, mean|d|, mean|d|/mean|ref| and ||d||_F/||ref||_F (the three statistics of numeric_tests.py:49-52
    plus the mean-relative gate)."""
    d = out.detach().cpu().double() - ref.detach().cpu().double()
    r = ref.detach().cpu().double()
    max_abs = d.abs().max().item() if d.numel() else 0.0
    mean_abs = d.abs().mean().item() if d.numel() else 0.0
    mean_ref = r.abs().mean().item() if r.numel() else 0.0
    fro_ref = r.norm().item() if r.numel() else 0.0
    return {
        "max_abs": max_abs,
        "mean_abs": mean_abs,
        "mean_rel": mean_abs / mean_ref if mean_ref > 0 else (0.0 if mean_abs == 0 else float("inf")),
        "fro_rel": d.norm().item() / fro_ref if fro_ref > 0 else (0.0 if mean_abs == 0 else float("inf")),
    }


def passes(metrics, max_abs_tol=MAX_ABS_TOL, mean_rel_tol=MEAN_REL_TOL):
    return (metrics["max_abs"] <= max_abs_tol and metrics["mean_rel"] <= mean_rel_tol
            and metrics["fro_rel"] <= mean_rel_tol)


def assert_parity(out, ref, what="", max_abs_tol=MAX_ABS_TOL, mean_rel_tol=MEAN_REL_TOL):
    assert tuple(out.shape) == tuple(ref.shape), "%s: shape %s vs %s" % (what, tuple(out.shape), tuple(ref.shape))
    assert torch.isfinite(out.float()).all(), "%s: non-finite values in the output" % what
    m = error_metrics(out, ref)
    assert passes(m, max_abs_tol, mean_rel_tol), "%s: parity failed %s (gates: max_abs<=%g, mean_rel<=%g)" % (
        what, m, max_abs_tol, mean_rel_tol)
    return m
