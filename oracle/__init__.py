"""CPU oracle for the gated linear scan -- TEST INFRASTRUCTURE, never the product path.

Only tests/, `__graft_entry__.smoke()` and bench.py's `cpu_baseline` leg import this package.
quick_ssm_amd never does.

  scan_oracle.c          C restatement of the reference's sequential algorithm (float64 truth and
                         an fp32 flavour in the reference's operation order)
  reference_cpu_path.py  torch restatement of the reference's CPU execution path, loop for loop,
                         including its rounding points; what the cpu_baseline leg times

Parity status: every function here is pinned by tests/test_oracle.py (exact rational vectors in
tests/golden, closed forms, finite differences, cross-checks between the C and torch flavours).
Nothing is "parity unpinned".
"""
from __future__ import annotations

import ctypes
import os
import subprocess
from pathlib import Path
from typing import Optional, Tuple

import numpy as np

ORACLE_DIR = Path(__file__).resolve().parent
LIB_PATH = ORACLE_DIR / "liboracle_scan.so"

_lib: Optional[ctypes.CDLL] = None


def build(force: bool = False) -> Path:
    """Compile scan_oracle.c with gcc (seconds)."""
    if force and LIB_PATH.exists():
        LIB_PATH.unlink()
    subprocess.run(["make", "-C", os.fspath(ORACLE_DIR), "liboracle_scan.so"], check=True, capture_output=True)
    return LIB_PATH


def _load() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not LIB_PATH.exists():
            build()
        lib = ctypes.CDLL(os.fspath(LIB_PATH))
        fp = ctypes.POINTER(ctypes.c_float)
        dp = ctypes.POINTER(ctypes.c_double)
        i = ctypes.c_int
        lib.oracle_scan_forward_f64.argtypes = [fp, fp, fp, fp, dp, dp, i, i, i]
        lib.oracle_scan_backward_f64.argtypes = [fp, fp, fp, fp, fp, dp, dp, dp, dp, i, i, i]
        lib.oracle_scan_forward_carry_f64.argtypes = [fp, fp, fp, fp, fp, dp, dp, dp, i, i, i]
        lib.oracle_scan_backward_carry_f64.argtypes = [fp] * 7 + [dp] * 5 + [i, i, i]
        lib.oracle_scan_forward_f32_seq.argtypes = [fp, fp, fp, fp, i, i, i]
        lib.oracle_scan_backward_f32_seq.argtypes = [fp] * 6 + [fp] * 4 + [i, i, i]
        for fn in (lib.oracle_scan_forward_f64, lib.oracle_scan_backward_f64,
                   lib.oracle_scan_forward_carry_f64, lib.oracle_scan_backward_carry_f64,
                   lib.oracle_scan_forward_f32_seq, lib.oracle_scan_backward_f32_seq):
            fn.restype = None
        _lib = lib
    return _lib


def _f32(t) -> np.ndarray:
    """Any tensor/array -> contiguous float32 numpy array holding exactly the stored values."""
    if hasattr(t, "detach"):
        t = t.detach().to("cpu").float().numpy()
    return np.ascontiguousarray(t, dtype=np.float32)


def _fp(arr: np.ndarray):
    return arr.ctypes.data_as(ctypes.POINTER(ctypes.c_float))


def _dp(arr: Optional[np.ndarray]):
    if arr is None:
        return ctypes.POINTER(ctypes.c_double)()
    return arr.ctypes.data_as(ctypes.POINTER(ctypes.c_double))


def forward_f64(x, a, b, c=None) -> Tuple[np.ndarray, np.ndarray]:
    """(h, y) in float64 from the stored values of x, a, b, c (c=None means c = 1)."""
    x, a, b = _f32(x), _f32(a), _f32(b)
    cc = _f32(c) if c is not None else None
    B, L, D = x.shape
    h = np.empty((B, L, D), dtype=np.float64)
    y = np.empty((B, L, D), dtype=np.float64)
    _load().oracle_scan_forward_f64(_fp(x), _fp(a), _fp(b), _fp(cc) if cc is not None else None,
                                    _dp(h), _dp(y), B, L, D)
    return h, y


def backward_f64(x, a, b, c, dy) -> Tuple[np.ndarray, np.ndarray, np.ndarray, np.ndarray]:
    """(dx, da, db, dc) in float64 for the loss sum(y * dy)."""
    x, a, b, c, dy = (_f32(t) for t in (x, a, b, c, dy))
    B, L, D = x.shape
    outs = [np.empty((B, L, D), dtype=np.float64) for _ in range(4)]
    _load().oracle_scan_backward_f64(_fp(x), _fp(a), _fp(b), _fp(c), _fp(dy), *[_dp(o) for o in outs], B, L, D)
    return tuple(outs)


def forward_carry_f64(x, a, b, c, h0=None) -> Tuple[np.ndarray, np.ndarray, np.ndarray]:
    """(h, y, h_final) in float64, the recurrence started from h(-1) = h0 ([B, D], None = zero)."""
    x, a, b, c = (_f32(t) for t in (x, a, b, c))
    B, L, D = x.shape
    h0f = _f32(h0) if h0 is not None else None
    h = np.empty((B, L, D), dtype=np.float64)
    y = np.empty((B, L, D), dtype=np.float64)
    hf = np.empty((B, D), dtype=np.float64)
    _load().oracle_scan_forward_carry_f64(_fp(x), _fp(a), _fp(b), _fp(c), _fp(h0f) if h0f is not None else None,
                                          _dp(h), _dp(y), _dp(hf), B, L, D)
    return h, y, hf


def backward_carry_f64(x, a, b, c, dy, h0=None, g_final=None):
    """(dx, da, db, dc, dh0) in float64 for the loss sum(y * dy) + sum(h_final * g_final)."""
    x, a, b, c, dy = (_f32(t) for t in (x, a, b, c, dy))
    B, L, D = x.shape
    h0f = _f32(h0) if h0 is not None else None
    gf = _f32(g_final) if g_final is not None else None
    outs = [np.empty((B, L, D), dtype=np.float64) for _ in range(4)]
    dh0 = np.empty((B, D), dtype=np.float64)
    _load().oracle_scan_backward_carry_f64(
        _fp(x), _fp(a), _fp(b), _fp(c), _fp(dy), _fp(h0f) if h0f is not None else None,
        _fp(gf) if gf is not None else None, *[_dp(o) for o in outs], _dp(dh0), B, L, D)
    return tuple(outs) + (dh0,)


def forward_f32_seq(x, a, b) -> np.ndarray:
    """h in float32, computed with the reference's operation order (mul, mul, add per step)."""
    x, a, b = _f32(x), _f32(a), _f32(b)
    B, L, D = x.shape
    h = np.empty((B, L, D), dtype=np.float32)
    _load().oracle_scan_forward_f32_seq(_fp(x), _fp(a), _fp(b), _fp(h), B, L, D)
    return h


def backward_f32_seq(x, a, b, c, dy, h) -> Tuple[np.ndarray, np.ndarray, np.ndarray, np.ndarray]:
    """(dx, da, db, dc) in float32 with the reference's operation order, given the forward h."""
    x, a, b, c, dy, h = (_f32(t) for t in (x, a, b, c, dy, h))
    B, L, D = x.shape
    outs = [np.empty((B, L, D), dtype=np.float32) for _ in range(4)]
    _load().oracle_scan_backward_f32_seq(_fp(x), _fp(a), _fp(b), _fp(c), _fp(dy), _fp(h),
                                         *[_fp(o) for o in outs], B, L, D)
    return tuple(outs)


def error_report(got, ref, floor_frac: float = 1e-3) -> dict:
    """Per-tensor error figures against a float64 reference.

    scaled  = max|got - ref| / max|ref|
    rel     = max over elements of |got - ref| / max(|ref|, floor), floor = floor_frac * max|ref|
    """
    if hasattr(got, "detach"):
        got = got.detach().to("cpu").double().numpy()
    got = np.asarray(got, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    if ref.size == 0:
        return {"scaled": 0.0, "rel": 0.0, "max_abs": 0.0, "ref_max": 0.0}
    diff = np.abs(got - ref)
    ref_max = float(np.max(np.abs(ref)))
    floor = max(floor_frac * ref_max, 1e-300)
    return {
        "scaled": float(diff.max() / max(ref_max, 1e-300)),
        "rel": float(np.max(diff / np.maximum(np.abs(ref), floor))),
        "max_abs": float(diff.max()),
        "ref_max": ref_max,
    }
