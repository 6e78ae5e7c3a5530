"""CPU oracle for the SSM layer's gate prologue -- TEST INFRASTRUCTURE, not part of the product.
Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import this.

Restates in float64 numpy what the reference's SSM.forward does between its projections and the scan
(quick_ssm/layers.py:76-88):

    a = sigmoid(A_proj(u))                      layers.py:76
    b = B_proj(u)            (the scan's x)     layers.py:77
    c = silu(C_proj_a(u)) * C_proj_b(u)         layers.py:79-81
    d = sigmoid(D_proj(u))   (the scan's b)     layers.py:82

and the gradients autograd derives from those lines.  Inputs are the stored values of the projection
outputs (already rounded to their storage type by the caller); every intermediate is float64.

Pinned by tests/test_oracle.py: against torch's own sigmoid / silu and autograd in float64 (library
routines), and by central differences.
"""
from __future__ import annotations

import numpy as np


def _f64(t) -> np.ndarray:
    if hasattr(t, "detach"):
        t = t.detach().to("cpu").double().numpy()
    return np.asarray(t, dtype=np.float64)


def _sigmoid(z: np.ndarray) -> np.ndarray:
    out = np.empty_like(z)
    pos = z >= 0
    out[pos] = 1.0 / (1.0 + np.exp(-z[pos]))
    ez = np.exp(z[~pos])
    out[~pos] = ez / (1.0 + ez)
    return out


def gates_forward_f64(A_pre, B_in, Ca, Cb, D_pre):
    """(a, x, c, b): the scan's forget gate, drive, output gate and input gate."""
    A_pre, B_in, Ca, Cb, D_pre = (_f64(t) for t in (A_pre, B_in, Ca, Cb, D_pre))
    return _sigmoid(A_pre), B_in.copy(), Ca * _sigmoid(Ca) * Cb, _sigmoid(D_pre)


def gates_backward_f64(g_a, g_x, g_c, g_b, A_pre, Ca, Cb, D_pre):
    """(dA_pre, dB_in, dCa, dCb, dD_pre) for the loss sum(a g_a + x g_x + c g_c + b g_b)."""
    g_a, g_x, g_c, g_b, A_pre, Ca, Cb, D_pre = (_f64(t) for t in (g_a, g_x, g_c, g_b, A_pre, Ca, Cb, D_pre))
    a, s, b = _sigmoid(A_pre), _sigmoid(Ca), _sigmoid(D_pre)
    return (g_a * a * (1.0 - a), g_x.copy(), g_c * Cb * s * (1.0 + Ca * (1.0 - s)), g_c * Ca * s,
            g_b * b * (1.0 - b))
