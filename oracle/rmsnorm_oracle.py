"""CPU oracle for the SSM layer's RMSNorm -- TEST INFRASTRUCTURE, not part of the product.
Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import this.

Restates in float64 numpy what the reference's RMSNorm.forward computes (quick_ssm/layers.py:15-17):

    norm = sqrt(mean(x^2, last axis) + eps)         layers.py:15
    y    = x * (weight / norm)                      layers.py:16

and the gradients autograd derives from those two lines.  Inputs are the stored values (already
rounded to their storage type by the caller); every intermediate is float64.

Pinned by tests/test_oracle.py: against torch.nn.functional.rms_norm and torch autograd in float64
(library routines), by central differences, and by the invariances the formula fixes (y unchanged in
direction under scaling of x when eps = 0; dx orthogonal to x when eps = 0).
"""
from __future__ import annotations

import numpy as np


def _f64(t) -> np.ndarray:
    if hasattr(t, "detach"):
        t = t.detach().to("cpu").double().numpy()
    return np.asarray(t, dtype=np.float64)


def rmsnorm_forward_f64(x, weight, eps: float):
    """y [.., H] for x [.., H], weight [H]."""
    x, w = _f64(x), _f64(weight)
    norm = np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps)
    return x * (w / norm)


def rmsnorm_backward_f64(dy, x, weight, eps: float):
    """(dx [.., H], dweight [H]) for the loss sum(y * dy)."""
    dy, x, w = _f64(dy), _f64(x), _f64(weight)
    H = x.shape[-1]
    r = 1.0 / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps)
    g = dy * w
    s = np.sum(g * x, axis=-1, keepdims=True)
    dx = r * g - x * (r ** 3) * s / H
    dw = np.sum((dy * x * r).reshape(-1, H), axis=0)
    return dx, dw
