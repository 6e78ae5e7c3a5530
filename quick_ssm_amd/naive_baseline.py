"""Sequential (one time step after another) scan in plain torch.

This is the path `scan(..., backend="torch")` runs and the one CPU tensors take.  It keeps the
reference's rounding points (quick_ssm/naive_baseline.py:28-40): 16-bit inputs are accumulated
in fp32, h is rounded to x.dtype once at the end, and callers multiply c * h in the input
dtype.  Unlike the reference's loop it advances all batch rows together and gathers the steps
with one `stack`, so autograd through it costs O(L) instead of one whole-tensor copy per step;
every element still sees the same operations in the same order.
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch

Tensor = torch.Tensor

_HALF = (torch.float16, torch.bfloat16)


def naive_forward_3d(x: Tensor, a: Tensor, b: Tensor, h_init: Optional[Tensor] = None,
                     return_final: bool = False):
    """h(t) = a(t) * h(t-1) + b(t) * x(t) for [B, L, D] tensors; returns h in x.dtype.

    h(-1) is zero, as in the reference, unless `h_init` ([B, D]) is given.  With `return_final` the
    state after the last step comes back too, in the accumulation dtype: (h, h_final).
    """
    B, L, D = x.shape
    acc = torch.float32 if x.dtype in _HALF else x.dtype
    xs, as_, bs = x.to(acc), a.to(acc), b.to(acc)
    if h_init is None:
        state = torch.zeros((B, D), device=x.device, dtype=acc)
    else:
        state = h_init.to(acc)
    steps = []
    for t in range(L):
        state = as_[:, t] * state + bs[:, t] * xs[:, t]
        steps.append(state)
    h = torch.stack(steps, dim=1).to(x.dtype) if L > 0 else torch.zeros((B, L, D), device=x.device, dtype=x.dtype)
    return (h, state) if return_final else h


def naive_full_3d(x: Tensor, a: Tensor, b: Tensor, c: Tensor) -> Tuple[Tensor, Tensor]:
    """Returns (h, y) with y = c * h (reference: quick_ssm/naive_baseline.py:43-64)."""
    h = naive_forward_3d(x, a, b)
    return h, c * h


def naive_backward_3d(x: Tensor, a: Tensor, b: Tensor, c: Tensor, grad_y: Tensor
                      ) -> Tuple[Tensor, Tensor, Tensor, Tensor]:
    """Analytic gradients of sum(y * grad_y): the reverse recurrence, one step at a time.

        dH(t) = c(t) grad_y(t) + a(t+1) dH(t+1);  dx = b dH, db = x dH, da(t) = h(t-1) dH(t), dc = grad_y h

    Follows quick_ssm/naive_baseline.py:67-137 (all arithmetic in the input dtype).
    """
    B, L, D = x.shape
    h = naive_forward_3d(x, a, b)
    dx, da, db, dc = (torch.zeros_like(t) for t in (x, a, b, c))
    flow = torch.zeros((B, D), device=x.device, dtype=x.dtype)  # a(t+1) * dH(t+1)
    zero = torch.zeros((B, D), device=x.device, dtype=x.dtype)
    for t in range(L - 1, -1, -1):
        dH = grad_y[:, t] * c[:, t] + flow
        dc[:, t] = grad_y[:, t] * h[:, t]
        db[:, t] = dH * x[:, t]
        da[:, t] = dH * (h[:, t - 1] if t > 0 else zero)
        dx[:, t] = dH * b[:, t]
        flow = dH * a[:, t]
    return dx, da, db, dc
