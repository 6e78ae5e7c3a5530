"""Torch restatement of the reference's CPU execution path -- TEST INFRASTRUCTURE.

Follows, loop for loop, what `scan(..., backend="torch")` runs in the reference:
quick_ssm/scan_interface.py:161-166 (`_torch_scan`: h = naive_forward_3d(x, a, b); y = c * h;
cast to out_dtype) on top of quick_ssm/naive_baseline.py:28-40 (per batch row, per time step,
one D-vector update written into a preallocated h; 16-bit inputs accumulate in fp32 and h is
rounded back to x.dtype).  Gradients come from torch autograd through those steps, as in the
reference.  It is deliberately as slow as the original: bench.py times it for `cpu_baseline`.
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch

Tensor = torch.Tensor


def reference_forward_states(x: Tensor, a: Tensor, b: Tensor) -> Tensor:
    rows, steps, width = x.shape
    wide = x.dtype in (torch.float16, torch.bfloat16)
    work = torch.float32 if wide else x.dtype
    xw, aw, bw = x.to(work), a.to(work), b.to(work)
    out = torch.zeros((rows, steps, width), dtype=work, device=x.device)
    for r in range(rows):
        carry = torch.zeros(width, dtype=work, device=x.device)
        for t in range(steps):
            carry = aw[r, t] * carry + bw[r, t] * xw[r, t]
            out[r, t] = carry
    return out.to(x.dtype)


def reference_scan(x: Tensor, a: Tensor, b: Tensor, c: Tensor, out_dtype: Optional[torch.dtype] = None) -> Tensor:
    states = reference_forward_states(x, a, b)
    return (c * states).to(out_dtype or x.dtype)


def reference_scan_with_grads(x: Tensor, a: Tensor, b: Tensor, c: Tensor, dy: Tensor,
                              out_dtype: Optional[torch.dtype] = None
                              ) -> Tuple[Tensor, Tensor, Tensor, Tensor, Tensor]:
    """y and the four gradients of sum(y * dy), through autograd, as the reference's tests do."""
    leaves = [t.detach().clone().requires_grad_(True) for t in (x, a, b, c)]
    y = reference_scan(*leaves, out_dtype=out_dtype)
    (y * dy).sum().backward()
    return (y.detach(),) + tuple(t.grad for t in leaves)
