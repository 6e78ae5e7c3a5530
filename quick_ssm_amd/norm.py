"""RMSNorm of the SSM layer: y = x * weight / sqrt(mean(x^2) + eps) over the last axis.

The reference writes it as torch ops (quick_ssm/layers.py:14-17): pow, mean, add, sqrt, divide and
multiply, each a pass over [.., H], with their intermediates kept for autograd.  Here GPU tensors take
one HIP pass forward (`qssm_rmsnorm_forward`: x read once, y written once, one fp32 per row saved) and
one backward (`qssm_rmsnorm_backward`: dy and x read once, dx written once, dweight summed in a fixed
order).  Arithmetic is fp32 whatever the storage, each result rounded once.  CPU tensors, and inputs
whose storage type differs from the weight's, take the same formula as torch ops.
"""
from __future__ import annotations

import torch

from . import _lib

Tensor = torch.Tensor

_CODES = {torch.float32: _lib.QSSM_F32, torch.float16: _lib.QSSM_F16, torch.bfloat16: _lib.QSSM_BF16}
PARTIAL_ROWS = 512  # rows of fp32 scratch the backward may spread dweight over (one per workgroup)


def _rows(t: Tensor, H: int) -> Tensor:
    """[.., H] -> [rows, H] with unit column stride (a view whenever the layout allows)."""
    t2 = t.reshape(-1, H)
    return t2 if t2.stride(1) == 1 or t2.shape[0] == 0 else t2.contiguous()


def _ld(t2: Tensor, H: int) -> int:
    return t2.stride(0) if t2.shape[0] > 1 else H


def rms_norm_reference(x: Tensor, weight: Tensor, eps: float) -> Tensor:
    """The reference's own order of operations (quick_ssm/layers.py:15-17)."""
    rms = torch.sqrt(x.pow(2).mean(dim=-1, keepdim=True) + eps)
    return x * (weight / rms)


class _RmsNorm(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x: Tensor, weight: Tensor, eps: float):
        H = x.shape[-1]
        x2 = _rows(x, H)
        rows = x2.shape[0]
        w = weight.contiguous()
        y = torch.empty((rows, H), dtype=x.dtype, device=x.device)
        rstd = torch.empty((rows,), dtype=torch.float32, device=x.device)
        with _lib.launch_stream(x.device) as stream:
            _lib.check(_lib.load().qssm_rmsnorm_forward(
                x2.data_ptr(), _ld(x2, H), w.data_ptr(), y.data_ptr(), rstd.data_ptr(), rows, H, float(eps),
                _CODES[x.dtype], stream))
        ctx.save_for_backward(x2, w, rstd)
        ctx.shape, ctx.eps = x.shape, float(eps)
        return y.view(x.shape)

    @staticmethod
    def backward(ctx, dy: Tensor):
        x2, w, rstd = ctx.saved_tensors
        rows, H = x2.shape
        dev = x2.device
        g = dy.reshape(rows, H)
        if g.dtype != x2.dtype:
            g = g.to(x2.dtype)
        if rows > 0 and g.stride(1) != 1:
            g = g.contiguous()
        dx = torch.empty((rows, H), dtype=x2.dtype, device=dev)
        dw = torch.empty((H,), dtype=w.dtype, device=dev)
        n_part = max(_lib.QSSM_RMSNORM_MIN_PARTIAL_ROWS, min(PARTIAL_ROWS, (rows + 7) // 8))
        partial = torch.empty((n_part, H), dtype=torch.float32, device=dev)
        with _lib.launch_stream(dev) as stream:
            _lib.check(_lib.load().qssm_rmsnorm_backward(
                g.data_ptr(), _ld(g, H), x2.data_ptr(), _ld(x2, H), w.data_ptr(), rstd.data_ptr(), dx.data_ptr(),
                dw.data_ptr(), partial.data_ptr(), n_part, rows, H, ctx.eps, _CODES[x2.dtype], stream))
        return dx.view(ctx.shape), dw, None


def rms_norm(x: Tensor, weight: Tensor, eps: float = 1e-5) -> Tensor:
    """RMSNorm over the last axis of x with a [H] weight.

    GPU tensors whose storage type is the weight's (f32, f16 or bf16) take the fused HIP passes;
    everything else takes `rms_norm_reference`.
    """
    if weight.dim() != 1 or x.dim() < 1 or x.shape[-1] != weight.shape[0]:
        raise ValueError(f"weight {tuple(weight.shape)} does not match the last axis of x {tuple(x.shape)}")
    fused = (x.device.type == "cuda" and weight.device == x.device and x.dtype == weight.dtype
             and x.dtype in _CODES and x.numel() > 0)
    if fused:
        return _RmsNorm.apply(x, weight, eps)
    return rms_norm_reference(x, weight, eps)


__all__ = ["rms_norm", "rms_norm_reference"]
