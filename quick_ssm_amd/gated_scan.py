"""The scan with the layer's gate activations inside it: projection outputs in, y out, one launch each way.

    a = sigmoid(A_pre)   x = B_in   b = sigmoid(D_pre)   c = silu(Ca) * Cb
    h(t) = a(t) h(t-1) + b(t) x(t),   y(t) = c(t) h(t)

The reference's layer forms a, x, b, c with separate torch ops, casts them to its compute dtype and hands them to
`scan` (quick_ssm/layers.py:76-104); autograd then walks the same chain back.  Here `qssm_scan_gated_forward` /
`qssm_scan_gated_backward` read the five projection outputs themselves and return y / the projections' gradients:
the operands and their gradients never exist in HBM.  Values are rounded where the layer rounds them (gate outputs
to the compute dtype, the scan's gradients to the compute dtype), so the result is that of `gate_prologue` followed
by `scan`, to the last rounding of the activations' derivatives.

Built for 16-bit projections whose storage type is the compute dtype, and for fp32 projections with any compute
dtype and fp32 y (the reference's default layer: fp32 parameters, fp16 compute; the 16-bit operands then exist in
registers only); checkpoint=True, S >= 128 and a multiple of 4, rows 16-byte aligned.  `supported()` says whether a
call qualifies, and the layer takes the two-pass route (quick_ssm_amd/gates.py + scan) otherwise.
"""
from __future__ import annotations

import ctypes
from typing import Optional, Sequence, Tuple

import torch

from . import _lib, hip_scan
from ._lib import Plan, Strides
from .gates import gate_prologue, gate_prologue_wide

Tensor = torch.Tensor

_CODES = {torch.float32: _lib.QSSM_F32, torch.float16: _lib.QSSM_F16, torch.bfloat16: _lib.QSSM_BF16}
_plans: dict = {}


def supported(pre: Sequence[Tensor], compute_dtype: torch.dtype, out_dtype: torch.dtype, checkpoint: bool = True) -> bool:
    """Whether the five projection outputs can take the gated launches."""
    t0 = pre[0]
    if t0.device.type != "cuda" or t0.dim() != 3 or not checkpoint:
        return False
    if t0.dtype in (torch.float16, torch.bfloat16):
        if compute_dtype != t0.dtype or out_dtype not in (t0.dtype, torch.float32):
            return False
    elif t0.dtype == torch.float32:
        if compute_dtype not in _CODES or out_dtype != torch.float32:
            return False
    else:
        return False
    B, L, S = t0.shape
    if B == 0 or L == 0 or S < 128 or S % 4 != 0:
        return False
    es = t0.element_size()
    for t in pre:
        if t.shape != t0.shape or t.dtype != t0.dtype or t.device != t0.device or t.stride(2) != 1:
            return False
        if t.data_ptr() % 16 or (t.stride(0) * es) % 16 or (t.stride(1) * es) % 16:
            return False
    return True


def _plan(B: int, L: int, S: int, dtype: torch.dtype, compute_dtype: torch.dtype, out_dtype: torch.dtype,
          direction: int, ckpt_stride: int) -> Plan:
    key = (B, L, S, dtype, compute_dtype, out_dtype, direction, ckpt_stride)
    plan = _plans.get(key)
    if plan is None:
        plan = Plan()
        _lib.check(_lib.load().qssm_plan_scan_gated(B, L, S, _CODES[dtype], _CODES[compute_dtype], _CODES[out_dtype],
                                                    direction, 8, ckpt_stride, ctypes.byref(plan)))
        if len(_plans) >= 1024:
            _plans.clear()
        _plans[key] = plan
    return plan


def _st(t: Tensor) -> Strides:
    return Strides(t.stride(0), t.stride(1))


def _launch(plan: Plan, dev: torch.device, fn, *args) -> None:
    with torch.cuda.device(dev):
        stream = hip_scan._raw_stream(dev.index)
        buf, epoch, capturing = hip_scan._launch_buffers(dev, dev.index, stream, int(plan.control_bytes),
                                                         int(plan.workspace_bytes))
        _lib.check(fn(ctypes.byref(plan), *args, buf.ctl_ptr, buf.ctl_size, buf.ws_ptr, buf.ws_size, epoch, stream))
        hip_scan._after_launch(buf, stream, capturing)


def _forward_launch(pre: Sequence[Tensor], compute_dtype: torch.dtype, out_dtype: torch.dtype, train: bool = True):
    """y, the saved states and their spacing for the five projection outputs.  `train`: a backward will follow, so
    the last tiles of every chain may leave their operands in the caches for it (`hip_scan.set_forward_keep`)."""
    A_pre, B_in, Ca, Cb, D_pre = pre
    B, L, S = A_pre.shape
    dev, dtype = A_pre.device, A_pre.dtype
    # the backward's tile length decides how far apart the saved states are; it takes dy stored as the projections are
    stride = _plan(B, L, S, dtype, compute_dtype, dtype, _lib.QSSM_BACKWARD, 0).seg_len
    plan = _plan(B, L, S, dtype, compute_dtype, out_dtype, _lib.QSSM_FORWARD, stride)
    keep = hip_scan._forward_keep if train else False
    if keep is not True:
        plan = Plan.from_buffer_copy(plan)   # cached plans are shared: change a copy
        plan.keep_tiles = 0 if keep is False else min(int(plan.keep_tiles), int(keep))
    y = torch.empty((B, L, S), dtype=out_dtype, device=dev)
    ckpt = torch.empty((B, plan.n_ckpt, S), dtype=torch.float32, device=dev)
    _launch(plan, dev, _lib.load().qssm_scan_gated_forward,
            A_pre.data_ptr(), _st(A_pre), B_in.data_ptr(), _st(B_in), Ca.data_ptr(), _st(Ca), Cb.data_ptr(), _st(Cb),
            D_pre.data_ptr(), _st(D_pre), y.data_ptr(), _st(y), ckpt.data_ptr())
    return y, ckpt, int(plan.ckpt_stride)


def _fits_fused_backward(grad_y: Tensor, dtype: torch.dtype) -> bool:
    es = grad_y.element_size()
    return not (grad_y.dtype != dtype or grad_y.stride(2) != 1 or grad_y.data_ptr() % 16 or (grad_y.stride(0) * es) % 16
                or (grad_y.stride(1) * es) % 16)


def _backward_launch(pre: Sequence[Tensor], compute_dtype: torch.dtype, grad_y: Tensor, ckpt: Tensor, stride: int,
                     grads: Sequence[Tensor]) -> None:
    """The five projection gradients, written into `grads` (any batch and time strides)."""
    A_pre, B_in, Ca, Cb, D_pre = pre
    dA, dB, dCa, dCb, dD = grads
    B, L, S = A_pre.shape
    dtype = A_pre.dtype
    plan = _plan(B, L, S, dtype, compute_dtype, dtype, _lib.QSSM_BACKWARD, stride)
    _launch(plan, A_pre.device, _lib.load().qssm_scan_gated_backward,
            A_pre.data_ptr(), _st(A_pre), B_in.data_ptr(), _st(B_in), Ca.data_ptr(), _st(Ca), Cb.data_ptr(), _st(Cb),
            D_pre.data_ptr(), _st(D_pre), grad_y.data_ptr(), _st(grad_y), ckpt.data_ptr(),
            dA.data_ptr(), _st(dA), dB.data_ptr(), _st(dB), dCa.data_ptr(), _st(dCa), dCb.data_ptr(), _st(dCb),
            dD.data_ptr(), _st(dD))


class _GatedScanFunction(torch.autograd.Function):
    """(A_pre, B_in, Ca, Cb, D_pre) -> y, one HIP launch forward, one backward."""

    @staticmethod
    def forward(ctx, A_pre: Tensor, B_in: Tensor, Ca: Tensor, Cb: Tensor, D_pre: Tensor, out_dtype: torch.dtype,
                compute_dtype: torch.dtype) -> Tensor:
        y, ckpt, stride = _forward_launch((A_pre, B_in, Ca, Cb, D_pre), compute_dtype, out_dtype,
                                          any(ctx.needs_input_grad[:5]))
        ctx.save_for_backward(A_pre, B_in, Ca, Cb, D_pre, ckpt)
        ctx.stride, ctx.out_dtype, ctx.compute_dtype = stride, out_dtype, compute_dtype
        return y

    @staticmethod
    def backward(ctx, grad_y: Tensor):
        *pre, ckpt = ctx.saved_tensors
        B, L, S = pre[0].shape
        dev, dtype = pre[0].device, pre[0].dtype
        if not _fits_fused_backward(grad_y, dtype):
            if ctx.out_dtype == dtype:
                grad_y = grad_y.to(dtype).contiguous()
            else:
                return _two_pass_backward(ctx, grad_y)
        grads = [torch.empty((B, L, S), dtype=dtype, device=dev) for _ in range(5)]
        _backward_launch(pre, ctx.compute_dtype, grad_y, ckpt, ctx.stride, grads)
        return (*grads, None, None)


def _blocks(wide: Tensor) -> Tuple[Tensor, ...]:
    S = wide.shape[-1] // 5
    return tuple(wide[..., k * S:(k + 1) * S] for k in range(5))


class _GatedScanWide(torch.autograd.Function):
    """The same on one wide [B, L, 5 S] tensor whose column blocks are the five projection outputs (one GEMM over the
    stacked weights): the gradients are written into the blocks of one wide gradient."""

    @staticmethod
    def forward(ctx, wide: Tensor, out_dtype: torch.dtype, compute_dtype: torch.dtype) -> Tensor:
        y, ckpt, stride = _forward_launch(_blocks(wide), compute_dtype, out_dtype, ctx.needs_input_grad[0])
        ctx.save_for_backward(wide, ckpt)
        ctx.stride, ctx.out_dtype, ctx.compute_dtype = stride, out_dtype, compute_dtype
        return y

    @staticmethod
    def backward(ctx, grad_y: Tensor):
        wide, ckpt = ctx.saved_tensors
        dtype = wide.dtype
        if not _fits_fused_backward(grad_y, dtype):
            if ctx.out_dtype == dtype:
                grad_y = grad_y.to(dtype).contiguous()
            else:
                with torch.enable_grad():
                    leaf = wide.detach().requires_grad_(True)
                    a, x, c, b = gate_prologue_wide(leaf, ctx.compute_dtype)
                k_in, k_out = hip_scan.kernel_dtypes([x.dtype], ctx.out_dtype)
                dy = grad_y if grad_y.dtype == k_out else grad_y.to(k_out)
                dx, da, db, dc = hip_scan.scan_backward(x.detach(), a.detach(), b.detach(), c.detach(), dy, ckpt=ckpt,
                                                        ckpt_stride=ctx.stride)
                (dwide,) = torch.autograd.grad((a, x, c, b), (leaf,), (da, dx, dc, db))
                return dwide, None, None
        dwide = torch.empty_like(wide, memory_format=torch.contiguous_format)
        _backward_launch(_blocks(wide), ctx.compute_dtype, grad_y, ckpt, ctx.stride, _blocks(dwide))
        return dwide, None, None


def _two_pass_backward(ctx, grad_y: Tensor):
    """The backward for a y that is not stored as the projections are (fp32 y from 16-bit projections): the gate
    prologue again, the plain backward scan on its operands with the states the gated forward saved, and the
    prologue's own backward."""
    A_pre, B_in, Ca, Cb, D_pre, ckpt = ctx.saved_tensors
    with torch.enable_grad():
        leaves = [t.detach().requires_grad_(True) for t in (A_pre, B_in, Ca, Cb, D_pre)]
        a, x, c, b = gate_prologue(*leaves, ctx.compute_dtype)
    k_in, k_out = hip_scan.kernel_dtypes([x.dtype], ctx.out_dtype)
    dy = grad_y if grad_y.dtype == k_out else grad_y.to(k_out)
    dx, da, db, dc = hip_scan.scan_backward(x.detach(), a.detach(), b.detach(), c.detach(), dy, ckpt=ckpt,
                                            ckpt_stride=ctx.stride)
    grads = torch.autograd.grad((a, x, c, b), leaves, (da, dx, dc, db))
    return tuple(grads) + (None, None)


def gated_scan(A_pre: Tensor, B_in: Tensor, Ca: Tensor, Cb: Tensor, D_pre: Tensor, *,
               out_dtype: Optional[torch.dtype] = None, compute_dtype: Optional[torch.dtype] = None) -> Tensor:
    """y of the scan whose operands are sigmoid(A_pre), B_in, sigmoid(D_pre), silu(Ca) * Cb (all [B, L, S]), each
    rounded to `compute_dtype` (default: the projections' own dtype) as the layer's casts round them.

    Call `supported()` first; tensors that do not qualify raise from the library."""
    return _GatedScanFunction.apply(A_pre, B_in, Ca, Cb, D_pre, out_dtype or A_pre.dtype, compute_dtype or A_pre.dtype)


def gated_scan_wide(wide: Tensor, *, out_dtype: Optional[torch.dtype] = None,
                    compute_dtype: Optional[torch.dtype] = None) -> Tensor:
    """`gated_scan` on one [B, L, 5 S] tensor holding A_pre, B_in, Ca, Cb, D_pre side by side; call `supported()` on
    its five blocks first."""
    return _GatedScanWide.apply(wide, out_dtype or wide.dtype, compute_dtype or wide.dtype)


__all__ = ["gated_scan", "gated_scan_wide", "supported"]
