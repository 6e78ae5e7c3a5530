"""Gate prologue of the SSM layer: the five projection outputs become the scan's operands.

    a = sigmoid(A_pre)    x = B_in    c = silu(Ca) * Cb    b = sigmoid(D_pre)

The reference does this with separate torch ops (quick_ssm/layers.py:76-88): two sigmoids, a silu,
a product and four casts, each a pass over a [B, L, state] tensor, and autograd keeps their
intermediates.  Here GPU tensors take one HIP pass forward (`qssm_gates_forward`) and one backward
(`qssm_gates_backward`); only the projection outputs are saved.  Arithmetic is fp32 whatever the
storage, each result rounded once.  CPU tensors, and storage pairs the library is not built for,
take the same formulas as torch ops.
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch
import torch.nn.functional as F

from . import _lib

Tensor = torch.Tensor

_CODES = {torch.float32: _lib.QSSM_F32, torch.float16: _lib.QSSM_F16, torch.bfloat16: _lib.QSSM_BF16}
_BUILT = {
    (torch.float32, torch.float32), (torch.float32, torch.float16), (torch.float32, torch.bfloat16),
    (torch.float16, torch.float16), (torch.float16, torch.float32),
    (torch.bfloat16, torch.bfloat16), (torch.bfloat16, torch.float32),
}


def _rows(t: Tensor, S: int) -> Tensor:
    """[.., S] -> [rows, S] with unit column stride (a view whenever the layout allows)."""
    t2 = t.reshape(-1, S)
    return t2 if t2.stride(1) == 1 or t2.shape[0] == 0 else t2.contiguous()


def gates_reference(A_pre: Tensor, B_in: Tensor, Ca: Tensor, Cb: Tensor, D_pre: Tensor, compute_dtype: torch.dtype
                    ) -> Tuple[Tensor, Tensor, Tensor, Tensor]:
    """The same four operands as separate torch ops, in the reference's order of operations."""
    a = torch.sigmoid(A_pre).to(compute_dtype)
    x = B_in.to(compute_dtype)
    c = (F.silu(Ca) * Cb).to(compute_dtype)
    b = torch.sigmoid(D_pre).to(compute_dtype)
    return a, x, c, b


class _GatePrologue(torch.autograd.Function):
    @staticmethod
    def forward(ctx, A_pre: Tensor, B_in: Tensor, Ca: Tensor, Cb: Tensor, D_pre: Tensor, compute_dtype: torch.dtype):
        shape = A_pre.shape
        S = shape[-1]
        ins = [_rows(t, S) for t in (A_pre, B_in, Ca, Cb, D_pre)]
        rows = ins[0].shape[0]
        outs = [torch.empty((rows, S), dtype=compute_dtype, device=A_pre.device) for _ in range(4)]
        with _lib.launch_stream(A_pre.device) as stream:
            args = []
            for t in ins:
                args += [t.data_ptr(), t.stride(0) if rows > 1 else S]
            _lib.check(_lib.load().qssm_gates_forward(
                *args, *[o.data_ptr() for o in outs], rows, S, _CODES[A_pre.dtype], _CODES[compute_dtype], stream))
        ctx.save_for_backward(ins[0], ins[2], ins[3], ins[4])
        ctx.shape, ctx.in_dtype, ctx.out_dtype = shape, A_pre.dtype, compute_dtype
        return tuple(o.view(shape) for o in outs)

    @staticmethod
    def backward(ctx, g_a: Optional[Tensor], g_x: Optional[Tensor], g_c: Optional[Tensor], g_b: Optional[Tensor]):
        A_pre, Ca, Cb, D_pre = ctx.saved_tensors
        rows, S = A_pre.shape
        dev = A_pre.device

        def dense(g: Optional[Tensor]) -> Tensor:
            if g is None:
                return torch.zeros((rows, S), dtype=ctx.out_dtype, device=dev)
            g = g.reshape(rows, S)
            return g if g.is_contiguous() and g.dtype == ctx.out_dtype else g.to(ctx.out_dtype).contiguous()

        gs = [dense(g) for g in (g_a, g_x, g_c, g_b)]
        outs = [torch.empty((rows, S), dtype=ctx.in_dtype, device=dev) for _ in range(5)]
        with _lib.launch_stream(dev) as stream:
            args = [g.data_ptr() for g in gs]
            for t in (A_pre, Ca, Cb, D_pre):
                args += [t.data_ptr(), t.stride(0) if rows > 1 else S]
            _lib.check(_lib.load().qssm_gates_backward(
                *args, *[o.data_ptr() for o in outs], rows, S, _CODES[ctx.in_dtype], _CODES[ctx.out_dtype], stream))
        return tuple(o.view(ctx.shape) for o in outs) + (None,)


class _GatePrologueWide(torch.autograd.Function):
    """The prologue on one wide [.., 5 S] tensor whose column blocks are A_pre, B_in, Ca, Cb, D_pre (the output of a
    single GEMM over the five stacked projection weights): the kernels read the blocks in place and the backward
    writes the five gradients into the blocks of one wide gradient, which is what that GEMM's backward wants."""

    @staticmethod
    def forward(ctx, wide: Tensor, compute_dtype: torch.dtype):
        S = wide.shape[-1] // 5
        w2 = _rows(wide, 5 * S)
        rows = w2.shape[0]
        ld = w2.stride(0) if rows > 1 else 5 * S
        es = w2.element_size()
        outs = [torch.empty((rows, S), dtype=compute_dtype, device=wide.device) for _ in range(4)]
        with _lib.launch_stream(wide.device) as stream:
            args = []
            for k in range(5):
                args += [w2.data_ptr() + k * S * es, ld]
            _lib.check(_lib.load().qssm_gates_forward(
                *args, *[o.data_ptr() for o in outs], rows, S, _CODES[wide.dtype], _CODES[compute_dtype], stream))
        ctx.save_for_backward(w2)
        ctx.shape, ctx.out_dtype = wide.shape, compute_dtype
        lead = wide.shape[:-1]
        return tuple(o.view(*lead, S) for o in outs)

    @staticmethod
    def backward(ctx, g_a: Optional[Tensor], g_x: Optional[Tensor], g_c: Optional[Tensor], g_b: Optional[Tensor]):
        (w2,) = ctx.saved_tensors
        rows, S = w2.shape[0], w2.shape[1] // 5
        dev, es = w2.device, w2.element_size()
        ld = w2.stride(0) if rows > 1 else 5 * S

        def dense(g: Optional[Tensor]) -> Tensor:
            if g is None:
                return torch.zeros((rows, S), dtype=ctx.out_dtype, device=dev)
            g = g.reshape(rows, S)
            return g if g.is_contiguous() and g.dtype == ctx.out_dtype else g.to(ctx.out_dtype).contiguous()

        gs = [dense(g) for g in (g_a, g_x, g_c, g_b)]
        dwide = torch.empty((rows, 5 * S), dtype=w2.dtype, device=dev)
        with _lib.launch_stream(dev) as stream:
            args = [g.data_ptr() for g in gs]
            for k in (0, 2, 3, 4):                     # A_pre, Ca, Cb, D_pre
                args += [w2.data_ptr() + k * S * es, ld]
            _lib.check(_lib.load().qssm_gates_backward_strided(
                *args, *[dwide.data_ptr() + k * S * es for k in range(5)], 5 * S, rows, S, _CODES[w2.dtype],
                _CODES[ctx.out_dtype], stream))
        return dwide.view(ctx.shape), None


def gate_prologue_wide(wide: Tensor, compute_dtype: torch.dtype) -> Tuple[Tensor, Tensor, Tensor, Tensor]:
    """(a, x, c, b) from one [.., 5 S] tensor holding A_pre, B_in, Ca, Cb, D_pre side by side."""
    if wide.shape[-1] % 5 != 0:
        raise ValueError("the last axis must hold five blocks of equal width")
    S = wide.shape[-1] // 5
    fused = wide.device.type == "cuda" and (wide.dtype, compute_dtype) in _BUILT and wide.numel() > 0
    if fused:
        return _GatePrologueWide.apply(wide, compute_dtype)
    return gates_reference(*(wide[..., k * S:(k + 1) * S] for k in range(5)), compute_dtype)


def gate_prologue(A_pre: Tensor, B_in: Tensor, Ca: Tensor, Cb: Tensor, D_pre: Tensor, compute_dtype: torch.dtype
                  ) -> Tuple[Tensor, Tensor, Tensor, Tensor]:
    """(a, x, c, b) in `compute_dtype` from the five projection outputs (all of one shape and dtype).

    GPU tensors of a storage pair the library is built for take the fused HIP pass; everything else
    takes `gates_reference`.
    """
    tensors = (A_pre, B_in, Ca, Cb, D_pre)
    same = all(t.shape == A_pre.shape and t.dtype == A_pre.dtype and t.device == A_pre.device for t in tensors)
    if not same:
        raise ValueError("the five projection outputs must share shape, dtype and device")
    fused = (A_pre.device.type == "cuda" and (A_pre.dtype, compute_dtype) in _BUILT and A_pre.dim() >= 1
             and A_pre.numel() > 0)
    if fused:
        return _GatePrologue.apply(A_pre, B_in, Ca, Cb, D_pre, compute_dtype)
    return gates_reference(A_pre, B_in, Ca, Cb, D_pre, compute_dtype)


__all__ = ["gate_prologue", "gate_prologue_wide", "gates_reference"]
