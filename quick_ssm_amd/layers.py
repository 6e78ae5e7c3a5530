"""`SSM` and `RMSNorm`: the layer that feeds the scan.

Same constructor arguments, parameter names (so state dicts interchange) and forward keywords as
the reference's quick_ssm/layers.py:9-107.  The projections stay on torch GEMMs; the gate
activations and casts between them and the scan happen inside the scan's own launches when the
projections are stored as the 16-bit compute dtype (quick_ssm_amd/gated_scan.py) and are one fused HIP
pass otherwise (quick_ssm_amd/gates.py),
the pre-norm is one fused HIP pass each way (quick_ssm_amd/norm.py), and the scan is the HIP path.  Roles of the projections
(quick_ssm/test_swiglu_equiv.py:60-70): A_proj -> forget gate a, B_proj -> the scan's input x,
D_proj -> input gate b, C_proj_a/C_proj_b -> SwiGLU output gate c, out_proj -> output.
"""
from __future__ import annotations

from typing import Optional

import torch
import torch.nn as nn

from . import _lib
from . import gated_scan as _gated
from . import scan_interface as _scan_interface
from .gates import gate_prologue, gate_prologue_wide
from .norm import rms_norm
from .scan_interface import scan


class RMSNorm(nn.Module):
    """x * weight / sqrt(mean(x^2) + eps) over the last axis (quick_ssm/layers.py:9-17)."""

    def __init__(self, hidden_size: int, eps: float = 1e-5, dtype=torch.float32, device=None):
        super().__init__()
        self.eps = eps
        self.weight = nn.Parameter(torch.ones(hidden_size, dtype=dtype, device=device))

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return rms_norm(x, self.weight, self.eps)


_CODES = {torch.float32: _lib.QSSM_F32, torch.float16: _lib.QSSM_F16, torch.bfloat16: _lib.QSSM_BF16}
_COLSUM_PARTIAL_ROWS = 64


def column_sum(g2: torch.Tensor) -> torch.Tensor:
    """Sum over the rows of a [rows, S] matrix: the bias gradient of a linear map from its output's gradient.

    GPU matrices with unit column stride (a column block of a wider matrix is fine) take `qssm_colsum`: two small
    launches, a fixed summation order; a library reduction of this shape costs as much as the layer's scan at the
    copy task's size.  Everything else is `g2.sum(0)`."""
    rows, S = g2.shape
    if not (g2.is_cuda and g2.dtype in _CODES and S > 0 and rows > 0 and g2.stride(1) == 1 and g2.stride(0) >= S):
        return g2.sum(0)
    out = torch.empty((S,), dtype=g2.dtype, device=g2.device)
    partial = torch.empty((_COLSUM_PARTIAL_ROWS, S), dtype=torch.float32, device=g2.device)
    with _lib.launch_stream(g2.device) as stream:
        _lib.check(_lib.load().qssm_colsum(g2.data_ptr(), g2.stride(0), rows, S, _CODES[g2.dtype], partial.data_ptr(),
                                           _COLSUM_PARTIAL_ROWS, out.data_ptr(), stream))
    return out


class _LinearBias(torch.autograd.Function):
    """u @ weight^T + bias, as `torch.nn.functional.linear`, with the bias gradient from `column_sum`."""

    @staticmethod
    def forward(ctx, u, weight, bias):
        ctx.save_for_backward(u, weight)
        return torch.nn.functional.linear(u, weight, bias)

    @staticmethod
    def backward(ctx, g):
        u, weight = ctx.saved_tensors
        need = ctx.needs_input_grad
        g2 = g.reshape(-1, g.shape[-1])
        du = (g2 @ weight).view_as(u) if need[0] else None
        dw = g2.t() @ u.reshape(-1, u.shape[-1]) if need[1] else None
        db = column_sum(g2) if need[2] else None
        return du, dw, db


class _PackedProjection(torch.autograd.Function):
    """u -> u @ wide_w^T + wide_b, where wide_w [5 S, H] and wide_b [5 S] are the memory of the five projection
    weights and of A_proj's bias (`SSM._packed_parameters`).  The five weights and the bias are passed as well so
    that autograd routes their gradients: one GEMM gives the gradient of the wide weight, whose row blocks go to the
    five parameters; the bias gradient is summed over A_proj's block only."""

    @staticmethod
    def forward(ctx, u, w_a, w_b, w_ca, w_cb, w_d, bias_a, wide_w, wide_b):
        ctx.save_for_backward(u, wide_w)
        return torch.nn.functional.linear(u, wide_w, wide_b)

    @staticmethod
    def backward(ctx, g):
        u, wide_w = ctx.saved_tensors
        need = ctx.needs_input_grad
        S = wide_w.shape[0] // 5
        g2 = g.reshape(-1, g.shape[-1])
        du = (g2 @ wide_w).view_as(u) if need[0] else None
        blocks = [None] * 5
        if any(need[1:6]):
            dw = g2.t() @ u.reshape(-1, u.shape[-1])                              # [5 S, H]
            blocks = [dw[k * S:(k + 1) * S] if need[1 + k] else None for k in range(5)]
        dbias = column_sum(g2[:, :S]) if need[6] else None
        return (du, *blocks, dbias, None, None)


class SSM(nn.Module):
    """Gated linear recurrence layer: norm -> five projections -> scan -> out projection (+ residual)."""

    def __init__(
        self,
        hidden_size: int,
        state_size_mult: float = 1.0,
        eps: float = 1e-5,
        dtype: torch.dtype = torch.float32,
        device: Optional[torch.device] = None,
        compute_dtype: torch.dtype = torch.float16,
        use_residual: bool = True,
        use_norm: bool = True,
    ):
        super().__init__()
        self.hidden_size = hidden_size
        self.state_size_dim = int(hidden_size * state_size_mult)
        self.compute_dtype = compute_dtype
        self.use_residual = use_residual
        self.use_norm = use_norm

        def proj(n_in: int, n_out: int, bias: bool) -> nn.Linear:
            return nn.Linear(n_in, n_out, bias=bias, device=device, dtype=dtype)

        # Creation order matches the reference so that seeded initialisation matches too.
        self.A_proj = proj(hidden_size, self.state_size_dim, True)
        self.B_proj = proj(hidden_size, self.state_size_dim, False)
        self.C_proj_a = proj(hidden_size, self.state_size_dim, False)
        self.C_proj_b = proj(hidden_size, self.state_size_dim, False)
        self.D_proj = proj(hidden_size, self.state_size_dim, False)
        self.out_proj = proj(self.state_size_dim, hidden_size, True)
        self.pre_norm = RMSNorm(hidden_size, eps=eps, dtype=dtype, device=device) if use_norm else nn.Identity()

    # Below this many elements per projection output a layer's step is bound by launches, not by their work.
    _BATCHED_PROJECTION_LIMIT = 1 << 23

    def _packed_parameters(self):
        """The five projection weights as one [5 S, H] tensor and a [5 S] bias (A_proj's, then zeros) that ARE the
        parameters' memory: each `nn.Linear.weight` is a row block of the wide tensor, `A_proj.bias` the head of the
        wide bias.  Parameter objects, names and values stay what they were (state dicts and optimizers see no
        difference); only where their data lives changes, once.  Whatever gives the parameters storage of their own
        again (`.to()`, `.half()`, loading into fresh tensors) is noticed here by their addresses and packed again."""
        ws = (self.A_proj.weight, self.B_proj.weight, self.C_proj_a.weight, self.C_proj_b.weight, self.D_proj.weight)
        S, H = self.state_size_dim, self.hidden_size
        packed = self.__dict__.get("_packed")
        if packed is not None:
            wide_w, wide_b = packed
            base, step = wide_w.data_ptr(), S * H * wide_w.element_size()
            if (wide_w.dtype == ws[0].dtype and wide_b.dtype == self.A_proj.bias.dtype
                    and all(w.data_ptr() == base + k * step for k, w in enumerate(ws))
                    and self.A_proj.bias.data_ptr() == wide_b.data_ptr()):
                return wide_w, wide_b
        with torch.no_grad():
            wide_w = torch.cat([w.data for w in ws])                              # [5 S, H]
            for k, w in enumerate(ws):
                w.data = wide_w[k * S:(k + 1) * S]
            bias = self.A_proj.bias
            wide_b = torch.cat((bias.data, bias.data.new_zeros(4 * S)))
            bias.data = wide_b[:S]
        self.__dict__["_packed"] = (wide_w, wide_b)
        return wide_w, wide_b

    def _wide_projection(self, u: torch.Tensor) -> Optional[torch.Tensor]:
        """All five projection outputs as one [.., 5 S] tensor (blocks in A, B, C_a, C_b, D order) from a single GEMM
        over the packed weights, for small layers; None for the others.

        The copy task's 12 x hidden 256 stack spends a training step on about a thousand launches of a few
        microseconds each: one GEMM forward and two backward per layer instead of five and ten cut both the host's
        and the GPU's time (the wide tensor's blocks are read in place by the gate kernels, and their gradients are
        written as blocks of one wide gradient).  The weights are not concatenated per call: the five parameters
        live in one tensor (`_packed_parameters`), and the gradient of that tensor is handed back as five row blocks.
        Large layers keep the separate GEMMs: theirs are efficient already."""
        S, H = self.state_size_dim, self.hidden_size
        rows = u.numel() // H
        if not (u.is_cuda and 0 < rows * S <= self._BATCHED_PROJECTION_LIMIT):
            return None
        wide_w, wide_b = self._packed_parameters()
        return _PackedProjection.apply(u, self.A_proj.weight, self.B_proj.weight, self.C_proj_a.weight,
                                       self.C_proj_b.weight, self.D_proj.weight, self.A_proj.bias, wide_w, wide_b)

    def gates(self, u: torch.Tensor):
        """The scan's four operands (x, a, b, c) from the normalised input, in `compute_dtype`."""
        forget, drive, out_gate, in_gate = gate_prologue(
            self.A_proj(u), self.B_proj(u), self.C_proj_a(u), self.C_proj_b(u), self.D_proj(u), self.compute_dtype)
        return drive, forget, in_gate, out_gate

    def forward(
        self,
        x: torch.Tensor,
        *,
        block_l: int = 256,
        checkpoint: bool = True,
        tile_b: Optional[int] = None,
        tile_d: Optional[int] = None,
        backend: str = "auto",
        scan_out_dtype: Optional[torch.dtype] = None,
    ) -> torch.Tensor:
        if (x.is_cuda and torch.cuda.is_current_stream_capturing() and torch.is_grad_enabled()
                and (x.requires_grad or any(p.requires_grad for p in self.parameters()))):
            # a recorded training step would also record the backward of the projections' bias and weight gradients
            # (library reductions with memset nodes), which does not replay reliably on this platform
            raise RuntimeError(
                "quick_ssm_amd.SSM: recording a differentiable forward into a HIP graph is not supported (the backward's "
                "torch library calls record memset nodes that do not replay reliably on this platform); record under "
                "torch.no_grad(), or run the training step eagerly.")
        skip = x if self.use_residual else 0
        u = self.pre_norm(x) if self.use_norm else x
        w_dtype = self.out_proj.weight.dtype
        out_dtype = w_dtype if scan_out_dtype is None else scan_out_dtype
        if backend in ("auto", "hip", "triton") and u.is_cuda and not _scan_interface._HONOR_TILES:
            # 16-bit projections stored as the compute dtype, or fp32 projections with fp32 y: the activations (and the
            # casts to the compute dtype) happen inside the scan's launches
            wide = self._wide_projection(u)
            if wide is not None:
                S = self.state_size_dim
                pre = tuple(wide[..., k * S:(k + 1) * S] for k in range(5))
            else:
                pre = (self.A_proj(u), self.B_proj(u), self.C_proj_a(u), self.C_proj_b(u), self.D_proj(u))
            if wide is not None and wide.dim() == 3 and _gated.supported(pre, self.compute_dtype, out_dtype, checkpoint):
                y = _gated.gated_scan_wide(wide, out_dtype=out_dtype, compute_dtype=self.compute_dtype)
            elif _gated.supported(pre, self.compute_dtype, out_dtype, checkpoint):
                y = _gated.gated_scan(*pre, out_dtype=out_dtype, compute_dtype=self.compute_dtype)
            else:
                if wide is not None:
                    forget, drive, out_gate, in_gate = gate_prologue_wide(wide, self.compute_dtype)
                else:
                    forget, drive, out_gate, in_gate = gate_prologue(*pre, self.compute_dtype)
                y = scan(x=drive, a=forget, b=in_gate, c=out_gate, block_l=block_l, checkpoint=checkpoint,
                         tile_b=tile_b, tile_d=tile_d, out_dtype=out_dtype, backend=backend)
            y = y if y.dtype == w_dtype else y.to(w_dtype)
            return _LinearBias.apply(y, self.out_proj.weight, self.out_proj.bias) + skip
        drive, forget, in_gate, out_gate = self.gates(u)
        y = scan(
            x=drive, a=forget, b=in_gate, c=out_gate,
            block_l=block_l, checkpoint=checkpoint, tile_b=tile_b, tile_d=tile_d,
            out_dtype=out_dtype,
            backend=backend,
        )
        return self.out_proj(y.to(w_dtype)) + skip


__all__ = ["SSM", "RMSNorm"]
