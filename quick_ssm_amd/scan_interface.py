"""Public scan entry point: `scan(x, a, b, c, *, block_l, checkpoint, tile_b, tile_d, backend, out_dtype)`.

    h(t) = a(t) * h(t-1) + b(t) * x(t)        (all tensors [B, L, D])
    y(t) = c(t) * h(t)

Same surface as the reference's `quick_ssm/scan_interface.py` (`scan` :169-213, the autograd
Function :49-158, `_chunk_ranges` :36-46, `_torch_scan` :161-166); the device work behind it is one
HIP launch per direction on gfx950 instead of Triton kernels inside a Python tile loop.

What the knobs mean here
  block_l     accepted and recorded.  The kernels pick their own time tiling (tile length and
              the spacing of the states kept for the backward); results do not depend on it.
  checkpoint  True: the forward keeps only the fp32 state at every `ckpt_stride`-th step (about
              1/64 of one tensor) and the backward rebuilds h inside each tile.  False: the
              forward also keeps the full fp32 h (`ctx.h_saved`, as the reference does) and the
              backward reads it.
  tile_b/d    accepted.  They bound the reference's N-sized fp32 scratch, which does not exist
              here, and rows (b, d) are independent, so by default one launch covers the whole
              tensor.  `honor_tiles(True)` makes every tile its own launch on a strided view
              (no copies); batch tiles give bitwise the same results, feature tiles agree to
              fp32 rounding (a narrower tile changes how lanes split the time axis).
  backend     "auto": the HIP kernels for GPU tensors, the sequential torch recurrence for CPU
              tensors.  "triton" is kept as the legacy name of the device path, "hip" is its
              proper name.  "torch": the sequential recurrence on whatever device the tensors
              are on.  A GPU tensor never takes the sequential path unless "torch" is asked for
              by name, and the device path raises if libquick_ssm_hip.so is not built.
"""
from __future__ import annotations

from typing import List, Optional, Tuple

import torch

from . import hip_scan
from .naive_baseline import naive_forward_3d

Tensor = torch.Tensor

_HONOR_TILES = False


def honor_tiles(flag: bool) -> bool:
    """Launch once per (tile_b, tile_d) tile instead of once per call.  Returns the old setting."""
    global _HONOR_TILES
    old, _HONOR_TILES = _HONOR_TILES, bool(flag)
    return old


def _chunk_ranges(total: int, tile: Optional[int]) -> List[Tuple[int, int]]:
    """Half-open ranges covering [0, total); no tile, a non-positive one or one >= total gives one range."""
    if tile is None or tile <= 0 or tile >= total:
        return [(0, total)]
    edges = list(range(0, total, tile)) + [total]
    return list(zip(edges[:-1], edges[1:]))


def _launch_tiles(shape, tile_b, tile_d) -> List[Tuple[slice, slice]]:
    if not _HONOR_TILES:
        return [(slice(0, shape[0]), slice(0, shape[2]))]
    return [
        (slice(b0, b1), slice(d0, d1))
        for b0, b1 in _chunk_ranges(shape[0], tile_b)
        for d0, d1 in _chunk_ranges(shape[2], tile_d)
    ]


class _HipScanFunction(torch.autograd.Function):
    """Autograd node of the device scan: one HIP launch forward, one backward.

    Argument list, saved state and returned gradients follow the reference's
    `_TritonScanFunction` (quick_ssm/scan_interface.py:49-158): forward takes
    (x, a, b, c, block_l, checkpoint, tile_b, tile_d, out_dtype); backward returns
    (dx, da, db, dc, None x 5) with every gradient in its operand's dtype.
    """

    @staticmethod
    def forward(ctx, x: Tensor, a: Tensor, b: Tensor, c: Tensor, block_l: int, checkpoint: bool,
                tile_b: Optional[int], tile_d: Optional[int], out_dtype: torch.dtype) -> Tensor:
        if x.shape != a.shape or x.shape != b.shape or x.shape != c.shape:
            raise ValueError("x, a, b, c must share the same shape [B, L, D].")
        if x.dim() != 3:
            raise ValueError("x, a, b, c must be 3-D tensors [B, L, D].")
        if x.device.type != "cuda":
            raise RuntimeError("HIP scan backend requires GPU tensors.")

        ctx.block_l = int(block_l)
        ctx.checkpoint = bool(checkpoint)
        ctx.tile_b = tile_b
        ctx.tile_d = tile_d
        ctx.out_dtype = out_dtype
        ctx.save_for_backward(x, a, b, c)

        k_in, k_out = hip_scan.kernel_dtypes([x.dtype, a.dtype, b.dtype, c.dtype], out_dtype)
        xs, as_, bs, cs = (t if t.dtype == k_in else t.to(k_in) for t in (x, a, b, c))
        ctx.k_in, ctx.k_out = k_in, k_out

        tiles = _launch_tiles(x.shape, tile_b, tile_d)
        ctx.tiles = tiles
        ctx.tile_states = []
        whole = len(tiles) == 1
        y = None if whole else torch.empty(x.shape, dtype=k_out, device=x.device)
        # No operand wants a gradient (inference, torch.no_grad()): no backward will come, so no state is saved and
        # the launch streams its operands past the caches.
        train = any(ctx.needs_input_grad[:4])
        h_saved = None
        if train and not checkpoint and not whole:
            h_saved = torch.empty(x.shape, dtype=torch.float32, device=x.device)
        for bs_, ds_ in tiles:
            # the common case, one launch over the whole tensor, skips four view constructions
            ops = (xs, as_, bs, cs) if whole else tuple(t[bs_, :, ds_] for t in (xs, as_, bs, cs))
            yt, ht, ckpt, stride = hip_scan.scan_forward(
                *ops, out_dtype=k_out, want_h=train and not checkpoint, want_ckpt=train and bool(checkpoint),
            )
            ctx.tile_states.append((ckpt, stride))
            if whole:
                y, h_saved = yt, ht
            else:
                y[bs_, :, ds_] = yt
                if h_saved is not None:
                    h_saved[bs_, :, ds_] = ht
        ctx.h_saved = h_saved
        return y if y.dtype == out_dtype else y.to(out_dtype)

    @staticmethod
    def backward(ctx, grad_output: Tensor):
        x, a, b, c = ctx.saved_tensors
        k_in, k_out = ctx.k_in, ctx.k_out
        xs, as_, bs, cs = (t if t.dtype == k_in else t.to(k_in) for t in (x, a, b, c))
        dy = grad_output if grad_output.dtype == k_out else grad_output.to(k_out)
        need = tuple(ctx.needs_input_grad[:4])

        whole = len(ctx.tiles) == 1
        grads = [None, None, None, None]
        if not whole:
            grads = [torch.empty(x.shape, dtype=k_in, device=x.device) if n else None for n in need]
        for (bs_, ds_), (ckpt, stride) in zip(ctx.tiles, ctx.tile_states):
            if whole:
                ops, h_tile = (xs, as_, bs, cs, dy), ctx.h_saved
            else:
                ops = tuple(t[bs_, :, ds_] for t in (xs, as_, bs, cs, dy))
                h_tile = None if ctx.h_saved is None else ctx.h_saved[bs_, :, ds_]
            out = hip_scan.scan_backward(
                *ops, h=h_tile, ckpt=None if h_tile is not None else ckpt, ckpt_stride=stride, need=need,
            )
            if whole:
                grads = list(out)
            else:
                for gfull, gt in zip(grads, out):
                    if gfull is not None:
                        gfull[bs_, :, ds_] = gt

        def _as(g: Optional[Tensor], like: Tensor) -> Optional[Tensor]:
            if g is None:
                return None
            return g if g.dtype == like.dtype else g.to(like.dtype)

        return (_as(grads[0], x), _as(grads[1], a), _as(grads[2], b), _as(grads[3], c),
                None, None, None, None, None)


# The reference's name for the autograd node; kept so that code reaching for it still works.
_TritonScanFunction = _HipScanFunction


def _torch_scan(x: Tensor, a: Tensor, b: Tensor, c: Tensor, out_dtype: torch.dtype) -> Tensor:
    """Sequential recurrence in plain torch (the reference's CPU path, scan_interface.py:161-166)."""
    h = naive_forward_3d(x, a, b)
    return (c * h).to(out_dtype)


class _HipScanCarryFunction(torch.autograd.Function):
    """Autograd node of the device scan with a carried state: (x, a, b, c, h_init) -> (y, h_final).

    One HIP launch forward, one backward, like `_HipScanFunction`; the backward also takes the
    gradient arriving at h_final and returns the gradient of h_init, so pieces of a sequence
    chain through autograd exactly as the whole sequence would.
    """

    @staticmethod
    def forward(ctx, x: Tensor, a: Tensor, b: Tensor, c: Tensor, h_init: Optional[Tensor], checkpoint: bool,
                out_dtype: torch.dtype):
        if x.shape != a.shape or x.shape != b.shape or x.shape != c.shape:
            raise ValueError("x, a, b, c must share the same shape [B, L, D].")
        if x.dim() != 3:
            raise ValueError("x, a, b, c must be 3-D tensors [B, L, D].")
        if x.device.type != "cuda":
            raise RuntimeError("HIP scan backend requires GPU tensors.")
        B, L, D = x.shape
        if h_init is not None and tuple(h_init.shape) != (B, D):
            raise ValueError(f"state must have shape {(B, D)}, got {tuple(h_init.shape)}.")
        k_in, k_out = hip_scan.kernel_dtypes([x.dtype, a.dtype, b.dtype, c.dtype], out_dtype)
        xs, as_, bs, cs = (t if t.dtype == k_in else t.to(k_in) for t in (x, a, b, c))
        h0 = None
        if h_init is not None:
            h0 = h_init.detach().to(torch.float32).contiguous()
            if h0.data_ptr() % 16 != 0:
                h0 = h0.clone()
        h_final = torch.empty((B, D), dtype=torch.float32, device=x.device)
        train = any(ctx.needs_input_grad[:5])   # generation mode saves no states and leaves nothing in the caches
        y, h_full, ckpt, stride = hip_scan.scan_forward(
            xs, as_, bs, cs, out_dtype=k_out, want_h=train and not checkpoint, want_ckpt=train and bool(checkpoint),
            h_init=h0, h_final=h_final,
        )
        ctx.save_for_backward(x, a, b, c)
        ctx.k_in, ctx.k_out = k_in, k_out
        ctx.h0, ctx.h_saved, ctx.ckpt, ctx.stride = h0, h_full, ckpt, stride
        ctx.state_dtype = None if h_init is None else h_init.dtype
        return (y if y.dtype == out_dtype else y.to(out_dtype)), h_final

    @staticmethod
    def backward(ctx, grad_y: Optional[Tensor], grad_state: Optional[Tensor]):
        x, a, b, c = ctx.saved_tensors
        k_in, k_out = ctx.k_in, ctx.k_out
        B, L, D = x.shape
        xs, as_, bs, cs = (t if t.dtype == k_in else t.to(k_in) for t in (x, a, b, c))
        if grad_y is None:
            grad_y = torch.zeros((B, L, D), dtype=k_out, device=x.device)
        dy = grad_y if grad_y.dtype == k_out else grad_y.to(k_out)
        dh_final = None
        if grad_state is not None:
            dh_final = grad_state.to(torch.float32).contiguous()
            if dh_final.data_ptr() % 16 != 0:
                dh_final = dh_final.clone()
        need = tuple(ctx.needs_input_grad[:4])
        dh_init = None
        if ctx.needs_input_grad[4]:
            dh_init = torch.empty((B, D), dtype=torch.float32, device=x.device)
        out = hip_scan.scan_backward(
            xs, as_, bs, cs, dy, h=ctx.h_saved, ckpt=None if ctx.h_saved is not None else ctx.ckpt,
            ckpt_stride=ctx.stride, need=need, h_init=ctx.h0, dh_final=dh_final, dh_init=dh_init,
        )

        def _as(g: Optional[Tensor], like_dtype) -> Optional[Tensor]:
            if g is None:
                return None
            return g if g.dtype == like_dtype else g.to(like_dtype)

        return (_as(out[0], x.dtype), _as(out[1], a.dtype), _as(out[2], b.dtype), _as(out[3], c.dtype),
                _as(dh_init, ctx.state_dtype), None, None)


def scan_chunk(
    x: Tensor,
    a: Tensor,
    b: Tensor,
    c: Tensor,
    state: Optional[Tensor] = None,
    *,
    checkpoint: bool = True,
    backend: str = "auto",
    out_dtype: Optional[torch.dtype] = None,
) -> Tuple[Tensor, Tensor]:
    """One piece of a longer scan: starts from `state` (h before the piece's first step, [B, D]; None
    = zero) and returns `(y, new_state)` with new_state = h after its last step, in float32 (on the
    sequential CPU path: in the dtype the recurrence is accumulated in).

    Feeding each piece's `new_state` to the next gives the same y, and through autograd the same
    gradients, as one `scan` over the concatenated sequence: chunked prefill and token-by-token
    generation (L = 1).  The reference's scan always starts from zero
    (quick_ssm/scan_interface.py:15-21) and lists a generation mode as future work (README.md:176-184);
    this is that mode on the same kernels.
    """
    out_dtype = out_dtype or x.dtype
    chosen = backend
    if backend == "auto":
        chosen = "hip" if x.device.type == "cuda" else "torch"
    if chosen in ("hip", "triton"):
        return _HipScanCarryFunction.apply(x, a, b, c, state, checkpoint, out_dtype)
    if chosen == "torch":
        h, final = naive_forward_3d(x, a, b, h_init=state, return_final=True)
        return (c * h).to(out_dtype), final
    raise ValueError(f"Unsupported backend '{backend}'. Use 'auto', 'hip', 'triton', or 'torch'.")


def scan(
    x: Tensor,
    a: Tensor,
    b: Tensor,
    c: Tensor,
    *,
    block_l: int = 256,
    checkpoint: bool = True,
    tile_b: Optional[int] = None,
    tile_d: Optional[int] = None,
    backend: str = "auto",
    out_dtype: Optional[torch.dtype] = None,
) -> Tensor:
    """Gated linear scan y = c * h, h(t) = a(t) h(t-1) + b(t) x(t), differentiable in x, a, b, c.

    Args:
        x, a, b, c: tensors of shape [B, L, D].
        block_l, checkpoint, tile_b, tile_d: see the module docstring.
        backend: "auto" (default), "hip" / "triton" (device kernels), or "torch".
        out_dtype: dtype of the returned tensor; defaults to x.dtype.

    Returns:
        y of shape [B, L, D] and dtype `out_dtype`.
    """
    out_dtype = out_dtype or x.dtype
    chosen = backend
    if backend == "auto":
        chosen = "hip" if x.device.type == "cuda" else "torch"
    if chosen in ("hip", "triton"):
        return _HipScanFunction.apply(x, a, b, c, block_l, checkpoint, tile_b, tile_d, out_dtype)
    if chosen == "torch":
        return _torch_scan(x, a, b, c, out_dtype)
    raise ValueError(f"Unsupported backend '{backend}'. Use 'auto', 'hip', 'triton', or 'torch'.")


__all__ = ["scan", "scan_chunk", "honor_tiles"]
