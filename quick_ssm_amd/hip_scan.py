"""Host side of the HIP scan: tensor checks, launch planning, workspace, and the two launches.

Everything here is plumbing around `qssm_scan_forward` / `qssm_scan_backward`
(include/quick_ssm_hip.h).  It takes the place of the launch code in the reference's
`block_scan_forward_3d` (quick_ssm/triton_forwards.py:134-172) and `block_scan_backward_3d`
(quick_ssm/triton_backwards.py:168-209): no fp32 upcast copies, no N-sized scratch, one launch per
direction.
"""
from __future__ import annotations

import ctypes
import threading
from typing import Dict, Optional, Sequence, Tuple

import torch

from . import _lib
from ._lib import Plan, Strides

Tensor = torch.Tensor

_DTYPE_CODE = {torch.float32: _lib.QSSM_F32, torch.float16: _lib.QSSM_F16, torch.bfloat16: _lib.QSSM_BF16}
# (storage of x,a,b,c) -> storages of y the kernels are built for
_BUILT_OUT = {
    torch.float32: (torch.float32,),
    torch.float16: (torch.float16, torch.float32),
    torch.bfloat16: (torch.bfloat16, torch.float32),
}

_ws_lock = threading.Lock()
_EPOCH_MAX = 0xFFFFFFFF


class _Buffers:
    """Per (device, stream, who numbers the launches): control block, workspace, and the host's launch count."""

    __slots__ = ("control", "workspace", "epoch")

    def __init__(self):
        self.control: Optional[Tensor] = None
        self.workspace: Optional[Tensor] = None
        self.epoch = 0


_buffers: Dict[Tuple[int, int, bool], _Buffers] = {}


def kernel_dtypes(in_dtypes: Sequence[torch.dtype], out_dtype: torch.dtype) -> Tuple[torch.dtype, torch.dtype]:
    """Storage types the launch will use for (x,a,b,c / grads) and for (y / dy).

    Arithmetic is fp32 in every case.  Operands of mixed or unsupported storage are cast to a
    common supported one on the host; an unsupported y storage is produced as fp32 and cast.
    """
    common = in_dtypes[0]
    for dt in in_dtypes[1:]:
        common = torch.promote_types(common, dt)
    if common not in _DTYPE_CODE:
        common = torch.float32
    k_out = out_dtype if out_dtype in _BUILT_OUT[common] else torch.float32
    return common, k_out


def _unit_inner(t: Tensor) -> Tensor:
    """A view or copy of `t` whose last axis is contiguous."""
    if t.size(-1) > 1 and t.stride(-1) != 1:
        return t.contiguous()
    if t.size(-1) == 1 and t.stride(-1) != 1:
        return t.contiguous()
    return t


def _strides(t: Optional[Tensor]) -> Strides:
    if t is None:
        return Strides(0, 0)
    return Strides(t.stride(0), t.stride(1))


def _ptr(t: Optional[Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


def _align_elems(tensors: Sequence[Optional[Tensor]], D: int) -> int:
    """Largest v in (8, 4, 2, 1) such that D, every stride and every base address (in elements) divide by v."""
    for v in (8, 4, 2):
        ok = D % v == 0
        for t in tensors:
            if not ok:
                break
            if t is None:
                continue
            es = t.element_size()
            ok = t.data_ptr() % (es * v) == 0 and t.stride(0) % v == 0 and t.stride(1) % v == 0
        if ok:
            return v
    return 1


_device_counted_depth = 0  # contexts open right now, in any thread (guarded by _ws_lock)


class device_counted_launches:
    """Context manager: scan launches made while it is open, from any thread (autograd runs the backward on its
    own), number themselves in their control block (epoch argument 0), as launches recorded into a graph do, and use
    the buffers kept for such launches.

    Launches being recorded into a graph do this by themselves, but cannot allocate: run the work once inside this
    context, on the stream that will capture, and the control block and workspace exist (large enough) when the
    capture starts.
    """

    def __enter__(self):
        global _device_counted_depth
        with _ws_lock:
            _device_counted_depth += 1
        return self

    def __exit__(self, *exc):
        global _device_counted_depth
        with _ws_lock:
            _device_counted_depth -= 1
        return False


def _launch_buffers(device: torch.device, stream: int, plan: Plan) -> Tuple[Tensor, Tensor, int]:
    """Control block, workspace and epoch argument for the next launch on (device, stream).

    Both buffers are zero-filled when they are allocated (torch.zeros runs a fill kernel on the
    current stream, ahead of the launch that uses them) and grown on demand.  Every launch leaves
    the control block's status word and ticket counters zero.  The workspace is never cleared:
    every launch gets the next epoch.  Eager launches are numbered here.  Launches recorded into a
    graph (and those inside `device_counted_launches`) use a pair of buffers of their own and are
    numbered in the control block itself (epoch argument 0), so that replays number themselves, at
    the price of a one-lane counting kernel behind each launch.  A workspace that has to grow, or
    whose 32-bit host numbering is used up, is replaced by a fresh zeroed one.
    """
    capturing = bool(torch.cuda.is_current_stream_capturing())
    on_device = capturing or _device_counted_depth > 0
    key = (device.index if device.index is not None else torch.cuda.current_device(), stream, on_device)
    with _ws_lock:
        buf = _buffers.get(key)
        if buf is None:
            buf = _Buffers()
        need_c, need_w = int(plan.control_bytes), max(int(plan.workspace_bytes), 256)
        grow_c = buf.control is None or buf.control.numel() < need_c
        grow_w = grow_c or buf.workspace is None or buf.workspace.numel() < need_w or buf.epoch >= _EPOCH_MAX
        if capturing and grow_w:
            raise RuntimeError(
                "quick_ssm_amd: a scan launch being recorded into a graph cannot allocate its control block and "
                "workspace; run the same work once inside `hip_scan.device_counted_launches()` on this stream first")
        _buffers[key] = buf
        if grow_c:
            # a new control block restarts the device-side count: the workspace must not keep words of the old numbering
            buf.control = torch.zeros(max(1 << 16, 1 << (need_c - 1).bit_length()), dtype=torch.uint8, device=device)
        if grow_w:
            buf.workspace = torch.zeros(max(1 << 20, 1 << (need_w - 1).bit_length()), dtype=torch.uint8, device=device)
            buf.epoch = 0
        if on_device:
            return buf.control, buf.workspace, 0
        buf.epoch += 1
        return buf.control, buf.workspace, buf.epoch


def workspace_status(device: Optional[torch.device] = None) -> int:
    """Status words of the current stream's control blocks, or-ed (synchronises).  0 = all launches completed."""
    device = torch.device("cuda", torch.cuda.current_device()) if device is None else device
    stream = torch.cuda.current_stream(device).cuda_stream
    index = device.index if device.index is not None else torch.cuda.current_device()
    status = 0
    for on_device in (False, True):
        with _ws_lock:
            buf = _buffers.get((index, stream, on_device))
        if buf is None or buf.control is None:
            continue
        out = ctypes.c_int32(0)
        _lib.check(_lib.load().qssm_control_status(buf.control.data_ptr(), stream, ctypes.byref(out)))
        status |= int(out.value)
    return status


def reset_workspaces() -> None:
    """Drop every cached buffer (the next launch allocates fresh zeroed ones)."""
    with _ws_lock:
        _buffers.clear()


_plans: Dict[tuple, Plan] = {}


def make_plan(B: int, L: int, D: int, in_dtype: torch.dtype, out_dtype: torch.dtype, direction: int,
              align_elems: int, ckpt_stride: int = 0, tune: int = 0) -> Plan:
    """Launch geometry for a shape (qssm_plan_scan).  Plans depend on nothing but the arguments, so they are
    kept: small problems are bound by the host side of a launch.  Callers must not modify the result."""
    key = (B, L, D, in_dtype, out_dtype, direction, align_elems, ckpt_stride, tune)
    plan = _plans.get(key)
    if plan is None:
        plan = Plan()
        _lib.check(
            _lib.load().qssm_plan_scan(B, L, D, _DTYPE_CODE[in_dtype], _DTYPE_CODE[out_dtype], direction,
                                       align_elems, ckpt_stride, tune, ctypes.byref(plan))
        )
        if len(_plans) >= 4096:
            _plans.clear()
        _plans[key] = plan
    return plan


def _require_gpu(*tensors: Tensor) -> torch.device:
    dev = tensors[0].device
    for t in tensors:
        if t.device.type != "cuda":
            raise RuntimeError("HIP scan backend requires GPU tensors.")
        if t.device != dev:
            raise RuntimeError("all scan operands must live on one GPU")
    return dev


def _check_state(t: Optional[Tensor], B: int, D: int, dev: torch.device, name: str) -> None:
    """A carried state / its gradient: fp32 [B, D], contiguous, on the operands' device."""
    if t is None:
        return
    if tuple(t.shape) != (B, D) or t.dtype != torch.float32 or not t.is_contiguous() or t.device != dev:
        raise ValueError(f"{name} must be a contiguous float32 tensor of shape {(B, D)} on {dev}, "
                         f"got {t.dtype} {tuple(t.shape)} on {t.device}")


def scan_forward(
    x: Tensor, a: Tensor, b: Tensor, c: Optional[Tensor], *,
    out_dtype: torch.dtype,
    want_y: bool = True,
    want_h: bool = False,
    want_ckpt: bool = True,
    tune: int = 0,
    bwd_tune: int = 0,
    h_init: Optional[Tensor] = None,
    h_final: Optional[Tensor] = None,
) -> Tuple[Optional[Tensor], Optional[Tensor], Optional[Tensor], int]:
    """One forward launch.  Operands must already share one supported storage type.

    Returns (y, h, ckpt, ckpt_stride): y in `out_dtype` (a storage the kernels are built for), h
    the full fp32 state if `want_h`, ckpt the fp32 states h(t-1) at t = k*ckpt_stride if
    `want_ckpt` (what the backward rebuilds h from).  `h_init` (fp32 [B, D], contiguous) is the
    state before the first step instead of zero; `h_final` (same layout) receives h(L-1).
    """
    ops = [x, a, b] + ([c] if c is not None else [])
    dev = _require_gpu(*ops)
    B, L, D = x.shape
    in_dtype = x.dtype
    y = torch.empty((B, L, D), dtype=out_dtype, device=dev) if want_y else None
    h = torch.empty((B, L, D), dtype=torch.float32, device=dev) if want_h else None
    _check_state(h_init, B, D, dev, "h_init")
    _check_state(h_final, B, D, dev, "h_final")
    if B == 0 or L == 0 or D == 0:
        if h_final is not None:  # nothing happened to the state
            h_final.copy_(h_init) if h_init is not None else h_final.zero_()
        return y, h, (torch.empty((B, 0, D), dtype=torch.float32, device=dev) if want_ckpt else None), 0

    x, a, b = _unit_inner(x), _unit_inner(a), _unit_inner(b)
    c = _unit_inner(c) if c is not None else None
    align = _align_elems([x, a, b, c, y, h], D)

    ckpt_stride = 0
    if want_ckpt:
        # The backward decides how far apart the saved states may be; the forward follows.
        ckpt_stride = make_plan(B, L, D, in_dtype, out_dtype, _lib.QSSM_BACKWARD, align, 0, bwd_tune).seg_len
    plan = make_plan(B, L, D, in_dtype, out_dtype, _lib.QSSM_FORWARD, align, ckpt_stride, tune)
    ckpt = None
    if want_ckpt:
        ckpt = torch.empty((B, plan.n_ckpt, D), dtype=torch.float32, device=dev)

    with torch.cuda.device(dev):
        stream = torch.cuda.current_stream(dev).cuda_stream
        ctl, ws, epoch = _launch_buffers(dev, stream, plan)
        _lib.check(
            _lib.load().qssm_scan_forward_carry(
                ctypes.byref(plan),
                _ptr(x), _strides(x), _ptr(a), _strides(a), _ptr(b), _strides(b), _ptr(c), _strides(c),
                _ptr(y), _strides(y), _ptr(h), _strides(h), _ptr(ckpt), _ptr(h_init), _ptr(h_final),
                ctl.data_ptr(), ctl.numel(), ws.data_ptr(), ws.numel(), epoch, stream,
            )
        )
    return y, h, ckpt, int(plan.ckpt_stride)


def scan_backward(
    x: Tensor, a: Tensor, b: Tensor, c: Tensor, dy: Tensor, *,
    h: Optional[Tensor] = None,
    ckpt: Optional[Tensor] = None,
    ckpt_stride: int = 0,
    need: Sequence[bool] = (True, True, True, True),
    tune: int = 0,
    h_init: Optional[Tensor] = None,
    dh_final: Optional[Tensor] = None,
    dh_init: Optional[Tensor] = None,
) -> Tuple[Optional[Tensor], Optional[Tensor], Optional[Tensor], Optional[Tensor]]:
    """One backward launch.  x, a, b, c share one storage type; dy has the storage of y.

    Exactly one of `h` (full fp32 state) and `ckpt` (+ its `ckpt_stride`) must be given.  Returns
    (dx, da, db, dc) in the storage type of the operands; entries not in `need` are None.
    `h_init` is the state the forward started from, `dh_final` the gradient arriving at h(L-1),
    `dh_init` receives the gradient of h(-1); all fp32 [B, D], contiguous, optional.
    """
    dev = _require_gpu(x, a, b, c, dy)
    B, L, D = x.shape
    in_dtype = x.dtype
    grads = [torch.empty((B, L, D), dtype=in_dtype, device=dev) if n else None for n in need]
    for name, t in (("h_init", h_init), ("dh_final", dh_final), ("dh_init", dh_init)):
        _check_state(t, B, D, dev, name)
    if B == 0 or L == 0 or D == 0:
        if dh_init is not None:  # the state passed through untouched
            dh_init.copy_(dh_final) if dh_final is not None else dh_init.zero_()
        return tuple(grads)
    if (h is None) == (ckpt is None):
        raise ValueError("pass exactly one of h and ckpt")

    x, a, b, c, dy = (_unit_inner(t) for t in (x, a, b, c, dy))
    if h is not None:
        h = _unit_inner(h if h.dtype == torch.float32 else h.float())
    else:
        ckpt = ckpt.contiguous()
    align = _align_elems([x, a, b, c, dy, h, *grads], D)
    plan = make_plan(B, L, D, in_dtype, dy.dtype, _lib.QSSM_BACKWARD, align, ckpt_stride if h is None else 0, tune)
    if ckpt is not None and tuple(ckpt.shape) != (B, plan.n_ckpt, D):
        raise ValueError(f"ckpt has shape {tuple(ckpt.shape)}, expected {(B, plan.n_ckpt, D)}")

    with torch.cuda.device(dev):
        stream = torch.cuda.current_stream(dev).cuda_stream
        ctl, ws, epoch = _launch_buffers(dev, stream, plan)
        _lib.check(
            _lib.load().qssm_scan_backward_carry(
                ctypes.byref(plan),
                _ptr(x), _strides(x), _ptr(a), _strides(a), _ptr(b), _strides(b), _ptr(c), _strides(c),
                _ptr(dy), _strides(dy), _ptr(h), _strides(h), _ptr(ckpt),
                _ptr(h_init), _ptr(dh_final), _ptr(dh_init),
                _ptr(grads[0]), _strides(grads[0]), _ptr(grads[1]), _strides(grads[1]),
                _ptr(grads[2]), _strides(grads[2]), _ptr(grads[3]), _strides(grads[3]),
                ctl.data_ptr(), ctl.numel(), ws.data_ptr(), ws.numel(), epoch, stream,
            )
        )
    return tuple(grads)


def block_scan_forward_3d(x: Tensor, a: Tensor, b: Tensor, BLOCK_L: int = 256) -> Tuple[Tensor, Tensor]:
    """Device forward of h(t) = a(t) h(t-1) + b(t) x(t).

    Same contract as the reference's function of this name (quick_ssm/triton_forwards.py:134-172):
    3-D GPU inputs, returns fp32 `(out_a, out_x)` with out_x = h and out_a the running product of
    a.  `BLOCK_L` is accepted for compatibility; the launch geometry no longer depends on it.
    """
    for t in (x, a, b):
        assert t.dim() == 3, "All inputs should be [B, L, D]."
        assert t.device.type == "cuda", "Inputs must be on a GPU device."
    B, L, D = x.shape
    if L == 0:
        return torch.empty_like(a), torch.empty_like(x)
    k_in, _ = kernel_dtypes([x.dtype, a.dtype, b.dtype], torch.float32)
    xs, as_, bs = (t if t.dtype == k_in else t.to(k_in) for t in (x, a, b))
    h, _, _, _ = scan_forward(xs, as_, bs, None, out_dtype=torch.float32, want_ckpt=False)
    # out_a is discarded by every caller of the reference; it is kept for the tuple's shape.
    out_a = torch.cumprod(a.to(torch.float32), dim=1)
    return out_a, h


def block_scan_backward_3d(a: Tensor, b: Tensor, c: Tensor, x: Tensor, h: Tensor, grad_y: Tensor,
                           BLOCK_L: int = 256) -> Tuple[Tensor, Tensor, Tensor, Tensor]:
    """Device backward given the forward states h; returns fp32 (dx, da, db, dc).

    Same contract and argument order as the reference's function of this name
    (quick_ssm/triton_backwards.py:168-209), which upcasts every operand to fp32 first.
    """
    for t in (a, b, c, x, h, grad_y):
        assert t.dim() == 3, "All inputs should be [B, L, D]."
        assert t.device.type == "cuda", "Inputs must be on a GPU device."
    B, L, D = x.shape
    if L == 0:
        return (torch.empty_like(x), torch.empty_like(a), torch.empty_like(b), torch.empty_like(c))
    f32 = torch.float32
    a, b, c, x, h, grad_y = (t if t.dtype == f32 else t.to(f32) for t in (a, b, c, x, h, grad_y))
    return scan_backward(x, a, b, c, grad_y, h=h)
