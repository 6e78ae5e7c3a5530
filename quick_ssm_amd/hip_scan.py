"""Host side of the HIP scan: tensor checks, launch planning, workspace, and the two launches.

Everything here is plumbing around `qssm_scan_forward` / `qssm_scan_backward`
(include/quick_ssm_hip.h).  It takes the place of the launch code in the reference's
`block_scan_forward_3d` (quick_ssm/triton_forwards.py:134-172) and `block_scan_backward_3d`
(quick_ssm/triton_backwards.py:168-209): no fp32 upcast copies, no N-sized scratch, one launch per
direction.
"""
from __future__ import annotations

import ctypes
import os
import threading
from typing import Dict, List, Optional, Sequence, Tuple

import torch

from . import _lib
from ._lib import BackwardCall, ForwardCall, Plan, Strides

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


class ScanLaunchError(RuntimeError):
    """A scan launch reported failure through its control block's status word.

    status 1: a tile gave up waiting for a neighbour's word (about a second); outputs downstream of it are NaN.
    status 2: a ticket counter was not zero when the launch started; every output of the launch is NaN.
    By the time this is raised the control block and workspace have been zero-filled again, so the next launch
    on the stream starts clean; results of launches since the last check must be discarded.
    """

    def __init__(self, status: int, where: str):
        super().__init__(
            f"quick_ssm_amd: a scan launch on {where} failed with status {status} "
            f"({'a tile gave up waiting for a neighbour' if status == 1 else 'the control block was not zero on entry' if status == 2 else 'both kinds of failure'}); "
            "its outputs are NaN. Control block and workspace have been reset; repeat the step.")
        self.status = status


def _env_int(name: str, default: int) -> int:
    try:
        return int(os.environ.get(name, default))
    except ValueError:
        return default


# Every `_check_every`-th launch on a pair of buffers is followed by an asynchronous copy of the status word to
# pinned host memory, looked at (without waiting) before each later launch: a failed launch is reported within two
# such periods.  QSSM_CHECK_STATUS=1 checks behind every launch, 0 never; set_status_check_period() at run time.
_check_every = _env_int("QSSM_CHECK_STATUS", 64)


def set_status_check_period(launches: int) -> int:
    """Look at the status word every `launches`-th launch (0: never).  Returns the old period."""
    global _check_every
    old, _check_every = _check_every, max(0, int(launches))
    return old


class _Buffers:
    """Per (device, stream, who numbers the launches): control block, workspace, the host's launch count, and the
    pinned word the status is copied to."""

    __slots__ = ("control", "workspace", "epoch", "ctl_ptr", "ctl_size", "ws_ptr", "ws_size", "captured",
                 "pinned", "seen", "since_check", "device", "where")

    def __init__(self, device: torch.device, where: str):
        self.control: Optional[Tensor] = None
        self.workspace: Optional[Tensor] = None
        self.epoch = 0
        self.ctl_ptr = self.ctl_size = self.ws_ptr = self.ws_size = 0
        self.captured = False          # a graph holds these addresses: never free or move them
        # The status word is copied here by a raw asynchronous copy that torch's pinned-memory allocator knows
        # nothing about: the block must never go back to it, or a copy still queued when the entry is dropped
        # would land in somebody else's tensor.  Four bytes per (device, stream) ever used.
        self.pinned = torch.zeros(1, dtype=torch.int32, pin_memory=True)
        _pinned_words.append(self.pinned)
        self.seen = ctypes.c_int32.from_address(self.pinned.data_ptr())
        self.since_check = 0
        self.device = device
        self.where = where


# One entry per (device, raw stream handle, device-counted) ever launched on.  Entries stay until reset_workspaces():
# a stream handle says nothing about whether its stream still exists, and an entry costs its control block and
# workspace (tens of MiB for large shapes), so a program that keeps making streams should call reset_workspaces()
# now and then.
_buffers: Dict[Tuple[int, int, bool], _Buffers] = {}
_pinned_words: List[Tensor] = []
# Buffers a recorded graph still points to, after they have been replaced by larger ones or dropped by
# reset_workspaces(): kept alive until the process ends, because replaying that graph writes to them.
_retired: List[Tensor] = []


def kernel_dtypes(in_dtypes: Sequence[torch.dtype], out_dtype: torch.dtype) -> Tuple[torch.dtype, torch.dtype]:
    """Storage types the launch will use for (x,a,b,c / grads) and for (y / dy).

    Arithmetic is fp32 in every case.  Operands of mixed or unsupported storage are cast to a
    common supported one on the host; an unsupported y storage is produced as fp32 and cast.
    """
    common = in_dtypes[0]
    for dt in in_dtypes[1:]:
        if dt != common:
            common = torch.promote_types(common, dt)
    if common not in _DTYPE_CODE:
        common = torch.float32
    k_out = out_dtype if out_dtype in _BUILT_OUT[common] else torch.float32
    return common, k_out


def _align_elems(tensors: Sequence[Optional[Tensor]], D: int) -> int:
    """Largest v in (8, 4, 2, 1) such that D, every stride and every base address (in elements) divide by v."""
    bits = D
    for t in tensors:
        if t is None:
            continue
        es = t.element_size()
        ptr = t.data_ptr()
        if ptr % es:
            return 1
        bits |= (ptr // es) | t.stride(0) | t.stride(1)
    low = bits & -bits
    return 8 if low == 0 or low > 8 else low


_ELEM_BYTES = {torch.float32: 4, torch.float16: 2, torch.bfloat16: 2}


def _describe(given: Sequence[Optional[Tensor]], fresh: Sequence[Optional[Tensor]], L: int, D: int):
    """What a launch needs of its tensors, with as few calls into torch as possible (small launches are bound by
    the host): the caller's tensors made contiguous in their last axis, then strides, base addresses and the
    alignment in elements (see `_align_elems`) of those and of the freshly allocated, contiguous outputs."""
    kept, strides, ptrs = [], [], []
    bits = D
    for t in given:
        if t is None:
            kept.append(None)
            strides.append(_NO_STRIDE)
            ptrs.append(None)
            continue
        st = t.stride()
        if st[2] != 1:
            t = t.contiguous()
            st = t.stride()
        ptr = t.data_ptr()
        es = _ELEM_BYTES[t.dtype]
        bits |= 1 if ptr % es else (ptr // es) | st[0] | st[1]
        kept.append(t)
        strides.append(st)
        ptrs.append(ptr)
    out_stride = (L * D, D, 1)
    for t in fresh:
        if t is None:
            strides.append(_NO_STRIDE)
            ptrs.append(None)
            continue
        ptr = t.data_ptr()
        bits |= (ptr // _ELEM_BYTES[t.dtype]) | out_stride[0]
        strides.append(out_stride)
        ptrs.append(ptr)
    low = bits & -bits
    return kept, tuple(strides), ptrs, (8 if low == 0 or low > 8 else low)


# (device index, stream handle) -> how many `device_counted_launches` contexts are open on it
_device_counted: Dict[Tuple[int, int], int] = {}


def _raw_stream(dev_index: int) -> int:
    return torch._C._cuda_getCurrentRawStream(dev_index)


class device_counted_launches:
    """Context manager: scan launches made on the stream that is current when it is entered, while it is open and
    from any thread (autograd runs the backward on its own, on the forward's stream), number themselves in their
    control block (epoch argument 0), as launches recorded into a graph do, and use the buffers kept for such
    launches.  Launches on other streams or devices are not affected.

    Launches being recorded into a graph do this by themselves, but cannot allocate: run the work once inside this
    context, on the stream that will capture, and the control block and workspace exist (large enough) when the
    capture starts.  Buffers a capture has used are never freed: if a later launch needs larger ones, new buffers
    take their place for new launches and the old ones stay alive for the graph that points to them.  Two graphs
    recorded on one stream share their buffers: replay them on that stream, one at a time.
    """

    def __enter__(self):
        index = torch.cuda.current_device()
        self._key = (index, _raw_stream(index))
        with _ws_lock:
            _device_counted[self._key] = _device_counted.get(self._key, 0) + 1
        return self

    def __exit__(self, *exc):
        with _ws_lock:
            left = _device_counted.get(self._key, 0) - 1
            if left > 0:
                _device_counted[self._key] = left
            else:
                _device_counted.pop(self._key, None)
        return False


def _grow_buffers(key: Tuple[int, int, bool], device: torch.device, need_c: int, need_w: int, capturing: bool) -> _Buffers:
    """Slow path of `_launch_buffers`: first use of a (device, stream), a larger shape, or a used-up numbering."""
    with _ws_lock:
        return _grow_buffers_locked(key, device, need_c, need_w, capturing)


def _grow_buffers_locked(key: Tuple[int, int, bool], device: torch.device, need_c: int, need_w: int, capturing: bool) -> _Buffers:
    """`_grow_buffers` for a caller that holds `_ws_lock`."""
    buf = _buffers.get(key)
    grow_c = buf is None or buf.control is None or buf.ctl_size < need_c
    grow_w = grow_c or buf.workspace is None or buf.ws_size < need_w or buf.epoch >= _EPOCH_MAX
    if capturing and grow_w:   # before anything is allocated: an allocation would spoil the recording
        raise RuntimeError(
            "quick_ssm_amd: a scan launch being recorded into a graph cannot allocate its control block and "
            "workspace; run the same work once inside `hip_scan.device_counted_launches()` on this stream first")
    if buf is None:
        buf = _Buffers(device, f"device {key[0]}, stream {key[1]:#x}")
    if buf.captured and grow_w:
        # a recorded graph points at the old pair: keep it alive and untouched, new launches get a new pair
        _retired.extend(t for t in (buf.control, buf.workspace) if t is not None)
        buf.captured = False
        grow_c = True
    if grow_c:
        # a new control block restarts the device-side count: the workspace must not keep words of the old numbering
        buf.control = torch.zeros(max(1 << 16, 1 << (need_c - 1).bit_length()), dtype=torch.uint8, device=device)
        buf.ctl_ptr, buf.ctl_size = buf.control.data_ptr(), buf.control.numel()
    if grow_w:
        buf.workspace = torch.zeros(max(1 << 20, 1 << (need_w - 1).bit_length()), dtype=torch.uint8, device=device)
        buf.ws_ptr, buf.ws_size = buf.workspace.data_ptr(), buf.workspace.numel()
        buf.epoch = 0
    _buffers[key] = buf
    return buf


def _recover(buf: _Buffers, stream: int) -> int:
    """Zero-fill a failed pair of buffers on `stream`, forget the host's numbering, and return the status seen."""
    lib = _lib.load()
    with torch.cuda.device(buf.device):
        _lib.check(lib.qssm_zero_fill(buf.ctl_ptr, buf.ctl_size, stream))
        _lib.check(lib.qssm_zero_fill(buf.ws_ptr, buf.ws_size, stream))
        out = ctypes.c_int32(0)
        _lib.check(lib.qssm_control_status(buf.ctl_ptr, stream, ctypes.byref(out)))   # waits: copies in flight have landed
    with _ws_lock:
        status = int(buf.seen.value)
        buf.seen.value = 0
        buf.epoch = 0
        buf.since_check = 0
    return status


def _launch_buffers(device: torch.device, dev_index: int, stream: int, need_c: int, need_w: int) -> Tuple[_Buffers, int, bool]:
    """Control block, workspace and epoch argument for the next launch on (device, stream).

    Both buffers are zero-filled when they are allocated (torch.zeros runs a fill kernel on the
    current stream, ahead of the launch that uses them) and grown on demand.  Every launch leaves
    the control block's status word and ticket counters zero.  The workspace is never cleared:
    every launch gets the next epoch.  Eager launches are numbered here.  Launches recorded into a
    graph (and those inside `device_counted_launches`) use a pair of buffers of their own and are
    numbered in the control block itself (epoch argument 0), so that replays number themselves, at
    the price of a one-lane counting kernel behind each launch.  A workspace that has to grow, or
    whose 32-bit host numbering is used up, is replaced by a fresh zeroed one.  A status word that an
    earlier check found nonzero raises ScanLaunchError here, after the buffers have been reset.
    """
    capturing = torch._C._cuda_isCurrentStreamCapturing()
    on_device = capturing or ((dev_index, stream) in _device_counted)
    key = (dev_index, stream, on_device)
    # Looking the buffers up and taking the next number is one step under the lock: the forward of the next step on
    # the caller's thread and a backward on autograd's thread may launch on one stream at the same time, and two
    # launches with one number would read each other's words as their own.
    with _ws_lock:
        buf = _buffers.get(key)
        if buf is None or buf.ctl_size < need_c or buf.ws_size < need_w or buf.epoch >= _EPOCH_MAX:
            buf = _grow_buffers_locked(key, device, need_c, max(need_w, 256), capturing)
        failed = buf.seen.value != 0 and not capturing
        epoch = 0
        if not failed:
            if capturing:
                buf.captured = True
            if not on_device:
                buf.epoch += 1
                epoch = buf.epoch
    if failed:
        raise ScanLaunchError(_recover(buf, stream), buf.where)
    return buf, epoch, capturing


def _after_launch(buf: _Buffers, stream: int, capturing: bool) -> None:
    """Every `_check_every`-th launch: ask for the status word, to be looked at before a later launch."""
    if _check_every <= 0 or capturing:
        return
    with _ws_lock:
        buf.since_check += 1
        due = buf.since_check >= _check_every
        if due:
            buf.since_check = 0
    if due:
        _lib.check(_lib.load().qssm_control_status_async(buf.ctl_ptr, buf.pinned.data_ptr(), stream))


def workspace_status(device: Optional[torch.device] = None, all_streams: bool = False) -> int:
    """Status words of the current stream's control blocks (of every stream of the device with `all_streams`),
    or-ed; synchronises those streams.  0 = all launches completed."""
    device = torch.device("cuda", torch.cuda.current_device()) if device is None else device
    index = device.index if device.index is not None else torch.cuda.current_device()
    stream = _raw_stream(index)
    with _ws_lock:
        bufs = [(k, b) for k, b in _buffers.items()
                if k[0] == index and (all_streams or k[1] == stream) and b.control is not None]
    status = 0
    for key, buf in bufs:
        out = ctypes.c_int32(0)
        with torch.cuda.device(device):
            _lib.check(_lib.load().qssm_control_status(buf.ctl_ptr, key[1], ctypes.byref(out)))
        status |= int(out.value)
    return status


def reset_workspaces() -> None:
    """Drop every cached buffer (the next launch allocates fresh zeroed ones).  Buffers that a recorded graph
    points to are not freed, but no later launch uses them: such graphs still replay, on their own old buffers."""
    with _ws_lock:
        for buf in _buffers.values():
            if buf.captured:
                _retired.extend(t for t in (buf.control, buf.workspace) if t is not None)
        _buffers.clear()


_plans: Dict[tuple, Plan] = {}
_forward_keep = True


def set_forward_keep(flag):
    """Whether forwards that save states for a backward (plain and gated) follow the planner's cache policy from now
    on (`plan.keep_tiles`: the last tiles of every chain load their operands with ordinary loads, for a backward
    that starts there; True), stream every operand past the caches (False), or keep at most that many tiles per
    chain (an int).  Forwards that save nothing always stream.  Results are the same bit for bit; only what a launch
    leaves in the caches differs.  Returns the old setting."""
    global _forward_keep
    old = _forward_keep
    _forward_keep = flag if isinstance(flag, bool) else max(0, int(flag))
    return old


def make_plan(B: int, L: int, D: int, in_dtype: torch.dtype, out_dtype: torch.dtype, direction: int,
              align_elems: int, ckpt_stride: int = 0, tune: int = 0) -> Plan:
    """Launch geometry for a shape (qssm_plan_scan; qssm_plan_scan_tuned when a test or sweep overrides single
    choices with `tune`).  Plans depend on nothing but the arguments, so they are kept: small problems are bound by
    the host side of a launch.  Callers must not modify the result."""
    key = (B, L, D, in_dtype, out_dtype, direction, align_elems, ckpt_stride, tune)
    plan = _plans.get(key)
    if plan is None:
        plan = Plan()
        lib = _lib.load()
        if tune:
            rc = lib.qssm_plan_scan_tuned(B, L, D, _DTYPE_CODE[in_dtype], _DTYPE_CODE[out_dtype], direction,
                                          align_elems, ckpt_stride, tune, ctypes.byref(plan))
        else:
            rc = lib.qssm_plan_scan(B, L, D, _DTYPE_CODE[in_dtype], _DTYPE_CODE[out_dtype], direction,
                                    align_elems, ckpt_stride, ctypes.byref(plan))
        _lib.check(rc)
        if len(_plans) >= 4096:
            _plans.clear()
        _plans[key] = plan
    return plan


class _Launch:
    """A ready-made argument block for one (direction, shape, storage, alignment, geometry): the plan, what the
    host needs from it as plain ints, and the ctypes block whose pointers a call patches."""

    __slots__ = ("plan", "call", "call_ref", "need_c", "need_w", "n_ckpt", "ckpt_stride", "strides")

    def __init__(self, plan: Plan, call):
        self.plan = plan
        self.call = call
        self.call_ref = ctypes.byref(call)
        call.plan = ctypes.pointer(plan)
        self.need_c = int(plan.control_bytes)
        self.need_w = int(plan.workspace_bytes)
        self.n_ckpt = int(plan.n_ckpt)
        self.ckpt_stride = int(plan.ckpt_stride)
        self.strides = None   # the stride tuples the block's stride fields were last filled from


_tls = threading.local()   # argument blocks are patched in place, so every thread keeps its own


def _launch_entry(key: tuple, make) -> _Launch:
    cache = getattr(_tls, "launches", None)
    if cache is None:
        cache = _tls.launches = {}
    entry = cache.get(key)
    if entry is None:
        if len(cache) >= 1024:
            cache.clear()
        entry = cache[key] = make()
    return entry


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


_NO_STRIDE = (0, 0, 0)


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
    dev = _require_gpu(x, a, b) if c is None else _require_gpu(x, a, b, c)
    B, L, D = x.shape
    in_dtype = x.dtype
    y = torch.empty((B, L, D), dtype=out_dtype, device=dev) if want_y else None
    h = torch.empty((B, L, D), dtype=torch.float32, device=dev) if want_h else None
    if h_init is not None or h_final is not None:
        _check_state(h_init, B, D, dev, "h_init")
        _check_state(h_final, B, D, dev, "h_final")
    if B == 0 or L == 0 or D == 0:
        if h_final is not None:  # nothing happened to the state
            h_final.copy_(h_init) if h_init is not None else h_final.zero_()
        return y, h, (torch.empty((B, 0, D), dtype=torch.float32, device=dev) if want_ckpt else None), 0

    (x, a, b, c), strides, ptrs, align = _describe((x, a, b, c), (y, h), L, D)

    # Operands are left in the caches only for a backward: a forward that saves no states has none coming.
    keep = _forward_keep if (want_ckpt or want_h) else False

    def make() -> _Launch:
        stride = 0
        if want_ckpt:
            # The backward decides how far apart the saved states may be; the forward follows.
            stride = make_plan(B, L, D, in_dtype, out_dtype, _lib.QSSM_BACKWARD, align, 0, bwd_tune).seg_len
        plan = make_plan(B, L, D, in_dtype, out_dtype, _lib.QSSM_FORWARD, align, stride, tune)
        if keep is not True:
            plan = Plan.from_buffer_copy(plan)   # cached plans are shared: change a copy
            plan.keep_tiles = 0 if keep is False else min(int(plan.keep_tiles), int(keep))
        return _Launch(plan, ForwardCall())

    entry = _launch_entry((0, B, L, D, in_dtype, out_dtype, align, want_ckpt, tune, bwd_tune, keep), make)
    ckpt = torch.empty((B, entry.n_ckpt, D), dtype=torch.float32, device=dev) if want_ckpt else None

    k = entry.call
    if entry.strides != strides:
        k.sx, k.sa, k.sb, k.sc, k.sy, k.sh = (Strides(s[0], s[1]) for s in strides)
        entry.strides = strides
    k.x, k.a, k.b, k.c, k.y, k.h_out = ptrs
    k.ckpt = None if ckpt is None else ckpt.data_ptr()
    k.h_init = None if h_init is None else h_init.data_ptr()
    k.h_final = None if h_final is None else h_final.data_ptr()

    index = dev.index
    if index == torch.cuda.current_device():
        _launch_on(index, dev, entry, _lib.load().qssm_scan_forward_call)
    else:
        with torch.cuda.device(dev):
            _launch_on(index, dev, entry, _lib.load().qssm_scan_forward_call)
    return y, h, ckpt, entry.ckpt_stride


def _launch_on(index: int, dev: torch.device, entry: _Launch, fn) -> None:
    """Fill in stream, buffers and epoch of a ready argument block and make the call (device `index` is current)."""
    stream = _raw_stream(index)
    buf, epoch, capturing = _launch_buffers(dev, index, stream, entry.need_c, entry.need_w)
    k = entry.call
    k.control, k.control_size, k.workspace, k.workspace_bytes = buf.ctl_ptr, buf.ctl_size, buf.ws_ptr, buf.ws_size
    k.epoch = epoch
    k.stream = stream
    rc = fn(entry.call_ref)
    if rc != 0:
        _lib.check(rc)
    _after_launch(buf, stream, capturing)


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
    if h_init is not None or dh_final is not None or dh_init is not None:
        for name, t in (("h_init", h_init), ("dh_final", dh_final), ("dh_init", dh_init)):
            _check_state(t, B, D, dev, name)
    if B == 0 or L == 0 or D == 0:
        if dh_init is not None:  # the state passed through untouched
            dh_init.copy_(dh_final) if dh_final is not None else dh_init.zero_()
        return tuple(grads)
    if (h is None) == (ckpt is None):
        raise ValueError("pass exactly one of h and ckpt")

    if h is not None:
        if h.dtype != torch.float32:
            h = h.float()
    elif not ckpt.is_contiguous():
        ckpt = ckpt.contiguous()
    (x, a, b, c, dy, h), strides, ptrs, align = _describe((x, a, b, c, dy, h), grads, L, D)
    stride_arg = ckpt_stride if h is None else 0
    out_dtype = dy.dtype

    def make() -> _Launch:
        return _Launch(make_plan(B, L, D, in_dtype, out_dtype, _lib.QSSM_BACKWARD, align, stride_arg, tune), BackwardCall())

    entry = _launch_entry((1, B, L, D, in_dtype, out_dtype, align, stride_arg, tune), make)
    if ckpt is not None and tuple(ckpt.shape) != (B, entry.n_ckpt, D):
        raise ValueError(f"ckpt has shape {tuple(ckpt.shape)}, expected {(B, entry.n_ckpt, D)}")

    k = entry.call
    if entry.strides != strides:
        (k.sx, k.sa, k.sb, k.sc, k.sdy, k.sh, k.sdx, k.sda, k.sdb, k.sdc) = (Strides(s[0], s[1]) for s in strides)
        entry.strides = strides
    k.x, k.a, k.b, k.c, k.dy, k.h, k.dx, k.da, k.db, k.dc = ptrs
    k.ckpt = None if ckpt is None else ckpt.data_ptr()
    k.h_init = None if h_init is None else h_init.data_ptr()
    k.dh_final = None if dh_final is None else dh_final.data_ptr()
    k.dh_init = None if dh_init is None else dh_init.data_ptr()

    index = dev.index
    if index == torch.cuda.current_device():
        _launch_on(index, dev, entry, _lib.load().qssm_scan_backward_call)
    else:
        with torch.cuda.device(dev):
            _launch_on(index, dev, entry, _lib.load().qssm_scan_backward_call)
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
