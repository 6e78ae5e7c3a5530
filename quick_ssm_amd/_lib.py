"""ctypes binding of libquick_ssm_hip.so (the C ABI declared in include/quick_ssm_hip.h).

The library is looked up next to this file.  It is never replaced by another implementation:
if it cannot be loaded, every device entry point raises.
"""
from __future__ import annotations

import ctypes
import os
import threading
from pathlib import Path
from typing import Optional

LIB_NAME = "libquick_ssm_hip.so"
LIB_PATH = Path(__file__).resolve().parent / LIB_NAME

# The QSSM_VERSION of include/quick_ssm_hip.h this binding was written against (same minor version = same ABI).
QSSM_VERSION = 200
QSSM_F32, QSSM_F16, QSSM_BF16 = 0, 1, 2
QSSM_FORWARD, QSSM_BACKWARD = 0, 1
QSSM_RMSNORM_MIN_PARTIAL_ROWS = 8
QSSM_STATIC_SCRATCH_BYTES = 32 << 20
QSSM_EINVAL, QSSM_EALIGN, QSSM_EWORKSPACE, QSSM_ESTATE = -1, -2, -3, -4

EXPORTED_SYMBOLS = (
    "qssm_version",
    "qssm_error_string",
    "qssm_plan_scan",
    "qssm_plan_scan_tuned",
    "qssm_zero_fill",
    "qssm_control_status",
    "qssm_control_status_async",
    "qssm_scan_forward",
    "qssm_scan_backward",
    "qssm_scan_forward_carry",
    "qssm_scan_backward_carry",
    "qssm_scan_forward_static",
    "qssm_scan_forward_call",
    "qssm_scan_backward_call",
    "qssm_plan_scan_gated",
    "qssm_scan_gated_forward",
    "qssm_scan_gated_backward",
    "qssm_gates_forward",
    "qssm_gates_backward",
    "qssm_gates_backward_strided",
    "qssm_rmsnorm_forward",
    "qssm_rmsnorm_backward",
    "qssm_colsum",
    "qssm_copy_bytes",
    "qssm_launch_count_step",
)


class Plan(ctypes.Structure):
    """Mirror of `qssm_plan`."""

    _fields_ = [
        ("B", ctypes.c_int32),
        ("L", ctypes.c_int32),
        ("D", ctypes.c_int32),
        ("in_dtype", ctypes.c_int32),
        ("out_dtype", ctypes.c_int32),
        ("direction", ctypes.c_int32),
        ("vec", ctypes.c_int32),
        ("steps", ctypes.c_int32),
        ("threads", ctypes.c_int32),
        ("g_log2", ctypes.c_int32),
        ("strip_cols", ctypes.c_int32),
        ("seg_len", ctypes.c_int32),
        ("n_strips", ctypes.c_int32),
        ("n_seg", ctypes.c_int32),
        ("cluster", ctypes.c_int32),
        ("n_super", ctypes.c_int32),
        ("ckpt_stride", ctypes.c_int32),
        ("n_ckpt", ctypes.c_int32),
        ("lds_bytes", ctypes.c_int32),
        ("keep_tiles", ctypes.c_int32),
        ("compute_dtype", ctypes.c_int32),
        ("control_bytes", ctypes.c_uint64),
        ("workspace_bytes", ctypes.c_uint64),
        ("ckpt_elems", ctypes.c_uint64),
    ]

    def describe(self) -> dict:
        return {name: int(getattr(self, name)) for name, _ in self._fields_}


class Strides(ctypes.Structure):
    """Mirror of `qssm_strides` (element strides of the batch and time axes)."""

    _fields_ = [("b", ctypes.c_int64), ("l", ctypes.c_int64)]


class ForwardCall(ctypes.Structure):
    """Mirror of `qssm_forward_call`."""

    _fields_ = (
        [("plan", ctypes.POINTER(Plan))]
        + [(n, ctypes.c_void_p) for n in ("x", "a", "b", "c", "y", "h_out", "ckpt", "h_init", "h_final")]
        + [(n, Strides) for n in ("sx", "sa", "sb", "sc", "sy", "sh")]
        + [("control", ctypes.c_void_p), ("control_size", ctypes.c_uint64), ("workspace", ctypes.c_void_p),
           ("workspace_bytes", ctypes.c_uint64), ("epoch", ctypes.c_uint32), ("reserved", ctypes.c_uint32),
           ("stream", ctypes.c_void_p)]
    )


class BackwardCall(ctypes.Structure):
    """Mirror of `qssm_backward_call`."""

    _fields_ = (
        [("plan", ctypes.POINTER(Plan))]
        + [(n, ctypes.c_void_p) for n in ("x", "a", "b", "c", "dy", "h", "ckpt", "h_init", "dh_final", "dh_init",
                                          "dx", "da", "db", "dc")]
        + [(n, Strides) for n in ("sx", "sa", "sb", "sc", "sdy", "sh", "sdx", "sda", "sdb", "sdc")]
        + [("control", ctypes.c_void_p), ("control_size", ctypes.c_uint64), ("workspace", ctypes.c_void_p),
           ("workspace_bytes", ctypes.c_uint64), ("epoch", ctypes.c_uint32), ("reserved", ctypes.c_uint32),
           ("stream", ctypes.c_void_p)]
    )


class QssmError(RuntimeError):
    def __init__(self, code: int, message: str):
        super().__init__(f"libquick_ssm_hip: {message} (code {code})")
        self.code = code


_lock = threading.Lock()
_lib: Optional[ctypes.CDLL] = None


def _declare(lib: ctypes.CDLL) -> None:
    vp, u64, i32 = ctypes.c_void_p, ctypes.c_uint64, ctypes.c_int32
    lib.qssm_version.restype = ctypes.c_int
    lib.qssm_version.argtypes = []
    lib.qssm_error_string.restype = ctypes.c_char_p
    lib.qssm_error_string.argtypes = []
    lib.qssm_plan_scan.restype = ctypes.c_int
    lib.qssm_plan_scan.argtypes = [i32] * 8 + [ctypes.POINTER(Plan)]
    lib.qssm_plan_scan_tuned.restype = ctypes.c_int
    lib.qssm_plan_scan_tuned.argtypes = [i32] * 9 + [ctypes.POINTER(Plan)]
    lib.qssm_control_status_async.restype = ctypes.c_int
    lib.qssm_control_status_async.argtypes = [vp, vp, vp]
    lib.qssm_scan_forward_call.restype = ctypes.c_int
    lib.qssm_scan_forward_call.argtypes = [vp]
    lib.qssm_scan_backward_call.restype = ctypes.c_int
    lib.qssm_scan_backward_call.argtypes = [vp]
    lib.qssm_zero_fill.restype = ctypes.c_int
    lib.qssm_zero_fill.argtypes = [vp, u64, vp]
    lib.qssm_control_status.restype = ctypes.c_int
    lib.qssm_control_status.argtypes = [vp, vp, ctypes.POINTER(i32)]
    lib.qssm_scan_forward.restype = ctypes.c_int
    lib.qssm_scan_forward.argtypes = (
        [ctypes.POINTER(Plan)] + [vp, Strides] * 6 + [vp] + [vp, u64, vp, u64, ctypes.c_uint32, vp]
    )
    lib.qssm_scan_forward_static.restype = ctypes.c_int
    lib.qssm_scan_forward_static.argtypes = [ctypes.POINTER(Plan)] + [vp, Strides] * 6 + [vp] + [vp]
    lib.qssm_scan_backward.restype = ctypes.c_int
    lib.qssm_scan_backward.argtypes = (
        [ctypes.POINTER(Plan)] + [vp, Strides] * 6 + [vp] + [vp, Strides] * 4 + [vp, u64, vp, u64, ctypes.c_uint32, vp]
    )
    lib.qssm_scan_forward_carry.restype = ctypes.c_int
    lib.qssm_scan_forward_carry.argtypes = (
        [ctypes.POINTER(Plan)] + [vp, Strides] * 6 + [vp] + [vp, vp] + [vp, u64, vp, u64, ctypes.c_uint32, vp]
    )
    lib.qssm_scan_backward_carry.restype = ctypes.c_int
    lib.qssm_scan_backward_carry.argtypes = (
        [ctypes.POINTER(Plan)] + [vp, Strides] * 6 + [vp] + [vp, vp, vp] + [vp, Strides] * 4
        + [vp, u64, vp, u64, ctypes.c_uint32, vp]
    )
    lib.qssm_plan_scan_gated.restype = ctypes.c_int
    lib.qssm_plan_scan_gated.argtypes = [i32] * 9 + [ctypes.POINTER(Plan)]
    lib.qssm_scan_gated_forward.restype = ctypes.c_int
    lib.qssm_scan_gated_forward.argtypes = (
        [ctypes.POINTER(Plan)] + [vp, Strides] * 6 + [vp] + [vp, u64, vp, u64, ctypes.c_uint32, vp]
    )
    lib.qssm_scan_gated_backward.restype = ctypes.c_int
    lib.qssm_scan_gated_backward.argtypes = (
        [ctypes.POINTER(Plan)] + [vp, Strides] * 6 + [vp] + [vp, Strides] * 5 + [vp, u64, vp, u64, ctypes.c_uint32, vp]
    )
    i64 = ctypes.c_int64
    lib.qssm_gates_forward.restype = ctypes.c_int
    lib.qssm_gates_forward.argtypes = [vp, i64] * 5 + [vp] * 4 + [i64, i32, i32, i32, vp]
    lib.qssm_gates_backward.restype = ctypes.c_int
    lib.qssm_gates_backward.argtypes = [vp] * 4 + [vp, i64] * 4 + [vp] * 5 + [i64, i32, i32, i32, vp]
    lib.qssm_gates_backward_strided.restype = ctypes.c_int
    lib.qssm_gates_backward_strided.argtypes = [vp] * 4 + [vp, i64] * 4 + [vp] * 5 + [i64, i64, i32, i32, i32, vp]
    lib.qssm_rmsnorm_forward.restype = ctypes.c_int
    lib.qssm_rmsnorm_forward.argtypes = [vp, i64, vp, vp, vp, i64, i32, ctypes.c_float, i32, vp]
    lib.qssm_rmsnorm_backward.restype = ctypes.c_int
    lib.qssm_rmsnorm_backward.argtypes = [vp, i64, vp, i64, vp, vp, vp, vp, vp, i32, i64, i32, ctypes.c_float, i32, vp]
    lib.qssm_colsum.restype = ctypes.c_int
    lib.qssm_colsum.argtypes = [vp, i64, i64, i32, i32, vp, i32, vp, vp]
    lib.qssm_copy_bytes.restype = ctypes.c_int
    lib.qssm_copy_bytes.argtypes = [vp, vp, u64, vp]
    lib.qssm_launch_count_step.restype = ctypes.c_int
    lib.qssm_launch_count_step.argtypes = [ctypes.c_uint32, i32, ctypes.POINTER(ctypes.c_uint32),
                                           ctypes.POINTER(ctypes.c_uint32), ctypes.POINTER(i32)]


def is_built() -> bool:
    return LIB_PATH.exists()


def load() -> ctypes.CDLL:
    """Load the shared library (once).  Raises RuntimeError if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is None:
            if not LIB_PATH.exists():
                raise RuntimeError(
                    f"{LIB_PATH} is missing: the HIP scan kernels are not built. "
                    "Run `python -m quick_ssm_amd.build` (needs hipcc). There is no other device path."
                )
            lib = ctypes.CDLL(os.fspath(LIB_PATH))
            lib.qssm_version.restype = ctypes.c_int
            built = int(lib.qssm_version())
            if built // 100 != QSSM_VERSION // 100:
                raise RuntimeError(
                    f"{LIB_PATH} was built from version {built} of the C ABI, this package binds version "
                    f"{QSSM_VERSION}: the argument lists differ. Rebuild with `python -m quick_ssm_amd.build`.")
            _declare(lib)
            _lib = lib
    return _lib


class launch_stream:
    """`with launch_stream(device) as stream:` makes `device` current if it is not already (the common case costs
    two cheap calls instead of a device context and a Stream object) and yields the raw handle of its current
    stream, which is what the library's entry points take."""

    __slots__ = ("device", "guard")

    def __init__(self, device):
        self.device = device
        self.guard = None

    def __enter__(self) -> int:
        import torch

        index = self.device.index
        if index is None:
            index = torch.cuda.current_device()
        elif index != torch.cuda.current_device():
            self.guard = torch.cuda.device(self.device)
            self.guard.__enter__()
        return torch._C._cuda_getCurrentRawStream(index)

    def __exit__(self, *exc):
        if self.guard is not None:
            self.guard.__exit__(*exc)
        return False


def check(code: int) -> None:
    """Raise QssmError for a nonzero return code of a library call."""
    if code != 0:
        message = load().qssm_error_string().decode("utf-8", "replace")
        raise QssmError(code, message or "call failed")
