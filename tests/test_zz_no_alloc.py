"""The forward entry point that allocates nothing (`qssm_scan_forward_static`), through the C ABI.

Its control block and workspace live in an array inside the library's device image, so its results must be
those of `qssm_scan_forward` with caller-owned buffers for the same plan: bit for bit, both being the same
kernels on the same geometry.  Two calls in a row share the array, the second with a smaller input and another
geometry, so words of the first call are still lying in the array when the second runs.
"""
import ctypes

import pytest
import torch

from helpers import TOL, assert_close, make_inputs
from quick_ssm_amd import _lib, hip_scan
from quick_ssm_amd._lib import Plan, Strides

pytestmark = pytest.mark.gpu


def _st(t):
    return Strides(t.stride(0), t.stride(1))


def _forward_both_ways(lib, gpu, shape, dtype, seed):
    """(y, ckpt) from qssm_scan_forward with buffers of the caller, and from qssm_scan_forward_static."""
    import oracle

    x, a, b, c, _ = make_inputs(shape, dtype=dtype, seed=seed)
    B, L, D = shape
    code = {torch.float32: _lib.QSSM_F32, torch.float16: _lib.QSSM_F16, torch.bfloat16: _lib.QSSM_BF16}[dtype]
    stride = hip_scan.make_plan(B, L, D, dtype, dtype, _lib.QSSM_BACKWARD, 8, 0).seg_len
    plan = Plan()
    assert lib.qssm_plan_scan(B, L, D, code, code, _lib.QSSM_FORWARD, 8, stride, ctypes.byref(plan)) == 0
    xd, ad, bd, cd = (t.to(gpu) for t in (x, a, b, c))
    stream = torch.cuda.current_stream(gpu).cuda_stream
    none = Strides(0, 0)

    y0 = torch.empty(shape, dtype=dtype, device=gpu)
    k0 = torch.empty((B, plan.n_ckpt, D), dtype=torch.float32, device=gpu)
    ctl = torch.zeros(max(int(plan.control_bytes), 64), dtype=torch.uint8, device=gpu)
    ws = torch.zeros(max(int(plan.workspace_bytes), 256), dtype=torch.uint8, device=gpu)
    rc = lib.qssm_scan_forward(ctypes.byref(plan), xd.data_ptr(), _st(xd), ad.data_ptr(), _st(ad), bd.data_ptr(),
                               _st(bd), cd.data_ptr(), _st(cd), y0.data_ptr(), _st(y0), None, none, k0.data_ptr(),
                               ctl.data_ptr(), ctl.numel(), ws.data_ptr(), ws.numel(), 1, stream)
    assert rc == 0, lib.qssm_error_string()
    out = ctypes.c_int32(-1)
    assert lib.qssm_control_status(ctl.data_ptr(), stream, ctypes.byref(out)) == 0 and out.value == 0

    y1 = torch.full(shape, float("nan"), dtype=dtype, device=gpu)
    k1 = torch.full((B, plan.n_ckpt, D), float("nan"), dtype=torch.float32, device=gpu)
    rc = lib.qssm_scan_forward_static(ctypes.byref(plan), xd.data_ptr(), _st(xd), ad.data_ptr(), _st(ad),
                                      bd.data_ptr(), _st(bd), cd.data_ptr(), _st(cd), y1.data_ptr(), _st(y1),
                                      None, none, k1.data_ptr(), stream)
    assert rc == 0, lib.qssm_error_string()
    torch.cuda.synchronize()
    _, y_ref = oracle.forward_f64(x, a, b, c)
    assert_close("y of the static entry point against the oracle", y1.cpu(), y_ref, TOL[dtype])
    return plan, (y0, k0), (y1, k1)


def test_static_entry_point_equals_the_caller_buffer_one_twice_in_a_row(gpu, hip_lib):
    lib = hip_lib
    # several clusters per chain; then a smaller input with narrower strips and a ragged last tile
    first = _forward_both_ways(lib, gpu, (2, 2048, 512), torch.bfloat16, seed=11)
    second = _forward_both_ways(lib, gpu, (1, 300, 264), torch.bfloat16, seed=12)
    for plan, (y0, k0), (y1, k1) in (first, second):
        assert plan.n_seg > 1 and plan.workspace_bytes > 0      # the scratch array is really in use
        assert torch.equal(y0, y1)
        assert torch.equal(k0, k1)
    # the same call again: the array now holds this very geometry's words from one launch earlier
    again = _forward_both_ways(lib, gpu, (1, 300, 264), torch.bfloat16, seed=12)
    assert torch.equal(again[1][0], again[2][0]) and torch.equal(second[2][0], again[2][0])


def test_static_entry_point_over_a_seeded_run_of_shapes(gpu, hip_lib):
    # 25 calls in a row with changing shapes, storage and geometry, all through the one scratch array: each equals
    # the caller-buffer entry point bit for bit (and meets the oracle, inside the helper)
    import numpy as np

    rng = np.random.default_rng(606)
    dtypes = (torch.bfloat16, torch.float32, torch.float16)
    for case in range(25):
        dtype = dtypes[case % 3]
        B = int(rng.integers(1, 4))
        L = int(rng.choice([int(rng.integers(1, 100)), int(rng.integers(100, 1200)), int(rng.integers(1200, 4000))]))
        D = 8 * int(rng.choice([int(rng.integers(1, 12)), int(rng.integers(12, 70)), 32 * int(rng.integers(1, 3))]))
        print(f"case static {case} shape=({B}, {L}, {D}) {dtype}", flush=True)
        plan, (y0, k0), (y1, k1) = _forward_both_ways(hip_lib, gpu, (B, L, D), dtype, seed=200 + case)
        assert torch.equal(y0, y1) and torch.equal(k0, k1), (case, (B, L, D), dtype)


def test_static_entry_point_refuses_what_does_not_fit(gpu, hip_lib):
    lib = hip_lib
    B, L, D = 64, 8192, 4096     # 8.6 G elements' worth of tiles: far more workspace than the array holds
    plan = Plan()
    assert lib.qssm_plan_scan(B, L, D, _lib.QSSM_BF16, _lib.QSSM_BF16, _lib.QSSM_FORWARD, 8, 32,
                              ctypes.byref(plan)) == 0
    assert plan.workspace_bytes > _lib.QSSM_STATIC_SCRATCH_BYTES
    t = torch.zeros(8, dtype=torch.bfloat16, device=gpu)     # never touched: the call is refused first
    s = Strides(L * D, D)
    rc = lib.qssm_scan_forward_static(ctypes.byref(plan), t.data_ptr(), s, t.data_ptr(), s, t.data_ptr(), s,
                                      t.data_ptr(), s, t.data_ptr(), s, None, Strides(0, 0), None,
                                      torch.cuda.current_stream(gpu).cuda_stream)
    assert rc == _lib.QSSM_EWORKSPACE
    assert b"scratch array" in lib.qssm_error_string()
