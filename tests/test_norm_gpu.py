"""GPU parity of the SSM layer's RMSNorm (quick_ssm_amd/csrc/rmsnorm.hip) through the C ABI.

Oracle: oracle/rmsnorm_oracle.py (float64) on the same stored inputs.  Tolerances: 1e-5 of the tensor's
largest magnitude for fp32 results, 1e-2 for fp16 / bf16 results (one rounding to the storage type);
dweight sums `rows` rounded products, so its fp32 tolerance carries a factor sqrt(rows).
"""
from __future__ import annotations

import ctypes

import numpy as np
import pytest
import torch

from helpers import TOL, assert_close
from oracle import rmsnorm_oracle
from quick_ssm_amd import _lib
from quick_ssm_amd.layers import RMSNorm
from quick_ssm_amd.norm import rms_norm, rms_norm_reference

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.float16, torch.bfloat16]
# H: one chunk, several chunks, the widest register-resident row, wider than that, odd widths (1 or 2 per lane)
SHAPES = [(2, 33, 64), (3, 50, 256), (4, 64, 1024), (2, 9, 4096), (1, 5, 8192), (3, 7, 37), (2, 5, 1030), (1, 1, 6),
          (2, 3, 5000), (1, 2, 3001)]


def _inputs(shape, dtype, seed):
    gen = torch.Generator().manual_seed(seed)
    x = (torch.randn(*shape, generator=gen) * 1.7 + 0.3).to(dtype)
    w = (torch.rand(shape[-1], generator=gen) + 0.5).to(dtype)
    dy = torch.randn(*shape, generator=gen).to(dtype)
    return x, w, dy


@pytest.mark.parametrize("dtype", DTYPES, ids=lambda d: str(d).replace("torch.", ""))
@pytest.mark.parametrize("shape", SHAPES, ids=lambda s: "x".join(map(str, s)))
def test_rms_norm_matches_oracle(gpu, dtype, shape):
    x, w, dy = _inputs(shape, dtype, seed=sum(shape))
    eps = 1e-5
    xg, wg = x.to(gpu).requires_grad_(True), w.to(gpu).requires_grad_(True)
    y = rms_norm(xg, wg, eps)
    assert y.dtype == dtype and y.shape == torch.Size(shape)
    assert_close("y", y.detach().cpu(), rmsnorm_oracle.rmsnorm_forward_f64(x, w, eps), TOL[dtype])
    y.backward(dy.to(gpu))
    dx, dw = rmsnorm_oracle.rmsnorm_backward_f64(dy, x, w, eps)
    rows = int(np.prod(shape[:-1]))
    assert xg.grad.dtype == dtype and wg.grad.dtype == dtype
    assert_close("dx", xg.grad.cpu(), dx, TOL[dtype])
    assert_close("dweight", wg.grad.cpu(), dw, TOL[dtype] * max(1.0, rows ** 0.5) if dtype == torch.float32 else TOL[dtype])


def test_rms_norm_many_rows_strided_input_and_repeatable_dweight(gpu):
    # more rows than one pass of the grid covers; x is a column slice of a wider tensor (row stride 3 H)
    rows, H = 9000, 512
    gen = torch.Generator().manual_seed(3)
    wide = torch.randn(rows, 3 * H, generator=gen).to(gpu)
    x = wide[:, H:2 * H].detach().requires_grad_(True)
    w = (torch.rand(H, generator=gen) + 0.5).to(gpu).requires_grad_(True)
    dy = torch.randn(rows, H, generator=gen).to(gpu)
    y = rms_norm(x, w, 1e-6)
    assert_close("y", y.detach().cpu(), rmsnorm_oracle.rmsnorm_forward_f64(x, w, 1e-6), 1e-5)
    y.backward(dy)
    dx, dw = rmsnorm_oracle.rmsnorm_backward_f64(dy, x, w, 1e-6)
    assert_close("dx", x.grad.cpu(), dx, 1e-5)
    assert_close("dweight", w.grad.cpu(), dw, 1e-5 * rows ** 0.5)
    first = w.grad.clone()
    for _ in range(3):
        x.grad = None
        w.grad = None
        rms_norm(x, w, 1e-6).backward(dy)
        assert torch.equal(w.grad, first)  # summed in a fixed order


def test_rms_norm_backward_without_saved_rstd_and_error_codes(gpu):
    rows, H = 37, 200
    x, w, dy = (t.to(gpu) for t in _inputs((rows, H), torch.float32, seed=8))
    lib = _lib.load()
    stream = torch.cuda.current_stream(gpu).cuda_stream
    dx = torch.empty_like(x)
    dw = torch.empty_like(w)
    partial = torch.empty(8, H, device=gpu)
    rc = lib.qssm_rmsnorm_backward(dy.data_ptr(), H, x.data_ptr(), H, w.data_ptr(), None, dx.data_ptr(), dw.data_ptr(),
                                   partial.data_ptr(), 8, rows, H, 1e-5, _lib.QSSM_F32, stream)
    assert rc == 0, _lib.load().qssm_error_string()
    rdx, rdw = rmsnorm_oracle.rmsnorm_backward_f64(dy, x, w, 1e-5)
    assert_close("dx", dx.cpu(), rdx, 1e-5)
    assert_close("dweight", dw.cpu(), rdw, 1e-5 * rows ** 0.5)
    # too little scratch, a row stride below H, an unknown storage code
    assert lib.qssm_rmsnorm_backward(dy.data_ptr(), H, x.data_ptr(), H, w.data_ptr(), None, dx.data_ptr(),
                                     dw.data_ptr(), partial.data_ptr(), 4, rows, H, 1e-5, _lib.QSSM_F32, stream) != 0
    y = torch.empty_like(x)
    assert lib.qssm_rmsnorm_forward(x.data_ptr(), H - 1, w.data_ptr(), y.data_ptr(), None, rows, H, 1e-5,
                                    _lib.QSSM_F32, stream) != 0
    assert lib.qssm_rmsnorm_forward(x.data_ptr(), H, w.data_ptr(), y.data_ptr(), None, rows, H, 1e-5, 77, stream) != 0
    # no rows: nothing to do forward; backward still defines dweight = 0
    assert lib.qssm_rmsnorm_forward(None, H, w.data_ptr(), None, None, 0, H, 1e-5, _lib.QSSM_F32, stream) == 0
    dw.fill_(5.0)
    assert lib.qssm_rmsnorm_backward(None, H, None, H, w.data_ptr(), None, None, dw.data_ptr(), partial.data_ptr(), 8,
                                     0, H, 1e-5, _lib.QSSM_F32, stream) == 0
    assert torch.count_nonzero(dw) == 0


def test_rmsnorm_module_mixed_storage_takes_the_reference_formula(gpu):
    # fp16 activations under an fp32 weight: torch promotes to fp32, as the reference does
    gen = torch.Generator().manual_seed(2)
    norm = RMSNorm(48, eps=1e-5, dtype=torch.float32, device=gpu)
    x = torch.randn(2, 5, 48, generator=gen).half().to(gpu)
    y = norm(x)
    assert y.dtype == torch.float32
    assert torch.equal(y, rms_norm_reference(x, norm.weight, 1e-5))
    with pytest.raises(ValueError):
        rms_norm(x, torch.ones(47, device=gpu))
