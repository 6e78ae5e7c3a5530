"""GPU parity of qssm_colsum (through the C ABI): the bias gradients of the layer's linear maps.

Oracle: numpy's float64 sum over the rows of the stored values (a library routine).  Bar: 1e-5 of the largest
column sum for fp32 storage, 1e-2 for 16-bit storage (the result is rounded once to the storage type).
"""
from __future__ import annotations

import numpy as np
import pytest
import torch

from helpers import TOL, assert_close
from quick_ssm_amd.layers import _LinearBias, column_sum

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16], ids=["f32", "f16", "bf16"])
@pytest.mark.parametrize("rows,S", [(4096, 1024), (4096, 256), (1000, 100), (1, 7), (63, 130), (70000, 64), (5, 2048)])
def test_column_sums_match_float64(gpu, dtype, rows, S):
    g = torch.Generator().manual_seed(rows + S)
    x = (torch.randn(rows, S, generator=g) + 0.25).to(dtype)
    want = x.double().numpy().sum(axis=0)
    got = column_sum(x.to(gpu))
    assert got.dtype == dtype and got.shape == (S,)
    assert_close("colsum", got, want, TOL[dtype])
    again = column_sum(x.to(gpu))
    assert torch.equal(got, again)                        # fixed summation order


def test_column_sums_of_a_block_of_a_wider_matrix(gpu):
    # A_proj's bias gradient is summed over the first S columns of the wide [rows, 5 S] gradient, in place
    rows, S = 4096, 1024
    wide = torch.randn(rows, 5 * S, generator=torch.Generator().manual_seed(3)).to(gpu)
    for k in (0, 3):
        block = wide[:, k * S:(k + 1) * S]
        assert_close("colsum", column_sum(block), block.double().sum(0).cpu().numpy(), 1e-5)
    odd = wide[:, 3:3 + 1001]                             # rows that start off 16 bytes: one column per lane
    assert_close("colsum", column_sum(odd), odd.double().sum(0).cpu().numpy(), 1e-5)


def test_linear_with_bias_matches_torch(gpu):
    torch.manual_seed(0)
    lin = torch.nn.Linear(96, 40).to(gpu)
    u = torch.randn(3, 50, 96, device=gpu, requires_grad=True)
    g = torch.randn(3, 50, 40, device=gpu)
    out = _LinearBias.apply(u, lin.weight, lin.bias)
    ref = lin(u)
    assert torch.equal(out, ref)
    got = torch.autograd.grad(out, [u, lin.weight, lin.bias], g)
    want = torch.autograd.grad(ref, [u, lin.weight, lin.bias], g)
    for a, b, n in zip(got, want, ("du", "dw", "db")):
        assert_close(n, a, b.double().cpu().numpy(), 1e-5)
