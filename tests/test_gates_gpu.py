"""GPU parity of the SSM layer's gate prologue (quick_ssm_amd/csrc/gates.hip) through the C ABI.

Oracle: oracle/gates_oracle.py (float64) on the same stored inputs.  Tolerances: 1e-5 of the tensor's
largest magnitude for fp32 results, 1e-2 for fp16 / bf16 results (one rounding to the storage type).
"""
from __future__ import annotations

import numpy as np
import pytest
import torch

from helpers import TOL, assert_close
from oracle import gates_oracle
from quick_ssm_amd.gates import gate_prologue, gate_prologue_wide, gates_reference

pytestmark = pytest.mark.gpu

PAIRS = [
    (torch.float32, torch.float32), (torch.float32, torch.float16), (torch.float32, torch.bfloat16),
    (torch.float16, torch.float16), (torch.float16, torch.float32),
    (torch.bfloat16, torch.bfloat16), (torch.bfloat16, torch.float32),
]


def _inputs(shape, dtype, seed):
    gen = torch.Generator().manual_seed(seed)
    return [(torch.randn(*shape, generator=gen) * 2.5).to(dtype) for _ in range(5)]


@pytest.mark.parametrize("in_dtype,out_dtype", PAIRS, ids=lambda d: str(d).replace("torch.", ""))
@pytest.mark.parametrize("shape", [(2, 33, 64), (3, 5, 7), (1, 1, 6), (4, 128, 1024)], ids=lambda s: "x".join(map(str, s)))
def test_gate_prologue_matches_oracle(gpu, in_dtype, out_dtype, shape):
    z = _inputs(shape, in_dtype, seed=sum(shape))
    gen = torch.Generator().manual_seed(99)
    g = [torch.randn(*shape, generator=gen).to(out_dtype) for _ in range(4)]
    leaves = [t.to(gpu).requires_grad_(True) for t in z]
    outs = gate_prologue(*leaves, out_dtype)
    assert all(o.dtype == out_dtype and o.shape == torch.Size(shape) for o in outs)
    ref = gates_oracle.gates_forward_f64(*z)
    for name, got, want in zip("axcb", outs, ref):
        assert_close(name, got.detach().cpu(), want, TOL[out_dtype])
    torch.autograd.backward(outs, [t.to(gpu) for t in g])
    gref = gates_oracle.gates_backward_f64(*g, z[0], z[2], z[3], z[4])
    for name, leaf, want in zip(("dA_pre", "dB_in", "dCa", "dCb", "dD_pre"), leaves, gref):
        assert leaf.grad.dtype == in_dtype
        assert_close(name, leaf.grad.cpu(), want, TOL[in_dtype])


def test_gate_prologue_on_column_slices_of_one_wide_tensor_and_partial_gradients(gpu):
    # the five projections as slices of one [rows, 5 S] GEMM output (row stride 5 S), S odd -> one element per lane
    B, L, S = 2, 50, 37
    gen = torch.Generator().manual_seed(5)
    wide = (torch.randn(B, L, 5 * S, generator=gen) * 2).to(gpu).requires_grad_(True)
    parts = [wide[..., k * S:(k + 1) * S] for k in range(5)]
    a, x, c, b = gate_prologue(*parts, torch.float16)
    z = [p.detach().cpu() for p in parts]
    ref = gates_oracle.gates_forward_f64(*z)
    for name, got, want in zip("axcb", (a, x, c, b), ref):
        assert_close(name, got.detach().cpu(), want, TOL[torch.float16])
    # only a and c feed the loss: the other gradients are zero, dB_in and dD_pre vanish
    w = torch.randn(B, L, S, generator=gen).to(gpu)
    ((a.float() * w).sum() + (c.float() * w).sum()).backward()
    zero = np.zeros((B, L, S))
    gref = gates_oracle.gates_backward_f64(w.half().cpu(), zero, w.half().cpu(), zero, z[0], z[2], z[3], z[4])
    got = wide.grad.cpu()
    for k, name in enumerate(("dA_pre", "dB_in", "dCa", "dCb", "dD_pre")):
        piece = got[..., k * S:(k + 1) * S]
        if np.abs(gref[k]).max() == 0:
            assert torch.count_nonzero(piece) == 0, name
        else:
            assert_close(name, piece, gref[k], 1e-5)


def test_gate_prologue_saturates_and_falls_back_for_unbuilt_pairs(gpu):
    z = [torch.tensor([[-200.0, -20.0, 0.0, 20.0, 200.0, 3.0e38, -3.0e38, 1.0]], device=gpu) for _ in range(5)]
    a, x, c, b = gate_prologue(*z, torch.float32)
    assert torch.isfinite(a).all() and torch.isfinite(b).all()
    assert a[0, 0] == 0 and a[0, 4] == 1 and c[0, 0] == 0 and c[0, 6] == 0
    # fp16 projections with bf16 operands: not a built pair, same formulas through torch
    zh = _inputs((2, 9, 8), torch.float16, seed=1)
    got = gate_prologue(*[t.to(gpu) for t in zh], torch.bfloat16)
    want = gates_reference(*[t.to(gpu) for t in zh], torch.bfloat16)
    for g_, w_ in zip(got, want):
        assert torch.equal(g_, w_)
    with pytest.raises(ValueError):
        gate_prologue(z[0], z[1], z[2], z[3], z[4][:, :4], torch.float32)


@pytest.mark.parametrize("in_dtype,out_dtype", [(torch.float32, torch.float16), (torch.bfloat16, torch.bfloat16),
                                                (torch.float32, torch.float32)], ids=lambda d: str(d).replace("torch.", ""))
@pytest.mark.parametrize("shape", [(2, 33, 64), (3, 5, 7), (4, 128, 256)], ids=lambda s: "x".join(map(str, s)))
def test_wide_prologue_equals_the_prologue_on_its_blocks(gpu, in_dtype, out_dtype, shape):
    # one [.., 5 S] tensor (a single GEMM's output): blocks read in place, gradients written as blocks of one wide
    # gradient (qssm_gates_backward_strided); same kernels, so the same bits as five separate tensors
    z = _inputs(shape, in_dtype, seed=7 + sum(shape))
    gen = torch.Generator().manual_seed(5)
    g = [torch.randn(*shape, generator=gen).to(out_dtype).to(gpu) for _ in range(4)]
    leaves = [t.to(gpu).requires_grad_(True) for t in z]
    outs = gate_prologue(*leaves, out_dtype)
    torch.autograd.backward(outs, g)
    wide = torch.cat(z, dim=-1).to(gpu).requires_grad_(True)
    outs_w = gate_prologue_wide(wide, out_dtype)
    torch.autograd.backward(outs_w, g)
    S = shape[-1]
    for a, b in zip(outs, outs_w):
        assert torch.equal(a, b)
    assert wide.grad.shape == wide.shape
    for k, leaf in enumerate(leaves):
        assert torch.equal(wide.grad[..., k * S:(k + 1) * S], leaf.grad)
    ref = gates_oracle.gates_forward_f64(*z)
    for name, got, want in zip("axcb", outs_w, ref):
        assert_close(name, got.detach().cpu(), want, TOL[out_dtype])
