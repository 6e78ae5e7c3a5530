"""Shared input generators and comparison bars for the tests."""
from __future__ import annotations

import numpy as np
import torch

import oracle

# Tolerances of the parity bar: max|got - ref| / max|ref| per tensor, against the float64 oracle
# evaluated on the same stored (dtype-rounded) inputs.
TOL = {torch.float32: 1e-5, torch.float16: 1e-2, torch.bfloat16: 1e-2}


def make_inputs(shape, dtype=torch.float32, seed=0, a_lo=0.9, a_span=0.1, out_dtype=None, unit_bc=False):
    """Seeded operands with the reference's distributions, generated on the CPU in fp32 and cast.

    x ~ N(0,1); a = U(0,1)*a_span + a_lo; b = N(0,1)*0.1; c = sigmoid(N(0,1)); dy ~ N(0,1) in
    out_dtype (quick_ssm/test_forwards.py:51-53, README usage).  With unit_bc, b and c are N(0,1)
    as in quick_ssm/test_backwards.py:50-53.
    """
    g = torch.Generator(device="cpu").manual_seed(seed)
    x = torch.randn(shape, generator=g)
    a = torch.rand(shape, generator=g) * a_span + a_lo
    if unit_bc:
        b = torch.randn(shape, generator=g)
        c = torch.randn(shape, generator=g)
    else:
        b = torch.randn(shape, generator=g) * 0.1
        c = torch.sigmoid(torch.randn(shape, generator=g))
    dy = torch.randn(shape, generator=g)
    out_dtype = out_dtype or dtype
    return x.to(dtype), a.to(dtype), b.to(dtype), c.to(dtype), dy.to(out_dtype)


def oracle_all(x, a, b, c, dy):
    """float64 y and gradients from the oracle, on the stored values of the operands."""
    _, y = oracle.forward_f64(x, a, b, c)
    dx, da, db, dc = oracle.backward_f64(x, a, b, c, dy)
    return {"y": y, "dx": dx, "da": da, "db": db, "dc": dc}


def assert_close(name, got, ref, tol, report=None):
    rep = oracle.error_report(got, ref)
    if report is not None:
        report[name] = rep
    assert np.isfinite(rep["scaled"]), f"{name}: non-finite error"
    assert rep["scaled"] <= tol, f"{name}: max|d|/max|ref| = {rep['scaled']:.3e} > {tol:.1e} ({rep})"


def run_scan_with_grads(scan_fn, x, a, b, c, dy, device, **kw):
    """y and grads of sum(y*dy) through `scan_fn` on `device`; results as CPU tensors."""
    leaves = [t.detach().to(device).clone().requires_grad_(True) for t in (x, a, b, c)]
    y = scan_fn(*leaves, **kw)
    y.backward(dy.to(device=device, dtype=y.dtype))
    out = {"y": y.detach().cpu()}
    for name, t in zip(("dx", "da", "db", "dc"), leaves):
        out[name] = t.grad.detach().cpu()
    return out
