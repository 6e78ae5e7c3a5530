"""Pins the CPU oracle (oracle/) before anything is compared with it.

Checks chosen so that a dropped term, a wrong sign or index, or a transposed operand fails one:
exact rational vectors from the scan's definition as an explicit sum (tests/golden), closed forms,
finite differences, structural invariants, and agreement between the independently written C and
torch flavours.  None of these retypes the oracle's recurrence.
"""
import json
from pathlib import Path

import numpy as np
import pytest
import torch

import oracle
from oracle.reference_cpu_path import reference_forward_states, reference_scan, reference_scan_with_grads
from helpers import make_inputs, oracle_all

GOLDEN = json.loads((Path(__file__).parent / "golden" / "exact_scan_vectors.json").read_text())


@pytest.mark.parametrize("case", GOLDEN["cases"], ids=lambda c: c["name"])
def test_oracle_matches_exact_rational_vectors(case):
    ops = [np.array(case[k], dtype=np.float32) for k in ("x", "a", "b", "c", "dy")]
    for k, arr in zip(("x", "a", "b", "c", "dy"), ops):  # inputs are exactly representable
        assert np.array_equal(arr.astype(np.float64), np.array(case[k]))
    x, a, b, c, dy = ops
    h, y = oracle.forward_f64(x, a, b, c)
    grads = dict(zip(("dx", "da", "db", "dc"), oracle.backward_f64(x, a, b, c, dy)))
    np.testing.assert_allclose(h, np.array(case["h"]), rtol=1e-14, atol=1e-14)
    np.testing.assert_allclose(y, np.array(case["y"]), rtol=1e-14, atol=1e-14)
    for k, g in grads.items():
        np.testing.assert_allclose(g, np.array(case[k]), rtol=1e-13, atol=1e-13, err_msg=k)


@pytest.mark.parametrize("case", GOLDEN["cases"], ids=lambda c: c["name"])
def test_torch_restatement_matches_exact_rational_vectors(case):
    x, a, b, c, dy = (torch.tensor(case[k], dtype=torch.float64) for k in ("x", "a", "b", "c", "dy"))
    y, dx, da, db, dc = reference_scan_with_grads(x, a, b, c, dy)
    for k, got in (("y", y), ("dx", dx), ("da", da), ("db", db), ("dc", dc)):
        np.testing.assert_allclose(got.numpy(), np.array(case[k]), rtol=1e-13, atol=1e-13, err_msg=k)


def test_closed_form_geometric_decay():
    # x = delta(t=0), b = 1, a = g  =>  h(t) = g^t  (the reference's precision test, forward_only.py:592-600,
    # at a length where g^L stays a normal number)
    L, g = 4096, 0.999
    x = np.zeros((1, L, 2), np.float32)
    x[:, 0] = 1.0
    a = np.full_like(x, g)
    b = np.ones_like(x)
    h, _ = oracle.forward_f64(x, a, b)
    expect = np.float64(np.float32(g)) ** np.arange(L)
    np.testing.assert_allclose(h[0, :, 0], expect, rtol=1e-12)


def test_closed_forms_cumsum_and_memoryless_and_geometric_sum():
    rng = np.random.default_rng(0)
    x = rng.standard_normal((2, 300, 3)).astype(np.float32)
    b = rng.standard_normal((2, 300, 3)).astype(np.float32)
    ones, zeros = np.ones_like(x), np.zeros_like(x)
    h, _ = oracle.forward_f64(x, ones, b)                      # a = 1: running sum of b*x
    np.testing.assert_allclose(h, np.cumsum(b.astype(np.float64) * x, axis=1), rtol=1e-12, atol=1e-12)
    h, _ = oracle.forward_f64(x, zeros, b)                     # a = 0: no memory
    np.testing.assert_allclose(h, b.astype(np.float64) * x, rtol=0, atol=0)
    g = np.float32(0.75)
    h, _ = oracle.forward_f64(ones, np.full_like(x, g), ones)  # a = g, b*x = 1: (1 - g^(t+1)) / (1 - g)
    t = np.arange(300)
    np.testing.assert_allclose(h[1, :, 2], (1 - np.float64(g) ** (t + 1)) / (1 - np.float64(g)), rtol=1e-13)


def test_gradients_match_finite_differences():
    x, a, b, c, dy = (t.double().numpy() for t in make_inputs((1, 7, 2), seed=5))
    f32 = [t.astype(np.float32) for t in (x, a, b, c, dy)]
    grads = oracle.backward_f64(*f32)

    def loss(ops):
        _, y = oracle.forward_f64(ops[0], ops[1], ops[2], ops[3])
        return float((y * f32[4].astype(np.float64)).sum())

    # the loss is affine in each single input, so a wide central difference is exact up to rounding
    step = np.float32(0.25)
    for which, g in enumerate(grads):
        for idx in np.ndindex(f32[which].shape):
            hi = [t.copy() for t in f32[:4]]
            lo = [t.copy() for t in f32[:4]]
            hi[which][idx] += step
            lo[which][idx] -= step
            fd = (loss(hi) - loss(lo)) / (float(hi[which][idx]) - float(lo[which][idx]))  # the step as stored
            assert abs(fd - g[idx]) <= 1e-9 * max(1.0, abs(fd)), (which, idx, fd, g[idx])


def test_gradient_invariants():
    x, a, b, c, dy = make_inputs((2, 65, 4), seed=9)
    r = oracle_all(x, a, b, c, dy)
    h, _ = oracle.forward_f64(x, a, b, c)
    assert np.all(r["da"][:, 0, :] == 0.0)                                    # h(-1) = 0
    np.testing.assert_allclose(r["dc"], dy.double().numpy() * h, rtol=1e-14)  # dc = dy * h
    np.testing.assert_allclose(r["dx"] * x.double().numpy(), r["db"] * b.double().numpy(), rtol=1e-12, atol=1e-15)
    # linearity of every gradient in dy
    r2 = oracle_all(x, a, b, c, (2 * dy))
    for k in ("dx", "da", "db", "dc"):
        np.testing.assert_allclose(r2[k], 2 * r[k], rtol=1e-14)


def test_time_concatenation_property():
    # scanning [0, L) equals scanning [0, k) and then [k, L) seeded with h(k-1); the seed enters as an
    # extra drive term a(k) * h(k-1) folded into step k
    x, a, b, c, _ = make_inputs((1, 40, 3), seed=11)
    h_full, _ = oracle.forward_f64(x, a, b, c)
    k = 17
    h_head, _ = oracle.forward_f64(x[:, :k], a[:, :k], b[:, :k], c[:, :k])
    x2, b2 = x[:, k:].double().numpy().copy(), b[:, k:].double().numpy().copy()
    # fold the seed into the first step: b*x + a*h_prev (kept in float64 by passing b = 1, x = drive)
    drive = b2 * x2
    drive[:, 0] += a[:, k].double().numpy() * h_head[:, -1]
    state = np.zeros_like(drive[:, 0])
    tail = []
    for t in range(drive.shape[1]):
        state = (a[:, k + t].double().numpy() if t > 0 else 0.0) * state + drive[:, t]
        tail.append(state)
    np.testing.assert_allclose(np.stack(tail, axis=1), h_full[:, k:], rtol=1e-13)


def test_carried_state_pieces_reproduce_the_whole_sequence():
    # Pins the carried-state oracle functions on the whole-sequence ones (which the exact vectors, closed forms and
    # finite differences above pin): scanning [0, L) in pieces, handing h_final on as the next piece's h0, must give
    # the same h and y; and running the pieces' backward passes last piece first, handing dh0 back as the previous
    # piece's incoming gradient of h_final, must give the same gradients.  The carried values are float32 (what the
    # device hands over), so agreement is to float32 rounding of the state, not to float64.
    x, a, b, c, dy = make_inputs((2, 61, 5), seed=23)
    h_full, y_full = oracle.forward_f64(x, a, b, c)
    g_full = oracle.backward_f64(x, a, b, c, dy)
    cuts = [0, 1, 18, 19, 40, 61]
    pieces = list(zip(cuts[:-1], cuts[1:]))
    h0, states, hs, ys = None, [], [], []
    for k0, k1 in pieces:
        states.append(h0)
        h, y, hf = oracle.forward_carry_f64(x[:, k0:k1], a[:, k0:k1], b[:, k0:k1], c[:, k0:k1], h0)
        np.testing.assert_array_equal(hf, h[:, -1])
        hs.append(h)
        ys.append(y)
        h0 = hf.astype(np.float32)
    np.testing.assert_allclose(np.concatenate(hs, 1), h_full, rtol=0, atol=2e-7 * np.abs(h_full).max())
    np.testing.assert_allclose(np.concatenate(ys, 1), y_full, rtol=0, atol=2e-7 * np.abs(y_full).max())
    g_in, grads = None, []
    for (k0, k1), st in reversed(list(zip(pieces, states))):
        out = oracle.backward_carry_f64(x[:, k0:k1], a[:, k0:k1], b[:, k0:k1], c[:, k0:k1], dy[:, k0:k1], st, g_in)
        grads.append(out[:4])
        g_in = out[4].astype(np.float32)
    grads.reverse()
    for k in range(4):
        got = np.concatenate([g[k] for g in grads], 1)
        np.testing.assert_allclose(got, g_full[k], rtol=0, atol=1e-6 * np.abs(g_full[k]).max())


def test_carried_state_gradients_by_finite_differences():
    # d loss / d h0 and the effect of an incoming gradient on h_final, checked against central differences of
    # loss(h0) = sum(y * dy) + sum(h_final * g_final), which is affine in h0 (so the difference is exact up to rounding).
    x, a, b, c, dy = make_inputs((1, 9, 3), seed=29)
    rng = np.random.default_rng(5)
    h0 = rng.standard_normal((1, 3)).astype(np.float32)
    g_final = rng.standard_normal((1, 3)).astype(np.float32)

    def loss(h0v):
        _, y, hf = oracle.forward_carry_f64(x, a, b, c, h0v)
        return float((y * dy.double().numpy()).sum() + (hf * g_final).sum())

    dh0 = oracle.backward_carry_f64(x, a, b, c, dy, h0, g_final)[4]
    for d in range(3):
        step = np.zeros_like(h0)
        step[0, d] = 0.5
        fd = (loss(h0 + step) - loss(h0 - step)) / float((h0 + step)[0, d] - (h0 - step)[0, d])
        assert abs(fd - dh0[0, d]) <= 1e-6 * max(1.0, abs(fd))
    # with L = 0 nothing touches the state: dh0 is the incoming gradient
    e = np.zeros((1, 0, 3), dtype=np.float32)
    np.testing.assert_array_equal(oracle.backward_carry_f64(e, e, e, e, e, h0, g_final)[4], g_final.astype(np.float64))


def test_gate_oracle_against_torch_library_routines_and_differences():
    # Pins oracle/gates_oracle.py: forward against torch.sigmoid / silu in float64, backward against torch's autograd
    # of those library routines and against central differences of the float64 forward.
    from oracle import gates_oracle
    import torch.nn.functional as F
    gen = torch.Generator().manual_seed(17)
    z = [(torch.randn(3, 7, 5, generator=gen, dtype=torch.float64) * 3).requires_grad_(True) for _ in range(5)]
    g = [torch.randn(3, 7, 5, generator=gen, dtype=torch.float64) for _ in range(4)]
    a, x, c, b = torch.sigmoid(z[0]), z[1] * 1.0, F.silu(z[2]) * z[3], torch.sigmoid(z[4])
    got = gates_oracle.gates_forward_f64(*z)
    for name, mine, lib in zip("axcb", got, (a, x, c, b)):
        np.testing.assert_allclose(mine, lib.detach().numpy(), rtol=1e-14, atol=1e-16, err_msg=name)
    (a * g[0] + x * g[1] + c * g[2] + b * g[3]).sum().backward()
    grads = gates_oracle.gates_backward_f64(*g, z[0], z[2], z[3], z[4])
    for name, mine, leaf in zip(("dA", "dB", "dCa", "dCb", "dD"), grads, z):
        np.testing.assert_allclose(mine, leaf.grad.numpy(), rtol=1e-12, atol=1e-15, err_msg=name)
    # central differences on one element of every input
    zs = [t.detach().numpy().copy() for t in z]
    gs = [t.numpy() for t in g]

    def loss(vals):
        out = gates_oracle.gates_forward_f64(*vals)
        return sum(float((o * w).sum()) for o, w in zip(out, gs))

    for k in range(5):
        bump = [v.copy() for v in zs]
        lo = [v.copy() for v in zs]
        bump[k][1, 2, 3] += 1e-6
        lo[k][1, 2, 3] -= 1e-6
        fd = (loss(bump) - loss(lo)) / 2e-6
        assert abs(fd - grads[k][1, 2, 3]) <= 1e-7 * max(1.0, abs(fd))
    # saturation: large |z| must not overflow
    big = np.array([[-800.0, 800.0]])
    sat = gates_oracle.gates_forward_f64(big, big, big, big, big)
    assert np.all(np.isfinite(sat[0])) and sat[0][0, 0] == 0.0 and sat[0][0, 1] == 1.0 and sat[2][0, 0] == 0.0


def test_rmsnorm_oracle_against_torch_library_routine_and_differences():
    # Pins oracle/rmsnorm_oracle.py: forward against torch.nn.functional.rms_norm in float64, backward against
    # torch's autograd of that library routine, against central differences, and through what the formula fixes.
    from oracle import rmsnorm_oracle
    import torch.nn.functional as F
    gen = torch.Generator().manual_seed(23)
    x = (torch.randn(3, 5, 11, generator=gen, dtype=torch.float64) * 2).requires_grad_(True)
    w = (torch.rand(11, generator=gen, dtype=torch.float64) + 0.5).requires_grad_(True)
    dy = torch.randn(3, 5, 11, generator=gen, dtype=torch.float64)
    eps = 1e-5
    y = F.rms_norm(x, (11,), w, eps)
    np.testing.assert_allclose(rmsnorm_oracle.rmsnorm_forward_f64(x, w, eps), y.detach().numpy(), rtol=1e-14)
    (y * dy).sum().backward()
    dx, dw = rmsnorm_oracle.rmsnorm_backward_f64(dy, x, w, eps)
    np.testing.assert_allclose(dx, x.grad.numpy(), rtol=1e-11, atol=1e-14)
    np.testing.assert_allclose(dw, w.grad.numpy(), rtol=1e-11, atol=1e-14)
    # central differences on one element of x and of the weight
    xs, ws, gs = x.detach().numpy().copy(), w.detach().numpy().copy(), dy.numpy()

    def loss(xv, wv):
        return float((rmsnorm_oracle.rmsnorm_forward_f64(xv, wv, eps) * gs).sum())

    hi, lo = xs.copy(), xs.copy()
    hi[1, 2, 3] += 1e-6
    lo[1, 2, 3] -= 1e-6
    fd = (loss(hi, ws) - loss(lo, ws)) / 2e-6
    assert abs(fd - dx[1, 2, 3]) <= 1e-7 * max(1.0, abs(fd))
    hi, lo = ws.copy(), ws.copy()
    hi[4] += 1e-6
    lo[4] -= 1e-6
    fd = (loss(xs, hi) - loss(xs, lo)) / 2e-6
    assert abs(fd - dw[4]) <= 1e-7 * max(1.0, abs(fd))
    # eps = 0: y does not change when x is scaled, every row of y / w has unit mean square, and dx is
    # orthogonal to x (the loss cannot change along the direction that only rescales the row)
    y0 = rmsnorm_oracle.rmsnorm_forward_f64(xs, ws, 0.0)
    np.testing.assert_allclose(rmsnorm_oracle.rmsnorm_forward_f64(7.5 * xs, ws, 0.0), y0, rtol=1e-13)
    np.testing.assert_allclose(np.mean((y0 / ws) ** 2, axis=-1), 1.0, rtol=1e-13)
    dx0, _ = rmsnorm_oracle.rmsnorm_backward_f64(gs, xs, ws, 0.0)
    assert np.max(np.abs(np.sum(dx0 * xs, axis=-1))) <= 1e-12 * np.max(np.abs(dx0)) * np.max(np.abs(xs)) * 11


def test_c_and_torch_flavours_agree_bitwise_in_fp32():
    x, a, b, c, dy = make_inputs((2, 130, 5), seed=3)
    h_c = oracle.forward_f32_seq(x, a, b)
    h_t = reference_forward_states(x, a, b)
    assert np.array_equal(h_c, h_t.numpy())
    y, dx, da, db, dc = reference_scan_with_grads(x, a, b, c, dy)
    got = oracle.backward_f32_seq(x, a, b, c, dy, h_c)
    # autograd accumulates the same products; sums of two terms may associate differently only in dH,
    # where both sides add (dy*c) + carried term in that order
    for name, g_c, g_t in zip(("dx", "da", "db", "dc"), got, (dx, da, db, dc)):
        np.testing.assert_allclose(g_c, g_t.numpy(), rtol=2e-6, atol=1e-7, err_msg=name)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_torch_restatement_rounding_points(dtype):
    # 16-bit inputs: fp32 accumulation, h rounded to the input dtype, then c*h in the input dtype
    x, a, b, c, _ = make_inputs((1, 33, 4), dtype=dtype, seed=4)
    h64, _ = oracle.forward_f64(x, a, b, c)
    h = reference_forward_states(x, a, b)
    assert h.dtype == dtype
    expect_h = torch.from_numpy(oracle.forward_f32_seq(x, a, b)).to(dtype)
    assert torch.equal(h, expect_h)
    y = reference_scan(x, a, b, c)
    assert torch.equal(y, c * expect_h)
    assert oracle.error_report(y, h64 * c.double().numpy())["scaled"] < 1e-2


def test_product_cpu_path_equals_reference_cpu_path():
    # quick_ssm_amd's own backend="torch" path advances all batch rows at once; element for element it
    # must do what the reference's loop does
    from quick_ssm_amd.scan_interface import scan

    for dtype in (torch.float32, torch.float16, torch.bfloat16):
        x, a, b, c, dy = make_inputs((3, 70, 6), dtype=dtype, seed=8)
        leaves = [t.clone().requires_grad_(True) for t in (x, a, b, c)]
        y = scan(*leaves, backend="torch")
        y.backward(dy)
        y_ref, *g_ref = reference_scan_with_grads(x, a, b, c, dy)
        assert torch.equal(y, y_ref)
        for t, g in zip(leaves, g_ref):
            assert torch.allclose(t.grad.float(), g.float(), rtol=1e-5, atol=1e-6)
