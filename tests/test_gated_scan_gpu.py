"""GPU parity of the gated scan (qssm_scan_gated_forward / _backward through the C ABI): projection outputs in,
y and the projections' gradients out, with the gate activations inside the scan's launches.

Oracle: gates_oracle (float64) -> the operands rounded to the storage type where the layer rounds them
(quick_ssm/layers.py:85-88) -> scan oracle (float64) -> scan gradients -> gates_oracle backward.  Both oracles are
pinned in tests/test_oracle.py.  Tolerance: 1e-2 of each tensor's largest magnitude (16-bit storage).
"""
from __future__ import annotations

import numpy as np
import pytest
import torch

import oracle
from helpers import TOL, assert_close
from oracle import gates_oracle
from quick_ssm_amd import gated_scan, hip_scan
from quick_ssm_amd.gates import gate_prologue
from quick_ssm_amd.scan_interface import scan

pytestmark = pytest.mark.gpu

NAMES = ("dA_pre", "dB_in", "dCa", "dCb", "dD_pre")


def _projections(shape, dtype, seed):
    """Pre-activations with the spread a trained layer shows: forget gate around sigmoid^-1(0.9 .. 0.99)."""
    gen = torch.Generator().manual_seed(seed)
    A_pre = torch.randn(shape, generator=gen) * 0.8 + 3.0
    B_in = torch.randn(shape, generator=gen)
    Ca = torch.randn(shape, generator=gen) * 1.5
    Cb = torch.randn(shape, generator=gen)
    D_pre = torch.randn(shape, generator=gen) * 1.5 - 1.0
    return [t.to(dtype) for t in (A_pre, B_in, Ca, Cb, D_pre)]


def _oracle(pre, dy, dtype):
    A_pre, B_in, Ca, Cb, D_pre = pre
    a, x, c, b = gates_oracle.gates_forward_f64(A_pre, B_in, Ca, Cb, D_pre)
    ops = [torch.from_numpy(t).to(dtype) for t in (x, a, b, c)]          # as the layer stores them
    _, y = oracle.forward_f64(*ops)
    dx, da, db, dc = oracle.backward_f64(*ops, dy)
    grads = gates_oracle.gates_backward_f64(da, dx, dc, db, A_pre, Ca, Cb, D_pre)
    return y, grads


def _run(pre, dy, gpu, out_dtype, place=lambda t, dev: t.to(dev), compute_dtype=None):
    leaves = [place(t, gpu).detach().requires_grad_(True) for t in pre]
    compute_dtype = compute_dtype or pre[0].dtype
    assert gated_scan.supported(leaves, compute_dtype, out_dtype)
    y = gated_scan.gated_scan(*leaves, out_dtype=out_dtype, compute_dtype=compute_dtype)
    y.backward(place(dy, gpu))
    assert hip_scan.workspace_status() == 0
    return y.detach().cpu(), [t.grad.cpu() for t in leaves]


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=["f16", "bf16"])
@pytest.mark.parametrize("shape", [(2, 700, 512), (2, 1100, 264), (1, 97, 256), (3, 33, 128), (1, 2100, 136)],
                         ids=lambda s: "x".join(map(str, s)))
def test_gated_scan_matches_oracle_composition(gpu, dtype, shape):
    # whole and ragged tiles, a partial last strip, several clusters per chain, rows of 64 and of 32 lanes
    pre = _projections(shape, dtype, seed=sum(shape))
    dy = torch.randn(shape, generator=torch.Generator().manual_seed(7)).to(dtype)
    y_ref, g_ref = _oracle(pre, dy, dtype)
    y, grads = _run(pre, dy, gpu, dtype)
    assert_close("y", y, y_ref, TOL[dtype])
    for name, got, want in zip(NAMES, grads, g_ref):
        assert got.dtype == dtype
        assert_close(name, got, want, TOL[dtype])


@pytest.mark.parametrize("compute", [torch.float16, torch.bfloat16, torch.float32], ids=["c16", "cbf16", "c32"])
@pytest.mark.parametrize("shape", [(2, 700, 512), (2, 1100, 264), (1, 97, 256), (3, 33, 128), (1, 2100, 136), (4, 2048, 1024)],
                         ids=lambda s: "x".join(map(str, s)))
def test_gated_scan_over_fp32_projections_matches_oracle_composition(gpu, compute, shape):
    # The reference's default layer: fp32 projection outputs, gates and scan operands cast to the compute dtype
    # (quick_ssm/layers.py:85-88), fp32 y and dy.  One launch each way; the 16-bit operands exist in registers only.
    # Oracle: float64 gates, operands rounded to the compute dtype, float64 scan, float64 gate derivatives.
    pre = _projections(shape, torch.float32, seed=sum(shape) + 5)
    dy = torch.randn(shape, generator=torch.Generator().manual_seed(12))
    y_ref, g_ref = _oracle(pre, dy, compute)
    y, grads = _run(pre, dy, gpu, torch.float32, compute_dtype=compute)
    assert y.dtype == torch.float32
    # 16-bit compute: a gate within an fp32 ulp of a rounding tie rounds the other way than the float64 oracle's, so y
    # carries differences the size of the compute dtype's spacing; fp32 compute meets the fp32 bar but for the
    # hardware's 1-ulp exp and reciprocal inside the sigmoids
    tol = {torch.float32: 2e-5, torch.float16: 1e-3, torch.bfloat16: 1e-2}[compute]
    assert_close("y", y, y_ref, tol)
    for name, got, want in zip(NAMES, grads, g_ref):
        assert got.dtype == torch.float32
        assert_close(name, got, want, 2e-5 if compute == torch.float32 else 1e-2)


def test_gated_scan_over_fp32_projections_equals_prologue_plus_scan(gpu):
    # the same values through the two-pass route (gate prologue kernel, then the plain scan on fp16 operands with
    # fp32 y): the operands are the same bits, so y differs by the order of the fp32 sums only (another tile
    # geometry); gradients to the rounding of the activations' derivatives
    shape, compute = (2, 900, 384), torch.float16
    pre = _projections(shape, torch.float32, seed=4)
    dy = torch.randn(shape, generator=torch.Generator().manual_seed(13))
    y, grads = _run(pre, dy, gpu, torch.float32, compute_dtype=compute)
    leaves = [t.to(gpu).requires_grad_(True) for t in pre]
    a, x, c, b = gate_prologue(*leaves, compute)
    y2 = scan(x, a, b, c, out_dtype=torch.float32)
    y2.backward(dy.to(gpu))
    assert_close("y", y, y2.detach().cpu().double().numpy(), 1e-5)
    for name, got, leaf in zip(NAMES, grads, leaves):
        assert_close(name, got, leaf.grad.cpu().double().numpy(), 1e-2)


def test_gated_scan_over_fp32_projections_as_blocks_of_one_wide_tensor(gpu):
    # the five fp32 projections as column blocks of one [B, L, 5 S] GEMM output, gradients into one wide tensor:
    # the same launches on strided views, so the same bits as the five-tensor entry
    B, L, S, compute = 2, 500, 256, torch.bfloat16
    pre = _projections((B, L, S), torch.float32, seed=18)
    dy = torch.randn((B, L, S), generator=torch.Generator().manual_seed(14)).to(gpu)
    leaves = [t.to(gpu).requires_grad_(True) for t in pre]
    y = gated_scan.gated_scan(*leaves, out_dtype=torch.float32, compute_dtype=compute)
    y.backward(dy)
    wide = torch.cat(pre, dim=-1).to(gpu).requires_grad_(True)
    assert gated_scan.supported([wide[..., k * S:(k + 1) * S] for k in range(5)], compute, torch.float32)
    y_w = gated_scan.gated_scan_wide(wide, out_dtype=torch.float32, compute_dtype=compute)
    y_w.backward(dy)
    assert hip_scan.workspace_status() == 0
    assert torch.equal(y, y_w)
    for k, leaf in enumerate(leaves):
        assert torch.equal(wide.grad[..., k * S:(k + 1) * S], leaf.grad), NAMES[k]


@pytest.mark.timeout(600)
def test_gated_scan_over_a_wide_tensor_past_4_gib(gpu):
    # [32, 2048, 5 x 4096] fp32 is 5 GiB: the projections of the last batch rows lie past 2^32 bytes.  Drawn on the
    # device; windows of columns of the first and the last batch row go to the float64 oracle composition.
    B, L, S, compute = 32, 2048, 4096, torch.float16
    free, _ = torch.cuda.mem_get_info(gpu)
    if free < (40 << 30):
        pytest.skip("needs 40 GiB of free device memory")
    print("case gated scan over 5 GiB of projections", flush=True)
    gen = torch.Generator(device=gpu).manual_seed(23)
    wide = torch.empty((B, L, 5 * S), dtype=torch.float32, device=gpu).normal_(generator=gen)
    wide[..., 0 * S:1 * S].mul_(0.8).add_(3.0)
    wide[..., 2 * S:3 * S].mul_(1.5)
    wide[..., 4 * S:5 * S].mul_(1.5).sub_(1.0)
    wide.requires_grad_(True)
    dy = torch.empty((B, L, S), dtype=torch.float32, device=gpu).normal_(generator=gen)
    assert gated_scan.supported([wide[..., k * S:(k + 1) * S] for k in range(5)], compute, torch.float32)
    y = gated_scan.gated_scan_wide(wide, out_dtype=torch.float32, compute_dtype=compute)
    y.backward(dy)
    assert hip_scan.workspace_status() == 0
    assert bool(torch.isfinite(y).all()) and bool(torch.isfinite(wide.grad).all())
    for row in (0, B - 1):
        for c0 in (0, S - 64):
            pre = [wide.detach()[row:row + 1, :, k * S + c0:k * S + c0 + 64].cpu() for k in range(5)]
            y_ref, g_ref = _oracle(pre, dy[row:row + 1, :, c0:c0 + 64].cpu(), compute)
            assert_close(f"y[row {row}, cols {c0}]", y[row:row + 1, :, c0:c0 + 64].detach().cpu(), y_ref, 1e-2)
            for k, (name, ref) in enumerate(zip(NAMES, g_ref)):
                got = wide.grad[row:row + 1, :, k * S + c0:k * S + c0 + 64].cpu()
                assert_close(f"{name}[row {row}, cols {c0}]", got, ref, 1e-2)
    del y, dy, wide
    torch.cuda.empty_cache()


@pytest.mark.timeout(600)
def test_seeded_random_gated_shapes_match_the_oracle(gpu):
    # A fixed-seed draw over (shape, projection storage, compute dtype): whatever geometry the planner picks for the
    # gated launches (state widths from 128 up, clusters, partial strips, ragged last tiles) must meet the composed
    # float64 oracle.  QSSM_RANDOM_GATED_CASES=n draws n cases instead of 60.
    import os
    n_cases = int(os.environ.get("QSSM_RANDOM_GATED_CASES", "60"))
    rng = np.random.default_rng(20250911)
    kinds = [(torch.float16, torch.float16), (torch.bfloat16, torch.bfloat16), (torch.float32, torch.float16),
             (torch.float32, torch.bfloat16), (torch.float32, torch.float32)]
    for case in range(n_cases):
        dtype, compute = kinds[case % len(kinds)]
        unit = 8 if dtype != torch.float32 else 4                 # 16 bytes of a row
        B = int(rng.integers(1, 4))
        L = int(rng.choice([int(rng.integers(1, 100)), int(rng.integers(100, 1500)), int(rng.integers(1500, 5000))]))
        S = max(128, unit * int(rng.choice([int(rng.integers(16, 40)), int(rng.integers(40, 130)), 32 * int(rng.integers(1, 5))])))
        if B * L * S > 1_500_000:
            L = max(1, 1_500_000 // (B * S))
        shape = (B, L, S)
        pre = _projections(shape, dtype, seed=3000 + case)
        dy = torch.randn(shape, generator=torch.Generator().manual_seed(4000 + case)).to(dtype)
        if case < 20 or case % 10 == 0:
            print(f"case random gated {case} shape={shape} storage={dtype} compute={compute}", flush=True)
        y_ref, g_ref = _oracle(pre, dy, compute)
        y, grads = _run(pre, dy, gpu, dtype, compute_dtype=compute)
        y_tol = {torch.float32: 2e-5, torch.float16: 1e-3, torch.bfloat16: 1e-2}[compute] if dtype == torch.float32 \
            else TOL[dtype]
        g_tol = (2e-5 if compute == torch.float32 else 1e-2) if dtype == torch.float32 else TOL[dtype]
        assert_close(f"y (case {case})", y, y_ref, y_tol)
        for name, got, want in zip(NAMES, grads, g_ref):
            assert got.dtype == dtype
            assert_close(f"{name} (case {case})", got, want, g_tol)


def test_gated_forward_without_a_backward_equals_the_one_with(gpu):
    # no projection wants a gradient: the launch is planned with keep_tiles = 0; y is the same bit for bit
    pre = [t.to(gpu) for t in _projections((2, 900, 512), torch.bfloat16, seed=41)]
    with torch.no_grad():
        y0 = gated_scan.gated_scan(*pre, out_dtype=torch.bfloat16)
    y1 = gated_scan.gated_scan(*[t.clone().requires_grad_(True) for t in pre], out_dtype=torch.bfloat16)
    assert y0.grad_fn is None and y1.grad_fn is not None
    assert torch.equal(y0, y1.detach())
    assert hip_scan.workspace_status() == 0


def test_gated_scan_with_fp32_y_takes_the_two_pass_backward(gpu):
    # y stored as fp32 (the layer's scan_out_dtype): forward fused, backward through the prologue and the plain scan
    shape, dtype = (2, 600, 256), torch.float16
    pre = _projections(shape, dtype, seed=21)
    dy = torch.randn(shape, generator=torch.Generator().manual_seed(8))
    y_ref, g_ref = _oracle(pre, dy, dtype)
    y, grads = _run(pre, dy, gpu, torch.float32)
    assert y.dtype == torch.float32
    # the operands themselves are computed here and rounded to fp16: a gate within an fp32 ulp of a tie rounds the
    # other way than the float64 oracle's, so y carries fp16-sized differences however it is stored
    assert_close("y", y, y_ref, 1e-3)
    for name, got, want in zip(NAMES, grads, g_ref):
        assert_close(name, got, want, TOL[dtype])


def test_gated_scan_equals_prologue_plus_scan(gpu):
    # the same values through the two-pass route: y bit for bit (same activations, same roundings, same recurrence
    # geometry is not guaranteed, so to fp32 rounding of the carries), gradients to the rounding of a(1 - a)
    shape, dtype = (2, 900, 384), torch.bfloat16
    pre = _projections(shape, dtype, seed=3)
    dy = torch.randn(shape, generator=torch.Generator().manual_seed(9)).to(dtype)
    y, grads = _run(pre, dy, gpu, dtype)
    leaves = [t.to(gpu).requires_grad_(True) for t in pre]
    a, x, c, b = gate_prologue(*leaves, dtype)
    y2 = scan(x, a, b, c)
    y2.backward(dy.to(gpu))
    assert_close("y", y, y2.detach().cpu().double().numpy(), 1e-2)
    frac_equal = (y == y2.detach().cpu()).float().mean().item()
    assert frac_equal > 0.99, frac_equal
    for name, got, leaf in zip(NAMES, grads, leaves):
        assert_close(name, got, leaf.grad.cpu().double().numpy(), 1e-2)


def test_gated_scan_on_column_slices_of_one_wide_tensor(gpu):
    # the five projections as slices of one [B, L, 5 S] GEMM output (time stride 5 S), gradients into one wide tensor
    B, L, S, dtype = 2, 300, 256, torch.bfloat16
    pre = _projections((B, L, S), dtype, seed=11)
    dy = torch.randn((B, L, S), generator=torch.Generator().manual_seed(10)).to(dtype)
    y_ref, g_ref = _oracle(pre, dy, dtype)
    wide = torch.cat(pre, dim=-1).to(gpu).requires_grad_(True)
    parts = [wide[..., k * S:(k + 1) * S] for k in range(5)]
    assert gated_scan.supported(parts, dtype, dtype)
    y = gated_scan.gated_scan(*parts)
    y.backward(dy.to(gpu))
    assert hip_scan.workspace_status() == 0
    assert_close("y", y.detach().cpu(), y_ref, TOL[dtype])
    for k, (name, want) in enumerate(zip(NAMES, g_ref)):
        assert_close(name, wide.grad[..., k * S:(k + 1) * S].cpu(), want, TOL[dtype])


def test_what_the_gated_launches_do_not_take(gpu):
    pre = [t.to(gpu) for t in _projections((2, 64, 256), torch.bfloat16, seed=1)]
    assert gated_scan.supported(pre, torch.bfloat16, torch.bfloat16)
    assert not gated_scan.supported(pre, torch.float16, torch.float16)              # compute dtype differs from storage
    assert not gated_scan.supported(pre, torch.bfloat16, torch.bfloat16, checkpoint=False)
    wide32 = [t.float() for t in pre]
    assert gated_scan.supported(wide32, torch.float32, torch.float32)               # fp32 projections: any compute dtype,
    assert gated_scan.supported(wide32, torch.float16, torch.float32)               # fp32 y only
    assert not gated_scan.supported(wide32, torch.float16, torch.float16)
    assert not gated_scan.supported([t[..., 2:] for t in wide32], torch.float16, torch.float32)   # rows off 16 bytes
    assert not gated_scan.supported([t[..., :100] for t in pre], torch.bfloat16, torch.bfloat16)     # S < 128
    assert not gated_scan.supported([t[..., 4:] for t in pre], torch.bfloat16, torch.bfloat16)       # rows off 16 bytes
    assert not gated_scan.supported([t.cpu() for t in pre], torch.bfloat16, torch.bfloat16)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "f16"])
def test_ssm_layer_with_16_bit_parameters_uses_the_gated_scan_and_matches_the_sequential_path(gpu, dtype, monkeypatch):
    from quick_ssm_amd.layers import SSM

    torch.manual_seed(0)
    layer = SSM(hidden_size=64, state_size_mult=4.0, compute_dtype=dtype, dtype=dtype)
    xin = torch.randn(2, 192, 64).to(dtype)
    gout = torch.randn(2, 192, 64).to(dtype)
    calls = []
    real, real_wide = gated_scan.gated_scan, gated_scan.gated_scan_wide
    monkeypatch.setattr(gated_scan, "gated_scan", lambda *a, **k: (calls.append(1), real(*a, **k))[1])
    monkeypatch.setattr(gated_scan, "gated_scan_wide", lambda *a, **k: (calls.append(1), real_wide(*a, **k))[1])

    def run(mod, inp, backend):
        mod.zero_grad(set_to_none=True)
        inp = inp.clone().requires_grad_(True)
        out = mod(inp, backend=backend)
        out.backward(gout.to(inp.device))
        return out.detach().cpu().float(), inp.grad.cpu().float(), {n: p.grad.cpu().float() for n, p in mod.named_parameters()}

    ref_layer = SSM(hidden_size=64, state_size_mult=4.0, compute_dtype=dtype, dtype=dtype)
    ref_layer.load_state_dict(layer.state_dict())
    y_ref, dx_ref, g_ref = run(ref_layer, xin, "torch")
    y, dx, g = run(layer.to(gpu), xin.to(gpu), "auto")
    assert calls, "the layer did not take the gated launches"
    tol = 2e-2 if dtype == torch.float16 else 4e-2      # 16-bit GEMMs and 16-bit parameters on both sides
    assert_close("layer out", y, y_ref.double().numpy(), tol)
    assert_close("layer dx", dx, dx_ref.double().numpy(), tol)
    for n in g_ref:
        assert_close(f"grad {n}", g[n], g_ref[n].double().numpy(), tol)


@pytest.mark.timeout(600)
def test_seeded_random_layers_with_16_bit_parameters_match_the_sequential_path(gpu):
    # A fixed-seed draw over layer sizes, batch, sequence length (down to one step) and 16-bit parameter types: the
    # device layer (gated scan, fused or two-pass backward, wide or separate projections) against the same layer with
    # the same parameter values in float64 on the product's sequential torch path on the CPU (a 16-bit run of that
    # path is itself several roundings away from it).  QSSM_RANDOM_LAYER16_CASES=n draws n cases instead of 24.
    import os
    from quick_ssm_amd.layers import SSM

    n_cases = int(os.environ.get("QSSM_RANDOM_LAYER16_CASES", "24"))
    rng = np.random.default_rng(4242)
    for case in range(n_cases):
        dtype = (torch.bfloat16, torch.float16)[case % 2]
        hidden = int(rng.choice([32, 64, 128, 256]))
        mult = float(rng.choice([1.0, 2.0, 4.0]))
        B = int(rng.integers(1, 3))
        L = int(rng.choice([int(rng.integers(1, 12)), int(rng.integers(12, 120)), int(rng.integers(120, 260))]))
        out32 = bool(rng.integers(0, 2))            # fp32 scan output: the two-pass backward
        torch.manual_seed(700 + case)
        layer = SSM(hidden_size=hidden, state_size_mult=mult, compute_dtype=dtype, dtype=dtype)
        ref_layer = SSM(hidden_size=hidden, state_size_mult=mult, compute_dtype=torch.float64, dtype=torch.float64)
        ref_layer.load_state_dict(layer.state_dict())           # the 16-bit values, exactly
        layer = layer.to(gpu)
        g = torch.Generator(device="cpu").manual_seed(800 + case)
        xin = torch.randn(B, L, hidden, generator=g).to(dtype)
        gout = torch.randn(B, L, hidden, generator=g).to(dtype)
        kw = {"scan_out_dtype": torch.float32} if out32 else {}
        print(f"case random 16-bit layer {case} B={B} L={L} hidden={hidden} state={int(hidden * mult)} {dtype} {kw}", flush=True)

        def run(mod, inp, backend):
            mod.zero_grad(set_to_none=True)
            inp = inp.clone().requires_grad_(True)
            out = mod(inp, backend=backend, **kw)
            out.backward(gout.to(inp.device))
            return (out.detach().cpu().float(), inp.grad.cpu().float(),
                    {n: p.grad.cpu().float() for n, p in mod.named_parameters()})

        def run_ref():
            ref_layer.zero_grad(set_to_none=True)
            inp = xin.double().requires_grad_(True)
            out = ref_layer(inp, backend="torch", **({"scan_out_dtype": torch.float64} if out32 else {}))
            out.backward(gout.double())
            return out.detach(), inp.grad, {n: p.grad for n, p in ref_layer.named_parameters()}

        y_ref, dx_ref, g_ref = run_ref()
        y, dx, grads = run(layer, xin.to(gpu), "auto")
        assert hip_scan.workspace_status() == 0
        tol = 1e-2 if dtype == torch.float16 else 4e-2      # 16-bit parameters, activations and GEMM outputs
        assert_close(f"layer out (case {case})", y, y_ref.numpy(), tol)
        assert_close(f"layer dx (case {case})", dx, dx_ref.numpy(), tol)
        for n in g_ref:
            assert_close(f"grad {n} (case {case})", grads[n], g_ref[n].numpy(), tol)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
def test_batched_projection_gemm_equals_the_five_separate_ones(gpu, dtype, monkeypatch):
    # small layers stack the five projection weights into one batched GEMM; same values and gradients as five
    # nn.Linear calls, to GEMM rounding, and the parameters (and so the state dict) stay the reference's
    from quick_ssm_amd.layers import SSM

    torch.manual_seed(1)
    layer = SSM(hidden_size=64, state_size_mult=4.0, compute_dtype=torch.bfloat16, dtype=dtype).to(gpu)
    assert sorted(n for n, _ in layer.named_parameters()) == sorted(
        f"{m}.{p}" for m, ps in (("A_proj", ("weight", "bias")), ("B_proj", ("weight",)), ("C_proj_a", ("weight",)),
                                 ("C_proj_b", ("weight",)), ("D_proj", ("weight",)), ("out_proj", ("weight", "bias")),
                                 ("pre_norm", ("weight",))) for p in ps)
    xin = torch.randn(2, 160, 64, device=gpu).to(dtype)
    gout = torch.randn(2, 160, 64, device=gpu).to(dtype)

    def run():
        layer.zero_grad(set_to_none=True)
        inp = xin.clone().requires_grad_(True)
        out = layer(inp)
        out.backward(gout)
        return out.detach().float().cpu(), inp.grad.float().cpu(), {n: p.grad.float().cpu() for n, p in layer.named_parameters()}

    y_b, dx_b, g_b = run()
    monkeypatch.setattr(SSM, "_BATCHED_PROJECTION_LIMIT", 0)
    y_s, dx_s, g_s = run()
    tol = 1e-4 if dtype == torch.float32 else 3e-2
    assert_close("layer out", y_b, y_s.double().numpy(), tol)
    assert_close("layer dx", dx_b, dx_s.double().numpy(), tol)
    for n in g_s:
        assert_close(f"grad {n}", g_b[n], g_s[n].double().numpy(), tol)


@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float32], ids=["y16", "y32"])
def test_gated_scan_on_one_wide_tensor_equals_five_tensors(gpu, out_dtype):
    # the wide entry (one GEMM's [B, L, 5 S] output in, one wide gradient out): same launches on strided views, so
    # the same bits as the five-tensor entry; with fp32 y the backward takes the two-pass route in both
    B, L, S, dtype = 2, 500, 256, torch.bfloat16
    pre = _projections((B, L, S), dtype, seed=17)
    dy = torch.randn((B, L, S), generator=torch.Generator().manual_seed(3)).to(out_dtype).to(gpu)
    leaves = [t.to(gpu).requires_grad_(True) for t in pre]
    y = gated_scan.gated_scan(*leaves, out_dtype=out_dtype)
    y.backward(dy)
    wide = torch.cat(pre, dim=-1).to(gpu).requires_grad_(True)
    y_w = gated_scan.gated_scan_wide(wide, out_dtype=out_dtype)
    y_w.backward(dy)
    assert hip_scan.workspace_status() == 0
    assert torch.equal(y, y_w)
    for k, leaf in enumerate(leaves):
        assert torch.equal(wide.grad[..., k * S:(k + 1) * S], leaf.grad), NAMES[k]
