"""Parity of the HIP scan (through the C ABI) with the CPU oracle, on a real MI355X.

Bar: per tensor, max|got - oracle| / max|oracle| <= 1e-5 for fp32 storage and <= 1e-2 for fp16 / bf16
storage, the oracle being float64 arithmetic on the same stored inputs.  fp32 cases are also held
to the reference tests' own allclose(rtol=1e-3, atol=1e-5) against the fp32 sequential recurrence.
"""
import json
import os
from pathlib import Path

import numpy as np
import pytest
import torch

import oracle
from helpers import TOL, assert_close, make_inputs, oracle_all, run_scan_with_grads
from quick_ssm_amd import _lib, hip_scan
from quick_ssm_amd.scan_interface import honor_tiles, scan, scan_chunk

pytestmark = pytest.mark.gpu

GOLDEN = json.loads((Path(__file__).parent / "golden" / "exact_scan_vectors.json").read_text())


def _check_all(got, ref, tol):
    report = {}
    for k in ("y", "dx", "da", "db", "dc"):
        assert_close(k, got[k], ref[k], tol, report)
    return report


# ---- the reference's own test cases ----------------------------------------------------------------

@pytest.mark.parametrize("shape,block_l,seed", [((2, 512, 8), 128, 42), ((1, 4, 1), 8, 3), ((1, 1024, 1), 1024, 4)])
def test_forward_cases_of_reference_test_forwards(gpu, shape, block_l, seed):
    # quick_ssm/test_forwards.py:108-114: fp32 h against the sequential recurrence, rtol 1e-3 atol 1e-5
    x, a, b, _, _ = make_inputs(shape, seed=seed)
    print(f"case fwd shape={shape} block_l={block_l} seed={seed}", flush=True)
    out_a, h = hip_scan.block_scan_forward_3d(x.to(gpu), a.to(gpu), b.to(gpu), BLOCK_L=block_l)
    assert h.dtype == torch.float32 and out_a.shape == h.shape
    h_seq = torch.from_numpy(oracle.forward_f32_seq(x, a, b))
    assert torch.allclose(h.cpu(), h_seq, rtol=1e-3, atol=1e-5)
    h64, _ = oracle.forward_f64(x, a, b)
    assert_close("h", h, h64, 1e-5)
    assert_close("out_a", out_a, np.cumprod(a.double().numpy(), axis=1), 1e-5)


@pytest.mark.parametrize("shape", [(2, 2048, 8), (1, 1024, 1)])
def test_backward_cases_of_reference_test_backwards(gpu, shape):
    # quick_ssm/test_backwards.py:120-125: b, c ~ N(0,1), h from the sequential recurrence fed in, fp32
    x, a, b, c, dy = make_inputs(shape, seed=0, unit_bc=True)
    print(f"case bwd shape={shape}", flush=True)
    h_seq = torch.from_numpy(oracle.forward_f32_seq(x, a, b))
    got = hip_scan.block_scan_backward_3d(*(t.to(gpu) for t in (a, b, c, x, h_seq, dy)))
    ref = oracle.backward_f64(x, a, b, c, dy)
    seq = oracle.backward_f32_seq(x, a, b, c, dy, h_seq)
    for name, g, r, s in zip(("dx", "da", "db", "dc"), got, ref, seq):
        assert g.dtype == torch.float32
        assert_close(name, g, r, 1e-5)
        assert torch.allclose(g.cpu(), torch.from_numpy(s), rtol=1e-3, atol=1e-5 * max(1.0, float(np.abs(r).max())))


def test_scan_interface_case_of_reference(gpu):
    # quick_ssm/test_scan_interface.py:8-31: B2 L32 D4, block_l 16, fp16 on the device, grads within atol 1e-4 rtol 1e-3
    # of the sequential path (here: of the float64 oracle, at the fp16 bar)
    x, a, b, c, dy = make_inputs((2, 32, 4), dtype=torch.float16, seed=0)
    got = run_scan_with_grads(scan, x, a, b, c, dy, gpu, block_l=16, checkpoint=True)
    _check_all(got, oracle_all(x, a, b, c, dy), TOL[torch.float16])


# ---- exact vectors and closed forms -----------------------------------------------------------------

# What one rounding of an exact result to the storage type may cost, per element (half an ulp: 2^-24, 2^-11, 2^-8),
# on top of fp32 arithmetic inside the kernels.
_STORE_RTOL = {torch.float32: 2e-6, torch.float16: 6e-4, torch.bfloat16: 4.5e-3}


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16], ids=["f32", "f16", "bf16"])
@pytest.mark.parametrize("case", GOLDEN["cases"], ids=lambda c: c["name"])
def test_exact_rational_vectors(gpu, case, dtype):
    # The inputs are small dyadic rationals, exact in all three storage types; the expected values are the exact
    # rationals, so a 16-bit run may differ from them by the one rounding of each result and nothing else.
    x, a, b, c, dy = (torch.tensor(case[k], dtype=torch.float32) for k in ("x", "a", "b", "c", "dy"))
    for t, k in zip((x, a, b, c, dy), "xabcg"):
        assert torch.equal(t.to(dtype).float(), t), f"{k} is not exact in {dtype}"
    got = run_scan_with_grads(scan, *(t.to(dtype) for t in (x, a, b, c, dy)), gpu)
    rtol = _STORE_RTOL[dtype]
    for k in ("y", "dx", "da", "db", "dc"):
        assert got[k].dtype == dtype
        np.testing.assert_allclose(got[k].double().numpy(), np.array(case[k]), rtol=rtol, atol=rtol, err_msg=k)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
def test_closed_form_geometric_decay(gpu, dtype):
    # x = delta(t=0), b = 1, a = g: h(t) = g^t (the idea of quick_ssm/forward_only.py:548-629)
    L, g = 4096, 0.999
    x = torch.zeros(1, L, 2, dtype=dtype)
    x[:, 0] = 1
    a = torch.full_like(x, g)
    b = torch.ones_like(x)
    _, h = hip_scan.block_scan_forward_3d(x.to(gpu), a.to(gpu), b.to(gpu))
    g_stored = float(a[0, 0, 0].double())
    expect = g_stored ** np.arange(L)
    rel = np.abs(h[0, :, 0].double().cpu().numpy() - expect) / expect
    assert rel.max() < (1e-5 if dtype == torch.float32 else 1e-2) * 30  # error grows with t; ~L * eps / 2
    assert rel[-1] < 3e-4


def test_a_million_steps_of_near_unit_decay(gpu):
    # The reference's precision test at its own length (quick_ssm/forward_only.py:548-629: L = 2^20, an impulse at
    # t = 0, b = 1, a = g), with g chosen so that g^L stays a normal number: h(t) = g^t over 2^20 steps and the
    # thousands of hand-overs between tiles they take, against float64 powers of the stored g; and y, with the
    # gradients of a random dy, against the float64 oracle on a second, random, input of the same length.
    L, D = 1 << 20, 16
    g = float(torch.tensor(0.99999, dtype=torch.float32).double())
    x = torch.zeros(1, L, D)
    x[:, 0] = 1
    a = torch.full_like(x, g)
    b = torch.ones_like(x)
    print("case 2^20 steps", flush=True)
    _, h = hip_scan.block_scan_forward_3d(x.to(gpu), a.to(gpu), b.to(gpu))
    expect = g ** np.arange(L)
    rel = np.abs(h[0].double().cpu().numpy() - expect[:, None]) / expect[:, None]
    print(f"  g^t: worst relative error {rel.max():.2e}, at the last step {rel[-1].max():.2e}", flush=True)
    # With one g for every step every tile carries the same product g^64 with the same rounding error, which the
    # 16 384 tiles of the chain then repeat instead of averaging out: 1.3e-3 at the last step (measured), where the
    # sequential fp32 recurrence on this input reaches 1.3e-4.  Any evaluation by blocks has this property, the
    # reference's per-block running products (quick_ssm/triton_forwards.py:63-70) included; operands that vary from
    # step to step do not show it (second half of this test: 1e-5 of the largest value over the same 2^20 steps).
    worst_abs = np.abs(h[0].double().cpu().numpy() - expect[:, None]).max()
    print(f"  g^t: largest absolute error {worst_abs:.2e}", flush=True)
    assert rel.max() < 5e-3, (rel.max(), rel[-1].max())
    assert worst_abs < 2e-4
    x, a, b, c, dy = make_inputs((1, L, D), seed=31, a_lo=0.999, a_span=0.001)
    got = run_scan_with_grads(scan, x, a, b, c, dy, gpu)
    ref = oracle_all(x, a, b, c, dy)
    assert hip_scan.workspace_status() == 0
    _check_all(got, ref, 1e-5)


# ---- shapes, dtypes, edges ---------------------------------------------------------------------------

SHAPES = [
    (4, 2048, 16),    # config 0
    (2, 300, 5),      # ragged L, odd D (1 column per lane)
    (1, 1, 1),
    (3, 7, 2),
    (2, 1000, 6),     # D multiple of 2 only
    (2, 777, 64),     # several tiles per chain, ragged last tile
    (1, 4096, 128),
    (2, 1500, 260),   # two strips, the second partial
    (5, 64, 1024),    # config 4's per-layer shape (smaller batch)
    (2, 1100, 264),   # 16-bit: operands through LDS, ragged last tile, second strip of 8 columns
    (3, 200, 512),    # 16-bit: operands through LDS, whole strips, short ragged sequence
]


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16], ids=["f32", "f16", "bf16"])
@pytest.mark.parametrize("shape", SHAPES, ids=lambda s: "x".join(map(str, s)))
def test_scan_matches_oracle(gpu, shape, dtype):
    x, a, b, c, dy = make_inputs(shape, dtype=dtype, seed=sum(shape))
    print(f"case scan shape={shape} dtype={dtype}", flush=True)
    got = run_scan_with_grads(scan, x, a, b, c, dy, gpu)
    assert got["y"].dtype == dtype and got["dx"].dtype == dtype
    _check_all(got, oracle_all(x, a, b, c, dy), TOL[dtype])
    assert torch.all(got["da"][:, 0, :] == 0)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=["f16", "bf16"])
def test_fp32_output_from_16bit_operands(gpu, dtype):
    # what SSM does with fp32 parameters: 16-bit operands, y and dy in fp32 (quick_ssm/layers.py:85-91)
    x, a, b, c, dy = make_inputs((2, 700, 96), dtype=dtype, seed=21, out_dtype=torch.float32)
    got = run_scan_with_grads(scan, x, a, b, c, dy, gpu, out_dtype=torch.float32)
    assert got["y"].dtype == torch.float32 and got["da"].dtype == dtype
    ref = oracle_all(x, a, b, c, dy)
    assert_close("y", got["y"], ref["y"], 1e-5)  # fp32 storage of y: only fp32 arithmetic error remains
    for k in ("dx", "da", "db", "dc"):
        assert_close(k, got[k], ref[k], TOL[dtype])


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=["f16", "bf16"])
@pytest.mark.parametrize("g_log2", [6, 5], ids=["rows64", "rows32"])
@pytest.mark.parametrize("shape", [(2, 700, 512), (2, 1100, 264), (1, 97, 256)], ids=lambda s: "x".join(map(str, s)))
def test_lds_resident_operands_and_register_path_agree(gpu, dtype, shape, g_log2):
    # 64- or 32-lane rows whose bytes are 16-byte aligned take the kernels that load c (and dy) straight into LDS;
    # the same values at an offset of 4 elements take the register-only kernels.  Both must meet the oracle: ragged
    # last tiles, a partial last strip, checkpoint on and off, y in the operands' storage and in fp32.
    B, L, D = shape
    x, a, b, c, dy = make_inputs(shape, dtype=dtype, seed=31)
    ref = oracle_all(x, a, b, c, dy)
    tune = (g_log2 + 1) | (8 << 8)  # lanes per row, 8 steps per lane; workgroup size and clusters automatic

    def run(place, out_dtype=dtype, gy=dy, keep_h=False):
        ops = [place(t) for t in (x, a, b, c)]
        g = place(gy)
        y, h, ckpt, stride = hip_scan.scan_forward(*ops, out_dtype=out_dtype, want_h=keep_h, want_ckpt=not keep_h,
                                                   tune=tune, bwd_tune=tune)
        dx, da, db, dc = hip_scan.scan_backward(*ops, g, h=h, ckpt=ckpt, ckpt_stride=stride, tune=tune)
        assert hip_scan.workspace_status() == 0
        return {k: v.cpu() for k, v in zip(("y", "dx", "da", "db", "dc"), (y, dx, da, db, dc))}, ops

    def aligned(t):
        return t.to(gpu).contiguous()

    def shifted(t):  # same values, every row 8 bytes (4 elements) off a 16-byte boundary
        buf = torch.zeros(B, L, D + 8, dtype=t.dtype, device=gpu)
        buf[:, :, 4:4 + D] = t.to(gpu)
        return buf[:, :, 4:4 + D]

    got_lds, ops = run(aligned)
    assert all(t.data_ptr() % 16 == 0 for t in ops)
    fwd_plan = hip_scan.make_plan(B, L, D, dtype, dtype, _lib.QSSM_FORWARD, 8, 32, tune)
    bwd_plan = hip_scan.make_plan(B, L, D, dtype, dtype, _lib.QSSM_BACKWARD, 8, 0, tune)
    assert (fwd_plan.g_log2, fwd_plan.vec, fwd_plan.steps) == (g_log2, 4, 8) and fwd_plan.threads in (256, 512)
    assert (bwd_plan.g_log2, bwd_plan.vec, bwd_plan.steps, bwd_plan.threads) == (g_log2, 4, 8, 256)
    _check_all(got_lds, ref, TOL[dtype])
    _check_all(run(aligned, keep_h=True)[0], ref, TOL[dtype])

    got_reg, ops = run(shifted)
    assert all(t.data_ptr() % 16 == 8 for t in ops) and D % 8 == 0
    _check_all(got_reg, ref, TOL[dtype])

    x32, a32, b32, c32, dy32 = make_inputs(shape, dtype=dtype, seed=31, out_dtype=torch.float32)
    # fp32 y and dy: the forward keeps c in LDS, the backward dy alone (16 bytes per lane), c in registers
    got32, _ = run(aligned, out_dtype=torch.float32, gy=dy32)
    ref32 = oracle_all(x32, a32, b32, c32, dy32)
    got32_reg, _ = run(shifted, out_dtype=torch.float32, gy=dy32)   # and all of it through registers
    got32_h, _ = run(aligned, out_dtype=torch.float32, gy=dy32, keep_h=True)
    for got in (got32, got32_reg, got32_h):
        assert_close("y", got["y"], ref32["y"], 1e-5)
        for k in ("dx", "da", "db", "dc"):
            assert_close(k, got[k], ref32[k], TOL[dtype])


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=["f16", "bf16"])
@pytest.mark.parametrize("g_log2", [5, 4, 2], ids=["rows32", "rows16", "rows4"])
@pytest.mark.parametrize("shape", [(2, 700, 512), (2, 1100, 264), (1, 97, 256), (1, 2100, 40)],
                         ids=lambda s: "x".join(map(str, s)))
def test_forward_with_sixteen_bytes_per_lane(gpu, dtype, shape, g_log2):
    # The forward over 16-bit storage that large launches take by themselves (8 columns = 16 bytes per lane, c
    # loaded straight into LDS), forced here onto small shapes: ragged last tiles, a partial last strip, several
    # clusters per chain, rows narrower than a wavefront, y in the operands' storage and in fp32, the full fp32
    # state, rows off a 16-byte boundary (c then goes through registers), and its saved states feeding the
    # (unchanged) backward.
    B, L, D = shape
    x, a, b, c, dy = make_inputs(shape, dtype=dtype, seed=33)
    ref = oracle_all(x, a, b, c, dy)
    tune = (g_log2 + 1) | (8 << 16)
    bwd_tune = 7 | (8 << 8)      # the backward at its usual 64-lane rows: saved states 32 steps apart
    plan = hip_scan.make_plan(B, L, D, dtype, dtype, _lib.QSSM_FORWARD, 8, 32, tune)
    assert (plan.vec, plan.steps, plan.threads, plan.g_log2) == (8, 8, 256, g_log2)

    def run(place, out_dtype=dtype, gy=dy, keep_h=False):
        ops = [place(t) for t in (x, a, b, c)]
        y, h, ckpt, stride = hip_scan.scan_forward(*ops, out_dtype=out_dtype, want_h=keep_h, want_ckpt=not keep_h,
                                                   tune=tune, bwd_tune=bwd_tune)
        assert stride == 32 or keep_h
        dx, da, db, dc = hip_scan.scan_backward(*ops, place(gy), h=h, ckpt=ckpt, ckpt_stride=stride, tune=bwd_tune)
        assert hip_scan.workspace_status() == 0
        return {k: v.cpu() for k, v in zip(("y", "dx", "da", "db", "dc"), (y, dx, da, db, dc))}, h

    def aligned(t):
        return t.to(gpu).contiguous()

    def shifted(t):  # same values, every row 16 bytes off a 32-byte boundary but 8 elements apart in alignment
        buf = torch.zeros(B, L, D + 16, dtype=t.dtype, device=gpu)
        buf[:, :, 8:8 + D] = t.to(gpu)
        return buf[:, :, 8:8 + D]

    _check_all(run(aligned)[0], ref, TOL[dtype])
    got, h = run(aligned, keep_h=True)
    _check_all(got, ref, TOL[dtype])
    h64, _ = oracle.forward_f64(x, a, b, c)
    assert_close("h", h.cpu(), h64, 1e-5)
    _check_all(run(shifted)[0], ref, TOL[dtype])
    x32, a32, b32, c32, dy32 = make_inputs(shape, dtype=dtype, seed=33, out_dtype=torch.float32)
    got32, _ = run(aligned, out_dtype=torch.float32, gy=dy32)
    ref32 = oracle_all(x32, a32, b32, c32, dy32)
    assert_close("y", got32["y"], ref32["y"], 1e-5)
    for k in ("dx", "da", "db", "dc"):
        assert_close(k, got32[k], ref32[k], TOL[dtype])


def test_mixed_operand_dtypes_and_unbuilt_output_dtype(gpu):
    x, a, b, c, dy = make_inputs((2, 130, 8), seed=2)
    a16, c16 = a.to(torch.float16), c.to(torch.bfloat16)
    got = run_scan_with_grads(scan, x, a16, b, c16, dy.to(torch.float16), gpu, out_dtype=torch.float16)
    assert got["y"].dtype == torch.float16
    assert got["da"].dtype == torch.float16 and got["dc"].dtype == torch.bfloat16 and got["dx"].dtype == torch.float32
    ref = oracle_all(x, a16, b, c16, dy.to(torch.float16))
    for k in ("y", "dx", "da", "db", "dc"):
        assert_close(k, got[k], ref[k], 1e-2)


def test_empty_sequence_and_empty_batch(gpu):
    for shape in [(2, 0, 4), (0, 5, 4), (2, 5, 0)]:
        x = torch.zeros(shape, device=gpu, requires_grad=True)
        y = scan(x, x.detach(), x.detach(), x.detach())
        assert y.shape == torch.Size(shape)
        y.sum().backward()
        assert x.grad.shape == torch.Size(shape)
    o_a, o_x = hip_scan.block_scan_forward_3d(*(torch.zeros(1, 0, 3, device=gpu) for _ in range(3)))
    assert o_a.shape == (1, 0, 3) and o_x.shape == (1, 0, 3)


def test_non_contiguous_operands(gpu):
    shape = (3, 200, 24)
    x, a, b, c, dy = make_inputs(shape, seed=5)
    ref = oracle_all(x, a, b, c, dy)
    dev = [t.to(gpu) for t in (x, a, b, c)]
    big = torch.zeros(3, 400, 48, device=gpu)
    big[:, ::2, 8:32] = dev[0]
    views = [
        big[:, ::2, 8:32],                                      # strided in time, offset in D
        dev[1].transpose(0, 1).contiguous().transpose(0, 1),    # batch and time swapped in memory
        dev[2].permute(0, 2, 1).contiguous().permute(0, 2, 1),  # D not the fast axis: copied by the host
        dev[3][:, :, :],
    ]
    leaves = [v.detach().requires_grad_(True) for v in views]
    y = scan(*leaves)
    y.backward(dy.to(gpu).expand_as(y))
    got = {"y": y.detach().cpu()}
    for k, t in zip(("dx", "da", "db", "dc"), leaves):
        got[k] = t.grad.cpu()
    _check_all(got, ref, 1e-5)


# ---- carried state: a sequence scanned in pieces ------------------------------------------------------------

@pytest.mark.parametrize("dtype,shape,cuts", [
    (torch.float32, (2, 777, 64), [0, 1, 300, 301, 777]),
    (torch.bfloat16, (2, 1100, 264), [0, 5, 600, 1100]),
    (torch.float16, (3, 40, 6), [0, 1, 2, 3, 40]),
], ids=["f32", "bf16", "f16"])
def test_pieces_with_carried_state_equal_the_whole_scan(gpu, dtype, shape, cuts):
    x, a, b, c, dy = make_inputs(shape, dtype=dtype, seed=41)
    ref = oracle_all(x, a, b, c, dy)
    h64, _ = oracle.forward_f64(x, a, b, c)
    leaves = [t.to(gpu).requires_grad_(True) for t in (x, a, b, c)]
    state, ys = None, []
    for k0, k1 in zip(cuts[:-1], cuts[1:]):
        y, state = scan_chunk(*(t[:, k0:k1] for t in leaves), state)
        assert state.dtype == torch.float32 and state.shape == (shape[0], shape[2])
        assert_close(f"state after step {k1 - 1}", state.detach(), h64[:, k1 - 1], 1e-5)
        ys.append(y)
    y = torch.cat(ys, dim=1)
    y.backward(dy.to(gpu))
    got = {"y": y.detach().cpu()}
    for k, t in zip(("dx", "da", "db", "dc"), leaves):
        got[k] = t.grad.cpu()
    _check_all(got, ref, TOL[dtype])
    whole = run_scan_with_grads(scan, x, a, b, c, dy, gpu)
    for k in got:  # and the one-launch scan says the same
        assert_close(k + " (pieces vs whole)", got[k], whole[k].double().numpy(), TOL[dtype])


def test_seeded_random_pieces_with_carried_state_match_the_oracle(gpu):
    # A fixed-seed draw over (shape, storage, cut points, checkpoint on/off): a sequence scanned in pieces of random
    # lengths (single steps included) with the state carried through autograd must give the whole sequence's y and
    # gradients.  QSSM_RANDOM_PIECE_CASES=n draws n cases instead of 40.
    n_cases = int(os.environ.get("QSSM_RANDOM_PIECE_CASES", "40"))
    rng = np.random.default_rng(31337)
    dtypes = (torch.float32, torch.float16, torch.bfloat16)
    for case in range(n_cases):
        dtype = dtypes[case % 3]
        B = int(rng.integers(1, 4))
        L = int(rng.choice([int(rng.integers(2, 40)), int(rng.integers(40, 700)), int(rng.integers(700, 2500))]))
        D = int(rng.choice([int(rng.integers(1, 20)), 8 * int(rng.integers(1, 40)), 256 * int(rng.integers(1, 3))]))
        n_cuts = int(rng.integers(1, 6))
        cuts = sorted({0, L, *(int(v) for v in rng.integers(1, L, size=n_cuts))})
        if rng.integers(0, 3) == 0 and L > 3:      # a run of single steps somewhere
            t = int(rng.integers(1, L - 2))
            cuts = sorted({*cuts, t, t + 1, t + 2})
        checkpoint = bool(rng.integers(0, 2))
        x, a, b, c, dy = make_inputs((B, L, D), dtype=dtype, seed=5000 + case)
        if case < 12 or case % 10 == 0:
            print(f"case random pieces {case} shape=({B}, {L}, {D}) {dtype} cuts={cuts} checkpoint={checkpoint}", flush=True)
        ref = oracle_all(x, a, b, c, dy)
        h64, _ = oracle.forward_f64(x, a, b, c)
        leaves = [t.to(gpu).requires_grad_(True) for t in (x, a, b, c)]
        state, ys = None, []
        for k0, k1 in zip(cuts[:-1], cuts[1:]):
            y, state = scan_chunk(*(t[:, k0:k1] for t in leaves), state, checkpoint=checkpoint)
            ys.append(y)
        assert_close(f"final state (case {case})", state.detach(), h64[:, -1], 1e-5)
        y = torch.cat(ys, dim=1)
        y.backward(dy.to(gpu))
        assert hip_scan.workspace_status() == 0
        got = {"y": y.detach().cpu()}
        for k, t in zip(("dx", "da", "db", "dc"), leaves):
            got[k] = t.grad.cpu()
        for k in got:
            assert_close(f"{k} (case {case})", got[k], ref[k], TOL[dtype])


def test_token_by_token_generation_matches_scan(gpu):
    x, a, b, c, _ = make_inputs((2, 12, 520), dtype=torch.float16, seed=43)
    dev = [t.to(gpu) for t in (x, a, b, c)]
    whole = scan(*dev)
    state, steps = None, []
    with torch.no_grad():
        for t in range(12):
            y, state = scan_chunk(*(v[:, t:t + 1] for v in dev), state)
            steps.append(y)
    h64, y64 = oracle.forward_f64(x, a, b, c)
    assert_close("y", torch.cat(steps, 1).cpu(), y64, TOL[torch.float16])
    assert_close("y vs scan", torch.cat(steps, 1).cpu(), whole.double().cpu().numpy(), TOL[torch.float16])
    assert_close("state", state.cpu(), h64[:, -1], 1e-5)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("keep_h", [False, True], ids=["ckpt", "full_h"])
def test_carried_state_through_clustered_chains_and_its_gradients(gpu, dtype, keep_h):
    # 64-lane rows, clusters of two: the state enters the first cluster's tiles, the incoming gradient the last
    # cluster's, and both must come out right at the other end (oracle: the carried-state recurrence in float64).
    shape = (2, 700, 512)
    x, a, b, c, dy = make_inputs(shape, dtype=dtype, seed=47)
    rng = np.random.default_rng(7)
    h0 = torch.from_numpy(rng.standard_normal((shape[0], shape[2])).astype(np.float32))
    g_final = torch.from_numpy(rng.standard_normal((shape[0], shape[2])).astype(np.float32))
    _, y64, hf64 = oracle.forward_carry_f64(x, a, b, c, h0)
    ref = oracle.backward_carry_f64(x, a, b, c, dy, h0, g_final)
    tune = 7 | (8 << 8) | (2 << 28)
    ops = [t.to(gpu) for t in (x, a, b, c)]
    h_final = torch.empty(shape[0], shape[2], dtype=torch.float32, device=gpu)
    dh_init = torch.empty_like(h_final)
    y, h, ckpt, stride = hip_scan.scan_forward(*ops, out_dtype=dtype, want_h=keep_h, want_ckpt=not keep_h, tune=tune,
                                               bwd_tune=tune, h_init=h0.to(gpu), h_final=h_final)
    grads = hip_scan.scan_backward(*ops, dy.to(gpu), h=h, ckpt=ckpt, ckpt_stride=stride, tune=tune,
                                   h_init=h0.to(gpu), dh_final=g_final.to(gpu), dh_init=dh_init)
    assert hip_scan.workspace_status() == 0
    assert_close("y", y.cpu(), y64, TOL[dtype])
    assert_close("h_final", h_final.cpu(), hf64, 1e-5)
    for name, got, want in zip(("dx", "da", "db", "dc"), grads, ref[:4]):
        assert_close(name, got.cpu(), want, TOL[dtype])
    assert_close("dh_init", dh_init.cpu(), ref[4], 1e-5)


def test_carried_state_argument_errors_and_empty_piece(gpu):
    x, a, b, c, _ = make_inputs((2, 8, 4), seed=3)
    dev = [t.to(gpu) for t in (x, a, b, c)]
    with pytest.raises(ValueError):
        scan_chunk(*dev, torch.zeros(2, 5, device=gpu))
    with pytest.raises(ValueError):
        hip_scan.scan_forward(*dev, out_dtype=torch.float32, h_init=torch.zeros(2, 4, device=gpu, dtype=torch.float16))
    st = torch.arange(8, dtype=torch.float32, device=gpu).reshape(2, 4)
    y, out = scan_chunk(*(t[:, :0] for t in dev), st)
    assert y.shape == (2, 0, 4) and torch.equal(out, st)
    # CPU tensors take the sequential path with the same meaning
    yc, sc = scan_chunk(x[:, :5], a[:, :5], b[:, :5], c[:, :5])
    yc2, sc2 = scan_chunk(x[:, 5:], a[:, 5:], b[:, 5:], c[:, 5:], sc)
    h64, y64 = oracle.forward_f64(x, a, b, c)
    assert_close("cpu pieces", torch.cat([yc, yc2], 1), y64, 1e-5)
    assert_close("cpu state", sc2, h64[:, -1], 1e-5)


# ---- launch numbering: by the caller, by the library, and under graph replay --------------------------------

def test_c_abi_with_caller_counted_epochs(gpu):
    # the raw C ABI as a caller outside this package would use it: own control block and workspace, epochs 1, 2, 3 from the caller
    import ctypes
    lib = _lib.load()
    shape = (2, 900, 256)
    x, a, b, c, dy = make_inputs(shape, dtype=torch.bfloat16, seed=51)
    ref = oracle_all(x, a, b, c, dy)
    ops = [t.to(gpu).contiguous() for t in (x, a, b, c, dy)]
    B, L, D = shape
    tune = 7 | (8 << 8)
    bwd = hip_scan.make_plan(B, L, D, torch.bfloat16, torch.bfloat16, _lib.QSSM_BACKWARD, 8, 0, tune)
    fwd = hip_scan.make_plan(B, L, D, torch.bfloat16, torch.bfloat16, _lib.QSSM_FORWARD, 8, bwd.seg_len, tune)
    assert fwd.n_seg > 1 and bwd.n_seg > 1
    control = torch.zeros(max(fwd.control_bytes, bwd.control_bytes), dtype=torch.uint8, device=gpu)
    workspace = torch.zeros(max(fwd.workspace_bytes, bwd.workspace_bytes), dtype=torch.uint8, device=gpu)
    stream = torch.cuda.current_stream().cuda_stream
    st = lambda t: _lib.Strides(t.stride(0), t.stride(1))
    none = _lib.Strides(0, 0)
    epoch = 0
    for _ in range(3):  # same buffers, next epochs: old words must read as "not there yet"
        y = torch.empty(shape, dtype=torch.bfloat16, device=gpu)
        ckpt = torch.empty(B, fwd.n_ckpt, D, dtype=torch.float32, device=gpu)
        grads = [torch.empty(shape, dtype=torch.bfloat16, device=gpu) for _ in range(4)]
        epoch += 1
        _lib.check(lib.qssm_scan_forward(
            ctypes.byref(fwd), ops[0].data_ptr(), st(ops[0]), ops[1].data_ptr(), st(ops[1]), ops[2].data_ptr(), st(ops[2]),
            ops[3].data_ptr(), st(ops[3]), y.data_ptr(), st(y), None, none, ckpt.data_ptr(),
            control.data_ptr(), control.numel(), workspace.data_ptr(), workspace.numel(), epoch, stream))
        epoch += 1
        _lib.check(lib.qssm_scan_backward(
            ctypes.byref(bwd), ops[0].data_ptr(), st(ops[0]), ops[1].data_ptr(), st(ops[1]), ops[2].data_ptr(), st(ops[2]),
            ops[3].data_ptr(), st(ops[3]), ops[4].data_ptr(), st(ops[4]), None, none, ckpt.data_ptr(),
            grads[0].data_ptr(), st(grads[0]), grads[1].data_ptr(), st(grads[1]), grads[2].data_ptr(), st(grads[2]),
            grads[3].data_ptr(), st(grads[3]),
            control.data_ptr(), control.numel(), workspace.data_ptr(), workspace.numel(), epoch, stream))
        status = ctypes.c_int32(-1)
        _lib.check(lib.qssm_control_status(control.data_ptr(), stream, ctypes.byref(status)))
        assert status.value == 0
        got = {"y": y.cpu(), "dx": grads[0].cpu(), "da": grads[1].cpu(), "db": grads[2].cpu(), "dc": grads[3].cpu()}
        _check_all(got, ref, TOL[torch.bfloat16])
    assert int(control.view(torch.int32)[1]) == 0   # the library's own count was never used


def test_dirty_control_block_is_reported_and_zero_fill_recovers(gpu):
    # A control block that is not zero on entry (here: ticket counters far past the end) makes every workgroup leave
    # at once with status 2 instead of touching memory it does not own; after qssm_zero_fill the same buffers work.
    import ctypes
    lib = _lib.load()
    shape = (1, 600, 256)
    x, a, b, c, dy = make_inputs(shape, dtype=torch.float16, seed=71)
    ops = [t.to(gpu).contiguous() for t in (x, a, b, c)]
    B, L, D = shape
    plan = hip_scan.make_plan(B, L, D, torch.float16, torch.float16, _lib.QSSM_FORWARD, 8, 0, 7 | (8 << 8))
    assert plan.n_seg > 1
    control = torch.zeros(plan.control_bytes, dtype=torch.uint8, device=gpu)
    workspace = torch.zeros(plan.workspace_bytes, dtype=torch.uint8, device=gpu)
    control.view(torch.int32)[16:] = 0x7fff0000           # every ticket slot; the status word stays zero
    stream = torch.cuda.current_stream().cuda_stream
    st = lambda t: _lib.Strides(t.stride(0), t.stride(1))
    none = _lib.Strides(0, 0)

    def launch(epoch):
        y = torch.zeros(shape, dtype=torch.float16, device=gpu)
        _lib.check(lib.qssm_scan_forward(
            ctypes.byref(plan), ops[0].data_ptr(), st(ops[0]), ops[1].data_ptr(), st(ops[1]), ops[2].data_ptr(), st(ops[2]),
            ops[3].data_ptr(), st(ops[3]), y.data_ptr(), st(y), None, none, None,
            control.data_ptr(), control.numel(), workspace.data_ptr(), workspace.numel(), epoch, stream))
        status = ctypes.c_int32(-1)
        _lib.check(lib.qssm_control_status(control.data_ptr(), stream, ctypes.byref(status)))
        return y, status.value

    y, status = launch(1)
    assert status == 2 and torch.isnan(y).all()           # every tile of the output was poisoned, nothing else ran
    _lib.check(lib.qssm_zero_fill(control.data_ptr(), control.numel(), stream))
    y, status = launch(2)
    assert status == 0
    _, y64 = oracle.forward_f64(x, a, b, c)
    assert_close("y", y.cpu(), y64, TOL[torch.float16])


def test_failed_launch_is_reported_through_scan_and_the_stream_recovers(gpu):
    # The same dirty control block, this time under the public API: the launch poisons its outputs, the status
    # check behind it (period 1 here) brings the word to the host, the next scan() on the stream raises
    # ScanLaunchError after resetting the buffers, and the one after that is correct again.  Every kernel exits
    # normally throughout.
    shape = (2, 700, 256)
    x, a, b, c, dy = make_inputs(shape, dtype=torch.bfloat16, seed=72)
    ops = [t.to(gpu) for t in (x, a, b, c)]
    old = hip_scan.set_status_check_period(1)
    try:
        y = scan(*ops)                                     # the buffers of this stream exist and are large enough
        torch.cuda.synchronize()
        stream = torch.cuda.current_stream(gpu).cuda_stream
        buf = hip_scan._buffers[(gpu.index, stream, False)]
        buf.control.view(torch.int32)[16:] = 0x7fff0000    # every ticket slot; the status word stays zero
        y = scan(*ops)
        torch.cuda.synchronize()
        assert torch.isnan(y).all()
        with pytest.raises(hip_scan.ScanLaunchError) as err:
            scan(*ops)
        assert err.value.status == 2
        got = run_scan_with_grads(scan, x, a, b, c, dy, gpu)
        assert hip_scan.workspace_status() == 0
        _check_all(got, oracle_all(x, a, b, c, dy), TOL[torch.bfloat16])
    finally:
        hip_scan.set_status_check_period(old)


def test_buffers_of_a_recorded_graph_outlive_a_larger_shape(gpu):
    # A graph recorded for a small shape holds the addresses of its control block and workspace.  A larger shape on
    # the same stream needs larger buffers: the old pair must stay alive and untouched (it is retired, not freed),
    # and the old graph must still replay correctly afterwards.
    small, large = (1, 600, 256), (4, 4096, 1024)
    side = torch.cuda.Stream()
    xs = [t.to(gpu).contiguous() for t in make_inputs(small, dtype=torch.bfloat16, seed=81)]
    xl = [t.to(gpu).contiguous() for t in make_inputs(large, dtype=torch.bfloat16, seed=82)]

    def run(ops):
        y, _, ckpt, stride = hip_scan.scan_forward(*ops[:4], out_dtype=torch.bfloat16)
        return (y,) + tuple(hip_scan.scan_backward(*ops, ckpt=ckpt, ckpt_stride=stride))

    with torch.cuda.stream(side):
        with hip_scan.device_counted_launches():
            run(xs)
        side.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            outs = run(xs)
        key = (gpu.index, side.cuda_stream, True)
        before = hip_scan._buffers[key]
        old_ptrs = (before.ctl_ptr, before.ws_ptr)
        assert before.captured
        retired = len(hip_scan._retired)
        with hip_scan.device_counted_launches():
            big = run(xl)                                   # needs a larger workspace than the recorded pair
        side.synchronize()
        after = hip_scan._buffers[key]
        assert after.ws_ptr != old_ptrs[1] and len(hip_scan._retired) == retired + 2
        assert {t.data_ptr() for t in hip_scan._retired[-2:]} == set(old_ptrs)
        fresh = make_inputs(small, dtype=torch.bfloat16, seed=83)
        for dst, src in zip(xs, fresh):
            dst.copy_(src.to(gpu))
        for _ in range(2):
            graph.replay()
            side.synchronize()
            got = dict(zip(("y", "dx", "da", "db", "dc"), (t.cpu() for t in outs)))
            _check_all(got, oracle_all(*fresh), TOL[torch.bfloat16])
        assert hip_scan.workspace_status() == 0
        ref = oracle_all(*make_inputs(large, dtype=torch.bfloat16, seed=82))
        _check_all(dict(zip(("y", "dx", "da", "db", "dc"), (t.cpu() for t in big))), ref, TOL[torch.bfloat16])


def test_captured_launches_replay_with_new_inputs(gpu):
    # Forward and backward captured in one graph; every replay reads its epoch from device memory, so tiles of a
    # replay never mistake the previous replay's words for their neighbours'.  Replays alternate with eager launches
    # on the same buffers and with new input values, and each one is checked against the eager result.
    shape = (2, 1500, 512)
    tune = 7 | (8 << 8)
    side = torch.cuda.Stream()
    sets = [make_inputs(shape, dtype=torch.bfloat16, seed=60 + k) for k in range(3)]
    static = [t.to(gpu).contiguous() for t in sets[0]]

    def run():
        y, _, ckpt, stride = hip_scan.scan_forward(*static[:4], out_dtype=torch.bfloat16, tune=tune, bwd_tune=tune)
        return (y,) + tuple(hip_scan.scan_backward(*static, ckpt=ckpt, ckpt_stride=stride, tune=tune))

    import warnings
    with torch.cuda.stream(side):
        with warnings.catch_warnings():
            warnings.simplefilter("ignore")     # torch warns that the graph of the refused recording is empty
            with pytest.raises(RuntimeError):   # recording the very first launch would have to allocate
                with torch.cuda.graph(torch.cuda.CUDAGraph(), stream=side):
                    run()
        with hip_scan.device_counted_launches():   # warm-up: the buffers of captured launches exist afterwards
            run()
        run()
        side.synchronize()
        plan = hip_scan.make_plan(*shape, torch.bfloat16, torch.bfloat16, _lib.QSSM_BACKWARD, 8, 0, tune)
        assert plan.n_seg > 1 and plan.n_super > 1
        graph = torch.cuda.CUDAGraph()
        with warnings.catch_warnings():
            warnings.simplefilter("error")      # the real recording must not be empty
            with torch.cuda.graph(graph, stream=side):
                outs = run()
        for t in outs:
            t.fill_(float("nan"))               # whatever the outputs hold later, a replay wrote it
    for k in (1, 2, 0, 1):
        for dst, src in zip(static, sets[k]):
            dst.copy_(src.to(gpu))
        with torch.cuda.stream(side):
            side.wait_stream(torch.cuda.current_stream())
            eager = [t.clone() for t in run()]      # eager launch between the replays, same buffers
            graph.replay()
            side.synchronize()
            assert hip_scan.workspace_status() == 0
        ref = oracle_all(*sets[k])
        got = dict(zip(("y", "dx", "da", "db", "dc"), (t.cpu() for t in outs)))
        _check_all(got, ref, TOL[torch.bfloat16])
        for name, g_, e_ in zip(("y", "dx", "da", "db", "dc"), outs, eager):
            assert torch.equal(g_, e_), name


# ---- knobs must not change results ---------------------------------------------------------------------

def test_checkpoint_false_keeps_fp32_states_and_matches(gpu):
    x, a, b, c, dy = make_inputs((2, 900, 40), dtype=torch.float16, seed=6)
    on = run_scan_with_grads(scan, x, a, b, c, dy, gpu, checkpoint=True)
    off = run_scan_with_grads(scan, x, a, b, c, dy, gpu, checkpoint=False)
    assert torch.equal(on["y"], off["y"])
    ref = oracle_all(x, a, b, c, dy)
    _check_all(off, ref, TOL[torch.float16])
    # the saved states themselves
    leaves = [t.to(gpu).requires_grad_(True) for t in (x, a, b, c)]
    y = scan(*leaves, checkpoint=False)
    h_saved = y.grad_fn.h_saved
    assert h_saved is not None and h_saved.dtype == torch.float32
    h64, _ = oracle.forward_f64(x, a, b, c)
    assert_close("h_saved", h_saved, h64, 1e-5)
    y2 = scan(*leaves, checkpoint=True)
    assert y2.grad_fn.h_saved is None


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
def test_block_l_and_tiles_do_not_change_results(gpu, dtype):
    x, a, b, c, dy = make_inputs((4, 600, 48), dtype=dtype, seed=7)
    base = run_scan_with_grads(scan, x, a, b, c, dy, gpu)
    for block_l in (1, 7, 16, 256, 4096):
        other = run_scan_with_grads(scan, x, a, b, c, dy, gpu, block_l=block_l, tile_b=1, tile_d=16)
        for k in base:
            assert torch.equal(base[k], other[k]), (block_l, k)
    # One launch per tile: batch tiles keep the launch geometry, so results stay bitwise equal; feature tiles
    # narrower than a strip change how lanes split the time axis, so results agree to rounding.
    ref = oracle_all(x, a, b, c, dy)
    old = honor_tiles(True)
    try:
        for tb, td in ((1, None), (3, None), (1, 16), (3, 20), (None, 8)):
            tiled = run_scan_with_grads(scan, x, a, b, c, dy, gpu, tile_b=tb, tile_d=td)
            if td is None:
                for k in base:
                    assert torch.equal(base[k], tiled[k]), (tb, td, k)
            _check_all(tiled, ref, TOL[dtype])
    finally:
        honor_tiles(old)


def test_seeded_random_tiles_launched_one_by_one(gpu):
    # With one launch per (tile_b, tile_d) tile, as the reference loops (quick_ssm/scan_interface.py:88-103): a
    # fixed-seed draw over shapes, storage, odd tile sizes and checkpoint on/off; every tile is a strided view that
    # may start off the 16-byte grid.  QSSM_RANDOM_TILE_CASES=n draws n cases instead of 30.
    n_cases = int(os.environ.get("QSSM_RANDOM_TILE_CASES", "30"))
    rng = np.random.default_rng(2718)
    pairs = [(torch.float32, torch.float32), (torch.float16, torch.float16), (torch.bfloat16, torch.bfloat16),
             (torch.bfloat16, torch.float32)]
    old = honor_tiles(True)
    try:
        for case in range(n_cases):
            dtype, out_dtype = pairs[case % len(pairs)]
            B = int(rng.integers(1, 6))
            L = int(rng.choice([int(rng.integers(1, 50)), int(rng.integers(50, 900))]))
            D = int(rng.choice([int(rng.integers(1, 30)), 8 * int(rng.integers(1, 40)), 256 * int(rng.integers(1, 3))]))
            tile_b = [None, 1, 2, 3][int(rng.integers(0, 4))]
            tile_d = [None, 1, 7, 8, 13, 100, 256][int(rng.integers(0, 7))]
            checkpoint = bool(rng.integers(0, 2))
            x, a, b, c, dy = make_inputs((B, L, D), dtype=dtype, seed=9000 + case, out_dtype=out_dtype)
            if case < 10 or case % 10 == 0:
                print(f"case random tiles {case} shape=({B}, {L}, {D}) {dtype}->{out_dtype} tile_b={tile_b} tile_d={tile_d} "
                      f"checkpoint={checkpoint}", flush=True)
            got = run_scan_with_grads(scan, x, a, b, c, dy, gpu, tile_b=tile_b, tile_d=tile_d, checkpoint=checkpoint,
                                      out_dtype=out_dtype)
            assert hip_scan.workspace_status() == 0
            ref = oracle_all(x, a, b, c, dy)
            assert_close(f"y (case {case})", got["y"], ref["y"], TOL[out_dtype])
            for k in ("dx", "da", "db", "dc"):
                assert_close(f"{k} (case {case})", got[k], ref[k], TOL[dtype])
    finally:
        honor_tiles(old)


def test_launch_geometry_does_not_change_results_beyond_rounding(gpu):
    # every lanes-per-row / steps-per-lane geometry must agree with the oracle
    x, a, b, c, dy = make_inputs((2, 1100, 72), seed=8)
    ref = oracle_all(x, a, b, c, dy)
    dev = [t.to(gpu) for t in (x, a, b, c)]  # L=1100: up to 138 tiles per chain, clusters of 1..32
    for threads_code, g_log2, steps, cluster_code in [
        (1, 0, 8, 1), (1, 2, 4, 2), (1, 4, 8, 3), (1, 5, 4, 4), (1, 6, 8, 1), (1, 8, 4, 2),
        (2, 3, 8, 2), (2, 6, 4, 3), (2, 9, 8, 1), (3, 4, 4, 2), (3, 6, 8, 3), (3, 5, 4, 4), (3, 10, 4, 1),
        (1, 4, 4, 5), (1, 5, 8, 6), (1, 2, 4, 6), (2, 4, 4, 5),      # clusters of 16 and 32 tiles: more tiles than lane groups
    ]:
        tune = (g_log2 + 1) | (steps << 8) | (threads_code << 24) | (cluster_code << 28)
        y, _, ckpt, stride = hip_scan.scan_forward(*dev, out_dtype=torch.float32, tune=tune, bwd_tune=tune)
        grads = hip_scan.scan_backward(*dev, dy.to(gpu), ckpt=ckpt, ckpt_stride=stride, tune=tune)
        got = dict(zip(("y", "dx", "da", "db", "dc"), (y,) + grads))
        print(f"geometry threads={256 << (threads_code - 1)} g_log2={g_log2} steps={steps} "
              f"cluster={1 << (cluster_code - 1)} ckpt_stride={stride}", flush=True)
        _check_all(got, ref, 1e-5)
    assert hip_scan.workspace_status() == 0


def test_a_forward_that_no_backward_follows_saves_no_states(gpu, monkeypatch):
    # inference (no operand wants a gradient, or torch.no_grad()): same y bit for bit, no saved states, and the launch
    # is planned to stream its operands past the caches (plan.keep_tiles = 0)
    seen = []
    real = hip_scan.scan_forward

    def spy(*args, **kw):
        out = real(*args, **kw)
        seen.append((kw.get("want_h"), kw.get("want_ckpt"), out[2]))
        return out

    monkeypatch.setattr(hip_scan, "scan_forward", spy)
    x, a, b, c, _ = make_inputs((2, 700, 256), dtype=torch.bfloat16, seed=3)
    ops = [t.to(gpu) for t in (x, a, b, c)]
    with torch.no_grad():
        y0 = scan(*ops)
    assert seen[-1][:2] == (False, False) and seen[-1][2] is None and y0.grad_fn is None
    y1 = scan(*ops)                                   # grad mode on, but no operand requires a gradient
    assert seen[-1][:2] == (False, False) and seen[-1][2] is None
    leaves = [t.clone().requires_grad_(True) for t in ops]
    y2 = scan(*leaves)
    assert seen[-1][:2] == (False, True) and seen[-1][2] is not None
    assert torch.equal(y0, y1) and torch.equal(y0, y2.detach())
    with torch.no_grad():
        y3, state = scan_chunk(*ops, state=None)
    assert seen[-1][:2] == (False, False) and torch.equal(y3, y0)
    assert hip_scan.workspace_status() == 0


def test_partial_gradients(gpu):
    x, a, b, c, dy = make_inputs((2, 400, 16), seed=9)
    ref = oracle_all(x, a, b, c, dy)
    xs = x.to(gpu).requires_grad_(True)
    cs = c.to(gpu).requires_grad_(True)
    y = scan(xs, a.to(gpu), b.to(gpu), cs)
    y.backward(dy.to(gpu))
    assert_close("dx", xs.grad, ref["dx"], 1e-5)
    assert_close("dc", cs.grad, ref["dc"], 1e-5)


def test_float64_operands_run_in_fp32_and_come_back_as_float64(gpu):
    # quick_ssm/triton_forwards.py:7-16 casts whatever float type it gets to fp32; y comes back in x.dtype
    # (scan_interface.py:200) and every gradient in its operand's dtype (:148-151)
    x, a, b, c, dy = (t.double() for t in make_inputs((2, 300, 24), seed=21))
    ref = oracle_all(x, a, b, c, dy)
    got = run_scan_with_grads(scan, x, a, b, c, dy, gpu)
    for k in ("y", "dx", "da", "db", "dc"):
        assert got[k].dtype == torch.float64, k
        assert_close(k, got[k], ref[k], 1e-5)
    # mixed storage: the operands meet in the widest type among them, each gradient returns in its own
    leaves = [t.to(gpu).requires_grad_(True) for t in (x.half(), a.float(), b.bfloat16(), c.double())]
    y = scan(*leaves, out_dtype=torch.float32)
    y.backward(dy.to(gpu).float())
    assert y.dtype == torch.float32
    for t in leaves:
        assert t.grad.dtype == t.dtype and bool(torch.isfinite(t.grad).all())
    ref = oracle_all(x.half().double(), a.float().double(), b.bfloat16().double(), c, dy.float().double())
    assert_close("y", y, ref["y"], 1e-5)
    assert_close("da", leaves[1].grad, ref["da"], 1e-5)
    assert_close("dx", leaves[0].grad, ref["dx"], 1e-2)


def test_argument_errors(gpu):
    x = torch.zeros(2, 8, 4, device=gpu)
    with pytest.raises(ValueError):
        scan(x, x[:, :4], x, x)
    with pytest.raises(ValueError):
        scan(x, x, x, x, backend="cuda")
    with pytest.raises(RuntimeError):
        scan(x.cpu(), x.cpu(), x.cpu(), x.cpu(), backend="triton")


# ---- the headline shapes ---------------------------------------------------------------------------------

def _rows_check(got, ops, dy, rows, tol):
    """Compare whole batch rows (all of L and D) of every output with the oracle."""
    x, a, b, c = ops
    for r in rows:
        sl = slice(r, r + 1)
        ref = oracle_all(x[sl], a[sl], b[sl], c[sl], dy[sl])
        for k in ("y", "dx", "da", "db", "dc"):
            assert_close(f"{k}[row {r}]", got[k][sl], ref[k], tol)


def test_config1_bf16_full_shape(gpu):
    # B=8 L=4096 D=2048 bf16: every batch row of every output against the oracle, plus the properties that hold at
    # any size
    shape = (8, 4096, 2048)
    x, a, b, c, dy = make_inputs(shape, dtype=torch.bfloat16, seed=0)
    print("case config1 full shape", flush=True)
    got = run_scan_with_grads(scan, x, a, b, c, dy, gpu, block_l=256, checkpoint=True)
    assert hip_scan.workspace_status() == 0
    _rows_check(got, (x, a, b, c), dy, range(shape[0]), TOL[torch.bfloat16])
    assert torch.all(got["da"][:, 0, :] == 0)
    for k in got:
        assert torch.isfinite(got[k].float()).all(), k
    # dx * x and db * b are the same number b*x*dH up to one rounding each
    lhs = got["dx"].float() * x.float()
    rhs = got["db"].float() * b.float()
    assert torch.allclose(lhs, rhs, rtol=2e-2, atol=1e-6)
    # linearity in dy: doubling dy doubles every gradient exactly (power of two)
    twice = run_scan_with_grads(scan, x, a, b, c, dy * 2, gpu)
    for k in ("dx", "da", "db", "dc"):
        assert torch.equal(twice[k].float(), got[k].float() * 2), k
    assert hip_scan.workspace_status() == 0


@pytest.mark.timeout(600)
def test_tensors_past_4_gib_reach_their_last_batch_row(gpu):
    # 5 x 8192 x 65536 bf16 is 5 GiB per tensor: the last batch row starts 2^31 elements = 2^32 bytes into each of
    # them, past what 32-bit offsets reach.  Operands are drawn on the device; windows of columns of the first, the
    # fourth and the last row go to the float64 oracle.
    B, L, D = 5, 8192, 65536
    free, _ = torch.cuda.mem_get_info(gpu)
    if free < (80 << 30):
        pytest.skip("needs 80 GiB of free device memory")
    print("case tensors of 5 GiB", flush=True)
    gen = torch.Generator(device=gpu).manual_seed(7)

    def new():
        return torch.empty((B, L, D), dtype=torch.bfloat16, device=gpu)

    x = new().normal_(generator=gen)
    a = new().uniform_(0.9, 1.0, generator=gen)
    b = new().normal_(0.0, 0.1, generator=gen)
    c = new().uniform_(0.0, 1.0, generator=gen)
    dy = new().normal_(generator=gen)
    leaves = [t.requires_grad_(True) for t in (x, a, b, c)]
    y = scan(*leaves, block_l=256, checkpoint=True)
    y.backward(dy)
    assert hip_scan.workspace_status() == 0
    got = {"y": y.detach(), "dx": x.grad, "da": a.grad, "db": b.grad, "dc": c.grad}
    for k, t in got.items():
        assert t.shape == (B, L, D) and bool(torch.isfinite(t).all()), k
    for row in (0, 3, B - 1):
        for c0 in (0, D // 2 - 32, D - 64):
            win = (slice(row, row + 1), slice(None), slice(c0, c0 + 64))
            ref = oracle_all(*(t.detach()[win].cpu() for t in (x, a, b, c, dy)))
            for k in ("y", "dx", "da", "db", "dc"):
                assert_close(f"{k}[row {row}, cols {c0}:{c0 + 64}]", got[k][win].cpu(), ref[k], TOL[torch.bfloat16])
    del got, y, leaves, x, a, b, c, dy
    torch.cuda.empty_cache()


@pytest.mark.timeout(600)
def test_config2_fp16_long_sequence_near_unit_decay(gpu):
    # B=1 L=65536 D=4096 fp16, a in [0.99, 1], block_l=1024, tile_d=1024: every column over all of L, the oracle
    # taking 512 columns at a time
    shape = (1, 65536, 4096)
    x, a, b, c, dy = make_inputs(shape, dtype=torch.float16, seed=1, a_lo=0.99, a_span=0.01)
    print("case config2 full shape", flush=True)
    got = run_scan_with_grads(scan, x, a, b, c, dy, gpu, block_l=1024, checkpoint=True, tile_d=1024)
    assert hip_scan.workspace_status() == 0
    for k in got:
        assert torch.isfinite(got[k].float()).all(), k
    for c0 in range(0, shape[2], 512):
        cols = slice(c0, c0 + 512)
        print(f"  columns {c0}:{c0 + 512}", flush=True)
        ref = oracle_all(x[..., cols], a[..., cols], b[..., cols], c[..., cols], dy[..., cols])
        for k in ("y", "dx", "da", "db", "dc"):
            assert_close(f"{k}[cols {cols.start}:{cols.stop}]", got[k][..., cols], ref[k], TOL[torch.float16])


@pytest.mark.timeout(600)
def test_config3_scan_at_its_own_shape(gpu):
    # the scan inside the config-3 layer: B=16 L=2048 D=4096, fp16 operands, fp32 y and dy, checkpoint=True.
    # Every batch row against the oracle: 1e-5 for y (fp32 storage), 1e-2 for the gradients (fp16 storage).
    shape = (16, 2048, 4096)
    x, a, b, c, dy = make_inputs(shape, dtype=torch.float16, seed=3, out_dtype=torch.float32)
    print("case config3 scan full shape", flush=True)
    got = run_scan_with_grads(scan, x, a, b, c, dy, gpu, block_l=256, checkpoint=True, out_dtype=torch.float32)
    assert hip_scan.workspace_status() == 0
    assert got["y"].dtype == torch.float32 and got["dx"].dtype == torch.float16
    for r in range(shape[0]):
        sl = slice(r, r + 1)
        ref = oracle_all(x[sl], a[sl], b[sl], c[sl], dy[sl])
        assert_close(f"y[row {r}]", got["y"][sl], ref["y"], TOL[torch.float32])
        for k in ("dx", "da", "db", "dc"):
            assert_close(f"{k}[row {r}]", got[k][sl], ref[k], TOL[torch.float16])
    assert torch.all(got["da"][:, 0, :] == 0)


def _layer_oracle_f64(layer, xin, gout, gemm_device):
    """float64 composition of the committed oracles for one SSM layer step (quick_ssm/layers.py:60-107):
    rmsnorm_oracle -> float64 projections -> gates_oracle -> scan oracle -> float64 out projection (+ residual),
    and the same chain backwards.  The operands of the scan are rounded to `compute_dtype` where the layer rounds
    them (layers.py:85-88), so the scan oracle sees the stored values the kernels see up to the rounding of
    values within an ulp of a tie.  The matrix products (torch's library GEMM on both sides of the comparison, not
    part of the path under test) run in float64 on `gemm_device`; everything elementwise runs on the CPU oracles.
    """
    from oracle import gates_oracle, rmsnorm_oracle

    f64 = torch.float64
    P = {n: p.detach().to("cpu", f64) for n, p in layer.named_parameters()}
    B, L, H = xin.shape
    S = layer.state_size_dim
    x64 = xin.detach().to("cpu", f64)
    eps = layer.pre_norm.eps
    u = torch.from_numpy(rmsnorm_oracle.rmsnorm_forward_f64(x64.numpy(), P["pre_norm.weight"].numpy(), eps))

    def mm(lhs, rhs):
        return (lhs.to(gemm_device) @ rhs.to(gemm_device)).cpu()

    u2 = u.reshape(-1, H)
    pre = {n: mm(u2, P[f"{n}.weight"].t()) for n in ("A_proj", "B_proj", "C_proj_a", "C_proj_b", "D_proj")}
    pre["A_proj"] = pre["A_proj"] + P["A_proj.bias"]
    ga, gx, gc, gb = gates_oracle.gates_forward_f64(pre["A_proj"].numpy(), pre["B_proj"].numpy(),
                                                    pre["C_proj_a"].numpy(), pre["C_proj_b"].numpy(),
                                                    pre["D_proj"].numpy())
    cd = layer.compute_dtype
    ops = [torch.from_numpy(t).to(cd).reshape(B, L, S) for t in (gx, ga, gb, gc)]   # x, a, b, c as stored
    _, y = oracle.forward_f64(*ops)
    y2 = torch.from_numpy(y).reshape(-1, S)
    out = (mm(y2, P["out_proj.weight"].t()) + P["out_proj.bias"]).reshape(B, L, H) + x64

    g2 = gout.detach().to("cpu", f64).reshape(-1, H)
    grads = {"out_proj.bias": g2.sum(0), "out_proj.weight": mm(g2.t(), y2)}
    dy = mm(g2, P["out_proj.weight"])                                             # [rows, S]
    dx_s, da_s, db_s, dc_s = oracle.backward_f64(*ops, dy.reshape(B, L, S).float())
    # the scan's dy is the fp32 tensor autograd hands it; the oracle takes stored values
    dpre = gates_oracle.gates_backward_f64(da_s.reshape(-1, S), dx_s.reshape(-1, S), dc_s.reshape(-1, S),
                                           db_s.reshape(-1, S), pre["A_proj"].numpy(), pre["C_proj_a"].numpy(),
                                           pre["C_proj_b"].numpy(), pre["D_proj"].numpy())
    du = torch.zeros_like(u2)
    for n, g in zip(("A_proj", "B_proj", "C_proj_a", "C_proj_b", "D_proj"), dpre):
        g = torch.from_numpy(np.ascontiguousarray(g))
        grads[f"{n}.weight"] = mm(g.t(), u2)
        if n == "A_proj":
            grads["A_proj.bias"] = g.sum(0)
        du += mm(g, P[f"{n}.weight"])
    dxn, dw = rmsnorm_oracle.rmsnorm_backward_f64(du.reshape(B, L, H).numpy(), x64.numpy(),
                                                  P["pre_norm.weight"].numpy(), eps)
    grads["pre_norm.weight"] = torch.from_numpy(dw)
    dx = torch.from_numpy(dxn) + gout.detach().to("cpu", f64)
    return out, dx, grads


def _run_layer(mod, inp, gout):
    mod.zero_grad(set_to_none=True)
    inp = inp.clone().requires_grad_(True)
    out = mod(inp)
    out.backward(gout.to(inp.device))
    grads = {n: p.grad.detach().cpu().clone() for n, p in mod.named_parameters()}
    return out.detach().cpu(), inp.grad.detach().cpu(), grads


def test_ssm_layer_small_matches_oracle_composition(gpu):
    # the layer's whole step at a size the CPU does in a second, against the float64 composition of the oracles
    from quick_ssm_amd.layers import SSM

    torch.manual_seed(0)
    layer = SSM(hidden_size=64, state_size_mult=4.0, compute_dtype=torch.float16, dtype=torch.float32).to(gpu)
    xin = torch.randn(2, 192, 64)
    gout = torch.randn(2, 192, 64)
    out, dx, grads = _run_layer(layer, xin.to(gpu), gout)
    assert hip_scan.workspace_status() == 0
    ref_out, ref_dx, ref_grads = _layer_oracle_f64(layer, xin, gout, "cpu")
    assert_close("layer out", out, ref_out.numpy(), 1e-2)
    assert_close("layer dx", dx, ref_dx.numpy(), 1e-2)
    for n in ref_grads:
        assert_close(f"grad {n}", grads[n], ref_grads[n].numpy(), 1e-2)


@pytest.mark.timeout(600)
def test_seeded_random_layer_shapes_match_the_oracle_composition(gpu):
    # A fixed-seed draw over layer sizes, batch, sequence length (down to a single step) and compute dtype, fp32
    # parameters as the reference creates them: whichever route the layer takes (gated scan over one wide projection
    # or over five, gate pass + plain scan for narrow states) must meet the float64 composition of the oracles.
    # QSSM_RANDOM_LAYER_CASES=n draws n cases instead of 40.
    from quick_ssm_amd.layers import SSM

    n_cases = int(os.environ.get("QSSM_RANDOM_LAYER_CASES", "40"))
    rng = np.random.default_rng(977)
    computes = (torch.float16, torch.bfloat16, torch.float32)
    for case in range(n_cases):
        compute = computes[case % 3]
        hidden = int(rng.choice([32, 64, 96, 128, 256]))
        mult = float(rng.choice([1.0, 2.0, 4.0]))
        B = int(rng.integers(1, 4))
        L = int(rng.choice([int(rng.integers(1, 12)), int(rng.integers(12, 300)), int(rng.integers(300, 1200))]))
        torch.manual_seed(500 + case)
        layer = SSM(hidden_size=hidden, state_size_mult=mult, compute_dtype=compute, dtype=torch.float32).to(gpu)
        g = torch.Generator(device="cpu").manual_seed(600 + case)
        xin = torch.randn(B, L, hidden, generator=g)
        gout = torch.randn(B, L, hidden, generator=g)
        print(f"case random layer {case} B={B} L={L} hidden={hidden} state={int(hidden * mult)} compute={compute}", flush=True)
        out, dx, grads = _run_layer(layer, xin.to(gpu), gout)
        assert hip_scan.workspace_status() == 0
        ref_out, ref_dx, ref_grads = _layer_oracle_f64(layer, xin, gout, "cpu")
        tol = 1e-4 if compute == torch.float32 else 1e-2
        assert_close(f"layer out (case {case})", out, ref_out.numpy(), tol)
        assert_close(f"layer dx (case {case})", dx, ref_dx.numpy(), tol)
        for n in ref_grads:
            assert_close(f"grad {n} (case {case})", grads[n], ref_grads[n].numpy(), tol)


@pytest.mark.timeout(900)
def test_config3_ssm_layer_at_its_own_shape(gpu):
    # SSM(hidden 1024, state 4096), fp32 parameters, fp16 scan operands, fp32 scan output, B=16 L=2048, seeded
    # default initialisation (quick_ssm/layers.py:31-58) and N(0,1) activations: output, input gradient and every
    # parameter gradient against the float64 composition of the oracles (float64 GEMMs on the GPU: 5 TFLOP).
    from quick_ssm_amd.layers import SSM

    torch.manual_seed(0)
    layer = SSM(hidden_size=1024, state_size_mult=4.0, compute_dtype=torch.float16, dtype=torch.float32).to(gpu)
    g = torch.Generator(device="cpu").manual_seed(5)
    xin = torch.randn(16, 2048, 1024, generator=g)
    gout = torch.randn(16, 2048, 1024, generator=g)
    print("case config3 layer full shape", flush=True)
    out, dx, grads = _run_layer(layer, xin.to(gpu), gout)
    assert hip_scan.workspace_status() == 0
    ref_out, ref_dx, ref_grads = _layer_oracle_f64(layer, xin, gout, gpu)
    assert_close("layer out", out, ref_out.numpy(), 1e-2)
    assert_close("layer dx", dx, ref_dx.numpy(), 1e-2)
    for n in ref_grads:
        assert_close(f"grad {n}", grads[n], ref_grads[n].numpy(), 1e-2)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16], ids=["fp32", "fp16", "bf16"])
def test_copy_stack_layers_against_the_float64_oracle(gpu, dtype):
    # Two layers of the copy task's stack at its own shape (hidden 256, state 1024, B 32, 64 + 64 teacher-forced
    # steps, fp32 parameters, fp32 scan output), forward and backward, against the float64 composition of the norm,
    # gate and scan oracles chained through both layers: the oracle's activations stay float64 between the layers,
    # the device's are fp32.  Every tensor (stack output, input gradient, every parameter gradient of both layers)
    # meets the bar of its compute dtype.
    from quick_ssm_amd.layers import SSM

    torch.manual_seed(0)
    layers = [SSM(hidden_size=256, state_size_mult=4.0, compute_dtype=dtype, dtype=torch.float32).to(gpu) for _ in range(2)]
    g = torch.Generator(device="cpu").manual_seed(11)
    xin = torch.randn(32, 128, 256, generator=g)
    gout = torch.randn(32, 128, 256, generator=g)
    print(f"case copy stack 2 layers compute={dtype}", flush=True)
    x0 = xin.to(gpu).requires_grad_(True)
    h = x0
    for layer in layers:
        h = layer(h, block_l=128, checkpoint=True, scan_out_dtype=torch.float32)
    h.backward(gout.to(gpu))
    assert hip_scan.workspace_status() == 0
    mid, _, _ = _layer_oracle_f64(layers[0], xin, torch.zeros_like(gout), gpu)          # layer 1 forward
    ref_out, ref_dmid, ref_g2 = _layer_oracle_f64(layers[1], mid, gout, gpu)            # layer 2 both ways
    _, ref_dx, ref_g1 = _layer_oracle_f64(layers[0], xin, ref_dmid, gpu)                # layer 1 backward
    tol = 1e-4 if dtype == torch.float32 else 1e-2
    assert_close("stack out", h.detach(), ref_out.numpy(), tol)
    assert_close("stack dx", x0.grad, ref_dx.numpy(), tol)
    for layer, ref in ((layers[0], ref_g1), (layers[1], ref_g2)):
        got = {n: p.grad for n, p in layer.named_parameters()}
        for n in ref:
            assert_close(f"grad {n}", got[n], ref[n].numpy(), tol)


def test_ssm_layer_matches_sequential_path(gpu):
    # the device layer against the same layer on the product's sequential torch path (pinned on the reference's CPU
    # path by tests/test_oracle.py)
    from quick_ssm_amd.layers import SSM

    torch.manual_seed(0)
    layer = SSM(hidden_size=64, state_size_mult=4.0, compute_dtype=torch.float16, dtype=torch.float32)
    xin = torch.randn(2, 192, 64)
    gout = torch.randn(2, 192, 64)

    def run(mod, inp, backend):
        mod.zero_grad(set_to_none=True)
        inp = inp.clone().requires_grad_(True)
        out = mod(inp, backend=backend)
        out.backward(gout.to(inp.device))
        grads = {n: p.grad.detach().cpu().clone() for n, p in mod.named_parameters()}
        return out.detach().cpu(), inp.grad.detach().cpu(), grads

    y_ref, dx_ref, g_ref = run(layer, xin, "torch")
    layer_gpu = layer.to(gpu)
    y_gpu, dx_gpu, g_gpu = run(layer_gpu, xin.to(gpu), "auto")
    assert_close("layer out", y_gpu, y_ref.double().numpy(), 1e-2)
    assert_close("layer dx", dx_gpu, dx_ref.double().numpy(), 1e-2)
    for n in g_ref:
        assert_close(f"grad {n}", g_gpu[n], g_ref[n].double().numpy(), 2e-2)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("D", [1, 4, 16])
def test_narrow_rows_fold_across_lanes(gpu, D, dtype):
    # A few columns only: rows of 1 to 4 lanes, 64 to 256 lane groups per tile, whose maps are combined by exchanges
    # between the lanes of a wavefront (both directions in the backward).  Long enough for several tiles per chain.
    # Every output against the oracle; the launch time is printed for the record (run with -s).
    shape = (4, 6000, D)
    x, a, b, c, dy = make_inputs(shape, dtype=dtype, seed=90 + D)
    ref = oracle_all(x, a, b, c, dy)
    ops = [t.to(gpu) for t in (x, a, b, c)]
    g = dy.to(gpu)
    fwd = hip_scan.make_plan(*shape, dtype, dtype, _lib.QSSM_FORWARD, 1, 0)
    assert fwd.threads == 256 and fwd.g_log2 <= 4 and fwd.n_seg > 1
    y, _, ckpt, stride = hip_scan.scan_forward(*ops, out_dtype=dtype)
    grads = hip_scan.scan_backward(*ops, g, ckpt=ckpt, ckpt_stride=stride)
    assert hip_scan.workspace_status() == 0
    _check_all(dict(zip(("y", "dx", "da", "db", "dc"), (y,) + grads)), ref, TOL[dtype])
    full = hip_scan.scan_forward(*ops, out_dtype=dtype, want_h=True, want_ckpt=False)[1]
    grads_h = hip_scan.scan_backward(*ops, g, h=full)            # the backward that reads h folds one way only
    _check_all(dict(zip(("y", "dx", "da", "db", "dc"), (y,) + grads_h)), ref, TOL[dtype])
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(3)]
    ev[0].record()
    for _ in range(20):
        hip_scan.scan_forward(*ops, out_dtype=dtype)
    ev[1].record()
    for _ in range(20):
        hip_scan.scan_backward(*ops, g, ckpt=ckpt, ckpt_stride=stride)
    ev[2].record()
    torch.cuda.synchronize()
    print(f"narrow rows D={D} {dtype}: forward {ev[0].elapsed_time(ev[1]) * 50:.1f} us, backward "
          f"{ev[1].elapsed_time(ev[2]) * 50:.1f} us per launch ({fwd.n_seg} tiles per chain, "
          f"{fwd.threads >> fwd.g_log2} lane groups per tile)", flush=True)


def test_calibration_copy_moves_every_byte(gpu):
    # qssm_copy_bytes is the kernel of known traffic that the HBM counters are scaled by: sizes that are not a
    # multiple of a workgroup's 16 KiB, one 16-byte piece, nothing
    lib = _lib.load()
    stream = torch.cuda.current_stream(gpu).cuda_stream
    for nbytes in (16, 16 * 1023, 16 * 1024, 16 * 1025, (3 << 20) + 48):
        src = torch.randint(0, 256, (nbytes,), dtype=torch.uint8, device=gpu)
        dst = torch.zeros(nbytes + 16, dtype=torch.uint8, device=gpu)
        assert lib.qssm_copy_bytes(dst.data_ptr(), src.data_ptr(), nbytes, stream) == 0
        assert torch.equal(dst[:nbytes], src) and int(dst[nbytes:].sum()) == 0
    assert lib.qssm_copy_bytes(None, None, 0, stream) == 0


def test_random_shapes_layouts_and_storage_against_oracle(gpu):
    # a seeded sweep: shapes around the tile and strip boundaries, every built storage pair, operands that are
    # contiguous, column slices of a wider tensor, or every second time step of a longer one; checkpoint on and off
    import random
    rng = random.Random(7)
    pairs = [(torch.float32, torch.float32), (torch.float16, torch.float16), (torch.bfloat16, torch.bfloat16),
             (torch.float16, torch.float32), (torch.bfloat16, torch.float32)]
    for case in range(36):
        B = rng.choice([1, 2, 3])
        L = rng.choice([1, 2, 31, 33, 64, 65, 129, 255, 300, 513, 1030])
        D = rng.choice([1, 3, 4, 8, 12, 64, 100, 128, 256, 264, 520])
        dtype, out_dtype = rng.choice(pairs)
        layout = rng.choice(["dense", "columns", "steps"])
        checkpoint = rng.random() < 0.7
        print(f"case {case}: B{B} L{L} D{D} {dtype} -> {out_dtype} {layout} checkpoint={checkpoint}", flush=True)
        x, a, b, c, dy = make_inputs((B, L, D), dtype=dtype, seed=1000 + case, out_dtype=out_dtype)
        ref = oracle_all(x, a, b, c, dy)

        def place(t):
            if layout == "columns":      # a column slice: row stride D + 16, first column at 8
                wide = torch.zeros(B, L, D + 16, dtype=t.dtype, device=gpu)
                wide[:, :, 8:8 + D] = t.to(gpu)
                return wide[:, :, 8:8 + D]
            if layout == "steps":        # every second step of a sequence twice as long
                long = torch.zeros(B, 2 * L, D, dtype=t.dtype, device=gpu)
                long[:, ::2] = t.to(gpu)
                return long[:, ::2]
            return t.to(gpu)

        leaves = [place(t).detach().requires_grad_(True) for t in (x, a, b, c)]
        y = scan(*leaves, checkpoint=checkpoint, out_dtype=out_dtype)
        y.backward(place(dy))
        assert hip_scan.workspace_status() == 0
        tol_y, tol_g = TOL[out_dtype], TOL[dtype]
        assert_close(f"case {case} y", y.detach().cpu(), ref["y"], tol_y)
        for name, leaf in zip(("dx", "da", "db", "dc"), leaves):
            assert_close(f"case {case} {name}", leaf.grad.cpu(), ref[name], tol_g)


def test_seeded_random_operand_layouts_tiles_and_keywords(gpu):
    # A fixed-seed draw in which every operand gets a layout of its own (dense, time-major memory, broadcast over the
    # batch or over time through stride 0, a transposed last axis that needs a copy, a column block of a wider tensor,
    # an offset that breaks 16-byte alignment) and scan() random keywords (block_l, checkpoint, tile_b, tile_d,
    # out_dtype); gradients of broadcast operands come back summed by autograd.  QSSM_RANDOM_LAYOUT_CASES=n draws n
    # cases instead of 60.
    n_cases = int(os.environ.get("QSSM_RANDOM_LAYOUT_CASES", "60"))
    rng = np.random.default_rng(8088)
    pairs = [(torch.float32, torch.float32), (torch.float16, torch.float16), (torch.bfloat16, torch.bfloat16),
             (torch.float16, torch.float32), (torch.bfloat16, torch.float32)]
    layouts = ("dense", "time_major", "bcast_batch", "bcast_time", "transposed", "columns", "offset")

    def place(t, layout):
        B, L, D = t.shape
        t = t.to(gpu)
        if layout == "time_major":                      # memory is [L, B, D]
            return t.transpose(0, 1).contiguous().transpose(0, 1)
        if layout == "bcast_batch":                     # one batch row, stride 0 over the batch
            return t[:1].contiguous().expand(B, L, D)
        if layout == "bcast_time":                      # one step, stride 0 over time
            return t[:, :1].contiguous().expand(B, L, D)
        if layout == "transposed":                      # memory is [B, D, L]: the last axis is not contiguous
            return t.transpose(1, 2).contiguous().transpose(1, 2)
        if layout == "columns":
            wide = torch.zeros(B, L, D + 24, dtype=t.dtype, device=gpu)
            wide[:, :, 16:16 + D] = t
            return wide[:, :, 16:16 + D]
        if layout == "offset":                          # starts one element into its allocation
            flat = torch.zeros(B * L * D + 1, dtype=t.dtype, device=gpu)
            flat[1:] = t.reshape(-1)
            return flat[1:].view(B, L, D)
        return t

    for case in range(n_cases):
        dtype, out_dtype = pairs[case % len(pairs)]
        B = int(rng.integers(1, 4))
        L = int(rng.choice([int(rng.integers(1, 40)), int(rng.integers(40, 400)), int(rng.integers(400, 1500))]))
        D = int(rng.choice([int(rng.integers(1, 20)), 8 * int(rng.integers(1, 40)), 256 * int(rng.integers(1, 3))]))
        lay = [str(rng.choice(layouts)) for _ in range(5)]
        kw = {"block_l": int(rng.choice([1, 16, 100, 256, 1024])), "checkpoint": bool(rng.integers(0, 2)),
              "tile_b": [None, 1, 2][int(rng.integers(0, 3))], "tile_d": [None, 8, 100, 256][int(rng.integers(0, 4))]}
        x, a, b, c, dy = make_inputs((B, L, D), dtype=dtype, seed=7000 + case, out_dtype=out_dtype)
        # what the device sees: a broadcast operand repeats its first batch row or first step
        seen = []
        for t, how in zip((x, a, b, c, dy), lay):
            if how == "bcast_batch":
                t = t[:1].expand(B, L, D).contiguous()
            elif how == "bcast_time":
                t = t[:, :1].expand(B, L, D).contiguous()
            seen.append(t)
        if case < 12 or case % 10 == 0:
            print(f"case random layouts {case} shape=({B}, {L}, {D}) {dtype}->{out_dtype} {lay} {kw}", flush=True)
        ref = oracle_all(*seen)
        bases = [place(t, how) for t, how in zip((x, a, b, c), lay[:4])]
        leaves = [t.detach().requires_grad_(True) for t in bases]
        y = scan(*leaves, out_dtype=out_dtype, **kw)
        y.backward(place(dy, lay[4]))
        assert hip_scan.workspace_status() == 0
        assert_close(f"y (case {case})", y.detach().cpu(), ref["y"], TOL[out_dtype])
        for name, leaf in zip(("dx", "da", "db", "dc"), leaves):
            assert leaf.grad.shape == (B, L, D), name
            assert_close(f"{name} (case {case})", leaf.grad.cpu(), ref[name], TOL[dtype])


def test_scans_from_several_threads_on_shared_and_private_streams(gpu):
    # Six Python threads scan forward and backward at the same time, three on the default stream (one control block
    # and workspace between them, launches numbered under the lock) and three on streams of their own; autograd adds
    # its own thread for every backward.  Every result must be the bits the same call gives on a quiet device.
    import threading

    shapes = [((2, 900, 256), torch.bfloat16), ((1, 2100, 64), torch.float32), ((3, 300, 520), torch.float16)]
    cases = []
    for k, (shape, dtype) in enumerate(shapes):
        ops = [t.to(gpu) for t in make_inputs(shape, dtype=dtype, seed=90 + k)]
        leaves = [t.clone().requires_grad_(True) for t in ops[:4]]
        y = scan(*leaves)
        y.backward(ops[4])
        cases.append((ops, y.detach().clone(), [t.grad.clone() for t in leaves]))
    torch.cuda.synchronize()
    errors = []

    def work(idx, own_stream):
        try:
            ops, y_ref, g_ref = cases[idx % len(cases)]
            stream = torch.cuda.Stream(device=gpu) if own_stream else torch.cuda.current_stream(gpu)
            stream.wait_stream(torch.cuda.default_stream(gpu))
            with torch.cuda.stream(stream):
                for it in range(25):
                    leaves = [t.clone().requires_grad_(True) for t in ops[:4]]
                    y = scan(*leaves)
                    y.backward(ops[4])
                    stream.synchronize()
                    if not torch.equal(y, y_ref) or any(not torch.equal(t.grad, g) for t, g in zip(leaves, g_ref)):
                        errors.append(f"thread {idx} iteration {it}: results differ")
                        return
        except Exception as exc:  # noqa: BLE001 - reported by the main thread
            errors.append(f"thread {idx}: {type(exc).__name__}: {exc}")

    threads = [threading.Thread(target=work, args=(k, k >= 3)) for k in range(6)]
    for t in threads:
        t.start()
    for t in threads:
        t.join(timeout=120)
    assert not any(t.is_alive() for t in threads), "a worker thread did not finish"
    torch.cuda.synchronize()
    assert not errors, errors
    assert hip_scan.workspace_status() == 0


def test_nan_in_an_input_stays_in_its_column_and_nothing_hangs(gpu):
    # one NaN in x: from that step on y, da and dc of that column are NaN (the state carries it), db only at that
    # step, dx nowhere; every other column is untouched, no tile waits for ever (the tags of the exchanged words
    # do not depend on their payload), and the pattern is the oracle's
    shape = (2, 600, 260)
    x, a, b, c, dy = make_inputs(shape, dtype=torch.bfloat16, seed=77)
    x[0, 100, 5] = float("nan")
    got = run_scan_with_grads(scan, x, a, b, c, dy, gpu, checkpoint=True)
    assert hip_scan.workspace_status() == 0
    ref = oracle_all(x, a, b, c, dy)
    for name in ("y", "dx", "da", "db", "dc"):
        g = got[name].float().numpy()
        r = np.asarray(ref[name], dtype=np.float64)
        assert np.array_equal(np.isnan(g), np.isnan(r)), name
        ok = ~np.isnan(r)
        scale = np.abs(r[ok]).max()
        assert np.abs(g[ok] - r[ok]).max() <= TOL[torch.bfloat16] * scale, name
    y = got["y"].float()
    assert torch.isnan(y[0, 100:, 5]).all() and torch.isfinite(y[0, :100, 5]).all()
    assert torch.isfinite(got["dx"].float()).all()
    assert int(torch.isnan(got["db"].float()).sum()) == 1


def test_tiles_that_keep_their_operands_in_the_caches_change_nothing(gpu, hip_lib):
    # keep_tiles only chooses between streaming and ordinary loads: every setting gives the same bits
    import ctypes

    from quick_ssm_amd._lib import Plan, Strides

    lib = hip_lib
    stream = torch.cuda.current_stream(gpu).cuda_stream
    for shape, dtype in (((2, 1100, 512), torch.bfloat16), ((2, 700, 96), torch.float32), ((1, 900, 264), torch.float16)):
        B, L, D = shape
        x, a, b, c, _ = make_inputs(shape, dtype=dtype, seed=5)
        xd, ad, bd, cd = (t.to(gpu) for t in (x, a, b, c))
        stride = hip_scan.make_plan(B, L, D, dtype, dtype, _lib.QSSM_BACKWARD, 8, 0).seg_len
        base = hip_scan.make_plan(B, L, D, dtype, dtype, _lib.QSSM_FORWARD, 8, stride)
        assert base.n_seg > 2
        outs = []
        for keep in (0, 1, base.n_seg // 2, base.n_seg, base.n_seg + 5):
            plan = Plan.from_buffer_copy(base)
            plan.keep_tiles = keep
            y = torch.full(shape, float("nan"), dtype=dtype, device=gpu)
            ck = torch.full((B, plan.n_ckpt, D), float("nan"), dtype=torch.float32, device=gpu)
            ctl = torch.zeros(max(int(plan.control_bytes), 64), dtype=torch.uint8, device=gpu)
            ws = torch.zeros(max(int(plan.workspace_bytes), 256), dtype=torch.uint8, device=gpu)
            st = lambda t: Strides(t.stride(0), t.stride(1))
            rc = lib.qssm_scan_forward(ctypes.byref(plan), xd.data_ptr(), st(xd), ad.data_ptr(), st(ad), bd.data_ptr(),
                                       st(bd), cd.data_ptr(), st(cd), y.data_ptr(), st(y), None, Strides(0, 0),
                                       ck.data_ptr(), ctl.data_ptr(), ctl.numel(), ws.data_ptr(), ws.numel(), 1, stream)
            assert rc == 0, lib.qssm_error_string()
            torch.cuda.synchronize()
            outs.append((y, ck))
        _, y_ref = oracle.forward_f64(x, a, b, c)
        assert_close("y", outs[0][0].cpu(), y_ref, TOL[dtype])
        for y, ck in outs[1:]:
            assert torch.equal(y, outs[0][0]) and torch.equal(ck, outs[0][1])
        plan = Plan.from_buffer_copy(base)
        plan.keep_tiles = -1
        rc = lib.qssm_scan_forward(ctypes.byref(plan), xd.data_ptr(), st(xd), ad.data_ptr(), st(ad), bd.data_ptr(),
                                   st(bd), cd.data_ptr(), st(cd), y.data_ptr(), st(y), None, Strides(0, 0),
                                   ck.data_ptr(), ctl.data_ptr(), ctl.numel(), ws.data_ptr(), ws.numel(), 1, stream)
        assert rc == _lib.QSSM_EINVAL


def test_seeded_random_shapes_match_the_oracle(gpu):
    # Shapes, storage types and output types drawn from a fixed seed: whatever geometry the planner picks for them
    # (strip widths, lanes per row, clusters of 1 to 8, LDS-resident or register operands) must meet the oracle.
    # QSSM_RANDOM_CASES=n draws n cases instead of 300 (the first cases stay the same ones whatever n is).
    n_cases = int(os.environ.get("QSSM_RANDOM_CASES", "300"))
    rng = np.random.default_rng(20240607)
    pairs = [(torch.float32, torch.float32), (torch.float16, torch.float16), (torch.bfloat16, torch.bfloat16),
             (torch.float16, torch.float32), (torch.bfloat16, torch.float32)]
    seen = set()
    for case in range(n_cases):
        dtype, out_dtype = pairs[case % len(pairs)]
        B = int(rng.integers(1, 5))
        L = int(rng.choice([int(rng.integers(1, 200)), int(rng.integers(200, 3000)), int(rng.integers(3000, 9000))]))
        D = int(rng.choice([int(rng.integers(1, 40)), 8 * int(rng.integers(1, 80)), 256 * int(rng.integers(1, 4))]))
        if B * L * D > 6_000_000:
            L = max(1, 6_000_000 // (B * D))
        x, a, b, c, dy = make_inputs((B, L, D), dtype=dtype, seed=1000 + case, out_dtype=out_dtype)
        if case < 40 or case % 25 == 0:
            print(f"case random {case} shape=({B}, {L}, {D}) dtype={dtype} out={out_dtype}", flush=True)
        got = run_scan_with_grads(scan, x, a, b, c, dy, gpu, out_dtype=out_dtype)
        assert hip_scan.workspace_status() == 0
        ref = oracle_all(x, a, b, c, dy)
        assert_close("y", got["y"], ref["y"], TOL[out_dtype])
        for k in ("dx", "da", "db", "dc"):
            assert_close(k, got[k], ref[k], TOL[dtype])
        align = 8 if D % 8 == 0 else 4 if D % 4 == 0 else 2 if D % 2 == 0 else 1
        plan = hip_scan.make_plan(B, L, D, dtype, out_dtype, _lib.QSSM_BACKWARD, align, 0)
        seen.add((plan.vec, plan.g_log2, plan.cluster))
    assert len({c for _, _, c in seen}) >= 3, seen     # the draw really covers several cluster sizes
