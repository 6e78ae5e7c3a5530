"""Host-side logic and the C-ABI surface, without a GPU."""
import ctypes
import re
from pathlib import Path

import pytest
import torch

from quick_ssm_amd import _lib, hip_scan
from quick_ssm_amd.scan_interface import _chunk_ranges, scan

ROOT = Path(__file__).resolve().parents[1]


def test_library_exports_every_declared_symbol(hip_lib):
    header = (ROOT / "include" / "quick_ssm_hip.h").read_text()
    declared = set(re.findall(r"QSSM_API\s+[\w\s\*]+?\b(qssm_\w+)\s*\(", header))
    assert declared == set(_lib.EXPORTED_SYMBOLS)
    for name in declared:
        assert getattr(hip_lib, name) is not None
    assert hip_lib.qssm_version() == _lib.QSSM_VERSION == 200
    assert ctypes.sizeof(_lib.Plan) == 22 * 4 + 3 * 8   # 21 ints, padded to the 8-byte fields behind them


def test_chunk_ranges_follow_the_reference_rules():
    # quick_ssm/scan_interface.py:36-46
    assert _chunk_ranges(10, None) == [(0, 10)]
    assert _chunk_ranges(10, 0) == [(0, 10)]
    assert _chunk_ranges(10, -3) == [(0, 10)]
    assert _chunk_ranges(10, 10) == [(0, 10)]
    assert _chunk_ranges(10, 99) == [(0, 10)]
    assert _chunk_ranges(10, 4) == [(0, 4), (4, 8), (8, 10)]
    assert _chunk_ranges(8, 4) == [(0, 4), (4, 8)]
    assert _chunk_ranges(0, 4) == [(0, 0)]


SHAPES = [(8, 4096, 2048), (4, 2048, 16), (1, 65536, 4096), (32, 64, 1024), (1, 1024, 1), (1, 4, 1), (2, 300, 5),
          (3, 7, 2), (2, 1500, 260), (1, 1, 1)]


@pytest.mark.parametrize("shape", SHAPES, ids=lambda s: "x".join(map(str, s)))
@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
def test_plans_are_consistent_and_forward_follows_backward(hip_lib, shape, dtype):
    B, L, D = shape
    for align in (4, 2, 1):
        bwd = hip_scan.make_plan(B, L, D, dtype, dtype, _lib.QSSM_BACKWARD, align)
        fwd = hip_scan.make_plan(B, L, D, dtype, dtype, _lib.QSSM_FORWARD, align, bwd.seg_len)
        for p in (bwd, fwd):
            assert D % p.vec == 0 and p.vec <= align
            assert p.strip_cols == p.vec << p.g_log2
            assert p.threads in (256, 512, 1024) and p.seg_len == p.steps * (p.threads >> p.g_log2)
            assert p.n_super == -(-p.n_seg // p.cluster) and 0 < p.lds_bytes <= 64 * 1024
            assert p.n_strips * p.strip_cols >= D > (p.n_strips - 1) * p.strip_cols
            assert p.n_seg * p.seg_len >= L > (p.n_seg - 1) * p.seg_len
            assert p.seg_len % p.ckpt_stride == 0
            assert p.n_ckpt == -(-L // p.ckpt_stride)
        assert fwd.ckpt_stride == bwd.seg_len == bwd.ckpt_stride
        assert fwd.ckpt_stride % fwd.steps == 0
        # the forward leaves the operands of its last tiles in the caches, as far as 224 MiB reach; the backward none
        per_index = B * fwd.n_strips * fwd.strip_cols * fwd.seg_len * 4 * fwd_elem_bytes(dtype)
        assert fwd.keep_tiles == min(fwd.n_seg, (224 << 20) // per_index) and bwd.keep_tiles == 0
        # a backward planned later, with worse alignment, still reads the same saved states
        late = hip_scan.make_plan(B, L, D, dtype, dtype, _lib.QSSM_BACKWARD, 1, bwd.seg_len)
        assert late.ckpt_stride == bwd.seg_len and late.seg_len % late.ckpt_stride == 0


def fwd_elem_bytes(dtype):
    return torch.empty((), dtype=dtype).element_size()


def test_keep_tiles_of_the_headline_shape(hip_lib):
    bf = torch.bfloat16
    fwd = hip_scan.make_plan(8, 4096, 2048, bf, bf, _lib.QSSM_FORWARD, 8, 32)
    assert (fwd.vec, fwd.n_seg, fwd.keep_tiles) == (8, 64, 28)


def test_sixteen_bytes_per_lane_only_where_it_pays(hip_lib):
    bf, f16 = torch.bfloat16, torch.float16

    def fwd(B, L, D, dt):
        return hip_scan.make_plan(B, L, D, dt, dt, _lib.QSSM_FORWARD, 8, 32)

    assert (fwd(8, 4096, 2048, bf).vec, fwd(12, 4096, 2048, bf).vec) == (8, 8)
    small = fwd(16, 2048, 1024, bf)                      # 2048 tiles: too few
    assert (small.vec, small.threads) == (4, 512)
    long = fwd(1, 65536, 4096, f16)                      # 16 strips over a long sequence: rows of half the width instead
    assert (long.vec, long.threads, long.g_log2) == (4, 512, 5)


def test_cluster_size_follows_stream_time_against_chain_time(hip_lib):
    bf, f16 = torch.bfloat16, torch.float16

    def clusters(B, L, D, dt, odt):
        bwd = hip_scan.make_plan(B, L, D, dt, odt, _lib.QSSM_BACKWARD, 8, 0)
        fwd = hip_scan.make_plan(B, L, D, dt, odt, _lib.QSSM_FORWARD, 8, bwd.seg_len)
        return fwd.cluster, bwd.cluster

    assert clusters(8, 4096, 2048, bf, bf) == (2, 4)          # chain and stream in balance; the backward's hops cost more than its maps
    assert clusters(16, 4096, 2048, bf, bf) == (1, 1)         # stream time dwarfs the chain: no maps at all
    assert clusters(1, 65536, 4096, f16, f16) == (4, 4)       # very long chains
    assert clusters(2, 8192, 512, bf, bf) == (8, 8)           # little to stream, long chains: fewest hand-overs
    assert clusters(2, 4096, 2048, bf, bf) == (8, 4)          # the backward pays more per neighbour map
    assert clusters(32, 64, 1024, f16, torch.float32) == (1, 1)   # one tile per chain
    assert clusters(1, 16384, 256, bf, bf) == (32, 16)        # one long, narrow sequence: the chain is all there is
    assert clusters(1, 32768, 1024, bf, bf) == (8, 8)         # wider: the maps of 16 tiles would cost more than the hops


def test_plan_rejects_bad_arguments(hip_lib):
    with pytest.raises(_lib.QssmError):
        hip_scan.make_plan(-1, 4, 4, torch.float32, torch.float32, 0, 4)
    with pytest.raises(_lib.QssmError) as err:
        hip_scan.make_plan(1, 64, 4, torch.float32, torch.float32, 0, 4, ckpt_stride=48)
    assert "power of two" in str(err.value)
    plan = _lib.Plan()
    rc = hip_lib.qssm_plan_scan(1, 4, 4, 7, 0, 0, 4, 0, ctypes.byref(plan))
    assert rc == _lib.QSSM_EINVAL and b"dtype" in hip_lib.qssm_error_string()
    # fp32 operands with 16-bit y is not a built pair: the host casts instead
    assert hip_scan.kernel_dtypes([torch.float32] * 4, torch.float16) == (torch.float32, torch.float32)
    assert hip_scan.kernel_dtypes([torch.float16, torch.float32], torch.float32) == (torch.float32, torch.float32)
    assert hip_scan.kernel_dtypes([torch.bfloat16] * 4, torch.float32) == (torch.bfloat16, torch.float32)
    assert hip_scan.kernel_dtypes([torch.float64] * 4, torch.float64) == (torch.float32, torch.float32)


def test_launchers_validate_before_touching_the_gpu(hip_lib):
    plan = hip_scan.make_plan(2, 64, 8, torch.float32, torch.float32, _lib.QSSM_FORWARD, 4)
    z = _lib.Strides(0, 0)
    args = [ctypes.byref(plan)] + [None, z] * 6 + [None, None, 0, None, 0, 1, None]
    assert hip_lib.qssm_scan_forward(*args) == _lib.QSSM_EINVAL      # NULL operands
    bwd = [ctypes.byref(plan)] + [None, z] * 6 + [None] + [None, z] * 4 + [None, 0, None, 0, 1, None]
    assert hip_lib.qssm_scan_backward(*bwd) == _lib.QSSM_EINVAL      # forward plan given to the backward
    assert b"direction" in hip_lib.qssm_error_string()
    assert hip_lib.qssm_copy_bytes(8, 16, 10, None) == _lib.QSSM_EALIGN


def test_device_backend_refuses_cpu_tensors_and_unknown_backends():
    x = torch.zeros(2, 8, 4)
    for backend in ("triton", "hip"):
        with pytest.raises(RuntimeError):
            scan(x, x, x, x, backend=backend)
    with pytest.raises(ValueError):
        scan(x, x, x, x, backend="nope")
    y = scan(x, x, x, x)  # auto on CPU tensors: the sequential torch path, as in the reference
    assert y.shape == x.shape


def test_drop_in_import_paths():
    import quick_ssm
    from quick_ssm.layers import SSM, RMSNorm
    from quick_ssm.naive_baseline import naive_backward_3d, naive_forward_3d, naive_full_3d
    from quick_ssm.scan_interface import _TritonScanFunction, scan as scan2
    from quick_ssm.triton_backwards import block_scan_backward_3d
    from quick_ssm.triton_forwards import block_scan_forward_3d

    assert quick_ssm.__all__ == ["scan", "SSM", "RMSNorm"]
    assert scan2 is scan and callable(block_scan_forward_3d) and callable(block_scan_backward_3d)
    assert issubclass(_TritonScanFunction, torch.autograd.Function)


def test_naive_backward_matches_autograd_on_cpu():
    from quick_ssm_amd.naive_baseline import naive_backward_3d, naive_full_3d

    torch.manual_seed(1)
    x, a, b, c, dy = (torch.randn(2, 20, 3, dtype=torch.float64) for _ in range(5))
    leaves = [t.clone().requires_grad_(True) for t in (x, a, b, c)]
    _, y = naive_full_3d(*leaves)
    (y * dy).sum().backward()
    for got, t in zip(naive_backward_3d(x, a, b, c, dy), leaves):
        assert torch.allclose(got, t.grad, rtol=1e-12, atol=1e-12)


def test_ssm_layer_on_cpu_matches_hand_written_recurrence():
    # weight roles as documented in quick_ssm/test_swiglu_equiv.py:60-70
    from quick_ssm_amd.layers import SSM

    torch.manual_seed(0)
    layer = SSM(hidden_size=8, state_size_mult=2.0, compute_dtype=torch.float32)
    x = torch.randn(2, 12, 8)
    out = layer(x, backend="torch")
    u = layer.pre_norm(x)
    f = torch.sigmoid(layer.A_proj(u))
    z = layer.B_proj(u) * torch.sigmoid(layer.D_proj(u))
    gate = torch.nn.functional.silu(layer.C_proj_a(u)) * layer.C_proj_b(u)
    h = torch.zeros(2, 16)
    hs = []
    for t in range(12):
        h = f[:, t] * h + z[:, t]
        hs.append(h)
    expect = layer.out_proj(gate * torch.stack(hs, 1)) + x
    assert torch.allclose(out, expect, rtol=1e-5, atol=1e-6)
    assert [n for n, _ in layer.named_parameters()] == [
        "A_proj.weight", "A_proj.bias", "B_proj.weight", "C_proj_a.weight", "C_proj_b.weight", "D_proj.weight",
        "out_proj.weight", "out_proj.bias", "pre_norm.weight"]


def _tile_accesses(plan, B, L, D):
    """Element offsets (contiguous [B, L, D]) every lane of every tile touches, and the workspace words,
    following the index arithmetic of the kernels."""
    import numpy as np

    G = 1 << plan.g_log2
    NG = plan.threads >> plan.g_log2
    cols = plan.strip_cols
    tid = np.arange(plan.threads)
    j, dl = tid >> plan.g_log2, (tid & (G - 1)) * plan.vec
    n_chains = B * plan.n_strips
    hi_elem, hi_ckpt, hi_word = -1, -1, -1
    lo_elem = 0
    maps_off = 0
    states_off = (n_chains * plan.n_seg * cols * 16 + 255) // 256 * 256
    assert plan.control_bytes >= 64 + n_chains * 64
    for chain in range(n_chains):
        bi, strip = divmod(chain, plan.n_strips)
        d = strip * cols + dl
        dok = d < D
        for seg in range(plan.n_seg):
            t0 = seg * plan.seg_len + j * plan.steps
            for i in range(plan.steps):
                ok = dok & (t0 + i < L)
                if ok.any():
                    off = (bi * L + t0[ok] + i) * D + d[ok]
                    lo_elem = min(lo_elem, int(off.min()))
                    hi_elem = max(hi_elem, int(off.max()) + plan.vec - 1)
            ck = dok & (t0 < L) & (t0 % plan.ckpt_stride == 0)
            if ck.any():
                hi_ckpt = max(hi_ckpt, int(((bi * plan.n_ckpt + t0[ck] // plan.ckpt_stride) * D + d[ck]).max()) + plan.vec - 1)
            if plan.n_seg > 1:
                edge = dl[dok]
                hi_word = max(hi_word, maps_off + int((((chain * plan.n_seg + seg) * cols + edge) * 2).max() + 2 * plan.vec) * 8)
                s = seg // plan.cluster
                hi_word = max(hi_word, states_off + int(((chain * plan.n_super + s) * cols + edge).max() + plan.vec) * 8)
    assert NG * plan.steps == plan.seg_len
    return lo_elem, hi_elem, hi_ckpt, hi_word


@pytest.mark.parametrize("shape", [(2, 1500, 260), (2, 300, 5), (3, 7, 2), (2, 777, 64), (1, 2100, 520), (2, 64, 1024)],
                         ids=lambda s: "x".join(map(str, s)))
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_tile_index_arithmetic_stays_in_bounds(hip_lib, shape, dtype):
    B, L, D = shape
    for direction in (_lib.QSSM_BACKWARD, _lib.QSSM_FORWARD):
        for tune in (0, 1 | (4 << 8) | (1 << 24) | (2 << 28), 7 | (8 << 8) | (2 << 24) | (4 << 28)):
            plan = hip_scan.make_plan(B, L, D, dtype, dtype, direction, 4, 0, tune)
            lo, hi, hi_ckpt, hi_word = _tile_accesses(plan, B, L, D)
            assert lo >= 0 and hi == B * L * D - 1          # every element is covered, nothing beyond
            assert hi_ckpt < plan.ckpt_elems
            assert hi_word <= plan.workspace_bytes
    if dtype != torch.float32 and D % 8 == 0:
        # the forward with 8 columns (16 bytes) per lane, forced onto these small shapes
        for tune in (8 << 16, 3 | (8 << 16) | (3 << 28), 6 | (8 << 16) | (2 << 28)):
            plan = hip_scan.make_plan(B, L, D, dtype, dtype, _lib.QSSM_FORWARD, 8, 32, tune)
            assert plan.vec == 8 and plan.threads == 256
            lo, hi, hi_ckpt, hi_word = _tile_accesses(plan, B, L, D)
            assert lo >= 0 and hi == B * L * D - 1 and hi_ckpt < plan.ckpt_elems and hi_word <= plan.workspace_bytes


def test_plan_invariants_over_random_shapes(hip_lib):
    # a seeded sweep over shapes, alignments, storage pairs and directions: whatever the planner picks must describe
    # a launch the kernels can run (lane counts, tile lengths, LDS, buffer sizes), for the backward first and then for
    # a forward that saves the states that backward will read
    import random
    rng = random.Random(1234)
    pairs = [(torch.float32, torch.float32), (torch.float16, torch.float16), (torch.bfloat16, torch.bfloat16),
             (torch.float16, torch.float32), (torch.bfloat16, torch.float32)]
    for _ in range(400):
        B = rng.choice([1, 1, 2, 3, 8, 17, 64])
        L = rng.choice([1, 2, 7, 31, 32, 33, 64, 100, 255, 256, 1000, 4096, 5000, 65536, 100001])
        D = rng.choice([1, 2, 3, 4, 6, 8, 12, 60, 64, 100, 256, 260, 1024, 2048, 4100])
        dt, odt = rng.choice(pairs)
        align = rng.choice([1, 2, 4, 8])
        bwd = hip_scan.make_plan(B, L, D, dt, odt, _lib.QSSM_BACKWARD, align)
        fwd = hip_scan.make_plan(B, L, D, dt, odt, _lib.QSSM_FORWARD, align, bwd.seg_len)
        for p in (bwd, fwd):
            what = (B, L, D, dt, odt, align, p.describe())
            wide = p is fwd and dt != torch.float32 and odt == dt     # 16 bytes per lane: forward, 16-bit storage
            assert p.vec in ((1, 2, 4, 8) if wide else (1, 2, 4)) and D % p.vec == 0 and align % p.vec == 0, what
            assert p.steps in (4, 8) and p.threads in (256, 512, 1024), what
            assert 1 <= (1 << p.g_log2) <= p.threads and p.strip_cols == p.vec << p.g_log2, what
            assert p.seg_len == p.steps * (p.threads >> p.g_log2) and p.seg_len % p.ckpt_stride == 0, what
            assert p.n_strips == -(-D // p.strip_cols) and p.n_seg == -(-L // p.seg_len), what
            assert p.cluster in (1, 2, 4, 8, 16, 32) and p.n_super == -(-p.n_seg // p.cluster), what
            assert 0 < p.lds_bytes <= 64 * 1024, what
            chains = B * p.n_strips
            assert p.control_bytes >= 64 + 64 * chains and p.control_bytes % 256 == 0, what
            words = chains * (p.n_seg * 2 + p.n_super) * p.strip_cols * 8
            assert (p.workspace_bytes >= words if p.n_seg > 1 else p.workspace_bytes == 0), what
            assert p.ckpt_elems == B * p.n_ckpt * D and p.n_ckpt == -(-L // p.ckpt_stride), what
        assert fwd.ckpt_stride == bwd.ckpt_stride == bwd.seg_len


def test_gated_plans_of_both_directions_agree_on_the_saved_states(hip_lib):
    # The gated forward is handed the gated backward's tile length as the spacing of its saved states, and the
    # backward is handed it back: over a grid of shapes (very short sequences included, where the planner first
    # widens the rows and the gated kernels then narrow them again) both plans must exist, keep that spacing and
    # describe launches the gated kernels are built for.  (1, 6, 688) and (1, 7, 1008) failed to plan once.
    from quick_ssm_amd import gated_scan
    storage = ((torch.float16, (torch.float16,)), (torch.bfloat16, (torch.bfloat16,)),
               (torch.float32, (torch.float16, torch.bfloat16, torch.float32)))
    for dtype, computes in storage:
        for compute in computes:
            for B in (1, 2, 3, 16):
                for L in (1, 2, 5, 6, 7, 8, 9, 16, 17, 31, 33, 64, 100, 257, 1000, 4096, 65536):
                    for S in (128, 132, 136, 264, 512, 688, 1008, 1024, 4096):
                        outs = (dtype, torch.float32) if dtype != torch.float32 else (torch.float32,)
                        for out in outs:
                            what = (B, L, S, dtype, compute, out)
                            stride = gated_scan._plan(B, L, S, dtype, compute, dtype, _lib.QSSM_BACKWARD, 0).seg_len
                            fwd = gated_scan._plan(B, L, S, dtype, compute, out, _lib.QSSM_FORWARD, stride)
                            bwd = gated_scan._plan(B, L, S, dtype, compute, dtype, _lib.QSSM_BACKWARD, stride)
                            assert bwd.seg_len == stride and fwd.seg_len % stride == 0, what
                            assert fwd.ckpt_stride == bwd.ckpt_stride == stride, what
                            # the two-pass backward (gate pass, then the plain backward over operands in the compute
                            # dtype) reads the same saved states: the plain planner must take their spacing as well
                            # ((2, 5, 1024) with fp32 dy failed to plan once)
                            for align in (8, 4):
                                plain = hip_scan.make_plan(B, L, S, compute, out, _lib.QSSM_BACKWARD, align, stride)
                                assert plain.ckpt_stride == stride and plain.seg_len % stride == 0, (what, align)
                            for p in (fwd, bwd):
                                assert p.threads == 256 and p.steps == 8 and p.g_log2 in (5, 6), what
                                assert p.vec == 8 // torch.empty((), dtype=dtype).element_size() and p.cluster <= 2, what
                                assert p.compute_dtype == gated_scan._CODES[compute], what


def test_tile_index_arithmetic_over_random_shapes(hip_lib):
    # the same bounds model over a seeded sweep of small shapes, alignments, storage types and forced geometries
    import random
    rng = random.Random(99)
    for _ in range(60):
        B = rng.choice([1, 2, 3])
        L = rng.choice([1, 5, 31, 32, 33, 64, 65, 127, 200, 513, 1030])
        D = rng.choice([1, 2, 4, 6, 8, 20, 64, 72, 128, 136, 260, 512])
        dtype = rng.choice([torch.float32, torch.float16, torch.bfloat16])
        align = rng.choice([1, 2, 4, 8])
        g = rng.choice([0, 0, 4, 5, 6, 7, 8])                      # automatic, or 8 .. 128 lanes per row
        tune = g | (rng.choice([0, 4, 8]) << 8) | (rng.choice([0, 1, 2]) << 24) | (rng.choice([0, 1, 2, 3, 4]) << 28)
        for direction in (_lib.QSSM_BACKWARD, _lib.QSSM_FORWARD):
            try:
                plan = hip_scan.make_plan(B, L, D, dtype, dtype, direction, align, 0, tune)
            except Exception as exc:   # a forced geometry the planner refuses is fine; anything else is not
                assert "LDS" in str(exc) or "ckpt_stride" in str(exc), (B, L, D, dtype, align, tune, str(exc))
                continue
            lo, hi, hi_ckpt, hi_word = _tile_accesses(plan, B, L, D)
            what = (B, L, D, dtype, align, tune, plan.describe())
            assert lo >= 0 and hi == B * L * D - 1, what
            assert hi_ckpt < plan.ckpt_elems, what
            assert hi_word <= plan.workspace_bytes, what


class _FakeBuffers:
    """What `_launch_buffers` and `_after_launch` touch of a `_Buffers` entry, without device or pinned memory."""

    def __init__(self):
        self.control = self.workspace = object()
        self.ctl_ptr = self.ws_ptr = 256
        self.ctl_size = self.ws_size = 1 << 30
        self.epoch = 0
        self.captured = False
        self.seen = ctypes.c_int32(0)
        self.since_check = 0
        self.device = torch.device("cpu")
        self.where = "a fake device"


def test_launches_from_several_threads_get_distinct_numbers(monkeypatch):
    # The caller's thread (next forward) and autograd's thread (a backward) may launch on one stream at the same
    # time: two launches must never share a flag value, and every due status check must be asked for exactly once.
    import sys
    import threading

    monkeypatch.setattr(torch._C, "_cuda_isCurrentStreamCapturing", lambda: False, raising=False)
    asked = []
    monkeypatch.setattr(hip_scan._lib, "load", lambda: type("L", (), {
        "qssm_control_status_async": staticmethod(lambda *a: asked.append(1) or 0)})())
    old_period = hip_scan.set_status_check_period(7)
    key = (0, 0x1234, False)
    buf = _FakeBuffers()
    buf.pinned = type("P", (), {"data_ptr": staticmethod(lambda: 0)})()
    hip_scan._buffers[key] = buf
    n_threads, per_thread = 8, 4000
    got = [[] for _ in range(n_threads)]
    start = threading.Barrier(n_threads)
    old_switch = sys.getswitchinterval()
    sys.setswitchinterval(1e-6)   # hand the interpreter from thread to thread as often as it can

    def work(slot):
        start.wait()
        for _ in range(per_thread):
            b, epoch, capturing = hip_scan._launch_buffers(buf.device, 0, 0x1234, 64, 64)
            got[slot].append(epoch)
            hip_scan._after_launch(b, 0x1234, capturing)

    try:
        threads = [threading.Thread(target=work, args=(k,)) for k in range(n_threads)]
        for t in threads:
            t.start()
        for t in threads:
            t.join()
    finally:
        sys.setswitchinterval(old_switch)
        hip_scan.set_status_check_period(old_period)
        hip_scan._buffers.pop(key, None)
    flat = [e for part in got for e in part]
    total = n_threads * per_thread
    assert sorted(flat) == list(range(1, total + 1))
    assert all(a < b for part in got for a, b in zip(part, part[1:]))   # and in order within a thread
    assert len(asked) == total // 7 and buf.since_check == total % 7


def test_device_side_launch_count_never_repeats_a_flag_between_wipes(hip_lib):
    # Launches that number themselves (epoch argument 0) use flag count + 1 and the counting kernel stores the
    # next count.  Walk the arithmetic across both wraps: no flag is ever zero, flags grow by one between restarts,
    # and the static scratch array restarts its count only behind a launch whose prologue wiped it.
    def step(count, static):
        flag, nxt, wipes = ctypes.c_uint32(), ctypes.c_uint32(), ctypes.c_int32()
        assert hip_lib.qssm_launch_count_step(count, static, ctypes.byref(flag), ctypes.byref(nxt), ctypes.byref(wipes)) == 0
        return flag.value, nxt.value, wipes.value

    for static, restart_from in ((1, 0xFFFFFFF0), (0, 0xFFFFFFFE)):
        count, flags, wiped_at = restart_from - 3, [], []
        for _ in range(8):
            flag, nxt, wipes = step(count, static)
            assert flag != 0 and flag == (count + 1) & 0xFFFFFFFF
            if wipes:
                wiped_at.append(count)
            if nxt == 0:
                # the count restarts: with the static array only behind a wipe, so flag 1 cannot meet an old word
                assert count >= restart_from and (not static or wipes)
            else:
                assert nxt == count + 1
            flags.append(flag)
            count = nxt
        assert flags[:4] == [restart_from - 2, restart_from - 1, restart_from, restart_from + 1]
        assert flags[4:] == [1, 2, 3, 4]
        assert wiped_at == ([0xFFFFFFF0] if static else [])
    assert step(5, 1) == (6, 6, 0) and step(0, 0) == (1, 1, 0)


def test_packed_projection_parameters_stay_the_reference_parameters():
    # Small layers run one GEMM over the five projection weights, which then live in one [5 S, H] tensor.  Names,
    # values and Parameter objects stay the reference's; optimizer updates and state-dict loads keep the packing;
    # whatever moves the parameters to storage of their own is noticed and packed again; and the packed function
    # gives the values and gradients of the five separate nn.Linear calls.
    import copy

    from quick_ssm_amd.layers import SSM, _PackedProjection

    torch.manual_seed(0)
    layer = SSM(16, 2.0, compute_dtype=torch.float32)
    S, H = 32, 16
    before = {k: v.clone() for k, v in layer.state_dict().items()}
    params = dict(layer.named_parameters())
    wide_w, wide_b = layer._packed_parameters()
    assert wide_w.shape == (5 * S, H) and wide_b.shape == (5 * S,)
    assert dict(layer.named_parameters()).keys() == params.keys()
    assert all(p is params[n] for n, p in layer.named_parameters())
    for k, v in layer.state_dict().items():
        assert torch.equal(v, before[k]), k
    order = ("A_proj", "B_proj", "C_proj_a", "C_proj_b", "D_proj")
    for k, n in enumerate(order):
        assert getattr(layer, n).weight.data_ptr() == wide_w.data_ptr() + k * S * H * 4
    opt = torch.optim.AdamW(layer.parameters(), lr=0.1)
    for p in layer.parameters():
        p.grad = torch.ones_like(p)
    opt.step()
    again_w, again_b = layer._packed_parameters()
    assert again_w is wide_w and again_b is wide_b                       # in-place updates keep the packing
    assert torch.equal(wide_w[S:2 * S], layer.B_proj.weight) and not torch.equal(layer.B_proj.weight, before["B_proj.weight"])
    assert torch.equal(wide_b[:S], layer.A_proj.bias) and float(wide_b[S:].abs().max()) == 0.0
    twin = copy.deepcopy(layer)
    twin_w, _ = twin._packed_parameters()
    assert twin_w.data_ptr() != wide_w.data_ptr() and twin.A_proj.weight.data_ptr() == twin_w.data_ptr()
    layer.double()                                                       # new storage per parameter: packed again
    new_w, _ = layer._packed_parameters()
    assert new_w.dtype == torch.float64 and layer.D_proj.weight.data_ptr() == new_w.data_ptr() + 4 * S * H * 8
    layer.load_state_dict({k: v.double() for k, v in before.items()})
    kept_w, _ = layer._packed_parameters()
    assert kept_w is new_w and torch.equal(kept_w[S:2 * S].float(), before["B_proj.weight"])

    u = torch.randn(3, 5, H, dtype=torch.double, requires_grad=True)
    out = _PackedProjection.apply(u, *(getattr(layer, n).weight for n in order), layer.A_proj.bias, *layer._packed_parameters())
    ref = torch.cat([getattr(layer, n)(u) for n in order], dim=-1)
    assert torch.allclose(out, ref, rtol=1e-12, atol=1e-12)
    wrt = [u] + [getattr(layer, n).weight for n in order] + [layer.A_proj.bias]
    g = torch.randn_like(out)
    for got, want in zip(torch.autograd.grad(out, wrt, g), torch.autograd.grad(ref, wrt, g)):
        assert torch.allclose(got, want, rtol=1e-12, atol=1e-12)
