"""The copy-task harness (quick_ssm_amd/copy_task.py): host logic on the CPU, one training step on the GPU."""
from __future__ import annotations

import copy

import pytest
import torch

from quick_ssm_amd import copy_task


def test_teacher_batch_layout():
    gen = torch.Generator().manual_seed(0)
    inp, lab = copy_task.build_teacher_batch(3, 5, "cpu", start_token=7, generator=gen)
    assert inp.shape == (3, 10) and lab.shape == (3, 10)
    src = inp[:, :5]
    assert torch.equal(inp[:, 5], torch.full((3,), 7))
    assert torch.equal(inp[:, 6:], src[:, :-1])
    assert torch.all(lab[:, :5] == copy_task.IGNORE) and torch.equal(lab[:, 5:], src)
    assert int(src.max()) < copy_task.VOCAB_SIZE == 62


def test_small_stack_learns_on_the_sequential_path():
    torch.manual_seed(0)
    model = copy_task.CopyStack(hidden=32, layers=2, compute_dtype=torch.float32, device="cpu")
    opt = torch.optim.AdamW(model.parameters(), lr=3e-3, weight_decay=0.0)
    gen = torch.Generator().manual_seed(1)
    losses = []
    for _ in range(40):
        tokens = copy_task.sample_batch(8, 6, "cpu", gen)
        loss, _ = copy_task.train_step(model, opt, tokens, tokens)   # identity copy: every position is a label
        losses.append(float(loss))
    assert losses[-1] < 0.7 * losses[0]


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16], ids=["fp32", "fp16", "bf16"])
def test_training_step_on_hip_matches_sequential_path(gpu, dtype):
    # config 4's shape (12 layers, hidden 256, state 1024, B 32, L 64 + 64 teacher-forced); the same model and batch
    # stepped once with the HIP scan and once with the sequential torch scan on the same device
    torch.manual_seed(0)
    hip_model = copy_task.CopyStack(hidden=256, layers=12, compute_dtype=dtype, device=gpu)
    seq_model = copy.deepcopy(hip_model)
    seq_model.backend = "torch"
    gen = torch.Generator().manual_seed(2)
    tokens, labels = copy_task.build_teacher_batch(32, 64, gpu, generator=gen)
    out = []
    for model in (hip_model, seq_model):
        opt = torch.optim.AdamW(model.parameters(), lr=1e-3, weight_decay=0.0)
        loss, logits = copy_task.train_step(model, opt, tokens, labels)
        out.append((float(loss), logits.float().cpu(), [p.detach().float().cpu() for p in model.parameters()]))
    tol = {torch.float32: 1e-4, torch.float16: 2e-2, torch.bfloat16: 5e-2}[dtype]
    (l0, g0, p0), (l1, g1, p1) = out
    assert abs(l0 - l1) <= tol * max(1.0, abs(l1)), (l0, l1)
    assert (g0 - g1).abs().max() <= tol * g1.abs().max()
    # one AdamW step moves every weight by about lr whatever the gradient's size, so compare the updated weights
    # only loosely: the direction of a near-zero gradient component is rounding noise
    worst = max(float((a - b).abs().max()) for a, b in zip(p0, p1))
    assert worst <= 2.5e-3, worst


@pytest.mark.gpu
def test_recording_the_training_step_is_refused_before_anything_is_recorded(gpu):
    # whole-step graph capture is unsupported (library memset nodes do not replay reliably here): the harness and the
    # layer say so instead of recording; nothing is launched inside the refused recordings
    import warnings

    from quick_ssm_amd.layers import SSM

    torch.manual_seed(0)
    model = copy_task.CopyStack(hidden=32, layers=1, compute_dtype=torch.float32, device=gpu)
    opt = torch.optim.AdamW(model.parameters(), lr=1e-3)
    tokens, labels = copy_task.build_teacher_batch(2, 8, gpu, generator=torch.Generator().manual_seed(1))
    copy_task.train_step(model, opt, tokens, labels)            # eager: fine
    layer = SSM(32, 2.0, device=gpu)
    xin = torch.randn(2, 16, 32, device=gpu)
    side = torch.cuda.Stream()
    with torch.cuda.stream(side), warnings.catch_warnings():
        warnings.simplefilter("ignore")
        with pytest.raises(RuntimeError, match="cannot be recorded"):
            with torch.cuda.graph(torch.cuda.CUDAGraph(), stream=side):
                copy_task.train_step(model, opt, tokens, labels)
        with pytest.raises(RuntimeError, match="not supported"):
            with torch.cuda.graph(torch.cuda.CUDAGraph(), stream=side):
                layer(xin)
    torch.cuda.synchronize()
    loss, _ = copy_task.train_step(model, opt, tokens, labels)  # and the eager step still works afterwards
    assert torch.isfinite(loss)
