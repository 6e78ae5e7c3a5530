"""Copy-task training harness: Embedding -> N x SSM -> vocabulary head, cross-entropy, AdamW.

Modelled on the reference's copy_train.py (vocabulary :12-13, model :20-38, teacher-forced batches
:41-57, AdamW + gradient clipping loop :60-95), with a stack of SSM layers instead of one: the
12-layer, hidden-256 configuration whose training curves the reference's README shows.

    python -m quick_ssm_amd.copy_task --steps 200 --teacher-forcing

Every layer's scan goes through `quick_ssm_amd.scan` (HIP kernels for GPU tensors, the sequential
torch recurrence on CPU or with --backend torch).
"""
from __future__ import annotations

import argparse
import string
import time
from typing import Optional, Tuple

import torch
import torch.nn as nn
import torch.nn.functional as F

from .layers import SSM

VOCAB = string.ascii_letters + string.digits  # 62 symbols
VOCAB_SIZE = len(VOCAB)
IGNORE = -100


def sample_batch(batch_size: int, seq_len: int, device, generator: Optional[torch.Generator] = None) -> torch.Tensor:
    """Uniform random strings over the vocabulary, [batch_size, seq_len] int64."""
    tokens = torch.randint(0, VOCAB_SIZE, (batch_size, seq_len), dtype=torch.long, generator=generator)
    return tokens.to(device)


def build_teacher_batch(batch_size: int, seq_len: int, device, start_token: int = 0,
                        generator: Optional[torch.Generator] = None) -> Tuple[torch.Tensor, torch.Tensor]:
    """Teacher-forced copying: inputs = [src, start + src[:-1]], labels = [ignored, src]."""
    src = sample_batch(batch_size, seq_len, device, generator)
    start = torch.full((batch_size, 1), start_token, device=src.device, dtype=src.dtype)
    inputs = torch.cat([src, start, src[:, :-1]], dim=1)
    labels = torch.cat([torch.full_like(src, IGNORE), src], dim=1)
    return inputs, labels


class CopyStack(nn.Module):
    """Token embedding, `layers` SSM layers (fp32 parameters, `compute_dtype` scan), linear head."""

    def __init__(self, hidden: int = 256, layers: int = 12, compute_dtype: torch.dtype = torch.float16,
                 device=None, state_size_mult: float = 4.0, backend: str = "auto"):
        super().__init__()
        self.backend = backend
        self.embed = nn.Embedding(VOCAB_SIZE, hidden, device=device)
        self.layers = nn.ModuleList(
            SSM(hidden_size=hidden, state_size_mult=state_size_mult, compute_dtype=compute_dtype,
                dtype=torch.float32, use_residual=True, use_norm=True, device=device)
            for _ in range(layers)
        )
        self.head = nn.Linear(hidden, VOCAB_SIZE, device=device)

    def forward(self, tokens: torch.Tensor) -> torch.Tensor:
        h = self.embed(tokens)
        for layer in self.layers:
            # one chunk per sequence, as the reference's script asks for (block_l >= L); fp32 scan output
            h = layer(h, block_l=128, checkpoint=True, scan_out_dtype=torch.float32, backend=self.backend)
        return self.head(h)


def loss_fn(logits: torch.Tensor, labels: torch.Tensor) -> torch.Tensor:
    return F.cross_entropy(logits.view(-1, VOCAB_SIZE), labels.view(-1), ignore_index=IGNORE)


def train_step(model: nn.Module, opt: torch.optim.Optimizer, tokens: torch.Tensor, labels: torch.Tensor,
               max_norm: float = 1.0) -> Tuple[torch.Tensor, torch.Tensor]:
    """One optimisation step (forward, loss, backward, gradient clipping at `max_norm`, AdamW).  Returns (loss, logits).

    The step runs eagerly.  Recording it into a HIP graph is refused: the backward of its torch library calls (bias
    and embedding gradients, the loss reduction, gradient clipping) records memset nodes, which this platform does
    not replay reliably (a recording of the whole step drifted from the eager step after two replays, one of
    forward + backward faulted on replay).  The scan launches on their own can be recorded
    (`hip_scan.device_counted_launches`)."""
    if tokens.is_cuda and torch.cuda.is_current_stream_capturing():
        raise RuntimeError(
            "quick_ssm_amd.copy_task.train_step cannot be recorded into a HIP graph: its torch library calls record "
            "memset nodes that do not replay reliably on this platform. Run the step eagerly; scan launches alone "
            "can be recorded (hip_scan.device_counted_launches).")
    logits = model(tokens)
    loss = loss_fn(logits, labels)
    opt.zero_grad(set_to_none=True)
    # One GPU, one graph: the backward runs on the calling thread.  At this size the step is bound by the host
    # side of its ~1000 small launches, and handing each backward node to autograd's device thread and waiting for
    # it costs more than the node's own launch.
    with torch.autograd.set_multithreading_enabled(False):
        loss.backward()
    torch.nn.utils.clip_grad_norm_(model.parameters(), max_norm=max_norm)
    opt.step()
    return loss.detach(), logits.detach()


def token_accuracy(logits: torch.Tensor, labels: torch.Tensor) -> float:
    mask = labels != IGNORE
    return (logits.argmax(dim=-1)[mask] == labels[mask]).float().mean().item()


def train(args: argparse.Namespace) -> float:
    torch.manual_seed(args.seed)
    device = torch.device("cuda" if torch.cuda.is_available() and not args.cpu else "cpu")
    dtype = {"fp32": torch.float32, "fp16": torch.float16, "bf16": torch.bfloat16}[args.compute_dtype]
    if device.type == "cpu" and dtype == torch.float16:
        dtype = torch.float32
    model = CopyStack(args.hidden, args.layers, dtype, device, backend=args.backend)
    opt = torch.optim.AdamW(model.parameters(), lr=args.lr, weight_decay=0.0)
    loss = torch.zeros(())
    t0 = time.perf_counter()
    for step in range(1, args.steps + 1):
        if args.teacher_forcing:
            tokens, labels = build_teacher_batch(args.batch_size, args.seq_len, device)
        else:
            tokens = sample_batch(args.batch_size, args.seq_len, device)
            labels = tokens
        loss, logits = train_step(model, opt, tokens, labels)
        if step % args.log_interval == 0 or step == 1:
            print(f"step {step:04d} | loss {loss.item():.6f} | token-acc {token_accuracy(logits, labels):.4f}", flush=True)
    if device.type == "cuda":
        torch.cuda.synchronize()
    print(f"{args.steps} steps in {time.perf_counter() - t0:.2f} s")
    return float(loss)


def parse_args(argv=None) -> argparse.Namespace:
    p = argparse.ArgumentParser(description="Copying toy task on a stack of SSM layers")
    p.add_argument("--steps", type=int, default=200)
    p.add_argument("--batch-size", type=int, default=32)
    p.add_argument("--seq-len", type=int, default=64)
    p.add_argument("--hidden", type=int, default=256)
    p.add_argument("--layers", type=int, default=12)
    p.add_argument("--lr", type=float, default=1e-3)
    p.add_argument("--log-interval", type=int, default=20)
    p.add_argument("--seed", type=int, default=0)
    p.add_argument("--compute-dtype", choices=("fp32", "fp16", "bf16"), default="fp16")
    p.add_argument("--backend", choices=("auto", "hip", "torch"), default="auto")
    p.add_argument("--cpu", action="store_true", help="stay on the CPU even if a GPU is there")
    p.add_argument("--teacher-forcing", action="store_true", help="inputs [src, src], loss on the second half only")
    return p.parse_args(argv)


if __name__ == "__main__":
    train(parse_args())
