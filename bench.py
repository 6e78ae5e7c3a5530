#!/usr/bin/env python3
"""Benchmark of the gated linear scan hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload c1|c0|c2|c3scan|c4scan]

A step is one forward + backward of `scan()` (the public API, through autograd) over one batch
of synthetic operands already resident in HBM.  The default workload is the configuration the
headline metric is quoted on: bf16, B=8, L=4096, D=2048, block_l=256, checkpoint=True.

One JSON line is printed.  `value` is algorithmic HBM bytes per step (forward: read x, a, b, c,
write y; backward: read x, a, b, c, dy, write dx, da, db, dc; state rebuild and carries count as
zero) divided by the measured time per step.  `roofline` prices the dominant kernel (the
backward: 9 of the 14 tensor passes) from HIP-event timing of back-to-back launches on the
launch stream.  `cpu_baseline` times the torch restatement of the reference's CPU path on a
bounded slice of the same workload on this box's host cores.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))

HBM_PEAK_GBS = 8000.0  # MI355X published HBM3E peak, 8 TB/s
SETTLE_MS = 30.0        # untimed load in front of the first measurement (see main)
IDLE_MS = 250.0         # idle spell in front of the `after_idle` figure

WORKLOADS = {
    # name: (B, L, D, operand dtype, y/dy dtype, a_lo, a_span, block_l, description)
    "c0": (4, 2048, 16, "float32", "float32", 0.9, 0.1, 256, "fp32 B=4 L=2048 D=16"),
    "c1": (8, 4096, 2048, "bfloat16", "bfloat16", 0.9, 0.1, 256, "bf16 B=8 L=4096 D=2048"),
    "c2": (1, 65536, 4096, "float16", "float16", 0.99, 0.01, 1024, "fp16 B=1 L=65536 D=4096"),
    "c3scan": (16, 2048, 4096, "float16", "float32", 0.9, 0.1, 256, "fp16 operands, fp32 y/dy, B=16 L=2048 D=4096"),
    "c4scan": (32, 64, 1024, "float16", "float32", 0.9, 0.1, 256, "fp16 operands, fp32 y/dy, B=32 L=64 D=1024"),
}


def make_operands(torch, shape, dtype, out_dtype, a_lo, a_span, device, seed=0):
    g = torch.Generator(device="cpu").manual_seed(seed)
    x = torch.randn(shape, generator=g)
    a = torch.rand(shape, generator=g) * a_span + a_lo
    b = torch.randn(shape, generator=g) * 0.1
    c = torch.sigmoid(torch.randn(shape, generator=g))
    dy = torch.randn(shape, generator=g)
    ops = [t.to(dtype) for t in (x, a, b, c)] + [dy.to(out_dtype)]
    return ops, [t.to(device) for t in ops]


def event_time_ms(torch, fn, iters, warmup):
    """Average duration of `fn` over `iters` back-to-back calls, from events on the current stream."""
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    start = torch.cuda.Event(enable_timing=True)
    stop = torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(iters):
        fn()
    stop.record()
    torch.cuda.synchronize()
    return start.elapsed_time(stop) / iters


def alternating_times_ms(torch, first, second, iters, warmup):
    """Average durations of `first` and `second` when they run in turn, as the two launches of a step do (an event
    between every two launches on the current stream).  What the second finds in the caches is what the first left."""
    for _ in range(warmup):
        first()
        second()
    torch.cuda.synchronize()
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(2 * iters + 1)]
    ev[0].record()
    for k in range(iters):
        first()
        ev[2 * k + 1].record()
        second()
        ev[2 * k + 2].record()
    torch.cuda.synchronize()
    t1 = sum(ev[2 * k].elapsed_time(ev[2 * k + 1]) for k in range(iters)) / iters
    t2 = sum(ev[2 * k + 1].elapsed_time(ev[2 * k + 2]) for k in range(iters)) / iters
    return t1, t2


def kernel_source_hash() -> str:
    """Hash of the scan kernels' sources: measured traffic is only quoted for the kernels it was measured on."""
    import hashlib

    h = hashlib.sha256()
    for name in ("scan_common.h", "scan_fwd.hip", "scan_bwd.hip"):
        h.update((ROOT / "quick_ssm_amd" / "csrc" / name).read_bytes())
    return h.hexdigest()[:16]


def cpu_baseline(torch, workload, shape, dtype, out_dtype, a_lo, a_span):
    """The reference CPU path (torch restatement, oracle/reference_cpu_path.py) on a bounded slice, plus the two legs
    the path can do in full: the fp32 B=4 L=2048 D=16 configuration forward + backward, and this workload's forward
    at full shape under no_grad (both bounded by the clock: rows stop being added after 8 s)."""
    from oracle.reference_cpu_path import reference_scan, reference_scan_with_grads

    B, L, D = shape
    # One batch row with every column of the workload.  The reference's backward through its in-place slice writes
    # costs O(L^2) whole-row copies once a row outgrows the host's caches, so rows are cut to 2048 steps.
    sB, sL, sD = 1, min(L, 2048), D
    ops, _ = make_operands(torch, (sB, sL, sD), dtype, out_dtype, a_lo, a_span, "cpu")
    # Hosts differ by more than 10x on this path: repeat the row until about 10 s of CPU work are on the clock.
    rows, dt = 0, 0.0
    while dt < 10.0 and rows < 64:
        t0 = time.perf_counter()
        reference_scan_with_grads(*ops, out_dtype=out_dtype)
        dt += time.perf_counter() - t0
        rows += 1
    sB = rows
    n = sB * sL * sD
    es, os_ = ops[0].element_size(), ops[4].element_size()
    nbytes = n * (8 * es + 2 * os_)
    out = {
        "value": nbytes / dt / 1e9,
        "unit": "GB/s",
        "cores": torch.get_num_threads(),
        "kind": "port",
        "sample": f"reference CPU path (python loop over batch and time, torch autograd backward) fwd+bwd on a "
                  f"slice L={sL} D={sD} of {workload} run {sB} time(s), {dt:.2f} s, host cpu_count={os.cpu_count()}",
        "melem_per_s": n / dt / 1e6,
        "seconds": dt,
    }
    # the configuration the reference's CPU path runs in full: fp32 B=4 L=2048 D=16, forward + backward
    c0 = WORKLOADS["c0"]
    ops0, _ = make_operands(torch, c0[:3], torch.float32, torch.float32, c0[5], c0[6], "cpu")
    t0 = time.perf_counter()
    reference_scan_with_grads(*ops0, out_dtype=torch.float32)
    dt0 = time.perf_counter() - t0
    n0 = c0[0] * c0[1] * c0[2]
    out["c0_full"] = {"seconds": dt0, "melem_per_s": n0 / dt0 / 1e6, "gbs": n0 * 14 * 4 / dt0 / 1e9,
                      "sample": "fp32 B=4 L=2048 D=16 fwd+bwd, whole configuration"}
    # this workload's forward at its full shape under no_grad, batch row by batch row until the clock says stop
    with torch.no_grad():
        done, dtf = 0, 0.0
        ops1, _ = make_operands(torch, (1, L, D), dtype, out_dtype, a_lo, a_span, "cpu")
        while done < B and dtf < 8.0:
            t0 = time.perf_counter()
            reference_scan(*ops1[:4], out_dtype=out_dtype)
            dtf += time.perf_counter() - t0
            done += 1
    nf = done * L * D
    out["forward_full_shape"] = {"seconds": dtf, "rows_done": done, "rows": B, "melem_per_s": nf / dtf / 1e6,
                                 "gbs": nf * (4 * es + os_) / dtf / 1e9,
                                 "sample": f"forward only, no_grad, L={L} D={D}, {done} of {B} batch rows"}
    return out


def record_traffic(fetch_csv: str, write_csv: str, workload: str) -> int:
    """Turn two rocprofv3 counter runs of this script (`--pmc FETCH_SIZE`, `--pmc WRITE_SIZE`, each with
    `--kernel-trace --output-format csv`) into profiles/scan_bwd_<workload>_traffic.json: the backward's HBM bytes
    per launch, each counter scaled by what it reads for the calibration copy of known size in the same run, tagged
    with the hash of the kernel sources so that a later run only quotes it while they are unchanged."""
    import csv

    def mean_kib(path: str, counter: str, kernel: str) -> float:
        vals = [float(r["Counter_Value"]) for r in csv.DictReader(open(path))
                if kernel in r["Kernel_Name"] and r["Counter_Name"] == counter]
        if not vals:
            raise SystemExit(f"{path}: no {counter} rows for {kernel}")
        return sum(vals) / len(vals)

    B, L, D, dt_name, out_name = WORKLOADS[workload][:5]
    n = B * L * D
    es = {"float32": 4, "float16": 2, "bfloat16": 2}
    copy_kib = (n * (8 * es[dt_name] + es[out_name]) // 2 // 16) * 16 / 1024      # what the calibration copy moves each way
    fetch = mean_kib(fetch_csv, "FETCH_SIZE", "scan_bwd") * copy_kib / mean_kib(fetch_csv, "FETCH_SIZE", "copy_kernel")
    write = mean_kib(write_csv, "WRITE_SIZE", "scan_bwd") * copy_kib / mean_kib(write_csv, "WRITE_SIZE", "copy_kernel")
    rec = {"kernel": "scan_bwd_kernel", "workload": workload, "traffic_bytes_per_launch": int(fetch * 1024) + int(write * 1024),
           "fetch_bytes": int(fetch * 1024), "write_bytes": int(write * 1024), "kernel_source_hash": kernel_source_hash(),
           "source": f"profiles/scan_{workload}_{ {'float32': 'f32', 'float16': 'fp16', 'bfloat16': 'bf16'}[dt_name] }_hbm_traffic.md"}
    out = ROOT / "profiles" / f"scan_bwd_{workload}_traffic.json"
    out.write_text(json.dumps(rec, indent=1))
    print(json.dumps(rec))
    return 0


def settle_timeline(torch, step) -> int:
    """Per-step durations (HIP events between the steps) of 60 steps begun right after idle spells of different
    lengths, printed as text: how long the device takes to settle after a pause, and from which pause on."""
    def timeline(n):
        torch.cuda.synchronize()
        ev = [torch.cuda.Event(enable_timing=True) for _ in range(n + 1)]
        ev[0].record()
        for k in range(n):
            step()
            ev[k + 1].record()
        torch.cuda.synchronize()
        return [ev[k].elapsed_time(ev[k + 1]) * 1e3 for k in range(n)]

    for _ in range(100):     # 30 ms and more of load first: the settled rate
        step()
    base = timeline(60)
    print(f"settled: mean of 60 steps {sum(base[1:]) / 59:.1f} us (first step after the synchronize: {base[0]:.0f} us)")
    for idle_ms in (2, 5, 10, 20, 50, 200):
        time.sleep(idle_ms * 1e-3)
        per = timeline(60)
        print(f"after {idle_ms:3d} ms idle: steps 2-10 {sum(per[1:10]) / 9:.1f} us, 11-20 {sum(per[10:20]) / 10:.1f}, "
              f"21-30 {sum(per[20:30]) / 10:.1f}, 31-60 {sum(per[30:]) / 30:.1f} | " + " ".join(f"{p:.0f}" for p in per[:40]), flush=True)
    return 0


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--record-traffic", nargs=2, metavar=("FETCH_CSV", "WRITE_CSV"),
                    help="no GPU work: write profiles/scan_bwd_<workload>_traffic.json from two counter_collection.csv files")
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=30)
    ap.add_argument("--workload", default="c1", choices=sorted(WORKLOADS))
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--settle-timeline", action="store_true",
                    help="instead of the benchmark: per-step times of the steps that follow idle spells of 2 to 200 ms "
                         "(what the untimed run-in in front of the measurements is for)")
    args = ap.parse_args()
    if args.record_traffic:
        return record_traffic(args.record_traffic[0], args.record_traffic[1], args.workload)

    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py measures one GPU: rows (b, d) of the scan are independent, so more GPUs only shard B or D "
              "with no communication. Run with --gpus 1.", file=sys.stderr)
        return 2

    import torch

    from quick_ssm_amd import _lib, hip_scan
    from quick_ssm_amd.scan_interface import scan

    if not _lib.is_built():
        from quick_ssm_amd import build as builder

        builder.build(verbose=False)
    if not torch.cuda.is_available():
        print("bench.py needs a GPU (the scan has no CPU product path to measure)", file=sys.stderr)
        return 2
    dev = torch.device("cuda", 0)
    torch.cuda.set_device(dev)

    B, L, D, dt_name, odt_name, a_lo, a_span, block_l, desc = WORKLOADS[args.workload]
    dtype, out_dtype = getattr(torch, dt_name), getattr(torch, odt_name)
    shape = (B, L, D)
    n = B * L * D
    cpu_ops, (x, a, b, c, dy) = make_operands(torch, shape, dtype, out_dtype, a_lo, a_span, dev)
    del cpu_ops
    es, os_ = x.element_size(), dy.element_size()
    fwd_bytes = n * (4 * es + os_)
    bwd_bytes = n * (8 * es + os_)
    step_bytes = fwd_bytes + bwd_bytes

    leaves = [t.requires_grad_(True) for t in (x, a, b, c)]

    # Small workloads would otherwise be timed out of the 256 MB Infinity Cache: steps rotate over enough
    # copies of the operands that a step never finds its own data from the previous round in cache.
    working_set = step_bytes + n * 4   # operands, results and the gradients autograd keeps
    n_sets = 1 if working_set >= (512 << 20) else min(64, -(-(1 << 30) // working_set))
    sets = [(leaves, dy)]
    for _ in range(n_sets - 1):
        sets.append(([t.detach().clone().requires_grad_(True) for t in leaves], dy.clone()))
    turn = [0]

    def step():
        ops, gy = sets[turn[0] % n_sets]
        turn[0] += 1
        y = scan(*ops, block_l=block_l, checkpoint=True, out_dtype=out_dtype)
        # one device, one graph: run the backward on this thread instead of waking autograd's device thread (the
        # hand-over costs more than the launch it brackets when the workload is small; it changes nothing on the GPU)
        with torch.autograd.set_multithreading_enabled(False):
            y.backward(gy)
        # gradients are dropped at the end of the step, as a training loop's zero_grad(set_to_none=True) does: the
        # next step starts with its forward launch
        for t in ops:
            t.grad = None

    if args.settle_timeline:
        return settle_timeline(torch, step)

    # ---- everything the run needs exists before the first measured launch ------------------------
    # An allocation of this size is milliseconds of idle GPU, and an idle spell of 10 ms or more is followed by
    # about 10 ms in which the device runs the same launches up to 8 % slower (it starts fast, sags after 1-2 ms
    # and recovers; profiles/device_settle_timeline.md): every leg below therefore follows the one before without
    # a pause, behind a run of untimed launches that outlasts that spell, and what is reported is the settled
    # rate a job that keeps the device busy sees.  `after_idle` at the end reports the other case.
    xd, ad, bd, cd = (t.detach() for t in leaves)
    nb = (bwd_bytes // 2 // 16) * 16
    src = torch.empty(nb, dtype=torch.uint8, device=dev)
    dst = torch.empty(nb, dtype=torch.uint8, device=dev)
    stream = torch.cuda.current_stream().cuda_stream
    lib = _lib.load()
    step()          # plans, argument blocks, control block, workspace and the allocator's blocks for y and the gradients
    with torch.no_grad():
        _, _, ckpt, stride = hip_scan.scan_forward(xd, ad, bd, cd, out_dtype=out_dtype)
        detached = [tuple(t.detach() for t in ops) + (gy,) for ops, gy in sets]

        def fwd_once():
            xs, as_, bs, cs, _ = detached[turn[0] % n_sets]
            turn[0] += 1
            hip_scan.scan_forward(xs, as_, bs, cs, out_dtype=out_dtype)

        def bwd_once():
            xs, as_, bs, cs, gy = detached[turn[0] % n_sets]
            turn[0] += 1
            hip_scan.scan_backward(xs, as_, bs, cs, gy, ckpt=ckpt, ckpt_stride=stride)

        def fwd_same_set():
            xs, as_, bs, cs, _ = detached[turn[0] % n_sets]
            hip_scan.scan_forward(xs, as_, bs, cs, out_dtype=out_dtype)

        # untimed: the two launches in turn until the device has been busy for SETTLE_MS without a pause
        torch.cuda.synchronize()
        t_settle = time.perf_counter()
        settle_pairs = 0
        while (time.perf_counter() - t_settle) * 1e3 < SETTLE_MS:
            for _ in range(8):
                fwd_same_set()
                bwd_once()
            settle_pairs += 8
            torch.cuda.synchronize()

        # ---- the two kernels on their own, through the C ABI ---------------------------------------
        # each launch repeated on its own (a forward then finds the operands its predecessor kept in the caches for
        # a backward that never came, so this figure flatters it), and the two in turn as a step runs them
        fwd_alone_ms = event_time_ms(torch, fwd_once, args.steps, args.warmup)
        bwd_alone_ms = event_time_ms(torch, bwd_once, args.steps, args.warmup)
        # achievable ceiling on this box: a plain copy of the same number of bytes as the backward moves
        copy_ms = event_time_ms(torch, lambda: lib.qssm_copy_bytes(dst.data_ptr(), src.data_ptr(), nb, stream),
                                args.steps, args.warmup)
        # the forward without its cache policy (every operand streamed past the caches) and the backward behind it:
        # what the pair costs when other work runs between a layer's forward and its backward
        hip_scan.set_forward_keep(False)
        fwd_nokeep_ms, bwd_nokeep_ms = alternating_times_ms(torch, fwd_same_set, bwd_once, args.steps, args.warmup)
        hip_scan.set_forward_keep(True)
        fwd_ms, bwd_ms = alternating_times_ms(torch, fwd_same_set, bwd_once, args.steps, args.warmup)
    # ---- whole step through the public API: W warm-ups, then exactly K timed steps ---------------
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / args.steps
    ms_per_step = wall_ms
    # the same K steps once more between two HIP events, for the GPU's own clock beside the host's (the headline is
    # the wall clock above; events inside that region would only add host work in front of its first launch)
    ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    ev0.record()
    for _ in range(args.steps):
        step()
    ev1.record()
    torch.cuda.synchronize()
    gpu_ms = ev0.elapsed_time(ev1) / args.steps

    # the same K steps right after an idle spell, no warm-up: what a job that leaves the device idle between steps sees
    time.sleep(IDLE_MS * 1e-3)
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    after_idle_ms = (time.perf_counter() - t0) * 1e3 / args.steps
    del src, dst

    status = hip_scan.workspace_status()
    align = hip_scan._align_elems([xd, ad, bd, cd, dy], D)   # what the timed launches were planned with
    plan_b = hip_scan.make_plan(B, L, D, dtype, out_dtype, _lib.QSSM_BACKWARD, align, stride)
    plan_f = hip_scan.make_plan(B, L, D, dtype, out_dtype, _lib.QSSM_FORWARD, align, stride)

    # HBM bytes per launch of the dominant kernel, from rocprofv3 FETCH_SIZE / WRITE_SIZE runs of this command: only
    # quoted while the kernels are the ones it was measured on
    traffic, traffic_note = None, "not measured for this workload"
    traffic_file = ROOT / "profiles" / f"scan_bwd_{args.workload}_traffic.json"
    if traffic_file.exists():
        try:
            rec = json.loads(traffic_file.read_text())
            if rec.get("kernel_source_hash") == kernel_source_hash():
                traffic, traffic_note = rec.get("traffic_bytes_per_launch"), rec.get("source", "")
            else:
                traffic_note = "kernel sources changed since profiles/ was measured"
        except (ValueError, OSError):
            traffic = None

    bwd_gbs = bwd_bytes / (bwd_ms * 1e-3) / 1e9
    fwd_gbs = fwd_bytes / (fwd_ms * 1e-3) / 1e9
    value = step_bytes / (ms_per_step * 1e-3) / 1e9
    out = {
        "metric": f"scan fwd+bwd HBM GB/s (% of peak) + Melem/s, {desc}",
        "value": value,
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        # the arithmetic type the path computes in; storage of the operands noted beside it
        "dtype": "f32 (" + {"float32": "f32", "float16": "f16", "bfloat16": "bf16"}[dt_name] + " storage)",
        "data": "synthetic",
        "config": {"workload": f"{args.workload}: gated linear scan fwd+bwd through scan(), {desc}, "
                               f"block_l={block_l}, checkpoint=True", "B": B, "L": L, "D": D},
        "pct_of_hbm_peak": 100.0 * value / HBM_PEAK_GBS,
        "melem_per_s": n / (ms_per_step * 1e-3) / 1e6,
        "algorithmic_bytes_per_step": step_bytes,
        "gpu_ms_per_step_events": gpu_ms,
        "kernels_only_gbs": step_bytes / ((fwd_ms + bwd_ms) * 1e-3) / 1e9,
        "roofline": {
            "bound": "hbm",
            "kernel": "scan_bwd_kernel",
            "achieved": bwd_gbs,
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": bwd_gbs / HBM_PEAK_GBS,
            "traffic": traffic,
            "traffic_note": traffic_note,
            "algorithmic_bytes_per_launch": bwd_bytes,
            "avg_launch_ms": bwd_ms,
        },
        "kernels": {
            "scan_fwd_kernel": {"avg_launch_ms": fwd_ms, "repeated_on_its_own_ms": fwd_alone_ms,
                                "algorithmic_bytes": fwd_bytes, "gbs": fwd_gbs,
                                "frac": fwd_gbs / HBM_PEAK_GBS, "plan": plan_f.describe()},
            "scan_bwd_kernel": {"avg_launch_ms": bwd_ms, "repeated_on_its_own_ms": bwd_alone_ms,
                                "algorithmic_bytes": bwd_bytes, "gbs": bwd_gbs,
                                "frac": bwd_gbs / HBM_PEAK_GBS, "plan": plan_b.describe()},
            "copy_kernel": {"avg_launch_ms": copy_ms, "bytes_moved": 2 * nb, "gbs": 2 * nb / (copy_ms * 1e-3) / 1e9},
        },
        "workspace_status": status,
        "rotated_operand_sets": n_sets,
        # untimed fwd+bwd pairs in front of every measurement (the device settles for about 10 ms after an idle spell)
        "settle": {"ms": SETTLE_MS, "pairs": settle_pairs},
        # the same K steps begun right after an idle spell, no warm-up
        "after_idle": {"idle_ms": IDLE_MS, "steps": args.steps, "ms_per_step": after_idle_ms,
                       "pct_of_hbm_peak": 100.0 * step_bytes / (after_idle_ms * 1e-3) / 1e9 / HBM_PEAK_GBS},
        # the two launches in turn with every operand of the forward streamed past the caches (plan.keep_tiles = 0):
        # the pair's cost when other work runs between a forward and its backward
        "without_cache_policy": {"fwd_ms": fwd_nokeep_ms, "bwd_ms": bwd_nokeep_ms,
                                 "pct_of_hbm_peak": 100.0 * step_bytes / ((fwd_nokeep_ms + bwd_nokeep_ms) * 1e-3) / 1e9 / HBM_PEAK_GBS},
    }
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(torch, args.workload, shape, dtype, out_dtype, a_lo, a_span)
    print(json.dumps(out), flush=True)
    return 0 if status == 0 else 1


if __name__ == "__main__":
    sys.exit(main())
