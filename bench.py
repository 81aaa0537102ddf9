#!/usr/bin/env python3
"""Benchmark of the fused linear cross-entropy (forward + backward) on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME]

A step is one forward + backward of ``tiled_linear_cross_entropy`` over one
synthetic batch that is already resident in HBM.  Prints ONE JSON line:
tokens/s (loss-bearing rows per second), the roofline of the dominant kernel
class measured live with HIP events, and the CPU oracle timed on a bounded row
sample of the same workload on this box's host cores.
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time
from pathlib import Path

REPO_ROOT = Path(__file__).resolve().parent
if str(REPO_ROOT) not in sys.path:
    sys.path.insert(0, str(REPO_ROOT))

PEAK_BF16_TFLOPS = 2500.0      # MI355X dense bf16 MFMA
PEAK_HBM_GBS = 8000.0          # MI355X HBM3E


def build_workload(name: str, seed: int):
    from turbo_dllm_amd import workloads

    if name == "block_diffusion_shard_all_rows":
        return workloads.block_diffusion_shard(seed=seed, all_rows_loss_bearing=True)
    return workloads.CONFIGS[name](seed=seed)


def _median(values):
    values = sorted(values)
    return values[len(values) // 2]


def _time_cpu_paths(hidden, weight, labels, softcap, iterations, warmup):
    """Median seconds (forward, backward) of the two CPU paths on the given rows:
    the float32 oracle (unfused matmul -> log-softmax -> masked NLL, analytic
    gradients) and this package's host implementation of the loss API
    (vocabulary tiles of 8192, autograd backward)."""
    import torch

    sys.path.insert(0, str(REPO_ROOT / "oracle"))
    import linear_ce_oracle as oracle
    from turbo_dllm_amd.tiled_linear_cross_entropy import tiled_linear_cross_entropy

    h32, w32 = hidden.float(), weight.float()
    unfused, tiled = [], []
    for it in range(warmup + iterations):
        t0 = time.perf_counter()
        oracle.dense_linear_ce(h32, w32, labels, logit_softcap=softcap, dtype=torch.float32)
        t1 = time.perf_counter()
        oracle.dense_linear_ce_grads(h32, w32, labels, logit_softcap=softcap, dtype=torch.float32)
        t2 = time.perf_counter()
        h = hidden.clone().requires_grad_(True)
        w = weight.clone().requires_grad_(True)
        t3 = time.perf_counter()
        loss = tiled_linear_cross_entropy(h, w, labels, vocab_block_size=8192,
                                          logit_softcap=softcap, dtype=torch.float32,
                                          weight_layout="vocab_first")
        t4 = time.perf_counter()
        loss.backward()
        t5 = time.perf_counter()
        if it >= warmup:
            unfused.append((t1 - t0, t2 - t1))
            tiled.append((t4 - t3, t5 - t4))

    def summary(samples, rows):
        fwd = _median([a for a, _ in samples])
        bwd = _median([b for _, b in samples])
        both = _median([a + b for a, b in samples])
        return {"forward_s": fwd, "backward_s": bwd, "forward_backward_s": both,
                "tokens_per_s": rows / both}

    rows = int((labels != -100).sum())
    return summary(unfused, rows), summary(tiled, rows)


def cpu_baseline(wl, sample_rows: int, iterations: int = 5, warmup: int = 2):
    """The CPU paths timed on this box's host cores beside the GPU kernels.

    ``value`` is the float32 oracle's forward+backward throughput on the first
    ``sample_rows`` loss-bearing rows of the workload at its full H and V (rows
    are independent, so tokens/s carries over to the whole batch up to the
    fixed cost of the [V, H] weight gradient, which the slice pays in full:
    the figure is an extrapolation that favours neither side much).  Also
    reported: this package's host implementation of the loss API on the same
    rows, and both paths on the small-head configuration at its full size
    (2048 rows, H=1024, V=32000).  Two warm-up and ``iterations`` timed passes
    each, medians."""
    import torch

    from turbo_dllm_amd import workloads

    keep = torch.nonzero(wl.labels != -100).flatten()[:sample_rows]
    hidden = wl.hidden.index_select(0, keep)
    labels = wl.labels.index_select(0, keep)
    cores = torch.get_num_threads()
    t_start = time.perf_counter()
    unfused, tiled = _time_cpu_paths(hidden, wl.weight, labels, wl.logit_softcap, iterations,
                                     warmup)
    small = workloads.small_head(seed=wl.seed)
    small_unfused, small_tiled = _time_cpu_paths(small.hidden, small.weight, small.labels, None,
                                                 iterations, warmup)
    rows = int(keep.numel())
    return {
        "value": unfused["tokens_per_s"],
        "unit": "tokens/s",
        "cores": cores,
        "kind": "port",
        "sample": f"float32 oracle (unfused path + analytic gradients), forward+backward on the "
                  f"first {rows} loss-bearing rows at full H and V, median of {iterations} "
                  f"after {warmup} warm-up passes; extrapolated per row to the whole batch",
        "oracle_unfused": unfused,
        "host_tiled_path": dict(tiled, note="turbo_dllm_amd host implementation of the loss "
                                            "API, vocabulary tile 8192, same rows"),
        "small_head_full_size": {
            "rows": small.n_rows, "loss_rows": small.n_loss_rows,
            "oracle_unfused": small_unfused, "host_tiled_path": small_tiled,
            "input_rows_per_s_unfused": small.n_rows / small_unfused["forward_backward_s"],
        },
        "cpu_seconds_spent": time.perf_counter() - t_start,
    }


def measure_compaction_gather(torch, native, device, n, h, hidden):
    """Ballot/prefix-sum compaction of a block-diffusion label mask plus the row
    gather of hidden and labels, timed with HIP events on the launch stream.
    Algorithmic bytes: 8N labels read twice is not counted, only 8N + 8M + 4MH
    (labels once, indices, rows read + written)."""
    gen = torch.Generator().manual_seed(7)
    half = n // 2
    blocks = max(half // 32, 1)
    t = torch.rand(blocks, generator=gen)
    noisy = (torch.rand(blocks, 32, generator=gen) < t[:, None]).reshape(-1)[:half]
    keep = torch.cat([torch.zeros(n - noisy.numel(), dtype=torch.bool), noisy])
    labels = torch.where(keep, torch.randint(0, 1000, (n,), generator=gen),
                         torch.full((n,), -100)).to(device)
    for _ in range(3):
        idx, m = native.compact_rows(labels, -100)
        native.gather_rows(hidden, idx)
    torch.cuda.synchronize()
    reps = 20
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(reps):
        idx, m = native.compact_rows(labels, -100)
        native.gather_rows(hidden, idx)
        native.gather_rows(labels, idx)
    stop.record()
    torch.cuda.synchronize()
    ms = start.elapsed_time(stop) / reps
    nbytes = 8 * n + 8 * m + 4 * m * h
    # the gather alone (no host read-back of the count inside the timed region)
    start.record()
    for _ in range(reps):
        native.gather_rows(hidden, idx)
    stop.record()
    torch.cuda.synchronize()
    gather_ms = start.elapsed_time(stop) / reps
    # the same pass without any host read-back: scan, then ONE gather of hidden rows, labels
    # and loss weights with the count read on the device
    weights = torch.ones(n, device=device)
    for _ in range(3):
        idx_all, count = native.compact_rows_device(labels, -100)
        native.gather_loss_rows(hidden, labels, weights, idx_all, count, -100)
    torch.cuda.synchronize()
    start.record()
    for _ in range(reps):
        idx_all, count = native.compact_rows_device(labels, -100)
        native.gather_loss_rows(hidden, labels, weights, idx_all, count, -100)
    stop.record()
    torch.cuda.synchronize()
    device_ms = start.elapsed_time(stop) / reps
    device_bytes = 8 * n + 8 * m + 4 * m * h + 24 * m
    return {
        "device_count_ms": device_ms, "device_count_algorithmic_bytes": device_bytes,
        "device_count_GB_per_s": device_bytes / device_ms / 1e6,
        "rows": n, "loss_rows": m, "ms": ms, "algorithmic_bytes": nbytes,
        "GB_per_s": nbytes / ms / 1e6,
        "gather_only_ms": gather_ms,
        "gather_only_GB_per_s": 4 * m * h / gather_ms / 1e6,
        "hbm_peak_GB_per_s": PEAK_HBM_GBS,
        "note": "compaction includes the host read-back of the row count",
    }


def source_fingerprint() -> str:
    """Short hash of the HIP sources: names the build a profile was taken from."""
    import hashlib

    digest = hashlib.sha256()
    csrc = REPO_ROOT / "turbo_dllm_amd" / "csrc"
    for path in sorted(csrc.glob("*.h")) + sorted(csrc.glob("*.hip")):
        digest.update(path.name.encode())
        digest.update(path.read_bytes())
    return digest.hexdigest()[:12]


TRAFFIC_PROFILE = REPO_ROOT / "profiles" / "hbm_traffic_per_kernel.txt"


def measured_traffic(workload: str, kernel: str):
    """Bytes between L2 and the memory fabric per launch of ``kernel`` on
    ``workload``, from the rocprofv3 FETCH_SIZE / WRITE_SIZE summary under
    profiles/ (counters cannot be read from inside the process).  The summary
    names the source fingerprint it was measured at; a figure measured on other
    sources is reported as stale, not as this build's."""
    if not TRAFFIC_PROFILE.exists():
        return None, "no traffic profile"
    current = source_fingerprint()
    for line in TRAFFIC_PROFILE.read_text().splitlines():
        fields = line.split()
        if len(fields) == 6 and fields[0] == "traffic" and fields[1] == workload \
                and fields[2] == kernel:
            total = float(fields[4]) + float(fields[5])
            if fields[3] == current:
                return total, f"measured on this build ({current})"
            return None, (f"stale: {total:.3g} B per launch was measured on sources "
                          f"{fields[3]}, these are {current}")
    return None, "not measured for this workload"


def library_gemm_reference(torch, device, h, v, rows=8192, panel=16384, reps=5):
    """What the vendor GEMM (torch.matmul -> hipBLASLt) reaches on this box for
    the three operand layouts of the path, bf16 with float32 accumulation: the
    logits contraction [rows,h] x [v,h]^T, and one vocabulary panel of the two
    gradient contractions, G [rows,panel] x W [panel,h] and G^T x hidden.  The
    practical ceiling for a plain GEMM, reported next to the fused kernels."""
    def timed(fn):
        for _ in range(2):
            fn()
        torch.cuda.synchronize()
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        for _ in range(reps):
            fn()
        stop.record()
        torch.cuda.synchronize()
        return start.elapsed_time(stop) / reps

    def entry(shape, ms, flops):
        tflops = flops / 1e12 / (ms / 1e3)
        return {"shape": shape, "ms": ms, "TFLOP_per_s": tflops,
                "frac_of_bf16_peak": tflops / PEAK_BF16_TFLOPS}

    bf16 = dict(device=device, dtype=torch.bfloat16)
    hidden = torch.randn(rows, h, **bf16)
    weight = torch.randn(v, h, **bf16) * 0.02
    out = torch.empty(rows, v, **bf16)
    result = entry(f"[{rows},{h}] x [{v},{h}]^T bf16",
                   timed(lambda: torch.matmul(hidden, weight.t(), out=out)), 2.0 * rows * h * v)
    del out
    m = 4 * rows
    g = torch.randn(m, panel, **bf16) * 0.01
    w_panel = weight[:panel]
    hidden_m = torch.randn(m, h, **bf16)
    flops = 2.0 * m * panel * h
    result["grad_hidden_panel"] = entry(f"[{m},{panel}] x [{panel},{h}] bf16",
                                        timed(lambda: torch.matmul(g, w_panel)), flops)
    result["grad_weight_panel"] = entry(f"[{m},{panel}]^T x [{m},{h}] bf16",
                                        timed(lambda: torch.matmul(g.t(), hidden_m)), flops)
    return result


def bench_masked_loss(args) -> int:
    """The loss method around the operator (output multiplier, mask token excluded,
    per-token weights, / valid_token_count) on the block-diffusion shard: the fused
    path against the reference's sequence of calls on the same kernels."""
    import torch

    from turbo_dllm_amd import chunked_linear_ce_native as native
    from turbo_dllm_amd import workloads
    from turbo_dllm_amd.compaction import compact_valid_loss_rows
    from turbo_dllm_amd.layers import VocabParallelLinear
    from turbo_dllm_amd.loss import masked_token_loss
    from turbo_dllm_amd.tiled_linear_cross_entropy import tiled_linear_cross_entropy

    device = torch.device("cuda:0")
    native.verify_device(0)
    wl = workloads.block_diffusion_shard(seed=args.seed)
    n, m = wl.n_rows, wl.n_loss_rows
    h, v = wl.hidden.shape[1], wl.weight.shape[0]
    head = VocabParallelLinear(h, v, bias=False).to(device=device, dtype=torch.bfloat16)
    with torch.no_grad():
        head.weight.copy_(wl.weight.to(device))
    hidden = wl.hidden.to(device).requires_grad_(True)
    labels = wl.labels.to(device)
    weights = (torch.rand(n, generator=torch.Generator().manual_seed(args.seed)) + 0.5).to(device)

    def fused():
        hidden.grad = None
        head.weight.grad = None
        loss = masked_token_loss(hidden, labels, weights, head, valid_token_count=float(m),
                                 mask_token_id=5, output_multiplier=0.5)
        loss.backward()
        return loss

    def reference_sequence():          # nemotron/model.py:2078-2151, unfused
        hidden.grad = None
        head.weight.grad = None
        rows, targets, w = compact_valid_loss_rows(hidden, labels, weights, ignore_index=-100)
        rows = rows * 0.5
        token_losses = tiled_linear_cross_entropy(rows, head.weight, targets, reduction="none",
                                                  exclude_index=5, dtype=rows.dtype,
                                                  weight_layout="vocab_first")
        loss = (token_losses.reshape(-1).float() * w).sum() / float(m)
        loss.backward()
        return loss

    def timed(fn):
        for _ in range(args.warmup):
            fn()
        torch.cuda.synchronize()
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        for _ in range(args.steps):
            loss = fn()
        stop.record()
        torch.cuda.synchronize()
        return start.elapsed_time(stop) / args.steps, float(loss.detach())

    from turbo_dllm_amd import options

    ms, loss = timed(fused)
    # the reference's own sequence of calls: per-token losses (reduction "none") whose
    # per-row upstream gradients reach the operator's backward; with the gradients formed
    # in the forward (3 contractions) and with the recomputing backward (4)
    ref_ms, ref_loss = timed(reference_sequence)
    with options.gradient_mode("recompute"):
        ref4_ms, _ = timed(reference_sequence)
    print(json.dumps({
        "metric": "masked-token loss fwd+bwd tokens/s", "value": m / (ms / 1e3),
        "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": f"masked_token_loss on {wl.name}: N={n} rows, M={m} loss-bearing, "
                               f"H={h}, V={v}, multiplier 0.5, mask token excluded, seed={args.seed}",
                   "compaction_mode": args.compaction_mode},
        "loss": loss,
        "reference_sequence_ms_per_step": ref_ms, "reference_sequence_loss": ref_loss,
        "reference_sequence_recompute_ms_per_step": ref4_ms,
    }), flush=True)
    return 0


def bench_next_objective(args) -> int:
    """The objectives built on the same kernels: frozen-head forward KL
    (forward + backward) and the streaming soft embedding (forward only)."""
    import torch

    from turbo_dllm_amd import _lib
    from turbo_dllm_amd import chunked_linear_ce_native as native
    from turbo_dllm_amd.dflash_kl import frozen_linear_kl
    from turbo_dllm_amd.streaming_soft_embedding import streaming_soft_embedding

    device = torch.device("cuda:0")
    native.verify_device(0)
    gen = torch.Generator().manual_seed(args.seed)
    m = args.rows

    def randn(rows, cols, std):
        return (torch.randn(rows, cols, generator=gen) * std).bfloat16().to(device)

    if args.objective == "kl":
        h, v = 4096, 151936
        draft_w, teacher_w = randn(v, h, 0.02), randn(v, h, 0.02)
        draft_h = randn(m, h, 1.0).requires_grad_(True)
        teacher_h = randn(m, h, 1.0)

        def step():
            draft_h.grad = None
            frozen_linear_kl(draft_h, draft_w, teacher_h, teacher_w).sum().backward()

        # one pass over the teacher head, one over the draft head, and the gradient
        # contraction, all in the forward; the backward scales rows
        # (--gradients recompute: 3 + 3)
        contractions = 3 if args.gradients == "forward" else 6
        name = "frozen-head KL fwd+bwd"
        shape = f"M={m}, H_draft=H_teacher={h}, V={v}"
    elif args.objective == "ce_topk":
        from turbo_dllm_amd.dflash_linear_topk import frozen_linear_ce_topk

        h, v, k = 4096, 151936, 16
        weight = randn(v, h, 0.02)
        hidden = randn(m, h, 1.0).requires_grad_(True)
        labels = torch.randint(0, v, (m,), generator=gen).to(device)

        def step():
            hidden.grad = None
            loss, prob, values, _ = frozen_linear_ce_topk(hidden, weight, labels, top_k=k)
            (loss.sum() + prob.sum() + values.sum()).backward()

        # the logits and, in the same forward, d lse / d hidden; the backward is a row pass
        # (--gradients recompute: 1 forward + 2 backward)
        contractions = 2 if args.gradients == "forward" else 3
        name = "frozen-head CE + top-16 fwd+bwd"
        shape = f"M={m}, H={h}, V={v}, top_k={k}"
    else:
        h, v = 3840, 262144
        weight, hidden = randn(v, h, 0.02), randn(m, h, 1.0)

        def step():
            streaming_soft_embedding(hidden, weight, row_chunk_size=1024, vocab_chunk_size=8192,
                                     logit_softcap=30.0)

        contractions, name = 2, "streaming soft embedding fwd"
        shape = f"M={m}, H={h}, V={v}, softcap=30"
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(args.steps):
        step()
    stop.record()
    torch.cuda.synchronize()
    ms = start.elapsed_time(stop) / args.steps
    with _lib.kernel_profile() as prof:
        step()
    torch.cuda.synchronize()
    executed = contractions * 2.0 * m * h * v / 1e12 / (ms / 1e3)
    print(json.dumps({
        "metric": f"{name} tokens/s", "value": m / (ms / 1e3), "unit": "tokens/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms, "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": f"{args.objective}: {shape}, seed={args.seed}"},
        "contractions_executed": contractions, "tflops_executed": executed,
        "mfma_util_executed": executed / PEAK_BF16_TFLOPS,
        "kernel_ms": {k: round(x, 3) for k, x in prof.ms.items()},
        "kernel_launches": prof.launches,
    }), flush=True)
    return 0


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--objective",
                    choices=("ce", "masked_loss", "kl", "soft_embedding", "ce_topk"), default="ce",
                    help="ce: the headline fused linear cross-entropy (default); masked_loss: the "
                         "loss method around it on the block-diffusion shard; kl / soft_embedding "
                         "/ ce_topk: the objectives built on the same kernels")
    ap.add_argument("--rows", type=int, default=8192, help="rows for --objective kl / soft_embedding")
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default="block_diffusion_shard_all_rows")
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--cpu-rows", type=int, default=512,
                    help="loss-bearing rows of the workload the CPU paths are timed on")
    ap.add_argument("--compaction-mode", choices=("sync", "device", "none"), default="sync",
                    help="how ignored rows are handled (tiled_linear_cross_entropy."
                         "set_compaction_mode): exact launches after one host read-back of "
                         "the row count, no read-back (device-side count), or no compaction")
    ap.add_argument("--panel-mib", type=int, default=0,
                    help="budget of the staging panel between the contractions in MiB (0: the "
                         "library's default, 2.5 GiB with --gradients forward, 1 GiB with "
                         "recompute)")
    ap.add_argument("--gradients", choices=("forward", "recompute"), default="forward",
                    help="form the gradients in the forward while a block's logits exist "
                         "(3 contractions per step; the package default) or in a backward "
                         "that recomputes the logits (4)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run one plain row copy of the weight matrix (known HBM bytes) "
                         "so rocprofv3 FETCH_SIZE / WRITE_SIZE readings can be scaled")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-library-gemm", action="store_true",
                    help="skip timing torch.matmul (hipBLASLt) on one contraction of this shape")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path "
              f"(--gpus {args.gpus} is not supported; use --gpus 1)", file=sys.stderr)
        return 2

    import torch

    from turbo_dllm_amd import _lib, options
    from turbo_dllm_amd import chunked_linear_ce_native as native
    from turbo_dllm_amd.tiled_linear_cross_entropy import (set_compaction_mode,
                                                           tiled_linear_cross_entropy)

    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        return 1
    set_compaction_mode(args.compaction_mode)
    options.set_panel_bytes(args.panel_mib << 20)
    options.set_gradient_mode(args.gradients)
    if args.objective == "masked_loss":
        return bench_masked_loss(args)
    if args.objective != "ce":
        return bench_next_objective(args)
    device = torch.device("cuda:0")
    native.verify_device(0)

    wl = build_workload(args.workload, args.seed)
    n, m = wl.n_rows, wl.n_loss_rows
    h, v = wl.hidden.shape[1], wl.weight.shape[0]
    hidden = wl.hidden.to(device).requires_grad_(True)
    weight = wl.weight.to(device).requires_grad_(True)
    labels = wl.labels.to(device)

    def step():
        hidden.grad = None
        weight.grad = None
        loss = tiled_linear_cross_entropy(hidden, weight, labels, reduction="mean",
                                          logit_softcap=wl.logit_softcap, dtype=hidden.dtype,
                                          weight_layout="vocab_first")
        loss.backward()
        return loss

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    # the timed region: exactly `steps` steps between two synchronisations; the
    # events between steps only yield the per-step spread (median) afterwards
    marks = [torch.cuda.Event(enable_timing=True) for _ in range(args.steps + 1)]
    marks[0].record()
    for i in range(args.steps):
        loss = step()
        marks[i + 1].record()
    torch.cuda.synchronize()
    ms_per_step = marks[0].elapsed_time(marks[-1]) / args.steps
    per_step = sorted(marks[i].elapsed_time(marks[i + 1]) for i in range(args.steps))
    ms_median = per_step[len(per_step) // 2] if per_step else float("nan")
    loss_value = float(loss.detach())

    # the two halves of a step, a few more steps with an event between them (outside the
    # timed region): with the gradients formed in the forward the backward only scales and
    # rounds them (and runs the grad_weight contraction when that one was postponed)
    halves = []
    for _ in range(min(args.steps, 5)):
        hidden.grad = None
        weight.grad = None
        e0, e1, e2 = (torch.cuda.Event(enable_timing=True) for _ in range(3))
        e0.record()
        loss = tiled_linear_cross_entropy(hidden, weight, labels, reduction="mean",
                                          logit_softcap=wl.logit_softcap, dtype=hidden.dtype,
                                          weight_layout="vocab_first")
        e1.record()
        loss.backward()
        e2.record()
        torch.cuda.synchronize()
        halves.append((e0.elapsed_time(e1), e1.elapsed_time(e2)))
    forward_ms = _median([a for a, _ in halves])
    backward_ms = _median([b for _, b in halves])

    # per-kernel-class durations of one forward + backward (HIP events on the launch stream;
    # the library calls are made directly so that all of them run on this thread)
    softcap = float(wl.logit_softcap or 0.0)
    go = torch.ones(1, device=device)
    with torch.no_grad():
        # the same operands and entry points the loss API uses for this compaction mode
        rows, targets, _, row_idx, count, m_rows = native.compact_loss_rows(
            hidden.detach(), labels, None, -100, args.compaction_mode)
        fused = (args.gradients == "forward"
                 and native.fused_gradients_supported(rows, weight.detach(), None, False))
        on_device = count if args.compaction_mode == "device" else None
        if fused:
            # as the autograd functions do: one block of rows -> the grad_weight contraction
            # waits for the upstream gradient and is stored in bf16 at once
            postpone = native.weight_grad_can_wait(m_rows, h, v, hidden.dtype)
            with _lib.kernel_profile() as prof:
                out = native.forward_with_gradients(
                    rows[:m_rows], weight.detach(), targets[:m_rows], ignore_index=-100,
                    exclude_index=-1, logit_softcap=softcap, compute_weight_grad=True,
                    row_idx=row_idx, n_out=n, row_count=on_device,
                    postpone_weight_grad=postpone)
                native.apply_grad_output(out[3], None if postpone else out[4], go, out[2],
                                         reduction="mean", dtype=hidden.dtype, row_idx=row_idx,
                                         n_out=n, row_count=on_device, vocab=v)
                if postpone:
                    native.grad_weight_from_panel(
                        rows[:m_rows], out[4], go, out[2], reduction="mean", vocab=v,
                        panel_bytes=options.get_panel_bytes(), row_count=on_device)
            del out
        elif count is not None:
            kw = dict(m=m_rows, row_idx=row_idx, row_count=count, n_out=n, ignore_index=-100,
                      exclude_index=-1, logit_softcap=softcap)
            with _lib.kernel_profile() as prof:
                _, lse, valid, _ = native.masked_loss_forward(
                    rows, weight.detach(), None, targets, None, want_losses=True, want_sum=False,
                    **kw)
                native.masked_loss_backward(rows, weight.detach(), None, targets, None, lse, valid,
                                            go, reduction="mean", **kw)
        else:
            kw = dict(row_block_size=0, ignore_index=-100, exclude_index=-1,
                      logit_softcap=softcap, compute_dtype=hidden.dtype,
                      weight_dim_first=False, row_idx=row_idx, n_out=n)
            with _lib.kernel_profile() as prof:
                _, lse, valid = native.forward(rows, weight.detach(), None, targets, **kw)
                native.backward(rows, weight.detach(), None, targets, lse, valid, go,
                                reduction="mean", **kw)
        torch.cuda.synchronize()

    if args.calibrate_copy:
        # gather_rows_kernel with identity indices = a plain copy: reads and writes v*h*2 bytes
        ident = torch.arange(v, device=device)
        native.gather_rows(weight.detach(), ident)
        torch.cuda.synchronize()

    # compaction + gather pass on the block-diffusion mask of this shape (HBM-bound)
    compaction = measure_compaction_gather(torch, native, device, n, h, hidden.detach())

    # kernels by symbol: both gradient contractions are launches of lce_gemm_nt_kernel
    contraction_tflop = 2.0 * m * h * v / 1e12          # algorithmic FLOPs of one contraction
    kernels = {
        "lce_forward_stats_kernel": (prof.ms["forward_stats"], prof.launches["forward_stats"], 1),
        "lce_grad_logits_panel_kernel": (prof.ms["grad_logits_panel"],
                                         prof.launches["grad_logits_panel"], 1),
        # every block of rows launches this kernel twice; the second launch is the
        # second try, which exits at once unless the block asked for it
        "lce_exp_logits_panel_kernel": (prof.ms["exp_logits_panel"],
                                        prof.launches["exp_logits_panel"] // 2, 1),
        "lce_gemm_nt_kernel": (prof.ms["grad_hidden_gemm"] + prof.ms["grad_weight_gemm"],
                               prof.launches["grad_hidden_gemm"]
                               + prof.launches["grad_weight_gemm"], 2),
    }
    dominant = max(kernels, key=lambda name: kernels[name][0])
    total_ms, launches, contractions = kernels[dominant]
    launches = max(launches, 1)
    avg_ms = total_ms / launches
    flops_per_launch = contractions * contraction_tflop * 1e12 / launches
    achieved = flops_per_launch / 1e12 / (avg_ms / 1e3)
    executed_contractions = 3 if fused else 4
    useful_tflops = 3.0 * contraction_tflop / (ms_per_step / 1e3)
    executed_tflops = executed_contractions * contraction_tflop / (ms_per_step / 1e3)
    # launches are sized for the loss-bearing rows, or for all rows when the count is not
    # read back / rows are not compacted
    plan_rows = m if args.compaction_mode == "sync" else n
    if fused:
        plan = {"engine": "mfma_direct", "tile": 256,
                **_lib.query_fused_plan(plan_rows, h, v, _lib.DTYPE_BF16, options.get_panel_bytes())}
    else:
        plan = _lib.query_plan(plan_rows, h, v, _lib.DTYPE_BF16, True, options.get_panel_bytes())
    traffic, traffic_note = measured_traffic(wl.name, dominant)

    result = {
        "metric": "fused linear-CE fwd+bwd tokens/s",
        "value": m / (ms_per_step / 1e3),
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {
            "workload": f"{wl.name}: N={n} rows, M={m} loss-bearing, H={h}, V={v}, "
                        f"softcap={wl.logit_softcap}, seed={args.seed}",
            "input_rows_per_s": n / (ms_per_step / 1e3),
            "compaction_mode": args.compaction_mode,
            "gradients": "forward" if fused else "recompute",
            "panel_bytes": options.get_panel_bytes() or ((5 << 29) if fused else (1 << 30)),
            "plan": plan,
            "sources": source_fingerprint(),
        },
        "loss": loss_value,
        "tflops_useful_6MHV": useful_tflops,
        "contractions_executed": executed_contractions,
        "tflops_executed": executed_tflops,
        "frac_of_bf16_peak_useful": useful_tflops / PEAK_BF16_TFLOPS,
        "mfma_util_executed": executed_tflops / PEAK_BF16_TFLOPS,
        "ms_per_step_median": ms_median,
        "forward_only_ms": round(forward_ms, 3),
        "backward_only_ms": round(backward_ms, 3),
        "kernel_ms": {k: round(x, 3) for k, x in prof.ms.items()},
        "kernel_launches": prof.launches,
        "roofline": {
            "kernel": dominant,
            "bound": "mfma",
            "achieved": achieved,
            "peak": PEAK_BF16_TFLOPS,
            "unit": "TFLOP/s",
            "frac": achieved / PEAK_BF16_TFLOPS,
            "traffic": traffic,
            "traffic_source": traffic_note,
            "avg_launch_ms": avg_ms,
            "launches_per_step": launches,
            "flops_per_launch": flops_per_launch,
        },
    }
    result["compaction_gather"] = compaction
    if not args.no_library_gemm:
        result["library_gemm"] = library_gemm_reference(torch, device, h, v)
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(wl, args.cpu_rows)
    print(json.dumps(result), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
