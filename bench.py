#!/usr/bin/env python3
"""Benchmark of the GRPO log-prob + loss forward/backward path on one MI355X.

One "step" = one pass of the hot path over one synthetic batch that is already resident in HBM.  For the headline
workload (benchmark configuration "GRPO loss fwd+bwd": bf16 logits [64, 1024, 151936], temperature 0.9) the step
is timed four ways -- two passes over the logits (K1 log-prob kernel, [B, T] loss kernel, K3 gradient kernel) and one
pass (K7, which writes a row's gradient from the registers that hold the row), each with and without the rows outside
the completion mask -- and the headline is the fastest that produces every stated output.  Prints ONE JSON line.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--loss-type dapo] [--no-cpu-baseline]

`value` is token positions per second over the K timed steps (events on torch's current stream, which is the stream
the kernels are enqueued on, bracketed by device synchronisation).  `roofline` is for the dominant kernel of the
headline step: algorithmic bytes per launch / average launch time, measured live with events around back-to-back
launches of that kernel alone; `step_hbm_GBps` prices the whole step by the bytes its kernels move.
`cpu_baseline` times the CPU oracle (a port of the reference path, oracle/) on a bounded row sample of the same
workload on this host's cores.  Without `--workload` the line also carries `secondary`: the other loss types of the
headline workload and the other benchmark configurations (fused head, long context, DPO, and the fp32 forward-only
configuration small enough for the host to run whole), each with its step time,
its dominant kernel's roofline figures and -- where the one-pass kernel runs -- the relative L2 distance between its
gradient and the two-pass gradient.  The fused-head record also times the SFT chunked cross-entropy on its operands,
the DPO record the KTO loss on its logits.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0  # MI355X HBM3E, published peak
# HBM bytes per launch of the dominant kernel from rocprofv3 FETCH_SIZE / WRITE_SIZE: two --pmc runs of
# `bench.py --workload W --only-leg LEG --calibrate-copy` per entry (every dispatch of the kernel in such a run is the
# same launch), each counter scaled by its reading for the 1 GiB device copy of the same run (FETCH x 2.000,
# WRITE x 1.000 KiB; summaries under profiles/).  The inputs are seeded, so the figures are stable; they are records of
# those runs, not measured by the run that prints them, and None where no counter run was made.
MEASURED_TRAFFIC_BYTES = {
    ("K3", "grpo_c3", "dapo"): (2 * 5056283 + 19450543) * 1024,       # --only-leg k3
    ("K7", "grpo_c3", "dapo"): (2 * 5055232 + 19469108) * 1024,       # --only-leg k7_masked
    ("K3", "grpo_c4", "dapo"): (2 * 10689829 + 38900940) * 1024,
    ("K7", "grpo_c4", "dapo"): (2 * 10686914 + 38943851) * 1024,
    ("K3", "dpo_c2", None): (2 * 6608991 + 32838146) * 1024,
    ("K1", "logp_c1", None): (2 * 128206 + 192) * 1024,
    # (the forward's operand re-reads vary from launch to launch with how closely the workgroups of an XCD stay in
    # step: 59.7-70.4 M KiB of fetches over four launches; the stash itself is 10.04 M KiB of writes)
    ("head_fwd", "head_c5", "dapo"): (2 * 31333262 + 10492504) * 1024,  # --only-leg head_fwd_stash
}
# the loss type changes per-row scalars only: the same rows are read and written, by the same launches
for _k in ("K3", "K7"):
    for _lt in ("grpo", "dr_grpo"):
        MEASURED_TRAFFIC_BYTES[(_k, "grpo_c3", _lt)] = MEASURED_TRAFFIC_BYTES[(_k, "grpo_c3", "dapo")]

WORKLOADS = {
    # name: (n_seq, completion_len, vocab, temperature, group_size, min_len)
    "grpo_c3": dict(B=64, T=1024, V=151936, temperature=0.9, G=8, min_len=64, beta=0.04, eps_low=0.2, eps_high=0.2,
                    rewards="normal", desc="GRPO fwd+bwd, bf16 logits [64,1024,151936], T=0.9, G=8, lens~U[64,1024]"),
    "grpo_c4": dict(B=32, T=4096, V=151936, temperature=1.0, G=16, min_len=512, beta=0.0, eps_low=0.2, eps_high=0.28,
                    rewards="bernoulli", desc="long-context GRPO fwd+bwd, bf16 logits [32,4096,151936], G=16"),
    "head_c5": dict(B=16, T=2048, V=151936, H=3584, temperature=1.0, G=8, min_len=64, beta=0.04, eps_low=0.2,
                    eps_high=0.2, rewards="normal", head=True,
                    desc="fused lm_head + log-prob + GRPO loss fwd+bwd, hidden bf16 [16x2048,3584], W bf16 [151936,3584]"),
    "dpo_c2": dict(B=64, T=2048, V=128256, beta=0.1, dpo=True,
                   desc="DPO sequence log-probs + sigmoid loss fwd+bwd, bf16 logits [64,2048,128256], 32 pairs, "
                        "prompt~U[64,512], completion~U[128,1536]"),
    "logp_c1": dict(B=8, T=256, V=32000, logp=True,
                    desc="selective_log_softmax + entropy_from_logits forward, fp32 logits [8,256,32000] = 3*randn (seed 0)"),
    "tiny": dict(B=8, T=64, V=151936, temperature=0.9, G=8, min_len=8, beta=0.04, eps_low=0.2, eps_high=0.2,
                 rewards="normal", desc="reduced-size functional check (not a benchmark configuration)"),
}


def make_inputs(w, device, seed=0):
    """Synthetic batch of the workload's shape, generated on the device one sequence at a time."""
    g = torch.Generator(device=device).manual_seed(seed)
    B, T, V = w["B"], w["T"], w["V"]
    logits = torch.empty((B, T, V), dtype=torch.bfloat16, device=device)
    for b in range(B):
        logits[b] = (2.0 * torch.randn((T, V), generator=g, device=device)).bfloat16()
    ids = torch.randint(0, V, (B, T), generator=g, device=device)
    lengths = torch.randint(w["min_len"], T + 1, (B,), generator=g, device=device)
    mask = (torch.arange(T, device=device)[None] < lengths[:, None]).long()
    if w["rewards"] == "normal":
        rewards = torch.randn((B,), generator=g, device=device)
    else:
        rewards = (torch.rand((B,), generator=g, device=device) < 0.3).float()
    return logits, ids, mask, rewards, g


def cpu_baseline(w, loss_type, rows_per_seq=512, n_seq=32, repeats=2):
    """The oracle (CPU port of the reference path: row-looped log_softmax / 128-row entropy chunks /
    autograd backward) on a [n_seq, rows_per_seq, V] bf16 sample of the workload."""
    import oracle

    torch.set_num_threads(os.cpu_count() or 1)
    g = torch.Generator().manual_seed(0)
    V, G = w["V"], min(w["G"], n_seq)
    logits = (2.0 * torch.randn(n_seq, rows_per_seq + 1, V, generator=g)).bfloat16()
    ids = torch.randint(0, V, (n_seq, rows_per_seq + 1), generator=g)
    lengths = torch.randint(max(1, rows_per_seq // 16), rows_per_seq + 1, (n_seq,), generator=g)
    mask = (torch.arange(rows_per_seq)[None] < lengths[:, None]).long()
    adv = oracle.group_advantages(torch.randn(n_seq, generator=g), G)
    with torch.no_grad():
        base, _ = oracle.logps_and_entropies_from_logits(logits, ids, rows_per_seq, w["temperature"], False)
    base = base.float()
    old = base + 0.05 * torch.randn(base.shape, generator=g)
    ref = base + 0.1 * torch.randn(base.shape, generator=g)
    best = float("inf")
    for _ in range(repeats):
        leaf = logits.clone().requires_grad_(True)
        t0 = time.perf_counter()
        lp, ent = oracle.logps_and_entropies_from_logits(leaf, ids, rows_per_seq, w["temperature"], True)
        loss, _ = oracle.grpo_loss(
            lp, adv, mask, entropies=ent, old_per_token_logps=old, ref_per_token_logps=ref if w["beta"] else None,
            loss_type=loss_type, epsilon_low=w["eps_low"], epsilon_high=w["eps_high"], beta=w["beta"],
            max_completion_length=rows_per_seq, num_items_in_batch=mask.sum().float())
        loss.backward()
        best = min(best, time.perf_counter() - t0)
    rows = n_seq * rows_per_seq
    return {
        "value": rows / best,
        "unit": "tokens/s",
        "cores": torch.get_num_threads(),
        "kind": "port",
        "sample": f"oracle fwd+bwd on bf16 logits [{n_seq},{rows_per_seq}+1,{V}] ({rows} of the workload's rows), "
                  f"best of {repeats}, {best:.2f} s; torch {torch.__version__} CPU",
    }


def cpu_baseline_head(w, rows=128, chunk=8192):
    """The oracle's chunked lm_head + log-prob operator (the reference's algorithm: vocabulary slabs, online
    log-sum-exp, recompute backward with fp32 products) forward + backward on `rows` tokens of the workload's
    hidden size and vocabulary."""
    import oracle

    torch.set_num_threads(os.cpu_count() or 1)
    g = torch.Generator().manual_seed(0)
    H, V = w["H"], w["V"]
    # a 2048-row random block repeated down the vocabulary: the timing does not depend on the values, and drawing
    # 5.4e8 normals on the host would take longer than the measurement
    block = (0.02 * torch.randn(2048, H, generator=g)).bfloat16()
    weight = block.repeat((V + 2047) // 2048, 1)[:V].contiguous().requires_grad_(True)

    def run(n):
        hid = torch.randn(n, H, generator=g).bfloat16().requires_grad_(True)
        targets = torch.randint(0, V, (n,), generator=g)
        gout = torch.randn(n, generator=g)
        weight.grad = None
        t0 = time.perf_counter()
        lp, _ = oracle.ChunkedLogProbOracle.apply(hid, weight, targets, w["temperature"], chunk)
        (lp * gout).sum().backward()
        return time.perf_counter() - t0

    dt = run(rows)
    if dt < 5.0:  # a fast host: grow the sample towards ~10 s of work
        rows = int(min(4096, rows * 10.0 / max(dt, 1e-3))) // 64 * 64
        dt = run(rows)
    return {"value": rows / dt, "unit": "tokens/s", "cores": torch.get_num_threads(), "kind": "port",
            "sample": f"oracle chunked head fwd+bwd on hidden bf16 [{rows},{H}], W bf16 [{V},{H}], chunk {chunk}, one run, "
                      f"{dt:.2f} s; torch {torch.__version__} CPU"}


def cpu_baseline_dpo(w, n_pairs=2, length=257):
    """The oracle's `DPOTrainer._compute_loss` restatement (sigmoid loss, all logged metrics) forward + backward on
    `2 * n_pairs` sequences of `length` tokens at the workload's vocabulary."""
    import oracle

    torch.set_num_threads(os.cpu_count() or 1)
    g = torch.Generator().manual_seed(0)
    V = w["V"]

    def run(pairs):
        B = 2 * pairs
        logits = (2.0 * torch.randn(B, length, V, generator=g)).bfloat16()
        ids = torch.randint(0, V, (B, length), generator=g)
        cm = torch.zeros(B, length, dtype=torch.long)
        cm[:, length // 8:] = 1
        ref = -8.0 * (length - length // 8) + torch.randn(B, generator=g)
        best = float("inf")
        for _ in range(2):
            leaf = logits.clone().requires_grad_(True)
            t0 = time.perf_counter()
            loss, _ = oracle.dpo_compute_loss(leaf, ids, cm, ref[:pairs], ref[pairs:], w["beta"])
            loss.backward()
            best = min(best, time.perf_counter() - t0)
        return best

    best = run(n_pairs)
    if best < 2.0:  # a fast host: grow the sample towards ~5 s per run
        n_pairs = int(min(16, max(n_pairs, n_pairs * 5.0 / max(best, 1e-3))))
        best = run(n_pairs)
    B = 2 * n_pairs
    rows = B * length
    return {"value": rows / best, "unit": "tokens/s", "cores": torch.get_num_threads(), "kind": "port",
            "sample": f"oracle DPO loss fwd+bwd on bf16 logits [{B},{length},{V}] ({rows} token rows), best of 2, "
                      f"{best:.2f} s; torch {torch.__version__} CPU"}


MFMA_BF16_PEAK_TFLOPS = 2500.0  # MI355X dense bf16, published peak


# Vocabulary rows per backward chunk of the fused head.  The operator's `chunk_size` only sizes the
# dz workspace (2 x N x chunk bf16); 32768 rows = 4.3 GB at this shape, a small share of the card's
# HBM, and leaves 5 chunks instead of 19 (fewer partial waves and dHidden accumulation passes).
HEAD_CHUNK = int(os.environ.get("TRL_AMD_BENCH_HEAD_CHUNK", "32768"))


def bench_head(args, w):
    """benchmark configuration 5: the logits are never materialised.  Step = fused head forward, GRPO loss,
    fused head backward (dHidden and dW)."""
    import trl_amd
    from trl_amd import ops

    dev = torch.device("cuda:0")
    B, T, V, H = w["B"], w["T"], w["V"], w["H"]
    N = B * T
    g = torch.Generator(device=dev).manual_seed(0)
    hidden = torch.randn((N, H), generator=g, device=dev).bfloat16().requires_grad_(True)
    weight = (0.02 * torch.randn((V, H), generator=g, device=dev)).bfloat16().requires_grad_(True)
    targets = torch.randint(0, V, (N,), generator=g, device=dev)
    lengths = torch.randint(w["min_len"], T + 1, (B,), generator=g, device=dev)
    mask = (torch.arange(T, device=dev)[None] < lengths[:, None]).long()
    adv = trl_amd.group_advantages(torch.randn((B,), generator=g, device=dev), w["G"])
    with torch.no_grad():
        base = ops.fused_head_fwd(hidden, weight, targets, w["temperature"], 0.0, 1.0)[0]
    base = base.view(B, T)
    old = base + 0.05 * torch.randn(base.shape, generator=g, device=dev)
    ref = base + 0.1 * torch.randn(base.shape, generator=g, device=dev)
    n_items = mask.sum().float()

    def step():
        hidden.grad = weight.grad = None
        lp, ent = trl_amd._ChunkedLogProbFunction.apply(hidden, weight, targets, w["temperature"], HEAD_CHUNK)
        loss, _ = trl_amd.grpo_loss(lp.view(B, T), adv, mask, entropies=ent.view(B, T), old_per_token_logps=old,
                                    ref_per_token_logps=ref, loss_type=args.loss_type, epsilon_low=w["eps_low"],
                                    epsilon_high=w["eps_high"], beta=w["beta"], max_completion_length=T,
                                    num_items_in_batch=n_items)
        loss.backward()
        return loss

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(args.steps):
        loss = step()
    e1.record()
    torch.cuda.synchronize()
    ms_per_step = max((time.perf_counter() - t0) * 1e3, e0.elapsed_time(e1)) / args.steps

    def time_op(fn, reps=3):
        fn()
        torch.cuda.synchronize()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        for _ in range(reps):
            fn()
        b.record()
        torch.cuda.synchronize()
        return a.elapsed_time(b) / reps

    # the same loss through the fused-linear operator (the call behind `use_liger_kernel`): it compacts the hidden
    # states to the rows of the completion mask before the head, so forward and backward both run on those rows only
    fl = trl_amd.FusedLinearGRPOLoss(beta=w["beta"], epsilon_low=w["eps_low"], epsilon_high=w["eps_high"],
                                     temperature=w["temperature"], use_ref_model=w["beta"] != 0.0,
                                     loss_type=args.loss_type, max_completion_length=T, chunk_size=HEAD_CHUNK)
    h3, t3 = hidden.view(B, T, H), targets.view(B, T)

    def fl_step():
        hidden.grad = weight.grad = None
        loss_fl, _ = fl(h3, weight, t3, mask, adv, None, old, ref if w["beta"] else None)
        loss_fl.backward()
        return loss_fl

    fl_ms = time_op(fl_step, reps=max(2, args.steps // 2))
    fl_loss = float(fl_step().detach())
    stash = ops.head_stash_fits(N, V)  # what the step above did: keep the forward's products, or recompute them
    flop = 2.0 * N * H * V
    with torch.no_grad():
        gl = torch.randn((N,), generator=g, device=dev)
        fwd_args = (hidden, weight, targets, w["temperature"], 0.0, 1.0)
        out = ops.fused_head_fwd(*fwd_args, None, stash)
        log_z, saved = out[2], (out[4] if stash else None)
        del out
        fwd_ms = time_op(lambda: ops.fused_head_fwd(*fwd_args, None, stash))
        bwd_ms = time_op(lambda: ops.fused_head_bwd(*fwd_args, log_z, gl, HEAD_CHUNK, None, saved))
        # the step's backward: the loss gives the tokens outside the completion mask an upstream gradient of exactly
        # zero, and those tokens are dropped before the two products (their dz rows are zero)
        g_step = gl * mask.reshape(-1).float()
        bwd_step_ms = time_op(lambda: ops.head_backward(*fwd_args, log_z, g_step, HEAD_CHUNK, None, saved))
        kernels = {}
        if stash:  # the reference's scheme (recompute the logits in the backward) on the same kernels, for comparison
            del saved
            fwd_plain = time_op(lambda: ops.fused_head_fwd(*fwd_args))
            bwd_rec = time_op(lambda: ops.fused_head_bwd(*fwd_args, log_z, gl, HEAD_CHUNK))
            kernels["fused_head_fwd_no_grad"] = {
                "avg_ms": fwd_plain, "TFLOPs": flop / (fwd_plain * 1e-3) / 1e12,
                "frac": flop / (fwd_plain * 1e-3) / 1e12 / MFMA_BF16_PEAK_TFLOPS,
                "note": "the forward when nothing asks for a gradient (log-probs of the old and of the reference "
                        "policy): same kernel, no products kept for a backward"}
            kernels["recompute_scheme"] = {
                "fwd_ms": fwd_plain, "bwd_ms": bwd_rec, "fwd_TFLOPs": flop / (fwd_plain * 1e-3) / 1e12,
                "bwd_TFLOPs": 3 * flop / (bwd_rec * 1e-3) / 1e12,
                "TFLOPs": 4 * flop / ((fwd_plain + bwd_rec) * 1e-3) / 1e12}
    # the SFT loss on the same operands: next-token cross-entropy of the completion tokens (prompt and padding
    # positions labelled -100 and dropped before the head), forward + backward, through the same kernels
    from trl_amd.trainer.sft_trainer import _chunked_cross_entropy_loss
    sft_labels = torch.where(mask.bool(), targets.view(B, T), torch.full_like(targets.view(B, T), -100))

    def sft_step():
        hidden.grad = weight.grad = None
        out = _chunked_cross_entropy_loss(hidden.view(B, T, H), weight, HEAD_CHUNK, shift_labels=sft_labels)
        out[0].backward()
        return out

    sft_ms = time_op(sft_step)
    sft_out = sft_step()
    n_sft = int(sft_out[3])
    hidden.grad = weight.grad = None
    kernels["sft_chunked_nll_step"] = {
        "ms_per_step": sft_ms, "tokens_with_label": n_sft, "tokens_per_s": N / (sft_ms * 1e-3),
        "loss": float(sft_out[0].detach()), "TFLOPs": 3 * 2.0 * n_sft * H * V / (sft_ms * 1e-3) / 1e12,
        "note": "SFTTrainer's chunked_nll loss (loss, correct-token count, entropy sum) forward + backward on the "
                "tokens that carry a label; three products of 2*n*H*V flop"}
    bwd_flop = (2 if stash else 3) * flop  # products actually executed by the backward
    fwd_tf, bwd_tf = flop / (fwd_ms * 1e-3) / 1e12, bwd_flop / (bwd_ms * 1e-3) / 1e12
    total_tf = (flop + bwd_flop) / ((fwd_ms + bwd_ms) * 1e-3) / 1e12
    result = {
        "metric": "tokens/sec + MFMA bf16 utilisation for fused lm_head+logprob+GRPO loss fwd+bwd",
        "value": N / (ms_per_step * 1e-3), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": args.workload, "description": w["desc"], "tokens": N, "hidden": H, "vocab": V,
                   "backward_chunk_rows": HEAD_CHUNK,
                   "backward_logits": "softmax numerators stashed by the forward (fp16, 2.07 bytes per logit)" if stash else "recomputed per chunk",
                   "tokens_with_gradient": int(mask.sum()),
                   "loss_type": args.loss_type, "loss": float(loss.detach())},
        # the dominant kernel: the forward sweep (2*N*H*V flop per launch; the event-timed interval also holds its
        # two sub-0.1 ms helper kernels)
        "roofline": {"bound": "mfma", "kernel": "fused_head_fwd_kernel", "achieved": fwd_tf,
                     "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s", "frac": fwd_tf / MFMA_BF16_PEAK_TFLOPS,
                     "traffic": MEASURED_TRAFFIC_BYTES.get(("head_fwd", args.workload, "dapo")) if stash else None,
                     "algorithmic_flop": flop, "avg_launch_ms": fwd_ms,
                     "forward_plus_backward": {"achieved": total_tf, "frac": total_tf / MFMA_BF16_PEAK_TFLOPS,
                                               "executed_flop": flop + bwd_flop, "ms": fwd_ms + bwd_ms}},
        "kernels": dict(kernels, **{
            "fused_head_fwd": {"avg_ms": fwd_ms, "TFLOPs": fwd_tf, "frac": fwd_tf / MFMA_BF16_PEAK_TFLOPS},
            "fused_head_bwd": {"avg_ms": bwd_ms, "TFLOPs": bwd_tf, "frac": bwd_tf / MFMA_BF16_PEAK_TFLOPS,
                               "products": 2 if stash else 3, "note": "every token with an upstream gradient"},
            "fused_head_bwd_step": {"avg_ms": bwd_step_ms, "tokens": int(mask.sum()),
                                    "note": "as in the step: tokens whose upstream gradient is zero are dropped"},
            "step_if_every_token_had_a_gradient_ms": ms_per_step - bwd_step_ms + bwd_ms}),
        "mask_aware": {"ms_per_step": fl_ms, "tokens_per_s": N / (fl_ms * 1e-3), "loss": fl_loss,
                       "note": "FusedLinearGRPOLoss: only the rows of the completion mask go through the head, forward "
                               "and backward; same loss"},
        "cpu_baseline": None if args.no_cpu_baseline else cpu_baseline_head(w),
    }
    if args.calibrate_copy:
        dst = torch.empty_like(weight)
        for _ in range(3):
            dst.copy_(weight.detach())  # reads and writes V*H*2 bytes each
        torch.cuda.synchronize()
        result["calibration_copy_bytes_each_way"] = V * H * 2
        del dst
    return result


def bench_dpo(args, w):
    """Config 2: `DPOTrainer._compute_loss` arithmetic (sigmoid loss, given reference log-probs) forward + backward
    to dlogits.  Headline = every shifted row computed; `mask_aware` = only the completion rows are read."""
    import trl_amd
    from trl_amd import ops

    dev = torch.device("cuda:0")
    B, L, V = w["B"], w["T"], w["V"]
    g = torch.Generator(device=dev).manual_seed(0)
    logits = torch.empty((B, L, V), dtype=torch.bfloat16, device=dev)
    for b in range(B):
        logits[b] = (2.0 * torch.randn((L, V), generator=g, device=dev)).bfloat16()
    ids = torch.randint(0, V, (B, L), generator=g, device=dev)
    prompt = torch.randint(64, 513, (B // 2,), generator=g, device=dev).repeat(2)
    comp = torch.randint(128, 1537, (B,), generator=g, device=dev)
    pos = torch.arange(L, device=dev)[None]
    cmask = ((pos >= prompt[:, None]) & (pos < (prompt + comp)[:, None])).long()
    with torch.no_grad():
        seq = trl_amd.dpo_sequence_logps(logits, ids, cmask)
    ref = seq + 0.5 * torch.randn((B,), generator=g, device=dev)
    leaf = logits.requires_grad_(True)
    R = B * (L - 1)

    def step(skip):
        leaf.grad = None
        loss, _ = trl_amd.dpo_compute_loss(leaf, ids, cmask, ref[: B // 2], ref[B // 2:], beta=w["beta"],
                                           skip_masked_rows=skip)
        loss.backward()
        return loss

    def timed(skip):
        for _ in range(args.warmup):
            step(skip)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(args.steps):
            loss = step(skip)
        e1.record()
        torch.cuda.synchronize()
        return max((time.perf_counter() - t0) * 1e3, e0.elapsed_time(e1)) / args.steps, float(loss.detach())

    ms_dense, loss_dense = timed(False)
    ms_aware, loss_aware = timed(True)
    assert abs(loss_dense - loss_aware) <= 1e-6 * max(1.0, abs(loss_dense)), "mask-aware loss differs"
    idx = ids[:, 1:].reshape(R, 1).contiguous()
    active = int(cmask[:, 1:].sum())
    with torch.no_grad():
        _, _, lse, _ = ops.logp_entropy_stats_fwd(logits.detach(), idx, 1.0, 0, L - 1, None)
        g_logp = (cmask[:, 1:].reshape(R, 1) * 0.01).float().contiguous()

        def time_kernel(fn, reps=5):
            fn()
            torch.cuda.synchronize()
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            for _ in range(reps):
                out = fn()
                del out
            b.record()
            torch.cuda.synchronize()
            return a.elapsed_time(b) / reps

        # (as the step above runs it: without the sum of squared probabilities, which only the WPO weights read)
        fwd_ms = time_kernel(lambda: ops.logp_entropy_stats_fwd(logits.detach(), idx, 1.0, 0, L - 1, None, False))
        fwd_p2_ms = time_kernel(lambda: ops.logp_entropy_stats_fwd(logits.detach(), idx, 1.0, 0, L - 1, None, True))
        bwd_ms = time_kernel(lambda: ops.logp_entropy_bwd(logits.detach(), idx, 1.0, 0, L - 1, lse, None, g_logp, None))
    # the KTO loss on the same logits (first half of the batch desirable, second half undesirable; no KL batch):
    # one pass with row statistics, [B]-sized arithmetic, the gradient kernel
    kto_label = torch.arange(B, device=dev) < B // 2

    def kto_step():
        leaf.grad = None
        loss, _ = trl_amd.kto_compute_loss(leaf, ids, cmask, kto_label, ref, beta=w["beta"], skip_masked_rows=False)
        loss.backward()
        return loss

    kto_ms = time_kernel(kto_step, reps=3)
    leaf.grad = None
    row_bytes = V * 2
    fwd_bytes = R * row_bytes
    bwd_bytes = active * 2 * row_bytes + (B * L - active) * row_bytes  # masked rows and the last position: zero fill
    result = {
        "metric": "tokens/sec + achieved HBM TB/s (% of peak) for DPO sequence logps + sigmoid loss fwd+bwd",
        "value": R / (ms_dense * 1e-3), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_dense, "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": args.workload, "description": w["desc"], "rows": R, "vocab": V, "active_rows": active,
                   "loss": loss_dense},
        "roofline": {"bound": "hbm", "kernel": "logp_entropy_bwd_kernel (K3)", "achieved": bwd_bytes / (bwd_ms * 1e-3) / 1e9,
                     "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": bwd_bytes / (bwd_ms * 1e-3) / 1e9 / HBM_PEAK_GBPS,
                     "traffic": MEASURED_TRAFFIC_BYTES.get(("K3", args.workload, None)), "algorithmic_bytes": bwd_bytes,
                     "avg_launch_ms": bwd_ms},
        "kernels": {"logp_entropy_fwd_kernel with row statistics (K1)": {
            "avg_launch_ms": fwd_ms, "algorithmic_bytes": fwd_bytes, "achieved_GBps": fwd_bytes / (fwd_ms * 1e-3) / 1e9,
            "frac": fwd_bytes / (fwd_ms * 1e-3) / 1e9 / HBM_PEAK_GBPS,
            "with_sum_of_squared_probabilities_ms": fwd_p2_ms}},
        "kto": {"ms_per_step": kto_ms, "tokens_per_s": R / (kto_ms * 1e-3),
                "note": "KTOTrainer's loss (kto, no KL batch) forward + backward on the same logits: the same two kernels"},
        "mask_aware": {"ms_per_step": ms_aware, "tokens_per_s": R / (ms_aware * 1e-3),
                       "note": "only rows inside the completion mask are read; loss, metrics and dlogits identical"},
        "cpu_baseline": None if args.no_cpu_baseline else cpu_baseline_dpo(w),
    }
    return result


def bench_logp_c1(args, w):
    """Config 1, the reference's CPU-runnable case: per-token log-probs and entropies of fp32 logits, forward only.
    The inputs come from a CPU generator, so the oracle on the host sees the same bits and the whole output is
    compared with it (1e-5, against its fp64 evaluation) before anything is timed.  The 262 MB of logits would stay in the memory-side cache
    between launches: the timed launches rotate over eight copies."""
    import oracle
    import trl_amd
    from trl_amd import ops

    dev = torch.device("cuda:0")
    B, T, V = w["B"], w["T"], w["V"]
    R = B * T
    g = torch.Generator().manual_seed(0)
    host_logits = 3.0 * torch.randn((B, T, V), generator=g)
    host_ids = torch.randint(0, V, (B, T), generator=g)
    torch.set_num_threads(os.cpu_count() or 1)
    best = float("inf")
    for _ in range(3):
        t0 = time.perf_counter()
        want_lp = oracle.selective_log_softmax(host_logits, host_ids)
        want_h = oracle.entropy_from_logits(host_logits)
        best = min(best, time.perf_counter() - t0)
    # parity against the same functions in fp64 (the fp32 host result carries ~2e-5 of summation error itself)
    want_lp = oracle.selective_log_softmax(host_logits.double(), host_ids)
    want_h = oracle.entropy_from_logits(host_logits.double())
    copies = [host_logits.to(dev) for _ in range(8)]
    ids = host_ids.to(dev)
    lp, ent = trl_amd.logps_and_entropies(copies[0], ids)
    err_lp = float((lp.cpu().double() - want_lp).abs().max())
    err_h = float((ent.cpu().double() - want_h).abs().max())
    assert err_lp <= 1e-5 and err_h <= 1e-5, (err_lp, err_h)
    idx = ids.reshape(R, 1)

    def timed(fn, reps):
        for c in copies:
            fn(c)
        torch.cuda.synchronize()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        t0 = time.perf_counter()
        a.record()
        for i in range(reps):
            fn(copies[i % len(copies)])
        b.record()
        torch.cuda.synchronize()
        return max((time.perf_counter() - t0) * 1e3, a.elapsed_time(b)) / reps, a.elapsed_time(b) / reps

    reps = max(args.steps, 10) * 8
    ms_step, _ = timed(lambda x: trl_amd.logps_and_entropies(x, ids), reps)
    ms_two, _ = timed(lambda x: (trl_amd.selective_log_softmax(x, ids), trl_amd.entropy_from_logits(x)), reps)
    _, ms_kernel = timed(lambda x: ops.logp_entropy_fwd(x, idx, 1.0, 0, T, None), reps)
    nbytes = R * V * 4
    gbps = nbytes / (ms_kernel * 1e-3) / 1e9
    return {
        "metric": "tokens/sec + achieved HBM TB/s (% of peak) for log-prob + entropy forward",
        "value": R / (ms_step * 1e-3), "unit": "tokens/s", "n_gpus": 1, "steps": reps, "warmup": len(copies),
        "ms_per_step": ms_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": args.workload, "description": w["desc"], "rows": R, "vocab": V,
                   "max_abs_err_logps_vs_oracle": err_lp, "max_abs_err_entropy_vs_oracle": err_h},
        "roofline": {"bound": "hbm", "kernel": "logp_entropy_fwd_kernel (K1)", "achieved": gbps, "peak": HBM_PEAK_GBPS,
                     "unit": "GB/s", "frac": gbps / HBM_PEAK_GBPS,
                     "traffic": MEASURED_TRAFFIC_BYTES.get(("K1", args.workload, None)), "algorithmic_bytes": nbytes,
                     "avg_launch_ms": ms_kernel,
                     "note": "back-to-back launches over eight copies of the logits (each launch reads cold data)"},
        "two_calls_ms_per_step": ms_two,
        "cpu_baseline": {"value": R / best, "unit": "tokens/s", "cores": torch.get_num_threads(), "kind": "port",
                         "sample": f"oracle selective_log_softmax + entropy_from_logits on the full configuration, "
                                   f"best of 3, {best:.3f} s; torch {torch.__version__} CPU"},
    }


def _trainer_step_legs(args, w, loss_type, shared, timed):
    """`GRPOLossMixin._compute_loss` as a `transformers.Trainer` runs it with 4 gradient-accumulation steps: the parent
    class divides the returned loss by 4 before `backward` (a trainer with `model_accepts_loss_kwargs = False` and no
    `compute_loss_func`).  Three ways: the mix-in as it is (it announces the divisor to the single pass), the same
    with the announcement switched off (`backward` then rescales the whole gradient), and the two-pass path.  The
    model is a stand-in that returns the resident logits; one prompt token, T - 1 completion tokens."""
    from collections import defaultdict
    from types import SimpleNamespace

    import trl_amd

    logits, ids, mask, adv, old, ref, leaf = (shared[k] for k in ("logits", "ids", "mask", "adv", "old", "ref", "leaf"))
    B, T = ids.shape
    K = T - 1

    class Accelerator:
        num_processes, sync_gradients, scaler, gradient_accumulation_steps = 1, True, None, 1
        gather = gather_for_metrics = staticmethod(lambda x: x)
        reduce = staticmethod(lambda x, reduction="sum": x)

    class Trainer(trl_amd.GRPOLossMixin):
        pass

    inputs = dict(prompt_ids=ids[:, :1], prompt_mask=torch.ones_like(ids[:, :1]), completion_ids=ids[:, 1:],
                  completion_mask=mask[:, 1:], advantages=adv, old_per_token_logps=old[:, 1:],
                  num_items_in_batch=mask[:, 1:].sum().float())
    if ref is not None:
        inputs["ref_per_token_logps"] = ref[:, 1:]
    out = {}
    for name, single, announce in (("single_pass", True, True), ("single_pass_divisor_not_announced", True, False),
                                   ("two_pass", False, True)):
        tr = Trainer()
        tr.accelerator, tr.temperature, tr.model_kwarg_keys = Accelerator(), w["temperature"], set()
        tr._entropy_bonus_enabled, tr.entropy_coef, tr.use_adaptive_entropy, tr.aux_loss_enabled = False, 0.0, False, False
        tr.top_entropy_quantile, tr.off_policy_mask_threshold, tr.importance_sampling_level = 1.0, None, "token"
        tr.beta, tr.loss_type, tr.epsilon_low, tr.epsilon_high = w["beta"], loss_type, w["eps_low"], w["eps_high"]
        tr.use_vllm = tr.vllm_importance_sampling_correction = False
        tr.max_completion_length, tr.current_gradient_accumulation_steps = K, 4
        tr.args = SimpleNamespace(delta=None, use_bias_correction_kl=False)
        tr._metrics = {"train": defaultdict(list), "eval": defaultdict(list)}
        tr.model = SimpleNamespace(training=True)
        tr.model_accepts_loss_kwargs, tr.compute_loss_func = False, None
        tr.trl_amd_single_pass, tr.trl_amd_trainer_divides_loss = single, announce

        def training_step(tr=tr):
            leaf.grad = None
            loss = tr._compute_loss(lambda **kw: SimpleNamespace(logits=leaf, aux_loss=None), inputs)
            loss = loss / tr.current_gradient_accumulation_steps  # transformers Trainer.training_step
            loss.backward()
            return loss, None

        out[name] = timed(training_step)[0]
    leaf.grad = None
    return out


def _parity_sample(w, loss_type, shared, run_step, n_rows=24):
    """The headline step's outputs against the CPU oracle on a sample of rows, inside the run that times it: the
    log-prob and entropy of `n_rows` token rows from the stored bf16 logits (fp32 arithmetic on the host), the loss from
    the oracle's loss on the step's log-probs, and those rows of the gradient from the oracle's d loss / d log-prob
    through the host's log-softmax.  Bars as in the tests: 2e-3 absolute (bf16 logits), loss 1e-3 relative, gradient rows
    5e-3 relative L2 (the device rounds them to bf16)."""
    import oracle

    logits, ids, mask, adv, old, ref, n_items, leaf = (shared[k] for k in ("logits", "ids", "mask", "adv", "old", "ref",
                                                                        "n_items", "leaf"))
    B, T = ids.shape
    loss, lp, ent = run_step()
    grad = leaf.grad
    pick = torch.Generator().manual_seed(1)
    active = torch.nonzero(mask.cpu().reshape(-1)).reshape(-1)
    rows = active[torch.randperm(active.numel(), generator=pick)[:n_rows]]
    rows = torch.cat([rows, torch.tensor([0, int(active[-1])])]).unique()
    b_idx, t_idx = (rows // T).to(logits.device), (rows % T).to(logits.device)
    x = logits.detach()[b_idx, t_idx].cpu().float().requires_grad_(True)
    tok = ids.cpu().reshape(-1)[rows]
    temp = w["temperature"]
    want_lp = oracle.selective_log_softmax_f32(x.detach(), tok, temp)
    want_ent = oracle.entropy_from_logits_f32(x.detach(), temp)
    err_lp = float((lp.detach().cpu().reshape(-1)[rows] - want_lp).abs().max())
    err_ent = float((ent.detach().cpu().reshape(-1)[rows] - want_ent).abs().max())
    lp_host = lp.detach().cpu().clone().requires_grad_(True)
    oloss, _ = oracle.grpo_loss(
        lp_host, adv.cpu(), mask.cpu(), entropies=ent.detach().cpu(), old_per_token_logps=old.cpu(),
        ref_per_token_logps=None if ref is None else ref.cpu(), loss_type=loss_type, epsilon_low=w["eps_low"],
        epsilon_high=w["eps_high"], beta=w["beta"], max_completion_length=T, num_items_in_batch=n_items.cpu())
    oloss.backward()
    g_tok = lp_host.grad.reshape(-1)[rows]
    z = x / temp
    (torch.log_softmax(z, -1).gather(-1, tok[:, None]).squeeze(-1) * g_tok).sum().backward()
    got = grad[b_idx, t_idx].cpu().float()
    rel = float((got - x.grad).norm() / x.grad.norm().clamp(min=1e-30))
    loss_rel = abs(float(loss.detach()) - float(oloss.detach())) / max(1e-12, abs(float(oloss.detach())))
    leaf.grad = None
    assert err_lp <= 2e-3 and err_ent <= 2e-3 and loss_rel <= 1e-3 and rel <= 5e-3, (err_lp, err_ent, loss_rel, rel)
    return {"rows": int(rows.numel()), "max_abs_err_logp": err_lp, "max_abs_err_entropy": err_ent,
            "loss_rel_err": loss_rel, "dlogits_rel_l2": rel,
            "note": "the step's outputs on a sample of token rows against the CPU oracle (fp32 arithmetic on the stored "
                    "bf16 logits; gradient rows through the oracle's loss gradient and the host's log-softmax)"}


def _grad_distance(run_a, run_b, leaf):
    """Relative L2 distance between the gradients two step functions leave in `leaf.grad`, accumulated sequence
    by sequence (no logits-sized fp32 temporaries)."""
    run_a()
    ga = leaf.grad
    leaf.grad = None
    run_b()
    gb = leaf.grad
    num = den = 0.0
    for b in range(ga.shape[0]):
        x, y = ga[b].float(), gb[b].float()
        num += float((x - y).square().sum())
        den += float(y.square().sum())
    leaf.grad = None
    del ga, gb
    return (num / max(den, 1e-300)) ** 0.5


def bench_grpo(args, w, loss_type, shared=None, full=True):
    """One GRPO workload and loss type.  `shared` carries the inputs of an earlier call on the same workload;
    `full` adds the two-pass kernel timings, the mask-aware two-pass leg and the scaled-upstream-gradient leg."""
    import trl_amd
    from trl_amd import ops

    dev = torch.device("cuda:0")
    B, T, V = w["B"], w["T"], w["V"]
    R = B * T
    if shared is None:
        logits, ids, mask, rewards, g = make_inputs(w, dev)
        adv = trl_amd.group_advantages(rewards, w["G"])
        with torch.no_grad():
            base, _ = trl_amd.logps_and_entropies(logits, ids, w["temperature"])
        old = base + 0.05 * torch.randn(base.shape, generator=g, device=dev)
        ref = base + 0.1 * torch.randn(base.shape, generator=g, device=dev) if w["beta"] else None
        shared = dict(logits=logits, ids=ids, mask=mask, adv=adv, old=old, ref=ref, n_items=mask.sum().float(),
                      leaf=logits.requires_grad_(True))
    logits, ids, mask, adv, old, ref, n_items, leaf = (shared[k] for k in ("logits", "ids", "mask", "adv", "old", "ref",
                                                                        "n_items", "leaf"))

    def step(row_mask=None):
        leaf.grad = None
        lp, ent = trl_amd.logps_and_entropies(leaf, ids, w["temperature"], row_mask=row_mask)
        loss, metrics = trl_amd.grpo_loss(
            lp, adv, mask, entropies=ent.detach(), old_per_token_logps=old, ref_per_token_logps=ref,
            loss_type=loss_type, epsilon_low=w["eps_low"], epsilon_high=w["eps_high"], beta=w["beta"],
            max_completion_length=T, num_items_in_batch=n_items)
        loss.backward()
        return loss, metrics

    def timed(fn):
        for _ in range(args.warmup):
            fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(args.steps):
            loss, _ = fn()
        e1.record()
        torch.cuda.synchronize()
        wall_ms = (time.perf_counter() - t0) * 1e3
        return max(wall_ms, e0.elapsed_time(e1)) / args.steps, float(loss.detach())

    # two passes over the logits (log-prob kernel, [B, T] loss kernel, gradient kernel); every row's log-prob and
    # entropy is produced (the configuration's stated outputs)
    ms_two_pass, loss_value = timed(lambda: step(None))
    assert loss_value == loss_value, "loss is NaN"
    ms_mask_aware = None
    if full:  # the forward also skips the rows the completion mask zeroes (what `_compute_loss` does by default)
        ms_mask_aware, loss_mask_aware = timed(lambda: step(mask))
        assert abs(loss_mask_aware - loss_value) <= 1e-6 * max(1.0, abs(loss_value)), "mask-aware loss differs"

    # one pass over the logits: the kernel that computes a row's log-prob also writes that row's gradient
    single = None
    if trl_amd.grpo_single_pass_supported(leaf, loss_type):
        def sp_step(skip, factor=None, tell=False):
            leaf.grad = None
            loss, metrics, _, _ = trl_amd.grpo_loss_from_logits(
                leaf, ids, adv, mask, temperature=w["temperature"], old_per_token_logps=old, ref_per_token_logps=ref,
                loss_type=loss_type, epsilon_low=w["eps_low"], epsilon_high=w["eps_high"], beta=w["beta"],
                max_completion_length=T, num_items_in_batch=n_items, keep_start=0, skip_masked_rows=skip,
                upstream_scale=factor if tell else None)
            (loss if factor is None else loss * factor).backward()
            return loss, metrics

        ms_sp_all, loss_sp = timed(lambda: sp_step(False))
        assert abs(loss_sp - loss_value) <= 1e-6 * max(1.0, abs(loss_value)), "single-pass loss differs"
        ms_sp_skip, loss_sp2 = timed(lambda: sp_step(True))
        assert abs(loss_sp2 - loss_value) <= 1e-6 * max(1.0, abs(loss_value)), "single-pass (mask-aware) loss differs"
        single = {"all_rows_ms": ms_sp_all, "mask_aware_ms": ms_sp_skip,
                  # the gradient of the one pass against the gradient of the two passes (both rounded to bf16 once)
                  "dlogits_rel_l2_vs_two_pass": _grad_distance(lambda: sp_step(False), lambda: step(None), leaf)}
        if full and not args.no_cpu_baseline:
            def sp_outputs():
                leaf.grad = None
                out = trl_amd.grpo_loss_from_logits(
                    leaf, ids, adv, mask, temperature=w["temperature"], old_per_token_logps=old, ref_per_token_logps=ref,
                    loss_type=loss_type, epsilon_low=w["eps_low"], epsilon_high=w["eps_high"], beta=w["beta"],
                    max_completion_length=T, num_items_in_batch=n_items, keep_start=0, skip_masked_rows=False)
                out[0].backward()
                return out[0], out[2], out[3]

            single["parity_vs_oracle"] = _parity_sample(w, loss_type, shared, sp_outputs)
        if full:
            # an upstream gradient other than 1 (a gradient scaler): announced to the forward it costs nothing,
            # unannounced it costs a further read + write of the gradient in `backward`
            single["scaled_upstream_ms"] = {"announced": timed(lambda: sp_step(True, 1024.0, True))[0],
                                            "unannounced": timed(lambda: sp_step(True, 1024.0, False))[0]}
            single["trainer_step_grad_accum_4_ms"] = _trainer_step_legs(args, w, loss_type, shared, timed)
    # headline: the fastest path that produces every stated output (log-prob and entropy of every row, loss, dlogits)
    ms_per_step = min(ms_two_pass, single["all_rows_ms"]) if single else ms_two_pass
    headline_single = single is not None and single["all_rows_ms"] <= ms_two_pass
    tokens_per_s = R / (ms_per_step * 1e-3)

    # ---- per-kernel timing: each kernel alone, events around `reps` back-to-back launches -----------
    idx = ids.reshape(R, 1)
    with torch.no_grad():
        lp_flat, ent_flat, lse = ops.logp_entropy_fwd(logits.detach(), idx, w["temperature"], 0, T, None)
    loss2, _, dlogp, _ = ops.grpo_loss_op(
        lp_flat.view(B, T), old, ref, ent_flat.view(B, T), adv, mask, None, None, n_items,
        ops.LOSS_TYPES[loss_type][0], w["eps_low"], w["eps_high"], float("nan"), w["beta"], False, 1.0,
        float(B * T), 1.0, 0.0, ops.LOSS_TYPES[loss_type][1])
    g_logp = dlogp.reshape(R, 1).contiguous()
    leaf.grad = None
    reps = max(3, min(args.steps, 10))

    def time_kernel(fn):
        fn()
        torch.cuda.synchronize()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        for _ in range(reps):
            out = fn()
            del out
        b.record()
        torch.cuda.synchronize()
        return a.elapsed_time(b) / reps

    row_bytes = V * 2
    active_rows = int((g_logp != 0).sum())
    fwd_bytes = R * row_bytes
    bwd_bytes = active_rows * 2 * row_bytes + (R - active_rows) * row_bytes  # masked rows: zero-fill write only
    kernels = {}
    roofline = None
    fwd_ms = bwd_ms = None
    if full or not headline_single:
        with torch.no_grad():
            fwd_ms = time_kernel(lambda: ops.logp_entropy_fwd(logits.detach(), idx, w["temperature"], 0, T, None))
            bwd_ms = time_kernel(lambda: ops.logp_entropy_bwd(logits.detach(), idx, w["temperature"], 0, T, lse, None,
                                                              g_logp, None))
        fwd_gbps = fwd_bytes / (fwd_ms * 1e-3) / 1e9
        bwd_gbps = bwd_bytes / (bwd_ms * 1e-3) / 1e9
        roofline = {
            "bound": "hbm", "kernel": "logp_entropy_bwd_kernel (K3)", "achieved": bwd_gbps, "peak": HBM_PEAK_GBPS,
            "unit": "GB/s", "frac": bwd_gbps / HBM_PEAK_GBPS,
            "traffic": MEASURED_TRAFFIC_BYTES.get(("K3", args.workload, loss_type)), "algorithmic_bytes": bwd_bytes,
            "avg_launch_ms": bwd_ms,
        }
        kernels.update({
            "logp_entropy_fwd_kernel (K1)": {"avg_launch_ms": fwd_ms, "algorithmic_bytes": fwd_bytes,
                                             "achieved_GBps": fwd_gbps, "frac": fwd_gbps / HBM_PEAK_GBPS},
            "logp_entropy_bwd_kernel (K3)": {"avg_launch_ms": bwd_ms, "algorithmic_bytes": bwd_bytes,
                                             "achieved_GBps": bwd_gbps, "frac": bwd_gbps / HBM_PEAK_GBPS},
            "two_pass_step_hbm_GBps": (fwd_bytes + bwd_bytes) / (ms_two_pass * 1e-3) / 1e9,
        })
    step_bytes = fwd_bytes + bwd_bytes  # what the two-pass step moves
    if single:
        reduce_code, term_code = ops.LOSS_TYPES[loss_type]
        if reduce_code == 0:  # per-sequence mean
            row_scale = 1.0 / B / mask.float().sum(1).clamp(min=1.0)
        elif loss_type == "dr_grpo":
            row_scale = torch.full((B,), 1.0 / (B * T), device=dev)
        else:
            row_scale = (1.0 / n_items.clamp(min=1.0)).expand(B)

        def fused(all_rows):
            return ops.grpo_fused_fwd_bwd(logits.detach(), ids, w["temperature"], 0, T, mask, adv, row_scale, old, ref, None,
                                          None, term_code, w["eps_low"], w["eps_high"], float("nan"), w["beta"], False,
                                          1.0, 1.05, all_rows)

        def fused_dense():  # every row inside the mask: each is read and its gradient written
            return ops.grpo_fused_fwd_bwd(logits.detach(), ids, w["temperature"], 0, T, torch.ones_like(mask), adv,
                                          row_scale, old, ref, None, None, term_code, w["eps_low"], w["eps_high"],
                                          float("nan"), w["beta"], False, 1.0, 1.05, False)

        with torch.no_grad():
            sp_skip_ms = time_kernel(lambda: fused(False))
            sp_all_ms = time_kernel(lambda: fused(True)) if full else None
            sp_dense_ms = time_kernel(fused_dense) if full else None
        sp_all_bytes = 2 * R * row_bytes                              # every row read, every gradient row written
        sp_skip_bytes = active_rows * 2 * row_bytes + (R - active_rows) * row_bytes
        for name, ms_k, nbytes in (("grpo_fused_kernel (K7), masked rows not read", sp_skip_ms, sp_skip_bytes),
                                   ("grpo_fused_kernel (K7), every row read (C entry only)", sp_all_ms, sp_all_bytes),
                                   ("grpo_fused_kernel (K7), every row active (a mask of ones)", sp_dense_ms, sp_all_bytes)):
            if ms_k is not None:
                kernels[name] = {"avg_launch_ms": ms_k, "algorithmic_bytes": nbytes,
                                 "achieved_GBps": nbytes / (ms_k * 1e-3) / 1e9,
                                 "frac": nbytes / (ms_k * 1e-3) / 1e9 / HBM_PEAK_GBPS}
        if headline_single:
            # the headline step = this kernel on the rows with gradient (the others zero-filled) + the forward kernel
            # on the rows without gradient, for their log-probs and entropies
            gbps = sp_skip_bytes / (sp_skip_ms * 1e-3) / 1e9
            step_bytes = sp_skip_bytes + (R - active_rows) * row_bytes
            roofline = {"bound": "hbm", "kernel": "grpo_fused_kernel (K7)", "achieved": gbps, "peak": HBM_PEAK_GBPS,
                        "unit": "GB/s", "frac": gbps / HBM_PEAK_GBPS,
                        "traffic": MEASURED_TRAFFIC_BYTES.get(("K7", args.workload, loss_type)),
                        "algorithmic_bytes": sp_skip_bytes, "avg_launch_ms": sp_skip_ms}
    # the whole step priced by the bytes its own kernels move (K7's bytes + the forward read of the other rows, or
    # K1's + K3's): bytes / step time
    roofline["step_hbm_bytes"] = step_bytes
    roofline["step_hbm_GBps"] = step_bytes / (ms_per_step * 1e-3) / 1e9
    roofline["step_hbm_frac"] = roofline["step_hbm_GBps"] / HBM_PEAK_GBPS

    result = {
        "metric": "tokens/sec + achieved HBM TB/s (% of peak) for GRPO logprob+loss fwd+bwd",
        "value": tokens_per_s,
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
        "config": {"workload": args.workload, "description": w["desc"], "rows": R, "vocab": V,
                   "loss_type": loss_type, "active_rows": active_rows, "loss": loss_value,
                   "path": "single pass over the logits (K7) for the rows with gradient + forward kernel (K1) for the "
                           "log-probs and entropies of the others" if headline_single
                           else "two passes over the logits (K1, K3)"},
        "roofline": roofline,
        "kernels": kernels,
        "two_pass": {"ms_per_step": ms_two_pass, "tokens_per_s": R / (ms_two_pass * 1e-3),
                     "note": "log-prob kernel (K1), [B, T] loss kernel, gradient kernel (K3): two reads and one write "
                             "of the logits-sized data; the path of every configuration the single pass does not take"},
        "single_pass": None if single is None else {
            "ms_per_step": single["all_rows_ms"], "tokens_per_s": R / (single["all_rows_ms"] * 1e-3),
            "mask_aware_ms_per_step": single["mask_aware_ms"],
            "mask_aware_tokens_per_s": R / (single["mask_aware_ms"] * 1e-3),
            "dlogits_rel_l2_vs_two_pass": single["dlogits_rel_l2_vs_two_pass"],
            "parity_vs_oracle": single.get("parity_vs_oracle"),
            "scaled_upstream_ms": single.get("scaled_upstream_ms"),
            "trainer_step_grad_accum_4_ms": single.get("trainer_step_grad_accum_4_ms"),
            "note": "grpo_loss_from_logits: the rows with gradient are read once and their gradient written by the same "
                    "kernel; same loss, log-probs, entropies and dlogits; the log-probs and entropies of the other rows "
                    "come from the forward kernel; mask-aware = those rows are not read at all (what `_compute_loss` "
                    "does by default); scaled_upstream_ms = mask-aware step with loss * 1024 before backward; "
                    "trainer_step_grad_accum_4_ms = `GRPOLossMixin._compute_loss` on a trainer whose parent class divides "
                    "the loss by 4 accumulation steps before backward, host-side metrics copy included"},
    }
    if ms_mask_aware is not None:
        result["mask_aware"] = {"ms_per_step": ms_mask_aware, "tokens_per_s": R / (ms_mask_aware * 1e-3),
                                "note": "forward also skips rows with completion_mask == 0 (their outputs are 0); "
                                        "loss, metrics and dlogits identical"}
    if args.calibrate_copy and full:
        dst = torch.empty_like(logits)
        for _ in range(3):
            dst.copy_(logits.detach())  # reads and writes R*V*2 bytes each
        torch.cuda.synchronize()
        result["calibration_copy_bytes_each_way"] = fwd_bytes
        del dst
    return result, shared


def _brief(r):
    """What a secondary entry keeps of a full result."""
    out = {"workload": r["config"]["workload"], "loss_type": r["config"].get("loss_type"), "value": r["value"],
           "unit": r["unit"], "ms_per_step": r["ms_per_step"], "path": r["config"].get("path"),
           "roofline": r["roofline"]}
    if r.get("single_pass"):
        out["single_pass_ms_per_step"] = r["single_pass"]["ms_per_step"]
        out["single_pass_mask_aware_ms_per_step"] = r["single_pass"]["mask_aware_ms_per_step"]
        out["dlogits_rel_l2_vs_two_pass"] = r["single_pass"]["dlogits_rel_l2_vs_two_pass"]
    if r.get("two_pass"):
        out["two_pass_ms_per_step"] = r["two_pass"]["ms_per_step"]
    if r.get("mask_aware"):
        out["mask_aware_ms_per_step"] = r["mask_aware"]["ms_per_step"]
    if "kernels" in r:
        out["kernels"] = {k: v for k, v in r["kernels"].items() if isinstance(v, dict) and ("frac" in v or "avg_ms" in v)}
        if "sft_chunked_nll_step" in r["kernels"]:  # the SFT loss on the head workload's operands
            out["sft_chunked_nll_step"] = r["kernels"]["sft_chunked_nll_step"]
    if r.get("kto"):  # the KTO loss on the DPO workload's logits
        out["kto"] = r["kto"]
    if r["config"]["workload"] == "logp_c1":  # small enough for the host to run whole: its own baseline and parity
        out["cpu_baseline"] = r["cpu_baseline"]
        out["two_calls_ms_per_step"] = r["two_calls_ms_per_step"]
        out["max_abs_err_vs_oracle"] = max(r["config"]["max_abs_err_logps_vs_oracle"],
                                           r["config"]["max_abs_err_entropy_vs_oracle"])
    return out


LEGS = ("k1", "k1_stats", "k3", "k7_masked", "k7_all_rows", "k7_dense_mask", "head_fwd_stash", "head_fwd_plain",
        "head_bwd_every_token", "head_bwd_step")


def bench_one_leg(args, w):
    """One kernel of one workload in one mode, `--steps` launches back to back between two events.  Under a profiler
    every launch of the kernel in the trace then moves the same bytes (or does the same flop), so the trace's average
    duration belongs to one figure:
      k1 / k1_stats          log-prob forward kernel (with row statistics: the DPO workload's form), every row
      k3                     gradient kernel with the workload's mask (rows outside it are zero-filled, not read)
      k7_masked              single-pass kernel, rows outside the mask zero-filled without being read
      k7_all_rows            single-pass kernel, rows outside the mask read for their log-prob and entropy
      k7_dense_mask          single-pass kernel with a mask of ones: every row read and written
      head_fwd_stash/_plain  fused head forward with / without keeping its softmax numerators
      head_bwd_every_token   fused head backward (from the kept products) with a gradient on every token
      head_bwd_step          the same with the benchmark's mask (tokens without gradient dropped first)"""
    import trl_amd
    from trl_amd import ops

    dev = torch.device("cuda:0")
    leg = args.only_leg
    B, T, V = w["B"], w["T"], w["V"]
    g = torch.Generator(device=dev).manual_seed(0)
    unit, peak = "GB/s", HBM_PEAK_GBPS
    if w.get("head"):
        if not leg.startswith("head_"):
            sys.exit(f"bench.py: leg {leg} does not belong to workload {args.workload}")
        N, H = B * T, w["H"]
        hidden = torch.randn((N, H), generator=g, device=dev).bfloat16()
        weight = (0.02 * torch.randn((V, H), generator=g, device=dev)).bfloat16()
        targets = torch.randint(0, V, (N,), generator=g, device=dev)
        lengths = torch.randint(w["min_len"], T + 1, (B,), generator=g, device=dev)
        mask = (torch.arange(T, device=dev)[None] < lengths[:, None]).reshape(-1)
        fwd_args = (hidden, weight, targets, w["temperature"], 0.0, 1.0)
        gl = torch.randn((N,), generator=g, device=dev)
        work = 2.0 * N * H * V
        unit, peak = "TFLOP/s", MFMA_BF16_PEAK_TFLOPS
        with torch.no_grad():
            if leg == "head_fwd_plain":
                fn = lambda: ops.fused_head_fwd(*fwd_args)  # noqa: E731
            elif leg == "head_fwd_stash":
                fn = lambda: ops.fused_head_fwd(*fwd_args, None, True)  # noqa: E731
            else:
                out = ops.fused_head_fwd(*fwd_args, None, True)
                log_z, saved = out[2], out[4]
                del out
                if leg == "head_bwd_every_token":
                    work *= 2
                    fn = lambda: ops.fused_head_bwd(*fwd_args, log_z, gl, HEAD_CHUNK, None, saved)  # noqa: E731
                else:
                    g_step = gl * mask.float()
                    work *= 2.0 * float(mask.sum()) / N
                    fn = lambda: ops.head_backward(*fwd_args, log_z, g_step, HEAD_CHUNK, None, saved)  # noqa: E731
    elif w.get("logp") or w.get("dpo"):
        if leg not in ("k1", "k1_stats", "k3") or (w.get("logp") and leg != "k1"):
            sys.exit(f"bench.py: leg {leg} does not belong to workload {args.workload}")
        dtype = torch.float32 if w.get("logp") else torch.bfloat16
        L = T
        K = T if w.get("logp") else T - 1
        logits = torch.empty((B, L, V), dtype=dtype, device=dev)
        for b in range(B):
            logits[b] = ((3.0 if w.get("logp") else 2.0) * torch.randn((L, V), generator=g, device=dev)).to(dtype)
        ids = torch.randint(0, V, (B, L), generator=g, device=dev)
        R = B * K
        idx = (ids if w.get("logp") else ids[:, 1:]).reshape(R, 1).contiguous()
        row_bytes = V * logits.element_size()
        if leg == "k1" and w.get("logp"):
            # 262 MB would stay in the memory-side cache between launches: rotate over eight copies, as the workload's
            # own bench leg does, so that every launch reads cold data
            work = R * row_bytes
            copies = [logits] + [logits.clone() for _ in range(7)]
            turn = [0]

            def fn():
                turn[0] += 1
                return ops.logp_entropy_fwd(copies[turn[0] % 8], idx, 1.0, 0, K, None)
        elif leg == "k1":
            work = R * row_bytes
            fn = lambda: ops.logp_entropy_fwd(logits, idx, 1.0, 0, K, None)  # noqa: E731
        elif leg == "k1_stats":
            work = R * row_bytes
            fn = lambda: ops.logp_entropy_stats_fwd(logits, idx, 1.0, 0, K, None, False)  # noqa: E731
        else:
            prompt = torch.randint(64, 513, (B // 2,), generator=g, device=dev).repeat(2)
            comp = torch.randint(128, 1537, (B,), generator=g, device=dev)
            pos = torch.arange(L, device=dev)[None]
            cmask = ((pos >= prompt[:, None]) & (pos < (prompt + comp)[:, None])).long()
            lse = ops.logp_entropy_fwd(logits, idx, 1.0, 0, K, None)[2]
            g_logp = (cmask[:, 1:].reshape(R, 1) * 0.01).float().contiguous()
            active = int(cmask[:, 1:].sum())
            work = active * 2 * row_bytes + (B * L - active) * row_bytes
            fn = lambda: ops.logp_entropy_bwd(logits, idx, 1.0, 0, K, lse, None, g_logp, None)  # noqa: E731
    else:
        if leg not in ("k1", "k3", "k7_masked", "k7_all_rows", "k7_dense_mask"):
            sys.exit(f"bench.py: leg {leg} does not belong to workload {args.workload}")
        logits, ids, mask, rewards, g = make_inputs(w, dev)
        R = B * T
        idx = ids.reshape(R, 1)
        adv = trl_amd.group_advantages(rewards, w["G"])
        row_bytes = V * 2
        active = int(mask.sum())
        with torch.no_grad():
            base, _, lse = ops.logp_entropy_fwd(logits, idx, w["temperature"], 0, T, None)
        base = base.view(B, T)
        old = base + 0.05 * torch.randn(base.shape, generator=g, device=dev)
        ref = base + 0.1 * torch.randn(base.shape, generator=g, device=dev) if w["beta"] else None
        n_items = mask.sum().float()
        row_scale = (1.0 / n_items.clamp(min=1.0)).expand(B)
        if leg == "k1":
            work = R * row_bytes
            fn = lambda: ops.logp_entropy_fwd(logits, idx, w["temperature"], 0, T, None)  # noqa: E731
        elif leg == "k3":
            g_logp = (mask.reshape(R, 1) * 0.01).float().contiguous()
            work = active * 2 * row_bytes + (R - active) * row_bytes
            fn = lambda: ops.logp_entropy_bwd(logits, idx, w["temperature"], 0, T, lse, None, g_logp, None)  # noqa: E731
        else:
            m = torch.ones_like(mask) if leg == "k7_dense_mask" else mask
            every = leg == "k7_all_rows"
            work = 2 * R * row_bytes if leg != "k7_masked" else active * 2 * row_bytes + (R - active) * row_bytes
            fn = lambda: ops.grpo_fused_fwd_bwd(logits, ids, w["temperature"], 0, T, m, adv, row_scale, old, ref, None,  # noqa: E731
                                                None, 0, w["eps_low"], w["eps_high"], float("nan"), w["beta"], False,
                                                1.0, 1.05, every)
    with torch.no_grad():
        for _ in range(max(1, args.warmup)):
            out = fn()
            del out
        torch.cuda.synchronize()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        for _ in range(args.steps):
            out = fn()
            del out
        b.record()
        torch.cuda.synchronize()
    ms = a.elapsed_time(b) / args.steps
    achieved = work / (ms * 1e-3) / (1e9 if unit == "GB/s" else 1e12)
    if args.calibrate_copy:  # a plain device copy of known size, to scale the profiler's byte counters by
        src = torch.empty((1 << 28,), dtype=torch.float32, device=dev).normal_()
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)  # reads and writes 1 GiB each
        torch.cuda.synchronize()
    return {"workload": args.workload, "leg": leg, "launches": args.steps, "warmup_launches": max(1, args.warmup),
            "avg_launch_ms": ms, "algorithmic_bytes" if unit == "GB/s" else "algorithmic_flop": work,
            "achieved": achieved, "unit": unit, "peak": peak, "frac": achieved / peak}


def _summary_rows(r):
    """Compact rows for the end of the line: per workload / loss type the step time, the dominant kernel's fraction of
    its roofline and the step's own (HBM workloads) or the TFLOP/s (matrix workload); numbers rounded."""
    cfg = r.get("config", {})
    name, lt = r.get("workload") or cfg.get("workload"), r.get("loss_type") or cfg.get("loss_type")
    if "error" in r:
        return [{"w": name, "lt": lt, "error": r["error"][:80]}]
    roof = r["roofline"]
    kern = {"grpo_fused_kernel (K7)": "K7", "logp_entropy_bwd_kernel (K3)": "K3", "logp_entropy_fwd_kernel (K1)": "K1",
            "fused_head_fwd_kernel": "head_fwd"}.get(roof["kernel"], roof["kernel"])
    row = {"w": name, "lt": lt, "ms": round(r["ms_per_step"], 3), "k": kern, "frac": round(roof["frac"], 3)}
    if roof.get("step_hbm_frac") is not None:
        row["step_frac"] = round(roof["step_hbm_frac"], 3)
    rows = [row]
    kernels = r.get("kernels") or {}
    if roof["bound"] == "mfma":
        row["TFLOPs"] = round(roof["achieved"])
        bwd = kernels.get("fused_head_bwd")
        if bwd:
            rows.append({"w": name, "k": "head_bwd_every_token", "ms": round(bwd["avg_ms"], 2), "frac": round(bwd["frac"], 3),
                         "TFLOPs": round(bwd["TFLOPs"])})
        plain = kernels.get("fused_head_fwd_no_grad")
        if plain:
            rows.append({"w": name, "k": "head_fwd_no_stash", "ms": round(plain["avg_ms"], 2), "frac": round(plain["frac"], 3)})
    for key, short in (("grpo_fused_kernel (K7), every row active (a mask of ones)", "K7_dense_mask"),
                       ("logp_entropy_fwd_kernel (K1)", "K1"), ("logp_entropy_bwd_kernel (K3)", "K3"),
                       ("logp_entropy_fwd_kernel with row statistics (K1)", "K1_stats")):
        k = kernels.get(key)
        if k and short != kern:
            rows.append({"w": name, "k": short, "ms": round(k["avg_launch_ms"], 3), "frac": round(k["frac"], 3)})
    return rows


def _is_hip_runtime_error(exc):
    text = f"{type(exc).__name__}: {exc}"
    return "HIP error" in text or "hipError" in text or "AcceleratorError" in text


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default=None, choices=sorted(WORKLOADS),
                    help="one workload only (default: grpo_c3 as the headline plus the others as `secondary`)")
    ap.add_argument("--loss-type", default="dapo", choices=["grpo", "dapo", "dr_grpo", "bnpo"])
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-secondary", action="store_true")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run a plain device copy of the logits (known bytes) to scale profiler counters by")
    ap.add_argument("--only-leg", default=None, choices=sorted(LEGS),
                    help="launch ONE kernel of --workload in ONE mode --steps times and print its event-timed average "
                         "(for profiler runs: every launch of that kernel in the trace then moves the same bytes)")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        sys.exit("bench.py: this build runs on ONE GPU; rows are independent, so N GPUs would each run this same "
                 "kernel on B/N sequences and exchange a handful of scalars per step. Run with --gpus 1.")
    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible; the hot path has no CPU fallback.")
    torch.cuda.set_device(0)
    secondary_wanted = args.workload is None and not args.no_secondary
    args.workload = args.workload or "grpo_c3"
    w = WORKLOADS[args.workload]
    if args.only_leg:
        return print(json.dumps(bench_one_leg(args, w)))
    if w.get("head"):
        return print(json.dumps(bench_head(args, w)))
    if w.get("dpo"):
        return print(json.dumps(bench_dpo(args, w)))
    if w.get("logp"):
        return print(json.dumps(bench_logp_c1(args, w)))
    result, shared = bench_grpo(args, w, args.loss_type)
    secondary = []
    device_lost = False  # after a HIP runtime error every later launch fails the same way: no further legs
    if secondary_wanted:
        few = argparse.Namespace(**{**vars(args), "steps": max(3, args.steps // 2), "warmup": 2, "no_cpu_baseline": True,
                                    "calibrate_copy": False})
        for lt in ("grpo", "dr_grpo"):
            if lt != args.loss_type and not device_lost:
                try:
                    secondary.append(_brief(bench_grpo(few, w, lt, shared, full=False)[0]))
                except Exception as exc:
                    secondary.append({"workload": args.workload, "loss_type": lt, "error": f"{type(exc).__name__}: {exc}"[:500]})
                    device_lost = _is_hip_runtime_error(exc)
    del shared
    if secondary_wanted:
        # (the matrix-core workload first: its clock is set by the power budget and falls as the part warms up,
        # the streaming workloads are bound by memory and hardly notice)
        for name in ("head_c5", "grpo_c4", "dpo_c2", "logp_c1"):
            if device_lost:
                secondary.append({"workload": name, "error": "not run: an earlier workload ended in a HIP runtime error"})
                continue
            torch.cuda.empty_cache()
            few.workload = name
            w2 = WORKLOADS[name]
            try:
                r = (bench_head(few, w2) if w2.get("head") else bench_dpo(few, w2) if w2.get("dpo")
                     else bench_logp_c1(few, w2) if w2.get("logp") else bench_grpo(few, w2, "dapo")[0])
                secondary.append(_brief(r))
                del r
            except Exception as exc:  # a secondary workload never takes the headline line with it
                secondary.append({"workload": name, "error": f"{type(exc).__name__}: {exc}"[:500]})
                device_lost = _is_hip_runtime_error(exc)
        result["secondary"] = secondary
    if not args.no_cpu_baseline:
        base = cpu_baseline(w, args.loss_type, repeats=1)
        secs = 32 * 512 / base["value"]
        if secs < 5.0:  # a fast host: the sample grows towards ~10 s of work per run
            base = cpu_baseline(w, args.loss_type, n_seq=int(min(96, max(32, 32 * 10.0 / secs))) // 8 * 8)
        result["cpu_baseline"] = base
    else:
        result["cpu_baseline"] = None
    # the end of the line: what a reader of its last 2000 characters needs -- every workload's step time and roofline
    # fractions, and whether a secondary workload failed
    errors = [f"{r.get('workload')}/{r.get('loss_type')}: {r['error']}"[:200] for r in secondary if "error" in r]
    result["secondary_errors"] = errors
    summary = _summary_rows(result)
    for r in secondary:
        summary += _summary_rows(r)
    result["summary"] = summary
    print(json.dumps(result))
    if errors:
        sys.exit(f"bench.py: {len(errors)} secondary workload(s) failed: {errors}")


if __name__ == "__main__":
    main()
