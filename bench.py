#!/usr/bin/env python3
"""Benchmark of the transducer-loss hot path on one MI355X.

A step is one forward + backward of the loss module over one resident batch:
    costs = loss(acts, labels, act_lens, label_lens); costs.sum().backward()
on the north-star workload (RNNT, B=16, T=375, U+1=121, V=1025, fp32, variable
lengths), inputs already in HBM.  The timed steps are training steps, not replays: every step gets length tensors it
has not seen (so the module's shape-vs-lengths check runs, with its read-back and host wait, as it does for a fresh
batch) and the logits alternate between two buffers (so no step starts on what the step before left in the
last-level cache).  The same loop over one set of tensors is timed beside it (`whole_job.same_tensors_ms_per_step`).
Prints ONE JSON line:
  value        logit elements per second (B*T*U*V / step time)
  roofline     the gradient pass (the dominant kernel; its name for this shape is reported):
               algorithmic bytes per launch / its mean duration, measured with HIP events around
               its launches in a second pass over the same steps (an event pair costs queue time, so
               the steps that give ms_per_step carry none)
  cpu_baseline the C restatement of the reference's CPU path on a bounded sample, host cores (all threads, one
               thread, and the interpreted per-cell restatement at configuration 1)
  other_workloads  configurations 3, 4, 5 and the multi-blank one: median ms/step, bytes, fraction of peak
  kernels      mean duration of each pipeline kernel over the timed steps (ms)
  copy_probe   bandwidth a plain device copy reaches on this GPU (GB/s, read + write)

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload 0..5] [--op loss|logprobs|joint] [--no-cpu-baseline]

--op logprobs measures the compact log-prob op on the same tensors instead (speech_amd.k2.rnnt_logprobs
forward + backward with given upstream gradients; RNNT workloads only).
--op joint measures the fused joint + loss (speech_amd.joint.joint_rnnt_loss, forward + backward to f, g, weight,
bias) on joint inputs of the same lattice shape (H = 640, bf16); its roofline is the matrix cores: useful
flops of the logit recomputation kernel (2 * valid cells * V * H) over its mean duration, against 2.5 PFLOP/s.
"""

import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0  # MI355X HBM3E, published peak

# HBM bytes per launch of the gradient-pass kernel from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of
# this script, scaled by what the same counters read for mi_transducer_copy_probe of known size
# (summaries under profiles/).  None = not measured for that workload.
MEASURED_TRAFFIC_KIB = {
    # workload: (FETCH_SIZE, WRITE_SIZE) of the gradient-pass kernel in KiB per dispatch; the factors below are what the
    # same counters need to read a 1 GiB copy right (profiles/transducer_kernels_<cfg>_hbm_traffic.md)
    "cfg2_rnnt_B16_T375_U121_V1025_f32": (807541, 2598715),
    "cfg3_rnnt_B32_T750_U201_V1025_bf16": (2938583, 8566134),
    "cfg4_tdt_B16_T375_U121_V1025_D5_f32": (760714, 1786097),
    "cfg5_rnnt_B8_T250_U101_V16385_f32": (3669187, 12770381),
    "cfg6_multiblank_B16_T375_U121_V1028_f32": (684890, 1978605),
}
TRAFFIC_SCALE = (2.0, 1.0)


def measured_traffic(name):
    kib = MEASURED_TRAFFIC_KIB.get(name)
    return None if kib is None else int((kib[0] * TRAFFIC_SCALE[0] + kib[1] * TRAFFIC_SCALE[1]) * 1024)


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=30)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", type=int, default=1, help="index into speech_amd.synthetic.CONFIGS (1 = north star)")
    ap.add_argument("--op", choices=["loss", "logprobs", "joint"], default="loss")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-graph", action="store_true", help="skip the HIP-graph replay timing of the same step")
    ap.add_argument("--no-other-workloads", action="store_true",
                    help="skip the short runs of the other benchmark configurations (default run of workload 1 only)")
    ap.add_argument("--same-tensors", action="store_true",
                    help="headline loop over ONE set of tensors (the length check is then remembered and pass 1 starts "
                         "in the last step's cache tail); default: fresh length tensors and alternating logits buffers")
    ap.add_argument("--full-lengths", action="store_true",
                    help="every utterance at full length (act_lens = T, label_lens = U-1): the same kernels without "
                         "padding, for counter profiles that hold ragged against full lengths")
    ap.add_argument("--cpu-sample-utterances", type=int, default=16)
    return ap.parse_args()


def cpu_baseline(cfg, acts, labels, act_lens, label_lens, n_utt):
    """The reference's CPU path (log_softmax, per-utterance lattice, sparse gradient, softmax
    Jacobian) restated in C, timed on the host cores over the first n_utt utterances: on all threads (`value`), on one
    thread over fewer utterances (`c1_value`), and -- for RNNT -- the interpreted per-cell restatement (what a user of
    the reference gets on a CPU) on the reference's own CPU-sized configuration (`interpreted_cfg1`)."""
    import numpy as np

    import oracle

    threads = max(1, min(16, os.cpu_count() or 1))
    n_utt = min(n_utt, cfg.B)
    lam, clamp = cfg.fastemit_lambda, max(cfg.clamp, 0.0)

    def timed(n, nthreads, budget_core_s, max_passes):
        x = acts[:n].float().cpu().numpy()
        lab, al, ll = labels[:n].cpu().numpy(), act_lens[:n].cpu().numpy(), label_lens[:n].cpu().numpy()

        def one_pass():
            if cfg.D:
                oracle.tdt_loss(x, lab, al, ll, cfg.blank, cfg.durations, cfg.sigma, lam, clamp, dtype=np.float32,
                                num_threads=nthreads)  # fmt: skip
            elif cfg.big_blank_durations:
                oracle.multiblank_loss(x, lab, al, ll, cfg.blank, cfg.big_blank_durations, cfg.sigma, lam, clamp,
                                       dtype=np.float32, num_threads=nthreads)  # fmt: skip
            else:
                oracle.rnnt_cpu_path(x, lab, al, ll, cfg.blank, lam, clamp, dtype=np.float32, num_threads=nthreads)

        passes, t0 = 0, time.perf_counter()
        while passes < max_passes and (passes == 0 or (time.perf_counter() - t0) * nthreads < budget_core_s):
            one_pass()
            passes += 1
        dt = time.perf_counter() - t0
        return passes * x.size / dt, passes, dt

    # whole passes until about 20 core-seconds of work are spent (at most 8 passes)
    value, passes, dt = timed(n_utt, threads, 20.0, 8)
    n1 = max(1, min(2, n_utt))
    c1_value, c1_passes, c1_dt = timed(n1, 1, 5.0, 4)
    out = {
        "value": value,
        "unit": "logit elems/s",
        "cores": threads,
        "kind": "port",
        "sample": f"first {n_utt} of {cfg.B} utterances of the same batch, full T x U x V, {passes} pass(es), "
                  f"{dt:.2f} s wall on {threads} threads",
        "c1_value": c1_value,
        "c1_sample": f"first {n1} utterance(s), {c1_passes} pass(es), {c1_dt:.2f} s wall on 1 thread",
    }  # fmt: skip
    if not cfg.D and not cfg.big_blank_durations:
        out["interpreted_cfg1"] = interpreted_baseline()
    return out


def interpreted_baseline():
    """The interpreted restatement of the reference's CPU path (per-cell loops over 0-d torch tensors, one thread) on
    configuration 1 (B=4, T=50, U=21, V=129), checked against the C restatement before its time is reported."""
    import numpy as np

    import oracle
    from oracle.cpu_path_interpreted import rnnt_cpu_path_interpreted
    from speech_amd import synthetic

    cfg1, acts, labels, act_lens, label_lens = synthetic.make_inputs(0)
    x, lab, al, ll = acts.numpy(), labels.numpy(), act_lens.numpy(), label_lens.numpy()
    t0 = time.perf_counter()
    costs, grads = rnnt_cpu_path_interpreted(x, lab, al, ll, cfg1.blank)
    dt = time.perf_counter() - t0
    c_ref, g_ref = oracle.rnnt_cpu_path(x, lab, al, ll, cfg1.blank, dtype=np.float64)
    # the interpreted path keeps its lattice in float32, as the reference does: 5e-4 on the gradient, not 1e-4
    assert np.allclose(costs, c_ref, rtol=1e-5) and np.abs(grads - g_ref).max() < 5e-4
    return {"value": x.size / dt, "unit": "logit elems/s", "cores": 1, "workload": cfg1.name, "seconds": dt}


def cpu_baseline_logprobs(cfg, acts, labels, act_lens, label_lens, g_target, g_blank, n_utt):
    """The numpy restatement of the compact log-prob op (forward + backward), one host thread."""
    import oracle

    n_utt = min(n_utt, cfg.B)
    x = acts[:n_utt].float().cpu().numpy()
    lab = labels[:n_utt].cpu().numpy()
    al = act_lens[:n_utt].cpu().numpy()
    ll = label_lens[:n_utt].cpu().numpy()
    gt, gb = g_target[:n_utt].cpu().numpy(), g_blank[:n_utt].cpu().numpy()
    t0 = time.perf_counter()
    oracle.rnnt_logprobs(x, lab, cfg.blank, al, ll)
    oracle.rnnt_logprobs_grad(x, lab, cfg.blank, gt, gb, al, ll)
    dt = time.perf_counter() - t0
    return {
        "value": x.size / dt,
        "unit": "logit elems/s",
        "cores": 1,
        "kind": "port",
        "sample": f"first {n_utt} of {cfg.B} utterances of the same batch, full T x U x V, forward + backward, "
                  f"{dt:.2f} s wall (numpy, float64)",
    }  # fmt: skip


def median(sorted_values):
    n = len(sorted_values)
    return sorted_values[n // 2] if n % 2 else 0.5 * (sorted_values[n // 2 - 1] + sorted_values[n // 2])


def run_steps(torch, step_fn, bufs, act_lens, label_lens, steps, fresh):
    """`steps` forward + backward steps, each timed by the stream events on either side of it.
    step_fn(acts, act_lens, label_lens) -> costs.  fresh (a training loop): every step is given length tensors of its
    own (cloned here, before the clock starts, so the module has not seen them and checks them against the shape as
    it must for a new batch) and the next of the logits buffers in `bufs`; otherwise one set of tensors serves
    every step.  Returns (sorted per-step ms, wall seconds, event ms over the whole loop, last costs)."""
    if fresh:
        lens = [(act_lens.clone(), label_lens.clone()) for _ in range(steps)]
    else:
        lens = [(act_lens, label_lens)] * steps
    marks = [torch.cuda.Event(enable_timing=True) for _ in range(steps + 1)]
    costs = None
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    marks[0].record()
    for i in range(steps):
        costs = step_fn(bufs[i % len(bufs)] if fresh else bufs[0], *lens[i])
        marks[i + 1].record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    per_step = sorted(marks[i].elapsed_time(marks[i + 1]) for i in range(steps))
    return per_step, wall, marks[0].elapsed_time(marks[-1]), costs


PROTOCOLS = {
    True: "training steps: length tensors the module has not seen (its shape check runs every step) and two "
          "alternating logits buffers",
    False: "one set of tensors for every step (the length check is remembered after the first, and pass 1 starts on "
           "what the last step left in the last-level cache)",
}  # fmt: skip


def riders_filled_bytes(torch, cfg, acts, labels, act_lens, label_lens, reps=5):
    """Bytes of gradient padding that the riders of the lattice launch zero-fill per step (median over a few forward
    calls at the function-level seam; it varies a little with how the workgroups were placed), or 0 where the
    modules do not use them."""
    from speech_amd.rnnt_loss import rnnt, rnnt_pytorch

    if not rnnt_pytorch._prefill_wanted(acts):
        return 0
    nd = cfg.D or len(cfg.big_blank_durations)
    ws = rnnt.new_workspace(acts, nd)
    costs = torch.empty(cfg.B, dtype=torch.float32, device=acts.device)
    grads = torch.empty_like(acts)
    lam = cfg.fastemit_lambda
    filled = []
    for _ in range(reps):
        if cfg.D:
            rnnt.tdt_forward(acts, labels, act_lens, label_lens, costs, cfg.blank, cfg.durations, lam, cfg.sigma, False,
                             True, ws, grads)  # fmt: skip
        elif cfg.big_blank_durations:
            rnnt.multiblank_forward(acts, labels, act_lens, label_lens, costs, cfg.blank, cfg.big_blank_durations, lam,
                                    cfg.sigma, True, ws, grads)  # fmt: skip
        else:
            rnnt.rnnt_forward(acts, labels, act_lens, label_lens, costs, cfg.blank, lam, True, ws, grads)
        cells = rnnt.prefilled_cells(ws, act_lens, label_lens, cfg.B, cfg.T, cfg.U, acts.shape[-1], acts.element_size(), nd)
        filled.append(int(cells.sum().item()) * acts.shape[-1] * acts.element_size())
    del grads
    return sorted(filled)[len(filled) // 2]


def graph_replay(torch, cfg, acts, labels, act_lens, label_lens, steps):
    """The same forward + backward at the function-level seam (caller-owned costs / grads / workspace, grad_output
    = ones), captured once into a HIP graph and replayed: what a training loop with static shapes pays per step
    when launch gaps and the Python/autograd layer are out of the picture.  Reported beside the headline, not as it."""
    from speech_amd.rnnt_loss import rnnt

    B = cfg.B
    costs = torch.empty(B, dtype=torch.float32, device=acts.device)
    grads = torch.empty_like(acts)
    ones = torch.ones(B, dtype=torch.float32, device=acts.device)
    lam, clamp = cfg.fastemit_lambda, max(cfg.clamp, 0.0)
    if cfg.D:
        ws = rnnt.new_workspace(acts, cfg.D)

        def run():
            rnnt.tdt_forward(acts, labels, act_lens, label_lens, costs, cfg.blank, cfg.durations, lam, cfg.sigma, False,
                             True, ws, grads)  # fmt: skip
            rnnt.tdt_backward(acts, labels, act_lens, label_lens, grads, ones, cfg.blank, cfg.durations, lam, clamp,
                              cfg.sigma, False, ws, padding_zeroed=2)  # fmt: skip
    elif cfg.big_blank_durations:
        ws = rnnt.new_workspace(acts, len(cfg.big_blank_durations))

        def run():
            rnnt.multiblank_forward(acts, labels, act_lens, label_lens, costs, cfg.blank, cfg.big_blank_durations, lam,
                                    cfg.sigma, True, ws, grads)  # fmt: skip
            rnnt.multiblank_backward(acts, labels, act_lens, label_lens, grads, ones, cfg.blank,
                                     cfg.big_blank_durations, lam, clamp, cfg.sigma, ws, padding_zeroed=2)  # fmt: skip
    else:
        ws = rnnt.new_workspace(acts)

        def run():
            rnnt.rnnt_forward(acts, labels, act_lens, label_lens, costs, cfg.blank, lam, True, ws, grads)
            rnnt.rnnt_backward(acts, labels, act_lens, label_lens, grads, ones, cfg.blank, lam, clamp, ws,
                               padding_zeroed=2)

    run()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        run()
    for _ in range(3):
        graph.replay()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        graph.replay()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / steps
    assert bool(torch.isfinite(costs).all())
    del grads
    return {"ms_per_step": ms, "logit_elems_per_s": cfg.elems / (ms * 1e-3),
            "what": "mi_*_forward + mi_*_backward (grad_output = 1) replayed from one captured HIP graph"}  # fmt: skip


def other_workloads(torch, dev, indices, steps=8, warmup=3):
    """The remaining benchmark configurations, a few steps each, outside the headline's timed region: median step
    time by stream events, algorithmic bytes and the fraction of the HBM peak of the whole fwd+bwd step."""
    from speech_amd import MultiblankRNNTLossNumba, RNNTLossNumba, TDTLossNumba, _native, synthetic

    out = []
    for index in indices:
        cfg, acts, labels, act_lens, label_lens = synthetic.make_inputs(index, device=dev, generate_on_device=True)
        acts.requires_grad_(True)
        if cfg.D:
            loss = TDTLossNumba(blank=cfg.blank, durations=cfg.durations, reduction='none',
                                fastemit_lambda=cfg.fastemit_lambda, clamp=cfg.clamp, sigma=cfg.sigma)  # fmt: skip
        elif cfg.big_blank_durations:
            loss = MultiblankRNNTLossNumba(blank=cfg.blank, big_blank_durations=cfg.big_blank_durations,
                                           reduction='none', fastemit_lambda=cfg.fastemit_lambda, clamp=cfg.clamp,
                                           sigma=cfg.sigma)  # fmt: skip
        else:
            loss = RNNTLossNumba(blank=cfg.blank, reduction='none', fastemit_lambda=cfg.fastemit_lambda,
                                 clamp=cfg.clamp)  # fmt: skip
        nbytes = synthetic.algorithmic_bytes(cfg, act_lens, label_lens)
        bufs = [acts, acts.detach().clone().requires_grad_(True)]

        def step(a, al, ll):
            a.grad = None
            costs = loss(a, labels, al, ll)
            costs.sum().backward()
            return costs

        run_steps(torch, step, bufs, act_lens, label_lens, warmup, True)
        per_step, _, _, costs = run_steps(torch, step, bufs, act_lens, label_lens, steps, True)
        assert bool(torch.isfinite(costs.float()).all()), "non-finite costs"
        ms = median(per_step)
        # a second pass with every pipeline kernel bracketed by events (not part of ms_per_step: the brackets cost
        # queue time): where the step goes, and how close the dominant kernel, the gradient pass, is to the HBM peak
        _native.profile_enable(steps)
        run_steps(torch, step, bufs, act_lens, label_lens, steps, True)
        kernels = {k: v[0] / max(v[1], 1) for k, v in _native.profile_read().items()}
        _native.profile_disable()
        for a in bufs:
            a.grad = None
        grad_ms = kernels.get("gradient_pass", 0.0)
        riders_bytes = riders_filled_bytes(torch, cfg, acts.detach(), labels, act_lens, label_lens)
        out.append({
            "workload": cfg.name, "steps": steps, "ms_per_step": ms, "logit_elems_per_s": cfg.elems / (ms * 1e-3),
            "algorithmic_bytes": nbytes["total"], "achieved_GBps": nbytes["total"] / (ms * 1e-3) / 1e9,
            "frac_of_peak": nbytes["total"] / (ms * 1e-3) / 1e9 / HBM_PEAK_GBPS,
            "dtype": {torch.float32: "f32", torch.bfloat16: "bf16", torch.float16: "f16"}[cfg.dtype],
            "kernel_ms": kernels,
            "riders_filled_bytes": riders_bytes,
            "gradient_pass_frac_of_peak": (((nbytes["grad_stream"] - riders_bytes) / (grad_ms * 1e-3) / 1e9 / HBM_PEAK_GBPS)
                                           if grad_ms else None),
            "gradient_pass_traffic_bytes": measured_traffic(cfg.name),
            "protocol": PROTOCOLS[True],
        })  # fmt: skip
        del acts, bufs, costs, loss
        torch.cuda.empty_cache()
    return out


MFMA_BF16_PEAK_TFLOPS = 2500.0  # MI355X dense bf16, published peak
JOINT_HIDDEN = 640  # joint_hidden of the reference's FastConformer transducer configs


def run_joint(args, torch, dev, cfg, labels, act_lens, label_lens):
    """--op joint: one step = joint_rnnt_loss (joint_tdt_loss for the TDT workload) forward + backward
    (gradients of f, g, weight, bias)."""
    from speech_amd import _native
    from speech_amd.joint import joint_multiblank_loss, joint_rnnt_loss, joint_tdt_loss

    B, T, U, H = cfg.B, cfg.T, cfg.U, JOINT_HIDDEN
    V = cfg.V + cfg.D  # outputs of the joint's Linear layer (token logits, then duration logits)
    gen = torch.Generator(device=dev).manual_seed(1234)
    f = torch.randn(B, T, H, device=dev, generator=gen).to(torch.bfloat16).requires_grad_(True)
    g = torch.randn(B, U, H, device=dev, generator=gen).to(torch.bfloat16).requires_grad_(True)
    weight = (torch.randn(V, H, device=dev, generator=gen) / H**0.5).requires_grad_(True)
    bias = (torch.randn(V, device=dev, generator=gen) * 0.1).requires_grad_(True)
    valid = int((act_lens * (label_lens + 1)).sum())

    def step():
        for p in (f, g, weight, bias):
            p.grad = None
        if cfg.D:
            costs = joint_tdt_loss(f, g, weight, bias, labels, act_lens, label_lens, cfg.blank, cfg.durations, cfg.sigma,
                                   cfg.fastemit_lambda, max(cfg.clamp, 0.0))  # fmt: skip
        elif cfg.big_blank_durations:
            costs = joint_multiblank_loss(f, g, weight, bias, labels, act_lens, label_lens, cfg.blank,
                                          cfg.big_blank_durations, cfg.sigma, cfg.fastemit_lambda, max(cfg.clamp, 0.0))  # fmt: skip
        else:
            costs = joint_rnnt_loss(f, g, weight, bias, labels, act_lens, label_lens, cfg.blank, cfg.fastemit_lambda,
                                    max(cfg.clamp, 0.0))  # fmt: skip
        costs.sum().backward()
        return costs

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    # the timed steps carry no events; the kernels' own times come from a second pass with the library's event pairs
    torch.cuda.reset_peak_memory_stats(dev)
    base_bytes = torch.cuda.memory_allocated(dev)
    t0 = time.perf_counter()
    for _ in range(args.steps):
        costs = step()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    step_peak_bytes = torch.cuda.max_memory_allocated(dev) - base_bytes  # what a step allocates on top of its inputs
    _native.profile_enable(args.steps, ["denominator_pass", "lattice", "cells", "gradient_pass", "weight_gradient"])
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    kernels = _native.profile_read()
    _native.profile_disable()
    assert bool(torch.isfinite(costs).all()), "non-finite costs"
    ms_per_step = wall * 1e3 / args.steps
    # three matrix products of 2 * valid cells * V * H flops each: logits (forward kernel), d hidden, d weight
    flops = 2.0 * valid * V * H
    stage_s = {k: ms * 1e-3 / max(n_, 1) for k, (ms, n_) in kernels.items() if n_}
    names = {"denominator_pass": "joint_lse_kernel (logits -> denominators, arc log-probs, saved logits and activations)",
             "gradient_pass": "joint_dhidden_kernel (saved logits -> gradient entries -> d hidden)",
             "weight_gradient": "joint_dweight_kernel (saved logits -> gradient entries -> d weight, d bias)"}
    products = {names[k]: {"avg_launch_ms": stage_s[k] * 1e3, "achieved_tflops": flops / stage_s[k] / 1e12,
                           "frac_of_peak": flops / stage_s[k] / 1e12 / MFMA_BF16_PEAK_TFLOPS}
                for k in names if k in stage_s}  # fmt: skip
    fwd_s = stage_s["denominator_pass"]
    achieved = flops / fwd_s / 1e12
    result = {
        "metric": "fused joint + %s loss fwd+bwd: logit elems/s and achieved MFMA TFLOP/s vs peak" % ("TDT" if cfg.D else ("multi-blank" if cfg.big_blank_durations else "RNNT")),
        "value": cfg.elems / (ms_per_step * 1e-3),
        "unit": "logit elems/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms_per_step,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": cfg.name.replace("_f32", "") + "_joint_H%d_bf16" % H, "B": B, "T": T, "U": U, "V": V, "H": H,
                   "valid_cells": valid, "cells": B * T * U},
        "roofline": {
            "kernel": "joint_lse_kernel<H=%d> (the longest of the three product kernels)" % H, "bound": "mfma",
            "achieved": achieved, "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s", "frac": achieved / MFMA_BF16_PEAK_TFLOPS,
            "traffic": None, "algorithmic_flops_per_launch": flops, "avg_launch_ms": fwd_s * 1e3,
            "launches": kernels["denominator_pass"][1],
        },
        "kernels": {k: v * 1e3 for k, v in stage_s.items()},
        "product_kernels": products,
        "whole_job": {"useful_tflop_per_step": 3 * flops / 1e12,
                      "achieved_tflops": 3 * flops / (ms_per_step * 1e-3) / 1e12,
                      "step_peak_memory_GB": step_peak_bytes / 1e9,
                      "note": "three products per step (logits, d hidden, d weight), each in a kernel of this library; "
                              "no library GEMM and no host wait in the step"},
    }  # fmt: skip
    if not args.no_cpu_baseline:
        import oracle

        Tb, Ub = int(act_lens[0]), int(label_lens[0]) + 1
        x = (f[:1, :Tb].detach().float().cpu().numpy(), g[:1, :Ub].detach().float().cpu().numpy(),
             weight.detach().cpu().numpy(), bias.detach().cpu().numpy())  # fmt: skip
        t0 = time.perf_counter()
        oracle.joint_rnnt_loss(*x, labels[:1, : Ub - 1].cpu().numpy(), [Tb], [Ub - 1], cfg.blank,
                               durations=cfg.durations if cfg.D else None, sigma=cfg.sigma,
                               big_blank_durations=cfg.big_blank_durations or None)
        dt = time.perf_counter() - t0
        result["cpu_baseline"] = {
            "value": Tb * Ub * V / dt, "unit": "logit elems/s", "cores": 1, "kind": "port",
            "sample": f"utterance 0 of {B} at its own lengths ({Tb} x {Ub} cells), forward + backward, {dt:.2f} s "
                      "wall (numpy float64; the lattice part in interpreted per-cell loops)",
        }  # fmt: skip
    print(json.dumps(result))


def main():
    args = parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build measures one GPU only; run with --gpus 1 (the loss is data-parallel over "
              "utterances, nothing is exchanged between GPUs)", file=sys.stderr)  # fmt: skip
        sys.exit(2)

    import torch

    from speech_amd import MultiblankRNNTLossNumba, RNNTLossNumba, TDTLossNumba, _native, synthetic

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(2)
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    _native.lib()  # fail now if the HIP library is missing

    cfg, acts, labels, act_lens, label_lens = synthetic.make_inputs(args.workload, device=dev, generate_on_device=True)
    if args.full_lengths:
        act_lens.fill_(cfg.T)
        label_lens.fill_(cfg.U - 1)
    if args.op == "joint":
        del acts
        return run_joint(args, torch, dev, cfg, labels, act_lens, label_lens)
    acts.requires_grad_(True)
    if cfg.D:
        loss = TDTLossNumba(blank=cfg.blank, durations=cfg.durations, reduction='none',
                            fastemit_lambda=cfg.fastemit_lambda, clamp=cfg.clamp, sigma=cfg.sigma)  # fmt: skip
    elif cfg.big_blank_durations:
        loss = MultiblankRNNTLossNumba(blank=cfg.blank, big_blank_durations=cfg.big_blank_durations, reduction='none',
                                       fastemit_lambda=cfg.fastemit_lambda, clamp=cfg.clamp, sigma=cfg.sigma)  # fmt: skip
    else:
        loss = RNNTLossNumba(blank=cfg.blank, reduction='none', fastemit_lambda=cfg.fastemit_lambda, clamp=cfg.clamp)
    nbytes = synthetic.algorithmic_bytes(cfg, act_lens, label_lens)

    def step(a, al, ll):
        a.grad = None
        costs = loss(a, labels, al, ll)
        costs.sum().backward()
        return costs

    logprobs = args.op == "logprobs"
    if logprobs:
        if cfg.D or cfg.big_blank_durations:
            print("bench.py: --op logprobs runs on the RNNT workloads (0, 1, 2, 4)", file=sys.stderr)
            sys.exit(2)
        from speech_amd.k2 import rnnt_logprobs

        g_target = torch.rand(cfg.B, cfg.T, cfg.U, device=dev)
        g_blank = torch.rand(cfg.B, cfg.T, cfg.U, device=dev)
        # forward reads the valid rows and writes two score arrays; backward reads them, the two upstream
        # gradients and the valid rows again and writes every gradient element
        s_in = acts.element_size()
        nbytes = dict(nbytes)
        nbytes["total"] = 2 * nbytes["c_valid"] * cfg.V * s_in + nbytes["cells"] * cfg.V * s_in + 16 * nbytes["cells"]

        def step(a, al, ll):  # noqa: F811
            a.grad = None
            target_scores, blank_scores = rnnt_logprobs(a, labels, cfg.blank, al, ll)
            torch.autograd.backward([target_scores, blank_scores], [g_target, g_blank])
            return blank_scores

    bufs = [acts, acts.detach().clone().requires_grad_(True)]
    fresh = not args.same_tensors
    run_steps(torch, step, bufs, act_lens, label_lens, args.warmup, fresh)
    # the timed region: nothing but the steps (no kernel is bracketed by events here)
    per_step, wall, event_ms, costs = run_steps(torch, step, bufs, act_lens, label_lens, args.steps, fresh)
    assert bool(torch.isfinite(costs).all()), "non-finite costs"
    # the headline is the MEDIAN step (stream events between the steps of the one timed loop); the mean of the same
    # loop by the host clock and by the events is reported beside it
    ms_per_step = median(per_step)
    mean_wall_ms = wall * 1e3 / args.steps
    event_ms_per_step = event_ms / args.steps
    # the same loop under the other protocol, for comparison
    run_steps(torch, step, bufs, act_lens, label_lens, min(args.warmup, 2), not fresh)
    other_protocol_ms = median(run_steps(torch, step, bufs, act_lens, label_lens, args.steps, not fresh)[0])
    # per-kernel durations from a pass of their own: every pipeline kernel bracketed by a pair of HIP events on its
    # stream (the brackets cost queue time, so the steps above carry none)
    _native.profile_enable(args.steps)
    run_steps(torch, step, bufs, act_lens, label_lens, args.steps, fresh)
    kernels = breakdown = _native.profile_read()
    _native.profile_disable()
    bufs[1].grad = None
    del bufs

    # copy yardstick: 1 GiB device-to-device
    n = 1 << 30
    src = torch.empty(n, dtype=torch.uint8, device=dev)
    dst = torch.empty_like(src)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    for _ in range(3):
        _native.lib().mi_transducer_copy_probe(src.data_ptr(), dst.data_ptr(), n, stream)
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(10):
        _native.lib().mi_transducer_copy_probe(src.data_ptr(), dst.data_ptr(), n, stream)
    e1.record()
    torch.cuda.synchronize()
    copy_gbps = 2 * n * 10 / (e0.elapsed_time(e1) * 1e-3) / 1e9
    del src, dst

    from speech_amd.rnnt_loss import rnnt, rnnt_pytorch

    plan = _native.describe_plan(rnnt._dtype_code(acts), cfg.B, cfg.T, cfg.U, cfg.V, cfg.D,
                                 max(cfg.durations) if cfg.D else max(cfg.big_blank_durations, default=0),
                                 num_big_blanks=len(cfg.big_blank_durations))  # fmt: skip

    grad_ms, grad_n = kernels["gradient_pass"]
    grad_avg_s = grad_ms * 1e-3 / max(grad_n, 1)
    if logprobs:  # the op's backward always streams the coefficient records of its own cell kernel
        plan["lattice"], plan["cells"] = "none", "logprobs_export_kernel + logprobs_cell_kernel"
        plan["gradient"] = plan["gradient"].replace("fused>", "coef>")
    grad_bytes = nbytes["grad_stream"]
    # the riders of the lattice launch zero-fill part of the padding while the recursion runs; those bytes are the
    # lattice launch's, not the gradient pass's
    riders_bytes = 0 if logprobs else riders_filled_bytes(torch, cfg, acts.detach(), labels, act_lens, label_lens)
    grad_bytes -= riders_bytes
    achieved = grad_bytes / grad_avg_s / 1e9
    result = {
        "metric": ("compact log-prob op fwd+bwd: logit elems/s and achieved HBM GB/s vs peak" if logprobs else
                   "RNNT/TDT loss fwd+bwd: logit elems/s and achieved HBM GB/s vs peak"),
        "value": cfg.elems / (ms_per_step * 1e-3),
        "unit": "logit elems/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": {torch.float32: "f32", torch.bfloat16: "bf16", torch.float16: "f16"}[cfg.dtype],
        "data": "synthetic",
        "config": {
            "workload": cfg.name + ("_logprobs" if logprobs else "") + ("_full_lengths" if args.full_lengths else ""),
            "B": cfg.B, "T": cfg.T, "U": cfg.U, "V": cfg.V, "D": cfg.D,
            "valid_cells": nbytes["c_valid"], "cells": nbytes["cells"],
            "fastemit_lambda": cfg.fastemit_lambda, "clamp": cfg.clamp, "sigma": cfg.sigma,
        },
        "whole_job": {
            "algorithmic_bytes": nbytes["total"],
            "achieved_GBps": nbytes["total"] / (ms_per_step * 1e-3) / 1e9,
            "frac_of_peak": nbytes["total"] / (ms_per_step * 1e-3) / 1e9 / HBM_PEAK_GBPS,
            "event_ms_per_step": event_ms_per_step,
            "mean_wall_ms_per_step": mean_wall_ms,
            "min_ms_per_step": per_step[0],
            "max_ms_per_step": per_step[-1],
            "timing": "ms_per_step = median over the timed steps of the stream-event interval of each step",
            "protocol": PROTOCOLS[fresh],
            ("same_tensors_ms_per_step" if fresh else "training_steps_ms_per_step"): other_protocol_ms,
        },
        "roofline": {
            "kernel": plan["gradient"],
            "bound": "hbm",
            "achieved": achieved,
            "peak": HBM_PEAK_GBPS,
            "unit": "GB/s",
            "frac": achieved / HBM_PEAK_GBPS,
            "traffic": None if logprobs else measured_traffic(cfg.name),
            "algorithmic_bytes_per_launch": grad_bytes,
            "padding_zero_filled_by": "this kernel, less what the riders of the lattice launch did",
            "riders_filled_bytes": riders_bytes,
            "avg_launch_ms": grad_avg_s * 1e3,
            "launches": grad_n,
            "timed_in": "a second pass over the same steps with every pipeline kernel bracketed by HIP events",
        },
        "kernels": {k: (ms / max(n_, 1)) for k, (ms, n_) in breakdown.items()},
        "plan": plan,
        "copy_probe_GBps": copy_gbps,
    }  # fmt: skip
    if args.workload == 1 and not logprobs and not args.no_other_workloads:
        del acts, costs
        torch.cuda.empty_cache()
        result["other_workloads"] = other_workloads(torch, dev, [2, 3, 4, 5])
        cfg, acts, labels, act_lens, label_lens = synthetic.make_inputs(1, device=dev, generate_on_device=True)
    if not args.no_graph and not logprobs:
        result["graph_replay"] = graph_replay(torch, cfg, acts.detach(), labels, act_lens, label_lens, args.steps)
    if not args.no_cpu_baseline and logprobs:
        result["cpu_baseline"] = cpu_baseline_logprobs(
            cfg, acts.detach(), labels, act_lens, label_lens, g_target, g_blank, min(args.cpu_sample_utterances, 8)
        )
    elif not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(
            cfg, acts.detach(), labels, act_lens, label_lens, args.cpu_sample_utterances
        )
    print(json.dumps(result))


if __name__ == "__main__":
    main()
