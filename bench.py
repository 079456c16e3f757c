#!/usr/bin/env python3
"""Benchmark of bitfield-masked attention on one MI355X.

A step is one pass of the hot path over one batch of synthetic input that is already
resident in HBM: tile flags -> forward -> delta -> dK/dV -> dQ (gradients written in the
input dtype), i.e. everything ``bitfield_attn_func(...).backward(dO)`` launches.  The figure of merit is effective
TFLOP/s over UNMASKED (query, key) pairs: fwd 4*D*Hq*pairs, bwd 10*D*Hq*pairs.

Prints one JSON line (see --help for the knobs).  Next to the kernel-level step it reports the same work
driven through the public entry point (``bitfield_attn_func`` + ``torch.autograd.grad``, "api_ms_per_step"),
mean and median, the MFMA FLOPs the kernels issue according to their tile lists, a short record for the other
three GPU workloads, and the CPU baseline: the oracle's materialized-mask SDPA in fp32 on the host cores on a
bounded sample.
"""

from __future__ import annotations

import argparse
import json
import math
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_BF16_DENSE_TFLOPS = 2500.0  # MI355X published dense bf16 MFMA peak
PEAK_HBM_GBPS = 8000.0           # MI355X published HBM3E bandwidth


def library_gemm_tflops(dev, n=8192, reps=10):
    """bf16 GEMM of the vendor library (torch.matmul) on n x n x n, TFLOP/s: a reference point for what the MFMA
    units of this box sustain, measured next to the attention kernels."""
    import torch

    a = torch.randn(n, n, device=dev, dtype=torch.bfloat16)
    b = torch.randn(n, n, device=dev, dtype=torch.bfloat16)
    for _ in range(3):
        torch.matmul(a, b)
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    e0.record()
    for _ in range(reps):
        torch.matmul(a, b)
    e1.record()
    torch.cuda.synchronize()
    return round(2 * n ** 3 * reps / (e0.elapsed_time(e1) * 1e-3) / 1e12, 1)


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="C2", choices=["C1", "C2", "C3", "C4", "C5"],
                    help="C1 is the forward-only plumbing configuration (fp32 values rounded to bf16 for the kernels)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-other-workloads", action="store_true",
                    help="skip the short C3 / C4 / C5 records that accompany the default (C2) run")
    ap.add_argument("--other-steps", type=int, default=5)
    ap.add_argument("--copy-calibration", action="store_true",
                    help="after the timed region, run a plain 1 GiB device copy (reads 1 GiB, writes 1 GiB) so that "
                         "a rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE run of this command also holds a kernel of known traffic")
    return ap.parse_args()


def cpu_baseline(name):
    """Oracle (port of the reference tests' ground truth): bool mask from the bitfields +
    library SDPA in fp32 on the host, fwd+bwd (forward only for C1).  Bounded sample: the first KV group is timed
    first; if that took under 2 s (C1, C2, C4) the whole workload is timed, otherwise the one group stands."""
    import torch

    from cornstarch_amd import workloads as W
    from oracle import bam_oracle as O

    w = W.WORKLOADS[name]
    G = w.Hq // w.Hkv
    # every core this process may use: the scheduler's share where the environment states one, else all of them
    torch.set_num_threads(int(os.environ.get("OMP_NUM_THREADS") or 0) or os.cpu_count() or 1)
    bf = W.make_bitfields(name)

    def timed(heads, backward):
        q, k, v, do = (t.float() for t in W.make_tensors(name, heads=heads))
        t0 = time.perf_counter()
        O.sdpa_forward_backward(q, k, v, bf, do if backward else None, row_chunk=2048)
        return time.perf_counter() - t0

    backward = w.backward
    heads, q_heads, sample = (0, G), G, f"{name} q-heads 0..{G - 1} + kv-head 0, all {w.B} sequences"
    t = timed(heads, backward)
    if t < 2.0 and w.Hkv > 1:
        heads, q_heads, sample = None, w.Hq, f"{name}, the whole workload"
        t = timed(heads, backward)
    if t < 10.0:  # a second repetition where it is cheap; the faster one counts
        t = min(t, timed(heads, backward))
    t_fwd = timed(heads, False) if backward else t
    flops = (14 if backward else 4) * w.D * q_heads * O.unmasked_pairs(bf)
    return {
        "value": flops / t / 1e12,
        "unit": "TFLOP/s",
        "cores": torch.get_num_threads(),
        "kind": "port",
        "seconds": t,
        "fwd_seconds": t_fwd,
        "sample": sample + (", fwd+bwd" if backward else ", forward only") + " fp32 materialized-mask SDPA (oracle)",
    }


def measured_traffic(workload, kernel):
    """HBM bytes per launch of `kernel`, measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE and
    recorded in profiles/hbm_traffic.txt as lines `<workload> <kernel> <bytes>`; None if absent."""
    path = os.path.join(ROOT, "profiles", "hbm_traffic.txt")
    if not os.path.exists(path):
        return None
    with open(path) as f:
        for line in f:
            parts = line.split()
            if len(parts) >= 3 and parts[0] == workload and parts[1] == kernel:
                return float(parts[2])
    return None


def issued_flops(flags, plan, w, handover=False):
    """MFMA FLOPs the three attention kernels issue, from the tile lists they build: a wave of the forward
    and dQ kernels computes a 32-row slice against every 64-key tile in which the slice has a non-empty class
    (4 resp. 6 D-deep products per pair), a wave of dK/dV a 32-row slice against a 32-key group (8).  Partial
    tiles count in full.  Without a plan a slice inherits the classes of its 128-row block.  With the dS hand-over
    the dQ kernel runs one product per pair of the 32 x 32 blocks that have work (2)."""
    import torch.nn.functional as F

    cls = plan.fine_classes() if plan is not None else flags.repeat_interleave(4, dim=1)
    nz = cls > 0
    if nz.shape[-1] % 2:
        nz = F.pad(nz, (0, 1))
    tiles64 = int((nz[..., 0::2] | nz[..., 1::2]).sum())
    tiles32 = int(nz.sum())
    per_pair = w.D * w.Hq
    return {
        "fwd": 4 * per_pair * tiles64 * 32 * 64,
        "dkdv": 8 * per_pair * tiles32 * 32 * 32,
        "dq": 2 * per_pair * tiles32 * 32 * 32 if handover else 6 * per_pair * tiles64 * 32 * 64,
    }


def run_workload(name, steps, warmup, dev):
    """Times `steps` steps of workload `name` (after `warmup` untimed ones), kernel level and through the public
    entry point.  Returns a dict of measurements."""
    import torch

    from cornstarch_amd import workloads as W
    from cornstarch_amd.kernel import bitfield_attention as BA
    from oracle import bam_oracle as O  # checker / baseline only

    w = W.WORKLOADS[name]
    q, k, v, do = (t.to(dev) for t in W.make_tensors(name))
    if q.dtype == torch.float32:  # C1: the kernels take the fp32 values rounded to bf16
        q, k, v, do = (t.bfloat16() for t in (q, k, v, do))
    backward = w.backward
    bf = W.make_bitfields(name).to(dev)
    pairs = O.unmasked_pairs(bf)  # exact, on the GPU through torch ops (setup, untimed)
    f_fwd = 4 * w.D * w.Hq * pairs
    f_bwd = 10 * w.D * w.Hq * pairs if backward else 0
    scale = 1.0 / math.sqrt(w.D)

    stages = ["flags", "fwd", "alloc", "delta", "dkdv", "dq"]
    n_ev = len(stages) + 1
    handover = [False]  # did the last step hand dS from dK/dV to dQ through a workspace?

    def step(ev=None):
        def mark(i):
            if ev is not None:
                ev[i].record()

        mark(0)
        BA.BitfieldUtils.clear_cache()
        flags = BA.BitfieldUtils.materialize_compressed_mask_from_bitfield_mask(bf)
        plan = BA.BitfieldUtils.plan_for(flags, bf)  # built by the same launch as the flags
        mark(1)
        o, lse, _ = BA._bitfield_attn_forward(q, k, v, bf, flags, softmax_scale=scale)
        mark(2)
        if not backward:
            for i in range(3, n_ev):
                mark(i)
            return o, None
        dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
        delta = torch.empty_like(lse)
        # the dS workspace of the backward (head dim 128), sized from the plan's pair count, as the autograd path does
        ds_ws = plan.attach_ds_workspace(w.Hq, w.D, w.S) if plan is not None else None
        handover[0] = ds_ws is not None
        mark(3)
        BA._launch_bwd_preprocess(o, do, delta)
        mark(4)
        BA._launch_bwd_dkdv(q, k, v, do, lse, delta, dk, dv, bf, flags, scale, accumulate=False, plan=plan)
        mark(5)
        BA._launch_bwd_dq(q, k, v, do, lse, delta, dq, bf, flags, scale, accumulate=False, plan=plan)
        mark(6)
        if plan is not None:
            plan.detach_ds_workspace()
        return o, (dq, dk, dv)

    for _ in range(warmup):
        step()
    torch.cuda.synchronize()

    events = [[torch.cuda.Event(enable_timing=True) for _ in range(n_ev)] for _ in range(steps)]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(steps):
        step(events[i])
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0

    ms_per_step = wall * 1e3 / steps
    per_step = [ev[0].elapsed_time(ev[-1]) for ev in events]
    stage_ms, stage_med = {}, {}
    for si, s in enumerate(stages):
        xs = [ev[si].elapsed_time(ev[si + 1]) for ev in events]
        stage_ms[s] = sum(xs) / steps
        stage_med[s] = statistics.median(xs)

    # the same work through the entry point callers use: autograd Function, flag cache cleared every step
    qg, kg, vg = (t.detach().requires_grad_(True) for t in (q, k, v))

    def api_step():
        BA.BitfieldUtils.clear_cache()
        if not backward:
            with torch.no_grad():
                return BA.bitfield_attn_func(qg, kg, vg, bf)
        o = BA.bitfield_attn_func(qg, kg, vg, bf)
        return torch.autograd.grad(o, (qg, kg, vg), do)

    for _ in range(min(warmup, 3)):
        api_step()
    torch.cuda.synchronize()
    api_ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(steps)]
    t0 = time.perf_counter()
    for a, b in api_ev:
        a.record()
        api_step()
        b.record()
    torch.cuda.synchronize()
    api_wall = time.perf_counter() - t0
    api_times = [a.elapsed_time(b) for a, b in api_ev]

    BA.BitfieldUtils.clear_cache()
    flags = BA.BitfieldUtils.materialize_compressed_mask_from_bitfield_mask(bf)
    the_plan = BA.BitfieldUtils.plan_for(flags, bf)
    issued = issued_flops(flags, the_plan, w, handover[0])
    ds_bytes = the_plan.ds_pairs() * w.Hq * 8192 if (handover[0] and the_plan is not None) else 0
    BA.BitfieldUtils.clear_cache()
    return {
        "w": w, "pairs": pairs, "f_fwd": f_fwd, "f_bwd": f_bwd, "handover": handover[0], "ds_workspace_bytes": ds_bytes,
        "ms_per_step": ms_per_step, "median_ms_per_step": statistics.median(per_step),
        "stage_ms": stage_ms, "stage_median_ms": stage_med,
        "api_ms_per_step": api_wall * 1e3 / steps, "api_median_ms_per_step": statistics.median(api_times),
        "issued": issued,
    }


def run_neighbouring_entry_points(dev, steps):
    """C2-shaped records for the entry points either side of plain bitfield attention, forward + backward each:
    a context-parallel shard (index tensors: rank 0 of a two-rank zigzag split, 4096 rows against all 8192 keys,
    through `_bitfield_attn_forward` / `_bitfield_attn_backward`), the materialized C2 mask through `flash_attn_func`,
    and an ALiBi-like bias vector through `bitfield_attn_func`.  Effective TFLOP/s over each case's unmasked pairs.
    Last, the single-token decode step (HBM-bound: rate at which the key / value cache is read)."""
    import torch

    from cornstarch_amd import workloads as W
    from cornstarch_amd.kernel import attention as A
    from cornstarch_amd.kernel import bitfield_attention as BA
    from oracle import bam_oracle as O  # pair counts only (setup, untimed)

    w = W.WORKLOADS["C2"]
    q, k, v, do = (t.to(dev) for t in W.make_tensors("C2"))
    bf = W.make_bitfields("C2").to(dev)
    per_pair = 14 * w.D * w.Hq

    def timed(fn):
        for _ in range(3):
            fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            fn()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) * 1e3 / steps

    def issued_ratio(plan, pairs, handover):
        nz = plan.fine_classes() > 0
        if nz.shape[-1] % 2:
            nz = torch.nn.functional.pad(nz, (0, 1))
        t64, t32 = int((nz[..., 0::2] | nz[..., 1::2]).sum()), int(nz.sum())
        issued = 4 * t64 * 2048 + 8 * t32 * 1024 + (2 * t32 * 1024 if handover else 6 * t64 * 2048)
        return round(issued / ((14 if handover else 18) * pairs), 4)

    out = {}
    # --- context-parallel shard
    chunks = torch.arange(w.S, device=dev).chunk(4)
    idx_q = torch.cat([chunks[0], chunks[3]])
    idx_k = torch.cat([chunks[0], chunks[3], chunks[1], chunks[2]])
    pairs = sum(int(O.allow_rows(bf[0], r0, min(r0 + 1024, idx_q.numel()), idx_q, idx_k).sum())
                for r0 in range(0, idx_q.numel(), 1024))
    ql, dol = q[:, idx_q].contiguous(), do[:, idx_q].contiguous()
    kl, vl = k[:, idx_k].contiguous(), v[:, idx_k].contiguous()
    BA.BitfieldUtils.clear_cache()
    glob = BA.BitfieldUtils.materialize_compressed_mask_from_bitfield_mask(bf)
    # the caller's recipe for the shard's 128 x 32 flags (reference shardformer/layers/utils.py:331-353)
    flags = glob[:, idx_q[::128] // 128][:, :, idx_k[::32] // 32].contiguous()
    grads = [torch.zeros_like(t, dtype=torch.float32) for t in (ql, kl, vl)]

    def shard_step():
        o, lse, sc = BA._bitfield_attn_forward(ql, kl, vl, bf, flags, idx_q, idx_k)
        BA._bitfield_attn_backward(dol, ql, kl, vl, o, bf, flags, lse, *grads, offsets_q=idx_q, offsets_k=idx_k, softmax_scale=sc)

    ms = timed(shard_step)
    view = BA._IndexView.get(bf, idx_q, idx_k)
    out["index_tensors_zigzag_rank0"] = {
        "ms_per_step": round(ms, 4), "tflops": round(per_pair * pairs / (ms * 1e-3) / 1e12, 3), "unmasked_pairs": pairs,
        "issued_over_unmasked": issued_ratio(view.plan, pairs, True), "steps": steps,
    }
    BA.BitfieldUtils.clear_cache()
    # --- materialized mask
    mask = BA.materialize_bitfield_mask(bf)
    pairs = int(mask.sum())
    qg, kg, vg = (t.detach().requires_grad_(True) for t in (q, k, v))

    def mask_step():
        A._MaskPlan.forget()  # flags and plan of the mask are rebuilt every step, like the bitfield flags in the headline
        o = A.flash_attn_func(qg, kg, vg, mask=mask)
        torch.autograd.grad(o, (qg, kg, vg), do)

    ms = timed(mask_step)
    _, mplan = A._MaskPlan.get(mask, w.B, w.S, w.S, dev)
    out["materialized_mask"] = {
        "ms_per_step": round(ms, 4), "tflops": round(per_pair * pairs / (ms * 1e-3) / 1e12, 3), "unmasked_pairs": pairs,
        "issued_over_unmasked": issued_ratio(mplan, pairs, True), "steps": steps,
    }
    A._MaskPlan.forget()
    del mask
    # --- bias vector
    slopes = torch.tensor([2.0 ** (-8.0 * (i + 1) / w.Hq) for i in range(w.Hq)], device=dev)
    bias = (-torch.arange(w.S, device=dev, dtype=torch.float32))[None, None, None, :] * slopes[None, :, None, None] * 1e-3

    def bias_step():
        BA.BitfieldUtils.clear_cache()
        o = BA.bitfield_attn_func(qg, kg, vg, bf, bias)
        torch.autograd.grad(o, (qg, kg, vg), do)

    ms = timed(bias_step)
    out["alibi_bias_vector"] = {
        "ms_per_step": round(ms, 4), "tflops": round(per_pair * pairs / (ms * 1e-3) / 1e12, 3), "unmasked_pairs": pairs,
        "steps": steps,
    }
    BA.BitfieldUtils.clear_cache()
    del qg, kg, vg, bias
    # --- single-token decode step of the HF adapter (eval mode): 8 sequences, a cache of C2's length and head layout
    from cornstarch_amd.kernel import interface as I

    Bd = 8
    qd = torch.randn(Bd, w.Hq, 1, w.D, device=dev, dtype=torch.bfloat16)
    kd = torch.randn(Bd, w.Hkv, w.S, w.D, device=dev, dtype=torch.bfloat16)
    vd = torch.randn(Bd, w.Hkv, w.S, w.D, device=dev, dtype=torch.bfloat16)
    ms = timed(lambda: I._decode_attention(qd, kd, vd, None, 0.0, None, None))
    cache_bytes = 2 * Bd * w.S * w.Hkv * w.D * 2
    out["decode_step"] = {
        "ms_per_step": round(ms, 4), "batch": Bd, "cache_len": w.S, "cache_gbytes_per_s": round(cache_bytes / (ms * 1e-3) / 1e9, 1),
        "hbm_frac": round(cache_bytes / (ms * 1e-3) / 1e9 / PEAK_HBM_GBPS, 4), "steps": steps,
    }
    return out


def main():
    args = parse()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)", file=sys.stderr)
        sys.exit(2)

    import torch

    assert torch.cuda.is_available(), "bench.py needs the GPU"
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    name = args.workload
    r = run_workload(name, args.steps, args.warmup, dev)
    w, pairs, f_fwd, f_bwd = r["w"], r["pairs"], r["f_fwd"], r["f_bwd"]
    stage_ms, ms_per_step = r["stage_ms"], r["ms_per_step"]

    if args.copy_calibration:
        src = torch.empty(1 << 28, dtype=torch.float32, device=dev).normal_()
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    fwd_ms = stage_ms["flags"] + stage_ms["fwd"]
    bwd_ms = stage_ms["alloc"] + stage_ms["delta"] + stage_ms["dkdv"] + stage_ms["dq"]

    # Per kernel: algorithmic FLOPs (5-GEMM accounting of the backward: the dK/dV kernel owns S, dP, dV, dK; the dQ
    # kernel owns dQ) and algorithmic HBM bytes (every operand and result once; with the dS hand-over the workspace
    # is written once by dK/dV and read once by dQ).
    esz = 2
    t_q, t_kv, t_row = w.B * w.S * w.Hq * w.D * esz, w.B * w.S * w.Hkv * w.D * esz, w.B * w.Hq * w.S * 4
    ds_bytes = r["ds_workspace_bytes"]
    algo = {"fwd": f_fwd, "dkdv": 8 * w.D * w.Hq * pairs, "dq": 2 * w.D * w.Hq * pairs}
    algo_bytes = {
        "fwd": 2 * t_q + 2 * t_kv + t_row,
        "dkdv": 2 * t_q + 4 * t_kv + 2 * t_row + ds_bytes,
        "dq": (ds_bytes + t_kv + t_q) if r["handover"] else (3 * t_q + 2 * t_kv + 2 * t_row),
    }
    kname = {"fwd": "fwd_kernel", "dkdv": "bwd_dkdv_kernel", "dq": "bwd_dq_saved_kernel" if r["handover"] else "bwd_dq_kernel"}
    kernels = {}
    for s_ in algo:
        sec = stage_ms[s_] * 1e-3
        kernels[kname[s_]] = {
            "avg_launch_ms": round(stage_ms[s_], 4),
            "algorithmic_tflops": round(algo[s_] / sec / 1e12, 3),
            "mfma_frac": round(algo[s_] / sec / 1e12 / PEAK_BF16_DENSE_TFLOPS, 4),
            "algorithmic_gbytes_per_s": round(algo_bytes[s_] / sec / 1e9, 1),
            "hbm_frac": round(algo_bytes[s_] / sec / 1e9 / PEAK_HBM_GBPS, 4),
            "issued_tflops": round(r["issued"][s_] / sec / 1e12, 3),
        }
    dom = max(algo, key=lambda s_: stage_ms[s_])
    dk = kernels[kname[dom]]
    # the roof the dominant kernel sits closer to, by its own measured fractions
    bound = "mfma" if dk["mfma_frac"] >= dk["hbm_frac"] else "hbm"
    traffic = measured_traffic(name, kname[dom])

    value = (f_fwd + f_bwd) / (ms_per_step * 1e-3) / 1e12
    dq_gemms = 2 if r["handover"] else 6
    result = {
        "metric": "bitfield attention fwd+bwd effective TFLOP/s over unmasked pairs (S=8192 GQA bf16)"
        if name == "C2"
        else f"bitfield attention fwd+bwd effective TFLOP/s over unmasked pairs ({name})",
        "value": round(value, 3),
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {
            "workload": f"{name}: B={w.B} S={w.S} Hq={w.Hq} Hkv={w.Hkv} D={w.D} bf16 "
                        f"{'fwd+bwd' if w.backward else 'forward only'}, {w.description}",
            "unmasked_pairs": pairs,
            "flops_fwd": f_fwd,
            "flops_bwd": f_bwd,
        },
        "median_ms_per_step": round(r["median_ms_per_step"], 4),
        "api_ms_per_step": round(r["api_ms_per_step"], 4),
        "api_median_ms_per_step": round(r["api_median_ms_per_step"], 4),
        "fwd_ms": round(fwd_ms, 4),
        "bwd_ms": round(bwd_ms, 4),
        "fwd_tflops": round(f_fwd / (fwd_ms * 1e-3) / 1e12, 3),
        "mfma_util_unmasked": round(value / PEAK_BF16_DENSE_TFLOPS, 4),
        "stage_ms": {s_: round(x, 4) for s_, x in stage_ms.items()},
        "stage_median_ms": {s_: round(x, 4) for s_, x in r["stage_median_ms"].items()},
        # backward decomposition in use: with the hand-over the dK/dV kernel stores its dS blocks (8 KiB per q head and
        # (32-row slice, 128-key tile) pair) and the dQ kernel is one GEMM over them; without, dQ recomputes S and dP
        "ds_handover": r["handover"],
        "ds_workspace_bytes": ds_bytes,
        # MFMA FLOPs issued according to the tile lists, and their ratio to the algorithmic (unmasked-pair) FLOPs of
        # the GEMMs each kernel runs (forward 2, dK/dV 4, dQ 1 with the hand-over, 3 without)
        "issued_mfma_flops": r["issued"],
        "issued_over_unmasked": {
            "fwd": round(r["issued"]["fwd"] / f_fwd, 4),
            "dkdv": round(r["issued"]["dkdv"] / (8 * w.D * w.Hq * pairs), 4),
            "dq": round(r["issued"]["dq"] / (dq_gemms * w.D * w.Hq * pairs), 4),
        },
        "kernels": kernels,
        # the library's bf16 GEMM on this very box, same process: what a pure MFMA kernel sustains here
        "library_gemm_tflops": library_gemm_tflops(dev),
        "roofline": {
            "kernel": kname[dom],
            "bound": bound,
            "achieved": dk["algorithmic_tflops"] if bound == "mfma" else dk["algorithmic_gbytes_per_s"],
            "peak": PEAK_BF16_DENSE_TFLOPS if bound == "mfma" else PEAK_HBM_GBPS,
            "unit": "TFLOP/s" if bound == "mfma" else "GB/s",
            "frac": dk["mfma_frac"] if bound == "mfma" else dk["hbm_frac"],
            "traffic": traffic,
            "traffic_source": "profiles/hbm_traffic.txt (rocprofv3 --pmc run of this command on another box)"
            if traffic is not None else None,
            "avg_launch_ms": dk["avg_launch_ms"],
            "issued_tflops": dk["issued_tflops"],
        },
    }
    if name == "C2" and not args.no_other_workloads:
        others = {}
        for other in ("C3", "C4", "C5"):
            torch.cuda.empty_cache()
            # short steps get more repetitions: with a handful of them the start of the queue dominates the wall time
            other_steps = args.other_steps * {"C3": 2, "C4": 4}.get(other, 1)
            ro = run_workload(other, other_steps, 3, dev)
            tot = ro["f_fwd"] + ro["f_bwd"]
            others[other] = {
                "ms_per_step": round(ro["ms_per_step"], 4),
                "api_ms_per_step": round(ro["api_ms_per_step"], 4),
                "tflops": round(tot / (ro["ms_per_step"] * 1e-3) / 1e12, 3),
                "steps": other_steps,
                "unmasked_pairs": ro["pairs"],
                "stage_ms": {s: round(x, 4) for s, x in ro["stage_ms"].items()},
                "ds_handover": ro["handover"],
                "issued_over_unmasked": round(sum(ro["issued"].values()) /
                                              ((14 if ro["handover"] else 18) * ro["w"].D * ro["w"].Hq * ro["pairs"]), 4),
            }
        result["other_workloads"] = others
        result["neighbouring_entry_points"] = run_neighbouring_entry_points(dev, args.other_steps * 2)
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(name)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
