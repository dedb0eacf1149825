#!/usr/bin/env python3
"""Headline benchmark: bf16 causal attention forward + recompute backward at
B=4, H=16, T=4096, head_dim=128 on ONE MI355X, through the C ABI.

A "step" is one forward (O + LSE) plus one backward (dQ, dK, dV) over one
batch of synthetic inputs already resident in HBM. Prints ONE JSON line.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu-baseline]

Work model (same for every rate printed here): FLOPs = 14 * dk * pairs * B*Hq
(forward 2 GEMMs = 4*dk*pairs, backward 5 GEMMs = 10*dk*pairs; masked tiles
and recomputation earn nothing), pairs = T(T+1)/2 for causal. Bytes = one
read of Q,K,V + one write of O,LSE (forward) + one read of Q,K,V,O,dO,LSE and
one write of dQ,dK,dV (backward).
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2500.0  # MI355X dense bf16 MFMA, published
PEAK_HBM_GBS = 8000.0      # MI355X HBM3E, published
PEAK_FP32_TFLOPS = 157.3   # MI355X dense fp32 MFMA, published

PMC_SUMMARY = os.path.join(ROOT, "profiles", "attn_fwd_bwd_causal_B4_H16_T4096_d128_pmc.txt")
PMC_SUMMARY_WINDOW = os.path.join(ROOT, "profiles", "attn_fwd_bwd_window256_sinks4_B4_H16_T4096_d128_pmc.txt")
TRAFFIC_SOURCE = ("rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE of this kernel as committed under profiles/ (a constant read "
                  "from that summary, not a measurement of this run)")


def measured_traffic_bytes(path=PMC_SUMMARY):
    """HBM bytes per launch of each kernel of a workload, read from the committed summary of the two `rocprofv3 --pmc`
    runs (FETCH_SIZE, WRITE_SIZE, each scaled by what the same counter reads for a copy kernel of known size; the
    factors are stated in that file). Returns {} when the summary is missing: traffic is then reported as null."""
    import re
    out, kernel = {}, None
    try:
        for line in open(path):
            m = re.match(r"(mfma_\w+)<", line)
            if m:
                kernel = {"mfma_fwd": "fwd", "mfma_dq": "dq", "mfma_dq3": "dq", "mfma_dkdv2": "dkdv",
                          "mfma_dkdv3": "dkdv"}.get(m.group(1))
            m = re.search(r"HBM traffic per launch: .* total ([0-9.]+) MB", line)
            if m and kernel:
                out[kernel] = float(m.group(1)) * 1e6
    except OSError:
        pass
    return out


def cpu_baseline(B, T, H, dk, scale):
    """The reference's CPU attention (ops.cpp path) on two of the (batch, head) units of
    the same workload, single thread, timed with a wall clock; the rate is
    FLOPs-per-unit / time, so it compares with `value` directly."""
    import numpy as np
    from oracle.bindings import Oracle, load_reference
    from paperkiln_amd import synth

    units = 2  # about 8 s each on one core
    flops_unit = 14.0 * dk * (T * (T + 1) // 2)
    # The reference's GEMM announces its SIMD level on stdout when the library is loaded; this script's
    # stdout carries exactly one JSON line, so file descriptor 1 points at stderr while the CPU leg runs.
    sys.stdout.flush()
    saved_stdout = os.dup(1)
    os.dup2(2, 1)
    try:
        ref = load_reference()
        orc = None if ref is not None else Oracle()
        kind = "reference" if ref is not None else "port"
        dt = _cpu_units(units, ref, orc, T, dk, scale, synth)
    finally:
        import ctypes
        ctypes.CDLL(None).fflush(None)  # the C library's own stdout buffer, before descriptor 1 goes back
        sys.stdout.flush()
        os.dup2(saved_stdout, 1)
        os.close(saved_stdout)
    cpu = "unknown"
    try:
        for line in open("/proc/cpuinfo"):
            if line.startswith("model name"):
                cpu = line.split(":", 1)[1].strip()
                break
    except OSError:
        pass
    return {"value": units * flops_unit / dt / 1e12, "unit": "TFLOP/s", "cores": 1, "kind": kind,
            "sample": f"{units} of {B * H} (batch, head) units of the same workload, fwd+bwd, {dt:.2f} s wall; "
                      f"whole job would take ~{dt / units * B * H:.0f} s on one core",
            "host_cpu": cpu, "host_nproc": os.cpu_count()}


def _cpu_units(units, ref, orc, T, dk, scale, synth):
    dt = 0.0
    for u in range(units):
        q = synth.bf16_round(synth.randn(11 + 10 * u, (T, dk), 0.5))
        k = synth.bf16_round(synth.randn(12 + 10 * u, (T, dk), 0.5))
        v = synth.bf16_round(synth.randn(13 + 10 * u, (T, dk), 0.5))
        g = synth.bf16_round(synth.randn(14 + 10 * u, (T, dk), 1.0))
        t0 = time.perf_counter()
        if ref is not None:
            ref.fused_attention(q, k, v, scale, 0, True, dy=g)
        else:
            _, _, A = orc.head_fwd(q, k, v, scale, 0, True, 0, 0)
            orc.head_bwd(q, k, v, A, g, scale, 0, True, 0, 0)
        dt += time.perf_counter() - t0
    return dt


def window_variant(ops, q, k, v, d_o, out, scale, B, H, T, dk, warmup, steps):
    """Same shape, window=256 + 4 sink keys (BASELINE config 4b): 12% of the causal pairs are live, every
    byte still moves once, so this one is priced against the HBM roofline."""
    import torch
    from paperkiln_amd import synth
    W, S = 256, 4

    def step():
        o, lse = ops.attn_fwd(q, k, v, scale, True, W, S)
        ops.attn_bwd(q, k, v, o, lse, d_o, scale, True, W, S, out=out)

    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) / steps * 1e3
    pairs = synth.visible_pairs(T, True, W, S)
    nbytes = 12.0 * B * T * H * dk * 2 + 2.0 * B * H * T * 4
    traffic = measured_traffic_bytes(PMC_SUMMARY_WINDOW)  # the three kernels of one step together
    return {"workload": "same shape, window=256, sinks=4", "ms_per_step": round(ms, 4),
            "tflops": round(14.0 * dk * pairs * B * H / (ms * 1e-3) / 1e12, 2),
            "roofline": {"bound": "hbm", "achieved": round(nbytes / (ms * 1e-3) / 1e9, 1), "peak": PEAK_HBM_GBS,
                         "unit": "GB/s", "frac": round(nbytes / (ms * 1e-3) / 1e9 / PEAK_HBM_GBS, 4),
                         "algorithmic_bytes": nbytes,
                         "traffic": sum(traffic.values()) if len(traffic) == 3 else None,
                         "traffic_source": TRAFFIC_SOURCE}}


def other_config(ops, name, B, Hq, Hkv, T, dk, theta, bound, steps=400, warmup=50):
    """BASELINE configs 2 and 3 at their full shapes (bf16, causal, RoPE pre-applied to Q and K on the host in
    fp32 before rounding): forward + backward in one loop, with per-kernel HIP events on every 8th step."""
    import numpy as np
    import torch
    from paperkiln_amd import synth
    dev = torch.device("cuda:0")
    scale = float(np.float32(1.0 / np.sqrt(dk)))
    q = synth.bf16_round(synth.rope_interleaved(synth.randn(21, (B, T, Hq, dk)), theta))
    k = synth.bf16_round(synth.rope_interleaved(synth.randn(22, (B, T, Hkv, dk)), theta))
    v = synth.bf16_round(synth.randn(23, (B, T, Hkv, dk)))
    g = synth.bf16_round(synth.randn(24, (B, T, Hq, dk)))
    q, k, v, g = (torch.from_numpy(x).to(dev).bfloat16() for x in (q, k, v, g))
    out = (torch.empty_like(q), torch.empty_like(k), torch.empty_like(v),
           torch.empty(max(ops.bwd_workspace_bytes(q, k), 16), dtype=torch.uint8, device=dev))

    def step(events=None):
        def mark(nm):
            if events is not None:
                e = torch.cuda.Event(enable_timing=True)
                e.record()
                events.append((nm, e))
        mark("start")
        o, lse = ops.attn_fwd(q, k, v, scale, True)
        mark("fwd")
        ops.attn_bwd(q, k, v, o, lse, g, scale, True, out=out)
        mark("bwd")

    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    evs = []
    t0 = time.perf_counter()
    for i in range(steps):
        if i % 8 == 0:
            ev = []
            step(ev)
            evs.append(ev)
        else:
            step()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) / steps * 1e3
    kern = {}
    for ev in evs:
        for (_, e0), (nm, e1) in zip(ev[:-1], ev[1:]):
            kern[nm] = kern.get(nm, 0.0) + e0.elapsed_time(e1) / len(evs)
    pairs = synth.visible_pairs(T, True, 0, 0)
    flops = 14.0 * dk * pairs * B * Hq
    nbytes = (6.0 * Hq + 6.0 * Hkv) * B * T * dk * 2 + 2.0 * B * Hq * T * 4
    tf, gbs = flops / (ms * 1e-3) / 1e12, nbytes / (ms * 1e-3) / 1e9
    roof = ({"bound": "mfma", "achieved": round(tf, 2), "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
             "frac": round(tf / PEAK_BF16_TFLOPS, 4)} if bound == "mfma" else
            {"bound": "hbm", "achieved": round(gbs, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
             "frac": round(gbs / PEAK_HBM_GBS, 4)})
    return {"workload": name, "steps": steps, "ms_per_step": round(ms, 4), "tflops": round(tf, 2),
            "hbm_gb_per_s_algorithmic": round(gbs, 1), "tokens_per_s": round(B * T / (ms * 1e-3), 1),
            "kernel_ms": {n: round(t, 4) for n, t in kern.items()}, "roofline": roof}


def fp32_variant(ops, q, k, v, d_o, scale, B, H, T, dk):
    """Same shape with fp32 tensors (the reference's own element type): the kernels built on the fp32
    matrix instruction, priced against the fp32 MFMA peak."""
    import torch
    from paperkiln_amd import synth
    q, k, v, d_o = (x.float() for x in (q, k, v, d_o))
    out = (torch.empty_like(q), torch.empty_like(k), torch.empty_like(v),
           torch.empty(ops.bwd_workspace_bytes(q, k), dtype=torch.uint8, device=q.device))

    def step():
        o, lse = ops.attn_fwd(q, k, v, scale, True)
        ops.attn_bwd(q, k, v, o, lse, d_o, scale, True, out=out)

    warmup, steps = 3, 10
    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) / steps * 1e3
    tf = 14.0 * dk * synth.visible_pairs(T, True, 0, 0) * B * H / (ms * 1e-3) / 1e12
    return {"workload": "same shape, fp32 in/out", "steps": steps, "ms_per_step": round(ms, 3), "tflops": round(tf, 2),
            "roofline": {"bound": "mfma", "achieved": round(tf, 2), "peak": PEAK_FP32_TFLOPS, "unit": "TFLOP/s",
                         "frac": round(tf / PEAK_FP32_TFLOPS, 4)}}


def llama_step():
    """Activation-checkpointed Llama training step (BASELINE config 5): 6 layers, d=512, 8 heads, SwiGLU 1376,
    vocab 32000 tied, B=8 x T=1024 tokens, bf16 compute with fp32 master weights. Reports tokens/s, the loss
    with and without per-block checkpointing, and the allocator's peak activation bytes for both."""
    from paperkiln_amd import synth
    from paperkiln_amd.llama import Llama
    cfg = dict(vocab=32000, d=512, n_layers=6, n_heads=8, d_ff=1376)
    B, T = 8, 1024
    m = Llama(compute_dtype="bf16", seed=0, **cfg)
    toks = synth.randint(9, B * T + 1, cfg["vocab"])
    x, y = toks[:-1], toks[1:]
    out = {"workload": "Llama L6 d512 H8 d_ff1376 V32000 tied, B=8 T=1024, bf16 compute / fp32 master, fwd+bwd+AdamW",
           "params": m.parameter_count()}
    for ck in (False, True):
        for _ in range(2):
            m.loss_backward(x, y, T, checkpoint=ck)
        t0 = time.perf_counter()
        n = 3
        for _ in range(n):
            loss, st = m.loss_backward(x, y, T, checkpoint=ck)
        dt = (time.perf_counter() - t0) / n
        tag = "checkpointed" if ck else "plain"
        out[tag] = {"loss": round(loss, 6), "ms_fwd_bwd": round(dt * 1e3, 2), "tokens_per_s_fwd_bwd": round(B * T / dt, 0),
                    "peak_activation_bytes": st["peak_activation_bytes"],
                    "activation_bytes_after_forward": st["activation_bytes_after_forward"],
                    "live_vars_after_forward": st["live_vars_after_forward"]}
    m.adamw_step(1e-3, max_norm=1.0)  # the first step also allocates the moments
    t0 = time.perf_counter()
    for _ in range(3):
        m.adamw_step(1e-3, max_norm=1.0)
    out["ms_clip_adamw"] = round((time.perf_counter() - t0) / 3 * 1e3, 2)
    out["loss_abs_diff"] = abs(out["plain"]["loss"] - out["checkpointed"]["loss"])
    out["peak_activation_ratio"] = round(out["plain"]["peak_activation_bytes"] / out["checkpointed"]["peak_activation_bytes"], 2)
    # the whole training step as it repeats: forward + backward with checkpointing, clip, AdamW, and the refresh of the
    # bf16 weight copies that every optimiser step makes necessary
    for _ in range(2):
        m.loss_backward(x, y, T, checkpoint=True)
        m.adamw_step(1e-3, max_norm=1.0)
    t0 = time.perf_counter()
    for _ in range(3):
        m.loss_backward(x, y, T, checkpoint=True)
        m.adamw_step(1e-3, max_norm=1.0)
    full = (time.perf_counter() - t0) / 3
    out["ms_step_checkpointed"] = round(full * 1e3, 2)
    out["tokens_per_s_step_checkpointed"] = round(B * T / full, 0)
    m.close()
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    # the card leaves its idle clock state only under sustained load: a short warm-up would time the ramp
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--event-every", type=int, default=8,
                    help="steps of the timed region that carry per-kernel HIP events: every N-th (each event "
                         "costs a few microseconds on the stream, so instrumenting every step slows the job)")
    ap.add_argument("--preheat-ms", type=float, default=500.0,
                    help="untimed run of the same step for this long before the counted warm-up: the card leaves its "
                         "idle clock state only under sustained load, and --warmup counts steps, not time")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--sections", default="window,cfg2,cfg3,fp32,llama",
                    help="extra measurements beside the headline: any of window,cfg2,cfg3,fp32,llama (empty = headline only, "
                         "which is what the profiles under profiles/ were taken with)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on ONE GPU (one process, one MI355X); --gpus must be 1. "
                 "Each (batch, KV-head group) is an independent unit, so N GPUs would each take B*Hkv/N of them.")

    import numpy as np
    import torch
    from paperkiln_amd import _lib, ops, synth

    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible; paperkiln_amd has no CPU path")
    _lib.check(_lib.lib().pk_init(0, None, 0))
    dev = torch.device("cuda:0")

    B, H, T, dk = 4, 16, 4096, 128
    scale = float(np.float32(1.0 / np.sqrt(dk)))
    gen = torch.Generator(device=dev).manual_seed(4)
    q = (torch.randn((B, T, H, dk), generator=gen, device=dev) * 0.5).bfloat16()
    k = (torch.randn((B, T, H, dk), generator=gen, device=dev) * 0.5).bfloat16()
    v = (torch.randn((B, T, H, dk), generator=gen, device=dev) * 0.5).bfloat16()
    d_o = torch.randn((B, T, H, dk), generator=gen, device=dev).bfloat16()
    # outputs and scratch are allocated once; the timed region allocates nothing but O/LSE views
    dq, dkk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    ws = torch.empty(max(ops.bwd_workspace_bytes(q, k), ops.bwd_workspace_bytes(q, k, window=256, sinks=4)),
                     dtype=torch.uint8, device=dev)
    out = (dq, dkk, dv, ws)

    pairs = synth.visible_pairs(T, True, 0, 0)
    unit = dk * pairs * B * H
    flops_step = 14.0 * unit
    bytes_step = 12.0 * B * T * H * dk * 2 + 2.0 * B * H * T * 4
    # algorithmic work per launch: forward = S and PV; dkdv = S, dP, dV, dK; dq = dQ only
    # (its S and dP are recomputation and earn nothing; it also forms delta = rowsum(O .* dO)).
    alg_flops = {"fwd": 4.0 * unit, "dkdv": 8.0 * unit, "dq": 2.0 * unit}

    def step(events=None):
        def mark(name):
            if events is not None:
                e = torch.cuda.Event(enable_timing=True)
                e.record()
                events.append((name, e))
        mark("start")
        o, lse = ops.attn_fwd(q, k, v, scale, True)
        mark("fwd")
        # the backward as one call launches exactly these two kernels in this order; it is split
        # here only so that an event can sit between them
        ops.attn_bwd(q, k, v, o, lse, d_o, scale, True, out=out, stages=ops.BWD_DELTA | ops.BWD_DQ)
        mark("dq")
        ops.attn_bwd(q, k, v, o, lse, d_o, scale, True, out=out, stages=ops.BWD_DKDV)
        mark("dkdv")

    t_pre = time.perf_counter()
    while (time.perf_counter() - t_pre) * 1e3 < args.preheat_ms:
        for _ in range(10):
            step()
        torch.cuda.synchronize()
    preheat_ms = (time.perf_counter() - t_pre) * 1e3
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    all_events = []
    # per-kernel events on at least 8 steps of the timed region, whatever --steps is (spread evenly)
    every = max(1, min(args.event_every, args.steps // 8))
    t0 = time.perf_counter()
    for i in range(args.steps):
        if i % every == 0:
            ev = []
            step(ev)
            all_events.append(ev)
        else:
            step()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0

    ms_per_step = dt / args.steps * 1e3
    kern_ms = {}
    for ev in all_events:
        for (_, e0), (name, e1) in zip(ev[:-1], ev[1:]):
            kern_ms[name] = kern_ms.get(name, 0.0) + e0.elapsed_time(e1)
    kern_ms = {n: t / len(all_events) for n, t in kern_ms.items()}
    dominant = max(alg_flops, key=lambda n: kern_ms[n])
    achieved = alg_flops[dominant] / (kern_ms[dominant] * 1e-3) / 1e12
    value = flops_step / (ms_per_step * 1e-3) / 1e12

    res = {
        "metric": "causal attn fwd+bwd TFLOP/s (% bf16 MFMA peak) at T=4096; peak activation bytes",
        "value": round(value, 2), "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "preheat_ms": round(preheat_ms, 1), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "causal attention fwd + recompute bwd, B=4 H=16 T=4096 head_dim=128, bf16 in/out, "
                               "fp32 accumulate (BASELINE config 4, full causal)", "B": B, "H": H, "T": T,
                   "head_dim": dk, "causal": True},
        "pct_of_bf16_mfma_peak": round(100.0 * value / PEAK_BF16_TFLOPS, 2),
        "tokens_per_s": round(B * T / (ms_per_step * 1e-3), 1),
        "hbm_gb_per_s_algorithmic": round(bytes_step / (ms_per_step * 1e-3) / 1e9, 1),
        "kernel_ms": {n: round(t, 4) for n, t in kern_ms.items()}, "kernel_event_steps": len(all_events),
        "roofline": {"bound": "mfma", "kernel": dominant, "achieved": round(achieved, 2), "peak": PEAK_BF16_TFLOPS,
                     "unit": "TFLOP/s", "frac": round(achieved / PEAK_BF16_TFLOPS, 4),
                     "traffic": measured_traffic_bytes().get(dominant),
                     "traffic_source": TRAFFIC_SOURCE},
    }
    extras = [x for x in args.sections.split(",") if x]
    if "window" in extras:
        res["window_variant"] = window_variant(ops, q, k, v, d_o, out, scale, B, H, T, dk, args.warmup,
                                               max(args.steps // 2, 1))
    if "cfg2" in extras:
        # 15.1 GFLOP against 101 MB: about 6 us of matrix work and 13 us of HBM time at peak, so the HBM roofline
        res["cfg2"] = other_config(ops, "BASELINE config 2: causal MHA B=16 H=8 T=512 head_dim=64, RoPE theta=1e4 "
                                   "pre-applied, bf16", 16, 8, 8, 512, 64, 1e4, "hbm")
    if "cfg3" in extras:
        res["cfg3"] = other_config(ops, "BASELINE config 3: causal GQA B=4 Hq=14 Hkv=2 T=2048 head_dim=64, RoPE "
                                   "theta=1e6 pre-applied, bf16", 4, 14, 2, 2048, 64, 1e6, "mfma")
    if "fp32" in extras:
        res["fp32_variant"] = fp32_variant(ops, q, k, v, d_o, scale, B, H, T, dk)
    if "llama" in extras:
        res["llama_step"] = llama_step()
        # the second half of the metric, lifted to the top level: checkpointed against plain, config 5
        res["peak_activation_bytes"] = {"checkpointed": res["llama_step"]["checkpointed"]["peak_activation_bytes"],
                                        "plain": res["llama_step"]["plain"]["peak_activation_bytes"],
                                        "ratio": res["llama_step"]["peak_activation_ratio"]}
    if not args.no_cpu_baseline:
        res["cpu_baseline"] = cpu_baseline(B, T, H, dk, scale)
    print(json.dumps(res), flush=True)


if __name__ == "__main__":
    main()
