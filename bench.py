#!/usr/bin/env python3
"""Benchmark of the SLA hot path on one MI355X.

A step is one full ``SparseLinearAttention`` forward (block-mask build, block-sparse
attention, linear branch, projection, sum) on the configuration the headline metric is
quoted on: B=1 H=12 L=32760 D=128, BLKQ=BLKK=64, topk=0.05, feature map elu, bf16,
structured synthetic q/k.  Inputs are resident in HBM before the timed region.

Prints one JSON line.  ``value`` is the reference's "effective TFLOPS" convention
(dense-equivalent 4*B*H*L^2*D / time, evaluate/bench_kernel.py:93-94 of the reference);
``roofline`` is the executed MFMA rate of the dominant kernel (block-sparse forward);
``cpu_baseline`` is the CPU oracle on a bounded sample of the same workload.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2500.0     # MI355X dense bf16 MFMA
PEAK_HBM_GBS = 8000.0

PEAK_I8F8_TOPS = 5000.0        # MI355X dense int8 / fp8 MFMA

# HBM bytes per launch of the dominant kernel come from two `rocprofv3 --pmc` runs of this script (FETCH_SIZE, then
# WRITE_SIZE), each scaled by what the same counter reads for the 1 GiB-read / 1 GiB-write elementwise kernel of
# --pmc-calibration.  A plain bench run cannot re-measure them, so the figures live in a small file next to the
# profiler summaries, stamped with a fingerprint of the kernel's sources: when the kernel changes the stamp no
# longer matches and `traffic` is reported as null until the counters have been read again (--record-traffic).
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "sparse_fwd_cfg3_hbm_traffic.json")
KERNEL_SOURCES = ("sla_amd/csrc/sparse_fwd.hip", "sla_amd/csrc/sparse_fwd_pair.h", "sla_amd/csrc/common.h",
                  "sla_amd/csrc/linear_state.h", "sla_amd/csrc/linear_common.h")


def kernel_fingerprint() -> str:
    import hashlib
    h = hashlib.sha256()
    for rel in KERNEL_SOURCES:
        with open(os.path.join(ROOT, rel), "rb") as f:
            h.update(f.read())
    return h.hexdigest()[:16]


def measured_traffic(workload: str):
    """(bytes per launch, note) from the committed counter readings, or (None, why not)."""
    try:
        with open(TRAFFIC_FILE) as f:
            t = json.load(f)
    except (OSError, ValueError):
        return None, "no counter readings recorded"
    if t.get("workload") != workload:
        return None, f"counter readings are for {t.get('workload')}"
    if t.get("kernel_sources_sha256_16") != kernel_fingerprint():
        return None, "the kernel's sources changed after the counters were read"
    return (t["fetch_size_kib"] * 1024 * t["fetch_factor"] + t["write_size_kib"] * 1024 * t["write_factor"],
            "rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, scaled by a copy kernel of known size")


def measured_clock_mhz(workload: str):
    """Shader clock while the dominant kernel runs, from the committed counter readings: GRBM_GUI_ACTIVE (cycles the
    graphics engine was busy during one dispatch, summed over the device's 8 XCDs) / 8 over the dispatch's duration
    in the same profiler run.  None when the readings are missing or older than the kernel's sources."""
    try:
        with open(TRAFFIC_FILE) as f:
            t = json.load(f)
    except (OSError, ValueError):
        return None
    if t.get("workload") != workload or t.get("kernel_sources_sha256_16") != kernel_fingerprint():
        return None
    if not t.get("gui_active_cycles") or not t.get("dispatch_duration_us"):
        return None
    return t["gui_active_cycles"] / 8.0 / t["dispatch_duration_us"]


def record_traffic(values):
    fetch_kib, write_kib, fetch_factor, write_factor = values[:4]
    t = {"workload": "cfg3", "kernel": "sparse_fwd_pair_kernel<FUSED>", "fetch_size_kib": fetch_kib, "write_size_kib": write_kib,
         "fetch_factor": fetch_factor, "write_factor": write_factor, "kernel_sources_sha256_16": kernel_fingerprint(),
         "kernel_sources": list(KERNEL_SOURCES)}
    if len(values) >= 6:
        t["gui_active_cycles"], t["dispatch_duration_us"] = values[4], values[5]
    with open(TRAFFIC_FILE, "w") as f:
        json.dump(t, f, indent=1)
        f.write("\n")


def _events(torch):
    return torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)


def time_region(torch, fn, steps, warmup, preheat_s=0.15):
    """Average milliseconds per call over exactly `steps` calls, on the current stream.

    Before the `warmup` untimed calls the same call is repeated for `preheat_s` seconds (untimed as well):
    the GPU needs that long under load to leave its idle clocks, and a handful of sub-millisecond
    warm-up calls does not get it there.
    """
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < preheat_s:
        for _ in range(10):
            fn()
        torch.cuda.synchronize()
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    e0, e1 = _events(torch)
    e0.record()
    for _ in range(steps):
        fn()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / steps


def _median(xs):
    xs = sorted(xs)
    n = len(xs)
    return xs[n // 2] if n % 2 else 0.5 * (xs[n // 2 - 1] + xs[n // 2])


def time_steps(torch, fn, steps, warmup, preheat_s=0.15, flush=None):
    """Times exactly `steps` calls, one event pair per call, on the current stream; returns their median and mean in ms.

    Without `flush` the calls run back to back (caches warm from the call before, as the reference's README figures
    were not: its script times with triton.testing.do_bench, which clears the L2 between calls).  With `flush`, a
    tensor larger than the L2s and the memory-side cache together, that tensor is overwritten before every call,
    outside the timed pair: every call then starts from cold caches.
    """
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < preheat_s:
        for _ in range(10):
            fn()
        torch.cuda.synchronize()
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    pairs = [_events(torch) for _ in range(steps)]
    for e0, e1 in pairs:
        if flush is not None:
            flush.fill_(0)
        e0.record()
        fn()
        e1.record()
    torch.cuda.synchronize()
    ms = [e0.elapsed_time(e1) for e0, e1 in pairs]
    return _median(ms), sum(ms) / len(ms)


def boundary_margins(torch, dev, path):
    """Writes, per benchmark configuration, how far apart the last selected and the first rejected pooled score of a
    query block lie, in units of the 16-bit format's spacing at that magnitude: a margin of 0 is a tie, which the
    lowest block index decides; small margins are where a different summation order would select another block."""
    from sla_amd import get_block_map
    from sla_amd.block_map import mean_pool
    from sla_amd.inputs import CONFIGS, make_inputs, make_inputs_on_device
    lines = ["# Margin between the last selected and the first rejected pooled score, per query block", "",
             "Written by `python3 bench.py --margins` on the GPU box.  Scores are formed as the mask builder forms them (block means of q",
             "and of the smoothed k in the input dtype, fp32 products, rounded to the input dtype); the margin of a query block is the",
             "T-th largest score of its row minus the (T+1)-th, in units of the dtype's spacing at the T-th score's magnitude.", "",
             "| config | rows | T of N | margin 0 (ties) | 1 | 2-3 | 4-7 | 8-15 | 16-63 | >= 64 |", "|---|---|---|---|---|---|---|---|---|---|"]
    for name in ("cfg1", "cfg2", "cfg3", "cfg4", "cfg5"):
        cfg = CONFIGS[name]
        if cfg.L > 40000:
            q, k, _, _ = make_inputs_on_device(cfg, dev, 4, False)
        else:
            d = make_inputs(cfg)
            q, k = d["q"].to(dev), d["k"].to(dev)
        _, _, T = get_block_map(q, k, cfg.topk, cfg.BLKQ, cfg.BLKK)
        km = k.float().mean(dim=-2, keepdim=True).to(k.dtype)
        pq = mean_pool(q, cfg.BLKQ).float()
        pk = mean_pool((k - km).contiguous(), cfg.BLKK).float()
        s = torch.matmul(pq, pk.transpose(-1, -2)).to(q.dtype)
        N = s.shape[-1]
        if T >= N:
            lines.append(f"| {name} | {s[..., 0].numel()} | {T} of {N} | every block selected | | | | | | |")
            continue
        top = torch.sort(s.float(), dim=-1, descending=True).values
        a, b_ = top[..., T - 1], top[..., T]
        mant = 8 if q.dtype == torch.bfloat16 else (11 if q.dtype == torch.float16 else 24)
        ulp = torch.exp2(torch.floor(torch.log2(a.abs().clamp_min(1e-30))) - (mant - 1))
        mg = torch.round((a - b_) / ulp).flatten()
        edges = [0, 1, 2, 4, 8, 16, 64]
        counts = [int(((mg >= lo) & (mg < hi)).sum()) for lo, hi in zip(edges, edges[1:] + [float("inf")])]
        lines.append(f"| {name} | {mg.numel()} | {T} of {N} | " + " | ".join(str(c) for c in counts) + " |")
        del q, k, s, top
    with open(path, "w") as f:
        f.write("\n".join(lines) + "\n")


def cpu_baseline(cfg, heads, torch):
    """Oracle module forward on `heads` heads of the workload, all host threads."""
    from oracle import sla_oracle as O
    from sla_amd.inputs import make_inputs, make_proj
    cores = min(os.cpu_count() or 1, 16)
    torch.set_num_threads(cores)
    d = make_inputs(cfg, H=heads)
    w, b = make_proj(cfg.D)
    t0 = time.perf_counter()
    O.sla_forward(d["q"], d["k"], d["v"], w, b, cfg.topk, cfg.feature_map, cfg.BLKQ, cfg.BLKK)
    dt = time.perf_counter() - t0
    eff = 4.0 * cfg.B * heads * cfg.L * cfg.L * cfg.D / dt / 1e12
    return {"value": eff, "unit": "TFLOP/s (dense-equivalent)", "cores": cores, "kind": "port",
            "sample": f"{heads} of {cfg.H} heads of the same workload, full module forward in the eager CPU oracle, "
                      f"{dt:.2f} s wall", "ms_per_step_scaled_to_all_heads": dt * 1e3 * cfg.H / heads}


def other_configs(torch, dev, steps):
    """The figures of the other benchmark configurations (a handful of steps each, inputs generated on the device):
    the quantised forward on cfg5, forward and forward + backward on cfg4, the sparse backward alone on cfg3, and
    the reference-convention kernel benchmark (evaluate/bench_kernel.py)."""
    import dataclasses
    import importlib.util
    from sla_amd import SageSparseLinearAttention, SparseLinearAttention, get_block_map
    from sla_amd.inputs import CONFIGS, make_inputs_on_device, make_proj
    from sla_amd.sage import sage_attn_fwd, sage_prepare, quant_v
    from sla_amd.sparse_attn import sparse_attn_bwd, sparse_attn_fwd
    ex = {}
    w, b = make_proj(128)

    def seeded(mod):
        with torch.no_grad():
            mod.proj_l.weight.copy_(w)
            mod.proj_l.bias.copy_(b)
        return mod

    # ---- cfg3: sparse backward alone (delta, lists, dq, dk/dv): 7 products per selected tile executed ----
    cfg = CONFIGS["cfg3"]
    q, k, v, do = make_inputs_on_device(cfg, dev, 3, True)
    m, lut, T = get_block_map(q, k, cfg.topk, cfg.BLKQ, cfg.BLKK)
    o, lse = sparse_attn_fwd(q, k, v, lut, T, cfg.BLKQ, cfg.BLKK, cfg.D ** -0.5)
    ms = time_region(torch, lambda: sparse_attn_bwd(q, k, v, o, do, lse, m, lut, T, cfg.BLKQ, cfg.BLKK, cfg.D ** -0.5),
                     steps, 2, preheat_s=0.05)
    tiles = cfg.B * cfg.H * (-(-cfg.L // cfg.BLKQ)) * T
    ex["cfg3_sparse_bwd_ms"] = ms
    # two conventions: the seven products per tile that the kernels execute (three in dQ, four in dK/dV: 2 flops
    # each = 14), and the reference's "backward = 2.5 x forward" (evaluate/bench_kernel.py:97-98), i.e. five
    # products per tile (10): it counts the scores recomputed once and dP formed once, where the two kernels
    # here each form both
    ex["cfg3_sparse_bwd_mfma_frac"] = 14.0 * tiles * cfg.BLKQ * 64 * cfg.D / ms / 1e9 / PEAK_BF16_TFLOPS
    ex["cfg3_sparse_bwd_mfma_frac_2p5x_fwd"] = 10.0 * tiles * cfg.BLKQ * 64 * cfg.D / ms / 1e9 / PEAK_BF16_TFLOPS
    del q, k, v, do, o, lse, m, lut

    # ---- cfg5: SageSLA module forward, and its attention kernel against the int8 / fp8 peak ----
    cfg = CONFIGS["cfg5"]
    q, k, v, _ = make_inputs_on_device(cfg, dev, 5, False)
    sage = seeded(SageSparseLinearAttention(cfg.D, cfg.topk, cfg.feature_map).to(dev))
    with torch.no_grad():
        ex["cfg5_sage_fwd_ms"] = time_region(torch, lambda: sage(q, k, v), steps, 2, preheat_s=0.05)
        m, lut, T, q8, qs, k8, ks, _, _ = sage_prepare(q, k, None, cfg.topk)
        v8, vs = quant_v(v)
        ms = time_region(torch, lambda: sage_attn_fwd(q8, qs, k8, ks, v8, vs, lut, T, torch.bfloat16), steps, 2,
                         preheat_s=0.05)
    ops = 4.0 * cfg.B * cfg.H * (-(-cfg.L // 128)) * T * 128 * 64 * cfg.D
    ex["cfg5_sage_attention_kernel_ms"] = ms
    ex["cfg5_sage_attention_kernel_frac_of_5_pops"] = ops / ms / 1e9 / PEAK_I8F8_TOPS
    ex["cfg5_sage_effective_tflops"] = 4.0 * cfg.B * cfg.H * cfg.L * cfg.L * cfg.D / ex["cfg5_sage_fwd_ms"] / 1e9
    del q8, k8, v8, m, lut, sage
    # the 16-bit module on the same inputs and block sizes
    mod = seeded(SparseLinearAttention(cfg.D, cfg.topk, cfg.feature_map, cfg.BLKQ, cfg.BLKK).to(dev))
    with torch.no_grad():
        ex["cfg5_sla_bf16_fwd_ms"] = time_region(torch, lambda: mod(q, k, v), steps, 2, preheat_s=0.05)
    del q, k, v, mod

    # ---- cfg4: module forward and forward + backward ----
    cfg = CONFIGS["cfg4"]
    q, k, v, do = make_inputs_on_device(cfg, dev, 4, True)
    mod = seeded(SparseLinearAttention(cfg.D, cfg.topk, cfg.feature_map, cfg.BLKQ, cfg.BLKK).to(dev))
    dense = 4.0 * cfg.B * cfg.H * cfg.L * cfg.L * cfg.D
    with torch.no_grad():
        ex["cfg4_sla_fwd_ms"] = time_region(torch, lambda: mod(q, k, v), steps, 1, preheat_s=0.05)
        ms = time_region(torch, lambda: get_block_map(q, k, cfg.topk, cfg.BLKQ, cfg.BLKK), steps, 1, preheat_s=0.05)
    ex["cfg4_fwd_effective_tflops"] = dense / ex["cfg4_sla_fwd_ms"] / 1e9
    ex["cfg4_mask_ms"] = ms
    ex["cfg4_mask_hbm_gbs"] = 2.0 * q.numel() * 2 / ms / 1e6
    # the attention kernel of that forward alone, against the bf16 MFMA peak (the cfg3 convention: executed flops of the
    # selected tiles and of the epilogue's products)
    from sla_amd.linear import linear_state_fwd
    from sla_amd.sparse_attn import sparse_attn_linear_fwd
    with torch.no_grad():
        _, lut4, T4 = get_block_map(q, k, cfg.topk, cfg.BLKQ, cfg.BLKK)
        ws4 = linear_state_fwd(k, v, mod.proj_l.weight, cfg.feature_map)
        ms = time_region(torch, lambda: sparse_attn_linear_fwd(q, k, v, lut4, T4, cfg.BLKQ, cfg.BLKK, cfg.D ** -0.5, ws4,
                                                               mod.proj_l.bias, cfg.feature_map, False),
                         steps, 1, preheat_s=0.05)
    flops4 = (4.0 * cfg.B * cfg.H * (-(-cfg.L // cfg.BLKQ)) * T4 * cfg.BLKQ * 64 * cfg.D
              + 2.0 * cfg.B * cfg.H * cfg.L * cfg.D * cfg.D)
    ex["cfg4_attention_fused_ms"] = ms
    ex["cfg4_attention_fused_mfma_frac"] = flops4 / ms / 1e9 / PEAK_BF16_TFLOPS
    del lut4, ws4
    qg, kg, vg = (t.requires_grad_(True) for t in (q, k, v))

    def fwd_bwd():
        mod(qg, kg, vg).backward(do)
        qg.grad = kg.grad = vg.grad = None
    ex["cfg4_sla_fwd_bwd_ms"] = time_region(torch, fwd_bwd, steps, 1, preheat_s=0.05)
    ex["cfg4_fwd_bwd_effective_tflops"] = 3.5 * dense / ex["cfg4_sla_fwd_bwd_ms"] / 1e9
    del q, k, v, do, qg, kg, vg, mod
    torch.cuda.empty_cache()

    # ---- the reference's own kernel benchmark: B2 H16 L32760 D128 randn, sparsity .95, BLKQ 128 ----
    spec = importlib.util.spec_from_file_location("bench_kernel", os.path.join(ROOT, "evaluate", "bench_kernel.py"))
    bk = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(bk)
    for r in bk.run(iters=steps, warmup=2):
        ex[f"bench_kernel_{r['mode']}_ms"] = r["ms"]
        ex[f"bench_kernel_{r['mode']}_effective_tflops"] = r["effective_tflops"]
        if "attention_kernel_ms" in r:
            ex["bench_kernel_attention_kernel_ms"] = r["attention_kernel_ms"]
    return ex


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="cfg3")
    ap.add_argument("--cpu-heads", type=int, default=12, help="heads of the workload timed on the CPU oracle (0 = skip)")
    ap.add_argument("--no-extras", action="store_true", help="skip the per-kernel, backward and SageSLA timings")
    ap.add_argument("--one-config", action="store_true",
                    help="keep the extras of the workload itself, skip the other configurations (for profiler runs)")
    ap.add_argument("--pmc-calibration", action="store_true",
                    help="also run one plain 1 GiB read + 1 GiB write elementwise kernel, the known-size reference for "
                         "scaling the FETCH_SIZE / WRITE_SIZE counters of a rocprofv3 --pmc run")
    ap.add_argument("--record-traffic", type=float, nargs="+",
                    metavar="FETCH_KIB WRITE_KIB FETCH_FACTOR WRITE_FACTOR [GUI_ACTIVE_CYCLES DISPATCH_US]",
                    help="store the FETCH_SIZE / WRITE_SIZE readings (KiB per dispatch of the dominant kernel) and the "
                         "calibration factors of two rocprofv3 --pmc runs and, optionally, GRBM_GUI_ACTIVE and the duration "
                         "(us) of one dispatch from a third, stamped with the kernel sources' fingerprint; needs no GPU")
    ap.add_argument("--margins", action="store_true",
                    help="write profiles/pooled_score_boundary_margins.md (how close the block selection of every "
                         "configuration is to a tie) and exit")
    args = ap.parse_args()
    if args.record_traffic:
        assert len(args.record_traffic) in (4, 6), "--record-traffic takes 4 or 6 values"
        record_traffic(args.record_traffic)
        return
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (heads shard with no collective in "
              "forward); run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    from sla_amd import build as _build
    if not os.path.exists(_build.LIBPATH):
        _build.build(force=True)
    import torch
    from sla_amd import SparseLinearAttention, get_block_map
    from sla_amd.inputs import CONFIGS, make_inputs, make_proj
    from sla_amd.linear import linear_fwd
    from sla_amd.linear import linear_state_fwd
    from sla_amd.sparse_attn import sparse_attn_fwd, sparse_attn_linear_fwd

    cfg = CONFIGS[args.workload]
    dev = torch.device("cuda:0")
    if args.margins:
        boundary_margins(torch, dev, os.path.join(ROOT, "profiles", "pooled_score_boundary_margins.md"))
        return
    d = make_inputs(cfg, with_do=True)
    q, k, v, do = (d[x].to(dev) for x in ("q", "k", "v", "do"))
    w, b = make_proj(cfg.D)
    mod = SparseLinearAttention(cfg.D, cfg.topk, cfg.feature_map, cfg.BLKQ, cfg.BLKK).to(dev)
    with torch.no_grad():
        mod.proj_l.weight.copy_(w)
        mod.proj_l.bias.copy_(b)
    B, H, L, D = q.shape
    M = -(-L // cfg.BLKQ)
    N = -(-L // cfg.BLKK)

    # ---- the step: full module forward; exactly `steps` calls are timed, each with its own event pair; the
    # headline is their median ----
    flush_buf = torch.empty(512 << 20, dtype=torch.uint8, device=dev)      # larger than 8 x 4 MB of L2 + 256 MB behind them
    with torch.no_grad():
        ms_fwd, ms_fwd_mean = time_steps(torch, lambda: mod(q, k, v), args.steps, args.warmup)
        ms_fwd_cold, _ = time_steps(torch, lambda: mod(q, k, v), max(args.steps // 2, 5), 2, preheat_s=0.05, flush=flush_buf)
    dense_flops = 4.0 * B * H * L * L * D
    eff_tflops = dense_flops / ms_fwd / 1e9

    # ---- dominant kernel: the attention kernel the module launches (block-sparse forward with the linear
    # branch, projection and sum in its epilogue), timed alone with events on its stream ----
    m, lut, T = get_block_map(q, k, cfg.topk, cfg.BLKQ, cfg.BLKK)
    scale = D ** -0.5
    wdev, bdev = mod.proj_l.weight.detach().contiguous(), mod.proj_l.bias.detach().contiguous()
    state_ws = linear_state_fwd(k, v, wdev, cfg.feature_map)
    def attention():
        return sparse_attn_linear_fwd(q, k, v, lut, T, cfg.BLKQ, cfg.BLKK, scale, state_ws, bdev, cfg.feature_map, False)
    ms_sparse, ms_sparse_mean = time_steps(torch, attention, args.steps, args.warmup)
    ms_sparse_cold, _ = time_steps(torch, attention, max(args.steps // 2, 5), 2, preheat_s=0.05, flush=flush_buf)
    # the same launch where the module makes it: behind the mask builder on this stream and the state build on the
    # module's second stream, caches as those kernels leave them
    from sla_amd.module import _StateBuild
    in_module = []
    with torch.no_grad():
        for i in range(args.warmup + args.steps):
            st_build = _StateBuild(k, v, wdev, cfg.feature_map)
            _, lut_i, _ = get_block_map(q, k, cfg.topk, cfg.BLKQ, cfg.BLKK)
            ws_i = st_build.join()
            e0, e1 = _events(torch)
            e0.record()
            sparse_attn_linear_fwd(q, k, v, lut_i, T, cfg.BLKQ, cfg.BLKK, scale, ws_i, bdev, cfg.feature_map, False)
            e1.record()
            if i >= args.warmup:
                in_module.append((e0, e1))
        torch.cuda.synchronize()
    ms_sparse_in_module = _median([e0.elapsed_time(e1) for e0, e1 in in_module])
    # executed MFMA work: QK^T and PV over the selected tiles + phi(q) KVW of the epilogue
    sparse_flops = 4.0 * B * H * M * T * cfg.BLKQ * cfg.BLKK * D + 2.0 * B * H * L * D * D
    achieved = sparse_flops / ms_sparse / 1e9
    traffic, traffic_note = measured_traffic(cfg.name)
    out = {
        "metric": "sla_forward_effective_tflops",
        "value": eff_tflops,
        "unit": "TFLOP/s (dense-equivalent 4*B*H*L^2*D per full module forward)",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms_fwd,
        "ms_per_step_note": "median of the timed steps (one event pair each, back to back)",
        "ms_per_step_mean": ms_fwd_mean, "ms_per_step_l2_flushed": ms_fwd_cold,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": f"{cfg.name}: SLA module forward B{B} H{H} L{L} D{D} BLKQ{cfg.BLKQ} BLKK{cfg.BLKK} "
                               f"topk{cfg.topk} (T={T} of N={N}) feature_map={cfg.feature_map}, structured q/k",
                   "B": B, "H": H, "L": L, "D": D, "topk": cfg.topk, "T": T},
        "roofline": {"bound": "mfma", "achieved": achieved, "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                     "frac": achieved / PEAK_BF16_TFLOPS,
                     "traffic": traffic, "traffic_note": traffic_note,
                     "traffic_unit": "HBM bytes per launch (fetch + write)", "kernel": "sparse_fwd_pair_kernel<FUSED=true>",
                     "flops_per_launch": sparse_flops, "ms_per_launch": ms_sparse,
                     "frac_note": "frac = flops_per_launch / ms_per_launch / peak; ms_per_launch is the median of the "
                                  "kernel launched back to back (warm caches)",
                     "ms_per_launch_mean": ms_sparse_mean, "ms_per_launch_l2_flushed": ms_sparse_cold,
                     "ms_per_launch_in_module": ms_sparse_in_module,
                     "frac_in_module": sparse_flops / ms_sparse_in_module / 1e9 / PEAK_BF16_TFLOPS,
                     "frac_l2_flushed": sparse_flops / ms_sparse_cold / 1e9 / PEAK_BF16_TFLOPS,
                     "clock_mhz": measured_clock_mhz(cfg.name),
                     "clock_note": "GRBM_GUI_ACTIVE / dispatch duration of the kernel in a rocprofv3 --pmc run; the peak "
                                   "is quoted at 2400 MHz"},
    }
    extra = {"sla_fwd_ms": ms_fwd, "attention_fused_ms": ms_sparse}
    if not args.no_extras:
        extra["mask_ms"] = time_region(torch, lambda: get_block_map(q, k, cfg.topk, cfg.BLKQ, cfg.BLKK), args.steps,
                                       args.warmup)
        extra["mask_hbm_gbs"] = 2.0 * q.numel() * 2 / extra["mask_ms"] / 1e6
        extra["sparse_fwd_alone_ms"] = time_region(torch, lambda: sparse_attn_fwd(q, k, v, lut, T, cfg.BLKQ, cfg.BLKK, scale),
                                                   args.steps, args.warmup)
        extra["linear_state_ms"] = time_region(torch, lambda: linear_state_fwd(k, v, wdev, cfg.feature_map), args.steps,
                                               args.warmup)
        extra["state_hbm_gbs"] = 2.0 * q.numel() * 2 / extra["linear_state_ms"] / 1e6
        o_s, _ = sparse_attn_fwd(q, k, v, lut, T, cfg.BLKQ, cfg.BLKK, scale)
        extra["linear_proj_sum_unfused_ms"] = time_region(torch, lambda: linear_fwd(q, k, v, wdev, bdev, o_s, cfg.feature_map),
                                                          args.steps, args.warmup)
        extra["mfma_frac_module_fwd"] = (sparse_flops + 2.0 * B * H * L * D * D) / ms_fwd / 1e9 / PEAK_BF16_TFLOPS
        try:
            qg, kg, vg = (t.clone().requires_grad_(True) for t in (q, k, v))

            def fwd_bwd():
                o = mod(qg, kg, vg)
                o.backward(do)
                qg.grad = kg.grad = vg.grad = None
            extra["sla_fwd_bwd_ms"] = time_region(torch, fwd_bwd, max(args.steps // 2, 1), min(args.warmup, 2))
            extra["fwd_bwd_effective_tflops"] = 3.5 * dense_flops / extra["sla_fwd_bwd_ms"] / 1e9
        except (AssertionError, RuntimeError) as e:
            extra["sla_fwd_bwd_ms"] = None
            extra["fwd_bwd_note"] = str(e)[:200]
        try:
            from sla_amd import SageSparseLinearAttention
            sage = SageSparseLinearAttention(cfg.D, cfg.topk, cfg.feature_map).to(dev)
            with torch.no_grad():
                sage.proj_l.weight.copy_(w)
                sage.proj_l.bias.copy_(b)
                extra["sage_fwd_ms"] = time_region(torch, lambda: sage(q, k, v), args.steps, args.warmup)
        except (ImportError, AssertionError, RuntimeError) as e:
            extra["sage_fwd_ms"] = None
            extra["sage_note"] = str(e)[:200]
        try:
            cmod = SparseLinearAttention(cfg.D, cfg.topk, cfg.feature_map, cfg.BLKQ, cfg.BLKK,
                                         linear_mode="complement").to(dev)
            with torch.no_grad():
                cmod.proj_l.weight.copy_(w)
                cmod.proj_l.bias.copy_(b)
                extra["sla_fwd_complement_mode_ms"] = time_region(torch, lambda: cmod(q, k, v), args.steps, args.warmup)

            def cfwd_bwd():
                o = cmod(qg, kg, vg)
                o.backward(do)
                qg.grad = kg.grad = vg.grad = None
            extra["sla_fwd_bwd_complement_mode_ms"] = time_region(torch, cfwd_bwd, max(args.steps // 2, 1), min(args.warmup, 2))
        except (AssertionError, RuntimeError, NotImplementedError) as e:
            extra["sla_fwd_complement_mode_ms"] = None
            extra["complement_note"] = str(e)[:200]
    if not args.no_extras and not args.one_config and cfg.name == "cfg3":
        extra.update(other_configs(torch, dev, max(args.steps // 10, 3)))
    if args.pmc_calibration:
        x = torch.empty(1 << 28, dtype=torch.float32, device=dev).normal_()
        y = torch.empty_like(x)
        torch.add(x, 1.0, out=y)          # 1 GiB read + 1 GiB written by one elementwise kernel
        torch.cuda.synchronize()
        extra["pmc_calibration"] = "torch.add on 2^28 fp32: 1 GiB read, 1 GiB written"
    out["extra"] = extra
    if args.cpu_heads > 0:
        out["cpu_baseline"] = cpu_baseline(cfg, min(args.cpu_heads, cfg.H), torch)
    else:
        out["cpu_baseline"] = None
    print(json.dumps(out))


if __name__ == "__main__":
    main()
