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

# HBM bytes per launch of the dominant kernel, from two `rocprofv3 --pmc` runs of this script
# (FETCH_SIZE, then WRITE_SIZE; summaries under profiles/), each scaled by what the same counter reads for
# the 1 GiB-read / 1 GiB-write elementwise kernel of --pmc-calibration (FETCH_SIZE x2.0, WRITE_SIZE x1.0).
# It is a property of the kernel and the workload, not re-measured by a plain bench run.
MEASURED_TRAFFIC_BYTES = {
    "cfg3": {"kernel": "sparse_fwd_kernel<FUSED>", "fetch": 208656.1 * 1024 * 2.0, "write": 99869.7 * 1024 * 1.0},
}


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


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="cfg3")
    ap.add_argument("--cpu-heads", type=int, default=12, help="heads of the workload timed on the CPU oracle (0 = skip)")
    ap.add_argument("--no-extras", action="store_true", help="skip the per-kernel, backward and SageSLA timings")
    ap.add_argument("--pmc-calibration", action="store_true",
                    help="also run one plain 1 GiB read + 1 GiB write elementwise kernel, the known-size reference for "
                         "scaling the FETCH_SIZE / WRITE_SIZE counters of a rocprofv3 --pmc run")
    args = ap.parse_args()
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

    # ---- the step: full module forward ----
    with torch.no_grad():
        ms_fwd = time_region(torch, lambda: mod(q, k, v), args.steps, args.warmup)
    dense_flops = 4.0 * B * H * L * L * D
    eff_tflops = dense_flops / ms_fwd / 1e9

    # ---- dominant kernel: the attention kernel the module launches (block-sparse forward with the linear
    # branch, projection and sum in its epilogue), timed alone with events on its stream ----
    m, lut, T = get_block_map(q, k, cfg.topk, cfg.BLKQ, cfg.BLKK)
    scale = D ** -0.5
    wdev, bdev = mod.proj_l.weight.detach().contiguous(), mod.proj_l.bias.detach().contiguous()
    state_ws = linear_state_fwd(k, v, wdev, cfg.feature_map)
    ms_sparse = time_region(torch, lambda: sparse_attn_linear_fwd(q, k, v, lut, T, cfg.BLKQ, cfg.BLKK, scale, state_ws,
                                                                  bdev, cfg.feature_map, False), args.steps, args.warmup)
    # executed MFMA work: QK^T and PV over the selected tiles + phi(q) KVW of the epilogue
    sparse_flops = 4.0 * B * H * M * T * cfg.BLKQ * cfg.BLKK * D + 2.0 * B * H * L * D * D
    achieved = sparse_flops / ms_sparse / 1e9
    out = {
        "metric": "sla_forward_effective_tflops",
        "value": eff_tflops,
        "unit": "TFLOP/s (dense-equivalent 4*B*H*L^2*D per full module forward)",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms_fwd,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": f"{cfg.name}: SLA module forward B{B} H{H} L{L} D{D} BLKQ{cfg.BLKQ} BLKK{cfg.BLKK} "
                               f"topk{cfg.topk} (T={T} of N={N}) feature_map={cfg.feature_map}, structured q/k",
                   "B": B, "H": H, "L": L, "D": D, "topk": cfg.topk, "T": T},
        "roofline": {"bound": "mfma", "achieved": achieved, "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                     "frac": achieved / PEAK_BF16_TFLOPS,
                     "traffic": (sum(v for k_, v in MEASURED_TRAFFIC_BYTES[cfg.name].items() if k_ != "kernel")
                                 if cfg.name in MEASURED_TRAFFIC_BYTES else None),
                     "traffic_unit": "HBM bytes per launch (fetch + write)", "kernel": "sparse_fwd_kernel<FUSED=true>",
                     "flops_per_launch": sparse_flops, "ms_per_launch": ms_sparse},
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
