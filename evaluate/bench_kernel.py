"""Kernel benchmark in the convention of the reference's ``evaluate/bench_kernel.py``.

Workload of that script (reference ``bench_kernel.py:31,41,62-65,79,104``): bf16 ``randn`` q, k, v of shape
(2, 16, 32760, 128), sparsity 0.95 (``topk_ratio = 0.05``), ``BLKQ=128, BLKK=64``; the mask is built once
outside the timed body; the timed body is ``_attention.apply`` plus the plain ``calc_linear`` of raw q, k
(no feature map, no projection: reference ``:81-85``); "bwd" times ``o.backward(do, retain_graph=True)`` of
``o = o_s + o_l`` (``:87-90``).  TFLOPS = dense-equivalent ``4 B H L^2 D / t`` (x2.5 for bwd, ``:93-98``).

Here the attention runs on the HIP kernels of this repository; ``calc_linear`` stays the three eager torch
expressions the reference script times (rocBLAS GEMMs).  One JSON line per mode.

    python evaluate/bench_kernel.py [--batch 2 --heads 16 --seq 32760 --sparsity 0.95 --blkq 128]
"""
from __future__ import annotations

import argparse
import json
import os
import sys

import torch

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))

from sparse_linear_attention.kernel import _attention  # noqa: E402
from sparse_linear_attention.utils import get_block_map  # noqa: E402


def calc_linear(q, k, v):
    kvsum = k.transpose(-1, -2) @ v
    ksum = torch.sum(k, dim=-2, keepdim=True)
    return (q @ kvsum) / (1e-5 + (q * ksum).sum(dim=-1, keepdim=True))


def time_ms(fn, warmup=5, iters=20):
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    e0 = torch.cuda.Event(enable_timing=True)
    e1 = torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(iters):
        fn()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / iters


def run(batch=2, heads=16, seq=32760, dim=128, sparsity=0.95, blkq=128, iters=20, warmup=5):
    """Times the two modes; returns the two result dicts (``mode`` "fwd" and "bwd")."""
    dev = torch.device("cuda:0")
    torch.manual_seed(42)
    shape = (batch, heads, seq, dim)
    q, k, v = (torch.randn(shape, dtype=torch.bfloat16, device=dev, requires_grad=True) for _ in range(3))
    do = torch.randn_like(v)
    with torch.no_grad():
        sparse_map, lut, real_topk = get_block_map(q, k, topk_ratio=1 - sparsity, BLKQ=blkq, BLKK=64)

    def fwd():
        return _attention.apply(q, k, v, sparse_map, lut, real_topk, blkq, 64), calc_linear(q, k, v)

    def fwd_attention_only():
        with torch.no_grad():
            return _attention.apply(q, k, v, sparse_map, lut, real_topk, blkq, 64)

    dense_flops = 4.0 * batch * heads * seq * seq * dim
    common = {"B": batch, "H": heads, "L": seq, "D": dim, "sparsity": sparsity, "BLKQ": blkq, "BLKK": 64, "T": real_topk,
              "dtype": "bf16", "data": "randn, seed 42"}
    ms = time_ms(fwd, warmup=warmup, iters=iters)
    ms_attn = time_ms(fwd_attention_only, warmup=warmup, iters=iters)
    results = [{"mode": "fwd", "ms": ms, "effective_tflops": dense_flops / ms * 1e-9, "attention_kernel_ms": ms_attn,
                **common}]
    o_s, o_l = fwd()
    o = o_s + o_l

    def bwd():
        q.grad = k.grad = v.grad = None
        o.backward(do, retain_graph=True)

    ms = time_ms(bwd, warmup=warmup, iters=iters)
    results.append({"mode": "bwd", "ms": ms, "effective_tflops": 2.5 * dense_flops / ms * 1e-9, **common})
    return results


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--batch", type=int, default=2)
    ap.add_argument("--heads", type=int, default=16)
    ap.add_argument("--seq", type=int, default=32760)
    ap.add_argument("--dim", type=int, default=128)
    ap.add_argument("--sparsity", type=float, default=0.95)
    ap.add_argument("--blkq", type=int, default=128)
    ap.add_argument("--iters", type=int, default=20)
    args = ap.parse_args()
    if not torch.cuda.is_available():
        sys.exit("evaluate/bench_kernel.py needs a GPU")
    for r in run(args.batch, args.heads, args.seq, args.dim, args.sparsity, args.blkq, args.iters):
        print(json.dumps(r))


if __name__ == "__main__":
    main()
