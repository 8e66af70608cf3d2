"""Writes tests/golden/sla_small.npz: known-answer vectors of the CPU oracle for one small ragged case.

The reference ships no golden vectors (it has no tests at all), so these are regression vectors of the
oracle itself, not outputs of the reference: they pin what the oracle computed when its functions were
checked against closed forms and library routines, so that a later change of the oracle (or of a torch
version underneath it) that moves a result is noticed, and they give the HIP path one fixed target that
does not depend on a random generator.  Inputs are stored in the file (bf16 bit patterns), not re-drawn.

Run from the repository root:  python tests/golden/make_vectors.py
"""
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import sla_oracle as O  # noqa: E402

B, H, L, D = 1, 1, 200, 64          # L is not a multiple of the block size: the last blocks are ragged
BLKQ = BLKK = 64
TOPK = 0.5                          # 2 of 4 key blocks
FMAP = "elu"


def bits(x):                        # bf16 tensor -> uint16 array
    return x.view(torch.int16).numpy().view(np.uint16)


def main():
    g = torch.Generator().manual_seed(20240607)
    q, k, v, do = (torch.randn(B, H, L, D, generator=g).to(torch.bfloat16) for _ in range(4))
    k = (k.float() + 0.75 * torch.randn(1, H, 1, D, generator=g)).to(torch.bfloat16)   # a column offset to smooth away
    w = (torch.randn(D, D, generator=g) / D ** 0.5).float()
    b = (0.1 * torch.randn(D, generator=g)).float()

    o, o_s, o_l, sparse_map, lut, T = O.sla_forward(q, k, v, w, b, TOPK, FMAP, BLKQ, BLKK, linear_dtype=torch.float32)
    _, lse2 = O.sparse_attn_fwd_gather(q, k, v, lut, BLKQ, BLKK, dtype=torch.float32)
    # gradients of sum(out * do) by autograd through the dense-masked float64 restatement
    qd, kd, vd = (t.double().requires_grad_(True) for t in (q, k, v))
    wd, bd = w.double().requires_grad_(True), b.double().requires_grad_(True)
    out, _, _ = O.sla_forward_autograd(qd, kd, vd, wd, bd, sparse_map, FMAP, BLKQ, BLKK)
    (out * do.double()).sum().backward()

    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "sla_small.npz")
    np.savez_compressed(
        path,
        shape=np.array([B, H, L, D, BLKQ, BLKK, T], dtype=np.int32), topk=np.float64(TOPK), fmap=np.array(FMAP),
        q=bits(q), k=bits(k), v=bits(v), do=bits(do), weight=w.numpy(), bias=b.numpy(),
        lut=lut.numpy().astype(np.int16), sparse_map=sparse_map.numpy(),
        o_s=o_s.float().numpy(), lse2=lse2.float().numpy(), out=o.float().numpy(),
        dq=qd.grad.float().numpy(), dk=kd.grad.float().numpy(), dv=vd.grad.float().numpy(),
        dw=wd.grad.float().numpy(), db=bd.grad.float().numpy())
    print("wrote", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
