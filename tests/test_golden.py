"""Known-answer vectors (tests/golden/sla_small.npz, written by tests/golden/make_vectors.py).

They are regression vectors of the CPU oracle (the reference ships no vectors of its own): the CPU test
checks that the oracle still reproduces them, the GPU test checks the HIP path against the same file.
"""
import os

import numpy as np
import pytest
import torch

from conftest import cos_sim, max_abs
from oracle import sla_oracle as O

PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "sla_small.npz")


def _load():
    z = np.load(PATH, allow_pickle=False)
    B, H, L, D, BLKQ, BLKK, T = (int(x) for x in z["shape"])
    bf = lambda name: torch.from_numpy(z[name].view(np.int16).copy()).view(torch.bfloat16)  # noqa: E731
    t = lambda name: torch.from_numpy(z[name].copy())  # noqa: E731
    return dict(B=B, H=H, L=L, D=D, BLKQ=BLKQ, BLKK=BLKK, T=T, topk=float(z["topk"]), fmap=str(z["fmap"]),
                q=bf("q"), k=bf("k"), v=bf("v"), do=bf("do"), weight=t("weight"), bias=t("bias"),
                lut=t("lut").long(), sparse_map=t("sparse_map"), o_s=t("o_s"), lse2=t("lse2"), out=t("out"),
                dq=t("dq"), dk=t("dk"), dv=t("dv"), dw=t("dw"), db=t("db"))


def test_oracle_reproduces_the_vectors():
    g = _load()
    o, o_s, _, sparse_map, lut, T = O.sla_forward(g["q"], g["k"], g["v"], g["weight"], g["bias"], g["topk"], g["fmap"],
                                                  g["BLKQ"], g["BLKK"], linear_dtype=torch.float32)
    assert T == g["T"] and torch.equal(lut, g["lut"]) and torch.equal(sparse_map, g["sparse_map"])
    assert max_abs(o_s.float(), g["o_s"]) <= 1e-5
    assert max_abs(o.float(), g["out"]) <= 2 ** -6          # one bf16 step at the output's magnitude
    _, lse2 = O.sparse_attn_fwd_gather(g["q"], g["k"], g["v"], lut, g["BLKQ"], g["BLKK"], dtype=torch.float32)
    assert max_abs(lse2.float(), g["lse2"]) <= 1e-4
    # the explicit backward formulas of the oracle against the stored autograd gradients of the sparse branch
    # plus nothing else would not be comparable (the stored ones include the linear branch); compare the
    # full restatement instead
    qd, kd, vd = (x.double().requires_grad_(True) for x in (g["q"], g["k"], g["v"]))
    wd, bd = g["weight"].double().requires_grad_(True), g["bias"].double().requires_grad_(True)
    out, _, _ = O.sla_forward_autograd(qd, kd, vd, wd, bd, sparse_map, g["fmap"], g["BLKQ"], g["BLKK"])
    (out * g["do"].double()).sum().backward()
    for name, grad in (("dq", qd.grad), ("dk", kd.grad), ("dv", vd.grad), ("dw", wd.grad), ("db", bd.grad)):
        assert max_abs(grad.float(), g[name]) <= 1e-4 * max(1.0, float(g[name].abs().max())), name


@pytest.mark.gpu
def test_hip_path_against_the_vectors(dev):
    from sla_amd import SparseLinearAttention, get_block_map

    g = _load()
    q, k, v = (g[x].to(dev).requires_grad_(True) for x in "qkv")
    sparse_map, lut, T = get_block_map(q.detach(), k.detach(), g["topk"], g["BLKQ"], g["BLKK"])
    assert T == g["T"] and torch.equal(lut.cpu().long(), g["lut"]) and torch.equal(sparse_map.cpu(), g["sparse_map"])
    mod = SparseLinearAttention(g["D"], g["topk"], g["fmap"], g["BLKQ"], g["BLKK"]).to(dev)
    with torch.no_grad():
        mod.proj_l.weight.copy_(g["weight"])
        mod.proj_l.bias.copy_(g["bias"])
    out = mod(q, k, v)
    o = out.detach().float().cpu()
    assert max_abs(o, g["out"]) <= 2e-2 and cos_sim(o, g["out"]) >= 0.999
    out.backward(g["do"].to(dev))
    for name, grad in (("dq", q.grad), ("dk", k.grad), ("dv", v.grad), ("dw", mod.proj_l.weight.grad),
                       ("db", mod.proj_l.bias.grad)):
        ref = g[name]
        scale = max(1.0, float(ref.abs().max()))
        assert max_abs(grad.float().cpu(), ref) <= 2e-2 * scale, name
        assert cos_sim(grad.float().cpu(), ref) >= 0.999, name
