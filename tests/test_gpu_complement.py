"""Complement-mode linear branch (linear attention over the non-selected key blocks) vs the brute-force oracle."""
import pytest
import torch

from conftest import cos_sim, max_abs
from oracle import sla_oracle as O
from sla_amd import SparseLinearAttention
from sla_amd.inputs import CONFIGS, make_inputs, make_proj
from sla_amd.linear import linear_bwd, linear_complement_bwd, linear_complement_fwd, linear_fwd

pytestmark = pytest.mark.gpu

TOL_ABS = 2e-2
TOL_COS = 0.999


@pytest.mark.parametrize("fmap", ["elu", "relu", "softmax"])
@pytest.mark.parametrize("L,D,BLKQ,ratio", [(512, 128, 64, 0.25), (1000, 128, 128, 0.3), (333, 64, 64, 0.5), (700, 64, 128, 0.2)])
def test_complement_vs_oracle(dev, fmap, L, D, BLKQ, ratio):
    g = torch.Generator().manual_seed(L + D)
    q, k, v, res = (torch.randn(1, 2, L, D, generator=g).to(torch.bfloat16) for _ in range(4))
    w, b = make_proj(D)
    m, lut, T = O.get_block_map(q, k, ratio, BLKQ, 64)
    ref = O.linear_branch_complement(q, k, v, lut, w, b, fmap, BLKQ, 64, torch.float32).float() + res.float()
    out = linear_complement_fwd(q.to(dev), k.to(dev), v.to(dev), lut.to(dev), T, w.to(dev), b.to(dev), res.to(dev), fmap,
                                BLKQ, 64).cpu()
    assert out.dtype == torch.bfloat16
    assert max_abs(out, ref) <= TOL_ABS and cos_sim(out, ref) >= TOL_COS


def test_empty_selection_equals_global_branch(dev):
    """With nothing selected the complement is everything: same result as the global linear branch up to the
    16-bit rounding of the per-block states and of the unfolded projection."""
    g = torch.Generator().manual_seed(11)
    q, k, v = (torch.randn(1, 2, 640, 128, generator=g).to(torch.bfloat16).to(dev) for _ in range(3))
    w, b = (t.to(dev) for t in make_proj(128))
    lut = torch.zeros((1, 2, 10, 0), dtype=torch.int64, device=dev)
    out = linear_complement_fwd(q, k, v, lut, 0, w, b, None, "elu")
    ref = linear_fwd(q, k, v, w, b, None, "elu")
    assert max_abs(out.cpu(), ref.cpu()) <= TOL_ABS and cos_sim(out.cpu(), ref.cpu()) >= TOL_COS


def test_int32_lut_and_module_option(dev):
    cfg = CONFIGS["cfg2"]
    d = make_inputs(cfg, H=2)
    q, k, v = (d[x] for x in "qkv")
    w, b = make_proj(cfg.D)
    mod = SparseLinearAttention(cfg.D, cfg.topk, "relu", cfg.BLKQ, cfg.BLKK, linear_mode="complement").to(dev)
    with torch.no_grad():
        mod.proj_l.weight.copy_(w)
        mod.proj_l.bias.copy_(b)
        o = mod(q.to(dev), k.to(dev), v.to(dev)).cpu()
    m, lut, T = O.get_block_map(q, k, cfg.topk, cfg.BLKQ, cfg.BLKK)
    o_s, _ = O.sparse_attn_fwd_gather(q, k, v, lut, cfg.BLKQ, cfg.BLKK)
    ref = o_s.float() + O.linear_branch_complement(q, k, v, lut, w, b, "relu", cfg.BLKQ, cfg.BLKK, torch.float32).float()
    assert max_abs(o, ref) <= TOL_ABS and cos_sim(o, ref) >= TOL_COS
    out32 = linear_complement_fwd(q.to(dev), k.to(dev), v.to(dev), lut.to(dev).int(), T, w.to(dev), b.to(dev), None, "relu")
    out64 = linear_complement_fwd(q.to(dev), k.to(dev), v.to(dev), lut.to(dev), T, w.to(dev), b.to(dev), None, "relu")
    assert torch.equal(out32, out64)
    with pytest.raises(NotImplementedError):
        SparseLinearAttention(cfg.D, cfg.topk, "relu", linear_mode="selected")


def _oracle_grads(q, k, v, lut, w, b, g, fmap, BLKQ):
    leaves = [t.float().clone().requires_grad_(True) for t in (q, k, v, w, b)]
    O.linear_branch_complement(*leaves[:3], lut, *leaves[3:], fmap, BLKQ, 64, torch.float32).backward(g.float())
    return [t.grad for t in leaves]


def _check_grads(got, refs):
    for name, a, r in zip(("dq", "dk", "dv", "dW", "db"), got, refs):
        a = a.cpu()
        scale = max(1.0, float(r.abs().max()))          # dW/db are sums over B*H*L rows
        assert max_abs(a, r) <= TOL_ABS * scale, (name, max_abs(a, r), scale)
        assert cos_sim(a, r) >= TOL_COS, (name, cos_sim(a, r))


@pytest.mark.parametrize("fmap", ["elu", "relu", "softmax"])
@pytest.mark.parametrize("L,D,BLKQ,ratio", [(512, 128, 64, 0.25), (1000, 128, 128, 0.3), (333, 64, 64, 0.5), (700, 64, 128, 0.2),
                                            (150, 128, 64, 0.4)])
def test_complement_backward_vs_autograd_oracle(dev, fmap, L, D, BLKQ, ratio):
    gen = torch.Generator().manual_seed(L + D + 1)
    q, k, v, g = (torch.randn(2, 2, L, D, generator=gen).to(torch.bfloat16) for _ in range(4))
    w, b = make_proj(D)
    m, lut, T = O.get_block_map(q, k, ratio, BLKQ, 64)
    refs = _oracle_grads(q, k, v, lut, w, b, g, fmap, BLKQ)
    args = [t.to(dev) for t in (q, k, v, m, lut)]
    got = linear_complement_bwd(*args, T, w.to(dev), b.to(dev), g.to(dev), fmap, BLKQ, 64)
    _check_grads(got, refs)
    # adding into existing gradients: one more 16-bit rounding of the sum
    base = [torch.randn(2, 2, L, D, generator=gen).to(torch.bfloat16).to(dev) for _ in range(3)]
    acc = linear_complement_bwd(*args, T, w.to(dev), b.to(dev), g.to(dev), fmap, BLKQ, 64,
                                accumulate_into=tuple(t.clone() for t in base))
    for a, x, y in zip(acc[:3], base, got[:3]):
        assert torch.equal(a, (x.float() + y.float()).to(torch.bfloat16))
    assert torch.equal(acc[3], got[3]) and torch.equal(acc[4], got[4])


def test_backward_with_nothing_selected_equals_the_global_backward(dev):
    gen = torch.Generator().manual_seed(13)
    q, k, v, g = (torch.randn(1, 2, 640, 128, generator=gen).to(torch.bfloat16).to(dev) for _ in range(4))
    w, b = (t.to(dev) for t in make_proj(128))
    lut = torch.zeros((1, 2, 10, 0), dtype=torch.int64, device=dev)
    m = torch.zeros((1, 2, 10, 10), dtype=torch.int8, device=dev)
    got = linear_complement_bwd(q, k, v, m, lut, 0, w, b, g, "elu")
    ref = linear_bwd(q, k, v, w, b, g, "elu")
    _check_grads(got, [t.cpu().float() for t in ref])


def test_module_trains_in_complement_mode(dev):
    cfg = CONFIGS["cfg2"]
    d = make_inputs(cfg, H=2)
    q, k, v, do = (d[x] for x in ("q", "k", "v", "do"))
    w, b = make_proj(cfg.D)
    mod = SparseLinearAttention(cfg.D, cfg.topk, "softmax", cfg.BLKQ, cfg.BLKK, linear_mode="complement").to(dev)
    with torch.no_grad():
        mod.proj_l.weight.copy_(w)
        mod.proj_l.bias.copy_(b)
    qd, kd, vd = (t.to(dev).requires_grad_(True) for t in (q, k, v))
    mod(qd, kd, vd).backward(do.to(dev))
    m, lut, T = O.get_block_map(q, k, cfg.topk, cfg.BLKQ, cfg.BLKK)
    o_s, lse = O.sparse_attn_fwd_gather(q, k, v, lut, cfg.BLKQ, cfg.BLKK)
    sp = O.sparse_attn_bwd_gather(q, k, v, o_s, do, lse, lut, cfg.BLKQ, cfg.BLKK)
    lin = _oracle_grads(q, k, v, lut, w, b, do, "softmax", cfg.BLKQ)
    refs = [a + c for a, c in zip(sp, lin[:3])] + lin[3:]
    _check_grads((qd.grad, kd.grad, vd.grad, mod.proj_l.weight.grad, mod.proj_l.bias.grad), refs)


def test_everything_selected_leaves_the_bias_and_no_gradient(dev):
    """topk = 1: the complement is empty.  The difference of the two state sums is then exactly zero (not their
    rounding residue, which the 1e-5 of the divisor would amplify): the branch is the bias, and only the bias has a gradient."""
    from sla_amd import _attention
    gen = torch.Generator().manual_seed(17)
    q, k, v, g = (torch.randn(1, 2, 333, 128, generator=gen).to(torch.bfloat16).to(dev) for _ in range(4))
    w, b = (t.to(dev) for t in make_proj(128))
    for BLKQ in (64, 128):
        M, N = -(-333 // BLKQ), 6
        lut = torch.arange(N, device=dev).expand(1, 2, M, N).contiguous()
        m = torch.ones(1, 2, M, N, dtype=torch.int8, device=dev)
        out = linear_complement_fwd(q, k, v, lut, N, w, b, None, "elu", BLKQ, 64)
        assert torch.equal(out, b.to(torch.bfloat16).expand_as(out))
        dq, dk, dv, dw, db = linear_complement_bwd(q, k, v, m, lut, N, w, b, g, "elu", BLKQ, 64)
        for t in (dq, dk, dv, dw):
            assert int(torch.count_nonzero(t)) == 0
        assert max_abs(db.cpu(), g.float().sum((0, 1, 2)).cpu()) <= 1e-2 * float(g.float().sum((0, 1, 2)).abs().max())
