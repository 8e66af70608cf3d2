"""Pins the sparse-attention part of the CPU oracle: library SDPA, independent autograd,
gradcheck, brute force and invariants (the reference ships no vectors)."""
import math

import pytest
import torch
import torch.nn.functional as F

from oracle import sla_oracle as O

LN2 = math.log(2.0)


def _rand(B, H, L, D, seed=0, dtype=torch.float64):
    g = torch.Generator().manual_seed(seed)
    return tuple(torch.randn(B, H, L, D, generator=g, dtype=torch.float64).to(dtype) for _ in range(3))


def _full_map(B, H, L, BLKQ, BLKK):
    M, N = -(-L // BLKQ), -(-L // BLKK)
    m = torch.ones(B, H, M, N, dtype=torch.int8)
    lut = torch.arange(N).expand(B, H, M, N).contiguous()
    return m, lut


@pytest.mark.parametrize("L,BLKQ", [(256, 64), (200, 64), (100, 128), (64, 64), (37, 64)])
def test_full_selection_is_sdpa(L, BLKQ):
    q, k, v = _rand(1, 2, L, 32)
    m, lut = _full_map(1, 2, L, BLKQ, 64)
    ref = F.scaled_dot_product_attention(q, k, v)
    o1, lse1 = O.sparse_attn_fwd_dense(q, k, v, m, BLKQ, 64)
    o2, lse2 = O.sparse_attn_fwd_gather(q, k, v, lut, BLKQ, 64, dtype=torch.float64)
    assert (o1 - ref).abs().max() < 1e-12 and (o2 - ref).abs().max() < 1e-12
    s = (q @ k.transpose(-1, -2)) / math.sqrt(32)
    assert (lse1 * LN2 - torch.logsumexp(s, -1)).abs().max() < 1e-12
    assert (lse2 * LN2 - torch.logsumexp(s, -1)).abs().max() < 1e-12


def test_sparse_is_masked_softmax_brute_force():
    # brute force per query row with python loops over selected blocks
    q, k, v = _rand(1, 1, 150, 8, seed=1)
    m, lut, T = O.get_block_map(q.float(), k.float(), 0.67, 64, 64)
    assert T == 2
    o, lse = O.sparse_attn_fwd_dense(q, k, v, m, 64, 64)
    for i in (0, 63, 64, 149):
        keys = [j for b in lut[0, 0, i // 64].tolist() for j in range(b * 64, min(150, b * 64 + 64))]
        w = torch.tensor([float(q[0, 0, i] @ k[0, 0, j]) / math.sqrt(8) for j in keys], dtype=torch.float64)
        p = torch.exp(w - w.max())
        ref = sum(p[n] * v[0, 0, j] for n, j in enumerate(keys)) / p.sum()
        assert (o[0, 0, i] - ref).abs().max() < 1e-12
        assert abs(lse[0, 0, i] * LN2 - (w.max() + torch.log(p.sum()))) < 1e-12


@pytest.mark.parametrize("L,BLKQ,ratio", [(512, 64, 0.25), (300, 128, 0.5), (130, 64, 0.4)])
def test_gather_equals_dense_and_lut_order_is_irrelevant(L, BLKQ, ratio):
    q, k, v = _rand(2, 2, L, 16, seed=2)
    m, lut, T = O.get_block_map(q.float(), k.float(), ratio, BLKQ, 64)
    o1, lse1 = O.sparse_attn_fwd_dense(q, k, v, m, BLKQ, 64)
    o2, lse2 = O.sparse_attn_fwd_gather(q, k, v, lut, BLKQ, 64, dtype=torch.float64)
    o3, _ = O.sparse_attn_fwd_gather(q, k, v, lut.flip(-1), BLKQ, 64, dtype=torch.float64)
    assert (o1 - o2).abs().max() < 1e-12 and (lse1 - lse2).abs().max() < 1e-12
    assert (o2 - o3).abs().max() < 1e-12
    o4, _ = O.sparse_attn_fwd_gather(q, k, v, lut, BLKQ, 64, heads=[1, 3], dtype=torch.float64)
    assert (o4[0, 1] - o1[0, 1]).abs().max() < 1e-12 and (o4[1, 1] - o1[1, 1]).abs().max() < 1e-12
    assert float(o4[0, 0].abs().max()) == 0.0


def _autograd_reference(q, k, v, m, do, BLKQ):
    q, k, v = (t.clone().requires_grad_(True) for t in (q, k, v))
    L, D = q.shape[-2:]
    mask = O.expand_block_map(m, L, BLKQ, 64)
    s = (q @ k.transpose(-1, -2)) / math.sqrt(D)
    o = torch.softmax(s.masked_fill(~mask, float("-inf")), -1) @ v
    o.backward(do)
    return o.detach(), q.grad, k.grad, v.grad


@pytest.mark.parametrize("L,BLKQ,ratio", [(256, 64, 0.5), (200, 128, 0.5), (150, 64, 0.67)])
def test_backward_formulas_equal_autograd(L, BLKQ, ratio):
    q, k, v = _rand(1, 2, L, 16, seed=3)
    do = torch.randn(1, 2, L, 16, dtype=torch.float64, generator=torch.Generator().manual_seed(9))
    m, lut, T = O.get_block_map(q.float(), k.float(), ratio, BLKQ, 64)
    o_ref, dq_ref, dk_ref, dv_ref = _autograd_reference(q, k, v, m, do, BLKQ)
    o, lse = O.sparse_attn_fwd_dense(q, k, v, m, BLKQ, 64)
    dq, dk, dv = O.sparse_attn_bwd_dense(q, k, v, o, do, lse, m, BLKQ, 64)
    for a, b in ((dq, dq_ref), (dk, dk_ref), (dv, dv_ref)):
        assert (a - b).abs().max() < 1e-11
    dq2, dk2, dv2 = O.sparse_attn_bwd_gather(q, k, v, o, do, lse, lut, BLKQ, 64, dtype=torch.float64)
    for a, b in ((dq2, dq_ref), (dk2, dk_ref), (dv2, dv_ref)):
        assert (a - b).abs().max() < 1e-11
    # invariants the full-size GPU tests rely on
    assert (dv.sum(-2) - do.sum(-2)).abs().max() < 1e-10            # rows of P sum to one
    assert ((q * dq).sum() - (k * dk).sum()).abs() < 1e-9           # q.k is invariant under q*a, k/a


def test_gradcheck_of_differentiable_restatement():
    g = torch.Generator().manual_seed(4)
    q, k, v = (torch.randn(1, 1, 96, 4, generator=g, dtype=torch.float64, requires_grad=True) for _ in range(3))
    w = torch.randn(4, 4, generator=g, dtype=torch.float64, requires_grad=True)
    b = torch.randn(4, generator=g, dtype=torch.float64, requires_grad=True)
    m = torch.tensor([[[[1, 0], [1, 1]]]], dtype=torch.int8)
    for fmap in ("elu", "relu", "softmax"):
        fn = lambda q, k, v, w, b: O.sla_forward_autograd(q, k, v, w, b, m, fmap, 64, 64)[0]
        assert torch.autograd.gradcheck(fn, (q, k, v, w, b), eps=1e-6, atol=1e-5, rtol=1e-4)


def test_p_dtype_rounding_is_small_and_l_unrounded():
    q, k, v = _rand(1, 1, 256, 32, seed=5, dtype=torch.bfloat16)
    m, lut, T = O.get_block_map(q, k, 0.5)
    o1, _ = O.sparse_attn_fwd_gather(q, k, v, lut, 64, 64)
    o2, _ = O.sparse_attn_fwd_gather(q, k, v, lut, 64, 64, p_dtype=torch.bfloat16)
    assert 0 < (o1 - o2).abs().max() < 5e-3


def test_qk_scale_argument():
    """``qk_scale`` (kernel.py:242, 251-252): the library attention with ``scale=`` when every block is selected;
    and doubling the scale is the same as doubling q (exact in floating point), which fixes the forward, lse and
    the factor of every gradient."""
    g = torch.Generator().manual_seed(31)
    q, k, v, do = (torch.randn(1, 2, 200, 32, generator=g) for _ in range(4))
    full = torch.ones(1, 2, 4, 4, dtype=torch.int8)
    o, lse = O.sparse_attn_fwd_dense(q, k, v, full, 64, 64, qk_scale=0.07)
    sd = torch.nn.functional.scaled_dot_product_attention(q.double(), k.double(), v.double(), scale=0.07)
    assert (o - sd).abs().max() < 1e-12
    m, lut, T = O.get_block_map(q, k, 0.5, 64, 64)
    s0 = 32 ** -0.5
    a, lse_a = O.sparse_attn_fwd_dense(q, k, v, m, 64, 64, qk_scale=2 * s0)
    b, lse_b = O.sparse_attn_fwd_dense(2 * q, k, v, m, 64, 64)
    assert torch.equal(a, b) and torch.equal(lse_a, lse_b)
    ag, _ = O.sparse_attn_fwd_gather(q, k, v, lut, 64, 64, qk_scale=2 * s0, dtype=torch.float64)
    assert (ag - a).abs().max() < 1e-12
    ga = O.sparse_attn_bwd_dense(q, k, v, a, do, lse_a, m, 64, 64, qk_scale=2 * s0)
    gb = O.sparse_attn_bwd_dense(2 * q, k, v, b, do, lse_b, m, 64, 64)
    assert (ga[0] - 2 * gb[0]).abs().max() < 1e-12       # d/dq f(2q) = 2 f'(2q)
    assert (ga[1] - gb[1]).abs().max() < 1e-12 and (ga[2] - gb[2]).abs().max() < 1e-12
    gg = O.sparse_attn_bwd_gather(q, k, v, a, do, lse_a, lut, 64, 64, qk_scale=2 * s0, dtype=torch.float64)
    for x, y in zip(gg, ga):
        assert (x - y).abs().max() < 1e-10
