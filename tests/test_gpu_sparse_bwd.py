"""HIP block-sparse attention backward vs the CPU oracle (tolerance 2e-2 abs, cos >= 0.999)."""
import pytest
import torch

from conftest import cos_sim, max_abs
from oracle import sla_oracle as O
from sla_amd import _attention
from sla_amd.inputs import CONFIGS, make_inputs

pytestmark = pytest.mark.gpu

TOL_ABS = 2e-2
TOL_COS = 0.999


def _grads(q, k, v, do, m, lut, T, BLKQ, dev):
    qd, kd, vd = (t.to(dev).requires_grad_(True) for t in (q, k, v))
    o = _attention.apply(qd, kd, vd, m.to(dev), lut.to(dev), T, BLKQ, 64)
    o.backward(do.to(dev))
    torch.cuda.synchronize()
    return o.detach().cpu(), qd.grad.cpu(), kd.grad.cpu(), vd.grad.cpu()


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("L,D,BLKQ,ratio", [(512, 128, 64, 0.25), (1000, 128, 64, 0.3), (777, 128, 128, 0.4),
                                            (640, 64, 64, 0.5), (333, 64, 128, 0.34), (50, 128, 64, 1.0)])
def test_against_dense_oracle(dev, dtype, L, D, BLKQ, ratio):
    g = torch.Generator().manual_seed(L + D)
    q, k, v, do = (torch.randn(1, 3, L, D, generator=g).to(dtype) for _ in range(4))
    m, lut, T = O.get_block_map(q, k, ratio, BLKQ, 64)
    o_ref, lse_ref = O.sparse_attn_fwd_dense(q, k, v, m, BLKQ, 64)
    refs = O.sparse_attn_bwd_dense(q, k, v, o_ref, do, lse_ref, m, BLKQ, 64)
    o, dq, dk, dv = _grads(q, k, v, do, m, lut, T, BLKQ, dev)
    for name, a, b in zip(("dq", "dk", "dv"), (dq, dk, dv), refs):
        assert a.dtype == dtype
        assert max_abs(a, b) <= TOL_ABS, name
        assert cos_sim(a, b) >= TOL_COS, name


@pytest.mark.parametrize("H,L,dtype,ratio", [(64, 1024, torch.bfloat16, 0.25), (70, 970, torch.float16, 0.3),
                                              (65, 1000, torch.bfloat16, 0.2)])
def test_many_query_blocks(dev, H, L, dtype, ratio):
    """At least 1024 query blocks of 64 rows at head dim 128: the launch size from which dQ comes from the kernel that
    gives a whole query block to one wave (and dK / dV from its counterpart); ragged last key blocks with fewer and
    with more than 32 rows."""
    g = torch.Generator().manual_seed(H + L)
    q, k, v, do = (torch.randn(1, H, L, 128, generator=g).to(dtype) for _ in range(4))
    m, lut, T = O.get_block_map(q, k, ratio, 64, 64)
    o_ref, lse_ref = O.sparse_attn_fwd_dense(q, k, v, m, 64, 64)
    refs = O.sparse_attn_bwd_dense(q, k, v, o_ref, do, lse_ref, m, 64, 64)
    o, dq, dk, dv = _grads(q, k, v, do, m, lut, T, 64, dev)
    for name, a, b in zip(("dq", "dk", "dv"), (dq, dk, dv), refs):
        assert torch.isfinite(a.float()).all(), name
        assert max_abs(a, b) <= TOL_ABS, name
        assert cos_sim(a, b) >= TOL_COS, name


@pytest.mark.parametrize("H,L,dtype,ratio", [(64, 1024, torch.bfloat16, 0.25),   # whole 128-row blocks
                                              (70, 970, torch.float16, 0.3),      # second half of the last block ragged
                                              (68, 960, torch.bfloat16, 0.25)])   # last block without a second half
def test_many_query_blocks_of_128_rows(dev, H, L, dtype, ratio):
    """BLOCK_M = 128 (the reference's evaluate/bench_kernel.py:60-61) at the same launch sizes: the kernels above walk a
    128-row query block as its two halves, both following the block's row of the table / its entry of the lists."""
    g = torch.Generator().manual_seed(H + L + 1)
    q, k, v, do = (torch.randn(1, H, L, 128, generator=g).to(dtype) for _ in range(4))
    m, lut, T = O.get_block_map(q, k, ratio, 128, 64)
    o_ref, lse_ref = O.sparse_attn_fwd_dense(q, k, v, m, 128, 64)
    refs = O.sparse_attn_bwd_dense(q, k, v, o_ref, do, lse_ref, m, 128, 64)
    o, dq, dk, dv = _grads(q, k, v, do, m, lut, T, 128, dev)
    assert max_abs(o, o_ref) <= TOL_ABS
    for name, a, b in zip(("dq", "dk", "dv"), (dq, dk, dv), refs):
        assert torch.isfinite(a.float()).all(), name
        assert max_abs(a, b) <= TOL_ABS, name
        assert cos_sim(a, b) >= TOL_COS, name


def test_full_selection_equals_sdpa_autograd(dev):
    g = torch.Generator().manual_seed(21)
    q, k, v, do = (torch.randn(2, 2, 300, 128, generator=g).to(torch.bfloat16) for _ in range(4))
    N = 5
    lut = torch.arange(N).expand(2, 2, N, N).contiguous()
    m = torch.ones(2, 2, N, N, dtype=torch.int8)
    qr, kr, vr = (t.double().requires_grad_(True) for t in (q, k, v))
    torch.nn.functional.scaled_dot_product_attention(qr, kr, vr).backward(do.double())
    o, dq, dk, dv = _grads(q, k, v, do, m, lut, N, 64, dev)
    for a, b in ((dq, qr.grad), (dk, kr.grad), (dv, vr.grad)):
        assert max_abs(a, b) <= TOL_ABS and cos_sim(a, b) >= TOL_COS


def test_cfg2_backward(dev):
    cfg = CONFIGS["cfg2"]
    d = make_inputs(cfg)
    m, lut, T = O.get_block_map(d["q"], d["k"], cfg.topk, 64, 64)
    o_ref, lse_ref = O.sparse_attn_fwd_gather(d["q"], d["k"], d["v"], lut, 64, 64)
    refs = O.sparse_attn_bwd_gather(d["q"], d["k"], d["v"], o_ref, d["do"], lse_ref, lut, 64, 64)
    o, dq, dk, dv = _grads(d["q"], d["k"], d["v"], d["do"], m, lut, T, 64, dev)
    for name, a, b in zip(("dq", "dk", "dv"), (dq, dk, dv), refs):
        assert max_abs(a, b) <= TOL_ABS, name
        assert cos_sim(a, b) >= TOL_COS, name


def test_cfg3_shape_invariants_and_two_heads(dev):
    # long sequence with a partial last block: oracle on two heads + size-independent identities
    cfg = CONFIGS["cfg3"]
    d = make_inputs(cfg, H=2, with_do=True)
    m, lut, T = O.get_block_map(d["q"], d["k"], cfg.topk, 64, 64)
    o_ref, lse_ref = O.sparse_attn_fwd_gather(d["q"], d["k"], d["v"], lut, 64, 64)
    refs = O.sparse_attn_bwd_gather(d["q"], d["k"], d["v"], o_ref, d["do"], lse_ref, lut, 64, 64)
    o, dq, dk, dv = _grads(d["q"], d["k"], d["v"], d["do"], m, lut, T, 64, dev)
    for name, a, b in zip(("dq", "dk", "dv"), (dq, dk, dv), refs):
        assert max_abs(a, b) <= TOL_ABS, name
        assert cos_sim(a, b) >= TOL_COS, name
    # rows of P sum to one: sum_keys dV == sum_queries dO
    assert max_abs(dv.double().sum(-2), d["do"].double().sum(-2)) <= 0.5
    # q.k is invariant under (q*a, k/a): sum q.dq == sum k.dk
    # (signed sums of bf16-rounded terms: the tolerance scales with the sum of magnitudes)
    ta, tb = d["q"].double() * dq.double(), d["k"].double() * dk.double()
    assert abs(ta.sum() - tb.sum()) <= 1e-3 * float(ta.abs().sum() + tb.abs().sum())


def test_more_query_blocks_than_one_round_of_the_list_builder(dev):
    """L = 40000 at BLKQ 64 is 625 query blocks: the per-key-block lists are built in two rounds of row chunks and
    the last round is ragged.  dK / dV (the consumers of the lists) against the gather oracle."""
    g = torch.Generator().manual_seed(41)
    L, D = 40000, 64
    q, k, v, do = (torch.randn(1, 1, L, D, generator=g).to(torch.bfloat16) for _ in range(4))
    m, lut, T = O.get_block_map(q, k, 0.01, 64, 64)
    assert m.shape[-2] == 625 and T == 6
    o_ref, lse_ref = O.sparse_attn_fwd_gather(q, k, v, lut, 64, 64)
    refs = O.sparse_attn_bwd_gather(q, k, v, o_ref, do, lse_ref, lut, 64, 64)
    o, dq, dk, dv = _grads(q, k, v, do, m, lut, T, 64, dev)
    for name, a, b in zip(("dq", "dk", "dv"), (dq, dk, dv), refs):
        assert max_abs(a, b) <= TOL_ABS, name
        assert cos_sim(a, b) >= TOL_COS, name


@pytest.mark.parametrize("L,D,BLKQ,T,sinks", [(12800, 64, 64, 8, 2), (12790, 128, 128, 6, 1), (9000, 128, 64, 5, 5)])
def test_key_blocks_selected_by_every_query_block(dev, L, D, BLKQ, T, sinks):
    """Attention "sinks": a few key blocks are in every look-up row, so their lists hold every query block and are cut
    into segments whose fp32 partials a second kernel adds; the other key blocks keep short lists."""
    g = torch.Generator().manual_seed(L + T)
    q, k, v, do = (torch.randn(1, 2, L, D, generator=g).to(torch.bfloat16) for _ in range(4))
    M, N = -(-L // BLKQ), -(-L // 64)
    lut = torch.empty(1, 2, M, T, dtype=torch.int64)
    for h in range(2):
        for i in range(M):
            rest = torch.randperm(N - sinks, generator=g)[:T - sinks] + sinks
            lut[0, h, i] = torch.cat([torch.arange(sinks), rest]).sort().values
    m = torch.zeros(1, 2, M, N, dtype=torch.int8).scatter_(-1, lut, 1)
    assert int(m[0, 0, :, 0].sum()) == M > 64
    o_ref, lse_ref = O.sparse_attn_fwd_gather(q, k, v, lut, BLKQ, 64)
    refs = O.sparse_attn_bwd_gather(q, k, v, o_ref, do, lse_ref, lut, BLKQ, 64)
    o, dq, dk, dv = _grads(q, k, v, do, m, lut, T, BLKQ, dev)
    for name, a, b in zip(("dq", "dk", "dv"), (dq, dk, dv), refs):
        # (a sink block's dK / dV rows are sums over all L queries: scale the absolute bound with their size)
        scale = max(1.0, float(b.abs().max()) / 8)
        assert max_abs(a, b) <= TOL_ABS * scale, (name, max_abs(a, b), scale)
        assert cos_sim(a, b) >= TOL_COS, name
    # the sink rows themselves, separately (they are a small part of the tensor)
    rows = slice(0, sinks * 64)
    for a, b in ((dk, refs[1]), (dv, refs[2])):
        assert cos_sim(a[:, :, rows], b[:, :, rows]) >= TOL_COS
