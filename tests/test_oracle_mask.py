"""Pins the block-mask part of the CPU oracle without the reference (it ships no tests):
library routines, brute force on tiny inputs, exact-arithmetic inputs and invariants."""
import pytest
import torch

from oracle import sla_oracle as O
from sla_amd.inputs import integer_inputs


def test_topk_count_table():
    # T = min(N, int(ratio*N)) for the five configurations (N = ceil(L/64))
    assert O.topk_count(16, 0.2) == 3
    assert O.topk_count(64, 0.2) == 12
    assert O.topk_count(512, 0.05) == 25
    assert O.topk_count(1182, 0.05) == 59
    assert O.topk_count(512, 0.1) == 51
    assert O.topk_count(10, 1.5) == 10
    assert O.topk_count(10, 0.01) == 0


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-6), (torch.bfloat16, 8e-3), (torch.float16, 1e-3)])
def test_mean_pool_full_blocks_closed_form(dtype, tol):
    x = torch.randn(2, 2, 256, 32).to(dtype)
    ref = x.view(2, 2, 4, 64, 32).double().mean(-2)
    out = O.mean_pool(x, 64)
    assert out.dtype == dtype and out.shape == (2, 2, 4, 32)
    assert (out.double() - ref).abs().max() <= tol


def test_mean_pool_tail_divides_by_real_count():
    x = torch.ones(1, 1, 70, 8)
    x[..., 64:, :] = 3.0
    out = O.mean_pool(x, 64)
    assert torch.equal(out[0, 0, 0], torch.ones(8))
    assert torch.equal(out[0, 0, 1], torch.full((8,), 3.0))     # 6 rows of 3 / 6, not / 64


def test_mean_pool_exact_on_integers():
    x = torch.randint(-4, 5, (1, 2, 200, 16)).to(torch.bfloat16)
    out = O.mean_pool(x, 64)
    for i, (a, b) in enumerate([(0, 64), (64, 128), (128, 192), (192, 200)]):
        exact = (x[:, :, a:b].double().sum(-2) / (b - a)).to(torch.bfloat16)
        assert torch.equal(out[:, :, i], exact)


def test_k_column_mean_matches_library():
    k = torch.randn(2, 3, 1000, 16)
    assert (O.k_column_mean(k) - torch.mean(k, dim=-2, keepdim=True)).abs().max() < 1e-6
    kb = (torch.randn(1, 2, 500, 16) + 2).to(torch.bfloat16)
    ref = torch.mean(kb.double(), dim=-2, keepdim=True)
    assert (O.k_column_mean(kb).double() - ref).abs().max() < 1.6e-2   # one bf16 ulp at |x|~2
    ki = torch.randint(-3, 4, (1, 1, 640, 8)).to(torch.bfloat16)
    assert torch.equal(O.k_column_mean(ki), (ki.double().sum(-2, keepdim=True) / 640).to(torch.bfloat16))


def test_pooled_score_matches_matmul():
    a, b = torch.randn(2, 5, 32), torch.randn(2, 7, 32)
    ref = a.double() @ b.double().transpose(-1, -2)
    assert (O.pooled_score(a, b).double() - ref).abs().max() < 1e-5
    ai = torch.randint(-3, 4, (1, 4, 64)).to(torch.bfloat16)
    bi = torch.randint(-3, 4, (1, 6, 64)).to(torch.bfloat16)
    assert torch.equal(O.pooled_score(ai, bi), (ai.double() @ bi.double().transpose(-1, -2)).to(torch.bfloat16))


def _brute_topk(row, T):
    order = sorted(range(len(row)), key=lambda i: (-row[i], i))
    return sorted(order[:T])


def test_select_topk_brute_force_with_planted_ties():
    g = torch.Generator().manual_seed(0)
    score = torch.randint(0, 6, (3, 4, 23), generator=g).float()   # few distinct values -> many ties
    score[0, 0, :] = 1.0
    score[0, 1, 5] = -0.0
    score[0, 1, 7] = 0.0
    for T in (1, 5, 22, 23):
        lut = O.select_topk(score, T)
        for a in range(3):
            for b in range(4):
                assert lut[a, b].tolist() == _brute_topk(score[a, b].tolist(), T)
    assert O.select_topk(score, 5)[0, 0].tolist() == [0, 1, 2, 3, 4]


def test_select_topk_equals_library_topk_without_ties():
    score = torch.randn(4, 50, dtype=torch.float64).float()
    assert score.unique().numel() == score.numel()
    lib = torch.topk(score, 9, dim=-1, sorted=False).indices.sort(-1).values
    assert torch.equal(O.select_topk(score, 9), lib)


def test_negative_and_positive_zero_tie():
    score = torch.tensor([[-0.0, 0.0, -1.0, 0.0]])
    assert O.select_topk(score, 2).tolist() == [[0, 1]]


@pytest.mark.parametrize("L,BLKQ,BLKK,ratio", [(512, 64, 64, 0.25), (500, 128, 64, 0.4), (100, 64, 64, 5.0)])
def test_block_map_invariants(L, BLKQ, BLKK, ratio):
    q, k = torch.randn(1, 2, L, 32), torch.randn(1, 2, L, 32)
    m, lut, T = O.get_block_map(q, k, ratio, BLKQ, BLKK)
    M, N = -(-L // BLKQ), -(-L // BLKK)
    assert m.shape == (1, 2, M, N) and m.dtype == torch.int8 and lut.shape == (1, 2, M, T)
    assert T == min(N, int(ratio * N))
    assert bool((m.sum(-1) == T).all())
    assert bool((torch.gather(m, -1, lut) == 1).all())
    assert bool((lut[..., 1:] > lut[..., :-1]).all())
    if ratio >= 1:
        assert bool((m == 1).all())


def test_block_map_ignores_constant_key_offset():
    # smoothing subtracts the column mean; on exact-arithmetic inputs a constant shift of all
    # keys therefore leaves the selection unchanged (and without smoothing it would not)
    q, k = integer_inputs(1, 2, 1024, 32, seed=4)
    k = torch.cat([k[:, :, :512], -k[:, :, :512]], dim=2)        # column means are exactly 0
    m1, lut1, _ = O.get_block_map(q, k, 0.25)
    m2, lut2, _ = O.get_block_map(q, (k.float() + 8).to(k.dtype), 0.25)
    assert torch.equal(lut1, lut2)
    raw = O.select_topk(O.pooled_score(O.mean_pool(q, 64), O.mean_pool((k.float() + 8).to(k.dtype), 64)), lut1.shape[-1])
    assert not torch.equal(raw, lut1)


def test_block_map_selects_blocks_with_highest_exact_scores():
    # independent float64 restatement on tie-free data: the chosen set is the true top-T
    g = torch.Generator().manual_seed(2)
    q = torch.randn(1, 1, 640, 16, dtype=torch.float64, generator=g)
    k = torch.randn(1, 1, 640, 16, dtype=torch.float64, generator=g)
    pq = q.view(1, 1, 10, 64, 16).mean(-2)
    pk = (k - k.mean(-2, keepdim=True)).view(1, 1, 10, 64, 16).mean(-2)
    score = pq @ pk.transpose(-1, -2)
    lib = torch.topk(score, 3, dim=-1).indices.sort(-1).values
    gap = (score.sort(-1, descending=True).values[..., 2] - score.sort(-1, descending=True).values[..., 3]).min()
    assert gap > 1e-5
    _, lut, _ = O.get_block_map(q.float(), k.float(), 0.3)
    assert torch.equal(lut, lib)
