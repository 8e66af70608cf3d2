"""HIP block-mask builder vs the CPU oracle: index sets must be bit-exact."""
import pytest
import torch

from oracle import sla_oracle as O
from sla_amd import get_block_map, mean_pool
from sla_amd.inputs import CONFIGS, integer_inputs, make_inputs

pytestmark = pytest.mark.gpu


def _compare(q, k, ratio, BLKQ, BLKK, dev):
    m_ref, lut_ref, T_ref = O.get_block_map(q, k, ratio, BLKQ, BLKK)
    m, lut, T = get_block_map(q.to(dev), k.to(dev), ratio, BLKQ, BLKK)
    assert T == T_ref
    assert m.dtype == torch.int8 and lut.dtype == torch.int64
    assert torch.equal(m.cpu(), m_ref), f"map differs in {(m.cpu() != m_ref).sum().item()} cells"
    assert torch.equal(lut.cpu(), lut_ref)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("L,BLKQ,BLKK,ratio", [(1024, 64, 64, 0.2), (1000, 64, 64, 0.3), (777, 128, 64, 0.5),
                                               (64, 64, 64, 1.0), (130, 64, 64, 0.05)])
def test_random_inputs(dev, dtype, L, BLKQ, BLKK, ratio):
    g = torch.Generator().manual_seed(L)
    q = torch.randn(2, 3, L, 64, generator=g).to(dtype)
    k = (torch.randn(2, 3, L, 64, generator=g) + 0.7).to(dtype)
    _compare(q, k, ratio, BLKQ, BLKK, dev)


@pytest.mark.parametrize("D,dtype", [(128, torch.bfloat16), (64, torch.float16)])
def test_many_rows_of_small_blocks(dev, D, dtype):
    """256 heads of 255 x 255 blocks of 8 rows: many rows, ragged at both edges of the score tiles, both head dims
    of the matrix-core score kernel."""
    g = torch.Generator().manual_seed(D)
    q = torch.randn(2, 128, 2036, D, generator=g).to(dtype)
    k = (torch.randn(2, 128, 2036, D, generator=g) + 0.3).to(dtype)
    _compare(q, k, 0.1, 8, 8, dev)


def test_integer_inputs_with_ties(dev):
    # every sum is exact in fp32, many exact score ties: only the tie rule decides
    q, k = integer_inputs(1, 2, 2048, 128, seed=3, lo=-1, hi=1)
    m_ref, lut_ref, T = O.get_block_map(q, k, 0.25, 64, 64)
    _compare(q, k, 0.25, 64, 64, dev)


def test_all_equal_scores_pick_lowest_indices(dev):
    q = torch.zeros(1, 1, 640, 64, dtype=torch.bfloat16)
    k = torch.ones(1, 1, 640, 64, dtype=torch.bfloat16)
    m, lut, T = get_block_map(q.to(dev), k.to(dev), 0.3, 64, 64)
    assert T == 3
    assert lut.cpu().tolist() == [[[[0, 1, 2]] * 10]]


def test_cfg1_and_cfg2(dev):
    for name in ("cfg1", "cfg2"):
        cfg = CONFIGS[name]
        d = make_inputs(cfg)
        _compare(d["q"], d["k"], cfg.topk, cfg.BLKQ, cfg.BLKK, dev)


def test_cfg3_two_heads(dev):
    cfg = CONFIGS["cfg3"]
    d = make_inputs(cfg, H=2)
    _compare(d["q"], d["k"], cfg.topk, cfg.BLKQ, cfg.BLKK, dev)


def test_cfg5_shape_one_head(dev):
    cfg = CONFIGS["cfg5"]
    d = make_inputs(cfg, H=1)
    _compare(d["q"], d["k"], cfg.topk, 128, 64, dev)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_mean_pool(dev, dtype):
    g = torch.Generator().manual_seed(5)
    x = torch.randn(2, 2, 333, 128, generator=g).to(dtype)
    for BLK in (64, 128):
        ref = O.mean_pool(x, BLK)
        out = mean_pool(x.to(dev), BLK).cpu()
        assert torch.equal(out, ref)


def test_full_size_invariants(dev):
    # cfg3 at full size on the GPU only: structural properties of the outputs
    cfg = CONFIGS["cfg3"]
    d = make_inputs(cfg, H=4)
    m, lut, T = get_block_map(d["q"].to(dev), d["k"].to(dev), cfg.topk, 64, 64)
    assert T == 25
    assert bool((m.sum(-1) == T).all())
    assert bool((lut[..., 1:] > lut[..., :-1]).all())
    assert bool((torch.gather(m, -1, lut) == 1).all())
    # adding a constant vector to every key must not change the selection (smoothing removes it)
    # on exact-arithmetic inputs
    q, k = integer_inputs(1, 2, 4096, 128, seed=9)
    k = torch.cat([k[:, :, :2048], -k[:, :, :2048]], dim=2)      # column means are exactly 0
    m1, lut1, _ = get_block_map(q.to(dev), k.to(dev), 0.1, 64, 64)
    m2, lut2, _ = get_block_map(q.to(dev), (k.float() + 8.0).to(k.dtype).to(dev), 0.1, 64, 64)
    assert torch.equal(lut1, lut2)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_negative_scores_and_wide_rows(dev, dtype):
    # all pooled scores negative (threshold key is a negative number) and N beyond 512 / 1280 / 2048
    g = torch.Generator().manual_seed(77)
    for L, ratio in ((64 * 70, 0.1), (64 * 600, 0.05), (64 * 1300, 0.02), (64 * 2100, 0.01)):
        q = (torch.rand(1, 1, L, 32, generator=g) + 0.5).to(dtype)
        k = -(torch.rand(1, 1, L, 32, generator=g) * torch.linspace(0.5, 2.0, L).view(1, 1, L, 1) + 0.5).to(dtype)
        _compare(q, k, ratio, 64, 64, dev)


def test_widest_supported_row(dev):
    # 4096 key blocks is the limit of the top-k kernel (the keys of four rows share 64 KB of LDS); 4097 is refused
    g = torch.Generator().manual_seed(78)
    L = 64 * 4096
    q = (torch.rand(1, 1, L, 32, generator=g) - 0.3).to(torch.bfloat16)
    k = (torch.rand(1, 1, L, 32, generator=g) * torch.linspace(0.5, 2.0, L).view(1, 1, L, 1) - 0.6).to(torch.bfloat16)
    _compare(q, k, 0.01, 128, 64, dev)
    with pytest.raises(AssertionError, match="4096"):
        get_block_map(torch.zeros(1, 1, L + 1, 32, dtype=torch.bfloat16, device=dev),
                      torch.zeros(1, 1, L + 1, 32, dtype=torch.bfloat16, device=dev), 0.01, 128, 64)
