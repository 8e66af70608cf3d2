"""The DiT-style caller around the operator: layouts, state_dict round trip, gradients reach every parameter."""
import pytest
import torch

from conftest import cos_sim
from oracle import sla_oracle as O
from sla_amd import SLASelfAttention

pytestmark = pytest.mark.gpu


def _block(dev, seed=0):
    torch.manual_seed(seed)
    blk = SLASelfAttention(dim=256, num_heads=2, topk=0.25, feature_map="elu").to(dev).to(torch.bfloat16)
    blk.attn.proj_l.float()                     # proj_l stays fp32 as in the reference module
    with torch.no_grad():
        blk.attn.proj_l.weight.normal_(0, 128 ** -0.5)
        blk.attn.proj_l.bias.normal_(0, 0.1)
    return blk


def test_block_matches_oracle_and_round_trips(dev):
    blk = _block(dev)
    x = torch.randn(2, 640, 256, device=dev, dtype=torch.bfloat16)
    with torch.no_grad():
        y = blk(x)
        # the same block with the attention replaced by the CPU oracle
        qkv = blk.qkv(x).view(2, 640, 3, 2, 128).permute(2, 0, 3, 1, 4).contiguous().cpu()
        o_ref, *_ = O.sla_forward(qkv[0], qkv[1], qkv[2], blk.attn.proj_l.weight.cpu(), blk.attn.proj_l.bias.cpu(), 0.25,
                                  "elu", linear_dtype=torch.float32)
        y_ref = blk.proj(o_ref.to(dev).to(torch.bfloat16).transpose(1, 2).reshape(2, 640, 256))
    assert y.shape == x.shape and cos_sim(y.cpu(), y_ref.cpu()) >= 0.999
    sd = blk.state_dict()
    assert {"qkv.weight", "qkv.bias", "attn.proj_l.weight", "attn.proj_l.bias", "proj.weight", "proj.bias"} == set(sd)
    assert sd["attn.proj_l.weight"].dtype == torch.float32
    blk2 = _block(dev, seed=1)
    blk2.load_state_dict(sd)
    with torch.no_grad():
        assert torch.equal(blk2(x), y)


def test_gradients_reach_all_parameters(dev):
    blk = _block(dev)
    x = torch.randn(1, 512, 256, device=dev, dtype=torch.bfloat16, requires_grad=True)
    blk(x).float().square().mean().backward()
    assert x.grad is not None and torch.isfinite(x.grad.float()).all()
    for n, p in blk.named_parameters():
        assert p.grad is not None and torch.isfinite(p.grad.float()).all() and float(p.grad.float().abs().max()) > 0, n


def test_quantised_block_loads_the_16_bit_block_and_agrees(dev):
    """Train with SLA, serve with SageSLA: same parameter names, outputs agree to the quantised operator's bound
    (both blocks at 128/64 blocks, so both attend to the same key blocks)."""
    torch.manual_seed(3)
    kw = dict(dim=256, num_heads=2, topk=0.25, feature_map="softmax")
    blk = SLASelfAttention(BLKQ=128, BLKK=64, **kw).to(dev).to(torch.bfloat16)
    blk.attn.proj_l.float()
    with torch.no_grad():
        blk.attn.proj_l.weight.normal_(0, 128 ** -0.5)
        blk.attn.proj_l.bias.normal_(0, 0.1)
    qblk = SLASelfAttention(quantized=True, **kw).to(dev).to(torch.bfloat16)
    qblk.attn.proj_l.float()
    qblk.load_state_dict(blk.state_dict())
    x = torch.randn(2, 1000, 256, device=dev, dtype=torch.bfloat16)
    with torch.no_grad():
        y, yq = blk(x), qblk(x)
    assert yq.shape == y.shape and cos_sim(yq.cpu(), y.cpu()) >= 0.995
    with pytest.raises(NotImplementedError):
        SLASelfAttention(quantized=True, linear_mode="complement", **kw)
