"""Whole-module forward (mask -> sparse -> linear -> proj -> sum) vs the CPU oracle."""
import pytest
import torch

from conftest import cos_sim, max_abs
from oracle import sla_oracle as O
from sla_amd import SparseLinearAttention
from sla_amd.inputs import CONFIGS, make_inputs, make_proj

pytestmark = pytest.mark.gpu

TOL_ABS = 2e-2
TOL_COS = 0.999


def _module(cfg, dev, seeded=True):
    mod = SparseLinearAttention(cfg.D, cfg.topk, cfg.feature_map, cfg.BLKQ, cfg.BLKK).to(dev)
    w, b = make_proj(cfg.D)
    if seeded:
        with torch.no_grad():
            mod.proj_l.weight.copy_(w)
            mod.proj_l.bias.copy_(b)
    else:
        w, b = torch.zeros_like(w), torch.zeros_like(b)
    return mod, w, b


def test_cfg1_fp32_inputs(dev):
    cfg = CONFIGS["cfg1"]
    d = make_inputs(cfg)
    for seeded in (False, True):
        mod, w, b = _module(cfg, dev, seeded)
        o_ref, o_s, o_l, m, lut, T = O.sla_forward(d["q"], d["k"], d["v"], w, b, cfg.topk, cfg.feature_map,
                                                   linear_dtype=torch.float32)
        o, dens = mod(d["q"].to(dev), d["k"].to(dev), d["v"].to(dev), return_sparsity=True)
        assert o.dtype == torch.float32 and dens == T / m.shape[-1] == 3 / 16
        assert max_abs(o.cpu(), o_ref) <= TOL_ABS and cos_sim(o.cpu(), o_ref) >= TOL_COS


def test_cfg2_forward(dev):
    cfg = CONFIGS["cfg2"]
    d = make_inputs(cfg)
    mod, w, b = _module(cfg, dev)
    o_ref, *_ = O.sla_forward(d["q"], d["k"], d["v"], w, b, cfg.topk, cfg.feature_map, linear_dtype=torch.float32)
    o = mod(d["q"].to(dev), d["k"].to(dev), d["v"].to(dev)).cpu()
    assert o.dtype == torch.bfloat16
    assert max_abs(o, o_ref) <= TOL_ABS and cos_sim(o, o_ref) >= TOL_COS


def test_zero_init_module_returns_sparse_branch(dev):
    cfg = CONFIGS["cfg2"]
    d = make_inputs(cfg)
    mod, _, _ = _module(cfg, dev, seeded=False)
    from sla_amd import _attention, get_block_map
    q, k, v = (d[x].to(dev) for x in "qkv")
    m, lut, T = get_block_map(q, k, cfg.topk)
    o_s = _attention.apply(q, k, v, m, lut, T, 64, 64)
    assert torch.equal(mod(q, k, v), o_s)


def test_state_dict_layout_and_errors(dev):
    mod = SparseLinearAttention(128, 0.2)
    sd = mod.state_dict()
    assert set(sd) == {"proj_l.weight", "proj_l.bias"}
    assert sd["proj_l.weight"].shape == (128, 128) and sd["proj_l.weight"].dtype == torch.float32
    assert float(sd["proj_l.weight"].abs().max()) == 0.0 and float(sd["proj_l.bias"].abs().max()) == 0.0
    with pytest.raises(NotImplementedError):
        SparseLinearAttention(128, 0.2, feature_map="hedgehog")


def test_cfg3_three_heads_forward(dev):
    cfg = CONFIGS["cfg3"]
    d = make_inputs(cfg, H=3)
    mod, w, b = _module(cfg, dev)
    o_ref, *_ = O.sla_forward(d["q"], d["k"], d["v"], w, b, cfg.topk, cfg.feature_map, linear_dtype=torch.float32)
    o = mod(d["q"].to(dev), d["k"].to(dev), d["v"].to(dev)).cpu()
    assert max_abs(o, o_ref) <= TOL_ABS and cos_sim(o, o_ref) >= TOL_COS


def test_forward_in_a_hip_graph(dev):
    """The whole forward (mask builder, attention, linear branch) is capturable: the library allocates
    nothing, clears nothing with memset nodes, and under capture the module keeps all work on the capturing
    stream.  Every replay is checked against the eager result, with eager work between the replays."""
    cfg = CONFIGS["cfg2"]
    d = make_inputs(cfg, H=2)
    mod, _, _ = _module(cfg, dev)
    q, k, v = (d[x].to(dev) for x in "qkv")
    with torch.no_grad():
        ref = mod(q, k, v)
        torch.cuda.synchronize()
        s = torch.cuda.Stream(device=dev)
        s.wait_stream(torch.cuda.current_stream(dev))
        with torch.cuda.stream(s):
            mod(q, k, v)                      # warm-up on the capture stream
        torch.cuda.current_stream(dev).wait_stream(s)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            out = mod(q, k, v)
        for i in range(3):
            out.zero_()
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(out, ref), f"replay {i}"
            assert torch.equal(mod(q, k, v), ref)   # eager work between the replays
            torch.cuda.synchronize()
        # new inputs in the captured buffers
        q2 = torch.roll(q, 3, dims=2)
        ref2 = mod(q2, k, v)
        q.copy_(q2)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, ref2)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("L,D,BLKQ,fmap", [(1000, 128, 64, "elu"), (700, 128, 128, "softmax"), (333, 64, 64, "relu"),
                                            (512, 64, 128, "elu")])
def test_fused_epilogue_equals_the_two_kernel_path(dev, dtype, L, D, BLKQ, fmap):
    """sla_sparse_attn_linear_fwd == sla_sparse_attn_fwd followed by sla_linear_out_fwd(residual = o_s),
    bit for bit, for out, o_s and lse (ragged L, both block sizes, both head dims, all feature maps)."""
    from sla_amd import get_block_map
    from sla_amd.linear import linear_out_fwd, linear_state_fwd
    from sla_amd.sparse_attn import sparse_attn_fwd, sparse_attn_linear_fwd
    g = torch.Generator().manual_seed(L)
    q, k, v = (torch.randn(1, 3, L, D, generator=g).to(dtype).to(dev) for _ in range(3))
    w, b = (t.to(dev) for t in make_proj(D))
    m, lut, T = get_block_map(q, k, 0.3, BLKQ, 64)
    ws = linear_state_fwd(k, v, w, fmap)
    o_s, lse = sparse_attn_fwd(q, k, v, lut, T, BLKQ, 64, D ** -0.5)
    ref = linear_out_fwd(q, b, o_s, ws, fmap)
    out, o_s2, lse2 = sparse_attn_linear_fwd(q, k, v, lut, T, BLKQ, 64, D ** -0.5, ws, b, fmap, want_o_s=True)
    bits = lambda t: t.view(torch.int16)            # bit patterns: equal also where float16 overflowed to inf/nan
    assert torch.equal(o_s2, o_s) and torch.equal(lse2, lse)
    assert torch.equal(bits(out), bits(ref))
    out3, none, _ = sparse_attn_linear_fwd(q, k, v, lut, T, BLKQ, 64, D ** -0.5, ws, b, fmap, want_o_s=False)
    assert none is None and torch.equal(bits(out3), bits(ref))
