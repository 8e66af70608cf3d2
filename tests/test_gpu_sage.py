"""SageSLA quantised forward: integer/fp8 tensors bit-exact vs the oracle's quantisers, attention
output cosine similarity >= 0.995 vs the fp32 math (the stated contract; the third-party kernels the
reference calls are not available, so their exact rounding is parity-unpinned)."""
import pytest
import torch

from conftest import cos_sim
from oracle import sla_oracle as O
from sla_amd import SageSparseLinearAttention
from sla_amd.inputs import CONFIGS, make_inputs, make_proj
from sla_amd import get_block_map
from sla_amd.sage import quant_qk, quant_v, sage_attn_fwd, sage_prepare

pytestmark = pytest.mark.gpu

TOL_COS = 0.995


def _qkv(L, D, seed, bias=2.0):
    g = torch.Generator().manual_seed(seed)
    q, k, v = (torch.randn(1, 3, L, D, generator=g) for _ in range(3))
    k = k + bias * torch.randn(1, 3, 1, D, generator=g)
    return q.to(torch.bfloat16), k.to(torch.bfloat16), v.to(torch.bfloat16)


@pytest.mark.parametrize("L,D", [(512, 128), (1000, 128), (333, 64)])
def test_quantisers_bit_exact(dev, L, D):
    q, k, v = _qkv(L, D, L)
    q8r, qsr, k8r, ksr, _ = O.sage_quant_qk(q, k, 128, 64)
    v8r, vsr = O.sage_quant_v(v)
    q8, qs, k8, ks = quant_qk(q.to(dev), k.to(dev))
    v8, vs = quant_v(v.to(dev))
    assert torch.equal(qs.cpu(), qsr) and torch.equal(ks.cpu(), ksr) and torch.equal(vs.cpu(), vsr)
    assert torch.equal(q8.cpu(), q8r) and torch.equal(k8.cpu(), k8r)
    assert torch.equal(v8.cpu().view(torch.uint8), v8r.view(torch.uint8))


def test_int8_quantiser_near_half_integers(dev):
    """The kernel rounds x * (1 / scale) and takes the division only where that product lies close to a half-integer.
    Two million elements hold a few hundred such quotients by chance; block 0 of q is planted with exact ties
    (scale 1: values k + 0.5 round to even) and block 1 with a scale of 3 / 127, whose reciprocal is inexact."""
    g = torch.Generator().manual_seed(5)
    q = torch.randn(1, 2, 8192, 128, generator=g)
    k = torch.randn(1, 2, 8192, 128, generator=g) + torch.randn(1, 2, 1, 128, generator=g)
    halves = (torch.arange(128 * 128) % 253 - 126).float() + 0.5        # -125.5 .. 126.5, exact in bf16
    q[0, 0, :128] = halves.view(128, 128)
    q[0, 0, 0, 0] = 127.0
    q[0, 0, 128:256] = (torch.arange(128 * 128) % 255 - 127).float().view(128, 128) * (3.0 / 254.0)
    q[0, 0, 128, 0] = 3.0
    q, k = q.to(torch.bfloat16), k.to(torch.bfloat16)
    q8r, qsr, k8r, ksr, _ = O.sage_quant_qk(q, k, 128, 64)
    quotient = q[0, 0].float().view(64, 128 * 128) / qsr[0, 0].view(64, 1)
    assert int(((quotient - quotient.round()).abs() > 0.4999).sum()) > 100     # the slow path is exercised
    q8, qs, k8, ks = quant_qk(q.to(dev), k.to(dev))
    assert torch.equal(qs.cpu(), qsr) and torch.equal(ks.cpu(), ksr)
    assert torch.equal(q8.cpu(), q8r) and torch.equal(k8.cpu(), k8r)
    *_, q8p, qsp, k8p, ksp, _, _ = sage_prepare(q.to(dev), k.to(dev), None, 0.25)
    assert torch.equal(q8p.cpu(), q8r) and torch.equal(k8p.cpu(), k8r)


@pytest.mark.parametrize("L,D,ratio,dtype", [(512, 128, 0.5, torch.bfloat16), (1000, 128, 0.3, torch.bfloat16),
                                              (333, 64, 0.5, torch.float16), (2048, 128, 0.1, torch.float16),
                                              (100, 64, 1.0, torch.bfloat16)])
def test_one_call_preparation_equals_the_separate_calls(dev, L, D, ratio, dtype):
    """Block map + both quantisers in one call: bit-identical to get_block_map, quant_qk, quant_v and to the oracle's map."""
    q, k, v = (x.to(dtype) for x in _qkv(L, D, 7 * L + D))
    m_ref, lut_ref, T_ref = O.get_block_map(q, k, ratio, 128, 64)
    qd, kd, vd = q.to(dev), k.to(dev), v.to(dev)
    m, lut, T, q8, qs, k8, ks, v8, vs = sage_prepare(qd, kd, vd, ratio)
    assert T == T_ref and torch.equal(lut.cpu(), lut_ref) and torch.equal(m.cpu(), m_ref)
    # without v: the same map and q / k results, the v part left to the caller
    m3, lut3, T3, q8c, qsc, k8c, ksc, none_a, none_b = sage_prepare(qd, kd, None, ratio)
    assert none_a is None and none_b is None and T3 == T and torch.equal(lut3, lut) and torch.equal(m3, m)
    assert torch.equal(q8c, q8) and torch.equal(qsc, qs) and torch.equal(k8c, k8) and torch.equal(ksc, ks)
    m2, lut2, T2 = get_block_map(qd, kd, ratio, 128, 64)
    assert T2 == T and torch.equal(lut2, lut) and torch.equal(m2, m)
    q8b, qsb, k8b, ksb = quant_qk(qd, kd)
    v8b, vsb = quant_v(vd)
    assert torch.equal(q8, q8b) and torch.equal(qs, qsb) and torch.equal(k8, k8b) and torch.equal(ks, ksb)
    assert torch.equal(v8.view(torch.uint8), v8b.view(torch.uint8)) and torch.equal(vs, vsb)


@pytest.mark.parametrize("L,D,dtype,fmap,v_range", [(512, 128, torch.bfloat16, "softmax", 448.0), (1000, 128, torch.bfloat16, "elu", 2.25),
                                                    (333, 64, torch.float16, "relu", 448.0), (4100, 128, torch.float16, "elu", 448.0)])
def test_state_build_with_v_quantised_in_the_same_call(dev, L, D, dtype, fmap, v_range):
    """The state kernel's column maxima of |v| instead of the quantiser's own pass over v: the states, the FP8 copy of v
    and its scales are bit for bit those of the two separate calls (and so of the oracle's quantiser), also on a
    (B, L, H, D) activation read in place."""
    from sla_amd.linear import linear_out_fwd, linear_state_fwd, linear_state_quant_v_fwd
    q, k, v = (x.to(dtype) for x in _qkv(L, D, 11 * L + D))
    v = v * torch.logspace(-2, 1, D).to(dtype)            # channels of very different size
    w, b = make_proj(D)
    qd, kd, vd, wd, bd = q.to(dev), k.to(dev), v.to(dev), w.to(dev), b.to(dev)
    ws_ref = linear_state_fwd(kd, vd, wd, fmap)
    out_ref = linear_out_fwd(qd, bd, None, ws_ref, fmap)
    v8_ref, vs_ref = quant_v(vd, v_range)
    ws, v8, vs = linear_state_quant_v_fwd(kd, vd, wd, fmap, v_range)
    assert torch.equal(vs, vs_ref) and torch.equal(v8.view(torch.uint8), v8_ref.view(torch.uint8))
    assert torch.equal(linear_out_fwd(qd, bd, None, ws, fmap), out_ref)          # (the states, through what reads them)
    v8o, vso = O.sage_quant_v(v, v_range)
    assert torch.equal(vs.cpu(), vso) and torch.equal(v8.cpu().view(torch.uint8), v8o.view(torch.uint8))
    # rows as they lie in a (B, L, H, D) activation
    kt, vt = (x.transpose(1, 2).contiguous().transpose(1, 2) for x in (kd, vd))
    ws2, v82, vs2 = linear_state_quant_v_fwd(kt, vt, wd, fmap, v_range)
    assert torch.equal(vs2, vs_ref) and torch.equal(v82.view(torch.uint8), v8_ref.view(torch.uint8))
    assert torch.equal(linear_out_fwd(qd, bd, None, ws2, fmap), out_ref)


@pytest.mark.parametrize("L,D,ratio", [(512, 128, 0.5), (1000, 128, 0.3), (333, 64, 0.5), (2048, 128, 0.1)])
def test_attention_vs_fp32_and_vs_quantised_oracle(dev, L, D, ratio):
    q, k, v = _qkv(L, D, L + 1)
    m, lut, T = O.get_block_map(q, k, ratio, 128, 64)
    ref, _ = O.sparse_attn_fwd_gather(q, k, v, lut, 128, 64)
    ref_q = O.sage_sparse_attn_fwd(q, k, v, lut, 128, 64)
    q8, qs, k8, ks = quant_qk(q.to(dev), k.to(dev))
    v8, vs = quant_v(v.to(dev))
    o = sage_attn_fwd(q8, qs, k8, ks, v8, vs, lut.to(dev), T, torch.bfloat16).cpu()
    assert cos_sim(o, ref) >= TOL_COS
    # Same quantised scheme as the oracle.  The kernel rounds P to e4m3 against a reference maximum that may
    # lag the running maximum by up to 2 (log2 units) and uses 448/4 as P scale; the oracle rounds against the
    # running maximum with scale 448: equal up to e4m3 rounding of P at slightly different points.
    assert cos_sim(o, ref_q) >= 0.9995
    assert float((o.float() - ref_q).abs().max()) <= 3e-2
    assert float((o.float() - ref).abs().max()) <= float((ref_q - ref).abs().max()) * 1.5 + 5e-3


def test_full_selection_vs_sdpa(dev):
    q, k, v = _qkv(640, 128, 5)
    lut = torch.arange(10).expand(1, 3, 5, 10).contiguous()
    q8, qs, k8, ks = quant_qk(q.to(dev), k.to(dev))
    v8, vs = quant_v(v.to(dev))
    o = sage_attn_fwd(q8, qs, k8, ks, v8, vs, lut.to(dev), 10, torch.bfloat16).cpu()
    ref = torch.nn.functional.scaled_dot_product_attention(q.float(), k.float(), v.float())
    assert cos_sim(o, ref) >= TOL_COS


def test_module_cfg5_two_heads(dev):
    cfg = CONFIGS["cfg5"]
    d = make_inputs(cfg, H=2)
    w, b = make_proj(cfg.D)
    mod = SageSparseLinearAttention(cfg.D, cfg.topk, cfg.feature_map, BLKQ=128, BLKK=64).to(dev)
    with torch.no_grad():
        mod.proj_l.weight.copy_(w)
        mod.proj_l.bias.copy_(b)
    o, dens = mod(d["q"].to(dev), d["k"].to(dev), d["v"].to(dev), return_sparsity=True)
    assert dens == 51 / 512
    o_ref, o_s, o_l, m, lut, T = O.sla_forward(d["q"], d["k"], d["v"], w, b, cfg.topk, cfg.feature_map, 128, 64,
                                               linear_dtype=torch.float32)
    assert cos_sim(o.cpu(), o_ref) >= TOL_COS
    with pytest.raises(AssertionError):
        SageSparseLinearAttention(128, 0.1, BLKQ=64, BLKK=64)
    with pytest.raises(NotImplementedError):
        SageSparseLinearAttention(128, 0.1, feature_map="hedgehog")


def test_quantised_forward_in_a_hip_graph(dev):
    """The quantised forward is capturable too (under capture the k/v state build and the v quantiser stay on the
    capturing stream); every replay is checked against the eager result, with eager work between the replays."""
    cfg = CONFIGS["cfg2"]
    d = make_inputs(cfg, H=2)
    w, b = make_proj(cfg.D)
    mod = SageSparseLinearAttention(cfg.D, cfg.topk, "elu").to(dev)
    q, k, v = (d[x].to(dev) for x in "qkv")
    with torch.no_grad():
        mod.proj_l.weight.copy_(w)
        mod.proj_l.bias.copy_(b)
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
        v2 = torch.roll(v, 5, dims=2)
        ref2 = mod(q, k, v2)
        v.copy_(v2)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, ref2)
