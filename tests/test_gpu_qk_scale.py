"""Non-default ``qk_scale`` (reference kernel.py:242, 251-252) through the forward, the backward and the quantised
forward, and the reference's e4m3 range 2.25 for v (SageSLA/core.py:129) through the quantiser and the kernel."""
import pytest
import torch

from conftest import cos_sim, max_abs
from oracle import sla_oracle as O
from sla_amd import _attention
from sla_amd.sage import V_RANGE_REFERENCE, quant_qk, quant_v, sage_attn_fwd
from sla_amd.sparse_attn import sparse_attn_fwd

pytestmark = pytest.mark.gpu

TOL_ABS = 2e-2
TOL_COS = 0.999


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("L,D,BLKQ,ratio,scale", [(512, 128, 64, 0.25, 0.05), (777, 128, 128, 0.4, 0.12),
                                                  (333, 64, 64, 0.5, 0.03), (640, 64, 128, 0.5, 0.18)])
def test_forward_and_backward_with_a_scale_of_the_callers(dev, dtype, L, D, BLKQ, ratio, scale):
    assert abs(scale - D ** -0.5) > 0.01
    g = torch.Generator().manual_seed(L + D)
    q, k, v, do = (torch.randn(1, 3, L, D, generator=g).to(dtype) for _ in range(4))
    m, lut, T = O.get_block_map(q, k, ratio, BLKQ, 64)
    o_ref, lse_ref = O.sparse_attn_fwd_dense(q, k, v, m, BLKQ, 64, qk_scale=scale)
    refs = O.sparse_attn_bwd_dense(q, k, v, o_ref, do, lse_ref, m, BLKQ, 64, qk_scale=scale)
    qd, kd, vd = (t.to(dev).requires_grad_(True) for t in (q, k, v))
    o = _attention.apply(qd, kd, vd, m.to(dev), lut.to(dev), T, BLKQ, 64, scale)
    o.backward(do.to(dev))
    _, lse = sparse_attn_fwd(qd.detach(), kd.detach(), vd.detach(), lut.to(dev), T, BLKQ, 64, scale)
    torch.cuda.synchronize()
    assert max_abs(o.cpu(), o_ref) <= TOL_ABS and cos_sim(o.cpu(), o_ref) >= TOL_COS
    assert max_abs(lse.cpu(), lse_ref) <= 1e-3 * max(1.0, float(lse_ref.abs().max()))
    for name, a, b in zip(("dq", "dk", "dv"), (qd.grad, kd.grad, vd.grad), refs):
        assert max_abs(a.cpu(), b) <= TOL_ABS, name
        assert cos_sim(a.cpu(), b) >= TOL_COS, name
    # and it is not the default scale that was used: the default's result differs by far more than the tolerance
    o_def, _ = O.sparse_attn_fwd_dense(q, k, v, m, BLKQ, 64)
    assert max_abs(o_def, o_ref) > 3 * TOL_ABS


def test_full_selection_equals_the_library_attention_with_that_scale(dev):
    g = torch.Generator().manual_seed(9)
    q, k, v, do = (torch.randn(2, 2, 300, 128, generator=g).to(torch.bfloat16) for _ in range(4))
    N = 5
    lut = torch.arange(N).expand(2, 2, N, N).contiguous()
    m = torch.ones(2, 2, N, N, dtype=torch.int8)
    qr, kr, vr = (t.double().requires_grad_(True) for t in (q, k, v))
    ref = torch.nn.functional.scaled_dot_product_attention(qr, kr, vr, scale=0.04)
    ref.backward(do.double())
    qd, kd, vd = (t.to(dev).requires_grad_(True) for t in (q, k, v))
    o = _attention.apply(qd, kd, vd, m.to(dev), lut.to(dev), N, 64, 64, 0.04)
    o.backward(do.to(dev))
    torch.cuda.synchronize()
    assert max_abs(o.cpu(), ref) <= TOL_ABS and cos_sim(o.cpu(), ref) >= TOL_COS
    for a, b in ((qd.grad, qr.grad), (kd.grad, kr.grad), (vd.grad, vr.grad)):
        assert max_abs(a.cpu(), b) <= TOL_ABS and cos_sim(a.cpu(), b) >= TOL_COS


def _qkv(L, D, seed, bias=2.0):
    g = torch.Generator().manual_seed(seed)
    q, k, v = (torch.randn(1, 3, L, D, generator=g) for _ in range(3))
    k = k + bias * torch.randn(1, 3, 1, D, generator=g)
    return q.to(torch.bfloat16), k.to(torch.bfloat16), v.to(torch.bfloat16)


@pytest.mark.parametrize("L,D,ratio,scale", [(512, 128, 0.5, 0.05), (1000, 128, 0.3, 0.15), (333, 64, 0.5, 0.05)])
def test_quantised_forward_with_a_scale_of_the_callers(dev, L, D, ratio, scale):
    q, k, v = _qkv(L, D, L + 3)
    m, lut, T = O.get_block_map(q, k, ratio, 128, 64)
    ref, _ = O.sparse_attn_fwd_gather(q, k, v, lut, 128, 64, qk_scale=scale)
    ref_q = O.sage_sparse_attn_fwd(q, k, v, lut, 128, 64, qk_scale=scale)
    ref_default, _ = O.sparse_attn_fwd_gather(q, k, v, lut, 128, 64)
    q8, qs, k8, ks = quant_qk(q.to(dev), k.to(dev))
    v8, vs = quant_v(v.to(dev))
    o = sage_attn_fwd(q8, qs, k8, ks, v8, vs, lut.to(dev), T, torch.bfloat16, qk_scale=scale).cpu()
    assert cos_sim(o, ref) >= 0.995
    # (same quantised scheme as the oracle up to the points where P is rounded to e4m3: a flatter softmax spreads the
    #  weight over more, individually rounded, probabilities)
    assert cos_sim(o, ref_q) >= 0.999 and max_abs(o, ref_q) <= 6e-2   # (a sharper softmax: single e4m3-rounded terms weigh more)
    assert max_abs(ref_default, ref) > 0.1          # the scale matters on these inputs


@pytest.mark.parametrize("L,D", [(512, 128), (1000, 128), (333, 64)])
def test_reference_range_of_v(dev, L, D):
    """v quantised to +-2.25 as the reference's call does: codes and scales bit-exact against the oracle, and the
    attention kernel, which only multiplies by v_scale at the end, gives the same output as with the full range."""
    q, k, v = _qkv(L, D, L + 11)
    v8r, vsr = O.sage_quant_v(v, O.SAGE_V_RANGE_REFERENCE)
    v8, vs = quant_v(v.to(dev), V_RANGE_REFERENCE)
    assert torch.equal(vs.cpu(), vsr)
    assert torch.equal(v8.cpu().view(torch.uint8), v8r.view(torch.uint8))
    assert float(v8.float().abs().max()) == 2.25
    # a strided view takes the other entry point
    vt = v.to(dev).transpose(1, 2).contiguous().transpose(1, 2)
    v8s, vss = quant_v(vt, V_RANGE_REFERENCE)
    assert torch.equal(v8s.view(torch.uint8), v8.view(torch.uint8)) and torch.equal(vss, vs)
    m, lut, T = O.get_block_map(q, k, 0.4, 128, 64)
    ref, _ = O.sparse_attn_fwd_gather(q, k, v, lut, 128, 64)
    ref_q = O.sage_sparse_attn_fwd(q, k, v, lut, 128, 64, v_range=O.SAGE_V_RANGE_REFERENCE)
    q8, qs, k8, ks = quant_qk(q.to(dev), k.to(dev))
    o = sage_attn_fwd(q8, qs, k8, ks, v8, vs, lut.to(dev), T, torch.bfloat16).cpu()
    assert cos_sim(o, ref) >= 0.995
    assert cos_sim(o, ref_q) >= 0.9995 and max_abs(o, ref_q) <= 3e-2
