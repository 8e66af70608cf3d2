"""Size-independent properties checked at the full benchmark size (cfg3: B1 H12 L32760 D128), where the
CPU oracle is too slow to serve as the checker for every head."""
import pytest
import torch

from sla_amd import SparseLinearAttention, get_block_map
from sla_amd.inputs import CONFIGS, make_inputs, make_proj
from sla_amd.sparse_attn import sparse_attn_fwd

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def full(dev):
    cfg = CONFIGS["cfg3"]
    d = make_inputs(cfg)
    q, k, v = (d[x].to(dev) for x in "qkv")
    m, lut, T = get_block_map(q, k, cfg.topk, cfg.BLKQ, cfg.BLKK)
    return cfg, q, k, v, m, lut, T


def test_heads_do_not_interact(dev, full):
    """Two heads computed inside the 12-head launch equal the same heads computed alone, bit for bit
    (mask builder and attention kernel; covers the workgroup-to-tile remapping at the full grid.  Two heads, not
    one: that is the smallest launch at this length that takes the same forward kernel as the full one)."""
    cfg, q, k, v, m, lut, T = full
    o, lse = sparse_attn_fwd(q, k, v, lut, T, cfg.BLKQ, cfg.BLKK, cfg.D ** -0.5)
    for h in (0, 7, 10):
        qs, ks, vs = (t[:, h:h + 2].contiguous() for t in (q, k, v))
        m1, lut1, T1 = get_block_map(qs, ks, cfg.topk, cfg.BLKQ, cfg.BLKK)
        assert T1 == T and torch.equal(m1, m[:, h:h + 2]) and torch.equal(lut1, lut[:, h:h + 2])
        o1, lse1 = sparse_attn_fwd(qs, ks, vs, lut1, T1, cfg.BLKQ, cfg.BLKK, cfg.D ** -0.5)
        assert torch.equal(o1, o[:, h:h + 2]) and torch.equal(lse1, lse[:, h:h + 2])


def test_output_is_homogeneous_in_v(dev, full):
    """out(q, k, 2v) == 2 out(q, k, v) exactly: doubling is exact in bf16 and fp32, and with a zero bias both
    branches are linear in v (the probabilities, the divisor and the mask do not depend on v)."""
    cfg, q, k, v, *_ = full
    mod = SparseLinearAttention(cfg.D, cfg.topk, cfg.feature_map, cfg.BLKQ, cfg.BLKK).to(dev)
    w, _ = make_proj(cfg.D)
    with torch.no_grad():
        mod.proj_l.weight.copy_(w)
        o1 = mod(q, k, v)
        o2 = mod(q, k, v * 2)
    assert torch.isfinite(o1.float()).all()
    assert torch.equal(o2, o1 * 2)


def test_rows_are_convex_combinations(dev, full):
    """With v = 1 everywhere every attention output is exactly 1 up to the bf16 rounding of P and of the
    result (sum_j p_j / l): checks the normalisation over all 6144 query blocks, including the ragged last one."""
    cfg, q, k, v, m, lut, T = full
    ones = torch.ones_like(v)
    o, _ = sparse_attn_fwd(q, k, ones, lut, T, cfg.BLKQ, cfg.BLKK, cfg.D ** -0.5)
    assert float((o.float() - 1).abs().max()) <= 2 ** -7


# ---------------------------------------------------------------------------------------------------------------
# The largest configuration (cfg4: B1 H40 L75600 D128, relu, forward + backward).  The inputs are generated on
# the device (the CPU generator needs minutes at this size); the oracle checks the LAST head, copied to the host,
# whose offsets are the largest the kernels form.
# ---------------------------------------------------------------------------------------------------------------
def _device_inputs(cfg, dev, seed, with_do):
    from sla_amd.inputs import make_inputs_on_device
    return make_inputs_on_device(cfg, dev, seed, with_do)


def _check_map(m, lut, T, N):
    assert lut.shape[-1] == T and m.shape[-1] == N
    assert int(m.sum(-1).min()) == T and int(m.sum(-1).max()) == T
    assert bool((lut[..., 1:] > lut[..., :-1]).all())                      # ascending, hence unique
    assert int(lut.min()) >= 0 and int(lut.max()) < N
    assert bool(torch.gather(m, -1, lut.long()).all())


def test_largest_configuration_forward_backward(dev):
    from conftest import cos_sim, max_abs
    from oracle import sla_oracle as O
    from sla_amd import _attention

    cfg = CONFIGS["cfg4"]
    q, k, v, do = _device_inputs(cfg, dev, 4, True)
    m, lut, T = get_block_map(q, k, cfg.topk, cfg.BLKQ, cfg.BLKK)
    assert T == 59
    _check_map(m, lut, T, 1182)

    # block-sparse attention, all 40 heads
    qd, kd, vd = (t.clone().requires_grad_(True) for t in (q, k, v))
    o = _attention.apply(qd, kd, vd, m, lut, T, cfg.BLKQ, cfg.BLKK)
    o.backward(do)
    dq, dk, dv = qd.grad, kd.grad, vd.grad
    for t in (o, dq, dk, dv):
        assert bool(torch.isfinite(t.float()).all())
    # rows of P sum to one: sum over keys of dV == sum over queries of dO, per head and channel
    assert max_abs(dv.double().sum(-2), do.double().sum(-2)) <= 1.0
    # q.k is invariant under (q a, k / a): sum q.dq == sum k.dk, per head
    ta, tb = (q.double() * dq.double()).sum((-1, -2)), (k.double() * dk.double()).sum((-1, -2))
    scale = (q.double() * dq.double()).abs().sum((-1, -2)) + (k.double() * dk.double()).abs().sum((-1, -2))
    assert bool(((ta - tb).abs() <= 1e-3 * scale).all())

    # the index sets of the first, a middle and the last head against the oracle's mask builder
    for hh in (0, cfg.H // 2 - 1, cfg.H - 1):
        m_h, lut_h, T_h = O.get_block_map(q[:, hh:hh + 1].cpu(), k[:, hh:hh + 1].cpu(), cfg.topk, cfg.BLKQ, cfg.BLKK)
        assert T_h == T and torch.equal(m_h, m[:, hh:hh + 1].cpu()), f"map of head {hh} differs from the oracle's"
        assert torch.equal(lut_h.long(), lut[:, hh:hh + 1].cpu().long()), f"look-up table of head {hh} differs"

    # the last head against the oracle (mask builder, forward, backward)
    h = cfg.H - 1
    qc, kc, vc, doc = (t[:, h:h + 1].cpu() for t in (q, k, v, do))
    m_ref, lut_ref, T_ref = O.get_block_map(qc, kc, cfg.topk, cfg.BLKQ, cfg.BLKK)
    assert T_ref == T and torch.equal(m_ref, m[:, h:h + 1].cpu())
    assert torch.equal(lut_ref.long(), lut[:, h:h + 1].cpu().long())
    o_ref, lse_ref = O.sparse_attn_fwd_gather(qc, kc, vc, lut_ref, cfg.BLKQ, cfg.BLKK)
    refs = O.sparse_attn_bwd_gather(qc, kc, vc, o_ref, doc, lse_ref, lut_ref, cfg.BLKQ, cfg.BLKK)
    got = (o.detach(), dq, dk, dv)
    for name, a, r in zip(("o", "dq", "dk", "dv"), got, (o_ref,) + tuple(refs)):
        a = a[:, h:h + 1].cpu()
        assert max_abs(a, r) <= 2e-2, (name, max_abs(a, r))
        assert cos_sim(a, r) >= 0.999, (name, cos_sim(a, r))
    del qd, kd, vd, o, dq, dk, dv

    # the whole module (relu feature map, seeded projection): forward + backward run at this size, the linear
    # branch of the last head agrees with the oracle, and the module output is attention + linear branch
    w, b = make_proj(cfg.D)
    mod = SparseLinearAttention(cfg.D, cfg.topk, cfg.feature_map, cfg.BLKQ, cfg.BLKK).to(dev)
    with torch.no_grad():
        mod.proj_l.weight.copy_(w)
        mod.proj_l.bias.copy_(b)
    qd, kd, vd = (t.clone().requires_grad_(True) for t in (q, k, v))
    out = mod(qd, kd, vd)
    out.backward(do)
    for t in (out, qd.grad, kd.grad, vd.grad, mod.proj_l.weight.grad, mod.proj_l.bias.grad):
        assert bool(torch.isfinite(t.float()).all())
    lin_ref = O.linear_branch(qc, kc, vc, w, b, cfg.feature_map, torch.float32)
    a = out.detach()[:, h:h + 1].cpu()
    assert max_abs(a, o_ref + lin_ref) <= 2e-2 and cos_sim(a, o_ref + lin_ref) >= 0.999
    # module gradient = attention gradient (above) + gradient of the linear branch (fp64 autograd of the oracle)
    qr, kr, vr = (t.double().requires_grad_(True) for t in (qc, kc, vc))
    O.linear_branch(qr, kr, vr, w.double(), b.double(), cfg.feature_map, torch.float64).backward(doc.double())
    for name, a, r_lin, r_sp in zip(("dq", "dk", "dv"), (qd.grad, kd.grad, vd.grad), (qr.grad, kr.grad, vr.grad), refs):
        a = a[:, h:h + 1].cpu()
        r = r_lin + r_sp.double()
        assert max_abs(a, r) <= 2e-2, (name, max_abs(a, r))
        assert cos_sim(a, r) >= 0.999, (name, cos_sim(a, r))


def test_largest_quantised_configuration(dev):
    """cfg5 in full (B1 H40 L32760 D128, 128/64 blocks, topk 0.1, biased k): finite everywhere, the map is
    well-formed, v = 1 gives 1 (normalisation of the fp8 P V product with its per-channel scale), and the last
    head agrees with the fp32 mathematics of the same mask to the cosine bound."""
    from conftest import cos_sim
    from oracle import sla_oracle as O
    from sla_amd import SageSparseLinearAttention
    from sla_amd.sage import sage_attn_fwd, sage_prepare

    cfg = CONFIGS["cfg5"]
    q, k, v, _ = _device_inputs(cfg, dev, 5, False)
    m, lut, T = get_block_map(q, k, cfg.topk, cfg.BLKQ, cfg.BLKK)
    assert T == 51
    _check_map(m, lut, T, 512)
    mod = SageSparseLinearAttention(cfg.D, cfg.topk, cfg.feature_map).to(dev)
    w, b = make_proj(cfg.D)
    with torch.no_grad():
        mod.proj_l.weight.copy_(w)
        mod.proj_l.bias.copy_(b)
        out = mod(q, k, v)
        m2, lut2, T2, q8, qs, k8, ks, v8, vs = sage_prepare(q, k, torch.ones_like(v), cfg.topk)
        assert T2 == T and torch.equal(lut2, lut) and torch.equal(m2, m)
        ones = sage_attn_fwd(q8, qs, k8, ks, v8, vs, lut, T, torch.bfloat16)
    assert bool(torch.isfinite(out.float()).all())
    assert float((ones.float() - 1).abs().max()) <= 2 ** -4
    h = cfg.H - 1
    qc, kc, vc = (t[:, h:h + 1].cpu() for t in (q, k, v))
    ref = O.sla_forward(qc, kc, vc, w, b, cfg.topk, cfg.feature_map, cfg.BLKQ, cfg.BLKK, linear_dtype=torch.float32)[0]
    assert cos_sim(out[:, h:h + 1].cpu(), ref) >= 0.995
