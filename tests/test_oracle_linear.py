"""Pins the linear branch / projection / sum of the CPU oracle."""
import pytest
import torch

from oracle import sla_oracle as O
from sla_amd.inputs import make_proj


def _rand(L=96, D=8, seed=0):
    g = torch.Generator().manual_seed(seed)
    return tuple(torch.randn(1, 2, L, D, generator=g, dtype=torch.float64) for _ in range(3))


def test_feature_maps_known_values():
    x = torch.tensor([[-1.0, 0.0, 2.0]], dtype=torch.float64)
    assert torch.allclose(O.feature_map("elu")(x), torch.tensor([[torch.exp(torch.tensor(-1.0)).item(), 1.0, 3.0]],
                                                                 dtype=torch.float64))
    assert torch.equal(O.feature_map("relu")(x), torch.tensor([[0.0, 0.0, 2.0]], dtype=torch.float64))
    sm = O.feature_map("softmax")(x)
    assert abs(float(sm.sum()) - 1.0) < 1e-12 and sm[0, 2] > sm[0, 1] > sm[0, 0]
    with pytest.raises(NotImplementedError):
        O.feature_map("hedgehog")


@pytest.mark.parametrize("fmap", ["elu", "relu", "softmax"])
def test_calc_linear_is_kernelised_attention(fmap):
    # independent quadratic form: o_i = sum_j (phi(q_i).phi(k_j)) v_j / (1e-5 + sum_j phi(q_i).phi(k_j))
    q, k, v = _rand()
    phi = O.feature_map(fmap)
    fq, fk = phi(q), phi(k)
    a = fq @ fk.transpose(-1, -2)
    ref = (a @ v) / (1e-5 + a.sum(-1, keepdim=True))
    assert (O.calc_linear(fq, fk, v) - ref).abs().max() < 1e-10


def test_block_state_decomposition_and_softmax_mass():
    q, k, v = _rand(L=200)
    fk = O.feature_map("softmax")(k)
    total = fk.transpose(-1, -2) @ v
    parts = sum(fk[:, :, a:a + 64].transpose(-1, -2) @ v[:, :, a:a + 64] for a in range(0, 200, 64))
    assert (total - parts).abs().max() < 1e-12
    assert abs(float(fk.sum(dim=(-1, -2))[0, 0]) - 200.0) < 1e-9


def test_zero_init_projection_returns_sparse_output_exactly():
    g = torch.Generator().manual_seed(1)
    q, k, v = (torch.randn(1, 2, 256, 32, generator=g).to(torch.bfloat16) for _ in range(3))
    o, o_s, o_l, *_ = O.sla_forward(q, k, v, torch.zeros(32, 32), torch.zeros(32), 0.5, "softmax")
    assert float(o_l.abs().max()) == 0.0
    assert torch.equal(o, o_s.to(torch.bfloat16))


def test_projection_is_linear_layer():
    q, k, v = _rand(D=16)
    w, b = make_proj(16)
    lin = torch.nn.Linear(16, 16, dtype=torch.float64)
    with torch.no_grad():
        lin.weight.copy_(w)
        lin.bias.copy_(b)
    phi = O.feature_map("elu")
    ref = lin(O.calc_linear(phi(q), phi(k), v))
    out = O.linear_branch(q, k, v, w, b, "elu", torch.float64)
    assert (out - ref).abs().max() < 1e-12


def test_reference_rounding_mode_close_to_fp32():
    g = torch.Generator().manual_seed(2)
    q, k, v = (torch.randn(1, 2, 512, 64, generator=g).to(torch.bfloat16) for _ in range(3))
    w, b = make_proj(64)
    for fmap in ("elu", "relu", "softmax"):
        lo = O.linear_branch(q, k, v, w, b, fmap, torch.bfloat16)
        hi = O.linear_branch(q, k, v, w, b, fmap, torch.float32)
        assert lo.dtype == torch.bfloat16
        assert (lo.float() - hi).abs().max() < 2e-2


def test_module_forward_is_sum_of_branches():
    g = torch.Generator().manual_seed(3)
    q, k, v = (torch.randn(1, 2, 256, 32, generator=g) for _ in range(3))
    w, b = make_proj(32)
    o, o_s, o_l, m, lut, T = O.sla_forward(q, k, v, w, b, 0.5, "elu", compute_dtype=torch.float32)
    ref, ref_s, ref_l = O.sla_forward_autograd(q, k, v, w, b, m, "elu", 64, 64)
    assert (o.double() - ref).abs().max() < 1e-4


# ---- complement mode (linear branch over the non-selected key blocks) ----------------------------------
def _complement_case(L=300, D=16, BLKQ=64, BLKK=64, ratio=0.4, seed=3):
    g = torch.Generator().manual_seed(seed)
    q, k, v = (torch.randn(1, 2, L, D, generator=g) for _ in range(3))
    m, lut, T = O.get_block_map(q, k, ratio, BLKQ, BLKK)
    w = torch.randn(D, D, generator=g) / D ** 0.5
    b = torch.randn(D, generator=g)
    return q, k, v, m, lut, T, w, b


@pytest.mark.parametrize("fmap", ["elu", "relu", "softmax"])
def test_complement_equals_masked_dense_linear_attention(fmap):
    """Independent restatement: dense (L x L) kernelised attention with the selected blocks masked out."""
    q, k, v, m, lut, T, w, b = _complement_case()
    L = q.shape[2]
    phi = O.feature_map(fmap)
    a = phi(q.double()) @ phi(k.double()).transpose(-1, -2)              # (B,H,L,L)
    keep = ~O.expand_block_map(m, L, 64, 64)
    a = a * keep
    o = (a @ v.double()) / (1e-5 + a.sum(dim=-1, keepdim=True))
    ref = torch.nn.functional.linear(o, w.double(), b.double())
    got = O.linear_branch_complement(q, k, v, lut, w, b, fmap, 64, 64, torch.float32)
    assert float((got.double() - ref).abs().max()) < 1e-4


def test_complement_with_nothing_selected_is_the_global_branch():
    q, k, v, m, lut, T, w, b = _complement_case()
    empty = lut[..., :0]
    got = O.linear_branch_complement(q, k, v, empty, w, b, "elu", 64, 64, torch.float32)
    ref = O.linear_branch(q, k, v, w, b, "elu", torch.float32)
    assert float((got - ref).abs().max()) < 1e-4


def test_complement_with_everything_selected_is_the_bias():
    q, k, v, m, lut, T, w, b = _complement_case(ratio=1.0)
    got = O.linear_branch_complement(q, k, v, lut, w, b, "relu", 64, 64, torch.float32)
    # numerator and divisor state are (numerically) zero: o_l = 0 / 1e-5, so only the bias is left
    assert float((got - b).abs().max()) < 1e-2


@pytest.mark.parametrize("fmap", ["elu", "relu", "softmax"])
def test_complement_gradients_equal_those_of_the_masked_dense_form(fmap):
    """Autograd through the block-state formulation (what the GPU tests use as the gradient oracle) against
    autograd through the dense masked kernelised attention in fp64."""
    q, k, v, m, lut, T, w, b = _complement_case()
    L = q.shape[2]
    g = torch.randn(q.shape, generator=torch.Generator().manual_seed(9))
    leaves = [t.clone().requires_grad_(True) for t in (q, k, v, w, b)]
    O.linear_branch_complement(*leaves[:3], lut, *leaves[3:], fmap, 64, 64, torch.float32).backward(g)
    ref = [t.double().requires_grad_(True) for t in (q, k, v, w, b)]
    phi = O.feature_map(fmap)
    a = (phi(ref[0]) @ phi(ref[1]).transpose(-1, -2)) * ~O.expand_block_map(m, L, 64, 64)
    o = (a @ ref[2]) / (1e-5 + a.sum(dim=-1, keepdim=True))
    torch.nn.functional.linear(o, ref[3], ref[4]).backward(g.double())
    for x, r in zip(leaves, ref):
        assert float((x.grad.double() - r.grad).abs().max()) <= 1e-3 * max(1.0, float(r.grad.abs().max()))
