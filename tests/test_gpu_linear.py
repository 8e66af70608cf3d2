"""HIP linear branch + projection + sum vs the CPU oracle."""
import pytest
import torch

from conftest import cos_sim, max_abs
from oracle import sla_oracle as O
from sla_amd.inputs import CONFIGS, make_inputs, make_proj
from sla_amd.linear import linear_bwd, linear_fwd, linear_out_fwd, linear_state_fwd

pytestmark = pytest.mark.gpu

TOL_ABS = 2e-2
TOL_COS = 0.999


@pytest.mark.parametrize("fmap", ["elu", "relu", "softmax"])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("L,D", [(512, 128), (1000, 128), (333, 64), (50, 128)])
def test_linear_branch_vs_oracle(dev, fmap, dtype, L, D):
    g = torch.Generator().manual_seed(L)
    q, k, v = (torch.randn(2, 2, L, D, generator=g).to(dtype) for _ in range(3))
    res = torch.randn(2, 2, L, D, generator=g).to(dtype)
    w, b = make_proj(D)
    ref32 = O.linear_branch(q, k, v, w, b, fmap, torch.float32) + res.float()
    ref16 = O.linear_branch(q, k, v, w, b, fmap, dtype).float() + res.float()
    out = linear_fwd(q.to(dev), k.to(dev), v.to(dev), w.to(dev), b.to(dev), res.to(dev), fmap).cpu()
    assert out.dtype == dtype
    # The reference keeps every intermediate in the 16-bit dtype.  In float16 its divisor
    # sum_d phi(q)*ksum overflows to inf for elu once L*D is large (the branch then returns the
    # bias only); the kernel follows that arithmetic, so float16 is checked against the
    # 16-bit evaluation only.
    if dtype == torch.bfloat16:
        assert max_abs(out, ref32) <= TOL_ABS and cos_sim(out, ref32) >= TOL_COS
    assert max_abs(out, ref16) <= TOL_ABS and cos_sim(out, ref16) >= TOL_COS
    out0 = linear_fwd(q.to(dev), k.to(dev), v.to(dev), w.to(dev), b.to(dev), None, fmap).cpu()
    assert max_abs(out0, ref16 - res.float()) <= TOL_ABS


def test_zero_projection_returns_residual_exactly(dev):
    g = torch.Generator().manual_seed(3)
    q, k, v, res = (torch.randn(1, 2, 700, 128, generator=g).to(torch.bfloat16) for _ in range(4))
    out = linear_fwd(q.to(dev), k.to(dev), v.to(dev), torch.zeros(128, 128, device=dev), torch.zeros(128, device=dev),
                     res.to(dev), "softmax").cpu()
    assert torch.equal(out, res)


def test_cfg3_shape_two_heads(dev):
    cfg = CONFIGS["cfg3"]
    d = make_inputs(cfg, H=2)
    w, b = make_proj(128)
    ref = O.linear_branch(d["q"], d["k"], d["v"], w, b, cfg.feature_map, torch.float32)
    out = linear_fwd(d["q"].to(dev), d["k"].to(dev), d["v"].to(dev), w.to(dev), b.to(dev), None, cfg.feature_map).cpu()
    assert max_abs(out, ref) <= TOL_ABS and cos_sim(out, ref) >= TOL_COS


def _oracle_linear_grads(q, k, v, w, b, g, fmap):
    qd, kd, vd = (t.double().requires_grad_(True) for t in (q, k, v))
    wd, bd = w.double().requires_grad_(True), b.double().requires_grad_(True)
    out = O.linear_branch(qd, kd, vd, wd, bd, fmap, torch.float64)
    out.backward(g.double())
    return qd.grad, kd.grad, vd.grad, wd.grad, bd.grad


@pytest.mark.parametrize("fmap", ["elu", "relu", "softmax"])
@pytest.mark.parametrize("L,D", [(512, 128), (1000, 128), (333, 64)])
def test_linear_branch_backward_vs_autograd_oracle(dev, fmap, L, D):
    from sla_amd.linear import _linear_proj_add
    gen = torch.Generator().manual_seed(L + 7)
    q, k, v, res, g = (torch.randn(2, 2, L, D, generator=gen).to(torch.bfloat16) for _ in range(5))
    w, b = make_proj(D)
    refs = _oracle_linear_grads(q, k, v, w, b, g, fmap)
    qd, kd, vd, rd = (t.to(dev).requires_grad_(True) for t in (q, k, v, res))
    wd, bd = w.to(dev).requires_grad_(True), b.to(dev).requires_grad_(True)
    out = _linear_proj_add.apply(qd, kd, vd, wd, bd, rd, fmap)
    out.backward(g.to(dev))
    torch.cuda.synchronize()
    assert torch.equal(rd.grad.cpu(), g)
    names = ("dq", "dk", "dv", "dW", "db")
    for name, a, r in zip(names, (qd.grad, kd.grad, vd.grad, wd.grad, bd.grad), refs):
        a = a.cpu()
        scale = max(1.0, float(r.abs().max()))          # dW/db are sums over B*H*L rows
        assert max_abs(a, r) <= TOL_ABS * scale, (name, max_abs(a, r), scale)
        assert cos_sim(a, r) >= TOL_COS, (name, cos_sim(a, r))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("fmap", ["elu", "relu", "softmax"])
@pytest.mark.parametrize("B,H,L", [(1, 2, 50), (1, 3, 4099), (1, 1, 129), (2, 1, 2048)])
def test_backward_head_dim_128_slices_and_tails(dev, dtype, fmap, B, H, L):
    """The one-pass query-side kernel of head dim 128: a length below one 128-row step, lengths that end a slice in the
    middle of a step, many slices per head, both 16-bit types (inputs scaled down so that float16 stays finite)."""
    gen = torch.Generator().manual_seed(L + H)
    q, k, v, g = (torch.randn(B, H, L, 128, generator=gen).mul(0.5).to(dtype) for _ in range(4))
    w, b = make_proj(128)
    refs = _oracle_linear_grads(q, k, v, w, b, g, fmap)
    out = linear_bwd(q.to(dev), k.to(dev), v.to(dev), w.to(dev), b.to(dev), g.to(dev), fmap)
    torch.cuda.synchronize()
    for name, a, r in zip(("dq", "dk", "dv", "dW", "db"), out, refs):
        a = a.cpu()
        assert torch.isfinite(a.float()).all(), name
        scale = max(1.0, float(r.abs().max()))
        assert max_abs(a, r) <= TOL_ABS * scale, (name, max_abs(a, r), scale)
        assert cos_sim(a, r) >= TOL_COS, (name, cos_sim(a, r))


@pytest.mark.parametrize("D", [128, 64])
def test_backward_accumulates_like_a_16_bit_addition(dev, D):
    """accumulate_into: the gradient is rounded to 16 bit, then added to what the tensor held, rounded once more."""
    gen = torch.Generator().manual_seed(5)
    q, k, v, g = (torch.randn(1, 2, 700, D, generator=gen).to(torch.bfloat16).to(dev) for _ in range(4))
    w, b = (t.to(dev) for t in make_proj(D))
    fresh = linear_bwd(q, k, v, w, b, g, "elu")
    base = [torch.randn_like(q) for _ in range(3)]
    acc = linear_bwd(q, k, v, w, b, g, "elu", accumulate_into=tuple(t.clone() for t in base))
    for a, f, b0 in zip(acc[:3], fresh[:3], base):
        assert torch.equal(a, (b0.float() + f.float()).to(torch.bfloat16))
    assert torch.equal(acc[3], fresh[3]) and torch.equal(acc[4], fresh[4])


def test_split_entry_points_equal_the_fused_one(dev):
    """state half on a side stream + output half on the main one == sla_linear_fwd, bit for bit."""
    g = torch.Generator().manual_seed(7)
    q, k, v, res = (torch.randn(1, 3, 700, 128, generator=g).to(torch.bfloat16).to(dev) for _ in range(4))
    w, b = (t.to(dev) for t in make_proj(128))
    ref = linear_fwd(q, k, v, w, b, res, "elu")
    side = torch.cuda.Stream(device=dev)
    side.wait_stream(torch.cuda.current_stream(dev))
    with torch.cuda.stream(side):
        ws = linear_state_fwd(k, v, w, "elu")
    torch.cuda.current_stream(dev).wait_stream(side)
    ws.record_stream(torch.cuda.current_stream(dev))
    out = linear_out_fwd(q, b, res, ws, "elu")
    assert torch.equal(out, ref)


@pytest.mark.parametrize("fmap,D", [("elu", 128), ("softmax", 64)])
def test_backward_with_the_forward_states_handed_over(dev, fmap, D):
    """States copied from the forward's workspace instead of rebuilt in the backward: same gradients, bit for bit."""
    from sla_amd.linear import saved_states

    g = torch.Generator().manual_seed(11)
    q, k, v, do = (torch.randn(2, 2, 450, D, generator=g).to(torch.bfloat16).to(dev) for _ in range(4))
    w, b = (t.to(dev) for t in make_proj(D))
    ref = linear_bwd(q, k, v, w, b, do, fmap)
    states = saved_states(linear_state_fwd(k, v, w, fmap), q)
    assert states.numel() < 4 * 4 * D * D * 2 + 4096          # a few D x D matrices per head, no partial sums
    out = linear_bwd(q, k, v, w, b, do, fmap, states=states)
    for a, r in zip(out, ref):
        assert torch.equal(a, r)
    # accumulating variant
    base = [torch.randn_like(q) for _ in range(3)]
    acc_ref = linear_bwd(q, k, v, w, b, do, fmap, accumulate_into=tuple(t.clone() for t in base))
    acc = linear_bwd(q, k, v, w, b, do, fmap, accumulate_into=tuple(t.clone() for t in base), states=states)
    for a, r in zip(acc, acc_ref):
        assert torch.equal(a, r)
