"""Whole-module forward+backward (cfg2, README shape) vs autograd of the fp64 dense oracle."""
import pytest
import torch

from conftest import cos_sim, max_abs
from oracle import sla_oracle as O
from sla_amd import SparseLinearAttention
from sla_amd.inputs import CONFIGS, make_inputs, make_proj

pytestmark = pytest.mark.gpu

TOL_ABS = 2e-2
TOL_COS = 0.999


@pytest.mark.parametrize("fmap", ["softmax", "elu", "relu"])
def test_cfg2_gradients(dev, fmap):
    cfg = CONFIGS["cfg2"]
    d = make_inputs(cfg)
    w, b = make_proj(cfg.D)
    mod = SparseLinearAttention(cfg.D, cfg.topk, fmap, cfg.BLKQ, cfg.BLKK).to(dev)
    with torch.no_grad():
        mod.proj_l.weight.copy_(w)
        mod.proj_l.bias.copy_(b)
    qd, kd, vd = (d[x].to(dev).requires_grad_(True) for x in "qkv")
    o = mod(qd, kd, vd)
    o.backward(d["do"].to(dev))
    torch.cuda.synchronize()

    m, lut, T = O.get_block_map(d["q"], d["k"], cfg.topk, cfg.BLKQ, cfg.BLKK)
    grads = {}
    # the dense oracle needs L^2 scores per head: one (b,h) at a time
    dw_ref = torch.zeros(cfg.D, cfg.D, dtype=torch.float64)
    db_ref = torch.zeros(cfg.D, dtype=torch.float64)
    for bi in range(cfg.B):
        for hi in range(cfg.H):
            sl = (slice(bi, bi + 1), slice(hi, hi + 1))
            qr, kr, vr = (d[x][sl].double().requires_grad_(True) for x in "qkv")
            wr, br = w.double().requires_grad_(True), b.double().requires_grad_(True)
            out, _, _ = O.sla_forward_autograd(qr, kr, vr, wr, br, m[sl], fmap, cfg.BLKQ, cfg.BLKK)
            out.backward(d["do"][sl].double())
            dw_ref += wr.grad
            db_ref += br.grad
            for name, a, r in (("dq", qd.grad[sl], qr.grad), ("dk", kd.grad[sl], kr.grad), ("dv", vd.grad[sl], vr.grad)):
                assert max_abs(a.cpu(), r) <= TOL_ABS, (name, bi, hi, max_abs(a.cpu(), r))
                assert cos_sim(a.cpu(), r) >= TOL_COS, (name, bi, hi)
            if bi == 0 and hi == 0:
                assert max_abs(o[sl].detach().cpu(), out.detach()) <= TOL_ABS
    for name, a, r in (("dW", mod.proj_l.weight.grad, dw_ref), ("db", mod.proj_l.bias.grad, db_ref)):
        scale = max(1.0, float(r.abs().max()))
        assert max_abs(a.cpu(), r) <= TOL_ABS * scale, (name, max_abs(a.cpu(), r), scale)
        assert cos_sim(a.cpu(), r) >= TOL_COS, name


@pytest.mark.parametrize("mode", ["global", "complement"])
def test_forward_and_gradients_are_bit_reproducible(dev, mode):
    """No atomics anywhere on the path: two runs give the same bits, also with a key block that every query block
    selects (its list is cut into segments whose partial sums are added in a fixed order)."""
    cfg = CONFIGS["cfg2"]
    d = make_inputs(cfg, H=2)
    d["k"][:, :, :64] += 3 * d["q"].float().mean(-2, keepdim=True).to(d["k"].dtype)   # pulls key block 0 into most rows
    w, b = make_proj(cfg.D)
    mod = SparseLinearAttention(cfg.D, cfg.topk, "elu", cfg.BLKQ, cfg.BLKK, linear_mode=mode).to(dev)
    with torch.no_grad():
        mod.proj_l.weight.copy_(w)
        mod.proj_l.bias.copy_(b)
    runs = []
    for _ in range(2):
        qd, kd, vd = (d[x].to(dev).requires_grad_(True) for x in "qkv")
        mod.zero_grad()
        o = mod(qd, kd, vd)
        o.backward(d["do"].to(dev))
        runs.append([t.detach().clone() for t in (o, qd.grad, kd.grad, vd.grad, mod.proj_l.weight.grad, mod.proj_l.bias.grad)])
    for a, c in zip(*runs):
        assert torch.equal(a, c)


def test_training_step_in_a_hip_graph(dev):
    """Forward + backward captured once and replayed: the library allocates nothing itself and clears nothing with
    memset nodes, so every replay gives the eager step's output and gradients bit for bit."""
    cfg = CONFIGS["cfg2"]
    d = make_inputs(cfg, H=2)
    w, b = make_proj(cfg.D)
    mod = SparseLinearAttention(cfg.D, cfg.topk, "elu", cfg.BLKQ, cfg.BLKK).to(dev)
    with torch.no_grad():
        mod.proj_l.weight.copy_(w)
        mod.proj_l.bias.copy_(b)
    do = d["do"].to(dev)
    qg, kg, vg = (d[x].to(dev).requires_grad_(True) for x in "qkv")
    leaves = (qg, kg, vg, mod.proj_l.weight, mod.proj_l.bias)

    def step():
        o = mod(qg, kg, vg)
        o.backward(do)
        return o

    o_ref = step().detach().clone()
    ref = [t.grad.clone() for t in leaves]
    for t in leaves:
        t.grad = None
    s = torch.cuda.Stream(device=dev)
    s.wait_stream(torch.cuda.current_stream(dev))
    with torch.cuda.stream(s):
        for _ in range(3):                    # warm-up on the capture stream
            step()
            for t in leaves:
                t.grad = None
    torch.cuda.current_stream(dev).wait_stream(s)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        o = step()
    for i in range(3):
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(o, o_ref), f"replay {i}"
        for t, r in zip(leaves, ref):
            assert torch.equal(t.grad, r), f"replay {i}"
        with torch.no_grad():
            mod(qg, kg, vg)                   # eager work between the replays
        torch.cuda.synchronize()


@pytest.mark.parametrize("layout", ["contiguous", "packed"])
@pytest.mark.parametrize("with_states", [False, True])
@pytest.mark.parametrize("dtype,L,D,BLKQ", [(torch.bfloat16, 2100, 128, 64), (torch.float16, 1000, 64, 128)])
def test_one_call_backward_equals_the_two_calls(dev, layout, with_states, dtype, L, D, BLKQ):
    """sla_module_bwd, on one stream and with the short kernels on a second one, against sla_sparse_attn_bwd followed
    by the accumulating sla_linear_bwd: the same bits.  Ran twice with the side stream (the events are reused)."""
    from sla_amd import get_block_map
    from sla_amd.linear import linear_bwd, linear_state_fwd, saved_states
    from sla_amd.module import module_bwd
    from sla_amd.sparse_attn import sparse_attn_bwd, sparse_attn_linear_fwd

    B, H, topk_ratio, fmap = 1, 3, 0.2, "elu"
    gen = torch.Generator().manual_seed(L)
    if layout == "packed":
        qkv = torch.randn(B, L, 3, H, D, generator=gen).to(dtype).to(dev)
        q, k, v = (qkv[:, :, i].permute(0, 2, 1, 3) for i in range(3))
        d_out = torch.randn(B, L, H, D, generator=gen).to(dtype).to(dev).permute(0, 2, 1, 3)
    else:
        q, k, v, d_out = (torch.randn(B, H, L, D, generator=gen).to(dtype).to(dev) for _ in range(4))
    w, b = (t.to(dev) for t in make_proj(D))
    sparse_map, lut, topk = get_block_map(q, k, topk_ratio=topk_ratio, BLKQ=BLKQ, BLKK=64)
    state_ws = linear_state_fwd(k, v, w, fmap)
    _, o_s, lse = sparse_attn_linear_fwd(q, k, v, lut, topk, BLKQ, 64, D ** -0.5, state_ws, b, fmap, want_o_s=True)
    states = saved_states(state_ws, q) if with_states else None

    def new_grads():
        if layout == "packed":
            g = torch.full((B, L, 3, H, D), float("nan"), dtype=dtype, device=dev)
            return g, tuple(g[:, :, i].permute(0, 2, 1, 3) for i in range(3))
        g = tuple(torch.full((B, H, L, D), float("nan"), dtype=dtype, device=dev) for _ in range(3))
        return g, g

    _, ref = new_grads()
    sparse_attn_bwd(q, k, v, o_s, d_out, lse, sparse_map, lut, topk, BLKQ, 64, D ** -0.5, grads=ref)
    _, _, _, dw_ref, db_ref = linear_bwd(q, k, v, w, b, d_out, fmap, accumulate_into=ref, states=states)
    side = torch.cuda.Stream(device=dev)
    for side_stream in (None, side, side):
        _, grads = new_grads()
        out = module_bwd(q, k, v, o_s, d_out, lse, sparse_map, lut, topk, BLKQ, 64, D ** -0.5, w, b, fmap, states=states,
                         grads=grads, side_stream=side_stream)
        torch.cuda.synchronize()
        for name, a, r in zip(("dq", "dk", "dv", "dW", "db"), out, (*ref, dw_ref, db_ref)):
            assert torch.equal(a, r), (name, side_stream is not None)
