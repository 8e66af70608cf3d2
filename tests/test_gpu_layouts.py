"""Row-contiguous views as inputs: a (B, L, H, D) activation or the slices of a packed (B, L, 3, H, D) projection,
seen as (B, H, L, D), must give bit for bit what the contiguous copies give, without being copied."""
import pytest
import torch

from sla_amd import SLASelfAttention, SparseLinearAttention, get_block_map
from sla_amd.inputs import make_proj
from sla_amd.linear import linear_out_fwd, linear_state_fwd

pytestmark = pytest.mark.gpu


def _views(kind, B, H, L, D, dtype, dev, seed):
    g = torch.Generator().manual_seed(seed)
    if kind == "blhd":
        return tuple(torch.randn(B, L, H, D, generator=g).to(dtype).to(dev).permute(0, 2, 1, 3) for _ in range(3))
    packed = torch.randn(B, L, 3, H, D, generator=g).to(dtype).to(dev)
    return tuple(packed[:, :, i].permute(0, 2, 1, 3) for i in range(3))


@pytest.mark.parametrize("kind", ["blhd", "packed"])
@pytest.mark.parametrize("B,H,L,D,BLKQ,fmap,dtype,ratio", [(2, 3, 700, 128, 64, "elu", torch.bfloat16, 0.3),
                                                           (1, 2, 333, 64, 128, "softmax", torch.float16, 0.3),
                                                           (1, 1, 50, 128, 64, "relu", torch.bfloat16, 1.0)])
def test_module_reads_views_in_place(dev, kind, B, H, L, D, BLKQ, fmap, dtype, ratio):
    q, k, v = _views(kind, B, H, L, D, dtype, dev, L)
    assert not q.is_contiguous() or B * H == 1
    mod = SparseLinearAttention(D, ratio, fmap, BLKQ, 64, use_bf16=dtype == torch.bfloat16).to(dev)
    w, b = make_proj(D)
    with torch.no_grad():
        mod.proj_l.weight.copy_(w)
        mod.proj_l.bias.copy_(b)
        ref = mod(q.contiguous(), k.contiguous(), v.contiguous())
        m_ref, lut_ref, T = get_block_map(q.contiguous(), k.contiguous(), ratio, BLKQ, 64)
        m, lut, T2 = get_block_map(q, k, ratio, BLKQ, 64)
        assert T == T2 and torch.equal(lut, lut_ref) and torch.equal(m, m_ref)
        out = mod(q, k, v)
    assert out.shape == ref.shape and torch.equal(out, ref)
    if not q.is_contiguous():
        # the output is laid out like the inputs' dimension order: (B, L, H, D) in memory
        assert out.transpose(1, 2).is_contiguous()
    # the two-kernel linear branch on views
    ws = linear_state_fwd(k, v, mod.proj_l.weight.detach(), fmap)
    ws_ref = linear_state_fwd(k.contiguous(), v.contiguous(), mod.proj_l.weight.detach(), fmap)
    a = linear_out_fwd(q.contiguous(), mod.proj_l.bias.detach(), None, ws, fmap)
    b2 = linear_out_fwd(q.contiguous(), mod.proj_l.bias.detach(), None, ws_ref, fmap)
    assert torch.equal(a, b2)


def test_training_on_views_takes_the_contiguous_route(dev):
    q, k, v = _views("packed", 1, 2, 512, 128, torch.bfloat16, dev, 5)
    mod = SparseLinearAttention(128, 0.25, "elu").to(dev)
    w, b = make_proj(128)
    with torch.no_grad():
        mod.proj_l.weight.copy_(w)
        mod.proj_l.bias.copy_(b)
    qg, kg, vg = (t.detach().requires_grad_(True) for t in (q, k, v))
    out = mod(qg, kg, vg)
    out.float().square().mean().backward()
    with torch.no_grad():
        ref = mod(q.contiguous(), k.contiguous(), v.contiguous())
    assert torch.equal(out.detach(), ref) and qg.grad is not None and torch.isfinite(qg.grad.float()).all()


def test_block_inference_equals_block_with_copies(dev):
    torch.manual_seed(0)
    blk = SLASelfAttention(dim=256, num_heads=2, topk=0.25, feature_map="elu").to(dev).to(torch.bfloat16)
    blk.attn.proj_l.float()
    with torch.no_grad():
        blk.attn.proj_l.weight.normal_(0, 128 ** -0.5)
        x = torch.randn(2, 640, 256, device=dev, dtype=torch.bfloat16)
        y = blk(x)
        qkv = blk.qkv(x).view(2, 640, 3, 2, 128).permute(2, 0, 3, 1, 4).contiguous()
        o = blk.attn(qkv[0], qkv[1], qkv[2])
        y_ref = blk.proj(o.transpose(1, 2).reshape(2, 640, 256))
    assert torch.equal(y, y_ref)


@pytest.mark.parametrize("B,H,L,D,BLKQ,fmap,dtype", [(2, 2, 700, 128, 64, "elu", torch.bfloat16),
                                                     (1, 3, 333, 64, 128, "softmax", torch.float16)])
def test_packed_training_equals_the_contiguous_route(dev, B, H, L, D, BLKQ, fmap, dtype):
    """forward_packed: output and all gradients (the packed one included) bit for bit what the module gives on
    contiguous (B, H, L, D) copies."""
    g = torch.Generator().manual_seed(L + 1)
    qkv = torch.randn(B, L, 3, H, D, generator=g).to(dtype).to(dev)
    do = torch.randn(B, L, H, D, generator=g).to(dtype).to(dev)
    mod = SparseLinearAttention(D, 0.3, fmap, BLKQ, 64, use_bf16=dtype == torch.bfloat16).to(dev)
    w, b = make_proj(D)
    with torch.no_grad():
        mod.proj_l.weight.copy_(w)
        mod.proj_l.bias.copy_(b)
    # contiguous route
    q, k, v = (qkv[:, :, i].permute(0, 2, 1, 3).contiguous().requires_grad_(True) for i in range(3))
    out_ref = mod(q, k, v)
    out_ref.backward(do.permute(0, 2, 1, 3).contiguous())
    gw, gb = mod.proj_l.weight.grad.clone(), mod.proj_l.bias.grad.clone()
    mod.zero_grad()
    # packed route
    qkv_g = qkv.clone().requires_grad_(True)
    out, dens = mod.forward_packed(qkv_g, return_sparsity=True)
    assert out.shape == (B, L, H, D) and out.is_contiguous() and 0 < dens <= 1
    assert torch.equal(out.detach().permute(0, 2, 1, 3), out_ref.detach())
    out.backward(do)
    for i, t in enumerate((q, k, v)):
        assert torch.equal(qkv_g.grad[:, :, i].permute(0, 2, 1, 3), t.grad), "qkv"[i]
    assert torch.equal(mod.proj_l.weight.grad, gw) and torch.equal(mod.proj_l.bias.grad, gb)
    # inference through the same entry
    with torch.no_grad():
        assert torch.equal(mod.forward_packed(qkv), out.detach())


@pytest.mark.parametrize("kind", ["blhd", "packed"])
@pytest.mark.parametrize("B,H,L,D,fmap,dtype", [(2, 3, 700, 128, "elu", torch.bfloat16), (1, 2, 333, 64, "softmax", torch.float16)])
def test_quantised_module_reads_views_in_place(dev, kind, B, H, L, D, fmap, dtype):
    """SageSLA on (B, L, H, D) activations / packed projections viewed as (B, H, L, D): bit for bit what the contiguous
    copies give (quantisers, state build and output kernel all read the views), output in the views' memory order."""
    from sla_amd import SageSparseLinearAttention
    from sla_amd.sage import quant_v, sage_prepare
    q, k, v = _views(kind, B, H, L, D, dtype, dev, L + 1)
    mod = SageSparseLinearAttention(D, 0.3, fmap, use_bf16=dtype == torch.bfloat16).to(dev)
    w, b = make_proj(D)
    with torch.no_grad():
        mod.proj_l.weight.copy_(w)
        mod.proj_l.bias.copy_(b)
        ref = mod(q.contiguous(), k.contiguous(), v.contiguous())
        out = mod(q, k, v)
    assert out.shape == ref.shape and torch.equal(out, ref)
    assert out.permute(0, 2, 1, 3).is_contiguous()
    # the pieces: one-call preparation and the separate v quantiser on views
    a = sage_prepare(q, k, v, 0.3)
    c = sage_prepare(q.contiguous(), k.contiguous(), v.contiguous(), 0.3)
    for x, y in zip(a, c):
        assert x == y if isinstance(x, int) else torch.equal(x.view(torch.uint8) if x.dtype == torch.float8_e4m3fn else x,
                                                             y.view(torch.uint8) if y.dtype == torch.float8_e4m3fn else y)
    v8, vs = quant_v(v)
    assert torch.equal(v8.view(torch.uint8), c[7].view(torch.uint8)) and torch.equal(vs, c[8])


def test_quantised_block_inference_equals_block_with_copies(dev):
    torch.manual_seed(5)
    blk = SLASelfAttention(dim=256, num_heads=2, topk=0.25, feature_map="relu", quantized=True).to(dev).to(torch.bfloat16)
    blk.attn.proj_l.float()
    with torch.no_grad():
        blk.attn.proj_l.weight.normal_(0, 128 ** -0.5)
        x = torch.randn(2, 640, 256, device=dev, dtype=torch.bfloat16)
        y = blk(x)
        q, k, v = blk.qkv(x).view(2, 640, 3, 2, 128).permute(2, 0, 3, 1, 4).contiguous()
        y_ref = blk.proj(blk.attn(q, k, v).transpose(1, 2).reshape(2, 640, 256))
    assert torch.equal(y, y_ref)
