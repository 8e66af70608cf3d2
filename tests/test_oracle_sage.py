"""Closed-form properties of the SageSLA quantisation oracle (parity unpinned against
spas_sage_attn, which is not available; the contract is cos >= 0.995 vs the fp32 math)."""
import torch

from conftest import cos_sim
from oracle import sla_oracle as O


def test_int8_quant_closed_forms():
    g = torch.Generator().manual_seed(0)
    q = torch.randn(1, 2, 300, 64, generator=g).to(torch.bfloat16)
    k = (torch.randn(1, 2, 300, 64, generator=g) + 3).to(torch.bfloat16)
    q8, qs, k8, ks, km = O.sage_quant_qk(q, k, 128, 64)
    assert q8.dtype == torch.int8 and qs.shape == (1, 2, 3) and ks.shape == (1, 2, 5)
    qb = q.float()
    for blk in range(3):
        rows = slice(blk * 128, min(300, blk * 128 + 128))
        s = qs[0, 0, blk]
        assert (qb[0, 0, rows] - s * q8[0, 0, rows].float()).abs().max() <= s / 2 + 1e-7
        assert int(q8[0, 0, rows].abs().max()) == 127
    ksm = k.float() - km.float()
    assert (ksm[0, 1, :64] - ks[0, 1, 0] * k8[0, 1, :64].float()).abs().max() <= ks[0, 1, 0] / 2 + 1e-7
    assert ksm.mean(-2).abs().max() < 0.05      # smoothing removed the +3 offset


def test_fp8_v_quant_closed_forms():
    v = torch.randn(1, 2, 200, 32).to(torch.bfloat16)
    v8, vs = O.sage_quant_v(v)
    assert v8.dtype == torch.float8_e4m3fn and vs.shape == (1, 2, 32)
    assert torch.equal(v8.float().abs().amax(-2), torch.full((1, 2, 32), 448.0))
    rel = ((v8.float() * vs.unsqueeze(-2) - v.float()).abs() / v.float().abs().clamp_min(1e-3)).max()
    assert rel < 0.07                              # e4m3: 3 mantissa bits -> 2^-4 relative


def test_quantised_attention_close_to_fp32_and_shift_invariant():
    g = torch.Generator().manual_seed(1)
    q, k, v = (torch.randn(1, 2, 512, 64, generator=g).to(torch.bfloat16) for _ in range(3))
    kb = (k.float() + 2 * torch.randn(1, 2, 1, 64, generator=g)).to(torch.bfloat16)
    m, lut, T = O.get_block_map(q, kb, 0.5, 128, 64)
    ref, _ = O.sparse_attn_fwd_gather(q, kb, v, lut, 128, 64)
    out = O.sage_sparse_attn_fwd(q, kb, v, lut, 128, 64)
    assert cos_sim(out, ref) >= 0.995
    N = lut.shape[-1]
    full = torch.arange(8).expand(1, 2, 4, 8).contiguous()
    sd = torch.nn.functional.scaled_dot_product_attention(q.float(), kb.float(), v.float())
    assert cos_sim(O.sage_sparse_attn_fwd(q, kb, v, full, 128, 64), sd) >= 0.995
