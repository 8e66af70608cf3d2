"""Closed-form properties of the SageSLA quantisation oracle (parity unpinned against
spas_sage_attn, which is not available; the contract is cos >= 0.995 vs the fp32 math)."""
import torch

from conftest import cos_sim, max_abs
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


# ---- scale-sensitive pins of the quantised attention: cosine similarity is blind to a wrong global factor and
# ---- nearly blind to a dropped per-channel scale, the checks below are not ----

def _sage_case(seed=2, L=512, D=64, H=2, ratio=0.5):
    g = torch.Generator().manual_seed(seed)
    q, k, v = (torch.randn(1, H, L, D, generator=g).to(torch.bfloat16) for _ in range(3))
    _, lut, _ = O.get_block_map(q, k, ratio, 128, 64)
    return q, k, v, lut


def test_quantised_attention_absolute_error_against_fp32_math():
    q, k, v, lut = _sage_case()
    ref, _ = O.sparse_attn_fwd_gather(q, k, v, lut, 128, 64)
    out = O.sage_sparse_attn_fwd(q, k, v, lut, 128, 64)
    assert max_abs(out, ref) <= 5e-2               # a factor of 448, 1/448 or 2 in the output fails this
    assert abs(float(out.norm() / ref.float().norm()) - 1.0) < 2e-2


def test_constant_v_gives_constant_output():
    # v == 1: every channel has scale 1/448 and v_fp8 == 448 exactly, so out = sum(p8) / (448 sum(p)),
    # 1 up to the e4m3 rounding of the probabilities (relative 2^-4 each, far less in the sum)
    q, k, v, lut = _sage_case(seed=3)
    out = O.sage_sparse_attn_fwd(q, k, torch.ones_like(v), lut, 128, 64)
    assert float((out - 1).abs().max()) < 3e-2
    out3 = O.sage_sparse_attn_fwd(q, k, torch.full_like(v, -3.0), lut, 128, 64)
    assert float((out3 + 3).abs().max()) < 9e-2


def test_power_of_two_channel_scales_pass_through_exactly():
    # scaling channel d of v by 2^(d % 8) changes only that channel's v_scale, by exactly that factor:
    # the e4m3 codes are unchanged, so the output scales bit for bit.  A dropped or mis-indexed per-channel
    # scale fails this.
    q, k, v, lut = _sage_case(seed=4)
    D = v.shape[-1]
    f = torch.tensor([2.0 ** (d % 8) for d in range(D)])
    v2 = (v.float() * f).to(torch.bfloat16)
    assert torch.equal(v2.float(), v.float() * f)
    a = O.sage_sparse_attn_fwd(q, k, v, lut, 128, 64)
    b = O.sage_sparse_attn_fwd(q, k, v2, lut, 128, 64)
    assert torch.equal(b, a * f)
    v8a, sa = O.sage_quant_v(v)
    v8b, sb = O.sage_quant_v(v2)
    assert torch.equal(v8a.view(torch.uint8), v8b.view(torch.uint8)) and torch.equal(sb, sa * f)


def test_one_tile_against_python_loops_with_explicit_casts():
    # a 64-row sequence, D = 16: one (ragged) query block, one key block; every step written out element by element
    g = torch.Generator().manual_seed(5)
    D = 16
    qq = torch.randn(1, 1, 64, D, generator=g).to(torch.bfloat16)
    k = (torch.randn(1, 1, 64, D, generator=g) + 1.5).to(torch.bfloat16)
    v = (torch.randn(1, 1, 64, D, generator=g) * torch.linspace(0.5, 4, D)).to(torch.bfloat16)
    lut = torch.zeros(1, 1, 1, 1, dtype=torch.int64)       # query block 0 -> key block 0
    out = O.sage_sparse_attn_fwd(qq, k, v, lut, 128, 64)[0, 0]
    qf, kf, vf = qq[0, 0].float(), k[0, 0].float(), v[0, 0].float()
    km = kf.mean(0).to(torch.bfloat16).float()          # one chunk, one group: plain mean is the fixed order here
    assert torch.equal(km, O.k_column_mean(k)[0, 0, 0].float())
    ks = kf - km
    sq = float(qf.abs().max()) / 127.0
    sk = float(ks.abs().max()) / 127.0
    import math
    q8 = [[max(-127, min(127, int(torch.round(qf[i, d] / torch.tensor(sq, dtype=torch.float32))))) for d in range(D)]
          for i in range(64)]
    k8 = [[max(-127, min(127, int(torch.round(ks[j, d] / torch.tensor(sk, dtype=torch.float32))))) for d in range(D)]
          for j in range(64)]
    vs = [float(vf[:, d].abs().max()) / 448.0 for d in range(D)]
    v8 = [[float((vf[j, d] / torch.tensor(vs[d], dtype=torch.float32)).to(torch.float8_e4m3fn).float()) for d in range(D)]
          for j in range(64)]
    scale = D ** -0.5 * math.log2(math.e)
    worst = 0.0
    for i in range(0, 64, 7):
        s = [sum(q8[i][d] * k8[j][d] for d in range(D)) * sq * sk * scale for j in range(64)]
        m = max(s)
        p = [2.0 ** (x - m) for x in s]
        l = sum(p)
        p8 = [float(torch.tensor(x * 448.0, dtype=torch.float32).to(torch.float8_e4m3fn).float()) for x in p]
        for d in range(D):
            o = sum(p8[j] * v8[j][d] for j in range(64)) * vs[d] / (448.0 * l)
            worst = max(worst, abs(o - float(out[i, d])))
    assert worst < 2e-5


def test_reference_v_range():
    # the reference quantises v to +-2.25 (SageSLA/core.py:129): same scheme, coarser use of the e4m3 grid
    q, k, v, lut = _sage_case(seed=6)
    v8, vs = O.sage_quant_v(v, O.SAGE_V_RANGE_REFERENCE)
    assert torch.equal(v8.float().abs().amax(-2), torch.full_like(vs, 2.25))
    assert torch.equal(vs, v.float().abs().amax(-2) / 2.25)
    ref, _ = O.sparse_attn_fwd_gather(q, k, v, lut, 128, 64)
    out = O.sage_sparse_attn_fwd(q, k, v, lut, 128, 64, v_range=O.SAGE_V_RANGE_REFERENCE)
    assert cos_sim(out, ref) >= 0.995 and max_abs(out, ref) <= 5e-2
