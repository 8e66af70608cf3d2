"""The forward kernel for head dim 128 / 64-row query blocks walks two neighbouring query blocks together and
splits their look-up rows into shared and own key blocks.  These cases fix the look-up rows by hand so that every
shape of that split occurs, and compare with the CPU oracle, which follows a look-up table entry by entry
(bf16 tolerance 2e-2, cos >= 0.999; log-sum-exp 1e-3).  The library takes that kernel only for launches of at
least 512 pairs of query blocks (two workgroups for each of the 256 compute units): every case has that many heads."""
import pytest
import torch

from conftest import cos_sim, max_abs
from oracle import sla_oracle as O
from sla_amd.sparse_attn import sparse_attn_fwd

pytestmark = pytest.mark.gpu

TOL_ABS = 2e-2
TOL_COS = 0.999
TOL_LSE = 1e-3



def _sum_tol(ref):
    """Bound on the module output o_s + o_l: 2e-2 where the values stay below 4.  Above, the 16-bit format itself is the
    limit: bf16 values in [4, 8) are 2^-5 apart, so the one rounding of the sum may already be 1.6e-2 off, before the
    rounding of the linear branch (values of several units with this test's projection) that both sides carry; the bound
    grows with the largest magnitude the way that spacing does."""
    return 2e-2 * max(1.0, float(ref.abs().max()) / 4.0)

def _heads(L):
    pairs_per_head = ((L + 63) // 64 + 1) // 2
    return -(-512 // pairs_per_head)


def _qkv(H, L, seed, dtype=torch.bfloat16):
    g = torch.Generator().manual_seed(seed)
    return tuple(torch.randn(1, H, L, 128, generator=g).to(dtype) for _ in range(3))


def _check(q, k, v, lut, dev, lut_dtype=torch.int64):
    T = lut.shape[-1]
    o_ref, lse_ref = O.sparse_attn_fwd_gather(q, k, v, lut, 64, 64)
    o, lse = sparse_attn_fwd(q.to(dev), k.to(dev), v.to(dev), lut.to(lut_dtype).to(dev), T, 64, 64, 128 ** -0.5)
    torch.cuda.synchronize()
    assert torch.isfinite(o.float()).all()
    assert max_abs(o.cpu(), o_ref) <= TOL_ABS and cos_sim(o.cpu(), o_ref) >= TOL_COS
    assert max_abs(lse.cpu(), lse_ref) <= TOL_LSE


def _rows(M, N, T, shared, g):
    """Look-up rows for M query blocks: blocks 2j and 2j+1 have exactly `shared` key blocks in common."""
    lut = torch.empty(M, T, dtype=torch.int64)
    for j in range(0, M, 2):
        perm = torch.randperm(N, generator=g)
        a = perm[:T]
        b = torch.cat([perm[:shared], perm[T:2 * T - shared]])
        lut[j] = a[torch.randperm(T, generator=g)]
        if j + 1 < M:
            lut[j + 1] = b[torch.randperm(T, generator=g)]
    return lut


@pytest.mark.parametrize("L,T,shared", [(1024, 5, 0), (1024, 5, 5), (1024, 6, 1), (1024, 6, 5), (1024, 1, 0), (1024, 1, 1),
                                        (1000, 7, 3),      # ragged last key block
                                        (960, 4, 2),       # odd number of query blocks: the last one has no partner
                                        (1217, 8, 4)])     # both
def test_split_of_a_pair(dev, L, T, shared):
    g = torch.Generator().manual_seed(L + 10 * T + shared)
    H = _heads(L)
    q, k, v = _qkv(H, L, 100 + L + T)
    M = N = (L + 63) // 64
    lut = torch.stack([_rows(M, N, T, shared, g) for _ in range(H)]).view(1, H, M, T)
    _check(q, k, v, lut, dev)
    _check(q, k, v, lut, dev, lut_dtype=torch.int32)


def test_last_key_block_in_every_position(dev):
    """The ragged key block as first, middle and last entry of a row, shared and not."""
    L, T = 1000, 4
    N = 16
    H = _heads(L)
    q, k, v = _qkv(H, L, 7)
    lut = torch.tensor([[15, 1, 2, 3], [4, 15, 5, 6],      # shared by the pair
                        [0, 1, 15, 2], [0, 1, 3, 2],       # only in the first row
                        [7, 8, 9, 10], [11, 12, 13, 15],   # only in the second row, last
                        [15, 14, 13, 12], [12, 13, 14, 15]] * 2).view(1, 1, N, T).expand(1, H, N, T).contiguous()
    _check(q, k, v, lut, dev)


def test_rows_longer_than_a_wavefront(dev):
    """More than 64 entries per row: the split is formed 64 entries at a time."""
    L, T = 64 * 160, 70
    g = torch.Generator().manual_seed(5)
    H = _heads(L)
    q, k, v = _qkv(H, L, 9)
    M = N = 160
    lut = torch.stack([_rows(M, N, T, 37, g) for _ in range(H)]).view(1, H, M, T)
    _check(q, k, v, lut, dev)


def test_a_row_that_names_a_block_twice(dev):
    """Not what the mask builder produces, but the reference kernel would visit the block twice, and so must this."""
    L, T = 768, 4
    H = _heads(L)
    q, k, v = _qkv(H, L, 21)
    lut = torch.tensor([[3, 3, 5, 7], [3, 5, 7, 7],
                        [0, 1, 2, 3], [4, 4, 4, 4],
                        [11, 10, 11, 10], [1, 2, 3, 4],
                        [6, 7, 8, 9], [9, 8, 7, 6],
                        [0, 0, 0, 0], [0, 0, 0, 0],
                        [2, 4, 6, 8], [8, 6, 4, 2]]).view(1, 1, 12, T).expand(1, H, 12, T).contiguous()
    _check(q, k, v, lut, dev)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_fused_linear_branch_on_a_split_pair(dev, dtype):
    """The fused entry (attention + linear branch + projection) on hand-made rows, against the oracle's forward."""
    from sla_amd.inputs import make_proj
    from sla_amd.linear import linear_state_fwd
    from sla_amd.sparse_attn import sparse_attn_linear_fwd

    L, T = 1217, 6
    g = torch.Generator().manual_seed(33)
    H = _heads(L)
    q, k, v = _qkv(H, L, 34, dtype)
    M = N = (L + 63) // 64
    lut = torch.stack([_rows(M, N, T, 4, g) for _ in range(H)]).view(1, H, M, T)
    w, b = make_proj(128)
    o_s_ref, _ = O.sparse_attn_fwd_gather(q, k, v, lut, 64, 64)
    ref = o_s_ref + O.linear_branch(q, k, v, w, b, "softmax", dtype).float()
    qd, kd, vd = q.to(dev), k.to(dev), v.to(dev)
    ws = linear_state_fwd(kd, vd, w.to(dev), "softmax")
    out, o_s, lse = sparse_attn_linear_fwd(qd, kd, vd, lut.to(dev), T, 64, 64, 128 ** -0.5, ws, b.to(dev), "softmax",
                                           want_o_s=True)
    assert max_abs(o_s.cpu(), o_s_ref) <= TOL_ABS
    assert max_abs(out.cpu(), ref) <= _sum_tol(ref) and cos_sim(out.cpu(), ref) >= TOL_COS


@pytest.mark.parametrize("L", [1024,      # whole 128-row blocks
                               1000,      # the last block's second half is ragged (and so is the last key block)
                               960,       # the last block has no second half at all
                               1217])
def test_query_blocks_of_128_rows(dev, L):
    """A 128-row query block goes through the same kernel as a pair of 64-row blocks whose two look-up rows are its one
    row: against the oracle at BLOCK_M = 128 (the shape of the reference's evaluate/bench_kernel.py:60-61), and bit for
    bit against the 64-row call with every row of the table written twice."""
    T = 5
    M, N = (L + 127) // 128, (L + 63) // 64
    pairs_per_head = M
    H = -(-512 // pairs_per_head)
    g = torch.Generator().manual_seed(L)
    q, k, v = _qkv(H, L, 200 + L)
    lut = torch.stack([torch.stack([torch.randperm(N, generator=g)[:T] for _ in range(M)]) for _ in range(H)]).view(1, H, M, T)
    o_ref, lse_ref = O.sparse_attn_fwd_gather(q, k, v, lut, 128, 64)
    qd, kd, vd = q.to(dev), k.to(dev), v.to(dev)
    o, lse = sparse_attn_fwd(qd, kd, vd, lut.to(dev), T, 128, 64, 128 ** -0.5)
    assert torch.isfinite(o.float()).all()
    assert max_abs(o.cpu(), o_ref) <= TOL_ABS and cos_sim(o.cpu(), o_ref) >= TOL_COS
    assert max_abs(lse.cpu(), lse_ref) <= TOL_LSE
    M64 = (L + 63) // 64
    lut64 = lut.repeat_interleave(2, dim=2)[:, :, :M64].contiguous()
    o2, lse2 = sparse_attn_fwd(qd, kd, vd, lut64.to(dev), T, 64, 64, 128 ** -0.5)
    assert torch.equal(o, o2) and torch.equal(lse, lse2)
    # the same with the linear branch in the epilogue
    from sla_amd.inputs import make_proj
    from sla_amd.linear import linear_state_fwd
    from sla_amd.sparse_attn import sparse_attn_linear_fwd
    w, b = make_proj(128)
    ws = linear_state_fwd(kd, vd, w.to(dev), "elu")
    out, o_s, lse3 = sparse_attn_linear_fwd(qd, kd, vd, lut.to(dev), T, 128, 64, 128 ** -0.5, ws, b.to(dev), "elu", want_o_s=True)
    out2, o_s2, lse4 = sparse_attn_linear_fwd(qd, kd, vd, lut64.to(dev), T, 64, 64, 128 ** -0.5, ws, b.to(dev), "elu", want_o_s=True)
    assert torch.equal(o_s, o) and torch.equal(lse3, lse)
    assert torch.equal(out, out2) and torch.equal(o_s, o_s2) and torch.equal(lse3, lse4)
    ref = o_ref + O.linear_branch(q, k, v, w, b, "elu", torch.bfloat16).float()
    assert max_abs(out.cpu(), ref) <= _sum_tol(ref) and cos_sim(out.cpu(), ref) >= TOL_COS
