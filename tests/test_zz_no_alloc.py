"""The block-mask builder's entry point that allocates nothing (``sla_block_map_fwd_static``: its workspace is a
fixed array in device memory) against ``sla_block_map_fwd`` with a caller-provided workspace: same map and
look-up table, bit for bit, on two calls in a row, the second on a smaller input."""
import pytest
import torch

from sla_amd import _lib, get_block_map
from sla_amd.block_map import topk_count
from sla_amd.inputs import CONFIGS, make_inputs


def _static_map(q, k, ratio, BLKQ, BLKK, lut_dtype=torch.int64):
    """Calls the entry point through the C ABI; the only device memory involved besides the library's own array is
    the inputs and outputs allocated here, before the call."""
    B, H, L, D = q.shape
    M, N = -(-L // BLKQ), -(-L // BLKK)
    T = topk_count(N, ratio)
    sparse_map = torch.full((B, H, M, N), -1, dtype=torch.int8, device=q.device)
    lut = torch.full((B, H, M, T), -1, dtype=lut_dtype, device=q.device)
    def call():
        rc = _lib.load().sla_block_map_fwd_static(q.data_ptr(), k.data_ptr(), _lib.dtype_code(q.dtype), B, H, L, D, BLKQ,
                                                  BLKK, T, sparse_map.data_ptr(), lut.data_ptr(), lut.element_size(),
                                                  _lib.stream_ptr(q.device))
        _lib.check(rc)
        torch.cuda.synchronize()

    call()                       # the first call on a device looks the array's address up and loads the kernels
    # The second one is watched at the driver's level: torch's own counters only see torch's allocator, and a
    # hipMalloc inside the library, made through ctypes, would pass them by.
    torch.cuda.synchronize()
    free_before, _ = torch.cuda.mem_get_info(q.device)
    torch_before = torch.cuda.memory_allocated(q.device)
    sparse_map.fill_(-1)
    lut.fill_(-1)
    call()
    free_after, _ = torch.cuda.mem_get_info(q.device)
    assert free_after == free_before, f"device memory in use changed by {free_before - free_after} bytes during the call"
    assert torch.cuda.memory_allocated(q.device) == torch_before
    return sparse_map, lut, T


@pytest.mark.gpu
def test_static_scratch_entry_point_matches_the_workspace_one(dev):
    g = torch.Generator().manual_seed(11)
    # first call: two heads of the headline shape (ragged last blocks); second call: a smaller input of another
    # dtype and block size, so that stale contents of the shared array would show
    cfg = CONFIGS["cfg3"]
    d = make_inputs(cfg, H=2)
    q1, k1 = d["q"].to(dev), d["k"].to(dev)
    q2 = torch.randn(2, 3, 777, 64, generator=g).to(torch.float16).to(dev)
    k2 = (torch.randn(2, 3, 777, 64, generator=g) + 0.7).to(torch.float16).to(dev)
    q3 = torch.randn(1, 2, 1024, 64, generator=g).to(dev)              # fp32 inputs, as the reference's own dtype order
    k3 = torch.randn(1, 2, 1024, 64, generator=g).to(dev)
    for q, k, ratio, BLKQ, lut_dtype in ((q1, k1, cfg.topk, 64, torch.int64), (q2, k2, 0.3, 128, torch.int32),
                                         (q3, k3, 0.2, 64, torch.int64), (q1, k1, cfg.topk, 64, torch.int64)):
        m_ref, lut_ref, T_ref = get_block_map(q, k, ratio, BLKQ, 64)
        m, lut, T = _static_map(q, k, ratio, BLKQ, 64, lut_dtype)
        assert T == T_ref
        assert torch.equal(m, m_ref), f"map differs in {(m != m_ref).sum().item()} cells"
        assert torch.equal(lut.long(), lut_ref)


@pytest.mark.gpu
def test_static_scratch_entry_point_refuses_what_does_not_fit(dev):
    # the whole headline shape fits (12.7 MB of 16 MiB) ...
    need = _lib.load().sla_workspace_bytes(_lib.WS_BLOCK_MAP, _lib.SLA_BF16, 1, 12, 32760, 128, 64, 64, 25)
    assert 0 < need <= _lib.STATIC_SCRATCH_BYTES
    # ... forty heads of it do not: a clear error before anything is launched, outputs untouched
    q = torch.zeros(1, 40, 32760, 128, dtype=torch.bfloat16, device=dev)
    sparse_map = torch.full((1, 40, 512, 512), -1, dtype=torch.int8, device=dev)
    lut = torch.full((1, 40, 512, 25), -1, dtype=torch.int64, device=dev)
    rc = _lib.load().sla_block_map_fwd_static(q.data_ptr(), q.data_ptr(), _lib.SLA_BF16, 1, 40, 32760, 128, 64, 64, 25,
                                              sparse_map.data_ptr(), lut.data_ptr(), 8, _lib.stream_ptr(dev))
    assert rc == _lib.ERR_WORKSPACE and "static buffer" in _lib.last_error()
    torch.cuda.synchronize()
    assert bool((sparse_map == -1).all()) and bool((lut == -1).all())


def test_size_limit_is_checked_before_any_device_work():
    """No GPU needed: a problem that does not fit the fixed array is refused from its sizes alone."""
    lib = _lib.load()
    FAKE = 0x1000
    assert lib.sla_block_map_fwd_static(FAKE, FAKE, _lib.SLA_BF16, 1, 40, 32760, 128, 64, 64, 25, FAKE, FAKE, 8,
                                        None) == _lib.ERR_WORKSPACE
    assert "static buffer" in _lib.last_error() and str(_lib.STATIC_SCRATCH_BYTES) in _lib.last_error()
    assert lib.sla_block_map_fwd_static(FAKE, FAKE, 7, 1, 1, 64, 64, 64, 64, 1, FAKE, FAKE, 8, None) == _lib.ERR_BAD_ARG
    assert lib.sla_block_map_fwd_static(None, FAKE, _lib.SLA_BF16, 1, 1, 64, 64, 64, 64, 1, FAKE, FAKE, 8,
                                        None) == _lib.ERR_BAD_ARG
