"""CPU-only checks of the C ABI: the library loads, exports every symbol the header declares,
and validates arguments before touching the device (so error paths need no GPU)."""
import os
import re

import pytest

from sla_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "sla_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(sla_\w+|sage_\w+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = _lib.load()
    names = _declared_symbols()
    assert len(names) >= 12
    for n in names:
        assert hasattr(lib, n), n
    assert set(names) == set(_lib.SIGNATURES), "python binding and header disagree"
    assert lib.sla_version() >= 1


def test_workspace_sizes():
    lib = _lib.load()
    n = lib.sla_workspace_bytes(_lib.WS_BLOCK_MAP, _lib.SLA_BF16, 1, 12, 32760, 128, 64, 64, 25)
    # chunk sums + column mean + pooled q/k + scores for cfg3
    assert n >= 12 * (512 * 128 * 4 + 2 * 512 * 128 * 2 + 512 * 512 * 2)
    assert lib.sla_workspace_bytes(_lib.WS_BLOCK_MAP, 7, 1, 1, 64, 64, 64, 64, 1) == _lib.ERR_BAD_ARG
    assert lib.sla_workspace_bytes(99, 1, 1, 1, 64, 64, 64, 64, 1) == _lib.ERR_BAD_ARG
    assert lib.sla_workspace_bytes(_lib.WS_SPARSE_BWD, 1, 0, 1, 64, 64, 64, 64, 1) == _lib.ERR_BAD_ARG
    for op in (_lib.WS_SPARSE_BWD, _lib.WS_LINEAR_FWD, _lib.WS_LINEAR_BWD, _lib.WS_SAGE_QUANT):
        assert lib.sla_workspace_bytes(op, 1, 2, 4, 4096, 128, 64, 64, 12) > 0


FAKE = 0x1000  # non-null, 16-byte aligned; never dereferenced because validation fails first


def test_attention_rejects_bad_shapes_before_launch():
    lib = _lib.load()
    args = dict(q=FAKE, k=FAKE, v=FAKE, lut=FAKE, lb=8, o=FAKE, lse=FAKE)

    def call(dtype=1, B=1, H=1, L=128, D=128, BLKQ=64, BLKK=64, topk=1, **kw):
        a = {**args, **kw}
        return lib.sla_sparse_attn_fwd(a["q"], a["k"], a["v"], a["lut"], a["lb"], a["o"], a["lse"], dtype, B, H, L, D,
                                       BLKQ, BLKK, topk, 0.1, None)
    assert call(BLKQ=32) == _lib.ERR_UNSUPPORTED and "BLOCK_M" in _lib.last_error()
    assert call(BLKK=128) == _lib.ERR_UNSUPPORTED and "BLOCK_N" in _lib.last_error()
    assert call(D=96) == _lib.ERR_UNSUPPORTED
    assert call(dtype=0) == _lib.ERR_UNSUPPORTED
    assert call(topk=3) == _lib.ERR_BAD_ARG
    assert call(L=0) == _lib.ERR_BAD_ARG
    assert call(lb=2) == _lib.ERR_BAD_ARG
    assert call(q=None) == _lib.ERR_BAD_ARG and "null" in _lib.last_error()
    assert call(q=FAKE + 2) == _lib.ERR_BAD_ARG and "aligned" in _lib.last_error()
    with pytest.raises(AssertionError):
        _lib.check(call(BLKQ=32))
    with pytest.raises(ValueError):
        _lib.check(call(q=None))


def test_other_entry_points_validate():
    import ctypes
    lib = _lib.load()
    assert lib.sla_mean_pool(None, FAKE, 1, 1, 64, 64, 64, None) == _lib.ERR_BAD_ARG
    assert lib.sla_mean_pool(FAKE, FAKE, 1, 1, 64, 60, 64, None) == _lib.ERR_UNSUPPORTED
    assert lib.sla_block_map_fwd(FAKE, FAKE, 1, 1, 1, 128, 64, 64, 64, 5, FAKE, 1 << 30, FAKE, FAKE, 8, None) == _lib.ERR_BAD_ARG
    assert lib.sla_block_map_fwd(FAKE, FAKE, 1, 1, 1, 128, 64, 64, 64, 1, FAKE, 16, FAKE, FAKE, 8, None) == _lib.ERR_WORKSPACE
    assert lib.sla_linear_fwd(FAKE, FAKE, FAKE, FAKE, FAKE, None, FAKE, 1, 9, 1, 1, 64, 128, FAKE, 1 << 30, None) == _lib.ERR_BAD_ARG
    assert lib.sla_linear_fwd(FAKE, FAKE, FAKE, FAKE, FAKE, None, FAKE, 1, 0, 1, 1, 64, 96, FAKE, 1 << 30, None) == _lib.ERR_UNSUPPORTED
    assert lib.sla_sparse_attn_linear_fwd(FAKE, FAKE, FAKE, FAKE, 8, FAKE, 8, FAKE, None, FAKE, FAKE, 1, 0, 1, 1, 128, 128,
                                          64, 64, 1, 0.1, None) == _lib.ERR_WORKSPACE
    assert lib.sla_sparse_attn_linear_fwd(FAKE, FAKE, FAKE, FAKE, 8, FAKE, 1 << 30, FAKE, None, FAKE, FAKE, 1, 7, 1, 1, 128,
                                          128, 64, 64, 1, 0.1, None) == _lib.ERR_BAD_ARG
    assert lib.sla_linear_complement_fwd(FAKE, FAKE, FAKE, FAKE, 8, FAKE, FAKE, None, FAKE, 1, 0, 1, 1, 128, 128, 64, 32, 1,
                                         FAKE, 1 << 30, None) == _lib.ERR_UNSUPPORTED
    cb = lambda **kw: lib.sla_linear_complement_bwd(  # noqa: E731
        FAKE, FAKE, FAKE, kw.get("m", FAKE), FAKE, 8, FAKE, FAKE, FAKE, FAKE, FAKE, FAKE, FAKE, FAKE, 1, 0, 1, 1, 128, 128,
        kw.get("BLKQ", 64), 64, 1, kw.get("flags", 0), FAKE, kw.get("ws", 1 << 30), None)
    assert cb(ws=8) == _lib.ERR_WORKSPACE
    assert cb(flags=2) == _lib.ERR_BAD_ARG and "flag" in _lib.last_error()
    assert cb(m=None) == _lib.ERR_BAD_ARG
    assert cb(BLKQ=32) == _lib.ERR_UNSUPPORTED
    need = lib.sla_workspace_bytes(_lib.WS_LINEAR_COMPLEMENT_BWD, 1, 1, 2, 128, 128, 64, 64, 1)
    assert need > lib.sla_workspace_bytes(_lib.WS_LINEAR_COMPLEMENT, 1, 1, 2, 128, 128, 64, 64, 1) > 0
    assert lib.sla_linear_state_fwd(FAKE, FAKE, FAKE, 1, 0, 1, 1, 64, 128, FAKE, 8, None) == _lib.ERR_WORKSPACE
    assert lib.sla_linear_state_fwd(FAKE, None, FAKE, 1, 0, 1, 1, 64, 128, FAKE, 1 << 30, None) == _lib.ERR_BAD_ARG
    # the state build with the FP8 quantisation of v in the same call: the checks of both
    sq = lib.sla_linear_state_quant_v_fwd
    assert sq(FAKE, FAKE, FAKE, 1, 0, 1, 1, 64, 128, FAKE, 8, FAKE, FAKE, 448.0, None) == _lib.ERR_WORKSPACE
    assert sq(FAKE, FAKE, FAKE, 1, 0, 1, 1, 64, 128, FAKE, 1 << 30, None, FAKE, 448.0, None) == _lib.ERR_BAD_ARG
    assert sq(FAKE, FAKE, FAKE, 1, 0, 1, 1, 64, 128, FAKE, 1 << 30, FAKE, FAKE, 449.0, None) == _lib.ERR_BAD_ARG
    assert "v_range" in _lib.last_error()
    assert sq(FAKE, FAKE, FAKE, 1, 7, 1, 1, 64, 128, FAKE, 1 << 30, FAKE, FAKE, 448.0, None) == _lib.ERR_BAD_ARG
    assert lib.sla_linear_state_quant_v_fwd_strided(FAKE, FAKE, None, FAKE, 1, 0, 1, 1, 64, 128, FAKE, 1 << 30, FAKE, FAKE,
                                                    448.0, None) == _lib.ERR_BAD_ARG
    assert lib.sla_linear_out_fwd(FAKE, FAKE, None, FAKE, 0, 0, 1, 1, 64, 128, FAKE, 1 << 30, None) == _lib.ERR_UNSUPPORTED
    assert lib.sla_linear_out_fwd(FAKE, FAKE, None, FAKE, 1, 0, 1, 1, 64, 128, None, 1 << 30, None) == _lib.ERR_BAD_ARG
    assert lib.sla_linear_bwd(FAKE, FAKE, FAKE, FAKE, FAKE, FAKE, FAKE, FAKE, FAKE, FAKE, FAKE, 1, 0, 1, 1, 64, 128, 0, FAKE,
                              8, None) == _lib.ERR_WORKSPACE
    assert lib.sla_linear_bwd(FAKE, FAKE, FAKE, FAKE, FAKE, FAKE, FAKE, FAKE, FAKE, FAKE, FAKE, 1, 0, 1, 1, 64, 128, 4, FAKE,
                              1 << 30, None) == _lib.ERR_BAD_ARG and "flag" in _lib.last_error()
    states = lib.sla_workspace_bytes(_lib.WS_LINEAR_STATES, 1, 1, 12, 32760, 128, 64, 64, 0)
    assert 0 < states <= 12 * 3 * 128 * 128 * 2 + 12 * 128 * 2 + 128 * 128 * 2 + 5 * 256
    assert states < lib.sla_workspace_bytes(_lib.WS_LINEAR_FWD, 1, 1, 12, 32760, 128, 64, 64, 0)
    assert lib.sla_sparse_attn_bwd(FAKE, FAKE, FAKE, FAKE, FAKE, FAKE, FAKE, FAKE, 8, FAKE, FAKE, FAKE, 1, 1, 1, 128, 128, 64,
                                   64, 1, 0.1, FAKE, 8, None) == _lib.ERR_WORKSPACE
    # the one-call backward: its own arguments first, then what the two calls it stands for check
    mb = lambda **kw: lib.sla_module_bwd(  # noqa: E731
        FAKE, FAKE, FAKE, kw.get("qs"), FAKE, FAKE, kw.get("dos"), FAKE, FAKE, FAKE, 8, kw.get("w", FAKE), FAKE, FAKE, FAKE,
        FAKE, FAKE, FAKE, 1, kw.get("fmap", 0), 1, 1, 128, 128, 64, 64, 1, 0.1, kw.get("flags", 0), FAKE,
        kw.get("ws_s", 1 << 30), FAKE, kw.get("ws_l", 1 << 30), None, None)
    assert mb(flags=1) == _lib.ERR_BAD_ARG and "flag" in _lib.last_error()           # accumulation is implied, not a flag
    assert mb(qs=(ctypes.c_int64 * 3)(16384, 16384, 128)) == _lib.ERR_BAD_ARG and "stride" in _lib.last_error()
    assert mb(ws_s=8) == _lib.ERR_WORKSPACE
    assert mb(ws_l=8) == _lib.ERR_WORKSPACE
    assert mb(w=None) == _lib.ERR_BAD_ARG
    assert mb(fmap=5) == _lib.ERR_BAD_ARG
    assert lib.sage_quant_qk(FAKE, FAKE, 1, 1, 1, 128, 128, 64, 64, FAKE, FAKE, FAKE, FAKE, FAKE, 1 << 30, None) == _lib.ERR_UNSUPPORTED
    assert "BLKQ=128" in _lib.last_error()
    assert lib.sage_quant_v(FAKE, 1, 1, 1, 128, 32, FAKE, FAKE, 448.0, FAKE, 1 << 30, None) == _lib.ERR_UNSUPPORTED
    assert "headdim" in _lib.last_error()
    # range of the e4m3 values: (0, 448]; 2.25 is the reference's constant (SageSLA/core.py:129)
    for bad in (0.0, -1.0, 449.0, float("nan")):
        assert lib.sage_quant_v(FAKE, 1, 1, 1, 128, 128, FAKE, FAKE, bad, FAKE, 1 << 30, None) == _lib.ERR_BAD_ARG
        assert "v_range" in _lib.last_error()
    assert lib.sage_quant_v(FAKE, 1, 1, 1, 128, 128, FAKE, FAKE, 2.25, FAKE, 8, None) == _lib.ERR_WORKSPACE
    assert lib.sage_sparse_attn_fwd(FAKE, FAKE, FAKE, FAKE, FAKE, FAKE, FAKE, 8, FAKE, 1, 1, 1, 128, 128, 128, 64, 9, 0.1,
                                    None) == _lib.ERR_BAD_ARG
    # strided variants: strides are {batch, head, row} in elements, checked before anything is launched
    import ctypes
    st = lambda *v: (ctypes.c_int64 * 3)(*v)  # noqa: E731
    bm = lambda strides: lib.sla_block_map_fwd_strided(FAKE, FAKE, strides, 1, 1, 2, 256, 128, 64, 64, 1, FAKE, 1 << 30,  # noqa: E731
                                                       FAKE, FAKE, 8, None)
    assert bm(None) == _lib.ERR_BAD_ARG and "strides" in _lib.last_error()
    assert bm(st(65536, 128, 100)) == _lib.ERR_BAD_ARG          # row stride below D
    assert bm(st(65536, 128, 260)) == _lib.ERR_BAD_ARG and "16-byte" in _lib.last_error()
    assert bm(st(1 << 40, 128, 1 << 30)) == _lib.ERR_UNSUPPORTED and "4 GiB" in _lib.last_error()
    # heads whose rows alias each other: head stride D with row stride D puts row l of head 1 on row l + 1 of head 0
    assert bm(st(65536, 128, 128)) == _lib.ERR_BAD_ARG and "overlap" in _lib.last_error()
    assert bm(st(65536, 128, 136)) == _lib.ERR_BAD_ARG and "overlap" in _lib.last_error()     # interleaved, row too short
    assert bm(st(65536, 256 * 128 - 8, 128)) == _lib.ERR_BAD_ARG and "overlap" in _lib.last_error()  # disjoint but 8 short
    assert lib.sla_linear_state_fwd_strided(FAKE, FAKE, st(65536, 128, 257), FAKE, 1, 0, 1, 2, 256, 128, FAKE, 1 << 30,
                                            None) == _lib.ERR_BAD_ARG
    assert lib.sla_sparse_attn_linear_fwd_strided(FAKE, FAKE, FAKE, st(65536, 128, 256), FAKE, 8, FAKE, 1 << 30, FAKE, None,
                                                  FAKE, st(65536, 128, 4), FAKE, 1, 0, 1, 2, 256, 128, 64, 64, 1, 0.1,
                                                  None) == _lib.ERR_BAD_ARG
    assert lib.sla_linear_out_fwd_strided(FAKE, st(65536, 128, 256), FAKE, None, FAKE, st(65536, 128, 100), 1, 0, 1, 2, 256, 128,
                                          FAKE, 1 << 30, None) == _lib.ERR_BAD_ARG
    assert lib.sla_linear_out_fwd_strided(FAKE, None, FAKE, None, FAKE, st(65536, 128, 256), 1, 0, 1, 2, 256, 128, FAKE, 1 << 30,
                                          None) == _lib.ERR_BAD_ARG and "strides" in _lib.last_error()
    assert lib.sage_quant_v_strided(FAKE, st(65536, 128, 260), 1, 1, 2, 256, 128, FAKE, FAKE, 448.0, FAKE, 1 << 30,
                                    None) == _lib.ERR_BAD_ARG and "16-byte" in _lib.last_error()
    assert lib.sage_prepare_strided(FAKE, FAKE, None, st(65536, 128, 64), 1, 1, 2, 256, 128, 128, 64, 1, FAKE, FAKE, 8, FAKE, FAKE,
                                    FAKE, FAKE, None, None, 448.0, FAKE, 1 << 30, None) == _lib.ERR_BAD_ARG
    # one-call SageSLA preparation: block sizes, topk range and workspace are checked before any launch
    # (v and its two outputs may be left out together, not separately)
    assert lib.sage_prepare(FAKE, FAKE, None, 1, 1, 1, 256, 128, 128, 64, 2, FAKE, FAKE, 8, FAKE, FAKE, FAKE, FAKE, FAKE, None,
                            448.0, FAKE, 1 << 30, None) == _lib.ERR_BAD_ARG
    prep = lambda BLKQ, topk, ws: lib.sage_prepare(FAKE, FAKE, FAKE, 1, 1, 1, 256, 128, BLKQ, 64, topk, FAKE, FAKE, 8, FAKE,  # noqa: E731
                                                   FAKE, FAKE, FAKE, FAKE, FAKE, 448.0, FAKE, ws, None)
    assert prep(64, 1, 1 << 30) == _lib.ERR_UNSUPPORTED
    assert prep(128, 5, 1 << 30) == _lib.ERR_BAD_ARG and "topk" in _lib.last_error()
    assert prep(128, 2, 8) == _lib.ERR_WORKSPACE
    need = lib.sla_workspace_bytes(_lib.WS_SAGE_PREPARE, 1, 1, 1, 256, 128, 128, 64, 2)
    assert need > lib.sla_workspace_bytes(_lib.WS_SAGE_QUANT, 1, 1, 1, 256, 128, 128, 64, 2) > 0


def test_host_api_mirrors_reference_names_and_errors():
    import torch

    import SageSLA
    import sparse_linear_attention as sla
    from sparse_linear_attention.kernel import _attention
    from sparse_linear_attention.utils import get_block_map, mean_pool  # noqa: F401
    mod = sla.SparseLinearAttention(head_dim=128, topk=0.2, feature_map="softmax", BLKQ=64, BLKK=64)
    assert set(mod.state_dict()) == {"proj_l.weight", "proj_l.bias"}
    assert mod.dtype == torch.bfloat16 and sla.SparseLinearAttention(64, 0.1, use_bf16=False).dtype == torch.float16
    with pytest.raises(NotImplementedError):
        sla.SparseLinearAttention(128, 0.2, feature_map="hedgehog")
    sage = SageSLA.SageSparseLinearAttention(head_dim=128, topk=0.2, feature_map="softmax", BLKQ=128, BLKK=64)
    assert set(sage.state_dict()) == {"proj_l.weight", "proj_l.bias"}
    x = torch.zeros(1, 1, 128, 128, dtype=torch.bfloat16)
    with pytest.raises(AssertionError):          # reference asserts contiguity first (kernel.py:243)
        _attention.apply(x.transpose(-1, -2), x, x, torch.zeros(1, 1, 2, 2, dtype=torch.int8),
                         torch.zeros(1, 1, 2, 1, dtype=torch.int64), 1, 64, 64)
    with pytest.raises(AssertionError):          # BLOCK_M must be 64 or 128 (kernel.py:247)
        _attention.apply(x, x, x, torch.zeros(1, 1, 2, 2, dtype=torch.int8), torch.zeros(1, 1, 2, 1, dtype=torch.int64),
                         1, 32, 64)
    with pytest.raises(RuntimeError):            # no CPU fallback: CPU tensors are refused loudly
        mod(x, x, x)


def test_missing_library_fails_loudly(monkeypatch):
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", "/nonexistent/libsla_hip.so")
    with pytest.raises(ImportError):
        _lib.load()
