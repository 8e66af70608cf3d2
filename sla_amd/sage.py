"""SageSLA: quantised forward of Sparse-Linear Attention (INT8 QK^T, FP8 PV).

Mirrors ``SageSparseLinearAttention`` of ``SageSLA/core.py:33-163``: same constructor,
parameters and forward; inference only.  The reference picks block sizes from the CUDA
architecture (``SageSLA/core.py:90-94``); gfx950 has one path, BLKQ=128 / BLKK=64.
"""
from __future__ import annotations

import torch
import torch.nn as nn

from . import _lib
from .block_map import get_block_map, topk_count
from .linear import linear_out_fwd
from .module import FEATURE_MAPS, _StateBuild

SAGE_BLKQ, SAGE_BLKK = 128, 64
# Range of the e4m3 values v is quantised to.  The reference's call passes 2.25 (SageSLA/core.py:129), which keeps the
# fp16 accumulators of its PV product finite; the kernel here accumulates in fp32 and uses the whole e4m3 range.
V_RANGE_E4M3, V_RANGE_REFERENCE = 448.0, 2.25


def quant_qk(q, k):
    """Per-block INT8 q and mean-smoothed k.  Returns (q_int8, q_scale, k_int8, k_scale)."""
    _lib.require_gpu(q, k)
    B, H, L, D = q.shape
    dt = _lib.dtype_code(q.dtype)
    M, N = (L + SAGE_BLKQ - 1) // SAGE_BLKQ, (L + SAGE_BLKK - 1) // SAGE_BLKK
    ws = _lib.workspace(_lib.WS_SAGE_QUANT, dt, B, H, L, D, SAGE_BLKQ, SAGE_BLKK, 0, q.device)
    q8 = torch.empty((B, H, L, D), dtype=torch.int8, device=q.device)
    k8 = torch.empty((B, H, L, D), dtype=torch.int8, device=q.device)
    qs = torch.empty((B, H, M), dtype=torch.float32, device=q.device)
    ks = torch.empty((B, H, N), dtype=torch.float32, device=q.device)
    rc = _lib.load().sage_quant_qk(q.data_ptr(), k.data_ptr(), dt, B, H, L, D, SAGE_BLKQ, SAGE_BLKK, q8.data_ptr(),
                                   qs.data_ptr(), k8.data_ptr(), ks.data_ptr(), ws.data_ptr(), ws.numel(),
                                   _lib.stream_ptr(q.device))
    _lib.check(rc)
    return q8, qs, k8, ks


def quant_v(v, v_range=V_RANGE_E4M3):
    """Per-channel FP8 e4m3 v (contiguous or a row-contiguous view).  Returns (v_fp8 (B,H,L,D) float8_e4m3fn, contiguous,
    v_scale (B,H,D) fp32 = max_L|v| / v_range).  ``v_range=2.25`` is the reference's constant (SageSLA/core.py:129)."""
    _lib.require_gpu(v)
    B, H, L, D = v.shape
    dt = _lib.dtype_code(v.dtype)
    ws = _lib.workspace(_lib.WS_SAGE_QUANT, dt, B, H, L, D, SAGE_BLKQ, SAGE_BLKK, 0, v.device)
    v8 = torch.empty((B, H, L, D), dtype=torch.float8_e4m3fn, device=v.device)
    vs = torch.empty((B, H, D), dtype=torch.float32, device=v.device)
    if v.is_contiguous():
        rc = _lib.load().sage_quant_v(v.data_ptr(), dt, B, H, L, D, v8.data_ptr(), vs.data_ptr(), float(v_range), ws.data_ptr(),
                                      ws.numel(), _lib.stream_ptr(v.device))
    else:
        assert _lib.row_strided(v), "v must be contiguous or a row-contiguous view"
        rc = _lib.load().sage_quant_v_strided(v.data_ptr(), _lib.strides_arg(v), dt, B, H, L, D, v8.data_ptr(), vs.data_ptr(),
                                              float(v_range), ws.data_ptr(), ws.numel(), _lib.stream_ptr(v.device))
    _lib.check(rc)
    return v8, vs


def sage_prepare(q, k, v, topk_ratio, v_range=V_RANGE_E4M3):
    """Block map, INT8 q / k and FP8 v in one library call (q, k, v already in the compute dtype; contiguous, or
    row-contiguous views with common strides: the quantised tensors are contiguous (B, H, L, D) either way).

    Returns ``(sparse_map, lut, T, q_int8, q_scale, k_int8, k_scale, v_fp8, v_scale)``, identical to
    ``get_block_map`` + ``quant_qk`` + ``quant_v`` on the same tensors; the k column mean and the block
    means are shared between the mask and the quantisers instead of being formed twice.  With ``v=None`` the
    v part is left out (``v_fp8`` and ``v_scale`` are returned as None) for a caller that runs ``quant_v`` elsewhere.
    """
    _lib.require_gpu(q, k)
    tensors = (q, k) if v is None else (q, k, v)
    contiguous = all(t.is_contiguous() for t in tensors)
    assert contiguous or _lib.row_strided(*tensors), "q, k, v must be contiguous or share row-contiguous strides"
    assert q.shape == k.shape and q.dtype == k.dtype
    if v is not None:
        _lib.require_gpu(v)
        assert v.shape == q.shape and v.dtype == q.dtype
    B, H, L, D = q.shape
    dt = _lib.dtype_code(q.dtype)
    M, N = (L + SAGE_BLKQ - 1) // SAGE_BLKQ, (L + SAGE_BLKK - 1) // SAGE_BLKK
    T = topk_count(N, topk_ratio)
    dev = q.device
    ws = _lib.workspace(_lib.WS_SAGE_PREPARE, dt, B, H, L, D, SAGE_BLKQ, SAGE_BLKK, T, dev)
    sparse_map = torch.empty((B, H, M, N), dtype=torch.int8, device=dev)
    lut = torch.empty((B, H, M, T), dtype=torch.int64, device=dev)
    q8 = torch.empty((B, H, L, D), dtype=torch.int8, device=dev)
    k8 = torch.empty((B, H, L, D), dtype=torch.int8, device=dev)
    qs = torch.empty((B, H, M), dtype=torch.float32, device=dev)
    ks = torch.empty((B, H, N), dtype=torch.float32, device=dev)
    v8 = vs = None
    if v is not None:
        v8 = torch.empty((B, H, L, D), dtype=torch.float8_e4m3fn, device=dev)
        vs = torch.empty((B, H, D), dtype=torch.float32, device=dev)
    tail = (dt, B, H, L, D, SAGE_BLKQ, SAGE_BLKK, T, sparse_map.data_ptr(), lut.data_ptr(), 8, q8.data_ptr(), qs.data_ptr(),
            k8.data_ptr(), ks.data_ptr(), None if v is None else v8.data_ptr(), None if v is None else vs.data_ptr(),
            float(v_range), ws.data_ptr(), ws.numel(), _lib.stream_ptr(dev))
    vp = None if v is None else v.data_ptr()
    if contiguous:
        rc = _lib.load().sage_prepare(q.data_ptr(), k.data_ptr(), vp, *tail)
    else:
        rc = _lib.load().sage_prepare_strided(q.data_ptr(), k.data_ptr(), vp, _lib.strides_arg(q), *tail)
    _lib.check(rc)
    return sparse_map, lut, T, q8, qs, k8, ks, v8, vs


def sage_attn_fwd(q8, qs, k8, ks, v8, vs, lut, topk, out_dtype, qk_scale=None):
    B, H, L, D = q8.shape
    if qk_scale is None:
        qk_scale = D ** -0.5
    o = torch.empty((B, H, L, D), dtype=out_dtype, device=q8.device)
    lut_bytes = 8 if lut.dtype == torch.int64 else 4
    rc = _lib.load().sage_sparse_attn_fwd(q8.data_ptr(), qs.data_ptr(), k8.data_ptr(), ks.data_ptr(), v8.data_ptr(),
                                          vs.data_ptr(), lut.data_ptr(), lut_bytes, o.data_ptr(),
                                          _lib.dtype_code(out_dtype), B, H, L, D, SAGE_BLKQ, SAGE_BLKK, topk,
                                          float(qk_scale), _lib.stream_ptr(q8.device))
    _lib.check(rc)
    return o


class SageSparseLinearAttention(nn.Module):
    def __init__(self, head_dim, topk, feature_map="softmax", use_bf16=True, tie_feature_map_qk=True, BLKQ=SAGE_BLKQ,
                 BLKK=SAGE_BLKK):
        r"""
        Args:
            head_dim: dimension of each head (64 or 128).
            topk: ratio of keys selected for sparse attention, shared across all queries.
            feature_map: feature map for linear attention, one of ['elu', 'relu', 'softmax'].
            use_bf16: bfloat16 (default) or float16 compute.
            tie_feature_map_qk: kept for signature compatibility.
            BLKQ, BLKK: accepted because the reference's README passes them; only 128 / 64 exist.
        """
        super().__init__()
        assert BLKQ == SAGE_BLKQ and BLKK == SAGE_BLKK, "SageSLA only supports BLKQ=128 and BLKK=64"
        self.dtype = torch.bfloat16 if use_bf16 else torch.float16
        self.topk = topk
        self.proj_l = nn.Linear(head_dim, head_dim, dtype=torch.float32)
        if feature_map not in FEATURE_MAPS:
            raise NotImplementedError(f"Not supported feature map {feature_map}.")
        self.feature_map = feature_map
        self.init_weights_()

    def init_weights_(self):
        with torch.no_grad():
            nn.init.zeros_(self.proj_l.weight)
            nn.init.zeros_(self.proj_l.bias)

    @torch.no_grad()
    def forward(self, q, k, v, return_sparsity=False):
        _lib.require_gpu(q, k, v)          # no CPU path: refuse loudly before anything touches a stream
        dtype = q.dtype
        # (B, L, H, D) activations or slices of a packed projection, viewed as (B, H, L, D), are read where they lie
        # and the output is written in the same order; anything else is copied as in the reference (core.py:85-87)
        in_place = (q.dtype == k.dtype == v.dtype == self.dtype and _lib.row_strided(q, k, v))
        if not in_place:
            q = q.contiguous()
            k = k.contiguous()
            v = v.contiguous()
        headdim = q.size(-1)
        assert headdim in [64, 128], "headdim should be in [64, 128]. For other headdim, you can use padding and specify the softmax scale."
        # The k/v half of the linear branch runs on a side stream beside the preparation and the attention
        # kernel (measured best when started first: 0.570 against 0.593 ms serial at H12 L32760).
        if q.dtype == k.dtype == v.dtype == self.dtype:
            # v, which neither the mask nor the q / k quantisers need, is quantised with the state build on the side
            # stream: the state kernel streams v anyway and finds the column maxima the quantiser starts from
            state = _StateBuild(k, v, self.proj_l.weight, self.feature_map, quant_v_range=V_RANGE_E4M3)
            v8, vs = state.v_fp8, state.v_scale
            # the mask sees the same values as the quantisers: one pass structure for both
            sparse_map, lut, real_topk, q8, qs, k8, ks, _, _ = sage_prepare(q, k, None, self.topk)
            state.join()
        else:
            # the mask is built from the inputs as given, the quantisers work in the compute dtype (core.py:96-100)
            sparse_map, lut, real_topk = get_block_map(q, k, topk_ratio=self.topk, BLKQ=SAGE_BLKQ, BLKK=SAGE_BLKK)
            q = q.to(self.dtype)
            k = k.to(self.dtype)
            v = v.to(self.dtype)
            state = _StateBuild(k, v, self.proj_l.weight, self.feature_map)
            q8, qs, k8, ks = quant_qk(q, k)
            v8, vs = quant_v(v)
        o_s = sage_attn_fwd(q8, qs, k8, ks, v8, vs, lut, real_topk, self.dtype)
        o = linear_out_fwd(q, self.proj_l.bias, o_s, state.join(), self.feature_map).to(dtype)
        if return_sparsity:
            return o, real_topk / sparse_map.shape[-1]
        return o
