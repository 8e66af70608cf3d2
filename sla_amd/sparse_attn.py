"""Host side of the block-sparse attention operator.

Mirrors ``_attention`` of ``sparse_linear_attention/kernel.py:240-320``: an
``autograd.Function`` with the same argument list, the same saved tensors and
the same assertions.
"""
from __future__ import annotations

import torch

from . import _lib


def _lut_bytes(lut: torch.Tensor) -> int:
    if lut.dtype == torch.int64:
        return 8
    if lut.dtype == torch.int32:
        return 4
    raise TypeError(f"lut must be int32 or int64, got {lut.dtype}")


def sparse_attn_fwd(q, k, v, lut, topk, BLOCK_M, BLOCK_N, qk_scale):
    """Launches the forward kernel; returns ``(o_s, lse)`` with lse in base-2 units."""
    _lib.require_gpu(q, k, v, lut)
    B, H, L, D = q.shape
    o = torch.empty_like(v)
    lse = torch.empty(q.shape[:-1], device=q.device, dtype=torch.float32)
    rc = _lib.load().sla_sparse_attn_fwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), lut.data_ptr(), _lut_bytes(lut),
                                         o.data_ptr(), lse.data_ptr(), _lib.dtype_code(q.dtype), B, H, L, D,
                                         BLOCK_M, BLOCK_N, topk, float(qk_scale), _lib.stream_ptr(q.device))
    _lib.check(rc)
    return o, lse


def sparse_attn_linear_fwd(q, k, v, lut, topk, BLOCK_M, BLOCK_N, qk_scale, state_ws, bias, fmap: str, want_o_s: bool):
    """Attention forward with the linear branch, projection and sum fused into its epilogue.

    ``state_ws`` is the workspace :func:`sla_amd.linear.linear_state_fwd` filled.  Returns ``(out, o_s, lse)``;
    ``o_s`` (the attention output alone, needed by the backward) is ``None`` unless ``want_o_s``.

    q, k, v may be row-contiguous views that share their strides (a ``(B, L, H, D)`` activation seen as
    ``(B, H, L, D)``, slices of a packed projection): ``out`` then has its dimensions ordered in memory like q."""
    _lib.require_gpu(q, k, v, lut, state_ws, bias)
    B, H, L, D = q.shape
    lse = torch.empty(q.shape[:-1], device=q.device, dtype=torch.float32)
    o_s = torch.empty(q.shape, dtype=q.dtype, device=q.device) if want_o_s else None
    if q.is_contiguous() and k.is_contiguous() and v.is_contiguous():
        out = torch.empty_like(v)
        rc = _lib.load().sla_sparse_attn_linear_fwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), lut.data_ptr(),
                                                    _lut_bytes(lut), state_ws.data_ptr(), state_ws.numel(), bias.data_ptr(),
                                                    0 if o_s is None else o_s.data_ptr(), out.data_ptr(), lse.data_ptr(),
                                                    _lib.dtype_code(q.dtype), _lib.FMAP[fmap], B, H, L, D, BLOCK_M,
                                                    BLOCK_N, topk, float(qk_scale), _lib.stream_ptr(q.device))
    else:
        assert _lib.row_strided(q, k, v), "q, k, v must be contiguous or share row-contiguous strides"
        out = _lib.empty_like_rows(q)
        rc = _lib.load().sla_sparse_attn_linear_fwd_strided(
            q.data_ptr(), k.data_ptr(), v.data_ptr(), _lib.strides_arg(q), lut.data_ptr(), _lut_bytes(lut),
            state_ws.data_ptr(), state_ws.numel(), bias.data_ptr(), 0 if o_s is None else o_s.data_ptr(), out.data_ptr(),
            _lib.strides_arg(out), lse.data_ptr(), _lib.dtype_code(q.dtype), _lib.FMAP[fmap], B, H, L, D, BLOCK_M, BLOCK_N,
            topk, float(qk_scale), _lib.stream_ptr(q.device))
    _lib.check(rc)
    return out, o_s, lse


def sparse_attn_bwd(q, k, v, o, do, lse, k_block_id, lut, topk, BLOCK_M, BLOCK_N, qk_scale, grads=None):
    """Launches delta + dQ + dK/dV; returns ``(dq, dk, dv)``.

    ``grads=(dq, dk, dv)``: write into these tensors instead of new ones.  q, k, v (and the gradient tensors)
    may be row-contiguous views sharing their strides, ``do`` a row-contiguous view of its own; ``o`` (the saved
    attention output) and ``lse`` are contiguous."""
    B, H, L, D = q.shape
    dq, dk, dv = (torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)) if grads is None else grads
    dt = _lib.dtype_code(q.dtype)
    ws = _lib.workspace(_lib.WS_SPARSE_BWD, dt, B, H, L, D, BLOCK_M, BLOCK_N, topk, q.device)
    assert o.is_contiguous() and lse.is_contiguous()
    if all(t.is_contiguous() for t in (q, k, v, do, dq, dk, dv)):
        rc = _lib.load().sla_sparse_attn_bwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), do.data_ptr(),
                                             lse.data_ptr(), k_block_id.data_ptr(), lut.data_ptr(), _lut_bytes(lut),
                                             dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), dt, B, H, L, D, BLOCK_M,
                                             BLOCK_N, topk, float(qk_scale), ws.data_ptr(), ws.numel(),
                                             _lib.stream_ptr(q.device))
    else:
        assert _lib.row_strided(q, k, v, dq, dk, dv) and _lib.row_strided(do), "tensors must be row-contiguous views"
        rc = _lib.load().sla_sparse_attn_bwd_strided(
            q.data_ptr(), k.data_ptr(), v.data_ptr(), _lib.strides_arg(q), o.data_ptr(), do.data_ptr(),
            _lib.strides_arg(do), lse.data_ptr(), k_block_id.data_ptr(), lut.data_ptr(), _lut_bytes(lut), dq.data_ptr(),
            dk.data_ptr(), dv.data_ptr(), dt, B, H, L, D, BLOCK_M, BLOCK_N, topk, float(qk_scale), ws.data_ptr(),
            ws.numel(), _lib.stream_ptr(q.device))
    _lib.check(rc)
    return dq, dk, dv


class _attention(torch.autograd.Function):
    """Block-sparse FlashAttention over the selected key blocks (reference kernel.py:240-320)."""

    @staticmethod
    def forward(ctx, q, k, v, k_block_id, lut, topk, BLOCK_M, BLOCK_N, qk_scale=None):
        assert q.is_contiguous() and k.is_contiguous() and v.is_contiguous()
        assert k_block_id.is_contiguous() and lut.is_contiguous()
        assert BLOCK_M == 64 or BLOCK_M == 128
        assert BLOCK_N == 64
        B, H, L, D = q.shape
        if qk_scale is None:
            qk_scale = D ** -0.5
        o_s, lse = sparse_attn_fwd(q, k, v, lut, topk, BLOCK_M, BLOCK_N, qk_scale)
        ctx.save_for_backward(q, k, v, k_block_id, lut, lse, o_s)
        ctx.qk_scale = qk_scale
        ctx.topk = topk
        ctx.BLOCK_M = BLOCK_M
        ctx.BLOCK_N = BLOCK_N
        return o_s

    @staticmethod
    def backward(ctx, do_s):
        q, k, v, k_block_id, lut, lse, o_s = ctx.saved_tensors
        do_s = do_s.contiguous()
        dq, dk, dv = sparse_attn_bwd(q, k, v, o_s, do_s, lse, k_block_id, lut, ctx.topk, ctx.BLOCK_M, ctx.BLOCK_N,
                                     ctx.qk_scale)
        return dq, dk, dv, None, None, None, None, None, None
