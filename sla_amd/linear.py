"""Host side of the linear-attention branch + projection + sum.

Replaces the eager block of ``sparse_linear_attention/core.py:90-100`` (feature
maps, ``calc_linear``, ``proj_l`` under autocast, ``o_s + o_l``) with one fused
operator: ``out = residual + proj_l(calc_linear(phi(q), phi(k), v))``.
"""
from __future__ import annotations

import torch

from . import _lib


def linear_fwd(q, k, v, weight, bias, residual, fmap: str):
    _lib.require_gpu(q, k, v, weight, bias)
    B, H, L, D = q.shape
    dt = _lib.dtype_code(q.dtype)
    ws = _lib.workspace(_lib.WS_LINEAR_FWD, dt, B, H, L, D, 64, 64, 0, q.device)
    out = torch.empty_like(q)
    rc = _lib.load().sla_linear_fwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), weight.data_ptr(), bias.data_ptr(),
                                    0 if residual is None else residual.data_ptr(), out.data_ptr(), dt,
                                    _lib.FMAP[fmap], B, H, L, D, ws.data_ptr(), ws.numel(), _lib.stream_ptr(q.device))
    _lib.check(rc)
    return out


def linear_state_fwd(k, v, weight, fmap: str):
    """First half of :func:`linear_fwd`: builds the per-head states from ``k`` and ``v`` on the current
    stream and returns the workspace that :func:`linear_out_fwd` consumes."""
    _lib.require_gpu(k, v, weight)
    B, H, L, D = k.shape
    dt = _lib.dtype_code(k.dtype)
    ws = _lib.workspace(_lib.WS_LINEAR_FWD, dt, B, H, L, D, 64, 64, 0, k.device)
    if k.is_contiguous() and v.is_contiguous():
        rc = _lib.load().sla_linear_state_fwd(k.data_ptr(), v.data_ptr(), weight.data_ptr(), dt, _lib.FMAP[fmap], B, H, L,
                                              D, ws.data_ptr(), ws.numel(), _lib.stream_ptr(k.device))
    else:
        assert _lib.row_strided(k, v), "k and v must be contiguous or share row-contiguous strides"
        rc = _lib.load().sla_linear_state_fwd_strided(k.data_ptr(), v.data_ptr(), _lib.strides_arg(k), weight.data_ptr(), dt,
                                                      _lib.FMAP[fmap], B, H, L, D, ws.data_ptr(), ws.numel(),
                                                      _lib.stream_ptr(k.device))
    _lib.check(rc)
    return ws


def linear_state_quant_v_fwd(k, v, weight, fmap: str, v_range: float = 448.0):
    """:func:`linear_state_fwd` and the per-channel FP8 quantisation of ``v`` (``sage.quant_v``) in one library call:
    the state kernel streams ``v`` anyway and leaves the column maxima the quantiser needs, which spares the
    quantiser's own pass over ``v`` for them.  Returns ``(workspace, v_fp8, v_scale)``, bit for bit what the two
    calls return."""
    _lib.require_gpu(k, v, weight)
    B, H, L, D = k.shape
    dt = _lib.dtype_code(k.dtype)
    ws = _lib.workspace(_lib.WS_LINEAR_FWD, dt, B, H, L, D, 64, 64, 0, k.device)
    v8 = torch.empty((B, H, L, D), dtype=torch.float8_e4m3fn, device=v.device)
    vs = torch.empty((B, H, D), dtype=torch.float32, device=v.device)
    if k.is_contiguous() and v.is_contiguous():
        rc = _lib.load().sla_linear_state_quant_v_fwd(k.data_ptr(), v.data_ptr(), weight.data_ptr(), dt, _lib.FMAP[fmap], B,
                                                      H, L, D, ws.data_ptr(), ws.numel(), v8.data_ptr(), vs.data_ptr(),
                                                      float(v_range), _lib.stream_ptr(k.device))
    else:
        assert _lib.row_strided(k, v), "k and v must be contiguous or share row-contiguous strides"
        rc = _lib.load().sla_linear_state_quant_v_fwd_strided(k.data_ptr(), v.data_ptr(), _lib.strides_arg(k),
                                                              weight.data_ptr(), dt, _lib.FMAP[fmap], B, H, L, D,
                                                              ws.data_ptr(), ws.numel(), v8.data_ptr(), vs.data_ptr(),
                                                              float(v_range), _lib.stream_ptr(k.device))
    _lib.check(rc)
    return ws, v8, vs


def linear_out_fwd(q, bias, residual, state_ws, fmap: str):
    """Second half of :func:`linear_fwd`: ``residual + proj(phi(q) state / divisor)``.

    ``q`` may be a row-contiguous view (see ``_lib.row_strided``); the output then has q's memory order.
    ``residual`` is always a contiguous (B, H, L, D) tensor."""
    _lib.require_gpu(q, bias, state_ws)
    B, H, L, D = q.shape
    dt = _lib.dtype_code(q.dtype)
    res_ptr = 0 if residual is None else residual.data_ptr()
    assert residual is None or residual.is_contiguous()
    if q.is_contiguous():
        out = torch.empty_like(q)
        rc = _lib.load().sla_linear_out_fwd(q.data_ptr(), bias.data_ptr(), res_ptr, out.data_ptr(), dt, _lib.FMAP[fmap], B, H,
                                            L, D, state_ws.data_ptr(), state_ws.numel(), _lib.stream_ptr(q.device))
    else:
        assert _lib.row_strided(q), "q must be contiguous or a row-contiguous view"
        out = _lib.empty_like_rows(q)
        rc = _lib.load().sla_linear_out_fwd_strided(q.data_ptr(), _lib.strides_arg(q), bias.data_ptr(), res_ptr, out.data_ptr(),
                                                    _lib.strides_arg(out), dt, _lib.FMAP[fmap], B, H, L, D,
                                                    state_ws.data_ptr(), state_ws.numel(), _lib.stream_ptr(q.device))
    _lib.check(rc)
    return out


def linear_complement_fwd(q, k, v, lut, topk, weight, bias, residual, fmap: str, BLKQ: int = 64, BLKK: int = 64):
    """Linear branch over the key blocks each query block did NOT select, + projection + ``residual``.

    Opt-in variant (the paper's formulation); the reference module computes the global branch
    (``core.py:92-96``).  :func:`linear_complement_bwd` is its backward."""
    _lib.require_gpu(q, k, v, lut, weight, bias)
    B, H, L, D = q.shape
    dt = _lib.dtype_code(q.dtype)
    if lut.dtype not in (torch.int32, torch.int64):
        raise TypeError(f"lut must be int32 or int64, got {lut.dtype}")
    ws = _lib.workspace(_lib.WS_LINEAR_COMPLEMENT, dt, B, H, L, D, BLKQ, BLKK, topk, q.device)
    out = torch.empty_like(q)
    rc = _lib.load().sla_linear_complement_fwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), lut.data_ptr(),
                                               lut.element_size(), weight.data_ptr(), bias.data_ptr(),
                                               0 if residual is None else residual.data_ptr(), out.data_ptr(), dt,
                                               _lib.FMAP[fmap], B, H, L, D, BLKQ, BLKK, topk, ws.data_ptr(),
                                               ws.numel(), _lib.stream_ptr(q.device))
    _lib.check(rc)
    return out


def linear_complement_bwd(q, k, v, sparse_map, lut, topk, weight, bias, d_out, fmap: str, BLKQ: int = 64, BLKK: int = 64,
                          accumulate_into=None):
    """Gradients of :func:`linear_complement_fwd` (the linear branch only; the residual's gradient is ``d_out``).

    ``sparse_map`` and ``lut`` are the pair ``get_block_map`` returned.  ``accumulate_into=(dq, dk, dv)`` adds to
    existing gradient tensors instead of allocating new ones.  Returns ``(dq, dk, dv, d_weight, d_bias)``."""
    _lib.require_gpu(q, k, v, sparse_map, lut, weight, bias, d_out)
    B, H, L, D = q.shape
    dt = _lib.dtype_code(q.dtype)
    if lut.dtype not in (torch.int32, torch.int64):
        raise TypeError(f"lut must be int32 or int64, got {lut.dtype}")
    assert sparse_map.dtype == torch.int8 and sparse_map.is_contiguous() and lut.is_contiguous()
    assert q.is_contiguous() and k.is_contiguous() and v.is_contiguous() and d_out.is_contiguous()
    ws = _lib.workspace(_lib.WS_LINEAR_COMPLEMENT_BWD, dt, B, H, L, D, BLKQ, BLKK, topk, q.device)
    if accumulate_into is None:
        dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
        flags = 0
    else:
        dq, dk, dv = accumulate_into
        flags = _lib.BWD_ACCUMULATE
    dw = torch.empty((D, D), dtype=torch.float32, device=q.device)
    db = torch.empty((D,), dtype=torch.float32, device=q.device)
    rc = _lib.load().sla_linear_complement_bwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), sparse_map.data_ptr(),
                                               lut.data_ptr(), lut.element_size(), weight.data_ptr(), bias.data_ptr(),
                                               d_out.data_ptr(), dq.data_ptr(), dk.data_ptr(), dv.data_ptr(),
                                               dw.data_ptr(), db.data_ptr(), dt, _lib.FMAP[fmap], B, H, L, D, BLKQ, BLKK,
                                               topk, flags, ws.data_ptr(), ws.numel(), _lib.stream_ptr(q.device))
    _lib.check(rc)
    return dq, dk, dv, dw, db


def saved_states(state_ws, q):
    """Copy of the finished per-head states at the head of a :func:`linear_state_fwd` workspace (about
    ``3 B H D^2`` 16-bit values): what :func:`linear_bwd` needs of the forward, without the partial sums."""
    B, H, L, D = q.shape
    n = _lib.load().sla_workspace_bytes(_lib.WS_LINEAR_STATES, _lib.dtype_code(q.dtype), B, H, L, D, 64, 64, 0)
    if n < 0:
        _lib.check(int(n))
    return state_ws[:int(n)].clone()


def linear_bwd(q, k, v, weight, bias, d_out, fmap: str, accumulate_into=None, states=None):
    """Gradients of the linear branch.  ``accumulate_into=(dq, dk, dv)`` adds them to existing
    gradient tensors (those of the sparse branch) instead of allocating new ones.  ``states``
    (from :func:`saved_states`, same k, v, weight) spares the backward rebuilding the forward's states."""
    B, H, L, D = q.shape
    dt = _lib.dtype_code(q.dtype)
    ws = _lib.workspace(_lib.WS_LINEAR_BWD, dt, B, H, L, D, 64, 64, 0, q.device)
    flags = 0 if accumulate_into is None else _lib.BWD_ACCUMULATE
    if states is not None:
        ws[:states.numel()].copy_(states)
        flags |= _lib.BWD_STATES_READY
    if accumulate_into is None:
        dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    else:
        dq, dk, dv = accumulate_into
    dw = torch.empty((D, D), dtype=torch.float32, device=q.device)
    db = torch.empty((D,), dtype=torch.float32, device=q.device)
    if all(t.is_contiguous() for t in (q, k, v, d_out, dq, dk, dv)):
        rc = _lib.load().sla_linear_bwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), weight.data_ptr(), bias.data_ptr(),
                                        d_out.data_ptr(), dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), dw.data_ptr(),
                                        db.data_ptr(), dt, _lib.FMAP[fmap], B, H, L, D, flags, ws.data_ptr(), ws.numel(),
                                        _lib.stream_ptr(q.device))
    else:
        # row-contiguous views: q, k, v and the gradient tensors share their strides, d_out has its own
        assert _lib.row_strided(q, k, v, dq, dk, dv) and _lib.row_strided(d_out), "tensors must be row-contiguous views"
        rc = _lib.load().sla_linear_bwd_strided(q.data_ptr(), k.data_ptr(), v.data_ptr(), _lib.strides_arg(q),
                                                weight.data_ptr(), bias.data_ptr(), d_out.data_ptr(),
                                                _lib.strides_arg(d_out), dq.data_ptr(), dk.data_ptr(), dv.data_ptr(),
                                                dw.data_ptr(), db.data_ptr(), dt, _lib.FMAP[fmap], B, H, L, D, flags,
                                                ws.data_ptr(), ws.numel(), _lib.stream_ptr(q.device))
    _lib.check(rc)
    return dq, dk, dv, dw, db


class _linear_proj_add(torch.autograd.Function):
    """out = residual + proj(calc_linear(phi(q), phi(k), v)); weight/bias are the fp32 ``proj_l`` parameters."""

    @staticmethod
    def forward(ctx, q, k, v, weight, bias, residual, fmap):
        weight = weight.contiguous()
        bias = bias.contiguous()
        out = linear_fwd(q, k, v, weight, bias, residual, fmap)
        ctx.save_for_backward(q, k, v, weight, bias)
        ctx.fmap = fmap
        ctx.has_residual = residual is not None
        return out

    @staticmethod
    def backward(ctx, d_out):
        q, k, v, weight, bias = ctx.saved_tensors
        d_out = d_out.contiguous()
        dq, dk, dv, dw, db = linear_bwd(q, k, v, weight, bias, d_out, ctx.fmap)
        return dq, dk, dv, dw, db, (d_out if ctx.has_residual else None), None
