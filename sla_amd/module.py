"""``SparseLinearAttention`` with the constructor, parameters and forward of the reference
module (``sparse_linear_attention/core.py:24-105``), running on the HIP kernels."""
from __future__ import annotations

import torch
import torch.nn as nn

from . import _lib
from .block_map import get_block_map
from .linear import linear_complement_bwd, linear_complement_fwd, linear_state_fwd, linear_state_quant_v_fwd, saved_states
from .sparse_attn import sparse_attn_bwd, sparse_attn_fwd, sparse_attn_linear_fwd

FEATURE_MAPS = ("elu", "relu", "softmax")


def module_bwd(q, k, v, o_s, d_out, lse, sparse_map, lut, topk, BLKQ, BLKK, qk_scale, weight, bias, fmap, states=None,
               grads=None, side_stream=None):
    """Backward of the whole operator in one library call (``sla_module_bwd``): the kernels of
    :func:`sparse_attn_bwd` and of :func:`linear_bwd` accumulating into the same gradients, bit for bit, with the
    short kernels on ``side_stream`` beside the long ones when one is given.  Returns ``(dq, dk, dv, d_weight, d_bias)``.

    q, k, v (and ``grads=(dq, dk, dv)`` when given) may be row-contiguous views sharing their strides, ``d_out`` a
    row-contiguous view of its own; ``o_s`` and ``lse`` are contiguous.  ``states`` as in :func:`linear_bwd`."""
    _lib.require_gpu(q, k, v, o_s, d_out, lse, sparse_map, lut, weight, bias)
    B, H, L, D = q.shape
    dev = q.device
    dt = _lib.dtype_code(q.dtype)
    dq, dk, dv = (torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)) if grads is None else grads
    assert o_s.is_contiguous() and lse.is_contiguous() and sparse_map.is_contiguous() and lut.is_contiguous()
    ws_s = _lib.workspace(_lib.WS_SPARSE_BWD, dt, B, H, L, D, BLKQ, BLKK, topk, dev)
    ws_l = _lib.workspace(_lib.WS_LINEAR_BWD, dt, B, H, L, D, 64, 64, 0, dev)
    flags = 0
    if states is not None:
        ws_l[:states.numel()].copy_(states)
        flags |= _lib.BWD_STATES_READY
    dw = torch.empty((D, D), dtype=torch.float32, device=dev)
    db = torch.empty((D,), dtype=torch.float32, device=dev)
    if all(t.is_contiguous() for t in (q, k, v, d_out, dq, dk, dv)):
        s_qkv = s_do = None
    else:
        assert _lib.row_strided(q, k, v, dq, dk, dv) and _lib.row_strided(d_out), "tensors must be row-contiguous views"
        s_qkv, s_do = _lib.strides_arg(q), _lib.strides_arg(d_out)
    side = 0 if side_stream is None else side_stream.cuda_stream
    rc = _lib.load().sla_module_bwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), s_qkv, o_s.data_ptr(), d_out.data_ptr(), s_do,
                                    lse.data_ptr(), sparse_map.data_ptr(), lut.data_ptr(), lut.element_size(),
                                    weight.data_ptr(), bias.data_ptr(), dq.data_ptr(), dk.data_ptr(), dv.data_ptr(),
                                    dw.data_ptr(), db.data_ptr(), dt, _lib.FMAP[fmap], B, H, L, D, BLKQ, BLKK, topk,
                                    float(qk_scale), flags, ws_s.data_ptr(), ws_s.numel(), ws_l.data_ptr(), ws_l.numel(),
                                    _lib.stream_ptr(dev), side)
    _lib.check(rc)
    return dq, dk, dv, dw, db


def _backward_side_stream(dev):
    """The stream the short kernels of the backward go to: the one the forward's state build uses (default priority,
    one per device); none while a graph is being captured (the work then stays on the capturing stream)."""
    if torch.cuda.is_current_stream_capturing():
        return None
    side = _StateBuild._side.get(dev.index)
    if side is None:
        side = _StateBuild._side[dev.index] = torch.cuda.Stream(device=dev)
    return side


class _sla_core(torch.autograd.Function):
    """Sparse branch + linear branch + projection + sum as one differentiable operator.

    Same function as ``_attention`` followed by ``_linear_proj_add`` (reference core.py:88-100); fusing
    them lets the backward add the linear-branch gradients into the sparse-branch ones in place.
    """

    @staticmethod
    def forward(ctx, q, k, v, weight, bias, sparse_map, lut, topk, BLKQ, BLKK, fmap, state, needs_grad=True):
        # (row-contiguous views are accepted on the inference path only: the backward kernels take (B, H, L, D))
        assert (q.is_contiguous() and k.is_contiguous() and v.is_contiguous()) or not needs_grad
        assert sparse_map.is_contiguous() and lut.is_contiguous()
        assert BLKQ == 64 or BLKQ == 128
        assert BLKK == 64
        qk_scale = q.shape[-1] ** -0.5
        bias = bias.contiguous()
        # one kernel: attention over the selected blocks, then the linear branch of the same rows from the
        # per-head state, projection and sum in its epilogue; o_s is only written when a backward will need it
        state_ws = state.join()
        out, o_s, lse = sparse_attn_linear_fwd(q, k, v, lut, topk, BLKQ, BLKK, qk_scale, state_ws, bias, fmap,
                                               want_o_s=needs_grad)
        if not needs_grad:
            return out
        # the finished states (a few D x D matrices per head) are kept for the backward, the partial sums are not
        ctx.save_for_backward(q, k, v, weight, bias, sparse_map, lut, lse, o_s, saved_states(state_ws, q))
        ctx.cfg = (topk, BLKQ, BLKK, fmap, qk_scale)
        return out

    @staticmethod
    def backward(ctx, d_out):
        q, k, v, weight, bias, sparse_map, lut, lse, o_s, states = ctx.saved_tensors
        topk, BLKQ, BLKK, fmap, qk_scale = ctx.cfg
        d_out = d_out.contiguous()
        dq, dk, dv, dw, db = module_bwd(q, k, v, o_s, d_out, lse, sparse_map, lut, topk, BLKQ, BLKK, qk_scale, weight, bias,
                                        fmap, states=states, side_stream=_backward_side_stream(q.device))
        return dq, dk, dv, dw, db, None, None, None, None, None, None, None, None


class _sla_complement(torch.autograd.Function):
    """Sparse branch + complement-mode linear branch (over the key blocks a query block did not select) + projection
    + sum.  The reference has no such variant; the definition is ``linear_complement_fwd``'s."""

    @staticmethod
    def forward(ctx, q, k, v, weight, bias, sparse_map, lut, topk, BLKQ, BLKK, fmap):
        assert q.is_contiguous() and k.is_contiguous() and v.is_contiguous()
        assert sparse_map.is_contiguous() and lut.is_contiguous()
        assert BLKQ in (64, 128) and BLKK == 64
        qk_scale = q.shape[-1] ** -0.5
        weight, bias = weight.contiguous(), bias.contiguous()
        o_s, lse = sparse_attn_fwd(q, k, v, lut, topk, BLKQ, BLKK, qk_scale)
        out = linear_complement_fwd(q, k, v, lut, topk, weight, bias, o_s, fmap, BLKQ, BLKK)
        if any(ctx.needs_input_grad[:5]):
            ctx.save_for_backward(q, k, v, weight, bias, sparse_map, lut, lse, o_s)
            ctx.cfg = (topk, BLKQ, BLKK, fmap, qk_scale)
        return out

    @staticmethod
    def backward(ctx, d_out):
        q, k, v, weight, bias, sparse_map, lut, lse, o_s = ctx.saved_tensors
        topk, BLKQ, BLKK, fmap, qk_scale = ctx.cfg
        d_out = d_out.contiguous()
        dq, dk, dv = sparse_attn_bwd(q, k, v, o_s, d_out, lse, sparse_map, lut, topk, BLKQ, BLKK, qk_scale)
        _, _, _, dw, db = linear_complement_bwd(q, k, v, sparse_map, lut, topk, weight, bias, d_out, fmap, BLKQ, BLKK,
                                                accumulate_into=(dq, dk, dv))
        return dq, dk, dv, dw, db, None, None, None, None, None, None


class _sla_packed(torch.autograd.Function):
    """The same operator on a packed ``(B, L, 3, H, D)`` projection output, returning ``(B, L, H, D)``.

    A transformer block produces q, k, v as one packed tensor in token-major order and consumes the attention
    output in token-major order.  Fed to ``_sla_core`` through views, autograd would rebuild the packed gradient
    with three zero-fill-and-copy passes; here the kernels read q, k, v where they lie (row stride ``3*H*D``) and
    the backward kernels write dq, dk, dv straight into one packed gradient tensor, so neither direction copies.
    """

    @staticmethod
    def forward(ctx, qkv, weight, bias, topk_ratio, BLKQ, BLKK, fmap):
        assert qkv.dim() == 5 and qkv.shape[2] == 3 and qkv.is_contiguous()
        q, k, v = (qkv[:, :, i].permute(0, 2, 1, 3) for i in range(3))          # (B, H, L, D) views
        weight = weight.contiguous()
        bias = bias.contiguous()
        state_ws = _StateBuild(k, v, weight, fmap)
        sparse_map, lut, topk = get_block_map(q, k, topk_ratio=topk_ratio, BLKQ=BLKQ, BLKK=BLKK)
        needs_grad = any(ctx.needs_input_grad[:3])
        qk_scale = q.shape[-1] ** -0.5
        out, o_s, lse = sparse_attn_linear_fwd(q, k, v, lut, topk, BLKQ, BLKK, qk_scale, state_ws.join(), bias, fmap,
                                               want_o_s=needs_grad)
        if needs_grad:
            ctx.save_for_backward(qkv, weight, bias, sparse_map, lut, lse, o_s, saved_states(state_ws.ws, q))
            ctx.cfg = (topk, BLKQ, BLKK, fmap, qk_scale)
        ctx.density = topk / sparse_map.shape[-1]
        return out.permute(0, 2, 1, 3)                                            # (B, L, H, D), contiguous

    @staticmethod
    def backward(ctx, d_out):
        qkv, weight, bias, sparse_map, lut, lse, o_s, states = ctx.saved_tensors
        topk, BLKQ, BLKK, fmap, qk_scale = ctx.cfg
        q, k, v = (qkv[:, :, i].permute(0, 2, 1, 3) for i in range(3))
        d_out = d_out.permute(0, 2, 1, 3)                                         # (B, H, L, D) view
        if not _lib.row_strided(d_out):
            d_out = d_out.contiguous()
        d_qkv = torch.empty_like(qkv)
        grads = tuple(d_qkv[:, :, i].permute(0, 2, 1, 3) for i in range(3))
        _, _, _, dw, db = module_bwd(q, k, v, o_s, d_out, lse, sparse_map, lut, topk, BLKQ, BLKK, qk_scale, weight, bias,
                                     fmap, states=states, grads=grads, side_stream=_backward_side_stream(qkv.device))
        return d_qkv, dw, db, None, None, None, None


class _StateBuild:
    """The k/v-only half of the linear branch, started on a side stream so that it runs beside the mask
    builder (both are short memory-bound kernels; neither fills the device on its own).  ``join`` makes
    the calling stream wait for it and hands over the workspace it filled."""

    _side = {}

    def __init__(self, k, v, weight, fmap, quant_v_range=None):
        """``quant_v_range``: also quantise ``v`` to FP8 with that range in the same library call (``self.v_fp8``,
        ``self.v_scale``, ready after ``join``)."""
        dev = k.device
        self.v_fp8 = self.v_scale = None

        def build():
            if quant_v_range is None:
                self.ws = linear_state_fwd(k, v, weight, fmap)
            else:
                self.ws, self.v_fp8, self.v_scale = linear_state_quant_v_fwd(k, v, weight, fmap, quant_v_range)

        cur = torch.cuda.current_stream(dev)
        if torch.cuda.is_current_stream_capturing():
            side = None          # inside a graph capture the work stays on the capturing stream
        else:
            side = self._side.get(dev.index)
            if side is None:
                side = self._side[dev.index] = torch.cuda.Stream(device=dev)
        self.side = side
        if side is None:
            build()
            return
        side.wait_stream(cur)    # k, v and the weight were produced on the calling stream
        with torch.cuda.stream(side):
            build()
        for t in (self.v_fp8, self.v_scale):
            if t is not None:
                t.record_stream(cur)         # allocated under the side stream, consumed on the calling one

    def also(self, fn, *args):
        """Runs ``fn(*args)`` behind the state build, on the same side stream; its results are ready after ``join``."""
        if self.side is None:
            return fn(*args)
        with torch.cuda.stream(self.side):
            res = fn(*args)
        for t in (res if isinstance(res, tuple) else (res,)):
            t.record_stream(torch.cuda.current_stream(t.device))
        return res

    def join(self):
        if self.side is not None:
            torch.cuda.current_stream(self.ws.device).wait_stream(self.side)
            # the workspace was allocated under the side stream; it is consumed on the calling one
            self.ws.record_stream(torch.cuda.current_stream(self.ws.device))
        return self.ws


class SparseLinearAttention(nn.Module):
    def __init__(self, head_dim, topk, feature_map="softmax", BLKQ=64, BLKK=64, use_bf16=True,
                 tie_feature_map_qk=True, linear_mode="global"):
        r"""
        Args:
            head_dim: dimension of each head.
            topk: ratio of keys selected for sparse attention, shared across all queries.
            feature_map: feature map for linear attention, one of ['elu', 'relu', 'softmax'].
            BLKQ: block size for query.
            BLKK: block size for key.
            use_bf16: bfloat16 (default) or float16 compute; inputs are converted inside the module.
            tie_feature_map_qk: kept for signature compatibility; q and k always use the same map
                (as in the reference, core.py:43-60).
            linear_mode: "global" (default, what the reference computes: the linear branch sees every key)
                or "complement" (extension: it sees only the key blocks the query block did not select).
        """
        super().__init__()
        self.dtype = torch.bfloat16 if use_bf16 else torch.float16
        self.topk = topk
        self.BLKQ = BLKQ
        self.BLKK = BLKK
        self.proj_l = nn.Linear(head_dim, head_dim, dtype=torch.float32)
        if feature_map not in FEATURE_MAPS:
            raise NotImplementedError(f"Not supported feature map {feature_map}.")
        self.feature_map = feature_map
        self.tie_feature_map_qk = tie_feature_map_qk
        if linear_mode not in ("global", "complement"):
            raise NotImplementedError(f"Not supported linear mode {linear_mode}.")
        self.linear_mode = linear_mode
        self.init_weights_()

    def init_weights_(self):
        with torch.no_grad():
            nn.init.zeros_(self.proj_l.weight)
            nn.init.zeros_(self.proj_l.bias)

    def forward(self, q, k, v, return_sparsity=False):
        r"""
        Args:
            q, k, v: (B, H, L, D).
            return_sparsity: also return real_topk / n_key_blocks (reference core.py:102-103).
        """
        _lib.require_gpu(q, k, v)          # no CPU path: refuse loudly before anything touches a stream
        dtype = q.dtype
        needs_grad = torch.is_grad_enabled() and any(
            t.requires_grad for t in (q, k, v, self.proj_l.weight, self.proj_l.bias))
        # Inference on activations that are not laid out as (B, H, L, D) -- a (B, L, H, D) tensor or the slices
        # of a packed QKV projection, viewed as (B, H, L, D) -- reads them where they are and writes the output
        # in the same dimension order, instead of copying three tensors in and one out (the reference makes
        # the copies: core.py:77-79).  Training and the other cases take the contiguous route.
        in_place = (not needs_grad and self.linear_mode == "global" and dtype == self.dtype
                    and not (q.is_contiguous() and k.is_contiguous() and v.is_contiguous())
                    and _lib.row_strided(q, k, v))
        if not in_place:
            q = q.contiguous()
            k = k.contiguous()
            v = v.contiguous()

        qc = q.to(self.dtype)
        kc = k.to(self.dtype)
        vc = v.to(self.dtype)
        if self.linear_mode == "complement":
            return self._forward_complement(q, k, qc, kc, vc, dtype, return_sparsity)
        weight = self.proj_l.weight.contiguous()
        with torch.no_grad():
            state = _StateBuild(kc, vc, weight, self.feature_map)

        # the mask is built from the inputs in their own dtype (reference core.py:83)
        sparse_map, lut, real_topk = get_block_map(q, k, topk_ratio=self.topk, BLKQ=self.BLKQ, BLKK=self.BLKK)

        o = _sla_core.apply(qc, kc, vc, weight, self.proj_l.bias, sparse_map, lut, real_topk, self.BLKQ,
                            self.BLKK, self.feature_map, state, needs_grad)
        o = o.to(dtype)

        if return_sparsity:
            return o, real_topk / sparse_map.shape[-1]
        return o

    def forward_packed(self, qkv, return_sparsity=False):
        r"""
        The forward on a packed projection output, without layout copies in either direction (extension; the
        reference takes separate ``(B, H, L, D)`` tensors).

        Args:
            qkv: (B, L, 3, H, D), as ``nn.Linear(dim, 3 * dim)(x).view(B, L, 3, H, D)`` gives it.
        Returns:
            (B, L, H, D), ready for ``reshape(B, L, H * D)``.
        """
        if qkv.dtype != self.dtype or self.linear_mode != "global" or not _lib.row_strided(qkv[:, :, 0].permute(0, 2, 1, 3)):
            q, k, v = (qkv[:, :, i].permute(0, 2, 1, 3) for i in range(3))
            res = self.forward(q, k, v, return_sparsity)
            o = res[0] if return_sparsity else res
            o = o.permute(0, 2, 1, 3)
            return (o, res[1]) if return_sparsity else o
        o = _sla_packed.apply(qkv.contiguous(), self.proj_l.weight, self.proj_l.bias, self.topk, self.BLKQ, self.BLKK,
                              self.feature_map)
        if return_sparsity:
            N = (qkv.shape[1] + self.BLKK - 1) // self.BLKK
            return o, min(N, int(self.topk * N)) / N
        return o

    def _forward_complement(self, q, k, qc, kc, vc, dtype, return_sparsity):
        sparse_map, lut, real_topk = get_block_map(q, k, topk_ratio=self.topk, BLKQ=self.BLKQ, BLKK=self.BLKK)
        o = _sla_complement.apply(qc, kc, vc, self.proj_l.weight, self.proj_l.bias, sparse_map, lut, real_topk, self.BLKQ,
                                  self.BLKK, self.feature_map).to(dtype)
        if return_sparsity:
            return o, real_topk / sparse_map.shape[-1]
        return o
