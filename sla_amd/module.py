"""``SparseLinearAttention`` with the constructor, parameters and forward of the reference
module (``sparse_linear_attention/core.py:24-105``), running on the HIP kernels."""
from __future__ import annotations

import torch
import torch.nn as nn

from .block_map import get_block_map
from .linear import _linear_proj_add
from .sparse_attn import _attention

FEATURE_MAPS = ("elu", "relu", "softmax")


class SparseLinearAttention(nn.Module):
    def __init__(self, head_dim, topk, feature_map="softmax", BLKQ=64, BLKK=64, use_bf16=True,
                 tie_feature_map_qk=True):
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
        dtype = q.dtype
        q = q.contiguous()
        k = k.contiguous()
        v = v.contiguous()

        # the mask is built from the inputs in their own dtype (reference core.py:83)
        sparse_map, lut, real_topk = get_block_map(q, k, topk_ratio=self.topk, BLKQ=self.BLKQ, BLKK=self.BLKK)

        q = q.to(self.dtype)
        k = k.to(self.dtype)
        v = v.to(self.dtype)
        o_s = _attention.apply(q, k, v, sparse_map, lut, real_topk, self.BLKQ, self.BLKK)
        o = _linear_proj_add.apply(q, k, v, self.proj_l.weight, self.proj_l.bias, o_s, self.feature_map)
        o = o.to(dtype)

        if return_sparsity:
            return o, real_topk / sparse_map.shape[-1]
        return o
