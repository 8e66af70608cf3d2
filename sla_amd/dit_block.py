"""A DiT-style self-attention block around ``SparseLinearAttention``: the caller either side of the path.

The reference README (``README.md:2``, usage at ``README.md:30-50``) motivates SLA as a replacement of the
attention call inside a video-diffusion transformer block that is then fine-tuned; its benchmark moves between
the ``(B, L, H, D)`` layout of such blocks and the operator's ``(B, H, L, D)`` (``evaluate/bench_kernel.py:68-71``).
This module is that caller: QKV projection -> head split -> SLA -> head merge -> output projection.  The two
projections are plain library GEMMs.  The head split and merge cost nothing, in training as at inference: the
packed ``(B, L, 3, H, D)`` projection goes to ``SparseLinearAttention.forward_packed``, whose kernels read the
q, k, v rows where they lie, write the output in ``(B, L, H, D)`` order, which the output projection takes as
it is, and whose backward kernels write dq, dk, dv straight into one packed gradient tensor.
"""
from __future__ import annotations

import torch.nn as nn

from .module import SparseLinearAttention
from .sage import SageSparseLinearAttention


class SLASelfAttention(nn.Module):
    def __init__(self, dim, num_heads, topk, feature_map="softmax", BLKQ=64, BLKK=64, use_bf16=True, qkv_bias=True,
                 linear_mode="global", quantized=False):
        """``quantized=True`` puts ``SageSparseLinearAttention`` (INT8 / FP8, inference only, 128/64 blocks) in the place
        of ``SparseLinearAttention``; the parameter names are the same, so a block fine-tuned with the 16-bit operator
        loads into a quantised one (the pairing the reference's README describes: train with SLA, serve with SageSLA)."""
        super().__init__()
        if dim % num_heads != 0:
            raise ValueError(f"dim {dim} is not a multiple of num_heads {num_heads}")
        self.num_heads = num_heads
        self.head_dim = dim // num_heads
        self.qkv = nn.Linear(dim, 3 * dim, bias=qkv_bias)
        self.quantized = quantized
        if quantized:
            if linear_mode != "global":
                raise NotImplementedError("the quantised operator has the global linear branch only")
            self.attn = SageSparseLinearAttention(self.head_dim, topk, feature_map, use_bf16=use_bf16)
        else:
            self.attn = SparseLinearAttention(self.head_dim, topk, feature_map, BLKQ, BLKK, use_bf16=use_bf16,
                                              linear_mode=linear_mode)
        self.proj = nn.Linear(dim, dim)

    def forward(self, x):
        """x: (B, L, dim) -> (B, L, dim)."""
        B, L, C = x.shape
        H, D = self.num_heads, self.head_dim
        qkv = self.qkv(x).view(B, L, 3, H, D)
        if self.quantized:
            # (B, H, L, D) views of the packed projection: the quantisers read them where they lie and the output
            # comes back in (B, L, H, D) memory order
            q, k, v = (qkv[:, :, i].permute(0, 2, 1, 3) for i in range(3))
            o = self.attn(q, k, v).permute(0, 2, 1, 3)
        else:
            o = self.attn.forward_packed(qkv)                               # (B, L, H, D)
        return self.proj(o.reshape(B, L, C))
