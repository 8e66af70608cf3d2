"""Host side of the block-mask builder.

Mirrors ``sparse_linear_attention/utils.py:43-67`` of the reference: same
function names, arguments and return values; the device work is one call into
the HIP library.
"""
from __future__ import annotations

import torch

from . import _lib


def topk_count(n_blocks: int, topk_ratio: float) -> int:
    """``min(K, int(topk_ratio * K))`` — reference utils.py:61-62."""
    return min(n_blocks, int(topk_ratio * n_blocks))


def mean_pool(x: torch.Tensor, BLK: int) -> torch.Tensor:
    """Per-block mean over the sequence axis — reference utils.py:43-52."""
    assert x.is_contiguous()
    _lib.require_gpu(x)
    B, H, L, D = x.shape
    nblk = (L + BLK - 1) // BLK
    out = torch.empty((B, H, nblk, D), device=x.device, dtype=x.dtype)
    rc = _lib.load().sla_mean_pool(x.data_ptr(), out.data_ptr(), _lib.dtype_code(x.dtype), B * H, L, D, BLK,
                                   _lib.stream_ptr(x.device))
    _lib.check(rc)
    return out


def get_block_map(q: torch.Tensor, k: torch.Tensor, topk_ratio: float, BLKQ: int = 64, BLKK: int = 64):
    """Returns ``(sparse_map int8 (B,H,M,N), lut int64 (B,H,M,T), T)`` — reference utils.py:55-67.

    The look-up table lists, per query block, the selected key blocks in
    ascending order (the reference leaves the order unspecified); equal scores
    are resolved towards the lowest block index.
    """
    assert q.shape == k.shape and q.dtype == k.dtype
    strided = not (q.is_contiguous() and k.is_contiguous())
    assert not strided or _lib.row_strided(q, k), "q and k must be contiguous or share row-contiguous strides"
    _lib.require_gpu(q, k)
    B, H, L, D = q.shape
    M = (L + BLKQ - 1) // BLKQ
    N = (L + BLKK - 1) // BLKK
    T = topk_count(N, topk_ratio)
    dt = _lib.dtype_code(q.dtype)
    ws = _lib.workspace(_lib.WS_BLOCK_MAP, dt, B, H, L, D, BLKQ, BLKK, T, q.device)
    sparse_map = torch.empty((B, H, M, N), dtype=torch.int8, device=q.device)
    lut = torch.empty((B, H, M, T), dtype=torch.int64, device=q.device)
    if strided:
        rc = _lib.load().sla_block_map_fwd_strided(q.data_ptr(), k.data_ptr(), _lib.strides_arg(q), dt, B, H, L, D, BLKQ,
                                                   BLKK, T, ws.data_ptr(), ws.numel(), sparse_map.data_ptr(),
                                                   lut.data_ptr(), 8, _lib.stream_ptr(q.device))
    else:
        rc = _lib.load().sla_block_map_fwd(q.data_ptr(), k.data_ptr(), dt, B, H, L, D, BLKQ, BLKK, T, ws.data_ptr(),
                                           ws.numel(), sparse_map.data_ptr(), lut.data_ptr(), 8,
                                           _lib.stream_ptr(q.device))
    _lib.check(rc)
    return sparse_map, lut, T
