"""Seeded synthetic inputs for the five benchmark / parity configurations.

Everything is generated on the CPU from a ``torch.Generator`` so that the
oracle and the HIP path see identical values; callers move the tensors to the
device.  Nothing upstream defines the "structured" q/k: the generator below is
this repository's definition (a smooth low-frequency field over the 3-D latent
grid shared by q and k, plus iid noise), chosen so pooled block scores are
non-uniform and neighbouring query blocks prefer similar key blocks.
"""
from __future__ import annotations

import math
from dataclasses import dataclass

import torch


@dataclass(frozen=True)
class Config:
    name: str
    B: int
    H: int
    L: int
    D: int
    BLKQ: int
    BLKK: int
    topk: float
    feature_map: str
    dtype: torch.dtype
    grid: tuple | None = None       # (F, Y, X) latent grid for structured q/k
    k_bias_std: float = 0.0         # per-channel bias on k (exercises smoothing)
    backward: bool = False
    sage: bool = False


CONFIGS = {
    "cfg1": Config("cfg1", 1, 2, 1024, 64, 64, 64, 0.2, "softmax", torch.float32),
    "cfg2": Config("cfg2", 2, 4, 4096, 128, 64, 64, 0.2, "softmax", torch.bfloat16, backward=True),
    "cfg3": Config("cfg3", 1, 12, 32760, 128, 64, 64, 0.05, "elu", torch.bfloat16, grid=(21, 30, 52)),
    "cfg4": Config("cfg4", 1, 40, 75600, 128, 64, 64, 0.05, "relu", torch.bfloat16, grid=(21, 45, 80),
                   backward=True),
    "cfg5": Config("cfg5", 1, 40, 32760, 128, 128, 64, 0.1, "softmax", torch.bfloat16, grid=(21, 30, 52),
                   k_bias_std=2.0, sage=True),
}

_FREQS = ((1, 0, 0), (0, 1, 0), (0, 0, 1), (1, 1, 0), (0, 1, 1), (2, 0, 1))


def structured_field(gen: torch.Generator, H: int, grid, D: int) -> torch.Tensor:
    """(H, L, D) fp32: sum of six low-frequency sinusoids over the (F,Y,X) grid.

    field[h,t,d] = sum_a A * sin(2*pi*(af*f/F + ay*y/Y + ax*x/X) + phase[a,h,d]),
    t = (f*Y + y)*X + x, A = 1/sqrt(len(freqs)/2) so the field has unit variance.
    """
    Fg, Y, X = grid
    f = torch.arange(Fg, dtype=torch.float32).view(Fg, 1, 1) / Fg
    y = torch.arange(Y, dtype=torch.float32).view(1, Y, 1) / Y
    x = torch.arange(X, dtype=torch.float32).view(1, 1, X) / X
    L = Fg * Y * X
    amp = 1.0 / math.sqrt(len(_FREQS) / 2.0)
    field = torch.zeros(H, L, D, dtype=torch.float32)
    for (af, ay, ax) in _FREQS:
        arg = (2 * math.pi) * (af * f + ay * y + ax * x)          # (F,Y,X)
        phase = torch.rand(H, 1, D, generator=gen) * (2 * math.pi)
        field += amp * torch.sin(arg.reshape(1, L, 1) + phase)
    return field


def make_inputs(cfg: Config, seed: int = 0, H: int | None = None, with_do: bool | None = None):
    """Returns dict(q,k,v[,do]) of CPU tensors in cfg.dtype, shape (B,H,L,D).

    ``H`` overrides the head count (used for bounded CPU baselines); heads are
    generated in order so the first heads are identical to the full set.
    """
    gen = torch.Generator().manual_seed(seed)
    B, Hn, L, D = cfg.B, (cfg.H if H is None else H), cfg.L, cfg.D
    shape = (B, Hn, L, D)
    if cfg.grid is None:
        q = torch.randn(shape, generator=gen)
        k = torch.randn(shape, generator=gen)
        v = torch.randn(shape, generator=gen)
    else:
        assert cfg.grid[0] * cfg.grid[1] * cfg.grid[2] == L
        q = torch.empty(shape)
        k = torch.empty(shape)
        for b in range(B):
            for h in range(Hn):
                fld = structured_field(gen, 1, cfg.grid, D)[0]
                q[b, h] = 0.5 * torch.randn(L, D, generator=gen) + fld
                k[b, h] = 0.5 * torch.randn(L, D, generator=gen) + fld
                if cfg.k_bias_std > 0:
                    k[b, h] += cfg.k_bias_std * torch.randn(1, D, generator=gen)
        v = torch.randn(shape, generator=gen)
    out = {"q": q.to(cfg.dtype), "k": k.to(cfg.dtype), "v": v.to(cfg.dtype)}
    if cfg.backward if with_do is None else with_do:
        out["do"] = torch.randn(shape, generator=gen).to(cfg.dtype)
    return out


def make_inputs_on_device(cfg: Config, device, seed: int = 0, with_do: bool = False):
    """The structured generator of :func:`make_inputs` run on the GPU (same field definition, the device's own random
    streams, so not the same values): for the large configurations, where the CPU generator needs minutes.
    Returns ``(q, k, v, do)`` on ``device``; ``do`` is None unless ``with_do``."""
    assert cfg.grid is not None
    g = torch.Generator(device=device).manual_seed(seed)
    Fg, Y, X = cfg.grid
    f = torch.arange(Fg, device=device, dtype=torch.float32).view(Fg, 1, 1) / Fg
    y = torch.arange(Y, device=device, dtype=torch.float32).view(1, Y, 1) / Y
    x = torch.arange(X, device=device, dtype=torch.float32).view(1, 1, X) / X
    amp = 1.0 / math.sqrt(len(_FREQS) / 2.0)
    shape = (cfg.B, cfg.H, cfg.L, cfg.D)
    q = torch.empty(shape, device=device, dtype=cfg.dtype)
    k = torch.empty(shape, device=device, dtype=cfg.dtype)
    for b in range(cfg.B):
        for h in range(cfg.H):
            fld = torch.zeros(cfg.L, cfg.D, device=device)
            for af, ay, ax in _FREQS:
                arg = (2 * math.pi) * (af * f + ay * y + ax * x).reshape(cfg.L, 1)
                fld += amp * torch.sin(arg + torch.rand(1, cfg.D, device=device, generator=g) * (2 * math.pi))
            q[b, h] = 0.5 * torch.randn(cfg.L, cfg.D, device=device, generator=g) + fld
            k[b, h] = 0.5 * torch.randn(cfg.L, cfg.D, device=device, generator=g) + fld
            if cfg.k_bias_std > 0:
                k[b, h] += cfg.k_bias_std * torch.randn(1, cfg.D, device=device, generator=g)
    v = torch.randn(shape, device=device, generator=g).to(cfg.dtype)
    do = torch.randn(shape, device=device, generator=g).to(cfg.dtype) if with_do else None
    return q, k, v, do


def make_proj(D: int, seed: int = 1):
    """Seeded non-zero proj_l parameters (weight (D,D), bias (D,)) in fp32.

    The module initialises proj_l to zero; tests of the linear branch load
    these so the branch contributes to the output.
    """
    gen = torch.Generator().manual_seed(seed)
    w = torch.randn(D, D, generator=gen) / math.sqrt(D)
    b = 0.1 * torch.randn(D, generator=gen)
    return w, b


def integer_inputs(B, H, L, D, seed=0, dtype=torch.bfloat16, lo=-3, hi=3):
    """q,k with small integer values: every fp32 sum on the mask path is exact,
    so block index sets do not depend on summation order (ties included)."""
    gen = torch.Generator().manual_seed(seed)
    q = torch.randint(lo, hi + 1, (B, H, L, D), generator=gen).to(dtype)
    k = torch.randint(lo, hi + 1, (B, H, L, D), generator=gen).to(dtype)
    return q, k
