"""ctypes binding of the C ABI declared in ``include/sla_hip.h``.

The shared library is the only compute path of this package: if it is missing
the import of any operator raises, there is no eager fallback.
"""
from __future__ import annotations

import ctypes
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
# (SLA_HIP_LIB names another build of the same library, e.g. the one with sanitizers in its host code)
LIB_PATH = os.environ.get("SLA_HIP_LIB") or os.path.join(_HERE, "lib", "libsla_hip.so")

SLA_F32, SLA_BF16, SLA_F16 = 0, 1, 2
FMAP = {"elu": 0, "relu": 1, "softmax": 2}
(WS_BLOCK_MAP, WS_SPARSE_BWD, WS_LINEAR_FWD, WS_LINEAR_BWD, WS_SAGE_QUANT, WS_LINEAR_COMPLEMENT, WS_SAGE_PREPARE,
 WS_LINEAR_STATES, WS_LINEAR_COMPLEMENT_BWD) = range(9)
BWD_ACCUMULATE, BWD_STATES_READY = 1, 2

ERR_BAD_ARG, ERR_UNSUPPORTED, ERR_LAUNCH, ERR_WORKSPACE = -1, -2, -3, -4
STATIC_SCRATCH_BYTES = 16 << 20

_c = ctypes
_P, _I, _F, _I64 = _c.c_void_p, _c.c_int, _c.c_float, _c.c_int64

# name -> (restype, argtypes); must list every symbol of include/sla_hip.h
SIGNATURES = {
    "sla_version": (_I, []),
    "sla_last_error": (_c.c_char_p, []),
    "sla_workspace_bytes": (_I64, [_I] * 9),
    "sla_mean_pool": (_I, [_P, _P, _I, _I, _I, _I, _I, _P]),
    "sla_block_map_fwd": (_I, [_P, _P, _I, _I, _I, _I, _I, _I, _I, _I, _P, _I64, _P, _P, _I, _P]),
    "sla_block_map_fwd_static": (_I, [_P, _P, _I, _I, _I, _I, _I, _I, _I, _I, _P, _P, _I, _P]),
    "sla_block_map_fwd_strided": (_I, [_P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _I, _P, _I64, _P, _P, _I, _P]),
    "sla_linear_state_fwd_strided": (_I, [_P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _P, _I64, _P]),
    "sla_linear_state_quant_v_fwd": (_I, [_P, _P, _P, _I, _I, _I, _I, _I, _I, _P, _I64, _P, _P, _F, _P]),
    "sla_linear_state_quant_v_fwd_strided": (_I, [_P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _P, _I64, _P, _P, _F, _P]),
    "sla_sparse_attn_linear_fwd_strided": (_I, [_P, _P, _P, _P, _P, _I, _P, _I64, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I,
                                                _I, _I, _I, _I, _F, _P]),
    "sla_sparse_attn_bwd_strided": (_I, [_P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _I, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I,
                                         _I, _F, _P, _I64, _P]),
    "sla_linear_bwd_strided": (_I, [_P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _P, _I64,
                                    _P]),
    "sla_sparse_attn_fwd": (_I, [_P, _P, _P, _P, _I, _P, _P, _I, _I, _I, _I, _I, _I, _I, _I, _F, _P]),
    "sla_sparse_attn_linear_fwd": (_I, [_P, _P, _P, _P, _I, _P, _I64, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _I, _I,
                                        _F, _P]),
    "sla_sparse_attn_bwd": (_I, [_P, _P, _P, _P, _P, _P, _P, _P, _I, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I,
                                 _I, _F, _P, _I64, _P]),
    "sla_linear_fwd": (_I, [_P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _P, _I64, _P]),
    "sla_linear_state_fwd": (_I, [_P, _P, _P, _I, _I, _I, _I, _I, _I, _P, _I64, _P]),
    "sla_linear_out_fwd": (_I, [_P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _P, _I64, _P]),
    "sla_linear_complement_fwd": (_I, [_P, _P, _P, _P, _I, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _I, _I, _P, _I64,
                                       _P]),
    "sla_linear_complement_bwd": (_I, [_P, _P, _P, _P, _P, _I, _P, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I,
                                       _I, _I, _I, _P, _I64, _P]),
    "sla_linear_bwd": (_I, [_P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _P, _I64, _P]),
    "sla_module_bwd": (_I, [_P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _I, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I,
                            _I, _I, _F, _I, _P, _I64, _P, _I64, _P, _P]),
    "sage_quant_qk": (_I, [_P, _P, _I, _I, _I, _I, _I, _I, _I, _P, _P, _P, _P, _P, _I64, _P]),
    "sage_prepare": (_I, [_P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _I, _P, _P, _I, _P, _P, _P, _P, _P, _P, _F, _P, _I64, _P]),
    "sage_quant_v": (_I, [_P, _I, _I, _I, _I, _I, _P, _P, _F, _P, _I64, _P]),
    "sage_sparse_attn_fwd": (_I, [_P, _P, _P, _P, _P, _P, _P, _I, _P, _I, _I, _I, _I, _I, _I, _I, _I, _F, _P]),
    "sage_prepare_strided": (_I, [_P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _I, _P, _P, _I, _P, _P, _P, _P, _P, _P, _F, _P,
                                  _I64, _P]),
    "sage_quant_v_strided": (_I, [_P, _P, _I, _I, _I, _I, _I, _P, _P, _F, _P, _I64, _P]),
    "sla_linear_out_fwd_strided": (_I, [_P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _P, _I64, _P]),
}

_lib = None


def load() -> ctypes.CDLL:
    """Loads the library once; raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                f"{LIB_PATH} not found: build the HIP kernels first (python -m sla_amd.build). "
                "This package has no fallback path.")
        lib = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype = res
            fn.argtypes = args
        _lib = lib
    return _lib


class SlaError(RuntimeError):
    pass


def last_error() -> str:
    return load().sla_last_error().decode()


def check(rc: int) -> None:
    """Maps a negative status to the exception the reference raises for the same mistake."""
    if rc >= 0:
        return
    msg = last_error()
    if rc == ERR_UNSUPPORTED:
        raise AssertionError(msg)          # reference: assert BLOCK_M in (64,128), BLOCK_N == 64, headdim ...
    if rc == ERR_BAD_ARG:
        raise ValueError(msg)
    raise SlaError(f"status {rc}: {msg}")


def dtype_code(dt: torch.dtype) -> int:
    if dt == torch.float32:
        return SLA_F32
    if dt == torch.bfloat16:
        return SLA_BF16
    if dt == torch.float16:
        return SLA_F16
    raise TypeError(f"unsupported dtype {dt}")


def stream_ptr(device) -> int:
    return torch.cuda.current_stream(device).cuda_stream


def require_gpu(*tensors) -> None:
    for t in tensors:
        if not t.is_cuda:
            raise RuntimeError("sla_amd runs on the GPU only: got a tensor on " + str(t.device))


def _significant_strides(t):
    """Strides of the batch, head and row dimensions; None where the dimension has one entry (its stride is never used)."""
    return tuple(st if n > 1 else None for n, st in zip(t.shape[:3], t.stride()[:3]))


def row_strided(*tensors) -> bool:
    """True when the (B, H, L, D) tensors can be handed to the ``*_strided`` entry points as they are: same
    strides, contiguous last dimension, every row 16-byte aligned, rows not overlapping."""
    t0 = tensors[0]
    if t0.dim() != 4 or t0.stride(-1) != 1:
        return False
    vec = 16 // t0.element_size()
    for t in tensors:
        if (t.shape != t0.shape or t.dtype != t0.dtype or t.stride(-1) != 1 or t.data_ptr() % 16
                or _significant_strides(t) != _significant_strides(t0)):
            return False
    sb, sh, sl = _significant_strides(t0)
    if any(st is not None and (st <= 0 or st % vec) for st in (sb, sh, sl)):
        return False
    return sl is None or sl >= t0.shape[-1]


def strides_arg(t):
    """{batch, head, row} strides of a (B, H, L, D) tensor as the int64[3] the ``*_strided`` entry points take
    (dimensions with one entry get a harmless aligned value)."""
    B, H, L, D = t.shape
    sb, sh, sl = _significant_strides(t)
    sl = D if sl is None else sl
    sh = L * sl if sh is None else sh
    sb = H * L * sl if sb is None else sb
    return (ctypes.c_int64 * 3)(sb, sh, sl)


def empty_like_rows(t):
    """Uninitialised tensor of t's shape and dtype whose dimensions are ordered in memory like t's (so a
    (B, L, H, D) activation viewed as (B, H, L, D) gets an output it can view back for free), densely packed."""
    order = sorted(range(t.dim() - 1), key=lambda i: (-t.stride(i), i)) + [t.dim() - 1]
    shape = [t.shape[i] for i in order]
    out = torch.empty(shape, dtype=t.dtype, device=t.device)
    inv = [order.index(i) for i in range(t.dim())]
    return out.permute(inv)


def workspace(op: int, dtype: int, B, H, L, D, BLKQ, BLKK, topk, device) -> torch.Tensor:
    n = load().sla_workspace_bytes(op, dtype, B, H, L, D, BLKQ, BLKK, topk)
    if n < 0:
        check(int(n))
    return torch.empty(max(int(n), 256), dtype=torch.uint8, device=device)
