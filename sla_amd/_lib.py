"""ctypes binding of the C ABI declared in ``include/sla_hip.h``.

The shared library is the only compute path of this package: if it is missing
the import of any operator raises, there is no eager fallback.
"""
from __future__ import annotations

import ctypes
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libsla_hip.so")

SLA_F32, SLA_BF16, SLA_F16 = 0, 1, 2
FMAP = {"elu": 0, "relu": 1, "softmax": 2}
WS_BLOCK_MAP, WS_SPARSE_BWD, WS_LINEAR_FWD, WS_LINEAR_BWD, WS_SAGE_QUANT, WS_LINEAR_COMPLEMENT, WS_SAGE_PREPARE, WS_LINEAR_STATES = range(8)
BWD_ACCUMULATE, BWD_STATES_READY = 1, 2

ERR_BAD_ARG, ERR_UNSUPPORTED, ERR_LAUNCH, ERR_WORKSPACE = -1, -2, -3, -4

_c = ctypes
_P, _I, _F, _I64 = _c.c_void_p, _c.c_int, _c.c_float, _c.c_int64

# name -> (restype, argtypes); must list every symbol of include/sla_hip.h
SIGNATURES = {
    "sla_version": (_I, []),
    "sla_last_error": (_c.c_char_p, []),
    "sla_workspace_bytes": (_I64, [_I] * 9),
    "sla_mean_pool": (_I, [_P, _P, _I, _I, _I, _I, _I, _P]),
    "sla_block_map_fwd": (_I, [_P, _P, _I, _I, _I, _I, _I, _I, _I, _I, _P, _I64, _P, _P, _I, _P]),
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
    "sla_linear_bwd": (_I, [_P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _P, _I64, _P]),
    "sage_quant_qk": (_I, [_P, _P, _I, _I, _I, _I, _I, _I, _I, _P, _P, _P, _P, _P, _I64, _P]),
    "sage_prepare": (_I, [_P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _I, _P, _P, _I, _P, _P, _P, _P, _P, _P, _P, _I64, _P]),
    "sage_quant_v": (_I, [_P, _I, _I, _I, _I, _I, _P, _P, _P, _I64, _P]),
    "sage_sparse_attn_fwd": (_I, [_P, _P, _P, _P, _P, _P, _P, _I, _P, _I, _I, _I, _I, _I, _I, _I, _I, _F, _P]),
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


def workspace(op: int, dtype: int, B, H, L, D, BLKQ, BLKK, topk, device) -> torch.Tensor:
    n = load().sla_workspace_bytes(op, dtype, B, H, L, D, BLKQ, BLKK, topk)
    if n < 0:
        check(int(n))
    return torch.empty(max(int(n), 256), dtype=torch.uint8, device=device)
