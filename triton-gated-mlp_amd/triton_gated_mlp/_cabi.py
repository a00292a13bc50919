"""ctypes binding of libgmlp.so (C ABI declared in include/gmlp.h).

The library is the only implementation of the fused operators: if it cannot be found or loaded the
import of the operators raises, there is no CPU or PyTorch fallback.
"""

from __future__ import annotations

import ctypes
import os
from pathlib import Path
from typing import Optional

import torch
from torch import Tensor

GMLP_F16, GMLP_BF16, GMLP_F32 = 0, 1, 2
GMLP_OP_DECODE_FWD, GMLP_OP_COLSUM, GMLP_OP_LINEAR_FWD, GMLP_OP_DX_BWD, GMLP_OP_GATEUP_FWD = 0, 1, 2, 3, 4
GMLP_OP_DH_BWD, GMLP_OP_DW_BWD, GMLP_OP_DW_BWD_GROUPED = 5, 6, 7
ABI_VERSION = 8
GMLP_PASS_FWD, GMLP_PASS_BWD = 0, 1

# hidden_act name -> GMLP_ACT_* code.  The names are those of the reference's ACT2CLS / ACT_FWD
# tables (src/triton_gated_mlp/gated_mlp.py:17-37).
ACT_CODES = {
    "silu": 0,
    "swish": 0,
    "gelu": 1,
    "relu": 2,
    "leaky_relu": 3,
    "sigmoid": 4,
    "tanh": 5,
    "no_act": 6,
}

_STATUS_EXC = {-1: ValueError, -2: NotImplementedError, -3: ValueError, -4: RuntimeError}

_c_ptr = ctypes.c_void_p
_i64 = ctypes.c_int64
_u64 = ctypes.c_uint64
_int = ctypes.c_int
_f32 = ctypes.c_float

_SIGNATURES = {
    "gmlp_abi_version": (_int, []),
    "gmlp_last_error": (ctypes.c_char_p, []),
    "gmlp_init": (_int, []),
    "gmlp_workspace_bytes": (ctypes.c_size_t, [_int, _i64, _i64, _i64, _int]),
    "gmlp_gateup_fwd": (
        _int,
        [_c_ptr] * 9 + [_i64, _i64, _i64, _int, _int, _f32, _u64, _u64, _c_ptr, ctypes.c_size_t, _c_ptr],
    ),
    "gmlp_linear_fwd": (_int, [_c_ptr] * 4 + [_i64, _i64, _i64, _int, _c_ptr, ctypes.c_size_t, _c_ptr]),
    "gmlp_dh_bwd": (
        _int,
        [_c_ptr] * 6 + [_i64, _i64, _i64, _int, _int, _f32, _u64, _u64, _c_ptr, ctypes.c_size_t, _c_ptr],
    ),
    "gmlp_gating_bwd": (_int, [_c_ptr] * 5 + [_i64, _i64, _int, _int, _f32, _u64, _u64, _c_ptr]),
    "gmlp_dx_bwd": (_int, [_c_ptr] * 5 + [_i64, _i64, _i64, _int, _c_ptr, ctypes.c_size_t, _c_ptr]),
    "gmlp_dw_bwd": (_int, [_c_ptr] * 3 + [_i64, _i64, _i64, _int, _c_ptr, ctypes.c_size_t, _c_ptr]),
    "gmlp_dw_bwd_grouped_workspace_bytes": (ctypes.c_size_t, [_int, _i64, _c_ptr, _c_ptr, _int]),
    "gmlp_dw_bwd_grouped": (
        _int,
        [_int, _c_ptr, _c_ptr, _c_ptr, _i64, _c_ptr, _c_ptr, _int, _c_ptr, ctypes.c_size_t, _c_ptr],
    ),
    "gmlp_colsum": (_int, [_c_ptr] * 3 + [_i64, _i64, _int, _c_ptr]),
    "gmlp_colsum_static": (_int, [_c_ptr] * 2 + [_i64, _i64, _int, _c_ptr]),
    "gmlp_colsum_grouped": (_int, [_int, _c_ptr, _c_ptr, _c_ptr, _i64, _c_ptr, _int, _c_ptr]),
    "gmlp_decode_fwd": (_int, [_c_ptr] * 10 + [_i64, _i64, _i64, _int, _int, _c_ptr]),
    "gmlp_dropout_mask": (_int, [_c_ptr, _i64, _i64, _f32, _u64, _u64, _c_ptr]),
    "gmlp_mlp_workspace_bytes": (ctypes.c_size_t, [_int, _i64, _i64, _i64, _int]),
    "gmlp_mlp_fwd": (
        _int,
        [_c_ptr] * 11 + [_i64, _i64, _i64, _int, _int, _f32, _u64, _u64, _c_ptr, ctypes.c_size_t, _c_ptr],
    ),
    "gmlp_mlp_bwd": (
        _int,
        [_c_ptr] * 17 + [_i64, _i64, _i64, _int, _int, _f32, _u64, _u64, _c_ptr, ctypes.c_size_t, _c_ptr],
    ),
}

EXPORTED_SYMBOLS = tuple(_SIGNATURES)


def library_path() -> Path:
    env = os.environ.get("GMLP_LIB")
    if env:
        return Path(env)
    return Path(__file__).resolve().parent.parent / "lib" / "libgmlp.so"


_lib: Optional[ctypes.CDLL] = None


def lib() -> ctypes.CDLL:
    """Load libgmlp.so once; raise if it is missing (there is no other implementation)."""
    global _lib
    if _lib is None:
        path = library_path()
        if not path.exists():
            raise RuntimeError(
                f"libgmlp.so not found at {path}: build it with `make -C {path.parent.parent}` "
                "(or set GMLP_LIB); the fused gated-MLP operators have no fallback path"
            )
        handle = ctypes.CDLL(str(path))
        for name, (restype, argtypes) in _SIGNATURES.items():
            fn = getattr(handle, name)
            fn.restype = restype
            fn.argtypes = argtypes
        got = handle.gmlp_abi_version()
        if got != ABI_VERSION:
            raise RuntimeError(f"libgmlp.so ABI version {got}, expected {ABI_VERSION}")
        _lib = handle
    return _lib


def check(status: int) -> None:
    if status != 0:
        msg = lib().gmlp_last_error().decode("utf-8", "replace")
        raise _STATUS_EXC.get(status, RuntimeError)(msg)


def dtype_code(dtype: torch.dtype) -> int:
    if dtype == torch.float16:
        return GMLP_F16
    if dtype == torch.bfloat16:
        return GMLP_BF16
    if dtype == torch.float32:
        return GMLP_F32
    raise TypeError(f"fused gated-MLP kernels take float16, bfloat16 or float32 tensors, got {dtype}")


def act_code(act_fn: str) -> int:
    try:
        return ACT_CODES[act_fn]
    except KeyError:
        raise NotImplementedError(
            f"hidden_act {act_fn!r} is not one of {sorted(ACT_CODES)}"
        ) from None


def require_gpu(*tensors: Optional[Tensor]) -> torch.device:
    """All given tensors must live on one HIP device and share a dtype; returns the device."""
    dev = None
    dt = None
    for t in tensors:
        if t is None:
            continue
        if not t.is_cuda:
            raise RuntimeError(
                "fused gated-MLP operators run on an AMD GPU only (tensor is on "
                f"{t.device}); use EagerGatedMLP for CPU execution"
            )
        if dev is None:
            dev, dt = t.device, t.dtype
        elif t.device != dev:
            raise RuntimeError(f"tensors on different devices: {dev} and {t.device}")
        elif t.dtype != dt:
            raise TypeError(f"tensors of different dtypes: {dt} and {t.dtype}")
    assert dev is not None
    return dev


def workspace(op: int, M: int, K: int, N: int, code: int, device: torch.device) -> Optional[Tensor]:
    """Scratch buffer of the size the library asks for (None if it needs none)."""
    nbytes = lib().gmlp_workspace_bytes(op, M, K, N, code)
    return torch.empty((nbytes,), dtype=torch.uint8, device=device) if nbytes else None


def ptr(t: Optional[Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


def stream_ptr(device: torch.device) -> int:
    return torch.cuda.current_stream(device).cuda_stream


_MLP_WS = {}


def mlp_workspace_bytes(which: int, M: int, K: int, N: int, code: int, device: torch.device) -> int:
    """gmlp_mlp_workspace_bytes, remembered per problem and device (the plan depends on the device's
    compute-unit count; call with `device` current)."""
    key = (which, M, K, N, code, device.index)
    n = _MLP_WS.get(key)
    if n is None:
        n = _MLP_WS[key] = lib().gmlp_mlp_workspace_bytes(which, M, K, N, code)
    return n

