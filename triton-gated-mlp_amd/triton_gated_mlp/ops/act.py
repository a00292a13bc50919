"""Activation forms of the fused path, as plain torch functions.

Names follow src/triton_gated_mlp/ops/act.py (Triton device functions there): `_compute_sigma`
(:28-30), `_silu_fwd` (:33-35), `_silu_bwd` (:42-45) and the dispatchers `_act_fwd` / `_act_bwd`
(:5-22).  The kernels evaluate the same forms in fp32 (csrc/common.hpp).  `_act_bwd` returns the
DERIVATIVE act'(x); for "no_act" that is 1 (the reference returns x there).
"""

from __future__ import annotations

import math

import torch
from torch import Tensor


def _compute_sigma(x: Tensor) -> Tensor:
    return 1 / (1 + torch.exp(-x))


def _silu_fwd(x: Tensor) -> Tensor:
    return x * _compute_sigma(x)


def _silu_bwd(x: Tensor) -> Tensor:
    sigma = _compute_sigma(x)
    return sigma * (1 + x * (1 - sigma))


_FWD = {
    "silu": _silu_fwd,
    "swish": _silu_fwd,
    "gelu": lambda x: 0.5 * x * (1 + torch.erf(x / math.sqrt(2.0))),
    "relu": lambda x: torch.clamp_min(x, 0),
    "leaky_relu": lambda x: torch.where(x > 0, x, 0.01 * x),
    "sigmoid": _compute_sigma,
    "tanh": torch.tanh,
    "no_act": lambda x: x,
}

_BWD = {
    "silu": _silu_bwd,
    "swish": _silu_bwd,
    "gelu": lambda x: 0.5 * (1 + torch.erf(x / math.sqrt(2.0)))
    + x * torch.exp(-0.5 * x * x) / math.sqrt(2.0 * math.pi),
    "relu": lambda x: (x > 0).to(x.dtype),
    "leaky_relu": lambda x: torch.where(x > 0, torch.ones_like(x), torch.full_like(x, 0.01)),
    "sigmoid": lambda x: _compute_sigma(x) * (1 - _compute_sigma(x)),
    "tanh": lambda x: 1 - torch.tanh(x) ** 2,
    "no_act": torch.ones_like,
}


def _act_fwd(x: Tensor, act_name: str) -> Tensor:
    if act_name not in _FWD:
        raise NotImplementedError(act_name)
    return _FWD[act_name](x)


def _act_bwd(x: Tensor, act_name: str) -> Tensor:
    if act_name not in _BWD:
        raise NotImplementedError(act_name)
    return _BWD[act_name](x)
