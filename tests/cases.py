"""Seeded inputs of the five benchmark configurations, generated on the CPU so that the HIP path and the
oracle see bit-identical tensors."""

from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, Optional

import torch


@dataclass(frozen=True)
class Case:
    name: str
    M: int
    K: int
    N: int
    dtype: torch.dtype
    bias: bool = False
    p: float = 0.0
    backward: bool = False
    seed: int = 0
    dropout_seed: int = 1234
    act: str = "silu"


CFG2 = Case("cfg2_llama7b_fwd", 4096, 4096, 11008, torch.float16)
CFG3 = Case("cfg3_llama3_8b_fwdbwd", 8192, 4096, 14336, torch.float16, backward=True)
CFG4 = Case("cfg4_bf16_bias_dropout", 2048, 2048, 5632, torch.bfloat16, bias=True, p=0.1, backward=True)
CFG5 = Case("cfg5_decode", 16, 8192, 28672, torch.float16)


def make_inputs(c: Case) -> Dict[str, Optional[torch.Tensor]]:
    """x ~ N(0,1); weights ~ N(0, 0.02); biases ~ U(-0.01, 0.01); dY ~ N(0,1); rounded to c.dtype."""
    g = torch.Generator().manual_seed(c.seed)
    t = {
        "x": torch.randn(c.M, c.K, generator=g),
        "W_gate": 0.02 * torch.randn(c.N, c.K, generator=g),
        "W_up": 0.02 * torch.randn(c.N, c.K, generator=g),
        "W_down": 0.02 * torch.randn(c.K, c.N, generator=g),
        "b_gate": None,
        "b_up": None,
        "b_down": None,
        "dY": None,
    }
    if c.bias:
        t["b_gate"] = (torch.rand(c.N, generator=g) - 0.5) * 0.02
        t["b_up"] = (torch.rand(c.N, generator=g) - 0.5) * 0.02
        t["b_down"] = (torch.rand(c.K, generator=g) - 0.5) * 0.02
    if c.backward:
        t["dY"] = torch.randn(c.M, c.K, generator=g)
    return {k: (None if v is None else v.to(c.dtype)) for k, v in t.items()}
