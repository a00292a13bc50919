"""CPU oracle (test infrastructure, not product code) of the gated MLP, in plain torch.

Restates the reference's eager module and closed forms (paths relative to the reference repo):
  forward    EagerGatedMLP.forward          src/triton_gated_mlp/gated_mlp.py:92-98
             eager_fwd                      src/triton_gated_mlp/gated_mlp.py:105-128
  backward   eager_bwd (hidden-state part)  src/triton_gated_mlp/gated_mlp.py:131-156
             _silu_op_bwd                   src/triton_gated_mlp/gated_mlp.py:40-43
             _silu_bwd / _compute_sigma     src/triton_gated_mlp/ops/act.py:28-45
  activations ACT2CLS / ACT_FWD table       src/triton_gated_mlp/gated_mlp.py:17-37
Dropout is expressed with an explicit keep mask D (nn.Dropout, gated_mlp.py:90,96, scales kept
values by 1/(1-p)):  H = act(G) * U * D / (1-p), act = silu unless stated.

Pinned by tests/test_oracle.py: brute-force loops on tiny shapes, an independent NumPy fp64
restatement, the C restatement in oracle/gated_mlp_ref.c, torch.autograd and gradcheck for the
backward, known values of silu and silu', and algebraic special cases; the other activations and
their closed-form derivatives (ACTS) against torch.nn.functional under torch.autograd, tabulated
values and central differences.  The reference holds no
stored vectors for this path (its tests compare fused against eager live), so nothing here is
pinned against reference fixtures; no function depends on one.
"""

from __future__ import annotations

import math
from typing import Dict, Optional

import torch
from torch import Tensor


def silu(x: Tensor) -> Tensor:
    return x * torch.sigmoid(x)


def silu_grad(x: Tensor) -> Tensor:
    s = torch.sigmoid(x)
    return s * (1 + x * (1 - s))


def _gelu(x: Tensor) -> Tensor:
    return 0.5 * x * (1 + torch.erf(x / math.sqrt(2.0)))


def _gelu_grad(x: Tensor) -> Tensor:
    return 0.5 * (1 + torch.erf(x / math.sqrt(2.0))) + x * torch.exp(-0.5 * x * x) / math.sqrt(2.0 * math.pi)


def _sigmoid_grad(x: Tensor) -> Tensor:
    s = torch.sigmoid(x)
    return s * (1 - s)


# name -> (act, act'): torch's defaults (erf GELU, LeakyReLU slope 0.01); at the kinks the
# derivative is torch.autograd's (relu'(0) = 0, leaky_relu'(0) = 0.01).
ACTS = {
    "silu": (silu, silu_grad),
    "swish": (silu, silu_grad),
    "gelu": (_gelu, _gelu_grad),
    "relu": (lambda x: torch.where(x > 0, x, torch.zeros_like(x)), lambda x: (x > 0).to(x.dtype)),
    "leaky_relu": (
        lambda x: torch.where(x > 0, x, 0.01 * x),
        lambda x: torch.where(x > 0, torch.ones_like(x), torch.full_like(x, 0.01)),
    ),
    "sigmoid": (torch.sigmoid, _sigmoid_grad),
    "tanh": (torch.tanh, lambda x: 1 - torch.tanh(x) ** 2),
    "no_act": (lambda x: x, torch.ones_like),
}


def hidden_forward(
    x: Tensor,
    W_gate: Tensor,
    b_gate: Optional[Tensor],
    W_up: Tensor,
    b_up: Optional[Tensor],
    keep: Optional[Tensor] = None,
    p: float = 0.0,
    act: str = "silu",
) -> Dict[str, Tensor]:
    G = x @ W_gate.T
    if b_gate is not None:
        G = G + b_gate
    U = x @ W_up.T
    if b_up is not None:
        U = U + b_up
    H = ACTS[act][0](G) * U
    if keep is not None and p > 0.0:
        H = H * keep.to(H.dtype) / (1.0 - p)
    return {"G": G, "U": U, "H": H}


def forward(
    x: Tensor,
    W_gate: Tensor,
    b_gate: Optional[Tensor],
    W_up: Tensor,
    b_up: Optional[Tensor],
    W_down: Tensor,
    b_down: Optional[Tensor],
    keep: Optional[Tensor] = None,
    p: float = 0.0,
    act: str = "silu",
) -> Dict[str, Tensor]:
    """Y = (act(xW_gᵀ+b_g) ⊙ (xW_uᵀ+b_u) ⊙ D/(1-p)) W_dᵀ + b_d for 2-D x; returns Y and G, U, H."""
    out = hidden_forward(x, W_gate, b_gate, W_up, b_up, keep, p, act)
    Y = out["H"] @ W_down.T
    if b_down is not None:
        Y = Y + b_down
    out["Y"] = Y
    return out


def hidden_backward(
    dH: Tensor, G: Tensor, U: Tensor, keep: Optional[Tensor] = None, p: float = 0.0, act: str = "silu"
) -> Dict[str, Tensor]:
    dA = dH
    if keep is not None and p > 0.0:
        dA = dH * keep.to(dH.dtype) / (1.0 - p)
    f, df = ACTS[act]
    return {"dU": dA * f(G), "dG": dA * U * df(G)}


def backward(
    x: Tensor,
    W_gate: Tensor,
    b_gate: Optional[Tensor],
    W_up: Tensor,
    b_up: Optional[Tensor],
    W_down: Tensor,
    b_down: Optional[Tensor],
    dY: Tensor,
    keep: Optional[Tensor] = None,
    p: float = 0.0,
    act: str = "silu",
) -> Dict[str, Tensor]:
    """Closed-form gradients of `forward` for upstream gradient dY (all 2-D)."""
    f = forward(x, W_gate, b_gate, W_up, b_up, W_down, b_down, keep, p, act)
    dH = dY @ W_down
    hb = hidden_backward(dH, f["G"], f["U"], keep, p, act)
    dG, dU = hb["dG"], hb["dU"]
    out = {
        "dX": dU @ W_up + dG @ W_gate,
        "dW_gate": dG.T @ x,
        "dW_up": dU.T @ x,
        "dW_down": dY.T @ f["H"],
        "dG": dG,
        "dU": dU,
        "dH": dH,
    }
    if b_gate is not None:
        out["db_gate"] = dG.sum(0)
    if b_up is not None:
        out["db_up"] = dU.sum(0)
    if b_down is not None:
        out["db_down"] = dY.sum(0)
    out.update(f)
    return out


class OracleGatedMLP(torch.nn.Module):
    """Module form (same parameter names and registration order gate, up, down as
    EagerGatedMLP.__init__, src/triton_gated_mlp/gated_mlp.py:74-90) with an explicit keep mask."""

    def __init__(self, hidden_size=256, intermediate_size=512, bias=True, dropout_p=0.0):
        super().__init__()
        self.hidden_size, self.intermediate_size, self.p = hidden_size, intermediate_size, dropout_p
        self.gate_proj = torch.nn.Linear(hidden_size, intermediate_size, bias=bias)
        self.up_proj = torch.nn.Linear(hidden_size, intermediate_size, bias=bias)
        self.down_proj = torch.nn.Linear(intermediate_size, hidden_size, bias=bias)

    def forward(self, x: Tensor, keep: Optional[Tensor] = None) -> Tensor:
        lead = x.shape[:-1]
        x2 = x.reshape(-1, x.shape[-1])
        h = torch.nn.functional.silu(self.gate_proj(x2)) * self.up_proj(x2)
        if keep is not None and self.p > 0.0 and self.training:
            h = h * keep.to(h.dtype) / (1.0 - self.p)
        return self.down_proj(h).reshape(*lead, self.hidden_size)
