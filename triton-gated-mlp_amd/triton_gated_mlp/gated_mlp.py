"""Gated-MLP modules with the public surface of matteobonotto/triton-gated-mlp.

  FusedGatedMLP(hidden_size, intermediate_size, bias, hidden_act, dropout_p)   nn.Module, HIP kernels
  EagerGatedMLP(...)                                                           same math in plain torch
  FusedGatedMLPFunction.apply(x, W_up, b_up, W_gp, b_gp)                       hidden-state autograd op
  mlp_hidden_states_fwd / mlp_hidden_states_bwd, eager_fwd / eager_bwd, ACT_FWD

Reference: src/triton_gated_mlp/gated_mlp.py (EagerGatedMLP :73-98, eager_fwd/bwd :105-156,
FusedGatedMLPFunction :159-200, FusedGatedMLP :203-237).  Differences, all towards the eager
semantics: the fused path applies the gate/up/down biases and dropout (the reference drops them),
returns bias gradients, keeps G and U from the forward pass instead of recomputing them, runs the
down projection and its backward in the same kernels family (one autograd node for the MLP), and
implements every hidden_act of ACT_FWD (the reference's fused kernels know silu and no_act only).
"""

from __future__ import annotations

from typing import Optional

import torch
from torch import Tensor, nn
from torch.autograd.function import Function

from .ops import bwd as _bwd
from .ops import fwd as _fwd
from .ops.bwd import mlp_hidden_states_bwd
from .ops.fwd import mlp_hidden_states_fwd

class _FreshModule(dict):
    """Mapping name -> module class whose lookup hands out a NEW module instance (a value may be a
    (class, kwargs) pair): the behaviour of the reference's ACT2FN table
    (src/triton_gated_mlp/gated_mlp.py:10-26)."""

    def __getitem__(self, key):
        entry = super().__getitem__(key)
        cls, kwargs = entry if isinstance(entry, tuple) else (entry, {})
        return cls(**kwargs)


ACT2CLS = {name: type(mod) for name, mod in (
    ("gelu", nn.GELU()), ("leaky_relu", nn.LeakyReLU()), ("relu", nn.ReLU()), ("sigmoid", nn.Sigmoid()),
    ("silu", nn.SiLU()), ("swish", nn.SiLU()), ("tanh", nn.Tanh()))}
ACT2FN = _FreshModule(ACT2CLS)
ClassInstantier = _FreshModule  # the reference's name for it

ACT_FWD = {
    "gelu": nn.GELU(),
    "leaky_relu": nn.LeakyReLU(),
    "relu": nn.ReLU(),
    "sigmoid": nn.Sigmoid(),
    "silu": nn.SiLU(),
    "swish": nn.SiLU(),
    "tanh": nn.Tanh(),
    "no_act": nn.Identity(),
}


def _silu_op_bwd(x: Tensor, grad_output: Tensor) -> Tensor:
    sigma = torch.sigmoid(x)
    return grad_output * (sigma * (1 + x * (1 - sigma)))


ACT_BWD = {"silu": _silu_op_bwd, "swish": _silu_op_bwd}


class _GatedMLPBase(nn.Module):
    """Parameters and attributes shared by the eager and the fused module (same names, same order)."""

    def __init__(
        self,
        hidden_size: int = 256,
        intermediate_size: int = 512,
        bias: bool = True,
        hidden_act: str = "silu",
        dropout_p: float = 0.0,
    ):
        super().__init__()
        self.hidden_size = hidden_size
        self.intermediate_size = intermediate_size
        self.gate_proj = nn.Linear(hidden_size, intermediate_size, bias=bias)
        self.up_proj = nn.Linear(hidden_size, intermediate_size, bias=bias)
        self.down_proj = nn.Linear(intermediate_size, hidden_size, bias=bias)
        self.act = ACT_FWD[hidden_act]
        self.act_fn = hidden_act
        self.dropout = nn.Dropout(dropout_p)


class EagerGatedMLP(_GatedMLPBase):
    """down_proj(dropout(act(gate_proj(x)) * up_proj(x))) with stock torch operators."""

    def forward(self, x: Tensor) -> Tensor:
        lead = x.shape[:-1]
        x2 = x.reshape(-1, x.shape[-1])
        hidden = self.dropout(self.act(self.gate_proj(x2)) * self.up_proj(x2))
        return self.down_proj(hidden).reshape(*lead, self.hidden_size)


def eager_fwd(x: Tensor, WT_up: Tensor, b_up: Optional[Tensor], WT_gp: Tensor, b_gp: Optional[Tensor]) -> Tensor:
    """silu(x·W_gpᵀ + b_gp) * (x·W_upᵀ + b_up) in plain torch."""
    up = torch.nn.functional.linear(x, WT_up, b_up)
    gate = torch.nn.functional.linear(x, WT_gp, b_gp)
    return torch.nn.functional.silu(gate) * up


def eager_bwd(x: Tensor, W_up: Tensor, W_gp: Tensor, grad_output: Tensor):
    """Closed-form gradients (dx, dW_up, dW_gp) of eager_fwd without biases."""
    up = x @ W_up.T
    gate = x @ W_gp.T
    d_up = grad_output * torch.nn.functional.silu(gate)
    d_gate = _silu_op_bwd(gate, grad_output * up)
    return d_up @ W_up + d_gate @ W_gp, d_up.T @ x, d_gate.T @ x


class FusedGatedMLPFunction(Function):
    """Hidden-state operator hidden = dropout(act_fn(x·W_gpᵀ+b_gp) * (x·W_upᵀ+b_up)).

    Argument order (x, W_up, b_up, W_gp, b_gp) as in the reference; dropout_p, seed, offset and
    act_fn (default "silu") are optional.
    """

    @staticmethod
    def forward(
        ctx, x, W_up, b_up, W_gp, b_gp, dropout_p: float = 0.0, seed: int = 0, offset: int = 0, act_fn: str = "silu"
    ):
        needs_grad = any(ctx.needs_input_grad[:5])
        out = _fwd.gateup_fwd(
            x, W_gp, b_gp, W_up, b_up, dropout_p, seed, offset, save_activations=needs_grad, act_fn=act_fn
        )
        if needs_grad:
            ctx.save_for_backward(x, W_up, W_gp, out.gate, out.up)
        ctx.act_fn = act_fn
        ctx.dropout = (float(dropout_p), int(seed), int(offset))
        ctx.has_bias = (b_up is not None, b_gp is not None)
        return out.hidden

    @staticmethod
    def backward(ctx, grad_output):
        x, W_up, W_gp, gate, up = ctx.saved_tensors
        p, seed, offset = ctx.dropout
        need = ctx.needs_input_grad
        dg, du = _bwd.gating_bwd(grad_output, gate, up, p, seed, offset, ctx.act_fn)
        dx = _bwd.dx_bwd(dg, du, W_gp, W_up) if need[0] else None
        dW_up = _bwd.dw_bwd(du, x) if need[1] else None
        db_up = _bwd.colsum(du) if ctx.has_bias[0] and need[2] else None
        dW_gp = _bwd.dw_bwd(dg, x) if need[3] else None
        db_gp = _bwd.colsum(dg) if ctx.has_bias[1] and need[4] else None
        grads = (dx, dW_up, db_up, dW_gp, db_gp, None, None, None, None)
        return grads[: len(need)]  # apply() may have been called with the 5 reference arguments only


_CU_COUNT = {}


def _compute_units(device: torch.device) -> int:
    index = device.index if device.index is not None else torch.cuda.current_device()
    if index not in _CU_COUNT:
        _CU_COUNT[index] = torch.cuda.get_device_properties(index).multi_processor_count
    return _CU_COUNT[index]


class FusedGatedMLPFullFunction(Function):
    """Whole MLP as one autograd node, so dY -> (dG, dU) is a single GEMM with a fused epilogue."""

    @staticmethod
    def forward(
        ctx, x, W_gate, b_gate, W_up, b_up, W_down, b_down, dropout_p, seed, offset, recompute=False, act_fn="silu"
    ):
        needs_grad = any(ctx.needs_input_grad[:7])
        keep = needs_grad and not recompute
        # one library call enqueues the whole pass
        y, hs = _fwd.mlp_fwd(
            x, W_gate, b_gate, W_up, b_up, W_down, b_down, dropout_p, seed, offset, save_activations=keep, act_fn=act_fn
        )
        if keep:
            ctx.save_for_backward(x, W_gate, W_up, W_down, hs.gate, hs.up, hs.hidden)
        elif needs_grad:
            # memory-lean mode: keep the inputs only (as the reference does, gated_mlp.py:182) and
            # run the gate/up GEMM again in backward; the dropout mask is a function of the seed
            ctx.save_for_backward(x, W_gate, W_up, W_down, b_gate, b_up)
        ctx.recompute = bool(recompute)
        ctx.act_fn = act_fn
        ctx.dropout = (float(dropout_p), int(seed), int(offset))
        ctx.has_bias = (b_gate is not None, b_up is not None, b_down is not None)
        return y

    @staticmethod
    def backward(ctx, dy):
        p, seed, offset = ctx.dropout
        if ctx.recompute:
            x, W_gate, W_up, W_down, b_gate, b_up = ctx.saved_tensors
            hs = _fwd.gateup_fwd(
                x, W_gate, b_gate, W_up, b_up, p, seed, offset, save_activations=True, act_fn=ctx.act_fn
            )
            gate, up, hidden = hs.gate, hs.up, hs.hidden
        else:
            x, W_gate, W_up, W_down, gate, up, hidden = ctx.saved_tensors
        need = ctx.needs_input_grad
        has = ctx.has_bias
        want = (need[0], need[1], has[0] and need[2], need[3], has[1] and need[4], need[5], has[2] and need[6])
        # one library call enqueues the whole pass: dH with the gating epilogue, dX, the three
        # weight gradients as one grid, the bias gradients as one pair of launches
        grads = _bwd.mlp_bwd(dy, x, W_gate, W_up, W_down, gate, up, hidden, want, p, seed, offset, ctx.act_fn)
        return grads + (None, None, None, None, None)


class FusedGatedMLP(_GatedMLPBase):
    """Drop-in gated MLP running on hand-written gfx950 kernels (float16 / bfloat16 tuned; float32
    on a compatibility path).  `hidden_act` is any key of ACT_FWD.

    Dropout is active in training mode only.  The keep mask comes from a counter-based generator:
    set `dropout_seed` (int) for a fixed mask stream, otherwise each forward draws a seed from
    torch's default CPU generator (so `torch.manual_seed` makes runs repeatable).  The seed and
    offset of the last training forward are kept in `last_dropout_state`; a batch that ran as
    several row chunks (see `_forward_2d`) drew one mask per chunk, and `last_dropout_states` lists
    them all as (first row, rows, seed, offset), the mask of a chunk being that of a [rows, N] tensor.

    Under `torch.autocast("cuda")` the module casts its input and parameters to the autocast dtype
    for the kernels (fp32 master weights keep fp32 gradients), as nn.Linear does.

    `recompute_activations = True` selects the memory-lean backward: only x is kept from the forward
    pass and G, U, H are recomputed (one more gate/up GEMM) instead of holding 3*M*N elements.
    """

    def __init__(self, *args, **kwargs):
        super().__init__(*args, **kwargs)
        self.dropout_seed: Optional[int] = None
        self.recompute_activations = False
        self._dropout_calls = 0
        self.last_dropout_state = (0, 0)
        self.last_dropout_states = []

    def _next_dropout_state(self):
        if self.dropout_seed is None:
            seed, offset = int(torch.randint(0, 2**62, (1,)).item()), 0
        else:
            seed, offset = int(self.dropout_seed), self._dropout_calls
            self._dropout_calls += 1
        self.last_dropout_state = (seed, offset)
        return seed, offset

    def forward(self, x: Tensor) -> Tensor:
        lead = x.shape[:-1]
        x2 = x.reshape(-1, x.shape[-1])
        p = float(self.dropout.p) if self.training else 0.0
        gate, up, down = self.gate_proj, self.up_proj, self.down_proj
        self.last_dropout_states = []
        if x2.is_cuda and torch.is_autocast_enabled("cuda"):
            # Mixed precision as nn.Linear does it under torch.autocast: activations and (master)
            # weights are cast to the autocast dtype for the kernels; autograd casts the gradients back.
            with torch.autocast("cuda", enabled=False):
                return self._forward_cast(x2, torch.get_autocast_dtype("cuda"), p).reshape(*lead, self.hidden_size)
        return self._forward_2d(
            x2, gate.weight, gate.bias, up.weight, up.bias, down.weight, down.bias, p
        ).reshape(*lead, self.hidden_size)

    def _forward_cast(self, x2: Tensor, dtype: torch.dtype, p: float) -> Tensor:
        cast = lambda t: None if t is None else t.to(dtype)
        g, u, d = self.gate_proj, self.up_proj, self.down_proj
        return self._forward_2d(
            cast(x2), cast(g.weight), cast(g.bias), cast(u.weight), cast(u.bias), cast(d.weight), cast(d.bias), p
        )

    def _forward_2d(self, x2, W_gate, b_gate, W_up, b_up, W_down, b_down, p: float, row0: int = 0) -> Tensor:
        M, K = x2.shape
        limit = _fwd.max_rows_32bit(K, self.intermediate_size, x2.dtype) if x2.is_cuda else None
        if limit is not None and M > limit:
            # Token rows are independent: a batch too tall for the pipelined kernels' 32-bit operand
            # offsets runs as near-equal row chunks (autograd sums the chunks' weight gradients; with
            # dropout every chunk draws its own mask, recorded in `last_dropout_states`).
            chunks = -(-M // limit)
            rows = -(-M // (chunks * 256)) * 256
            return torch.cat(
                [
                    self._forward_2d(x2[i : i + rows], W_gate, b_gate, W_up, b_up, W_down, b_down, p, row0 + i)
                    for i in range(0, M, rows)
                ]
            )
        inference = not torch.is_grad_enabled() or not any(
            t is not None and t.requires_grad for t in (x2, W_gate, b_gate, W_up, b_up, W_down, b_down)
        )
        if inference and p == 0.0 and x2.is_cuda:
            # Nothing to differentiate: no autograd node (its bookkeeping costs more host time than a
            # short batch's kernels take to enqueue), and the weight-streaming kernels for skinny M.
            if _fwd.decode_preferred(M, K, self.intermediate_size, x2.dtype, _compute_units(x2.device)):
                return _fwd.decode_fwd(x2, W_gate, b_gate, W_up, b_up, W_down, b_down, self.act_fn)
            return _fwd.mlp_fwd(x2, W_gate, b_gate, W_up, b_up, W_down, b_down, act_fn=self.act_fn)[0]
        if x2.is_cuda and torch.cuda.is_current_stream_capturing():
            # Capturing forward + backward with torch.cuda.graph has ended in a host-side crash inside
            # the runtime's end-of-capture call on ROCm 7.2; until its cause is known the module
            # refuses rather than take the process down.  Inference forwards capture fine.
            raise RuntimeError(
                "FusedGatedMLP: capturing a step that records an autograd graph (training forward) into a "
                "HIP graph is not supported; capture inference forwards (torch.no_grad(), eval mode) only"
            )
        seed, offset = self._next_dropout_state() if p > 0.0 else (0, 0)
        if p > 0.0:
            self.last_dropout_states.append((row0, M, seed, offset))
        return FusedGatedMLPFullFunction.apply(
            x2, W_gate, b_gate, W_up, b_up, W_down, b_down, p, seed, offset, self.recompute_activations, self.act_fn
        )
