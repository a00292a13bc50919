"""Forward operators of the gated MLP on MI355X (host wrappers over libgmlp.so).

`mlp_hidden_states_fwd` keeps the positional signature of the reference operator
(src/triton_gated_mlp/ops/fwd.py:198-206); the keyword-only arguments are extensions (dropout seed,
saving G and U for the backward pass).  Unlike the reference it applies the biases and the dropout
it is given, and makes its inputs contiguous instead of assuming it.
"""

from __future__ import annotations

from typing import NamedTuple, Optional

import torch
from torch import Tensor

from .. import _cabi


def validate_dimensions(
    x: Tensor, WT_up: Tensor, b_up: Optional[Tensor], WT_gp: Tensor, b_gp: Optional[Tensor]
) -> None:
    """Same conditions as the reference (src/triton_gated_mlp/ops/fwd.py:169-184), raised as ValueError."""
    if x.ndim != 2:
        raise ValueError(f"input tensor must be 2-D [M, K], got {x.ndim} dims")
    if WT_up.ndim != 2 or WT_up.shape[1] != x.shape[1]:
        raise ValueError(f"dimension mismatch in WT_up {tuple(WT_up.shape)} or x {tuple(x.shape)}")
    if WT_gp.shape != WT_up.shape:
        raise ValueError(f"dimension mismatch in WT_up {tuple(WT_up.shape)} or WT_gp {tuple(WT_gp.shape)}")
    if b_up is not None and tuple(b_up.shape) != (WT_up.shape[0],):
        raise ValueError("dimension mismatch in b_up")
    if b_gp is not None and tuple(b_gp.shape) != (WT_up.shape[0],):
        raise ValueError("dimension mismatch in b_gp")


class HiddenStates(NamedTuple):
    hidden: Tensor
    gate: Optional[Tensor]  # G = x·W_gateᵀ + b_gate (kept for backward)
    up: Optional[Tensor]  # U = x·W_upᵀ + b_up
    mask: Optional[Tensor]  # uint8 keep mask


def _c(t: Optional[Tensor]) -> Optional[Tensor]:
    return None if t is None else t.contiguous()


def gateup_fwd(
    x: Tensor,
    W_gate: Tensor,
    b_gate: Optional[Tensor],
    W_up: Tensor,
    b_up: Optional[Tensor],
    dropout_p: float = 0.0,
    seed: int = 0,
    offset: int = 0,
    save_activations: bool = False,
    return_mask: bool = False,
    act_fn: str = "silu",
) -> HiddenStates:
    """H = dropout(act_fn(x·W_gateᵀ + b_gate) * (x·W_upᵀ + b_up)) in one kernel."""
    validate_dimensions(x, W_up, b_up, W_gate, b_gate)
    act = _cabi.act_code(act_fn)
    dev = _cabi.require_gpu(x, W_gate, b_gate, W_up, b_up)
    code = _cabi.dtype_code(x.dtype)
    x, W_gate, W_up, b_gate, b_up = _c(x), _c(W_gate), _c(W_up), _c(b_gate), _c(b_up)
    M, K = x.shape
    N = W_up.shape[0]
    h = torch.empty((M, N), dtype=x.dtype, device=dev)
    g = torch.empty_like(h) if save_activations else None
    u = torch.empty_like(h) if save_activations else None
    mask = torch.empty((M, N), dtype=torch.uint8, device=dev) if return_mask else None
    if M > 0:
        with torch.cuda.device(dev):
            ws = _cabi.workspace(_cabi.GMLP_OP_GATEUP_FWD, M, K, N, code, dev)
            _cabi.check(
                _cabi.lib().gmlp_gateup_fwd(
                    _cabi.ptr(x), _cabi.ptr(W_gate), _cabi.ptr(W_up), _cabi.ptr(b_gate), _cabi.ptr(b_up),
                    _cabi.ptr(h), _cabi.ptr(g), _cabi.ptr(u), _cabi.ptr(mask),
                    M, K, N, code, act, float(dropout_p), int(seed), int(offset),
                    _cabi.ptr(ws), 0 if ws is None else ws.numel(), _cabi.stream_ptr(dev),
                )
            )
    return HiddenStates(h, g, u, mask)


def mlp_hidden_states_fwd(
    x: Tensor,
    WT_up: Tensor,
    b_up: Optional[Tensor],
    WT_gp: Tensor,
    b_gp: Optional[Tensor],
    act_fn: str = "silu",
    dropout_p: float = 0.0,
    *,
    seed: int = 0,
    offset: int = 0,
) -> Tensor:
    """dropout(act_fn(gate_proj(x)) * up_proj(x)) fused; weights in nn.Linear [N, K] layout.

    act_fn is any name of the reference's activation table (silu, swish, gelu, relu, leaky_relu,
    sigmoid, tanh, no_act); an unknown name raises NotImplementedError like the reference's
    _act_fwd (src/triton_gated_mlp/ops/act.py:5-12).
    """
    return gateup_fwd(x, WT_gp, b_gp, WT_up, b_up, dropout_p, seed, offset, act_fn=act_fn).hidden


def linear_fwd(a: Tensor, W: Tensor, bias: Optional[Tensor] = None) -> Tensor:
    """a[M,R]·W[C,R]ᵀ + bias: the down projection (reference: nn.Linear, gated_mlp.py:236)."""
    if a.ndim != 2 or W.ndim != 2 or W.shape[1] != a.shape[1]:
        raise ValueError(f"dimension mismatch: a {tuple(a.shape)}, W {tuple(W.shape)}")
    if bias is not None and tuple(bias.shape) != (W.shape[0],):
        raise ValueError("dimension mismatch in bias")
    dev = _cabi.require_gpu(a, W, bias)
    code = _cabi.dtype_code(a.dtype)
    a, W, bias = _c(a), _c(W), _c(bias)
    M, R = a.shape
    C = W.shape[0]
    out = torch.empty((M, C), dtype=a.dtype, device=dev)
    if M > 0:
        with torch.cuda.device(dev):
            ws = _cabi.workspace(_cabi.GMLP_OP_LINEAR_FWD, M, R, C, code, dev)
            _cabi.check(
                _cabi.lib().gmlp_linear_fwd(
                    _cabi.ptr(a), _cabi.ptr(W), _cabi.ptr(bias), _cabi.ptr(out), M, R, C, code,
                    _cabi.ptr(ws), 0 if ws is None else ws.numel(), _cabi.stream_ptr(dev),
                )
            )
    return out


def mlp_fwd(
    x: Tensor,
    W_gate: Tensor,
    b_gate: Optional[Tensor],
    W_up: Tensor,
    b_up: Optional[Tensor],
    W_down: Tensor,
    b_down: Optional[Tensor],
    dropout_p: float = 0.0,
    seed: int = 0,
    offset: int = 0,
    save_activations: bool = False,
    act_fn: str = "silu",
):
    """Whole forward pass in one library call (gmlp_mlp_fwd): returns (y, HiddenStates).

    The same kernels as gateup_fwd followed by linear_fwd, enqueued by one foreign call; G, U and H
    share one allocation when they are kept for the backward pass."""
    validate_dimensions(x, W_up, b_up, W_gate, b_gate)
    M, K = x.shape
    N = W_up.shape[0]
    if tuple(W_down.shape) != (K, N):
        raise ValueError(f"dimension mismatch in W_down {tuple(W_down.shape)}")
    if b_down is not None and tuple(b_down.shape) != (K,):
        raise ValueError("dimension mismatch in b_down")
    act = _cabi.act_code(act_fn)
    dev = _cabi.require_gpu(x, W_gate, b_gate, W_up, b_up, W_down, b_down)
    code = _cabi.dtype_code(x.dtype)
    x, W_gate, W_up, W_down = _c(x), _c(W_gate), _c(W_up), _c(W_down)
    b_gate, b_up, b_down = _c(b_gate), _c(b_up), _c(b_down)
    y = torch.empty((M, K), dtype=x.dtype, device=dev)
    if save_activations:
        g, u, h = torch.empty((3, M, N), dtype=x.dtype, device=dev).unbind(0)
    else:
        g = u = None
        h = torch.empty((M, N), dtype=x.dtype, device=dev)
    if M > 0:
        with torch.cuda.device(dev):
            nbytes = _cabi.mlp_workspace_bytes(_cabi.GMLP_PASS_FWD, M, K, N, code, dev)
            ws = torch.empty((nbytes,), dtype=torch.uint8, device=dev) if nbytes else None
            _cabi.check(
                _cabi.lib().gmlp_mlp_fwd(
                    _cabi.ptr(x), _cabi.ptr(W_gate), _cabi.ptr(W_up), _cabi.ptr(W_down), _cabi.ptr(b_gate),
                    _cabi.ptr(b_up), _cabi.ptr(b_down), _cabi.ptr(y), _cabi.ptr(h), _cabi.ptr(g), _cabi.ptr(u),
                    M, K, N, code, act, float(dropout_p), int(seed), int(offset),
                    _cabi.ptr(ws), nbytes, _cabi.stream_ptr(dev),
                )
            )
    return y, HiddenStates(h, g, u, None)


DECODE_MAX_M = 32
DECODE_PREFERRED_MAX_M = 32


def max_rows_32bit(K: int, N: int, dtype: torch.dtype) -> Optional[int]:
    """Largest token count (a multiple of 256) whose [M, K] and [M, N] operands the pipelined kernels
    can address, or None when there is no such limit (float32).

    Those kernels read their operands through buffer descriptors with 32-bit byte offsets, padded
    to whole tiles; the library runs anything larger on its slower predicated kernels.  Rows of the
    MLP are independent, so the module splits such a batch into row chunks instead.
    """
    if dtype == torch.float32:
        return None
    width = (max(K, N) + 255) // 256 * 256
    limit = (1 << 31) - 4096  # the descriptor base sits up to 4 KB below the operand
    return max(256, (limit - 1) // (2 * width) // 256 * 256)


def _decode_streams(K: int, N: int) -> bool:
    """Shapes the LDS-ring streaming kernels take (the others run on plainer skinny-M kernels)."""
    return K % 256 == 0 and N % 256 == 0 and K >= 768 and N >= 768 and K * N < (1 << 30)


def decode_supported(M: int, K: int, N: int, dtype: torch.dtype = torch.float16) -> bool:
    if dtype not in (torch.float16, torch.bfloat16) or K % 32 != 0 or N % 256 != 0:
        return False
    return 1 <= M <= 16 or (16 < M <= DECODE_MAX_M and _decode_streams(K, N))


def decode_preferred(M: int, K: int, N: int, dtype: torch.dtype = torch.float16, num_cu: int = 256) -> bool:
    """True when the skinny-M streaming kernels are the faster way to run the forward pass.

    They give every compute unit the same share of the weight rows (in blocks of 16 rows of
    W_gate/W_up, and of 32 or 16 rows of W_down), so they need widths that give each unit at least
    a block of W_gate/W_up rows and half a block of W_down rows; from there they beat or match the
    general path (GEMMs with split reductions) for every M <= 16 (measured on MI355X at the widths
    of Llama-2-7B/13B, Llama-3-8B/70B, 6144 x 16384 and 2048 x 8192).  With two token tiles
    (16 < M <= 32) the token operands cost L2 traffic of the order of the weights' HBM traffic: the
    kernels win by 4 to 17 % at M = 17 and by 0 to 10 % at M = 24 and 32 for hidden sizes from 3584
    up; below that they tie or lose (2560 x 10240: -12 %), so the module asks for 14 rows of W_down
    per compute unit there.
    """
    if M > DECODE_PREFERRED_MAX_M or not decode_supported(M, K, N, dtype) or K % 256 != 0 or N < 16 * num_cu:
        return False
    return K >= (8 if M <= 16 else 14) * num_cu


def decode_fwd(
    x: Tensor,
    W_gate: Tensor,
    b_gate: Optional[Tensor],
    W_up: Tensor,
    b_up: Optional[Tensor],
    W_down: Tensor,
    b_down: Optional[Tensor],
    act_fn: str = "silu",
) -> Tensor:
    """Whole-MLP forward for M <= 32 token rows: every weight byte is read from HBM once."""
    validate_dimensions(x, W_up, b_up, W_gate, b_gate)
    M, K = x.shape
    N = W_up.shape[0]
    if tuple(W_down.shape) != (K, N):
        raise ValueError(f"dimension mismatch in W_down {tuple(W_down.shape)}")
    dev = _cabi.require_gpu(x, W_gate, b_gate, W_up, b_up, W_down, b_down)
    code = _cabi.dtype_code(x.dtype)
    act = _cabi.act_code(act_fn)
    x, W_gate, W_up, W_down = _c(x), _c(W_gate), _c(W_up), _c(W_down)
    b_gate, b_up, b_down = _c(b_gate), _c(b_up), _c(b_down)
    # scratch: H for 16 or 32 token slots, in the library's layout
    h = torch.empty((16 if M <= 16 else 32, N), dtype=x.dtype, device=dev)
    y = torch.empty((M, K), dtype=x.dtype, device=dev)
    with torch.cuda.device(dev):
        _cabi.check(
            _cabi.lib().gmlp_decode_fwd(
                _cabi.ptr(x), _cabi.ptr(W_gate), _cabi.ptr(W_up), _cabi.ptr(W_down), _cabi.ptr(b_gate),
                _cabi.ptr(b_up), _cabi.ptr(b_down), _cabi.ptr(h), _cabi.ptr(y), None, M, K, N, code, act,
                _cabi.stream_ptr(dev),
            )
        )
    return y


def dropout_mask(M: int, N: int, dropout_p: float, seed: int, offset: int = 0, device=None) -> Tensor:
    """uint8 [M,N] keep mask of the kernels' counter-based generator (1 = keep)."""
    dev = torch.device("cuda", torch.cuda.current_device()) if device is None else torch.device(device)
    mask = torch.empty((M, N), dtype=torch.uint8, device=dev)
    if M * N > 0:
        with torch.cuda.device(dev):
            _cabi.check(
                _cabi.lib().gmlp_dropout_mask(
                    _cabi.ptr(mask), M, N, float(dropout_p), int(seed), int(offset), _cabi.stream_ptr(dev)
                )
            )
    return mask
