"""Backward operators of the gated MLP on MI355X (host wrappers over libgmlp.so).

`mlp_hidden_states_bwd(x, W_up, W_gp, grad_output)` keeps the reference signature and return
order `(dx, dW_up, dW_gp)` (src/triton_gated_mlp/ops/bwd.py:466-468,602).  The reference
recomputes G and U inside its first backward kernel; callers that kept them from the forward pass
hand them in through the keyword arguments and skip that GEMM.
"""

from __future__ import annotations

from typing import Optional, Tuple

import torch
from torch import Tensor

from .. import _cabi
from .fwd import _c, gateup_fwd


def dh_bwd(
    dy: Tensor,
    W_down: Tensor,
    g: Tensor,
    u: Tensor,
    dropout_p: float = 0.0,
    seed: int = 0,
    offset: int = 0,
    act_fn: str = "silu",
) -> Tuple[Tensor, Tensor]:
    """(dG, dU) from dY: dH = dY·W_down with dropout and gating backward fused in the epilogue."""
    M, K = dy.shape
    N = W_down.shape[1]
    if tuple(W_down.shape) != (K, N) or tuple(g.shape) != (M, N) or tuple(u.shape) != (M, N):
        raise ValueError("dimension mismatch among dy, W_down, g, u")
    dev = _cabi.require_gpu(dy, W_down, g, u)
    code = _cabi.dtype_code(dy.dtype)
    act = _cabi.act_code(act_fn)
    dy, W_down, g, u = _c(dy), _c(W_down), _c(g), _c(u)
    dg = torch.empty_like(g)
    du = torch.empty_like(u)
    if M > 0:
        with torch.cuda.device(dev):
            ws = _cabi.workspace(_cabi.GMLP_OP_DH_BWD, M, K, N, code, dev)
            _cabi.check(
                _cabi.lib().gmlp_dh_bwd(
                    _cabi.ptr(dy), _cabi.ptr(W_down), _cabi.ptr(g), _cabi.ptr(u), _cabi.ptr(dg), _cabi.ptr(du),
                    M, K, N, code, act, float(dropout_p), int(seed), int(offset),
                    _cabi.ptr(ws), 0 if ws is None else ws.numel(), _cabi.stream_ptr(dev),
                )
            )
    return dg, du


def gating_bwd(
    dh: Tensor,
    g: Tensor,
    u: Tensor,
    dropout_p: float = 0.0,
    seed: int = 0,
    offset: int = 0,
    act_fn: str = "silu",
) -> Tuple[Tensor, Tensor]:
    """(dG, dU) from dH (element-wise): dU = dA*act(G), dG = dA*U*act'(G), dA = dH*keep/(1-p)."""
    if g.shape != dh.shape or u.shape != dh.shape or dh.ndim != 2:
        raise ValueError("dh, g, u must be 2-D tensors of one shape")
    dev = _cabi.require_gpu(dh, g, u)
    code = _cabi.dtype_code(dh.dtype)
    act = _cabi.act_code(act_fn)
    dh, g, u = _c(dh), _c(g), _c(u)
    M, N = dh.shape
    dg = torch.empty_like(g)
    du = torch.empty_like(u)
    if M > 0:
        with torch.cuda.device(dev):
            _cabi.check(
                _cabi.lib().gmlp_gating_bwd(
                    _cabi.ptr(dh), _cabi.ptr(g), _cabi.ptr(u), _cabi.ptr(dg), _cabi.ptr(du), M, N, code, act,
                    float(dropout_p), int(seed), int(offset), _cabi.stream_ptr(dev),
                )
            )
    return dg, du


def dx_bwd(dg: Tensor, du: Tensor, W_gate: Tensor, W_up: Tensor) -> Tensor:
    """dX = dG·W_gate + dU·W_up as one GEMM over the concatenated reduction."""
    M, N = dg.shape
    K = W_gate.shape[1]
    if du.shape != dg.shape or tuple(W_gate.shape) != (N, K) or tuple(W_up.shape) != (N, K):
        raise ValueError("dimension mismatch among dg, du, W_gate, W_up")
    dev = _cabi.require_gpu(dg, du, W_gate, W_up)
    code = _cabi.dtype_code(dg.dtype)
    dg, du, W_gate, W_up = _c(dg), _c(du), _c(W_gate), _c(W_up)
    dx = torch.empty((M, K), dtype=dg.dtype, device=dev)
    if M > 0:
        with torch.cuda.device(dev):
            ws = _cabi.workspace(_cabi.GMLP_OP_DX_BWD, M, K, N, code, dev)
            _cabi.check(
                _cabi.lib().gmlp_dx_bwd(
                    _cabi.ptr(dg), _cabi.ptr(du), _cabi.ptr(W_gate), _cabi.ptr(W_up), _cabi.ptr(dx), M, K, N,
                    code, _cabi.ptr(ws), 0 if ws is None else ws.numel(), _cabi.stream_ptr(dev),
                )
            )
    return dx


def dw_bwd(lhs: Tensor, rhs: Tensor) -> Tensor:
    """dW[R,C] = lhs[M,R]ᵀ · rhs[M,C] (weight gradient of a linear layer)."""
    if lhs.ndim != 2 or rhs.ndim != 2 or lhs.shape[0] != rhs.shape[0]:
        raise ValueError(f"dimension mismatch: lhs {tuple(lhs.shape)}, rhs {tuple(rhs.shape)}")
    dev = _cabi.require_gpu(lhs, rhs)
    code = _cabi.dtype_code(lhs.dtype)
    lhs, rhs = _c(lhs), _c(rhs)
    M, R = lhs.shape
    C = rhs.shape[1]
    if M == 0:
        return torch.zeros((R, C), dtype=lhs.dtype, device=dev)
    dw = torch.empty((R, C), dtype=lhs.dtype, device=dev)
    with torch.cuda.device(dev):
        ws = _cabi.workspace(_cabi.GMLP_OP_DW_BWD, M, R, C, code, dev)
        _cabi.check(
            _cabi.lib().gmlp_dw_bwd(
                _cabi.ptr(lhs), _cabi.ptr(rhs), _cabi.ptr(dw), M, R, C, code,
                _cabi.ptr(ws), 0 if ws is None else ws.numel(), _cabi.stream_ptr(dev),
            )
        )
    return dw


def dw_bwd_grouped(pairs):
    """Weight gradients [lhs_iᵀ · rhs_i for (lhs_i, rhs_i) in pairs] (at most 3 pairs sharing the
    reduction length) enqueued as one grid when every problem fits the full-tile kernel."""
    import ctypes

    pairs = [(_c(a), _c(b)) for a, b in pairs]
    if not 1 <= len(pairs) <= 3:
        raise ValueError("dw_bwd_grouped takes 1 to 3 (lhs, rhs) pairs")
    M = pairs[0][0].shape[0]
    for a, b in pairs:
        if a.ndim != 2 or b.ndim != 2 or a.shape[0] != M or b.shape[0] != M:
            raise ValueError("every pair must be 2-D with the same number of rows")
    dev = _cabi.require_gpu(*[t for p in pairs for t in p])
    code = _cabi.dtype_code(pairs[0][0].dtype)
    if M == 0:
        return [torch.zeros((a.shape[1], b.shape[1]), dtype=a.dtype, device=dev) for a, b in pairs]
    outs = [torch.empty((a.shape[1], b.shape[1]), dtype=a.dtype, device=dev) for a, b in pairs]
    n = len(pairs)
    PtrArr, I64Arr = ctypes.c_void_p * n, ctypes.c_int64 * n
    lhs = PtrArr(*[a.data_ptr() for a, _ in pairs])
    rhs = PtrArr(*[b.data_ptr() for _, b in pairs])
    dws = PtrArr(*[o.data_ptr() for o in outs])
    R = I64Arr(*[a.shape[1] for a, _ in pairs])
    C = I64Arr(*[b.shape[1] for _, b in pairs])
    with torch.cuda.device(dev):
        nbytes = _cabi.lib().gmlp_dw_bwd_grouped_workspace_bytes(
            n, M, ctypes.cast(R, ctypes.c_void_p), ctypes.cast(C, ctypes.c_void_p), code
        )
        ws = torch.empty((nbytes,), dtype=torch.uint8, device=dev) if nbytes else None
        _cabi.check(
            _cabi.lib().gmlp_dw_bwd_grouped(
                n, ctypes.cast(lhs, ctypes.c_void_p), ctypes.cast(rhs, ctypes.c_void_p),
                ctypes.cast(dws, ctypes.c_void_p), M, ctypes.cast(R, ctypes.c_void_p),
                ctypes.cast(C, ctypes.c_void_p), code, _cabi.ptr(ws), 0 if ws is None else ws.numel(),
                _cabi.stream_ptr(dev),
            )
        )
    return outs


def colsum(a: Tensor) -> Tensor:
    """Σ_m a[m,:] with fp32 accumulation in a fixed order (bias gradient)."""
    if a.ndim != 2:
        raise ValueError("colsum takes a 2-D tensor")
    dev = _cabi.require_gpu(a)
    code = _cabi.dtype_code(a.dtype)
    a = _c(a)
    M, C = a.shape
    if M == 0:
        return torch.zeros((C,), dtype=a.dtype, device=dev)
    out = torch.empty((C,), dtype=a.dtype, device=dev)
    nbytes = _cabi.lib().gmlp_workspace_bytes(_cabi.GMLP_OP_COLSUM, M, 0, C, code)
    ws = torch.empty((nbytes,), dtype=torch.uint8, device=dev)
    with torch.cuda.device(dev):
        _cabi.check(
            _cabi.lib().gmlp_colsum(_cabi.ptr(a), _cabi.ptr(out), _cabi.ptr(ws), M, C, code, _cabi.stream_ptr(dev))
        )
    return out


def colsum_static(a: Tensor, out: Optional[Tensor] = None) -> Tensor:
    """colsum through the entry point that allocates nothing (gmlp_colsum_static): the partial sums
    live in a static device array of the library, so only `out` is the caller's (pass one to make
    the call allocation-free, e.g. under graph capture).  At most 32768 columns; calls that overlap
    on one GPU share the array and race."""
    if a.ndim != 2 or a.shape[0] < 1:
        raise ValueError("colsum_static takes a 2-D tensor with at least one row")
    dev = _cabi.require_gpu(a, out)
    code = _cabi.dtype_code(a.dtype)
    if not a.is_contiguous():
        raise ValueError("colsum_static takes a contiguous tensor (it would have to allocate a copy)")
    M, C = a.shape
    if out is None:
        out = torch.empty((C,), dtype=a.dtype, device=dev)
    elif tuple(out.shape) != (C,) or not out.is_contiguous():
        raise ValueError("out must be a contiguous tensor of C elements")
    with torch.cuda.device(dev):
        _cabi.check(
            _cabi.lib().gmlp_colsum_static(_cabi.ptr(a), _cabi.ptr(out), M, C, code, _cabi.stream_ptr(dev))
        )
    return out


def colsum_grouped(arrays):
    """[Σ_m a[m,:] for a in arrays] (at most 3 arrays with the same number of rows) in one pair of
    launches: the bias gradients of one backward pass."""
    import ctypes

    arrays = [_c(a) for a in arrays]
    if not 1 <= len(arrays) <= 3:
        raise ValueError("colsum_grouped takes 1 to 3 arrays")
    M = arrays[0].shape[0]
    for a in arrays:
        if a.ndim != 2 or a.shape[0] != M:
            raise ValueError("every array must be 2-D with the same number of rows")
    dev = _cabi.require_gpu(*arrays)
    code = _cabi.dtype_code(arrays[0].dtype)
    if M == 0:
        return [torch.zeros((a.shape[1],), dtype=a.dtype, device=dev) for a in arrays]
    outs = [torch.empty((a.shape[1],), dtype=a.dtype, device=dev) for a in arrays]
    n = len(arrays)
    nbytes = sum(_cabi.lib().gmlp_workspace_bytes(_cabi.GMLP_OP_COLSUM, M, 0, a.shape[1], code) for a in arrays)
    ws = torch.empty((nbytes,), dtype=torch.uint8, device=dev)
    PtrArr, I64Arr = ctypes.c_void_p * n, ctypes.c_int64 * n
    srcs = PtrArr(*[a.data_ptr() for a in arrays])
    dsts = PtrArr(*[o.data_ptr() for o in outs])
    C = I64Arr(*[a.shape[1] for a in arrays])
    with torch.cuda.device(dev):
        _cabi.check(
            _cabi.lib().gmlp_colsum_grouped(
                n, ctypes.cast(srcs, ctypes.c_void_p), ctypes.cast(dsts, ctypes.c_void_p), _cabi.ptr(ws), M,
                ctypes.cast(C, ctypes.c_void_p), code, _cabi.stream_ptr(dev),
            )
        )
    return outs


def mlp_bwd(
    dy: Tensor,
    x: Tensor,
    W_gate: Tensor,
    W_up: Tensor,
    W_down: Tensor,
    g: Tensor,
    u: Tensor,
    h: Tensor,
    need=(True,) * 7,
    dropout_p: float = 0.0,
    seed: int = 0,
    offset: int = 0,
    act_fn: str = "silu",
):
    """Whole backward pass in one library call (gmlp_mlp_bwd).

    `need` = which of (dx, dW_gate, db_gate, dW_up, db_up, dW_down, db_down) to compute; returns
    that 7-tuple with None for the others.  dG, dU and the library's workspace share one scratch
    allocation that is dropped on return."""
    M, K = dy.shape
    N = W_down.shape[1]
    if (
        tuple(x.shape) != (M, K) or tuple(W_gate.shape) != (N, K) or tuple(W_up.shape) != (N, K)
        or tuple(W_down.shape) != (K, N) or tuple(g.shape) != (M, N) or tuple(u.shape) != (M, N)
        or tuple(h.shape) != (M, N)
    ):
        raise ValueError("dimension mismatch among dy, x, the weights and the kept activations")
    dev = _cabi.require_gpu(dy, x, W_gate, W_up, W_down, g, u, h)
    code = _cabi.dtype_code(dy.dtype)
    act = _cabi.act_code(act_fn)
    dy, x, W_gate, W_up, W_down, g, u, h = (_c(t) for t in (dy, x, W_gate, W_up, W_down, g, u, h))
    shapes = ((M, K), (N, K), (N,), (N, K), (N,), (K, N), (K,))
    if M == 0:
        return tuple(torch.zeros(s, dtype=dy.dtype, device=dev) if n else None for s, n in zip(shapes, need))
    outs = [torch.empty(s, dtype=dy.dtype, device=dev) if n else None for s, n in zip(shapes, need)]
    dx, dwg, dbg, dwu, dbu, dwd, dbd = outs
    with torch.cuda.device(dev):
        nbytes = _cabi.mlp_workspace_bytes(_cabi.GMLP_PASS_BWD, M, K, N, code, dev)
        plane = (M * N * dy.element_size() + 255) // 256 * 256
        arena = torch.empty((2 * plane + nbytes,), dtype=torch.uint8, device=dev)
        base = arena.data_ptr()
        _cabi.check(
            _cabi.lib().gmlp_mlp_bwd(
                _cabi.ptr(dy), _cabi.ptr(x), _cabi.ptr(W_gate), _cabi.ptr(W_up), _cabi.ptr(W_down),
                _cabi.ptr(g), _cabi.ptr(u), _cabi.ptr(h), base, base + plane,
                _cabi.ptr(dx), _cabi.ptr(dwg), _cabi.ptr(dwu), _cabi.ptr(dwd), _cabi.ptr(dbg), _cabi.ptr(dbu),
                _cabi.ptr(dbd), M, K, N, code, act, float(dropout_p), int(seed), int(offset),
                base + 2 * plane if nbytes else None, nbytes, _cabi.stream_ptr(dev),
            )
        )
    return tuple(outs)


def mlp_hidden_states_bwd(
    x: Tensor,
    W_up: Tensor,
    W_gp: Tensor,
    grad_output: Tensor,
    *,
    b_up: Optional[Tensor] = None,
    b_gp: Optional[Tensor] = None,
    gate: Optional[Tensor] = None,
    up: Optional[Tensor] = None,
    dropout_p: float = 0.0,
    seed: int = 0,
    offset: int = 0,
    return_bias_grads: bool = False,
    act_fn: str = "silu",
):
    """Gradients of hidden = dropout(act_fn(x·W_gpᵀ+b_gp) * (x·W_upᵀ+b_up)) w.r.t. x, W_up, W_gp.

    Returns (dx, dW_up, dW_gp), or (dx, dW_up, db_up, dW_gp, db_gp) with return_bias_grads.
    """
    if gate is None or up is None:
        fwd = gateup_fwd(x, W_gp, b_gp, W_up, b_up, 0.0, 0, 0, save_activations=True, act_fn=act_fn)
        gate, up = fwd.gate, fwd.up
    dg, du = gating_bwd(grad_output, gate, up, dropout_p, seed, offset, act_fn)
    dx = dx_bwd(dg, du, W_gp, W_up)
    dW_up = dw_bwd(du, x)
    dW_gp = dw_bwd(dg, x)
    if return_bias_grads:
        db_up, db_gp = colsum_grouped([du, dg])
        return dx, dW_up, db_up, dW_gp, db_gp
    return dx, dW_up, dW_gp
