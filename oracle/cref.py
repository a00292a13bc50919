"""ctypes wrapper of oracle/_build/libgmlp_ref.so (the plain-C checker; test infrastructure)."""

from __future__ import annotations

import ctypes
import subprocess
from pathlib import Path

import numpy as np

_HERE = Path(__file__).resolve().parent
_LIB = _HERE / "_build" / "libgmlp_ref.so"
_lib = None


def build() -> Path:
    subprocess.run(["make", "-C", str(_HERE), "-s"], check=True)
    return _LIB


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not _LIB.exists():
            build()
        _lib = ctypes.CDLL(str(_LIB))
    return _lib


def _d(a):
    return None if a is None else np.ascontiguousarray(a, dtype=np.float64)


def _p(a, t=ctypes.c_double):
    return None if a is None else a.ctypes.data_as(ctypes.POINTER(t))


ACT_CODES = {"silu": 0, "swish": 0, "gelu": 1, "relu": 2, "leaky_relu": 3, "sigmoid": 4, "tanh": 5, "no_act": 6}


def forward(x, wg, bg, wu, bu, wd, bd, keep=None, p=0.0, act="silu"):
    x, wg, bg, wu, bu, wd, bd = map(_d, (x, wg, bg, wu, bu, wd, bd))
    M, K = x.shape
    N = wg.shape[0]
    keep = None if keep is None else np.ascontiguousarray(keep, dtype=np.uint8)
    G, U, H, Y = (np.empty((M, N)), np.empty((M, N)), np.empty((M, N)), np.empty((M, K)))
    lib().gmlp_ref_forward(
        _p(x), _p(wg), _p(bg), _p(wu), _p(bu), _p(wd), _p(bd), _p(keep, ctypes.c_uint8), ctypes.c_double(p),
        ctypes.c_int(ACT_CODES[act]), ctypes.c_int64(M), ctypes.c_int64(K), ctypes.c_int64(N), _p(G), _p(U), _p(H),
        _p(Y),
    )
    return {"G": G, "U": U, "H": H, "Y": Y}


def backward(x, wg, bg, wu, bu, wd, bd, dY, keep=None, p=0.0, act="silu"):
    f = forward(x, wg, bg, wu, bu, wd, bd, keep, p, act)
    x, wg, wu, wd, dY = map(_d, (x, wg, wu, wd, dY))
    M, K = x.shape
    N = wg.shape[0]
    keep = None if keep is None else np.ascontiguousarray(keep, dtype=np.uint8)
    out = {
        "dX": np.empty((M, K)), "dW_gate": np.empty((N, K)), "dW_up": np.empty((N, K)), "dW_down": np.empty((K, N)),
        "db_gate": np.empty(N), "db_up": np.empty(N), "db_down": np.empty(K),
    }
    lib().gmlp_ref_backward(
        _p(x), _p(wg), _p(wu), _p(wd), _p(keep, ctypes.c_uint8), ctypes.c_double(p),
        ctypes.c_int(ACT_CODES[act]), _p(f["G"]), _p(f["U"]),
        _p(f["H"]), _p(dY), ctypes.c_int64(M), ctypes.c_int64(K), ctypes.c_int64(N), _p(out["dX"]),
        _p(out["dW_gate"]), _p(out["dW_up"]), _p(out["dW_down"]), _p(out["db_gate"]), _p(out["db_up"]),
        _p(out["db_down"]),
    )
    out.update(f)
    return out


def philox4x32_10(ctr, key):
    c = (ctypes.c_uint32 * 4)(*[int(v) for v in ctr])
    k = (ctypes.c_uint32 * 2)(*[int(v) for v in key])
    o = (ctypes.c_uint32 * 4)()
    lib().gmlp_ref_philox4x32_10(c, k, o)
    return [int(v) for v in o]


def keep_mask(M, N, threshold, seed, offset=0):
    keep = np.empty((M, N), dtype=np.uint8)
    lib().gmlp_ref_keep_mask(
        _p(keep, ctypes.c_uint8), ctypes.c_int64(M), ctypes.c_int64(N), ctypes.c_uint32(threshold),
        ctypes.c_uint64(seed), ctypes.c_uint64(offset),
    )
    return keep
