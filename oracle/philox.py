"""NumPy oracle (test infrastructure) of the dropout keep mask used by the HIP kernels.

Philox4x32-10 after Salmon, Moraes, Dror, Shaw, "Parallel Random Numbers: As Easy as 1, 2, 3"
(SC'11); multipliers 0xD2511F53 / 0xCD9E8D57, Weyl constants 0x9E3779B9 / 0xBB67AE85, 10 rounds.
Pinned in tests/test_oracle.py by the Random123 known-answer vectors, against the independent C
restatement in oracle/gated_mlp_ref.c, and by keep-rate statistics.

Mask definition (the library's contract, include/gmlp.h): for element e = m*N + n,
    words = philox4x32_10(ctr = [lo32(e//4), hi32(e//4), lo32(offset), hi32(offset)],
                          key = [lo32(seed), hi32(seed)])
    keep  = words[e % 4] >= floor(p * 2**32)
The reference applies torch's nn.Dropout (src/triton_gated_mlp/gated_mlp.py:90,96), whose mask
depends on torch's device generator; parity is therefore defined with this explicit mask.
"""

from __future__ import annotations

import numpy as np

M0, M1 = np.uint64(0xD2511F53), np.uint64(0xCD9E8D57)
W0, W1 = 0x9E3779B9, 0xBB67AE85
MASK32 = np.uint64(0xFFFFFFFF)


def philox4x32_10(ctr: np.ndarray, key: np.ndarray) -> np.ndarray:
    """ctr: uint32 [..., 4]; key: uint32 [..., 2] (broadcastable).  Returns uint32 [..., 4]."""
    c = [np.asarray(ctr[..., i], dtype=np.uint64) for i in range(4)]
    k0 = np.asarray(key[..., 0], dtype=np.uint64)
    k1 = np.asarray(key[..., 1], dtype=np.uint64)
    for _ in range(10):
        p0 = M0 * c[0]
        p1 = M1 * c[2]
        hi0, lo0 = p0 >> np.uint64(32), p0 & MASK32
        hi1, lo1 = p1 >> np.uint64(32), p1 & MASK32
        c = [hi1 ^ c[1] ^ k0, lo1, hi0 ^ c[3] ^ k1, lo0]
        k0 = (k0 + np.uint64(W0)) & MASK32
        k1 = (k1 + np.uint64(W1)) & MASK32
    return np.stack(c, axis=-1).astype(np.uint32)


def threshold(p: float) -> int:
    return min(int(np.floor(np.float64(np.float32(p)) * 4294967296.0)), 0xFFFFFFFF)


def keep_mask(M: int, N: int, p: float, seed: int, offset: int = 0) -> np.ndarray:
    """uint8 [M, N]; 1 = keep."""
    if p <= 0.0:
        return np.ones((M, N), dtype=np.uint8)
    total = M * N
    n4 = (total + 3) // 4
    e4 = np.arange(n4, dtype=np.uint64)
    ctr = np.stack(
        [e4 & MASK32, e4 >> np.uint64(32),
         np.full(n4, offset & 0xFFFFFFFF, dtype=np.uint64), np.full(n4, (offset >> 32) & 0xFFFFFFFF, dtype=np.uint64)],
        axis=-1,
    ).astype(np.uint32)
    key = np.array([seed & 0xFFFFFFFF, (seed >> 32) & 0xFFFFFFFF], dtype=np.uint32)
    words = philox4x32_10(ctr, key[None, :]).reshape(-1)[:total]
    return (words >= np.uint32(threshold(p))).astype(np.uint8).reshape(M, N)
