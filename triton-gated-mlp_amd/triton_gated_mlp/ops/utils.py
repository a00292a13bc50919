"""Host helpers with the names of the reference's ops/utils.py.

`get_num_streaming_multiprocessors` (src/triton_gated_mlp/ops/utils.py:6-11) sizes persistent grids
in the reference; here the library reads the compute-unit count itself, the function is kept for
callers.  `map_pid_m_n` restates on the host the grouped tile order of the reference's
`map_pid_m_n_L2_optim` (ops/utils.py:29-44), which is also the order `tile_of` in csrc/gemm.hpp walks
inside one XCD's run of tiles.
"""

from __future__ import annotations

from typing import Tuple

import torch


def get_num_streaming_multiprocessors() -> int:
    """Compute units of GPU 0 (2 without a GPU, as the reference's debugging stand-in)."""
    if not torch.cuda.is_available():
        return 2
    return torch.cuda.get_device_properties(0).multi_processor_count


def map_pid_m_n(
    pid: int, M: int, N: int, block_m: int, block_n: int, group_m: int, optimize_L2: bool = True
) -> Tuple[int, int]:
    """Tile (row, column) of program `pid` over ceil(M/block_m) x ceil(N/block_n) tiles."""
    tiles_m = -(-M // block_m)
    tiles_n = -(-N // block_n)
    if not optimize_L2:
        return pid // tiles_n, pid % tiles_n
    in_group = group_m * tiles_n
    first_m = (pid // in_group) * group_m
    rows = min(group_m, tiles_m - first_m)
    r = pid % in_group
    return first_m + r % rows, r // rows
