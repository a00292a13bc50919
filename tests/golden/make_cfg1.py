"""Writes tests/golden/cfg1.npz: config 1 of the baseline (CPU eager gated MLP, fp32, M=128,
K=512, N=256, bias=False, dropout_p=0, x ~ U[0,1) with torch.rand, nn.Linear default
Kaiming-uniform weights, seed 0, forward only).

Convention (the baseline does not fix the order of seeding): torch.manual_seed(0), construct the
three nn.Linear layers in the order gate, up, down (EagerGatedMLP.__init__,
src/triton_gated_mlp/gated_mlp.py:85-87), then torch.manual_seed(0) again and x = torch.rand(128, 512).
The fixture holds a strided slice of Y, its sum, and the first values of x and W_gate (to detect a
change in torch's generator or init).  Produced by this repository's own oracle; the reference
package is not importable here and is not needed for it.

Run:  python tests/golden/make_cfg1.py
"""

from pathlib import Path

import numpy as np
import torch

FIXTURE = Path(__file__).resolve().parent / "cfg1.npz"


def compute():
    import sys

    sys.path.insert(0, str(Path(__file__).resolve().parent.parent.parent))
    from oracle import eager as oracle

    torch.manual_seed(0)
    m = oracle.OracleGatedMLP(hidden_size=512, intermediate_size=256, bias=False, dropout_p=0.0).float()
    torch.manual_seed(0)
    x = torch.rand(128, 512)
    with torch.no_grad():
        y = m(x)
    return {
        "y_strided": y[::16, ::64].numpy().copy(),
        "y_sum": np.float64(y.double().sum().item()),
        "x_head": x[0, :8].numpy().copy(),
        "w_gate_head": m.gate_proj.weight[0, :8].detach().numpy().copy(),
    }


if __name__ == "__main__":
    np.savez(FIXTURE, **compute())
    print("wrote", FIXTURE)
