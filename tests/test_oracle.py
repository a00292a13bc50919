"""Pins the CPU oracle (oracle/eager.py, oracle/philox.py, oracle/gated_mlp_ref.c) without a GPU.

The reference stores no vectors for this path (its tests compare fused and eager outputs live), so
each oracle function is pinned by independent restatements and by what the mathematics fixes.
"""

import math

import numpy as np
import pytest
import torch

from oracle import cref
from oracle import eager as oracle
from oracle import philox

torch.set_default_dtype(torch.float32)


def _rand_problem(M, K, N, bias, seed, dtype=torch.float64):
    g = torch.Generator().manual_seed(seed)
    r = lambda *s: torch.randn(*s, generator=g, dtype=dtype)
    t = dict(x=r(M, K), W_gate=0.5 * r(N, K), W_up=0.5 * r(N, K), W_down=0.5 * r(K, N), dY=r(M, K))
    t.update(b_gate=r(N) if bias else None, b_up=r(N) if bias else None, b_down=r(K) if bias else None)
    t["keep"] = (torch.rand(M, N, generator=g) > 0.3).to(torch.uint8)
    return t


def _args(t):
    return (t["x"], t["W_gate"], t["b_gate"], t["W_up"], t["b_up"], t["W_down"], t["b_down"])


def _loops_forward(t, p):
    """Brute force with Python loops and math.exp only."""
    x, Wg, bg, Wu, bu, Wd, bd = [None if v is None else v.tolist() for v in _args(t)]
    keep = t["keep"].tolist()
    M, K, N = len(x), len(x[0]), len(Wg)
    Y = [[0.0] * K for _ in range(M)]
    for m in range(M):
        h = []
        for n in range(N):
            g = sum(x[m][k] * Wg[n][k] for k in range(K)) + (bg[n] if bg else 0.0)
            u = sum(x[m][k] * Wu[n][k] for k in range(K)) + (bu[n] if bu else 0.0)
            v = g / (1.0 + math.exp(-g)) * u
            if p > 0:
                v = v / (1 - p) if keep[m][n] else 0.0
            h.append(v)
        for k in range(K):
            Y[m][k] = sum(h[n] * Wd[k][n] for n in range(N)) + (bd[k] if bd else 0.0)
    return torch.tensor(Y, dtype=torch.float64)


@pytest.mark.parametrize("bias", [False, True])
@pytest.mark.parametrize("p", [0.0, 0.3])
def test_forward_against_python_loops(bias, p):
    t = _rand_problem(3, 4, 5, bias, seed=1)
    ref = _loops_forward(t, p)
    got = oracle.forward(*_args(t), keep=t["keep"], p=p)["Y"]
    assert torch.allclose(got, ref, rtol=1e-12, atol=1e-12)


@pytest.mark.parametrize("bias", [False, True])
@pytest.mark.parametrize("p", [0.0, 0.25])
def test_forward_backward_against_numpy_and_c(bias, p):
    t = _rand_problem(7, 6, 9, bias, seed=2)
    got = oracle.backward(*_args(t), t["dY"], keep=t["keep"], p=p)
    # NumPy fp64 restatement written from the formula, not from the oracle's code
    x, Wg, bg, Wu, bu, Wd, bd = [None if v is None else v.numpy() for v in _args(t)]
    D = t["keep"].numpy() / (1 - p) if p > 0 else np.ones((7, 9))
    G = x @ Wg.T + (0 if bg is None else bg)
    U = x @ Wu.T + (0 if bu is None else bu)
    S = 1 / (1 + np.exp(-G))
    H = G * S * U * D
    Y = H @ Wd.T + (0 if bd is None else bd)
    dY = t["dY"].numpy()
    dA = (dY @ Wd) * D
    dU = dA * G * S
    dG = dA * U * (S * (1 + G * (1 - S)))
    exp = {"Y": Y, "H": H, "dX": dU @ Wu + dG @ Wg, "dW_gate": dG.T @ x, "dW_up": dU.T @ x, "dW_down": dY.T @ H}
    if bias:
        exp.update(db_gate=dG.sum(0), db_up=dU.sum(0), db_down=dY.sum(0))
    for k, v in exp.items():
        assert np.allclose(got[k].numpy(), v, rtol=1e-11, atol=1e-11), k
    # plain-C restatement (scalar loops)
    c = cref.backward(x, Wg, bg, Wu, bu, Wd, bd, dY, keep=t["keep"].numpy(), p=p)
    for k in exp:
        assert np.allclose(c[k], got[k].numpy(), rtol=1e-11, atol=1e-11), k


@pytest.mark.parametrize("bias", [False, True])
def test_backward_against_autograd_and_gradcheck(bias):
    t = _rand_problem(5, 4, 6, bias, seed=3)
    p = 0.3
    leaves = {k: (None if v is None else v.clone().requires_grad_(True)) for k, v in t.items() if k not in ("dY", "keep")}
    y = oracle.forward(leaves["x"], leaves["W_gate"], leaves["b_gate"], leaves["W_up"], leaves["b_up"],
                       leaves["W_down"], leaves["b_down"], keep=t["keep"], p=p)["Y"]
    names = [k for k, v in leaves.items() if v is not None]
    grads = torch.autograd.grad(y, [leaves[k] for k in names], grad_outputs=t["dY"])
    got = oracle.backward(*_args(t), t["dY"], keep=t["keep"], p=p)
    key = {"x": "dX", "W_gate": "dW_gate", "W_up": "dW_up", "W_down": "dW_down", "b_gate": "db_gate", "b_up": "db_up",
           "b_down": "db_down"}
    for n, g in zip(names, grads):
        assert torch.allclose(got[key[n]], g, rtol=1e-11, atol=1e-11), n
    f = lambda x, wg, wu, wd: oracle.forward(x, wg, t["b_gate"], wu, t["b_up"], wd, t["b_down"], t["keep"], p)["Y"]
    ins = [t[k].clone().requires_grad_(True) for k in ("x", "W_gate", "W_up", "W_down")]
    assert torch.autograd.gradcheck(f, ins, eps=1e-6, atol=1e-6)


def test_module_form_matches_functional_and_torch_layers():
    torch.manual_seed(0)
    m = oracle.OracleGatedMLP(8, 12, bias=True).double()
    x = torch.randn(2, 3, 8, dtype=torch.float64)
    y = m(x)
    ref = oracle.forward(x.view(-1, 8), m.gate_proj.weight, m.gate_proj.bias, m.up_proj.weight, m.up_proj.bias,
                         m.down_proj.weight, m.down_proj.bias)["Y"]
    assert torch.allclose(y.view(-1, 8), ref, rtol=1e-13, atol=1e-13)
    assert [n for n, _ in m.named_parameters()] == [
        "gate_proj.weight", "gate_proj.bias", "up_proj.weight", "up_proj.bias", "down_proj.weight", "down_proj.bias"]


def test_silu_known_values_and_derivative():
    x = torch.tensor([0.0, 1.0, -1.0, 20.0, -20.0], dtype=torch.float64)
    assert torch.allclose(oracle.silu(x)[:2], torch.tensor([0.0, 0.7310585786300049], dtype=torch.float64), atol=1e-12)
    assert torch.allclose(oracle.silu_grad(x)[:2], torch.tensor([0.5, 0.9276705118714869], dtype=torch.float64), atol=1e-12)
    assert torch.allclose(oracle.silu(x), torch.nn.functional.silu(x), atol=1e-12)
    xs = torch.linspace(-6, 6, 101, dtype=torch.float64)
    h = 1e-6
    fd = (oracle.silu(xs + h) - oracle.silu(xs - h)) / (2 * h)
    assert torch.allclose(oracle.silu_grad(xs), fd, atol=1e-8)
    xa = xs.clone().requires_grad_(True)
    (ga,) = torch.autograd.grad(torch.nn.functional.silu(xa).sum(), xa)
    assert torch.allclose(oracle.silu_grad(xs), ga, atol=1e-12)


TORCH_ACT = {
    "silu": torch.nn.functional.silu,
    "swish": torch.nn.functional.silu,
    "gelu": torch.nn.functional.gelu,
    "relu": torch.nn.functional.relu,
    "leaky_relu": torch.nn.functional.leaky_relu,
    "sigmoid": torch.sigmoid,
    "tanh": torch.tanh,
    "no_act": lambda v: v,
}
# act(1), act(-1), act'(1), act'(-1) from the definitions: Phi(1) = 0.841344746..., phi(1) = 0.241970724...
ACT_TABLE = {
    "gelu": (0.8413447460685429, -0.15865525393145707, 1.0833154705876864, -0.08331547058768629),
    "relu": (1.0, 0.0, 1.0, 0.0),
    "leaky_relu": (1.0, -0.01, 1.0, 0.01),
    "sigmoid": (0.7310585786300049, 0.2689414213699951, 0.19661193324148185, 0.19661193324148185),
    "tanh": (0.7615941559557649, -0.7615941559557649, 0.41997434161402614, 0.41997434161402614),
    "no_act": (1.0, -1.0, 1.0, 1.0),
}


@pytest.mark.parametrize("act", sorted(TORCH_ACT))
def test_activation_table_against_torch_autograd_and_central_differences(act):
    f, df = oracle.ACTS[act]
    xs = torch.cat([torch.linspace(-6, 6, 101, dtype=torch.float64), torch.tensor([0.0], dtype=torch.float64)])
    xa = xs.clone().requires_grad_(True)
    ya = TORCH_ACT[act](xa)
    (ga,) = torch.autograd.grad(ya.sum(), xa)
    assert torch.allclose(f(xs), ya.detach(), atol=1e-12), "forward differs from torch.nn.functional"
    assert torch.allclose(df(xs), ga, atol=1e-12), "derivative differs from torch.autograd (kinks included)"
    smooth = xs[xs.abs() > 1e-3]  # central differences away from the kink at 0
    h = 1e-6
    assert torch.allclose(df(smooth), (f(smooth + h) - f(smooth - h)) / (2 * h), atol=1e-8)
    if act in ACT_TABLE:
        one = torch.tensor([1.0, -1.0], dtype=torch.float64)
        exp = torch.tensor(ACT_TABLE[act], dtype=torch.float64)
        assert torch.allclose(torch.cat([f(one), df(one)]), exp, atol=1e-12)


@pytest.mark.parametrize("act", ["gelu", "relu", "leaky_relu", "sigmoid", "tanh", "no_act"])
def test_other_activations_full_path_against_autograd_and_c(act):
    t = _rand_problem(5, 4, 6, True, seed=11)
    p = 0.25
    leaves = {k: v.clone().requires_grad_(True) for k, v in t.items() if k not in ("dY", "keep")}
    g = torch.nn.functional.linear(leaves["x"], leaves["W_gate"], leaves["b_gate"])
    u = torch.nn.functional.linear(leaves["x"], leaves["W_up"], leaves["b_up"])
    h = TORCH_ACT[act](g) * u * t["keep"].to(torch.float64) / (1 - p)
    y = torch.nn.functional.linear(h, leaves["W_down"], leaves["b_down"])
    names = list(leaves)
    grads = torch.autograd.grad(y, [leaves[k] for k in names], grad_outputs=t["dY"])
    got = oracle.backward(*_args(t), t["dY"], keep=t["keep"], p=p, act=act)
    key = {"x": "dX", "W_gate": "dW_gate", "W_up": "dW_up", "W_down": "dW_down", "b_gate": "db_gate", "b_up": "db_up",
           "b_down": "db_down"}
    assert torch.allclose(got["Y"], y.detach(), rtol=1e-12, atol=1e-12)
    for n, gr in zip(names, grads):
        assert torch.allclose(got[key[n]], gr, rtol=1e-11, atol=1e-11), n
    x, Wg, bg, Wu, bu, Wd, bd = [v.numpy() for v in _args(t)]
    c = cref.backward(x, Wg, bg, Wu, bu, Wd, bd, t["dY"].numpy(), keep=t["keep"].numpy(), p=p, act=act)
    for k in ("Y", "H", "dX", "dW_gate", "dW_up", "dW_down", "db_gate", "db_up", "db_down"):
        assert np.allclose(c[k], got[k].numpy(), rtol=1e-11, atol=1e-11), k


def test_algebraic_special_cases():
    t = _rand_problem(6, 5, 7, True, seed=4)
    a = list(_args(t))
    # zero gate weights and gate bias: silu(0) = 0, so Y = b_down
    z = list(a)
    z[1], z[2] = torch.zeros_like(a[1]), torch.zeros_like(a[2])
    assert torch.allclose(oracle.forward(*z)["Y"], a[6].expand(6, 5), atol=1e-14)
    # x = 0 without biases: Y = 0
    assert not oracle.forward(torch.zeros(6, 5, dtype=torch.float64), a[1], None, a[3], None, a[5], None)["Y"].any()
    # linear in W_up and in W_down (no biases)
    y1 = oracle.forward(a[0], a[1], None, a[3], None, a[5], None)["Y"]
    assert torch.allclose(oracle.forward(a[0], a[1], None, 3 * a[3], None, a[5], None)["Y"], 3 * y1, rtol=1e-12)
    assert torch.allclose(oracle.forward(a[0], a[1], None, a[3], None, -2 * a[5], None)["Y"], -2 * y1, rtol=1e-12)
    # large positive gate: silu(g) -> g
    big = oracle.forward(a[0], a[1], 50 + torch.zeros(7, dtype=torch.float64), a[3], None, a[5], None)
    G = a[0] @ a[1].T + 50
    assert torch.allclose(big["H"], G * (a[0] @ a[3].T), rtol=1e-12)
    # keep = all ones with p: plain scaling by 1/(1-p); keep = zeros: Y = b_down
    ones = torch.ones(6, 7, dtype=torch.uint8)
    assert torch.allclose(oracle.forward(*a, keep=ones, p=0.5)["H"], 2 * oracle.forward(*a)["H"], rtol=1e-13)
    assert torch.allclose(oracle.forward(*a, keep=0 * ones, p=0.5)["Y"], a[6].expand(6, 5), atol=1e-14)


# ------------------------------------------------------------------ Philox / dropout mask

KAT = [  # Random123 kat_vectors, philox4x32 10 rounds: counter, key, expected
    ([0, 0, 0, 0], [0, 0], [0x6627E8D5, 0xE169C58D, 0xBC57AC4C, 0x9B00DBD8]),
    ([0xFFFFFFFF] * 4, [0xFFFFFFFF] * 2, [0x408F276D, 0x41C83B0E, 0xA20BC7C6, 0x6D5451FD]),
    ([0x243F6A88, 0x85A308D3, 0x13198A2E, 0x03707344], [0xA4093822, 0x299F31D0],
     [0xD16CFE09, 0x94FDCCEB, 0x5001E420, 0x24126EA1]),
]


@pytest.mark.parametrize("ctr,key,exp", KAT)
def test_philox_known_answers(ctr, key, exp):
    got = philox.philox4x32_10(np.array(ctr, dtype=np.uint32), np.array(key, dtype=np.uint32))
    assert [int(v) for v in got] == exp
    assert cref.philox4x32_10(ctr, key) == exp


def test_philox_numpy_matches_c_on_random_counters():
    rng = np.random.default_rng(0)
    ctr = rng.integers(0, 2**32, size=(200, 4), dtype=np.uint64).astype(np.uint32)
    key = rng.integers(0, 2**32, size=(200, 2), dtype=np.uint64).astype(np.uint32)
    got = philox.philox4x32_10(ctr, key)
    for i in range(200):
        assert [int(v) for v in got[i]] == cref.philox4x32_10(ctr[i], key[i])


@pytest.mark.parametrize("M,N,p,seed,offset", [(5, 8, 0.5, 1, 0), (33, 72, 0.1, 2**40 + 17, 3), (64, 128, 0.9, 7, 2**33 + 1)])
def test_keep_mask_numpy_matches_c(M, N, p, seed, offset):
    a = philox.keep_mask(M, N, p, seed, offset)
    b = cref.keep_mask(M, N, philox.threshold(p), seed, offset)
    assert np.array_equal(a, b)


def test_keep_mask_statistics_and_edge_probabilities():
    assert philox.keep_mask(16, 16, 0.0, 5).all()
    for p in (0.1, 0.5, 0.75):
        m = philox.keep_mask(512, 1024, p, seed=42)
        n = m.size
        assert abs(m.mean() - (1 - p)) < 5 * math.sqrt(p * (1 - p) / n)
        # different seed / offset give different, equally distributed masks
        m2 = philox.keep_mask(512, 1024, p, seed=43)
        m3 = philox.keep_mask(512, 1024, p, seed=42, offset=1)
        assert (m != m2).mean() > 0.5 * 2 * p * (1 - p) and (m != m3).mean() > 0.5 * 2 * p * (1 - p)
    assert philox.threshold(0.1) == 429496736  # float32(0.1) * 2^32, floored
    assert philox.threshold(0.5) == 2**31


# ------------------------------------------------------------------ golden fixture (config 1)


def test_cfg1_golden_fixture():
    """Config 1 (fp32 CPU, M=128 K=512 N=256, bias=False, x ~ U[0,1), seed 0): the oracle must
    reproduce the committed fixture written by tests/golden/make_cfg1.py."""
    from golden import make_cfg1

    fx = np.load(make_cfg1.FIXTURE)
    out = make_cfg1.compute()
    assert out["y_strided"].shape == fx["y_strided"].shape
    assert np.allclose(out["y_strided"], fx["y_strided"], rtol=1e-5, atol=1e-6)
    assert abs(out["y_sum"] - fx["y_sum"]) < 1e-3 * abs(fx["y_sum"]) + 1e-3
    assert np.allclose(out["x_head"], fx["x_head"]) and np.allclose(out["w_gate_head"], fx["w_gate_head"])
