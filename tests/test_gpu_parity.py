"""Parity of the HIP path (through the C ABI) against the CPU oracle on identical seeded inputs.

Tolerance, one rule for every comparison in this file (`_close`): rtol = 2e-2 element-wise against the
reference evaluated in fp32 on the same (already rounded) inputs, atol = 2e-2 * max(1, mean|ref|), and a
relative Frobenius error below 1e-2.  The absolute term follows the magnitude of the tensor because
an element's rounding error is set by the size of the terms that were summed (which is what
mean|ref| measures), not by the element's own value: an element of a weight gradient that happens
to come out near zero from 8192 products of size 1 cannot be held to 2e-2 of itself.  For outputs
of typical size below one (Y, dX, G, U, H, dG, dU with the stated input distributions) the rule is
the plain rtol = atol = 2e-2.  `test_cfg3_fp16_forward_backward_llama3_8b` holds the rule against a
yardstick: torch's own fp16 module on the same inputs against the same oracle.
"""

import contextlib

import numpy as np
import pytest
import torch

from cases import CFG2, CFG3, CFG4, CFG5, Case, make_inputs
from oracle import eager as oracle
from oracle import philox

pytestmark = pytest.mark.gpu

RTOL = ATOL = 2e-2


def _dev():
    assert torch.cuda.is_available(), "GPU tests need a visible AMD GPU"
    return torch.device("cuda", 0)


def _close(name, got, ref):
    got = got.detach().float().cpu()
    ref = ref.detach().float().cpu()
    assert got.shape == ref.shape, f"{name}: shape {tuple(got.shape)} vs {tuple(ref.shape)}"
    assert torch.isfinite(got).all(), f"{name}: non-finite values"
    err = (got - ref).abs()
    atol = ATOL * max(1.0, ref.abs().mean().item() if ref.numel() else 0.0)
    bad = err > atol + RTOL * ref.abs()
    rel_fro = ((got - ref).norm() / ref.norm().clamp_min(1e-30)).item()
    # elements outside the plain band, whatever the magnitude of the tensor scaled the absolute term to
    plain = int((err > ATOL + RTOL * ref.abs()).sum()) if err.numel() else 0
    print(
        f"  {name}: max_abs_err={err.max().item() if err.numel() else 0.0:.3e} rel_fro={rel_fro:.3e} "
        f"atol={atol:.3g} outside_plain_{RTOL:g}_{ATOL:g}_band={plain}/{err.numel()}",
        flush=True,
    )
    assert not bad.any(), (
        f"{name}: {int(bad.sum())} of {bad.numel()} elements outside rtol={RTOL}, atol={atol:.3g}; "
        f"max_abs_err={err.max().item():.4e}, rel_fro={rel_fro:.3e}"
    )
    assert rel_fro < 1e-2, f"{name}: relative Frobenius error {rel_fro:.3e}"


def _oracle_inputs(t):
    return {k: (None if v is None else v.float()) for k, v in t.items()}


def _run_module_case(c: Case, lean: bool = False, yardstick: bool = False):
    from triton_gated_mlp import FusedGatedMLP
    from triton_gated_mlp.ops import fwd as ops_fwd

    dev = _dev()
    print(f"case {c.name}: M={c.M} K={c.K} N={c.N} dtype={c.dtype} bias={c.bias} p={c.p} act={c.act}", flush=True)
    t = make_inputs(c)
    mlp = FusedGatedMLP(hidden_size=c.K, intermediate_size=c.N, bias=c.bias, dropout_p=c.p, hidden_act=c.act)
    mlp = mlp.to(dev).to(c.dtype)
    with torch.no_grad():
        mlp.gate_proj.weight.copy_(t["W_gate"])
        mlp.up_proj.weight.copy_(t["W_up"])
        mlp.down_proj.weight.copy_(t["W_down"])
        if c.bias:
            mlp.gate_proj.bias.copy_(t["b_gate"])
            mlp.up_proj.bias.copy_(t["b_up"])
            mlp.down_proj.bias.copy_(t["b_down"])
    mlp.train(c.p > 0.0)
    mlp.dropout_seed = c.dropout_seed
    mlp.recompute_activations = lean
    x = t["x"].to(dev).requires_grad_(c.backward)

    with contextlib.nullcontext() if c.backward else torch.no_grad():
        y = mlp(x)
    keep = None
    if c.p > 0.0:
        # one mask per row chunk the module ran (a single one unless the batch was split)
        states = mlp.last_dropout_states
        assert states and states[0][0] == 0 and sum(s[1] for s in states) == c.M
        assert mlp.last_dropout_state == states[-1][2:]
        parts = []
        for row0, rows, seed, offset in states:
            keep_dev = ops_fwd.dropout_mask(rows, c.N, c.p, seed, offset, device=dev)
            keep_np = philox.keep_mask(rows, c.N, c.p, seed, offset)
            assert np.array_equal(keep_dev.cpu().numpy(), keep_np), "device keep mask differs from the NumPy Philox oracle"
            parts.append(keep_np)
        keep = torch.from_numpy(np.concatenate(parts, axis=0))

    o = _oracle_inputs(t)
    if not c.backward:
        ref = oracle.forward(
            o["x"], o["W_gate"], o["b_gate"], o["W_up"], o["b_up"], o["W_down"], o["b_down"], keep, c.p, c.act
        )
        _close("Y", y, ref["Y"])
        return
    grads_in = [x, mlp.gate_proj.weight, mlp.up_proj.weight, mlp.down_proj.weight]
    names = ["dX", "dW_gate", "dW_up", "dW_down"]
    if c.bias:
        grads_in += [mlp.gate_proj.bias, mlp.up_proj.bias, mlp.down_proj.bias]
        names += ["db_gate", "db_up", "db_down"]
    grads = torch.autograd.grad(y, grads_in, grad_outputs=t["dY"].to(dev))
    ref = oracle.backward(
        o["x"], o["W_gate"], o["b_gate"], o["W_up"], o["b_up"], o["W_down"], o["b_down"], o["dY"], keep, c.p, c.act
    )
    _close("Y", y, ref["Y"])
    for n, g in zip(names, grads):
        _close(n, g, ref[n])
    if yardstick:
        from triton_gated_mlp import EagerGatedMLP, copy_weights

        eager = EagerGatedMLP(hidden_size=c.K, intermediate_size=c.N, bias=c.bias, dropout_p=0.0, hidden_act=c.act)
        eager = eager.to(dev).to(c.dtype)
        copy_weights(mlp, eager)
        xe = t["x"].to(dev).requires_grad_(True)
        ge = torch.autograd.grad(eager(xe), [xe, eager.gate_proj.weight, eager.up_proj.weight, eager.down_proj.weight],
                                 grad_outputs=t["dY"].to(dev))
        for n, g_fused, g_eager in zip(names[:4], grads[:4], ge):
            r = ref[n]
            band = ATOL + RTOL * r.abs()
            e_f, e_e = (g_fused.float().cpu() - r).abs(), (g_eager.float().cpu() - r).abs()
            out_f, out_e = int((e_f > band).sum()), int((e_e > band).sum())
            print(f"  yardstick {n}: outside plain band fused {out_f}, torch fp16 {out_e} of {r.numel()}; "
                  f"max_abs_err fused {e_f.max().item():.3e}, torch fp16 {e_e.max().item():.3e}", flush=True)
            assert out_f <= 1.5 * out_e + 1000, f"{n}: the fused path leaves the plain band far more often than torch's fp16 path"
            assert e_f.max().item() <= 2.0 * e_e.max().item() + ATOL


def test_cfg2_fp16_forward_llama7b():
    _run_module_case(CFG2)


def test_cfg3_fp16_forward_backward_llama3_8b():
    """The headline configuration at full size.  Also the yardstick for the weight-gradient tolerance
    (atol = 2e-2 * max(1, mean|ref|)): an element of dW sums M = 8192 products of operands that were
    themselves rounded to fp16 on the way (dG, dU, H), so its error has an absolute size set by the
    typical magnitude of dW (tens), whatever the element's own value, and elements far below typical
    cannot meet a bound relative to themselves.  torch's own fp16 module (EagerGatedMLP on the GPU,
    hipBLASLt GEMMs) is run on the same inputs: against the same fp32 oracle it leaves the plain
    2e-2/2e-2 band for about as many elements, and the fused gradients are as close as torch's."""
    _run_module_case(CFG3, yardstick=True)


def test_cfg4_bf16_bias_dropout_forward_backward():
    _run_module_case(CFG4)


def test_cfg5_fp16_decode_forward():
    _run_module_case(CFG5)


def test_cfg1_fp32_forward_against_golden_fixture():
    """Baseline configuration 1 (fp32, M=128, K=512, N=256, bias=False, x ~ U[0,1) from torch.rand,
    nn.Linear default init, seed 0; EagerGatedMLP.forward, src/triton_gated_mlp/gated_mlp.py:92-98)
    through FusedGatedMLP on the float32 HIP path, against the committed fixture and the oracle.
    Inputs are built exactly as tests/golden/make_cfg1.py builds them."""
    from golden import make_cfg1
    from triton_gated_mlp import FusedGatedMLP, copy_weights

    dev = _dev()
    torch.manual_seed(0)
    ref_mod = oracle.OracleGatedMLP(hidden_size=512, intermediate_size=256, bias=False, dropout_p=0.0).float()
    torch.manual_seed(0)
    x = torch.rand(128, 512)
    fix = np.load(make_cfg1.FIXTURE)
    assert np.array_equal(fix["x_head"], x[0, :8].numpy()), "torch's generator changed: regenerate the fixture"
    assert np.array_equal(fix["w_gate_head"], ref_mod.gate_proj.weight[0, :8].detach().numpy())
    fused = FusedGatedMLP(hidden_size=512, intermediate_size=256, bias=False, dropout_p=0.0).float()
    copy_weights(ref_mod, fused)
    fused = fused.to(dev)
    with torch.no_grad():
        y = fused(x.to(dev)).cpu()
        y_ref = ref_mod(x)
    assert y.dtype == torch.float32 and y.shape == (128, 512)
    # fp32 operands, fp32 accumulation on both sides: only the summation order differs
    assert torch.allclose(y, y_ref, rtol=1e-4, atol=1e-5), f"max abs err {(y - y_ref).abs().max().item():.3e}"
    np.testing.assert_allclose(y[::16, ::64].numpy(), fix["y_strided"], rtol=1e-4, atol=1e-5)
    np.testing.assert_allclose(y.double().sum().item(), float(fix["y_sum"]), rtol=1e-5)
    print(f"  cfg1: max_abs_err={(y - y_ref).abs().max().item():.3e}", flush=True)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize(
    "M,K,N,bias,p",
    [
        (128, 256, 512, True, 0.0),  # the reference's module test shape (tests/test_gated_mlp_fwd.py:23-38)
        (512, 256, 512, False, 0.0),  # 3-D input case B=16, M=32 (tests/test_gated_mlp_bwd.py:27-45)
        (64, 256, 512, False, 0.0),  # B,M,N,K = 2,32,512,256 (tests/test_gated_mlp_bwd.py:97)
        (200, 136, 264, True, 0.25),  # ragged: nothing a multiple of the tile
        (1, 64, 128, True, 0.0),
        (256, 512, 1024, True, 0.5),
        (768, 1024, 2048, False, 0.0),
    ],
)
def test_small_shapes_forward_backward(M, K, N, bias, p, dtype):
    _run_module_case(Case(f"small_{M}x{K}x{N}", M, K, N, dtype, bias=bias, p=p, backward=True, seed=M + K + N))


@pytest.mark.parametrize(
    "M,K,N,dtype,bias,p",
    [
        (3001, 2048, 4096, torch.float16, False, 0.0),  # odd token count on the 256-tile and 128-tile kernels
        (1000, 1024, 4104, torch.bfloat16, True, 0.1),  # ragged tokens and ragged intermediate size
        (50, 512, 1024, torch.float16, True, 0.0),  # fewer rows than one tile
        (4099, 1024, 2048, torch.float16, False, 0.0),  # three rows into the last tile-row
    ],
)
def test_ragged_token_counts_on_the_pipelined_kernels(M, K, N, dtype, bias, p):
    """Token counts (and intermediate sizes) that are not multiples of the tile run on the same
    kernels as whole tiles: the part of a tile beyond the end of an operand reads as zero.  The
    weight gradients reduce over the ragged dimension."""
    _run_module_case(Case(f"ragged_{M}x{K}x{N}", M, K, N, dtype, bias=bias, p=p, backward=True, seed=M))


@pytest.mark.parametrize(
    "M,K,N,dtype,bias",
    [
        (17, 2048, 8192, torch.float16, True),  # one more row than the skinny-M kernels take
        (64, 1024, 4096, torch.float16, False),
        (300, 1024, 4096, torch.bfloat16, True),
        (130, 4096, 14336, torch.float16, False),  # Llama-3-8B widths, short batch
        (40, 1024, 4160, torch.float16, False),  # 130 reduction tiles for dX do not divide by 16 splits
        (100, 5120, 13824, torch.float16, True),  # Llama-2-13B widths: the gate/up GEMM splits as well
    ],
)
def test_short_batches_split_the_long_reductions(M, K, N, dtype, bias):
    """Down projection and input gradient of a short batch have a few output tiles and a long
    reduction; the library asks for a workspace and splits the reduction over several workgroups
    per tile.  Same results as ever, to the usual tolerance."""
    from triton_gated_mlp import _cabi

    code = _cabi.dtype_code(dtype)
    assert _cabi.lib().gmlp_workspace_bytes(_cabi.GMLP_OP_LINEAR_FWD, M, N, K, code) > 0
    assert _cabi.lib().gmlp_workspace_bytes(_cabi.GMLP_OP_DX_BWD, M, K, N, code) > 0
    if N == 13824:
        assert _cabi.lib().gmlp_workspace_bytes(_cabi.GMLP_OP_GATEUP_FWD, M, K, N, code) > 0
    _run_module_case(Case(f"short_{M}x{K}x{N}", M, K, N, dtype, bias=bias, p=0.0, backward=True, seed=M + 1))


def test_split_reduction_without_workspace_gives_the_unsplit_result():
    """NULL workspace is always accepted: one workgroup per tile, same numbers up to summation order."""
    from triton_gated_mlp import _cabi
    from triton_gated_mlp.ops import fwd as ops_fwd

    dev = _dev()
    g = torch.Generator().manual_seed(5)
    a = torch.randn(48, 8192, generator=g).to(torch.float16).to(dev)
    W = (0.02 * torch.randn(1024, 8192, generator=g)).to(torch.float16).to(dev)
    split = ops_fwd.linear_fwd(a, W)
    plain = torch.empty_like(split)
    _cabi.check(_cabi.lib().gmlp_linear_fwd(a.data_ptr(), W.data_ptr(), None, plain.data_ptr(), 48, 8192, 1024, 0,
                                            None, 0, _cabi.stream_ptr(dev)))
    ref = a.float().cpu() @ W.float().cpu().T
    _close("split", split, ref)
    _close("plain", plain, ref)
    assert (split.float() - plain.float()).abs().max().item() < 1e-2


OTHER_ACTS = ["gelu", "relu", "leaky_relu", "sigmoid", "tanh", "no_act"]


@pytest.mark.parametrize("act", OTHER_ACTS)
def test_other_activations_forward_backward(act):
    """hidden_act beyond silu (the reference's ACT_FWD table, src/triton_gated_mlp/gated_mlp.py:28-37):
    full-tile kernels, bias, dropout; fp16."""
    _run_module_case(Case(f"act_{act}", 384, 256, 640, torch.float16, bias=True, p=0.1, backward=True, seed=21, act=act))


@pytest.mark.parametrize("act,dtype", [("gelu", torch.bfloat16), ("relu", torch.bfloat16), ("tanh", torch.float32)])
def test_other_activations_ragged_shapes_and_dtypes(act, dtype):
    _run_module_case(Case(f"act_{act}_ragged", 200, 136, 264, dtype, bias=True, p=0.25, backward=True, seed=22, act=act))


@pytest.mark.parametrize("act", OTHER_ACTS)
def test_other_activations_decode_path(act):
    """The weight-streaming kernels for M <= 16 (both variants: K % 256 == 0 and not), called directly:
    the module only routes to them for widths that fill the chip."""
    from triton_gated_mlp.ops import fwd as ops_fwd

    dev = _dev()
    for c in (
        Case(f"act_{act}_decode", 8, 1024, 1536, torch.float16, bias=True, seed=23, act=act),
        Case(f"act_{act}_decode_generic", 16, 96, 512, torch.float16, bias=False, seed=24, act=act),
    ):
        t = make_inputs(c)
        d = {k: (None if v is None else v.to(dev)) for k, v in t.items()}
        y = ops_fwd.decode_fwd(d["x"], d["W_gate"], d["b_gate"], d["W_up"], d["b_up"], d["W_down"], d["b_down"], act)
        o = _oracle_inputs(t)
        ref = oracle.forward(o["x"], o["W_gate"], o["b_gate"], o["W_up"], o["b_up"], o["W_down"], o["b_down"], act=act)
        _close(f"{c.name} Y", y, ref["Y"])


@pytest.mark.parametrize("act", ["gelu", "no_act"])
def test_other_activations_operator_level(act):
    """mlp_hidden_states_fwd / _bwd with act_fn, the reference operator signatures
    (src/triton_gated_mlp/ops/fwd.py:198-206, ops/bwd.py:466-468).  The reference's no_act backward
    multiplies by G instead of 1 (_act_bwd, ops/act.py:15-18); the true derivative is checked here."""
    from triton_gated_mlp import mlp_hidden_states_bwd, mlp_hidden_states_fwd

    dev = _dev()
    c = Case(f"op_{act}", 256, 128, 384, torch.float16, backward=True, seed=25, act=act)
    t = make_inputs(c)
    g = torch.Generator().manual_seed(26)
    dH = torch.randn(c.M, c.N, generator=g).to(c.dtype)
    x, Wu, Wg = t["x"].to(dev), t["W_up"].to(dev), t["W_gate"].to(dev)
    h = mlp_hidden_states_fwd(x, Wu, None, Wg, None, act, 0.0)
    dx, dWu, dWg = mlp_hidden_states_bwd(x, Wu, Wg, dH.to(dev), act_fn=act)
    o = _oracle_inputs(t)
    f = oracle.hidden_forward(o["x"], o["W_gate"], None, o["W_up"], None, act=act)
    hb = oracle.hidden_backward(dH.float(), f["G"], f["U"], act=act)
    _close("H", h, f["H"])
    _close("dX", dx, hb["dU"] @ o["W_up"] + hb["dG"] @ o["W_gate"])
    _close("dW_up", dWu, hb["dU"].T @ o["x"])
    _close("dW_gate", dWg, hb["dG"].T @ o["x"])


def test_device_activation_functions_against_float64_closed_forms():
    """The kernels evaluate erf and tanh through short fp32 approximations; this pins them far below
    the storage tolerance.  gating_bwd in float32 with dH = U = 1 returns act(G) as dU and act'(G) as
    dG, compared with scipy / numpy in float64 on a dense grid that includes both tails and 0."""
    from scipy.special import erf, expit

    from triton_gated_mlp.ops import bwd as ops_bwd

    dev = _dev()
    x32 = torch.linspace(-12.0, 12.0, 64 * 4096, dtype=torch.float32).reshape(64, 4096).clone()
    x32[0, :2] = torch.tensor([0.0, -0.0])
    x = x32.double().numpy()
    cdf, pdf = 0.5 * (1.0 + erf(x / np.sqrt(2.0))), np.exp(-0.5 * x * x) / np.sqrt(2.0 * np.pi)
    closed = {
        "silu": (x * expit(x), expit(x) * (1.0 + x * (1.0 - expit(x)))),
        "gelu": (x * cdf, cdf + x * pdf),
        "sigmoid": (expit(x), expit(x) * (1.0 - expit(x))),
        "tanh": (np.tanh(x), 1.0 - np.tanh(x) ** 2),
    }
    one = torch.ones_like(x32).to(dev)
    for act, (f, df) in closed.items():
        dg, du = ops_bwd.gating_bwd(one, x32.to(dev), one, 0.0, 0, 0, act)
        err_f = np.abs(du.cpu().double().numpy() - f).max()
        err_d = np.abs(dg.cpu().double().numpy() - df).max()
        assert err_f < 2e-6 and err_d < 2e-6, (act, err_f, err_d)  # |x| <= 12: a few fp32 ulps of the value
    # tanh keeps its relative accuracy through 0 (no 1 - e^{-2x} cancellation)
    tiny = torch.logspace(-6, -1, 4096, dtype=torch.float32).reshape(1, -1)
    _, du = ops_bwd.gating_bwd(torch.ones_like(tiny).to(dev), tiny.to(dev), torch.ones_like(tiny).to(dev), 0.0, 0, 0, "tanh")
    rel = np.abs(du.cpu().double().numpy() / np.tanh(tiny.double().numpy()) - 1.0).max()
    assert rel < 1e-6, rel


def test_three_dimensional_input_matches_flattened():
    """[B, S, K] input gives the 2-D result on x.view(-1, K) (tests/test_gated_mlp_bwd.py:37-45)."""
    from triton_gated_mlp import FusedGatedMLP

    dev = _dev()
    torch.manual_seed(0)
    mlp = FusedGatedMLP(256, 512, bias=False).to(dev).to(torch.float16)
    x = torch.rand(16, 32, 256, device=dev, dtype=torch.float16)
    y3 = mlp(x)
    y2 = mlp(x.view(-1, 256))
    assert y3.shape == x.shape
    assert torch.equal(y3.view(-1, 256), y2)


def test_operator_level_fwd_bwd_match_closed_form():
    """mlp_hidden_states_fwd/bwd against the closed form (pattern of tests/test_gated_mlp_bwd.py:89-129)."""
    from triton_gated_mlp import mlp_hidden_states_bwd, mlp_hidden_states_fwd

    dev = _dev()
    g = torch.Generator().manual_seed(7)
    BM, N, K = 64, 512, 256
    x = torch.rand(BM, K, generator=g).half()
    W_up = (torch.rand(N, K, generator=g) / 8).half()
    W_gp = (torch.rand(N, K, generator=g) / 8).half()
    dH = torch.rand(BM, N, generator=g).half()
    h = mlp_hidden_states_fwd(x.to(dev), W_up.to(dev), None, W_gp.to(dev), None, "silu", 0.0)
    ref = oracle.hidden_forward(x.float(), W_gp.float(), None, W_up.float(), None)
    _close("hidden", h, ref["H"])
    dx, dW_up, dW_gp = mlp_hidden_states_bwd(x.to(dev), W_up.to(dev), W_gp.to(dev), dH.to(dev))
    hb = oracle.hidden_backward(dH.float(), ref["G"], ref["U"])
    _close("dx", dx, hb["dU"] @ W_up.float() + hb["dG"] @ W_gp.float())
    _close("dW_up", dW_up, hb["dU"].T @ x.float())
    _close("dW_gp", dW_gp, hb["dG"].T @ x.float())


def test_autograd_function_reference_signature():
    """FusedGatedMLPFunction.apply(x, W_up, b_up, W_gp, b_gp) with biases and bias gradients."""
    from triton_gated_mlp import FusedGatedMLPFunction

    dev = _dev()
    g = torch.Generator().manual_seed(11)
    M, K, N = 96, 128, 256
    mk = lambda *s: torch.randn(*s, generator=g).mul(0.1).half()
    x, W_up, b_up, W_gp, b_gp, dH = mk(M, K), mk(N, K), mk(N), mk(N, K), mk(N), mk(M, N)
    args = [a.to(dev).requires_grad_(True) for a in (x, W_up, b_up, W_gp, b_gp)]
    h = FusedGatedMLPFunction.apply(*args)
    grads = torch.autograd.grad(h, args, grad_outputs=dH.to(dev))
    ref_in = [a.float().requires_grad_(True) for a in (x, W_up, b_up, W_gp, b_gp)]
    ref = oracle.hidden_forward(ref_in[0], ref_in[3], ref_in[4], ref_in[1], ref_in[2])["H"]
    ref_grads = torch.autograd.grad(ref, ref_in, grad_outputs=dH.float())
    _close("hidden", h, ref)
    for n, a, b in zip(("dx", "dW_up", "db_up", "dW_gp", "db_gp"), grads, ref_grads):
        _close(n, a, b)


def test_eval_mode_ignores_dropout_and_is_deterministic():
    from triton_gated_mlp import FusedGatedMLP

    dev = _dev()
    torch.manual_seed(3)
    mlp = FusedGatedMLP(256, 512, bias=True, dropout_p=0.5).to(dev).to(torch.bfloat16)
    x = torch.randn(64, 256, device=dev, dtype=torch.bfloat16)
    mlp.eval()
    y0, y1 = mlp(x), mlp(x)
    assert torch.equal(y0, y1)
    mlp.train()
    mlp.dropout_seed = 5
    a = mlp(x)
    mlp._dropout_calls = 0
    b = mlp(x)
    assert torch.equal(a, b), "same seed and offset must give the same mask"
    assert not torch.equal(a, y0)


def test_dropout_mask_matches_numpy_philox_and_rate():
    from triton_gated_mlp.ops import fwd as ops_fwd

    dev = _dev()
    for (M, N, p, seed, off) in [(64, 128, 0.1, 1234, 0), (33, 72, 0.5, 2**40 + 17, 3), (1024, 2048, 0.25, 99, 2**33)]:
        got = ops_fwd.dropout_mask(M, N, p, seed, off, device=dev).cpu().numpy()
        ref = philox.keep_mask(M, N, p, seed, off)
        assert np.array_equal(got, ref)
        rate = got.mean()
        sigma = (p * (1 - p) / (M * N)) ** 0.5
        assert abs(rate - (1 - p)) < 5 * sigma + 1e-9


def test_forward_mask_output_equals_standalone_mask():
    from triton_gated_mlp.ops import fwd as ops_fwd

    dev = _dev()
    g = torch.Generator().manual_seed(5)
    M, K, N = 300, 128, 520
    x = torch.randn(M, K, generator=g).half().to(dev)
    Wg = (0.05 * torch.randn(N, K, generator=g)).half().to(dev)
    Wu = (0.05 * torch.randn(N, K, generator=g)).half().to(dev)
    hs = ops_fwd.gateup_fwd(x, Wg, None, Wu, None, 0.3, seed=77, offset=1, save_activations=True, return_mask=True)
    ref = philox.keep_mask(M, N, 0.3, 77, 1)
    assert np.array_equal(hs.mask.cpu().numpy(), ref)
    o = oracle.hidden_forward(x.float().cpu(), Wg.float().cpu(), None, Wu.float().cpu(), None, torch.from_numpy(ref), 0.3)
    _close("H", hs.hidden, o["H"])
    _close("G", hs.gate, o["G"])
    _close("U", hs.up, o["U"])


@pytest.mark.parametrize("with_mask", [False, True])
def test_gateup_as_whole_rounds_plus_remaining_columns(with_mask):
    """A grid of large tiles that ends in a thinly filled round of workgroups is launched as two
    column ranges (here 352 tiles on 256 compute units: 32 tile columns, then 12 on small tiles).
    Biases, kept G and U, and the dropout mask must line up across the seam: the mask of an element
    depends on its index in the whole tensor.  With and without the keep-mask output (the two
    epilogue implementations)."""
    from triton_gated_mlp.ops import fwd as ops_fwd

    dev = _dev()
    g = torch.Generator().manual_seed(6)
    M, K, N, p = 2048, 64, 5632, 0.3
    x = torch.randn(M, K, generator=g).half().to(dev)
    Wg = (0.1 * torch.randn(N, K, generator=g)).half().to(dev)
    Wu = (0.1 * torch.randn(N, K, generator=g)).half().to(dev)
    bg = (0.1 * torch.randn(N, generator=g)).half().to(dev)
    bu = (0.1 * torch.randn(N, generator=g)).half().to(dev)
    hs = ops_fwd.gateup_fwd(x, Wg, bg, Wu, bu, p, seed=123, offset=2, save_activations=True, return_mask=with_mask)
    ref = philox.keep_mask(M, N, p, 123, 2)
    if with_mask:
        assert np.array_equal(hs.mask.cpu().numpy(), ref)
    f = lambda t: t.float().cpu()
    o = oracle.hidden_forward(f(x), f(Wg), f(bg), f(Wu), f(bu), torch.from_numpy(ref), p)
    _close("H", hs.hidden, o["H"])
    _close("G", hs.gate, o["G"])
    _close("U", hs.up, o["U"])
    # dropped elements are exact zeros, kept ones are not (up to the odd underflow): the mask
    # itself, read off H on both sides of the seam at column 4096
    zero = (hs.hidden == 0).cpu().numpy()
    assert (zero[:, :4096] == (ref[:, :4096] == 0)).mean() > 0.999
    assert (zero[:, 4096:] == (ref[:, 4096:] == 0)).mean() > 0.999


def test_linear_as_whole_rounds_plus_remaining_columns():
    """The same two-launch form for the plain projection: 352 large tiles on 256 compute units,
    bias included; also a shape with exactly one round, which must stay a single launch's result."""
    from triton_gated_mlp.ops import fwd as ops_fwd

    dev = _dev()
    g = torch.Generator().manual_seed(8)
    for M, R, C in [(2048, 64, 11264), (2048, 64, 8192)]:
        a = torch.randn(M, R, generator=g).half().to(dev)
        W = (0.1 * torch.randn(C, R, generator=g)).half().to(dev)
        b = (0.1 * torch.randn(C, generator=g)).half().to(dev)
        y = ops_fwd.linear_fwd(a, W, b)
        ref = a.float().cpu() @ W.float().cpu().T + b.float().cpu()
        _close(f"linear {M}x{R}->{C}", y, ref)


def test_backward_gemms_as_whole_rounds_plus_remaining_rows():
    """dH (with the gating-backward epilogue and dropout) and dX with 352 large tiles on 256 compute
    units: launched as 11 tile rows that make a whole round plus the remaining 5 as a problem of
    their own.  G, U, dG, dU and the dropout counters must line up across the seam at row 2816."""
    from triton_gated_mlp.ops import bwd as ops_bwd

    dev = _dev()
    g = torch.Generator().manual_seed(9)
    M, K, N, p = 4096, 64, 5632, 0.25
    dy = torch.randn(M, K, generator=g).half().to(dev)
    Wd = (0.1 * torch.randn(K, N, generator=g)).half().to(dev)
    G = torch.randn(M, N, generator=g).half().to(dev)
    U = torch.randn(M, N, generator=g).half().to(dev)
    dg, du = ops_bwd.dh_bwd(dy, Wd, G, U, p, 321, 4)
    keep = torch.from_numpy(philox.keep_mask(M, N, p, 321, 4))
    f = lambda t: t.float().cpu()
    ref = oracle.hidden_backward(f(dy) @ f(Wd), f(G), f(U), keep, p)
    _close("dG", dg, ref["dG"])
    _close("dU", du, ref["dU"])
    zero = (du == 0).cpu().numpy()
    for rows in (slice(0, 2816), slice(2816, M)):
        assert (zero[rows] == (keep[rows].numpy() == 0)).mean() > 0.999

    M, K, N = 4096, 5632, 64
    dG = torch.randn(M, N, generator=g).half().to(dev)
    dU = torch.randn(M, N, generator=g).half().to(dev)
    Wg = (0.1 * torch.randn(N, K, generator=g)).half().to(dev)
    Wu = (0.1 * torch.randn(N, K, generator=g)).half().to(dev)
    dx = ops_bwd.dx_bwd(dG, dU, Wg, Wu)
    _close("dX", dx, f(dG) @ f(Wg) + f(dU) @ f(Wu))


@pytest.mark.parametrize("band", ["columns", "rows"])
def test_grouped_weight_gradients_with_a_band_of_the_last_problem_on_its_own(band):
    """528 large tiles on 256 compute units: the last problem of the group gives up a band of 16
    tiles (two tile columns, or two tile rows when it is the tall one), which runs as a launch of
    its own through a moved pointer and a trimmed buffer size.  A reduction length that is not a
    multiple of 64 makes the trimmed size matter: reduction rows past the end must read as zero."""
    from triton_gated_mlp.ops import bwd as ops_bwd

    dev = _dev()
    g = torch.Generator().manual_seed(10)
    Mred = 200
    shapes = [(5632, 2048), (5632, 2048), (2048, 5632)] if band == "columns" else [(2048, 5632), (2048, 5632), (5632, 2048)]
    pairs = []
    for R, C in shapes:
        pairs.append((torch.randn(Mred, R, generator=g).half().to(dev), torch.randn(Mred, C, generator=g).half().to(dev)))
    outs = ops_bwd.dw_bwd_grouped(pairs)
    for (lhs, rhs), out in zip(pairs, outs):
        ref = lhs.float().cpu().T @ rhs.float().cpu()
        _close(f"dW {tuple(out.shape)}", out, ref)


def test_full_size_properties_cfg3_linearity_and_zero():
    """Size-independent checks at the headline shape: x = 0 gives Y = 0 (no bias), and the down
    projection is linear in H (Y(2H) = 2Y(H))."""
    from triton_gated_mlp.ops import fwd as ops_fwd

    dev = _dev()
    c = CFG3
    g = torch.Generator(device="cpu").manual_seed(1)
    Wd = (0.02 * torch.randn(c.K, c.N, generator=g)).half().to(dev)
    H = torch.randn(c.M, c.N, generator=g).half().to(dev)
    y1 = ops_fwd.linear_fwd(H, Wd)
    y2 = ops_fwd.linear_fwd(H * 2, Wd)
    assert torch.allclose(y2.float(), 2 * y1.float(), rtol=2e-3, atol=2e-3)
    Wg = (0.02 * torch.randn(c.N, c.K, generator=g)).half().to(dev)
    z = ops_fwd.gateup_fwd(torch.zeros(c.M, c.K, dtype=torch.float16, device=dev), Wg, None, Wg, None)
    assert not z.hidden.any()


# ---- float32: the reference's own four tests run in float32 (tests/test_gated_mlp_fwd.py:23-82,
# tests/test_gated_mlp_bwd.py:27-129); same shapes, inputs and tolerances here.


def test_reference_fp32_module_forward():
    from triton_gated_mlp import EagerGatedMLP, FusedGatedMLP, copy_weights

    dev = _dev()
    torch.manual_seed(0)
    eager = EagerGatedMLP(dropout_p=0.0).to(dev).float()  # defaults: K=256, N=512, bias=True
    fused = FusedGatedMLP(dropout_p=0.0).to(dev).float()
    copy_weights(eager, fused)
    x = torch.rand((128, eager.hidden_size), device=dev, dtype=torch.float32)
    y_e, y_f = eager(x), fused(x)
    assert torch.allclose(y_f, y_e, rtol=1e-6, atol=1e-2)  # the reference's effective tolerance
    assert torch.allclose(y_f, y_e, rtol=1e-4, atol=1e-5)  # what fp32 accumulation actually gives
    ref = oracle.forward(x.cpu().double(), *[t.detach().cpu().double() for t in (
        eager.gate_proj.weight, eager.gate_proj.bias, eager.up_proj.weight, eager.up_proj.bias,
        eager.down_proj.weight, eager.down_proj.bias)])["Y"]
    assert torch.allclose(y_f.cpu().double(), ref, rtol=1e-4, atol=1e-5)


def test_reference_fp32_operator_forward():
    from triton_gated_mlp import EagerGatedMLP, eager_fwd, mlp_hidden_states_fwd

    dev = _dev()
    torch.manual_seed(1)
    m = EagerGatedMLP(dropout_p=0.0, bias=False).to(dev).float()
    x = torch.rand((128, m.hidden_size), device=dev)
    ref = eager_fwd(x, m.up_proj.weight, None, m.gate_proj.weight, None)
    out = mlp_hidden_states_fwd(x, m.up_proj.weight, None, m.gate_proj.weight, None, m.act_fn, m.dropout.p)
    assert torch.allclose(out, ref, rtol=1e-4, atol=1e-5)
    # the reference builds this test's module with hidden_act="no_act" (tests/test_gated_mlp_fwd.py:41-82)
    up = torch.nn.functional.linear(x, m.up_proj.weight)
    gate = torch.nn.functional.linear(x, m.gate_proj.weight)
    out = mlp_hidden_states_fwd(x, m.up_proj.weight, None, m.gate_proj.weight, None, "no_act", 0.0)
    assert torch.allclose(out, gate * up, rtol=1e-4, atol=1e-5)


def test_reference_fp32_module_backward_3d_input():
    from triton_gated_mlp import EagerGatedMLP, FusedGatedMLP, copy_weights

    dev = _dev()
    torch.manual_seed(2)
    eager = EagerGatedMLP(dropout_p=0.0, bias=False).to(dev).float()
    fused = FusedGatedMLP(dropout_p=0.0, bias=False).to(dev).float()
    copy_weights(eager, fused)
    x = torch.rand((16, 32, eager.hidden_size), device=dev, requires_grad=True)
    y_e, y_f = eager(x), fused(x)
    assert y_f.shape == x.shape
    assert torch.allclose(y_f, y_e, atol=1e-3)
    go = torch.rand_like(x)
    g_e = torch.autograd.grad(y_e, (x, eager.up_proj.weight, eager.gate_proj.weight, eager.down_proj.weight), grad_outputs=go)
    g_f = torch.autograd.grad(y_f, (x, fused.up_proj.weight, fused.gate_proj.weight, fused.down_proj.weight), grad_outputs=go)
    for a, b in zip(g_f, g_e):
        rel = ((a - b).norm() / b.norm()).item()
        assert rel < 1e-5, rel


def test_reference_fp32_operator_backward():
    from triton_gated_mlp import mlp_hidden_states_bwd

    dev = _dev()
    torch.manual_seed(3)
    B, M, N, K = 2, 32, 512, 256
    kw = dict(device=dev, dtype=torch.float32)
    x = torch.rand((B * M, K), **kw) / K
    W_up, W_gp = torch.rand((N, K), **kw) / K, torch.rand((N, K), **kw) / K
    go = torch.rand((B * M, N), **kw) / K
    a, b = x @ W_up.T, x @ W_gp.T
    sig = torch.sigmoid(b)
    goap = go * a * (sig * (1 + b * (1 - sig)))
    goc = go * torch.nn.functional.silu(b)
    dx, dW_up, dW_gp = mlp_hidden_states_bwd(x, W_up, W_gp, go)
    for got, ref in ((dx, goc @ W_up + goap @ W_gp), (dW_up, goc.T @ x), (dW_gp, goap.T @ x)):
        rel = ((got - ref).norm() / ref.norm()).item()
        assert rel < 1e-5, rel  # the reference asks 1e-7 of its own kernels; fp32 MFMA order differs from BLAS


def test_fp32_bias_dropout_forward_backward_against_oracle():
    _run_module_case(Case("fp32_200x136x264", 200, 136, 264, torch.float32, bias=True, p=0.25, backward=True, seed=5))


def test_empty_and_degenerate_inputs():
    from triton_gated_mlp import FusedGatedMLP

    dev = _dev()
    torch.manual_seed(6)
    mlp = FusedGatedMLP(256, 512, bias=True).to(dev).half()
    # no tokens
    x0 = torch.zeros(0, 256, device=dev, dtype=torch.float16, requires_grad=True)
    y0 = mlp(x0)
    assert y0.shape == (0, 256)
    g = torch.autograd.grad(y0, [x0, mlp.gate_proj.weight, mlp.down_proj.bias], grad_outputs=torch.zeros_like(y0))
    assert g[0].shape == (0, 256) and not g[1].any() and not g[2].any()
    assert mlp(torch.zeros(4, 0, 256, device=dev, dtype=torch.float16)).shape == (4, 0, 256)
    # leading dimensions of one and a single token, with gradients
    x1 = torch.randn(1, 1, 256, device=dev, dtype=torch.float16, requires_grad=True)
    y1 = mlp(x1)
    (gx,) = torch.autograd.grad(y1, [x1], grad_outputs=torch.ones_like(y1))
    f = lambda t: t.detach().float().cpu()
    ref = oracle.backward(f(x1).view(1, 256), f(mlp.gate_proj.weight), f(mlp.gate_proj.bias), f(mlp.up_proj.weight),
                          f(mlp.up_proj.bias), f(mlp.down_proj.weight), f(mlp.down_proj.bias), torch.ones(1, 256))
    _close("Y single token", y1.view(1, 256), ref["Y"])
    _close("dX single token", gx.view(1, 256), ref["dX"])


def test_non_contiguous_inputs_and_partial_gradients():
    from triton_gated_mlp import FusedGatedMLP

    dev = _dev()
    torch.manual_seed(7)
    mlp = FusedGatedMLP(256, 768, bias=False).to(dev).to(torch.bfloat16)
    base = torch.randn(96, 512, device=dev, dtype=torch.bfloat16)
    x_nc = base[:, ::2]  # stride 2 along the feature dimension
    assert not x_nc.is_contiguous()
    y_nc = mlp(x_nc)
    assert torch.equal(y_nc, mlp(x_nc.contiguous()))
    # only the input needs a gradient (weights frozen): no weight-gradient launches, same dX
    x = x_nc.contiguous().requires_grad_(True)
    y = mlp(x)
    dy = torch.randn_like(y)
    (dx_full,) = torch.autograd.grad(y, [x], grad_outputs=dy, retain_graph=True)
    for q in mlp.parameters():
        q.requires_grad_(False)
    (dx_frozen,) = torch.autograd.grad(mlp(x), [x], grad_outputs=dy)
    assert torch.equal(dx_full, dx_frozen)
    # only the weights need a gradient
    for q in mlp.parameters():
        q.requires_grad_(True)
    xw = x.detach()
    gw = torch.autograd.grad(mlp(xw), list(mlp.parameters()), grad_outputs=dy)
    f = lambda t: t.detach().float().cpu()
    ref = oracle.backward(f(xw), f(mlp.gate_proj.weight), None, f(mlp.up_proj.weight), None, f(mlp.down_proj.weight),
                          None, f(dy))
    for n, got in zip(("dW_gate", "dW_up", "dW_down"), gw):
        _close(n, got, ref[n])


def test_many_tokens_tall_shape():
    """M much larger than K and N (65536 tokens): 32-bit index paths and the tile scheduler."""
    _run_module_case(Case("tall_65536x256x512", 65536, 256, 512, torch.float16, bias=False, backward=True, seed=8))


def test_batches_beyond_32bit_offsets_run_as_row_chunks(monkeypatch):
    """A batch whose [M, N] activations exceed the pipelined kernels' 32-bit byte offsets is split
    into row chunks by the module (here the limit is lowered to 512 rows: three chunks, the last one
    ragged); outputs and all gradients, weight gradients summed over the chunks, match the oracle."""
    from triton_gated_mlp.ops import fwd as ops_fwd

    assert ops_fwd.max_rows_32bit(8192, 28672, torch.float16) * 28672 * 2 < 2**31
    monkeypatch.setattr(ops_fwd, "max_rows_32bit", lambda K, N, dtype: 512)
    _run_module_case(Case("chunked_1300x256x640", 1300, 256, 640, torch.float16, bias=True, backward=True, seed=31))
    _run_module_case(Case("chunked_1024x256x640", 1024, 256, 640, torch.bfloat16, bias=False, backward=True, seed=32))
    # with dropout every chunk draws a mask of its own; the oracle rebuilds them from last_dropout_states
    _run_module_case(Case("chunked_1300x256x640_p", 1300, 256, 640, torch.float16, bias=True, p=0.2, backward=True, seed=33))


def test_memory_lean_backward_is_bit_identical():
    """recompute_activations=True (keep x only, as the reference does) gives the same gradients."""
    from triton_gated_mlp import FusedGatedMLP

    dev = _dev()
    torch.manual_seed(4)
    mlp = FusedGatedMLP(512, 1024, bias=True, dropout_p=0.2).to(dev).to(torch.bfloat16).train()
    x = torch.randn(384, 512, device=dev, dtype=torch.bfloat16, requires_grad=True)
    dy = torch.randn(384, 512, device=dev, dtype=torch.bfloat16)
    grads = []
    for lean in (False, True):
        mlp.recompute_activations = lean
        mlp.dropout_seed, mlp._dropout_calls = 77, 0
        y = mlp(x)
        grads.append((y, *torch.autograd.grad(y, [x, *mlp.parameters()], grad_outputs=dy)))
    for a, b in zip(*grads):
        assert torch.equal(a, b)


@pytest.mark.parametrize(
    "case",
    [
        Case("lean_384x512x1024", 384, 512, 1024, torch.bfloat16, bias=True, p=0.2, backward=True, seed=4, dropout_seed=77),
        Case("lean_1000x1024x4104", 1000, 1024, 4104, torch.float16, bias=False, p=0.0, backward=True, seed=5),
        # the size of the bf16 baseline configuration (biases, dropout)
        Case("lean_cfg4", CFG4.M, CFG4.K, CFG4.N, CFG4.dtype, bias=True, p=CFG4.p, backward=True, seed=6),
    ],
    ids=lambda c: c.name,
)
def test_memory_lean_backward_against_oracle(case):
    """recompute_activations=True keeps x only and recomputes G, U, H in backward (what the
    reference does, src/triton_gated_mlp/gated_mlp.py:182, ops/bwd.py:184-193): Y and all seven
    gradients against the oracle, with the Philox mask rebuilt from the recorded seed and offset."""
    _run_module_case(case, lean=True)


def test_benchmark_sweep_reports_both_providers_and_step_memory():
    """The sweep harness (reference: src/triton_gated_mlp/benchmark.py:27-45, 69-123) on two small
    cubes: finite TFLOPS for torch eager and the fused module, and a peak-memory column that is
    the step's own (at least the three [M, N] activations the fused backward keeps, and far from
    the hundreds of MB the process holds besides)."""
    from triton_gated_mlp import benchmark

    dev = _dev()
    perf, mem = benchmark.sweep([256, 512], dev)
    assert [r["N"] for r in perf] == [256, 512] and [r["N"] for r in mem] == [256, 512]
    for rp, rm in zip(perf, mem):
        s = rp["N"]
        for prov in ("torch", "fused"):
            assert np.isfinite(rp[prov]) and rp[prov] > 0.0
            assert rp[prov + "_min"] <= rp[prov] <= rp[prov + "_max"]
            assert rm[prov + "_total"] >= rm[prov] > 0.0
        kept_mb = 3 * s * s * 2 / 1024 / 1024  # G, U, H in fp16
        assert kept_mb <= rm["fused"] < 40 * kept_mb, f"fused step peak {rm['fused']:.2f} MB at {s}"


def _streamk_expected(op, M, K, N, code=0):
    from triton_gated_mlp import _cabi

    return _cabi.lib().gmlp_workspace_bytes(op, M, K, N, code)


def test_streamk_seams_every_gemm_kind_against_fp32_matmul():
    """Grids of large tiles that end in a thinly filled round with a long reduction run their last
    round's tiles as stream-K pieces (several workgroups per tile, fp32 partial sums through the
    workspace, a second launch adds them up in a fixed order).  Every kind of GEMM of the MLP on a
    shape that takes that path (the workspace query says so), against fp32 products of the same
    rounded operands; twice, bit-identical (no dependence on timing)."""
    from triton_gated_mlp import _cabi
    from triton_gated_mlp.ops import bwd as ops_bwd
    from triton_gated_mlp.ops import fwd as ops_fwd

    dev = _dev()
    g = torch.Generator().manual_seed(17)
    rnd = lambda *shape, s=1.0: (s * torch.randn(*shape, generator=g)).half()
    f = lambda t: t.float()

    # down projection: out [2048, 11264] = 352 tiles (1.375 rounds), reduction 5184 = 81 tiles; 96 tiles
    # over 256 workgroups: ranges that straddle tiles (the other cases below cut every tile into a
    # whole number of pieces)
    M, R, C = 2048, 5184, 11264
    assert _streamk_expected(_cabi.GMLP_OP_LINEAR_FWD, M, R, C) == (96 + 256) * 65536 * 4
    a, w, b = rnd(M, R), rnd(C, R, s=0.02), rnd(C, s=0.1)
    y = ops_fwd.linear_fwd(a.to(dev), w.to(dev), b.to(dev))
    assert torch.equal(y, ops_fwd.linear_fwd(a.to(dev), w.to(dev), b.to(dev)))
    _close("linear stream-K", y, f(a) @ f(w).T + f(b))
    # the same call without a workspace (one workgroup per tile throughout): same values up to the
    # order of the fp32 additions in the shared-out tiles
    y0 = torch.empty_like(y)
    ad, wd, bd = a.to(dev), w.to(dev), b.to(dev)
    _cabi.check(_cabi.lib().gmlp_linear_fwd(ad.data_ptr(), wd.data_ptr(), bd.data_ptr(), y0.data_ptr(), M, R, C, 0, None, 0,
                                            _cabi.stream_ptr(dev)))
    torch.cuda.synchronize()
    assert (y.float() - y0.float()).abs().max().item() <= 2e-3 * y0.float().abs().max().item()
    assert not torch.equal(y, torch.zeros_like(y))

    # the same with ragged edges (2000 rows, 11256 columns) in bf16: pieces of edge tiles, predicated sums
    M, R, C = 2000, 5184, 11256
    assert _streamk_expected(_cabi.GMLP_OP_LINEAR_FWD, M, R, C, 1) == (96 + 256) * 65536 * 4
    a, w, b = [v.bfloat16() for v in (rnd(M, R), rnd(C, R, s=0.02), rnd(C, s=0.1))]
    y = ops_fwd.linear_fwd(a.to(dev), w.to(dev), b.to(dev))
    assert torch.equal(y, ops_fwd.linear_fwd(a.to(dev), w.to(dev), b.to(dev)))
    _close("linear stream-K ragged bf16", y, f(a) @ f(w).T + f(b))

    # gate/up: [2048, 5120] hidden = 8 x 40 tiles of 256 x 128, reduction 4352; biases, dropout, G and U kept
    M, K, N = 2048, 4352, 5120
    assert _streamk_expected(_cabi.GMLP_OP_GATEUP_FWD, M, K, N) > 0
    x, wg, wu, bg, bu = rnd(M, K), rnd(N, K, s=0.02), rnd(N, K, s=0.02), rnd(N, s=0.1), rnd(N, s=0.1)
    p, seed = 0.25, 4242
    hs = ops_fwd.gateup_fwd(x.to(dev), wg.to(dev), bg.to(dev), wu.to(dev), bu.to(dev), p, seed, 3, save_activations=True)
    hs2 = ops_fwd.gateup_fwd(x.to(dev), wg.to(dev), bg.to(dev), wu.to(dev), bu.to(dev), p, seed, 3, save_activations=True)
    assert torch.equal(hs.hidden, hs2.hidden) and torch.equal(hs.gate, hs2.gate) and torch.equal(hs.up, hs2.up)
    keep = torch.from_numpy(philox.keep_mask(M, N, p, seed, 3))
    ref = oracle.hidden_forward(f(x), f(wg), f(bg), f(wu), f(bu), keep, p)
    _close("gate/up stream-K H", hs.hidden, ref["H"])
    _close("gate/up stream-K G", hs.gate, ref["G"])
    _close("gate/up stream-K U", hs.up, ref["U"])

    # dH with the gating epilogue: [2048, 10240] = 320 tiles, reduction 4352
    M, K, N = 2048, 4352, 10240
    assert _streamk_expected(_cabi.GMLP_OP_DH_BWD, M, K, N) > 0
    dy, wdn, G, U = rnd(M, K), rnd(K, N, s=0.02), rnd(M, N), rnd(M, N)
    dg, du = ops_bwd.dh_bwd(dy.to(dev), wdn.to(dev), G.to(dev), U.to(dev), p, seed, 5)
    dg2, du2 = ops_bwd.dh_bwd(dy.to(dev), wdn.to(dev), G.to(dev), U.to(dev), p, seed, 5)
    assert torch.equal(dg, dg2) and torch.equal(du, du2)
    keep = torch.from_numpy(philox.keep_mask(M, N, p, seed, 5))
    hb = oracle.hidden_backward(f(dy) @ f(wdn), f(G), f(U), keep, p)
    _close("dH stream-K dG", dg, hb["dG"])
    _close("dH stream-K dU", du, hb["dU"])

    # dX: [2048, 10240] = 320 tiles, two reduction segments of 2176 = 68 tiles together
    M, K, N = 2048, 10240, 2176
    assert _streamk_expected(_cabi.GMLP_OP_DX_BWD, M, K, N) > 0
    dgv, duv, wg, wu = rnd(M, N), rnd(M, N), rnd(N, K, s=0.02), rnd(N, K, s=0.02)
    dx = ops_bwd.dx_bwd(dgv.to(dev), duv.to(dev), wg.to(dev), wu.to(dev))
    assert torch.equal(dx, ops_bwd.dx_bwd(dgv.to(dev), duv.to(dev), wg.to(dev), wu.to(dev)))
    _close("dX stream-K", dx, f(dgv) @ f(wg) + f(duv) @ f(wu))

    # dW, one problem: [10240, 2048] = 320 tiles, reduction over 4360 token rows (not a multiple of 64)
    Mred, R, C = 4360, 10240, 2048
    assert _streamk_expected(_cabi.GMLP_OP_DW_BWD, Mred, R, C) > 0
    lhs, rhs = rnd(Mred, R), rnd(Mred, C)
    dw = ops_bwd.dw_bwd(lhs.to(dev), rhs.to(dev))
    assert torch.equal(dw, ops_bwd.dw_bwd(lhs.to(dev), rhs.to(dev)))
    _close("dW stream-K", dw, f(lhs).T @ f(rhs))

    # dW, grouped: 64 + 64 + 256 = 384 tiles (1.5 rounds); the shared-out tiles are the last 128 of
    # the last problem (reduction of 102 tiles: half a round saved is worth the second launch)
    Mred = 6528
    pairs = [(rnd(Mred, 2048), rnd(Mred, 2048)), (rnd(Mred, 2048), rnd(Mred, 2048)), (rnd(Mred, 4096), rnd(Mred, 4096))]
    dev_pairs = [(a_.to(dev), b_.to(dev)) for a_, b_ in pairs]
    outs = ops_bwd.dw_bwd_grouped(dev_pairs)
    outs2 = ops_bwd.dw_bwd_grouped(dev_pairs)
    for (a_, b_), got, again in zip(pairs, outs, outs2):
        assert torch.equal(got, again)
        _close("dW grouped stream-K", got, f(a_).T @ f(b_))


def test_streamk_pieces_that_straddle_tiles_every_gemm_kind():
    """352 large tiles = one whole round and 96 tiles: 96 does not divide 256, so the shared-out
    tiles go to 256 workgroups as even ranges of (tile, reduction tile) pairs that begin and end
    inside tiles (the multi-piece loop, slot = workgroup + tile, the search for a tile's first
    workgroup in the second stage).  Every kind of GEMM: two accumulator sets (gate/up), the dH
    epilogue with its prefetch, a piece crossing the seam between dX's two reduction segments, both
    operands reduction-strided with a ragged reduction (dW); against fp32 products on the host."""
    from triton_gated_mlp import _cabi
    from triton_gated_mlp.ops import bwd as ops_bwd
    from triton_gated_mlp.ops import fwd as ops_fwd

    dev = _dev()
    g = torch.Generator().manual_seed(23)
    rnd = lambda *shape, s=1.0: (s * torch.randn(*shape, generator=g)).half()
    f = lambda t: t.float()
    straddling = (96 + 256) * 65536 * 4  # slots of a plan without whole pieces per tile

    M, K, N = 2048, 5184, 5632  # gate/up: 8 x 44 tiles of 256 x 128, 81 reduction tiles
    assert _streamk_expected(_cabi.GMLP_OP_GATEUP_FWD, M, K, N) == straddling
    x, wg, wu, bg = rnd(M, K), rnd(N, K, s=0.02), rnd(N, K, s=0.02), rnd(N, s=0.1)
    hs = ops_fwd.gateup_fwd(x.to(dev), wg.to(dev), bg.to(dev), wu.to(dev), None, save_activations=True)
    hs2 = ops_fwd.gateup_fwd(x.to(dev), wg.to(dev), bg.to(dev), wu.to(dev), None, save_activations=True)
    assert torch.equal(hs.hidden, hs2.hidden) and torch.equal(hs.gate, hs2.gate) and torch.equal(hs.up, hs2.up)
    ref = oracle.hidden_forward(f(x), f(wg), f(bg), f(wu), None, None, 0.0)
    _close("gate/up straddling H", hs.hidden, ref["H"])
    _close("gate/up straddling G", hs.gate, ref["G"])
    _close("gate/up straddling U", hs.up, ref["U"])

    M, K, N = 2048, 5184, 11264  # dH: 8 x 44 tiles of 256 x 256
    assert _streamk_expected(_cabi.GMLP_OP_DH_BWD, M, K, N) == straddling
    dy, wdn, G, U = rnd(M, K), rnd(K, N, s=0.02), rnd(M, N), rnd(M, N)
    dg, du = ops_bwd.dh_bwd(dy.to(dev), wdn.to(dev), G.to(dev), U.to(dev))
    dg2, du2 = ops_bwd.dh_bwd(dy.to(dev), wdn.to(dev), G.to(dev), U.to(dev))
    assert torch.equal(dg, dg2) and torch.equal(du, du2)
    hb = oracle.hidden_backward(f(dy) @ f(wdn), f(G), f(U), None, 0.0)
    _close("dH straddling dG", dg, hb["dG"])
    _close("dH straddling dU", du, hb["dU"])

    M, K, N = 2048, 11264, 2624  # dX: two segments of 41 reduction tiles; pieces of 30-31 cross the seam
    assert _streamk_expected(_cabi.GMLP_OP_DX_BWD, M, K, N) == straddling
    dgv, duv, wg, wu = rnd(M, N), rnd(M, N), rnd(N, K, s=0.02), rnd(N, K, s=0.02)
    dx = ops_bwd.dx_bwd(dgv.to(dev), duv.to(dev), wg.to(dev), wu.to(dev))
    assert torch.equal(dx, ops_bwd.dx_bwd(dgv.to(dev), duv.to(dev), wg.to(dev), wu.to(dev)))
    _close("dX straddling", dx, f(dgv) @ f(wg) + f(duv) @ f(wu))

    Mred, R, C = 5192, 2048, 11264  # dW: 82 reduction tiles, the last one of 8 rows
    assert _streamk_expected(_cabi.GMLP_OP_DW_BWD, Mred, R, C) == straddling
    lhs, rhs = rnd(Mred, R), rnd(Mred, C)
    dw = ops_bwd.dw_bwd(lhs.to(dev), rhs.to(dev))
    assert torch.equal(dw, ops_bwd.dw_bwd(lhs.to(dev), rhs.to(dev)))
    _close("dW straddling", dw, f(lhs).T @ f(rhs))


def test_grouped_launch_of_one_problem_whose_tiles_all_go_to_streamk():
    """A single weight gradient of 200 large tiles with a long reduction: fewer tiles than compute
    units, so the plan shares out every tile and the grouped launch has no whole-tile grid left to
    run (which must not be launched empty).  Against the fp32 product and gmlp_dw_bwd."""
    import ctypes

    from triton_gated_mlp import _cabi
    from triton_gated_mlp.ops import bwd as ops_bwd

    dev = _dev()
    Mred, R, C = 16384, 2560, 5120
    RC = (ctypes.c_int64 * 1)
    nbytes = _cabi.lib().gmlp_dw_bwd_grouped_workspace_bytes(
        1, Mred, ctypes.cast(RC(R), ctypes.c_void_p), ctypes.cast(RC(C), ctypes.c_void_p), 0)
    assert nbytes == (200 + 256) * 65536 * 4  # all 200 tiles shared out over 256 workgroups
    g = torch.Generator().manual_seed(29)
    lhs = torch.randn(Mred, R, generator=g).half()
    rhs = torch.randn(Mred, C, generator=g).half()
    (grouped,) = ops_bwd.dw_bwd_grouped([(lhs.to(dev), rhs.to(dev))])
    single = ops_bwd.dw_bwd(lhs.to(dev), rhs.to(dev))
    torch.cuda.synchronize()
    assert torch.equal(grouped, single)
    _close("dW, one problem, all tiles as pieces", grouped, lhs.float().T @ rhs.float())


@pytest.mark.parametrize(
    "M,K,N,dtype,bias,p",
    [
        (2048, 2048, 5632, torch.bfloat16, True, 0.1),   # mid-size grids, biases, dropout
        (300, 1024, 4096, torch.float16, True, 0.0),     # short batch: split reductions, ragged rows
        (2048, 4352, 5120, torch.float16, False, 0.25),  # stream-K in the forward GEMMs
        (1000, 520, 1048, torch.bfloat16, True, 0.0),    # widths that are multiples of 8 only (predicated kernels)
        (192, 512, 768, torch.float32, True, 0.1),       # float32 path
    ],
)
def test_whole_pass_entry_points_equal_the_separate_launches(M, K, N, dtype, bias, p):
    """gmlp_mlp_fwd and gmlp_mlp_bwd (one library call per pass; what the module uses) give, bit for
    bit, what the per-GEMM entry points give when called one after the other, call after call, and
    leave out exactly the gradients that were not asked for.  (The separate entry
    points are the ones held against the oracle throughout this file; the module-level cases go
    through the one-call entries and are held against the oracle as well.)"""
    from triton_gated_mlp.ops import bwd as ops_bwd
    from triton_gated_mlp.ops import fwd as ops_fwd

    dev = _dev()
    g = torch.Generator().manual_seed(31)
    rnd = lambda *shape, s=1.0: (s * torch.randn(*shape, generator=g)).to(dtype).to(dev)
    x, wg, wu, wd, dy = rnd(M, K), rnd(N, K, s=0.03), rnd(N, K, s=0.03), rnd(K, N, s=0.03), rnd(M, K)
    bg, bu, bd = (rnd(N, s=0.1), rnd(N, s=0.1), rnd(K, s=0.1)) if bias else (None, None, None)
    seed, off = 77, 2
    hs = ops_fwd.gateup_fwd(x, wg, bg, wu, bu, p, seed, off, save_activations=True)
    y_ref = ops_fwd.linear_fwd(hs.hidden, wd, bd)
    y, hs1 = ops_fwd.mlp_fwd(x, wg, bg, wu, bu, wd, bd, p, seed, off, save_activations=True)
    assert torch.equal(y, y_ref) and torch.equal(hs1.hidden, hs.hidden)
    assert torch.equal(hs1.gate, hs.gate) and torch.equal(hs1.up, hs.up)
    y2, hs2 = ops_fwd.mlp_fwd(x, wg, bg, wu, bu, wd, bd, p, seed, off, save_activations=False)
    assert torch.equal(y2, y_ref) and hs2.gate is None and hs2.up is None

    dg, du = ops_bwd.dh_bwd(dy, wd, hs.gate, hs.up, p, seed, off)
    ref = {
        "dx": ops_bwd.dx_bwd(dg, du, wg, wu),
        "dW_gate": None, "db_gate": None, "dW_up": None, "db_up": None, "dW_down": None, "db_down": None,
    }
    ref["dW_gate"], ref["dW_up"], ref["dW_down"] = ops_bwd.dw_bwd_grouped([(dg, x), (du, x), (dy, hs.hidden)])
    if bias:
        ref["db_gate"], ref["db_up"], ref["db_down"] = ops_bwd.colsum_grouped([dg, du, dy])
    names = list(ref)
    all_of = tuple(ref[n] is not None for n in names)
    for call in range(2):
        got = ops_bwd.mlp_bwd(dy, x, wg, wu, wd, hs.gate, hs.up, hs.hidden, all_of, p, seed, off)
        torch.cuda.synchronize()
        for n, a, b in zip(names, got, (ref[n] for n in names)):
            assert (a is None) == (b is None), n
            assert a is None or torch.equal(a, b), f"{n} differs (call {call})"
    # subsets: only the input gradient; only the down projection's gradients; everything but dX
    for want in ((True,) + (False,) * 6, (False,) * 5 + (True, bias), (False,) + all_of[1:]):
        got = ops_bwd.mlp_bwd(dy, x, wg, wu, wd, hs.gate, hs.up, hs.hidden, want, p, seed, off)
        torch.cuda.synchronize()
        for n, w, a in zip(names, want, got):
            assert (a is not None) == bool(w), n
            assert a is None or torch.equal(a, ref[n]), f"{n} differs for subset {want}"


def test_random_shapes_every_operator_against_fp32_products():
    """Two dozen seeded random shapes through the five GEMM operators: token counts from 1 to a few
    thousand, widths that are multiples of 64 (tuned kernels: large, medium, two-launch, split and
    stream-K grids as the dispatcher picks them) or only of 8 (predicated kernel), both 16-bit
    dtypes; each result against the fp32 product of the same rounded operands, computed on the host,
    and the gate/up and dH epilogues against the oracle's closed forms."""
    from triton_gated_mlp.ops import bwd as ops_bwd
    from triton_gated_mlp.ops import fwd as ops_fwd

    dev = _dev()
    rng = np.random.default_rng(20240611)
    g = torch.Generator(device="cpu").manual_seed(99)
    f = lambda t: t.float().cpu()
    for case in range(24):
        dtype = torch.float16 if case % 2 == 0 else torch.bfloat16
        unit = 8 if case % 6 == 5 else 64
        M = int(rng.choice([1, 7, 33, 100, 255, 256, 257, 700, 1500, 2304, 3000]))
        K = int(rng.integers(1, 3072 // unit + 1)) * unit
        N = int(rng.integers(1, 4096 // unit + 1)) * unit
        print(f"random case {case}: M={M} K={K} N={N} {dtype}", flush=True)
        rnd = lambda *shape, s=1.0: (s * torch.randn(*shape, generator=g)).to(dtype).to(dev)
        x, wg, wu, wd = rnd(M, K), rnd(N, K, s=0.03), rnd(N, K, s=0.03), rnd(K, N, s=0.03)
        dy = rnd(M, K)
        # forward
        hs = ops_fwd.gateup_fwd(x, wg, None, wu, None, save_activations=True)
        G, U = f(x) @ f(wg).T, f(x) @ f(wu).T
        _close("G", hs.gate, G)
        _close("U", hs.up, U)
        _close("H", hs.hidden, torch.nn.functional.silu(G) * U)
        y = ops_fwd.linear_fwd(hs.hidden, wd)
        _close("Y", y, f(hs.hidden) @ f(wd).T)
        # backward, from the device's own (rounded) G, U and H so that every operator is checked alone
        dg, du = ops_bwd.dh_bwd(dy, wd, hs.gate, hs.up)
        hb = oracle.hidden_backward(f(dy) @ f(wd), f(hs.gate), f(hs.up), None, 0.0)
        _close("dG", dg, hb["dG"])
        _close("dU", du, hb["dU"])
        dx = ops_bwd.dx_bwd(dg, du, wg, wu)
        ref_dx = f(dg) @ f(wg) + f(du) @ f(wu)
        _close("dX", dx, ref_dx)
        pairs = [(dg, x), (du, x), (dy, hs.hidden)]
        for name, got, (a_, b_) in zip(("dW_gate", "dW_up", "dW_down"), ops_bwd.dw_bwd_grouped(pairs), pairs):
            ref = f(a_).T @ f(b_)
            _close(name, got, ref)
        _close("dW_gate alone", ops_bwd.dw_bwd(dg, x), f(dg).T @ f(x))


def test_random_modules_through_the_one_call_entries_no_worse_than_torch_16bit():
    """Four dozen seeded random modules (token counts 1 to 6144, widths that are multiples of 8, 64
    or 256, both 16-bit dtypes, biases, dropout, five activations) through FusedGatedMLP, i.e. through
    gmlp_mlp_fwd / gmlp_mlp_bwd, against fp32 formulas on the same rounded inputs with the library's
    own keep mask.  Weights ~ N(0, 0.03) and biases ~ U(-0.1, 0.1): harsher than the baseline's
    distributions, so that 16-bit rounding of G, U, H and of the outputs shows as a few elements
    beyond the element-wise band of `_close` (bf16 resolves 2^-9).  Those are counted, not waved
    through: the fused path may
    leave the band at most twice as often as the same formulas run through torch's own 16-bit
    operators on the same inputs with the same mask (plus 16 elements + 2e-5 of the tensor).  The
    relative Frobenius error stays below 1e-2 throughout.  The activations are the smooth ones: a
    relu whose fp32 pre-activation lies within 1e-6 of zero falls on either side of the kink
    depending on the summation order of whoever computes it, the fp32 reference included, and then
    moves a whole row of dW_gate (relu and leaky_relu are held to the CPU oracle in
    test_other_activations_*)."""
    import random

    from triton_gated_mlp import FusedGatedMLP
    from triton_gated_mlp.ops import fwd as ops_fwd

    dev = _dev()
    rng = random.Random(1)
    acts = {"silu": torch.nn.functional.silu, "gelu": torch.nn.functional.gelu, "tanh": torch.tanh,
            "sigmoid": torch.sigmoid, "no_act": lambda t: t}

    def outside(got, ref):
        got, ref = got.float(), ref.float()
        assert torch.isfinite(got).all()
        atol = ATOL * max(1.0, ref.abs().mean().item())
        fro = ((got - ref).norm() / ref.norm().clamp_min(1e-30)).item()
        return int(((got - ref).abs() > atol + RTOL * ref.abs()).sum()), fro

    for case in range(48):
        dt = rng.choice([torch.float16, torch.bfloat16])
        unit = rng.choice([64, 64, 64, 8, 256])
        M = rng.choice([1, 3, 16, 17, 33, 100, 255, 256, 257, 511, 700, 1024, 1500, 2048, 2304, 3000, 4097, 6144])
        K = rng.randint(1, 4096 // unit) * unit
        N = rng.randint(1, 6144 // unit) * unit
        bias = rng.random() < 0.5
        p = rng.choice([0.0, 0.0, 0.1, 0.3])
        act = rng.choice(list(acts))
        print(f"random module {case}: M={M} K={K} N={N} {dt} bias={bias} p={p} act={act}", flush=True)
        g = torch.Generator(device=dev).manual_seed(case)
        mlp = FusedGatedMLP(K, N, bias=bias, dropout_p=p, hidden_act=act).to(dev).to(dt)
        with torch.no_grad():
            for lin in (mlp.gate_proj, mlp.up_proj, mlp.down_proj):
                lin.weight.copy_(torch.empty(lin.weight.shape, device=dev).normal_(0, 0.03, generator=g))
                if bias:
                    lin.bias.copy_(torch.empty(lin.bias.shape, device=dev).uniform_(-0.1, 0.1, generator=g))
        mlp.train(p > 0)
        mlp.dropout_seed = 99
        x = torch.empty(M, K, device=dev).normal_(0, 1, generator=g).to(dt)
        dy = torch.empty(M, K, device=dev).normal_(0, 1, generator=g).to(dt)
        xs = x.clone().requires_grad_(True)
        y = mlp(xs)
        fused = [y] + list(torch.autograd.grad(y, [xs] + list(mlp.parameters()), dy))
        # fp32 formulas, the same keep mask
        xf = x.float().requires_grad_(True)
        ps = [q.detach().float().requires_grad_(True) for q in mlp.parameters()]
        if bias:
            Wg, bg, Wu, bu, Wd, bd = ps
        else:
            (Wg, Wu, Wd), bg, bu, bd = ps, None, None, None
        H = acts[act](torch.nn.functional.linear(xf, Wg, bg)) * torch.nn.functional.linear(xf, Wu, bu)
        if p > 0:
            seed, off = mlp.last_dropout_state
            keep = ops_fwd.dropout_mask(M, N, p, seed, off, device=dev).float()
            H = H * keep / (1 - p)
        yr = torch.nn.functional.linear(H, Wd, bd)
        ref = [yr] + list(torch.autograd.grad(yr, [xf] + ps, dy.float()))
        # yardstick: the same formulas through torch's own 16-bit operators, same keep mask
        xe = x.clone().requires_grad_(True)
        pe = [q.detach().clone().requires_grad_(True) for q in mlp.parameters()]
        if bias:
            Wg, bg, Wu, bu, Wd, bd = pe
        else:
            (Wg, Wu, Wd), bg, bu, bd = pe, None, None, None
        He = acts[act](torch.nn.functional.linear(xe, Wg, bg)) * torch.nn.functional.linear(xe, Wu, bu)
        if p > 0:
            He = He * (keep.to(dt) * (1.0 / (1 - p)))
        ye = torch.nn.functional.linear(He, Wd, bd)
        yard = [ye] + list(torch.autograd.grad(ye, [xe] + pe, dy))
        names = ["Y", "dX"] + [n for n, _ in mlp.named_parameters()]
        for i, n in enumerate(names):
            bad, fro = outside(fused[i], ref[i])
            allowed = 16 + 2e-5 * ref[i].numel() + 2 * outside(yard[i], ref[i])[0]
            assert fro < 1e-2, f"{n}: relative Frobenius error {fro:.3e}"
            assert bad <= allowed, f"{n}: {bad} elements outside the band, {allowed:.0f} allowed"


def test_grouped_weight_gradients_equal_single_launches():
    """gmlp_dw_bwd_grouped (one grid) is bit-identical to three gmlp_dw_bwd launches."""
    from triton_gated_mlp.ops import bwd as ops_bwd

    dev = _dev()
    g = torch.Generator().manual_seed(9)
    for M, K, N in [(2048, 2048, 5632), (512, 256, 520)]:  # full-tile class and predicated class
        x = torch.randn(M, K, generator=g).half().to(dev)
        dg = torch.randn(M, N, generator=g).half().to(dev)
        du = torch.randn(M, N, generator=g).half().to(dev)
        dy = torch.randn(M, K, generator=g).half().to(dev)
        h = torch.randn(M, N, generator=g).half().to(dev)
        pairs = [(dg, x), (du, x), (dy, h)]
        grouped = ops_bwd.dw_bwd_grouped(pairs)
        for (a, b), got in zip(pairs, grouped):
            assert torch.equal(got, ops_bwd.dw_bwd(a, b))  # (neither form shares out tiles at these shapes)
        _close("dW_gate grouped", grouped[0], dg.float().cpu().T @ x.float().cpu())


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_decode_matches_general_path(dtype):
    """Skinny-M kernels against the oracle and the general path: both layouts of the intermediate H
    (row-major up to M = 10, fragment order above, with token slots past M), both streaming variants
    of the down projection, and shapes that only the register-streaming kernels take."""
    from triton_gated_mlp.ops import fwd as ops_fwd

    dev = _dev()
    g = torch.Generator().manual_seed(2)
    for M, K, N, bias in [(16, 1024, 2048, True), (3, 256, 512, False), (1, 4096, 11008, True), (5, 768, 1792, True),
                          (16, 4096, 11008, False), (12, 1024, 2048, True), (11, 768, 1792, False), (10, 8192, 512, True)]:
        x = torch.randn(M, K, generator=g).to(dtype).to(dev)
        Wg = (0.02 * torch.randn(N, K, generator=g)).to(dtype).to(dev)
        Wu = (0.02 * torch.randn(N, K, generator=g)).to(dtype).to(dev)
        Wd = (0.02 * torch.randn(K, N, generator=g)).to(dtype).to(dev)
        bg = bu = bd = None
        if bias:
            bg = (0.01 * torch.randn(N, generator=g)).to(dtype).to(dev)
            bu = (0.01 * torch.randn(N, generator=g)).to(dtype).to(dev)
            bd = (0.01 * torch.randn(K, generator=g)).to(dtype).to(dev)
        y = ops_fwd.decode_fwd(x, Wg, bg, Wu, bu, Wd, bd)
        f = lambda t: None if t is None else t.float().cpu()
        ref = oracle.forward(f(x), f(Wg), f(bg), f(Wu), f(bu), f(Wd), f(bd))
        _close(f"decode Y M={M}", y, ref["Y"])
        h = ops_fwd.gateup_fwd(x, Wg, bg, Wu, bu).hidden
        y_general = ops_fwd.linear_fwd(h, Wd, bd)
        _close(f"general Y M={M}", y_general, ref["Y"])


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_decode_with_two_token_tiles(dtype):
    """16 < M <= 32 on the streaming kernels (two MFMAs per weight fragment, H for 32 token slots):
    full and partly filled second tiles, both block heights of the down projection, widths whose
    rows do not fill a last round of blocks, with and without biases."""
    from triton_gated_mlp.ops import fwd as ops_fwd

    dev = _dev()
    g = torch.Generator().manual_seed(5)
    for M, K, N, bias in [(32, 1024, 2048, True), (17, 768, 1792, False), (24, 8192, 768, True), (31, 4096, 11008, True),
                          (20, 4352, 1024, False), (32, 5120, 13824, False)]:
        assert ops_fwd.decode_supported(M, K, N, dtype)
        print(f"decode two tiles {dtype} M={M} K={K} N={N} bias={bias}", flush=True)
        x = torch.randn(M, K, generator=g).to(dtype).to(dev)
        Wg = (0.02 * torch.randn(N, K, generator=g)).to(dtype).to(dev)
        Wu = (0.02 * torch.randn(N, K, generator=g)).to(dtype).to(dev)
        Wd = (0.02 * torch.randn(K, N, generator=g)).to(dtype).to(dev)
        bg = bu = bd = None
        if bias:
            bg = (0.01 * torch.randn(N, generator=g)).to(dtype).to(dev)
            bu = (0.01 * torch.randn(N, generator=g)).to(dtype).to(dev)
            bd = (0.01 * torch.randn(K, generator=g)).to(dtype).to(dev)
        y = ops_fwd.decode_fwd(x, Wg, bg, Wu, bu, Wd, bd)
        f = lambda t: None if t is None else t.float().cpu()
        ref = oracle.forward(f(x), f(Wg), f(bg), f(Wu), f(bu), f(Wd), f(bd))
        _close(f"decode Y M={M}", y, ref["Y"])
    # shapes the streaming kernels do not take keep the limit of 16 rows
    assert not ops_fwd.decode_supported(17, 512, 1024, dtype)
    with pytest.raises(NotImplementedError):
        ops_fwd.decode_fwd(torch.zeros(17, 512, dtype=dtype, device=dev), *[t for _ in range(2) for t in (torch.zeros(1024, 512, dtype=dtype, device=dev), None)],
                           torch.zeros(512, 1024, dtype=dtype, device=dev), None)


@pytest.mark.parametrize("M,K,N,streams", [(8, 2048, 4096, True), (24, 3584, 4096, True), (64, 1024, 4096, False)])
def test_inference_forward_under_hip_graph_replay(M, K, N, streams):
    """Serving loops replay a captured forward: the skinny-M streaming path (one and two token
    tiles) and the general path with split reductions are captured once and replayed with new
    inputs written into the captured input buffer; every replay must equal the eager result for
    that input, with eager work and synchronisations in between."""
    from triton_gated_mlp import FusedGatedMLP
    from triton_gated_mlp.ops import fwd as ops_fwd

    dev = _dev()
    cus = torch.cuda.get_device_properties(dev).multi_processor_count
    assert ops_fwd.decode_preferred(M, K, N, torch.float16, cus) == streams
    mlp = FusedGatedMLP(K, N, bias=True).to(dev).to(torch.float16).eval()
    g = torch.Generator().manual_seed(41)
    inputs = [torch.randn(M, K, generator=g).half().to(dev) for _ in range(3)]
    with torch.no_grad():
        eager = [mlp(v).clone() for v in inputs]
        x = inputs[0].clone()
        side = torch.cuda.Stream(device=dev)
        side.wait_stream(torch.cuda.current_stream(dev))
        with torch.cuda.stream(side):  # warm-up on a side stream, as torch's graph recipe asks
            mlp(x)
        torch.cuda.current_stream(dev).wait_stream(side)
        torch.cuda.synchronize(dev)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            y = mlp(x)
        for rep in (1, 2, 0, 1):
            x.copy_(inputs[rep])
            y.fill_(float("nan"))
            _ = (torch.randn(256, 256, device=dev) @ torch.randn(256, 256, device=dev)).sum().item()
            graph.replay()
            torch.cuda.synchronize(dev)
            assert torch.equal(y, eager[rep]), f"replay with input {rep} differs from the eager forward"


def test_training_step_under_stream_capture_is_refused(monkeypatch):
    """A forward that records an autograd graph while its stream is being captured raises a
    RuntimeError (no kernel is enqueued, nothing is captured); the capture state is simulated on
    the host, no stream is actually captured here."""
    from triton_gated_mlp import FusedGatedMLP

    dev = _dev()
    mlp = FusedGatedMLP(256, 512, bias=False).to(dev).half()
    x = torch.randn(64, 256, device=dev, dtype=torch.float16, requires_grad=True)
    monkeypatch.setattr(torch.cuda, "is_current_stream_capturing", lambda: True)
    with pytest.raises(RuntimeError, match="autograd graph"):
        mlp(x)
    with torch.no_grad():
        assert mlp(x).shape == (64, 256)  # inference is not affected


@pytest.mark.skip(
    reason="capturing the step with torch.cuda.graph ended in a host-side segmentation fault inside "
    "capture_end (hipStreamEndCapture) on this image; cause not established, so the case stays off the GPU"
)
def test_forward_backward_under_hip_graph_replay():
    """The entry points only enqueue kernels on the caller's stream (no allocation, no memset), so a
    training step can be captured once and replayed; every replay must equal the eager result."""
    from triton_gated_mlp import FusedGatedMLP

    dev = _dev()
    c = Case("graph", 512, 256, 768, torch.float16, bias=True, p=0.1, backward=True, seed=31)
    t = make_inputs(c)
    mlp = FusedGatedMLP(c.K, c.N, bias=True, dropout_p=c.p).to(dev).to(c.dtype).train()
    mlp.dropout_seed = 99
    x = t["x"].to(dev).requires_grad_(True)
    dY = t["dY"].to(dev)
    params = [x] + list(mlp.parameters())

    def step():
        mlp._dropout_calls = 0  # same mask stream for every step
        y = mlp(x)
        return (y,) + torch.autograd.grad(y, params, grad_outputs=dY)

    eager = [v.clone() for v in step()]
    side = torch.cuda.Stream(device=dev)
    side.wait_stream(torch.cuda.current_stream(dev))
    with torch.cuda.stream(side):  # warm-up on the capture stream, as torch's graph recipe asks
        step()
    torch.cuda.current_stream(dev).wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        outs = step()
    for rep in range(3):
        for o in outs:
            o.fill_(float("nan"))
        _ = (torch.randn(256, 256, device=dev) @ torch.randn(256, 256, device=dev)).sum().item()  # eager work between replays
        graph.replay()
        torch.cuda.synchronize(dev)
        for name, got, ref in zip(["Y", "dX"] + [n for n, _ in mlp.named_parameters()], outs, eager):
            assert torch.equal(got, ref), f"replay {rep}: {name} differs from the eager step"


@pytest.mark.parametrize("amp_dtype", [torch.float16, torch.bfloat16])
def test_autocast_with_fp32_master_weights(amp_dtype):
    """Mixed-precision training: fp32 parameters, torch.autocast picks the kernel dtype; gradients
    come back in fp32 and match the oracle evaluated on the rounded operands."""
    from triton_gated_mlp import FusedGatedMLP

    dev = _dev()
    c = Case("amp", 384, 256, 640, amp_dtype, bias=True, backward=True, seed=41)
    t = make_inputs(c)  # values already representable in amp_dtype
    mlp = FusedGatedMLP(c.K, c.N, bias=True).to(dev).float()
    with torch.no_grad():
        for name, key in (("gate_proj", "gate"), ("up_proj", "up"), ("down_proj", "down")):
            getattr(mlp, name).weight.copy_(t[f"W_{key}"].float())
            getattr(mlp, name).bias.copy_(t[f"b_{key}"].float())
    x = t["x"].float().to(dev).requires_grad_(True)
    with torch.autocast("cuda", dtype=amp_dtype):
        y = mlp(x)
    assert y.dtype == amp_dtype
    params = [x] + list(mlp.parameters())
    grads = torch.autograd.grad(y, params, grad_outputs=t["dY"].to(dev))
    assert all(g.dtype == torch.float32 for g in grads), "master-weight gradients must stay fp32"
    o = _oracle_inputs(t)
    ref = oracle.backward(o["x"], o["W_gate"], o["b_gate"], o["W_up"], o["b_up"], o["W_down"], o["b_down"], o["dY"])
    _close("Y", y, ref["Y"])
    names = ["dX", "dW_gate", "db_gate", "dW_up", "db_up", "dW_down", "db_down"]
    for n, g in zip(names, grads):
        _close(n, g, ref[n])
