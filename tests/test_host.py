"""Host-side checks that need no GPU: the C ABI loads and exports what include/gmlp.h declares,
argument validation returns error codes before any device work, and the Python surface mirrors the
reference's module/operator interface."""

import ctypes
import re
from pathlib import Path

import pytest
import torch

ROOT = Path(__file__).resolve().parent.parent

from triton_gated_mlp import _cabi  # noqa: E402
import triton_gated_mlp as tgm  # noqa: E402
from triton_gated_mlp.gated_mlp import ACT_FWD, EagerGatedMLP, FusedGatedMLP  # noqa: E402
from triton_gated_mlp.utils import copy_weights, get_device  # noqa: E402


def _declared_symbols():
    text = (ROOT / "include" / "gmlp.h").read_text()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(gmlp_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = _cabi.lib()
    declared = _declared_symbols()
    assert len(declared) >= 12
    for name in declared:
        assert hasattr(lib, name), f"libgmlp.so does not export {name}"
    assert sorted(_cabi.EXPORTED_SYMBOLS) == declared, "ctypes signature table and gmlp.h disagree"
    assert lib.gmlp_abi_version() == 8


def _buf(nbytes=4096):
    raw = ctypes.create_string_buffer(nbytes + 64)
    addr = (ctypes.addressof(raw) + 63) & ~63
    return raw, addr


def test_argument_validation_returns_codes_without_touching_the_device():
    lib = _cabi.lib()
    _, a = _buf()
    err = lambda: lib.gmlp_last_error().decode()
    # NULL pointer
    assert lib.gmlp_linear_fwd(None, a, None, a, 8, 8, 8, 0, None, 0, None) == -1 and "NULL" in err()
    # bad dtype; float32 is not available for the skinny-M kernels
    assert lib.gmlp_linear_fwd(a, a, None, a, 8, 8, 8, 7, None, 0, None) == -1 and "dtype" in err()
    assert lib.gmlp_decode_fwd(a, a, a, a, None, None, None, a, a, None, 16, 256, 256, 2, 0, None) == -2
    # shape: K not a multiple of 8, M < 1
    assert lib.gmlp_linear_fwd(a, a, None, a, 8, 12, 8, 0, None, 0, None) == -2 and "multiple of 8" in err()
    assert lib.gmlp_gateup_fwd(a, a, a, None, None, a, None, None, None, 0, 8, 8, 0, 0, 0.0, 0, 0, None, 0, None) == -2
    # alignment
    assert lib.gmlp_linear_fwd(a + 2, a, None, a, 8, 8, 8, 0, None, 0, None) == -3 and "aligned" in err()
    # dropout probability outside [0, 1)
    assert lib.gmlp_gateup_fwd(a, a, a, None, None, a, None, None, None, 8, 8, 8, 0, 0, 1.0, 0, 0, None, 0, None) == -1
    assert lib.gmlp_gateup_fwd(a, a, a, None, None, a, None, None, None, 8, 8, 8, 0, 0, -0.1, 0, 0, None, 0, None) == -1
    assert lib.gmlp_dropout_mask(a, 8, 8, float("nan"), 0, 0, None) == -1
    # activation code outside the GMLP_ACT_* range
    assert lib.gmlp_gateup_fwd(a, a, a, None, None, a, None, None, None, 8, 8, 8, 0, 7, 0.0, 0, 0, None, 0, None) == -1
    assert "act" in err()
    assert lib.gmlp_gating_bwd(a, a, a, a, a, 8, 8, 0, -1, 0.0, 0, 0, None) == -1
    # decode limits
    assert lib.gmlp_decode_fwd(a, a, a, a, None, None, None, a, a, None, 17, 256, 256, 0, 0, None) == -2 and "16" in err()
    assert lib.gmlp_decode_fwd(a, a, a, a, None, None, None, a, a, None, 16, 40, 256, 0, 0, None) == -2
    assert lib.gmlp_decode_fwd(a, a, a, a, None, None, None, a, a, None, 16, 256, 128, 0, 0, None) == -2
    for fn, args in [
        (lib.gmlp_dh_bwd, (a, a, a, None, a, a, 8, 8, 8, 0, 0, 0.0, 0, 0, None, 0, None)),
        (lib.gmlp_gating_bwd, (a, a, a, a, None, 8, 8, 0, 0, 0.0, 0, 0, None)),
        (lib.gmlp_dx_bwd, (a, a, a, a, None, 8, 8, 8, 0, None, 0, None)),
        (lib.gmlp_dw_bwd, (a, None, a, 8, 8, 8, 0, None, 0, None)),
        (lib.gmlp_colsum, (a, a, None, 8, 8, 0, None)),
    ]:
        assert fn(*args) == -1
    # the entry point without a workspace rejects more columns than its static array holds
    assert lib.gmlp_colsum_static(a, a, 8, 32768 + 8, 0, None) == -2 and "32768" in err()
    assert lib.gmlp_colsum_static(a, None, 8, 64, 0, None) == -1
    assert lib.gmlp_colsum_static(a, a, 8, 12, 0, None) == -2
    assert lib.gmlp_workspace_bytes(_cabi.GMLP_OP_COLSUM, 100, 0, 64, 0) == 64 * 64 * 4
    assert lib.gmlp_workspace_bytes(_cabi.GMLP_OP_DECODE_FWD, 16, 8192, 28672, 0) == 0
    # split reduction: asked for by short batches with a long reduction only, never for float32
    assert lib.gmlp_workspace_bytes(_cabi.GMLP_OP_LINEAR_FWD, 8192, 14336, 4096, 0) == 0
    assert lib.gmlp_workspace_bytes(_cabi.GMLP_OP_DX_BWD, 8192, 4096, 14336, 0) == 0
    assert lib.gmlp_workspace_bytes(_cabi.GMLP_OP_LINEAR_FWD, 64, 28672, 8192, 2) == 0
    n = lib.gmlp_workspace_bytes(_cabi.GMLP_OP_LINEAR_FWD, 64, 28672, 8192, 0)
    assert n > 0 and n % (64 * 8192 * 4) == 0 and 2 <= n // (64 * 8192 * 4) <= 16
    n = lib.gmlp_workspace_bytes(_cabi.GMLP_OP_DX_BWD, 300, 4096, 14336, 1)
    assert n > 0 and n % (300 * 4096 * 4) == 0
    # gate/up: two accumulator sets per split; only when its 128 x 64 tiles leave the chip half idle
    n = lib.gmlp_workspace_bytes(_cabi.GMLP_OP_GATEUP_FWD, 64, 5120, 13824, 0)
    assert n > 0 and n % (2 * 64 * 13824 * 4) == 0
    assert lib.gmlp_workspace_bytes(_cabi.GMLP_OP_GATEUP_FWD, 64, 8192, 28672, 0) == 0
    assert lib.gmlp_workspace_bytes(_cabi.GMLP_OP_GATEUP_FWD, 8192, 4096, 14336, 0) == 0
    # stream-K: asked for by grids of large tiles that end in a thinly filled round while the
    # reduction is long (256 compute units assumed without a GPU): 1.5 rounds of the down
    # projection share out 128 tiles over 256 workgroups, 384 slots of 256 x 256 floats
    assert lib.gmlp_workspace_bytes(_cabi.GMLP_OP_LINEAR_FWD, 6144, 14336, 4096, 0) == 384 * 65536 * 4
    assert lib.gmlp_workspace_bytes(_cabi.GMLP_OP_DW_BWD, 8192, 4096, 14336, 0) == 384 * 65536 * 4  # 3.5 rounds
    assert lib.gmlp_workspace_bytes(_cabi.GMLP_OP_DH_BWD, 8192, 4096, 14336, 0) == 0  # 7 whole rounds
    assert lib.gmlp_workspace_bytes(_cabi.GMLP_OP_DH_BWD, 2048, 2048, 5632, 1) == 0  # short reduction: not worth it
    assert lib.gmlp_workspace_bytes(_cabi.GMLP_OP_DW_BWD_GROUPED, 0, 0, 0, 0) == 512 * 65536 * 4
    assert lib.gmlp_workspace_bytes(_cabi.GMLP_OP_DW_BWD_GROUPED, 0, 0, 0, 2) == 0


def test_whole_pass_entry_points_validate_before_touching_the_device():
    """gmlp_mlp_fwd / gmlp_mlp_bwd: one call per pass.  Their own argument checks (and the workspace
    plan) run on the host before anything is enqueued."""
    lib = _cabi.lib()
    _, a = _buf()
    err = lambda: lib.gmlp_last_error().decode()
    fwd = lambda *ptrs, M=8, K=8, N=8, dt=0, act=0, p=0.0: lib.gmlp_mlp_fwd(*ptrs, M, K, N, dt, act, p, 0, 0, None, 0, None)
    full = (a, a, a, a, None, None, None, a, a, None, None)  # x, wg, wu, wd, biases, y, h, g_save, u_save
    for missing in (0, 1, 2, 3, 7, 8):  # x, the three weights, y, h
        ptrs = list(full)
        ptrs[missing] = None
        assert fwd(*ptrs) == -1 and "NULL" in err() and "gmlp_mlp_fwd" in err()
    assert fwd(*full, dt=5) == -1 and "dtype" in err()
    assert fwd(*full, act=9) == -1 and "act" in err()
    assert fwd(*full, p=1.0) == -1
    assert fwd(*full, K=12) == -2 and "multiple of 8" in err()
    assert fwd(*full, M=0) == -2
    misaligned = list(full)
    misaligned[4] = a + 2  # b_gate
    assert fwd(*misaligned) == -3 and "b_gate" in err()

    def bwd(dy=a, x=a, wg=a, wu=a, wd=a, g=a, u=a, h=a, dg=a, du=a, dx=a, dwg=a, dwu=a, dwd=a, dbg=None, dbu=None,
            dbd=None, M=8, K=8, N=8, dt=0, act=0, p=0.0, ws=None, nws=0):
        return lib.gmlp_mlp_bwd(dy, x, wg, wu, wd, g, u, h, dg, du, dx, dwg, dwu, dwd, dbg, dbu, dbd, M, K, N, dt, act, p,
                                0, 0, ws, nws, None)

    assert bwd(dy=None) == -1 and "'dy'" in err() and "gmlp_mlp_bwd" in err()
    # what a requested output needs must be there ...
    assert bwd(g=None) == -1 and "'g'" in err()
    assert bwd(dg=None) == -1 and "'dg'" in err()
    assert bwd(wd=None) == -1 and "'w_down'" in err()
    assert bwd(x=None) == -1 and "'x'" in err()
    assert bwd(h=None) == -1 and "'h'" in err()
    assert bwd(wg=None) == -1 and "'w_gate'" in err()
    # ... bad codes and shapes are refused like everywhere else
    assert bwd(dt=3) == -1 and bwd(act=-1) == -1 and bwd(p=float("nan")) == -1
    assert bwd(N=20) == -2 and bwd(M=0) == -2
    assert bwd(dx=a + 4) == -3 and "'dx'" in err()
    # bias gradients need the workspace (their partial sums live there); the others do without
    assert bwd(dbg=a) == -1 and "workspace" in err()
    # workspace plan: forward = the larger of its two launches; backward = the largest of its launches' requests
    q = lib.gmlp_workspace_bytes
    assert lib.gmlp_mlp_workspace_bytes(_cabi.GMLP_PASS_FWD, 64, 8192, 28672, 0) == max(
        q(_cabi.GMLP_OP_GATEUP_FWD, 64, 8192, 28672, 0), q(_cabi.GMLP_OP_LINEAR_FWD, 64, 28672, 8192, 0)) > 0
    assert lib.gmlp_mlp_workspace_bytes(_cabi.GMLP_PASS_FWD, 8192, 4096, 14336, 0) == 0
    cs = lambda M, C: q(_cabi.GMLP_OP_COLSUM, M, 0, C, 0)
    M, K, N = 8192, 4096, 14336  # nothing for dH / dX, stream-K for the grouped weight gradients, column sums
    assert lib.gmlp_mlp_workspace_bytes(_cabi.GMLP_PASS_BWD, M, K, N, 0) == max(384 * 65536 * 4, 2 * cs(M, N) + cs(M, K))
    M, K, N = 300, 4096, 14336  # a short batch: split reduction for dX
    assert lib.gmlp_mlp_workspace_bytes(_cabi.GMLP_PASS_BWD, M, K, N, 1) >= q(_cabi.GMLP_OP_DX_BWD, M, K, N, 1) > 0
    assert lib.gmlp_mlp_workspace_bytes(7, 8, 8, 8, 0) == 0 and lib.gmlp_mlp_workspace_bytes(0, 0, 8, 8, 0) == 0


def test_activation_tables_of_the_reference_are_importable():
    """ACT2CLS / ACT2FN / ClassInstantier (src/triton_gated_mlp/gated_mlp.py:10-26): name -> module
    class, and a table whose lookup instantiates."""
    from triton_gated_mlp.gated_mlp import ACT2CLS, ACT2FN, ClassInstantier

    assert set(ACT2CLS) == {"gelu", "leaky_relu", "relu", "sigmoid", "silu", "swish", "tanh"}
    assert ACT2CLS["swish"] is torch.nn.SiLU and ACT2CLS["gelu"] is torch.nn.GELU
    a, b = ACT2FN["silu"], ACT2FN["silu"]
    assert isinstance(a, torch.nn.SiLU) and a is not b
    table = ClassInstantier({"leaky": (torch.nn.LeakyReLU, {"negative_slope": 0.2})})
    assert table["leaky"].negative_slope == 0.2
    with pytest.raises(KeyError):
        ACT2FN["no_such_act"]


def test_error_codes_map_to_python_exceptions():
    lib = _cabi.lib()
    _, a = _buf()
    with pytest.raises(NotImplementedError, match="multiple of 8"):
        _cabi.check(lib.gmlp_linear_fwd(a, a, None, a, 8, 12, 8, 0, None, 0, None))
    with pytest.raises(ValueError, match="NULL"):
        _cabi.check(lib.gmlp_linear_fwd(None, a, None, a, 8, 8, 8, 0, None, 0, None))
    with pytest.raises(TypeError, match="float16, bfloat16 or float32"):
        _cabi.dtype_code(torch.float64)
    assert [_cabi.dtype_code(t) for t in (torch.float16, torch.bfloat16, torch.float32)] == [0, 1, 2]


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    monkeypatch.setenv("GMLP_LIB", str(tmp_path / "nope.so"))
    monkeypatch.setattr(_cabi, "_lib", None)
    with pytest.raises(RuntimeError, match="no fallback"):
        _cabi.lib()


def test_module_surface_matches_reference():
    """ctor kwargs, attributes and parameter names of src/triton_gated_mlp/gated_mlp.py:203-220."""
    m = FusedGatedMLP(hidden_size=64, intermediate_size=128, dropout_p=0.1, bias=True)
    names = [n for n, _ in m.named_parameters()]
    assert names == ["gate_proj.weight", "gate_proj.bias", "up_proj.weight", "up_proj.bias", "down_proj.weight",
                     "down_proj.bias"]
    assert m.gate_proj.weight.shape == (128, 64) and m.down_proj.weight.shape == (64, 128)
    assert m.hidden_size == 64 and m.intermediate_size == 128 and m.act_fn == "silu" and m.dropout.p == 0.1
    assert isinstance(m.act, torch.nn.SiLU)
    d = FusedGatedMLP()
    assert (d.hidden_size, d.intermediate_size, d.dropout.p) == (256, 512, 0.0) and d.gate_proj.bias is not None
    assert [n for n, _ in FusedGatedMLP(bias=False).named_parameters()] == [
        "gate_proj.weight", "up_proj.weight", "down_proj.weight"]
    assert set(ACT_FWD) >= {"silu", "swish", "gelu", "relu", "no_act"}
    # every activation of the reference's table constructs; an unknown name fails like its dict lookup
    for act in ACT_FWD:
        assert FusedGatedMLP(hidden_act=act).act_fn == act
        assert _cabi.act_code(act) in range(7)
    assert _cabi.act_code("swish") == _cabi.act_code("silu") == 0 and _cabi.act_code("no_act") == 6
    with pytest.raises(KeyError):
        FusedGatedMLP(hidden_act="softplus")
    with pytest.raises(NotImplementedError):
        _cabi.act_code("softplus")
    for name in ("EagerGatedMLP", "FusedGatedMLP", "FusedGatedMLPFunction", "mlp_hidden_states_fwd",
                 "mlp_hidden_states_bwd", "eager_fwd", "eager_bwd", "ACT_FWD"):
        assert hasattr(tgm.gated_mlp, name)


def test_state_dict_interchange_and_copy_weights():
    torch.manual_seed(0)
    e = EagerGatedMLP(32, 64, bias=True)
    f = FusedGatedMLP(32, 64, bias=True)
    f.load_state_dict(e.state_dict())
    for (n1, p1), (n2, p2) in zip(e.named_parameters(), f.named_parameters()):
        assert n1 == n2 and torch.equal(p1, p2)
    g = FusedGatedMLP(32, 64, bias=True)
    copy_weights(e, g)
    assert all(torch.equal(a, b) for a, b in zip(e.parameters(), g.parameters()))
    assert g.gate_proj.weight.data_ptr() != e.gate_proj.weight.data_ptr()
    assert get_device().type in ("cpu", "cuda")


def test_fused_module_has_no_cpu_path():
    m = FusedGatedMLP(64, 128).half()
    with pytest.raises(RuntimeError, match="AMD GPU only"):
        m(torch.randn(4, 64).half())


def test_eager_module_semantics_on_cpu():
    from oracle import eager as oracle

    torch.manual_seed(1)
    e = EagerGatedMLP(16, 24, bias=True).double()
    x = torch.randn(2, 5, 16, dtype=torch.float64)
    y = e(x)
    ref = oracle.forward(x.view(-1, 16), e.gate_proj.weight, e.gate_proj.bias, e.up_proj.weight, e.up_proj.bias,
                         e.down_proj.weight, e.down_proj.bias)["Y"]
    assert y.shape == x.shape and torch.allclose(y.view(-1, 16), ref, atol=1e-12)
    t = torch.randn(7, 16, dtype=torch.float64)
    Wu, Wg, dH = e.up_proj.weight.detach(), e.gate_proj.weight.detach(), torch.randn(7, 24, dtype=torch.float64)
    h = tgm.eager_fwd(t, Wu, None, Wg, None)
    assert torch.allclose(h, oracle.hidden_forward(t, Wg, None, Wu, None)["H"], atol=1e-12)
    dx, dWu, dWg = tgm.eager_bwd(t, Wu, Wg, dH)
    hb = oracle.hidden_backward(dH, t @ Wg.T, t @ Wu.T)
    assert torch.allclose(dx, hb["dU"] @ Wu + hb["dG"] @ Wg, atol=1e-12)
    assert torch.allclose(dWu, hb["dU"].T @ t, atol=1e-12) and torch.allclose(dWg, hb["dG"].T @ t, atol=1e-12)


def test_operator_shape_validation_happens_before_device_checks():
    from triton_gated_mlp.ops.fwd import validate_dimensions

    x, W = torch.zeros(4, 16), torch.zeros(8, 16)
    validate_dimensions(x, W, None, W, None)
    with pytest.raises(ValueError):
        validate_dimensions(torch.zeros(2, 4, 16), W, None, W, None)
    with pytest.raises(ValueError):
        validate_dimensions(x, torch.zeros(8, 12), None, W, None)
    with pytest.raises(ValueError):
        validate_dimensions(x, W, torch.zeros(7), W, None)
    with pytest.raises(NotImplementedError):
        tgm.mlp_hidden_states_fwd(x, W, None, W, None, "softplus", 0.0)


def test_host_activation_forms_match_the_oracle():
    """ops/act.py (names of src/triton_gated_mlp/ops/act.py:5-45) against the oracle's table, which is
    pinned against torch.autograd in test_oracle.py."""
    from oracle import eager as oracle
    from triton_gated_mlp.ops import act

    x = torch.cat([torch.linspace(-6, 6, 49, dtype=torch.float64), torch.zeros(1, dtype=torch.float64)])
    for name, (f, df) in oracle.ACTS.items():
        assert torch.allclose(act._act_fwd(x, name), f(x), atol=1e-12), name
        assert torch.allclose(act._act_bwd(x, name), df(x), atol=1e-12), name
    assert torch.allclose(act._silu_fwd(x), x * act._compute_sigma(x))
    with pytest.raises(NotImplementedError):
        act._act_fwd(x, "softplus")


@pytest.mark.parametrize("M,N,bm,bn,group", [(1024, 512, 128, 128, 4), (8192, 14336, 256, 128, 8), (300, 4104, 128, 64, 8),
                                              (257, 255, 256, 256, 8)])
def test_grouped_tile_order_visits_every_tile_once(M, N, bm, bn, group):
    from triton_gated_mlp.ops.utils import get_num_streaming_multiprocessors, map_pid_m_n

    tiles_m, tiles_n = -(-M // bm), -(-N // bn)
    for l2 in (True, False):
        seen = {map_pid_m_n(pid, M, N, bm, bn, group, l2) for pid in range(tiles_m * tiles_n)}
        assert seen == {(i, j) for i in range(tiles_m) for j in range(tiles_n)}
    # inside a group the walk is column-major: consecutive programs share the tile column
    assert map_pid_m_n(0, M, N, bm, bn, group)[1] == map_pid_m_n(min(group, tiles_m) - 1, M, N, bm, bn, group)[1]
    assert get_num_streaming_multiprocessors() >= 2


def test_small_helpers_of_the_reference_surface():
    from triton_gated_mlp import const, utils

    assert (const.ROOT_PATH / "triton-gated-mlp_amd" / "triton_gated_mlp" / "const.py").exists()
    a = torch.arange(12.0).reshape(3, 4)
    assert utils.validate_contiguous(a) is a
    assert utils.validate_contiguous(a.T).is_contiguous() and torch.equal(utils.validate_contiguous(a.T), a.T)
    with pytest.raises(RuntimeError, match="GPU"):
        utils.validate_tensor_device(a)


def test_max_rows_32bit_keeps_padded_operands_below_2_gib():
    """The module's chunk size for very tall batches: a multiple of 256 whose [rows, max(K, N)]
    operand, padded to whole 256-tiles, stays addressable with 32-bit byte offsets, and the next
    multiple of 256 does not."""
    from triton_gated_mlp.ops.fwd import max_rows_32bit

    limit = (1 << 31) - 4096
    for K, N in [(4096, 14336), (8192, 28672), (4096, 11008), (5120, 13824), (8, 8), (100, 72)]:
        for dtype in (torch.float16, torch.bfloat16):
            rows = max_rows_32bit(K, N, dtype)
            width = -(-max(K, N) // 256) * 256
            assert rows % 256 == 0 and rows >= 256
            assert rows * width * 2 < limit
            assert (rows + 256) * width * 2 >= limit
    assert max_rows_32bit(8192, 28672, torch.float16) == 37376
    assert max_rows_32bit(4096, 14336, torch.float32) is None


def test_decode_preferred_needs_widths_that_fill_the_chip():
    """Routing of M <= 16 inference between the streaming kernels and the general path."""
    from triton_gated_mlp.ops.fwd import decode_preferred

    for K, N in [(8192, 28672), (4096, 14336), (4096, 11008), (5120, 13824), (6144, 16384), (2048, 8192)]:
        assert all(decode_preferred(M, K, N) for M in (1, 8, 9, 16)), (K, N)
    assert decode_preferred(17, 8192, 28672) and decode_preferred(32, 4096, 14336)  # two token tiles
    assert not decode_preferred(33, 8192, 28672)  # beyond the skinny-M kernels
    assert decode_preferred(16, 2560, 10240) and not decode_preferred(17, 2560, 10240)  # two tiles want wider models
    assert decode_preferred(24, 3584, 18944)
    assert not decode_preferred(1, 4096 + 64, 14336)  # K must be a multiple of 256 for the streaming kernels
    assert not decode_preferred(1, 1024, 2048)  # fewer W_gate/W_up blocks than compute units
    assert not decode_preferred(1, 1024, 8192)  # a quarter of a W_down block per compute unit
    assert not decode_preferred(1, 8192, 28672, torch.float32)


def test_async_load_checker_flags_registers_touched_before_their_wait(tmp_path):
    """The build-time check of the streaming kernels' assembly: a load's destination registers may
    not be named by any instruction before the s_waitcnt that covers the load (in-order return: a
    wait for N leaves only the N youngest loads in flight; loads into LDS have no destination)."""
    import importlib.util

    spec = importlib.util.spec_from_file_location(
        "check_async_loads", ROOT / "triton-gated-mlp_amd" / "csrc" / "check_async_loads.py"
    )
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)

    good = tmp_path / "good.s"
    good.write_text(
        "_Z4kernv:\n"
        "\tbuffer_load_dwordx4 v[4:7], v1, s[0:3], s8 offen\n"
        "\tbuffer_load_dwordx4 v2, s[0:3], s8 offen lds\n"
        "\tbuffer_load_dwordx4 v[8:11], v1, s[0:3], s9 offen\n"
        "\tv_add_u32_e32 v1, 16, v1\n"            # the address register is free to change
        "\ts_waitcnt vmcnt(1)\n"                   # retires the first two loads
        "\tv_accvgpr_write_b32 a0, v4\n"
        "\ts_waitcnt vmcnt(0)\n"
        "\tv_mfma_f32_16x16x32_f16 a[0:3], v[4:7], v[8:11], a[0:3]\n"
        "\ts_endpgm\n"
    )
    assert mod.check(str(good)) == 0
    bad = tmp_path / "bad.s"
    bad.write_text(
        "_Z4kernv:\n"
        "\tbuffer_load_dwordx4 v[4:7], v1, s[0:3], s8 offen\n"
        "\tbuffer_load_dwordx4 v[8:11], v1, s[0:3], s9 offen\n"
        "\ts_waitcnt vmcnt(1)\n"
        "\tv_accvgpr_write_b32 a1, v9\n"           # the second load is still in flight
        "\ts_waitcnt vmcnt(0)\n"
        "\ts_endpgm\n"
        "_Z5kern2v:\n"
        "\ts_endpgm\n"
    )
    assert mod.check(str(bad)) == 1


def test_m0_checker_flags_compiler_generated_m0_uses(tmp_path):
    """csrc/check_m0.py (run on every GEMM unit by the build): M0 written inside the inline-assembly
    blocks is the kernels' own; a write or an implied use outside them, in a kernel that holds
    global->LDS loads, fails the build.  Kernels without such loads are not its business."""
    import importlib.util

    spec = importlib.util.spec_from_file_location("check_m0", ROOT / "triton-gated-mlp_amd" / "csrc" / "check_m0.py")
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    dma = "\t;;#ASMSTART\n\ts_mov_b32 m0, s4\n\ts_nop 0\n\t;;#ASMEND\n\t;;#ASMSTART\n\tbuffer_load_dwordx4 v1, s[8:11], s2 offen offset:1024 lds\n\t;;#ASMEND\n"
    good = "_Z4kern:\n" + dma + "\tv_mfma_f32_16x16x32_f16 a[0:3], v[0:3], v[4:7], a[0:3]\n\ts_endpgm\n"
    bad_write = "_Z4kern:\n" + dma + "\ts_mov_b32 m0, s9\n\ts_endpgm\n"
    bad_use = "_Z4kern:\n" + dma + "\tv_movrels_b32_e32 v0, v1\n\ts_endpgm\n"
    other = "_Z5plain:\n\ts_mov_b32 m0, s9\n\ts_endpgm\n"
    for text, expect in ((good, 0), (bad_write, 1), (bad_use, 1), (good + other, 0), (other + bad_write, 1)):
        f = tmp_path / "k.s"
        f.write_text(text)
        assert mod.check(str(f)) == expect
    # A unit in which the scan recognises no kernel with such loads has verified nothing: that
    # fails as well (kernel labels or inline-assembly markers the scan no longer matches), unless
    # the caller says the file is expected to have none.
    unmarked = "_Z4kern:\n\tbuffer_load_dwordx4 v1, s[8:11], s2 offen offset:1024 lds\n\ts_mov_b32 m0, s9\n\ts_endpgm\n"
    relabelled = good.replace("_Z4kern:", "kern$local:")
    for text in (other, unmarked, relabelled, ""):
        f = tmp_path / "k.s"
        f.write_text(text)
        assert mod.check(str(f)) == 1
        assert mod.check(str(f), minimum=0) == 0
    f.write_text(good)
    assert mod.check(str(f), minimum=2) == 1
