"""The entry point that allocates nothing (gmlp_colsum_static: partial sums in a static device
array of the library) against the entry point it is a variant of (gmlp_colsum with a caller's
workspace), through the C ABI: bit-identical, on two calls in a row of which the second is smaller,
and against the fp64 column sums of the same rounded inputs."""

import pytest
import torch

pytestmark = pytest.mark.gpu


def _call_pair(lib, _cabi, a, dev):
    M, C = a.shape
    code = _cabi.dtype_code(a.dtype)
    stream = _cabi.stream_ptr(dev)
    out_static = torch.full((C,), float("nan"), dtype=a.dtype, device=dev)
    out_ws = torch.full((C,), float("nan"), dtype=a.dtype, device=dev)
    ws = torch.empty((lib.gmlp_workspace_bytes(_cabi.GMLP_OP_COLSUM, M, 0, C, code),), dtype=torch.uint8, device=dev)
    torch.cuda.synchronize(dev)
    # torch's counter only sees torch's caching allocator; free device memory as the driver reports
    # it also moves when the library itself calls hipMalloc (gmlp_init has run: nothing is set up lazily)
    before, free_before = torch.cuda.memory_allocated(dev), torch.cuda.mem_get_info(dev)[0]
    _cabi.check(lib.gmlp_colsum_static(a.data_ptr(), out_static.data_ptr(), M, C, code, stream))
    torch.cuda.synchronize(dev)
    assert torch.cuda.memory_allocated(dev) == before
    assert torch.cuda.mem_get_info(dev)[0] == free_before, "free device memory changed across gmlp_colsum_static"
    _cabi.check(lib.gmlp_colsum(a.data_ptr(), out_ws.data_ptr(), ws.data_ptr(), M, C, code, stream))
    torch.cuda.synchronize(dev)
    return out_static, out_ws


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
def test_colsum_static_equals_colsum_on_two_calls_in_a_row(dtype):
    from triton_gated_mlp import _cabi

    assert torch.cuda.is_available(), "GPU tests need a visible AMD GPU"
    dev = torch.device("cuda", 0)
    lib = _cabi.lib()
    with torch.cuda.device(dev):
        _cabi.check(lib.gmlp_init())
        g = torch.Generator().manual_seed(11)
        # the second call is smaller in both directions: it must not see what the first left behind
        for M, C in [(3000, 5632), (77, 264), (2048, 32768), (1, 8)]:
            print(f"colsum_static M={M} C={C} {dtype}", flush=True)
            a = torch.randn(M, C, generator=g).to(dtype).to(dev)
            got, ref = _call_pair(lib, _cabi, a, dev)
            assert torch.equal(got, ref), f"M={M} C={C}: differs from gmlp_colsum"
            exact = a.double().sum(0).cpu()
            tol = 2e-2 if dtype != torch.float32 else 1e-4
            assert torch.allclose(got.double().cpu(), exact, rtol=tol, atol=tol * max(1.0, M ** 0.5))
        a = torch.zeros(8, 32768 + 8, dtype=dtype, device=dev)
        out = torch.empty(32768 + 8, dtype=dtype, device=dev)
        rc = lib.gmlp_colsum_static(a.data_ptr(), out.data_ptr(), 8, 32768 + 8, _cabi.dtype_code(dtype), _cabi.stream_ptr(dev))
        assert rc == -2 and "32768" in lib.gmlp_last_error().decode()
