"""cml_matmul_f32_static (the entry point that allocates nothing) against cml_matmul_f32,
through the C ABI: same bits, on two calls in a row that share the library's static staging
array, the second smaller than the first; sizes beyond the array are refused."""
import numpy as np
import pytest

from camelid_amd import binding as B
from camelid_amd.binding import DeviceBuffer, Weight, check, lib
from tests import gpu_util as G

pytestmark = pytest.mark.gpu

STATIC_BYTES = 1024 * 1024 + 128 * 1024  # CML_STATIC_WORKSPACE_BYTES


def static_matmul(w: Weight, x: np.ndarray) -> np.ndarray:
    n_tokens = x.shape[0]
    xd = DeviceBuffer.from_numpy(x)
    od = DeviceBuffer(n_tokens * w.rows * 4)
    od.fill(0xFF)
    check(lib().cml_matmul_f32_static(w.handle, xd.ptr, n_tokens, od.ptr, None), "cml_matmul_f32_static")
    check(lib().cml_stream_sync(None))
    return od.to_numpy(np.float32, (n_tokens, w.rows))


@pytest.mark.parametrize("fmt_name,rows,cols", [("Q4_K", 512, 4096), ("Q8_0", 384, 2048), ("Q4_0", 320, 1024), ("Q6_K", 256, 2048)])
def test_static_workspace_call_equals_the_workspace_call(fmt_name, rows, cols):
    fmt = B.FORMATS[fmt_name]
    B.init(0)
    wire = G.synth_weight(fmt, rows, cols, seed=11)
    w = Weight.upload(fmt, rows, cols, wire)
    rng = np.random.default_rng(5)
    # the second call is smaller: it must not see what the first one left in the shared array
    for n_tokens in (16, 4, 64, 3, 1):
        G.say(f"cml_matmul_f32_static {fmt_name} {rows}x{cols} tokens={n_tokens}")
        x = rng.standard_normal((n_tokens, cols)).astype(np.float32)
        want = G.gpu_matmul_f32(w, x)
        got = static_matmul(w, x)
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_static_workspace_refuses_what_does_not_fit():
    B.init(0)
    L = lib()
    fmt, rows, cols = B.CML_Q8_0, 32, 16384
    w = Weight.upload(fmt, rows, cols, G.synth_weight(fmt, rows, cols, seed=3))
    n_fit = 64
    assert L.cml_matmul_workspace_bytes(fmt, cols, n_fit) == STATIC_BYTES
    n_over = n_fit + 1
    xd = DeviceBuffer(n_over * cols * 4)
    xd.fill(0)
    od = DeviceBuffer(n_over * rows * 4)
    G.say(f"cml_matmul_f32_static refusal: {n_over} tokens of {cols} values")
    rc = L.cml_matmul_f32_static(w.handle, xd.ptr, n_over, od.ptr, None)
    assert rc == 3, rc  # CML_ERR_SHAPE
    assert b"static workspace" in L.cml_last_error()
    G.say(f"cml_matmul_f32_static at the limit: {n_fit} tokens of {cols} values")
    check(L.cml_matmul_f32_static(w.handle, xd.ptr, n_fit, od.ptr, None), "cml_matmul_f32_static")
    check(L.cml_stream_sync(None))
    assert np.all(od.to_numpy(np.float32, (n_fit, rows)) == 0)
    assert L.cml_matmul_f32_static(None, xd.ptr, 1, od.ptr, None) == 2  # CML_ERR_INVALID
