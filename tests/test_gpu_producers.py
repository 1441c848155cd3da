"""Fused producers on the device: rms_norm -> Q8_0 / Q8_K and silu(gate)*up -> Q8_0 / Q8_K,
through the C ABI, against the CPU oracle.  Bars: normalised f32 rows bit-exact (the kernel keeps
the reference's left-to-right sum of squares), quantized outputs bit-exact, fused == composed
(the reference's own claim, src/cuda_resident/tests.rs:4114-4190).  silu uses expf: its f32
values may differ from the host libm in the last bit, so that path is checked as fused ==
device-composed bit for bit and against the oracle within 1 quantization step."""
import numpy as np
import pytest

import oracle
from camelid_amd import binding as B
from camelid_amd.binding import DeviceBuffer, check, lib
from tests import gpu_util as G

pytestmark = pytest.mark.gpu

ACT_F32, ACT_Q8_0, ACT_Q8_K = 0, 1, 2


def setup_module(_m):
    B.init(0)


def gpu_rms_norm_quantize(act, x, w, eps, want_normed=True):
    n, cols = x.shape
    xd, wd = DeviceBuffer.from_numpy(x), DeviceBuffer.from_numpy(w)
    nd = DeviceBuffer(n * cols * 4) if want_normed else None
    per = 256 if act == ACT_Q8_K else 32
    qd = DeviceBuffer(n * cols) if act != ACT_F32 else None
    sd = DeviceBuffer(n * (cols // per) * 4) if act != ACT_F32 else None
    for b in (nd, qd, sd):
        if b is not None:
            b.fill(0xEE)
    check(lib().cml_rms_norm_quantize(act, xd.ptr, wd.ptr, eps, n, cols, nd.ptr if nd else None,
                                      qd.ptr if qd else None, sd.ptr if sd else None, None), "cml_rms_norm_quantize")
    check(lib().cml_stream_sync(None))
    normed = nd.to_numpy(np.float32, (n, cols)) if nd else None
    q = qd.to_numpy(np.int8, (n, cols)) if qd else None
    s = sd.to_numpy(np.float32, (n, cols // per)) if sd else None
    return normed, s, q


def _rows(n, cols, seed):
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((n, cols)).astype(np.float32)
    x[0] *= 37.0
    if n > 1:
        x[1, : cols // 2] = 0.0
    if n > 2:
        x[2, 0], x[2, 1:] = 4096.0, 1.0     # summation order decides the scale here
    w = (rng.standard_normal(cols) * 0.5 + 1.0).astype(np.float32)
    return x, w


@pytest.mark.parametrize("cols", [256, 2048, 2816, 4096, 14336])
def test_rms_norm_rows_are_bit_exact(cols):
    x, w = _rows(5, cols, 900 + cols)
    for eps in (1e-5, 1e-6, 0.0):
        G.say(f"rms_norm cols={cols} eps={eps}")
        got, _, _ = gpu_rms_norm_quantize(ACT_F32, x, w, eps)
        assert G.same_bits(got, oracle.rms_norm(x, w, eps))


@pytest.mark.parametrize("cols", [256, 2816, 4096, 14336])
def test_rms_norm_quantize_is_the_composed_result(cols):
    x, w = _rows(4, cols, 950 + cols)
    eps = 1e-6
    want_normed = oracle.rms_norm(x, w, eps)
    for act, per in ((ACT_Q8_0, 32), (ACT_Q8_K, 256)):
        if cols % per:
            continue
        G.say(f"rms_norm_quantize cols={cols} act={act}")
        normed, s, q = gpu_rms_norm_quantize(act, x, w, eps)
        assert G.same_bits(normed, want_normed)
        so, qo = (oracle.quantize_q8_0 if act == ACT_Q8_0 else oracle.quantize_q8_k)(want_normed)
        assert np.array_equal(q, qo) and np.array_equal(s.view(np.uint32), so.view(np.uint32))
        # the quantized form alone (no f32 round trip) and the separate device quantizer agree too
        _, s2, q2 = gpu_rms_norm_quantize(act, x, w, eps, want_normed=False)
        assert np.array_equal(q2, q) and np.array_equal(s2.view(np.uint32), s.view(np.uint32))
        s3, q3 = G.gpu_quantize(act == ACT_Q8_K, normed)
        assert np.array_equal(q3, q) and np.array_equal(s3.view(np.uint32), s.view(np.uint32))


def test_silu_mul_quantize():
    rng = np.random.default_rng(990)
    for n, cols in ((1, 14336), (3, 2048), (5, 256)):
        g = (rng.standard_normal((n, cols)) * 2).astype(np.float32)
        u = rng.standard_normal((n, cols)).astype(np.float32)
        g[0, :256] = 0.0
        h = oracle.silu_mul(g, u)
        gd, ud = DeviceBuffer.from_numpy(g), DeviceBuffer.from_numpy(u)
        for act, per in ((ACT_Q8_0, 32), (ACT_Q8_K, 256)):
            G.say(f"silu_mul_quantize {n}x{cols} act={act}")
            qd, sd = DeviceBuffer(n * cols), DeviceBuffer(n * (cols // per) * 4)
            check(lib().cml_silu_mul_quantize(act, gd.ptr, ud.ptr, n, cols, qd.ptr, sd.ptr, None), "cml_silu_mul_quantize")
            check(lib().cml_stream_sync(None))
            q = qd.to_numpy(np.int8, (n, cols)).astype(np.int32)
            s = sd.to_numpy(np.float32, (n, cols // per))
            so, qo = (oracle.quantize_q8_0 if act == ACT_Q8_0 else oracle.quantize_q8_k)(h)
            # expf on the device vs the host libm: h may differ in its last bit, hence at most one step
            assert np.max(np.abs(q - qo.astype(np.int32))) <= 1
            assert np.allclose(s, so, rtol=1e-6, atol=0)
            deq = q.reshape(n, cols // per, per) * s[:, :, None]
            assert np.max(np.abs(deq.reshape(n, cols) - h)) <= np.max(np.abs(s)) * 1.01 + 1e-12


def test_producer_error_paths():
    L = lib()
    d = DeviceBuffer(4096)
    assert L.cml_rms_norm_quantize(7, d.ptr, d.ptr, 1e-6, 1, 256, d.ptr, d.ptr, d.ptr, None) == 2
    assert L.cml_rms_norm_quantize(ACT_Q8_K, d.ptr, d.ptr, 1e-6, 1, 224, d.ptr, d.ptr, d.ptr, None) == 3
    assert L.cml_rms_norm_quantize(ACT_Q8_0, d.ptr, d.ptr, 1e-6, 1, 256, None, None, None, None) == 2
    assert L.cml_rms_norm_quantize(ACT_F32, d.ptr, d.ptr, 1e-6, 1, 32768, d.ptr, None, None, None) == 6   # row too long to stage
    assert L.cml_silu_mul_quantize(ACT_F32, d.ptr, d.ptr, 1, 256, d.ptr, d.ptr, None) == 2
    assert L.cml_rms_norm_quantize(ACT_F32, d.ptr, d.ptr, 1e-6, 0, 256, d.ptr, None, None, None) == 0
