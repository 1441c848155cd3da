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


def _ordered_sum_rows(cols, rng):
    """Rows that stress the in-order f32 sum of squares: plain, wide dynamic range, exact rounding
    ties, squares that underflow to subnormals, sums that overflow, sparse rows, constant rows with
    a few outliers, descending magnitudes, a large head (every later term is a fraction of an ulp),
    non-finite values."""
    n = cols
    rows = [
        rng.standard_normal(n),
        rng.standard_normal(n) * np.exp(rng.standard_normal(n) * 3),
        np.round(rng.standard_normal(n) * 8) / 8,
        np.round(rng.standard_normal(n) * 2) / 2 * 1024.0,
        rng.standard_normal(n) * 1e-20,
        rng.standard_normal(n) * 1e-23,
        rng.standard_normal(n) * 1e18,
        np.where(rng.random(n) < 0.9, 0.0, rng.standard_normal(n)),
        np.full(n, 1.5) * (1 + (rng.random(n) < 0.01)),
        np.full(n, 1.0),
        np.sort(np.abs(rng.standard_normal(n)))[::-1] * 1000.0,
        np.sort(np.abs(rng.standard_normal(n))) * 0.001,
        np.concatenate([[4096.0], np.ones(n - 1)]),
        np.concatenate([[1e10], rng.standard_normal(n - 1)]),
        np.zeros(n),
        np.concatenate([np.zeros(n - 1), [3.0]]),
        # sums that sit on or next to a power of two over a long stretch of small or zero terms
        np.concatenate([np.ones(n // 2), np.zeros(n - n // 2)]),
        np.concatenate([np.ones(n // 2) * 1.0001, np.full(n - n // 2, 1e-4)]),
        np.concatenate([np.ones(n // 2) * 0.9999, np.full(n - n // 2, 3e-3)]),
    ]
    x = np.stack(rows).astype(np.float32)
    extra = rng.standard_normal((3, n)).astype(np.float32)
    extra[0, n // 3] = np.inf
    extra[1, n // 2] = np.nan
    extra[2, min(5, n - 1)], extra[2, max(n - 7, 0)] = np.inf, np.nan
    return np.concatenate([x, extra])


@pytest.mark.parametrize("cols", [4, 64, 256, 1000, 2048, 2816, 4096, 5120, 8192, 14336, 16384])
def test_sum_of_squares_is_the_scalar_loop(cols):
    """cml_sum_squares_f32 adds the squares in parallel and must return the bits of the
    left-to-right scalar loop (the first pass of the reference's rms_norm)."""
    rng = np.random.default_rng(4200 + cols)
    for rep in range(3):
        x = _ordered_sum_rows(cols, rng)
        n = x.shape[0]
        G.say(f"sum of squares cols={cols} rep={rep}")
        xd, od = DeviceBuffer.from_numpy(x), DeviceBuffer(n * 4)
        check(lib().cml_sum_squares_f32(xd.ptr, n, cols, od.ptr, None), "cml_sum_squares_f32")
        check(lib().cml_stream_sync(None))
        got = od.to_numpy(np.float32, (n,))
        with np.errstate(over="ignore", invalid="ignore"):
            sq = (x * x).astype(np.float32)
            want = np.zeros(n, np.float32)
            for c in range(cols):                      # the scalar loop, all rows at once
                want = (want + sq[:, c]).astype(np.float32)
        finite = np.isfinite(want)
        assert np.array_equal(np.isnan(got), np.isnan(want))
        assert G.same_bits(got[~np.isnan(want)], want[~np.isnan(want)]), (cols, rep, np.nonzero(got.view(np.uint32) != want.view(np.uint32))[0][:8])
        assert finite.sum() >= 12


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


@pytest.mark.parametrize("cols", [256, 2816, 4096, 14336])
def test_rms_inv_norm_quantize_with_the_hosts_inverse(cols):
    """The norm with the inverse root-mean-square handed over by the host (the reference's CPU router has
    scanned the row already): value = (x * rms_inv) * weight with both multiplies rounded, then the
    quantizer -- the bits of the numpy float32 expression followed by the oracle's quantizer, on rows
    with zero blocks, rounding ties and the maximum held by both signs."""
    x, w = _rows(3, cols, 960 + cols)
    x[0, :256] = 0.0
    x[1, 5], x[1, 9] = 7.0, -7.0
    w[5], w[9] = 1.0, 1.0
    for r in range(3):
        # the host's scan: the sequential f32 sum of squares, (mean + eps)^-0.5 (reference src/tensor/mod.rs:2707-2760)
        acc = np.float32(0.0)
        for v in x[r]:
            acc = np.float32(acc + np.float32(v * v))
        rms_inv = np.float32(1.0) / np.sqrt(np.float32(acc / np.float32(cols) + np.float32(1e-6)), dtype=np.float32)
        value = ((x[r] * rms_inv).astype(np.float32) * w).astype(np.float32)
        for act, per in ((ACT_Q8_0, 32), (ACT_Q8_K, 256)):
            G.say(f"rms_inv_norm_quantize cols={cols} row={r} act={act}")
            xd, wd = DeviceBuffer.from_numpy(x[r]), DeviceBuffer.from_numpy(w)
            qd, sd = DeviceBuffer(cols), DeviceBuffer(cols // per * 4)
            with G.engaged(r"^producer\.rms_inv_norm\." + ("q8_0" if act == ACT_Q8_0 else "q8_k")):
                check(lib().cml_rms_inv_norm_quantize(act, xd.ptr, wd.ptr, float(rms_inv), cols, qd.ptr, sd.ptr, None), "cml_rms_inv_norm_quantize")
            check(lib().cml_stream_sync(None))
            q, s = qd.to_numpy(np.int8, (cols,)), sd.to_numpy(np.float32, (cols // per,))
            so, qo = (oracle.quantize_q8_0 if act == ACT_Q8_0 else oracle.quantize_q8_k)(value)
            assert np.array_equal(q, qo) and np.array_equal(s.view(np.uint32), so.view(np.uint32))
    assert lib().cml_rms_inv_norm_quantize(ACT_Q8_K, xd.ptr, wd.ptr, 1.0, 100, qd.ptr, sd.ptr, None) != 0   # not whole super-blocks
    assert lib().cml_rms_inv_norm_quantize(ACT_F32, xd.ptr, wd.ptr, 1.0, cols, qd.ptr, sd.ptr, None) != 0   # nothing to quantize into


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


def test_gelu_tanh_mul_quantize():
    """The Gemma-4 expert activation fused with the quantizer (reference geglu_quantize_routed,
    src/cuda_resident.rs:6301-6343).  tanhf on the device vs the host libm: h may differ in its
    last bits, hence at most one quantization step; all-zero blocks stay exact."""
    rng = np.random.default_rng(991)
    for n, cols in ((1, 704), (3, 2048), (8, 256)):
        g = (rng.standard_normal((n, cols)) * 2).astype(np.float32)
        u = rng.standard_normal((n, cols)).astype(np.float32)
        g[0, :256] = 0.0
        h = oracle.gelu_tanh_mul(g, u)
        gd, ud = DeviceBuffer.from_numpy(g), DeviceBuffer.from_numpy(u)
        for act, per in ((ACT_Q8_0, 32), (ACT_Q8_K, 256)):
            if cols % per:
                continue
            G.say(f"glu_quantize gelu_tanh {n}x{cols} act={act}")
            qd, sd = DeviceBuffer(n * cols), DeviceBuffer(n * (cols // per) * 4)
            check(lib().cml_glu_quantize(1, act, gd.ptr, ud.ptr, n, cols, qd.ptr, sd.ptr, None), "cml_glu_quantize")
            check(lib().cml_stream_sync(None))
            q = qd.to_numpy(np.int8, (n, cols)).astype(np.int32)
            s = sd.to_numpy(np.float32, (n, cols // per))
            so, qo = (oracle.quantize_q8_0 if act == ACT_Q8_0 else oracle.quantize_q8_k)(h)
            assert np.max(np.abs(q - qo.astype(np.int32))) <= 1
            assert np.allclose(s, so, rtol=2e-6, atol=0)
            assert not q[0, :256].any() and not s[0, :256 // per].any()
            deq = q.reshape(n, cols // per, per) * s[:, :, None]
            assert np.max(np.abs(deq.reshape(n, cols) - h)) <= np.max(np.abs(s)) * 1.01 + 1e-12
    # the selector 0 is cml_silu_mul_quantize, bit for bit
    g = (rng.standard_normal((2, 512)) * 2).astype(np.float32)
    u = rng.standard_normal((2, 512)).astype(np.float32)
    gd, ud = DeviceBuffer.from_numpy(g), DeviceBuffer.from_numpy(u)
    outs = []
    for call in (lambda q, s: lib().cml_glu_quantize(0, ACT_Q8_K, gd.ptr, ud.ptr, 2, 512, q, s, None),
                 lambda q, s: lib().cml_silu_mul_quantize(ACT_Q8_K, gd.ptr, ud.ptr, 2, 512, q, s, None)):
        qd, sd = DeviceBuffer(1024), DeviceBuffer(16)
        check(call(qd.ptr, sd.ptr))
        check(lib().cml_stream_sync(None))
        outs.append((qd.to_numpy(np.int8, (1024,)), sd.to_numpy(np.float32, (4,))))
    assert np.array_equal(outs[0][0], outs[1][0]) and np.array_equal(outs[0][1], outs[1][1])
    d = DeviceBuffer(4096)
    assert lib().cml_glu_quantize(2, ACT_Q8_0, d.ptr, d.ptr, 1, 256, d.ptr, d.ptr, None) == 2   # unknown activation


def test_producer_error_paths():
    L = lib()
    d = DeviceBuffer(4096)
    assert L.cml_rms_norm_quantize(7, d.ptr, d.ptr, 1e-6, 1, 256, d.ptr, d.ptr, d.ptr, None) == 2
    assert L.cml_rms_norm_quantize(ACT_Q8_K, d.ptr, d.ptr, 1e-6, 1, 224, d.ptr, d.ptr, d.ptr, None) == 3
    assert L.cml_rms_norm_quantize(ACT_Q8_0, d.ptr, d.ptr, 1e-6, 1, 256, None, None, None, None) == 2
    assert L.cml_rms_norm_quantize(ACT_F32, d.ptr, d.ptr, 1e-6, 1, 32768, d.ptr, None, None, None) == 6   # row too long to stage
    assert L.cml_silu_mul_quantize(ACT_F32, d.ptr, d.ptr, 1, 256, d.ptr, d.ptr, None) == 2
    assert L.cml_rms_norm_quantize(ACT_F32, d.ptr, d.ptr, 1e-6, 0, 256, d.ptr, None, None, None) == 0


# ------------------------------------------------- either side of the LM head ----

@pytest.mark.parametrize("name,fmt", [("Q8_0", oracle.Q8_0), ("Q4_0", oracle.Q4_0), ("Q4_K", oracle.Q4_K), ("Q6_K", oracle.Q6_K)])
def test_embed_gather_rows_are_the_block_decode(name, fmt):
    rows, cols = 77, 1024
    wire = G.synth_weight(fmt, rows, cols, seed=1200 + fmt)
    w = B.Weight.upload(fmt, rows, cols, wire)
    ref = oracle.dequant(fmt, wire).reshape(rows, cols)
    ids = np.array([0, 76, 5, 5, 33, 16, 15, 1000, 17], np.uint32)   # 1000 is outside the table
    G.say(f"embed_gather {name}")
    idd = DeviceBuffer.from_numpy(ids)
    out = DeviceBuffer(ids.size * cols * 4)
    out.fill(0)
    check(lib().cml_embed_gather(w.handle, idd.ptr, ids.size, out.ptr, None), "cml_embed_gather")
    check(lib().cml_stream_sync(None))
    got = out.to_numpy(np.float32, (ids.size, cols))
    for k, t in enumerate(ids):
        if t < rows:
            assert G.same_bits(got[k], ref[t]), (k, t)
        else:
            assert np.all(np.isnan(got[k]))
    # a band view gathers relative to the band
    band = w.slice(21, 40)
    check(lib().cml_embed_gather(band.handle, idd.ptr, 3, out.ptr, None), "cml_embed_gather")
    check(lib().cml_stream_sync(None))
    got = out.to_numpy(np.float32, (ids.size, cols))
    assert G.same_bits(got[0], ref[21]) and np.all(np.isnan(got[1])) and G.same_bits(got[2], ref[26])


def test_argmax_first_maximum_wins():
    rng = np.random.default_rng(1300)
    for n in (1, 3, 63, 1024, 1025, 4099, 20483, 128256):
        logits = rng.standard_normal((6, n)).astype(np.float32)
        if n > 3:
            logits[1, n // 2] = logits[1, 1] = 9.0          # equal maxima: the lower index
            logits[2, :] = -np.inf                          # nothing beats the starting value: index 0
            logits[3, 0] = np.nan
            logits[3, n - 1] = 50.0
            logits[4, :] = 2.5                              # all equal
            logits[5, n - 1] = 100.0                        # the very last element
        G.say(f"argmax n={n}")
        ld = DeviceBuffer.from_numpy(logits)
        od = DeviceBuffer(6 * 4)
        check(lib().cml_argmax_f32(ld.ptr, 6, n, od.ptr, None), "cml_argmax_f32")
        check(lib().cml_stream_sync(None))
        got = od.to_numpy(np.uint32, (6,))
        for r in range(6):
            best, besti = np.float32(-3.4e38), 0            # the reference's scan, spelled out
            for i, v in enumerate(logits[r]) if n <= 2048 else ():
                if v > best:
                    best, besti = v, i
            if n > 2048:
                row = np.where(np.isnan(logits[r]), -np.inf, logits[r])
                besti = int(np.argmax(row)) if row.max() > -3.4e38 else 0
            assert got[r] == besti, (n, r, got[r], besti)
    # argmax feeds embed_gather without leaving the device
    rows, cols = 300, 512
    wire = G.synth_weight(oracle.Q6_K, rows, cols, seed=1301)
    w = B.Weight.upload(oracle.Q6_K, rows, cols, wire)
    logits = rng.standard_normal((2, rows)).astype(np.float32)
    ld, od, out = DeviceBuffer.from_numpy(logits), DeviceBuffer(8), DeviceBuffer(2 * cols * 4)
    check(lib().cml_argmax_f32(ld.ptr, 2, rows, od.ptr, None), "cml_argmax_f32")
    check(lib().cml_embed_gather(w.handle, od.ptr, 2, out.ptr, None), "cml_embed_gather")
    check(lib().cml_stream_sync(None))
    ref = oracle.dequant(oracle.Q6_K, wire).reshape(rows, cols)
    got = out.to_numpy(np.float32, (2, cols))
    for r in range(2):
        assert G.same_bits(got[r], ref[int(np.argmax(logits[r]))])
