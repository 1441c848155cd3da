"""Pins for the parts of the oracle the golden dequant fixtures leave open.

Known answers are taken from the reference's own unit tests (cited per test);
the rest are closed forms, invariants, special cases where float arithmetic is
exact, and brute force over independently decoded integers (tests/npref.py,
itself pinned by the golden fixtures).
"""
import numpy as np
import pytest

import oracle
from oracle import Q4_0, Q4_K, Q6_K, Q8_0, ORDER_ALT, ORDER_PRIMARY
from tests import npref


# ---------------------------------------------------------------- f16 ------

def test_f16_to_f32_exhaustive_against_numpy():
    h = np.arange(65536, dtype=np.uint16)
    got = oracle.f16_bits_to_f32_array(h)
    want = h.view(np.float16).astype(np.float32)
    nan = np.isnan(want)
    assert np.array_equal(got.view(np.uint32)[~nan], want.view(np.uint32)[~nan])
    assert np.all(np.isnan(got[nan]))


def test_f32_to_f16_against_numpy_rne():
    rng = np.random.default_rng(1)
    # every exponent, random mantissas, plus all f16 midpoints' neighbourhoods
    bits = rng.integers(0, 2**32, size=4_000_000, dtype=np.uint64).astype(np.uint32)
    h = np.arange(65536, dtype=np.uint16).view(np.float16).astype(np.float32)
    h = h[np.isfinite(h)]
    mids = ((h[:-1].astype(np.float64) + h[1:].astype(np.float64)) / 2).astype(np.float32)
    near = np.concatenate([np.nextafter(mids, np.float32(np.inf)), mids, np.nextafter(mids, np.float32(-np.inf))])
    v = np.concatenate([bits.view(np.float32), near, np.array([0.0, -0.0, 65504.0, 65520.0, 65519.99, 1e-8, 5.96e-8, 2.98e-8, 2.9802322e-8, np.inf, -np.inf], np.float32)])
    v = v[~np.isnan(v)]
    got = oracle.f32_to_f16_bits_array(v)
    with np.errstate(over="ignore"):
        want = v.astype(np.float16).view(np.uint16)
    assert np.array_equal(got, want)
    assert oracle.f32_to_f16_bits(float("nan")) & 0x7fff == 0x7e00


# ------------------------------------------------------- Q8_0 quantize -----

def test_q8_0_quantize_ties_round_away_from_zero():
    # amax = 127 -> unrounded scale 1.0 -> inv 1.0: q = round-half-away(v).
    # (The reference CPU path uses `.round()`, src/inference.rs:22525; ties-to-even would give 2, 0, -2.)
    x = np.zeros(32, np.float32)
    x[0] = 127.0
    x[1:7] = [2.5, 0.5, -0.5, -2.5, 1.5, -1.5]
    s, q = oracle.quantize_q8_0(x)
    assert s[0] == np.float32(1.0)
    assert list(q[:7]) == [127, 3, 1, -1, -3, 2, -2]


def test_q8_0_quantize_inverse_uses_unrounded_scale():
    # amax/127 = 0.1/127 is not f16-representable; q must come from 1/(amax/127), not 1/f16(scale).
    x = np.full(32, 0.05, np.float32)
    x[0] = 0.1
    s, q = oracle.quantize_q8_0(x)
    u = np.float32(0.1) / np.float32(127.0)
    assert s[0] == np.float32(np.float16(u))
    inv = np.float32(1.0) / u
    assert q[0] == 127
    assert q[1] == int(np.floor(np.float64(np.float32(0.05) * inv) + 0.5))


def test_q8_0_quantize_random_against_numpy_restatement():
    rng = np.random.default_rng(2)
    x = rng.standard_normal((64, 2048)).astype(np.float32)
    x[3, 32:64] = 0.0  # an all-zero block
    s, q = oracle.quantize_q8_0(x)
    blk = x.reshape(-1, 32)
    amax = np.abs(blk).max(axis=1)
    u = (amax / np.float32(127.0)).astype(np.float32)
    assert np.array_equal(s.reshape(-1), u.astype(np.float16).astype(np.float32))
    with np.errstate(divide="ignore"):
        inv = np.where(u == 0, np.float32(0), np.float32(1.0) / u).astype(np.float32)
    prod = (blk * inv[:, None]).astype(np.float32).astype(np.float64)
    want = np.clip(np.sign(prod) * np.floor(np.abs(prod) + 0.5), -128, 127).astype(np.int8)
    assert np.array_equal(q.reshape(-1, 32), want)
    assert np.abs(q.astype(np.int32)).max() <= 127
    assert s[3, 1] == 0 and not q[3, 32:64].any()


# ------------------------------------------------------- Q8_K quantize -----

def test_q8_k_known_answers_from_reference_unit_test():
    # src/inference/tests.rs:17058-17074
    row = np.zeros(256, np.float32)
    row[0], row[1] = -10.0, 4.0
    d, q = oracle.quantize_q8_k(row)
    assert abs(d[0] - 1.0 / 12.7) < 1e-6
    assert q[0] == -127 and q[1] == 51
    dz, qz = oracle.quantize_q8_k(np.zeros(256, np.float32))
    assert dz[0] == 0.0 and not qz.any()


def test_q8_k_first_max_wins_and_positive_max_maps_to_minus_127():
    row = np.zeros(256, np.float32)
    row[5], row[9] = 3.0, -3.0      # equal magnitude: index 5 (positive) sets iscale
    d, q = oracle.quantize_q8_k(row)
    assert q[5] == -127 and q[9] == 127 and d[0] < 0
    row[5], row[9] = -3.0, 3.0
    d, q = oracle.quantize_q8_k(row)
    # iscale = 127/3 > 0: v=-3 -> -127, v=+3 -> +127
    assert q[5] == -127 and q[9] == 127 and d[0] > 0


def test_q8_k_rounding_is_nearest_even_and_clamps_above_only():
    # max = -127 -> iscale = 1.0 exactly; values pass through nearest-even rounding.
    row = np.zeros(256, np.float32)
    row[0] = -127.0
    row[1:7] = [2.5, 0.5, -0.5, -2.5, 1.5, 3.5]
    d, q = oracle.quantize_q8_k(row)
    assert d[0] == np.float32(1.0)
    assert list(q[:7]) == [-127, 2, 0, 0, -2, 2, 4]


def test_q8_k_random_against_numpy_rint():
    rng = np.random.default_rng(3)
    x = rng.standard_normal((32, 4096)).astype(np.float32) * 3
    d, q = oracle.quantize_q8_k(x)
    blk = x.reshape(-1, 256)
    i = np.argmax(np.abs(blk), axis=1)  # first maximum
    mx = blk[np.arange(blk.shape[0]), i]
    iscale = (np.float32(-127.0) / mx).astype(np.float32)
    want = np.minimum(np.rint((blk * iscale[:, None]).astype(np.float32)), 127).astype(np.int8)
    assert np.array_equal(q.reshape(-1, 256), want)
    assert np.array_equal(d.reshape(-1), (np.float32(1.0) / iscale).astype(np.float32))


# -------------------------------------------------- integer block dots -----

def _rand_wire(fmt, n_blocks, rng):
    """Random but valid wire blocks (finite, moderate f16 scales)."""
    bb = oracle.block_bytes(fmt)
    w = rng.integers(0, 256, size=(n_blocks, bb), dtype=np.uint8)

    def put(col, vals):
        h = vals.astype(np.float16).view(np.uint16)
        w[:, col] = h & 0xff
        w[:, col + 1] = h >> 8

    if fmt in (Q8_0, Q4_0):
        put(0, rng.uniform(-0.05, 0.05, n_blocks))
    elif fmt == Q4_K:
        put(0, rng.uniform(0.001, 0.05, n_blocks))
        put(2, rng.uniform(0.001, 0.05, n_blocks))
    else:
        put(208, rng.uniform(-0.01, 0.01, n_blocks))
    return w.reshape(-1)


@pytest.mark.parametrize("fmt,name", [(Q8_0, "Q8_0"), (Q4_0, "Q4_0"), (Q4_K, "Q4_K"), (Q6_K, "Q6_K")])
def test_block_ints_brute_force(fmt, name):
    rng = np.random.default_rng(10 + fmt)
    bv, bb = oracle.block_values(fmt), oracle.block_bytes(fmt)
    nb = 6
    wire = _rand_wire(fmt, nb, rng)
    y = rng.integers(-128, 128, size=nb * bv, dtype=np.int64).astype(np.int8)
    got = oracle.row_block_ints(fmt, wire, y)
    for b in range(nb):
        blk = wire[b * bb:(b + 1) * bb]
        yy = y[b * bv:(b + 1) * bv].astype(np.int64)
        if fmt == Q8_0:
            _, q = npref.q8_0_block(blk)
            assert got[b] == int((q * yy).sum())
        elif fmt == Q4_0:
            _, q = npref.q4_0_block(blk)
            assert got[b] == int((q * yy).sum())
        elif fmt == Q4_K:
            _, _, sc, m, q = npref.q4_k_block(blk)
            main = sum(int(sc[g]) * int((q[32 * g:32 * g + 32] * yy[32 * g:32 * g + 32]).sum()) for g in range(8))
            mins = sum(int(m[g]) * int(yy[32 * g:32 * g + 32].sum()) for g in range(8))
            assert got[2 * b] == main and got[2 * b + 1] == mins
        else:
            _, sc, q = npref.q6_k_block(blk)
            tot = sum(int(sc[j]) * int((q[16 * j:16 * j + 16] * yy[16 * j:16 * j + 16]).sum()) for j in range(16))
            assert got[b] == tot


# ------------------------------------------------------------ row dots -----

def _f64_reference(name, wire, act_scale, act_q, per):
    w = npref.dequant_f64(name, wire)
    a = np.repeat(act_scale.astype(np.float64), per) * act_q.astype(np.float64)
    return float((w * a).sum())


def test_q4_k_row_dots_match_f64_of_dequant_reference_vectors():
    # the synthetic wire of src/inference/tests.rs:16400-16433
    blocks = 3
    wire = np.array([(i * 131 + 17) % 256 for i in range(blocks * 144)], dtype=np.uint8)
    for b in range(blocks):
        for off, val in ((0, 0.0173), (2, 0.0049)):
            h = oracle.f32_to_f16_bits(val)
            wire[b * 144 + off] = h & 0xff
            wire[b * 144 + off + 1] = h >> 8
    act = (np.sin(np.arange(blocks * 256, dtype=np.float32) * np.float32(0.37)) * np.float32(3.0)).astype(np.float32)
    d, q = oracle.quantize_q8_k(act)
    ref = _f64_reference("Q4_K", wire, d, q, 256)
    for order in (ORDER_PRIMARY, ORDER_ALT):
        dot = float(oracle.row_dot(Q4_K, order, wire, d, q))
        assert abs(dot - ref) <= abs(ref) * 1e-4 + 1e-3, (order, dot, ref)


def test_q6_k_row_dots_match_f64_of_dequant_reference_vectors():
    # the synthetic super-block of src/inference/tests.rs:16301-16349
    blk = np.zeros(210, np.uint8)
    blk[:128] = [(i * 37 + 11) % 256 for i in range(128)]
    blk[128:192] = [(i * 73 + 5) % 256 for i in range(64)]
    blk[192:208] = [((i * 9 - 60) & 0xFF) for i in range(16)]
    h = oracle.f32_to_f16_bits(0.0375)
    blk[208], blk[209] = h & 0xff, h >> 8
    act = (np.cos(np.arange(256, dtype=np.float32) * np.float32(0.21)) * np.float32(4.0)).astype(np.float32)
    d, q = oracle.quantize_q8_k(act)
    ref = _f64_reference("Q6_K", blk, d, q, 256)
    for order in (ORDER_PRIMARY, ORDER_ALT):
        dot = float(oracle.row_dot(Q6_K, order, blk, d, q))
        assert abs(dot - ref) <= abs(ref) * 1e-5 + 1e-4, (order, dot, ref)


def test_q4_0_row_dot_matches_f64_of_dequant_reference_vectors():
    # the synthetic row of src/inference/tests.rs:16154-16212
    blocks = 4
    wire = np.zeros(blocks * 18, np.uint8)
    for b in range(blocks):
        h = oracle.f32_to_f16_bits(np.float32(0.0125) * np.float32(b + 1))
        wire[b * 18], wire[b * 18 + 1] = h & 0xff, h >> 8
        for j in range(16):
            lo, hi = (b * 7 + j * 3) % 16, (b * 11 + j * 5) % 16
            wire[b * 18 + 2 + j] = (hi << 4) | lo
    act = (np.sin(np.arange(blocks * 32, dtype=np.float32) * np.float32(0.37)) * np.float32(3.0)).astype(np.float32)
    s, q = oracle.quantize_q8_0(act)
    ref = _f64_reference("Q4_0", wire, s, q, 32)
    dot = float(oracle.row_dot(Q4_0, ORDER_PRIMARY, wire, s, q))
    assert abs(dot - ref) <= abs(ref) * 1e-6 + 1e-6


@pytest.mark.parametrize("fmt,name,per", [(Q8_0, "Q8_0", 32), (Q4_0, "Q4_0", 32), (Q4_K, "Q4_K", 256), (Q6_K, "Q6_K", 256)])
def test_row_dots_random_against_f64(fmt, name, per):
    rng = np.random.default_rng(20 + fmt)
    cols = 2048
    nb = cols // oracle.block_values(fmt)
    for _ in range(8):
        wire = _rand_wire(fmt, nb, rng)
        x = rng.standard_normal(cols).astype(np.float32)
        s, q = oracle.quantize_activation(fmt, x)
        ref = _f64_reference(name, wire, s, q, per)
        mag = float(np.abs(npref.dequant_f64(name, wire) * np.repeat(s.astype(np.float64), per) * q).sum())
        orders = (ORDER_PRIMARY, ORDER_ALT) if fmt in (Q4_K, Q6_K) else (ORDER_PRIMARY,)
        for order in orders:
            dot = float(oracle.row_dot(fmt, order, wire, s, q))
            assert abs(dot - ref) <= 2e-6 * mag + 1e-6, (name, order, dot, ref)


def test_k_quant_orders_agree_within_1e5():
    rng = np.random.default_rng(31)
    for fmt in (Q4_K, Q6_K):
        w = rng.standard_normal((64, 4096)).astype(np.float32) * 0.02
        wire = oracle.quantize_weights(fmt, w)
        x = rng.standard_normal(4096).astype(np.float32)
        a = oracle.matmul(fmt, wire, 4096, x, order=ORDER_PRIMARY)
        b = oracle.matmul(fmt, wire, 4096, x, order=ORDER_ALT)
        assert np.max(np.abs(a - b) / np.maximum(np.abs(b), 1.0)) <= 1e-5


def test_q4_k_exact_arithmetic_special_case_pins_signs_and_terms():
    # d = 1, dmin = 0.5, activation scale 1.0: every product is a small integer
    # or half-integer, so both float orders must return exactly D*S - M*prod.
    rng = np.random.default_rng(40)
    blk = rng.integers(0, 256, size=144, dtype=np.uint8)
    blk[0:2] = np.frombuffer(np.float16(1.0).tobytes(), np.uint8)
    blk[2:4] = np.frombuffer(np.float16(0.5).tobytes(), np.uint8)
    y = rng.integers(-20, 21, size=256).astype(np.int8)
    d = np.array([1.0], np.float32)
    _, _, sc, m, q = npref.q4_k_block(blk)
    yy = y.astype(np.int64)
    S = sum(int(sc[g]) * int((q[32 * g:32 * g + 32] * yy[32 * g:32 * g + 32]).sum()) for g in range(8))
    P = sum(int(m[g]) * int(yy[32 * g:32 * g + 32].sum()) for g in range(8))
    want = np.float32(S - 0.5 * P)
    assert abs(S) < 2**22 and abs(P) < 2**22
    assert oracle.row_dot(Q4_K, ORDER_PRIMARY, blk, d, y) == want
    assert oracle.row_dot(Q4_K, ORDER_ALT, blk, d, y) == want


def test_q6_k_exact_arithmetic_special_case():
    rng = np.random.default_rng(41)
    blk = rng.integers(0, 256, size=210, dtype=np.uint8)
    blk[192:208] = rng.integers(-8, 9, size=16).astype(np.int8).view(np.uint8)
    blk[208:210] = np.frombuffer(np.float16(0.25).tobytes(), np.uint8)
    y = rng.integers(-20, 21, size=256).astype(np.int8)
    d = np.array([2.0], np.float32)
    _, sc, q = npref.q6_k_block(blk)
    yy = y.astype(np.int64)
    T = sum(int(sc[j]) * int((q[16 * j:16 * j + 16] * yy[16 * j:16 * j + 16]).sum()) for j in range(16))
    assert abs(T) < 2**22
    want = np.float32(0.5 * T)
    assert oracle.row_dot(Q6_K, ORDER_PRIMARY, blk, d, y) == want
    assert oracle.row_dot(Q6_K, ORDER_ALT, blk, d, y) == want


def test_q8_0_and_q4_0_exact_arithmetic_special_case():
    rng = np.random.default_rng(42)
    for fmt, dec in ((Q8_0, npref.q8_0_block), (Q4_0, npref.q4_0_block)):
        bb = oracle.block_bytes(fmt)
        wire = rng.integers(0, 256, size=3 * bb, dtype=np.uint8)
        scales = [0.5, -2.0, 0.125]
        for b, s in enumerate(scales):
            wire[b * bb:b * bb + 2] = np.frombuffer(np.float16(s).tobytes(), np.uint8)
        y = rng.integers(-30, 31, size=96).astype(np.int8)
        xs = np.array([1.0, 0.25, 4.0], np.float32)
        want = 0.0
        for b in range(3):
            _, q = dec(wire[b * bb:(b + 1) * bb])
            want += float((q * y[32 * b:32 * b + 32].astype(np.int64)).sum()) * scales[b] * float(xs[b])
        assert oracle.row_dot(fmt, ORDER_PRIMARY, wire, xs, y) == np.float32(want)


# -------------------------------------------------------------- drivers ----

@pytest.mark.parametrize("fmt", [Q8_0, Q4_0, Q4_K, Q6_K])
def test_batched_band_and_threads_are_bitwise_the_single_row_dot(fmt):
    # src/gemma4_runtime.rs:22626-22677 pins band == full rows; matmul_q docs pin batched == single.
    rng = np.random.default_rng(50 + fmt)
    rows, cols = 200, 512
    wire = oracle.quantize_weights(fmt, rng.standard_normal((rows, cols)).astype(np.float32) * 0.02)
    x = rng.standard_normal((5, cols)).astype(np.float32)
    full = oracle.matmul(fmt, wire, cols, x)
    assert full.shape == (5, rows)
    for t in range(5):
        assert np.array_equal(oracle.matmul(fmt, wire, cols, x[t]).view(np.uint32), full[t].view(np.uint32))
    band = oracle.matmul(fmt, wire, cols, x, row_start=70, rows=100)
    assert np.array_equal(band.view(np.uint32), full[:, 70:170].view(np.uint32))
    thr = oracle.matmul(fmt, wire, cols, x, threads=4)
    assert np.array_equal(thr.view(np.uint32), full.view(np.uint32))
    s, q = oracle.quantize_activation(fmt, x[0])
    rb = oracle.row_bytes(fmt, cols)
    assert oracle.row_dot(fmt, ORDER_PRIMARY, wire[3 * rb:4 * rb], s, q) == full[0, 3]


# ------------------------------------------------------------------ MoE ----

def test_softmax_top_k_closed_forms():
    idx, w = oracle.softmax_top_k([0.0, 0.0, 0.0], 2)
    assert list(idx) == [0, 1] and list(w) == [0.5, 0.5]
    idx, w = oracle.softmax_top_k([1.0, 3.0, 2.0], 2)
    e = np.exp(np.float32(-1.0))
    assert list(idx) == [1, 2]
    assert np.allclose(w, [1 / (1 + e), e / (1 + e)], rtol=1e-6)
    assert abs(float(w.sum()) - 1) < 1e-6
    idx, w = oracle.softmax_top_k([5.0], 4)          # k > n
    assert list(idx) == [0] and w[0] == 1.0
    idx, w = oracle.softmax_top_k([], 2)
    assert idx.size == 0
    idx, w = oracle.softmax_top_k([-np.inf, -np.inf, 1.0], 2)  # non-finite gets weight 0
    assert idx[0] == 2 and w[0] == 1.0 and w[1] == 0.0
    idx, w = oracle.softmax_top_k([-np.inf, -np.inf], 2)        # all zero -> uniform
    assert list(w) == [0.5, 0.5] and list(idx) == [0, 1]


def test_softmax_top_k_brute_force():
    rng = np.random.default_rng(60)
    for _ in range(200):
        logits = rng.standard_normal(8).astype(np.float32)
        idx, w = oracle.softmax_top_k(logits, 2)
        order = sorted(range(8), key=lambda i: (-float(logits[i]), i))[:2]
        ex = np.exp(logits[order].astype(np.float64) - float(logits[order].max()))
        ww = ex / ex.sum()
        assert list(idx) == order
        assert np.allclose(w, ww, rtol=1e-6)
        assert w[0] >= w[1]


def test_silu_mul_against_f64():
    rng = np.random.default_rng(61)
    a = rng.standard_normal(4096).astype(np.float32) * 4
    b = rng.standard_normal(4096).astype(np.float32)
    got = oracle.silu_mul(a, b)
    want = (a.astype(np.float64) / (1 + np.exp(-a.astype(np.float64)))) * b
    assert np.allclose(got, want, rtol=1e-6, atol=1e-30)


def test_moe_ffn_is_the_composition_of_its_pieces():
    rng = np.random.default_rng(62)
    n_exp, hidden, ff = 4, 256, 512
    gate = oracle.quantize_weights(Q4_K, rng.standard_normal((n_exp * ff, hidden)).astype(np.float32) * 0.05)
    up = oracle.quantize_weights(Q4_K, rng.standard_normal((n_exp * ff, hidden)).astype(np.float32) * 0.05)
    down = oracle.quantize_weights(Q4_K, rng.standard_normal((n_exp * hidden, ff)).astype(np.float32) * 0.05)
    x = rng.standard_normal((3, hidden)).astype(np.float32)
    logits = rng.standard_normal((3, n_exp)).astype(np.float32)
    out = oracle.moe_ffn(Q4_K, gate, up, down, n_exp, 2, hidden, ff, logits, x)
    for t in range(3):
        acc = np.zeros(hidden, np.float32)
        idx, w = oracle.softmax_top_k(logits[t], 2)
        for e, wt in zip(idx, w):
            g = oracle.matmul(Q4_K, gate, hidden, x[t], row_start=e * ff, rows=ff)
            u = oracle.matmul(Q4_K, up, hidden, x[t], row_start=e * ff, rows=ff)
            y = oracle.matmul(Q4_K, down, ff, oracle.silu_mul(g, u), row_start=e * hidden, rows=hidden)
            acc = (acc + (y * wt).astype(np.float32)).astype(np.float32)
        assert np.array_equal(acc.view(np.uint32), out[t].view(np.uint32))


def test_router_softmax_top_k_reference_tie_vector():
    """The reference's own selection test (src/gemma4_runtime.rs:21548-21561): 128 values
    ((e*37+11)%17)/17 with many repeats, top-k must equal a full sort by (descending value,
    ascending index).  Fed as logits: exp is monotone and equal logits give equal probabilities,
    so the selection over probabilities is the selection over these values."""
    vals = np.array([((e * 37 + 11) % 17) / 17.0 for e in range(128)], np.float32)
    full = sorted(range(128), key=lambda i: (-float(vals[i]), i))
    for k in [1, 8, 17, 127, 128, 256]:
        idx, _ = oracle.router_softmax_top_k(vals, k)
        assert list(idx) == full[:min(k, 128)], k


def test_router_softmax_top_k_closed_forms():
    # all equal: p = 1/n each, the first k win, scale = (1/n) / (k/n) = 1/k
    idx, sc = oracle.router_softmax_top_k(np.zeros(8, np.float32), 4)
    assert list(idx) == [0, 1, 2, 3] and list(sc) == [0.25] * 4
    # softmax over ALL experts, renormalised over the selected ones: the ratio of two scales is
    # exp(logit difference) and they sum to 1, whatever the unselected logits are
    for rest in (-30.0, 0.5):
        idx, sc = oracle.router_softmax_top_k([1.0, rest, 3.0, 2.0, rest], 2)
        e = np.exp(-1.0)
        assert list(idx) == [2, 3]
        assert np.allclose(sc, [1 / (1 + e), e / (1 + e)], rtol=3e-7)
    # down_scale multiplies per selected expert after the renormalisation
    ds = np.array([2.0, 1.0, 0.5, 4.0, 1.0], np.float32)
    idx, sc2 = oracle.router_softmax_top_k([1.0, 0.5, 3.0, 2.0, 0.5], 2, down_scale=ds)
    assert list(idx) == [2, 3]
    assert np.array_equal(sc2, sc * np.array([0.5, 4.0], np.float32))
    # k = n: every expert, in descending order; the scales are the plain softmax
    lg = np.array([0.3, -1.0, 2.0, 0.3], np.float32)
    idx, sc = oracle.router_softmax_top_k(lg, 4)
    assert list(idx) == [2, 0, 3, 1]
    p = np.exp(lg.astype(np.float64) - 2.0)
    assert np.allclose(sc, (p / p.sum())[[2, 0, 3, 1]], rtol=5e-7)


def test_router_softmax_top_k_brute_force():
    rng = np.random.default_rng(63)
    for trial in range(200):
        n, k = (128, 8) if trial % 2 else (16, 3)
        logits = (rng.standard_normal(n) * 3).astype(np.float32)
        ds = rng.uniform(0.5, 2.0, n).astype(np.float32)
        idx, sc = oracle.router_softmax_top_k(logits, k, down_scale=ds)
        order = sorted(range(n), key=lambda i: (-float(logits[i]), i))[:k]
        assert list(idx) == order
        p = np.exp(logits.astype(np.float64) - float(logits.max()))
        want = ds[order] * (p[order] / p[order].sum())
        assert np.allclose(sc, want, rtol=2e-6)


def test_gelu_tanh_mul_reference_values_and_f64():
    """Known answers of the reference's unit tests (src/inference/gemma4.rs:90-111), then the
    formula in float64 (the libm tanhf's last bit is not pinned by anything the reference holds)."""
    one = np.ones(1, np.float32)
    for x, want, tol in [(0.0, 0.0, 1e-6), (1.0, 0.841192, 1e-4), (-1.0, -0.158808, 1e-4), (2.0, 1.954598, 1e-4),
                         (8.0, 8.0, 1e-3), (-8.0, 0.0, 1e-3)]:
        assert abs(float(oracle.gelu_tanh_mul(np.float32([x]), one)[0]) - want) <= tol, x
    got = oracle.gelu_tanh_mul(np.float32([0.0, 1.0, 2.0]), np.float32([3.0, 4.0, 5.0]))
    assert got[0] == 0.0
    assert got[1] == np.float32(oracle.gelu_tanh_mul(np.float32([1.0]), one)[0] * np.float32(4.0))
    assert got[2] == np.float32(oracle.gelu_tanh_mul(np.float32([2.0]), one)[0] * np.float32(5.0))
    rng = np.random.default_rng(64)
    a = (rng.standard_normal(8192) * 3).astype(np.float32)
    b = rng.standard_normal(8192).astype(np.float32)
    a64 = a.astype(np.float64)
    want = 0.5 * a64 * (1 + np.tanh(np.sqrt(2 / np.pi) * (a64 + 0.044715 * a64 ** 3))) * b
    got = oracle.gelu_tanh_mul(a, b)
    # 1 + tanh cancels for negative inputs: absolute error there is a few ulp of 1 times |0.5 a b|
    assert np.all(np.abs(got - want) <= 2e-6 * np.abs(want) + 4e-7 * np.abs(0.5 * a64 * b))
    # odd-part identity gelu(x) - gelu(-x) = x holds to rounding: pins the sign of the cubic term
    gp = oracle.gelu_tanh_mul(a, np.ones_like(a))
    gm = oracle.gelu_tanh_mul(-a, np.ones_like(a))
    assert np.allclose(gp - gm, a, rtol=1e-6, atol=1e-6)


def test_moe_ffn_ex_gemma4_is_the_composition_of_its_pieces():
    """Gemma-4 expert mix (reference moe_layer_ffn, src/gemma4_runtime.rs:5567-5708): route over
    the full softmax, fused gate|up band of 2*ff rows per expert, gelu_tanh(g)*u, down band,
    acc += y * (down_scale[e] * p[e]/wsum) in selection order.  Also: the separate-gate/up call on
    the de-interleaved halves gives the same bits."""
    rng = np.random.default_rng(65)
    n_exp, hidden, ff, k = 6, 256, 512, 3
    gate_up = oracle.quantize_weights(Q4_K, rng.standard_normal((n_exp * 2 * ff, hidden)).astype(np.float32) * 0.05)
    down = oracle.quantize_weights(Q4_K, rng.standard_normal((n_exp * hidden, ff)).astype(np.float32) * 0.05)
    ds = rng.uniform(0.5, 2.0, n_exp).astype(np.float32)
    x = rng.standard_normal((3, hidden)).astype(np.float32)
    logits = rng.standard_normal((3, n_exp)).astype(np.float32)
    out = oracle.moe_ffn_ex(Q4_K, gate_up, None, down, n_exp, k, hidden, ff, logits, x, variant=1, down_scale=ds)
    for t in range(3):
        acc = np.zeros(hidden, np.float32)
        idx, sc = oracle.router_softmax_top_k(logits[t], k, down_scale=ds)
        for e, wt in zip(idx, sc):
            gu = oracle.matmul(Q4_K, gate_up, hidden, x[t], row_start=e * 2 * ff, rows=2 * ff).reshape(-1)
            h = oracle.gelu_tanh_mul(gu[:ff], gu[ff:])
            y = oracle.matmul(Q4_K, down, ff, h, row_start=e * hidden, rows=hidden)
            acc = (acc + (y * wt).astype(np.float32)).astype(np.float32)
        assert np.array_equal(acc.view(np.uint32), out[t].view(np.uint32))
    rb = oracle.row_bytes(Q4_K, hidden)
    gu3 = gate_up.reshape(n_exp, 2, ff * rb)
    out2 = oracle.moe_ffn_ex(Q4_K, gu3[:, 0].copy(), gu3[:, 1].copy(), down, n_exp, k, hidden, ff, logits, x, variant=1,
                             down_scale=ds)
    assert np.array_equal(out.view(np.uint32), out2.view(np.uint32))
    # variant 0 through the extended entry is the plain entry
    a = oracle.moe_ffn_ex(Q4_K, gu3[:, 0].copy(), gu3[:, 1].copy(), down, n_exp, 2, hidden, ff, logits, x)
    b = oracle.moe_ffn(Q4_K, gu3[:, 0].copy(), gu3[:, 1].copy(), down, n_exp, 2, hidden, ff, logits, x)
    assert np.array_equal(a.view(np.uint32), b.view(np.uint32))


# ----------------------------------------------------- weight quantizers ---

def test_weight_quantizer_error_bounds_on_reference_ramps():
    # src/quantize.rs:731-809
    ramp = ((np.arange(32, dtype=np.float32) - 16.0) * 0.125).astype(np.float32)
    rec = oracle.dequant(Q8_0, oracle.quantize_weights(Q8_0, ramp, threads=1))
    assert np.max(np.abs(rec - ramp)) < 0.05
    ramp = ((np.arange(32, dtype=np.float32) - 16.0) * 0.25).astype(np.float32)
    wire = oracle.quantize_weights(Q4_0, ramp, threads=1)
    rec = oracle.dequant(Q4_0, wire)
    d = abs(float(oracle.f16_bits_to_f32(int(wire[0]) | (int(wire[1]) << 8))))
    assert np.array_equal(np.sign(rec), np.sign(ramp))
    assert np.all(np.abs(rec - ramp) <= d + 0.01)
    orig = np.zeros(256, np.float32)
    for g in range(8):
        off = 2.0 if g == 6 else (-2.0 if g == 7 else 0.0)
        orig[g * 32:(g + 1) * 32] = (np.arange(32, dtype=np.float32) - 15.5) * (g + 1.0) * 0.03125 + off
    rec = oracle.dequant(Q4_K, oracle.quantize_weights(Q4_K, orig, threads=1))
    assert np.max(np.abs(rec - orig).reshape(8, 32), axis=1).max() < 0.3


def test_q6_k_input_generator_round_trips_within_a_step():
    rng = np.random.default_rng(63)
    w = rng.standard_normal(4096).astype(np.float32) * 0.02
    w[256:512] = 0.0
    rec = oracle.dequant(Q6_K, oracle.quantize_weights(Q6_K, w, threads=1))
    assert not rec[256:512].any()
    step = np.abs(w.reshape(-1, 16)).max(axis=1) / 31.0
    assert np.all(np.abs(rec - w).reshape(-1, 16) <= step[:, None] * 1.05 + 1e-6)


# ------------------------------------------------------------------ rms_norm ----

def test_rms_norm_known_vector_of_the_reference():
    """tests/tensor_primitives.rs:83-93 of the reference: x = [3, 4], w = [1, 2], eps = 0."""
    out = oracle.rms_norm(np.array([[3.0, 4.0]], np.float32), np.array([1.0, 2.0], np.float32), 0.0)
    rms = np.sqrt(np.float32((9.0 + 16.0) / 2.0))
    assert abs(out[0, 0] - 3.0 / rms) < 1e-5 and abs(out[0, 1] - 4.0 / rms * 2.0) < 1e-5


def test_rms_norm_exact_cases_and_summation_order():
    # powers of two make every step exact: 256 values of 0.5 -> mean 0.25 -> scale 2 -> out = w
    w = np.linspace(-3, 3, 256, dtype=np.float32)
    out = oracle.rms_norm(np.full((1, 256), 0.5, np.float32), w, 0.0)
    assert np.array_equal(out[0].view(np.uint32), w.view(np.uint32))
    # eps enters under the root: x = 0 -> scale = 1/sqrt(eps), out = 0 * scale * w = 0
    assert np.all(oracle.rms_norm(np.zeros((1, 64), np.float32), np.ones(64, np.float32), 1e-5) == 0)
    # left-to-right f32 sum: 1 followed by 2^24 .. the small squares after a huge one vanish one by one,
    # whereas a pairwise sum would keep them
    x = np.zeros((1, 4096), np.float32)
    x[0, 0] = 4096.0                      # square 2^24
    x[0, 1:] = 1.0                        # 4095 squares of 1: sequentially each is absorbed (2^24 + 1 rounds to 2^24)
    out = oracle.rms_norm(x, np.ones(4096, np.float32), 0.0)
    seq_scale = np.float32(1.0) / np.sqrt(np.float32(2.0 ** 24) / np.float32(4096))
    assert out[0, 1].view(np.uint32) == np.float32(np.float32(1.0) * seq_scale).view(np.uint32)
    tree_scale = np.float32(1.0) / np.sqrt(np.float32(2.0 ** 24 + 4095) / np.float32(4096))
    assert out[0, 1] != np.float32(tree_scale)   # a reassociated sum would have given this
    # reversed order: the ones add up first (exactly 4095), then 2^24 + 4095 rounds to even
    out_r = oracle.rms_norm(x[:, ::-1].copy(), np.ones(4096, np.float32), 0.0)
    rev_scale = np.float32(1.0) / np.sqrt(np.float32(np.float32(4095.0) + np.float32(2.0 ** 24)) / np.float32(4096))
    assert out_r[0, 0].view(np.uint32) == np.float32(np.float32(1.0) * rev_scale).view(np.uint32)


def test_rms_norm_against_float64_and_rows_are_independent():
    rng = np.random.default_rng(77)
    x = rng.standard_normal((5, 3072)).astype(np.float32)
    w = (rng.standard_normal(3072) * 0.5 + 1.0).astype(np.float32)
    out = oracle.rms_norm(x, w, 1e-6)
    x64 = x.astype(np.float64)
    ref = x64 / np.sqrt((x64 ** 2).mean(axis=1, keepdims=True) + 1e-6) * w.astype(np.float64)
    assert np.max(np.abs(out - ref) / np.maximum(np.abs(ref), 1.0)) < 1e-6
    for r in range(5):
        assert np.array_equal(oracle.rms_norm(x[r:r + 1], w, 1e-6)[0].view(np.uint32), out[r].view(np.uint32))
