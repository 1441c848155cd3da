"""Pins the last-ulp association of the oracle's row dots.

The reference stores no output vectors for its dot products, so what fixes their bits is the
order of the float operations (reference src/inference.rs:22729-22798, :25535-25581,
:25806-25889; src/diffusion_gemma/refmath.rs:504-562, :678-721).  This file evaluates those
orders independently of the C code: integers from the numpy block decoders, every float step
in exact rational arithmetic followed by an explicit round-to-nearest-even to binary32.  For
each order it also evaluates plausible wrong variants (a fused step unfused, an unfused step
fused, the scale product associated the other way, terms added in another order) and checks
that they give different bits on these inputs -- so a mistake of that kind in the oracle
fails here -- and that the oracle returns the bits of the right one.
"""
from fractions import Fraction

import numpy as np
import pytest

import oracle
from oracle import ORDER_ALT, ORDER_PRIMARY, Q4_0, Q4_K, Q6_K, Q8_0
from tests import npref

TWO = Fraction(2)


def rnd(x: Fraction) -> Fraction:
    """Round an exact rational to the nearest binary32 value, ties to even (normal and
    subnormal range; the inputs here never overflow)."""
    if x == 0:
        return Fraction(0)
    sign = -1 if x < 0 else 1
    a = abs(x)
    e = a.numerator.bit_length() - a.denominator.bit_length()
    if TWO ** e > a:
        e -= 1
    elif TWO ** (e + 1) <= a:
        e += 1
    assert TWO ** e <= a < TWO ** (e + 1)
    e = max(e, -126)
    ulp = TWO ** (e - 23)
    q = a / ulp
    n = q.numerator // q.denominator
    r = q - n
    if r > Fraction(1, 2) or (r == Fraction(1, 2) and n % 2 == 1):
        n += 1
    assert n * ulp < TWO ** 128
    return sign * n * ulp


def F(v) -> Fraction:
    return Fraction(float(np.float32(v)))


def mul(a, b):
    return rnd(a * b)


def add(a, b):
    return rnd(a + b)


def fma(a, b, c):
    return rnd(a * b + c)


def i2f(i: int) -> Fraction:
    """An integer converted to f32 (rounds beyond 2^24)."""
    return rnd(Fraction(int(i)))


def bits(x: Fraction) -> int:
    f = np.float32(float(x))
    assert Fraction(float(f)) == x
    return int(f.view(np.uint32))


def test_the_rounding_helper_is_ieee_binary32():
    rng = np.random.default_rng(1)
    a = rng.standard_normal(2000).astype(np.float32) * np.float32(3.7)
    b = (rng.standard_normal(2000) * 10.0 ** rng.integers(-20, 20, 2000)).astype(np.float32)
    for x, y in zip(a, b):
        assert bits(mul(F(x), F(y))) == int(np.float32(x * y).view(np.uint32))
        assert bits(add(F(x), F(y))) == int(np.float32(x + y).view(np.uint32))
    # ties, subnormals, integers beyond 2^24
    assert rnd(Fraction(2 ** 24 + 1)) == 2 ** 24 and rnd(Fraction(2 ** 24 + 3)) == 2 ** 24 + 4
    assert rnd(TWO ** -149 / 2) == 0 and rnd(TWO ** -149 * 3 / 2) == TWO ** -148
    assert i2f(30_000_001) == 30_000_000 and i2f(-16_777_217) == -16_777_216


# ---- the orders, restated from the reference ------------------------------------------------

def q8_0_like(dec, bb, wire, xs, xq, variant="ref"):
    total = Fraction(0)
    for b in range(len(xs)):
        d, q = dec(wire[bb * b:bb * (b + 1)])
        isum = int((q.astype(np.int64) * xq[32 * b:32 * b + 32].astype(np.int64)).sum())
        if variant == "ref":        # total += (isum as f32 * scale) * x_scale
            term = mul(mul(i2f(isum), F(d)), F(xs[b]))
        elif variant == "scales_first":
            term = mul(i2f(isum), mul(F(d), F(xs[b])))
        elif variant == "fused":
            total = fma(mul(i2f(isum), F(d)), F(xs[b]), total)
            continue
        total = add(total, term)
    return total


def q4_k_ints(blk, y):
    d, dmin, sc, m, q = npref.q4_k_block(blk)
    y = y.astype(np.int64)
    S = sum(int(sc[g]) * int((q[32 * g:32 * g + 32] * y[32 * g:32 * g + 32]).sum()) for g in range(8))
    P = sum(int(m[g]) * int(y[32 * g:32 * g + 32].sum()) for g in range(8))
    aux = [sum(int(sc[g]) * int((q[32 * g + l:32 * g + 32:8] * y[32 * g + l:32 * g + 32:8]).sum()) for g in range(8)) for l in range(8)]
    assert sum(aux) == S
    return d, dmin, S, P, aux


def q4_k_arm(wire, xd, xq, variant="ref"):
    acc = Fraction(0)
    for i in range(len(xd)):
        d, dmin, S, P, _ = q4_k_ints(wire[144 * i:144 * (i + 1)], xq[256 * i:256 * (i + 1)])
        D, M = mul(F(xd[i]), F(d)), mul(F(xd[i]), F(dmin))
        if variant == "ref":          # sumf = fma(-dmin, prod, sumf); sumf = fma(d, sumi, sumf)
            acc = fma(-M, i2f(P), acc)
            acc = fma(D, i2f(S), acc)
        elif variant == "unfused":
            acc = add(acc, mul(-M, i2f(P)))
            acc = add(acc, mul(D, i2f(S)))
        elif variant == "main_first":
            acc = fma(D, i2f(S), acc)
            acc = fma(-M, i2f(P), acc)
        elif variant == "one_term":
            acc = add(acc, rnd(D * i2f(S) - M * i2f(P)))
        elif variant == "exact_ints":  # the integer not rounded to f32 before the multiply
            acc = fma(-M, Fraction(P), acc)
            acc = fma(D, Fraction(S), acc)
    return acc


def q4_k_generic(wire, xd, xq, variant="ref"):
    sums = [Fraction(0)] * 8
    sumf = Fraction(0)
    for i in range(len(xd)):
        d, dmin, S, P, aux = q4_k_ints(wire[144 * i:144 * (i + 1)], xq[256 * i:256 * (i + 1)])
        dd = mul(F(d), F(xd[i]))
        for l in range(8):
            sums[l] = fma(dd, i2f(aux[l]), sums[l]) if variant == "fused" else add(sums[l], mul(dd, i2f(aux[l])))
        if variant == "mins_other_way":   # dmin * (y.d * sumi)
            sumf = add(sumf, -mul(F(dmin), mul(F(xd[i]), i2f(P))))
        else:                             # sumf -= (dmin * y.d) * sumi
            sumf = add(sumf, -mul(mul(F(dmin), F(xd[i])), i2f(P)))
    if variant == "pairwise_fold":
        lanes = add(add(add(sums[0], sums[1]), add(sums[2], sums[3])), add(add(sums[4], sums[5]), add(sums[6], sums[7])))
    else:
        lanes = Fraction(0)
        for l in range(8):
            lanes = add(lanes, sums[l])
    if variant == "lanes_into_sumf":
        for l in range(8):
            sumf = add(sumf, sums[l])
        return sumf
    return add(sumf, lanes)


def q6_k_ints(blk, y):
    d, sc, q = npref.q6_k_block(blk)
    y = y.astype(np.int64)
    aux = [sum(int(sc[j]) * (int(q[16 * j + l]) * int(y[16 * j + l]) + int(q[16 * j + 8 + l]) * int(y[16 * j + 8 + l])) for j in range(16)) for l in range(8)]
    return d, sum(aux), aux


def q6_k_lanes(wire, xd, xq, variant="ref"):
    sums = [Fraction(0)] * 8
    for i in range(len(xd)):
        d, _, aux = q6_k_ints(wire[210 * i:210 * (i + 1)], xq[256 * i:256 * (i + 1)])
        dd = mul(F(d), F(xd[i]))
        for l in range(8):
            sums[l] = fma(dd, i2f(aux[l]), sums[l]) if variant == "fused" else add(sums[l], mul(dd, i2f(aux[l])))
    total = Fraction(0)
    order = range(7, -1, -1) if variant == "reverse_fold" else range(8)
    for l in order:
        total = add(total, sums[l])
    return total


def q6_k_arm(wire, xd, xq, variant="ref"):
    acc = Fraction(0)
    for i in range(len(xd)):
        d, T, _ = q6_k_ints(wire[210 * i:210 * (i + 1)], xq[256 * i:256 * (i + 1)])
        dd = mul(F(d), F(xd[i]))
        acc = add(acc, mul(dd, i2f(T))) if variant == "unfused" else fma(dd, i2f(T), acc)
    return acc


# ---- inputs: a few rows of several blocks, sized so that the running sums round at every step ----

def _rows(fmt, n_rows, n_blocks, seed):
    rng = np.random.default_rng(seed)
    cols = n_blocks * oracle.block_values(fmt)
    x = (rng.standard_normal(cols) * (1.0 + 3.0 * rng.random(cols))).astype(np.float32)
    w = (rng.standard_normal((n_rows, cols)) * 0.02).astype(np.float32)
    # half of the rows follow the signs of the activation: large block integers, whose products
    # with the scales no longer fit 24 bits (small ones would hide a wrong association)
    w[:n_rows // 2] = np.abs(w[:n_rows // 2]) * np.sign(x)
    wire = oracle.quantize_weights(fmt, w).reshape(n_rows, -1)
    s, q = oracle.quantize_activation(fmt, x)
    return wire, s, q


CASES = [
    (Q8_0, ORDER_PRIMARY, lambda w, s, q, v: q8_0_like(npref.q8_0_block, 34, w, s, q, v), ("scales_first", "fused")),
    (Q4_0, ORDER_PRIMARY, lambda w, s, q, v: q8_0_like(npref.q4_0_block, 18, w, s, q, v), ("scales_first", "fused")),
    (Q4_K, ORDER_PRIMARY, q4_k_arm, ("unfused", "main_first", "one_term", "exact_ints")),
    (Q4_K, ORDER_ALT, q4_k_generic, ("fused", "mins_other_way", "pairwise_fold", "lanes_into_sumf")),
    (Q6_K, ORDER_PRIMARY, q6_k_lanes, ("fused", "reverse_fold")),
    (Q6_K, ORDER_ALT, q6_k_arm, ("unfused",)),
]


@pytest.mark.parametrize("fmt,order,evaluate,variants", CASES, ids=[f"{f}-{o}" for f, o, _, _ in CASES])
def test_oracle_row_dot_has_the_bits_of_the_reference_order(fmt, order, evaluate, variants):
    n_rows = 12
    n_blocks = 24 if fmt in (Q8_0, Q4_0) else 4
    wire, s, q = _rows(fmt, n_rows, n_blocks, seed=100 + fmt + order)
    differs = {v: 0 for v in variants}
    for r in range(n_rows):
        want = bits(evaluate(wire[r], s, q, "ref"))
        got = int(oracle.row_dot(fmt, order, wire[r], s, q).view(np.uint32))
        assert got == want, (fmt, order, r, hex(got), hex(want))
        for v in variants:
            differs[v] += bits(evaluate(wire[r], s, q, v)) != want
    if fmt in (Q8_0, Q4_0):
        # single blocks with the largest integers the format allows (activation +-127 with the
        # sign of the weight) and random f16 scales: here (isum * d) itself rounds, which is what
        # tells (isum * d) * s from isum * (d * s)
        rng = np.random.default_rng(7 + fmt)
        bb, dec = (34, npref.q8_0_block) if fmt == Q8_0 else (18, npref.q4_0_block)
        for _ in range(600):
            blk = rng.integers(0, 256, bb, dtype=np.uint8)
            blk[0:2] = np.frombuffer(np.float16(rng.uniform(0.01, 0.05)).tobytes(), np.uint8)
            _, qw = dec(blk)
            xq = np.where(qw >= 0, 127, -127).astype(np.int8)
            xs = np.array([np.float16(rng.uniform(0.01, 0.2))], np.float32)
            want = bits(evaluate(blk, xs, xq, "ref"))
            got = int(oracle.row_dot(fmt, order, blk, xs, xq).view(np.uint32))
            assert got == want, (fmt, hex(got), hex(want))
            for v in variants:
                differs[v] += bits(evaluate(blk, xs, xq, v)) != want
    if fmt == Q4_K:
        # rows of three super-blocks at the top of the integer range (6-bit scales all ones, high
        # nibbles, activations 125..127): S passes 2^24, so `S as f32` itself rounds
        rng = np.random.default_rng(70 + order)
        for _ in range(40):
            blks = rng.integers(0xcc, 0x100, 3 * 144).astype(np.uint8)
            for i in range(3):
                blks[144 * i:144 * i + 2] = np.frombuffer(np.float16(rng.uniform(0.001, 0.004)).tobytes(), np.uint8)
                blks[144 * i + 2:144 * i + 4] = np.frombuffer(np.float16(rng.uniform(0.01, 0.04)).tobytes(), np.uint8)
                blks[144 * i + 4:144 * i + 16] = 0xff
            xq = rng.integers(125, 128, 3 * 256).astype(np.int8)
            xd = rng.uniform(0.01, 0.05, 3).astype(np.float32)
            want = bits(evaluate(blks, xd, xq, "ref"))
            got = int(oracle.row_dot(fmt, order, blks, xd, xq).view(np.uint32))
            assert got == want, (fmt, order, hex(got), hex(want))
            for v in variants:
                differs[v] += bits(evaluate(blks, xd, xq, v)) != want
    # the inputs tell every variant apart from the reference order on at least one row
    assert all(n > 0 for n in differs.values()), differs


def test_q4_k_top_of_range_blocks_really_round_their_integer():
    rng = np.random.default_rng(70)
    blk = rng.integers(0xcc, 0x100, 144).astype(np.uint8)
    blk[4:16] = 0xff
    xq = rng.integers(125, 128, 256).astype(np.int8)
    S = q4_k_ints(blk, xq)[2]
    assert S > 2 ** 24 and S < 2 ** 25
