"""Random shapes through the plain matvec / small-batch entry points: every format, ragged row
counts, 1..9 tokens, a band view that starts inside a tile -- bit for bit against the oracle in
the exact order, within 1e-5 max-rel under the default K-split policy."""
import numpy as np
import pytest

import oracle
from camelid_amd import binding as B
from camelid_amd.binding import Weight, lib
from tests import gpu_util as G

pytestmark = pytest.mark.gpu

EXACT = {oracle.Q8_0: oracle.ORDER_PRIMARY, oracle.Q4_0: oracle.ORDER_PRIMARY,
         oracle.Q4_K: oracle.ORDER_PRIMARY, oracle.Q6_K: oracle.ORDER_ALT}


@pytest.fixture(scope="module", autouse=True)
def _init():
    assert lib().cml_available() == 1
    B.init(0)
    yield


@pytest.mark.parametrize("seed", [3, 17])
def test_random_shapes_match_the_oracle(seed):
    rng = np.random.default_rng(seed)
    for case in range(48):
        fmt = [oracle.Q8_0, oracle.Q4_0, oracle.Q4_K, oracle.Q6_K][case % 4]
        unit = 256 if fmt in (oracle.Q4_K, oracle.Q6_K) else 32
        rows = int(rng.integers(1, 700))
        cols = unit * int(rng.integers(1, 24 if unit == 256 else 160))
        n = int(rng.choice([1, 1, 2, 3, 5, 9]))
        G.say(f"fuzz seed={seed} case={case} fmt={fmt} {rows}x{cols} n={n}")
        wire = G.synth_weight(fmt, rows, cols, seed=1000 * seed + case)
        w = Weight.upload(fmt, rows, cols, wire)
        x = rng.standard_normal((n, cols)).astype(np.float32)
        s, q = oracle.quantize_activation(fmt, x)
        want = oracle.matmul(fmt, wire, cols, x, order=EXACT[fmt], threads=8)
        with G.env(CAMELID_HIP_EXACT_ORDER="1"):
            got = G.gpu_gemm(w, s, q).reshape(n, rows)
            assert G.same_bits(got, want), (case, fmt, rows, cols, n)
            if n == 1:
                assert G.same_bits(G.gpu_matmul_f32(w, x[0]), want[0]), (case, fmt, rows, cols)
            else:   # two tokens also quantize inside the matvec kernel where the shape allows
                assert G.same_bits(G.gpu_matmul_f32(w, x), want), (case, fmt, rows, cols, n)
            if rows > 40:   # a band of rows that starts inside a tile
                start, count = int(rng.integers(1, 30)), int(rng.integers(1, rows - 30))
                band = w.slice(start, count)
                assert G.same_bits(G.gpu_gemm(band, s, q).reshape(n, count), want[:, start:start + count]), (case, start, count)
        default = G.gpu_gemm(w, s, q).reshape(n, rows)   # default K-split policy
        assert G.max_rel(default, want) <= 1e-5, (case, fmt, rows, cols, n)


@pytest.mark.parametrize("seed", [4, 29, 31])
def test_random_staged_once_walks_match_the_oracle(seed):
    """Q4_K batches of 3 to 32 tokens forced onto the staged-once matrix-core kernel at small sizes (the launch
    that serves tall weights and expert groups): random row counts and row lengths (2, 5, 8, 12, 14, 16, 20,
    24 or 32 super-blocks: with and without the row length known at compile time), one or two token groups per wave,
    one to eight groups of row tiles per workgroup, a band view that starts and ends inside a tile -- the
    oracle's chain bit for bit."""
    fmt = oracle.Q4_K
    rng = np.random.default_rng(seed)
    for case in range(32):
        rows = int(rng.integers(100, 6000))
        cols = 256 * int(rng.choice([2, 5, 8, 8, 12, 12, 14, 14, 16, 16, 16, 20, 24, 32]))
        n = int(rng.integers(3, 33)) if cols <= 4096 else int(rng.integers(3, 17))  # (longer rows: one token group per wave)
        units = int(rng.choice([0, 1, 2, 3, 5, 8]))
        fixed = int(rng.choice([0, 1, 1]))
        skip, tail = int(rng.integers(0, 16)), int(rng.integers(0, 16))
        G.say(f"walk fuzz seed={seed} case={case} {rows}x{cols} n={n} units={units} fixed={fixed} band=[{skip},{rows - tail})")
        wire = G.synth_weight(fmt, rows, cols, seed=7000 * seed + case)
        w = Weight.upload(fmt, rows, cols, wire)
        band = w.slice(skip, rows - skip - tail)
        x = rng.standard_normal((n, cols)).astype(np.float32)
        s, q = oracle.quantize_activation(fmt, x)
        want = oracle.matmul_q(fmt, wire, cols, s, q, order=oracle.ORDER_PRIMARY, threads=8)
        with G.env(CAMELID_HIP_EXACT_ORDER="1", CAMELID_HIP_Q4K_MFMA_PAIR_MAX_ROWS=64, CAMELID_HIP_Q4K_MFMA_ONCE_TWO_GROUPS_MIN_TILES=1,
                   CAMELID_HIP_Q4K_MFMA_ONCE_LONG_MIN_TILES=1, CAMELID_HIP_Q4K_MFMA_UNITS=units, CAMELID_HIP_Q4K_MFMA_FIXED_ROWS=fixed, CAMELID_HIP_Q4K_MFMA_MIN_TOKENS=3), \
                G.engaged(r"^q4k\.mfma\.tile\.g[12]t1\.once", none=(r"^q4k\.mfma\.pair", r"^q4k\.dot\.")):
            got = G.gpu_gemm(w, s, q)
            got_band = G.gpu_gemm(band, s, q)
        assert G.same_bits(got, want), (case, rows, cols, n, units, fixed)
        assert G.same_bits(got_band, want[:, skip:rows - tail]), (case, rows, cols, n, units, fixed, skip, tail)


@pytest.mark.parametrize("fmt", [oracle.Q8_0, oracle.Q4_0])
def test_block32_launch_shapes_agree(fmt):
    """The 32-value-block matvec under each of its launch shapes (4 or 8 waves per workgroup for
    the fused quantizer, 2 or 4 steps per register buffer, 8 or 16 lanes per row): the same bits."""
    lanes_knob = "CAMELID_HIP_Q8_0_LANES" if fmt == oracle.Q8_0 else "CAMELID_HIP_Q4_0_LANES"
    rng = np.random.default_rng(5)
    for rows, cols in [(77, 32), (1000, 2048), (530, 4096), (300, 8192 + 64), (64, 14336)]:
        wire = G.synth_weight(fmt, rows, cols, seed=rows + cols)
        w = Weight.upload(fmt, rows, cols, wire)
        x = rng.standard_normal((2, cols)).astype(np.float32)
        s, q = oracle.quantize_activation(fmt, x)
        want = oracle.matmul(fmt, wire, cols, x, order=EXACT[fmt], threads=8)
        for waves in ("2", "4", "8", "16"):
            for depth in ("2", "4"):
                for lanes in ("8", "16", "32", "64"):
                    G.say(f"block32 {fmt} {rows}x{cols} waves={waves} depth={depth} lanes={lanes}")
                    with G.env(CAMELID_HIP_EXACT_ORDER="1", CAMELID_HIP_B32_FUSED_WAVES=waves, CAMELID_HIP_B32_WAVES=("8" if waves == "8" else "4"), CAMELID_HIP_B32_DEPTH=depth, **{lanes_knob: lanes}):
                        assert G.same_bits(G.gpu_matmul_f32(w, x[0]), want[0]), (rows, cols, waves, depth, lanes)
                        assert G.same_bits(G.gpu_gemm(w, s[:1], q[:1]).reshape(rows), want[0]), (rows, cols, depth, lanes)
                        assert G.same_bits(G.gpu_gemm(w, s, q).reshape(2, rows), want), (rows, cols, depth, lanes)


def test_register_buffer_rings_cover_every_remainder():
    """The single-token matvecs that walk a row through a ring of small register buffers (Q4_K: three
    2-super-block slots under 8-row waves, four 1-super-block slots under 16-row waves; Q8_0:
    three one-step slots) against the oracle in the exact order, for every remainder of the row
    length modulo the ring, with the ring and without it (CAMELID_HIP_Q4K_RING / _B32_RING = 0),
    quantized and f32 activations, one and two tokens, K cut 1 and 2."""
    rng = np.random.default_rng(41)
    cases = [(oracle.Q4_K, 200, 256 * nsb) for nsb in (6, 8, 10, 12, 14, 16, 18, 20, 28, 32)]   # 8-row waves: 3..16 steps of two
    cases += [(oracle.Q4_K, 136, 256 * nsb) for nsb in (4, 5, 6, 7, 8, 9, 11, 12, 14, 16)]           # two tokens: 16-row waves, steps of one
    cases += [(oracle.Q8_0, 4200, 512 * steps) for steps in (3, 4, 5, 6, 7, 8)]          # 16-lane rows, eight-wave workgroups
    for fmt, rows, cols in cases:
        wire = G.synth_weight(fmt, rows, cols, seed=rows + cols)
        w = Weight.upload(fmt, rows, cols, wire)
        x = rng.standard_normal((2, cols)).astype(np.float32)
        s, q = oracle.quantize_activation(fmt, x)
        want = oracle.matmul(fmt, wire, cols, x, order=EXACT[fmt], threads=8)
        for ring in ("1", "0"):
            for ksplit in ("1", "2"):
                if fmt != oracle.Q4_K and ksplit != "1":
                    continue
                G.say(f"ring fmt={fmt} {rows}x{cols} ring={ring} ksplit={ksplit}")
                # the kernels that must (not) have served these calls: with the ring on and no K cut every test row is
                # a whole number of ring steps; with it off no ring kernel may run
                tag = "q4k" if fmt == oracle.Q4_K else "q8_0"
                if ring == "0":
                    proof = G.engaged(rf"^{tag}\.dot\.", none=(rf"^{tag}\.dot\..*ring", r"^q4k\.dot\.wg8"))
                elif ksplit == "1":
                    proof = G.engaged(rf"^{tag}\.dot\..*ring")
                else:
                    proof = G.engaged(rf"^{tag}\.dot\.")
                with G.env(CAMELID_HIP_Q4K_RING=ring, CAMELID_HIP_B32_RING=ring, CAMELID_HIP_Q4K_KSPLIT=ksplit), proof:
                    one = G.gpu_matmul_f32(w, x[0])
                    two = G.gpu_matmul_f32(w, x)
                    pre = G.gpu_gemm(w, s[:1], q[:1]).reshape(rows)
                    pre2 = G.gpu_gemm(w, s, q).reshape(2, rows)
                if ksplit == "1":
                    assert G.same_bits(one, want[0]), (fmt, rows, cols, ring)
                    assert G.same_bits(two, want), (fmt, rows, cols, ring)
                    assert G.same_bits(pre, want[0]), (fmt, rows, cols, ring)
                    assert G.same_bits(pre2, want), (fmt, rows, cols, ring)
                else:
                    for got, ref in ((one, want[0]), (two, want), (pre, want[0]), (pre2, want)):
                        assert G.max_rel(got, ref) <= 1e-5, (fmt, rows, cols, ring, ksplit)
                    if ring == "1":
                        cut = (one, two, pre, pre2)
                    else:   # the K cut decides the association, the ring does not
                        for got, ref in zip((one, two, pre, pre2), cut):
                            assert G.same_bits(got, ref), (fmt, rows, cols, "ring on/off under the K cut")
