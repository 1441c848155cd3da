"""GPU parity: the HIP path against the CPU oracle on the same seeded inputs,
through the C ABI.

Bars: activation quantization, per-block integer dots and dequantized weights
bit-exact; final f32 within max-relative error 1e-5 (|x-y| / max(|y|, 1), the
reference's own metric) of every accumulation order the reference has, and
bit-exact against the order each kernel follows when no K-split is in play.
"""
import ctypes as C
import json
import os

import numpy as np
import pytest

import oracle
from camelid_amd import binding as B
from camelid_amd.binding import DeviceBuffer, Weight, check, lib
from tests import gpu_util as G

pytestmark = pytest.mark.gpu

FMTS = [("Q8_0", B.CML_Q8_0), ("Q4_0", B.CML_Q4_0), ("Q4_K", B.CML_Q4_K), ("Q6_K", B.CML_Q6_K)]
TOL = 1e-5

# The accumulation order a kernel follows bit for bit (when it does not split K).
EXACT_ORDER = {B.CML_Q8_0: oracle.ORDER_PRIMARY, B.CML_Q4_0: oracle.ORDER_PRIMARY,
               B.CML_Q4_K: oracle.ORDER_PRIMARY, B.CML_Q6_K: oracle.ORDER_ALT}


@pytest.fixture(scope="module", autouse=True)
def _init():
    assert lib().cml_available() == 1, "a GPU node is present but libcamelid_hip cannot use it"
    B.init(0)
    yield


def check_outputs(fmt, wire, cols, x_scales, x_q, got, row_start=0, rows=None, expect_exact=True):
    for order in (oracle.ORDER_PRIMARY, oracle.ORDER_ALT):
        if order == oracle.ORDER_ALT and not G.is_k(fmt):
            continue
        want = oracle.matmul_q(fmt, wire, cols, x_scales, x_q, order=order, row_start=row_start, rows=rows, threads=8)
        err = G.max_rel(got, want)
        assert err <= TOL, f"order {order}: max rel err {err}"
        if expect_exact and order == EXACT_ORDER[fmt]:
            assert G.same_bits(got, want), f"not bit-identical to reference order {order}"


# ----------------------------------------------------------- quantizers ----

def _activation_cases(cols, rng):
    x = rng.standard_normal((6, cols)).astype(np.float32)
    x[1] *= 1e-3
    x[2] *= 50.0
    x[3, :cols // 2] = 0.0          # all-zero blocks
    x[4] = np.round(x[4] * 4) / 4   # many exact ties after scaling
    x[5, ::7] = -x[5, ::7]
    return x


def test_quantize_q8_0_bit_exact():
    rng = np.random.default_rng(100)
    for cols in (32, 2048, 3072, 4096 + 32):
        G.say(f"quantize_q8_0 cols={cols}")
        x = _activation_cases(cols, rng)
        # exact .5 ties: amax = 127 makes the inverse scale 1.0
        x[0, :32] = 0.0
        x[0, 0] = 127.0
        x[0, 1:7] = [2.5, 0.5, -0.5, -2.5, 1.5, -1.5]
        s, q = G.gpu_quantize(False, x)
        so, qo = oracle.quantize_q8_0(x)
        assert np.array_equal(s.view(np.uint32), so.view(np.uint32))
        assert np.array_equal(q, qo)
    assert list(q[0, :7]) == [127, 3, 1, -1, -3, 2, -2]


def test_quantize_q8_k_bit_exact():
    rng = np.random.default_rng(101)
    for cols in (256, 3072, 4096, 14336):
        G.say(f"quantize_q8_k cols={cols}")
        x = _activation_cases(cols, rng)
        x[0, :256] = 0.0
        x[0, 5], x[0, 9] = 3.0, -3.0   # equal magnitudes: the first one sets the sign
        x[0, 17:21] = [1.5 * 3 / 127, 2.5 * 3 / 127, -0.5 * 3 / 127, 0.5 * 3 / 127]
        d, q = G.gpu_quantize(True, x)
        do, qo = oracle.quantize_q8_k(x)
        assert np.array_equal(d.view(np.uint32), do.view(np.uint32))
        assert np.array_equal(q, qo)
    assert q[0, 5] == -127 and q[0, 9] == 127


# ------------------------------------------------- layout and dequantize ----

@pytest.mark.parametrize("name,fmt", FMTS)
def test_relayout_is_a_pure_permutation(name, fmt):
    rng = np.random.default_rng(110 + fmt)
    bv = oracle.block_values(fmt)
    for rows, cols in ((1, bv), (7, 3 * bv), (33, 8 * bv), (130, 5 * bv)):
        G.say(f"relayout {name} {rows}x{cols}")
        wire = rng.integers(0, 256, size=rows * oracle.row_bytes(fmt, cols), dtype=np.uint8)
        w = Weight.upload(fmt, rows, cols, wire)
        assert np.array_equal(w.download(), wire)
        rb = oracle.row_bytes(fmt, cols)
        for start, count in ((16, rows - 19), (2, 3), (5, rows - 6), (17, 1)):   # bands may start anywhere
            if start + count > rows or count <= 0:
                continue
            band = w.slice(start, count)
            assert np.array_equal(band.download(), wire[start * rb:(start + count) * rb])
            if count > 4:   # a band of a band
                inner = band.slice(3, count - 4)
                assert np.array_equal(inner.download(), wire[(start + 3) * rb:(start + count - 1) * rb])


@pytest.mark.parametrize("name,fmt", FMTS)
def test_dequantize_bit_exact_golden_and_random(name, fmt):
    gold = os.path.join(os.path.dirname(__file__), "golden", "dequant", f"{name}.json")
    fx = json.load(open(gold))
    wire = np.frombuffer(bytes.fromhex(fx["quant_hex"]), dtype=np.uint8)
    ref = np.array([int(v, 16) if isinstance(v, str) else int(v) for v in fx["ref_f32_bits"]], dtype=np.uint32)
    G.say(f"dequantize golden {name}")
    w = Weight.upload(fmt, 1, fx["n_elements"], wire)
    assert np.array_equal(G.gpu_dequant(w).view(np.uint32), ref)
    rng = np.random.default_rng(120 + fmt)
    rows, cols = 37, 4 * oracle.block_values(fmt)
    wire = G.synth_weight(fmt, rows, cols, seed=120 + fmt)
    # also arbitrary scale/min bytes, not only what the quantizer emits
    wire2 = rng.integers(0, 256, size=wire.size, dtype=np.uint8)
    bb = oracle.block_bytes(fmt)
    d_off = {B.CML_Q8_0: [0], B.CML_Q4_0: [0], B.CML_Q4_K: [0, 2], B.CML_Q6_K: [208]}[fmt]
    w2 = wire2.reshape(-1, bb)
    w1 = wire.reshape(-1, bb)
    for off in d_off:
        w2[:, off:off + 2] = w1[:, off:off + 2]  # keep finite f16 scales
    for wr in (wire, wire2):
        G.say(f"dequantize random {name}")
        w = Weight.upload(fmt, rows, cols, wr)
        got = G.gpu_dequant(w)
        assert np.array_equal(got.view(np.uint32), oracle.dequant(fmt, wr).view(np.uint32))


# ------------------------------------------------------- integer block dots ----

@pytest.mark.parametrize("name,fmt", FMTS)
def test_block_dots_bit_exact(name, fmt):
    rng = np.random.default_rng(130 + fmt)
    bv = oracle.block_values(fmt)
    for rows, cols in ((5, bv), (67, 6 * bv), (129, 16 * bv)):
        G.say(f"block_dots {name} {rows}x{cols}")
        wire = rng.integers(0, 256, size=rows * oracle.row_bytes(fmt, cols), dtype=np.uint8)
        q = rng.integers(-128, 128, size=cols).astype(np.int8)
        w = Weight.upload(fmt, rows, cols, wire)
        got = G.gpu_block_dots(w, q)
        want = oracle.block_ints(fmt, wire, cols, q)
        assert np.array_equal(got, want)


# ------------------------------------------------------------------- gemv ----

SMALL_SHAPES = {
    B.CML_Q8_0: [(1, 32), (9, 64), (130, 2048), (2049, 57 * 32), (513, 96 * 32)],
    B.CML_Q4_0: [(1, 32), (9, 64), (130, 2048), (2049, 57 * 32), (513, 96 * 32)],
    B.CML_Q4_K: [(1, 256), (9, 512), (130, 4096), (2049, 5 * 256), (300, 56 * 256)],
    B.CML_Q6_K: [(1, 256), (9, 512), (130, 3072), (2049, 5 * 256), (300, 56 * 256)],
}


@pytest.mark.parametrize("name,fmt", FMTS)
def test_gemv_matches_oracle_small_and_ragged(name, fmt):
    rng = np.random.default_rng(140 + fmt)
    for rows, cols in SMALL_SHAPES[fmt]:
        G.say(f"gemv {name} {rows}x{cols}")
        wire = G.synth_weight(fmt, rows, cols, seed=rows * 7 + cols)
        x = rng.standard_normal(cols).astype(np.float32)
        s, q = oracle.quantize_activation(fmt, x)
        w = Weight.upload(fmt, rows, cols, wire)
        with G.env(CAMELID_HIP_EXACT_ORDER="1"):
            got = G.gpu_gemm(w, s, q)
        check_outputs(fmt, wire, cols, s, q, got, expect_exact=True)
        got = G.gpu_gemm(w, s, q)  # default K-split policy: tolerance only
        check_outputs(fmt, wire, cols, s, q, got, expect_exact=False)
        if fmt == B.CML_Q6_K:
            # the deeper register buffers taken for weights with thousands of row tiles: same bits
            with G.env(CAMELID_HIP_Q6K_DEEP_MIN_TILES=1):
                assert G.same_bits(G.gpu_gemm(w, s, q), got)
                assert G.same_bits(G.gpu_matmul_f32(w, x), G.gpu_matmul_f32(w, x))
            with G.env(CAMELID_HIP_Q6K_DEEP_MIN_TILES=1, CAMELID_HIP_EXACT_ORDER="1"):
                check_outputs(fmt, wire, cols, s, q, G.gpu_gemm(w, s, q), expect_exact=True)


def test_q4k_gemv_every_configuration_agrees():
    rng = np.random.default_rng(150)
    rows, cols = 301, 56 * 256
    wire = G.synth_weight(B.CML_Q4_K, rows, cols, seed=150)
    x = rng.standard_normal(cols).astype(np.float32)
    s, q = oracle.quantize_activation(B.CML_Q4_K, x)
    w = Weight.upload(B.CML_Q4_K, rows, cols, wire)
    x2 = np.stack([x, rng.standard_normal(cols).astype(np.float32)])
    s2, q2 = oracle.quantize_activation(B.CML_Q4_K, x2)
    for ks, tpw in ((1, 1), (1, 2), (1, 4), (1, 8), (2, 1), (2, 4), (4, 1), (4, 2), (8, 1)):
        per_rpw = []
        for rpw in (16, 8):   # rows per wave: 8 = two lane groups per row on neighbouring super-blocks
            G.say(f"gemv Q4_K ksplit={ks} tiles_per_wg={tpw} rows_per_wave={rpw}")
            with G.env(CAMELID_HIP_Q4K_KSPLIT=ks, CAMELID_HIP_Q4K_TILES_PER_WG=tpw, CAMELID_HIP_Q4K_ROWS_PER_WAVE=rpw):
                got = G.gpu_gemm(w, s, q)
                ints = G.gpu_block_dots(w, q)
            check_outputs(B.CML_Q4_K, wire, cols, s, q, got, expect_exact=(ks == 1))
            assert np.array_equal(ints, oracle.block_ints(B.CML_Q4_K, wire, cols, q))
            per_rpw.append(got)
            # the load form with per-lane clamping (taken when a K part is not whole buffers) and
            # the one without: same bits, one and two tokens
            with G.env(CAMELID_HIP_Q4K_KSPLIT=ks, CAMELID_HIP_Q4K_TILES_PER_WG=tpw, CAMELID_HIP_Q4K_ROWS_PER_WAVE=rpw,
                       CAMELID_HIP_Q4K_MFMA_MIN_TOKENS=1 << 30):
                two = G.gpu_gemm(w, s2, q2)
                with G.env(CAMELID_HIP_Q4K_CLAMPED_LOADS=1):
                    assert G.same_bits(G.gpu_gemm(w, s, q), got)
                    assert G.same_bits(G.gpu_gemm(w, s2, q2), two)
                with G.env(CAMELID_HIP_Q4K_GENERAL_ENTRY=1):   # the kernel entry that also serves expert groups
                    assert G.same_bits(G.gpu_gemm(w, s, q), got)
                    assert G.same_bits(G.gpu_gemm(w, s2, q2), two)
            assert G.same_bits(two[0], got) and not G.same_bits(two[1], got)
        assert G.same_bits(per_rpw[0], per_rpw[1])


@pytest.mark.parametrize("name,fmt", FMTS)
def test_gemv_residual_and_band_view(name, fmt):
    rng = np.random.default_rng(160 + fmt)
    rows, cols = 96, 4 * oracle.block_values(fmt) * (2 if not G.is_k(fmt) else 1)
    wire = G.synth_weight(fmt, rows, cols, seed=160 + fmt)
    x = rng.standard_normal(cols).astype(np.float32)
    s, q = oracle.quantize_activation(fmt, x)
    w = Weight.upload(fmt, rows, cols, wire)
    res = rng.standard_normal(rows).astype(np.float32)
    for rpw in (16, 8):
        G.say(f"gemv residual {name} rows_per_wave={rpw}")
        with G.env(CAMELID_HIP_Q4K_ROWS_PER_WAVE=rpw):
            _residual_and_band_view(name, fmt, rows, cols, wire, w, x, s, q, res, rng)
        if fmt != oracle.Q4_K:
            break


def _residual_and_band_view(name, fmt, rows, cols, wire, w, x, s, q, res, rng):
    with G.env(CAMELID_HIP_EXACT_ORDER="1"):
        base = G.gpu_gemm(w, s, q)
        got = G.gpu_gemm(w, s, q, residual=res)
        assert G.same_bits(got, (base + res).astype(np.float32))
        G.say(f"gemv band view {name}")
        band = w.slice(32, 40)   # rows 32..71: an expert band of a stacked tensor
        got = G.gpu_gemm(band, s, q)
        assert G.same_bits(got, base[32:72])
        check_outputs(fmt, wire, cols, s, q, got, row_start=32, rows=40, expect_exact=True)
        # the reference's own band test starts inside a tile (matvec_rows_proj(2, 3, ..),
        # src/gemma4_runtime.rs:22666-22675): bands are bitwise the rows of the full matvec
        xs = rng.standard_normal((16, cols)).astype(np.float32)
        sb, qb = oracle.quantize_activation(fmt, xs)
        full16 = G.gpu_gemm(w, sb, qb)
        for start, count in ((2, 3), (5, 60), (47, 49)):
            G.say(f"gemv band view {name} rows {start}..{start + count}")
            band = w.slice(start, count)
            assert G.same_bits(G.gpu_gemm(band, s, q), base[start:start + count])
            assert G.same_bits(G.gpu_matmul_f32(band, x), G.gpu_matmul_f32(w, x)[start:start + count])
            assert G.same_bits(G.gpu_gemm(band, sb, qb), full16[:, start:start + count])   # batched (matrix cores for Q4_K)
            assert G.same_bits(G.gpu_dequant(band).reshape(count, cols), G.gpu_dequant(w).reshape(rows, cols)[start:start + count])


# ------------------------------------------------------------- batched ----

@pytest.mark.parametrize("name,fmt", FMTS)
def test_gemm_cells_are_bitwise_the_gemv(name, fmt):
    rng = np.random.default_rng(170 + fmt)
    rows, cols = 257, (4096 if G.is_k(fmt) else 2048)
    wire = G.synth_weight(fmt, rows, cols, seed=170 + fmt)
    w = Weight.upload(fmt, rows, cols, wire)
    for n in (2, 3, 4, 7, 8, 13, 16):
        G.say(f"gemm {name} n={n}")
        x = rng.standard_normal((n, cols)).astype(np.float32)
        s, q = oracle.quantize_activation(fmt, x)
        got = G.gpu_gemm(w, s, q)   # default K-split policy (a function of the weight shape only)
        for t in range(n):
            assert G.same_bits(got[t], G.gpu_gemm(w, s[t], q[t])), f"token {t}"
        check_outputs(fmt, wire, cols, s, q, got, expect_exact=False)
        with G.env(CAMELID_HIP_EXACT_ORDER="1"):
            got = G.gpu_gemm(w, s, q)
        check_outputs(fmt, wire, cols, s, q, got, expect_exact=True)


@pytest.mark.parametrize("name,fmt", FMTS)
def test_matmul_f32_is_quantize_then_gemm(name, fmt):
    rng = np.random.default_rng(180 + fmt)
    rows, cols = 190, (3072 if G.is_k(fmt) else 2048)
    wire = G.synth_weight(fmt, rows, cols, seed=180 + fmt)
    w = Weight.upload(fmt, rows, cols, wire)
    for n in (1, 4):
        G.say(f"matmul_f32 {name} n={n}")
        x = rng.standard_normal((n, cols)).astype(np.float32)
        with G.env(CAMELID_HIP_EXACT_ORDER="1"):
            got = G.gpu_matmul_f32(w, x)
        want = oracle.matmul(fmt, wire, cols, x, order=EXACT_ORDER[fmt], threads=8)
        assert G.same_bits(got, want)


@pytest.mark.parametrize("rows,cols", [(190, 3072), (64, 256), (333, 4096), (48, 14336), (77, 1280)])
def test_q4k_fused_quantize_matvec_is_the_two_step_path(rows, cols):
    """Single-token cml_matmul_f32 on Q4_K quantizes inside the matvec kernel: same bits as
    quantize_q8_k followed by the matvec, for every workgroup shape, on activations with zero
    super-blocks, equal magnitudes of both signs, exact rounding ties and NaNs."""
    fmt = oracle.Q4_K
    rng = np.random.default_rng(7000 + rows)
    wire = G.synth_weight(fmt, rows, cols, seed=7100 + rows)
    w = Weight.upload(fmt, rows, cols, wire)
    acts = _activation_cases(cols, rng)
    acts[0, :256] = 0.0
    acts[0, 5], acts[0, 9] = 3.0, -3.0
    acts[0, 17:21] = [1.5 * 3 / 127, 2.5 * 3 / 127, -0.5 * 3 / 127, 0.5 * 3 / 127]
    acts[1, 3] = np.nan
    acts[2, -256:] = 0.0
    for i, x in enumerate(acts):
        for tpw in (0, 1, 2, 3, 4, 7, 8):
            for ks in (0, 1, 2):
                if ks > cols // 256:
                    continue
                for rpw in (16, 8):
                    G.say(f"Q4_K fused quantize+matvec {rows}x{cols} act={i} tiles_per_wg={tpw} ksplit={ks} rows_per_wave={rpw}")
                    with G.env(CAMELID_HIP_Q4K_FUSED_TILES_PER_WG=tpw, CAMELID_HIP_Q4K_KSPLIT=ks, CAMELID_HIP_Q4K_ROWS_PER_WAVE=rpw):
                        with G.env(CAMELID_HIP_FUSED_QUANT=2):   # also where the shape policy would not fuse
                            fused = G.gpu_matmul_f32(w, x)
                            with G.env(CAMELID_HIP_Q4K_GENERAL_ENTRY=1):
                                assert G.same_bits(G.gpu_matmul_f32(w, x), fused)
                        with G.env(CAMELID_HIP_FUSED_QUANT=0, CAMELID_HIP_Q4K_ROWS_PER_WAVE=16):
                            two_step = G.gpu_matmul_f32(w, x)
                    assert G.same_bits(fused, two_step)
        if i != 1:  # the oracle's f64 criterion has no meaning for a NaN input; bits above cover it
            with G.env(CAMELID_HIP_EXACT_ORDER="1"):
                got = G.gpu_matmul_f32(w, x)
            want = oracle.matmul(fmt, wire, cols, x[None, :], order=EXACT_ORDER[fmt], threads=8)[0]
            assert G.same_bits(got, want)


def test_launch_shape_knobs_need_the_tuning_switch():
    """A knob that only chooses among kernels of equal bits is honoured when CAMELID_HIP_TUNING=1 is set
    with it and ignored otherwise (a stray variable cannot move a production call onto another kernel);
    the knobs that choose the accumulation order are honoured on their own.  The counters say which
    kernel ran."""
    fmt, rows, cols = oracle.Q4_K, 12288, 4096
    w = Weight.upload(fmt, rows, cols, G.synth_weight(fmt, rows, cols, seed=8801))
    x = np.random.default_rng(8802).standard_normal(cols).astype(np.float32)
    with G.engaged(r"^q4k\.dot\.wg8\.fused$"):
        want = G.gpu_matmul_f32(w, x)
    with G.env(CAMELID_HIP_Q4K_CU=0, CAMELID_HIP_TUNING=0), G.engaged(r"^q4k\.dot\.wg8\.fused$", none=(r"^q4k\.dot\.ring",)):
        assert G.same_bits(G.gpu_matmul_f32(w, x), want)
    with G.env(CAMELID_HIP_Q4K_CU=0, CAMELID_HIP_TUNING=1), G.engaged(r"^q4k\.dot\.ring\.fused$", none=(r"^q4k\.dot\.wg8",)):
        assert G.same_bits(G.gpu_matmul_f32(w, x), want)
    # an order knob without the switch: the 8-lane order of the reference's generic CPU lane
    with G.env(CAMELID_HIP_Q4K_LANE_ORDER=1, CAMELID_HIP_TUNING=0), G.engaged(r"^q4k\.lanes$", none=(r"^q4k\.dot\.",)):
        G.gpu_matmul_f32(w, x)


@pytest.mark.parametrize("rows", [12288, 14336, 14327, 16384])
def test_q4k_eight_wave_launch_is_the_four_wave_launch_and_the_two_step_path(rows):
    """Rows of 4096 values on 12288 to 16384 rows (no K cut): cml_matmul_f32 runs the eight-wave launch
    whose quantizer gives a 32-lane half wave to each super-block.  Same bits as the four-wave ring launch
    (CAMELID_HIP_Q4K_CU=0, 16-lane quantizer rows), as quantize_q8_k followed by the matvec, and as the
    oracle, on activations built to break a quantizer: zero super-blocks, the maximum magnitude held by both
    signs (first holder positive, first holder negative, inside one lane, in different lanes, in the two
    16-lane rows of a half wave, in the two halves), exact rounding ties, a super-block of equal values, NaNs;
    also on a row band that starts inside a 16-row tile.  The counters prove which launch ran."""
    fmt, cols = oracle.Q4_K, 4096
    rng = np.random.default_rng(8000 + rows)
    wire = G.synth_weight(fmt, rows, cols, seed=8100 + rows)
    w = Weight.upload(fmt, rows, cols, wire)
    acts = rng.standard_normal((6, cols)).astype(np.float32)
    a = acts[0]
    a[0:256] = 0.0                                    # an all-zero super-block
    a[256 + 5], a[256 + 6] = 3.5, -3.5                # both signs in one lane (values 8l..8l+7), positive first
    a[512 + 6], a[512 + 5] = 3.5, -3.5                # ... negative first
    a[768 + 3], a[768 + 100] = -4.0, 4.0              # different lanes of one 16-lane row, negative first
    a[1024 + 3], a[1024 + 200] = 4.0, -4.0            # the two 16-lane rows of a half wave, positive first
    a[1280 + 130], a[1280 + 255] = -4.5, 4.5          # upper row only, negative first
    a[1536:1792] = 2.0                                # a super-block of equal values
    a[1792:2048] = -2.0
    a[2048 + 7] = 127.0
    a[2048 + 8:2048 + 12] = [0.5, 1.5, -0.5, -2.5]    # exact .5 ties under iscale = -1
    a[2304 + 0], a[2304 + 255] = -6.0, 6.0            # first and last value of a super-block
    b = acts[1]
    b[3], b[300], b[1000] = np.nan, np.nan, np.nan    # NaNs are skipped by the maximum scan
    b[256 * 5:256 * 6] = np.nan                       # a whole super-block of NaNs
    acts[2, :] = 0.0                                  # everything zero
    acts[3, 1::2] = -acts[3, ::2]                     # every magnitude twice, alternating signs
    acts[4] = np.round(acts[4] * 8) / 8               # many repeated magnitudes
    band = w.slice(5, rows - 9)
    s_all, q_all = oracle.quantize_activation(fmt, np.nan_to_num(acts))
    for i, x in enumerate(acts):
        G.say(f"Q4_K eight-wave launch {rows}x4096 act={i}")
        with G.engaged(r"^q4k\.dot\.wg8\.fused$", none=(r"^q4k\.dot\.ring", r"^q4k\.dot\.buffers", r"^quantize\.")):
            got = G.gpu_matmul_f32(w, x)
            got_band = G.gpu_matmul_f32(band, x)
        with G.env(CAMELID_HIP_Q4K_CU=0), G.engaged(r"^q4k\.dot\.ring\.fused$", none=(r"^q4k\.dot\.wg8",)):
            four = G.gpu_matmul_f32(w, x)
        with G.env(CAMELID_HIP_FUSED_QUANT=0), G.engaged(r"^quantize\.q8_k$", r"^q4k\.dot\.ring$", none=(r"^q4k\.dot\.wg8", r"fused")):
            two_step = G.gpu_matmul_f32(w, x)
        assert G.same_bits(got, four), (rows, i)
        assert G.same_bits(got, two_step), (rows, i)
        assert G.same_bits(got_band, got[5:rows - 4]), (rows, i)
        if i != 1:   # the oracle's comparison has no meaning for NaN inputs; the two-step bits above cover them
            want = oracle.matmul(fmt, wire, cols, x[None, :], order=EXACT_ORDER[fmt], threads=16)[0]
            assert G.same_bits(got, want), (rows, i)
            d_gpu, q_gpu = G.gpu_quantize(True, x)
            assert np.array_equal(q_gpu, q_all[i]) and np.array_equal(d_gpu.view(np.uint32), s_all[i].view(np.uint32))


@pytest.mark.parametrize("rows", [12288, 14336, 14327])
def test_q4k_eight_wave_launch_replays_a_few_tokens(rows):
    """Two, three (and, under its knob, four) tokens on the eight-wave launch: the weight of a step unpacked once and
    replayed against every token's staged row.  Each cell is the single-token call's bits and the oracle's, the
    counters show the launch, and with it switched off (CAMELID_HIP_Q4K_CU_TOKENS=1) the former paths give the same
    bits: the 16-row-wave ring launch for two tokens, the matrix-core launch for three and four."""
    fmt, cols = oracle.Q4_K, 4096
    rng = np.random.default_rng(8400 + rows)
    wire = G.synth_weight(fmt, rows, cols, seed=8500 + rows)
    w = Weight.upload(fmt, rows, cols, wire)
    x = rng.standard_normal((4, cols)).astype(np.float32)
    x[1, :512] = 0.0
    x[2, 1::2] = -x[2, ::2]
    x[3, 7], x[3, 1000] = 9.0, -9.0
    singles = np.stack([G.gpu_matmul_f32(w, x[t]) for t in range(4)])
    want = oracle.matmul(fmt, wire, cols, x, order=EXACT_ORDER[fmt], threads=16)
    assert G.same_bits(singles, want)
    for n in (2, 3, 4):
        G.say(f"Q4_K eight-wave launch {rows}x4096, {n} tokens")
        with G.env(CAMELID_HIP_Q4K_CU_TOKENS=4), G.engaged(r"^q4k\.dot\.wg8\.fused\.tokens$", none=(r"^q4k\.mfma", r"^q4k\.dot\.ring", r"^quantize\.")):
            got = G.gpu_matmul_f32(w, x[:n])
        assert G.same_bits(got, singles[:n]), (rows, n)
        former = r"^q4k\.dot\.ring\.fused$" if n == 2 else r"^q4k\.mfma\.pair\.fused$"
        with G.env(CAMELID_HIP_Q4K_CU_TOKENS=1), G.engaged(former, none=(r"^q4k\.dot\.wg8",)):
            assert G.same_bits(G.gpu_matmul_f32(w, x[:n]), singles[:n]), (rows, n, "former path")
        default_kernel = r"^q4k\.dot\.wg8\.fused\.tokens$" if n <= 3 else r"^q4k\.mfma\.pair\.fused$"
        with G.engaged(default_kernel):
            assert G.same_bits(G.gpu_matmul_f32(w, x[:n]), singles[:n]), (rows, n, "default")


@pytest.mark.parametrize("rows,cols", [(12800, 1536), (12304, 2048), (13000, 2560), (12320, 3072), (16384, 3584),
                                       (13824, 5120), (12800, 6144), (12330, 8192)])
def test_q4k_eight_wave_launch_serves_rows_of_six_to_sixteen_super_blocks(rows, cols):
    """The eight-wave launch on the other row lengths it is built for (1536 to 3584 values: 6 to 14 super-blocks, an
    even count; 5120, 6144 and 8192 values: 20, 24 and 32 super-blocks, quantized in two passes), one to three tokens: the bits of the four-wave / matrix-core paths it replaces and of the oracle,
    also on a row band; the counters show the launch."""
    fmt = oracle.Q4_K
    rng = np.random.default_rng(8600 + cols)
    wire = G.synth_weight(fmt, rows, cols, seed=8700 + cols)
    w = Weight.upload(fmt, rows, cols, wire)
    x = rng.standard_normal((3, cols)).astype(np.float32)
    x[1, :256] = 0.0
    x[2, 5], x[2, cols - 3] = 7.0, -7.0
    want = oracle.matmul(fmt, wire, cols, x, order=EXACT_ORDER[fmt], threads=16)
    band = w.slice(3, rows - 20)
    for n in (1, 2, 3):
        G.say(f"Q4_K eight-wave launch {rows}x{cols}, {n} tokens")
        kernel = r"^q4k\.dot\.wg8\.fused$" if n == 1 else r"^q4k\.dot\.wg8\.fused\.tokens$"
        with G.engaged(kernel, none=(r"^q4k\.mfma", r"^q4k\.dot\.ring", r"^q4k\.dot\.buffers", r"^quantize\.")):
            got = G.gpu_matmul_f32(w, x[:n] if n > 1 else x[0])
            got_band = G.gpu_matmul_f32(band, x[:n] if n > 1 else x[0])
        got = np.asarray(got).reshape(n, rows)
        assert G.same_bits(got, want[:n]), (rows, cols, n)
        assert G.same_bits(np.asarray(got_band).reshape(n, rows - 20), got[:, 3:rows - 17]), (rows, cols, n, "band")
        with G.env(CAMELID_HIP_Q4K_CU=0), G.engaged(none=(r"^q4k\.dot\.wg8",)):
            former = np.asarray(G.gpu_matmul_f32(w, x[:n] if n > 1 else x[0])).reshape(n, rows)
        assert G.same_bits(former, got), (rows, cols, n, "former path")


@pytest.mark.parametrize("rows,cols,tokens,kernel", [
    (18944, 3584, (1, 2, 3), "wide"),     # ten waves per workgroup
    (24570, 4096, (1, 2, 3), "wide"),     # twelve, the last 16-row tile partly filled
    (17920, 5120, (1, 2, 3), "wide"),     # ten, two quantizer passes
    (28672, 4096, (3,), "wide"),          # sixteen: three tokens only
    (40000, 4096, (3, 4), "eight"),       # three and (from 24576 rows on) four tokens beyond one workgroup per compute unit: eight waves
    (24600, 3584, (4,), "eight"),
])
def test_q4k_wide_workgroups_beyond_one_eight_wave_workgroup_per_unit(rows, cols, tokens, kernel):
    """More than 16384 rows of 14 or 16 super-blocks: the one-workgroup-per-compute-unit launch with ten, twelve or
    sixteen waves per workgroup (and three tokens on eight waves at any row count).  The bits of the oracle and of
    the four-wave / matrix-core paths that served these shapes before, also on a row band; the counters show the launch."""
    fmt = oracle.Q4_K
    rng = np.random.default_rng(8800 + rows)
    wire = G.synth_weight(fmt, rows, cols, seed=8900 + rows)
    w = Weight.upload(fmt, rows, cols, wire)
    x = rng.standard_normal((4, cols)).astype(np.float32)
    x[1, :256] = 0.0
    x[2, 5], x[2, cols - 3] = 7.0, -7.0
    want = oracle.matmul(fmt, wire, cols, x, order=EXACT_ORDER[fmt], threads=16)
    band = w.slice(3, rows - 20)
    for n in tokens:
        G.say(f"Q4_K wide workgroups {rows}x{cols}, {n} tokens")
        name = r"^q4k\.dot\.wg8\.fused" + (r"\.tokens" if n > 1 else "") + (r"\.wide$" if kernel == "wide" else "$")
        with G.engaged(name, none=(r"^q4k\.mfma", r"^q4k\.dot\.ring", r"^q4k\.dot\.buffers", r"^quantize\.")):
            got = G.gpu_matmul_f32(w, x[:n] if n > 1 else x[0])
            got_band = G.gpu_matmul_f32(band, x[:n] if n > 1 else x[0])
        got = np.asarray(got).reshape(n, rows)
        assert G.same_bits(got, want[:n]), (rows, cols, n)
        assert G.same_bits(np.asarray(got_band).reshape(n, rows - 20), got[:, 3:rows - 17]), (rows, cols, n, "band")
        with G.env(CAMELID_HIP_Q4K_CU=0), G.engaged(none=(r"^q4k\.dot\.wg8",)):
            former = np.asarray(G.gpu_matmul_f32(w, x[:n] if n > 1 else x[0])).reshape(n, rows)
        assert G.same_bits(former, got), (rows, cols, n, "former path")


@pytest.mark.parametrize("rows", [4096, 3100, 6100])
def test_q4k_eight_wave_launch_under_the_k_cut_is_the_two_launch_path(rows):
    """Rows of 14336 values on 3072 to 6128 rows (the FFN down projection: the shape policy cuts K four ways):
    cml_matmul_f32 with one token runs ONE launch whose eight-wave workgroups quantize the row once each.  Same
    bits as the quantizing launch followed by the four-wave matvec (CAMELID_HIP_Q4K_CU=0), on the adversarial
    activations of the test above and on a row band; within 1e-5 of the oracle's uncut chain."""
    fmt, cols = oracle.Q4_K, 14336
    rng = np.random.default_rng(8200 + rows)
    wire = G.synth_weight(fmt, rows, cols, seed=8300 + rows)
    w = Weight.upload(fmt, rows, cols, wire)
    acts = rng.standard_normal((4, cols)).astype(np.float32)
    a = acts[0]
    a[0:256] = 0.0
    a[256 + 5], a[256 + 6] = 3.5, -3.5
    a[512 + 6], a[512 + 5] = 3.5, -3.5
    a[768 + 3], a[768 + 100] = -4.0, 4.0
    a[1024 + 3], a[1024 + 200] = 4.0, -4.0
    a[13 * 1024 + 130], a[13 * 1024 + 255] = -4.5, 4.5
    a[-256:] = 2.0                                    # the last super-block: equal values
    acts[1, 3], acts[1, 9000] = np.nan, np.nan
    acts[1, 256 * 55:] = np.nan
    acts[2, 1::2] = -acts[2, ::2]
    band = w.slice(5, rows - 9)
    for i, x in enumerate(acts):
        G.say(f"Q4_K eight-wave K-cut launch {rows}x14336 act={i}")
        # up to 4096 rows (one eight-wave workgroup per compute unit) the form of its own, beyond twelve-wave workgroups of the general one
        kernel = r"^q4k\.dot\.wg8\.kcut\.fused$" if rows <= 4096 else r"^q4k\.dot\.wg8\.kcut\.fused\.uneven$"
        with G.engaged(kernel, none=(r"^q4k\.dot\.ring", r"^q4k\.dot\.buffers", r"^quantize\.")):
            got = G.gpu_matmul_f32(w, x)
            got_band = G.gpu_matmul_f32(band, x)
        with G.env(CAMELID_HIP_Q4K_CU=0), G.engaged(r"^quantize\.q8_k$", r"^q4k\.dot\.", none=(r"^q4k\.dot\.wg8",)):
            two_launches = G.gpu_matmul_f32(w, x)
        with G.env(CAMELID_HIP_Q4K_KCUT_STAGED=0, CAMELID_HIP_Q4K_KCUT_ANY=2), \
                G.engaged(r"^q4k\.dot\.wg8\.kcut\.fused\.whole_row$", none=(r"^q4k\.dot\.wg8\.kcut\.fused$",)):
            whole_row = G.gpu_matmul_f32(w, x)   # the row quantized before the walk instead of pass by pass along it
        with G.env(CAMELID_HIP_Q4K_KCUT_ANY=2), G.engaged(r"^q4k\.dot\.wg8\.kcut\.fused$"):
            own_form = G.gpu_matmul_f32(w, x)
        assert G.same_bits(got, two_launches), (rows, i)
        assert G.same_bits(got, whole_row), (rows, i)
        assert G.same_bits(got, own_form), (rows, i)
        assert G.same_bits(got_band, got[5:rows - 4]), (rows, i)
        if i != 1:
            want = oracle.matmul(fmt, wire, cols, x[None, :], order=EXACT_ORDER[fmt], threads=16)[0]
            assert G.max_rel(got, want) <= TOL, (rows, i)


@pytest.mark.parametrize("rows,cols", [
    (4096, 4096), (5003, 4096), (4096, 6144), (3080, 8192),                       # cut four ways: parts of 2, 2, 3, 4 steps
    (8192, 3072), (11008, 4096), (9216, 5120), (6150, 6144), (10240, 8192),       # cut two ways: parts of 3, 4, 5, 6, 8 steps
    # parts that are no whole number of two-super-block steps, or longer than the forms above take
    (4096, 11008), (5120, 5120), (5125, 13824), (3584, 18944), (3584, 3584), (4100, 10240), (8192, 7168), (3300, 2304),
    (5000, 16384), (4096, 20480),
    # cut eight ways (fewer than 3072 rows), and rows of 2048 values cut two ways
    (2048, 8192), (2050, 14336), (2048, 11008), (2560, 10240), (3000, 12288), (8192, 2048), (2048, 5632),
])
def test_q4k_eight_wave_launch_under_the_k_cut_on_shorter_rows(rows, cols):
    """Rows of 2304 to 20480 values on fewer than 12288 rows (attention projections, smaller FFN matrices, the down
    projections of 11008-, 13824- and 18944-wide FFNs: the shape policy cuts K two or four ways, into parts that need
    not be whole steps or equal): one launch of eight-, twelve- or sixteen-wave workgroups that quantize the row once each.
    Same bits as the four-wave launch it replaces (CAMELID_HIP_Q4K_KCUT_SHORT=0), whatever the workgroup width, on
    activations built to break a quantizer and on a row band; within 1e-5 of the oracle's uncut chain."""
    fmt = oracle.Q4_K
    rng = np.random.default_rng(9400 + rows + cols)
    wire = G.synth_weight(fmt, rows, cols, seed=9500 + rows + cols)
    w = Weight.upload(fmt, rows, cols, wire)
    acts = rng.standard_normal((3, cols)).astype(np.float32)
    a = acts[0]
    a[0:256] = 0.0
    a[256 + 5], a[256 + 6] = 3.5, -3.5
    a[512 + 6], a[512 + 5] = 3.5, -3.5
    a[768 + 3], a[768 + 100] = -4.0, 4.0
    a[-256:] = 2.0
    acts[1, 3], acts[1, cols - 300] = np.nan, np.nan
    acts[2, 1::2] = -acts[2, ::2]
    band = w.slice(5, rows - 9)
    # below 3072 rows the policy would cut long rows eight ways; it stops at four by default and the eight-way forms stay selectable
    for most in ((4, 8) if rows < 3072 else (4,)):
        with G.env(CAMELID_HIP_Q4K_MAX_KSPLIT=most):
            _check_q4k_k_cut_forms(fmt, wire, w, band, acts, rows, cols, most)


def _check_q4k_k_cut_forms(fmt, wire, w, band, acts, rows, cols, most):
    served = r"^q4k\.dot\.wg8\.kcut\.fused(\.(short|uneven))?$"   # (rows of 14336 values cut four ways: the form of their own)
    for i, x in enumerate(acts):
        G.say(f"Q4_K K-cut launch on shorter rows {rows}x{cols} act={i} at most {most} parts")
        with G.engaged(served, none=(r"^q4k\.dot\.ring", r"^q4k\.dot\.buffers", r"^quantize\.")):
            got = G.gpu_matmul_f32(w, x)
            got_band = G.gpu_matmul_f32(band, x)
        with G.env(CAMELID_HIP_Q4K_KCUT_SHORT=0, CAMELID_HIP_Q4K_CU=0), G.engaged(r"^q4k\.dot\.", none=(r"^q4k\.dot\.wg8",)):
            four_wave = G.gpu_matmul_f32(w, x)
        assert G.same_bits(got, four_wave), (rows, cols, i, most)
        assert G.same_bits(got_band, got[5:rows - 4]), (rows, cols, i, most)
        for width in (8, 12, 16):
            with G.env(CAMELID_HIP_Q4K_KCUT_WAVES=width), G.engaged(served):
                assert G.same_bits(G.gpu_matmul_f32(w, x), got), (rows, cols, i, most, width)
        if i != 1:
            want = oracle.matmul(fmt, wire, cols, x[None, :], order=EXACT_ORDER[fmt], threads=16)[0]
            assert G.max_rel(got, want) <= TOL, (rows, cols, i, most)


@pytest.mark.parametrize("rows,cols", [(4096, 4096), (4096, 14336), (11008, 4096), (4096, 11008), (5120, 5120), (2048, 8192),
                                       (5003, 8192), (9216, 5120), (3584, 18944), (8192, 3072)])
def test_q4k_k_cut_launch_replays_two_and_three_tokens(rows, cols):
    """Two and three (on parts of up to four steps: four) tokens on a weight whose shape the policy cuts K for: one launch of the general K-cut form, each
    step's unpacked weight replayed against every token's staged row.  Every cell is the single-token call's bits,
    also on a row band; the counters show the launch, and with it switched off (CAMELID_HIP_Q4K_KCUT_TOKENS=0) the
    former paths (16-row waves for two tokens, the matrix cores for three) give the same bits."""
    fmt = oracle.Q4_K
    rng = np.random.default_rng(10100 + rows + cols)
    wire = G.synth_weight(fmt, rows, cols, seed=10200 + rows + cols)
    w = Weight.upload(fmt, rows, cols, wire)
    x = rng.standard_normal((4, cols)).astype(np.float32)
    x[0, :256] = 0.0
    x[1, 1::2] = -x[1, ::2]
    x[2, 5], x[2, cols - 3] = 7.0, -7.0
    x[2, 300] = np.nan
    singles = np.stack([G.gpu_matmul_f32(w, x[t]) for t in range(4)])
    band = w.slice(5, rows - 9)
    four = (rows, cols) in ((4096, 4096), (11008, 4096), (5120, 5120), (2048, 8192), (5003, 8192), (8192, 3072))   # parts of up to four steps
    for n in (2, 3, 4) if four else (2, 3):
        if n * (cols // 256) * 292 + 1536 > 64 * 1024:
            continue   # the tokens' staging does not fit LDS: the former paths serve the call
        G.say(f"Q4_K K-cut launch {rows}x{cols}, {n} tokens")
        with G.engaged(r"^q4k\.dot\.wg8\.kcut\.fused\.tokens$", none=(r"^q4k\.mfma", r"^q4k\.dot\.ring", r"^q4k\.dot\.buffers", r"^quantize\.")):
            got = np.asarray(G.gpu_matmul_f32(w, x[:n])).reshape(n, rows)
            got_band = np.asarray(G.gpu_matmul_f32(band, x[:n])).reshape(n, rows - 9)
        assert G.same_bits(got, singles[:n]), (rows, cols, n)
        assert G.same_bits(got_band, got[:, 5:rows - 4]), (rows, cols, n, "band")
        with G.env(CAMELID_HIP_Q4K_KCUT_TOKENS=0), G.engaged(none=(r"^q4k\.dot\.wg8\.kcut\.fused\.tokens$",)):
            former = np.asarray(G.gpu_matmul_f32(w, x[:n])).reshape(n, rows)
        assert G.same_bits(former, got), (rows, cols, n, "former path")
        for width in (8, 12, 16):
            with G.env(CAMELID_HIP_Q4K_KCUT_WAVES=width), G.engaged(r"^q4k\.dot\.wg8\.kcut\.fused\.tokens$"):
                assert G.same_bits(np.asarray(G.gpu_matmul_f32(w, x[:n])).reshape(n, rows), got), (rows, cols, n, width)


@pytest.mark.parametrize("rows", [4096, 3100, 6100])
def test_q6k_eight_wave_launch_under_the_k_cut_is_the_two_launch_path(rows):
    """Q6_K rows of 14336 values on up to 6136 rows (the FFN down projection: the shape policy cuts K four ways):
    cml_matmul_f32 with one token runs ONE launch whose eight-wave workgroups quantize the row once each, pass by
    pass along the walk.  Same bits as the quantizing launch followed by the four-wave matvec (CAMELID_HIP_Q6K_CU=0)
    on activations built to break a quantizer, and with a residual-free row count that is not a multiple of the
    workgroup's 16 rows; within 1e-5 of the oracle's uncut chain."""
    fmt, cols = oracle.Q6_K, 14336
    rng = np.random.default_rng(9200 + rows)
    wire = G.synth_weight(fmt, rows, cols, seed=9300 + rows)
    w = Weight.upload(fmt, rows, cols, wire)
    acts = rng.standard_normal((4, cols)).astype(np.float32)
    a = acts[0]
    a[0:256] = 0.0
    a[256 + 5], a[256 + 6] = 3.5, -3.5
    a[512 + 6], a[512 + 5] = 3.5, -3.5
    a[768 + 3], a[768 + 100] = -4.0, 4.0
    a[1024 + 3], a[1024 + 200] = 4.0, -4.0
    a[13 * 1024 + 130], a[13 * 1024 + 255] = -4.5, 4.5
    a[-256:] = 2.0                                    # the last super-block: equal values
    acts[1, 3], acts[1, 9000] = np.nan, np.nan
    acts[1, 256 * 55:] = np.nan
    acts[2, 1::2] = -acts[2, ::2]
    band = w.slice(5, rows - 9)
    for i, x in enumerate(acts):
        G.say(f"Q6_K eight-wave K-cut launch {rows}x14336 act={i}")
        # up to 4096 rows (one eight-wave workgroup per compute unit) the form of its own, beyond twelve-wave workgroups of the general one
        kernel = r"^q6k\.dot\.wg8\.kcut\.fused$" if rows <= 4096 else r"^q6k\.dot\.wg8\.kcut\.fused\.any$"
        with G.engaged(kernel, none=(r"^q6k\.dot\.buffers", r"^q6k\.dot\.deep", r"^quantize\.")):
            got = G.gpu_matmul_f32(w, x)
            got_band = G.gpu_matmul_f32(band, x)
        with G.env(CAMELID_HIP_Q6K_CU=0), G.engaged(r"^quantize\.q8_k$", r"^q6k\.dot\.", none=(r"^q6k\.dot\.wg8",)):
            two_launches = G.gpu_matmul_f32(w, x)
        assert G.same_bits(got, two_launches), (rows, i)
        assert G.same_bits(got_band, got[5:rows - 4]), (rows, i)
        if i != 1:
            want = oracle.matmul(fmt, wire, cols, x[None, :], order=EXACT_ORDER[fmt], threads=16)[0]
            assert G.max_rel(got, want) <= TOL, (rows, i)


@pytest.mark.parametrize("rows,cols", [
    (4096, 4096), (5003, 5120), (4096, 6144), (3080, 8192), (4096, 11008), (5125, 13824), (3584, 18944),   # cut four ways
    (8192, 2048), (6200, 3072), (3584, 3584), (11008, 4096), (9216, 5120), (6200, 6144), (8200, 8192),      # cut two ways
    (14336, 4096), (18944, 3584), (13000, 5120), (12300, 3072), (24570, 4096), (12400, 8192),                # no cut
])
def test_q6k_eight_wave_launch_under_the_k_cut_on_other_rows(rows, cols):
    """Q6_K rows of 2048 to 18944 values on fewer than 12288 rows (the shape policy cuts K two or four ways, into
    parts that need not be equal), and rows of 3072 to 8192 values on 12288 to 24576 rows (no cut): one launch of
    eight-, ten- or twelve-wave workgroups, at most one per compute unit, that quantize the row once each.
    Same bits as the four-wave launches they replace (CAMELID_HIP_Q6K_KCUT_ANY=0), whatever the workgroup width,
    on activations built to break a quantizer and on a row band; within 1e-5 of the oracle's uncut chain."""
    fmt = oracle.Q6_K
    rng = np.random.default_rng(9600 + rows + cols)
    wire = G.synth_weight(fmt, rows, cols, seed=9700 + rows + cols)
    w = Weight.upload(fmt, rows, cols, wire)
    acts = rng.standard_normal((3, cols)).astype(np.float32)
    a = acts[0]
    a[0:256] = 0.0
    a[256 + 5], a[256 + 6] = 3.5, -3.5
    a[512 + 6], a[512 + 5] = 3.5, -3.5
    a[768 + 3], a[768 + 100] = -4.0, 4.0
    a[-256:] = 2.0
    acts[1, 3], acts[1, cols - 300] = np.nan, np.nan
    acts[2, 1::2] = -acts[2, ::2]
    band = w.slice(5, rows - 9)
    for i, x in enumerate(acts):
        G.say(f"Q6_K K-cut launch {rows}x{cols} act={i}")
        with G.engaged(r"^q6k\.dot\.wg8\.kcut\.fused\.any$", none=(r"^q6k\.dot\.buffers", r"^q6k\.dot\.deep", r"^quantize\.")):
            got = G.gpu_matmul_f32(w, x)
            got_band = G.gpu_matmul_f32(band, x)
        with G.env(CAMELID_HIP_Q6K_KCUT_ANY=0), G.engaged(r"^q6k\.dot\.", none=(r"^q6k\.dot\.wg8",)):
            four_wave = G.gpu_matmul_f32(w, x)
        assert G.same_bits(got, four_wave), (rows, cols, i)
        assert G.same_bits(got_band, got[5:rows - 4]), (rows, cols, i)
        for width in (8, 12):
            for two_per_step in (1, 0):   # (the no-cut form: two super-blocks of a row per ring step, or one)
                with G.env(CAMELID_HIP_Q6K_KCUT_WAVES=width, CAMELID_HIP_Q6K_CU_U2=two_per_step), G.engaged(r"^q6k\.dot\.wg8\.kcut\.fused\.any$"):
                    assert G.same_bits(G.gpu_matmul_f32(w, x), got), (rows, cols, i, width, two_per_step)
        if i != 1:
            want = oracle.matmul(fmt, wire, cols, x[None, :], order=EXACT_ORDER[fmt], threads=16)[0]
            assert G.max_rel(got, want) <= TOL, (rows, cols, i)


@pytest.mark.parametrize("rows,cols", [(4096, 4096), (5003, 5120), (3080, 8192), (8192, 2048), (6200, 3072), (11008, 4096), (9216, 5120),
                                       (14336, 4096), (18944, 3584)])
def test_q6k_k_cut_launch_replays_two_tokens(rows, cols):
    """Two tokens on the Q6_K one-workgroup-per-unit launch (rows of up to 8192 values): each step's unpacked weight
    replayed against both staged rows.  Every cell is the single-token call's bits, also on a row band; the counters
    show the launch, and with it switched off (CAMELID_HIP_Q6K_KCUT_TOKENS=0) the four-wave launch gives the same bits."""
    fmt = oracle.Q6_K
    rng = np.random.default_rng(10300 + rows + cols)
    wire = G.synth_weight(fmt, rows, cols, seed=10400 + rows + cols)
    w = Weight.upload(fmt, rows, cols, wire)
    x = rng.standard_normal((2, cols)).astype(np.float32)
    x[0, :256] = 0.0
    x[1, 1::2] = -x[1, ::2]
    x[1, 300] = np.nan
    singles = np.stack([G.gpu_matmul_f32(w, x[t]) for t in range(2)])
    band = w.slice(8, rows - 16)   # (Q6_K views start on a row of the 8-row tiles or anywhere: the planes are row-major)
    G.say(f"Q6_K K-cut launch {rows}x{cols}, two tokens")
    with G.engaged(r"^q6k\.dot\.wg8\.kcut\.fused\.two$", none=(r"^q6k\.dot\.buffers", r"^q6k\.mfma", r"^quantize\.")):
        got = np.asarray(G.gpu_matmul_f32(w, x)).reshape(2, rows)
        got_band = np.asarray(G.gpu_matmul_f32(band, x)).reshape(2, rows - 16)
    assert G.same_bits(got, singles), (rows, cols)
    assert G.same_bits(got_band, got[:, 8:rows - 8]), (rows, cols, "band")
    with G.env(CAMELID_HIP_Q6K_KCUT_TOKENS=0), G.engaged(none=(r"^q6k\.dot\.wg8\.kcut\.fused\.two$",)):
        former = np.asarray(G.gpu_matmul_f32(w, x)).reshape(2, rows)
    assert G.same_bits(former, got), (rows, cols, "former path")


@pytest.mark.parametrize("rows,cols", [(190, 3072), (64, 256), (333, 4096), (40, 14336), (77, 1280)])
def test_q4k_fused_two_tokens_is_the_two_step_path(rows, cols):
    """Two-token cml_matmul_f32 on Q4_K quantizes both rows inside the matvec kernel: the bits of
    quantize_q8_k + matmul, and of the oracle, for every workgroup shape and K split."""
    fmt = oracle.Q4_K
    rng = np.random.default_rng(7200 + rows)
    wire = G.synth_weight(fmt, rows, cols, seed=7250 + rows)
    w = Weight.upload(fmt, rows, cols, wire)
    acts = _activation_cases(cols, rng)
    acts[0, :256] = 0.0
    acts[1, -256:] = 0.0
    acts[2, 17:21] = [1.5 * 3 / 127, 2.5 * 3 / 127, -0.5 * 3 / 127, 0.5 * 3 / 127]
    for pair in ((0, 1), (2, 0), (1, 2)):
        x = np.ascontiguousarray(acts[list(pair)])
        for tpw in (0, 1, 3, 8):
            for ks in (0, 1, 2):
                if ks > cols // 256:
                    continue
                G.say(f"Q4_K fused two tokens {rows}x{cols} pair={pair} tiles_per_wg={tpw} ksplit={ks}")
                with G.env(CAMELID_HIP_Q4K_FUSED_TILES_PER_WG=tpw, CAMELID_HIP_Q4K_KSPLIT=ks):
                    with G.env(CAMELID_HIP_FUSED_QUANT=2):
                        fused = G.gpu_matmul_f32(w, x)
                        with G.env(CAMELID_HIP_Q4K_CLAMPED_LOADS=1):
                            assert G.same_bits(G.gpu_matmul_f32(w, x), fused)
                    with G.env(CAMELID_HIP_FUSED_QUANT=0):
                        two_step = G.gpu_matmul_f32(w, x)
                assert G.same_bits(fused, two_step), (pair, tpw, ks)
        with G.env(CAMELID_HIP_EXACT_ORDER="1", CAMELID_HIP_FUSED_QUANT=2):
            got = G.gpu_matmul_f32(w, x)
        want = oracle.matmul(fmt, wire, cols, x, order=EXACT_ORDER[fmt], threads=8)
        assert G.same_bits(got, want)


@pytest.mark.parametrize("rows,cols", [(190, 3072), (64, 512), (333, 4096), (14336, 4096), (77, 1280)])
def test_q4k_fused_quantize_small_batches_are_the_two_step_path(rows, cols):
    """3 to 8 f32 rows against a Q4_K weight run as ONE launch (the matrix-core kernel quantizes them
    itself): bit for bit the quantize launch + matmul, on rows with zero blocks, equal magnitudes of
    both signs and exact rounding ties, for a full weight and a band that starts inside a tile."""
    fmt = B.CML_Q4_K
    rng = np.random.default_rng(rows + cols)
    wire = G.synth_weight(fmt, rows, cols, seed=rows * 11 + cols)
    w = Weight.upload(fmt, rows, cols, wire)
    band = w.slice(3, rows - 7) if rows > 20 else None
    for n in (3, 4, 5, 6, 8):                 # 8: served when CAMELID_HIP_FUSED_QUANT_BATCH_MAX allows it
        x = rng.standard_normal((n, cols)).astype(np.float32)
        x[0, :256] = 0.0                      # an empty super-block
        x[1, 256:512] = np.float32(0.5)       # every value the maximum
        x[n - 1, 0] = -x[n - 1, 1]            # two first holders of the maximum, opposite signs
        x[2, :256] = np.round(x[2, :256] * 4) / 4
        G.say(f"Q4_K fused quantize, {n} tokens, {rows}x{cols}")
        s, q = oracle.quantize_activation(fmt, x)
        with G.env(CAMELID_HIP_EXACT_ORDER="1", CAMELID_HIP_FUSED_QUANT_BATCH_MAX=8):
            got = G.gpu_matmul_f32(w, x)
            two_step = G.gpu_gemm(w, s, q)
            with G.env(CAMELID_HIP_EXACT_ORDER="1", CAMELID_HIP_FUSED_QUANT_BATCH=0):
                unfused = G.gpu_matmul_f32(w, x)
            if band is not None:
                got_band = G.gpu_matmul_f32(band, x)
        assert G.same_bits(got, two_step)
        assert G.same_bits(got, unfused)
        check_outputs(fmt, wire, cols, s, q, got, expect_exact=True)
        if band is not None:
            assert G.same_bits(got_band, got[:, 3:rows - 4])


@pytest.mark.parametrize("rows,cols", [(190, 3072), (61, 256), (333, 4096), (20, 14336), (2100, 1280)])
def test_q6k_fused_quantize_matvec_is_the_two_step_path(rows, cols):
    """One- and two-token cml_matmul_f32 on Q6_K quantizes inside the matvec kernel: the bits of
    quantize_q8_k + matmul for every K split and buffer depth, and of the oracle."""
    fmt = oracle.Q6_K
    rng = np.random.default_rng(7700 + rows)
    wire = G.synth_weight(fmt, rows, cols, seed=7750 + rows)
    w = Weight.upload(fmt, rows, cols, wire)
    acts = _activation_cases(cols, rng)
    acts[0, :256] = 0.0
    acts[0, 5], acts[0, 9] = 3.0, -3.0
    acts[1, 17:21] = [1.5 * 3 / 127, 2.5 * 3 / 127, -0.5 * 3 / 127, 0.5 * 3 / 127]
    acts[2, -256:] = 0.0
    for sel in ((0,), (1,), (2, 0), (1, 2)):
        x = np.ascontiguousarray(acts[list(sel)])
        xin = x[0] if len(sel) == 1 else x
        for ks in (0, 1, 2, 4):
            if ks > cols // 256:
                continue
            for deep in (2048, 1):
                G.say(f"Q6_K fused quantize+matvec {rows}x{cols} rows={sel} ksplit={ks} deep_min_tiles={deep}")
                with G.env(CAMELID_HIP_Q6K_KSPLIT=ks, CAMELID_HIP_Q6K_DEEP_MIN_TILES=deep):
                    with G.env(CAMELID_HIP_FUSED_QUANT=2):
                        fused = G.gpu_matmul_f32(w, xin)
                    with G.env(CAMELID_HIP_FUSED_QUANT=0):
                        two_step = G.gpu_matmul_f32(w, xin)
                assert G.same_bits(fused, two_step), (sel, ks, deep)
        with G.env(CAMELID_HIP_EXACT_ORDER="1", CAMELID_HIP_FUSED_QUANT=2):
            got = G.gpu_matmul_f32(w, xin)
        want = oracle.matmul(fmt, wire, cols, x, order=EXACT_ORDER[fmt], threads=8)
        assert G.same_bits(got.reshape(want.shape), want)


@pytest.mark.parametrize("name,fmt", [("Q8_0", oracle.Q8_0), ("Q4_0", oracle.Q4_0)])
@pytest.mark.parametrize("rows,cols", [(190, 2048), (33, 32), (70, 3072 + 32), (16, 14336)])
def test_b32_fused_quantize_matvec_is_the_two_step_path(name, fmt, rows, cols):
    """Single-token cml_matmul_f32 on Q8_0 / Q4_0 weights quantizes inside the matvec kernel: same
    bits as quantize_q8_0 followed by the matvec, on activations with zero blocks, exact .5 ties
    (rounded away from zero) and NaNs, for both lane mappings."""
    rng = np.random.default_rng(7300 + rows + fmt)
    wire = G.synth_weight(fmt, rows, cols, seed=7400 + rows + fmt)
    w = Weight.upload(fmt, rows, cols, wire)
    acts = _activation_cases(cols, rng)
    acts[0, :32] = 0.0
    acts[0, 0] = 127.0
    acts[0, 1:7] = [2.5, 0.5, -0.5, -2.5, 1.5, -1.5]
    acts[1, 3] = np.nan
    lanes_env = "CAMELID_HIP_Q8_0_LANES" if fmt == oracle.Q8_0 else "CAMELID_HIP_Q4_0_LANES"
    for i, x in enumerate(acts):
        for lanes in (0, 8, 16, 32, 64):
            G.say(f"{name} fused quantize+matvec {rows}x{cols} act={i} lanes={lanes}")
            with G.env(**{lanes_env: lanes}):
                with G.env(CAMELID_HIP_FUSED_QUANT=2):
                    fused = G.gpu_matmul_f32(w, x)
                with G.env(CAMELID_HIP_FUSED_QUANT=0):
                    two_step = G.gpu_matmul_f32(w, x)
            assert G.same_bits(fused, two_step)
        if i != 1:
            want = oracle.matmul(fmt, wire, cols, x[None, :], order=EXACT_ORDER[fmt], threads=8)[0]
            assert G.same_bits(fused, want)


@pytest.mark.parametrize("rows,cols", [(14336, 4096), (4096, 14336), (5120, 14336), (4096, 4096), (4096, 11008), (11008, 4096),
                                       (18944, 3584), (13824, 5120), (200, 2304), (32000, 4096)])
def test_q4k_loads_only_twin_runs_for_every_single_token_launch_shape(rows, cols):
    """cml_calibrate_weight_loads (the matvec's weight requests and nothing else, what bench.py prices a shape's
    ceiling with) is served whatever launch cml_matmul_f32 picks for the shape, and leaves the weight intact."""
    fmt = oracle.Q4_K
    wire = G.synth_weight(fmt, rows, cols, seed=9950 + rows + cols)
    w = Weight.upload(fmt, rows, cols, wire)
    x = np.random.default_rng(9960 + rows).standard_normal(cols).astype(np.float32)
    before = G.gpu_matmul_f32(w, x)
    scratch = DeviceBuffer(256)
    stream = C.c_void_p()
    check(lib().cml_stream_create(C.byref(stream)))
    G.say(f"Q4_K loads-only twin {rows}x{cols}")
    with G.engaged(r"^q4k\.calibrate\."):
        check(lib().cml_calibrate_weight_loads(w.handle, scratch.ptr, stream), "cml_calibrate_weight_loads")
        check(lib().cml_stream_sync(stream))
    assert G.same_bits(G.gpu_matmul_f32(w, x), before)


@pytest.mark.parametrize("name,fmt", [("Q8_0", oracle.Q8_0), ("Q4_0", oracle.Q4_0)])
@pytest.mark.parametrize("rows,cols", [(4096, 14336), (2050, 11008), (8192, 14336), (5120, 13824), (3000, 16384)])
def test_b32_rows_longer_than_8192_values_run_as_one_launch_where_the_token_fits_registers(name, fmt, rows, cols):
    """Single-token cml_matmul_f32 on Q8_0 / Q4_0 rows of 8193 to 16384 values: one launch (the quantizer inside, the
    token in registers) wherever the launch shape holds the token in registers, else a quantizing launch and the
    matvec -- the counters show which; both give the oracle's bits."""
    rng = np.random.default_rng(10500 + rows + fmt)
    wire = G.synth_weight(fmt, rows, cols, seed=10600 + rows + fmt)
    w = Weight.upload(fmt, rows, cols, wire)
    x = rng.standard_normal(cols).astype(np.float32)
    x[:64] = 0.0
    x[64:70] = [2.5, 0.5, -0.5, -2.5, 1.5, -1.5]
    x[-32:] = 3.0
    want = oracle.matmul(fmt, wire, cols, x[None, :], order=EXACT_ORDER[fmt], threads=16)[0]
    G.say(f"{name} {rows}x{cols}: default")
    before = G.launch_counts()
    got = G.gpu_matmul_f32(w, x)
    after = G.launch_counts()
    fired = {k: v - before.get(k, 0) for k, v in after.items() if v > before.get(k, 0)}
    assert G.same_bits(got, want), (name, rows, cols, fired)
    one_launch = not any(k.startswith("quantize.") for k in fired)
    # Q8_0 on 4097 to 8192 rows of at least 8192 values runs four-wave workgroups, which stage the token: two launches
    expect_one = not (fmt == oracle.Q8_0 and 4096 < rows <= 8192)
    assert one_launch == expect_one, (name, rows, cols, fired)
    with G.env(CAMELID_HIP_B32_LONG_ROWS_FUSE=0), G.engaged(r"^quantize\.q8_0$"):
        assert G.same_bits(G.gpu_matmul_f32(w, x), want), (name, rows, cols, "two launches")
    with G.env(CAMELID_HIP_FUSED_QUANT=2), G.engaged(none=(r"^quantize\.",)):
        assert G.same_bits(G.gpu_matmul_f32(w, x), want), (name, rows, cols, "one launch forced")


@pytest.mark.parametrize("name,fmt", [("Q8_0", oracle.Q8_0), ("Q4_0", oracle.Q4_0)])
@pytest.mark.parametrize("rows,cols", [(9001, 5120), (8192, 8192), (10250, 8192), (6000, 8192)])
def test_b32_fused_launch_shapes_on_rows_longer_than_4096_values(name, fmt, rows, cols):
    """Single-token cml_matmul_f32 on Q8_0 / Q4_0 rows of more than 4096 values (every workgroup stages the token
    through LDS): sixteen-wave workgroups beyond 8192 rows, four-wave ones with two-step buffers for Q8_0 rows of
    8192 values on up to 8192 rows, eight-wave ones otherwise.  The counters show which launch ran; each gives the
    oracle's bits and those of quantize + matvec, as does every workgroup width and buffer depth the knobs select."""
    rng = np.random.default_rng(9800 + rows + fmt)
    wire = G.synth_weight(fmt, rows, cols, seed=9900 + rows + fmt)
    w = Weight.upload(fmt, rows, cols, wire)
    x = rng.standard_normal(cols).astype(np.float32)
    x[:64] = 0.0
    x[64:70] = [2.5, 0.5, -0.5, -2.5, 1.5, -1.5]
    want = oracle.matmul(fmt, wire, cols, x[None, :], order=EXACT_ORDER[fmt], threads=16)[0]
    fam = "q8_0" if fmt == oracle.Q8_0 else "q4_0"
    if rows > 8192:
        kernel = rf"^{fam}\.dot\.p16\.w16\.fused$"
    elif fmt == oracle.Q8_0 and cols >= 8192:
        kernel = rf"^{fam}\.dot\.p16\.w4\.fused$"
    else:
        kernel = rf"^{fam}\.dot\.p16\.w8\.(deep\.)?fused$"
    G.say(f"{name} {rows}x{cols}: default launch")
    with G.engaged(kernel, none=(r"^quantize\.",)):
        got = G.gpu_matmul_f32(w, x)
    assert G.same_bits(got, want), (name, rows, cols)
    with G.env(CAMELID_HIP_FUSED_QUANT=0), G.engaged(r"^quantize\.q8_0$"):
        assert G.same_bits(G.gpu_matmul_f32(w, x), want), (name, rows, cols, "two launches")
    with G.env(CAMELID_HIP_B32_LONG_ROW_WAVES=0), G.engaged(rf"^{fam}\.dot\.p16\.w8\.(deep\.)?fused$"):
        assert G.same_bits(G.gpu_matmul_f32(w, x), want), (name, rows, cols, "eight waves")
    for most in (1, 2, 4, 8):   # how many float4 of the token a thread may hold in registers (beyond: staged through a loop)
        G.say(f"{name} {rows}x{cols}: at most {most} float4 of the token per thread")
        with G.env(CAMELID_HIP_B32_NXQ_MOST=most), G.engaged(rf"^{fam}\.dot\.p16\."):
            assert G.same_bits(G.gpu_matmul_f32(w, x), want), (name, rows, cols, "registers", most)
    for waves in (4, 8, 16):
        for depth in (2, 4):
            G.say(f"{name} {rows}x{cols}: waves={waves} depth={depth}")
            for most in (8, 1):
                with G.env(CAMELID_HIP_B32_FUSED_WAVES=waves, CAMELID_HIP_B32_DEPTH=depth, CAMELID_HIP_B32_NXQ_MOST=most), \
                        G.engaged(rf"^{fam}\.dot\.p16\.w{waves}\."):
                    assert G.same_bits(G.gpu_matmul_f32(w, x), want), (name, rows, cols, waves, depth, most)


@pytest.mark.parametrize("name,fmt", [("Q8_0", oracle.Q8_0), ("Q4_0", oracle.Q4_0)])
@pytest.mark.parametrize("rows,cols", [(190, 2048), (33, 32), (70, 3072 + 32), (5000, 1024), (16, 8192), (333, 4096), (14336, 4096)])
def test_b32_fused_two_tokens_is_the_two_step_path(name, fmt, rows, cols):
    """Two-token cml_matmul_f32 on Q8_0 / Q4_0 weights quantizes both rows inside the matvec
    kernel: the bits of quantize_q8_0 + matmul and of the oracle, for every lane mapping and
    workgroup size."""
    rng = np.random.default_rng(7500 + rows + fmt)
    wire = G.synth_weight(fmt, rows, cols, seed=7600 + rows + fmt)
    w = Weight.upload(fmt, rows, cols, wire)
    acts = _activation_cases(cols, rng)
    acts[0, :32] = 0.0
    acts[0, 1:7] = [2.5, 0.5, -0.5, -2.5, 1.5, -1.5]
    acts[2, -32:] = 0.0
    lanes_env = "CAMELID_HIP_Q8_0_LANES" if fmt == oracle.Q8_0 else "CAMELID_HIP_Q4_0_LANES"
    for pair in ((0, 2), (2, 1)):
        x = np.ascontiguousarray(acts[list(pair)])
        want = oracle.matmul(fmt, wire, cols, x, order=EXACT_ORDER[fmt], threads=8)
        for lanes in (0, 8, 16):
            for waves in (0, 4, 8):
                G.say(f"{name} fused two tokens {rows}x{cols} pair={pair} lanes={lanes} waves={waves}")
                with G.env(CAMELID_HIP_B32_FUSED_WAVES=waves, **{lanes_env: lanes}):
                    with G.env(CAMELID_HIP_FUSED_QUANT=2):
                        fused = G.gpu_matmul_f32(w, x)
                    with G.env(CAMELID_HIP_FUSED_QUANT=0):
                        two_step = G.gpu_matmul_f32(w, x)
                assert G.same_bits(fused, two_step), (pair, lanes, waves)
                assert G.same_bits(fused, want), (pair, lanes, waves)


# ----------------------------------------------------- errors and the seam ----

def test_error_paths_return_status_codes():
    L = lib()
    h = C.c_void_p()
    wire = np.zeros(144 * 3, np.uint8)
    assert L.cml_weight_upload(12, 3, 256, wire.ctypes.data, 100, C.byref(h)) == 3     # wrong byte count
    assert b"expected" in L.cml_last_error()
    assert L.cml_weight_upload(12, 3, 250, wire.ctypes.data, wire.nbytes, C.byref(h)) == 3  # cols not whole blocks
    assert L.cml_weight_upload(7, 3, 256, wire.ctypes.data, wire.nbytes, C.byref(h)) == 2   # unknown format
    w = Weight.upload(12, 3, 256, wire)
    assert L.cml_weight_slice(w.handle, 2, 5, C.byref(h)) == 3
    assert L.cml_gemv(w.handle, None, None, None, None, None) == 2
    empty = Weight.upload(12, 0, 256, np.zeros(0, np.uint8))   # zero rows: accepted, nothing to do
    assert L.cml_gemv(empty.handle, None, None, None, None, None) == 0
    d = DeviceBuffer(64)
    assert L.cml_quantize_q8_k(d.ptr, 1, 100, d.ptr, d.ptr, None) == 3


@pytest.mark.parametrize("name,fmt", FMTS)
def test_host_slice_seam(name, fmt):
    rng = np.random.default_rng(190 + fmt)
    rows, cols, n = 77, (1024 if G.is_k(fmt) else 512), 3
    wire = G.synth_weight(fmt, rows, cols, seed=190 + fmt)
    x = rng.standard_normal((n, cols)).astype(np.float32)
    s, q = oracle.quantize_activation(fmt, x)
    out = np.full((n, rows), np.nan, np.float32)
    before = lib().cml_run_count()
    G.say(f"try_linear_rows {name}")
    for _ in range(2):  # second call hits the device weight cache
        with G.env(CAMELID_HIP_EXACT_ORDER="1"):
            rc = lib().cml_try_linear_rows(fmt, s.ctypes.data, q.ctypes.data, wire.ctypes.data, wire.nbytes, n, rows,
                                           cols, out.ctypes.data)
        assert rc == 0, lib().cml_last_error()
        assert G.same_bits(out, oracle.matmul_q(fmt, wire, cols, s, q, order=EXACT_ORDER[fmt]))
    assert lib().cml_run_count() >= before + 2
    bad = lib().cml_try_linear_rows(fmt, s.ctypes.data, q.ctypes.data, wire.ctypes.data, wire.nbytes - 1, n, rows,
                                    cols, out.ctypes.data)
    assert bad != 0


def test_q8_0_block_seam_takes_in_memory_blocks():
    """The seam the reference's CPU linear calls on its decode path (try_q8_0_block_linear_row,
    src/cuda.rs:1089-1222, called at src/inference.rs:27944): weights as 36-byte in-memory blocks
    (f32 scale + 32 int8).  Same bits as the wire-format matvec; blocks whose scale is not an f16
    value, and wrong lengths, make the call decline."""
    rng = np.random.default_rng(195)
    rows, cols = 70, 2048
    nb = cols // 32
    wire = G.synth_weight(B.CML_Q8_0, rows, cols, seed=195).reshape(rows * nb, 34)
    blocks = np.zeros((rows * nb, 36), np.uint8)
    blocks[:, :4] = np.ascontiguousarray(wire[:, :2]).view(np.float16).astype(np.float32).view(np.uint8).reshape(-1, 4)
    blocks[:, 4:] = wire[:, 2:]
    x = rng.standard_normal((1, cols)).astype(np.float32)
    s, q = oracle.quantize_activation(B.CML_Q8_0, x)
    out = np.full(rows, np.nan, np.float32)
    G.say("try_q8_0_block_linear_row")
    L = lib()
    before = L.cml_run_count()
    for _ in range(2):   # second call hits the device weight cache
        rc = L.cml_try_q8_0_block_linear_row(s.ctypes.data, q.ctypes.data, blocks.ctypes.data, blocks.nbytes, rows, nb, out.ctypes.data)
        assert rc == 0, L.cml_last_error()
        assert G.same_bits(out, oracle.matmul_q(B.CML_Q8_0, wire.reshape(-1), cols, s, q)[0])
    assert L.cml_run_count() >= before + 2
    assert L.cml_try_q8_0_block_linear_row(s.ctypes.data, q.ctypes.data, blocks.ctypes.data, blocks.nbytes - 36, rows, nb, out.ctypes.data) != 0
    odd = blocks.copy()
    odd[5, :4] = np.float32([0.1]).view(np.uint8)          # 0.1 is not an f16 value
    assert L.cml_try_q8_0_block_linear_row(s.ctypes.data, q.ctypes.data, odd.ctypes.data, odd.nbytes, rows, nb, out.ctypes.data) == 6


# ------------------------------------------------- matrix-core path (n >= 16) ----

# CAMELID_HIP_*_MFMA_SHAPE -> the workgroup shape in the kernel-family counter names
# (g<token groups per wave>t<waves over the tokens of a row tile>)
MFMA_SHAPES = {1: "g1t1", 2: "g2t1", 3: "g4t1", 4: "g1t2", 5: "g2t2", 6: "g1t4"}

# (4096, 4096) and (2000, 18*256): the matvec kernel splits K four ways (even and uneven parts);
# (1600, 9*256) and (6400, 8*256): two ways; (300, 56*256): eight ways (reproduced inside the lane)
@pytest.mark.parametrize("rows,cols", [(130, 1024), (2049, 5 * 256), (300, 56 * 256), (16, 256), (4096, 4096), (2000, 18 * 256),
                                       (1600, 9 * 256), (6400, 8 * 256)])
def test_q4k_matrix_core_cells_are_bitwise_the_gemv(rows, cols):
    fmt = B.CML_Q4_K
    rng = np.random.default_rng(rows + cols)
    wire = G.synth_weight(fmt, rows, cols, seed=rows * 3 + cols)
    w = Weight.upload(fmt, rows, cols, wire)
    for n in (4, 5, 8, 16, 17, 33, 50, 64, 70):
        x = rng.standard_normal((n, cols)).astype(np.float32)
        s, q = oracle.quantize_activation(fmt, x)
        for shape in (0, 1, 2, 3, 4, 5, 6):   # 0 = the default workgroup shape, 1..6 = every other one
            G.say(f"Q4_K matrix-core {rows}x{cols} n={n} shape={shape}")
            # which kernel must have run: any matrix-core one by default, the named workgroup shape otherwise
            want_kernel = r"^q4k\.mfma\." if shape == 0 else r"^q4k\.mfma\.(tile|serial_split)\." + MFMA_SHAPES[shape] + r"(\.|$)"
            with G.env(CAMELID_HIP_Q4K_MFMA_SHAPE=shape), G.engaged(want_kernel, none=(r"^q4k\.dot\.",)):
                got = G.gpu_gemm(w, s, q)                      # default K-split policy, reproduced across waves or in-lane
            if shape == 0:
                with G.env(CAMELID_HIP_Q4K_MFMA_SERIAL_SPLIT=1), G.engaged(r"^q4k\.mfma\.", none=(r"^q4k\.mfma\.ksplit", r"^q4k\.dot\.")):
                    assert G.same_bits(got, G.gpu_gemm(w, s, q))
            with G.env(CAMELID_HIP_Q4K_MFMA_MIN_TOKENS=1 << 30), G.engaged(r"^q4k\.dot\.", none=(r"^q4k\.mfma\.",)):
                ref = G.gpu_gemm(w, s, q)                      # the packed-dot kernel on the same inputs
            assert G.same_bits(got, ref)
            check_outputs(fmt, wire, cols, s, q, got, expect_exact=False)
        with G.env(CAMELID_HIP_EXACT_ORDER="1"):
            got = G.gpu_gemm(w, s, q)
        check_outputs(fmt, wire, cols, s, q, got, expect_exact=True)


@pytest.mark.parametrize("rows,cols", [(200, 2 * 256), (75, 7 * 256), (1000, 15 * 256), (14336, 4096), (97, 4096), (300, 8 * 256)])
def test_q4k_two_waves_per_tile_keep_one_chain(rows, cols):
    """Up to 16 tokens against rows of 2..16 super-blocks with no K cut: two waves share a row tile
    and split K, the chain stays one chain -- the oracle's order bit for bit, the same bits as one
    wave per tile (CAMELID_HIP_Q4K_MFMA_PAIR=0), also on a row band that starts inside a tile."""
    fmt = B.CML_Q4_K
    rng = np.random.default_rng(rows * 7 + cols)
    wire = G.synth_weight(fmt, rows, cols, seed=rows + cols)
    w = Weight.upload(fmt, rows, cols, wire)
    band = w.slice(5, rows - 9)
    for n in (3, 9, 16):
        x = rng.standard_normal((n, cols)).astype(np.float32)
        s, q = oracle.quantize_activation(fmt, x)
        want = oracle.matmul_q(fmt, wire, cols, s, q, order=oracle.ORDER_PRIMARY, threads=8)
        G.say(f"Q4_K two waves per tile {rows}x{cols} n={n}")
        with G.env(CAMELID_HIP_EXACT_ORDER="1"):
            with G.engaged(r"^q4k\.mfma\.pair$", none=(r"^q4k\.mfma\.(tile|serial_split|ksplit)", r"^q4k\.dot\.")):
                got = G.gpu_gemm(w, s, q)
                got_band = G.gpu_gemm(band, s, q)
            with G.env(CAMELID_HIP_EXACT_ORDER="1", CAMELID_HIP_Q4K_MFMA_PAIR=0), G.engaged(r"^q4k\.mfma\.tile\.g1t1", none=(r"^q4k\.mfma\.pair", r"^q4k\.dot\.")):
                one_wave = G.gpu_gemm(w, s, q)
            # one wave per tile walking three groups of row tiles per workgroup (a last group partly past the end of
            # the weight, a band that starts inside a tile), with the row length known at compile time or not
            with G.env(CAMELID_HIP_EXACT_ORDER="1", CAMELID_HIP_Q4K_MFMA_PAIR=0, CAMELID_HIP_Q4K_MFMA_UNITS=3), \
                    G.engaged(r"^q4k\.mfma\.tile\.g1t1\.once.*\.units$" if rows > 64 else r"^q4k\.mfma\.tile\.g1t1\.once"):
                walk = G.gpu_gemm(w, s, q)
                walk_band = G.gpu_gemm(band, s, q)
            with G.env(CAMELID_HIP_EXACT_ORDER="1", CAMELID_HIP_Q4K_MFMA_PAIR=0, CAMELID_HIP_Q4K_MFMA_UNITS=2, CAMELID_HIP_Q4K_MFMA_FIXED_ROWS=0), \
                    G.engaged(r"^q4k\.mfma\.tile\.g1t1\.once", none=(r"\.k(8|16)",)):
                walk_any = G.gpu_gemm(w, s, q)
        assert G.same_bits(got, want)
        assert G.same_bits(got, one_wave)
        assert G.same_bits(got_band, want[:, 5:rows - 4])
        assert G.same_bits(walk, want)
        assert G.same_bits(walk_band, want[:, 5:rows - 4])
        assert G.same_bits(walk_any, want)


@pytest.mark.parametrize("rows,cols,tokens", [(16400, 2048, (9, 16, 17, 32)), (20000, 14 * 256, (5, 16, 25)), (49168, 4096, (3, 4, 7, 31))])
def test_q4k_tall_weights_take_the_resident_walk(rows, cols, tokens):
    """Up to 16 tokens against a Q4_K weight of more than 16384 rows (no K cut): one wave per row tile, the
    activation staged once per workgroup, the launch sized to about one resident workgroup per compute unit that
    walks its share of the weight -- from f32 rows (cml_matmul_f32: the quantizing launch, then this one) the
    oracle's chain bit for bit, and the bits of the two-waves-per-tile kernel that serves shorter weights.  Four
    tokens on a vocabulary-sized weight come here too (three on a weight of this size stay on the packed-dot
    launch), and 17 to 32 tokens as two token groups per wave; the last group of row tiles lies partly past the
    end of the weight."""
    fmt = B.CML_Q4_K
    rng = np.random.default_rng(rows + cols)
    wire = G.synth_weight(fmt, rows, cols, seed=rows * 3 + cols)
    w = Weight.upload(fmt, rows, cols, wire)
    for n in tokens:
        x = rng.standard_normal((n, cols)).astype(np.float32)
        s, q = oracle.quantize_activation(fmt, x)
        want = oracle.matmul_q(fmt, wire, cols, s, q, order=oracle.ORDER_PRIMARY, threads=8)
        G.say(f"Q4_K tall weight {rows}x{cols} n={n}")
        walk = r"^q4k\.dot\.wg8\.fused\.tokens$" if n == 3 else (r"^q4k\.mfma\.tile\.g1t1\.once" if n <= 16 else r"^q4k\.mfma\.tile\.g2t1\.once")
        with G.env(CAMELID_HIP_EXACT_ORDER="1"):
            with G.engaged(walk, none=(r"^q4k\.mfma\.pair",)):
                got = G.gpu_matmul_f32(w, x)
            # the launches that served these calls before: two waves per tile up to 16 tokens, the phased kernel beyond
            with G.env(CAMELID_HIP_EXACT_ORDER="1", CAMELID_HIP_Q4K_MFMA_PAIR_MAX_ROWS=1 << 30, CAMELID_HIP_Q4K_TALL_TOKENS_MFMA=0,
                       CAMELID_HIP_Q4K_MFMA_ONCE_TWO_GROUPS=0), \
                    G.engaged(r"^q4k\.mfma\.tile\.g2t1$" if n > 16 else (r"^q4k\.mfma\.pair" if n > 4 else r"^q4k\.(dot\.wg8\.fused\.tokens|mfma\.pair)")):
                former = G.gpu_matmul_f32(w, x)
        assert G.same_bits(got, want)
        assert G.same_bits(got, former)


@pytest.mark.parametrize("rows,cols", [(16700, 20 * 256), (3001, 24 * 256), (2000, 32 * 256)])
def test_q4k_long_rows_take_the_staged_once_walk(rows, cols):
    """Up to 16 tokens against a Q4_K weight whose rows are 5120 / 6144 / 8192 values (no K cut): the staged-once walk
    with 32 slabs of LDS (one resident workgroup per compute unit) -- the oracle's chain bit for bit, and the
    bits of the phased kernel that served these shapes."""
    fmt = B.CML_Q4_K
    rng = np.random.default_rng(rows + cols)
    wire = G.synth_weight(fmt, rows, cols, seed=rows * 5 + cols)
    w = Weight.upload(fmt, rows, cols, wire)
    min_tiles = 0
    for n in (4, 16):
        x = rng.standard_normal((n, cols)).astype(np.float32)
        s, q = oracle.quantize_activation(fmt, x)
        want = oracle.matmul_q(fmt, wire, cols, s, q, order=oracle.ORDER_PRIMARY, threads=8)
        G.say(f"Q4_K tall weight, long rows {rows}x{cols} n={n}")
        with G.env(CAMELID_HIP_EXACT_ORDER="1", CAMELID_HIP_Q4K_MFMA_ONCE_LONG_MIN_TILES=min_tiles, CAMELID_HIP_Q4K_MFMA_MIN_TOKENS=3), \
                G.engaged(rf"^q4k\.mfma\.tile\.g1t1\.once\.k{cols // 256}"):
            got = G.gpu_gemm(w, s, q)
        with G.env(CAMELID_HIP_EXACT_ORDER="1", CAMELID_HIP_Q4K_MFMA_ONCE_LONG_MIN_TILES=1 << 30, CAMELID_HIP_Q4K_MFMA_MIN_TOKENS=3), \
                G.engaged(r"^q4k\.mfma\.tile\.g1t1$"):
            former = G.gpu_gemm(w, s, q)
        assert G.same_bits(got, want)
        assert G.same_bits(got, former)


@pytest.mark.parametrize("name,fmt", [("Q8_0", oracle.Q8_0), ("Q4_0", oracle.Q4_0)])
@pytest.mark.parametrize("rows,cols", [(130, 1024), (2049, 5 * 256), (77, 12 * 256), (16, 256)])
def test_b32_matrix_core_cells_are_bitwise_the_gemv(name, fmt, rows, cols):
    """Q8_0 / Q4_0 batches on the matrix cores: every cell is the matvec kernel's block-ordered
    chain, bit for bit, and the oracle's (these formats have one accumulation order)."""
    rng = np.random.default_rng(rows + cols + fmt)
    wire = G.synth_weight(fmt, rows, cols, seed=rows * 5 + cols + fmt)
    w = Weight.upload(fmt, rows, cols, wire)
    for n in (4, 5, 8, 16, 17, 33, 50, 64, 70):
        x = rng.standard_normal((n, cols)).astype(np.float32)
        if n == 5:
            x[1] = 0.0              # an all-zero token: scale 0, sums 0
            x[2, :32] = -x[2, :32].max() * 4   # a block at the negative extreme
        s, q = oracle.quantize_activation(fmt, x)
        tag = name.lower()
        with G.env(CAMELID_HIP_B32_MFMA_MIN_TOKENS=1 << 30), G.engaged(rf"^{tag}\.dot\.", none=(rf"^{tag}\.mfma\.",)):
            ref = G.gpu_gemm(w, s, q)                      # the packed-dot kernel on the same inputs
        for shape in (0, 1, 2, 3, 4, 5, 6):   # 0 = the default workgroup shape, 1..6 = every other one
            G.say(f"{name} matrix-core {rows}x{cols} n={n} shape={shape}")
            for deep in (0, 1):          # short phases / shallow ring, long phases / deep ring
                # MIN_TOKENS=1: the matrix-core kernels also below the batch size from which they pay
                want_kernel = rf"^{tag}\.mfma\." if shape == 0 else rf"^{tag}\.mfma\.tile\." + MFMA_SHAPES[shape] + r"\.w\d+\." + ("r[48]" if deep else "r2")
                with G.env(CAMELID_HIP_B32_MFMA_SHAPE=shape, CAMELID_HIP_B32_MFMA_DEEP=deep, CAMELID_HIP_B32_MFMA_MIN_TOKENS=1), \
                        G.engaged(want_kernel, none=(rf"^{tag}\.dot\.",)):
                    got = G.gpu_gemm(w, s, q)
                assert G.same_bits(got, ref)
        check_outputs(fmt, wire, cols, s, q, got, expect_exact=True)


@pytest.mark.parametrize("name,fmt", [("Q8_0", oracle.Q8_0), ("Q4_0", oracle.Q4_0)])
@pytest.mark.parametrize("rows,cols", [(130, 2 * 256), (45, 3 * 256), (2049, 5 * 256), (500, 8 * 256), (77, 12 * 256),
                                       (4100, 16 * 256), (16, 4 * 256)])
def test_b32_waves_sharing_a_row_tile_keep_the_block_order(name, fmt, rows, cols):
    """Up to 16 tokens on a matrix of few row tiles: 2, 4 or 8 waves share a row tile, each taking a
    run of the row's slabs, and hand the running sums on in order -- the block-order chain of the
    reference bit for bit, in every workgroup shape (CAMELID_HIP_B32_MFMA_KPAR = 1..4; 0 = one wave
    per tile), on ragged row counts and with a token count that leaves cells unused."""
    rng = np.random.default_rng(rows * 3 + cols + fmt)
    wire = G.synth_weight(fmt, rows, cols, seed=rows + cols * 7 + fmt)
    w = Weight.upload(fmt, rows, cols, wire)
    for n in (3, 9, 16):
        x = rng.standard_normal((n, cols)).astype(np.float32)
        x[n - 1, :64] = 0.0
        s, q = oracle.quantize_activation(fmt, x)
        want = oracle.matmul_q(fmt, wire, cols, s, q, order=oracle.ORDER_PRIMARY, threads=8)
        with G.env(CAMELID_HIP_B32_MFMA_MIN_TOKENS=1):
            tag, slabs = name.lower(), cols // 256
            for variant in (-1, 0, 1, 2, 3, 4):
                G.say(f"{name} waves per tile, {rows}x{cols} n={n} variant={variant}")
                # the kernel each variant selects for rows of this many slabs (launch_b32_mfma_fmt); every test matrix
                # has few enough row tiles for the default (-1) to share tiles as well
                if variant == 0:
                    want_kernel, never = rf"^{tag}\.mfma\.tile\.", (rf"^{tag}\.mfma\.kpar", rf"^{tag}\.dot\.")
                else:
                    table = ({1: "k4s2t1", 2: "k4s2t2", 3: "k8s1t1", 4: "k8s1t2"} if 4 <= slabs <= 8 else
                             {1: "k4s4t1", 2: "k8s2t1", 3: "k8s2t2"} if 8 < slabs <= 16 else {1: "k2s2t1", 2: "k2s2t1", 3: "k2s2t1", 4: "k2s2t1"})
                    want_kernel = rf"^{tag}\.mfma\.kpar\." + table.get(variant, r"k\d")
                    never = (rf"^{tag}\.mfma\.tile\.", rf"^{tag}\.dot\.")
                with G.env(CAMELID_HIP_B32_MFMA_MIN_TOKENS=1, CAMELID_HIP_B32_MFMA_KPAR=variant), G.engaged(want_kernel, none=never):
                    got = G.gpu_gemm(w, s, q)
                assert G.same_bits(got, want)


@pytest.mark.parametrize("name,fmt", [("Q8_0", oracle.Q8_0), ("Q4_0", oracle.Q4_0)])
def test_b32_rows_that_are_not_whole_slabs_take_the_packed_dot_kernel(name, fmt):
    rows, cols, n = 40, 352, 9     # 11 blocks: not a multiple of 8
    wire = G.synth_weight(fmt, rows, cols, seed=77 + fmt)
    w = Weight.upload(fmt, rows, cols, wire)
    x = np.random.default_rng(78).standard_normal((n, cols)).astype(np.float32)
    s, q = oracle.quantize_activation(fmt, x)
    G.say(f"{name} 11-block rows, 9 tokens")
    got = G.gpu_gemm(w, s, q)
    check_outputs(fmt, wire, cols, s, q, got, expect_exact=True)


# K split by the matvec kernel: (300, 12*256) and (300, 13*256) two ways, (4000, 16*256) and
# (1000, 18*256) four ways (even and uneven parts); the others not at all
@pytest.mark.parametrize("rows,cols", [(130, 1024), (2049, 5 * 256), (300, 12 * 256), (16, 256), (4000, 16 * 256), (300, 13 * 256),
                                       (1000, 18 * 256)])
def test_q6k_matrix_core_cells_are_bitwise_the_gemv(rows, cols):
    """Q6_K batches on the matrix cores: every cell is the matvec kernel's chain (K-split policy
    included), bit for bit; with the split off it is the oracle's fused order."""
    fmt = B.CML_Q6_K
    rng = np.random.default_rng(rows + cols + 6)
    wire = G.synth_weight(fmt, rows, cols, seed=rows * 7 + cols)
    w = Weight.upload(fmt, rows, cols, wire)
    for n in (5, 8, 16, 17, 33, 50, 64, 70):
        x = rng.standard_normal((n, cols)).astype(np.float32)
        if n == 5:
            x[1] = 0.0
            x[2, :256] = -np.abs(x[2, :256]).max() * 4   # a super-block at the negative extreme
        s, q = oracle.quantize_activation(fmt, x)
        with G.env(CAMELID_HIP_Q6K_MFMA_MIN_TOKENS=1 << 30), G.engaged(r"^q6k\.dot\.", none=(r"^q6k\.mfma\.",)):
            ref = G.gpu_gemm(w, s, q)                      # the packed-dot kernel on the same inputs
        for shape in (0, 1, 2, 3, 4, 6):
            for deep in (0, 1):
                G.say(f"Q6_K matrix-core {rows}x{cols} n={n} shape={shape} deep={deep}")
                want_kernel = r"^q6k\.mfma\." if shape == 0 else r"^q6k\.mfma\.(tile|serial_split)\." + MFMA_SHAPES[shape] + r"\." + ("r4" if deep else "r2")
                with G.env(CAMELID_HIP_Q6K_MFMA_SHAPE=shape, CAMELID_HIP_Q6K_MFMA_DEEP=deep, CAMELID_HIP_Q6K_MFMA_MIN_TOKENS=1), \
                        G.engaged(want_kernel, none=(r"^q6k\.dot\.",)):
                    got = G.gpu_gemm(w, s, q)
                assert G.same_bits(got, ref)
        with G.env(CAMELID_HIP_Q6K_MFMA_SERIAL_SPLIT=1, CAMELID_HIP_Q6K_MFMA_MIN_TOKENS=1), \
                G.engaged(r"^q6k\.mfma\.", none=(r"^q6k\.mfma\.ksplit", r"^q6k\.dot\.")):   # the split inside the lane
            assert G.same_bits(G.gpu_gemm(w, s, q), ref)
        check_outputs(fmt, wire, cols, s, q, got, expect_exact=False)
        with G.env(CAMELID_HIP_EXACT_ORDER="1", CAMELID_HIP_Q6K_MFMA_MIN_TOKENS=1):
            got = G.gpu_gemm(w, s, q)
        check_outputs(fmt, wire, cols, s, q, got, expect_exact=True)


@pytest.mark.parametrize("name,fmt", FMTS)
def test_long_rows_in_small_batches_fit_the_staging_limit(name, fmt):
    """14336-value rows (an FFN down projection) with 2..8 tokens: the packed-dot kernels stage
    fewer tokens per pass instead of refusing the call."""
    rows, cols = 40, 14336
    wire = G.synth_weight(fmt, rows, cols, seed=900 + fmt)
    w = Weight.upload(fmt, rows, cols, wire)
    rng = np.random.default_rng(901)
    for n in (2, 4, 8):
        x = rng.standard_normal((n, cols)).astype(np.float32)
        s, q = oracle.quantize_activation(fmt, x)
        G.say(f"{name} {rows}x{cols} n={n} packed-dot")
        with G.env(CAMELID_HIP_Q4K_MFMA_MIN_TOKENS=1 << 30, CAMELID_HIP_B32_MFMA_MIN_TOKENS=1 << 30,
                   CAMELID_HIP_Q6K_MFMA_MIN_TOKENS=1 << 30, CAMELID_HIP_EXACT_ORDER="1"):
            got = G.gpu_gemm(w, s, q)
        check_outputs(fmt, wire, cols, s, q, got, expect_exact=True)


@pytest.mark.parametrize("name,fmt", FMTS)
def test_rows_too_long_for_the_matrix_core_staging_fall_back_to_the_packed_dot(name, fmt):
    """16384-value rows with 64 tokens: where the matrix-core kernel's LDS staging does not hold the
    batch, the call is served by the packed-dot kernel in passes of fewer tokens, not refused."""
    rows, cols, n = 24, 16384, 64
    wire = G.synth_weight(fmt, rows, cols, seed=950 + fmt)
    w = Weight.upload(fmt, rows, cols, wire)
    x = np.random.default_rng(951).standard_normal((n, cols)).astype(np.float32)
    s, q = oracle.quantize_activation(fmt, x)
    G.say(f"{name} {rows}x{cols} n={n} default dispatch")
    with G.env(CAMELID_HIP_EXACT_ORDER="1"):
        got = G.gpu_gemm(w, s, q)
    check_outputs(fmt, wire, cols, s, q, got, expect_exact=True)


@pytest.mark.parametrize("rows,cols", [(130, 1024), (33, 256), (61, 9 * 256), (300, 14336), (5, 16 * 256)])
def test_q6k_lane_order_is_the_reference_cpu_chain_bit_for_bit(rows, cols):
    """CAMELID_HIP_Q6K_LANE_ORDER=1: every plain Q6_K call (one token, a batch, a row band, with a
    residual, f32 or quantized activations in) returns the bits of q6_k_wire_row_dot's 8-lane order
    (reference src/inference.rs:25535-25581), the order both of the reference's CPU lanes run."""
    fmt = B.CML_Q6_K
    rng = np.random.default_rng(rows + cols)
    wire = G.synth_weight(fmt, rows, cols, seed=rows * 3 + cols)
    w = Weight.upload(fmt, rows, cols, wire)
    x = rng.standard_normal((5, cols)).astype(np.float32)
    x[1, :256] = 0.0
    s, q = oracle.quantize_activation(fmt, x)
    want = oracle.matmul_q(fmt, wire, cols, s, q, order=oracle.ORDER_PRIMARY, threads=8)
    res = rng.standard_normal(rows).astype(np.float32)
    G.say(f"Q6_K lane order {rows}x{cols}")
    with G.env(CAMELID_HIP_Q6K_LANE_ORDER="1"):
        assert G.same_bits(G.gpu_gemm(w, s[0], q[0]), want[0])
        assert G.same_bits(G.gpu_gemm(w, s[0], q[0], residual=res), want[0] + res)
        assert G.same_bits(G.gpu_gemm(w, s, q), want)
        assert G.same_bits(G.gpu_matmul_f32(w, x[2]), want[2])
        assert G.same_bits(G.gpu_matmul_f32(w, x), want)
        if rows > 20:
            band = w.slice(3, rows - 7)
            assert G.same_bits(G.gpu_gemm(band, s, q), want[:, 3:rows - 4])
    # without the switch: the fused chain, within tolerance of it
    assert G.max_rel(G.gpu_gemm(w, s, q), want) <= TOL


@pytest.mark.parametrize("rows,cols", [(130, 1024), (33, 256), (61, 9 * 256), (300, 14336), (5, 16 * 256), (2000, 4096)])
def test_q4k_lane_order_is_the_reference_wire_row_dot_bit_for_bit(rows, cols):
    """CAMELID_HIP_Q4K_LANE_ORDER=1: every plain Q4_K call (one token, a batch, a row band that
    starts inside a tile, with a residual, f32 or quantized activations in) returns the bits of
    q4_k_wire_row_dot's generic 8-lane order (reference src/inference.rs:25806-25889), the order of
    the Gemma-4 wire lane; the default kernels keep the fused order of q4_k_dot_arm."""
    fmt = B.CML_Q4_K
    rng = np.random.default_rng(rows + cols)
    wire = G.synth_weight(fmt, rows, cols, seed=rows * 3 + cols)
    w = Weight.upload(fmt, rows, cols, wire)
    x = rng.standard_normal((5, cols)).astype(np.float32)
    x[1, :256] = 0.0
    s, q = oracle.quantize_activation(fmt, x)
    want = oracle.matmul_q(fmt, wire, cols, s, q, order=oracle.ORDER_ALT, threads=8)
    fused = oracle.matmul_q(fmt, wire, cols, s, q, order=oracle.ORDER_PRIMARY, threads=8)
    res = rng.standard_normal(rows).astype(np.float32)
    G.say(f"Q4_K lane order {rows}x{cols}")
    with G.env(CAMELID_HIP_Q4K_LANE_ORDER="1"):
        assert G.same_bits(G.gpu_gemm(w, s[0], q[0]), want[0])
        assert G.same_bits(G.gpu_gemm(w, s[0], q[0], residual=res), want[0] + res)
        assert G.same_bits(G.gpu_gemm(w, s, q), want)
        assert G.same_bits(G.gpu_matmul_f32(w, x[2]), want[2])
        assert G.same_bits(G.gpu_matmul_f32(w, x), want)
        if rows > 20:
            band = w.slice(3, rows - 7)
            assert G.same_bits(G.gpu_gemm(band, s, q), want[:, 3:rows - 4])
    # without the switch: the fused chain (exactly, with the K cut forbidden), within tolerance of the 8-lane order
    with G.env(CAMELID_HIP_EXACT_ORDER="1"):
        got = G.gpu_gemm(w, s, q)
    assert G.same_bits(got, fused)
    assert G.max_rel(got, want) <= TOL
    if cols >= 1024:
        assert not G.same_bits(fused, want)    # the two orders do differ on this input


@pytest.mark.parametrize("rows,cols", [(512, 4096), (47, 4096), (3000, 4096), (9000, 4096), (14336, 4096), (4096, 14336),
                                       (300, 14336), (100, 8192), (1000, 2048), (70, 7 * 256), (33, 1024)])
def test_q4k_single_token_entry_points_give_the_same_bits(rows, cols):
    """A single-token Q4_K call through both entry points (quantized activation in, f32 activation
    in), with a residual, and on a row band that starts inside a 16-row tile: the oracle's fused
    order bit for bit with the K cut forbidden, and one set of bits under the default policy, which
    cuts K for weights of few row tiles."""
    fmt = B.CML_Q4_K
    rng = np.random.default_rng(rows * 5 + cols)
    wire = G.synth_weight(fmt, rows, cols, seed=rows + 3 * cols)
    w = Weight.upload(fmt, rows, cols, wire)
    x = rng.standard_normal(cols).astype(np.float32)
    x[:256] = 0.0
    s, q = oracle.quantize_activation(fmt, x)
    want = oracle.matmul(fmt, wire, cols, x, order=oracle.ORDER_PRIMARY, threads=8)
    res = rng.standard_normal(rows).astype(np.float32)
    band = w.slice(5, rows - 9) if rows > 20 else None
    G.say(f"Q4_K single token on {rows}x{cols}")
    default_bits = G.gpu_gemm(w, s, q)
    assert G.max_rel(default_bits, want) <= TOL
    assert G.same_bits(G.gpu_matmul_f32(w, x), default_bits)
    with G.env(CAMELID_HIP_EXACT_ORDER="1"):
        assert G.same_bits(G.gpu_gemm(w, s, q), want)
        assert G.same_bits(G.gpu_gemm(w, s, q, residual=res), want + res)
        assert G.same_bits(G.gpu_matmul_f32(w, x), want)
        if band is not None:
            assert G.same_bits(G.gpu_gemm(band, s, q), want[5:rows - 4])
            assert G.same_bits(G.gpu_matmul_f32(band, x), want[5:rows - 4])


@pytest.mark.parametrize("name,fmt,rows,cols", [("Q4_K", B.CML_Q4_K, 14336, 4096), ("Q4_K", B.CML_Q4_K, 200, 4096), ("Q4_K", B.CML_Q4_K, 1000, 3584),
                                                ("Q4_K", B.CML_Q4_K, 530, 2304), ("Q4_K", B.CML_Q4_K, 4096, 14336), ("Q4_K", B.CML_Q4_K, 17000, 1024),
                                                ("Q6_K", B.CML_Q6_K, 300, 1024), ("Q8_0", B.CML_Q8_0, 700, 2048), ("Q4_0", B.CML_Q4_0, 64, 96),
                                                ("Q8_0", B.CML_Q8_0, 8192, 2048), ("Q8_0", B.CML_Q8_0, 4099, 4096), ("Q4_0", B.CML_Q4_0, 4100, 4096),
                                                ("Q4_0", B.CML_Q4_0, 5000, 1056), ("Q8_0", B.CML_Q8_0, 4500, 96),
                                                # shapes the b32 pair launch does not take: served by the multi launch of two weights
                                                ("Q8_0", B.CML_Q8_0, 4096, 4096), ("Q4_0", B.CML_Q4_0, 6000, 5120), ("Q4_0", B.CML_Q4_0, 3000, 8192),
                                                ("Q6_K", B.CML_Q6_K, 14336, 4096), ("Q6_K", B.CML_Q6_K, 4100, 4096)])
def test_matmul_f32_pair_is_two_single_calls(name, fmt, rows, cols):
    """cml_matmul_f32_pair (one token, two weights that read it: gate and up of a dense FFN): the bits
    of two cml_matmul_f32 calls -- where it runs as one launch (Q4_K, with and without the ring of
    register buffers, 8- and 16-row waves; Q8_0 / Q4_0 on at least 4096 rows of 16 lanes), where it
    does not (Q6_K, few rows, long rows), and with
    the one-launch path switched off; weights of different shapes are two calls."""
    rng = np.random.default_rng(rows + cols)
    wa = Weight.upload(fmt, rows, cols, G.synth_weight(fmt, rows, cols, seed=rows + 1))
    wb = Weight.upload(fmt, rows, cols, G.synth_weight(fmt, rows, cols, seed=rows + 2))
    x = rng.standard_normal(cols).astype(np.float32)

    def pair(w1, w2):
        ws_bytes = lib().cml_matmul_workspace_bytes(fmt, cols, 1)
        xd = DeviceBuffer.from_numpy(x.reshape(1, -1))
        ws = DeviceBuffer(max(ws_bytes, 16))
        o1, o2 = DeviceBuffer(w1.rows * 4), DeviceBuffer(w2.rows * 4)
        o1.fill(0xFF)
        o2.fill(0xFF)
        check(lib().cml_matmul_f32_pair(w1.handle, w2.handle, xd.ptr, o1.ptr, o2.ptr, ws.ptr, ws_bytes, None), "cml_matmul_f32_pair")
        check(lib().cml_stream_sync(None))
        return o1.to_numpy(np.float32, (w1.rows,)), o2.to_numpy(np.float32, (w2.rows,))

    G.say(f"pair {name} {rows}x{cols}")
    want_a, want_b = G.gpu_matmul_f32(wa, x), G.gpu_matmul_f32(wb, x)
    if (name, rows, cols) in (("Q8_0", 4096, 4096), ("Q4_0", 6000, 5120), ("Q4_0", 3000, 8192)):
        with G.engaged(r"^q[48]_0\.dot\.p\d+\.w8\.fused\.multi$", none=(r"^quantize\.", r"pair")):
            got_a, got_b = pair(wa, wb)
        assert G.same_bits(got_a, want_a) and G.same_bits(got_b, want_b), (name, rows, cols, "multi launch of two")
    if name == "Q6_K" and rows >= 4096:
        with G.engaged(r"^q6k\.dot\.wg8\.kcut\.fused\.multi$", none=(r"^quantize\.",)):
            got_a, got_b = pair(wa, wb)
        assert G.same_bits(got_a, want_a) and G.same_bits(got_b, want_b), (name, rows, cols, "multi launch of two")
    for knobs in ({}, {"CAMELID_HIP_Q4K_RING": "0", "CAMELID_HIP_B32_RING": "0"}, {"CAMELID_HIP_PAIR_LAUNCH": "0"}, {"CAMELID_HIP_Q4K_ROWS_PER_WAVE": "16"},
                  {"CAMELID_HIP_Q4K_ROWS_PER_WAVE": "8"}, {"CAMELID_HIP_B32_MULTI": "0"}, {"CAMELID_HIP_Q6K_MULTI": "0"}):
        with G.env(**knobs):
            got_a, got_b = pair(wa, wb)
        assert G.same_bits(got_a, want_a), (name, rows, cols, knobs)
        assert G.same_bits(got_b, want_b), (name, rows, cols, knobs)
    if rows > 40:   # a second weight of another shape: two calls
        band = wb.slice(16, rows - 32)
        got_a, got_c = pair(wa, band)
        assert G.same_bits(got_a, want_a) and G.same_bits(got_c, want_b[16:rows - 16])
    L = lib()
    d = DeviceBuffer(64)
    assert L.cml_matmul_f32_pair(wa.handle, None, d.ptr, d.ptr, d.ptr, d.ptr, 64, None) == 2
    assert L.cml_matmul_f32_pair(wa.handle, wb.handle, None, d.ptr, d.ptr, d.ptr, 64, None) == 2


# ------------------------------------------------- the top of the integer range ----

def _saturated_weight(fmt, rows, cols, rng):
    """Wire rows whose every block sits at the top (or bottom) of what the format can encode, with
    small random f16 scales so that the f32 results stay finite."""
    nb = cols // oracle.block_values(fmt)
    bb = oracle.block_bytes(fmt)
    blk = np.empty((rows, nb, bb), np.uint8)

    def f16_bytes(lo, hi, shape):
        return rng.uniform(lo, hi, shape).astype(np.float16).view(np.uint8).reshape(*shape, 2)

    if fmt == B.CML_Q4_K:
        blk[:, :, 16:] = rng.integers(0xcc, 0x100, (rows, nb, 128), dtype=np.uint8)   # nibbles 12..15
        blk[:, :, 4:16] = 0xff                                                        # 6-bit scales and mins all 63
        blk[:, :, 0:2] = f16_bytes(0.001, 0.004, (rows, nb))
        blk[:, :, 2:4] = f16_bytes(0.01, 0.04, (rows, nb))
    elif fmt == B.CML_Q6_K:
        top = rng.integers(0, 2, (rows, nb, 1), dtype=np.uint8)                       # a super-block of all 63 or all 0 codes (+31 / -32)
        blk[:, :, 0:192] = np.where(top == 1, 0xff, 0x00)
        blk[:, :, 192:208] = rng.choice(np.array([127, -128, -127], np.int8), (rows, nb, 16)).view(np.uint8)
        blk[:, :, 208:210] = f16_bytes(0.0005, 0.002, (rows, nb))
    elif fmt == B.CML_Q8_0:
        blk[:, :, 0:2] = f16_bytes(0.01, 0.05, (rows, nb))
        blk[:, :, 2:] = rng.choice(np.array([127, -128], np.int8), (rows, nb, 32)).view(np.uint8)
    else:
        blk[:, :, 0:2] = f16_bytes(0.01, 0.05, (rows, nb))
        blk[:, :, 2:] = rng.choice(np.array([0x00, 0xff, 0xf0, 0x0f], np.uint8), (rows, nb, 16))   # nibbles 0 or 15: -8 or +7
    return np.ascontiguousarray(blk.reshape(-1))


@pytest.mark.parametrize("name,fmt", FMTS)
def test_saturated_blocks_and_activations_keep_every_bit(name, fmt):
    """Weights and activations at the top of the integer range -- 6-bit scales all 63 with nibbles 12..15,
    Q6_K codes all 63 or all 0 under int8 scales of +127 / -128, int8 weights of +127 / -128, activations of
    +127, of -128 (which no quantizer produces but a caller of cml_gemv may pass), of the weight's sign and
    of 125..127 -- through cml_block_dots, cml_gemv and cml_gemm at 2, 3, 16 and 64 tokens, in both
    accumulation orders of the K-quants: the oracle's bits.  The super-block integers pass 2^24 here, so
    their conversion to f32 rounds; 24-bit multiplies, digit-split scales and half-precision run sums inside
    the kernels would show up as wrong bits exactly on such inputs."""
    rng = np.random.default_rng(900 + fmt)
    bv = oracle.block_values(fmt)
    is_k = G.is_k(fmt)
    lane_knob = {B.CML_Q4_K: "CAMELID_HIP_Q4K_LANE_ORDER", B.CML_Q6_K: "CAMELID_HIP_Q6K_LANE_ORDER"}.get(fmt)
    # the order the fast kernels keep, and the one the lane-order kernels keep
    fast_order = EXACT_ORDER[fmt]
    lane_order = (oracle.ORDER_ALT if fast_order == oracle.ORDER_PRIMARY else oracle.ORDER_PRIMARY) if is_k else None
    for rows, nbr in ((37, 3), (300, 16), (130, 8 if not is_k else 5)):
        cols = nbr * (256 if is_k else 256)   # Q8_0 / Q4_0: whole 256-value slabs, so that the matrix-core kernels serve them
        wire = _saturated_weight(fmt, rows, cols, rng)
        w = Weight.upload(fmt, rows, cols, wire)
        n_max = 64
        q = np.empty((n_max, cols), np.int8)
        q[0] = 127
        q[1] = -128
        q[2] = rng.integers(125, 128, cols)
        q[3] = np.where(rng.integers(0, 2, cols) == 1, 127, -128)
        q[4:] = rng.choice(np.array([127, -128, -127, 126], np.int8), (n_max - 4, cols))
        s = rng.uniform(0.01, 0.05, (n_max, cols // (256 if is_k else 32))).astype(np.float32)
        G.say(f"{name} saturated {rows}x{cols}: block integers")
        for t in (0, 1, 3):
            assert np.array_equal(G.gpu_block_dots(w, q[t]), oracle.block_ints(fmt, wire, cols, q[t])), (name, rows, cols, t)
        for n in (1, 2, 3, 16, 64):
            want = oracle.matmul_q(fmt, wire, cols, s[:n], q[:n], order=fast_order, threads=8)
            G.say(f"{name} saturated {rows}x{cols} n={n}")
            with G.env(CAMELID_HIP_EXACT_ORDER="1"):
                got = G.gpu_gemm(w, s[0], q[0]) if n == 1 else G.gpu_gemm(w, s[:n], q[:n])
                assert G.same_bits(got.reshape(n, rows), want), (name, rows, cols, n, "fast kernels")
                if n >= 3:   # the packed-dot kernel on the same batch
                    knob = {B.CML_Q4_K: "CAMELID_HIP_Q4K_MFMA_MIN_TOKENS", B.CML_Q6_K: "CAMELID_HIP_Q6K_MFMA_MIN_TOKENS"}.get(fmt, "CAMELID_HIP_B32_MFMA_MIN_TOKENS")
                    with G.env(CAMELID_HIP_EXACT_ORDER="1", **{knob: 1 << 30}), G.engaged(r"\.dot\.", none=(r"\.mfma\.",)):
                        assert G.same_bits(G.gpu_gemm(w, s[:n], q[:n]), want), (name, rows, cols, n, "packed dot")
                    with G.env(CAMELID_HIP_EXACT_ORDER="1", **{knob: 1}), G.engaged(r"\.mfma\.", none=(r"\.dot\.",)):
                        assert G.same_bits(G.gpu_gemm(w, s[:n], q[:n]), want), (name, rows, cols, n, "matrix cores")
            if lane_knob and n <= 3:
                want_lane = oracle.matmul_q(fmt, wire, cols, s[:n], q[:n], order=lane_order, threads=8)
                with G.env(**{lane_knob: 1}), G.engaged(r"\.lanes$"):
                    got = G.gpu_gemm(w, s[0], q[0]) if n == 1 else G.gpu_gemm(w, s[:n], q[:n])
                assert G.same_bits(got.reshape(n, rows), want_lane), (name, rows, cols, n, "lane order")


# ------------------------------------------------- several projections of one token, one launch ----

def _multi(ws, x, stream=None):
    """cml_matmul_f32_multi through the C ABI: host arrays of weight handles and output pointers."""
    n = len(ws)
    cols = ws[0].cols
    ws_bytes = lib().cml_matmul_workspace_bytes(ws[0].fmt, cols, 1)
    xd = DeviceBuffer.from_numpy(np.ascontiguousarray(x, np.float32).reshape(1, -1))
    wsp = DeviceBuffer(max(ws_bytes, 16))
    outs = [DeviceBuffer(max(w.rows * 4, 16)) for w in ws]
    for o in outs:
        o.fill(0xFF)
    handles = (C.c_void_p * n)(*[w.handle for w in ws])
    optrs = (C.c_void_p * n)(*[o.ptr for o in outs])
    check(lib().cml_matmul_f32_multi(handles, n, xd.ptr, optrs, wsp.ptr, ws_bytes, stream), "cml_matmul_f32_multi")
    check(lib().cml_stream_sync(stream))
    return [o.to_numpy(np.float32, (w.rows,)) for o, w in zip(outs, ws)]


@pytest.mark.parametrize("case", ["qkv_4096", "gate_up_14336", "ragged_2304", "three_3584", "mixed_cut", "five", "q6k", "bands",
                                  "cut4_8192", "cut2_4096", "q8_0_qkv_4096", "q4_0_qkv_3584", "q8_0_ragged_2048", "q4_0_pair_8192",
                                  "q4_0_gate_up_14336", "q8_0_tiny", "q6k_qkv_4096", "q6k_gate_up_14336", "q6k_mixed_cut", "q6k_qkv_3584"])
def test_matmul_f32_multi_is_the_single_calls(case):
    """cml_matmul_f32_multi: several weights that read one token (q | k | v of an attention block, gate | up of an FFN).
    Runs of up to four Q4_K weights with one K cut go out as one launch -- the counters prove it -- and every
    output is the bits of a cml_matmul_f32 call of its own; sets the one launch does not serve (different K cuts,
    another format) fall back to single calls with the same results."""
    fmt = B.CML_Q4_K
    shapes, cols, one_launch = {
        "qkv_4096": ([4096, 1024, 1024], 4096, 1),          # K cut 4 for all three: the eight-wave K-cut form
        "cut4_8192": ([4000, 3100, 5000], 8192, 1),         # K cut 4, parts of four steps
        "cut2_4096": ([8192, 6144, 7001], 4096, 1),         # K cut 2, parts of four steps
        "gate_up_14336": ([14336, 14336], 4096, 1),         # no K cut: the ring kernel
        "ragged_2304": ([200, 77, 530, 16], 2304, 1),       # ragged row counts, 9 super-blocks
        "three_3584": ([1000, 333, 4100], 3584, 1),
        "mixed_cut": ([14336, 4096], 4096, 0),              # K cuts 1 and 4: two calls
        "five": ([512, 256, 256, 128, 640], 2048, 2),       # four in one launch, the fifth alone
        "q6k": ([300, 200], 1024, 0),
        "bands": ([700, 300, 650], 4096, 1),
        "q8_0_qkv_4096": ([4096, 1024, 1024], 4096, 1),     # the 32-value block formats: one launch too
        "q4_0_qkv_3584": ([3584, 512, 512], 3584, 1),
        "q8_0_ragged_2048": ([200, 77, 530, 16], 2048, 1),
        "q4_0_pair_8192": ([4096, 1030], 8192, 1),
        "q4_0_gate_up_14336": ([14336, 14336], 4096, 1),
        "q8_0_tiny": ([40, 24], 64, 1),
        "q6k_qkv_4096": ([4096, 1030, 1024], 4096, 1),      # Q6_K sets with one K cut: one launch of the one-workgroup-per-unit form
        "q6k_gate_up_14336": ([14336, 14336], 4096, 1),
        "q6k_qkv_3584": ([3584, 512, 512], 3584, 1),
        "q6k_mixed_cut": ([8192, 1024], 4096, 0),           # K cuts 2 and 4: two calls
    }[case]
    if case.startswith("q6k"):
        fmt = B.CML_Q6_K
    elif case.startswith("q8_0"):
        fmt = B.CML_Q8_0
    elif case.startswith("q4_0"):
        fmt = B.CML_Q4_0
    rng = np.random.default_rng(sum(shapes) + cols)
    ws = [Weight.upload(fmt, r, cols, G.synth_weight(fmt, r, cols, seed=r + cols + j)) for j, r in enumerate(shapes)]
    if case == "bands":   # views that start inside a 16-row tile
        ws = [ws[0].slice(5, 600), ws[1].slice(0, 300), ws[2].slice(17, 601)]
    x = rng.standard_normal(cols).astype(np.float32)
    x[:256] = 0.0
    G.say(f"multi {case}: single calls")
    want = [G.gpu_matmul_f32(w, x) for w in ws]
    G.say(f"multi {case}: one call")
    if fmt == B.CML_Q6_K and one_launch:
        proof = G.engaged(r"^q6k\.dot\.wg8\.kcut\.fused\.multi$", none=(r"^quantize\.",))
    elif fmt == B.CML_Q6_K:
        proof = G.engaged(r"^q6k\.dot\.", none=(r"multi",))
    elif fmt in (B.CML_Q8_0, B.CML_Q4_0):
        proof = G.engaged(r"^q[48]_0\.dot\.p\d+\.w8\.fused\.multi$", none=(r"^quantize\.",))
    elif one_launch == 0:
        proof = G.engaged(r"^q4k\.dot\.", none=(r"multi",))
    elif case in ("qkv_4096", "cut4_8192", "cut2_4096"):   # ("bands" is too small for eight-wave workgroups to fill the chip)
        proof = G.engaged(r"^q4k\.dot\.wg8\.kcut\.fused\.multi$", none=(r"^q4k\.dot\.(ring|buffers)",))
    else:
        proof = G.engaged(r"^q4k\.dot\.(ring|buffers)\.fused\.multi$")
    before = G.launch_counts()
    with proof:
        got = _multi(ws, x)
    after = G.launch_counts()
    launches = sum(after.values()) - sum(before.values())
    assert launches == {"five": 2}.get(case, 1 if one_launch else launches), (case, launches)
    for j, (g, wnt) in enumerate(zip(got, want)):
        assert G.same_bits(g, wnt), (case, j)
    with G.env(CAMELID_HIP_MULTI_LAUNCH=0), G.engaged(none=(r"multi",)):
        got = _multi(ws, x)
    for j, (g, wnt) in enumerate(zip(got, want)):
        assert G.same_bits(g, wnt), (case, j, "single calls inside")
    if fmt == B.CML_Q4_K and one_launch:
        with G.env(CAMELID_HIP_Q4K_KCUT_MULTI=0), G.engaged(r"^q4k\.dot\.(ring|buffers)\.fused\.multi$", none=(r"^q4k\.dot\.wg8",)):
            got = _multi(ws, x)
        for j, (g, wnt) in enumerate(zip(got, want)):
            assert G.same_bits(g, wnt), (case, j, "four-wave multi launch")
    if fmt == B.CML_Q4_K:
        with G.env(CAMELID_HIP_EXACT_ORDER="1"):
            got = _multi(ws, x)
            for j, (g, w) in enumerate(zip(got, ws)):
                assert G.same_bits(g, G.gpu_matmul_f32(w, x)), (case, j, "exact order")
