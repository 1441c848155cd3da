"""GPU parity at BASELINE.json's full shapes (configs 1-4), against the
multithreaded oracle on the same seeded inputs, plus size-independent
properties (linearity in the activation scale, batched == single)."""
import numpy as np
import pytest

import oracle
from camelid_amd import binding as B
from camelid_amd.binding import Weight, lib
from tests import gpu_util as G
from tests.test_gpu_parity import EXACT_ORDER, TOL

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module", autouse=True)
def _init():
    assert lib().cml_available() == 1
    B.init(0)
    yield


def _case(fmt, rows, cols, seed, exact):
    G.say(f"baseline shape fmt={fmt} {rows}x{cols}")
    wire = G.synth_weight(fmt, rows, cols, seed=seed)
    x = np.random.default_rng(seed + 1).standard_normal(cols).astype(np.float32)
    w = Weight.upload(fmt, rows, cols, wire)
    got = G.gpu_matmul_f32(w, x)
    s, q = oracle.quantize_activation(fmt, x)
    for order in ((oracle.ORDER_PRIMARY, oracle.ORDER_ALT) if G.is_k(fmt) else (oracle.ORDER_PRIMARY,)):
        want = oracle.matmul_q(fmt, wire, cols, s, q, order=order, threads=16)
        assert G.max_rel(got, want) <= TOL
        if exact and order == EXACT_ORDER[fmt]:
            assert G.same_bits(got, want)
    # linearity: doubling the activation scales doubles every output exactly (power of two)
    got2 = G.gpu_gemm(w, s * np.float32(2.0), q)
    assert G.same_bits(got2, got * np.float32(2.0))
    return w, wire, x


def test_c1_q8_0_8192x2048():
    _case(B.CML_Q8_0, 8192, 2048, seed=1001, exact=True)


def test_c2_q4_k_gate_up_14336x4096():
    w, wire, x = _case(B.CML_Q4_K, 14336, 4096, seed=1002, exact=True)
    # the generic 8-lane order of the reference's wire row dot (q4_k_wire_row_dot): bit for bit under its own switch
    G.say("Q4_K 14336x4096 in the 8-lane order")
    with G.env(CAMELID_HIP_Q4K_LANE_ORDER="1"):
        got = G.gpu_matmul_f32(w, x)
    want = oracle.matmul(B.CML_Q4_K, wire, 4096, x, order=oracle.ORDER_ALT, threads=16)
    assert G.same_bits(got, want)


def test_c2_q4_k_down_4096x14336():
    _case(B.CML_Q4_K, 4096, 14336, seed=1003, exact=False)  # K-split: tolerance only
    with G.env(CAMELID_HIP_EXACT_ORDER="1"):
        _case(B.CML_Q4_K, 4096, 14336, seed=1003, exact=True)


def test_c3_q6_k_lm_head_128256x3072():
    w, wire, x = _case(B.CML_Q6_K, 128256, 3072, seed=1004, exact=True)
    # the order the reference's CPU lanes run (8 lanes by index mod 8, q6_k_wire_row_dot): bit for bit
    # under its own switch
    G.say("Q6_K 128256x3072 in the 8-lane order")
    with G.env(CAMELID_HIP_Q6K_LANE_ORDER="1"):
        got = G.gpu_matmul_f32(w, x)
    want = oracle.matmul(B.CML_Q6_K, wire, 3072, x, order=oracle.ORDER_PRIMARY, threads=16)
    assert G.same_bits(got, want)


def test_c3_q4_0_lm_head_128256x3072():
    _case(B.CML_Q4_0, 128256, 3072, seed=1005, exact=True)


@pytest.mark.parametrize("n", [4, 8, 16, 64])
def test_c4_q4_k_batched_14336x4096(n):
    fmt, rows, cols = B.CML_Q4_K, 14336, 4096
    G.say(f"batched Q4_K n={n}")
    wire = G.synth_weight(fmt, rows, cols, seed=1002)
    w = Weight.upload(fmt, rows, cols, wire)
    x = np.random.default_rng(2000 + n).standard_normal((n, cols)).astype(np.float32)
    got = G.gpu_matmul_f32(w, x)   # 14336 rows: no K-split, the reference association
    want = oracle.matmul(fmt, wire, cols, x, order=oracle.ORDER_PRIMARY, threads=16)
    assert G.same_bits(got, want)
    alt = oracle.matmul(fmt, wire, cols, x, order=oracle.ORDER_ALT, threads=16)
    assert G.max_rel(got, alt) <= TOL
    one = G.gpu_matmul_f32(w, x[n // 2])
    assert G.same_bits(one, got[n // 2])
