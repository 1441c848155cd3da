"""The oracle against the golden vectors the reference's own tests hold.

tests/golden/dequant/*.json are the data files of the reference's
tests/fixtures/dequant (wire bytes + u32 bit patterns of gguf 0.19.0's
dequantizer), which the reference checks with zero tolerance
(tests/runnable_dequant.rs:121-158).
"""
import json
import os

import numpy as np
import pytest

import oracle
from tests import npref

GOLD = os.path.join(os.path.dirname(__file__), "golden", "dequant")


def load(name):
    with open(os.path.join(GOLD, f"{name}.json")) as f:
        fx = json.load(f)
    wire = np.frombuffer(bytes.fromhex(fx["quant_hex"]), dtype=np.uint8)
    ref = np.array([int(v, 16) if isinstance(v, str) else int(v) for v in fx["ref_f32_bits"]], dtype=np.uint32)
    return fx, wire, ref


@pytest.mark.parametrize("name", ["Q8_0", "Q4_0", "Q4_K", "Q6_K"])
def test_dequant_bit_exact_against_gguf_fixture(name):
    fx, wire, ref = load(name)
    assert wire.size == fx["n_blocks"] * fx["block_bytes"]
    out = oracle.dequant(oracle.FORMATS[name], wire)
    assert out.size == fx["n_elements"]
    assert np.array_equal(out.view(np.uint32), ref)


def test_f16_fixture_bit_exact():
    fx, wire, ref = load("F16")
    h = wire.view("<u2")
    out = oracle.f16_bits_to_f32_array(h)
    assert np.array_equal(out.view(np.uint32), ref)


@pytest.mark.parametrize("name", ["Q8_0", "Q4_0", "Q4_K", "Q6_K"])
def test_numpy_decoders_agree_with_fixture(name):
    """Pins tests/npref.py (used for the brute-force integer checks)."""
    fx, wire, ref = load(name)
    got = npref.dequant_f64(name, wire)
    want = ref.view(np.float32).astype(np.float64)
    # float64 evaluation of the same integers: equal up to one f32 rounding per product
    assert np.allclose(got, want, rtol=3e-7, atol=1e-30)
