"""The C++ host layer (camelid_amd/host: GGUF reader, WireQuant, SharedActivation) is tested by
C++ programs written like the reference's own tests of those interfaces; pytest runs them.
They are built by __graft_entry__.build() (camelid_amd/build.py: build_host, build_host_tests)."""
import hashlib
import os
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
BIN = os.path.join(HERE, "host", "bin")
GGUF_FIXTURES = os.path.join(HERE, "golden", "gguf")


def _ensure_built():
    exes = [os.path.join(BIN, n) for n in ("test_gguf_reader", "test_wire_quant")]
    if not all(os.path.exists(e) for e in exes):
        import sys
        sys.path.insert(0, os.path.dirname(HERE))
        import oracle
        from camelid_amd import build as b
        if not os.path.exists(b.LIB):
            b.build()
        b.build_host()
        oracle.lib()  # builds the checker if it is missing
        b.build_host_tests()
    return exes


def _run(cmd):
    r = subprocess.run(cmd, capture_output=True, text=True, timeout=240)
    assert r.returncode == 0, f"{' '.join(cmd)} failed ({r.returncode}):\n{r.stdout[-3000:]}\n{r.stderr[-3000:]}"
    return r.stdout


def test_gguf_fixture_bytes_are_the_reference_files():
    """tests/golden/gguf holds the reference's committed GGUF files; SHA256SUMS travelled with them
    and the reference's tests pin the same digests (tests/invariant_matrix_binding.rs:503-511)."""
    sums = dict(reversed(l.split()) for l in open(os.path.join(GGUF_FIXTURES, "SHA256SUMS")).read().splitlines() if l.strip())
    assert sums["nvfp4_unknown_type_trip.gguf"] == "23a93ec4973746af71086bfe891fc0f7218c0acea892a42224e15d2c39771791"
    assert sums["nvfp4_k_div_trip.gguf"] == "f05c7fbcc3440051c3e727ba514eee963bacc99dcaa7b0a4de213fd143ff8152"
    assert sums["nvfp4_sidecar_trip.gguf"] == "4220f812bfdc4cb7825241963604bf568963fad41e0bcba6a1c6e2b7e92b7d2d"
    for name, want in sums.items():
        got = hashlib.sha256(open(os.path.join(GGUF_FIXTURES, name), "rb").read()).hexdigest()
        assert got == want, name


def test_gguf_reader_program(tmp_path):
    exe, _ = _ensure_built()
    out = _run([exe, GGUF_FIXTURES, str(tmp_path)])
    assert "checks passed" in out


@pytest.mark.gpu
def test_wire_quant_program(tmp_path):
    _, exe = _ensure_built()
    print("[case] host layer: WireQuant / SharedActivation C++ test program", flush=True)
    out = _run([exe, str(tmp_path)])
    assert "checks passed" in out
