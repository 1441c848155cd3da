"""CPU-side checks of the C-ABI shared library: it loads, exports every symbol
the header declares, and fails closed (status codes, no aborts) without a GPU."""
import ctypes as C
import os
import re

import numpy as np
import pytest

from camelid_amd import binding as B

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "camelid_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(cml_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    L = B.lib()
    names = declared_symbols()
    assert len(names) >= 25
    for n in names:
        assert hasattr(L, n), f"{n} declared in include/camelid_hip.h but not exported"
    assert sorted(B.EXPORTS) == names


def test_geometry_helpers():
    L = B.lib()
    assert [(L.cml_block_values(f), L.cml_block_bytes(f)) for f in (2, 8, 12, 14)] == [
        (32, 18), (32, 34), (256, 144), (256, 210)]
    assert L.cml_block_values(3) == 0 and L.cml_block_bytes(99) == 0
    assert L.cml_matmul_workspace_bytes(12, 4096, 1) >= 4096 + 16 * 4
    assert L.cml_matmul_workspace_bytes(99, 4096, 1) == 0


@pytest.mark.skipif(os.path.exists("/dev/kfd"), reason="checks the no-GPU behaviour")
def test_fails_closed_without_a_gpu():
    L = B.lib()
    assert L.cml_available() == 0
    assert L.cml_init(0) == 1  # CML_ERR_UNAVAILABLE
    assert L.cml_last_error()
    h = C.c_void_p()
    wire = np.zeros(144, np.uint8)
    assert L.cml_weight_upload(12, 1, 256, wire.ctypes.data, 144, C.byref(h)) == 1
    assert h.value is None
    assert L.cml_gemv(None, None, None, None, None, None) == 2  # CML_ERR_INVALID: null weight
    out = np.zeros(4, np.float32)
    q = np.zeros(32, np.int8)
    s = np.zeros(1, np.float32)
    w = np.zeros(34 * 4, np.uint8)
    assert L.cml_try_linear_rows(8, s.ctypes.data, q.ctypes.data, w.ctypes.data, w.nbytes, 1, 4, 32,
                                 out.ctypes.data) != 0
    assert L.cml_run_count() == 0


def test_env_masking_is_honoured_before_the_driver():
    import subprocess
    import sys
    code = ("import os; os.environ['HIP_VISIBLE_DEVICES']='-1';"
            "from camelid_amd import binding as B; L=B.lib();"
            "print(L.cml_available(), L.cml_init(0))")
    r = subprocess.run([sys.executable, "-c", code], cwd=ROOT, capture_output=True, text=True, timeout=120)
    assert r.stdout.split() == ["0", "1"], r.stderr


def test_host_weight_quantizer_matches_the_oracle_restatement():
    import oracle
    rng = np.random.default_rng(7)
    for fmt in (2, 8, 12, 14):
        w = (rng.standard_normal((48, 2048)) * 0.02).astype(np.float32)
        w[3, :512] = 0.0
        assert np.array_equal(B.quantize_weights(fmt, w, threads=3), oracle.quantize_weights(fmt, w, threads=1))
    assert B.lib().cml_quantize_weights_host(12, None, 100, None, 1) == 3
