"""camelid_amd -- MI355X (gfx950) backend for the quantized weight-times-activation
path of the Camelid GGUF engine: fused dequantize + matvec / small-batch matmul over
Q8_0, Q4_0, Q4_K and Q6_K with Q8_0 / Q8_K activations.

The product is ``libcamelid_hip.so`` (C ABI in ``include/camelid_hip.h``); this package
is the thin ctypes plumbing the tests and the benchmark use to reach it.
"""
from .binding import (  # noqa: F401
    CML_Q4_0,
    CML_Q4_K,
    CML_Q6_K,
    CML_Q8_0,
    CamelidHipError,
    DeviceBuffer,
    Weight,
    lib,
    lib_path,
)
