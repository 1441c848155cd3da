"""Builds libcamelid_hip.so (gfx950) in-tree with hipcc.

hipcc cross-compiles without a GPU, so this runs in the build container; the
shared library then travels with the tree to the GPU box.
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(CSRC, "build")
LIB = os.path.join(HERE, "libcamelid_hip.so")

SOURCES = [
    "cml_api.hip",
    "quantize.hip",
    "layout.hip",
    "gemv_q4k.hip",
    "gemm_q4k_mfma.hip",
    "gemv_q8q4.hip",
    "gemv_q6k.hip",
    "moe.hip",
    "weight_quantize.cpp",
]

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")

# -ffp-contract=off: the reference arithmetic rounds every multiply and add on
# its own; the fused steps call fmaf explicitly.
# packed-fp32-ops is switched off for every device compile in this tree.
FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-ffp-contract=off",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # MFMA results straight into VGPRs: the integer epilogue reads every one of them
    "-mllvm", "-amdgpu-mfma-vgpr-form=1",
    "-Wall",
    "-Wno-unused-function",
    "-Wno-unknown-warning-option",
]


def _compile(src: str, extra: list[str]) -> str:
    obj = os.path.join(OBJ, os.path.splitext(src)[0] + ".o")
    cmd = [HIPCC, *FLAGS, *extra, "-c", os.path.join(CSRC, src), "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src}:\n{r.stdout}\n{r.stderr}")
    warnings = "\n".join(l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l and l.strip())
    if warnings and os.environ.get("CAMELID_BUILD_VERBOSE"):
        print(warnings, file=sys.stderr)
    return obj


def build(extra_flags: list[str] | None = None, jobs: int = 8) -> str:
    """Compile every HIP source and link libcamelid_hip.so.  Always recompiles."""
    os.makedirs(OBJ, exist_ok=True)
    extra = list(extra_flags or [])
    with ThreadPoolExecutor(max_workers=jobs) as pool:
        objs = list(pool.map(lambda s: _compile(s, extra), SOURCES))
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", *objs, "-o", LIB]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"link failed:\n{r.stdout}\n{r.stderr}")
    return LIB


if __name__ == "__main__":
    print(build(sys.argv[1:]))
