"""Builds libcamelid_hip.so (gfx950) in-tree with hipcc, the C++ host layer
libcamelid_host.so above it with g++, and the host layer's test programs.

hipcc cross-compiles without a GPU, so this runs in the build container; the
shared libraries then travel with the tree to the GPU box.
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
    "producers.hip",
    "layout.hip",
    "gemv_q4k.hip",
    "gemm_q4k_mfma.hip", "gemm_b32_mfma.hip", "gemm_q6k_mfma.hip",
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


# Per-file flags (none at present).
FILE_FLAGS: dict = {}


def _compile(src: str, extra: list[str]) -> str:
    obj = os.path.join(OBJ, os.path.splitext(src)[0] + ".o")
    cmd = [HIPCC, *FLAGS, *FILE_FLAGS.get(src, []), *extra, "-c", os.path.join(CSRC, src), "-o", obj]
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


HOST_DIR = os.path.join(HERE, "host")
HOST_LIB = os.path.join(HERE, "libcamelid_host.so")
HOST_SOURCES = ["gguf_reader.cpp", "wire_quant.cpp"]
CXX = os.environ.get("CXX", "g++")
CXXFLAGS = ["-O2", "-std=c++17", "-fPIC", "-Wall", "-Wextra"]


def build_host() -> str:
    """libcamelid_host.so: GGUF reader + WireQuant over the C ABI (plain C++, no HIP headers)."""
    cmd = [CXX, *CXXFLAGS, "-shared", *[os.path.join(HOST_DIR, s) for s in HOST_SOURCES],
           "-L" + HERE, "-lcamelid_hip", "-Wl,-rpath,$ORIGIN", "-o", HOST_LIB]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"host library build failed:\n{r.stdout}\n{r.stderr}")
    return HOST_LIB


def build_host_tests() -> list[str]:
    """The host layer's test programs (tests/host/*.cpp -> tests/host/bin/), run by pytest as
    subprocesses.  They link the CPU oracle as their checker, so it must be built first."""
    root = os.path.dirname(HERE)
    tdir = os.path.join(root, "tests", "host")
    bindir = os.path.join(tdir, "bin")
    os.makedirs(bindir, exist_ok=True)
    oracle_dir = os.path.join(root, "oracle")
    out = []
    for name, libs in (("test_gguf_reader", []), ("test_wire_quant", ["-L" + oracle_dir, "-loracle"])):
        exe = os.path.join(bindir, name)
        cmd = [CXX, *CXXFLAGS, os.path.join(tdir, name + ".cpp"), "-L" + HERE, "-lcamelid_host", "-lcamelid_hip", *libs,
               "-Wl,-rpath,$ORIGIN/../../../camelid_amd", "-Wl,-rpath,$ORIGIN/../../../oracle", "-o", exe]
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError(f"{name} build failed:\n{r.stdout}\n{r.stderr}")
        out.append(exe)
    return out


if __name__ == "__main__":
    print(build(sys.argv[1:]))
    print(build_host())
