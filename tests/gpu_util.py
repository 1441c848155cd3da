"""Helpers for the GPU parity tests: everything goes through the C ABI."""
from __future__ import annotations

import ctypes as C
import os
from contextlib import contextmanager

import numpy as np

import oracle
from camelid_amd import binding as B
from camelid_amd.binding import DeviceBuffer, Weight, check, lib


def say(msg: str) -> None:
    """Name the case before it touches the GPU (flushed, so it survives a lost box)."""
    print(f"[gpu-case] {msg}", flush=True)


@contextmanager
def env(**kv):
    """Knobs for the calls inside the block.  The library reads its environment once, so
    it is told to read it again on the way in and on the way out."""
    kv = dict(kv)
    kv.setdefault("CAMELID_HIP_TUNING", "1")  # launch-shape knobs are honoured only with this switch
    old = {k: os.environ.get(k) for k in kv}
    try:
        for k, v in kv.items():
            if v is None:
                os.environ.pop(k, None)
            else:
                os.environ[k] = str(v)
        check(lib().cml_reload_env(), "cml_reload_env")
        yield
    finally:
        for k, v in old.items():
            if v is None:
                os.environ.pop(k, None)
            else:
                os.environ[k] = v
        check(lib().cml_reload_env(), "cml_reload_env")


def launch_counts() -> dict:
    """{counter name: launches so far} from the library's kernel-family counters."""
    L = lib()
    need = L.cml_kernel_launch_report(None, 0)
    buf = C.create_string_buffer(int(need) + 256)
    L.cml_kernel_launch_report(buf, len(buf))
    out = {}
    for line in buf.value.decode().splitlines():
        name, _, n = line.rpartition(" ")
        out[name] = out.get(name, 0) + int(n)
    return out


@contextmanager
def engaged(*expect, none=()):
    """The calls inside the block launch at least one kernel whose counter name matches each regular
    expression of `expect`, and none whose name matches one of `none` (re.search on the dotted
    names).  Several kernels of this library return the same bits, so a comparison of results cannot
    tell which one served a call: this can (the reference's tests read its engaged counters for
    the same reason, src/inference/tests.rs:7158-7196)."""
    import re
    before = launch_counts()
    yield
    after = launch_counts()
    fired = {k: v - before.get(k, 0) for k, v in after.items() if v > before.get(k, 0)}
    for pat in expect:
        assert any(re.search(pat, k) for k in fired), f"no kernel matching {pat!r} ran; launched: {fired}"
    for pat in none:
        hit = {k: v for k, v in fired.items() if re.search(pat, k)}
        assert not hit, f"kernels matching {pat!r} ran: {hit}"


def is_k(fmt: int) -> bool:
    return fmt in (B.CML_Q4_K, B.CML_Q6_K)


def gpu_quantize(fmt_family_k: bool, x: np.ndarray):
    """x f32[n_tokens, cols] -> (scales f32[n_tokens, nb], q int8[n_tokens, cols]) on the device, copied back."""
    x = np.ascontiguousarray(x, np.float32)
    x2 = x.reshape(1, -1) if x.ndim == 1 else x
    n_tokens, cols = x2.shape
    per = 256 if fmt_family_k else 32
    xd = DeviceBuffer.from_numpy(x2)
    qd = DeviceBuffer(max(x2.size, 16))
    sd = DeviceBuffer(max(n_tokens * (cols // per) * 4, 16))
    f = lib().cml_quantize_q8_k if fmt_family_k else lib().cml_quantize_q8_0
    check(f(xd.ptr, n_tokens, cols, qd.ptr, sd.ptr, None), "cml_quantize")
    check(lib().cml_stream_sync(None))
    q = qd.to_numpy(np.int8, (n_tokens, cols))
    s = sd.to_numpy(np.float32, (n_tokens, cols // per))
    return (s[0], q[0]) if x.ndim == 1 else (s, q)


def gpu_gemm(w: Weight, scales: np.ndarray, q: np.ndarray, residual: np.ndarray | None = None) -> np.ndarray:
    """Quantized activations in, f32 out[n_tokens, rows] (cml_gemv for one row, cml_gemm otherwise)."""
    scales = np.ascontiguousarray(scales, np.float32)
    q = np.ascontiguousarray(q, np.int8)
    single = q.ndim == 1
    n_tokens = 1 if single else q.shape[0]
    qd = DeviceBuffer.from_numpy(q)
    sd = DeviceBuffer.from_numpy(scales)
    od = DeviceBuffer(max(n_tokens * w.rows * 4, 16))
    od.fill(0xFF)
    if single:
        rd = DeviceBuffer.from_numpy(np.ascontiguousarray(residual, np.float32)) if residual is not None else None
        check(lib().cml_gemv(w.handle, qd.ptr, sd.ptr, od.ptr, rd.ptr if rd else None, None), "cml_gemv")
    else:
        assert residual is None
        check(lib().cml_gemm(w.handle, qd.ptr, sd.ptr, n_tokens, od.ptr, None), "cml_gemm")
    check(lib().cml_stream_sync(None))
    out = od.to_numpy(np.float32, (n_tokens, w.rows))
    return out[0] if single else out


def gpu_block_dots(w: Weight, q: np.ndarray) -> np.ndarray:
    nb = w.cols // lib().cml_block_values(w.fmt)
    per = 2 if w.fmt == B.CML_Q4_K else 1
    qd = DeviceBuffer.from_numpy(np.ascontiguousarray(q, np.int8))
    idev = DeviceBuffer(max(w.rows * nb * per * 4, 16))
    idev.fill(0xFF)
    check(lib().cml_block_dots(w.handle, qd.ptr, idev.ptr, None), "cml_block_dots")
    out = idev.to_numpy(np.int32, (w.rows, nb * per))
    return out.reshape(w.rows, nb, 2) if per == 2 else out


def gpu_dequant(w: Weight) -> np.ndarray:
    od = DeviceBuffer(max(w.rows * w.cols * 4, 16))
    check(lib().cml_dequantize(w.handle, od.ptr, None), "cml_dequantize")
    check(lib().cml_stream_sync(None))
    return od.to_numpy(np.float32, (w.rows * w.cols,))


def gpu_matmul_f32(w: Weight, x: np.ndarray) -> np.ndarray:
    x = np.ascontiguousarray(x, np.float32)
    single = x.ndim == 1
    x2 = x.reshape(1, -1) if single else x
    n_tokens = x2.shape[0]
    ws_bytes = lib().cml_matmul_workspace_bytes(w.fmt, w.cols, n_tokens)
    xd = DeviceBuffer.from_numpy(x2)
    ws = DeviceBuffer(max(ws_bytes, 16))
    od = DeviceBuffer(max(n_tokens * w.rows * 4, 16))
    od.fill(0xFF)
    check(lib().cml_matmul_f32(w.handle, xd.ptr, n_tokens, od.ptr, ws.ptr, ws_bytes, None), "cml_matmul_f32")
    check(lib().cml_stream_sync(None))
    out = od.to_numpy(np.float32, (n_tokens, w.rows))
    return out[0] if single else out


def synth_weight(fmt: int, rows: int, cols: int, seed: int, sigma: float = 0.02) -> np.ndarray:
    """Seeded ~N(0, sigma) f32 weights quantized to `fmt` wire bytes (BASELINE's recipe)."""
    rng = np.random.default_rng(seed)
    out = np.empty(rows * oracle.row_bytes(fmt, cols), np.uint8)
    rb = oracle.row_bytes(fmt, cols)
    step = max(1, (1 << 24) // cols)  # ~64 MiB of f32 at a time
    for r0 in range(0, rows, step):
        r1 = min(rows, r0 + step)
        w = rng.standard_normal((r1 - r0, cols), dtype=np.float32) * np.float32(sigma)
        out[r0 * rb:r1 * rb] = oracle.quantize_weights(fmt, w)
    return out


def max_rel(got: np.ndarray, want: np.ndarray) -> float:
    """The reference's closeness metric, |x-y| / max(|y|, 1) (src/cuda_resident/tests.rs:3768)."""
    got = got.astype(np.float64)
    want = want.astype(np.float64)
    return float(np.max(np.abs(got - want) / np.maximum(np.abs(want), 1.0))) if got.size else 0.0


def same_bits(a: np.ndarray, b: np.ndarray) -> bool:
    """Bitwise equality, except that +0 and -0 compare equal."""
    a = np.ascontiguousarray(a, np.float32)
    b = np.ascontiguousarray(b, np.float32)
    return bool(np.all((a.view(np.uint32) == b.view(np.uint32)) | ((a == 0) & (b == 0))))
