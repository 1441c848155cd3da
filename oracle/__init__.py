"""ctypes binding of the CPU oracle (``liboracle.so``).

TEST INFRASTRUCTURE, NOT PRODUCT CODE.  Only the test-suite, the smoke check
and the benchmark's CPU-baseline leg import this module; the HIP library never
does.  The arithmetic lives in ``camelid_oracle.c``; this file only marshals
numpy arrays.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "liboracle.so")

Q4_0, Q8_0, Q4_K, Q6_K = 2, 8, 12, 14
ORDER_PRIMARY, ORDER_ALT = 0, 1

FORMATS = {"Q4_0": Q4_0, "Q8_0": Q8_0, "Q4_K": Q4_K, "Q6_K": Q6_K}


def build(force: bool = False) -> str:
    """Compile the oracle with the Makefile beside it."""
    if force:
        subprocess.run(["make", "-C", HERE, "clean"], check=True, capture_output=True)
    subprocess.run(["make", "-C", HERE], check=True, capture_output=True)
    return LIB_PATH


_lib = None


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            build()
        L = C.CDLL(LIB_PATH)
        vp, sz, i32 = C.c_void_p, C.c_size_t, C.c_int
        L.orc_block_values.restype = i32
        L.orc_block_bytes.restype = i32
        L.orc_f32_to_f16_bits.argtypes = [C.c_float]
        L.orc_f32_to_f16_bits.restype = C.c_uint16
        L.orc_f16_bits_to_f32.argtypes = [C.c_uint16]
        L.orc_f16_bits_to_f32.restype = C.c_float
        L.orc_f32_to_f16_bits_array.argtypes = [vp, sz, vp]
        L.orc_f16_bits_to_f32_array.argtypes = [vp, sz, vp]
        L.orc_quantize_q8_0.argtypes = [vp, sz, vp, vp]
        L.orc_quantize_q8_k.argtypes = [vp, sz, vp, vp]
        L.orc_dequant.argtypes = [i32, vp, sz, vp]
        for name in ("orc_q8_0_row_dot", "orc_q4_0_row_dot", "orc_q4_k_row_dot_arm",
                     "orc_q4_k_row_dot_generic", "orc_q6_k_row_dot_lanes", "orc_q6_k_row_dot_arm"):
            f = getattr(L, name)
            f.argtypes = [vp, vp, vp, sz]
            f.restype = C.c_float
        L.orc_row_block_ints.argtypes = [i32, vp, vp, sz, vp]
        L.orc_matmul.argtypes = [i32, i32, vp, sz, sz, sz, vp, sz, vp, i32]
        L.orc_matmul.restype = i32
        L.orc_matmul_q.argtypes = [i32, i32, vp, sz, sz, sz, vp, vp, sz, vp, i32]
        L.orc_matmul_q.restype = i32
        L.orc_softmax_top_k.argtypes = [vp, i32, i32, vp, vp]
        L.orc_softmax_top_k.restype = i32
        L.orc_silu_mul.argtypes = [vp, vp, sz, vp]
        L.orc_gelu_tanh_mul.argtypes = [vp, vp, sz, vp]
        L.orc_router_softmax_top_k.argtypes = [vp, i32, i32, vp, vp, vp]
        L.orc_router_softmax_top_k.restype = i32
        L.orc_moe_ffn_ex.argtypes = [i32, i32, vp, vp, vp, i32, i32, sz, sz, vp, vp, sz, vp, i32, i32, vp]
        L.orc_moe_ffn_ex.restype = i32
        L.orc_rms_norm.argtypes = [vp, vp, C.c_float, sz, sz, vp]
        L.orc_rms_norm.restype = None
        L.orc_moe_ffn.argtypes = [i32, vp, vp, vp, i32, i32, sz, sz, vp, vp, sz, vp, i32]
        L.orc_moe_ffn.restype = i32
        L.orc_quantize_weights.argtypes = [i32, vp, sz, vp, i32]
        L.orc_quantize_weights.restype = i32
        _lib = L
    return _lib


def _p(a: np.ndarray) -> int:
    return a.ctypes.data


def _c(a, dtype) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=dtype)


def block_values(fmt: int) -> int:
    return lib().orc_block_values(fmt)


def block_bytes(fmt: int) -> int:
    return lib().orc_block_bytes(fmt)


def is_k_family(fmt: int) -> bool:
    return fmt in (Q4_K, Q6_K)


def row_bytes(fmt: int, cols: int) -> int:
    return cols // block_values(fmt) * block_bytes(fmt)


def f32_to_f16_bits(v: float) -> int:
    return lib().orc_f32_to_f16_bits(float(np.float32(v)))


def f16_bits_to_f32(h: int) -> np.float32:
    return np.float32(lib().orc_f16_bits_to_f32(int(h)))


def f32_to_f16_bits_array(v) -> np.ndarray:
    v = _c(v, np.float32)
    out = np.empty(v.shape, np.uint16)
    lib().orc_f32_to_f16_bits_array(_p(v), v.size, _p(out))
    return out


def f16_bits_to_f32_array(h) -> np.ndarray:
    h = _c(h, np.uint16)
    out = np.empty(h.shape, np.float32)
    lib().orc_f16_bits_to_f32_array(_p(h), h.size, _p(out))
    return out


def quantize_q8_0(x):
    """f32[..., K] -> (scales f32[..., K/32], q int8[..., K])."""
    x = _c(x, np.float32)
    scales = np.empty(x.shape[:-1] + (x.shape[-1] // 32,), np.float32)
    q = np.empty(x.shape, np.int8)
    lib().orc_quantize_q8_0(_p(x), x.size, _p(scales), _p(q))
    return scales, q


def quantize_q8_k(x):
    """f32[..., K] -> (d f32[..., K/256], q int8[..., K])."""
    x = _c(x, np.float32)
    d = np.empty(x.shape[:-1] + (x.shape[-1] // 256,), np.float32)
    q = np.empty(x.shape, np.int8)
    lib().orc_quantize_q8_k(_p(x), x.size, _p(d), _p(q))
    return d, q


def quantize_activation(fmt: int, x):
    return quantize_q8_k(x) if is_k_family(fmt) else quantize_q8_0(x)


def dequant(fmt: int, wire) -> np.ndarray:
    wire = _c(wire, np.uint8).reshape(-1)
    nb = wire.size // block_bytes(fmt)
    out = np.empty(nb * block_values(fmt), np.float32)
    lib().orc_dequant(fmt, _p(wire), nb, _p(out))
    return out


_ROW_DOTS = {
    (Q8_0, ORDER_PRIMARY): "orc_q8_0_row_dot",
    (Q4_0, ORDER_PRIMARY): "orc_q4_0_row_dot",
    (Q4_K, ORDER_PRIMARY): "orc_q4_k_row_dot_arm",
    (Q4_K, ORDER_ALT): "orc_q4_k_row_dot_generic",
    (Q6_K, ORDER_PRIMARY): "orc_q6_k_row_dot_lanes",
    (Q6_K, ORDER_ALT): "orc_q6_k_row_dot_arm",
}


def row_dot(fmt: int, order: int, w_row, xscales, xq) -> np.float32:
    w_row = _c(w_row, np.uint8)
    xscales = _c(xscales, np.float32)
    xq = _c(xq, np.int8)
    f = getattr(lib(), _ROW_DOTS[(fmt, order)])
    return np.float32(f(_p(w_row), _p(xscales), _p(xq), xscales.size))


def row_block_ints(fmt: int, w_row, xq) -> np.ndarray:
    w_row = _c(w_row, np.uint8)
    xq = _c(xq, np.int8)
    nb = xq.size // block_values(fmt)
    out = np.empty(nb * (2 if fmt == Q4_K else 1), np.int32)
    lib().orc_row_block_ints(fmt, _p(w_row), _p(xq), nb, _p(out))
    return out


def block_ints(fmt: int, wire, cols: int, xq, row_start: int = 0, rows: int | None = None) -> np.ndarray:
    """Per-block integers of every row: int32[rows, n_blocks(, 2 for Q4_K)]."""
    wire = _c(wire, np.uint8).reshape(-1)
    rb = row_bytes(fmt, cols)
    if rows is None:
        rows = wire.size // rb - row_start
    nb = cols // block_values(fmt)
    per = 2 if fmt == Q4_K else 1
    out = np.empty((rows, nb * per), np.int32)
    xq = _c(xq, np.int8)
    for r in range(rows):
        off = (row_start + r) * rb
        lib().orc_row_block_ints(fmt, _p(wire) + off, _p(xq), nb, _p(out) + r * nb * per * 4)
    return out.reshape(rows, nb, per) if per == 2 else out


def matmul(fmt: int, wire, cols: int, x, order: int = ORDER_PRIMARY, row_start: int = 0,
           rows: int | None = None, threads: int = 1) -> np.ndarray:
    """x f32[n_tokens, cols] (or [cols]) -> out f32[n_tokens, rows] (or [rows])."""
    wire = _c(wire, np.uint8).reshape(-1)
    x = _c(x, np.float32)
    single = x.ndim == 1
    x2 = x.reshape(1, -1) if single else x
    if rows is None:
        rows = wire.size // row_bytes(fmt, cols) - row_start
    out = np.empty((x2.shape[0], rows), np.float32)
    rc = lib().orc_matmul(fmt, order, _p(wire), cols, row_start, rows, _p(x2), x2.shape[0], _p(out), threads)
    if rc != 0:
        raise ValueError(f"orc_matmul failed: {rc}")
    return out[0] if single else out


def matmul_q(fmt: int, wire, cols: int, xscales, xq, order: int = ORDER_PRIMARY, row_start: int = 0,
             rows: int | None = None, threads: int = 1) -> np.ndarray:
    wire = _c(wire, np.uint8).reshape(-1)
    xscales = _c(xscales, np.float32)
    xq = _c(xq, np.int8)
    single = xq.ndim == 1
    n_tokens = 1 if single else xq.shape[0]
    if rows is None:
        rows = wire.size // row_bytes(fmt, cols) - row_start
    out = np.empty((n_tokens, rows), np.float32)
    rc = lib().orc_matmul_q(fmt, order, _p(wire), cols, row_start, rows, _p(xscales), _p(xq), n_tokens,
                            _p(out), threads)
    if rc != 0:
        raise ValueError(f"orc_matmul_q failed: {rc}")
    return out[0] if single else out


def softmax_top_k(logits, k: int):
    logits = _c(logits, np.float32).reshape(-1)
    kk = min(k, logits.size)
    idx = np.empty(max(kk, 1), np.int32)
    w = np.empty(max(kk, 1), np.float32)
    n = lib().orc_softmax_top_k(_p(logits), logits.size, k, _p(idx), _p(w))
    return idx[:n].copy(), w[:n].copy()


def rms_norm(x, weight, eps: float) -> np.ndarray:
    """Rows of x normalised as the reference does (sequential f32 sum of squares)."""
    x = _c(x, np.float32)
    weight = _c(weight, np.float32)
    x2 = x.reshape(-1, weight.size)
    out = np.empty_like(x2)
    lib().orc_rms_norm(_p(x2), _p(weight), C.c_float(eps), x2.shape[0], x2.shape[1], _p(out))
    return out.reshape(x.shape)


def silu_mul(a, b) -> np.ndarray:
    a = _c(a, np.float32)
    b = _c(b, np.float32)
    out = np.empty_like(a)
    lib().orc_silu_mul(_p(a), _p(b), a.size, _p(out))
    return out


def gelu_tanh_mul(a, b) -> np.ndarray:
    a = _c(a, np.float32)
    b = _c(b, np.float32)
    out = np.empty_like(a)
    lib().orc_gelu_tanh_mul(_p(a), _p(b), a.size, _p(out))
    return out


def router_softmax_top_k(logits, k: int, down_scale=None):
    """Gemma-4 routing of one token: (idx int32[k'], scale f32[k'])."""
    logits = _c(logits, np.float32).reshape(-1)
    idx = np.zeros(k, np.int32)
    w = np.zeros(k, np.float32)
    ds = None if down_scale is None else _c(down_scale, np.float32)
    n = lib().orc_router_softmax_top_k(_p(logits), logits.size, k, None if ds is None else _p(ds), _p(idx), _p(w))
    return idx[:n], w[:n]


def moe_ffn_ex(fmt: int, gate, up, down, n_experts: int, top_k: int, hidden: int, ff: int, logits, x,
               variant: int = 0, down_scale=None, threads: int = 1, fmt_down: int | None = None) -> np.ndarray:
    """variant 0 = Mixtral, 1 = Gemma-4; up=None: `gate` holds fused gate|up experts;
    fmt_down: format of `down` when it differs from that of gate / up."""
    gate, down = (_c(a, np.uint8).reshape(-1) for a in (gate, down))
    upc = None if up is None else _c(up, np.uint8).reshape(-1)
    logits = _c(logits, np.float32).reshape(-1, n_experts)
    x = _c(x, np.float32).reshape(-1, hidden)
    ds = None if down_scale is None else _c(down_scale, np.float32)
    out = np.empty_like(x)
    rc = lib().orc_moe_ffn_ex(fmt, fmt if fmt_down is None else fmt_down, _p(gate), None if upc is None else _p(upc), _p(down), n_experts, top_k, hidden, ff,
                              _p(logits), _p(x), x.shape[0], _p(out), threads, variant, None if ds is None else _p(ds))
    if rc != 0:
        raise ValueError(f"orc_moe_ffn_ex failed: {rc}")
    return out


def moe_ffn(fmt: int, gate, up, down, n_experts: int, top_k: int, hidden: int, ff: int, logits, x,
            threads: int = 1) -> np.ndarray:
    gate, up, down = (_c(a, np.uint8).reshape(-1) for a in (gate, up, down))
    logits = _c(logits, np.float32).reshape(-1, n_experts)
    x = _c(x, np.float32).reshape(-1, hidden)
    out = np.empty_like(x)
    rc = lib().orc_moe_ffn(fmt, _p(gate), _p(up), _p(down), n_experts, top_k, hidden, ff, _p(logits), _p(x),
                           x.shape[0], _p(out), threads)
    if rc != 0:
        raise ValueError(f"orc_moe_ffn failed: {rc}")
    return out


def quantize_weights(fmt: int, w, threads: int = 8) -> np.ndarray:
    """f32 values (any shape, row-major, rows of whole blocks) -> wire bytes uint8[...]."""
    w = _c(w, np.float32)
    n = w.size
    out = np.empty(n // block_values(fmt) * block_bytes(fmt), np.uint8)
    rc = lib().orc_quantize_weights(fmt, _p(w), n, _p(out), threads)
    if rc != 0:
        raise ValueError(f"orc_quantize_weights failed: {rc}")
    return out
