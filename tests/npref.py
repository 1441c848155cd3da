"""Independent numpy decoders of the GGUF wire block layouts.

Written from the format description (field offsets and bit positions), not
from the oracle's C code, so that the oracle's integer arithmetic can be
checked by brute force.  Each decoder returns the *integers* of a block; the
tests first pin these decoders against the golden dequant fixtures and then
use them to check the oracle's integer block dots.
"""
import numpy as np


def f16(buf, off):
    return np.frombuffer(bytes(buf[off:off + 2]), dtype="<f2")[0].astype(np.float32)


def q8_0_block(blk):
    """-> (d f32, q int32[32])"""
    return f16(blk, 0), np.frombuffer(bytes(blk[2:34]), dtype=np.int8).astype(np.int32)


def q4_0_block(blk):
    """-> (d f32, q int32[32]) with the -8 bias applied"""
    b = np.frombuffer(bytes(blk[2:18]), dtype=np.uint8).astype(np.int32)
    q = np.concatenate([b & 15, b >> 4]) - 8
    return f16(blk, 0), q


def q4_k_block(blk):
    """-> (d, dmin, sc int32[8], m int32[8], q int32[256] in 0..15)"""
    d, dmin = f16(blk, 0), f16(blk, 2)
    s = np.frombuffer(bytes(blk[4:16]), dtype=np.uint8).astype(np.int32)
    sc = np.zeros(8, np.int32)
    m = np.zeros(8, np.int32)
    for g in range(8):
        if g < 4:
            sc[g] = s[g] & 63
            m[g] = s[g + 4] & 63
        else:
            sc[g] = (s[g + 4] & 15) | ((s[g - 4] >> 6) << 4)
            m[g] = (s[g + 4] >> 4) | ((s[g] >> 6) << 4)
    qs = np.frombuffer(bytes(blk[16:144]), dtype=np.uint8).astype(np.int32)
    q = np.zeros(256, np.int32)
    for c in range(4):
        q[64 * c:64 * c + 32] = qs[32 * c:32 * c + 32] & 15
        q[64 * c + 32:64 * c + 64] = qs[32 * c:32 * c + 32] >> 4
    return d, dmin, sc, m, q


def q6_k_block(blk):
    """-> (d, sc int32[16], q int32[256] in -32..31)"""
    ql = np.frombuffer(bytes(blk[0:128]), dtype=np.uint8).astype(np.int32)
    qh = np.frombuffer(bytes(blk[128:192]), dtype=np.uint8).astype(np.int32)
    sc = np.frombuffer(bytes(blk[192:208]), dtype=np.int8).astype(np.int32)
    d = f16(blk, 208)
    q = np.zeros(256, np.int32)
    for h in range(2):
        L = ql[64 * h:64 * h + 64]
        H = qh[32 * h:32 * h + 32]
        base = 128 * h
        q[base + 0:base + 32] = (L[0:32] & 15) | ((H & 3) << 4)
        q[base + 32:base + 64] = (L[32:64] & 15) | (((H >> 2) & 3) << 4)
        q[base + 64:base + 96] = (L[0:32] >> 4) | (((H >> 4) & 3) << 4)
        q[base + 96:base + 128] = (L[32:64] >> 4) | (((H >> 6) & 3) << 4)
    return d, sc, q - 32


def dequant_f64(fmt_name, wire):
    """Dequantize in float64 from the integers (not bit-exact: for f64 reference dots)."""
    wire = np.asarray(wire, np.uint8)
    out = []
    if fmt_name == "Q8_0":
        for b in range(wire.size // 34):
            d, q = q8_0_block(wire[34 * b:34 * b + 34])
            out.append(float(d) * q)
    elif fmt_name == "Q4_0":
        for b in range(wire.size // 18):
            d, q = q4_0_block(wire[18 * b:18 * b + 18])
            out.append(float(d) * q)
    elif fmt_name == "Q4_K":
        for b in range(wire.size // 144):
            d, dmin, sc, m, q = q4_k_block(wire[144 * b:144 * b + 144])
            scv = np.repeat(sc, 32).astype(np.float64)
            mv = np.repeat(m, 32).astype(np.float64)
            out.append(float(d) * scv * q - float(dmin) * mv)
    elif fmt_name == "Q6_K":
        for b in range(wire.size // 210):
            d, sc, q = q6_k_block(wire[210 * b:210 * b + 210])
            out.append(float(d) * np.repeat(sc, 16).astype(np.float64) * q)
    else:
        raise ValueError(fmt_name)
    return np.concatenate(out).astype(np.float64)
