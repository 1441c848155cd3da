"""ctypes binding of libcamelid_hip.so (the C ABI in include/camelid_hip.h).

There is no CPU fallback here on purpose: if the shared library is missing, or a
call returns a non-zero status, a CamelidHipError is raised.
"""
from __future__ import annotations

import ctypes as C
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))

CML_Q4_0, CML_Q8_0, CML_Q4_K, CML_Q6_K = 2, 8, 12, 14
FORMATS = {"Q4_0": CML_Q4_0, "Q8_0": CML_Q8_0, "Q4_K": CML_Q4_K, "Q6_K": CML_Q6_K}

EXPORTS = [
    "cml_available", "cml_init", "cml_shutdown", "cml_reload_env", "cml_last_error", "cml_run_count", "cml_kernel_launches", "cml_kernel_launch_report",
    "cml_block_values", "cml_block_bytes",
    "cml_dev_alloc", "cml_dev_free", "cml_memcpy_h2d", "cml_memcpy_d2h", "cml_memset_dev", "cml_copy_dev", "cml_calibrate_read", "cml_calibrate_weight_loads", "cml_calibrate_matvec_ablation", "cml_stream_sync",
    "cml_stream_create", "cml_stream_destroy", "cml_event_create", "cml_event_record", "cml_event_elapsed_ms",
    "cml_event_destroy", "cml_graph_begin_capture", "cml_graph_end_capture", "cml_graph_launch", "cml_graph_destroy",
    "cml_weight_upload", "cml_weight_upload_dev", "cml_weight_slice", "cml_weight_info",
    "cml_weight_download", "cml_weight_free",
    "cml_quantize_q8_0", "cml_quantize_q8_k", "cml_rms_norm_quantize", "cml_rms_inv_norm_quantize", "cml_sum_squares_f32", "cml_silu_mul_quantize", "cml_glu_quantize", "cml_embed_gather", "cml_argmax_f32", "cml_dequantize",
    "cml_gemv", "cml_gemm", "cml_block_dots", "cml_matmul_workspace_bytes", "cml_matmul_f32", "cml_matmul_f32_pair", "cml_matmul_f32_multi", "cml_matmul_f32_static",
    "cml_moe_route_top_k", "cml_moe_route_softmax_top_k", "cml_moe_workspace_bytes", "cml_moe_ffn", "cml_moe_ffn_ex", "cml_moe_ffn_logits",
    "cml_moe_plan", "cml_moe_gemv_routed", "cml_moe_weighted_sum",
    "cml_quantize_weights_host", "cml_try_linear_rows", "cml_try_q8_0_block_linear_row",
]


class CamelidHipError(RuntimeError):
    pass


def lib_path() -> str:
    return os.path.join(HERE, "libcamelid_hip.so")


_lib = None


def lib() -> C.CDLL:
    """Load libcamelid_hip.so; raises if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    path = lib_path()
    if not os.path.exists(path):
        raise CamelidHipError(
            f"{path} is missing: build it with `python -m camelid_amd.build` (needs hipcc); "
            "there is no CPU fallback")
    L = C.CDLL(path)
    vp, sz, i64, i32 = C.c_void_p, C.c_size_t, C.c_int64, C.c_int
    pp = C.POINTER(C.c_void_p)
    L.cml_available.restype = i32
    L.cml_init.argtypes = [i32]
    L.cml_last_error.restype = C.c_char_p
    L.cml_kernel_launches.argtypes = [C.c_char_p]
    L.cml_kernel_launches.restype = C.c_uint64
    L.cml_kernel_launch_report.argtypes = [C.c_char_p, sz]
    L.cml_kernel_launch_report.restype = sz
    L.cml_run_count.restype = C.c_uint64
    L.cml_block_values.argtypes = [i32]
    L.cml_block_bytes.argtypes = [i32]
    L.cml_dev_alloc.argtypes = [sz, pp]
    L.cml_dev_free.argtypes = [vp]
    L.cml_memcpy_h2d.argtypes = [vp, vp, sz, vp]
    L.cml_memcpy_d2h.argtypes = [vp, vp, sz, vp]
    L.cml_memset_dev.argtypes = [vp, i32, sz, vp]
    L.cml_copy_dev.argtypes = [vp, vp, sz, vp]
    L.cml_calibrate_read.argtypes = [vp, sz, i32, i32, vp]
    L.cml_calibrate_weight_loads.argtypes = [vp, vp, vp]
    L.cml_calibrate_matvec_ablation.argtypes = [vp, vp, vp, i32, vp]
    L.cml_stream_sync.argtypes = [vp]
    L.cml_stream_create.argtypes = [pp]
    L.cml_stream_destroy.argtypes = [vp]
    L.cml_event_create.argtypes = [pp]
    L.cml_event_record.argtypes = [vp, vp]
    L.cml_event_elapsed_ms.argtypes = [vp, vp, C.POINTER(C.c_float)]
    L.cml_event_destroy.argtypes = [vp]
    L.cml_graph_begin_capture.argtypes = [vp]
    L.cml_graph_end_capture.argtypes = [vp, pp]
    L.cml_graph_launch.argtypes = [vp, vp]
    L.cml_graph_destroy.argtypes = [vp]
    L.cml_weight_upload.argtypes = [i32, i64, i64, vp, sz, pp]
    L.cml_weight_upload_dev.argtypes = [i32, i64, i64, vp, sz, vp, pp]
    L.cml_weight_slice.argtypes = [vp, i64, i64, pp]
    L.cml_weight_info.argtypes = [vp, C.POINTER(i32), C.POINTER(i64), C.POINTER(i64), C.POINTER(sz)]
    L.cml_weight_download.argtypes = [vp, vp, sz]
    L.cml_weight_free.argtypes = [vp]
    L.cml_weight_free.restype = None
    L.cml_quantize_q8_0.argtypes = [vp, i64, i64, vp, vp, vp]
    L.cml_quantize_q8_k.argtypes = [vp, i64, i64, vp, vp, vp]
    L.cml_rms_norm_quantize.argtypes = [i32, vp, vp, C.c_float, i64, i64, vp, vp, vp, vp]
    L.cml_rms_inv_norm_quantize.argtypes = [i32, vp, vp, C.c_float, i64, vp, vp, vp]
    L.cml_sum_squares_f32.argtypes = [vp, i64, i64, vp, vp]
    L.cml_silu_mul_quantize.argtypes = [i32, vp, vp, i64, i64, vp, vp, vp]
    L.cml_embed_gather.argtypes = [vp, vp, i64, vp, vp]
    L.cml_argmax_f32.argtypes = [vp, i64, i64, vp, vp]
    L.cml_dequantize.argtypes = [vp, vp, vp]
    L.cml_gemv.argtypes = [vp, vp, vp, vp, vp, vp]
    L.cml_gemm.argtypes = [vp, vp, vp, i64, vp, vp]
    L.cml_block_dots.argtypes = [vp, vp, vp, vp]
    L.cml_matmul_workspace_bytes.argtypes = [i32, i64, i64]
    L.cml_matmul_workspace_bytes.restype = sz
    L.cml_matmul_f32.argtypes = [vp, vp, i64, vp, vp, sz, vp]
    L.cml_matmul_f32_static.argtypes = [vp, vp, i64, vp, vp]
    L.cml_matmul_f32_pair.argtypes = [vp, vp, vp, vp, vp, vp, sz, vp]
    L.cml_matmul_f32_multi.argtypes = [vp, i32, vp, vp, vp, sz, vp]
    L.cml_moe_route_top_k.argtypes = [vp, i64, i32, i32, vp, vp, vp]
    L.cml_moe_workspace_bytes.argtypes = [i32, i64, i64, i64, i32, i32]
    L.cml_moe_workspace_bytes.restype = sz
    L.cml_moe_ffn.argtypes = [vp, vp, vp, i32, i32, vp, vp, vp, i64, vp, vp, sz, vp]
    L.cml_moe_ffn_ex.argtypes = [vp, vp, vp, i32, i32, vp, vp, vp, i64, vp, vp, sz, i32, vp]
    L.cml_moe_ffn_logits.argtypes = [vp, vp, vp, i32, i32, vp, vp, i64, vp, vp, sz, vp]
    L.cml_moe_route_softmax_top_k.argtypes = [vp, i64, i32, i32, vp, vp, vp, vp]
    L.cml_moe_plan.argtypes = [vp, i64, i32, i32, vp, vp, vp, vp, vp]
    L.cml_moe_gemv_routed.argtypes = [vp, i32, vp, vp, vp, vp, vp, i32, i64, vp, vp]
    L.cml_moe_weighted_sum.argtypes = [vp, vp, vp, i64, i32, i64, vp, vp]
    L.cml_glu_quantize.argtypes = [i32, i32, vp, vp, i64, i64, vp, vp, vp]
    L.cml_quantize_weights_host.argtypes = [i32, vp, sz, vp, i32]
    L.cml_try_linear_rows.argtypes = [i32, vp, vp, vp, sz, i64, i64, i64, vp]
    L.cml_try_q8_0_block_linear_row.argtypes = [vp, vp, vp, sz, i64, i64, vp]
    _lib = L
    return L


def check(rc: int, what: str = "") -> None:
    if rc != 0:
        msg = lib().cml_last_error().decode(errors="replace")
        raise CamelidHipError(f"{what or 'camelid_hip call'} failed with status {rc}: {msg}")


_initialised = False


def init(device: int = 0) -> None:
    """cml_init once per process; raises when no gfx950 device is usable."""
    global _initialised
    if not _initialised:
        check(lib().cml_init(device), "cml_init")
        _initialised = True


class DeviceBuffer:
    """A device allocation made through the C ABI (cml_dev_alloc)."""

    def __init__(self, nbytes: int):
        init()
        self.nbytes = int(nbytes)
        p = C.c_void_p()
        check(lib().cml_dev_alloc(self.nbytes, C.byref(p)), "cml_dev_alloc")
        self.ptr = p.value

    @classmethod
    def from_numpy(cls, a: np.ndarray) -> "DeviceBuffer":
        a = np.ascontiguousarray(a)
        buf = cls(a.nbytes)
        if a.nbytes:
            check(lib().cml_memcpy_h2d(buf.ptr, a.ctypes.data, a.nbytes, None), "cml_memcpy_h2d")
        return buf

    def to_numpy(self, dtype, shape) -> np.ndarray:
        out = np.empty(shape, dtype=dtype)
        assert out.nbytes <= self.nbytes
        if out.nbytes:
            check(lib().cml_memcpy_d2h(out.ctypes.data, self.ptr, out.nbytes, None), "cml_memcpy_d2h")
        return out

    def fill(self, byte: int = 0) -> None:
        check(lib().cml_memset_dev(self.ptr, byte, self.nbytes, None), "cml_memset_dev")
        check(lib().cml_stream_sync(None), "cml_stream_sync")

    def free(self) -> None:
        if self.ptr:
            lib().cml_dev_free(self.ptr)
            self.ptr = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


class Weight:
    """A device-resident weight handle (cml_weight_upload / cml_weight_slice)."""

    def __init__(self, handle: int, fmt: int, rows: int, cols: int, parent: "Weight | None" = None):
        self.handle, self.fmt, self.rows, self.cols, self.parent = handle, fmt, rows, cols, parent

    @classmethod
    def upload(cls, fmt: int, rows: int, cols: int, wire: np.ndarray) -> "Weight":
        init()
        wire = np.ascontiguousarray(wire, dtype=np.uint8).reshape(-1)
        h = C.c_void_p()
        check(lib().cml_weight_upload(fmt, rows, cols, wire.ctypes.data, wire.nbytes, C.byref(h)), "cml_weight_upload")
        return cls(h.value, fmt, rows, cols)

    def slice(self, row_start: int, rows: int) -> "Weight":
        h = C.c_void_p()
        check(lib().cml_weight_slice(self.handle, row_start, rows, C.byref(h)), "cml_weight_slice")
        return Weight(h.value, self.fmt, rows, self.cols, parent=self)

    @property
    def wire_bytes(self) -> int:
        L = lib()
        return self.rows * (self.cols // L.cml_block_values(self.fmt)) * L.cml_block_bytes(self.fmt)

    def download(self) -> np.ndarray:
        out = np.empty(self.wire_bytes, np.uint8)
        check(lib().cml_weight_download(self.handle, out.ctypes.data, out.nbytes), "cml_weight_download")
        return out

    def free(self) -> None:
        if self.handle:
            lib().cml_weight_free(self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


def quantize_weights(fmt: int, values: np.ndarray, threads: int = 8) -> np.ndarray:
    """f32 values (rows of whole blocks) -> GGUF wire bytes, on the host (cml_quantize_weights_host)."""
    L = lib()
    values = np.ascontiguousarray(values, np.float32)
    out = np.empty(values.size // L.cml_block_values(fmt) * L.cml_block_bytes(fmt), np.uint8)
    check(L.cml_quantize_weights_host(fmt, values.ctypes.data, values.size, out.ctypes.data, threads),
          "cml_quantize_weights_host")
    return out
