//! `src/hip.rs` for the reference engine: the MI355X lane behind the same seams the CUDA lane
//! sits behind (`src/cuda.rs:276-319`, `src/cuda_resident.rs`), bound to `libcamelid_hip.so`
//! (`include/camelid_hip.h`).  Every `extern "C"` item of the header is declared here; above
//! them are the three host-pointer seams with the reference's own argument checks
//! (`src/cuda.rs:953-966`), a resident weight type, and `HipWireQuant`, whose methods mirror
//! `WireQuant::{matvec, matmul_proj, matvec_rows_proj, dequantize_elements}`
//! (`src/gemma4_runtime.rs:826-1150`).
//!
//! This file is not compiled in this tree (no Rust toolchain here); the same boundary is
//! exercised by the C++ host layer (`camelid_amd/host/`) and by every GPU test through ctypes.
//! Convention throughout: status 0 = handled, anything else = the caller runs its CPU path;
//! nothing here panics across the seam.
#![allow(clippy::too_many_arguments, dead_code)]

use core::ffi::{c_char, c_void};
use std::collections::HashMap;
use std::sync::{Mutex, OnceLock};

// GGUF tensor type ids pass through unchanged (src/gguf/reader.rs:94-127).
pub const CML_Q4_0: i32 = 2;
pub const CML_Q8_0: i32 = 8;
pub const CML_Q4_K: i32 = 12;
pub const CML_Q6_K: i32 = 14;

pub const CML_OK: i32 = 0;
pub const CML_ERR_UNAVAILABLE: i32 = 1;
pub const CML_ERR_INVALID: i32 = 2;
pub const CML_ERR_SHAPE: i32 = 3;
pub const CML_ERR_HIP: i32 = 4;
pub const CML_ERR_OOM: i32 = 5;
pub const CML_ERR_UNSUPPORTED: i32 = 6;

pub const CML_ACT_F32: i32 = 0;
pub const CML_ACT_Q8_0: i32 = 1;
pub const CML_ACT_Q8_K: i32 = 2;
pub const CML_GLU_SILU: i32 = 0;
pub const CML_GLU_GELU_TANH: i32 = 1;
pub const CML_STATIC_WORKSPACE_BYTES: usize = 1024 * 1024 + 128 * 1024;

#[repr(C)]
pub struct CmlWeight {
    _private: [u8; 0],
}
pub type Stream = *mut c_void;
pub type Event = *mut c_void;
pub type Graph = *mut c_void;

#[link(name = "camelid_hip")]
extern "C" {
    // ---- lifecycle, gating, counters
    pub fn cml_available() -> i32;
    pub fn cml_init(device: i32) -> i32;
    pub fn cml_shutdown();
    pub fn cml_reload_env() -> i32;
    pub fn cml_last_error() -> *const c_char;
    pub fn cml_run_count() -> u64;
    pub fn cml_kernel_launches(prefix: *const c_char) -> u64;
    pub fn cml_kernel_launch_report(buf: *mut c_char, cap: usize) -> usize;
    pub fn cml_block_values(fmt: i32) -> i32;
    pub fn cml_block_bytes(fmt: i32) -> i32;
    // ---- device memory, streams, events, graphs
    pub fn cml_dev_alloc(nbytes: usize, out_dev: *mut *mut c_void) -> i32;
    pub fn cml_dev_free(ptr_dev: *mut c_void) -> i32;
    pub fn cml_memcpy_h2d(dst_dev: *mut c_void, src_host: *const c_void, nbytes: usize, stream: Stream) -> i32;
    pub fn cml_memcpy_d2h(dst_host: *mut c_void, src_dev: *const c_void, nbytes: usize, stream: Stream) -> i32;
    pub fn cml_memset_dev(dst_dev: *mut c_void, value: i32, nbytes: usize, stream: Stream) -> i32;
    pub fn cml_stream_sync(stream: Stream) -> i32;
    pub fn cml_stream_create(out: *mut Stream) -> i32;
    pub fn cml_stream_destroy(stream: Stream) -> i32;
    pub fn cml_event_create(out: *mut Event) -> i32;
    pub fn cml_event_record(event: Event, stream: Stream) -> i32;
    pub fn cml_event_elapsed_ms(start: Event, stop: Event, ms: *mut f32) -> i32;
    pub fn cml_event_destroy(event: Event) -> i32;
    pub fn cml_graph_begin_capture(stream: Stream) -> i32;
    pub fn cml_graph_end_capture(stream: Stream, out: *mut Graph) -> i32;
    pub fn cml_graph_launch(graph: Graph, stream: Stream) -> i32;
    pub fn cml_graph_destroy(graph: Graph) -> i32;
    // ---- diagnostics (bench.py only; a production host never calls these)
    pub fn cml_copy_dev(dst_dev: *mut c_void, src_dev: *const c_void, nbytes: usize, stream: Stream) -> i32;
    pub fn cml_calibrate_read(src_dev: *const c_void, nbytes: usize, in_flight: i32, workgroups: i32, stream: Stream) -> i32;
    pub fn cml_calibrate_weight_loads(w: *const CmlWeight, scratch_dev: *mut c_void, stream: Stream) -> i32;
    pub fn cml_calibrate_matvec_ablation(w: *const CmlWeight, x_dev: *const f32, out_dev: *mut f32, mask: i32, stream: Stream) -> i32;
    // ---- weights
    pub fn cml_weight_upload(fmt: i32, rows: i64, cols: i64, wire_host: *const c_void, nbytes: usize, out: *mut *mut CmlWeight) -> i32;
    pub fn cml_weight_upload_dev(fmt: i32, rows: i64, cols: i64, wire_dev: *const c_void, nbytes: usize, stream: Stream, out: *mut *mut CmlWeight) -> i32;
    pub fn cml_weight_slice(parent: *const CmlWeight, row_start: i64, rows: i64, out: *mut *mut CmlWeight) -> i32;
    pub fn cml_weight_info(w: *const CmlWeight, fmt: *mut i32, rows: *mut i64, cols: *mut i64, wire_bytes: *mut usize) -> i32;
    pub fn cml_weight_download(w: *const CmlWeight, wire_host: *mut c_void, nbytes: usize) -> i32;
    pub fn cml_weight_free(w: *mut CmlWeight);
    // ---- activation quantizers and fused producers
    pub fn cml_quantize_q8_0(x_dev: *const f32, n_tokens: i64, cols: i64, q_dev: *mut i8, scales_dev: *mut f32, stream: Stream) -> i32;
    pub fn cml_quantize_q8_k(x_dev: *const f32, n_tokens: i64, cols: i64, q_dev: *mut i8, d_dev: *mut f32, stream: Stream) -> i32;
    pub fn cml_rms_norm_quantize(act: i32, x_dev: *const f32, weight_dev: *const f32, eps: f32, n_tokens: i64, cols: i64,
                                 normed_dev: *mut f32, q_dev: *mut i8, scales_dev: *mut f32, stream: Stream) -> i32;
    pub fn cml_rms_inv_norm_quantize(act: i32, x_dev: *const f32, weight_dev: *const f32, rms_inv: f32, cols: i64,
                                     q_dev: *mut i8, scales_dev: *mut f32, stream: Stream) -> i32;
    pub fn cml_sum_squares_f32(x_dev: *const f32, n_rows: i64, cols: i64, out_dev: *mut f32, stream: Stream) -> i32;
    pub fn cml_silu_mul_quantize(act: i32, gate_dev: *const f32, up_dev: *const f32, n_tokens: i64, cols: i64,
                                 q_dev: *mut i8, scales_dev: *mut f32, stream: Stream) -> i32;
    pub fn cml_glu_quantize(glu: i32, act: i32, gate_dev: *const f32, up_dev: *const f32, n_tokens: i64, cols: i64,
                            q_dev: *mut i8, scales_dev: *mut f32, stream: Stream) -> i32;
    pub fn cml_dequantize(w: *const CmlWeight, out_dev: *mut f32, stream: Stream) -> i32;
    pub fn cml_embed_gather(table: *const CmlWeight, token_ids_dev: *const u32, n_tokens: i64, out_dev: *mut f32, stream: Stream) -> i32;
    pub fn cml_argmax_f32(logits_dev: *const f32, n_rows: i64, n: i64, out_idx_dev: *mut u32, stream: Stream) -> i32;
    // ---- matvec / matmul
    pub fn cml_gemv(w: *const CmlWeight, q_dev: *const i8, scales_dev: *const f32, out_dev: *mut f32, residual_dev: *const f32, stream: Stream) -> i32;
    pub fn cml_gemm(w: *const CmlWeight, q_dev: *const i8, scales_dev: *const f32, n_tokens: i64, out_dev: *mut f32, stream: Stream) -> i32;
    pub fn cml_block_dots(w: *const CmlWeight, q_dev: *const i8, ints_dev: *mut i32, stream: Stream) -> i32;
    pub fn cml_matmul_workspace_bytes(fmt: i32, cols: i64, n_tokens: i64) -> usize;
    pub fn cml_matmul_f32(w: *const CmlWeight, x_dev: *const f32, n_tokens: i64, out_dev: *mut f32,
                          workspace_dev: *mut c_void, workspace_bytes: usize, stream: Stream) -> i32;
    pub fn cml_matmul_f32_pair(w_a: *const CmlWeight, w_b: *const CmlWeight, x_dev: *const f32, out_a_dev: *mut f32, out_b_dev: *mut f32,
                               workspace_dev: *mut c_void, workspace_bytes: usize, stream: Stream) -> i32;
    pub fn cml_matmul_f32_multi(weights: *const *const CmlWeight, n_weights: i32, x_dev: *const f32, outs_dev: *const *mut f32,
                                workspace_dev: *mut c_void, workspace_bytes: usize, stream: Stream) -> i32;
    pub fn cml_matmul_f32_static(w: *const CmlWeight, x_dev: *const f32, n_tokens: i64, out_dev: *mut f32, stream: Stream) -> i32;
    // ---- mixture of experts
    pub fn cml_moe_route_top_k(logits_dev: *const f32, n_tokens: i64, n_experts: i32, k: i32, idx_dev: *mut i32, weight_dev: *mut f32, stream: Stream) -> i32;
    pub fn cml_moe_route_softmax_top_k(logits_dev: *const f32, n_tokens: i64, n_experts: i32, k: i32, down_scale_dev: *const f32,
                                       idx_dev: *mut i32, weight_dev: *mut f32, stream: Stream) -> i32;
    pub fn cml_moe_workspace_bytes(fmt: i32, hidden: i64, ff: i64, n_tokens: i64, k: i32, n_experts: i32) -> usize;
    pub fn cml_moe_ffn(gate: *const CmlWeight, up: *const CmlWeight, down: *const CmlWeight, n_experts: i32, k: i32, idx_dev: *const i32,
                       weight_dev: *const f32, x_dev: *const f32, n_tokens: i64, out_dev: *mut f32, workspace_dev: *mut c_void,
                       workspace_bytes: usize, stream: Stream) -> i32;
    pub fn cml_moe_ffn_ex(gate: *const CmlWeight, up: *const CmlWeight, down: *const CmlWeight, n_experts: i32, k: i32, idx_dev: *const i32,
                          weight_dev: *const f32, x_dev: *const f32, n_tokens: i64, out_dev: *mut f32, workspace_dev: *mut c_void,
                          workspace_bytes: usize, glu: i32, stream: Stream) -> i32;
    pub fn cml_moe_ffn_logits(gate: *const CmlWeight, up: *const CmlWeight, down: *const CmlWeight, n_experts: i32, k: i32,
                              logits_dev: *const f32, x_dev: *const f32, n_tokens: i64, out_dev: *mut f32, workspace_dev: *mut c_void,
                              workspace_bytes: usize, stream: Stream) -> i32;
    pub fn cml_moe_plan(idx_dev: *const i32, n_tokens: i64, k: i32, n_experts: i32, token_offsets_dev: *mut i32, token_ids_dev: *mut i32,
                        route_to_assignment_dev: *mut i32, union_experts_dev: *mut i32, stream: Stream) -> i32;
    pub fn cml_moe_gemv_routed(experts: *const CmlWeight, n_experts: i32, q_dev: *const i8, scales_dev: *const f32,
                               token_offsets_dev: *const i32, token_ids_dev: *const i32, union_experts_dev: *const i32, max_union: i32,
                               max_assignments_per_expert: i64, out_dev: *mut f32, stream: Stream) -> i32;
    pub fn cml_moe_weighted_sum(y_dev: *const f32, route_to_assignment_dev: *const i32, weight_dev: *const f32, n_tokens: i64, k: i32,
                                hidden: i64, out_dev: *mut f32, stream: Stream) -> i32;
    // ---- host-side helpers and the host-pointer seams
    pub fn cml_quantize_weights_host(fmt: i32, src: *const f32, n_values: usize, dst: *mut u8, threads: i32) -> i32;
    pub fn cml_try_linear_rows(fmt: i32, input_scales: *const f32, input_quants: *const i8, weight_wire: *const u8, weight_nbytes: usize,
                               input_rows: i64, weight_rows: i64, cols: i64, output: *mut f32) -> i32;
    pub fn cml_try_q8_0_block_linear_row(input_scales: *const f32, input_quants: *const i8, weight_block_bytes: *const u8,
                                         weight_nbytes: usize, rows: i64, blocks_per_row: i64, output: *mut f32) -> i32;
}

// ---- gating ---------------------------------------------------------------------------------------

/// Once per process: is there a usable gfx950 device that the environment does not mask, and did
/// the library initialise on it?  (Reference: `gpu_accel_enabled`, `devices_masked_by_env`,
/// `src/cuda.rs:167, 206`; the backend `OnceLock`, `:691-699`.)  `CAMELID_HIP=0` switches the
/// lane off; `cml_available` checks that and the `*_VISIBLE_DEVICES` masks before touching the
/// driver.  The `CAMELID_HIP_*` tuning knobs are read here, once.
pub fn available() -> bool {
    static READY: OnceLock<bool> = OnceLock::new();
    *READY.get_or_init(|| unsafe { cml_available() == 1 && cml_init(-1) == CML_OK })
}

/// Matvec / matmul launches this process has completed on the device (reference
/// `cuda_q8_run_count`, `src/cuda.rs:346-358`): zero means the lane never ran.
pub fn hip_run_count() -> u64 {
    unsafe { cml_run_count() }
}

/// Launches of the kernel families whose dotted counter name starts with `prefix`
/// (e.g. `"q4k.dot.wg8"`, `"q4k.mfma."`): what a test reads before and after a call to prove which
/// kernel served it (reference: the engaged counters of `src/inference.rs:23740, 24596-24603`).
pub fn kernel_launches(prefix: &str) -> u64 {
    match std::ffi::CString::new(prefix) {
        Ok(p) => unsafe { cml_kernel_launches(p.as_ptr()) },
        Err(_) => 0,
    }
}

pub fn last_error() -> String {
    unsafe {
        let p = cml_last_error();
        if p.is_null() {
            String::new()
        } else {
            std::ffi::CStr::from_ptr(p).to_string_lossy().into_owned()
        }
    }
}

// ---- the three host-pointer seams of src/cuda.rs --------------------------------------------------
//
// Same names, arguments and `bool` convention as the CUDA lane's; the caller adds
// `|| hip::try_…(…)` next to the existing call (src/inference.rs:27938-27955).  Weight slices must
// outlive the process-wide device cache entry keyed by their address, the contract the CUDA seam
// already has (src/cuda.rs:1158-1168).

/// Decode-shaped Q8_0 linear over 34-byte wire blocks: one input row against `rows` weight rows.
pub fn try_q8_0_encoded_linear_row(
    input_scales: &[f32], input_quants: &[i8], weight_bytes: &[u8], weight_scales: &[f32],
    rows: usize, blocks_per_row: usize, output: &mut [f32],
) -> bool {
    try_q8_0_encoded_linear_rows(input_scales, input_quants, weight_bytes, weight_scales, 1, rows, blocks_per_row, output)
}

/// Prefill-shaped Q8_0 linear (`input_rows` x `weight_rows`), token-major output.
/// The shape guards are the reference's (`src/cuda.rs:953-966`), `weight_scales` included: the
/// library does not need that slice (the 34-byte blocks carry their f16 scales), but a caller
/// that passes a wrong one has a bug the CUDA lane would also have refused.
pub fn try_q8_0_encoded_linear_rows(
    input_scales: &[f32], input_quants: &[i8], weight_bytes: &[u8], weight_scales: &[f32],
    input_rows: usize, weight_rows: usize, blocks_per_row: usize, output: &mut [f32],
) -> bool {
    if input_rows == 0 || weight_rows == 0 || blocks_per_row == 0 {
        return false;
    }
    if input_scales.len() != input_rows * blocks_per_row
        || input_quants.len() != input_rows * blocks_per_row * 32
        || weight_bytes.len() != weight_rows * blocks_per_row * 34
        || weight_scales.len() != weight_rows * blocks_per_row
        || output.len() != input_rows * weight_rows
    {
        return false;
    }
    if !available() {
        return false;
    }
    unsafe {
        cml_try_linear_rows(
            CML_Q8_0, input_scales.as_ptr(), input_quants.as_ptr(), weight_bytes.as_ptr(), weight_bytes.len(),
            input_rows as i64, weight_rows as i64, (blocks_per_row * 32) as i64, output.as_mut_ptr(),
        ) == CML_OK
    }
}

/// Decode-shaped Q8_0 linear over the in-memory `Q8_0Block` layout (36 bytes per block: f32 scale +
/// 32 i8), the call at `src/inference.rs:27944`.  Guards as in `run_block` (`src/cuda.rs:1089-1110`).
pub fn try_q8_0_block_linear_row(
    input_scales: &[f32], input_quants: &[i8], weight_block_bytes: &[u8],
    rows: usize, blocks_per_row: usize, output: &mut [f32],
) -> bool {
    if rows == 0 || blocks_per_row == 0 {
        return false;
    }
    if input_scales.len() != blocks_per_row
        || input_quants.len() != blocks_per_row * 32
        || weight_block_bytes.len() != rows * blocks_per_row * 36
        || output.len() != rows
    {
        return false;
    }
    if !available() {
        return false;
    }
    unsafe {
        cml_try_q8_0_block_linear_row(
            input_scales.as_ptr(), input_quants.as_ptr(), weight_block_bytes.as_ptr(), weight_block_bytes.len(),
            rows as i64, blocks_per_row as i64, output.as_mut_ptr(),
        ) == CML_OK
    }
}

// ---- device memory --------------------------------------------------------------------------------

/// A device allocation owned by this process (freed on drop).
pub struct DeviceBuffer {
    ptr: *mut c_void,
    bytes: usize,
}
unsafe impl Send for DeviceBuffer {}

impl DeviceBuffer {
    pub fn new(bytes: usize) -> Option<Self> {
        let mut ptr = core::ptr::null_mut();
        let rc = unsafe { cml_dev_alloc(bytes.max(16), &mut ptr) };
        (rc == CML_OK && !ptr.is_null()).then_some(Self { ptr, bytes: bytes.max(16) })
    }
    pub fn from_slice<T: Copy>(src: &[T]) -> Option<Self> {
        let buf = Self::new(core::mem::size_of_val(src))?;
        buf.upload(src).then_some(buf)
    }
    pub fn upload<T: Copy>(&self, src: &[T]) -> bool {
        let n = core::mem::size_of_val(src);
        n <= self.bytes && unsafe { cml_memcpy_h2d(self.ptr, src.as_ptr() as *const c_void, n, core::ptr::null_mut()) } == CML_OK
    }
    pub fn download<T: Copy>(&self, dst: &mut [T]) -> bool {
        let n = core::mem::size_of_val(dst);
        n <= self.bytes && unsafe { cml_memcpy_d2h(dst.as_mut_ptr() as *mut c_void, self.ptr, n, core::ptr::null_mut()) } == CML_OK
    }
    pub fn ptr(&self) -> *mut c_void {
        self.ptr
    }
    pub fn bytes(&self) -> usize {
        self.bytes
    }
}
impl Drop for DeviceBuffer {
    fn drop(&mut self) {
        unsafe { cml_dev_free(self.ptr) };
    }
}

// ---- the operator API: WireQuant on the device -------------------------------------------------------

/// The wire formats of this path (`WireFormat`, `src/gemma4_runtime.rs:609-647`, restricted to
/// the four the library serves; the others stay on the CPU lane).
#[derive(Clone, Copy, PartialEq, Eq, Debug)]
pub enum HipWireFormat {
    Q8_0,
    Q4_0,
    Q4K,
    Q6K,
}
impl HipWireFormat {
    pub fn ggml_type(self) -> i32 {
        match self {
            Self::Q8_0 => CML_Q8_0,
            Self::Q4_0 => CML_Q4_0,
            Self::Q4K => CML_Q4_K,
            Self::Q6K => CML_Q6_K,
        }
    }
    pub fn values_per_block(self) -> usize {
        match self {
            Self::Q8_0 | Self::Q4_0 => 32,
            Self::Q4K | Self::Q6K => 256,
        }
    }
    pub fn block_bytes(self) -> usize {
        match self {
            Self::Q8_0 => 34,
            Self::Q4_0 => 18,
            Self::Q4K => 144,
            Self::Q6K => 210,
        }
    }
}

struct Scratch {
    x: DeviceBuffer,
    out: DeviceBuffer,
    workspace: DeviceBuffer,
}

/// A weight resident in HBM with `WireQuant`'s methods.  `None` from any method means "not
/// handled": the caller continues on its CPU path, exactly as it does when the CUDA lane
/// declines (`src/inference.rs:16377-16380`).
pub struct HipWireQuant {
    w: *mut CmlWeight,
    format: HipWireFormat,
    rows: usize,
    cols: usize,
    scratch: Mutex<Option<Scratch>>,
    bands: Mutex<HashMap<(usize, usize), usize>>, // (row_start, rows) -> *mut CmlWeight of the cached band view
}
unsafe impl Send for HipWireQuant {}
unsafe impl Sync for HipWireQuant {}

impl HipWireQuant {
    /// Mirrors `WireQuant::from_wire`: row-major wire bytes `[rows][cols / blk]` blocks, uploaded
    /// once (and re-laid on the device, losslessly) and kept resident.
    pub fn from_wire(format: HipWireFormat, bytes: &[u8], rows: usize, cols: usize) -> Option<Self> {
        if cols % format.values_per_block() != 0 || bytes.len() != rows * (cols / format.values_per_block()) * format.block_bytes() {
            return None;
        }
        if !available() {
            return None;
        }
        let mut w = core::ptr::null_mut();
        let rc = unsafe {
            cml_weight_upload(format.ggml_type(), rows as i64, cols as i64, bytes.as_ptr() as *const c_void, bytes.len(), &mut w)
        };
        (rc == CML_OK && !w.is_null()).then(|| Self {
            w,
            format,
            rows,
            cols,
            scratch: Mutex::new(None),
            bands: Mutex::new(HashMap::new()),
        })
    }

    pub fn out_dim(&self) -> usize {
        self.rows
    }
    pub fn in_dim(&self) -> usize {
        self.cols
    }

    fn run(&self, w: *const CmlWeight, w_rows: usize, x: &[f32], k_tokens: usize) -> Option<Vec<f32>> {
        if k_tokens == 0 || x.len() != k_tokens * self.cols {
            return None;
        }
        let ws_bytes = unsafe { cml_matmul_workspace_bytes(self.format.ggml_type(), self.cols as i64, k_tokens as i64) };
        let mut guard = self.scratch.lock().ok()?;
        let need_x = x.len() * 4;
        let need_out = k_tokens * w_rows * 4;
        let fits = guard.as_ref().map_or(false, |s| s.x.bytes() >= need_x && s.out.bytes() >= need_out && s.workspace.bytes() >= ws_bytes);
        if !fits {
            *guard = Some(Scratch {
                x: DeviceBuffer::new(need_x)?,
                out: DeviceBuffer::new(need_out)?,
                workspace: DeviceBuffer::new(ws_bytes)?,
            });
        }
        let s = guard.as_ref()?;
        if !s.x.upload(x) {
            return None;
        }
        let rc = unsafe {
            cml_matmul_f32(w, s.x.ptr() as *const f32, k_tokens as i64, s.out.ptr() as *mut f32, s.workspace.ptr(), s.workspace.bytes(),
                           core::ptr::null_mut())
        };
        if rc != CML_OK {
            return None;
        }
        let mut out = vec![0.0f32; k_tokens * w_rows];
        s.out.download(&mut out).then_some(out) // the download synchronises the stream
    }

    /// `WireQuant::matvec` (`src/gemma4_runtime.rs:826-851`): one activation row, quantized on the
    /// device to the weight's family (Q8_0 or Q8_K) exactly as the CPU lane quantizes it.
    pub fn matvec(&self, in_dim: usize, out_dim: usize, x: &[f32]) -> Option<Vec<f32>> {
        if in_dim != self.cols || out_dim != self.rows {
            return None;
        }
        self.run(self.w, self.rows, x, 1)
    }

    /// `WireQuant::matmul_proj` (`:1040-1082`): K activation rows, output `out[k][o]` token-major,
    /// every cell bit-identical to the single-token call.
    pub fn matmul_proj(&self, out_dim: usize, x: &[f32], k_tokens: usize) -> Option<Vec<f32>> {
        if out_dim != self.rows {
            return None;
        }
        self.run(self.w, self.rows, x, k_tokens)
    }

    /// `WireQuant::matvec_rows_proj` (`:1084-1110`): the row band `[row_start, row_start + rows)`
    /// (an expert of a stacked tensor); bit-identical to the same rows of the full matvec.
    pub fn matvec_rows_proj(&self, x: &[f32], row_start: usize, rows: usize) -> Option<Vec<f32>> {
        if rows == 0 || row_start + rows > self.rows {
            return None;
        }
        let band = {
            let mut bands = self.bands.lock().ok()?;
            match bands.get(&(row_start, rows)) {
                Some(&p) => p as *mut CmlWeight,
                None => {
                    let mut view = core::ptr::null_mut();
                    if unsafe { cml_weight_slice(self.w, row_start as i64, rows as i64, &mut view) } != CML_OK || view.is_null() {
                        return None;
                    }
                    bands.insert((row_start, rows), view as usize);
                    view
                }
            }
        };
        self.run(band, rows, x, 1)
    }

    /// `WireQuant::dequantize_elements` (`:1112-1150`, embedding rows): f32 values of the flat
    /// element range `[start, start + len)`, decoded on the device with the reference's block
    /// arithmetic.
    pub fn dequantize_elements(&self, start: usize, len: usize) -> Option<Vec<f32>> {
        if len == 0 || start + len > self.rows * self.cols {
            return None;
        }
        let (row0, row1) = (start / self.cols, (start + len - 1) / self.cols + 1);
        let mut view = core::ptr::null_mut();
        if unsafe { cml_weight_slice(self.w, row0 as i64, (row1 - row0) as i64, &mut view) } != CML_OK {
            return None;
        }
        let n = (row1 - row0) * self.cols;
        let result = (|| {
            let out = DeviceBuffer::new(n * 4)?;
            if unsafe { cml_dequantize(view, out.ptr() as *mut f32, core::ptr::null_mut()) } != CML_OK {
                return None;
            }
            let mut host = vec![0.0f32; n];
            out.download(&mut host).then_some(())?;
            let off = start - row0 * self.cols;
            Some(host[off..off + len].to_vec())
        })();
        unsafe { cml_weight_free(view) };
        result
    }
}

impl Drop for HipWireQuant {
    fn drop(&mut self) {
        if let Ok(bands) = self.bands.lock() {
            for &p in bands.values() {
                unsafe { cml_weight_free(p as *mut CmlWeight) };
            }
        }
        unsafe { cml_weight_free(self.w) };
    }
}

/// Gate and up of a dense FFN off one activation (`ffn_gate` / `ffn_up` on one `SharedActivation`,
/// `src/gemma4_runtime.rs:5591-5592`): one launch for two weights of one shape.
pub fn matvec_pair(gate: &HipWireQuant, up: &HipWireQuant, x: &[f32]) -> Option<(Vec<f32>, Vec<f32>)> {
    if gate.cols != up.cols || gate.format != up.format || x.len() != gate.cols {
        return None;
    }
    let ws_bytes = unsafe { cml_matmul_workspace_bytes(gate.format.ggml_type(), gate.cols as i64, 1) };
    let xd = DeviceBuffer::from_slice(x)?;
    let (oa, ob, ws) = (DeviceBuffer::new(gate.rows * 4)?, DeviceBuffer::new(up.rows * 4)?, DeviceBuffer::new(ws_bytes)?);
    let rc = unsafe {
        cml_matmul_f32_pair(gate.w, up.w, xd.ptr() as *const f32, oa.ptr() as *mut f32, ob.ptr() as *mut f32, ws.ptr(), ws.bytes(),
                            core::ptr::null_mut())
    };
    if rc != CML_OK {
        return None;
    }
    let (mut a, mut b) = (vec![0.0f32; gate.rows], vec![0.0f32; up.rows]);
    (oa.download(&mut a) && ob.download(&mut b)).then_some((a, b))
}
