/*
 * camelid_hip.h -- C ABI of the MI355X (gfx950) quantized matvec / small-batch
 * matmul backend for GGUF block formats Q8_0, Q4_0, Q4_K and Q6_K.
 *
 * This is the boundary a host engine binds over FFI.  It replaces, for this
 * one path, the device back end of the reference engine:
 *   - the per-matmul "try" seam that takes host slices and returns whether the
 *     device handled the call (reference src/cuda.rs:276-319, real
 *     implementation :1044-1218), and
 *   - the resident operator API that keeps weights on the device and
 *     dispatches quantize / gemv / batched gemm / routed expert kernels
 *     (reference src/cuda_resident.rs:9838 repack_for_lane, :9935
 *     launch_quantize, :11761 launch_quantize_q8k, :11370 dispatch_gemv,
 *     :11550 dispatch_gemm_batched, :12215-12508 routed launchers,
 *     :16133 set_layer_located).
 *
 * Conventions (the reference's, src/cuda.rs:257-345 and :1044-1218):
 *   - every entry point returns an int status: 0 = handled, non-zero = not
 *     handled, the caller keeps its own fallback; nothing aborts or throws
 *     across this boundary; cml_last_error() describes the last failure of the
 *     calling thread;
 *   - plain pointers and sizes only; host buffers stay owned by the caller;
 *     device buffers created here are freed through the matching call here;
 *   - all pointers named *_dev are device addresses on the initialised GPU;
 *   - `stream` is a hipStream_t passed as void* (NULL = the default stream);
 *     calls only enqueue work, except where a host pointer is read or written;
 *   - one GPU; no collectives;
 *   - threads: the host-slice seam (cml_try_*) serialises its callers on one
 *     process-wide lock, as the reference's backend does (src/cuda.rs:691-699).
 *     The resident entry points (quantize / gemv / gemm / matmul / moe / producers)
 *     take no lock: they only enqueue kernels on the caller's stream; what they
 *     share is atomic (the launch counters, and one flag per kernel that needs
 *     more than 64 KB of LDS, set the first time it is launched) -- and the static
 *     array of cml_matmul_f32_static, see there -- so any number of threads may
 *     call them, each on its own stream, on weights that nobody frees meanwhile.  cml_init / cml_shutdown / cml_reload_env must not
 *     run concurrently with anything else;
 *   - knobs (environment variables named CAMELID_HIP_*) are read once, by
 *     cml_init, the way the reference reads its CAMELID_* knobs once per process
 *     (src/inference.rs:23679-23692); cml_reload_env() reads them again.  Four
 *     are always honoured because they choose what is computed or where:
 *     CAMELID_HIP_DEVICE, CAMELID_HIP_EXACT_ORDER, CAMELID_HIP_Q4K_LANE_ORDER,
 *     CAMELID_HIP_Q6K_LANE_ORDER.  All others choose among kernels that give the
 *     same bits (launch shapes, ring depths, thresholds: the switches of this
 *     library's tests and measurements) and are ignored unless
 *     CAMELID_HIP_TUNING=1 is set as well.
 *
 * Tensor conventions (reference src/tensor/mod.rs:79-89, src/inference.rs:
 * 23728-23749): a weight is `rows` output rows of `cols` contraction values,
 * row-major in whole blocks; row o occupies wire bytes
 * [o*row_bytes, (o+1)*row_bytes) with row_bytes = cols/block_values*block_bytes.
 * Activations: int8 quants q[n_tokens*cols], f32 scales s[n_tokens*cols/32]
 * (Q8_0 family) or s[n_tokens*cols/256] (Q8_K, for Q4_K/Q6_K weights), token
 * major.  Outputs: f32 out[t*rows + row] (reference src/cuda_resident.rs:4442).
 */
#ifndef CAMELID_HIP_H
#define CAMELID_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Weight formats: the GGUF tensor type ids (reference src/gguf/reader.rs:94-127). */
#define CML_Q4_0 2
#define CML_Q8_0 8
#define CML_Q4_K 12
#define CML_Q6_K 14

/* Status codes. */
#define CML_OK 0
#define CML_ERR_UNAVAILABLE 1 /* no usable GPU / not initialised / masked by env */
#define CML_ERR_INVALID 2     /* null pointer, bad format id, bad flag */
#define CML_ERR_SHAPE 3       /* sizes do not fit the format or each other */
#define CML_ERR_HIP 4         /* a HIP runtime call failed */
#define CML_ERR_OOM 5         /* device allocation failed */
#define CML_ERR_UNSUPPORTED 6 /* valid request this build does not serve */

typedef struct cml_weight cml_weight; /* opaque device-resident weight */
typedef void *cml_stream_t;           /* hipStream_t */
typedef void *cml_event_t;            /* hipEvent_t */
typedef void *cml_graph_t;            /* an instantiated hipGraphExec_t */

/* ---- lifecycle (reference src/cuda.rs:167-236, :691-699, :350-358) ------- */

/* 1 when a gfx950 device can be used.  Honours HIP_VISIBLE_DEVICES /
 * ROCR_VISIBLE_DEVICES / CAMELID_HIP=0 masking before touching the driver
 * (reference devices_masked_by_env, src/cuda.rs:206-218). */
int cml_available(void);
/* Select the device (CAMELID_HIP_DEVICE overrides when device < 0). Idempotent. */
int cml_init(int device);
/* Frees what the library itself holds on the device (the seam's weight cache and
 * staging buffer); handles and buffers the caller created stay the caller's to
 * free, before or after (cml_weight_free, cml_dev_free). */
void cml_shutdown(void);
/* Takes a new snapshot of the CAMELID_HIP_* environment variables (tests change
 * them between calls; a production host never needs this). */
int cml_reload_env(void);
/* Message for the last non-zero status returned to this thread ("" if none). */
const char *cml_last_error(void);
/* Number of gemv/gemm launches completed by this process: proves the device
 * lane ran (reference cuda_q8_run_count, src/cuda.rs:350-358). */
uint64_t cml_run_count(void);
/* Launches, by kernel family, since the library was loaded: the sum of the counters whose dotted
 * name starts with `prefix` (null or "" = all).  Names are "<format>.<family>[.<variant>...]",
 * e.g. "q4k.dot.wg8", "q4k.dot.ring.fused", "q4k.mfma.pair", "q8_0.mfma.kpar", "q6k.lanes",
 * "moe.plan": a test (or a host) reads the counter before and after a call to prove WHICH kernel
 * served it -- several kernels give the same bits, so results alone cannot (reference: the
 * engaged counters of src/inference.rs:23740, 24596-24603 and the test that reads them,
 * src/inference/tests.rs:7158-7196; cuda_q8_run_count, src/cuda.rs:346-358).
 * cml_kernel_launch_report writes "name count" lines for every counter that has fired into buf
 * (at most cap bytes, always terminated) and returns the size the whole report needs. */
uint64_t cml_kernel_launches(const char *prefix);
size_t cml_kernel_launch_report(char *buf, size_t cap);
/* Block geometry helpers: 0 for an unknown format. */
int cml_block_values(int fmt);
int cml_block_bytes(int fmt);

/* ---- device memory plumbing for hosts without their own HIP bindings ----- */
int cml_dev_alloc(size_t nbytes, void **out_dev);
int cml_dev_free(void *ptr_dev);
int cml_memcpy_h2d(void *dst_dev, const void *src_host, size_t nbytes, cml_stream_t stream);
int cml_memcpy_d2h(void *dst_host, const void *src_dev, size_t nbytes, cml_stream_t stream);
int cml_memset_dev(void *dst_dev, int value, size_t nbytes, cml_stream_t stream);
int cml_stream_sync(cml_stream_t stream);
/* Streams (default priority), timing events and captured launch sequences, for
 * hosts that drive a decode loop through this library alone.  The reference's
 * resident engine owns one stream, syncs once per token and may replay a
 * captured graph (src/cuda_resident.rs:15195-15205); these are the pieces for
 * the same pattern.  Every matvec / matmul / quantize / mixture-of-experts entry
 * point may be captured; uploads, downloads, cml_memset_dev and cml_block_dots may not. */
int cml_stream_create(cml_stream_t *out);
int cml_stream_destroy(cml_stream_t stream);
int cml_event_create(cml_event_t *out);
int cml_event_record(cml_event_t event, cml_stream_t stream);
/* Waits for `stop`, then returns the milliseconds between the two events. */
int cml_event_elapsed_ms(cml_event_t start, cml_event_t stop, float *ms);
int cml_event_destroy(cml_event_t event);
int cml_graph_begin_capture(cml_stream_t stream);
int cml_graph_end_capture(cml_stream_t stream, cml_graph_t *out);
int cml_graph_launch(cml_graph_t graph, cml_stream_t stream);
int cml_graph_destroy(cml_graph_t graph);

/* ---- weights (reference repack_for_lane + set_layer_located,
 *      src/cuda_resident.rs:9838, :16133-16253) ---------------------------- */

/* Copy `nbytes` of GGUF wire bytes (host memory) to the device, re-laid at load
 * time so that every device load is a naturally aligned 128-bit load:
 *  - Q8_0, Q4_0, Q6_K: per-field planes of exactly the wire size
 *    (quants | scales, or ql | qh | scales | d);
 *  - Q4_K: super-block major, tiles of 16 rows; a tile is 2304 bytes =
 *    16 x 16 header bytes (d, dmin, scales) then the 16 rows' nibbles
 *    interleaved in 16-byte pieces, so one wave reads whole 1 KB runs.  The
 *    last tile of a weight whose row count is not a multiple of 16 is padded
 *    with zero blocks (device size = ceil(rows/16)*16 rows).
 * Both are pure permutations of the wire bytes: cml_weight_download returns the
 * original bytes (cf. the reference's lossless repacks,
 * src/cuda_resident.rs:9741-9753, :9878-9911). */
int cml_weight_upload(int fmt, int64_t rows, int64_t cols, const void *wire_host, size_t nbytes,
                      cml_weight **out);
/* Same, from wire bytes that already live in device memory. */
int cml_weight_upload_dev(int fmt, int64_t rows, int64_t cols, const void *wire_dev, size_t nbytes,
                          cml_stream_t stream, cml_weight **out);
/* A view of rows [row_start, row_start+rows) of `parent`: the expert band of a
 * stacked expert tensor (reference matvec_q8k_rows, src/gemma4_runtime.rs:
 * 1084-1110).  Any row range is accepted; the mixture-of-experts entry points
 * additionally need Q4_K bands that are whole 16-row tiles.  The parent must
 * outlive the view. */
int cml_weight_slice(const cml_weight *parent, int64_t row_start, int64_t rows, cml_weight **out);
int cml_weight_info(const cml_weight *w, int *fmt, int64_t *rows, int64_t *cols, size_t *wire_bytes);
/* Reconstruct the GGUF wire bytes of `w` (a view yields its rows only). */
int cml_weight_download(const cml_weight *w, void *wire_host, size_t nbytes);
void cml_weight_free(cml_weight *w);

/* ---- activation quantizers (reference quantize_q8_0_block,
 *      src/inference.rs:22510-22528; quantize_q8_k_blocks, :23121-23152;
 *      device lane launch_quantize / launch_quantize_q8k,
 *      src/cuda_resident.rs:9935, :11761) ---------------------------------- */
int cml_quantize_q8_0(const float *x_dev, int64_t n_tokens, int64_t cols, int8_t *q_dev,
                      float *scales_dev, cml_stream_t stream);
int cml_quantize_q8_k(const float *x_dev, int64_t n_tokens, int64_t cols, int8_t *q_dev,
                      float *d_dev, cml_stream_t stream);

/* ---- fused producers: the step upstream of a projection, quantizing as it goes.
 *      act selects the activation format: CML_ACT_F32 (no quantized output),
 *      CML_ACT_Q8_0 (scales per 32 values) or CML_ACT_Q8_K (per 256). -------- */
enum { CML_ACT_F32 = 0, CML_ACT_Q8_0 = 1, CML_ACT_Q8_K = 2 };
/* RMS norm of every row (reference CpuTensor::rms_norm_into, src/tensor/mod.rs:
 * 2707-2760: squares summed left to right in f32, scale = 1/sqrt(mean + eps),
 * out = (x*scale)*weight), then the quantizer above on the normalised row
 * (reference rms_norm_quantize / rms_norm_quantize_q8k, src/cuda_resident.rs:
 * 236-270, :4152-4177).  normed_dev (f32[n_tokens*cols]) may be null when only
 * the quantized form is wanted; q_dev/scales_dev are ignored for CML_ACT_F32.
 * Rows of up to 16384 values. */
int cml_rms_norm_quantize(int act, const float *x_dev, const float *weight_dev, float eps,
                          int64_t n_tokens, int64_t cols, float *normed_dev, int8_t *q_dev,
                          float *scales_dev, cml_stream_t stream);
/* The same norm with the inverse root-mean-square supplied by the host (reference
 * rms_inv_norm_quantize_q8_0 / _q8k, src/cuda_resident.rs:272-315, 4272-4291: the CPU router has
 * already scanned the row and hands over its exact sequential (mean_square + eps)^-0.5): one row,
 * value[i] = (x[i] * rms_inv) * weight[i], each multiply rounded, then the quantizer above.
 * act is CML_ACT_Q8_0 (cols a multiple of 32) or CML_ACT_Q8_K (a multiple of 256). */
int cml_rms_inv_norm_quantize(int act, const float *x_dev, const float *weight_dev, float rms_inv,
                              int64_t cols, int8_t *q_dev, float *scales_dev, cml_stream_t stream);
/* The first pass of the norm on its own: out_dev[r] = (((0 + x[r][0]^2) + x[r][1]^2) + ...) in f32,
 * every product and every sum rounded, in index order -- the bits of the scalar
 * loop (reference rms_norm's ordered sum, src/cuda_resident.rs:124-131;
 * src/tensor/mod.rs:2707-2760), computed in parallel.  cols a multiple of 4, up
 * to 16384. */
int cml_sum_squares_f32(const float *x_dev, int64_t n_rows, int64_t cols, float *out_dev,
                        cml_stream_t stream);
/* silu(gate) * up = (g / (1 + exp(-g))) * u per element (reference
 * CpuTensor::silu_mul, src/tensor/mod.rs:2610-2634), quantized (reference
 * silu_mul_quantize / _q8k, src/cuda_resident.rs:4289-4341).  act must be
 * CML_ACT_Q8_0 or CML_ACT_Q8_K. */
int cml_silu_mul_quantize(int act, const float *gate_dev, const float *up_dev, int64_t n_tokens,
                          int64_t cols, int8_t *q_dev, float *scales_dev, cml_stream_t stream);
/* The same with the expert activation named: CML_GLU_SILU as above, or
 * CML_GLU_GELU_TANH: (0.5*g*(1 + tanh(0.7978846*(g + 0.044715*g*g*g)))) * u,
 * evaluated left to right (reference gelu_tanh, src/gemma4_mtp.rs:172-175; the
 * Gemma-4 expert activation, src/gemma4_runtime.rs:5689-5691; device lane
 * geglu_quantize_routed, src/cuda_resident.rs:6301-6343). */
enum { CML_GLU_SILU = 0, CML_GLU_GELU_TANH = 1 };
int cml_glu_quantize(int glu, int act, const float *gate_dev, const float *up_dev, int64_t n_tokens,
                     int64_t cols, int8_t *q_dev, float *scales_dev, cml_stream_t stream);

/* ---- dequantize (reference Q4KBlock::dequantize & siblings,
 *      src/tensor/mod.rs:5365-5409, :5547-5572, :5903-5924, :6039-6066) ----- */
/* out_dev: f32[rows*cols], bit-identical to the reference decoders. */
int cml_dequantize(const cml_weight *w, float *out_dev, cml_stream_t stream);

/* ---- either side of the largest matvec (the output projection) ------------- */
/* Dequantizes rows token_ids[0..n_tokens) of an embedding table into
 * out_dev f32[n_tokens*cols]; the ids are read on the device, e.g. straight
 * from cml_argmax_f32 (reference embed_gather_q4k / _q6k / _q8_0,
 * src/cuda_resident.rs:8248-8383: element for element the block decode of
 * cml_dequantize).  An id outside the table yields a row of NaNs. */
int cml_embed_gather(const cml_weight *table, const uint32_t *token_ids_dev, int64_t n_tokens,
                     float *out_dev, cml_stream_t stream);
/* Greedy pick per row of logits_dev f32[n_rows*n]: strict >, the first index
 * wins ties, scanning from (-3.4e38, index 0) (reference argmax_f32,
 * src/cuda_resident.rs:6391-6417).  out_idx_dev u32[n_rows]. */
int cml_argmax_f32(const float *logits_dev, int64_t n_rows, int64_t n, uint32_t *out_idx_dev,
                   cml_stream_t stream);

/* ---- matvec / small-batch matmul (reference dispatch_gemv,
 *      src/cuda_resident.rs:11370; dispatch_gemm_batched, :11550; CPU
 *      semantics WireQuant::matvec_q / matvec_q8k / matmul_q / matmul_q8k,
 *      src/gemma4_runtime.rs:922-1150) ------------------------------------- */
/* One activation row.  residual_dev may be NULL; when given,
 * out[row] = dot + residual[row] (reference q8_gemv fused residual,
 * src/cuda_resident.rs:334-413). */
int cml_gemv(const cml_weight *w, const int8_t *q_dev, const float *scales_dev, float *out_dev,
             const float *residual_dev, cml_stream_t stream);
/* Accumulation order of cml_gemv / cml_gemm / cml_matmul_f32 (every path gives the
 * same bits for one weight, whatever the token count):
 *   Q8_0, Q4_0: the reference's block-order chain, always (src/inference.rs:22729-22798).
 *   Q4_K: the fused per-super-block chain of q4_k_dot_arm (src/diffusion_gemma/
 *         refmath.rs:504-562).  By default a weight with few row tiles and long rows
 *         (an FFN down projection, e.g. 4096 x 14336) has its K range cut into 2 / 4 / 8
 *         parts whose partial chains are added left to right: within 1e-5 (typically
 *         1e-7) of the reference chain, not its bits.  CAMELID_HIP_EXACT_ORDER=1
 *         forbids the cut: then every Q4_K result is the reference chain bit for bit.
 *         The other Q4_K order of the reference, the generic 8-lane one of
 *         q4_k_wire_row_dot (src/inference.rs:25806-25889, the Gemma-4 wire lane), is
 *         matched within 1e-5 by default and bit for bit under
 *         CAMELID_HIP_Q4K_LANE_ORDER=1 (plain calls; slower).
 *   Q6_K: the fused chain of q6_k_dot_arm (refmath.rs:678-721), K cut as for Q4_K;
 *         within 1e-5 of the 8-lane order of q6_k_wire_row_dot (src/inference.rs:
 *         25535-25581), which CAMELID_HIP_Q6K_LANE_ORDER=1 reproduces bit for bit
 *         (plain calls; slower). */
/* n_tokens activation rows; out_dev[t*rows + row].  A few tokens run on the
 * packed-dot kernel (up to 8 per pass over the weight), larger batches on the
 * int8 matrix cores (all four formats; Q8_0 / Q4_0 rows must be whole multiples
 * of 256 values for that, other lengths stay on the packed-dot kernel).  Every
 * cell equals the cml_gemv result for that token bit for bit. */
int cml_gemm(const cml_weight *w, const int8_t *q_dev, const float *scales_dev, int64_t n_tokens,
             float *out_dev, cml_stream_t stream);
/* The exact per-block integer dot products of cml_gemv, for parity checks:
 * Q8_0/Q4_0 int32[rows][cols/32]; Q4_K int32[rows][cols/256][2] =
 * {sum_g sc_g*dot_g, sum_g m_g*bsum_g}; Q6_K int32[rows][cols/256]. */
int cml_block_dots(const cml_weight *w, const int8_t *q_dev, int32_t *ints_dev, cml_stream_t stream);

/* f32 activations in, f32 out: quantize (Q8_0 or Q8_K by weight family) into
 * the caller's workspace, then gemv/gemm (reference WireQuant::matvec,
 * src/gemma4_runtime.rs:826-856).  workspace_dev needs
 * cml_matmul_workspace_bytes(fmt, cols, n_tokens) bytes.  Calls with one or two
 * tokens on short rows, and Q4_K calls with three to six tokens on rows of up
 * to 4096 values, quantize inside the product kernel (one launch, the
 * workspace is left untouched); the result bits do not depend on which way ran. */
size_t cml_matmul_workspace_bytes(int fmt, int64_t cols, int64_t n_tokens);
int cml_matmul_f32(const cml_weight *w, const float *x_dev, int64_t n_tokens, float *out_dev,
                   void *workspace_dev, size_t workspace_bytes, cml_stream_t stream);

/* cml_matmul_f32 for ONE token against TWO weights that read the same
 * activation -- the gate and up projections of a dense FFN, which the reference
 * runs as two matvecs on one shared quantized activation (SharedActivation,
 * src/gemma4_runtime.rs:1288-1340; gate / up at :5591-5592 and :5965-5966).
 * Two weights of one shape run as ONE launch (the token quantized once per
 * workgroup, both weights streamed) for Q4_K rows of up to 8192 values and for
 * Q8_0 / Q4_0 matrices of 4096 to 32768 rows of up to 4096 values where the
 * single call runs eight-wave workgroups with 16 lanes per row (the launcher
 * decides: not, for one, Q8_0 rows of 4096 values on 14336 rows or more, which
 * run sixteen-wave workgroups); every other pair is two cml_matmul_f32 calls.
 * Same bits as the two calls.  workspace as for cml_matmul_f32 with n_tokens = 1. */
int cml_matmul_f32_pair(const cml_weight *w_a, const cml_weight *w_b, const float *x_dev,
                        float *out_a_dev, float *out_b_dev, void *workspace_dev,
                        size_t workspace_bytes, cml_stream_t stream);

/* cml_matmul_f32 without a workspace argument, for callers that cannot allocate
 * device memory (a stream under HIP graph capture, a serving loop with a fixed
 * memory budget, a harness that forbids hipMalloc).  It has no counterpart in
 * the reference.  The quantized activation rows are staged in a static device
 * array of CML_STATIC_WORKSPACE_BYTES that the library holds on every GPU it is
 * initialised on until the process ends; the call allocates and frees nothing.
 * A call whose staging (cml_matmul_workspace_bytes(fmt, cols, n_tokens)) exceeds
 * that size returns CML_ERR_SHAPE.  Every call on one GPU shares the one array:
 * calls that overlap on one GPU (two streams, two threads) race on it; calls on
 * one stream do not.  Results are the bits of cml_matmul_f32. */
/* One token against n weights that read it (the q, k and v projections of an attention block,
 * gate and up of an FFN -- the projections the reference runs off one SharedActivation,
 * src/gemma4_runtime.rs:1288-1340; the per-layer dispatch_gemv calls of the device lane,
 * src/cuda_resident.rs:18161-19525): outs_dev[j][rows_j] = weights[j] x.  All weights read rows of
 * the same length; runs of up to four Q4_K or Q6_K weights whose shapes take the same K cut, and of
 * up to four Q8_0 or Q4_0 weights, go out as ONE launch (their workgroups end to end, the token quantized
 * once per workgroup), everything else as calls of its own.  The bits of n cml_matmul_f32 calls either way.  workspace as for
 * cml_matmul_f32 with one token.  weights / outs_dev are host arrays of n pointers. */
int cml_matmul_f32_multi(const cml_weight *const *weights, int n_weights, const float *x_dev,
                         float *const *outs_dev, void *workspace_dev, size_t workspace_bytes,
                         cml_stream_t stream);
#define CML_STATIC_WORKSPACE_BYTES (1024 * 1024 + 128 * 1024)
int cml_matmul_f32_static(const cml_weight *w, const float *x_dev, int64_t n_tokens, float *out_dev,
                          cml_stream_t stream);

/* ---- mixture of experts (reference softmax_top_k, src/inference.rs:
 *      13940-13991; mixtral_moe_ffn, :14142-14280; routed launchers,
 *      src/cuda_resident.rs:12215-12508; moe_weighted_sum_*, :6347-6389) ---- */
/* Mixtral routing on the device: for each token the top-k experts by logit
 * (ties to the lower index), softmax over the selected, renormalised, sorted
 * by weight.  idx_dev int32[n_tokens*k], weight_dev f32[n_tokens*k]. */
int cml_moe_route_top_k(const float *logits_dev, int64_t n_tokens, int n_experts, int k,
                        int32_t *idx_dev, float *weight_dev, cml_stream_t stream);
/* Gemma-4 routing on the device (reference moe_layer_ffn, src/gemma4_runtime.rs:
 * 5567-5610; router_top_k, :61-84): softmax over ALL experts, the k most
 * probable (ties to the lower index), weight = down_scale[e] * (p[e] /
 * max(sum of the selected p, 6.103515e-5)) in selection order.  down_scale_dev
 * f32[n_experts] may be null (= 1).  Up to 128 experts. */
int cml_moe_route_softmax_top_k(const float *logits_dev, int64_t n_tokens, int n_experts, int k,
                                const float *down_scale_dev, int32_t *idx_dev, float *weight_dev,
                                cml_stream_t stream);
/* Whole expert FFN for quantized stacked experts: gate/up hold n_experts*ff
 * rows of `hidden` values, down holds n_experts*hidden rows of `ff` values.
 * For every token, in routed order: y = down_e(silu(gate_e x) * up_e x),
 * out += y * weight.  Tokens that share an expert are grouped so each touched
 * expert matrix is streamed once.  x_dev/out_dev: f32[n_tokens*hidden];
 * idx/weight as produced by cml_moe_route_top_k.  workspace_dev needs
 * cml_moe_workspace_bytes(...) bytes. */
size_t cml_moe_workspace_bytes(int fmt, int64_t hidden, int64_t ff, int64_t n_tokens, int k,
                               int n_experts);
int cml_moe_ffn(const cml_weight *gate, const cml_weight *up, const cml_weight *down, int n_experts,
                int k, const int32_t *idx_dev, const float *weight_dev, const float *x_dev,
                int64_t n_tokens, float *out_dev, void *workspace_dev, size_t workspace_bytes,
                cml_stream_t stream);

/* The same with the expert activation named (CML_GLU_SILU / CML_GLU_GELU_TANH)
 * and, when up == NULL, with `gate` holding fused gate|up experts of 2*ff rows
 * each, gate rows first (the Gemma-4 lane's gate_up_exps, reference
 * src/gemma4_runtime.rs:5676-5691): one projection launch instead of two. */
int cml_moe_ffn_ex(const cml_weight *gate, const cml_weight *up, const cml_weight *down, int n_experts,
                   int k, const int32_t *idx_dev, const float *weight_dev, const float *x_dev,
                   int64_t n_tokens, float *out_dev, void *workspace_dev, size_t workspace_bytes,
                   int glu, cml_stream_t stream);

/* cml_moe_route_top_k and cml_moe_ffn as one call: logits_dev f32[n_tokens *
 * n_experts] are the router's outputs (what the reference's mixtral_moe_ffn
 * has after its router projection, src/inference.rs:14168-14172; routing and
 * expert lane :14173-14280).  Same results, bit for bit, as the two calls.  One
 * token on Q4_K experts with rows of 4096 values is routed inside the gate|up
 * launch (three launches per layer instead of four); every other shape runs
 * the routing launch first.  The routed experts and weights are kept in the
 * workspace. */
int cml_moe_ffn_logits(const cml_weight *gate, const cml_weight *up, const cml_weight *down,
                       int n_experts, int k, const float *logits_dev, const float *x_dev,
                       int64_t n_tokens, float *out_dev, void *workspace_dev, size_t workspace_bytes,
                       cml_stream_t stream);

/* The pieces cml_moe_ffn is made of, for callers that schedule the expert
 * lane themselves.
 * cml_moe_plan groups the n_tokens*k routed slots by expert, keeping (token,
 * rank) order inside each group (reference gemma4_plan_route_union,
 * src/gemma4_runtime.rs:12309-12424): token_offsets_dev int32[n_experts+1]
 * (CSR over expert ids), token_ids_dev int32[n_tokens*k] (assignment -> token),
 * route_to_assignment_dev int32[n_tokens*k] (slot t*k+s -> assignment; -1 for
 * an expert id out of range), union_experts_dev int32[n_experts] (the experts
 * in use, ascending, then -1). */
int cml_moe_plan(const int32_t *idx_dev, int64_t n_tokens, int k, int n_experts,
                 int32_t *token_offsets_dev, int32_t *token_ids_dev,
                 int32_t *route_to_assignment_dev, int32_t *union_experts_dev, cml_stream_t stream);
/* Expert-grouped matvec on quantized activations (reference
 * launch_q4_wire_gemm_routed, src/cuda_resident.rs:12215-12313): `experts`
 * stacks n_experts bands of rows/n_experts rows; assignment j of expert e (j in
 * [token_offsets[e], token_offsets[e+1])) dots band e with activation row
 * token_ids[j] (j itself when token_ids_dev is null) and writes
 * out_dev[j][band rows].  Activations are Q8_K for Q4_K experts, Q8_0 for Q8_0 /
 * Q4_0 (cml_quantize_*).  union_experts_dev (nullable) compacts the launch to
 * max_union grid slots; max_assignments_per_expert bounds any one group. */
int cml_moe_gemv_routed(const cml_weight *experts, int n_experts, const int8_t *q_dev,
                        const float *scales_dev, const int32_t *token_offsets_dev,
                        const int32_t *token_ids_dev, const int32_t *union_experts_dev, int max_union,
                        int64_t max_assignments_per_expert, float *out_dev, cml_stream_t stream);
/* out[t][c] = sum over s in routed order of y[route_to_assignment[t*k+s]][c] *
 * weight[t*k+s], multiply and add rounded separately (reference
 * moe_weighted_sum_batched, src/cuda_resident.rs:6369-6389; CPU accumulate,
 * src/inference.rs:14255-14257).  route_to_assignment_dev null = identity. */
int cml_moe_weighted_sum(const float *y_dev, const int32_t *route_to_assignment_dev,
                         const float *weight_dev, int64_t n_tokens, int k, int64_t hidden,
                         float *out_dev, cml_stream_t stream);

/* ---- weight quantizer tool (reference quantize_block_q8_0 / q4_0 / q4_k,
 *      src/quantize.rs:98-244): f32 values -> GGUF wire bytes on the host, in
 *      whole blocks, on `threads` threads.  Q6_K has no counterpart in the
 *      reference; its encoder here only produces valid super-blocks. -------- */
int cml_quantize_weights_host(int fmt, const float *src, size_t n_values, uint8_t *dst, int threads);

/* ---- host-slice seam (reference try_q8_0_encoded_linear_rows,
 *      src/cuda.rs:1044-1218): everything in host memory, synchronous.
 *      Returns 0 when the device produced `output`, non-zero when the caller
 *      must run its CPU path.  Weights are cached on the device keyed by
 *      (pointer, length), so they must stay alive and unchanged. ------------ */
/* The reference signature also passes `weight_scales: &[f32]` (src/cuda.rs:1044-1052,
 * the f16 scales of weight_bytes widened by the caller); the wire bytes already hold
 * them, so a binding drops that slice, and passes the format id the reference leaves
 * implicit (its seam is Q8_0 only; this one takes all four formats). */
int cml_try_linear_rows(int fmt, const float *input_scales, const int8_t *input_quants,
                        const uint8_t *weight_wire, size_t weight_nbytes, int64_t input_rows,
                        int64_t weight_rows, int64_t cols, float *output);
/* The seam the reference's CPU linear consults on its decode path (reference
 * try_q8_0_block_linear_row, src/cuda.rs:1089-1222; call site
 * src/inference.rs:27939-27955): one input row against `rows` weight rows held
 * as in-memory Q8_0Block values, 36 bytes each = f32 scale + 32 int8
 * (src/tensor/mod.rs:105-110); weight_nbytes must be rows*blocks_per_row*36.
 * The blocks are converted to wire form once per (pointer, length) and cached
 * on the device; a scale that is not an f16 value (blocks that were not decoded
 * from Q8_0 wire bytes) makes the call decline.  Same return convention. */
int cml_try_q8_0_block_linear_row(const float *input_scales, const int8_t *input_quants,
                                  const uint8_t *weight_block_bytes, size_t weight_nbytes,
                                  int64_t rows, int64_t blocks_per_row, float *output);

/* ==== Diagnostics: measurement yardsticks of bench.py ==========================================
 * None of these has a counterpart in the reference and a production host never calls them:
 * they exist so that the roofline reading of the matvec kernels (bench.py: roofline.shape_ceiling,
 * --calibrate-copy, --calibrate-read) rests on launches anybody can re-run, not on constants.
 * They share the library's launch path and may be captured into graphs; they change no state. */
/* Device-to-device streaming copy by a plain kernel (16-byte aligned pointers and
 * size; may be captured).  Also the yardstick bench.py reads byte counters and
 * matvec bandwidth against: it moves nbytes in, nbytes out and nothing else. */
int cml_copy_dev(void *dst_dev, const void *src_dev, size_t nbytes, cml_stream_t stream);
/* Two more yardsticks for the roofline reading of the matvec kernels (bench.py --calibrate-read /
 * roofline.shape_ceiling); neither has a counterpart in the reference.
 * cml_calibrate_read: a launch that only READS nbytes (16-byte aligned), every lane keeping
 * in_flight (1, 2, 4 or 8) 16-byte non-temporal loads out over a grid-stride walk with `workgroups`
 * workgroups of 256 lanes (0 = 2048), and stores nothing.
 * cml_calibrate_weight_loads: the plain single-token Q4_K matvec launch for `w` -- same grid, same
 * lane addresses, same load instructions and register buffers -- with the activation, the
 * arithmetic and the stores taken out (scratch_dev: 4 writable bytes, never written in practice).
 * What these two take for a weight's bytes is what the SHAPE allows a single launch on this chip;
 * what the real kernel takes beyond that is the kernel's own cost. */
int cml_calibrate_read(const void *src_dev, size_t nbytes, int in_flight, int workgroups, cml_stream_t stream);
int cml_calibrate_weight_loads(const cml_weight *w, void *scratch_dev, cml_stream_t stream);
/* cml_calibrate_matvec_ablation: the single-token Q4_K launch of cml_matmul_f32 for `w` with parts
 * taken out, to time what each part costs: mask 1 = no activation (no f32 loads, no quantizer, no
 * barrier), 4 = no output store, 7 = the weight requests alone.  Served for rows of 4096 values on
 * 12288 to 16384 rows (the eight-wave launch) and for rows of 14336 values on 3072 to 6128 rows (its
 * eight-wave K-cut form, which is also what cml_matmul_f32 launches up to 4096 rows; beyond it launches
 * twelve-wave workgroups); CML_ERR_UNSUPPORTED otherwise.  out_dev must hold w's rows and is garbage afterwards. */
int cml_calibrate_matvec_ablation(const cml_weight *w, const float *x_dev, float *out_dev, int mask, cml_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif
