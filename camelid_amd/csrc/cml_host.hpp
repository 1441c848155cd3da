// Host-side internals of libcamelid_hip: status/last-error plumbing, the
// weight handle, and the launcher prototypes each kernel file implements.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

#include <atomic>
#include <string>

#include "../../include/camelid_hip.h"

namespace cml {

// Records the message for cml_last_error() and returns `code`.
int fail(int code, const char *fmt, ...) __attribute__((format(printf, 2, 3)));
void clear_error();
bool ready();  // cml_init succeeded and the device is current

#define CML_HIP_TRY(expr)                                                                  \
    do {                                                                                   \
        hipError_t e_ = (expr);                                                            \
        if (e_ != hipSuccess) {                                                            \
            return ::cml::fail(e_ == hipErrorOutOfMemory ? CML_ERR_OOM : CML_ERR_HIP,      \
                               "%s failed: %s", #expr, hipGetErrorString(e_));             \
        }                                                                                  \
    } while (0)

inline hipStream_t as_stream(cml_stream_t s) { return reinterpret_cast<hipStream_t>(s); }

// Which kernel family served a call (reference: the engaged counters its tests read to prove that a
// dispatch fired, src/inference.rs:23740, 24596-24603; src/cuda.rs:346-358).  Every launcher counts
// under a dotted name, "<format>.<family>[.<variant>...]"; cml_kernel_launches(prefix) sums the
// counters whose names start with the prefix.  One relaxed atomic add per launch.
struct LaunchCounter {
    const char *name;
    std::atomic<uint64_t> n{0};
    LaunchCounter *next = nullptr;
    explicit LaunchCounter(const char *nm);         // links itself into the registry; nm must outlive the process (a literal)
    explicit LaunchCounter(const std::string &nm);  // the same for a name built at the first launch (kept for good)
};
// name_ may be any expression (evaluated once, at the site's first launch)
#define CML_COUNT_LAUNCH(name_)                               \
    do {                                                      \
        static ::cml::LaunchCounter cml_counter_(name_);      \
        cml_counter_.n.fetch_add(1, std::memory_order_relaxed); \
    } while (0)

struct Geometry {
    int block_values;
    int block_bytes;
};
Geometry geometry(int fmt);  // {0,0} for unknown formats
inline bool is_k_family(int fmt) { return fmt == CML_Q4_K || fmt == CML_Q6_K; }

// Device layout of a weight.  Q4_K: one plane, the wire blocks.  The other
// formats: per-field planes, each indexed by absolute row of the allocation
// that owns them.  plane[i] already points at this handle's first row.
struct Planes {
    const uint8_t *p[4];
    int64_t row_stride[4];  // bytes per row in each plane
};

}  // namespace cml

struct cml_weight {
    int fmt;
    int64_t rows, cols, nb;  // nb = blocks per row
    cml::Planes planes;
    int row_skip;      // Q4_K views that start inside a 16-row tile: rows of the first tile that precede the view (else 0)
    void *allocation;  // non-null only for the owning handle
    size_t allocation_bytes;
};


namespace cml {

// Plane sizes for `rows` rows; returns the number of planes.
int plane_layout(int fmt, int64_t rows, int64_t nb, int64_t stride[4], size_t offset[4], size_t *total);

// weight_quantize.cpp: 36-byte in-memory Q8_0 blocks (f32 scale + 32 int8) -> 34-byte wire blocks; false if a scale is not an f16 value
bool q8_0_blocks_to_wire(const uint8_t *blocks, size_t n_blocks, uint8_t *wire);

// ---- launchers (one per kernel file) ------------------------------------------------------------

// quantize.hip
int launch_quantize_q8_0(const float *x, int64_t n_tokens, int64_t cols, int8_t *q, float *s, hipStream_t st);
int launch_quantize_q8_k(const float *x, int64_t n_tokens, int64_t cols, int8_t *q, float *d, hipStream_t st);

int launch_rms_inv_norm_quantize(int act, const float *x, const float *weight, float rms_inv, int64_t cols, int8_t *q, float *scales, hipStream_t st);

// producers.hip: act = 0 (f32 only), 1 (Q8_0), 2 (Q8_K)
int launch_rms_norm_quantize(int act, const float *x, const float *weight, float eps, int64_t n_tokens, int64_t cols,
                             float *normed, int8_t *q, float *scales, hipStream_t st);
int launch_glu_quantize(int glu, int act, const float *g, const float *u, int64_t n_tokens, int64_t cols, int64_t in_stride,
                        int8_t *q, float *scales, hipStream_t st);  // glu: 0 = silu, 1 = gelu_tanh
int launch_silu_mul_quantize(int act, const float *g, const float *u, int64_t n_tokens, int64_t cols, int8_t *q, float *scales,
                             hipStream_t st);

// layout.hip: wire <-> planes, dequantize
int launch_wire_to_planes(int fmt, const uint8_t *wire, int64_t rows, int64_t nb, const Planes &dst, hipStream_t st);
int launch_planes_to_wire(int fmt, const Planes &src, int64_t rows, int64_t nb, int row_skip, uint8_t *wire, hipStream_t st);
int launch_dequantize(const cml_weight *w, float *out, hipStream_t st);
int launch_embed_gather(const cml_weight *table, const uint32_t *token_ids, int64_t n_tokens, float *out, hipStream_t st);
int launch_argmax_f32(const float *logits, int64_t n_rows, int64_t n, uint32_t *out_idx, hipStream_t st);

// Arguments common to every gemv/gemm launcher.
struct MatArgs {
    const cml_weight *w;
    const int8_t *q;      // activation rows [*][cols]
    const float *scales;  // [*][nb]
    int64_t n_tokens;     // plain: activation rows; grouped: the most assignments one group can hold
    float *out;           // [*][rows]
    const float *residual;  // plain single-token calls only, may be null
    int32_t *ints;          // block-int diagnostics, may be null (plain single token only)
    // Grouped (mixture-of-experts) extension; null/zero for plain calls.  The
    // grid gets one y-slot per group (expert) e, which owns the band of rows
    // [e*band_rows, (e+1)*band_rows) of the stacked weight and the
    // assignments [group_offsets[e], group_offsets[e+1]); assignment j dots
    // activation row group_rows[j] (j itself when null) and writes out[j][band_rows].
    const int32_t *group_offsets;  // device, [n_groups + 1]
    const int32_t *group_rows;     // device, [assignments] or null
    // Optional compaction of the grid: group_ids[y] is the group that y-slot y serves, the groups
    // that hold assignments first, -1 in the slots after them; the grid then has max_active
    // y-slots (at least the number of groups that can be non-empty) instead of n_groups.
    const int32_t *group_ids;      // device, [n_groups] or null
    int max_active;
    int64_t n_assign_total;        // all assignments of a grouped call (0 = unknown): sizes the expected group
    int n_groups;
    int64_t band_rows;
    // Grouped Q4_K matrix-core calls only: a second stacked weight of the same shape against the same
    // activations, its cells to out2, in the same launch (gate and up of an expert layer).
    const cml_weight *w2;
    float *out2;
    // Direct Q4_K decode launch only: route the token inside the launch (Mixtral routing of the
    // n_groups logits, top route_k), y-slot = routed rank; experts and weights in routed order are
    // left in route_idx / route_w.  Null = the caller has routed (group_ids).
    const float *route_logits;
    int route_k;
    int32_t *route_idx;
    float *route_w;
};

int launch_gemv_q4k(const MatArgs &a, hipStream_t st);
// quantize + matvec for two stacked expert weights of one shape in one launch; a.q / a.scales unused, x = f32 rows
int launch_gemv_q4k_f32_grouped_pair(const MatArgs &a, const cml_weight *w2, float *out2, const float *x, hipStream_t st);
int launch_gemv_q4k_f32_pair(const cml_weight *w, const cml_weight *w2, const float *x, float *out, float *out2, hipStream_t st);
bool gemv_q6k_long_rows_fuse(const cml_weight *w);
bool gemv_b32_long_rows_fuse(const cml_weight *w);  // the same for Q8_0 / Q4_0 rows of more than 8192 values  // the same for Q6_K
bool gemv_q4k_long_rows_fuse(const cml_weight *w, int n_tokens = 1);  // a single f32 token on this weight is one launch although its rows exceed 8192 values
int launch_gemv_q4k_f32_multi(const cml_weight *const *ws, int n, const float *x, float *const *outs, hipStream_t st);  // -1: not served
// whether that launch, as a direct call on these two weights, can route the token itself (a.route_logits)
bool gemv_q4k_direct_can_route(const cml_weight *w, int64_t band_rows, int n_slots, bool pair);

int launch_gemv_q4k_f32(const cml_weight *w, const float *x, float *out, hipStream_t st, int n_tokens = 1);  // quantize + matvec, one or two tokens
int launch_gemm_q4k_mfma_f32(const cml_weight *w, const float *x, int64_t n_tokens, float *out, hipStream_t st);  // 3..8 tokens, quantize inside; -1: not served
// MoE decode: the routed experts' Q4_K down projections and the weighted sum in one launch; -1: shape not served
int launch_moe_down_sum_q4k(const cml_weight *down, int n_experts, int n_slots, const int32_t *idx, const float *weight, const int8_t *q,
                            const float *yd, float *out, hipStream_t st);
int launch_gemv_q4k_loads_only(const cml_weight *w, float *out, hipStream_t st);  // calibration: the single-token launch's loads alone
int launch_gemv_q4k_ablated(const cml_weight *w, const float *x, float *out, int mask, hipStream_t st);  // calibration: parts of the launch taken out
int launch_gemv_q6k_f32(const cml_weight *w, const float *x, float *out, hipStream_t st, int n_tokens = 1);  // Q6_K: quantize + matvec, one or two tokens
int launch_gemv_b32_f32(const cml_weight *w, const float *x, float *out, hipStream_t st, int n_tokens = 1);
int launch_gemv_b32_f32_multi(const cml_weight *const *ws, int n, const float *x, float *const *outs, hipStream_t st);  // -1 = not served
int launch_gemv_q6k_f32_multi(const cml_weight *const *ws, int n, const float *x, float *const *outs, hipStream_t st);  // -1 = not served  // quantize + matvec, one or two tokens
int launch_gemv_b32_f32_pair(const cml_weight *w, const cml_weight *w2, const float *x, float *out, float *out2, hipStream_t st);  // -1: not served
// Where a grouped matvec takes its activation rows from instead of MatArgs::q / scales:
//   kind 1: ONE f32 token x, quantized inside the kernel, read by every assignment
//   kind 2 / 3: assignment j's row is silu / gelu_tanh of x[j] times u[j] (f32 rows `stride` apart), quantized in the kernel
struct GroupedPrologue {
    int kind = 0;
    const float *x = nullptr;
    const float *u = nullptr;
    int64_t stride = 0;
};
// Q8_0 / Q4_0 grouped (mixture-of-experts) matvec
int launch_gemv_b32_grouped(const MatArgs &a, const GroupedPrologue &pro, hipStream_t st);
int launch_gemv_q8_0(const MatArgs &a, hipStream_t st);
int launch_gemv_q4_0(const MatArgs &a, hipStream_t st);
int launch_gemv_q6k(const MatArgs &a, hipStream_t st);

int launch_gemm_q4k(const MatArgs &a, hipStream_t st);
int launch_gemm_q4k_mfma(const MatArgs &a, hipStream_t st);  // plain calls, n_tokens >= 16
int launch_gemm_b32_mfma(const MatArgs &a, hipStream_t st);  // Q8_0 / Q4_0 on the matrix cores; plain or grouped
bool b32_mfma_usable(const cml_weight *w);                   // rows of whole 256-value slabs
int b32_mfma_min_tokens(int64_t rows);                       // batch size from which it pays
int launch_gemm_q8_0(const MatArgs &a, hipStream_t st);
int launch_gemm_q4_0(const MatArgs &a, hipStream_t st);
int launch_gemm_q6k(const MatArgs &a, hipStream_t st);
int launch_gemm_q6k_mfma(const MatArgs &a, hipStream_t st);  // Q6_K on the matrix cores; plain or grouped
int q6k_mfma_min_tokens(int64_t rows, int64_t n_sb);         // batch size from which it pays
bool q4k_lane_order();                                       // CAMELID_HIP_Q4K_LANE_ORDER: the reference wire row dot's generic 8-lane order, bit for bit
bool q6k_lane_order();                                       // CAMELID_HIP_Q6K_LANE_ORDER: the reference CPU lanes' 8-lane order, bit for bit

// Integer tuning knob read once from the environment (0 when unset).
int env_int(const char *name, int dflt);

}  // namespace cml
