// Mixture-of-experts dispatch for quantized stacked experts.
//
// What the reference does per token (mixtral_moe_ffn, src/inference.rs:14142-14280):
// route (softmax_top_k, :13940-13991), then for every selected expert in routed
// order  y = down_e( silu(gate_e x) * up_e x )  and  out += y * weight.
// The device version keeps that arithmetic per (token, expert) cell and only
// changes the schedule: assignments are grouped by expert (the reference's
// expert-grouped plan for K-token batches, Gemma4RouteUnionPlan,
// src/gemma4_runtime.rs:12309-12424), so each touched expert matrix is streamed
// once for all the tokens routed to it, and the weighted sum walks each token's
// experts in router order (moe_weighted_sum_batched, src/cuda_resident.rs:6369-6389).
// Nothing here synchronises with the host: the grouping is built on the device
// and the expert kernels are launched over all experts, idle ones exiting at once.
#include "cml_device.hpp"
#include "cml_host.hpp"

#pragma clang fp contract(off)

namespace cml {

constexpr int kMaxExperts = 128;

// f32::total_cmp as an integer key (larger key = greater value).
__device__ __forceinline__ int total_key(float v) {
    const int b = __builtin_bit_cast(int, v);
    return b ^ static_cast<int>(static_cast<unsigned>(b >> 31) >> 1);
}

// One thread per token.  reference softmax_top_k, src/inference.rs:13940-13991.
__global__ __launch_bounds__(64) void moe_route_kernel(const float *__restrict__ logits, int64_t n_tokens, int n_experts,
                                                       int k, int32_t *__restrict__ idx_out, float *__restrict__ w_out) {
    const int64_t t = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (t >= n_tokens) return;
    const float *lg = logits + t * n_experts;
    int sel_idx[kMaxExperts];
    float sel_w[kMaxExperts];
    unsigned long long taken[2] = {0, 0};
    // top-k by logit (total order, descending), ties to the lower index
    for (int s = 0; s < k; s++) {
        int best = -1, best_key = 0;
        for (int e = 0; e < n_experts; e++) {
            if ((taken[e >> 6] >> (e & 63)) & 1ull) continue;
            const int key = total_key(lg[e]);
            if (best < 0 || key > best_key) {
                best = e;
                best_key = key;
            }
        }
        taken[best >> 6] |= 1ull << (best & 63);
        sel_idx[s] = best;
        sel_w[s] = lg[best];
    }
    float mx = -INFINITY;
    for (int s = 0; s < k; s++) mx = fmaxf(mx, sel_w[s]);
    float sum = 0.0f;
    for (int s = 0; s < k; s++) {
        const float v = sel_w[s];
        const float wv = (fabsf(v) < INFINITY) ? expf(v - mx) : 0.0f;  // is_finite: NaN and inf give 0
        sel_w[s] = wv;
        sum = sum + wv;
    }
    if (sum > 0.0f) {
        for (int s = 0; s < k; s++) sel_w[s] = sel_w[s] / sum;
    } else {
        const float uniform = 1.0f / static_cast<float>(k);
        for (int s = 0; s < k; s++) sel_w[s] = uniform;
    }
    // re-sort by weight (descending), ties to the lower index: insertion sort, stable
    for (int i = 1; i < k; i++) {
        const int ci = sel_idx[i];
        const float cw = sel_w[i];
        const int ck = total_key(cw);
        int j = i - 1;
        while (j >= 0) {
            const int kj = total_key(sel_w[j]);
            const bool before = (ck > kj) || (ck == kj && ci < sel_idx[j]);
            if (!before) break;
            sel_idx[j + 1] = sel_idx[j];
            sel_w[j + 1] = sel_w[j];
            j--;
        }
        sel_idx[j + 1] = ci;
        sel_w[j + 1] = cw;
    }
    for (int s = 0; s < k; s++) {
        idx_out[t * k + s] = sel_idx[s];
        w_out[t * k + s] = sel_w[s];
    }
}

// One thread per token.  Gemma-4 routing (reference moe_layer_ffn, src/gemma4_runtime.rs:5567-5610;
// router_top_k, :61-84): softmax over ALL experts (max folded from f32::MIN, exp(v - max), sum in
// index order, p /= sum), top-k by probability (descending, ties to the lower index), then
// scale[s] = down_scale[e] * (p[e] / max(sum of the selected p in selection order, 6.103515e-5)).
__global__ __launch_bounds__(64) void moe_route_softmax_kernel(const float *__restrict__ logits, int64_t n_tokens, int n_experts,
                                                               int k, const float *__restrict__ down_scale,
                                                               int32_t *__restrict__ idx_out, float *__restrict__ w_out) {
    const int64_t t = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (t >= n_tokens) return;
    const float *lg = logits + t * n_experts;
    float p[kMaxExperts];
    int sel[kMaxExperts];
    float maxl = -3.4028235e38f;
    for (int e = 0; e < n_experts; e++) maxl = fmaxf(maxl, lg[e]);
    float sum = 0.0f;
    for (int e = 0; e < n_experts; e++) {
        p[e] = expf(lg[e] - maxl);
        sum = sum + p[e];
    }
    for (int e = 0; e < n_experts; e++) p[e] = p[e] / sum;
    int len = 0;
    for (int c = 0; c < n_experts; c++) {
        int at = -1;
        for (int j = 0; j < len; j++) {
            const int cur = sel[j];
            if (p[cur] < p[c] || (p[cur] == p[c] && c < cur)) {
                at = j;
                break;
            }
        }
        if (at >= 0) {
            const int last = len < k ? len : k - 1;
            for (int j = last; j > at; j--) sel[j] = sel[j - 1];
            sel[at] = c;
            if (len < k) len++;
        } else if (len < k) {
            sel[len++] = c;
        }
    }
    float wsum = 0.0f;
    for (int s = 0; s < k; s++) wsum = wsum + p[sel[s]];
    wsum = fmaxf(wsum, 6.103515e-5f);
    for (int s = 0; s < k; s++) {
        const int e = sel[s];
        const float ds = down_scale ? down_scale[e] : 1.0f;
        idx_out[t * k + s] = e;
        w_out[t * k + s] = ds * (p[e] / wsum);
    }
}

// Group the n_tokens*k assignments by expert, keeping (token, rank) order
// inside each group.  One workgroup; thread e builds group e.
//   offsets[e..e+1)   assignment range of expert e
//   assign_token[j]   token whose activation assignment j reads
//   slot_to_assign[t*k+s]  where (token t, rank s) landed
__global__ __launch_bounds__(kMaxExperts) void moe_plan_kernel(const int32_t *__restrict__ idx, int n_slots, int n_experts, int k,
                                                      int32_t *__restrict__ offsets, int32_t *__restrict__ assign_token,
                                                      int32_t *__restrict__ slot_to_assign) {
    __shared__ int count[kMaxExperts + 1];
    const int e = threadIdx.x;
    int mine = 0;
    if (e < n_experts) {
        for (int i = 0; i < n_slots; i++) mine += (idx[i] == e);
        count[e] = mine;
    }
    __syncthreads();
    if (e < n_experts) {
        int start = 0;
        for (int j = 0; j < e; j++) start += count[j];
        offsets[e] = start;
        if (e == n_experts - 1) offsets[n_experts] = start + mine;
        int at = start;
        for (int i = 0; i < n_slots; i++) {
            if (idx[i] == e) {
                assign_token[at] = i / k;
                slot_to_assign[i] = at;
                at++;
            }
        }
    }
}

// Expert-grouped matmul: the packed-dot kernel for a few tokens, the matrix cores from 4 tokens
// up (the same crossover as for plain calls).  Both produce the same bits per cell.
static int launch_expert_matmul(const MatArgs &a, hipStream_t st) {
    if (a.w->fmt != CML_Q4_K) return launch_gemv_b32_grouped(a, nullptr, st);
    if (a.n_tokens >= env_int("CAMELID_HIP_Q4K_MFMA_MIN_TOKENS", 4)) return launch_gemm_q4k_mfma(a, st);
    return launch_gemv_q4k(a, st);
}

static bool expert_format(int fmt) { return fmt == CML_Q4_K || fmt == CML_Q8_0 || fmt == CML_Q4_0; }
// Activation quantization an expert matrix of this format is dotted with: 2 = Q8_K, 1 = Q8_0.
static int act_of(int fmt) { return fmt == CML_Q4_K ? 2 : 1; }
static int launch_quantize_act(int act, const float *x, int64_t n, int64_t cols, int8_t *q, float *s, hipStream_t st) {
    return act == 2 ? launch_quantize_q8_k(x, n, cols, q, s, st) : launch_quantize_q8_0(x, n, cols, q, s, st);
}

// out[t][c] = ((0 + y[a(t,0)][c]*w[t][0]) + y[a(t,1)][c]*w[t][1]) + ...  (reference
// src/inference.rs:14255-14257: `output += expert_out * weight`, routed order,
// multiply and add rounded separately).
__global__ __launch_bounds__(256) void moe_weighted_sum_kernel(const float *__restrict__ y, const int32_t *__restrict__ slot_to_assign,
                                                               const float *__restrict__ weight, int k, int64_t hidden,
                                                               float *__restrict__ out) {
    const int64_t c = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    const int64_t t = blockIdx.y;
    if (c >= hidden) return;
    float acc = 0.0f;
    for (int s = 0; s < k; s++) {
        const int64_t a = slot_to_assign[t * k + s];
        acc = acc + y[a * hidden + c] * weight[t * k + s];
    }
    out[t * hidden + c] = acc;
}

struct MoeWorkspace {
    int8_t *xq;
    float *xd;
    int32_t *offsets, *assign_token, *slot_to_assign;
    float *g, *u, *y, *hd;
    int8_t *hq;
    size_t total;
};

static MoeWorkspace carve(void *base, int64_t hidden, int64_t ff, int64_t n_tokens, int k, int n_experts) {
    MoeWorkspace w;
    size_t at = 0;
    auto take = [&](size_t bytes) {
        const size_t here = at;
        at += (bytes + 255) & ~size_t(255);
        return base ? static_cast<uint8_t *>(base) + here : nullptr;
    };
    const size_t T = static_cast<size_t>(n_tokens), A = T * static_cast<size_t>(k);
    w.xq = reinterpret_cast<int8_t *>(take(T * hidden));
    // scale arrays are sized for 32-value blocks, the finest any expert format uses
    w.xd = reinterpret_cast<float *>(take(T * ((hidden + 31) / 32) * 4));
    w.offsets = reinterpret_cast<int32_t *>(take((static_cast<size_t>(n_experts) + 1) * 4));
    w.assign_token = reinterpret_cast<int32_t *>(take(A * 4));
    w.slot_to_assign = reinterpret_cast<int32_t *>(take(A * 4));
    w.g = reinterpret_cast<float *>(take(A * ff * 4));
    w.u = reinterpret_cast<float *>(take(A * ff * 4));
    w.hq = reinterpret_cast<int8_t *>(take(A * ff));
    w.hd = reinterpret_cast<float *>(take(A * ((ff + 31) / 32) * 4));
    w.y = reinterpret_cast<float *>(take(A * hidden * 4));
    w.total = at;
    return w;
}

}  // namespace cml

using namespace cml;

extern "C" {

int cml_moe_route_top_k(const float *logits_dev, int64_t n_tokens, int n_experts, int k, int32_t *idx_dev,
                        float *weight_dev, cml_stream_t stream) {
    if (!ready()) return fail(CML_ERR_UNAVAILABLE, "cml_init has not succeeded");
    if (n_tokens < 0 || n_experts <= 0 || k <= 0) return fail(CML_ERR_SHAPE, "bad routing shape");
    if (n_experts > kMaxExperts) return fail(CML_ERR_UNSUPPORTED, "at most %d experts", kMaxExperts);
    if (k > n_experts) return fail(CML_ERR_SHAPE, "top-%d of %d experts", k, n_experts);
    if (n_tokens == 0) return CML_OK;
    if (!logits_dev || !idx_dev || !weight_dev) return fail(CML_ERR_INVALID, "null pointer");
    const unsigned grid = static_cast<unsigned>((n_tokens + 63) / 64);
    hipLaunchKernelGGL(moe_route_kernel, dim3(grid), dim3(64), 0, as_stream(stream), logits_dev, n_tokens, n_experts, k, idx_dev, weight_dev);
    CML_HIP_TRY(hipGetLastError());
    return CML_OK;
}

int cml_moe_route_softmax_top_k(const float *logits_dev, int64_t n_tokens, int n_experts, int k, const float *down_scale_dev,
                                int32_t *idx_dev, float *weight_dev, cml_stream_t stream) {
    if (!ready()) return fail(CML_ERR_UNAVAILABLE, "cml_init has not succeeded");
    if (n_tokens < 0 || n_experts <= 0 || k <= 0) return fail(CML_ERR_SHAPE, "bad routing shape");
    if (n_experts > kMaxExperts) return fail(CML_ERR_UNSUPPORTED, "at most %d experts", kMaxExperts);
    if (k > n_experts) return fail(CML_ERR_SHAPE, "top-%d of %d experts", k, n_experts);
    if (n_tokens == 0) return CML_OK;
    if (!logits_dev || !idx_dev || !weight_dev) return fail(CML_ERR_INVALID, "null pointer");
    const unsigned grid = static_cast<unsigned>((n_tokens + 63) / 64);
    hipLaunchKernelGGL(moe_route_softmax_kernel, dim3(grid), dim3(64), 0, as_stream(stream), logits_dev, n_tokens, n_experts, k,
                       down_scale_dev, idx_dev, weight_dev);
    CML_HIP_TRY(hipGetLastError());
    return CML_OK;
}

size_t cml_moe_workspace_bytes(int fmt, int64_t hidden, int64_t ff, int64_t n_tokens, int k, int n_experts) {
    if (!expert_format(fmt) || hidden <= 0 || ff <= 0 || n_tokens <= 0 || k <= 0 || n_experts <= 0) return 0;
    return carve(nullptr, hidden, ff, n_tokens, k, n_experts).total;
}

int cml_moe_ffn(const cml_weight *gate, const cml_weight *up, const cml_weight *down, int n_experts, int k,
                const int32_t *idx_dev, const float *weight_dev, const float *x_dev, int64_t n_tokens, float *out_dev,
                void *workspace_dev, size_t workspace_bytes, cml_stream_t stream) {
    if (!up) return fail(CML_ERR_INVALID, "null weight");
    return cml_moe_ffn_ex(gate, up, down, n_experts, k, idx_dev, weight_dev, x_dev, n_tokens, out_dev, workspace_dev, workspace_bytes,
                          CML_GLU_SILU, stream);
}

int cml_moe_ffn_ex(const cml_weight *gate, const cml_weight *up, const cml_weight *down, int n_experts, int k,
                   const int32_t *idx_dev, const float *weight_dev, const float *x_dev, int64_t n_tokens, float *out_dev,
                   void *workspace_dev, size_t workspace_bytes, int glu, cml_stream_t stream) {
    if (!ready()) return fail(CML_ERR_UNAVAILABLE, "cml_init has not succeeded");
    if (!gate || !down) return fail(CML_ERR_INVALID, "null weight");
    if (glu != CML_GLU_SILU && glu != CML_GLU_GELU_TANH) return fail(CML_ERR_INVALID, "unknown expert activation %d", glu);
    const bool fused_gate_up = up == nullptr;  // `gate` holds gate|up experts of 2*ff rows each
    if (!expert_format(gate->fmt) || (up && up->fmt != gate->fmt) || !expert_format(down->fmt))
        return fail(CML_ERR_UNSUPPORTED, "mixture-of-experts dispatch is built for Q4_K, Q8_0 and Q4_0 expert matrices (gate and up alike)");
    if (n_experts <= 0 || n_experts > kMaxExperts || k <= 0 || k > n_experts || n_tokens < 0)
        return fail(CML_ERR_SHAPE, "bad routing shape (%d experts, top-%d)", n_experts, k);
    const int64_t hidden = gate->cols, ff = down->cols;
    if ((up && (up->cols != hidden || gate->rows != up->rows)) || gate->rows != (fused_gate_up ? 2 : 1) * ff * n_experts ||
        down->rows != hidden * n_experts)
        return fail(CML_ERR_SHAPE, "expert matrices do not stack to %d experts of %lld x %lld", n_experts, (long long)ff, (long long)hidden);
    const int act_in = act_of(gate->fmt), act_mid = act_of(down->fmt);
    if (hidden % (act_in == 2 ? 256 : 32) || ff % (act_mid == 2 ? 256 : 32))
        return fail(CML_ERR_SHAPE, "hidden and ff must be whole blocks of the expert formats");
    if (n_tokens == 0) return CML_OK;
    if (!idx_dev || !weight_dev || !x_dev || !out_dev || !workspace_dev) return fail(CML_ERR_INVALID, "null pointer");
    if ((reinterpret_cast<uintptr_t>(x_dev) & 15u) || (reinterpret_cast<uintptr_t>(workspace_dev) & 255u))
        return fail(CML_ERR_INVALID, "x must be 16-byte and the workspace 256-byte aligned");
    const MoeWorkspace ws = carve(workspace_dev, hidden, ff, n_tokens, k, n_experts);
    if (workspace_bytes < ws.total) return fail(CML_ERR_SHAPE, "workspace of %zu bytes given, %zu needed", workspace_bytes, ws.total);
    hipStream_t st = as_stream(stream);
    const int n_slots = static_cast<int>(n_tokens * k);

    // Decode (one token, rows of up to 4096 values): gate and up run as ONE launch that quantizes
    // the token inside every workgroup -- two launches and the quantized round trip fewer.
    const bool fused_decode = n_tokens == 1 && (act_in == 1 || hidden / 256 <= 16) && env_int("CAMELID_HIP_FUSED_QUANT", 1) != 0;
    // ws.g and ws.u are adjacent: a fused gate|up projection writes rows of 2*ff values across both
    const int64_t glu_stride = fused_gate_up ? 2 * ff : ff;
    if (!fused_decode) {
        if (int rc = launch_quantize_act(act_in, x_dev, n_tokens, hidden, ws.xq, ws.xd, st)) return rc;
    }
    hipLaunchKernelGGL(moe_plan_kernel, dim3(1), dim3(kMaxExperts), 0, st, idx_dev, n_slots, n_experts, k, ws.offsets, ws.assign_token, ws.slot_to_assign);
    CML_HIP_TRY(hipGetLastError());

    MatArgs a;
    a.residual = nullptr;
    a.ints = nullptr;
    a.group_offsets = ws.offsets;
    a.n_groups = n_experts;
    a.n_tokens = n_tokens;  // the most assignments one expert can receive
    // gate and up: every assignment reads its token's activation
    a.q = ws.xq;
    a.scales = ws.xd;
    a.group_rows = ws.assign_token;
    a.band_rows = fused_gate_up ? 2 * ff : ff;
    a.w = gate;
    a.out = ws.g;
    if (fused_decode && act_in == 1) {
        if (int rc = launch_gemv_b32_grouped(a, x_dev, st)) return rc;
        if (up) {
            a.w = up;
            a.out = ws.u;
            if (int rc = launch_gemv_b32_grouped(a, x_dev, st)) return rc;
        }
    } else if (fused_decode) {
        if (int rc = launch_gemv_q4k_f32_grouped_pair(a, up, up ? ws.u : nullptr, x_dev, st)) return rc;
    } else if (fused_gate_up) {
        if (int rc = launch_expert_matmul(a, st)) return rc;
    } else {
        if (int rc = launch_expert_matmul(a, st)) return rc;
        a.w = up;
        a.out = ws.u;
        if (int rc = launch_expert_matmul(a, st)) return rc;
    }
    // h = act(g) * u, quantized per assignment
    if (int rc = launch_glu_quantize(glu, act_mid, ws.g, fused_gate_up ? ws.g + ff : ws.u, n_slots, ff, glu_stride, ws.hq, ws.hd, st)) return rc;
    // down: assignment j reads its own h
    a.q = ws.hq;
    a.scales = ws.hd;
    a.group_rows = nullptr;
    a.band_rows = hidden;
    a.w = down;
    a.out = ws.y;
    if (int rc = launch_expert_matmul(a, st)) return rc;
    hipLaunchKernelGGL(moe_weighted_sum_kernel, dim3(static_cast<unsigned>((hidden + 255) / 256), static_cast<unsigned>(n_tokens)), dim3(256), 0, st,
                       ws.y, ws.slot_to_assign, weight_dev, k, hidden, out_dev);
    CML_HIP_TRY(hipGetLastError());
    return CML_OK;
}

}  // extern "C"
