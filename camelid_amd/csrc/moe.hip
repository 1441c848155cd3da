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

#include <algorithm>

#pragma clang fp contract(off)

namespace cml {

constexpr int kMaxExperts = 128;

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

// The same routing with one wave per token (k <= 64), lane l holding experts l and l + 64 during the
// selection and the l-th selected expert afterwards; the short sequential parts (maximum and sum over
// the k selected, in selection order) run redundantly in every lane.  Same arithmetic, value for
// value, as moe_route_kernel.
__global__ __launch_bounds__(256) void moe_route_wave_kernel(const float *__restrict__ logits, int64_t n_tokens, int n_experts, int k,
                                                             int32_t *__restrict__ idx_out, float *__restrict__ w_out) {
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int64_t t_raw = static_cast<int64_t>(blockIdx.x) * 4 + wave;
    const bool live = t_raw < n_tokens;
    const int64_t t = live ? t_raw : n_tokens - 1;  // spare waves repeat the last token and store nothing
    int sel_e, rank;
    float w;
    moe_route_wave(logits + t * n_experts, n_experts, k, lane, sel_e, w, rank);
    if (live && lane < k) {
        idx_out[t * k + rank] = sel_e;
        w_out[t * k + rank] = w;
    }
}

// One wave per token, lane l holding experts l and l + 64.  Gemma-4 routing (reference
// moe_layer_ffn, src/gemma4_runtime.rs:5567-5610; router_top_k, :61-84): softmax over ALL experts
// (max folded from f32::MIN, exp(v - max), sum left to right in index order, p /= sum), top-k by
// probability (descending, ties to the lower index), then
// scale[s] = down_scale[e] * (p[e] / max(sum of the selected p in selection order, 6.103515e-5)).
// The two sums are sequential chains, run redundantly in every lane; the rest is per lane plus
// one wave-wide maximum per selected expert.
__global__ __launch_bounds__(256) void moe_route_softmax_kernel(const float *__restrict__ logits, int64_t n_tokens, int n_experts,
                                                                int k, const float *__restrict__ down_scale,
                                                                int32_t *__restrict__ idx_out, float *__restrict__ w_out) {
    __shared__ float ps[4][kMaxExperts];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int64_t t_raw = static_cast<int64_t>(blockIdx.x) * 4 + wave;
    const bool live = t_raw < n_tokens;
    const int64_t t = live ? t_raw : n_tokens - 1;  // spare waves repeat the last token and store nothing
    const float *lg = logits + t * n_experts;
    const bool has0 = lane < n_experts, has1 = lane + 64 < n_experts;
    const float kLowest = -3.4028235e38f;
    const float l0 = has0 ? lg[lane] : kLowest, l1 = has1 ? lg[lane + 64] : kLowest;
    // The maximum does not depend on the order.  fmaxf drops NaNs as f32::max does; total_key
    // orders floats like the floats and is its own inverse.
    const int mkey = wave_allmax_i32(total_key(fmaxf(fmaxf(l0, l1), kLowest)));
    const float maxl = __builtin_bit_cast(float, mkey ^ static_cast<int>(static_cast<unsigned>(mkey >> 31) >> 1));
    float p0 = has0 ? expf(l0 - maxl) : 0.0f, p1 = has1 ? expf(l1 - maxl) : 0.0f;
    ps[wave][lane] = p0;
    ps[wave][lane + 64] = p1;
    __syncthreads();
    float sum = 0.0f;
#pragma unroll 8
    for (int e = 0; e < n_experts; e++) sum = sum + ps[wave][e];
    p0 = p0 / sum;
    p1 = p1 / sum;
    // selection: probabilities are >= 0, so their bit patterns order like the values; -1 = not a candidate
    int c0 = has0 ? __builtin_bit_cast(int, p0) : -1, c1 = has1 ? __builtin_bit_cast(int, p1) : -1;
    int se0 = 0, se1 = 0;       // lane s holds the s-th selected expert (se1: the (s + 64)-th)
    float sp0 = 0.0f, sp1 = 0.0f;
    float wsum = 0.0f;
    for (int s = 0; s < k; s++) {
        const int m = wave_allmax_i32(max(c0, c1));
        const unsigned long long b0 = __builtin_amdgcn_ballot_w64(c0 == m), b1 = __builtin_amdgcn_ballot_w64(c1 == m);
        const int e = b0 ? __builtin_ctzll(b0) : (b1 ? 64 + __builtin_ctzll(b1) : 0);
        const float pm = __builtin_bit_cast(float, m);
        if (e == lane) c0 = -1;
        if (e == lane + 64) c1 = -1;
        if (lane == (s & 63)) {
            if (s < 64) {
                se0 = e;
                sp0 = pm;
            } else {
                se1 = e;
                sp1 = pm;
            }
        }
        wsum = wsum + pm;
    }
    wsum = fmaxf(wsum, 6.103515e-5f);
    if (live && lane < k) {
        const float ds = down_scale ? down_scale[se0] : 1.0f;
        idx_out[t * k + lane] = se0;
        w_out[t * k + lane] = ds * (sp0 / wsum);
    }
    if (live && lane + 64 < k) {
        const float ds = down_scale ? down_scale[se1] : 1.0f;
        idx_out[t * k + lane + 64] = se1;
        w_out[t * k + lane + 64] = ds * (sp1 / wsum);
    }
}

// Group the n_tokens*k assignments by expert, keeping (token, rank) order inside each group (a
// stable counting sort).  One workgroup of 256 threads, one routed slot per thread and pass:
//   offsets[e..e+1)   assignment range of expert e
//   assign_token[j]   token whose activation assignment j reads
//   slot_to_assign[t*k+s]  where (token t, rank s) landed (-1: expert id out of range, slot dropped)
//   group_ids[y]      the experts that received assignments, ascending, then -1
// A slot's place = start of its expert's range + the slots of that expert before it: those of
// earlier passes (base), of earlier waves of this pass (wave_cnt), and of lower lanes of its own
// wave (a match mask built from 64 lane reads).
constexpr int kPlanThreads = 256;
__global__ __launch_bounds__(kPlanThreads) void moe_plan_kernel(const int32_t *__restrict__ idx, int n_slots, int n_experts, int k,
                                                                int32_t *__restrict__ offsets, int32_t *__restrict__ assign_token,
                                                                int32_t *__restrict__ slot_to_assign, int32_t *__restrict__ group_ids) {
    __shared__ int total[kMaxExperts];
    __shared__ int first[kMaxExperts];
    __shared__ int base[kMaxExperts];
    __shared__ int wave_cnt[kPlanThreads / 64][kMaxExperts];
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    if (tid < kMaxExperts) {
        total[tid] = 0;
        base[tid] = 0;
    }
    __syncthreads();
    for (int i = tid; i < n_slots; i += kPlanThreads) {
        const int e = idx[i];
        if (e >= 0 && e < n_experts) atomicAdd(&total[e], 1);
    }
    __syncthreads();
    if (tid < n_experts) {
        const int e = tid, mine = total[e];
        int start = 0, rank = 0, n_active = 0;
        for (int j = 0; j < n_experts; j++) {
            const int c = total[j];
            start += j < e ? c : 0;
            rank += (j < e && c > 0) ? 1 : 0;
            n_active += c > 0 ? 1 : 0;
        }
        first[e] = start;
        offsets[e] = start;
        if (e == n_experts - 1) offsets[n_experts] = start + mine;
        if (mine > 0) group_ids[rank] = e;
        else group_ids[n_active + (e - rank)] = -1;
    }
    for (int c0 = 0; c0 < n_slots; c0 += kPlanThreads) {
        const int i = c0 + tid;
        int e = i < n_slots ? idx[i] : -1;
        if (e >= n_experts) e = -1;
        wave_cnt[wave][lane] = 0;
        wave_cnt[wave][lane + 64] = 0;
        unsigned long long same = 0;  // lanes of this wave routed to the same expert
#pragma unroll
        for (int j = 0; j < 64; j++) same |= (__builtin_amdgcn_readlane(e, j) == e) ? (1ull << j) : 0ull;
        const int before = __builtin_popcountll(same & ((1ull << lane) - 1ull));
        if (e >= 0 && lane == 63 - __builtin_clzll(same)) wave_cnt[wave][e] = __builtin_popcountll(same);
        __syncthreads();  // also orders `first` / `base` before their first use
        if (e >= 0) {
            int at = first[e] + base[e] + before;
            for (int w = 0; w < wave; w++) at += wave_cnt[w][e];
            assign_token[at] = i / k;
            slot_to_assign[i] = at;
        } else if (i < n_slots) {
            slot_to_assign[i] = -1;
        }
        __syncthreads();
        if (c0 + kPlanThreads < n_slots) {
            if (tid < kMaxExperts) {
                int add = 0;
                for (int w = 0; w < kPlanThreads / 64; w++) add += wave_cnt[w][tid];
                base[tid] += add;
            }
            __syncthreads();
        }
    }
}

// Expert-grouped matmul: the packed-dot kernel for a few tokens, the matrix cores from 4 tokens
// up (the same crossover as for plain calls).  Both produce the same bits per cell.
static int launch_expert_matmul(const MatArgs &a, hipStream_t st) {
    if (a.w->fmt == CML_Q6_K) {
        const int64_t groups = a.group_ids ? a.max_active : a.n_groups;
        if (a.group_offsets && a.n_assign_total >= groups * env_int("CAMELID_HIP_Q6K_MFMA_MIN_GROUP", 6)) return launch_gemm_q6k_mfma(a, st);
        return launch_gemv_q6k(a, st);
    }
    if (a.w->fmt != CML_Q4_K) {
        // matrix cores once the groups in use hold enough assignments on average to fill a 16-token tile reasonably
        const int64_t groups = a.group_ids ? a.max_active : a.n_groups;
        if (a.group_offsets && b32_mfma_usable(a.w) && a.n_assign_total >= groups * env_int("CAMELID_HIP_B32_MFMA_MIN_GROUP", 6))
            return launch_gemm_b32_mfma(a, st);
        return launch_gemv_b32_grouped(a, GroupedPrologue{}, st);
    }
    if (a.group_offsets && a.n_tokens >= env_int("CAMELID_HIP_Q4K_MFMA_MIN_TOKENS", 4)) return launch_gemm_q4k_mfma(a, st);
    return launch_gemv_q4k(a, st);
}

static bool expert_format(int fmt) { return fmt == CML_Q4_K || fmt == CML_Q6_K || fmt == CML_Q8_0 || fmt == CML_Q4_0; }
// Activation quantization an expert matrix of this format is dotted with: 2 = Q8_K, 1 = Q8_0.
static int act_of(int fmt) { return is_k_family(fmt) ? 2 : 1; }
static int launch_quantize_act(int act, const float *x, int64_t n, int64_t cols, int8_t *q, float *s, hipStream_t st) {
    return act == 2 ? launch_quantize_q8_k(x, n, cols, q, s, st) : launch_quantize_q8_0(x, n, cols, q, s, st);
}

// out[t][c] = ((0 + y[a(t,0)][c]*w[t][0]) + y[a(t,1)][c]*w[t][1]) + ...  (reference
// src/inference.rs:14255-14257: `output += expert_out * weight`, routed order,
// multiply and add rounded separately).
// slot_expert (single-token decode without a grouping pass: slot s IS assignment s): the routed
// expert of every slot; a slot whose id is outside [0, n_experts) was served by nobody and is skipped.
__global__ __launch_bounds__(256) void moe_weighted_sum_kernel(const float *__restrict__ y, const int32_t *__restrict__ slot_to_assign,
                                                               const float *__restrict__ weight, int k, int64_t hidden,
                                                               int64_t n_assign, float *__restrict__ out,
                                                               const int32_t *__restrict__ slot_expert, int n_experts) {
    const int64_t c = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    const int64_t t = blockIdx.y;
    if (c >= hidden) return;
    float acc = 0.0f;
    // eight routed slots at a time: their loads go out together, the sum stays in routed order
    for (int s0 = 0; s0 < k; s0 += 8) {
        float yv[8], wv[8];
        bool ok[8];
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const int s = s0 + j;
            const int64_t slot = t * k + min(s, k - 1);
            const int64_t a = slot_to_assign ? slot_to_assign[slot] : slot;
            ok[j] = s < k && a >= 0 && a < n_assign;  // a dropped slot (expert id out of range) or a malformed map is skipped
            if (slot_expert) {
                const int e = slot_expert[slot];
                ok[j] = ok[j] && e >= 0 && e < n_experts;
            }
            yv[j] = y[(ok[j] ? a : 0) * hidden + c];
            wv[j] = weight[slot];
        }
#pragma unroll
        for (int j = 0; j < 8; j++)
            if (ok[j]) acc = acc + yv[j] * wv[j];
    }
    out[t * hidden + c] = acc;
}

struct MoeWorkspace {
    int8_t *xq;
    float *xd;
    int32_t *offsets, *assign_token, *slot_to_assign, *group_ids;
    float *g, *u, *y, *hd;
    int8_t *hq;
    int32_t *route_idx;  // routing results of the entry that takes logits
    float *route_w;
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
    w.group_ids = reinterpret_cast<int32_t *>(take(static_cast<size_t>(n_experts) * 4));
    w.assign_token = reinterpret_cast<int32_t *>(take(A * 4));
    w.slot_to_assign = reinterpret_cast<int32_t *>(take(A * 4));
    w.g = reinterpret_cast<float *>(take(A * ff * 4));
    w.u = reinterpret_cast<float *>(take(A * ff * 4));
    w.hq = reinterpret_cast<int8_t *>(take(A * ff));
    w.hd = reinterpret_cast<float *>(take(A * ((ff + 31) / 32) * 4));
    w.y = reinterpret_cast<float *>(take(A * hidden * 4));
    w.route_idx = reinterpret_cast<int32_t *>(take(A * 4));
    w.route_w = reinterpret_cast<float *>(take(A * 4));
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
    if (k <= 64) {
        hipLaunchKernelGGL(moe_route_wave_kernel, dim3(static_cast<unsigned>((n_tokens + 3) / 4)), dim3(256), 0, as_stream(stream), logits_dev,
                           n_tokens, n_experts, k, idx_dev, weight_dev);
        CML_COUNT_LAUNCH("moe.route.wave");
    } else {
        hipLaunchKernelGGL(moe_route_kernel, dim3(static_cast<unsigned>((n_tokens + 63) / 64)), dim3(64), 0, as_stream(stream), logits_dev,
                           n_tokens, n_experts, k, idx_dev, weight_dev);
        CML_COUNT_LAUNCH("moe.route.thread");
    }
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
    const unsigned grid = static_cast<unsigned>((n_tokens + 3) / 4);
    hipLaunchKernelGGL(moe_route_softmax_kernel, dim3(grid), dim3(256), 0, as_stream(stream), logits_dev, n_tokens, n_experts, k,
                       down_scale_dev, idx_dev, weight_dev);
    CML_COUNT_LAUNCH("moe.route.softmax");
    CML_HIP_TRY(hipGetLastError());
    return CML_OK;
}

int cml_moe_plan(const int32_t *idx_dev, int64_t n_tokens, int k, int n_experts, int32_t *token_offsets_dev,
                 int32_t *token_ids_dev, int32_t *route_to_assignment_dev, int32_t *union_experts_dev, cml_stream_t stream) {
    if (!ready()) return fail(CML_ERR_UNAVAILABLE, "cml_init has not succeeded");
    if (n_tokens < 0 || k <= 0 || n_experts <= 0 || n_tokens * k > INT32_MAX) return fail(CML_ERR_SHAPE, "bad routing shape");
    if (n_experts > kMaxExperts) return fail(CML_ERR_UNSUPPORTED, "at most %d experts", kMaxExperts);
    if (!token_offsets_dev || !union_experts_dev) return fail(CML_ERR_INVALID, "null pointer");
    if (n_tokens > 0 && (!idx_dev || !token_ids_dev || !route_to_assignment_dev)) return fail(CML_ERR_INVALID, "null pointer");
    hipLaunchKernelGGL(moe_plan_kernel, dim3(1), dim3(kPlanThreads), 0, as_stream(stream), idx_dev, static_cast<int>(n_tokens * k), n_experts, k,
                       token_offsets_dev, token_ids_dev, route_to_assignment_dev, union_experts_dev);
    CML_COUNT_LAUNCH("moe.plan");
    CML_HIP_TRY(hipGetLastError());
    return CML_OK;
}

int cml_moe_gemv_routed(const cml_weight *experts, int n_experts, const int8_t *q_dev, const float *scales_dev,
                        const int32_t *token_offsets_dev, const int32_t *token_ids_dev, const int32_t *union_experts_dev,
                        int max_union, int64_t max_assignments_per_expert, float *out_dev, cml_stream_t stream) {
    if (!ready()) return fail(CML_ERR_UNAVAILABLE, "cml_init has not succeeded");
    if (!experts) return fail(CML_ERR_INVALID, "null weight");
    if (!expert_format(experts->fmt)) return fail(CML_ERR_UNSUPPORTED, "routed matvec is built for Q4_K, Q6_K, Q8_0 and Q4_0 expert matrices");
    if (n_experts <= 0 || n_experts > kMaxExperts || experts->rows % n_experts != 0)
        return fail(CML_ERR_SHAPE, "%lld rows do not stack to %d experts", (long long)experts->rows, n_experts);
    if (max_assignments_per_expert < 0 || (union_experts_dev && (max_union <= 0 || max_union > n_experts)))
        return fail(CML_ERR_SHAPE, "bad routed shape");
    if (max_assignments_per_expert == 0) return CML_OK;
    if (!q_dev || !scales_dev || !token_offsets_dev || !out_dev) return fail(CML_ERR_INVALID, "null pointer");
    if ((reinterpret_cast<uintptr_t>(q_dev) & 15u) != 0) return fail(CML_ERR_INVALID, "quantized activations must be 16-byte aligned");
    MatArgs a{};
    a.w = experts;
    a.q = q_dev;
    a.scales = scales_dev;
    a.n_tokens = max_assignments_per_expert;
    a.out = out_dev;
    a.group_offsets = token_offsets_dev;
    a.group_rows = token_ids_dev;
    a.group_ids = union_experts_dev;
    a.max_active = max_union;
    a.n_groups = n_experts;
    a.band_rows = experts->rows / n_experts;
    return launch_expert_matmul(a, as_stream(stream));
}

int cml_moe_weighted_sum(const float *y_dev, const int32_t *route_to_assignment_dev, const float *weight_dev, int64_t n_tokens, int k,
                         int64_t hidden, float *out_dev, cml_stream_t stream) {
    if (!ready()) return fail(CML_ERR_UNAVAILABLE, "cml_init has not succeeded");
    if (n_tokens < 0 || k <= 0 || hidden <= 0 || n_tokens > 65535) return fail(CML_ERR_SHAPE, "bad shape");
    if (n_tokens == 0) return CML_OK;
    if (!y_dev || !weight_dev || !out_dev) return fail(CML_ERR_INVALID, "null pointer");
    hipLaunchKernelGGL(moe_weighted_sum_kernel, dim3(static_cast<unsigned>((hidden + 255) / 256), static_cast<unsigned>(n_tokens)), dim3(256), 0,
                       as_stream(stream), y_dev, route_to_assignment_dev, weight_dev, k, hidden, n_tokens * k, out_dev, nullptr, 0);
    CML_COUNT_LAUNCH("moe.weighted_sum");
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

// logits_dev non-null: the call routes itself (Mixtral routing) into the workspace; idx_dev / weight_dev are ignored.
static int moe_ffn_impl(const cml_weight *gate, const cml_weight *up, const cml_weight *down, int n_experts, int k,
                        const int32_t *idx_dev, const float *weight_dev, const float *logits_dev, const float *x_dev, int64_t n_tokens,
                        float *out_dev, void *workspace_dev, size_t workspace_bytes, int glu, cml_stream_t stream) {
    if (!ready()) return fail(CML_ERR_UNAVAILABLE, "cml_init has not succeeded");
    if (!gate || !down) return fail(CML_ERR_INVALID, "null weight");
    if (glu != CML_GLU_SILU && glu != CML_GLU_GELU_TANH) return fail(CML_ERR_INVALID, "unknown expert activation %d", glu);
    const bool fused_gate_up = up == nullptr;  // `gate` holds gate|up experts of 2*ff rows each
    if (!expert_format(gate->fmt) || (up && up->fmt != gate->fmt) || !expert_format(down->fmt))
        return fail(CML_ERR_UNSUPPORTED, "mixture-of-experts dispatch is built for Q4_K, Q6_K, Q8_0 and Q4_0 expert matrices (gate and up alike)");
    if (n_experts <= 0 || n_experts > kMaxExperts || k <= 0 || k > n_experts || n_tokens < 0)
        return fail(CML_ERR_SHAPE, "bad routing shape (%d experts, top-%d)", n_experts, k);
    if (n_tokens > 65535) return fail(CML_ERR_SHAPE, "at most 65535 tokens per call (%lld given)", (long long)n_tokens);
    const int64_t hidden = gate->cols, ff = down->cols;
    if ((up && (up->cols != hidden || gate->rows != up->rows)) || gate->rows != (fused_gate_up ? 2 : 1) * ff * n_experts ||
        down->rows != hidden * n_experts)
        return fail(CML_ERR_SHAPE, "expert matrices do not stack to %d experts of %lld x %lld", n_experts, (long long)ff, (long long)hidden);
    const int act_in = act_of(gate->fmt), act_mid = act_of(down->fmt);
    if (hidden % (act_in == 2 ? 256 : 32) || ff % (act_mid == 2 ? 256 : 32))
        return fail(CML_ERR_SHAPE, "hidden and ff must be whole blocks of the expert formats");
    if (n_tokens == 0) return CML_OK;
    if ((!logits_dev && (!idx_dev || !weight_dev)) || !x_dev || !out_dev || !workspace_dev) return fail(CML_ERR_INVALID, "null pointer");
    if ((reinterpret_cast<uintptr_t>(x_dev) & 15u) || (reinterpret_cast<uintptr_t>(workspace_dev) & 255u))
        return fail(CML_ERR_INVALID, "x must be 16-byte and the workspace 256-byte aligned");
    const MoeWorkspace ws = carve(workspace_dev, hidden, ff, n_tokens, k, n_experts);
    if (workspace_bytes < ws.total) return fail(CML_ERR_SHAPE, "workspace of %zu bytes given, %zu needed", workspace_bytes, ws.total);
    hipStream_t st = as_stream(stream);
    const int n_slots = static_cast<int>(n_tokens * k);

    // Decode (one token, rows of up to 4096 values): gate and up run as ONE launch that quantizes
    // the token inside every workgroup -- two launches and the quantized round trip fewer.
    const bool fused_decode = n_tokens == 1 && (act_in == 1 || (gate->fmt == CML_Q4_K && hidden / 256 <= 16)) &&
                              env_int("CAMELID_HIP_FUSED_QUANT", 1) != 0;
    // ws.g and ws.u are adjacent: a fused gate|up projection writes rows of 2*ff values across both
    const int64_t glu_stride = fused_gate_up ? 2 * ff : ff;
    const float *u_rows = fused_gate_up ? ws.g + ff : ws.u;
    // Decode with 32-value-block experts on both sides: the k routed slots ARE the assignments, so
    // no grouping pass runs (y-slot s of the grid serves expert idx[s]), and the down projection
    // computes act(g) * u and quantizes it in its own prologue: 4 launches after routing.
    const bool b32_direct = fused_decode && act_in == 1 && act_mid == 1 && ff <= 8192;
    // Q4_K on both sides: the same without the fused down prologue (a 56-super-block row is too
    // much to re-quantize in every workgroup).
    const bool q4k_direct = fused_decode && act_in == 2 && act_mid == 2;
    const bool direct = b32_direct || q4k_direct;
    // Routing: inside the gate|up launch where that launch can do it (one token, Q4_K experts, rows of
    // 4096 values: every wave routes the token itself and the first workgroup leaves the result for
    // the launches behind it), a launch of its own otherwise.
    bool route_in_launch = false;
    if (logits_dev) {
        idx_dev = ws.route_idx;
        weight_dev = ws.route_w;
        route_in_launch = q4k_direct && k <= 64 && env_int("CAMELID_HIP_MOE_FOLD_ROUTE", 1) &&
                          gemv_q4k_direct_can_route(gate, fused_gate_up ? 2 * ff : ff, n_slots, up != nullptr);
        if (!route_in_launch) {
            if (int rc = cml_moe_route_top_k(logits_dev, n_tokens, n_experts, k, ws.route_idx, ws.route_w, stream)) return rc;
        }
    }
    if (!fused_decode) {
        if (int rc = launch_quantize_act(act_in, x_dev, n_tokens, hidden, ws.xq, ws.xd, st)) return rc;
    }
    if (!direct) {
        hipLaunchKernelGGL(moe_plan_kernel, dim3(1), dim3(kPlanThreads), 0, st, idx_dev, n_slots, n_experts, k, ws.offsets, ws.assign_token,
                           ws.slot_to_assign, ws.group_ids);
        CML_COUNT_LAUNCH("moe.plan");
        CML_HIP_TRY(hipGetLastError());
    }

    MatArgs a{};
    a.group_offsets = direct ? nullptr : ws.offsets;
    a.group_ids = direct ? idx_dev : ws.group_ids;
    a.max_active = direct ? n_slots : static_cast<int>(std::min<int64_t>(n_experts, n_slots));
    a.n_assign_total = n_slots;
    a.n_groups = n_experts;
    a.n_tokens = n_tokens;  // the most assignments one expert can receive
    // gate and up: every assignment reads its token's activation
    a.q = ws.xq;
    a.scales = ws.xd;
    a.group_rows = direct ? nullptr : ws.assign_token;
    a.band_rows = fused_gate_up ? 2 * ff : ff;
    a.w = gate;
    a.out = ws.g;
    if (fused_decode && act_in == 1) {
        GroupedPrologue token;
        token.kind = 1;
        token.x = x_dev;
        if (int rc = launch_gemv_b32_grouped(a, token, st)) return rc;
        if (up) {
            a.w = up;
            a.out = ws.u;
            if (int rc = launch_gemv_b32_grouped(a, token, st)) return rc;
        }
    } else if (fused_decode) {
        if (route_in_launch) {
            a.route_logits = logits_dev;
            a.route_k = k;
            a.route_idx = ws.route_idx;
            a.route_w = ws.route_w;
        }
        int rc = launch_gemv_q4k_f32_grouped_pair(a, up, up ? ws.u : nullptr, x_dev, st);
        if (rc == CML_ERR_UNSUPPORTED && route_in_launch) {
            // the launch decided against routing inside it (its own shape checks are the authority): route in a
            // launch of its own and run the gate|up launch on the routed slots
            clear_error();
            route_in_launch = false;
            a.route_logits = nullptr;
            if (int rrc = cml_moe_route_top_k(logits_dev, n_tokens, n_experts, k, ws.route_idx, ws.route_w, stream)) return rrc;
            rc = launch_gemv_q4k_f32_grouped_pair(a, up, up ? ws.u : nullptr, x_dev, st);
        }
        if (rc) return rc;
        a.route_logits = nullptr;
    } else if (fused_gate_up) {
        if (int rc = launch_expert_matmul(a, st)) return rc;
    } else if (gate->fmt == CML_Q4_K && a.n_tokens >= env_int("CAMELID_HIP_Q4K_MFMA_MIN_TOKENS", 4) && env_int("CAMELID_HIP_MOE_PAIR_LAUNCH", 1)) {
        // gate and up on the matrix cores as ONE launch: twice the workgroups in one grid, one partly
        // filled last round of them instead of two
        a.w2 = up;
        a.out2 = ws.u;
        if (int rc = launch_gemm_q4k_mfma(a, st)) return rc;
        a.w2 = nullptr;
        a.out2 = nullptr;
    } else {
        if (int rc = launch_expert_matmul(a, st)) return rc;
        a.w = up;
        a.out = ws.u;
        if (int rc = launch_expert_matmul(a, st)) return rc;
    }
    // down: assignment j reads its own h = act(g) * u, quantized per assignment
    a.q = ws.hq;
    a.scales = ws.hd;
    a.group_rows = nullptr;
    a.band_rows = hidden;
    a.w = down;
    a.out = ws.y;
    if (b32_direct) {
        GroupedPrologue gated;
        gated.kind = 2 + glu;
        gated.x = ws.g;
        gated.u = u_rows;
        gated.stride = glu_stride;
        if (int rc = launch_gemv_b32_grouped(a, gated, st)) return rc;
    } else {
        if (int rc = launch_glu_quantize(glu, act_mid, ws.g, u_rows, n_slots, ff, glu_stride, ws.hq, ws.hd, st)) return rc;
        if (q4k_direct && down->fmt == CML_Q4_K && env_int("CAMELID_HIP_MOE_FOLD_SUM", 1)) {
            // decode: the routed experts' down projections and the weighted sum in one launch (a workgroup
            // owns a row tile for all slots); -1 = a shape that launch does not serve
            const int rc = launch_moe_down_sum_q4k(down, n_experts, n_slots, idx_dev, weight_dev, ws.hq, ws.hd, out_dev, st);
            if (rc != -1) return rc;
        }
        if (int rc = launch_expert_matmul(a, st)) return rc;
    }
    hipLaunchKernelGGL(moe_weighted_sum_kernel, dim3(static_cast<unsigned>((hidden + 255) / 256), static_cast<unsigned>(n_tokens)), dim3(256), 0, st,
                       ws.y, direct ? nullptr : ws.slot_to_assign, weight_dev, k, hidden, static_cast<int64_t>(n_slots), out_dev,
                       direct ? idx_dev : nullptr, n_experts);
    CML_COUNT_LAUNCH("moe.weighted_sum");
    CML_HIP_TRY(hipGetLastError());
    return CML_OK;
}

int cml_moe_ffn_ex(const cml_weight *gate, const cml_weight *up, const cml_weight *down, int n_experts, int k,
                   const int32_t *idx_dev, const float *weight_dev, const float *x_dev, int64_t n_tokens, float *out_dev,
                   void *workspace_dev, size_t workspace_bytes, int glu, cml_stream_t stream) {
    return moe_ffn_impl(gate, up, down, n_experts, k, idx_dev, weight_dev, nullptr, x_dev, n_tokens, out_dev, workspace_dev, workspace_bytes, glu,
                        stream);
}

int cml_moe_ffn_logits(const cml_weight *gate, const cml_weight *up, const cml_weight *down, int n_experts, int k,
                       const float *logits_dev, const float *x_dev, int64_t n_tokens, float *out_dev, void *workspace_dev,
                       size_t workspace_bytes, cml_stream_t stream) {
    if (!up) return fail(CML_ERR_INVALID, "null weight");
    if (!logits_dev && n_tokens > 0) return fail(CML_ERR_INVALID, "null pointer");
    return moe_ffn_impl(gate, up, down, n_experts, k, nullptr, nullptr, logits_dev, x_dev, n_tokens, out_dev, workspace_dev, workspace_bytes,
                        CML_GLU_SILU, stream);
}

}  // extern "C"
