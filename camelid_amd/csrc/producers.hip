// The steps immediately upstream of a quantized projection, fused with the
// activation quantizer so that the f32 intermediate never leaves the chip:
//   rms_norm -> Q8_0 / Q8_K      reference rms_norm_quantize, rms_norm_quantize_q8k
//                                (src/cuda_resident.rs:236-270, :4152-4177), CPU
//                                arithmetic CpuTensor::rms_norm_into, src/tensor/mod.rs:2707-2760
//   silu(gate) * up -> Q8_0/Q8_K reference silu_mul_quantize[_q8k] (src/cuda_resident.rs:
//                                4289-4341), CPU arithmetic CpuTensor::silu_mul,
//                                src/tensor/mod.rs:2610-2634
//   gelu_tanh(gate) * up -> ...  reference geglu_quantize_routed (src/cuda_resident.rs:6301-6343),
//                                CPU arithmetic src/gemma4_runtime.rs:5689-5691
// The quantizers are the ones of quantize.hip (same device functions), so the
// fused result equals the composed one bit for bit.
//
// rms_norm keeps the reference's arithmetic exactly, including the part that
// looks as if it could not be spread over lanes: the squares are summed left to
// right in f32 (a tree sum reassociates and changes greedy tokens, as the
// reference's device lane notes at src/cuda_resident.rs:124-131).
//
// The left-to-right sum in parallel, bit for bit.  While the running sum s stays inside one
// binade 2^E, s is an integer S in [2^23, 2^24) counted in units of ulp = 2^(E-150), and
// s + a rounds to S + round(a / ulp): the increment of a term does not depend on S, except for an
// exact tie (fraction one half), which goes to the even neighbour and so depends on the parity
// of S alone.  A run of terms is therefore a pair (D0, D1): the total increment when the run is
// entered with S even / odd -- and two runs compose like functions, which is associative.
//   1. every thread sums its own contiguous chunk and a workgroup scan gives each chunk an
//      APPROXIMATE incoming sum (any association);
//   2. a chunk whose approximate incoming and outgoing sums, widened by the worst-case
//      difference between any two f32 summation orders, lie in the same binade computes its
//      (D0, D1) in that binade's units; any other chunk (the few where the sum crosses a power of
//      two, the leading ones, anything not finite) is marked for in-order addition;
//   3. neighbouring chunks of the same binade are composed by a segmented scan;
//   4. one wave walks the groups in order: a composed run is applied in O(1) after checking on
//      the EXACT running sum that it enters in the assumed binade and does not leave it (if the
//      check fails the run's terms are added one by one -- the approximation only decides speed,
//      never the result); marked chunks are added term by term as the scalar loop would.
// 4096 values: about 12 marked chunks of 16 terms and as many runs instead of 4096 dependent
// additions.
// Rows are independent: one workgroup per token.
#include "cml_device.hpp"
#include "cml_host.hpp"

#pragma clang fp contract(off)

namespace cml {

constexpr uint32_t kRunBig = 1u << 26;  // saturation of run increments: anything >= 2^24 leaves the binade

__device__ __forceinline__ float readlane_f32(float v, int lane) {
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), lane));
}

// A run of terms as a function of the parity of the sum that enters it.
struct RunPair {
    uint32_t d0, d1;
};
// `left` runs first, then `right`
__device__ __forceinline__ RunPair run_then(const RunPair &left, const RunPair &right) {
    RunPair r;
    r.d0 = min(left.d0 + ((left.d0 & 1u) ? right.d1 : right.d0), kRunBig);
    r.d1 = min(left.d1 + ((left.d1 & 1u) ? right.d0 : right.d1), kRunBig);
    return r;
}

// Segmented inclusive scan over the 64 lanes of a wave: every lane ends up with the composition
// of the runs from its group's first lane to itself, and with that first lane's `first`.
// `seen` enters as 1 in the lanes that start a group.  Rows of 16 lanes by DPP, then row by row
// through lane reads.
__device__ __forceinline__ void run_scan64(RunPair &me, int &first, int &seen, int lane) {
    const int rl = lane & 15, row = lane >> 4;
    auto absorb = [&](uint32_t o0, uint32_t o1, int ofirst, int oseen, bool reach) __attribute__((always_inline)) {
        if (reach && !seen) {
            me = run_then(RunPair{o0, o1}, me);
            first = ofirst;
            seen = oseen;
        }
    };
    absorb(row_shr_i32<1>(me.d0), row_shr_i32<1>(me.d1), row_shr_i32<1>(first), row_shr_i32<1>(seen), rl >= 1);
    absorb(row_shr_i32<2>(me.d0), row_shr_i32<2>(me.d1), row_shr_i32<2>(first), row_shr_i32<2>(seen), rl >= 2);
    absorb(row_shr_i32<4>(me.d0), row_shr_i32<4>(me.d1), row_shr_i32<4>(first), row_shr_i32<4>(seen), rl >= 4);
    absorb(row_shr_i32<8>(me.d0), row_shr_i32<8>(me.d1), row_shr_i32<8>(first), row_shr_i32<8>(seen), rl >= 8);
#pragma unroll
    for (int r = 1; r < 4; r++) {  // the (by now complete) last lane of row r-1 into row r
        const int src = 16 * r - 1;
        absorb(__builtin_amdgcn_readlane(me.d0, src), __builtin_amdgcn_readlane(me.d1, src), __builtin_amdgcn_readlane(first, src),
               __builtin_amdgcn_readlane(seen, src), row == r);
    }
}

constexpr int kSumThreads = 1024, kSumWaves = kSumThreads / 64;

// Terms xs[0 .. 4*1024*c4) (non-negative f32, zero padded) in LDS, thread t owning the contiguous
// chunk of c4 float4 starting at t*c4.  Returns, in every lane of wave 0, the f32 sum
// (((0 + xs[0]) + xs[1]) + ...) exactly as a scalar loop produces it.  1024 threads (short
// chunks: the terms of a chunk that straddles a power of two are added one by one); n = number
// of real terms (sets the width of the binade guard).
__device__ __forceinline__ float ordered_sum_nonneg(const float4 *xs4, int c4, int n, int tid) {
    __shared__ float s_wave_total[kSumWaves];
    __shared__ int s_E[kSumThreads];         // binade of the group ending at thread t (0: add in order)
    __shared__ uint32_t s_D0[kSumThreads], s_D1[kSumThreads];
    __shared__ int s_head[kSumThreads];      // first thread of the group ending at thread t
    __shared__ int s_count[kSumWaves];       // groups per wave
    __shared__ uint16_t s_list[kSumWaves][64];  // the last threads of a wave's groups, in order
    const int lane = tid & 63, wave = tid >> 6, row = lane >> 4;
    const float4 *mine = xs4 + tid * c4;

    // 1. chunk sums and their exclusive scan (the association of this approximation is free):
    //    rows of 16 lanes by DPP, the three row totals by lane reads
    float local = 0.0f;
    for (int j = 0; j < c4; j++) {
        const float4 v = mine[j];
        local = local + v.x;
        local = local + v.y;
        local = local + v.z;
        local = local + v.w;
    }
    float incl = local;
    incl = incl + row_shr_f32<1>(incl);  // lanes at the start of a row receive 0
    incl = incl + row_shr_f32<2>(incl);
    incl = incl + row_shr_f32<4>(incl);
    incl = incl + row_shr_f32<8>(incl);
    const float r0 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, incl), 15));
    const float r1 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, incl), 31));
    const float r2 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, incl), 47));
    incl = incl + (row == 0 ? 0.0f : (row == 1 ? r0 : (row == 2 ? r0 + r1 : (r0 + r1) + r2)));
    if (lane == 63) s_wave_total[wave] = incl;
    __syncthreads();
    float before = 0.0f;
#pragma unroll
    for (int w = 0; w < kSumWaves - 1; w++) {  // all reads at once, then the additions
        const float tw = s_wave_total[w];
        before = before + (w < wave ? tw : 0.0f);
    }
    const float base = before + (incl - local), after = before + incl;

    // 2. same binade on both sides, with room for the difference between summation orders?
    const float delta = static_cast<float>(n + 64) * 2.384185791015625e-07f;  // (n + 64) * 2^-22
    const uint32_t e_lo = __float_as_uint(base * (1.0f - delta)) >> 23, e_hi = __float_as_uint(after * (1.0f + delta)) >> 23;
    const bool run = e_lo == e_hi && e_lo >= 1 && e_lo < 255;
    const int E = run ? static_cast<int>(e_lo) : 0;
    RunPair me{0u, 0u};
    if (run) {
        for (int j = 0; j < c4; j++) {
            const float4 v = mine[j];
            const float t4[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
            for (int k = 0; k < 4; k++) {
                // branch-free: a right shift by 1..31 covers every term below the sum's binade
                // (25 and more leave nothing: no increment, no tie), a left shift the others
                const uint32_t bits = __float_as_uint(t4[k]);
                const int Ea = static_cast<int>(bits >> 23);
                const uint32_t ma = (bits & 0x7fffffu) | (Ea ? 0x800000u : 0u);
                const int sh = E - max(Ea, 1);
                const int rs = min(max(sh, 1), 31);
                const uint32_t floor_r = ma >> rs, rem = ma & ((1u << rs) - 1u), half = 1u << (rs - 1);
                const uint32_t inc_r = floor_r + (rem > half ? 1u : 0u), tie_r = rem == half ? 1u : 0u;
                const int ls = min(-sh, 8);
                const uint32_t inc_l = ls == 8 ? (ma ? kRunBig : 0u) : min(ma << (ls & 7), kRunBig);
                const bool right = sh >= 1;
                const uint32_t inc = right ? inc_r : inc_l, floor_part = right ? floor_r : inc_l, tie = right ? tie_r : 0u;
                // a tie goes to the even neighbour: up exactly when S + floor is odd
                me.d0 = min(me.d0 + inc + (tie & (me.d0 ^ floor_part) & 1u), kRunBig);
                me.d1 = min(me.d1 + inc + (tie & (me.d1 ^ floor_part ^ 1u) & 1u), kRunBig);
            }
        }
    }

    // 3. compose neighbouring runs of one binade: a segmented inclusive scan, rows of 16 lanes by
    //    DPP, then row by row through lane reads (a wave boundary ends a group; the walk below
    //    simply meets one more group there)
    const int E_prev = __shfl_up(E, 1);
    const bool head = lane == 0 || E_prev != E;  // neighbouring in-order chunks (E = 0) form one range
    int first = tid;
    int seen = head ? 1 : 0;  // a group head lies inside the span composed so far
    run_scan64(me, first, seen, lane);
    // the zero padding behind the last real chunk is not walked at all
    const int n_chunks = (n + 4 * c4 - 1) / (4 * c4);
    const int next_head = __shfl_down(static_cast<int>(head), 1);
    const bool tail = tid < n_chunks && (lane == 63 || next_head != 0 || tid == n_chunks - 1);
    s_E[tid] = E;
    s_D0[tid] = me.d0;
    s_D1[tid] = me.d1;
    s_head[tid] = first;
    const unsigned long long tails = __ballot(tail);
    if (lane == 0) s_count[wave] = __builtin_popcountll(tails);
    if (tail) s_list[wave][__builtin_popcountll(tails & ((1ull << lane) - 1ull))] = static_cast<uint16_t>(tid);
    __syncthreads();
    if (wave != 0) return 0.0f;

    // 4. the walk, every lane of wave 0 alike.  Lane g first fetches the g-th group of a batch of
    //    up to 64 (its last thread from the tail masks, then the group's record), so that the
    //    chain through the running sum reads lanes, not memory.
    float s = 0.0f;
    auto add_in_order = [&](const float4 *p, int cnt) __attribute__((always_inline)) {  // cnt float4, the next one read ahead
        float4 v = p[0];
        for (int j = 0; j < cnt; j++) {
            const float4 nx = p[min(j + 1, cnt - 1)];
            s = s + v.x;
            s = s + v.y;
            s = s + v.z;
            s = s + v.w;
            v = nx;
        }
    };
    int cnt_w[kSumWaves];
#pragma unroll
    for (int w = 0; w < kSumWaves; w++) cnt_w[w] = s_count[w];
    int n_groups = 0;
#pragma unroll
    for (int w = 0; w < kSumWaves; w++) n_groups += cnt_w[w];
    for (int g0 = 0; g0 < n_groups; g0 += 64) {
        // the (g0 + lane)-th group: which wave's list, which entry
        int k = g0 + lane, w_mine = 0;
        bool found = false;
#pragma unroll
        for (int w = 0; w < kSumWaves; w++) {
            if (!found) {
                if (k < cnt_w[w]) {
                    found = true;
                    w_mine = w;
                } else {
                    k -= cnt_w[w];
                }
            }
        }
        const int t_mine = found ? s_list[w_mine][k] : kSumThreads - 1;
        // Groups that a wave boundary cut apart are put together again here, in parallel: the same
        // scan over the batch's records (lanes past the last group form groups of their own).
        const int gE = g0 + lane < n_groups ? s_E[t_mine] : -1 - lane;
        const int gE_prev = __shfl_up(gE, 1);
        RunPair gD{s_D0[t_mine], s_D1[t_mine]};
        int gH = s_head[t_mine];
        int gSeen = (lane == 0 || gE_prev != gE) ? 1 : 0;
        const int gE_next = __shfl_down(gE, 1);
        const bool gTail = g0 + lane < n_groups && (lane == 63 || gE_next != gE);
        run_scan64(gD, gH, gSeen, lane);
        // an in-order range usually is one or two float4 long: fetch those with the record
        const int gCnt = (t_mine - gH + 1) * c4;
        const float4 gV0 = xs4[gH * c4], gV1 = xs4[gH * c4 + (gCnt > 1 ? 1 : 0)];
        unsigned long long todo = __ballot(gTail);
        while (todo) {
            const int g = __builtin_ctzll(todo);
            todo &= todo - 1;
            const int Eg = __builtin_amdgcn_readlane(gE, g);
            if (Eg == 0) {
                const int cnt = __builtin_amdgcn_readlane(gCnt, g);
                s = s + readlane_f32(gV0.x, g);
                s = s + readlane_f32(gV0.y, g);
                s = s + readlane_f32(gV0.z, g);
                s = s + readlane_f32(gV0.w, g);
                if (cnt > 1) {
                    s = s + readlane_f32(gV1.x, g);
                    s = s + readlane_f32(gV1.y, g);
                    s = s + readlane_f32(gV1.z, g);
                    s = s + readlane_f32(gV1.w, g);
                    if (cnt > 2) add_in_order(xs4 + __builtin_amdgcn_readlane(gH, g) * c4 + 2, cnt - 2);
                }
                continue;
            }
            // The run enters with S even or odd; adding its increment to the BITS of s is adding it
            // to S as long as no carry reaches the exponent field -- which is also the test that
            // the sum stays in the binade.  D1 - D0 is a handful of ties: a 24-bit multiply.
            const uint32_t D0 = __builtin_amdgcn_readlane(gD.d0, g), D1 = __builtin_amdgcn_readlane(gD.d1, g);
            const uint32_t sb = __float_as_uint(s);
            const uint32_t after = sb + D0 + static_cast<uint32_t>(__mul24(static_cast<int>(sb & 1u), static_cast<int>(D1 - D0)));
            const uint32_t e_bits = static_cast<uint32_t>(Eg) << 23;
            if (((sb ^ e_bits) | (after ^ e_bits)) < (1u << 23) && D0 < (1u << 24)) {
                s = __uint_as_float(after);
            } else {  // the guard was too narrow for this data: still exact
                add_in_order(xs4 + __builtin_amdgcn_readlane(gH, g) * c4, __builtin_amdgcn_readlane(gCnt, g));
            }
        }
    }
    return s;
}

// ACT: 0 = f32 output only, 1 = Q8_0, 2 = Q8_K (normed may be written as well), 3 = the row's
// sum of squares alone (into normed[token]).
// Every thread keeps its share of the row in registers (up to kRmsRegs float4) and puts the
// squares into LDS, where ordered_sum_nonneg adds them up; the LDS row is reused for the
// normalised values the quantizers read.
constexpr int kRmsRegs = 4;  // float4 per thread: rows of up to 4 * 1024 * 4 = 16384 values

template <int ACT>
__global__ __launch_bounds__(kSumThreads) void rms_norm_quantize_kernel(const float *__restrict__ x, const float *__restrict__ weight,
                                                                float eps, int cols, float *__restrict__ normed,
                                                                int8_t *__restrict__ q, float *__restrict__ scales) {
    extern __shared__ float4 xs4[];  // the row, padded to whole batches: squares first, then the normalised values
    __shared__ float s_scale;
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int64_t token = blockIdx.x;
    const int n4 = cols >> 2;
    const float4 *x4 = reinterpret_cast<const float4 *>(x + token * cols);
    float4 xv[kRmsRegs];
#pragma unroll
    for (int k = 0; k < kRmsRegs; k++) {
        const int i = tid + k * kSumThreads;
        if (i < n4) {
            const float4 v = x4[i];
            xv[k] = v;
            xs4[i] = make_float4(v.x * v.x, v.y * v.y, v.z * v.z, v.w * v.w);
        }
    }
    // zeros from the end of the row up to 1024 whole chunks: sum + 0 == sum exactly (the sum of
    // squares is never negative) and a zero term has increment 0
    const int c4 = (n4 + kSumThreads - 1) / kSumThreads;  // float4 per thread chunk
    for (int i = n4 + tid; i < kSumThreads * c4; i += kSumThreads) xs4[i] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    __syncthreads();
    const float sum = ordered_sum_nonneg(xs4, c4, cols, tid);  // valid in wave 0
    if constexpr (ACT == 3) {
        if (tid == 0) normed[token] = sum;
        return;
    }
    if (wave == 0) {
        const float mean_square = sum / static_cast<float>(cols);
        if (lane == 0) s_scale = 1.0f / sqrtf(mean_square + eps);
    }
    __syncthreads();
    const float scale = s_scale;
    const float4 *w4 = reinterpret_cast<const float4 *>(weight);
    float4 *n4out = normed ? reinterpret_cast<float4 *>(normed + token * cols) : nullptr;
#pragma unroll
    for (int k = 0; k < kRmsRegs; k++) {
        const int i = tid + k * kSumThreads;
        if (i < n4) {
            const float4 v = xv[k], w = w4[i];
            float4 y;
            y.x = (v.x * scale) * w.x;
            y.y = (v.y * scale) * w.y;
            y.z = (v.z * scale) * w.z;
            y.w = (v.w * scale) * w.w;
            if (ACT != 0) xs4[i] = y;
            if (n4out) n4out[i] = y;
        }
    }
    if constexpr (ACT == 0) return;
    __syncthreads();
    uint32_t *q32 = reinterpret_cast<uint32_t *>(q + token * cols);
    if constexpr (ACT == 1) {
        // eight lanes per 32-value block; cols/4 is a multiple of 8, so groups enter and leave together
        float *sc = scales + token * (cols / 32);
        for (int i = tid; i < n4; i += kSumThreads) {
            float s;
            const uint32_t packed = q8_0_quantize_lane8(xs4[i], s);
            q32[i] = packed;
            if ((i & 7) == 0) sc[i >> 3] = s;
        }
    } else {
        // one wave per 256-value super-block
        float *d = scales + token * (cols / 256);
        for (int sb = wave; sb < cols / 256; sb += kSumWaves) {
            float dv;
            int bsum;
            const uint32_t packed = q8k_quantize_wave(xs4[sb * 64 + lane], dv, bsum);
            q32[sb * 64 + lane] = packed;
            if (lane == 0) d[sb] = dv;
        }
    }
}

int launch_rms_norm_quantize(int act, const float *x, const float *weight, float eps, int64_t n_tokens, int64_t cols,
                             float *normed, int8_t *q, float *scales, hipStream_t st) {
    if (n_tokens == 0 || cols == 0) return CML_OK;
    if (cols > static_cast<int64_t>(kRmsRegs) * kSumThreads * 4)
        return fail(CML_ERR_UNSUPPORTED, "rms_norm row of %lld values exceeds the staging limit of %d", (long long)cols, kRmsRegs * kSumThreads * 4);
    // the row in 1024 whole chunks (zero padded)
    const size_t lds = static_cast<size_t>((cols / 4 + kSumThreads - 1) / kSumThreads) * kSumThreads * sizeof(float4);
    static bool raised = false;
    if (!raised) {
        CML_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(&rms_norm_quantize_kernel<0>), hipFuncAttributeMaxDynamicSharedMemorySize, 96 * 1024));
        CML_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(&rms_norm_quantize_kernel<1>), hipFuncAttributeMaxDynamicSharedMemorySize, 96 * 1024));
        CML_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(&rms_norm_quantize_kernel<2>), hipFuncAttributeMaxDynamicSharedMemorySize, 96 * 1024));
        CML_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(&rms_norm_quantize_kernel<3>), hipFuncAttributeMaxDynamicSharedMemorySize, 96 * 1024));
        raised = true;
    }
    const dim3 grid(static_cast<unsigned>(n_tokens)), block(kSumThreads);
    const int c = static_cast<int>(cols);
    switch (act) {
        case 0: hipLaunchKernelGGL(rms_norm_quantize_kernel<0>, grid, block, lds, st, x, weight, eps, c, normed, q, scales); break;
        case 1: hipLaunchKernelGGL(rms_norm_quantize_kernel<1>, grid, block, lds, st, x, weight, eps, c, normed, q, scales); break;
        case 3: hipLaunchKernelGGL(rms_norm_quantize_kernel<3>, grid, block, lds, st, x, weight, eps, c, normed, q, scales); break;
        default: hipLaunchKernelGGL(rms_norm_quantize_kernel<2>, grid, block, lds, st, x, weight, eps, c, normed, q, scales); break;
    }
    CML_COUNT_LAUNCH("producer.rms_norm");
    CML_HIP_TRY(hipGetLastError());
    return CML_OK;
}

// h = silu(g) * u = (g / (1 + exp(-g))) * u, quantized on the fly.  Q8_K: one wave per
// 256-value super-block, lane l holding values 4l..4l+3 (the layout of quantize_q8_k_kernel).
// Row r of g / u starts at g + r * in_stride / u + r * in_stride (in_stride = cols for separate
// buffers; 2 * cols with u = g + cols when a fused gate|up projection wrote both halves of a row).
template <int GLU>
__global__ __launch_bounds__(256) void glu_quantize_q8k_kernel(const float *__restrict__ g, const float *__restrict__ u,
                                                               int64_t n_sb, int sb_per_row, int64_t in_stride,
                                                               int8_t *__restrict__ q, float *__restrict__ d) {
    const int lane = threadIdx.x & 63;
    const int64_t sb = static_cast<int64_t>(blockIdx.x) * (blockDim.x >> 6) + (threadIdx.x >> 6);
    if (sb >= n_sb) return;
    const int64_t r = sb / sb_per_row, c = (sb - r * sb_per_row) * 256;
    const float4 v = glu4<GLU>(reinterpret_cast<const float4 *>(g + r * in_stride + c)[lane],
                               reinterpret_cast<const float4 *>(u + r * in_stride + c)[lane]);
    float dv;
    int bsum;
    const uint32_t packed = q8k_quantize_wave(v, dv, bsum);
    reinterpret_cast<uint32_t *>(q + sb * 256)[lane] = packed;
    if (lane == 0) d[sb] = dv;
}

// Q8_0: one thread per 4 values, 8 threads per 32-value block (the layout of quantize_q8_0_kernel).
template <int GLU>
__global__ __launch_bounds__(256) void glu_quantize_q8_0_kernel(const float *__restrict__ g, const float *__restrict__ u,
                                                                int64_t n_blocks, int blocks_per_row, int64_t in_stride,
                                                                int8_t *__restrict__ q, float *__restrict__ scales) {
    const int64_t tid = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    const int64_t block = tid >> 3;
    const bool live = block < n_blocks;
    const int64_t bsafe = live ? block : 0;
    const int64_t r = bsafe / blocks_per_row, c = (bsafe - r * blocks_per_row) * 32 + (tid & 7) * 4;
    const float4 v = glu4<GLU>(*reinterpret_cast<const float4 *>(g + r * in_stride + c), *reinterpret_cast<const float4 *>(u + r * in_stride + c));
    float scale;
    const uint32_t packed = q8_0_quantize_lane8(v, scale);
    if (!live) return;
    reinterpret_cast<uint32_t *>(q)[tid] = packed;
    if ((tid & 7) == 0) scales[block] = scale;
}

// glu: 0 = silu, 1 = gelu_tanh; act: 1 = Q8_0, 2 = Q8_K.
int launch_glu_quantize(int glu, int act, const float *g, const float *u, int64_t n_tokens, int64_t cols, int64_t in_stride,
                        int8_t *q, float *scales, hipStream_t st) {
    if (n_tokens == 0 || cols == 0) return CML_OK;
    if (act == 1) {
        const int64_t n_blocks = n_tokens * (cols / 32);
        const dim3 grid(static_cast<unsigned>((n_blocks * 8 + 255) / 256));
        const int bpr = static_cast<int>(cols / 32);
        if (glu == 0) hipLaunchKernelGGL(glu_quantize_q8_0_kernel<0>, grid, dim3(256), 0, st, g, u, n_blocks, bpr, in_stride, q, scales);
        else hipLaunchKernelGGL(glu_quantize_q8_0_kernel<1>, grid, dim3(256), 0, st, g, u, n_blocks, bpr, in_stride, q, scales);
        CML_COUNT_LAUNCH("producer.glu.q8_0");
    } else {
        const int64_t n_sb = n_tokens * (cols / 256);
        const dim3 grid(static_cast<unsigned>((n_sb + 3) / 4));
        const int spr = static_cast<int>(cols / 256);
        if (glu == 0) hipLaunchKernelGGL(glu_quantize_q8k_kernel<0>, grid, dim3(256), 0, st, g, u, n_sb, spr, in_stride, q, scales);
        else hipLaunchKernelGGL(glu_quantize_q8k_kernel<1>, grid, dim3(256), 0, st, g, u, n_sb, spr, in_stride, q, scales);
        CML_COUNT_LAUNCH("producer.glu.q8_k");
    }
    CML_HIP_TRY(hipGetLastError());
    return CML_OK;
}

int launch_silu_mul_quantize(int act, const float *g, const float *u, int64_t n_tokens, int64_t cols, int8_t *q, float *scales,
                             hipStream_t st) {
    return launch_glu_quantize(0, act, g, u, n_tokens, cols, cols, q, scales, st);
}

}  // namespace cml
