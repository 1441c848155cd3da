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

// Terms xs[0 .. 1024*c4) (non-negative f32, zero padded) in LDS, thread t owning the contiguous
// chunk of c4 float4 starting at t*c4.  Returns, in every lane of wave 0, the f32 sum
// (((0 + xs[0]) + xs[1]) + ...) exactly as a scalar loop produces it.  256 threads; n = number of
// real terms (sets the width of the binade guard).
__device__ __forceinline__ float ordered_sum_nonneg(const float4 *xs4, int c4, int n, int tid) {
    __shared__ float s_wave_total[4];
    __shared__ int s_E[256];         // binade of the group ending at thread t (0: add in order)
    __shared__ uint32_t s_D0[256], s_D1[256];
    __shared__ int s_head[256];      // first thread of the group ending at thread t
    __shared__ unsigned long long s_tail[4];
    const int lane = tid & 63, wave = tid >> 6;
    const float4 *mine = xs4 + tid * c4;

    // 1. chunk sums and their exclusive scan (the association of this approximation is free)
    float local = 0.0f;
    for (int j = 0; j < c4; j++) {
        const float4 v = mine[j];
        local = local + v.x;
        local = local + v.y;
        local = local + v.z;
        local = local + v.w;
    }
    float incl = local;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
        const float o = __shfl_up(incl, d);
        if (lane >= d) incl = incl + o;
    }
    if (lane == 63) s_wave_total[wave] = incl;
    __syncthreads();
    float before = 0.0f;
    for (int w = 0; w < wave; w++) before = before + s_wave_total[w];
    const float base = before + (incl - local), after = before + incl;

    // 2. same binade on both sides, with room for the difference between summation orders?
    const float delta = static_cast<float>(n + 64) * 2.384185791015625e-07f;  // (n + 64) * 2^-22
    const uint32_t e_lo = __float_as_uint(base * (1.0f - delta)) >> 23, e_hi = __float_as_uint(after * (1.0f + delta)) >> 23;
    const bool run = e_lo == e_hi && e_lo >= 1 && e_lo < 255;
    const int E = run ? static_cast<int>(e_lo) : 0;
    uint32_t D0 = 0, D1 = 0;
    if (run) {
        for (int j = 0; j < c4; j++) {
            const float4 v = mine[j];
            const float t4[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
            for (int k = 0; k < 4; k++) {
                const uint32_t bits = __float_as_uint(t4[k]);
                const int Ea = static_cast<int>(bits >> 23);
                const uint32_t ma = (bits & 0x7fffffu) | (Ea ? 0x800000u : 0u);
                const int sh = E - max(Ea, 1);
                uint32_t inc, tie = 0, floor_part;
                if (sh <= 0) {
                    floor_part = inc = -sh > 7 ? (ma ? kRunBig : 0u) : min(ma << (-sh), kRunBig);
                } else if (sh >= 25) {
                    floor_part = inc = 0;
                } else {
                    floor_part = ma >> sh;
                    const uint32_t rem = ma & ((1u << sh) - 1u), half = 1u << (sh - 1);
                    inc = floor_part + (rem > half ? 1u : 0u);
                    tie = rem == half ? 1u : 0u;
                }
                // a tie goes to the even neighbour: up exactly when S + floor is odd
                D0 = min(D0 + inc + (tie & (D0 ^ floor_part) & 1u), kRunBig);
                D1 = min(D1 + inc + (tie & (D1 ^ floor_part ^ 1u) & 1u), kRunBig);
            }
        }
    }

    // 3. compose neighbouring runs of one binade (segmented inclusive scan inside each wave; a
    //    wave boundary ends a group, the walk below simply meets one more group there)
    const int E_prev = __shfl_up(E, 1);
    bool head = lane == 0 || E == 0 || E_prev != E;  // in-order chunks stand alone
    int first = tid;
    bool seen = head;  // a group head lies inside the span composed so far
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
        const uint32_t o0 = __shfl_up(D0, d), o1 = __shfl_up(D1, d);
        const int ofirst = __shfl_up(first, d);
        const bool oseen = __shfl_up(static_cast<int>(seen), d) != 0;
        if (lane >= d && !seen) {
            // the span to the left (o0, o1) runs first, then this one
            const uint32_t n0 = min(o0 + ((o0 & 1u) ? D1 : D0), kRunBig);
            const uint32_t n1 = min(o1 + ((o1 & 1u) ? D0 : D1), kRunBig);
            D0 = n0;
            D1 = n1;
            first = ofirst;
            seen = oseen;
        }
    }
    const int next_head = __shfl_down(static_cast<int>(head), 1);
    const bool tail = lane == 63 || next_head != 0;
    s_E[tid] = E;
    s_D0[tid] = D0;
    s_D1[tid] = D1;
    s_head[tid] = first;
    const unsigned long long tails = __ballot(tail);
    if (lane == 0) s_tail[wave] = tails;
    __syncthreads();
    if (wave != 0) return 0.0f;

    // 4. the walk, every lane of wave 0 alike (all reads are broadcasts)
    float s = 0.0f;
    auto add_in_order = [&](int t0, int t1) __attribute__((always_inline)) {  // chunks t0..t1
        const float4 *p = xs4 + t0 * c4;
        const int cnt = (t1 - t0 + 1) * c4;
        for (int j = 0; j < cnt; j++) {
            const float4 v = p[j];
            s = s + v.x;
            s = s + v.y;
            s = s + v.z;
            s = s + v.w;
        }
    };
    for (int w = 0; w < 4; w++) {
        unsigned long long m = s_tail[w];
        while (m) {
            const int t = w * 64 + __builtin_ctzll(m);
            m &= m - 1;
            const int Eg = s_E[t];
            if (Eg == 0) {
                add_in_order(t, t);
                continue;
            }
            const uint32_t sb = __float_as_uint(s);
            const uint32_t S = (sb & 0x7fffffu) | 0x800000u;
            const uint32_t D = (S & 1u) ? s_D1[t] : s_D0[t];
            if (static_cast<int>(sb >> 23) == Eg && S + D < (1u << 24)) {
                s = __uint_as_float((static_cast<uint32_t>(Eg) << 23) | ((S + D) & 0x7fffffu));
            } else {
                add_in_order(s_head[t], t);  // the guard was too narrow for this data: still exact
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
constexpr int kRmsRegs = 16;  // float4 per thread: rows of up to 16 * 256 * 4 = 16384 values

template <int ACT>
__global__ __launch_bounds__(256) void rms_norm_quantize_kernel(const float *__restrict__ x, const float *__restrict__ weight,
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
        const int i = tid + k * 256;
        if (i < n4) {
            const float4 v = x4[i];
            xv[k] = v;
            xs4[i] = make_float4(v.x * v.x, v.y * v.y, v.z * v.z, v.w * v.w);
        }
    }
    // zeros from the end of the row up to 256 whole chunks: sum + 0 == sum exactly (the sum of
    // squares is never negative) and a zero term has increment 0
    const int c4 = (n4 + 255) >> 8;  // float4 per thread chunk
    for (int i = n4 + tid; i < 256 * c4; i += 256) xs4[i] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
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
        const int i = tid + k * 256;
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
        for (int i = tid; i < n4; i += 256) {
            float s;
            const uint32_t packed = q8_0_quantize_lane8(xs4[i], s);
            q32[i] = packed;
            if ((i & 7) == 0) sc[i >> 3] = s;
        }
    } else {
        // one wave per 256-value super-block
        float *d = scales + token * (cols / 256);
        for (int sb = wave; sb < cols / 256; sb += 4) {
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
    if (cols > static_cast<int64_t>(kRmsRegs) * 1024)
        return fail(CML_ERR_UNSUPPORTED, "rms_norm row of %lld values exceeds the staging limit of %d", (long long)cols, kRmsRegs * 1024);
    // the row in 256 whole chunks (zero padded); rows past 64 KB need the larger dynamic LDS window
    const size_t lds = static_cast<size_t>((cols / 4 + 255) / 256) * 256 * sizeof(float4);
    static bool raised = false;
    if (!raised) {
        CML_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(&rms_norm_quantize_kernel<0>), hipFuncAttributeMaxDynamicSharedMemorySize, 96 * 1024));
        CML_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(&rms_norm_quantize_kernel<1>), hipFuncAttributeMaxDynamicSharedMemorySize, 96 * 1024));
        CML_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(&rms_norm_quantize_kernel<2>), hipFuncAttributeMaxDynamicSharedMemorySize, 96 * 1024));
        CML_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(&rms_norm_quantize_kernel<3>), hipFuncAttributeMaxDynamicSharedMemorySize, 96 * 1024));
        raised = true;
    }
    const dim3 grid(static_cast<unsigned>(n_tokens)), block(256);
    const int c = static_cast<int>(cols);
    switch (act) {
        case 0: hipLaunchKernelGGL(rms_norm_quantize_kernel<0>, grid, block, lds, st, x, weight, eps, c, normed, q, scales); break;
        case 1: hipLaunchKernelGGL(rms_norm_quantize_kernel<1>, grid, block, lds, st, x, weight, eps, c, normed, q, scales); break;
        case 3: hipLaunchKernelGGL(rms_norm_quantize_kernel<3>, grid, block, lds, st, x, weight, eps, c, normed, q, scales); break;
        default: hipLaunchKernelGGL(rms_norm_quantize_kernel<2>, grid, block, lds, st, x, weight, eps, c, normed, q, scales); break;
    }
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
    } else {
        const int64_t n_sb = n_tokens * (cols / 256);
        const dim3 grid(static_cast<unsigned>((n_sb + 3) / 4));
        const int spr = static_cast<int>(cols / 256);
        if (glu == 0) hipLaunchKernelGGL(glu_quantize_q8k_kernel<0>, grid, dim3(256), 0, st, g, u, n_sb, spr, in_stride, q, scales);
        else hipLaunchKernelGGL(glu_quantize_q8k_kernel<1>, grid, dim3(256), 0, st, g, u, n_sb, spr, in_stride, q, scales);
    }
    CML_HIP_TRY(hipGetLastError());
    return CML_OK;
}

int launch_silu_mul_quantize(int act, const float *g, const float *u, int64_t n_tokens, int64_t cols, int8_t *q, float *scales,
                             hipStream_t st) {
    return launch_glu_quantize(0, act, g, u, n_tokens, cols, cols, q, scales, st);
}

}  // namespace cml
