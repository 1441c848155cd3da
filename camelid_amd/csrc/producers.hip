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
// cannot be spread over lanes: the squares are summed left to right in f32 (a
// tree sum reassociates and changes greedy tokens, as the reference's device
// lane notes at src/cuda_resident.rs:124-131).  The row is staged in LDS, one
// wave walks it in order -- one dependent addition per element, a few microseconds
// for 4096 values, the price of that contract -- and every lane then applies
// (x * scale) * weight.
// Rows are independent: one workgroup per token.
#include "cml_device.hpp"
#include "cml_host.hpp"

#pragma clang fp contract(off)

namespace cml {

// ACT: 0 = f32 output only, 1 = Q8_0, 2 = Q8_K (normed may be written as well).
// Every thread keeps its share of the row in registers (up to kRmsRegs float4) and puts the
// squares into LDS; wave 0 then adds them up in order, reading ahead in batches so that the
// only thing on its critical path is the chain of additions; the LDS row is reused for the
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
    // zeros from the end of the row up to the next multiple of 16 float4 and one more batch pair:
    // the walk below runs in whole batches and reads one batch ahead, and sum + 0 == sum exactly
    // (the sum of squares is never negative)
    const int n4p = (n4 + 15) & ~15;
    if (tid < n4p + 16 - n4) xs4[n4 + tid] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    __syncthreads();
    if (wave == 0) {
        // Left to right, every sum rounded on its own (the products were rounded above).  All lanes
        // of the wave run the same chain on the same (broadcast) reads.  Two register batches
        // alternate so that nothing but the additions sits between consecutive LDS reads.
        constexpr int B = 8;
        float4 ra[B], rb[B];
#pragma unroll
        for (int j = 0; j < B; j++) ra[j] = xs4[j];
        float sum = 0.0f;
        for (int i = 0; i < n4p; i += 2 * B) {
#pragma unroll
            for (int j = 0; j < B; j++) rb[j] = xs4[i + B + j];
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int j = 0; j < B; j++) {
                sum = sum + ra[j].x;
                sum = sum + ra[j].y;
                sum = sum + ra[j].z;
                sum = sum + ra[j].w;
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int j = 0; j < B; j++) ra[j] = xs4[i + 2 * B + j];
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int j = 0; j < B; j++) {
                sum = sum + rb[j].x;
                sum = sum + rb[j].y;
                sum = sum + rb[j].z;
                sum = sum + rb[j].w;
            }
            __builtin_amdgcn_sched_barrier(0);
        }
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
    if (cols > static_cast<int64_t>(kRmsRegs) * 1024 - 32)
        return fail(CML_ERR_UNSUPPORTED, "rms_norm row of %lld values exceeds the staging limit of %d", (long long)cols, kRmsRegs * 1024 - 32);
    const size_t lds = (((static_cast<size_t>(cols) / 4 + 15) & ~size_t(15)) + 16) * sizeof(float4);
    const dim3 grid(static_cast<unsigned>(n_tokens)), block(256);
    const int c = static_cast<int>(cols);
    switch (act) {
        case 0: hipLaunchKernelGGL(rms_norm_quantize_kernel<0>, grid, block, lds, st, x, weight, eps, c, normed, q, scales); break;
        case 1: hipLaunchKernelGGL(rms_norm_quantize_kernel<1>, grid, block, lds, st, x, weight, eps, c, normed, q, scales); break;
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
