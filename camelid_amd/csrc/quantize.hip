// Activation quantizers: f32 -> Q8_0 blocks and f32 -> Q8_K super-blocks, with
// the reference CPU path's exact arithmetic.
//
// Q8_0 (reference quantize_q8_0_block, src/inference.rs:22510-22528):
//   amax = max |v| (NaN ignored); u = amax / 127; scale = f16(u) widened back;
//   inv = (u == 0) ? 0 : 1 / u  (the UNROUNDED u); q = clamp(round-half-away(v * inv), -128, 127).
// Q8_K (reference quantize_q8_k_blocks, src/inference.rs:23121-23152):
//   the first strictly greatest |v| picks the signed `max`; iscale = -127 / max;
//   q = min(nearest_int(iscale * v), 127) with the 1.5*2^23 magic-add rounding;
//   d = 1 / iscale; an all-zero super-block gives d = 0, q = 0.
//
// Both are O(K) per token and never on the roofline; the layout is chosen for
// simplicity: 8 lanes per Q8_0 block, one wave per Q8_K super-block, each lane
// holding four consecutive values.
#include "cml_device.hpp"
#include "cml_host.hpp"

#pragma clang fp contract(off)

namespace cml {

// One thread per 4 values, 8 threads per 32-value block.
__global__ __launch_bounds__(256) void quantize_q8_0_kernel(const float *__restrict__ x, int64_t n_blocks,
                                                            int8_t *__restrict__ q, float *__restrict__ scales) {
    const int64_t tid = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    const int64_t block = tid >> 3;
    const bool live = block < n_blocks;
    const int64_t src = live ? tid : 0;
    const float4 v = reinterpret_cast<const float4 *>(x)[src];
    float scale;
    const uint32_t packed = q8_0_quantize_lane8(v, scale);
    if (!live) return;
    reinterpret_cast<uint32_t *>(q)[tid] = packed;
    if ((tid & 7) == 0) scales[block] = scale;
}

// One wave per 256-value super-block; lane l holds values 4l..4l+3.
__global__ __launch_bounds__(256) void quantize_q8_k_kernel(const float *__restrict__ x, int64_t n_sb,
                                                            int8_t *__restrict__ q, float *__restrict__ d) {
    const int lane = threadIdx.x & 63;
    const int64_t sb = static_cast<int64_t>(blockIdx.x) * (blockDim.x >> 6) + (threadIdx.x >> 6);
    if (sb >= n_sb) return;  // whole wave leaves together
    const float4 v = reinterpret_cast<const float4 *>(x + sb * 256)[lane];
    float dv;
    int bsum;
    const uint32_t packed = q8k_quantize_wave(v, dv, bsum);
    reinterpret_cast<uint32_t *>(q + sb * 256)[lane] = packed;
    if (lane == 0) d[sb] = dv;
}

// Host-supplied inverse (reference rms_inv_norm_quantize_q8_0 / _q8k, src/cuda_resident.rs:272-315,
// 4272-4291): the caller's CPU scan of the row has already produced the exact sequential
// (mean_square + eps)^-0.5; the device applies (x[i] * rms_inv) * weight[i] -- two multiplies, each
// rounded, left to right as in rms_norm -- and quantizes the row.  The reference walks the block's
// maximum serially in one lane and rounds with roundf; the maximum of a set does not depend on the
// order it is scanned in and the quantizers here round half away from zero as well, so these are
// the same bits with the scan done by data-parallel moves.
__global__ __launch_bounds__(256) void rms_inv_norm_quantize_q8_0_kernel(const float *__restrict__ x, const float *__restrict__ weight, float rms_inv,
                                                                         int64_t n_blocks, int8_t *__restrict__ q, float *__restrict__ scales) {
    const int64_t tid = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    const int64_t block = tid >> 3;
    const bool live = block < n_blocks;
    const int64_t src = live ? tid : 0;
    const float4 xv = reinterpret_cast<const float4 *>(x)[src], wv = reinterpret_cast<const float4 *>(weight)[src];
    const float4 v = make_float4((xv.x * rms_inv) * wv.x, (xv.y * rms_inv) * wv.y, (xv.z * rms_inv) * wv.z, (xv.w * rms_inv) * wv.w);
    float scale;
    const uint32_t packed = q8_0_quantize_lane8(v, scale);
    if (!live) return;
    reinterpret_cast<uint32_t *>(q)[tid] = packed;
    if ((tid & 7) == 0) scales[block] = scale;
}

__global__ __launch_bounds__(256) void rms_inv_norm_quantize_q8_k_kernel(const float *__restrict__ x, const float *__restrict__ weight, float rms_inv,
                                                                         int64_t n_sb, int8_t *__restrict__ q, float *__restrict__ d) {
    const int lane = threadIdx.x & 63;
    const int64_t sb = static_cast<int64_t>(blockIdx.x) * (blockDim.x >> 6) + (threadIdx.x >> 6);
    if (sb >= n_sb) return;  // whole wave leaves together
    const float4 xv = reinterpret_cast<const float4 *>(x + sb * 256)[lane], wv = reinterpret_cast<const float4 *>(weight + sb * 256)[lane];
    const float4 v = make_float4((xv.x * rms_inv) * wv.x, (xv.y * rms_inv) * wv.y, (xv.z * rms_inv) * wv.z, (xv.w * rms_inv) * wv.w);
    float dv;
    int bsum;
    const uint32_t packed = q8k_quantize_wave(v, dv, bsum);
    reinterpret_cast<uint32_t *>(q + sb * 256)[lane] = packed;
    if (lane == 0) d[sb] = dv;
}

// act: 1 = Q8_0 (cols a multiple of 32), 2 = Q8_K (a multiple of 256); one row
int launch_rms_inv_norm_quantize(int act, const float *x, const float *weight, float rms_inv, int64_t cols, int8_t *q, float *scales, hipStream_t st) {
    if (cols == 0) return CML_OK;
    if (act == 1) {
        const int64_t n_blocks = cols / 32;
        hipLaunchKernelGGL(rms_inv_norm_quantize_q8_0_kernel, dim3(static_cast<unsigned>((n_blocks * 8 + 255) / 256)), dim3(256), 0, st, x, weight, rms_inv,
                           n_blocks, q, scales);
        CML_COUNT_LAUNCH("producer.rms_inv_norm.q8_0");
    } else {
        const int64_t n_sb = cols / 256;
        hipLaunchKernelGGL(rms_inv_norm_quantize_q8_k_kernel, dim3(static_cast<unsigned>((n_sb + 3) / 4)), dim3(256), 0, st, x, weight, rms_inv, n_sb, q,
                           scales);
        CML_COUNT_LAUNCH("producer.rms_inv_norm.q8_k");
    }
    CML_HIP_TRY(hipGetLastError());
    return CML_OK;
}

int launch_quantize_q8_0(const float *x, int64_t n_tokens, int64_t cols, int8_t *q, float *s, hipStream_t st) {
    const int64_t n_blocks = n_tokens * (cols / 32);
    if (n_blocks == 0) return CML_OK;
    const int64_t threads = n_blocks * 8;
    const unsigned grid = static_cast<unsigned>((threads + 255) / 256);
    hipLaunchKernelGGL(quantize_q8_0_kernel, dim3(grid), dim3(256), 0, st, x, n_blocks, q, s);
    CML_COUNT_LAUNCH("quantize.q8_0");
    CML_HIP_TRY(hipGetLastError());
    return CML_OK;
}

int launch_quantize_q8_k(const float *x, int64_t n_tokens, int64_t cols, int8_t *q, float *d, hipStream_t st) {
    const int64_t n_sb = n_tokens * (cols / 256);
    if (n_sb == 0) return CML_OK;
    const unsigned grid = static_cast<unsigned>((n_sb + 3) / 4);
    hipLaunchKernelGGL(quantize_q8_k_kernel, dim3(grid), dim3(256), 0, st, x, n_sb, q, d);
    CML_COUNT_LAUNCH("quantize.q8_k");
    CML_HIP_TRY(hipGetLastError());
    return CML_OK;
}

}  // namespace cml
