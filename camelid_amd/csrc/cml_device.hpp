// Device-side helpers shared by the gfx950 kernels: 128-bit loads, packed int8
// dot products, DPP lane-group reductions and the GGUF field decoders.
//
// Everything here assumes wave64 (CDNA).  DPP row operations act inside a row
// of 16 lanes, so every lane group used with them is a power of two <= 16 and
// aligned to its own size.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#pragma clang fp contract(off)

namespace cml {

constexpr int kWave = 64;

// ---- loads -------------------------------------------------------------------

__device__ __forceinline__ uint4 ldg16(const void *p) {
    return *reinterpret_cast<const uint4 *>(p);
}
__device__ __forceinline__ uint2 ldg8(const void *p) {
    return *reinterpret_cast<const uint2 *>(p);
}
__device__ __forceinline__ uint32_t ldg4(const void *p) {
    return *reinterpret_cast<const uint32_t *>(p);
}
__device__ __forceinline__ uint16_t ldg2(const void *p) {
    return *reinterpret_cast<const uint16_t *>(p);
}

// ---- f16 ---------------------------------------------------------------------

// f16 bits -> f32: exact for every input (the hardware conversion widens
// without rounding, subnormals included), so it matches the reference's
// f16_bits_to_f32 (src/inference.rs:27098-27125).
__device__ __forceinline__ float f16_bits_to_f32(uint32_t bits16) {
    _Float16 h = __builtin_bit_cast(_Float16, static_cast<uint16_t>(bits16));
    return static_cast<float>(h);
}

// ---- packed int8 dot ---------------------------------------------------------

// acc + sum of the four signed byte products (v_dot4_i32_i8).
__device__ __forceinline__ int sdot4(uint32_t a, uint32_t b, int acc) {
    return __builtin_amdgcn_sdot4(static_cast<int>(a), static_cast<int>(b), acc, false);
}

__device__ __forceinline__ int dot16(const uint4 &a, const uint4 &b, int acc) {
    acc = sdot4(a.x, b.x, acc);
    acc = sdot4(a.y, b.y, acc);
    acc = sdot4(a.z, b.z, acc);
    acc = sdot4(a.w, b.w, acc);
    return acc;
}

// Sum of the 16 signed bytes of v.
__device__ __forceinline__ int bytesum16(const uint4 &v) {
    const uint32_t ones = 0x01010101u;
    int s = sdot4(v.x, ones, 0);
    s = sdot4(v.y, ones, s);
    s = sdot4(v.z, ones, s);
    s = sdot4(v.w, ones, s);
    return s;
}

// ---- DPP ---------------------------------------------------------------------

// row_shr:N -- lane i reads lane i-N of its 16-lane row; lanes whose source
// falls outside the row read 0.
template <int N>
__device__ __forceinline__ int row_shr_i32(int v) {
    static_assert(N >= 1 && N <= 15, "row_shr distance");
    return __builtin_amdgcn_update_dpp(0, v, 0x110 + N, 0xf, 0xf, true);
}
template <int N>
__device__ __forceinline__ float row_shr_f32(float v) {
    return __builtin_bit_cast(float, row_shr_i32<N>(__builtin_bit_cast(int, v)));
}

// Integer sum over an aligned group of G lanes; the LAST lane of the group
// (lane % G == G-1) ends up with the total, other lanes hold partial sums.
template <int G>
__device__ __forceinline__ int group_sum_to_last(int v) {
    static_assert(G == 1 || G == 2 || G == 4 || G == 8 || G == 16, "group size");
    if constexpr (G >= 2) v += row_shr_i32<1>(v);
    if constexpr (G >= 4) v += row_shr_i32<2>(v);
    if constexpr (G >= 8) v += row_shr_i32<4>(v);
    if constexpr (G >= 16) v += row_shr_i32<8>(v);
    return v;
}

// Ordered float fold over an aligned group of G lanes: the last lane of the
// group returns ((((acc + t[0]) + t[1]) + ...) + t[G-1]) where t[k] is `term`
// of the group's k-th lane -- the same left-to-right association a scalar
// loop over consecutive blocks produces.  Other lanes return garbage.
template <int G, int K = 0>
__device__ __forceinline__ float group_fold_ordered(float acc, float term) {
    if constexpr (K == G - 1) {
        return acc + term;
    } else {
        acc = acc + row_shr_f32<G - 1 - K>(term);
        return group_fold_ordered<G, K + 1>(acc, term);
    }
}

// ---- GGUF Q4_K scale/min words ------------------------------------------------

// The 12 scale bytes of a Q4_K super-block as three little-endian words
// u0,u1,u2.  Returns the four words the kmask scheme builds (reference
// src/inference.rs:25829-25861): scales 0..3, scales 4..7, mins 0..3,
// mins 4..7, one byte each.
__device__ __forceinline__ void q4k_unpack_scales(uint32_t u0, uint32_t u1, uint32_t u2,
                                                  uint32_t &sc03, uint32_t &sc47,
                                                  uint32_t &m03, uint32_t &m47) {
    sc03 = u0 & 0x3f3f3f3fu;
    m03 = u1 & 0x3f3f3f3fu;
    sc47 = (u2 & 0x0f0f0f0fu) | (((u0 >> 6) & 0x03030303u) << 4);
    m47 = ((u2 >> 4) & 0x0f0f0f0fu) | (((u1 >> 6) & 0x03030303u) << 4);
}

}  // namespace cml
