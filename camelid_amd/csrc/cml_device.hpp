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
// The bulk of a weight is read once per launch: the non-temporal hint keeps it from displacing
// what is reused (activations, scale planes) on its way through the caches.  Measured on the
// 14336 x 4096 Q4_K matvec, cache-cold: 8.7 -> 8.1 us.
__device__ __forceinline__ uint4 ldg16_stream(const void *p) {
#ifdef CML_PLAIN_WEIGHT_LOADS
    return ldg16(p);
#else
    typedef uint32_t v4u __attribute__((ext_vector_type(4)));
    const v4u v = __builtin_nontemporal_load(reinterpret_cast<const v4u *>(p));
    return make_uint4(v.x, v.y, v.z, v.w);
#endif
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
template <int CTRL>
__device__ __forceinline__ float dpp_f32(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true));
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

__device__ __forceinline__ uint32_t pack4(int a, int b, int c, int d) {
    return (static_cast<uint32_t>(a) & 0xffu) | ((static_cast<uint32_t>(b) & 0xffu) << 8) |
           ((static_cast<uint32_t>(c) & 0xffu) << 16) | ((static_cast<uint32_t>(d) & 0xffu) << 24);
}

// ---- Q8_0 activation quantizer, eight lanes per block ---------------------------

// Rust's `(v).round().clamp(-128.0, 127.0) as i8`: NaN casts to 0.
__device__ __forceinline__ int q8_0_round(float v) {
    float r = roundf(v);  // ties away from zero
    if (r != r) return 0;
    r = fminf(fmaxf(r, -128.0f), 127.0f);
    return static_cast<int>(r);
}

// Quantizes one 32-value block held by eight consecutive lanes (lane l of the group holds
// values 4l..4l+3): reference quantize_q8_0_block, src/inference.rs:22510-22528 -- amax = max |v|
// (NaN ignored); u = amax / 127; scale = f16(u) widened back; inv = (u == 0) ? 0 : 1 / u (the
// UNROUNDED u); q = clamp(round-half-away(v * inv), -128, 127).  Returns the lane's four quants
// packed; `scale` is the same in all eight lanes.  All eight lanes of a group must call it together.
__device__ __forceinline__ uint32_t q8_0_quantize_lane8(const float4 v, float &scale) {
    float amax = fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w)));
    // maximum over the aligned group of eight lanes by data-parallel-primitive moves (no LDS
    // crossbar round trips): lanes 1 and 2 apart inside each quad, then the other quad of the
    // group through the mirror of the half row (lane i <-> 7 - i, which holds that quad's maximum)
    amax = fmaxf(amax, dpp_f32<0xB1>(amax));   // quad_perm [1,0,3,2]
    amax = fmaxf(amax, dpp_f32<0x4E>(amax));   // quad_perm [2,3,0,1]
    amax = fmaxf(amax, dpp_f32<0x141>(amax));  // row_half_mirror
    const float u = amax / 127.0f;
    const float inv = (u == 0.0f) ? 0.0f : 1.0f / u;
    // f32 -> f16 round-to-nearest-even -> f32 (reference f32_to_f16_bits, src/inference.rs:27062-27096)
    scale = static_cast<float>(static_cast<_Float16>(u));
    return pack4(q8_0_round(v.x * inv), q8_0_round(v.y * inv), q8_0_round(v.z * inv), q8_0_round(v.w * inv));
}

// ---- Q8_K activation quantizer, one wave per super-block ------------------------

// The reference's nearest_int (src/inference.rs:23112-23116).
__device__ __forceinline__ int nearest_int_magic(float f) {
    const float val = f + 12582912.0f;
    return static_cast<int>(__builtin_bit_cast(uint32_t, val) & 0x007fffffu) - 0x00400000;
}

// Quantizes one 256-value super-block held by a whole wave, lane l holding
// values 4l..4l+3 (reference quantize_q8_k_blocks, src/inference.rs:23121-23152):
// the first strictly greatest |v| picks the signed `max`; iscale = -127 / max;
// q = min(nearest_int(iscale * v), 127); d = 1 / iscale; an all-zero (or all-NaN)
// super-block gives d = 0, q = 0.  Returns the lane's four quants packed; `d` is
// the same in every lane; lanes with (lane & 7) == 7 get in `bsum` the sum of the
// 32 quants of group lane / 8 (other lanes hold partial sums).
// Must be called by all 64 lanes.
__device__ __forceinline__ uint32_t q8k_quantize_wave(const float4 v, float &d, int &bsum) {
    const float a0 = fabsf(v.x), a1 = fabsf(v.y), a2 = fabsf(v.z), a3 = fabsf(v.w);
    // fmaxf drops NaNs; the trailing 0 turns an all-NaN lane into 0
    const float lmax = fmaxf(fmaxf(fmaxf(a0, a1), fmaxf(a2, a3)), 0.0f);
    float m = lmax;  // row maxima gather in lanes 15, 31, 47, 63 (values are >= 0, so the 0 fill is neutral)
    m = fmaxf(m, row_shr_f32<1>(m));
    m = fmaxf(m, row_shr_f32<2>(m));
    m = fmaxf(m, row_shr_f32<4>(m));
    m = fmaxf(m, row_shr_f32<8>(m));
    const int mi = __builtin_bit_cast(int, m);  // non-negative floats order like their bit patterns
    const int r0 = __builtin_amdgcn_readlane(mi, 15), r1 = __builtin_amdgcn_readlane(mi, 31);
    const int r2 = __builtin_amdgcn_readlane(mi, 47), r3 = __builtin_amdgcn_readlane(mi, 63);
    const int amax_bits = max(max(r0, r1), max(r2, r3));
    // Straight-line on purpose (several super-blocks interleave in one wave): an all-zero or
    // all-NaN super-block runs through with iscale = inf or NaN and is forced to d = 0, q = 0 at the end.
    const bool empty = amax_bits == 0;  // wave-uniform
    const float amax = __builtin_bit_cast(float, amax_bits);
    const unsigned long long holders = __builtin_amdgcn_ballot_w64(lmax == amax);
    const int first_lane = holders ? __builtin_ctzll(holders) : 0;
    const float mine = (a0 == amax) ? v.x : ((a1 == amax) ? v.y : ((a2 == amax) ? v.z : v.w));
    const float vmax = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, mine), first_lane));
    const float iscale = -127.0f / vmax;
    const int q0 = min(nearest_int_magic(iscale * v.x), 127);
    const int q1 = min(nearest_int_magic(iscale * v.y), 127);
    const int q2 = min(nearest_int_magic(iscale * v.z), 127);
    const int q3 = min(nearest_int_magic(iscale * v.w), 127);
    const uint32_t packed = empty ? 0u : pack4(q0, q1, q2, q3);
    d = empty ? 0.0f : 1.0f / iscale;
    bsum = group_sum_to_last<8>(sdot4(packed, 0x01010101u, 0));
    return packed;
}

// row_ror:N -- lane i reads lane (i - N) mod 16 of its 16-lane row.  Four of
// them (1, 2, 4, 8) leave every lane of a row with the row's reduction.
template <int N>
__device__ __forceinline__ int row_ror_i32(int v) {
    static_assert(N >= 1 && N <= 15, "row_ror distance");
    return __builtin_amdgcn_update_dpp(0, v, 0x120 + N, 0xf, 0xf, false);
}
__device__ __forceinline__ float row_allmax_nonneg(float m) {
    m = fmaxf(m, __builtin_bit_cast(float, row_ror_i32<1>(__builtin_bit_cast(int, m))));
    m = fmaxf(m, __builtin_bit_cast(float, row_ror_i32<2>(__builtin_bit_cast(int, m))));
    m = fmaxf(m, __builtin_bit_cast(float, row_ror_i32<4>(__builtin_bit_cast(int, m))));
    m = fmaxf(m, __builtin_bit_cast(float, row_ror_i32<8>(__builtin_bit_cast(int, m))));
    return m;
}
__device__ __forceinline__ int row_allor(int v) {
    v |= row_ror_i32<1>(v);
    v |= row_ror_i32<2>(v);
    v |= row_ror_i32<4>(v);
    v |= row_ror_i32<8>(v);
    return v;
}

// ---- mixture-of-experts routing by one wave ------------------------------------------------------
// f32::total_cmp as an integer key (larger key = greater value).
__device__ __forceinline__ int total_key(float v) {
    const int b = __builtin_bit_cast(int, v);
    return b ^ static_cast<int>(static_cast<unsigned>(b >> 31) >> 1);
}

// Maximum over the 64 lanes of a wave, returned in every lane (all lanes must be active).
__device__ __forceinline__ int wave_allmax_i32(int v) {
    v = max(v, row_ror_i32<1>(v));
    v = max(v, row_ror_i32<2>(v));
    v = max(v, row_ror_i32<4>(v));
    v = max(v, row_ror_i32<8>(v));
    return max(max(__builtin_amdgcn_readlane(v, 0), __builtin_amdgcn_readlane(v, 16)),
               max(__builtin_amdgcn_readlane(v, 32), __builtin_amdgcn_readlane(v, 48)));
}

// Mixtral routing of ONE token by one whole wave (reference softmax_top_k, src/inference.rs:
// 13940-13991): top-k by logit (total order, descending, ties to the lower index), softmax over the
// selected in selection order, renormalised, re-sorted by weight (descending, ties to the lower
// index).  n_experts <= 128 (lane l holds experts l and l + 64 during the selection), k <= 64.
// On return lane s < k holds the s-th SELECTED expert, its weight and the rank it takes in the
// routed order; the short sequential parts run redundantly in every lane.
// moe_route_wave_values: the same on logits the caller has loaded (l0 = logit of expert `lane`, l1 of
// expert lane + 64; lanes past n_experts pass anything).
__device__ __forceinline__ void moe_route_wave_values(float l0, float l1, int n_experts, int k, int lane, int &sel_e, float &w, int &rank) {
    bool v0 = lane < n_experts, v1 = lane + 64 < n_experts;
    const int k0 = total_key(l0), k1 = total_key(l1);
    sel_e = 0;
    float sel_v = 0.0f;
    for (int s = 0; s < k; s++) {  // top-k by logit (total order, descending), ties to the lower index
        const int m = wave_allmax_i32(max(v0 ? k0 : INT32_MIN, v1 ? k1 : INT32_MIN));
        const unsigned long long b0 = __builtin_amdgcn_ballot_w64(v0 && k0 == m), b1 = __builtin_amdgcn_ballot_w64(v1 && k1 == m);
        const int e = b0 ? __builtin_ctzll(b0) : (b1 ? 64 + __builtin_ctzll(b1) : 0);
        const int from = __builtin_amdgcn_readlane(__builtin_bit_cast(int, e < 64 ? l0 : l1), e & 63);
        if (e == lane) v0 = false;
        if (e == lane + 64) v1 = false;
        if (lane == s) {
            sel_e = e;
            sel_v = __builtin_bit_cast(float, from);
        }
    }
    float mx = -INFINITY;
    for (int s = 0; s < k; s++) mx = fmaxf(mx, __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, sel_v), s)));
    const float wv = (lane < k && fabsf(sel_v) < INFINITY) ? expf(sel_v - mx) : 0.0f;  // is_finite: NaN and inf give 0
    float sum = 0.0f;
    for (int s = 0; s < k; s++) sum = sum + __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, wv), s));
    w = sum > 0.0f ? wv / sum : 1.0f / static_cast<float>(k);
    // re-sort by weight (descending), ties to the lower index: the rank of (w, index) in that total order
    const int wk = total_key(w);
    rank = 0;
    for (int s = 0; s < k; s++) {
        const int ok = total_key(__builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, w), s)));
        const int oe = __builtin_amdgcn_readlane(sel_e, s);
        rank += (ok > wk || (ok == wk && oe < sel_e)) ? 1 : 0;
    }
}
__device__ __forceinline__ void moe_route_wave(const float *lg, int n_experts, int k, int lane, int &sel_e, float &w, int &rank) {
    const float l0 = lane < n_experts ? lg[lane] : 0.0f, l1 = lane + 64 < n_experts ? lg[lane + 64] : 0.0f;
    moe_route_wave_values(l0, l1, n_experts, k, lane, sel_e, w, rank);
}

// ---- gated activations ------------------------------------------------------------------------
// GLU 0: silu(g) * u = (g / (1 + exp(-g))) * u (reference CpuTensor::silu_mul).
// GLU 1: gelu_pytorch_tanh(g) * u = (0.5 * g * (1 + tanh(C * (g + 0.044715 * g * g * g)))) * u,
//        evaluated left to right (reference gelu_tanh, src/gemma4_mtp.rs:172-175; the expert
//        activation of the Gemma-4 lane, src/gemma4_runtime.rs:5689-5691).
template <int GLU>
__device__ __forceinline__ float glu1(float g, float u) {
    if constexpr (GLU == 0) {
        return (g / (1.0f + expf(-g))) * u;
    } else {
        const float cube = ((0.044715f * g) * g) * g;
        return ((0.5f * g) * (1.0f + tanhf(0.7978846f * (g + cube)))) * u;
    }
}
template <int GLU>
__device__ __forceinline__ float4 glu4(const float4 gv, const float4 uv) {
    return make_float4(glu1<GLU>(gv.x, uv.x), glu1<GLU>(gv.y, uv.y), glu1<GLU>(gv.z, uv.z), glu1<GLU>(gv.w, uv.w));
}

// The same quantizer with a 16-lane row per super-block, so that one wave does
// four super-blocks in one pass and one dependency chain: lane l of a row holds
// values 16l..16l+15 (v[0..3]).  Returns the 16 quants packed in value order;
// `d` is the same in every lane of the row; odd lanes get in `bsum` the sum of
// the 32 quants of group l / 2.  Same arithmetic, value for value, as
// q8k_quantize_wave.  Must be called by all 64 lanes.
__device__ __forceinline__ uint4 q8k_quantize_row16(const float4 (&v)[4], int lane, float &d, int &bsum) {
    float a[16];
#pragma unroll
    for (int k = 0; k < 4; k++) {
        a[4 * k + 0] = fabsf(v[k].x);
        a[4 * k + 1] = fabsf(v[k].y);
        a[4 * k + 2] = fabsf(v[k].z);
        a[4 * k + 3] = fabsf(v[k].w);
    }
    float lmax = 0.0f;  // fmaxf drops NaNs
#pragma unroll
    for (int j = 0; j < 16; j++) lmax = fmaxf(lmax, a[j]);
    const float amax = row_allmax_nonneg(lmax);
    const bool empty = amax == 0.0f;
    // first holder of the maximum: lowest lane of the row, lowest value in the lane
    const unsigned long long holders = __builtin_amdgcn_ballot_w64(lmax == amax);
    const uint32_t row_holders = static_cast<uint32_t>(holders >> (lane & 48)) & 0xffffu;
    const bool first = row_holders != 0u && (lane & 15) == __builtin_ctz(row_holders);
    const float vals[16] = {v[0].x, v[0].y, v[0].z, v[0].w, v[1].x, v[1].y, v[1].z, v[1].w,
                            v[2].x, v[2].y, v[2].z, v[2].w, v[3].x, v[3].y, v[3].z, v[3].w};
    float mine = vals[15];
#pragma unroll
    for (int j = 14; j >= 0; j--) mine = (a[j] == amax) ? vals[j] : mine;
    const float vmax = __builtin_bit_cast(float, row_allor(first ? __builtin_bit_cast(int, mine) : 0));
    const float iscale = -127.0f / vmax;
    uint32_t pk[4];
#pragma unroll
    for (int k = 0; k < 4; k++) {
        const int q0 = min(nearest_int_magic(iscale * vals[4 * k + 0]), 127);
        const int q1 = min(nearest_int_magic(iscale * vals[4 * k + 1]), 127);
        const int q2 = min(nearest_int_magic(iscale * vals[4 * k + 2]), 127);
        const int q3 = min(nearest_int_magic(iscale * vals[4 * k + 3]), 127);
        pk[k] = empty ? 0u : pack4(q0, q1, q2, q3);
    }
    d = empty ? 0.0f : 1.0f / iscale;
    const uint4 packed = make_uint4(pk[0], pk[1], pk[2], pk[3]);
    const int s = bytesum16(packed);
    bsum = s + row_shr_i32<1>(s);
    return packed;
}

// The same quantizer with a 32-lane half wave per super-block (one wave does two super-blocks in
// one pass): lane l of a half holds values 8l..8l+7 (v[0], v[1]).  Returns the 8 quants packed in
// value order; `d` is the same in every lane of the half; lanes with (l & 3) == 3 get in `bsum`
// the sum of the 32 quants of group l / 4.  Same arithmetic, value for value, as
// q8k_quantize_wave.  The signed value of the first strictly greatest |v| is found without a
// per-element search in the common case: with hi / lo the lane's signed extremes, the holders of
// the maximum magnitude are the lanes with hi == amax (a positive holder) or -lo == amax (a
// negative one); unless a half has both kinds the sign is the one kind present.  A half that has
// both takes the element-by-element search (wave-uniform branch).  Must be called by all 64 lanes.
__device__ __forceinline__ uint2 q8k_quantize_row32(const float4 (&v)[2], int lane, float &d, int &bsum) {
    const float vals[8] = {v[0].x, v[0].y, v[0].z, v[0].w, v[1].x, v[1].y, v[1].z, v[1].w};
    float hi = vals[0], lo = vals[0];  // fmaxf / fminf drop NaNs
#pragma unroll
    for (int j = 1; j < 8; j++) {
        hi = fmaxf(hi, vals[j]);
        lo = fminf(lo, vals[j]);
    }
    const float lmax = fmaxf(fmaxf(hi, -lo), 0.0f);  // the trailing 0 turns an all-NaN lane into 0
    // non-negative floats order like their bit patterns: integer maxima fold into the DPP moves
    int m = __builtin_bit_cast(int, lmax);
    m = max(m, row_ror_i32<1>(m));
    m = max(m, row_ror_i32<2>(m));
    m = max(m, row_ror_i32<4>(m));
    m = max(m, row_ror_i32<8>(m));
    {
        typedef unsigned int v2u_dev __attribute__((ext_vector_type(2)));
        const v2u_dev r = __builtin_amdgcn_permlane16_swap(static_cast<unsigned>(m), static_cast<unsigned>(m), false, false);
        m = max(static_cast<int>(r.x), static_cast<int>(r.y));  // both 16-lane rows of the half
    }
    const float amax = __builtin_bit_cast(float, m);
    const bool empty = m == 0;
    const unsigned long long bp = __builtin_amdgcn_ballot_w64(hi == amax), bn = __builtin_amdgcn_ballot_w64(-lo == amax);
    const uint32_t bp0 = static_cast<uint32_t>(bp), bp1 = static_cast<uint32_t>(bp >> 32);
    const uint32_t bn0 = static_cast<uint32_t>(bn), bn1 = static_cast<uint32_t>(bn >> 32);
    const bool upper = (lane & 32) != 0;
    float vmax = ((upper ? bn1 : bn0) != 0u) ? -amax : amax;
    if ((bp0 != 0u && bn0 != 0u) || (bp1 != 0u && bn1 != 0u)) {
        // equal magnitudes of both signs in one super-block: the first holder decides (lowest lane of
        // the half, lowest value in the lane)
        const uint32_t holders = upper ? (bp1 | bn1) : (bp0 | bn0);
        const bool first = holders != 0u && (lane & 31) == __builtin_ctz(holders);
        float mine = vals[7];
#pragma unroll
        for (int j = 6; j >= 0; j--) mine = (fabsf(vals[j]) == amax) ? vals[j] : mine;
        int sv = row_allor(first ? __builtin_bit_cast(int, mine) : 0);
        typedef unsigned int v2u_dev __attribute__((ext_vector_type(2)));
        const v2u_dev r = __builtin_amdgcn_permlane16_swap(static_cast<unsigned>(sv), static_cast<unsigned>(sv), false, false);
        sv = static_cast<int>(r.x | r.y);
        vmax = __builtin_bit_cast(float, sv);
    }
    const float iscale = -127.0f / vmax;
    uint32_t pk[2];
#pragma unroll
    for (int k = 0; k < 2; k++) {
        const int q0 = min(nearest_int_magic(iscale * vals[4 * k + 0]), 127);
        const int q1 = min(nearest_int_magic(iscale * vals[4 * k + 1]), 127);
        const int q2 = min(nearest_int_magic(iscale * vals[4 * k + 2]), 127);
        const int q3 = min(nearest_int_magic(iscale * vals[4 * k + 3]), 127);
        pk[k] = empty ? 0u : pack4(q0, q1, q2, q3);
    }
    d = empty ? 0.0f : 1.0f / iscale;
    int s = sdot4(pk[1], 0x01010101u, sdot4(pk[0], 0x01010101u, 0));
    s += row_shr_i32<1>(s);
    s += row_shr_i32<2>(s);
    bsum = s;
    return make_uint2(pk[0], pk[1]);
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
