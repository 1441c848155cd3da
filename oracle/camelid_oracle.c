/*
 * camelid_oracle.c -- TEST INFRASTRUCTURE, NOT PRODUCT CODE.
 *
 * Scalar CPU restatement of the reference's quantized matvec path; see
 * camelid_oracle.h for what it is for and what pins each function.  Compile
 * with -ffp-contract=off (the Makefile does): every float multiply and add
 * below is meant to round on its own unless it is written as fmaf().
 */
#include "camelid_oracle.h"

#include <float.h>
#include <math.h>
#include <pthread.h>
#include <stdlib.h>
#include <string.h>

#define Q8_0_VALUES 32
#define QK_K 256

int orc_block_values(int fmt) {
    switch (fmt) {
    case ORC_Q8_0:
    case ORC_Q4_0:
        return 32;
    case ORC_Q4_K:
    case ORC_Q6_K:
        return 256;
    default:
        return 0;
    }
}

/* Block geometry: src/gguf/reader.rs:130-185, src/tensor/mod.rs:5494-5508. */
int orc_block_bytes(int fmt) {
    switch (fmt) {
    case ORC_Q8_0:
        return 34;
    case ORC_Q4_0:
        return 18;
    case ORC_Q4_K:
        return 144;
    case ORC_Q6_K:
        return 210;
    default:
        return 0;
    }
}

/* ---- f16 <-> f32 -------------------------------------------------------- */

static uint32_t f32_bits(float v) {
    uint32_t b;
    memcpy(&b, &v, 4);
    return b;
}

static float bits_f32(uint32_t b) {
    float v;
    memcpy(&v, &b, 4);
    return v;
}

/* src/inference.rs:27062-27096: IEEE round-to-nearest-even, subnormals kept,
 * every NaN becomes 0x7e00. */
uint16_t orc_f32_to_f16_bits(float value) {
    uint32_t bits = f32_bits(value);
    uint16_t sign = (uint16_t)((bits >> 16) & 0x8000u);
    int32_t exp = (int32_t)((bits >> 23) & 0xffu);
    uint32_t mant = bits & 0x007fffffu;

    if (exp == 0xff)
        return (uint16_t)(sign | (mant == 0 ? 0x7c00u : 0x7e00u));
    int32_t half_exp = exp - 127 + 15;
    if (half_exp >= 0x1f)
        return (uint16_t)(sign | 0x7c00u);
    if (half_exp <= 0) {
        if (half_exp < -10)
            return sign;
        uint32_t mantissa = mant | 0x00800000u;
        uint32_t shift = (uint32_t)(14 - half_exp);
        uint16_t half_mant = (uint16_t)(mantissa >> shift);
        uint32_t round_bit = 1u << (shift - 1);
        if ((mantissa & round_bit) != 0 &&
            ((mantissa & (round_bit - 1)) != 0 || (half_mant & 1) != 0))
            half_mant = (uint16_t)(half_mant + 1);
        return (uint16_t)(sign | half_mant);
    }
    uint16_t half = (uint16_t)(sign | ((uint16_t)half_exp << 10) | (uint16_t)(mant >> 13));
    if ((mant & 0x00001000u) != 0 && ((mant & 0x00000fffu) != 0 || (half & 1) != 0))
        half = (uint16_t)(half + 1);
    return half;
}

/* src/inference.rs:27098-27125. */
float orc_f16_bits_to_f32(uint16_t bits) {
    uint32_t sign = ((uint32_t)(bits & 0x8000u)) << 16;
    uint32_t exp = (bits & 0x7c00u) >> 10;
    uint32_t frac = bits & 0x03ffu;
    uint32_t out;
    if (exp == 0) {
        if (frac == 0) {
            out = sign;
        } else {
            uint32_t mant = frac;
            int32_t e = -14;
            while ((mant & 0x0400u) == 0) {
                mant <<= 1;
                e -= 1;
            }
            mant &= 0x03ffu;
            out = sign | ((uint32_t)(e + 127) << 23) | (mant << 13);
        }
    } else if (exp == 0x1f) {
        out = sign | 0x7f800000u | (frac << 13);
    } else {
        out = sign | ((exp + (127 - 15)) << 23) | (frac << 13);
    }
    return bits_f32(out);
}

/* Array forms of the two converters, for exhaustive checks. */
void orc_f32_to_f16_bits_array(const float *v, size_t n, uint16_t *out) {
    for (size_t i = 0; i < n; i++)
        out[i] = orc_f32_to_f16_bits(v[i]);
}

void orc_f16_bits_to_f32_array(const uint16_t *h, size_t n, float *out) {
    for (size_t i = 0; i < n; i++)
        out[i] = orc_f16_bits_to_f32(h[i]);
}

static float wire_f16(const uint8_t *p) {
    return orc_f16_bits_to_f32((uint16_t)(p[0] | ((uint16_t)p[1] << 8)));
}

/* ---- activation quantizers --------------------------------------------- */

/* src/inference.rs:22510-22528.  max_abs folds with f32::max (NaN ignored);
 * the stored scale is the f16-rounded amax/127 but the quantizing inverse is
 * taken from the UNROUNDED quotient; `.round()` is ties-away-from-zero. */
void orc_quantize_q8_0(const float *x, size_t n, float *scales, int8_t *q) {
    size_t n_blocks = n / Q8_0_VALUES;
    for (size_t b = 0; b < n_blocks; b++) {
        const float *blk = x + b * Q8_0_VALUES;
        float max_abs = 0.0f;
        for (int j = 0; j < Q8_0_VALUES; j++)
            max_abs = fmaxf(max_abs, fabsf(blk[j]));
        float unrounded = max_abs / 127.0f;
        scales[b] = orc_f16_bits_to_f32(orc_f32_to_f16_bits(unrounded));
        float inv = (unrounded == 0.0f) ? 0.0f : 1.0f / unrounded;
        for (int j = 0; j < Q8_0_VALUES; j++) {
            float r = roundf(blk[j] * inv);
            int8_t v;
            if (r != r)
                v = 0; /* `NaN as i8` saturating cast gives 0 */
            else if (r < -128.0f)
                v = -128;
            else if (r > 127.0f)
                v = 127;
            else
                v = (int8_t)r;
            q[b * Q8_0_VALUES + j] = v;
        }
    }
}

/* src/inference.rs:23112-23116: round-to-nearest-even through the 1.5*2^23
 * magic constant. */
static int32_t nearest_int_reference(float fval) {
    float val = fval + 12582912.0f;
    return (int32_t)(f32_bits(val) & 0x007fffffu) - 0x00400000;
}

/* src/inference.rs:23121-23152: the FIRST strictly greater |v| wins and its
 * signed value sets iscale = -127/max; clamp above at 127 only; d = 1/iscale. */
void orc_quantize_q8_k(const float *x, size_t n, float *d, int8_t *q) {
    size_t n_sb = n / QK_K;
    for (size_t i = 0; i < n_sb; i++) {
        const float *chunk = x + i * QK_K;
        float amax = 0.0f, max = 0.0f;
        for (int j = 0; j < QK_K; j++) {
            float v = chunk[j];
            if (fabsf(v) > amax) {
                amax = fabsf(v);
                max = v;
            }
        }
        if (amax == 0.0f) {
            d[i] = 0.0f;
            memset(q + i * QK_K, 0, QK_K);
            continue;
        }
        float iscale = -127.0f / max;
        for (int j = 0; j < QK_K; j++) {
            int32_t v = nearest_int_reference(iscale * chunk[j]);
            if (v > 127)
                v = 127;
            q[i * QK_K + j] = (int8_t)v;
        }
        d[i] = 1.0f / iscale;
    }
}

/* ---- Q4_K scale/min unpack --------------------------------------------- */

/* src/tensor/mod.rs:5997-6006 (q4_k_scale_min); same values as the kmask form
 * at src/inference.rs:25829-25861. */
static void q4_k_scale_min(int idx, const uint8_t *scales, uint8_t *sc, uint8_t *m) {
    if (idx < 4) {
        *sc = scales[idx] & 63;
        *m = scales[idx + 4] & 63;
    } else {
        *sc = (uint8_t)((scales[idx + 4] & 0x0f) | ((scales[idx - 4] >> 6) << 4));
        *m = (uint8_t)((scales[idx + 4] >> 4) | ((scales[idx] >> 6) << 4));
    }
}

/* Signed 6-bit weights of one Q6_K super-block, in value order:
 * src/inference.rs:25546-25566. */
static void q6_k_rebuild(const uint8_t *block, int8_t *a) {
    const uint8_t *ql = block;
    const uint8_t *qh = block + 128;
    int w = 0;
    for (int half = 0; half < 2; half++) {
        for (int l = 0; l < 32; l++) {
            a[w + l] = (int8_t)(((ql[l] & 0xF) | ((qh[l] & 3) << 4)) - 32);
            a[w + l + 32] = (int8_t)(((ql[l + 32] & 0xF) | (((qh[l] >> 2) & 3) << 4)) - 32);
            a[w + l + 64] = (int8_t)(((ql[l] >> 4) | (((qh[l] >> 4) & 3) << 4)) - 32);
            a[w + l + 96] = (int8_t)(((ql[l + 32] >> 4) | (((qh[l] >> 6) & 3) << 4)) - 32);
        }
        w += 128;
        ql += 64;
        qh += 32;
    }
}

/* ---- dequantizers ------------------------------------------------------- */

/* Q8_0: src/tensor/mod.rs:5365-5378 (scale * q). */
static void dequant_q8_0(const uint8_t *blk, float *out) {
    float scale = wire_f16(blk);
    for (int j = 0; j < 32; j++)
        out[j] = scale * (float)(int8_t)blk[2 + j];
}

/* Q4_0: src/inference.rs:25698-25708 ((nib - 8) as f32 * scale). */
static void dequant_q4_0(const uint8_t *blk, float *out) {
    float scale = wire_f16(blk);
    for (int j = 0; j < 16; j++) {
        uint8_t byte = blk[2 + j];
        out[j] = (float)((int)(byte & 0x0F) - 8) * scale;
        out[j + 16] = (float)((int)(byte >> 4) - 8) * scale;
    }
}

/* Q4_K: src/tensor/mod.rs:5903-5924: (d*sc)*q - (dmin*m), three roundings. */
static void dequant_q4_k(const uint8_t *blk, float *out) {
    float d = wire_f16(blk);
    float d_min = wire_f16(blk + 2);
    const uint8_t *scales = blk + 4;
    const uint8_t *values = blk + 16;
    for (int pair = 0; pair < 4; pair++) {
        uint8_t ls, lm, hs, hm;
        q4_k_scale_min(pair * 2, scales, &ls, &lm);
        q4_k_scale_min(pair * 2 + 1, scales, &hs, &hm);
        float low_scale = d * (float)ls;
        float high_scale = d * (float)hs;
        float low_min = d_min * (float)lm;
        float high_min = d_min * (float)hm;
        for (int l = 0; l < 32; l++) {
            uint8_t byte = values[pair * 32 + l];
            out[pair * 64 + l] = low_scale * (float)(byte & 0x0f) - low_min;
            out[pair * 64 + 32 + l] = high_scale * (float)(byte >> 4) - high_min;
        }
    }
}

/* Q6_K: src/tensor/mod.rs:6039-6066 == src/inference.rs:25496-25527:
 * (d * sc) * q. */
static void dequant_q6_k(const uint8_t *blk, float *out) {
    float d = wire_f16(blk + 208);
    int8_t a[QK_K];
    q6_k_rebuild(blk, a);
    const int8_t *sc = (const int8_t *)(blk + 192);
    for (int half = 0; half < 2; half++) {
        for (int l = 0; l < 32; l++) {
            int is = l / 16;
            int y = half * 128;
            const int8_t *s = sc + half * 8;
            out[y + l] = d * (float)s[is] * (float)a[y + l];
            out[y + l + 32] = d * (float)s[is + 2] * (float)a[y + l + 32];
            out[y + l + 64] = d * (float)s[is + 4] * (float)a[y + l + 64];
            out[y + l + 96] = d * (float)s[is + 6] * (float)a[y + l + 96];
        }
    }
}

void orc_dequant(int fmt, const uint8_t *wire, size_t n_blocks, float *out) {
    int bv = orc_block_values(fmt), bb = orc_block_bytes(fmt);
    for (size_t b = 0; b < n_blocks; b++) {
        const uint8_t *blk = wire + b * (size_t)bb;
        float *o = out + b * (size_t)bv;
        switch (fmt) {
        case ORC_Q8_0:
            dequant_q8_0(blk, o);
            break;
        case ORC_Q4_0:
            dequant_q4_0(blk, o);
            break;
        case ORC_Q4_K:
            dequant_q4_k(blk, o);
            break;
        case ORC_Q6_K:
            dequant_q6_k(blk, o);
            break;
        default:
            return;
        }
    }
}

/* ---- row dots ----------------------------------------------------------- */

/* src/inference.rs:22729-22745: total += (isum as f32 * scale) * x_scale. */
float orc_q8_0_row_dot(const uint8_t *w, const float *xs, const int8_t *xq, size_t n_blocks) {
    float total = 0.0f;
    for (size_t b = 0; b < n_blocks; b++) {
        const uint8_t *blk = w + b * 34;
        float scale = wire_f16(blk);
        int32_t isum = 0;
        for (int j = 0; j < 32; j++)
            isum += (int32_t)(int8_t)blk[2 + j] * (int32_t)xq[b * 32 + j];
        total += (float)isum * scale * xs[b];
    }
    return total;
}

/* src/inference.rs:22778-22798. */
float orc_q4_0_row_dot(const uint8_t *w, const float *xs, const int8_t *xq, size_t n_blocks) {
    float total = 0.0f;
    for (size_t b = 0; b < n_blocks; b++) {
        const uint8_t *blk = w + b * 18;
        float scale = wire_f16(blk);
        int32_t isum = 0;
        for (int j = 0; j < 16; j++) {
            uint8_t byte = blk[2 + j];
            int32_t lo = (int32_t)(byte & 0x0F) - 8;
            int32_t hi = (int32_t)(byte >> 4) - 8;
            isum += lo * (int32_t)xq[b * 32 + j];
            isum += hi * (int32_t)xq[b * 32 + j + 16];
        }
        total += (float)isum * scale * xs[b];
    }
    return total;
}

/* Exact integers of one Q4_K super-block against one Q8_K super-block:
 * *main = sum_g sc_g * (sum_t q*y), *mins = sum_g m_g * (sum_t y). */
static void q4_k_block_ints(const uint8_t *blk, const int8_t *y, int64_t *main_sum, int64_t *mins_sum) {
    const uint8_t *scales = blk + 4;
    const uint8_t *qs = blk + 16;
    int64_t prod = 0, s = 0;
    for (int g = 0; g < 8; g++) {
        uint8_t sc, m;
        q4_k_scale_min(g, scales, &sc, &m);
        int32_t bs = 0;
        for (int t = 0; t < 32; t++)
            bs += y[g * 32 + t];
        prod += (int64_t)bs * m;
        const uint8_t *q4 = qs + (g / 2) * 32;
        int64_t dot = 0;
        for (int t = 0; t < 32; t++) {
            int32_t q = (g & 1) ? (q4[t] >> 4) : (q4[t] & 0xf);
            dot += (int64_t)q * y[g * 32 + t];
        }
        s += dot * sc;
    }
    *main_sum = s;
    *mins_sum = prod;
}

/* src/diffusion_gemma/refmath.rs:504-562 (q4_k_dot_scalar, the body behind
 * q4_k_dot_arm): d and dmin are each multiplied by y.d first, then two fused
 * multiply-adds per super-block on one accumulator. */
float orc_q4_k_row_dot_arm(const uint8_t *w, const float *xd, const int8_t *xq, size_t n_sb) {
    float sumf = 0.0f;
    for (size_t i = 0; i < n_sb; i++) {
        const uint8_t *blk = w + i * 144;
        float d = xd[i] * wire_f16(blk);
        float dmin = xd[i] * wire_f16(blk + 2);
        int64_t s, prod;
        q4_k_block_ints(blk, xq + i * QK_K, &s, &prod);
        sumf = fmaf(-dmin, (float)prod, sumf);
        sumf = fmaf(d, (float)s, sumf);
    }
    return sumf;
}

/* src/inference.rs:25806-25889 (q4_k_wire_row_dot): 8 integer lanes by value
 * index mod 8, 8 f32 lane accumulators + 1 mins accumulator, no fusing. */
float orc_q4_k_row_dot_generic(const uint8_t *w, const float *xd, const int8_t *xq, size_t n_sb) {
    float sums[8] = {0};
    float sumf = 0.0f;
    for (size_t i = 0; i < n_sb; i++) {
        const uint8_t *blk = w + i * 144;
        const int8_t *y = xq + i * QK_K;
        float d = wire_f16(blk);
        float dmin = wire_f16(blk + 2);
        const uint8_t *qs = blk + 16;
        int8_t a[QK_K];
        for (int j = 0; j < 4; j++) {
            for (int l = 0; l < 32; l++) {
                a[j * 64 + l] = (int8_t)(qs[j * 32 + l] & 0xF);
                a[j * 64 + 32 + l] = (int8_t)(qs[j * 32 + l] >> 4);
            }
        }
        uint8_t scales[8], mins[8];
        for (int g = 0; g < 8; g++)
            q4_k_scale_min(g, blk + 4, &scales[g], &mins[g]);
        int32_t sumi = 0;
        for (int j = 0; j < 16; j++) {
            int32_t bsum = 0;
            for (int t = 0; t < 16; t++)
                bsum += y[j * 16 + t];
            sumi += bsum * (int32_t)mins[j / 2];
        }
        int32_t aux32[8] = {0};
        for (int j = 0; j < 8; j++) {
            int32_t scale = scales[j];
            for (int k = 0; k < 4; k++) {
                int off = j * 32 + k * 8;
                for (int l = 0; l < 8; l++)
                    aux32[l] += scale * (int32_t)y[off + l] * (int32_t)a[off + l];
            }
        }
        float dd = d * xd[i];
        for (int l = 0; l < 8; l++)
            sums[l] += dd * (float)aux32[l];
        sumf -= dmin * xd[i] * (float)sumi;
    }
    float lanes = 0.0f;
    for (int l = 0; l < 8; l++)
        lanes += sums[l];
    return sumf + lanes;
}

/* src/inference.rs:25535-25581 (q6_k_wire_row_dot): 8 lanes by value index
 * mod 8 within each 16-group, d = d_w * y.d, sequential final fold. */
float orc_q6_k_row_dot_lanes(const uint8_t *w, const float *xd, const int8_t *xq, size_t n_sb) {
    float sums[8] = {0};
    for (size_t i = 0; i < n_sb; i++) {
        const uint8_t *blk = w + i * 210;
        const int8_t *y = xq + i * QK_K;
        float d = wire_f16(blk + 208) * xd[i];
        int8_t a[QK_K];
        q6_k_rebuild(blk, a);
        int32_t aux32[8] = {0};
        for (int j = 0; j < 16; j++) {
            int32_t scale = (int8_t)blk[192 + j];
            int off = j * 16;
            for (int l = 0; l < 8; l++)
                aux32[l] += scale * (int32_t)y[off + l] * (int32_t)a[off + l];
            for (int l = 0; l < 8; l++)
                aux32[l] += scale * (int32_t)y[off + 8 + l] * (int32_t)a[off + 8 + l];
        }
        for (int l = 0; l < 8; l++)
            sums[l] += d * (float)aux32[l];
    }
    float total = 0.0f;
    for (int l = 0; l < 8; l++)
        total += sums[l];
    return total;
}

/* src/diffusion_gemma/refmath.rs:678-721 (q6_k_dot_scalar behind
 * q6_k_dot_arm): unsigned 6-bit dot, the -32 bias folded out through the
 * per-16 activation sums, one fused chain. */
float orc_q6_k_row_dot_arm(const uint8_t *w, const float *xd, const int8_t *xq, size_t n_sb) {
    float sum = 0.0f;
    for (size_t i = 0; i < n_sb; i++) {
        const uint8_t *blk = w + i * 210;
        const int8_t *y = xq + i * QK_K;
        float d_all = wire_f16(blk + 208);
        const uint8_t *ql = blk;
        const uint8_t *qh = blk + 128;
        const int8_t *scales = (const int8_t *)(blk + 192);
        int64_t isum_mins = 0;
        for (int t = 0; t < 16; t++) {
            int32_t bs = 0;
            for (int k = 0; k < 16; k++)
                bs += y[t * 16 + k];
            isum_mins += (int64_t)bs * scales[t];
        }
        int64_t isum = 0;
        for (int half = 0; half < 2; half++) {
            const uint8_t *qlh = ql + half * 64;
            const uint8_t *qhh = qh + half * 32;
            const int8_t *q8 = y + half * 128;
            const int8_t *sc = scales + half * 8;
            int64_t group_sums[8] = {0};
            for (int l = 0; l < 32; l++) {
                int64_t v0 = (qlh[l] & 0xf) | ((qhh[l] & 3) << 4);
                int64_t v1 = (qlh[32 + l] & 0xf) | (((qhh[l] >> 2) & 3) << 4);
                int64_t v2 = (qlh[l] >> 4) | (((qhh[l] >> 4) & 3) << 4);
                int64_t v3 = (qlh[32 + l] >> 4) | (((qhh[l] >> 6) & 3) << 4);
                group_sums[l / 16] += v0 * q8[l];
                group_sums[2 + l / 16] += v1 * q8[32 + l];
                group_sums[4 + l / 16] += v2 * q8[64 + l];
                group_sums[6 + l / 16] += v3 * q8[96 + l];
            }
            for (int g = 0; g < 8; g++)
                isum += group_sums[g] * sc[g];
        }
        sum = fmaf(d_all * xd[i], (float)(isum - 32 * isum_mins), sum);
    }
    return sum;
}

void orc_row_block_ints(int fmt, const uint8_t *w, const int8_t *xq, size_t n_blocks, int32_t *out) {
    for (size_t b = 0; b < n_blocks; b++) {
        switch (fmt) {
        case ORC_Q8_0: {
            const uint8_t *blk = w + b * 34;
            int32_t isum = 0;
            for (int j = 0; j < 32; j++)
                isum += (int32_t)(int8_t)blk[2 + j] * (int32_t)xq[b * 32 + j];
            out[b] = isum;
            break;
        }
        case ORC_Q4_0: {
            const uint8_t *blk = w + b * 18;
            int32_t isum = 0;
            for (int j = 0; j < 16; j++) {
                isum += ((int32_t)(blk[2 + j] & 0x0F) - 8) * (int32_t)xq[b * 32 + j];
                isum += ((int32_t)(blk[2 + j] >> 4) - 8) * (int32_t)xq[b * 32 + j + 16];
            }
            out[b] = isum;
            break;
        }
        case ORC_Q4_K: {
            int64_t s, prod;
            q4_k_block_ints(w + b * 144, xq + b * QK_K, &s, &prod);
            out[2 * b] = (int32_t)s;
            out[2 * b + 1] = (int32_t)prod;
            break;
        }
        case ORC_Q6_K: {
            const uint8_t *blk = w + b * 210;
            int8_t a[QK_K];
            q6_k_rebuild(blk, a);
            int64_t total = 0;
            for (int j = 0; j < 16; j++) {
                int32_t scale = (int8_t)blk[192 + j];
                int32_t dot = 0;
                for (int l = 0; l < 16; l++)
                    dot += (int32_t)xq[b * QK_K + j * 16 + l] * (int32_t)a[j * 16 + l];
                total += (int64_t)scale * dot;
            }
            out[b] = (int32_t)total;
            break;
        }
        default:
            return;
        }
    }
}

/* ---- drivers ------------------------------------------------------------ */

static int is_k_family(int fmt) { return fmt == ORC_Q4_K || fmt == ORC_Q6_K; }

static float row_dot(int fmt, int order, const uint8_t *w, const float *xs, const int8_t *xq, size_t nb) {
    switch (fmt) {
    case ORC_Q8_0:
        return orc_q8_0_row_dot(w, xs, xq, nb);
    case ORC_Q4_0:
        return orc_q4_0_row_dot(w, xs, xq, nb);
    case ORC_Q4_K:
        return order == ORC_ORDER_PRIMARY ? orc_q4_k_row_dot_arm(w, xs, xq, nb)
                                          : orc_q4_k_row_dot_generic(w, xs, xq, nb);
    case ORC_Q6_K:
        return order == ORC_ORDER_PRIMARY ? orc_q6_k_row_dot_lanes(w, xs, xq, nb)
                                          : orc_q6_k_row_dot_arm(w, xs, xq, nb);
    default:
        return 0.0f;
    }
}

struct matmul_job {
    int fmt, order;
    const uint8_t *wire;
    size_t row_bytes, nb, cols, row_start, rows, n_tokens;
    const float *xscales;
    const int8_t *xq;
    float *out;
    size_t next_chunk; /* handed out with __atomic_fetch_add */
};

#define ROW_CHUNK 64 /* src/gemma4_runtime.rs:923 */

/* src/gemma4_runtime.rs:1006-1050 / 1115-1150: the weight row is read once and
 * dotted against every activation; each cell is the single-row dot. */
static void *matmul_worker(void *arg) {
    struct matmul_job *job = (struct matmul_job *)arg;
    size_t n_chunks = (job->rows + ROW_CHUNK - 1) / ROW_CHUNK;
    for (;;) {
        size_t c = __atomic_fetch_add(&job->next_chunk, 1, __ATOMIC_RELAXED);
        if (c >= n_chunks)
            break;
        size_t lo = c * ROW_CHUNK;
        size_t hi = lo + ROW_CHUNK < job->rows ? lo + ROW_CHUNK : job->rows;
        for (size_t r = lo; r < hi; r++) {
            const uint8_t *w = job->wire + (job->row_start + r) * job->row_bytes;
            for (size_t t = 0; t < job->n_tokens; t++) {
                job->out[t * job->rows + r] =
                    row_dot(job->fmt, job->order, w, job->xscales + t * job->nb,
                            job->xq + t * job->cols, job->nb);
            }
        }
    }
    return NULL;
}

int orc_matmul_q(int fmt, int order, const uint8_t *wire, size_t cols,
                 size_t row_start, size_t rows,
                 const float *xscales, const int8_t *xq, size_t n_tokens,
                 float *out, int threads) {
    int bv = orc_block_values(fmt);
    if (bv == 0 || cols % (size_t)bv != 0)
        return -1;
    struct matmul_job job;
    job.fmt = fmt;
    job.order = order;
    job.wire = wire;
    job.nb = cols / (size_t)bv;
    job.row_bytes = job.nb * (size_t)orc_block_bytes(fmt);
    job.cols = cols;
    job.row_start = row_start;
    job.rows = rows;
    job.n_tokens = n_tokens;
    job.xscales = xscales;
    job.xq = xq;
    job.out = out;
    job.next_chunk = 0;
    if (threads <= 1) {
        matmul_worker(&job);
        return 0;
    }
    if (threads > 256)
        threads = 256;
    pthread_t tid[256];
    int started = 0;
    for (int i = 0; i < threads - 1; i++) {
        if (pthread_create(&tid[started], NULL, matmul_worker, &job) == 0)
            started++;
    }
    matmul_worker(&job);
    for (int i = 0; i < started; i++)
        pthread_join(tid[i], NULL);
    return 0;
}

int orc_matmul(int fmt, int order, const uint8_t *wire, size_t cols,
               size_t row_start, size_t rows,
               const float *x, size_t n_tokens, float *out, int threads) {
    int bv = orc_block_values(fmt);
    if (bv == 0 || cols % (size_t)bv != 0)
        return -1;
    size_t nb = cols / (size_t)bv;
    float *xs = (float *)malloc(sizeof(float) * nb * n_tokens + 4);
    int8_t *xq = (int8_t *)malloc(cols * n_tokens + 4);
    if (!xs || !xq) {
        free(xs);
        free(xq);
        return -2;
    }
    for (size_t t = 0; t < n_tokens; t++) {
        if (is_k_family(fmt))
            orc_quantize_q8_k(x + t * cols, cols, xs + t * nb, xq + t * cols);
        else
            orc_quantize_q8_0(x + t * cols, cols, xs + t * nb, xq + t * cols);
    }
    int rc = orc_matmul_q(fmt, order, wire, cols, row_start, rows, xs, xq, n_tokens, out, threads);
    free(xs);
    free(xq);
    return rc;
}

/* ---- mixture of experts -------------------------------------------------- */

/* f32::total_cmp key (src/inference.rs:13950-13955 sorts with it). */
static int32_t total_key(float v) {
    int32_t b = (int32_t)f32_bits(v);
    return b ^ (int32_t)(((uint32_t)(b >> 31)) >> 1);
}

struct pair {
    int32_t idx;
    float v;
};

/* Descending by value under total_cmp, ascending by index; insertion sort is
 * stable and the keys are unique by index, so any correct sort agrees. */
static void sort_desc(struct pair *p, int n) {
    for (int i = 1; i < n; i++) {
        struct pair cur = p[i];
        int j = i - 1;
        while (j >= 0) {
            int32_t kc = total_key(cur.v), kj = total_key(p[j].v);
            int before = (kc > kj) || (kc == kj && cur.idx < p[j].idx);
            if (!before)
                break;
            p[j + 1] = p[j];
            j--;
        }
        p[j + 1] = cur;
    }
}

/* src/inference.rs:13940-13991. */
int orc_softmax_top_k(const float *logits, int n, int k, int32_t *idx, float *w) {
    if (n <= 0 || k <= 0)
        return 0;
    struct pair *sel = (struct pair *)malloc(sizeof(struct pair) * (size_t)n);
    if (!sel)
        return 0;
    for (int i = 0; i < n; i++) {
        sel[i].idx = i;
        sel[i].v = logits[i];
    }
    sort_desc(sel, n);
    int kk = k < n ? k : n;
    float max = -INFINITY;
    for (int i = 0; i < kk; i++)
        max = fmaxf(max, sel[i].v);
    float sum = 0.0f;
    for (int i = 0; i < kk; i++) {
        float v = sel[i].v;
        sel[i].v = isfinite(v) ? expf(v - max) : 0.0f;
        sum += sel[i].v;
    }
    if (sum > 0.0f) {
        for (int i = 0; i < kk; i++)
            sel[i].v /= sum;
    } else {
        float uniform = 1.0f / (float)kk;
        for (int i = 0; i < kk; i++)
            sel[i].v = uniform;
    }
    sort_desc(sel, kk);
    for (int i = 0; i < kk; i++) {
        idx[i] = sel[i].idx;
        w[i] = sel[i].v;
    }
    free(sel);
    return kk;
}

/* Gemma-4 routing: src/gemma4_runtime.rs:5567-5580 (softmax over ALL experts: max folded
 * from f32::MIN, exp(v - max), sequential sum, p /= sum), router_top_k :61-84 (top-k by
 * probability, descending, ties to the lower index), route scale = down_scale[e] *
 * (p[e] / max(sum of the selected p in selection order, 6.103515e-5)) (:5580-5610). */
int orc_router_softmax_top_k(const float *logits, int n, int k, const float *down_scale, int32_t *idx, float *scale) {
    if (n <= 0 || k <= 0)
        return 0;
    float *p = (float *)malloc(sizeof(float) * (size_t)n);
    if (!p)
        return 0;
    float maxl = -FLT_MAX;
    for (int i = 0; i < n; i++)
        maxl = fmaxf(maxl, logits[i]);
    float sum = 0.0f;
    for (int i = 0; i < n; i++) {
        p[i] = expf(logits[i] - maxl);
        sum += p[i];
    }
    for (int i = 0; i < n; i++)
        p[i] /= sum;
    int keep = k < n ? k : n, len = 0;
    for (int c = 0; c < n; c++) {
        /* first position whose occupant ranks after the candidate: lower probability, or equal and a higher index */
        int at = -1;
        for (int j = 0; j < len; j++) {
            int cur = idx[j];
            if (p[cur] < p[c] || (p[cur] == p[c] && c < cur)) {
                at = j;
                break;
            }
        }
        if (at >= 0 && at < keep) {
            int last = len < keep ? len : keep - 1;
            for (int j = last; j > at; j--)
                idx[j] = idx[j - 1];
            idx[at] = c;
            if (len < keep)
                len++;
        } else if (at < 0 && len < keep) {
            idx[len++] = c;
        }
    }
    float wsum = 0.0f;
    for (int s = 0; s < len; s++)
        wsum += p[idx[s]];
    wsum = fmaxf(wsum, 6.103515e-5f);
    for (int s = 0; s < len; s++) {
        float ds = down_scale ? down_scale[idx[s]] : 1.0f;
        scale[s] = ds * (p[idx[s]] / wsum);
    }
    free(p);
    return len;
}

/* gelu_pytorch_tanh(g) * u: src/gemma4_mtp.rs:172-175 and src/gemma4_runtime.rs:5689-5691:
 * 0.5 * x * (1 + tanh(C * (x + 0.044715 * x * x * x))), C = 0.7978846, evaluated left to right. */
void orc_gelu_tanh_mul(const float *a, const float *b, size_t n, float *out) {
    const float C = 0.7978846f;
    for (size_t i = 0; i < n; i++) {
        float x = a[i];
        float cube = ((0.044715f * x) * x) * x;
        float g = (0.5f * x) * (1.0f + tanhf(C * (x + cube)));
        out[i] = g * b[i];
    }
}

/* src/tensor/mod.rs:2624: (a / (1.0 + (-a).exp())) * b. */
void orc_silu_mul(const float *a, const float *b, size_t n, float *out) {
    for (size_t i = 0; i < n; i++)
        out[i] = (a[i] / (1.0f + expf(-a[i]))) * b[i];
}

/* src/tensor/mod.rs:2707-2760 (the portable branch): per row, the squares are summed
 * left to right in f32, mean = sum / cols, scale = 1 / sqrt(mean + eps),
 * out = (x * scale) * weight. */
void orc_rms_norm(const float *x, const float *weight, float eps, size_t rows, size_t cols, float *out) {
    for (size_t r = 0; r < rows; r++) {
        const float *in = x + r * cols;
        float sum = 0.0f;
        for (size_t c = 0; c < cols; c++)
            sum = sum + in[c] * in[c];
        float mean_square = sum / (float)cols;
        float scale = 1.0f / sqrtf(mean_square + eps);
        for (size_t c = 0; c < cols; c++)
            out[r * cols + c] = (in[c] * scale) * weight[c];
    }
}

/* src/inference.rs:14142-14280 with quantized expert bands
 * (src/gemma4_runtime.rs:1084-1110 for the band matvec). */
int orc_moe_ffn(int fmt, const uint8_t *gate, const uint8_t *up, const uint8_t *down,
                int n_experts, int top_k, size_t hidden, size_t ff,
                const float *logits, const float *x, size_t n_tokens,
                float *out, int threads) {
    return orc_moe_ffn_ex(fmt, fmt, gate, up, down, n_experts, top_k, hidden, ff, logits, x, n_tokens, out, threads, 0, NULL);
}

/* variant 0: Mixtral (softmax_top_k routing, silu).  variant 1: Gemma-4 (softmax over all experts,
 * route scales with down_scale, gelu_tanh; src/gemma4_runtime.rs:5550-5710).  up == NULL: `gate`
 * holds fused gate|up experts, 2*ff rows each (gate rows first), as the Gemma-4 lane stores them.
 * fmt is the format of gate / up, fmt_down that of down (each projection quantizes its activation
 * for its own format, as SharedActivation does). */
int orc_moe_ffn_ex(int fmt, int fmt_down, const uint8_t *gate, const uint8_t *up, const uint8_t *down,
                   int n_experts, int top_k, size_t hidden, size_t ff,
                   const float *logits, const float *x, size_t n_tokens,
                   float *out, int threads, int variant, const float *down_scale) {
    if (n_experts <= 0 || top_k <= 0)
        return -1;
    float *g = (float *)malloc(sizeof(float) * ff);
    float *u = (float *)malloc(sizeof(float) * ff);
    float *h = (float *)malloc(sizeof(float) * ff);
    float *y = (float *)malloc(sizeof(float) * hidden);
    int32_t *idx = (int32_t *)malloc(sizeof(int32_t) * (size_t)top_k);
    float *wt = (float *)malloc(sizeof(float) * (size_t)top_k);
    int rc = 0;
    if (!g || !u || !h || !y || !idx || !wt) {
        rc = -2;
        goto done;
    }
    for (size_t t = 0; t < n_tokens; t++) {
        float *o = out + t * hidden;
        for (size_t c = 0; c < hidden; c++)
            o[c] = 0.0f;
        int kk = variant == 1 ? orc_router_softmax_top_k(logits + t * (size_t)n_experts, n_experts, top_k, down_scale, idx, wt)
                              : orc_softmax_top_k(logits + t * (size_t)n_experts, n_experts, top_k, idx, wt);
        for (int s = 0; s < kk; s++) {
            size_t e = (size_t)idx[s];
            if (up) {
                rc |= orc_matmul(fmt, ORC_ORDER_PRIMARY, gate, hidden, e * ff, ff, x + t * hidden, 1, g, threads);
                rc |= orc_matmul(fmt, ORC_ORDER_PRIMARY, up, hidden, e * ff, ff, x + t * hidden, 1, u, threads);
            } else {
                rc |= orc_matmul(fmt, ORC_ORDER_PRIMARY, gate, hidden, e * 2 * ff, ff, x + t * hidden, 1, g, threads);
                rc |= orc_matmul(fmt, ORC_ORDER_PRIMARY, gate, hidden, e * 2 * ff + ff, ff, x + t * hidden, 1, u, threads);
            }
            if (variant == 1)
                orc_gelu_tanh_mul(g, u, ff, h);
            else
                orc_silu_mul(g, u, ff, h);
            rc |= orc_matmul(fmt_down, ORC_ORDER_PRIMARY, down, ff, e * hidden, hidden, h, 1, y, threads);
            for (size_t c = 0; c < hidden; c++)
                o[c] += y[c] * wt[s];
        }
    }
done:
    free(g);
    free(u);
    free(h);
    free(y);
    free(idx);
    free(wt);
    return rc;
}

/* ---- weight quantizers (synthetic inputs only) --------------------------- */

static void put_f16(uint8_t *dst, float v) {
    uint16_t h = orc_f32_to_f16_bits(v);
    dst[0] = (uint8_t)(h & 0xff);
    dst[1] = (uint8_t)(h >> 8);
}

static float clampf(float v, float lo, float hi) { return v < lo ? lo : (v > hi ? hi : v); }

/* src/quantize.rs:98-119. */
static void quantize_block_q8_0(const float *src, uint8_t *dst) {
    float amax = 0.0f;
    for (int i = 0; i < 32; i++) {
        float a = fabsf(src[i]);
        if (a > amax)
            amax = a;
    }
    float d = amax / 127.0f;
    float id = d != 0.0f ? 1.0f / d : 0.0f;
    put_f16(dst, d);
    for (int i = 0; i < 32; i++)
        dst[2 + i] = (uint8_t)(int8_t)clampf(roundf(src[i] * id), -128.0f, 127.0f);
}

/* src/quantize.rs:122-149. */
static void quantize_block_q4_0(const float *src, uint8_t *dst) {
    float amax = 0.0f, vmax = 0.0f;
    for (int i = 0; i < 32; i++) {
        float a = fabsf(src[i]);
        if (a > amax) {
            amax = a;
            vmax = src[i];
        }
    }
    float d = vmax / -8.0f;
    float id = d != 0.0f ? 1.0f / d : 0.0f;
    put_f16(dst, d);
    for (int i = 0; i < 16; i++) {
        int x0 = (int)(int8_t)clampf(roundf(src[i] * id), -8.0f, 7.0f) + 8;
        int x1 = (int)(int8_t)clampf(roundf(src[i + 16] * id), -8.0f, 7.0f) + 8;
        dst[2 + i] = (uint8_t)((x0 & 0x0F) | ((x1 & 0x0F) << 4));
    }
}

/* src/quantize.rs:152-244. */
static void quantize_block_q4_k(const float *src, uint8_t *dst) {
    float mins[8], maxs[8];
    for (int g = 0; g < 8; g++) {
        float mn = INFINITY, mx = -INFINITY;
        for (int i = 0; i < 32; i++) {
            float v = src[g * 32 + i];
            if (v < mn)
                mn = v;
            if (v > mx)
                mx = v;
        }
        mins[g] = mn;
        maxs[g] = mx;
    }
    float super_min = 0.0f, super_max = 0.0f;
    for (int g = 0; g < 8; g++) {
        float effective_min = fminf(mins[g], 0.0f);
        float group_scale = fmaxf(maxs[g] - effective_min, 0.0f) / 15.0f;
        if (group_scale > super_max)
            super_max = group_scale;
        float min_magnitude = fmaxf(-mins[g], 0.0f);
        if (min_magnitude > super_min)
            super_min = min_magnitude;
    }
    float d = super_max / 63.0f;
    float dmin = super_min / 63.0f;
    float id = d != 0.0f ? 1.0f / d : 0.0f;
    float idmin = dmin != 0.0f ? 1.0f / dmin : 0.0f;
    put_f16(dst, d);
    put_f16(dst + 2, dmin);
    uint8_t sc[8], m[8];
    for (int g = 0; g < 8; g++) {
        float effective_min = fminf(mins[g], 0.0f);
        float group_scale = fmaxf(maxs[g] - effective_min, 0.0f) / 15.0f;
        sc[g] = (uint8_t)clampf(roundf(group_scale * id), 0.0f, 63.0f);
        m[g] = (uint8_t)clampf(roundf(fmaxf(-mins[g], 0.0f) * idmin), 0.0f, 63.0f);
    }
    uint8_t packed[12] = {0};
    for (int g = 0; g < 4; g++) {
        packed[g] = sc[g] & 0x3f;
        packed[g + 4] = m[g] & 0x3f;
    }
    for (int g = 4; g < 8; g++) {
        packed[g - 4] |= (uint8_t)((sc[g] >> 4) << 6);
        packed[g] |= (uint8_t)((m[g] >> 4) << 6);
        packed[g + 4] = (uint8_t)((sc[g] & 0x0f) | ((m[g] & 0x0f) << 4));
    }
    memcpy(dst + 4, packed, 12);
    uint8_t quantized[8][32];
    for (int g = 0; g < 8; g++) {
        float sub_d = d * (float)sc[g];
        float sub_min = -(dmin * (float)m[g]);
        float sub_id = sub_d != 0.0f ? 1.0f / sub_d : 0.0f;
        for (int i = 0; i < 32; i++)
            quantized[g][i] = (uint8_t)clampf(roundf((src[g * 32 + i] - sub_min) * sub_id), 0.0f, 15.0f);
    }
    for (int pair = 0; pair < 4; pair++)
        for (int i = 0; i < 32; i++)
            dst[16 + pair * 32 + i] =
                (uint8_t)((quantized[pair * 2][i] & 0x0f) | (quantized[pair * 2 + 1][i] << 4));
}

/* No counterpart in the reference (it has no Q6_K quantizer): a plain
 * max-magnitude scheme that emits valid Q6_K super-blocks in the layout
 * q6_k_rebuild() decodes.  Per 16-group scale = max/-32; super scale
 * d = max|scale|/127 stored as f16; values re-quantized against f16(d)*sc. */
static void quantize_block_q6_k(const float *src, uint8_t *dst) {
    float gscale[16];
    float max_scale = 0.0f, max_abs_scale = 0.0f;
    for (int g = 0; g < 16; g++) {
        float amax = 0.0f, vmax = 0.0f;
        for (int i = 0; i < 16; i++) {
            float a = fabsf(src[g * 16 + i]);
            if (a > amax) {
                amax = a;
                vmax = src[g * 16 + i];
            }
        }
        gscale[g] = vmax / -32.0f;
        if (fabsf(gscale[g]) > max_abs_scale) {
            max_abs_scale = fabsf(gscale[g]);
            max_scale = gscale[g];
        }
    }
    memset(dst, 0, 210);
    if (max_abs_scale == 0.0f) {
        for (int i = 0; i < 128; i++)
            dst[i] = 0; /* low nibbles of 32 */
        for (int i = 0; i < 64; i++)
            dst[128 + i] = 0xAA; /* high bits of 32 (0b10) in each 2-bit field */
        return;
    }
    float iscale = -128.0f / max_scale;
    put_f16(dst + 208, 1.0f / iscale);
    float d = wire_f16(dst + 208);
    int8_t sc[16];
    uint8_t L[QK_K];
    for (int g = 0; g < 16; g++) {
        float s = clampf(roundf(iscale * gscale[g]), -128.0f, 127.0f);
        sc[g] = (int8_t)s;
        dst[192 + g] = (uint8_t)sc[g];
        float dd = d * (float)sc[g];
        for (int i = 0; i < 16; i++) {
            float q = dd != 0.0f ? roundf(src[g * 16 + i] / dd) : 0.0f;
            L[g * 16 + i] = (uint8_t)((int)clampf(q, -32.0f, 31.0f) + 32);
        }
    }
    uint8_t *ql = dst, *qh = dst + 128;
    for (int half = 0; half < 2; half++) {
        const uint8_t *Lh = L + half * 128;
        for (int l = 0; l < 32; l++) {
            uint8_t q1 = Lh[l], q2 = Lh[l + 32], q3 = Lh[l + 64], q4 = Lh[l + 96];
            ql[half * 64 + l] = (uint8_t)((q1 & 0xF) | ((q3 & 0xF) << 4));
            ql[half * 64 + l + 32] = (uint8_t)((q2 & 0xF) | ((q4 & 0xF) << 4));
            qh[half * 32 + l] =
                (uint8_t)((q1 >> 4) | ((q2 >> 4) << 2) | ((q3 >> 4) << 4) | ((q4 >> 4) << 6));
        }
    }
}

struct quant_job {
    int fmt;
    const float *src;
    uint8_t *dst;
    size_t n_blocks;
    size_t next;
};

static void *quant_worker(void *arg) {
    struct quant_job *job = (struct quant_job *)arg;
    size_t bv = (size_t)orc_block_values(job->fmt), bb = (size_t)orc_block_bytes(job->fmt);
    const size_t step = 1024;
    for (;;) {
        size_t lo = __atomic_fetch_add(&job->next, step, __ATOMIC_RELAXED);
        if (lo >= job->n_blocks)
            break;
        size_t hi = lo + step < job->n_blocks ? lo + step : job->n_blocks;
        for (size_t b = lo; b < hi; b++) {
            const float *s = job->src + b * bv;
            uint8_t *d = job->dst + b * bb;
            switch (job->fmt) {
            case ORC_Q8_0:
                quantize_block_q8_0(s, d);
                break;
            case ORC_Q4_0:
                quantize_block_q4_0(s, d);
                break;
            case ORC_Q4_K:
                quantize_block_q4_k(s, d);
                break;
            case ORC_Q6_K:
                quantize_block_q6_k(s, d);
                break;
            }
        }
    }
    return NULL;
}

int orc_quantize_weights(int fmt, const float *src, size_t n, uint8_t *dst, int threads) {
    int bv = orc_block_values(fmt);
    if (bv == 0 || n % (size_t)bv != 0)
        return -1;
    struct quant_job job = {fmt, src, dst, n / (size_t)bv, 0};
    if (threads <= 1) {
        quant_worker(&job);
        return 0;
    }
    if (threads > 64)
        threads = 64;
    pthread_t tid[64];
    int started = 0;
    for (int i = 0; i < threads - 1; i++)
        if (pthread_create(&tid[started], NULL, quant_worker, &job) == 0)
            started++;
    quant_worker(&job);
    for (int i = 0; i < started; i++)
        pthread_join(tid[i], NULL);
    return 0;
}
