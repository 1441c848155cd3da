// Host-side f32 -> GGUF block quantizers (Q8_0, Q4_0, Q4_K, plus a Q6_K encoder).
//
// These follow the reference's converter (src/quantize.rs:98-244) and exist so
// that a host can produce wire bytes "as the reference would" -- the benchmark
// uses them to turn seeded N(0, sigma) matrices into Q4_K / Q8_0 / Q4_0 weights.
// The reference has no Q6_K quantizer; the one here is a plain max-magnitude
// encoder that emits valid Q6_K super-blocks.  All arithmetic is f32 with every
// operation rounded on its own (compile with -ffp-contract=off).
#include <math.h>
#include <stdint.h>
#include <string.h>

#include <atomic>
#include <thread>
#include <vector>

#include "../../include/camelid_hip.h"

namespace {

// f32 -> f16 bits, round to nearest even (reference f32_to_f16_bits, src/inference.rs:27062-27096).
uint16_t f16_bits(float value) {
    uint32_t bits;
    memcpy(&bits, &value, 4);
    const uint16_t sign = static_cast<uint16_t>((bits >> 16) & 0x8000u);
    const int32_t exp = static_cast<int32_t>((bits >> 23) & 0xffu);
    const uint32_t mant = bits & 0x007fffffu;
    if (exp == 0xff) return static_cast<uint16_t>(sign | (mant == 0 ? 0x7c00u : 0x7e00u));
    const int32_t he = exp - 127 + 15;
    if (he >= 0x1f) return static_cast<uint16_t>(sign | 0x7c00u);
    if (he <= 0) {
        if (he < -10) return sign;
        const uint32_t m = mant | 0x00800000u;
        const uint32_t shift = static_cast<uint32_t>(14 - he);
        uint16_t hm = static_cast<uint16_t>(m >> shift);
        const uint32_t rb = 1u << (shift - 1);
        if ((m & rb) && ((m & (rb - 1)) || (hm & 1))) hm = static_cast<uint16_t>(hm + 1);
        return static_cast<uint16_t>(sign | hm);
    }
    uint16_t h = static_cast<uint16_t>(sign | (static_cast<uint16_t>(he) << 10) | static_cast<uint16_t>(mant >> 13));
    if ((mant & 0x1000u) && ((mant & 0x0fffu) || (h & 1))) h = static_cast<uint16_t>(h + 1);
    return h;
}

float f16_value(uint16_t h) {
    const uint32_t sign = static_cast<uint32_t>(h & 0x8000u) << 16;
    const uint32_t exp = (h & 0x7c00u) >> 10;
    uint32_t frac = h & 0x03ffu;
    uint32_t out;
    if (exp == 0) {
        if (frac == 0) {
            out = sign;
        } else {
            int e = -14;
            while (!(frac & 0x0400u)) { frac <<= 1; e--; }
            out = sign | (static_cast<uint32_t>(e + 127) << 23) | ((frac & 0x03ffu) << 13);
        }
    } else if (exp == 0x1f) {
        out = sign | 0x7f800000u | (frac << 13);
    } else {
        out = sign | ((exp + 112) << 23) | (frac << 13);
    }
    float v;
    memcpy(&v, &out, 4);
    return v;
}

void put_f16(uint8_t *dst, float v) {
    const uint16_t h = f16_bits(v);
    dst[0] = static_cast<uint8_t>(h & 0xff);
    dst[1] = static_cast<uint8_t>(h >> 8);
}

float clampf(float v, float lo, float hi) { return v < lo ? lo : (v > hi ? hi : v); }

// src/quantize.rs:98-119
void block_q8_0(const float *src, uint8_t *dst) {
    float amax = 0.0f;
    for (int i = 0; i < 32; i++) amax = fabsf(src[i]) > amax ? fabsf(src[i]) : amax;
    const float d = amax / 127.0f;
    const float id = d != 0.0f ? 1.0f / d : 0.0f;
    put_f16(dst, d);
    for (int i = 0; i < 32; i++) dst[2 + i] = static_cast<uint8_t>(static_cast<int8_t>(clampf(roundf(src[i] * id), -128.0f, 127.0f)));
}

// src/quantize.rs:122-149
void block_q4_0(const float *src, uint8_t *dst) {
    float amax = 0.0f, vmax = 0.0f;
    for (int i = 0; i < 32; i++) {
        if (fabsf(src[i]) > amax) { amax = fabsf(src[i]); vmax = src[i]; }
    }
    const float d = vmax / -8.0f;
    const float id = d != 0.0f ? 1.0f / d : 0.0f;
    put_f16(dst, d);
    for (int i = 0; i < 16; i++) {
        const int x0 = static_cast<int>(static_cast<int8_t>(clampf(roundf(src[i] * id), -8.0f, 7.0f))) + 8;
        const int x1 = static_cast<int>(static_cast<int8_t>(clampf(roundf(src[i + 16] * id), -8.0f, 7.0f))) + 8;
        dst[2 + i] = static_cast<uint8_t>((x0 & 0x0F) | ((x1 & 0x0F) << 4));
    }
}

// src/quantize.rs:152-244
void block_q4_k(const float *src, uint8_t *dst) {
    float mins[8], maxs[8];
    for (int g = 0; g < 8; g++) {
        float mn = INFINITY, mx = -INFINITY;
        for (int i = 0; i < 32; i++) {
            const float v = src[g * 32 + i];
            if (v < mn) mn = v;
            if (v > mx) mx = v;
        }
        mins[g] = mn;
        maxs[g] = mx;
    }
    float super_min = 0.0f, super_max = 0.0f;
    for (int g = 0; g < 8; g++) {
        const float gs = fmaxf(maxs[g] - fminf(mins[g], 0.0f), 0.0f) / 15.0f;
        if (gs > super_max) super_max = gs;
        const float mm = fmaxf(-mins[g], 0.0f);
        if (mm > super_min) super_min = mm;
    }
    const float d = super_max / 63.0f, dmin = super_min / 63.0f;
    const float id = d != 0.0f ? 1.0f / d : 0.0f;
    const float idmin = dmin != 0.0f ? 1.0f / dmin : 0.0f;
    put_f16(dst, d);
    put_f16(dst + 2, dmin);
    uint8_t sc[8], m[8];
    for (int g = 0; g < 8; g++) {
        const float gs = fmaxf(maxs[g] - fminf(mins[g], 0.0f), 0.0f) / 15.0f;
        sc[g] = static_cast<uint8_t>(clampf(roundf(gs * id), 0.0f, 63.0f));
        m[g] = static_cast<uint8_t>(clampf(roundf(fmaxf(-mins[g], 0.0f) * idmin), 0.0f, 63.0f));
    }
    uint8_t packed[12] = {0};
    for (int g = 0; g < 4; g++) {
        packed[g] = sc[g] & 0x3f;
        packed[g + 4] = m[g] & 0x3f;
    }
    for (int g = 4; g < 8; g++) {
        packed[g - 4] |= static_cast<uint8_t>((sc[g] >> 4) << 6);
        packed[g] |= static_cast<uint8_t>((m[g] >> 4) << 6);
        packed[g + 4] = static_cast<uint8_t>((sc[g] & 0x0f) | ((m[g] & 0x0f) << 4));
    }
    memcpy(dst + 4, packed, 12);
    uint8_t qv[8][32];
    for (int g = 0; g < 8; g++) {
        const float sub_d = d * static_cast<float>(sc[g]);
        const float sub_min = -(dmin * static_cast<float>(m[g]));
        const float sub_id = sub_d != 0.0f ? 1.0f / sub_d : 0.0f;
        for (int i = 0; i < 32; i++) qv[g][i] = static_cast<uint8_t>(clampf(roundf((src[g * 32 + i] - sub_min) * sub_id), 0.0f, 15.0f));
    }
    for (int pair = 0; pair < 4; pair++)
        for (int i = 0; i < 32; i++)
            dst[16 + pair * 32 + i] = static_cast<uint8_t>((qv[pair * 2][i] & 0x0f) | (qv[pair * 2 + 1][i] << 4));
}

// No counterpart in the reference.  Per 16-group scale = (value of largest
// magnitude) / -32; super scale d = (largest group scale) / -128 stored as f16;
// 8-bit group scales against d; values re-quantized against f16(d) * scale.
void block_q6_k(const float *src, uint8_t *dst) {
    float gscale[16], max_scale = 0.0f, max_abs = 0.0f;
    for (int g = 0; g < 16; g++) {
        float amax = 0.0f, vmax = 0.0f;
        for (int i = 0; i < 16; i++) {
            if (fabsf(src[g * 16 + i]) > amax) { amax = fabsf(src[g * 16 + i]); vmax = src[g * 16 + i]; }
        }
        gscale[g] = vmax / -32.0f;
        if (fabsf(gscale[g]) > max_abs) { max_abs = fabsf(gscale[g]); max_scale = gscale[g]; }
    }
    memset(dst, 0, 210);
    if (max_abs == 0.0f) {
        memset(dst + 128, 0xAA, 64);  // code 32 (= value 0): low nibble 0, high bits 0b10
        return;
    }
    const float iscale = -128.0f / max_scale;
    put_f16(dst + 208, 1.0f / iscale);
    const float d = f16_value(static_cast<uint16_t>(dst[208] | (dst[209] << 8)));
    uint8_t L[256];
    for (int g = 0; g < 16; g++) {
        const int8_t sc = static_cast<int8_t>(clampf(roundf(iscale * gscale[g]), -128.0f, 127.0f));
        dst[192 + g] = static_cast<uint8_t>(sc);
        const float dd = d * static_cast<float>(sc);
        for (int i = 0; i < 16; i++) {
            const float q = dd != 0.0f ? roundf(src[g * 16 + i] / dd) : 0.0f;
            L[g * 16 + i] = static_cast<uint8_t>(static_cast<int>(clampf(q, -32.0f, 31.0f)) + 32);
        }
    }
    for (int half = 0; half < 2; half++) {
        const uint8_t *Lh = L + half * 128;
        for (int l = 0; l < 32; l++) {
            const uint8_t q1 = Lh[l], q2 = Lh[l + 32], q3 = Lh[l + 64], q4 = Lh[l + 96];
            dst[half * 64 + l] = static_cast<uint8_t>((q1 & 0xF) | ((q3 & 0xF) << 4));
            dst[half * 64 + l + 32] = static_cast<uint8_t>((q2 & 0xF) | ((q4 & 0xF) << 4));
            dst[128 + half * 32 + l] = static_cast<uint8_t>((q1 >> 4) | ((q2 >> 4) << 2) | ((q3 >> 4) << 4) | ((q4 >> 4) << 6));
        }
    }
}

}  // namespace

namespace cml {

// In-memory Q8_0 blocks (36 bytes: f32 scale + 32 int8; reference Q8_0Block, src/tensor/mod.rs:
// 105-110) -> 34-byte wire blocks.  The scale must be a value an f16 holds exactly (it is whenever
// the blocks were decoded from a GGUF file); returns false at the first one that is not.
bool q8_0_blocks_to_wire(const uint8_t *blocks, size_t n_blocks, uint8_t *wire) {
    for (size_t i = 0; i < n_blocks; i++) {
        float scale;
        memcpy(&scale, blocks + i * 36, 4);
        const uint16_t h = f16_bits(scale);
        const float back = f16_value(h);
        if (memcmp(&back, &scale, 4) != 0 && !(back == 0.0f && scale == 0.0f)) return false;
        uint8_t *dst = wire + i * 34;
        dst[0] = static_cast<uint8_t>(h & 0xff);
        dst[1] = static_cast<uint8_t>(h >> 8);
        memcpy(dst + 2, blocks + i * 36 + 4, 32);
    }
    return true;
}

}  // namespace cml

extern "C" int cml_quantize_weights_host(int fmt, const float *src, size_t n_values, uint8_t *dst, int threads) {
    const int bv = cml_block_values(fmt), bb = cml_block_bytes(fmt);
    if (bv == 0) return CML_ERR_INVALID;
    if (n_values % static_cast<size_t>(bv) != 0) return CML_ERR_SHAPE;
    if ((!src || !dst) && n_values) return CML_ERR_INVALID;
    const size_t n_blocks = n_values / static_cast<size_t>(bv);
    std::atomic<size_t> next{0};
    auto work = [&]() {
        const size_t step = 1024;
        for (;;) {
            const size_t lo = next.fetch_add(step);
            if (lo >= n_blocks) break;
            const size_t hi = lo + step < n_blocks ? lo + step : n_blocks;
            for (size_t b = lo; b < hi; b++) {
                const float *s = src + b * bv;
                uint8_t *d = dst + b * bb;
                switch (fmt) {
                    case CML_Q8_0: block_q8_0(s, d); break;
                    case CML_Q4_0: block_q4_0(s, d); break;
                    case CML_Q4_K: block_q4_k(s, d); break;
                    default: block_q6_k(s, d); break;
                }
            }
        }
    };
    if (threads < 1) threads = 1;
    if (threads > 64) threads = 64;
    std::vector<std::thread> pool;
    for (int i = 1; i < threads; i++) pool.emplace_back(work);
    work();
    for (auto &t : pool) t.join();
    return CML_OK;
}
