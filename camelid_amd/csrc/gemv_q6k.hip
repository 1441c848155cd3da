// Q6_K x Q8_K fused dequantize + matvec / small-batch matmul for gfx950.
//
// Arithmetic.  Per 256-value super-block the exact integer
//     T = sum_{j<16} sc_j * sum_{k<16} a[16j+k] * y[16j+k],   a = 6-bit code - 32
// is what every variant of the reference computes (8 lane-wise pieces in
// q6_k_wire_row_dot, src/inference.rs:25535-25581; "isum - 32*isum_mins" in
// q6_k_dot_scalar, src/diffusion_gemma/refmath.rs:678-721).  The f32 step
// follows the fused single-chain form of the latter:
//     acc = fma(d_w * yd, (float)T, acc)      super-blocks in order.
// The 8-lane form differs from it only by f32 association and is matched
// within the 1e-5 relative tolerance, not bit for bit: its lanes split the 16
// values of a group by (index mod 8), which a 4-wide packed dot cannot keep apart.
//
// Mapping.  Plane layout ql | qh | scales | d.  Eight lanes own a super-block.
// Lane (half h, pair p, side s) loads ql[64h+32p+16s .. +16) and
// qh[32h+16s .. +16) with 128-bit loads: the low nibbles plus qh bits 2p,2p+1
// are values 128h+32p+16s+(0..15) (scale 8h+2p+s), the high nibbles plus qh
// bits 4+2p,5+2p are the values 64 further on (scale 8h+4+2p+s).  The codes are
// rebuilt as unsigned bytes, dotted against the LDS-staged activation with
// v_dot4_i32_i8, and the -32 bias is applied through per-16 activation sums.
#include "cml_device.hpp"
#include "cml_host.hpp"

#include <type_traits>

#pragma clang fp contract(off)

namespace cml {

// LDS written by some lanes of a wave and read by others of the same wave.
__device__ __forceinline__ void wave_barrier_lds() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

struct Q6KArgs {
    const uint8_t *ql, *qh, *sc, *d;
    int64_t ql_stride, qh_stride, sc_stride, d_stride;
    int rows, n_sb;
    const int8_t *q;
    const float *yd;
    const float *x;  // fused-quantizer launches: the NT f32 activation rows, contiguous
    float *out;
    const float *residual;
    int32_t *ints;  // [rows][n_sb] or null
    // Plain call: blockIdx.y = 0, the NT activation rows 0..NT-1 go to output rows 0..NT-1.
    // Grouped call (mixture of experts): y-slot -> group e = group_ids[y] (y itself when null; -1 =
    // unused slot), which owns the band of rows [e*rows, (e+1)*rows) and the assignments
    // [group_offsets[e], group_offsets[e+1]); assignment j reads activation row group_rows[j] (j
    // itself when null) and writes output row j, NT assignments per pass.
    // Direct call (single-token decode; group_offsets null, group_ids set): y-slot y IS assignment
    // y and group_ids[y] its expert; ids outside [0, n_groups) are skipped.
    const int32_t *group_offsets;
    const int32_t *group_rows;
    const int32_t *group_ids;
    int n_groups;
    int ksplit;       // 1, 2 or 4 waves per row tile
    int ksplit_log2;
};

// One f32 token against up to four Q6_K weights of one row length and one K cut (any row counts) in one launch of the
// one-workgroup-per-unit form: their workgroups lie end to end along grid.x, every workgroup quantizes the token once.
struct Q6KMultiArgs {
    Q6KArgs base;  // what the weights share (n_sb, x, ksplit)
    const uint8_t *qlm[4], *qhm[4], *scm[4], *dm[4];
    int64_t ql_stridem[4], qh_stridem[4], sc_stridem[4], d_stridem[4];
    float *outm[4];
    int rowsm[4];
    int wg_end[4];  // workgroups of weights 0 .. j (INT32_MAX beyond the last weight)
};

template <int U_>
struct Q6KRegs {
    static constexpr int U = U_;  // super-blocks in flight per buffer
    uint4 ql[U];
    uint4 qh[U];
    uint4 sc[U];
    uint32_t d[U];
};

template <int U>
__device__ __forceinline__ void q6k_load(Q6KRegs<U> &r, const uint8_t *ql, const uint8_t *qh, const uint8_t *sc,
                                         const uint8_t *d, int l, int sb, int s1) {
    const int h = l >> 2, p = (l >> 1) & 1, s = l & 1;
    // Unconditional, clamped loads (results past the end are discarded by the
    // caller) keep the loop body straight-line so loads stay in flight.
#pragma unroll
    for (int u = 0; u < U; u++) {
        const int64_t i = min(sb + u, s1 - 1);
        r.ql[u] = ldg16_stream(ql + i * 128 + 64 * h + 32 * p + 16 * s);
        // half a line per instruction (the other half belongs to the next super-block): the line
        // must stay cached in between, so no streaming hint here (128256 x 3072: 55.1 -> 49.7 us)
        r.qh[u] = ldg16(qh + i * 64 + 32 * h + 16 * s);
        r.sc[u] = ldg16(sc + i * 16);
        r.d[u] = ldg2(d + i * 2);
    }
}

template <int NT, bool INTS, int U>
__device__ __forceinline__ void q6k_compute(const Q6KRegs<U> &r, int l, int sb, int s1, const int8_t *ys,
                                            const int *bsum16, const float *yds, int n_sb, float (&acc)[NT],
                                            int32_t *ints_row) {
    const int h = l >> 2, p = (l >> 1) & 1, s = l & 1;
    const int g_lo = 8 * h + 2 * p + s;  // scale / 16-group index of the low-nibble values
#pragma unroll
    for (int u = 0; u < U; u++) {
        const bool valid = sb + u < s1;  // wave-uniform
        const int i = valid ? sb + u : s1 - 1;
        // scales: byte g_lo of the 16, and byte g_lo + 4
        const uint32_t w_lo = h ? r.sc[u].z : r.sc[u].x;
        const uint32_t w_hi = h ? r.sc[u].w : r.sc[u].y;
        const int sh = 8 * (2 * p + s);
        const int sc_lo = static_cast<int8_t>((w_lo >> sh) & 0xff);
        const int sc_hi = static_cast<int8_t>((w_hi >> sh) & 0xff);
        const uint32_t qlw[4] = {r.ql[u].x, r.ql[u].y, r.ql[u].z, r.ql[u].w};
        const uint32_t qhw[4] = {r.qh[u].x, r.qh[u].y, r.qh[u].z, r.qh[u].w};
        uint32_t vlo[4], vhi[4];
#pragma unroll
        for (int k = 0; k < 4; k++) {
            const uint32_t hp = qhw[k] >> (2 * p);  // p = 0: bits 0-1 / 4-5; p = 1: bits 2-3 / 6-7
            vlo[k] = (qlw[k] & 0x0f0f0f0fu) | ((hp << 4) & 0x30303030u);
            vhi[k] = ((qlw[k] >> 4) & 0x0f0f0f0fu) | (hp & 0x30303030u);
        }
        const float dw = f16_bits_to_f32(r.d[u]);
#pragma unroll
        for (int t = 0; t < NT; t++) {
            const int8_t *y = ys + (static_cast<int64_t>(t) * n_sb + i) * 256 + 128 * h + 32 * p + 16 * s;
            const uint4 ylo = *reinterpret_cast<const uint4 *>(y);
            const uint4 yhi = *reinterpret_cast<const uint4 *>(y + 64);
            int lo = sdot4(vlo[0], ylo.x, 0);
            lo = sdot4(vlo[1], ylo.y, lo);
            lo = sdot4(vlo[2], ylo.z, lo);
            lo = sdot4(vlo[3], ylo.w, lo);
            int hi = sdot4(vhi[0], yhi.x, 0);
            hi = sdot4(vhi[1], yhi.y, hi);
            hi = sdot4(vhi[2], yhi.z, hi);
            hi = sdot4(vhi[3], yhi.w, hi);
            const int *bs = bsum16 + (t * n_sb + i) * 16;
            lo -= 32 * bs[g_lo];
            hi -= 32 * bs[g_lo + 4];
            // |lo|, |hi| <= 16*63*127 + 32*16*127 and int8 scales: every product fits 24 bits (full-rate multiplies)
            int total = group_sum_to_last<8>(__mul24(lo, sc_lo) + __mul24(hi, sc_hi));
            total = valid ? total : 0;  // fma(x, 0, acc) leaves acc unchanged
            const float dd = dw * yds[t * n_sb + i];
            acc[t] = __builtin_fmaf(dd, static_cast<float>(total), acc[t]);
            if constexpr (INTS) {
                if (ints_row != nullptr && valid) ints_row[i] = total;
            }
        }
    }
}

// U = super-blocks per register buffer: 2, or 4 for weights with thousands of row tiles (an LM
// head), where the deeper queue per wave pays (128256 x 3072: 49.3 -> 47.1 us; at 4096 x 14336 it
// costs 1 us).
template <int NT, bool INTS, bool GROUPED = false, int U = 2, bool FUSEQ = false>
__global__ __launch_bounds__(256) void gemv_q6k_kernel(Q6KArgs a) {
    static_assert(!(GROUPED && INTS), "block-int diagnostics are for plain calls");
    static_assert(!FUSEQ || (NT <= 2 && !INTS && !GROUPED), "the fused quantizer serves plain calls of one or two tokens");
    constexpr int LPS = 8, RPW = kWave / LPS;
    extern __shared__ uint4 smem[];
    const int n_sb = a.n_sb;
    int8_t *ys = reinterpret_cast<int8_t *>(smem);                  // [NT][n_sb*256]
    int *bsum16 = reinterpret_cast<int *>(ys + NT * n_sb * 256);    // [NT][n_sb*16]
    float *yds = reinterpret_cast<float *>(bsum16 + NT * n_sb * 16);
    float *part = yds + ((NT * n_sb + 3) & ~3);

    const int tid = threadIdx.x;
    int64_t band = 0;
    int a0 = 0, n_assign = NT;
    if constexpr (GROUPED) {
        const bool direct = a.group_offsets == nullptr;
        band = a.group_ids ? a.group_ids[blockIdx.y] : static_cast<int>(blockIdx.y);
        if (band < 0 || band >= a.n_groups) return;  // an unused y-slot or an id out of range: the workgroup leaves together
        a0 = direct ? static_cast<int>(blockIdx.y) : a.group_offsets[band];
        n_assign = direct ? 1 : a.group_offsets[band + 1] - a0;
        if (n_assign <= 0) return;
    }

    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
    // the K split is a power of two: shifts, not divisions, on the way to the first load
    const int W = a.ksplit;
    const int tiles_per_wg = 4 >> a.ksplit_log2;
    const int tile_in_wg = wave >> a.ksplit_log2, kpart = wave & (W - 1);
    const int tile = blockIdx.x * tiles_per_wg + tile_in_wg;
    const int s0 = (kpart * n_sb) >> a.ksplit_log2;  // == kpart * n_sb / W
    const int s1 = ((kpart + 1) * n_sb) >> a.ksplit_log2;
    const int r = lane / LPS, l = lane - r * LPS;
    const int row = tile * RPW + r;
    const bool live = row < a.rows;
    const int64_t arow = band * a.rows + (live ? row : a.rows - 1);
    const uint8_t *ql = a.ql + arow * a.ql_stride;
    const uint8_t *qh = a.qh + arow * a.qh_stride;
    const uint8_t *sc = a.sc + arow * a.sc_stride;
    const uint8_t *dp = a.d + arow * a.d_stride;
    const bool leader = (l == LPS - 1);
    int32_t *ints_row = nullptr;
    if constexpr (INTS) {
        if (a.ints && leader && live) ints_row = a.ints + arow * static_cast<int64_t>(n_sb);
    }

    for (int p0 = 0; p0 < n_assign; p0 += NT) {
        // activation row of local token t (clamped to the group's last assignment; extra tokens store nothing)
        auto act_row = [&](int t) -> int64_t {
            const int j = a0 + min(p0 + t, n_assign - 1);
            return a.group_rows ? a.group_rows[j] : j;
        };
        if (p0 > 0) __syncthreads();  // the previous pass's readers are done
        Q6KRegs<U> ra, rb;
        bool ra_loaded = false;
        if constexpr (!GROUPED) {
            const uint4 *src = reinterpret_cast<const uint4 *>(a.q);
            uint4 *dst = reinterpret_cast<uint4 *>(ys);
            const int n16 = NT * n_sb * 16;
            if constexpr (FUSEQ) {
                // The activation arrives as f32 and every workgroup quantizes it to Q8_K itself (the
                // arithmetic of quantize_q8_k_kernel, a 16-lane row per super-block, four per wave
                // pass), under the first weight loads: no second launch, no trip through memory.
                // Two tokens are simply 2 * n_sb super-blocks in a row (rows and staging areas contiguous).
                const int tq = NT * n_sb;
                const int qrow = lane >> 4, ql16 = lane & 15;
                const float4 *x4 = reinterpret_cast<const float4 *>(a.x);
                auto load_pass = [&](float4 (&xv)[4], int base) {
                    const int sbk = min(base + qrow, tq - 1);
#pragma unroll
                    for (int k = 0; k < 4; k++) xv[k] = x4[sbk * 64 + ql16 * 4 + k];
                };
                auto quantize_pass = [&](const float4 (&xv)[4], int base) {
                    const int sbk = base + qrow;
                    float dv;
                    int bs;
                    const uint4 packed = q8k_quantize_row16(xv, lane, dv, bs);
                    if (sbk < tq) {
                        dst[sbk * 16 + ql16] = packed;
                        bsum16[sbk * 16 + ql16] = bytesum16(packed);
                        if (ql16 == 0) yds[sbk] = dv;
                    }
                };
                float4 xa[4];
                load_pass(xa, 4 * wave);
                __builtin_amdgcn_sched_barrier(0);
                q6k_load(ra, ql, qh, sc, dp, l, s0, s1);
                ra_loaded = true;
                __builtin_amdgcn_sched_barrier(0);
                for (int base = 4 * wave;;) {
                    quantize_pass(xa, base);
                    base += 16;
                    if (base >= tq) break;  // uniform per wave
                    load_pass(xa, base);
                }
            } else if (NT == 1 && n16 <= 4 * 256) {  // uniform
                // The activation loads go out first, the first weight buffer right behind them, and
                // only then is the activation written to LDS: the weight requests are in flight
                // while it is staged (a wave's loads return in order).
                uint4 sv[4];
#pragma unroll
                for (int k = 0; k < 4; k++) sv[k] = src[min(tid + k * 256, n16 - 1)];
                const float yd0 = a.yd[min(tid, n_sb - 1)];
                __builtin_amdgcn_sched_barrier(0);
                q6k_load(ra, ql, qh, sc, dp, l, s0, s1);
                ra_loaded = true;
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int k = 0; k < 4; k++) {
                    const int i = tid + k * 256;
                    if (i < n16) {
                        dst[i] = sv[k];
                        bsum16[i] = bytesum16(sv[k]);
                    }
                }
                if (tid < n_sb) yds[tid] = yd0;
                for (int i = tid + 256; i < n_sb; i += 256) yds[i] = a.yd[i];
            } else {
                for (int i = tid; i < n16; i += 256) {
                    const uint4 v = src[i];
                    dst[i] = v;
                    bsum16[i] = bytesum16(v);
                }
                for (int i = tid; i < NT * n_sb; i += 256) yds[i] = a.yd[i];
            }
        } else {
            uint4 *dst = reinterpret_cast<uint4 *>(ys);
            const int c16 = n_sb * 16;
            for (int i = tid; i < NT * c16; i += 256) {
                const int t = i / c16;
                const uint4 v = reinterpret_cast<const uint4 *>(a.q + act_row(t) * n_sb * 256)[i - t * c16];
                dst[i] = v;
                bsum16[i] = bytesum16(v);
            }
            for (int i = tid; i < NT * n_sb; i += 256) {
                const int t = i / n_sb;
                yds[i] = a.yd[act_row(t) * n_sb + (i - t * n_sb)];
            }
        }
        __syncthreads();
        float *out = a.out + static_cast<int64_t>(a0 + p0) * a.rows;
        const int n_here = GROUPED ? min(NT, n_assign - p0) : NT;

        float acc[NT];
#pragma unroll
        for (int t = 0; t < NT; t++) acc[t] = 0.0f;

        if (!ra_loaded) q6k_load(ra, ql, qh, sc, dp, l, s0, s1);
        __builtin_amdgcn_sched_barrier(0);
        // Two register buffers alternate; the last one is consumed without issuing
        // further loads.
        for (int sb = s0;;) {
            if (sb + U >= s1) {
                q6k_compute<NT, INTS, U>(ra, l, sb, s1, ys, bsum16, yds, n_sb, acc, ints_row);
                break;
            }
            q6k_load(rb, ql, qh, sc, dp, l, sb + U, s1);
            __builtin_amdgcn_sched_barrier(0);
            q6k_compute<NT, INTS, U>(ra, l, sb, s1, ys, bsum16, yds, n_sb, acc, ints_row);
            __builtin_amdgcn_sched_barrier(0);
            sb += U;
            if (sb + U >= s1) {
                q6k_compute<NT, INTS, U>(rb, l, sb, s1, ys, bsum16, yds, n_sb, acc, ints_row);
                break;
            }
            q6k_load(ra, ql, qh, sc, dp, l, sb + U, s1);
            __builtin_amdgcn_sched_barrier(0);
            q6k_compute<NT, INTS, U>(rb, l, sb, s1, ys, bsum16, yds, n_sb, acc, ints_row);
            __builtin_amdgcn_sched_barrier(0);
            sb += U;
        }

        if (W == 1) {
            if (leader && live) {
#pragma unroll
                for (int t = 0; t < NT; t++) {
                    if (t >= n_here) break;
                    float v = acc[t];
                    if (NT == 1 && a.residual) v = v + a.residual[row];
                    out[static_cast<int64_t>(t) * a.rows + row] = v;
                }
            }
            continue;
        }
        if (leader) {
#pragma unroll
            for (int t = 0; t < NT; t++) part[(wave * NT + t) * RPW + r] = acc[t];
        }
        __syncthreads();
        for (int i = tid; i < tiles_per_wg * NT * RPW; i += 256) {
            const int rr = i % RPW;
            const int t = (i / RPW) % NT;
            const int tw = i / (RPW * NT);
            const int orow = (blockIdx.x * tiles_per_wg + tw) * RPW + rr;
            if (orow >= a.rows || t >= n_here) continue;
            float v = part[((tw * W) * NT + t) * RPW + rr];
            for (int k = 1; k < W; k++) v = v + part[((tw * W + k) * NT + t) * RPW + rr];
            if (NT == 1 && a.residual) v = v + a.residual[orow];
            out[static_cast<int64_t>(t) * a.rows + orow] = v;
        }
    }
}

// ---- one token on a weight whose shape the policy cuts K for: eight-wave workgroups, one launch ----
//
// Few row tiles, long rows -- the FFN down projection in Q6_K (4096 x 14336: 56 super-blocks cut four ways).  The
// two-launch form (a quantizing launch, then gemv_q6k_kernel) takes 12.3 us per step for a 10.1 us matvec.  Here a
// workgroup's eight waves are 8 / KS row tiles (8 rows each) x KS parts of NSTEPS super-blocks; the arithmetic is
// q6k_load / q6k_compute, one super-block per step, and the KS partial chains of a row are added left to right
// through LDS -- the association of gemv_q6k_kernel under the same cut, so the same bits.  The workgroup quantizes
// the row ONCE, a 32-lane half wave per super-block, pass by pass ALONG the walk: pass p produces, for every K part,
// the four super-blocks its steps 4p .. 4p + 3 read (the part's two waves take two each), so the walk starts after
// one pass and the others run between steps, with a barrier ahead of the first step that reads a pass.  Every f32
// request is out before the first weight request (an execution barrier), and the weights stream through a ring of
// NB one-super-block buffers.
// ANY: the row length is the launch's (n_sb super-blocks, staged in dynamic LDS), the parts are those of
// gemv_q6k_kernel, [k n / KS, (k + 1) n / KS) -- unequal when KS does not divide n -- and NSTEPS is the longest part:
// steps past a shorter part's end re-read its last super-block and add nothing.
// NT = 2 (with ANY): two contiguous f32 rows in, out[2][rows]; every pass quantizes its super-blocks of both tokens and a
// step's unpacked weight is replayed against them -- each cell the one-token launch's bits.
template <int KS, int NSTEPS, int NB = 4, int WAVES = 8, bool ANY = false, int NT = 1, int U = 1, bool MULTI = false>
__global__ __launch_bounds__(WAVES * 64) void gemv_q6k_cu_kcut_kernel(std::conditional_t<MULTI, Q6KMultiArgs, Q6KArgs> a_in) {
    static_assert(!MULTI || (ANY && NT == 1), "the multi launch: the general form, one token");
    Q6KArgs a_sel;        // MULTI: the shared arguments with this workgroup's weight filled in
    int bx = blockIdx.x;  // workgroup index within its weight
    if constexpr (MULTI) {
        Q6KArgs &a = a_sel;
        a = a_in.base;
        // which weight this workgroup belongs to (wave-uniform selects: no indexed access to the argument block)
        const int j = (bx >= a_in.wg_end[0]) + (bx >= a_in.wg_end[1]) + (bx >= a_in.wg_end[2]);
        auto pick = [&](auto v0, auto v1, auto v2, auto v3) { return j == 0 ? v0 : (j == 1 ? v1 : (j == 2 ? v2 : v3)); };
        a.ql = pick(a_in.qlm[0], a_in.qlm[1], a_in.qlm[2], a_in.qlm[3]);
        a.qh = pick(a_in.qhm[0], a_in.qhm[1], a_in.qhm[2], a_in.qhm[3]);
        a.sc = pick(a_in.scm[0], a_in.scm[1], a_in.scm[2], a_in.scm[3]);
        a.d = pick(a_in.dm[0], a_in.dm[1], a_in.dm[2], a_in.dm[3]);
        a.ql_stride = pick(a_in.ql_stridem[0], a_in.ql_stridem[1], a_in.ql_stridem[2], a_in.ql_stridem[3]);
        a.qh_stride = pick(a_in.qh_stridem[0], a_in.qh_stridem[1], a_in.qh_stridem[2], a_in.qh_stridem[3]);
        a.sc_stride = pick(a_in.sc_stridem[0], a_in.sc_stridem[1], a_in.sc_stridem[2], a_in.sc_stridem[3]);
        a.d_stride = pick(a_in.d_stridem[0], a_in.d_stridem[1], a_in.d_stridem[2], a_in.d_stridem[3]);
        a.out = pick(a_in.outm[0], a_in.outm[1], a_in.outm[2], a_in.outm[3]);
        a.rows = pick(a_in.rowsm[0], a_in.rowsm[1], a_in.rowsm[2], a_in.rowsm[3]);
        bx -= pick(0, a_in.wg_end[0], a_in.wg_end[1], a_in.wg_end[2]);
    }
    const Q6KArgs &a = [&]() -> const Q6KArgs & {
        if constexpr (MULTI) return a_sel;
        else return a_in;
    }();
    constexpr int LPS = 8, RPW = kWave / LPS, TPW = WAVES / KS, PRE = 2;
    constexpr int PER_PASS = 2 * TPW;                       // super-blocks a pass gives every part
    constexpr int PASSES = (NSTEPS + PER_PASS - 1) / PER_PASS;
    constexpr int USTEPS = (NSTEPS + U - 1) / U;  // ring steps: U super-blocks of a row each
    static_assert(USTEPS >= NB && WAVES % KS == 0 && PER_PASS % U == 0, "K parts of at least one full ring; whole steps per quantizer pass");
    static_assert(NT == 1 || (ANY && NT == 2), "two tokens: the general form");
    const int NSB = ANY ? a.n_sb : KS * NSTEPS;
    __shared__ __attribute__((aligned(16))) int8_t ys_fixed[ANY ? 16 : KS * NSTEPS * 256];
    __shared__ int bsum16_fixed[ANY ? 1 : KS * NSTEPS * 16];
    __shared__ float yds_fixed[ANY ? 1 : KS * NSTEPS];
    __shared__ float part[WAVES * NT * RPW];
    extern __shared__ uint4 smem_q6k_any[];
    int8_t *ys = ANY ? reinterpret_cast<int8_t *>(smem_q6k_any) : ys_fixed;
    int *bsum16 = ANY ? reinterpret_cast<int *>(ys + NT * NSB * 256) : bsum16_fixed;
    float *yds = ANY ? reinterpret_cast<float *>(bsum16 + NT * NSB * 16) : yds_fixed;
    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
    const int tile_in_wg = wave / KS, kpart = wave - tile_in_wg * KS;
    const int s0 = ANY ? (kpart * NSB) / KS : kpart * NSTEPS;  // first super-block of this wave's part
    const int s1 = ANY ? ((kpart + 1) * NSB) / KS : s0 + NSTEPS;

    // the f32 activation: in pass p this wave's halves take super-blocks PER_PASS * p + 2 * tile_in_wg + {0, 1} of its part
    const int half = lane >> 5, ql32 = lane & 31;
    auto unit_of = [&](int p) __attribute__((always_inline)) -> int { return PER_PASS * p + 2 * tile_in_wg + half; };
    float4 xv[PASSES][NT][2];
#pragma unroll
    for (int p = 0; p < PASSES; p++) {
#pragma unroll
        for (int t = 0; t < NT; t++) {
            const float4 *x4 = reinterpret_cast<const float4 *>(a.x) + (t * NSB + min(s0 + unit_of(p), s1 - 1)) * 64 + ql32 * 2;
            xv[p][t][0] = x4[0];
            xv[p][t][1] = x4[1];
        }
    }
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_barrier();  // execution only: every activation request of the workgroup is out
    __builtin_amdgcn_sched_barrier(0);

    const int r = lane / LPS, l = lane - r * LPS;
    const int row = (bx * TPW + tile_in_wg) * RPW + r;
    const bool live = row < a.rows;
    const int64_t arow = live ? row : a.rows - 1;  // rows past the end (grid rounding) re-read the last row and store nothing
    const uint8_t *ql = a.ql + arow * a.ql_stride;
    const uint8_t *qh = a.qh + arow * a.qh_stride;
    const uint8_t *sc = a.sc + arow * a.sc_stride;
    const uint8_t *dp = a.d + arow * a.d_stride;
    Q6KRegs<U> ring[NB];
    auto request = [&](Q6KRegs<U> &b, int step) __attribute__((always_inline)) {
        q6k_load(b, ql, qh, sc, dp, l, s0 + U * step, s1);
        __builtin_amdgcn_sched_barrier(0);
    };
#pragma unroll
    for (int k = 0; k < PRE; k++) request(ring[k], k);

    // every wave runs every pass (a half without a super-block of its own in the last pass redoes the part's last one
    // and stores nothing): the f32 loads above are used unconditionally and stay ahead of the weight requests
    auto quantize_pass = [&](int p) __attribute__((always_inline)) {
        const int u = unit_of(p);
#pragma unroll
        for (int t = 0; t < NT; t++) {
            float dv;
            int bs;
            const uint2 packed = q8k_quantize_row32(xv[p][t], lane, dv, bs);
            int s16 = sdot4(packed.y, 0x01010101u, sdot4(packed.x, 0x01010101u, 0));
            s16 += row_shr_i32<1>(s16);  // odd lanes: the sum of 16 consecutive quants
            if (s0 + u < s1) {
                const int sbk = t * NSB + s0 + u;
                reinterpret_cast<uint2 *>(ys)[sbk * 32 + ql32] = packed;
                if (ql32 & 1) bsum16[sbk * 16 + (ql32 >> 1)] = s16;
                if (ql32 == 0) yds[sbk] = dv;
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    quantize_pass(0);
    __syncthreads();

    float acc[NT];
#pragma unroll
    for (int t = 0; t < NT; t++) acc[t] = 0.0f;
    auto compute = [&](const Q6KRegs<U> &b, int step) __attribute__((always_inline)) {
        q6k_compute<NT, false, U>(b, l, s0 + U * step, s1, ys, bsum16, yds, NSB, acc, nullptr);
        __builtin_amdgcn_sched_barrier(0);
    };
#pragma unroll
    for (int j = PRE; j < NB; j++) request(ring[j], j);
#pragma unroll
    for (int i = 0; i < USTEPS; i++) {
        if ((U * i) % PER_PASS == 0) {  // the first step that reads pass U i / PER_PASS: the next pass goes ahead of it
            if ((U * i) / PER_PASS + 1 < PASSES) quantize_pass((U * i) / PER_PASS + 1);
            if (i > 0) __syncthreads();
        }
        compute(ring[i % NB], i);
        if (i + NB < USTEPS) request(ring[i % NB], i + NB);
    }
    if (l == LPS - 1) {
#pragma unroll
        for (int t = 0; t < NT; t++) part[(wave * NT + t) * RPW + r] = acc[t];
    }
    __syncthreads();
    if (tid < TPW * NT * RPW) {
        const int rr = tid % RPW, t = (tid / RPW) % NT, tw = tid / (RPW * NT);
        const int orow = (bx * TPW + tw) * RPW + rr;
        if (orow < a.rows) {
            float v = part[((tw * KS) * NT + t) * RPW + rr];
#pragma unroll
            for (int k = 1; k < KS; k++) v = v + part[((tw * KS + k) * NT + t) * RPW + rr];
            if (NT == 1 && a.residual) v = v + a.residual[orow];
            a.out[static_cast<int64_t>(t) * a.rows + orow] = v;
        }
    }
}

static int pick_ksplit_q6k(int64_t rows, int64_t n_sb) {
    const int forced = env_int("CAMELID_HIP_Q6K_KSPLIT", 0);
    if ((forced == 1 || forced == 2 || forced == 4) && forced <= n_sb) return forced;
    if (env_int("CAMELID_HIP_EXACT_ORDER", 0)) return 1;
    const int64_t tiles = (rows + 7) / 8;
    if (tiles >= 1536 || n_sb < 8) return 1;
    if (tiles * 2 >= 1536 || n_sb < 16) return 2;
    return 4;
}

int q6k_ksplit_for(int64_t rows, int64_t n_sb) { return pick_ksplit_q6k(rows, n_sb); }

// The K-cut eight-wave launch serves rows of 14336 values cut four ways (CAMELID_HIP_Q6K_CU=0: the two-launch form).
static bool q6k_cu_kcut_serves(int64_t rows, int64_t n_sb) {
    return n_sb == 56 && pick_ksplit_q6k(rows, n_sb) == 4 && env_int("CAMELID_HIP_Q6K_CU", 1) != 0;
}
// Steps per part (the longest part's super-blocks) of the general K-cut form, 0 where it does not serve.
// CAMELID_HIP_Q6K_KCUT_ANY=0 leaves these shapes to the four-wave launches.
static int q6k_cu_kcut_any_steps(int64_t rows, int64_t n_sb) {
    if (!env_int("CAMELID_HIP_Q6K_KCUT_ANY", 1) || !env_int("CAMELID_HIP_Q6K_CU", 1)) return 0;
    const int ks = pick_ksplit_q6k(rows, n_sb);
    if (ks == 1) {
        // no K cut: while twelve-wave workgroups still come to one per compute unit.  us per step against the four-wave
        // launches: 14336 x 4096 10.27 / 10.78, 18944 x 3584 (ten waves) 12.12 / 14.46, 16384 x 4096 10.6 / 11.18,
        // 12288 x 4096 9.9 / 10.5, 13824 x 5120 13.65 / 13.85, 24576 x 4096 (twelve) 14.8 / 15.05
        const bool length = n_sb == 12 || n_sb == 14 || n_sb == 16 || n_sb == 20 || n_sb == 24 || n_sb == 32;
        return length && (rows + 7) / 8 <= 12 * 256 ? static_cast<int>(n_sb) : 0;
    }
    if (ks != 2 && ks != 4) return 0;
    const int steps = static_cast<int>((n_sb + ks - 1) / ks);
    for (int served : {4, 5, 6, 8, 11, 14, 19, 7, 10, 12, 16}) {
        const bool four_ways = served == 5 || served == 11 || served == 14 || served == 19, two_ways = served == 7 || served == 10 || served == 12 || served == 16;
        if (steps == served && !(ks == 4 && two_ways) && !(ks == 2 && four_ways)) return steps;
    }
    return 0;
}
bool gemv_q6k_long_rows_fuse(const cml_weight *w) {
    return w->fmt == CML_Q6_K && (q6k_cu_kcut_serves(w->rows, w->nb) || q6k_cu_kcut_any_steps(w->rows, w->nb) != 0);
}

// One f32 token against two to four Q6_K weights of one row length whose shapes take the same K cut, in ONE launch of
// the one-workgroup-per-unit form (eight waves); every output is its own call's bits.  -1 = not a set this launch
// serves.  CAMELID_HIP_Q6K_MULTI=0: the caller makes the calls one by one.
int launch_gemv_q6k_f32_multi(const cml_weight *const *ws, int n, const float *x, float *const *outs, hipStream_t st) {
    if (n < 2 || n > 4 || !env_int("CAMELID_HIP_Q6K_MULTI", 1) || !env_int("CAMELID_HIP_MULTI_LAUNCH", 1)) return -1;
    const int64_t n_sb = ws[0]->nb;
    int ks = 0, steps = 0;
    for (int j = 0; j < n; j++) {
        if (ws[j]->fmt != CML_Q6_K || ws[j]->nb != n_sb || ws[j]->rows <= 0) return -1;
        const int k = pick_ksplit_q6k(ws[j]->rows, n_sb), st_j = q6k_cu_kcut_any_steps(ws[j]->rows, n_sb);
        if (st_j == 0 || (j && (k != ks || st_j != steps))) return -1;
        ks = k;
        steps = st_j;
    }
    if (!x) return fail(CML_ERR_INVALID, "null activation");
    Q6KMultiArgs ma{};
    ma.base.n_sb = static_cast<int>(n_sb);
    ma.base.x = x;
    ma.base.n_groups = 1;
    ma.base.ksplit = ks;
    ma.base.ksplit_log2 = ks >= 4 ? 2 : (ks >= 2 ? 1 : 0);
    const int tpw = 8 / ks;  // 8-row tiles per eight-wave workgroup
    int wg = 0;
    for (int j = 0; j < 4; j++) {
        const cml_weight *w = ws[std::min(j, n - 1)];
        ma.qlm[j] = w->planes.p[0]; ma.ql_stridem[j] = w->planes.row_stride[0];
        ma.qhm[j] = w->planes.p[1]; ma.qh_stridem[j] = w->planes.row_stride[1];
        ma.scm[j] = w->planes.p[2]; ma.sc_stridem[j] = w->planes.row_stride[2];
        ma.dm[j] = w->planes.p[3];  ma.d_stridem[j] = w->planes.row_stride[3];
        ma.outm[j] = outs[std::min(j, n - 1)];
        ma.rowsm[j] = static_cast<int>(w->rows);
        if (j < n) wg += static_cast<int>(((w->rows + 7) / 8 + tpw - 1) / tpw);
        ma.wg_end[j] = j < n ? wg : INT32_MAX;
    }
    const dim3 grid(static_cast<unsigned>(wg)), block(512);
    const size_t lds = static_cast<size_t>(n_sb) * (256 + 64 + 4);
#define CML_Q6K_MULTI(KS_, NS_) \
    case KS_ * 100 + NS_: hipLaunchKernelGGL((gemv_q6k_cu_kcut_kernel<KS_, NS_, 4, 8, true, 1, 1, true>), grid, block, lds, st, ma); break;
    switch (ks * 100 + steps) {
        CML_Q6K_MULTI(4, 4)
        CML_Q6K_MULTI(4, 5)
        CML_Q6K_MULTI(4, 6)
        CML_Q6K_MULTI(4, 8)
        CML_Q6K_MULTI(2, 4)
        CML_Q6K_MULTI(2, 6)
        CML_Q6K_MULTI(2, 7)
        CML_Q6K_MULTI(2, 8)
        CML_Q6K_MULTI(1, 12)
        CML_Q6K_MULTI(1, 14)
        CML_Q6K_MULTI(1, 16)
        CML_Q6K_MULTI(1, 20)
        default: return -1;
    }
#undef CML_Q6K_MULTI
    CML_COUNT_LAUNCH("q6k.dot.wg8.kcut.fused.multi");
    CML_HIP_TRY(hipGetLastError());
    return CML_OK;
}

static size_t q6k_lds_bytes(int nt, int n_sb) {
    return static_cast<size_t>(nt) * n_sb * (256 + 64) + ((static_cast<size_t>(nt) * n_sb + 3) & ~size_t(3)) * 4 + 4 * nt * 8 * 4;
}

template <int NT>
static int launch_q6k_nt(const Q6KArgs &ka, int n_bands, bool ints, bool grouped, hipStream_t st) {
    const int tiles_per_wg = 4 / ka.ksplit;
    const int64_t tiles = (ka.rows + 7) / 8;
    const unsigned gx = static_cast<unsigned>((tiles + tiles_per_wg - 1) / tiles_per_wg);
    const size_t lds = q6k_lds_bytes(NT, ka.n_sb);
    if (lds > 64 * 1024) return fail(CML_ERR_UNSUPPORTED, "Q6_K activation of %d super-blocks x %d tokens exceeds the LDS staging limit", ka.n_sb, NT);
    if (grouped) {
        hipLaunchKernelGGL((gemv_q6k_kernel<NT, false, true>), dim3(gx, n_bands), dim3(256), lds, st, ka);
        CML_COUNT_LAUNCH("q6k.dot.grouped");
    } else if (ints && NT == 1) {
        hipLaunchKernelGGL((gemv_q6k_kernel<1, true>), dim3(gx, n_bands), dim3(256), lds, st, ka);
        CML_COUNT_LAUNCH("q6k.dot.ints");
    } else if (NT == 1 && tiles >= env_int("CAMELID_HIP_Q6K_DEEP_MIN_TILES", 2048)) {
        hipLaunchKernelGGL((gemv_q6k_kernel<1, false, false, 4>), dim3(gx, n_bands), dim3(256), lds, st, ka);
        CML_COUNT_LAUNCH("q6k.dot.deep");
    } else {
        hipLaunchKernelGGL((gemv_q6k_kernel<NT, false>), dim3(gx, n_bands), dim3(256), lds, st, ka);
        CML_COUNT_LAUNCH("q6k.dot.buffers");
    }
    CML_HIP_TRY(hipGetLastError());
    return CML_OK;
}

// ---- the 8-lane order of the reference CPU lanes, bit for bit ------------------------------------
//
// q6_k_wire_row_dot (src/inference.rs:25535-25581, the Q6_K row dot both CPU lanes call) keeps
// eight integer lanes per super-block, lane l taking the values whose index is l modulo 8
// (aux32[l] += sc_j * y * a over j < 16 and both 8-value halves of group j), and eight f32 lane
// sums  sums[l] += (d_w * yd) * (float)aux32[l]  over the super-blocks in order, folded left to
// right at the end.  A 4-wide packed dot cannot keep those lanes apart, so the kernels above match
// this order to 1e-5 only.  This kernel reproduces it exactly and is selected by
// CAMELID_HIP_Q6K_LANE_ORDER=1 for every plain Q6_K call (one launch per token batch; speed is
// secondary here: byte loads, one wave per row).  Lane = 8 * g + l: eight super-blocks g in
// flight per pass, their integers independent; the f32 sums are then advanced in super-block
// order by the lanes of g = 0 through LDS.
__global__ __launch_bounds__(256) void gemv_q6k_lanes_kernel(Q6KArgs a, int64_t cols) {
    extern __shared__ uint4 smem[];
    int8_t *ys = reinterpret_cast<int8_t *>(smem);                              // [n_sb*256]
    float *yds = reinterpret_cast<float *>(ys + a.n_sb * 256);                  // [n_sb]
    float *xch = yds + ((a.n_sb + 3) & ~3);                                     // [4 waves][64]
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int token = blockIdx.y;
    const int8_t *q = a.q + static_cast<int64_t>(token) * cols;
    for (int i = tid; i < a.n_sb * 16; i += 256) reinterpret_cast<uint4 *>(ys)[i] = reinterpret_cast<const uint4 *>(q)[i];
    for (int i = tid; i < a.n_sb; i += 256) yds[i] = a.yd[static_cast<int64_t>(token) * a.n_sb + i];
    __syncthreads();
    const int row = blockIdx.x * 4 + wave;
    if (row >= a.rows) return;  // whole waves leave; no barrier follows
    const int g = lane >> 3, l = lane & 7;
    const uint8_t *ql = a.ql + static_cast<int64_t>(row) * a.ql_stride;
    const uint8_t *qh = a.qh + static_cast<int64_t>(row) * a.qh_stride;
    const int8_t *sc = reinterpret_cast<const int8_t *>(a.sc + static_cast<int64_t>(row) * a.sc_stride);
    const uint8_t *dw = a.d + static_cast<int64_t>(row) * a.d_stride;
    float *mine = xch + wave * 64;
    float sum_l = 0.0f;  // lanes of g == 0: sums[l]
    for (int sb0 = 0; sb0 < a.n_sb; sb0 += 8) {
        const int sb = sb0 + g;
        float term = 0.0f;
        if (sb < a.n_sb) {
            int aux = 0;
#pragma unroll
            for (int hh = 0; hh < 2; hh++) {
#pragma unroll
                for (int k = 0; k < 4; k++) {
                    const int ll = l + 8 * k;  // position inside the 32-value region
                    const int lo_b = ql[sb * 128 + 64 * hh + ll], hi_b = ql[sb * 128 + 64 * hh + 32 + ll], hb = qh[sb * 64 + 32 * hh + ll];
                    const int code[4] = {(lo_b & 15) | ((hb & 3) << 4), (hi_b & 15) | (((hb >> 2) & 3) << 4),
                                         (lo_b >> 4) | (((hb >> 4) & 3) << 4), (hi_b >> 4) | (((hb >> 6) & 3) << 4)};
#pragma unroll
                    for (int region = 0; region < 4; region++) {
                        const int v = 128 * hh + 32 * region + ll;
                        const int scale = sc[sb * 16 + (v >> 4)];
                        aux += scale * (static_cast<int>(ys[sb * 256 + v]) * (code[region] - 32));
                    }
                }
            }
            const float dd = f16_bits_to_f32(ldg2(dw + sb * 2)) * yds[sb];
            term = dd * static_cast<float>(aux);
        }
        mine[lane] = term;
        wave_barrier_lds();
        if (g == 0) {
            const int n = min(8, a.n_sb - sb0);
            for (int k = 0; k < n; k++) sum_l = sum_l + mine[8 * k + l];
        }
        wave_barrier_lds();
    }
    if (g == 0) mine[l] = sum_l;
    wave_barrier_lds();
    if (lane == 0) {
        float total = 0.0f;
        for (int k = 0; k < 8; k++) total = total + mine[k];
        if (a.residual) total = total + a.residual[row];
        a.out[static_cast<int64_t>(token) * a.rows + row] = total;
    }
}

static int launch_gemv_q6k_lanes(const MatArgs &a, hipStream_t st) {
    const cml_weight *w = a.w;
    Q6KArgs ka{};
    ka.ql = w->planes.p[0]; ka.ql_stride = w->planes.row_stride[0];
    ka.qh = w->planes.p[1]; ka.qh_stride = w->planes.row_stride[1];
    ka.sc = w->planes.p[2]; ka.sc_stride = w->planes.row_stride[2];
    ka.d = w->planes.p[3];  ka.d_stride = w->planes.row_stride[3];
    ka.rows = static_cast<int>(w->rows);
    ka.n_sb = static_cast<int>(w->nb);
    ka.q = a.q;
    ka.yd = a.scales;
    ka.out = a.out;
    ka.residual = a.residual;
    const size_t lds = static_cast<size_t>(ka.n_sb) * 256 + ((static_cast<size_t>(ka.n_sb) + 3) & ~size_t(3)) * 4 + 4 * 64 * 4;
    if (lds > 64 * 1024) return fail(CML_ERR_UNSUPPORTED, "Q6_K activation of %d super-blocks exceeds the LDS staging limit", ka.n_sb);
    if (a.n_tokens > 65535) return fail(CML_ERR_UNSUPPORTED, "at most 65535 tokens per call in the lane-order mode");
    hipLaunchKernelGGL(gemv_q6k_lanes_kernel, dim3(static_cast<unsigned>((ka.rows + 3) / 4), static_cast<unsigned>(a.n_tokens)), dim3(256), lds, st,
                       ka, static_cast<int64_t>(w->cols));
    CML_COUNT_LAUNCH("q6k.lanes");
    CML_HIP_TRY(hipGetLastError());
    return CML_OK;
}

bool q6k_lane_order() { return env_int("CAMELID_HIP_Q6K_LANE_ORDER", 0) != 0; }

int launch_gemv_q6k(const MatArgs &a, hipStream_t st) {
    const cml_weight *w = a.w;
    if (w->rows == 0 || a.n_tokens == 0) return CML_OK;
    const bool grouped = a.group_offsets != nullptr || a.group_ids != nullptr;
    if (!grouped && !a.ints && q6k_lane_order()) return launch_gemv_q6k_lanes(a, st);
    Q6KArgs ka{};
    ka.ql = w->planes.p[0]; ka.ql_stride = w->planes.row_stride[0];
    ka.qh = w->planes.p[1]; ka.qh_stride = w->planes.row_stride[1];
    ka.sc = w->planes.p[2]; ka.sc_stride = w->planes.row_stride[2];
    ka.d = w->planes.p[3];  ka.d_stride = w->planes.row_stride[3];
    ka.rows = static_cast<int>(grouped ? a.band_rows : w->rows);
    ka.n_sb = static_cast<int>(w->nb);
    ka.residual = a.residual;
    ka.ints = a.ints;
    ka.group_offsets = a.group_offsets;
    ka.group_rows = a.group_rows;
    ka.group_ids = a.group_ids;
    ka.n_groups = a.n_groups;
    ka.ksplit = pick_ksplit_q6k(ka.rows, ka.n_sb);
    ka.ksplit_log2 = ka.ksplit >= 4 ? 2 : (ka.ksplit >= 2 ? 1 : 0);
    if (grouped) {
        if (a.band_rows <= 0 || a.band_rows * a.n_groups != w->rows)
            return fail(CML_ERR_SHAPE, "%d bands of %lld rows do not cover %lld rows", a.n_groups, (long long)a.band_rows, (long long)w->rows);
        // One launch: every group walks its own assignments in passes of NT, NT sized for the most
        // a single group can hold and for the LDS staging limit.
        ka.q = a.q;
        ka.yd = a.scales;
        ka.out = a.out;
        int nt = a.n_tokens >= 8 ? 8 : (a.n_tokens >= 4 ? 4 : (a.n_tokens >= 2 ? 2 : 1));
        while (nt > 1 && q6k_lds_bytes(nt, ka.n_sb) > 64 * 1024) nt /= 2;
        const int slots = a.group_ids ? a.max_active : a.n_groups;
        switch (nt) {
            case 8: return launch_q6k_nt<8>(ka, slots, false, true, st);
            case 4: return launch_q6k_nt<4>(ka, slots, false, true, st);
            case 2: return launch_q6k_nt<2>(ka, slots, false, true, st);
            default: return launch_q6k_nt<1>(ka, slots, false, true, st);
        }
    }
    const int n_bands = 1;
    int64_t t0 = 0;
    while (t0 < a.n_tokens) {
        const int64_t left = a.n_tokens - t0;
        int nt = left >= 8 ? 8 : (left >= 4 ? 4 : (left >= 2 ? 2 : 1));
        while (nt > 1 && q6k_lds_bytes(nt, ka.n_sb) > 64 * 1024) nt /= 2;  // long rows: fewer tokens per pass
        ka.q = a.q + t0 * w->cols;
        ka.yd = a.scales + t0 * w->nb;
        ka.out = a.out + t0 * ka.rows;
        int rc;
        switch (nt) {
            case 8: rc = launch_q6k_nt<8>(ka, n_bands, false, false, st); break;
            case 4: rc = launch_q6k_nt<4>(ka, n_bands, false, false, st); break;
            case 2: rc = launch_q6k_nt<2>(ka, n_bands, false, false, st); break;
            default: rc = launch_q6k_nt<1>(ka, n_bands, a.ints != nullptr, false, st); break;
        }
        if (rc != CML_OK) return rc;
        t0 += nt;
    }
    return CML_OK;
}

int launch_gemm_q6k(const MatArgs &a, hipStream_t st) { return launch_gemv_q6k(a, st); }

// One or two tokens, f32 activation in: quantize + matvec in one launch (plain call).
int launch_gemv_q6k_f32(const cml_weight *w, const float *x, float *out, hipStream_t st, int n_tokens) {
    if (w->rows == 0) return CML_OK;
    if (n_tokens != 1 && n_tokens != 2) return fail(CML_ERR_UNSUPPORTED, "the fused Q6_K launch takes one or two tokens");
    Q6KArgs ka{};
    ka.ql = w->planes.p[0]; ka.ql_stride = w->planes.row_stride[0];
    ka.qh = w->planes.p[1]; ka.qh_stride = w->planes.row_stride[1];
    ka.sc = w->planes.p[2]; ka.sc_stride = w->planes.row_stride[2];
    ka.d = w->planes.p[3];  ka.d_stride = w->planes.row_stride[3];
    ka.rows = static_cast<int>(w->rows);
    ka.n_sb = static_cast<int>(w->nb);
    ka.x = x;
    ka.out = out;
    ka.n_groups = 1;
    ka.ksplit = pick_ksplit_q6k(ka.rows, ka.n_sb);
    ka.ksplit_log2 = ka.ksplit >= 4 ? 2 : (ka.ksplit >= 2 ? 1 : 0);
    const int tiles_per_wg = 4 / ka.ksplit;
    const int64_t tiles = (ka.rows + 7) / 8;
    const unsigned gx = static_cast<unsigned>((tiles + tiles_per_wg - 1) / tiles_per_wg);
    const size_t lds = q6k_lds_bytes(n_tokens, ka.n_sb);
    if (lds > 64 * 1024) return fail(CML_ERR_UNSUPPORTED, "Q6_K activation of %d super-blocks exceeds the LDS staging limit", ka.n_sb);
    if (n_tokens == 1 && q6k_cu_kcut_serves(ka.rows, ka.n_sb) && tiles <= 2 * 256) {
        // (ring of 3 / 4 / 5 / 6 one-super-block buffers: 10.61 / 10.42 / 10.86 / 11.32 us at 4096 x 14336)
        hipLaunchKernelGGL((gemv_q6k_cu_kcut_kernel<4, 14>), dim3(static_cast<unsigned>((tiles + 1) / 2)), dim3(512), 0, st, ka);
        CML_COUNT_LAUNCH("q6k.dot.wg8.kcut.fused");
        CML_HIP_TRY(hipGetLastError());
        return CML_OK;
    }
    if (const int two_steps = (n_tokens == 2 && env_int("CAMELID_HIP_Q6K_KCUT_TOKENS", 1)) ? q6k_cu_kcut_any_steps(ka.rows, ka.n_sb) : 0) {
        // two tokens on the general K-cut form (4096 x 4096: 6.65 us before on the four-wave launch that quantizes both rows in every workgroup)
        const int ks = ka.ksplit;
        int waves = 8;
        while (waves < 12 && (tiles + waves / ks - 1) / (waves / ks) > 256) waves += ks == 1 ? 2 : 4;
        const int tpw = waves / ks;
        const dim3 grid(static_cast<unsigned>((tiles + tpw - 1) / tpw)), block(64 * waves);
        const size_t lds_two = 2 * static_cast<size_t>(ka.n_sb) * (256 + 64 + 4);
        bool launched = lds_two <= 64 * 1024;
        if (launched) {
#define CML_Q6K_KCUT_TWO(KS_, NS_, W2_)                                                                                              \
    case KS_ * 100 + NS_:                                                                                                            \
        if (waves == 8) hipLaunchKernelGGL((gemv_q6k_cu_kcut_kernel<KS_, NS_, 4, 8, true, 2>), grid, block, lds_two, st, ka);         \
        else if (waves == W2_) hipLaunchKernelGGL((gemv_q6k_cu_kcut_kernel<KS_, NS_, 4, W2_, true, 2>), grid, block, lds_two, st, ka); \
        else launched = false;                                                                                                       \
        break;
            switch (ks * 100 + two_steps) {
                CML_Q6K_KCUT_TWO(4, 4, 12)
                CML_Q6K_KCUT_TWO(4, 5, 12)
                CML_Q6K_KCUT_TWO(4, 8, 12)
                CML_Q6K_KCUT_TWO(4, 11, 12)
                CML_Q6K_KCUT_TWO(4, 14, 12)
                CML_Q6K_KCUT_TWO(2, 4, 12)
                CML_Q6K_KCUT_TWO(2, 6, 12)
                CML_Q6K_KCUT_TWO(2, 8, 12)
                CML_Q6K_KCUT_TWO(2, 10, 12)
                CML_Q6K_KCUT_TWO(1, 14, 10)
                CML_Q6K_KCUT_TWO(1, 16, 10)
                default: launched = false; break;
            }
#undef CML_Q6K_KCUT_TWO
        }
        if (launched) {
            CML_COUNT_LAUNCH("q6k.dot.wg8.kcut.fused.two");
            CML_HIP_TRY(hipGetLastError());
            return CML_OK;
        }
    }
    if (const int any_steps = n_tokens == 1 ? q6k_cu_kcut_any_steps(ka.rows, ka.n_sb) : 0) {
        // the general K-cut form: eight waves, or twelve where eight would need more than one workgroup per compute unit
        const int ks = ka.ksplit;
        int waves = env_int("CAMELID_HIP_Q6K_KCUT_WAVES", 0);
        if (waves != 8 && waves != 12 && !(waves == 10 && ks == 1)) {
            waves = 8;
            while (waves < 12 && (tiles + waves / ks - 1) / (waves / ks) > 256) waves += ks == 1 ? 2 : 4;
        }
        const int tpw = waves / ks;
        const dim3 grid(static_cast<unsigned>((tiles + tpw - 1) / tpw)), block(64 * waves);
        const size_t lds_any = static_cast<size_t>(ka.n_sb) * (256 + 64 + 4);
#define CML_Q6K_KCUT_ANY(KS_, NS_)                                                                                          \
    case KS_ * 100 + NS_:                                                                                                   \
        if (waves == 8) hipLaunchKernelGGL((gemv_q6k_cu_kcut_kernel<KS_, NS_, 4, 8, true>), grid, block, lds_any, st, ka);   \
        else hipLaunchKernelGGL((gemv_q6k_cu_kcut_kernel<KS_, NS_, 4, 12, true>), grid, block, lds_any, st, ka);             \
        break;
        switch (ks * 100 + any_steps) {
            CML_Q6K_KCUT_ANY(4, 4)
            CML_Q6K_KCUT_ANY(4, 5)
            CML_Q6K_KCUT_ANY(4, 6)
            CML_Q6K_KCUT_ANY(4, 8)
            CML_Q6K_KCUT_ANY(4, 11)
            CML_Q6K_KCUT_ANY(4, 14)
            CML_Q6K_KCUT_ANY(4, 19)
            CML_Q6K_KCUT_ANY(2, 4)
            CML_Q6K_KCUT_ANY(2, 6)
            CML_Q6K_KCUT_ANY(2, 7)
            CML_Q6K_KCUT_ANY(2, 8)
            CML_Q6K_KCUT_ANY(2, 10)
            CML_Q6K_KCUT_ANY(2, 12)
            CML_Q6K_KCUT_ANY(2, 16)
            // no K cut (12288 to 24576 rows): the same launch, every wave a row tile of its own
            // two super-blocks of a row per ring step (256 contiguous bytes of each plane row per request), three slots: 13824 x 5120
            // 13.6 -> 12.7 us, 14336 x 8192 20.0 -> 18.8, 18944 x 3584 12.05 -> 11.8; rows of 4096 values keep four one-super-block slots
            // (16384 x 4096 10.55 against 10.6).  CAMELID_HIP_Q6K_CU_U2=0: one super-block per step everywhere.
#define CML_Q6K_CU_ANY(NS_)                                                                                                \
    case 100 + NS_:                                                                                                        \
        if (NS_ != 16 && env_int("CAMELID_HIP_Q6K_CU_U2", 1)) {                                                            \
            if (waves == 8) hipLaunchKernelGGL((gemv_q6k_cu_kcut_kernel<1, NS_, 3, 8, true, 1, 2>), grid, block, lds_any, st, ka);        \
            else if (waves == 10) hipLaunchKernelGGL((gemv_q6k_cu_kcut_kernel<1, NS_, 3, 10, true, 1, 2>), grid, block, lds_any, st, ka); \
            else hipLaunchKernelGGL((gemv_q6k_cu_kcut_kernel<1, NS_, 3, 12, true, 1, 2>), grid, block, lds_any, st, ka);                  \
            break;                                                                                                         \
        }                                                                                                                  \
        if (waves == 8) hipLaunchKernelGGL((gemv_q6k_cu_kcut_kernel<1, NS_, 4, 8, true>), grid, block, lds_any, st, ka);    \
        else if (waves == 10) hipLaunchKernelGGL((gemv_q6k_cu_kcut_kernel<1, NS_, 4, 10, true>), grid, block, lds_any, st, ka); \
        else hipLaunchKernelGGL((gemv_q6k_cu_kcut_kernel<1, NS_, 4, 12, true>), grid, block, lds_any, st, ka);              \
        break;
            CML_Q6K_CU_ANY(12)
            CML_Q6K_CU_ANY(14)
            CML_Q6K_CU_ANY(16)
            CML_Q6K_CU_ANY(20)
            CML_Q6K_CU_ANY(24)
            CML_Q6K_CU_ANY(32)
#undef CML_Q6K_CU_ANY
            default: return fail(CML_ERR_UNSUPPORTED, "no Q6_K K-cut form for %d super-blocks cut %d ways", ka.n_sb, ks);
        }
#undef CML_Q6K_KCUT_ANY
        CML_COUNT_LAUNCH("q6k.dot.wg8.kcut.fused.any");
        CML_HIP_TRY(hipGetLastError());
        return CML_OK;
    }
    if (n_tokens == 2) {
        hipLaunchKernelGGL((gemv_q6k_kernel<2, false, false, 2, true>), dim3(gx, 1), dim3(256), lds, st, ka);
        CML_COUNT_LAUNCH("q6k.dot.buffers.fused");
    } else if (tiles >= env_int("CAMELID_HIP_Q6K_DEEP_MIN_TILES", 2048)) {
        hipLaunchKernelGGL((gemv_q6k_kernel<1, false, false, 4, true>), dim3(gx, 1), dim3(256), lds, st, ka);
        CML_COUNT_LAUNCH("q6k.dot.deep.fused");
    } else {
        hipLaunchKernelGGL((gemv_q6k_kernel<1, false, false, 2, true>), dim3(gx, 1), dim3(256), lds, st, ka);
        CML_COUNT_LAUNCH("q6k.dot.buffers.fused");
    }
    CML_HIP_TRY(hipGetLastError());
    return CML_OK;
}

}  // namespace cml
