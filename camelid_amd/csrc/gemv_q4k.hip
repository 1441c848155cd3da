// Q4_K x Q8_K fused dequantize + matvec / small-batch matmul for gfx950.
//
// Arithmetic (reference q4_k_dot_scalar behind q4_k_dot_arm,
// src/diffusion_gemma/refmath.rs:504-562; the Llama lane's Q4_K row dot,
// src/inference.rs:23752): per 256-value super-block, in order,
//     D = yd * d;  M = yd * dmin;
//     P = sum_g m_g  * sum_{t<32} y[32g+t]              (exact integer)
//     S = sum_g sc_g * sum_{t<32} q[32g+t] * y[32g+t]   (exact integer)
//     acc = fma(-M, (float)P, acc);  acc = fma(D, (float)S, acc)
// S and P are what every variant of the reference agrees on bit for bit
// (src/inference.rs:25806-25889 computes the same integers lane-wise).
//
// Mapping.  At load time the 144-byte wire super-blocks are re-laid, losslessly
// and at the same density, into a tile-interleaved layout (layout.hip): for a
// tile of 16 consecutive rows and one super-block index there is one contiguous
// 2304-byte chunk, chunks ordered [super-block][tile] so that waves working on
// neighbouring tiles at the same super-block read neighbouring memory (a
// contiguous front sweeps the matrix, as in a grid-stride copy):
//     [16 headers x 16 B][16 rows x 4 x 16 B "a" pieces][16 rows x 4 x 16 B "b" pieces]
// (header = f16 d, f16 dmin, 12 packed 6-bit scale/min bytes; piece a/b of lane
// c = nibble bytes [32c, 32c+16) / [32c+16, 32c+32) of the block).  Four lanes
// own one super-block of one row, a wave owns a 16-row tile: each of its three
// 128-bit load instructions reads whole, consecutive 128-byte lines (256 B of
// headers, 1 KB, 1 KB) -- the same shape as a plain streaming copy.  The lane
// unpacks its 64 values in registers and dots them against the int8 activation
// staged in LDS with v_dot4_i32_i8.  All lanes of a group work on the same
// row, so the per-row f32 chain above lives in one lane and needs no
// cross-lane traffic; only the two integers are reduced inside the group (DPP
// row_shr).  A workgroup is TPW row tiles x KSPLIT waves: each tile's
// super-block range is cut into KSPLIT contiguous parts (one per wave) whose
// partial chains are added left to right.  With KSPLIT = 1 the result is the
// reference's own association, bit for bit.
//
// The kernel is short (a 33 MB matrix streams in a few microseconds), so the
// prologue is ordered to keep HBM busy from the first cycle: the activation
// loads are issued first, the first weight buffer right behind them, and only
// then is the activation written to LDS.
//
// NT > 1 holds the unpacked weight in registers and replays it against NT
// activation rows in LDS: the weight is streamed once per NT tokens and every
// (row, token) cell is the NT = 1 result exactly.
#include <algorithm>
#include <cmath>
#include <type_traits>

#include "cml_device.hpp"
#include "cml_host.hpp"

#pragma clang fp contract(off)

namespace cml {

struct Q4KArgs {
    const uint8_t *w;      // tiled layout: [super-block][tile][2304 B]
    int64_t sb_stride;     // bytes between consecutive super-blocks of one tile (= all tiles * 2304)
    int rows;              // rows of one band (a multiple of 16 when groups are used)
    int row_skip;          // leading rows of the first tile that are not part of this weight view (0..15; plain calls only)
    int n_sb;              // super-blocks per row
    const int8_t *q;       // activation rows [*][n_sb*256]
    const float *yd;       // activation scales [*][n_sb]
    const float *x;        // f32 activation row [n_sb*256]: only for the kernel that quantizes it itself
    float *out;            // [*][rows]
    const float *residual; // [rows] or null (plain single-token calls only)
    int32_t *ints;         // [rows][n_sb][2] or null
    // Plain call: blockIdx.y = 0, the NT activation rows 0..NT-1 go to output rows 0..NT-1.
    // Grouped call (mixture of experts): blockIdx.y = group e, which owns the
    // weight band of rows [e*rows, (e+1)*rows) and the assignments
    // [group_offsets[e], group_offsets[e+1]); assignment j reads activation row
    // group_rows[j] (j itself when null) and writes output row j.  A group
    // serves its assignments in passes of NT.
    const int32_t *group_offsets;
    const int32_t *group_rows;
    const int32_t *group_ids;  // y-slot -> group (-1: unused slot), or null (the y-slot is the group)
    // Direct call (single-token decode; group_offsets null, group_ids set): y-slot y IS assignment y
    // and group_ids[y] its expert (ids outside [0, n_groups) are skipped); its activation row is
    // row 0 (shared_act: every assignment reads the one token) or row y.
    int n_groups;
    int shared_act;
    // Direct call that routes the token itself (ROUTE): the n_groups router logits of the one token;
    // y-slot y serves the expert of routed rank y (Mixtral routing, top route_k), and the first
    // workgroup leaves experts and weights in routed order for the launches behind this one.
    const float *route_logits;
    int route_k;
    int32_t *route_idx;  // [route_k]
    float *route_w;      // [route_k]
    // Pair launch (gridDim.z == 2): blockIdx.z = 1 works on a second weight of the same shape
    // against the same activations and writes out2 (gate and up projections in one launch).
    const uint8_t *w2;
    float *out2;
    int ksplit;        // waves sharing one row tile (1, 2, 4 or 8)
    int ksplit_log2;
    int tiles_per_wg;  // row tiles per workgroup; blockDim.x = 64 * ksplit * tiles_per_wg
    // Multi launch (MULTI): up to four weights of one row length and one K cut against the same token, their workgroups
    // laid end to end along grid.x; weight j serves workgroups [wg_end[j-1], wg_end[j]) and writes outm[j].
    const uint8_t *wm[4];
    float *outm[4];
    int64_t stridem[4];
    int rowsm[4];
    int skipm[4];
    int wg_end[4];
};

constexpr int kQ4KStageRegs = 4;  // activation chunks a thread holds in registers during the prologue

constexpr int kQ4KChunk = 2304;  // bytes of one (tile, super-block) chunk
constexpr int LPS = 4;           // lanes per super-block

template <int U_>
struct Q4KRegs {
    static constexpr int U = U_;  // super-blocks in flight per buffer and 4-lane group
    uint4 hdr[U];
    uint4 qa[U];
    uint4 qb[U];
};

// Loads are unconditional (super-block indices past the end are clamped to the
// last one and their result is discarded by the caller): straight-line code
// lets the compiler keep the next buffer's loads in flight under the current
// buffer's arithmetic with partial vmcnt waits.  `tile` points at the tile's
// first chunk; row_in_tile = row in the 16-row layout tile, piece = 4*row_in_tile + c.  With SPR
// groups per row the group's own first super-block comes in `sb` and consecutive buffer entries
// are SPR super-blocks apart.
template <int U, int SPR>
__device__ __forceinline__ void q4k_load(Q4KRegs<U> &r, const uint8_t *tile, int64_t sb_stride, int row_in_tile, int piece,
                                         int sb, int s1) {
#pragma unroll
    for (int u = 0; u < U; u++) {
        const int i = min(sb + u * SPR, s1 - 1);
        const uint8_t *chunk = tile + static_cast<int64_t>(i) * sb_stride;
        r.hdr[u] = ldg16_stream(chunk + row_in_tile * 16);
        r.qa[u] = ldg16_stream(chunk + 256 + piece * 16);
        r.qb[u] = ldg16_stream(chunk + 1280 + piece * 16);
    }
}

// The same loads for a buffer that lies wholly inside the part (no clamping): a wave-uniform
// 64-bit base per entry plus two 32-bit lane constants.  The clamped form multiplies a per-lane
// index by the 64-bit stride for every entry -- quarter-rate instructions that were about a
// seventh of the loop's vector time.  `ubase` = the tile's chunk of super-block `sb` (uniform);
// hdr_off / q_off = the lane's own offsets inside a chunk plus h * stride.
template <int U, int SPR>
__device__ __forceinline__ void q4k_load_whole(Q4KRegs<U> &r, const uint8_t *ubase, int64_t sb_stride, uint32_t hdr_off, uint32_t q_off) {
#pragma unroll
    for (int u = 0; u < U; u++) {
        const uint8_t *chunk = ubase + static_cast<int64_t>(u * SPR) * sb_stride;
        r.hdr[u] = ldg16_stream(chunk + hdr_off);
        r.qa[u] = ldg16_stream(chunk + 256 + q_off);
        r.qb[u] = ldg16_stream(chunk + 1280 + q_off);
    }
}

__device__ __forceinline__ uint4 lo_nibbles(const uint4 &v) {
    return make_uint4(v.x & 0x0f0f0f0fu, v.y & 0x0f0f0f0fu, v.z & 0x0f0f0f0fu, v.w & 0x0f0f0f0fu);
}
__device__ __forceinline__ uint4 hi_nibbles(const uint4 &v) {
    return make_uint4((v.x >> 4) & 0x0f0f0f0fu, (v.y >> 4) & 0x0f0f0f0fu, (v.z >> 4) & 0x0f0f0f0fu,
                      (v.w >> 4) & 0x0f0f0f0fu);
}

// Per-lane constants of the scale/min extraction.  A lane works on chunk c of
// the super-block (values 64c..64c+63: scale groups 2c and 2c+1).  With
// sh = 16*(c&1), the pair (sc[2c], sc[2c+1]) sits in bytes 0,1 of
//   c < 2 :  (u0 >> sh) & 0x3f3f
//   c >= 2:  ((u2 >> sh) & 0x0f0f) | (((u0 >> sh) >> 2) & 0x3030)
// and the pair of mins in
//   c < 2 :  (u1 >> sh) & 0x3f3f
//   c >= 2:  (((u2 >> sh) >> 4) & 0x0f0f) | (((u1 >> sh) >> 2) & 0x3030)
// (u0,u1,u2 = the 12 scale bytes as little-endian words; this is the 6-bit
// packing of reference q4_k_scale_min, src/tensor/mod.rs:5997-6006.)
struct Q4KLane {
    int c;       // chunk
    int sh;      // 16 * (c & 1)
    bool upper;  // c >= 2
};

__device__ __forceinline__ void q4k_scale_pairs(const Q4KLane &ln, const uint4 &hdr, uint32_t &sc_pair,
                                                uint32_t &m_pair) {
    const uint32_t a0 = hdr.y >> ln.sh, a1 = hdr.z >> ln.sh, a2 = hdr.w >> ln.sh;
    const uint32_t sc_lo = a0 & 0x3f3fu, m_lo = a1 & 0x3f3fu;
    const uint32_t sc_up = (a2 & 0x0f0fu) | ((a0 >> 2) & 0x3030u);
    const uint32_t m_up = ((a2 >> 4) & 0x0f0fu) | ((a1 >> 2) & 0x3030u);
    sc_pair = ln.upper ? sc_up : sc_lo;
    m_pair = ln.upper ? m_up : m_lo;
}

// LOADONLY (calibration): every loaded register is folded into acc[0]'s bits and nothing else is
// done -- the kernel then issues exactly the matvec's weight requests, in its order and through
// its register buffers, with no activation and no arithmetic behind them.
template <int NT, bool INTS, int U, int SPR, bool WHOLE = false, bool LOADONLY = false>
__device__ __forceinline__ void q4k_compute(const Q4KRegs<U> &r, const Q4KLane &ln, int sb, int s1,
                                            const int8_t *ys, const int *bsum, const float *yds, int n_sb,
                                            float (&acc)[NT], int32_t *ints_row) {
    if constexpr (LOADONLY) {
        uint32_t sink = __builtin_bit_cast(uint32_t, acc[0]);
#pragma unroll
        for (int u = 0; u < U; u++)
            sink ^= r.hdr[u].x ^ r.hdr[u].y ^ r.hdr[u].z ^ r.hdr[u].w ^ r.qa[u].x ^ r.qa[u].y ^ r.qa[u].z ^ r.qa[u].w ^ r.qb[u].x ^ r.qb[u].y ^
                    r.qb[u].z ^ r.qb[u].w;
        acc[0] = __builtin_bit_cast(float, sink);
        return;
    }
#pragma unroll
    for (int u = 0; u < U; u++) {
        const bool valid = WHOLE || sb + u * SPR < s1;  // wave-uniform when SPR == 1
        const int i = valid ? sb + u * SPR : s1 - 1;
        uint32_t sc_pair, m_pair;
        q4k_scale_pairs(ln, r.hdr[u], sc_pair, m_pair);
        const int sc_lo = sc_pair & 0xff, sc_hi = sc_pair >> 8;
        const float dw = f16_bits_to_f32(r.hdr[u].x & 0xffffu);
        const float dminw = f16_bits_to_f32(r.hdr[u].x >> 16);
        const int c = ln.c;
        const uint4 alo = lo_nibbles(r.qa[u]), ahi = hi_nibbles(r.qa[u]);
        const uint4 blo = lo_nibbles(r.qb[u]), bhi = hi_nibbles(r.qb[u]);
        const int m_a = m_pair & 0xff, m_b = m_pair >> 8;
#pragma unroll
        for (int t = 0; t < NT; t++) {
            const int8_t *y = ys + (static_cast<int64_t>(t) * n_sb + i) * 256;
            const int *bs = bsum + (t * n_sb + i) * 8;
            const uint4 ylo0 = *reinterpret_cast<const uint4 *>(y + 64 * c);
            const uint4 ylo1 = *reinterpret_cast<const uint4 *>(y + 64 * c + 16);
            const uint4 yhi0 = *reinterpret_cast<const uint4 *>(y + 64 * c + 32);
            const uint4 yhi1 = *reinterpret_cast<const uint4 *>(y + 64 * c + 48);
            const int lo = dot16(blo, ylo1, dot16(alo, ylo0, 0));
            const int hi = dot16(bhi, yhi1, dot16(ahi, yhi0, 0));
            const int2 b2 = *reinterpret_cast<const int2 *>(bs + 2 * c);
            const int p = __mul24(b2.x, m_a) + __mul24(b2.y, m_b);
            // |lo|, |hi| <= 32*15*128 and the 6-bit scales keep every product inside 24 bits.
            int s_total = group_sum_to_last<LPS>(__mul24(lo, sc_lo) + __mul24(hi, sc_hi));
            int p_total = group_sum_to_last<LPS>(p);
            s_total = valid ? s_total : 0;  // fma(x, 0, acc) leaves acc unchanged
            p_total = valid ? p_total : 0;
            const float ydv = yds[t * n_sb + i];
            const float D = ydv * dw;
            const float M = ydv * dminw;
            if constexpr (SPR == 2) {
                // the row's first group hands its terms four lanes up: the second group's last lane
                // runs the chain in super-block order
                const float Mp = row_shr_f32<4>(M), Dp = row_shr_f32<4>(D);
                const float pp = row_shr_f32<4>(static_cast<float>(p_total)), sp = row_shr_f32<4>(static_cast<float>(s_total));
                acc[t] = __builtin_fmaf(-Mp, pp, acc[t]);
                acc[t] = __builtin_fmaf(Dp, sp, acc[t]);
            }
            acc[t] = __builtin_fmaf(-M, static_cast<float>(p_total), acc[t]);
            acc[t] = __builtin_fmaf(D, static_cast<float>(s_total), acc[t]);
            // The chain advances HERE.  Its only reader is the store of the one lane per row that owns it, under a
            // condition, and without this the compiler sinks every fused step of the row into that block: the
            // operands of all steps (eight registers per step and token) stay live to the end, and the whole dependent
            // chain -- 32 operations for a row of 4096 values -- runs after the last weight bytes have arrived,
            // where nothing is left to overlap it.
            asm volatile("" : "+v"(acc[t]));
            if constexpr (INTS) {
                if (ints_row != nullptr && valid) {
                    ints_row[2 * i] = s_total;
                    ints_row[2 * i + 1] = p_total;
                }
            }
            // one-entry buffers replayed against three or four tokens (the eight-wave launch): token by token, or the
            // scheduler holds every token's staged row in registers at once and the kernel no longer fits two waves per SIMD
            if constexpr (U == 1 && NT >= 3) __builtin_amdgcn_sched_barrier(0);
        }
    }
}

// FUSEQ (single token, plain call): the activation arrives as f32 and every
// workgroup quantizes it to Q8_K itself, wave w taking super-blocks w, w+waves, ...,
// straight into the LDS staging area -- the arithmetic of quantize_q8_k_kernel,
// without the launch and the round trip through memory.
//
// SPR = 2: a wave owns 8 rows and two 4-lane groups per row work on neighbouring super-blocks
// (lane = 8*row + 4*h + c).  Twice the waves with half the steps each, for weights whose 16-row
// tiles alone leave one wave per SIMD; every sum keeps its order, so the results are the same bits.
//
// PLAIN: a plain call (no groups, no second weight).  The general entry reads its arguments in
// several dependent rounds (group tables, then what they point to): with the split factors'
// integer divisions that was about 600 instructions and four scalar-load round trips before the
// first weight request -- 0.8 us of a kernel that lives for eight (14336 x 4096: 8.05 -> 7.25 us).
// The plain entry has none of it, and the K split (a power of two) is shifts.
//
// DIRECT: the decode launch of an expert layer (one shared f32 token, y-slot = routed assignment, z = which of up to
// two weights) with its mode known at compile time, for the same reason (one-token MoE layer 44.1 -> 42.6 us).
//
// RING = number of slots (0: two alternating 4-super-block register buffers): the K part walked through a ring of small
// register buffers, one super-block per 4-lane group and step; NSTEPS > 0: the part's length in steps known at compile
// time, the walk unrolled.  See the walk below for why and the measurements.
//
// ROUTE (with DIRECT): the launch routes the token itself from the router's logits (Mixtral routing by every wave,
// moe_route_wave_values); y-slot = routed rank; the first workgroup leaves experts and weights in routed order.
//
// PAIR (with PLAIN): grid.z = 2, blockIdx.z = 1 streams a second weight of the same shape against the same token
// (gate and up of a dense FFN in one launch).
//
// MULTI (with PLAIN): up to four weights of one row length and one K cut but different row counts against the same
// token (the q, k and v projections of an attention block), their workgroups end to end along grid.x.
template <int NT, bool INTS, bool FUSEQ = false, int SPR = 1, bool WHOLE = false, bool PLAIN = false, bool LOADONLY = false, bool DIRECT = false,
          int RING = 0, int NSTEPS = 0, bool ROUTE = false, bool PAIR = false, bool MULTI = false>
__global__ __launch_bounds__(512) void gemv_q4k_kernel(Q4KArgs a_in) {
    static_assert(!PAIR || (PLAIN && FUSEQ && NT == 1), "a plain pair: one f32 token against two weights of one shape (grid.z = 2)");
    static_assert(!MULTI || (PLAIN && FUSEQ && NT == 1 && !PAIR && !LOADONLY), "a multi launch: one f32 token against several plain weights");
    Q4KArgs a = a_in;
    int bx = blockIdx.x;  // workgroup index within its weight
    if constexpr (MULTI) {
        // which weight this workgroup belongs to (wave-uniform selects: no indexed access to the argument block)
        const int j = (bx >= a_in.wg_end[0]) + (bx >= a_in.wg_end[1]) + (bx >= a_in.wg_end[2]);
        auto pick = [&](auto v0, auto v1, auto v2, auto v3) { return j == 0 ? v0 : (j == 1 ? v1 : (j == 2 ? v2 : v3)); };
        a.w = pick(a_in.wm[0], a_in.wm[1], a_in.wm[2], a_in.wm[3]);
        a.out = pick(a_in.outm[0], a_in.outm[1], a_in.outm[2], a_in.outm[3]);
        a.sb_stride = pick(a_in.stridem[0], a_in.stridem[1], a_in.stridem[2], a_in.stridem[3]);
        a.rows = pick(a_in.rowsm[0], a_in.rowsm[1], a_in.rowsm[2], a_in.rowsm[3]);
        a.row_skip = pick(a_in.skipm[0], a_in.skipm[1], a_in.skipm[2], a_in.skipm[3]);
        bx -= pick(0, a_in.wg_end[0], a_in.wg_end[1], a_in.wg_end[2]);
    }
    static_assert(!ROUTE || DIRECT, "only the direct launch routes");
    static_assert(!FUSEQ || ((NT == 1 || (NT == 2 && PLAIN)) && !INTS),
                  "the fused quantizer serves single-token calls and plain two-token calls (contiguous f32 rows)");
    static_assert(SPR == 1 || SPR == 2, "groups per row");
    constexpr int RPW = kWave / (LPS * SPR);  // rows per wave tile
    static_assert(RING == 0 || (RING >= 3 && RING <= 6 && WHOLE && (PLAIN || DIRECT)), "the ring serves plain and direct calls and needs no clamping");
    constexpr int NB = RING ? RING : 1;  // ring slots
    constexpr int PRE = RING ? 2 : 1;  // slots requested before the activation is staged (the rest right after)
    constexpr int U = RING ? 1 : 4 / SPR;  // buffer entries per group: two buffers of 4 super-blocks of a row, or a ring of 2-super-block ones
    constexpr int UB = U * SPR;
    using Regs = Q4KRegs<U>;
    extern __shared__ uint4 smem[];
    const int n_sb = a.n_sb;
    int8_t *ys = reinterpret_cast<int8_t *>(smem);                     // [NT][n_sb*256]
    int *bsum = reinterpret_cast<int *>(ys + NT * n_sb * 256);         // [NT][n_sb*8]
    float *yds = reinterpret_cast<float *>(bsum + NT * n_sb * 8);      // [NT][n_sb]
    float *part = yds + ((NT * n_sb + 3) & ~3);                        // [waves][NT][RPW]

    const int tid = threadIdx.x;
    const int nthreads = blockDim.x;
    static_assert(!(DIRECT && PLAIN), "a direct launch is a grouped one");
    const bool direct = DIRECT || (!PLAIN && a.group_offsets == nullptr && a.group_ids != nullptr);
    const bool grouped = !DIRECT && !PLAIN && a.group_offsets != nullptr;
    int64_t band;
    float4 x_early[4];  // ROUTE: the wave's first quantizer pass of the token, requested before the routing
    if constexpr (ROUTE) {
        // every wave routes the token for itself (no barrier, nothing shared): a few dozen vector
        // instructions and one expf in front of the first weight request, instead of a launch
        // (the logits are requested first, the wave's share of the f32 token right behind them: the
        // selection runs while the token is on its way)
        const int rl0 = tid & 63;
        const float rl_lo = rl0 < a.n_groups ? a.route_logits[rl0] : 0.0f, rl_hi = rl0 + 64 < a.n_groups ? a.route_logits[rl0 + 64] : 0.0f;
        __builtin_amdgcn_sched_barrier(0);
        {
            const int sbk = min(4 * (tid >> 6) + (rl0 >> 4), a.n_sb - 1);
#pragma unroll
            for (int kk = 0; kk < 4; kk++) x_early[kk] = reinterpret_cast<const float4 *>(a.x)[sbk * 64 + (rl0 & 15) * 4 + kk];
        }
        __builtin_amdgcn_sched_barrier(0);
        int sel_e, rank;
        float rw;
        moe_route_wave_values(rl_lo, rl_hi, a.n_groups, a.route_k, rl0, sel_e, rw, rank);
        const unsigned long long mine = __builtin_amdgcn_ballot_w64(rl0 < a.route_k && rank == static_cast<int>(blockIdx.y));
        band = __builtin_amdgcn_readlane(sel_e, mine ? __builtin_ctzll(mine) : 0);
        if (blockIdx.x == 0 && blockIdx.y == 0 && blockIdx.z == 0 && tid < a.route_k) {
            a.route_idx[rank] = sel_e;
            a.route_w[rank] = rw;
        }
    } else {
        band = DIRECT ? a.group_ids[blockIdx.y] : (grouped || direct) ? (a.group_ids ? a.group_ids[blockIdx.y] : static_cast<int>(blockIdx.y)) : 0;
    }
    if (band < 0 || (direct && band >= a.n_groups)) return;  // a y-slot past the groups in use, or an id out of range
    const int a0 = DIRECT ? static_cast<int>(blockIdx.y) : grouped ? a.group_offsets[band] : (direct ? static_cast<int>(blockIdx.y) : 0);  // first assignment of this group
    const int n_assign = DIRECT ? 1 : grouped ? a.group_offsets[band + 1] - a0 : (direct ? 1 : NT);
    if (n_assign <= 0) return;  // an expert nobody routed to: the whole workgroup leaves
    const bool second = (DIRECT || PAIR) ? blockIdx.z == 1 : (!PLAIN && gridDim.z > 1 && blockIdx.z == 1);
    const uint8_t *w = (second ? a.w2 : a.w) + band * (a.rows / 16) * kQ4KChunk;

    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
    const int W = a.ksplit;  // 1, 2, 4 or 8
    const int tile_in_wg = wave >> a.ksplit_log2, kpart = wave & (W - 1);
    const int tile = bx * a.tiles_per_wg + tile_in_wg;
    const int s0 = (kpart * n_sb) >> a.ksplit_log2;  // == kpart * n_sb / W
    const int s1 = ((kpart + 1) * n_sb) >> a.ksplit_log2;
    const int g = lane / LPS, l = lane - g * LPS;
    const int r = g / SPR, h = g - r * SPR;
    const int row = tile * RPW + r - a.row_skip;  // output row; negative for the skipped head of a view's first tile
    const bool live = row >= 0 && row < a.rows;
    // the last tile is padded to 16 rows; tiles past the end (grid rounding) re-read it and store nothing
    const int rl = (tile % SPR) * RPW + r;  // row in the 16-row layout tile
    const uint8_t *wtile = w + static_cast<int64_t>(min(tile / SPR, (a.rows + a.row_skip + 15) / 16 - 1)) * kQ4KChunk;
    const int piece = rl * LPS + l;
    // lane constants of the unclamped loads (WHOLE: every part is a whole number of buffers and
    // the stride fits 31 bits -- the launcher checks both)
    const uint32_t hoff = WHOLE ? static_cast<uint32_t>(h) * static_cast<uint32_t>(a.sb_stride) : 0u;
    const uint32_t hdr_off = hoff + rl * 16, q_off = hoff + piece * 16;
    auto load_buffer = [&](Regs &dst, int sb) __attribute__((always_inline)) {  // super-blocks sb .. sb+UB-1 of the row
        if constexpr (WHOLE)
            q4k_load_whole<U, SPR>(dst, wtile + static_cast<int64_t>(sb) * a.sb_stride, a.sb_stride, hdr_off, q_off);
        else
            q4k_load<U, SPR>(dst, wtile, a.sb_stride, rl, piece, sb + h, s1);
    };
    const bool gleader = (l == LPS - 1);          // holds its group's integers
    const bool leader = gleader && h == SPR - 1;  // runs the row's f32 chain
    Q4KLane ln;
    ln.c = l;
    ln.sh = (ln.c & 1) * 16;
    ln.upper = ln.c >= 2;
    const int c16 = n_sb * 16;       // 16-byte chunks per activation row
    const int n16 = NT * c16;        // even; blockDim is even: lanes 2k, 2k+1 are in or out together

    for (int p0 = 0; p0 < n_assign; p0 += NT) {
        // Activation row of local token t (clamped to the group's last assignment; extra tokens store nothing).
        auto act_row = [&](int t) -> int64_t {
            const int j = a0 + min(p0 + t, n_assign - 1);
            if (PLAIN) return j;
            if (DIRECT || a.shared_act) return 0;
            return a.group_rows ? a.group_rows[j] : j;
        };
        Regs ra, rb;
        Regs ring[NB];
        auto ring_prologue = [&]() __attribute__((always_inline)) {
#pragma unroll
            for (int k = 0; k < PRE; k++) load_buffer(ring[k], s0 + k * UB);
        };
        if constexpr (LOADONLY) {
            if constexpr (RING) ring_prologue(); else
            load_buffer(ra, s0);
        } else if constexpr (FUSEQ) {
            // f32 loads of the first batch, the first weight buffer right behind
            // them, then the quantizer: HBM requests are in flight while it runs.
            // A 16-lane row per super-block: a wave quantizes four at a time (pass p of wave w
            // takes super-blocks 4*(w + p*waves) ..+3), lane l of a row holding values 16l..16l+15.
            const int nw = nthreads >> 6;
            const int qrow = lane >> 4, ql = lane & 15;
            const float4 *x4 = reinterpret_cast<const float4 *>(a.x + act_row(0) * n_sb * 256);
            // NT = 2 (plain call): the two f32 rows are contiguous and so are their staging areas, so
            // the tokens are simply 2 * n_sb super-blocks in a row.
            const int tq = NT * n_sb;
            auto load_pass = [&](float4 (&xv)[4], int base) {
                const int sbk = min(base + qrow, tq - 1);
#pragma unroll
                for (int k = 0; k < 4; k++) xv[k] = x4[sbk * 64 + ql * 4 + k];
            };
            auto quantize_pass = [&](const float4 (&xv)[4], int base) {
                const int sbk = base + qrow;
                float dv;
                int bs;
                const uint4 packed = q8k_quantize_row16(xv, lane, dv, bs);
                if (sbk < tq) {
                    reinterpret_cast<uint4 *>(ys)[sbk * 16 + ql] = packed;
                    if (ql & 1) bsum[sbk * 8 + (ql >> 1)] = bs;
                    if (ql == 0) yds[sbk] = dv;
                }
            };
            float4 xa[4], xb[4];
            if constexpr (ROUTE) {
#pragma unroll
                for (int kk = 0; kk < 4; kk++) xa[kk] = x_early[kk];
            } else {
                load_pass(xa, 4 * wave);
            }
            __builtin_amdgcn_sched_barrier(0);
            if constexpr (RING) ring_prologue(); else
            load_buffer(ra, s0);
            __builtin_amdgcn_sched_barrier(0);
            for (int base = 4 * wave;;) {
                const int next = base + 4 * nw;
                if (next >= tq) {
                    quantize_pass(xa, base);
                    break;
                }
                load_pass(xb, next);
                quantize_pass(xa, base);
#pragma unroll
                for (int k = 0; k < 4; k++) xa[k] = xb[k];
                base = next;
            }
            __syncthreads();
        } else {
            // Prologue: activation loads first, the first weight buffer right behind
            // them, then the LDS writes -- so HBM requests are in flight while the
            // activation is staged.
            uint4 *dst = reinterpret_cast<uint4 *>(ys);
            uint4 sv[kQ4KStageRegs];
    #pragma unroll
            for (int k = 0; k < kQ4KStageRegs; k++) {
                const int i = min(tid + k * nthreads, n16 - 1);
                const int t = NT == 1 ? 0 : i / c16;
                sv[k] = reinterpret_cast<const uint4 *>(a.q + act_row(t) * n_sb * 256)[i - t * c16];
            }
            float yd0;
            {
                const int i = min(tid, NT * n_sb - 1);
                const int t = NT == 1 ? 0 : i / n_sb;
                yd0 = a.yd[act_row(t) * n_sb + (i - t * n_sb)];
            }

            __builtin_amdgcn_sched_barrier(0);
            if constexpr (RING) ring_prologue(); else
            load_buffer(ra, s0);
            __builtin_amdgcn_sched_barrier(0);

    #pragma unroll
            for (int k = 0; k < kQ4KStageRegs; k++) {
                const int i = tid + k * nthreads;
                int s = bytesum16(sv[k]);
                s += row_shr_i32<1>(s);
                if (i < n16) {
                    dst[i] = sv[k];
                    if (i & 1) bsum[i >> 1] = s;
                }
            }
            for (int i = tid + kQ4KStageRegs * nthreads; i < n16; i += nthreads) {
                const int t = NT == 1 ? 0 : i / c16;
                const uint4 v = reinterpret_cast<const uint4 *>(a.q + act_row(t) * n_sb * 256)[i - t * c16];
                dst[i] = v;
                int s = bytesum16(v);
                s += row_shr_i32<1>(s);
                if (i & 1) bsum[i >> 1] = s;
            }
            if (tid < NT * n_sb) yds[tid] = yd0;
            for (int i = tid + nthreads; i < NT * n_sb; i += nthreads) {
                const int t = NT == 1 ? 0 : i / n_sb;
                yds[i] = a.yd[act_row(t) * n_sb + (i - t * n_sb)];
            }
            __syncthreads();

        }

        int32_t *ints_row = nullptr;
        if constexpr (INTS) {
            if (a.ints && gleader && live) ints_row = a.ints + (band * a.rows + row) * static_cast<int64_t>(n_sb) * 2;
        }

        float acc[NT];
#pragma unroll
        for (int t = 0; t < NT; t++) acc[t] = 0.0f;

        // Two register buffers alternate: the next buffer's loads are issued, then
        // the current one is consumed.  The last buffer is consumed without issuing
        // anything, so no load is wasted; sched_barrier keeps the loads ahead of
        // the arithmetic they overlap with.
        if constexpr (RING) {
            // A ring of NB small buffers (one super-block per 4-lane group and step: two
            // super-blocks of a row for 8-row waves, one for 16-row waves) instead of two
            // 4-super-block ones.  Fewer bytes are in flight per wave, but a slot is requested
            // again after one step's arithmetic instead of four super-blocks', so the wave's
            // requests never drop to half.  14336 x 4096, 8-row waves: 7.21 -> 6.78 us with three
            // slots (two slots 7.3-7.4, four 6.81, five 7.05, six 7.27; all three requested before
            // the quantizer 6.92, one 7.00).  16-row waves (two-token calls): four slots, 9.60 ->
            // 8.87 us (three 8.99, five 8.88, six 8.98).  The part holds n >= NB steps (the
            // launcher checks).  Whole turns of the ring run in a loop; the last NB..2NB-1 steps
            // are straight-line code per remainder, so that every wait counts exactly the loads
            // behind the buffer it needs -- a load under a condition would make each later wait
            // assume it had not been issued.
            auto compute = [&](const Regs &b, int step) __attribute__((always_inline)) {
                q4k_compute<NT, INTS, U, SPR, WHOLE, LOADONLY>(b, ln, s0 + step * UB + h, s1, ys, bsum, yds, n_sb, acc, ints_row);
                __builtin_amdgcn_sched_barrier(0);
            };
            auto request = [&](Regs &b, int step) __attribute__((always_inline)) {
                load_buffer(b, s0 + step * UB);
                __builtin_amdgcn_sched_barrier(0);
            };
#pragma unroll
            for (int j = PRE; j < NB; j++) request(ring[j], j);
            if constexpr (NSTEPS > 0) {
                // the part's length known at compile time (NSTEPS steps: the launcher checks): the
                // whole walk is straight-line code (14336 x 4096: 6.89 -> 6.81 us against the loop below)
                static_assert(NSTEPS >= NB, "a part holds at least one full ring");
#pragma unroll
                for (int i = 0; i < NSTEPS; i++) {
                    compute(ring[i % NB], i);
                    if (i + NB < NSTEPS) request(ring[i % NB], i + NB);
                }
            } else {
            const int n = (s1 - s0) / UB;
            int k = 0;
            for (; k + 2 * NB <= n; k += NB) {
#pragma unroll
                for (int j = 0; j < NB; j++) {
                    compute(ring[j], k + j);
                    request(ring[j], k + NB + j);
                }
            }
            auto tail = [&](auto extra) __attribute__((always_inline)) {  // `extra` steps are not requested yet
                constexpr int E = decltype(extra)::value;
#pragma unroll
                for (int j = 0; j < NB; j++) {
                    compute(ring[j], k + j);
                    if (j < E) request(ring[j], k + NB + j);
                }
#pragma unroll
                for (int j = 0; j < E; j++) compute(ring[j], k + NB + j);
            };
            switch (n - k - NB) {
                case 0: tail(std::integral_constant<int, 0>{}); break;
                case 1: tail(std::integral_constant<int, 1>{}); break;
                case 2: tail(std::integral_constant<int, 2>{}); break;
                case 3: if constexpr (NB > 3) tail(std::integral_constant<int, 3>{}); break;
                case 4: if constexpr (NB > 4) tail(std::integral_constant<int, 4>{}); break;
                default: if constexpr (NB > 5) tail(std::integral_constant<int, 5>{}); break;
            }
            }
        } else
        for (int sb = s0;;) {
            if (sb + UB >= s1) {
                q4k_compute<NT, INTS, U, SPR, WHOLE, LOADONLY>(ra, ln, sb + h, s1, ys, bsum, yds, n_sb, acc, ints_row);
                break;
            }
            load_buffer(rb, sb + UB);
            __builtin_amdgcn_sched_barrier(0);
            q4k_compute<NT, INTS, U, SPR, WHOLE, LOADONLY>(ra, ln, sb + h, s1, ys, bsum, yds, n_sb, acc, ints_row);
            __builtin_amdgcn_sched_barrier(0);
            sb += UB;
            if (sb + UB >= s1) {
                q4k_compute<NT, INTS, U, SPR, WHOLE, LOADONLY>(rb, ln, sb + h, s1, ys, bsum, yds, n_sb, acc, ints_row);
                break;
            }
            load_buffer(ra, sb + UB);
            __builtin_amdgcn_sched_barrier(0);
            q4k_compute<NT, INTS, U, SPR, WHOLE, LOADONLY>(rb, ln, sb + h, s1, ys, bsum, yds, n_sb, acc, ints_row);
            __builtin_amdgcn_sched_barrier(0);
            sb += UB;
        }

        if constexpr (LOADONLY) {
            // keeps the loads alive; the condition does not hold for weights written by this library's upload
            if (__builtin_bit_cast(uint32_t, acc[0]) == 0x12345679u && a.out) a.out[0] = 1.0f;
            return;
        }
        float *out = (second ? a.out2 : a.out) + static_cast<int64_t>(a0 + p0) * a.rows;  // output row of local token 0
        const int n_here = min(NT, n_assign - p0);
        if (W == 1) {
            if (leader && live) {
#pragma unroll
                for (int t = 0; t < NT; t++) {
                    if (t < n_here) {
                        float v = acc[t];
                        if (NT == 1 && a.residual) v = v + a.residual[row];
                        out[static_cast<int64_t>(t) * a.rows + row] = v;
                    }
                }
            }
        } else {
            if (leader) {
#pragma unroll
                for (int t = 0; t < NT; t++) part[(wave * NT + t) * RPW + r] = acc[t];
            }
            __syncthreads();
            for (int i = tid; i < a.tiles_per_wg * NT * RPW; i += nthreads) {
                const int rr = i % RPW;
                const int t = (i / RPW) % NT;
                const int tw = i / (RPW * NT);
                const int orow = (bx * a.tiles_per_wg + tw) * RPW + rr - a.row_skip;
                if (orow < 0 || orow >= a.rows || t >= n_here) continue;
                float v = part[((tw * W) * NT + t) * RPW + rr];
                for (int k = 1; k < W; k++) v = v + part[((tw * W + k) * NT + t) * RPW + rr];
                if (NT == 1 && a.residual) v = v + a.residual[orow];
                out[static_cast<int64_t>(t) * a.rows + orow] = v;
            }
        }
        if (p0 + NT < n_assign) __syncthreads();  // the next pass overwrites the staged activation
    }
}

// ---- the single-token launch of whole rows: eight-wave workgroups, scalar arguments ------------
//
// The plain fused single-token matvec of rows of 2 * NSTEPS super-blocks with no K cut (the decode
// shape: 14336 x 4096).  Arithmetic and association are exactly those of
// gemv_q4k_kernel<1, .., SPR = 2, RING = 3> above (same loads, same q4k_compute, same chain); the
// launch is rebuilt around its two ends, which is where a kernel that lives for six microseconds
// loses against its own weight stream:
//   * eight waves per workgroup -- 224 workgroups for 14336 rows, one per compute unit and two
//     waves per SIMD everywhere, instead of 448 four-wave ones of which most units got two and a
//     quarter got one; a unit's second workgroup had its f32 activation queued behind the first
//     one's weight requests in the unit's in-order memory pipe (0.7-1.0 us late);
//   * an execution barrier between the activation requests and the weight requests, so that in that
//     pipe every wave's share of the activation is ahead of every weight request of the workgroup;
//   * the quantizer with a 32-lane half wave per super-block: the eight waves quantize the sixteen
//     super-blocks of a row in ONE pass, eight values per lane, about half the instructions per wave
//     of the 16-lane form (q8k_quantize_row32);
//   * a 48-byte argument block and statically sized LDS: one scalar load and no size arithmetic
//     before the first address.  (Plain scalar arguments preloaded into SGPRs by the command
//     processor, -amdgpu-kernarg-preload-count, measured the same time to within noise, and
//     rocprofv3 could not follow graph replays of that form of the kernel; the argument block is a
//     struct by value like every other kernel's here.)
// Measured on 14336 x 4096, same box, same run: 6.84 -> 6.65 us.  With the activation taken out
// altogether (no f32 loads, no quantizer, no barriers: ABLATE = 1) the launch takes the same time,
// so nothing is left in the prologue; without the output store (4) 6.30; without arithmetic and
// store (the weight requests alone, 7) 6.0-6.06.  What remains above the bare request stream is the
// drain -- the last step's arithmetic after the last bytes arrive, and the store's way to L2.
//
// ABLATE (timing experiments, reachable only through cml_calibrate_matvec_ablation; results are
// wrong): 1 = no activation, 2 = no arithmetic, 4 = no store.
struct Q4KCuArgs {
    const uint8_t *w;       // tiled layout, as Q4KArgs::w
    const float *x;         // the f32 token
    float *out;             // [rows]
    const float *residual;  // [rows] or null
    uint32_t sb_stride;     // bytes between consecutive super-blocks of one tile (below 2 GiB)
    int rows, row_skip;     // as Q4KArgs
    int tiles16;            // 16-row layout tiles that hold the rows
};

// The K-cut form against up to four weights of one row length and one K cut (any row counts) in one launch: their
// workgroups lie end to end along grid.x, every workgroup quantizes the token once.
struct Q4KCuMultiArgs {
    const float *x;          // the f32 token
    const uint8_t *wm[4];    // tiled layouts
    float *outm[4];          // [rowsm[j]] each
    uint32_t stridem[4];     // bytes between consecutive super-blocks of one tile
    int rowsm[4], skipm[4], tiles16m[4];
    int wg_end[4];           // workgroups of weights 0 .. j (INT32_MAX beyond the last weight)
};

// NT (1 to 4) tokens: the f32 rows are contiguous ([NT][row length]), pass p of the quantizer takes token p, the
// unpacked weight of a step is replayed against the NT staged rows from registers, and token t writes out[t][rows]
// -- every cell the one-token result, bit for bit (the same q4k_compute).  The weight streams once for the NT tokens
// and the vector work per step grows by about 60 instructions per token, which the stream hides up to three
// tokens and nearly at four.
template <int NSTEPS, int ABLATE = 0, int NT = 1, int WAVES = 8>
__global__ __launch_bounds__(WAVES * 64) void gemv_q4k_cu_kernel(Q4KCuArgs a) {
    const uint8_t *__restrict__ w = a.w;
    const float *__restrict__ x = a.x;
    float *__restrict__ out = a.out;
    const float *__restrict__ residual = a.residual;
    const uint32_t sb_stride = a.sb_stride;
    const int rows = a.rows, row_skip = a.row_skip, tiles16 = a.tiles16;
    constexpr int NSB = 2 * NSTEPS;  // super-blocks per row
    constexpr int NB = 3, PRE = 2;   // ring slots; slots requested before the quantizer
    constexpr int PASSES = (NSB + 2 * WAVES - 1) / (2 * WAVES);  // quantizer passes per token: 2 * WAVES super-blocks each
    static_assert(NSTEPS >= NB && PASSES <= 2, "at most two quantizer passes cover a row");
    static_assert(NT >= 1 && NT <= 4 && (NT == 1 || ABLATE == 0), "up to four tokens; the ablations are one-token launches");
    constexpr bool NOACT = (ABLATE & 1) != 0, NOMATH = (ABLATE & 2) != 0, NOSTORE = (ABLATE & 4) != 0;
    using Regs = Q4KRegs<1>;
    __shared__ __attribute__((aligned(16))) int8_t ys[NT * NSB * 256];
    __shared__ int bsum[NT * NSB * 8];
    __shared__ float yds[NT * NSB];
    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;

    // the f32 activation: pass p of wave w quantizes super-blocks 2 (w + WAVES p) and the next of every token, a half wave each
    const int half = lane >> 5, ql = lane & 31;
    float4 xv[NT][PASSES][2];
    if constexpr (!NOACT) {
#pragma unroll
        for (int t = 0; t < NT; t++) {
#pragma unroll
            for (int p = 0; p < PASSES; p++) {
                const int sbk = 2 * (wave + WAVES * p) + half;
                const float4 *x4 = reinterpret_cast<const float4 *>(x) + (t * NSB + min(sbk, NSB - 1)) * 64 + ql * 2;
                xv[t][p][0] = x4[0];
                xv[t][p][1] = x4[1];
            }
        }
    }
    __builtin_amdgcn_sched_barrier(0);
    if constexpr (!NOACT) __builtin_amdgcn_s_barrier();  // execution only: every activation request of the workgroup is out
    __builtin_amdgcn_sched_barrier(0);

    const int tile = blockIdx.x * WAVES + wave;  // 8-row half tile
    const int g = lane / LPS, l = lane - g * LPS;
    const int r = g >> 1, h = g & 1;
    const int row = tile * 8 + r - row_skip;  // negative for the skipped head of a view's first tile
    const bool live = row >= 0 && row < rows;
    const int rl = (tile & 1) * 8 + r;        // row in the 16-row layout tile
    // half tiles past the end (grid rounding) re-read the last tile and store nothing
    const uint8_t *wtile = w + static_cast<int64_t>(min(tile >> 1, tiles16 - 1)) * kQ4KChunk;
    const uint32_t hoff = static_cast<uint32_t>(h) * sb_stride;
    const uint32_t hdr_off = hoff + rl * 16, q_off = hoff + (rl * LPS + l) * 16;
    Regs ring[NB];
    auto request = [&](Regs &b, int step) __attribute__((always_inline)) {
        q4k_load_whole<1, 2>(b, wtile + static_cast<int64_t>(2 * step) * sb_stride, sb_stride, hdr_off, q_off);
        __builtin_amdgcn_sched_barrier(0);
    };
#pragma unroll
    for (int k = 0; k < PRE; k++) request(ring[k], k);

    if constexpr (!NOACT) {
        // Every wave runs the quantizer (a wave without a super-block of its own redoes the last one and
        // stores nothing): the f32 loads above are then used unconditionally, and the compiler cannot
        // sink them into a conditional block behind the weight requests.
#pragma unroll
        for (int t = 0; t < NT; t++) {
#pragma unroll
            for (int p = 0; p < PASSES; p++) {
                const int sbk = 2 * (wave + WAVES * p) + half;
                const bool mine = NSB == 2 * WAVES * PASSES || sbk < NSB;
                float dv;
                int bs;
                const uint2 packed = q8k_quantize_row32(xv[t][p], lane, dv, bs);
                if (mine) {
                    const int at = t * NSB + sbk;
                    reinterpret_cast<uint2 *>(ys)[at * 32 + ql] = packed;
                    if ((ql & 3) == 3) bsum[at * 8 + (ql >> 2)] = bs;
                    if (ql == 0) yds[at] = dv;
                }
                if constexpr (NT * PASSES >= 3) __builtin_amdgcn_sched_barrier(0);  // one pass at a time: the passes interleaved need too many registers
            }
        }
        __syncthreads();
    }

    Q4KLane ln;
    ln.c = l;
    ln.sh = (l & 1) * 16;
    ln.upper = l >= 2;
    float acc[NT];
#pragma unroll
    for (int t = 0; t < NT; t++) acc[t] = 0.0f;
    auto compute = [&](const Regs &b, int step) __attribute__((always_inline)) {
        q4k_compute<NT, false, 1, 2, true, NOMATH>(b, ln, 2 * step + h, NSB, ys, bsum, yds, NSB, acc, nullptr);
        __builtin_amdgcn_sched_barrier(0);
    };
#pragma unroll
    for (int j = PRE; j < NB; j++) request(ring[j], j);
#pragma unroll
    for (int i = 0; i < NSTEPS; i++) {
        compute(ring[i % NB], i);
        if (i + NB < NSTEPS) request(ring[i % NB], i + NB);
    }
    if constexpr (NOSTORE) {
        // keeps the arithmetic alive; the condition does not hold for weights written by this library's upload
        if (__builtin_bit_cast(uint32_t, acc[0]) == 0x12345679u) out[0] = 1.0f;
        return;
    }
    if (l == LPS - 1 && h == 1 && live) {  // the second group's last lane ran the row's chains
#pragma unroll
        for (int t = 0; t < NT; t++) {
            float v = acc[t];
            if (NT == 1 && residual) v = v + residual[row];
            out[static_cast<int64_t>(t) * rows + row] = v;
        }
    }
}

// The same launch for a weight whose shape the policy cuts K for (few row tiles, long rows: the FFN down projection,
// 4096 x 14336): a workgroup's eight waves are 8 / KS half tiles x KS parts of NSTEPS steps each, the workgroup
// quantizes the WHOLE row once (56 super-blocks: 28 pairs over the eight waves, four passes of the 32-lane quantizer
// with every f32 request out before the first weight request), every wave then walks its own part, and the KS partial
// chains of a row are added left to right through LDS -- the association of gemv_q4k_kernel under the same K cut, so
// the same bits.  The two-launch form (a quantizing launch, then the matvec) takes 9.1 us per step at 4096 x 14336 for
// a 7.1 us matvec; the four-wave kernel with the quantizer inside took 10.0 (512 workgroups each quantizing the row).
// With the whole row quantized before the walk the launch takes 7.64 us, of which the activation path is 0.97 (6.66
// without it: every workgroup quantizes all 14336 values, four quantizer passes per wave against one in the uncut launch,
// where they hide), the combine and store 0.38 (7.26 without), the weight requests alone 6.02; STAGED brings it to 7.19.
// ABLATE: as in gemv_q4k_cu_kernel (timing experiments; results are wrong).
// STAGED: the quantizer passes are interleaved with the walk.  Pass p quantizes, for every K part, the two super-block
// pairs its steps 2p and 2p + 1 read (the part's two waves take one pair each), so after pass 0 and one barrier every
// wave starts walking, and pass p + 1 runs between the requests and the arithmetic of steps 2p, 2p + 1: the weight
// stream never waits for a whole row to be quantized.
template <int KS, int NSTEPS, int ABLATE = 0, bool STAGED = false, int WAVES = 8, bool MULTI = false>
__global__ __launch_bounds__(WAVES * 64) void gemv_q4k_cu_kcut_kernel(std::conditional_t<MULTI, Q4KCuMultiArgs, Q4KCuArgs> a) {
    static_assert(!STAGED || (KS == 4 && NSTEPS == 7 && WAVES == 8), "the staged quantizer: four K parts of seven steps, two waves each");
    static_assert(!MULTI || (ABLATE == 0 && !STAGED), "the multi launch: the plain short form");
    constexpr bool NOACT = (ABLATE & 1) != 0, NOMATH = (ABLATE & 2) != 0, NOSTORE = (ABLATE & 4) != 0;
    const uint8_t *__restrict__ w;
    const float *__restrict__ x = a.x;
    float *__restrict__ out;
    const float *__restrict__ residual;
    uint32_t sb_stride;
    int rows, row_skip, tiles16;
    int bx = blockIdx.x;  // workgroup index within its weight
    if constexpr (MULTI) {
        // which weight this workgroup belongs to (wave-uniform selects: no indexed access to the argument block)
        const int j = (bx >= a.wg_end[0]) + (bx >= a.wg_end[1]) + (bx >= a.wg_end[2]);
        auto pick = [&](auto v0, auto v1, auto v2, auto v3) { return j == 0 ? v0 : (j == 1 ? v1 : (j == 2 ? v2 : v3)); };
        w = pick(a.wm[0], a.wm[1], a.wm[2], a.wm[3]);
        out = pick(a.outm[0], a.outm[1], a.outm[2], a.outm[3]);
        residual = nullptr;
        sb_stride = pick(a.stridem[0], a.stridem[1], a.stridem[2], a.stridem[3]);
        rows = pick(a.rowsm[0], a.rowsm[1], a.rowsm[2], a.rowsm[3]);
        row_skip = pick(a.skipm[0], a.skipm[1], a.skipm[2], a.skipm[3]);
        tiles16 = pick(a.tiles16m[0], a.tiles16m[1], a.tiles16m[2], a.tiles16m[3]);
        bx -= pick(0, a.wg_end[0], a.wg_end[1], a.wg_end[2]);
    } else {
        w = a.w;
        out = a.out;
        residual = a.residual;
        sb_stride = a.sb_stride;
        rows = a.rows, row_skip = a.row_skip, tiles16 = a.tiles16;
    }
    constexpr int TPW = WAVES / KS;              // half tiles per workgroup
    constexpr int NSB = KS * 2 * NSTEPS;         // super-blocks per row
    constexpr int PAIRS = NSB / 2, PASSES = (PAIRS + WAVES - 1) / WAVES;
    // (more slots requested ahead of the quantizer are slower: 3 of 3 7.87 us, 4 of 4 7.85, 5 of 5 8.1, all 7 9.45 against 7.64 --
    // requests for several far-apart super-blocks per wave at once break up the front the grid sweeps the matrix with)
    constexpr int NB = NSTEPS < 3 ? NSTEPS : 3, PRE = 2;
    static_assert((KS == 2 || KS == 4 || KS == 8) && WAVES % KS == 0 && NSTEPS >= 2, "K parts of at least two steps");
    using Regs = Q4KRegs<1>;
    __shared__ __attribute__((aligned(16))) int8_t ys[NSB * 256];
    __shared__ int bsum[NSB * 8];
    __shared__ float yds[NSB];
    __shared__ float part[WAVES * 8];
    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;

    // the f32 activation: pass p of wave w quantizes the super-block pair w + 8 p (STAGED: pair 2p + (w / KS) of K part
    // w % KS), a half wave per super-block
    const int half = lane >> 5, ql = lane & 31;
    auto pair_of = [&](int p) __attribute__((always_inline)) -> int {
        if constexpr (STAGED) return NSTEPS * (wave % KS) + min(2 * p + wave / KS, NSTEPS - 1);
        else return min(wave + WAVES * p, PAIRS - 1);
    };
    auto pair_mine = [&](int p) __attribute__((always_inline)) -> bool {
        if constexpr (STAGED) return 2 * p + wave / KS < NSTEPS;
        else return WAVES * (p + 1) <= PAIRS || wave + WAVES * p < PAIRS;
    };
    float4 xv[PASSES][2];
    if constexpr (!NOACT) {
#pragma unroll
        for (int p = 0; p < PASSES; p++) {
            const int sbk = 2 * pair_of(p) + half;
            const float4 *x4 = reinterpret_cast<const float4 *>(x) + sbk * 64 + ql * 2;
            xv[p][0] = x4[0];
            xv[p][1] = x4[1];
        }
        __builtin_amdgcn_sched_barrier(0);
        __builtin_amdgcn_s_barrier();  // execution only: every activation request of the workgroup is out
        __builtin_amdgcn_sched_barrier(0);
    }

    const int tile_in_wg = wave / KS, kpart = wave - tile_in_wg * KS;
    const int tile = bx * TPW + tile_in_wg;  // 8-row half tile
    const int s0 = kpart * 2 * NSTEPS;               // first super-block of this wave's part
    const int g = lane / LPS, l = lane - g * LPS;
    const int r = g >> 1, h = g & 1;
    const int rl = (tile & 1) * 8 + r;
    const uint8_t *wtile = w + static_cast<int64_t>(min(tile >> 1, tiles16 - 1)) * kQ4KChunk;
    const uint32_t hoff = static_cast<uint32_t>(h) * sb_stride;
    const uint32_t hdr_off = hoff + rl * 16, q_off = hoff + (rl * LPS + l) * 16;
    Regs ring[NB];
    auto request = [&](Regs &b, int step) __attribute__((always_inline)) {
        q4k_load_whole<1, 2>(b, wtile + static_cast<int64_t>(s0 + 2 * step) * sb_stride, sb_stride, hdr_off, q_off);
        __builtin_amdgcn_sched_barrier(0);
    };
#pragma unroll
    for (int k = 0; k < PRE; k++) request(ring[k], k);

    // every wave runs every pass (a wave without a pair of its own in the last pass redoes the last pair and stores
    // nothing): the f32 loads above are then used unconditionally and stay ahead of the weight requests
    auto quantize_pass = [&](int p) __attribute__((always_inline)) {
        const int sbk = 2 * pair_of(p) + half;
        float dv;
        int bs;
        const uint2 packed = q8k_quantize_row32(xv[p], lane, dv, bs);
        if (pair_mine(p)) {
            reinterpret_cast<uint2 *>(ys)[sbk * 32 + ql] = packed;
            if ((ql & 3) == 3) bsum[sbk * 8 + (ql >> 2)] = bs;
            if (ql == 0) yds[sbk] = dv;
        }
        __builtin_amdgcn_sched_barrier(0);
    };
    if constexpr (!NOACT) {
        if constexpr (STAGED) {
            quantize_pass(0);
        } else {
#pragma unroll
            for (int p = 0; p < PASSES; p++) quantize_pass(p);
        }
        __syncthreads();
    }

    Q4KLane ln;
    ln.c = l;
    ln.sh = (l & 1) * 16;
    ln.upper = l >= 2;
    float acc[1] = {0.0f};
    auto compute = [&](const Regs &b, int step) __attribute__((always_inline)) {
        q4k_compute<1, false, 1, 2, true, NOMATH>(b, ln, s0 + 2 * step + h, NSB, ys, bsum, yds, NSB, acc, nullptr);
        __builtin_amdgcn_sched_barrier(0);
    };
#pragma unroll
    for (int j = PRE; j < NB; j++) request(ring[j], j);
#pragma unroll
    for (int i = 0; i < NSTEPS; i++) {
        if constexpr (STAGED && !NOACT) {
            // before steps 2p - 2 and 2p - 1: pass p, for steps 2p and 2p + 1; a barrier before step 2p makes it visible
            // (the pass behind the step's re-request instead of ahead of the step: 7.62 us against 7.19-7.3)
            if (i % 2 == 0 && i / 2 + 1 < PASSES) quantize_pass(i / 2 + 1);
            if (i % 2 == 0 && i > 0) __syncthreads();
        }
        compute(ring[i % NB], i);
        if (i + NB < NSTEPS) request(ring[i % NB], i + NB);
    }
    if constexpr (NOSTORE) {
        // keeps the arithmetic alive; the condition does not hold for weights written by this library's upload
        if (__builtin_bit_cast(uint32_t, acc[0]) == 0x12345679u) out[0] = 1.0f;
        return;
    }
    if (l == LPS - 1 && h == 1) part[wave * 8 + r] = acc[0];
    __syncthreads();
    if (tid < TPW * 8) {
        const int tw = tid >> 3, rr = tid & 7;
        const int orow = (bx * TPW + tw) * 8 + rr - row_skip;
        if (orow >= 0 && orow < rows) {
            float v = part[(tw * KS) * 8 + rr];
#pragma unroll
            for (int k = 1; k < KS; k++) v = v + part[(tw * KS + k) * 8 + rr];
            if (residual) v = v + residual[orow];
            out[orow] = v;
        }
    }
}

// The K-cut form for rows the cut does not divide into whole two-super-block steps (rows of 43 super-blocks cut four
// ways: parts of 10, 11, 11, 11; an odd part length; 5120 values cut four ways: parts of 5).  The parts are those of
// gemv_q4k_kernel, [k n / KS, (k + 1) n / KS), so the association and the bits are the same.  Every part runs MAXSTEPS
// steps: all but the last lie wholly inside every part (whole loads, no masks), the last one may be half or wholly
// outside its part (clamped loads, masked terms).  The quantizer is staged as in the 14336-value form: the wave of
// half tile t and part k quantizes the super-blocks of step TPW p + t of part k in pass p, a barrier in front of
// step TPW p makes them visible, and pass p + 1 runs ahead of that step's arithmetic.
struct Q4KCuAnyArgs {
    Q4KCuArgs one;
    int n_sb;  // super-blocks per row
};

// NT (1 to 3) tokens: contiguous f32 rows in, out[t][rows]; every pass quantizes its super-blocks of all the tokens,
// and a step's unpacked weight is replayed against them -- every cell the one-token launch's bits.
template <int KS, int MAXSTEPS, int WAVES = 8, int NT = 1>
__global__ __launch_bounds__(WAVES * 64) void gemv_q4k_cu_kcut_any_kernel(Q4KCuAnyArgs aa) {
    const Q4KCuArgs &a = aa.one;
    const uint8_t *__restrict__ w = a.w;
    const float *__restrict__ x = a.x;
    float *__restrict__ out = a.out;
    const float *__restrict__ residual = a.residual;
    const uint32_t sb_stride = a.sb_stride;
    const int rows = a.rows, row_skip = a.row_skip, tiles16 = a.tiles16, n_sb = aa.n_sb;
    constexpr int TPW = WAVES / KS;  // half tiles per workgroup = waves per K part
    static_assert(WAVES % KS == 0 && WAVES >= 8 && WAVES <= 16, "whole half tiles per workgroup");
    constexpr int PASSES = (MAXSTEPS + TPW - 1) / TPW;
    constexpr int NB = MAXSTEPS < 3 ? MAXSTEPS : 3, PRE = 2;
    static_assert((KS == 2 || KS == 4 || KS == 8) && MAXSTEPS >= 2, "K parts of at least two steps");
    static_assert(NT >= 1 && NT <= 4, "one to four tokens");
    using Regs = Q4KRegs<1>;
    extern __shared__ uint4 smem_any[];
    int8_t *ys = reinterpret_cast<int8_t *>(smem_any);               // [NT][n_sb * 256]
    int *bsum = reinterpret_cast<int *>(ys + NT * n_sb * 256);       // [NT][n_sb * 8]
    float *yds = reinterpret_cast<float *>(bsum + NT * n_sb * 8);    // [NT][n_sb]
    float *part = yds + ((NT * n_sb + 3) & ~3);                      // [WAVES][NT][8]
    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
    const int tile_in_wg = wave / KS, kpart = wave - tile_in_wg * KS;
    const int s0 = (kpart * n_sb) / KS, s1 = ((kpart + 1) * n_sb) / KS;  // this wave's part

    // the f32 activation: pass p of this wave takes the two super-blocks of step TPW p + tile_in_wg of its own part
    const int half = lane >> 5, ql = lane & 31;
    auto pass_sb = [&](int p) __attribute__((always_inline)) -> int { return s0 + 2 * (TPW * p + tile_in_wg) + half; };
    float4 xv[PASSES][NT][2];
#pragma unroll
    for (int p = 0; p < PASSES; p++) {
#pragma unroll
        for (int t = 0; t < NT; t++) {
            const float4 *x4 = reinterpret_cast<const float4 *>(x) + (t * n_sb + min(pass_sb(p), n_sb - 1)) * 64 + ql * 2;
            xv[p][t][0] = x4[0];
            xv[p][t][1] = x4[1];
        }
    }
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_barrier();  // execution only: every activation request of the workgroup is out
    __builtin_amdgcn_sched_barrier(0);

    const int tile = blockIdx.x * TPW + tile_in_wg;  // 8-row half tile
    const int g = lane / LPS, l = lane - g * LPS;
    const int r = g >> 1, h = g & 1;
    const int rl = (tile & 1) * 8 + r;
    const uint8_t *wtile = w + static_cast<int64_t>(min(tile >> 1, tiles16 - 1)) * kQ4KChunk;
    const uint32_t hoff = static_cast<uint32_t>(h) * sb_stride;
    const uint32_t hdr_off = hoff + rl * 16, q_off = hoff + (rl * LPS + l) * 16;
    Regs ring[NB];
    auto request = [&](Regs &b, int step) __attribute__((always_inline)) {
        if (step < MAXSTEPS - 1) q4k_load_whole<1, 2>(b, wtile + static_cast<int64_t>(s0 + 2 * step) * sb_stride, sb_stride, hdr_off, q_off);
        else q4k_load<1, 2>(b, wtile, sb_stride, rl, rl * LPS + l, s0 + 2 * step + h, s1);
        __builtin_amdgcn_sched_barrier(0);
    };
#pragma unroll
    for (int k = 0; k < PRE; k++) request(ring[k], k);

    // every wave runs every pass (super-blocks outside its part are redone from clamped values and not stored)
    auto quantize_pass = [&](int p) __attribute__((always_inline)) {
        const int sbk = pass_sb(p);
#pragma unroll
        for (int t = 0; t < NT; t++) {
            float dv;
            int bs;
            const uint2 packed = q8k_quantize_row32(xv[p][t], lane, dv, bs);
            if (sbk < s1) {
                const int at = t * n_sb + sbk;
                reinterpret_cast<uint2 *>(ys)[at * 32 + ql] = packed;
                if ((ql & 3) == 3) bsum[at * 8 + (ql >> 2)] = bs;
                if (ql == 0) yds[at] = dv;
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    quantize_pass(0);
    __syncthreads();

    Q4KLane ln;
    ln.c = l;
    ln.sh = (l & 1) * 16;
    ln.upper = l >= 2;
    float acc[NT];
#pragma unroll
    for (int t = 0; t < NT; t++) acc[t] = 0.0f;
    auto compute = [&](const Regs &b, int step) __attribute__((always_inline)) {
        if (step < MAXSTEPS - 1) q4k_compute<NT, false, 1, 2, true>(b, ln, s0 + 2 * step + h, s1, ys, bsum, yds, n_sb, acc, nullptr);
        else q4k_compute<NT, false, 1, 2, false>(b, ln, s0 + 2 * step + h, s1, ys, bsum, yds, n_sb, acc, nullptr);
        __builtin_amdgcn_sched_barrier(0);
    };
#pragma unroll
    for (int j = PRE; j < NB; j++) request(ring[j], j);
#pragma unroll
    for (int i = 0; i < MAXSTEPS; i++) {
        if (i % TPW == 0 && i / TPW + 1 < PASSES) quantize_pass(i / TPW + 1);
        if (i % TPW == 0 && i > 0) __syncthreads();
        compute(ring[i % NB], i);
        if (i + NB < MAXSTEPS) request(ring[i % NB], i + NB);
    }
    if (l == LPS - 1 && h == 1) {
#pragma unroll
        for (int t = 0; t < NT; t++) part[(wave * NT + t) * 8 + r] = acc[t];
    }
    __syncthreads();
    if (tid < TPW * NT * 8) {
        const int rr = tid & 7, t = (tid >> 3) % NT, tw = (tid >> 3) / NT;
        const int orow = (blockIdx.x * TPW + tw) * 8 + rr - row_skip;
        if (orow >= 0 && orow < rows) {
            float v = part[((tw * KS) * NT + t) * 8 + rr];
#pragma unroll
            for (int k = 1; k < KS; k++) v = v + part[((tw * KS + k) * NT + t) * 8 + rr];
            if (NT == 1 && residual) v = v + residual[orow];
            out[static_cast<int64_t>(t) * rows + orow] = v;
        }
    }
}

constexpr int kComputeUnits = 256;  // MI355X

// Steps per part of the form for uneven parts (gemv_q4k_cu_kcut_any_kernel), 0 where the whole-step forms or none
// serve: rows the cut leaves no whole number of two-super-block steps, or longer parts than the whole-step forms take
// (4096 x 11008: 43 super-blocks four ways, 8.20 -> 6.29 us; 5120 x 5120: 20 four ways, 7.2 -> 4.69; 5120 x 13824: 54,
// 11.6 -> 8.76; 3584 x 18944: 74, 10.76 -> 8.64; 4096 x 10240 7.70 -> 5.89).  CAMELID_HIP_Q4K_KCUT_ANY=0 leaves them
// to the four-wave launches.
static int q4k_cu_kcut_any_steps(const Q4KArgs &ka, int ksplit) {
    if (!env_int("CAMELID_HIP_Q4K_KCUT_ANY", 1)) return 0;
    if (ksplit == 4 && ka.n_sb == 56)  // rows of 14336 values: the form of its own while that is one workgroup per compute unit
        return (ka.rows + ka.row_skip + 15) / 16 > kComputeUnits && env_int("CAMELID_HIP_Q4K_KCUT_ANY", 1) != 2 ? 7 : 0;
    const int longest = (ka.n_sb + ksplit - 1) / ksplit, steps = (longest + 1) / 2;
    const bool whole_steps = ka.n_sb % (2 * ksplit) == 0;
    if (ksplit == 4) return (whole_steps ? steps > 4 && steps <= 10 : steps >= 3 && steps <= 10) ? steps : 0;
    if (ksplit == 2) return (whole_steps ? steps == 7 : steps >= 3 && steps <= 7) ? steps : 0;  // (28 steps, 8192 x 28672: 90-124 us against 26.6, the unrolled walk spills)
    if (ksplit == 8) return (whole_steps ? steps > 4 && steps <= 6 : steps >= 3 && steps <= 6) ? steps : 0;
    return 0;
}

// The K-cut form serves rows of 14336 values cut four ways (seven steps per part, the staged quantizer) and the
// shorter rows the policy cuts: four ways into parts of 2, 3 or 4 steps (rows of 4096, 6144, 8192 values on up to 6128
// rows), two ways into parts of 3, 4, 5, 6 or 8 steps (3072, 4096, 5120, 6144, 8192 values on up to 12272 rows), and
// what q4k_cu_kcut_any_steps lists; twelve (then sixteen) waves per workgroup where eight would need more than one
// workgroup per compute unit -- twelve always suffice below 12288 rows, and beat sixteen wherever both were measured
// (9216 x 5120: 8.13 / 5.97 / 6.75 us with 8 / 12 / 16 waves against 7.38 for the four-wave launch; 11008 x 4096:
// 6.64 / 5.75 / 6.13 against 6.54; 5120 x 8192: 7.29 / 5.83 / 6.17 against 8.02).  Returns the waves per workgroup,
// 0 when the form does not serve.  CAMELID_HIP_Q4K_KCUT_SHORT=0 leaves all but the 14336-value rows to the four-wave launch.
static int q4k_cu_kcut_waves(const Q4KArgs &ka, int ksplit) {
    if (ka.sb_stride >= (int64_t(1) << 31) || env_int("CAMELID_HIP_Q4K_CU", 1) == 0 || env_int("CAMELID_HIP_Q4K_CLAMPED_LOADS", 0) ||
        env_int("CAMELID_HIP_Q4K_RING", 1) == 0)
        return 0;
    if (ksplit == 4 && ka.n_sb == 56) return 8;
    if ((ksplit != 2 && ksplit != 4 && ksplit != 8) || !env_int("CAMELID_HIP_Q4K_KCUT_SHORT", 1)) return 0;
    // fewer than 96 eight-wave workgroups leave too many compute units idle (2048 x 2048, 64 of them: 2.95 us against 2.88)
    if (((ka.rows + ka.row_skip + 15) / 16 * 2 + 8 / ksplit - 1) / (8 / ksplit) < 96) return 0;
    if (q4k_cu_kcut_any_steps(ka, ksplit)) return 8;
    if (ka.n_sb % (2 * ksplit) != 0) return 0;
    const int nsteps = ka.n_sb / (2 * ksplit);
    if (ksplit == 2 ? (nsteps < 2 || nsteps == 7 || nsteps > 8) : (nsteps < 2 || nsteps > 4)) return 0;
    const int only = env_int("CAMELID_HIP_Q4K_KCUT_WAVES", 0);
    if (only == 8 || only == 16 || (only == 12 && ksplit != 8)) return only;  // whole half tiles per workgroup: eight parts take 8 or 16 waves
    const int half_tiles = (ka.rows + ka.row_skip + 15) / 16 * 2;
    int waves = 8;
    while (waves < 16 && (half_tiles + waves / ksplit - 1) / (waves / ksplit) > kComputeUnits) waves += ksplit == 8 ? 8 : 4;
    return waves;
}
static bool q4k_cu_kcut_serves(const Q4KArgs &ka, int ksplit) { return q4k_cu_kcut_waves(ka, ksplit) != 0; }

static int launch_q4k_cu_kcut(const Q4KArgs &ka, hipStream_t st, int ablate = 0) {
    if (!(ablate & 1) && !ka.x) return fail(CML_ERR_INVALID, "null activation");
    const int tiles16 = (ka.rows + ka.row_skip + 15) / 16;
    const Q4KCuArgs ca{ka.w, ka.x, ka.out, ka.residual, static_cast<uint32_t>(ka.sb_stride), ka.rows, ka.row_skip, tiles16};
    if (const int any_steps = ablate ? 0 : q4k_cu_kcut_any_steps(ka, ka.ksplit)) {
        // eight waves, or twelve / sixteen where eight would need more than one workgroup per compute unit
        const int ks = ka.ksplit;
        int waves = env_int("CAMELID_HIP_Q4K_KCUT_WAVES", 0);
        if (waves != 8 && waves != 12 && waves != 16) {
            waves = 8;
            while (waves < 16 && (2 * tiles16 + waves / ks - 1) / (waves / ks) > kComputeUnits) waves += ks == 8 ? 8 : 4;
        }
        if (ks == 8 && waves == 12) waves = 16;
        const int tpw = waves / ks;
        const dim3 grid(static_cast<unsigned>((2 * tiles16 + tpw - 1) / tpw)), block(64 * waves);
        const size_t lds = static_cast<size_t>(ka.n_sb) * (256 + 32) + ((static_cast<size_t>(ka.n_sb) + 3) & ~size_t(3)) * 4 + 16 * 8 * 4;
        const Q4KCuAnyArgs aa{ca, ka.n_sb};
#define CML_Q4K_KCUT_ANY(KS_, NS_)                                                                                        \
    case KS_ * 100 + NS_:                                                                                                 \
        if (waves == 8) hipLaunchKernelGGL((gemv_q4k_cu_kcut_any_kernel<KS_, NS_, 8>), grid, block, lds, st, aa);         \
        else if (waves == 12) hipLaunchKernelGGL((gemv_q4k_cu_kcut_any_kernel<KS_, NS_, 12>), grid, block, lds, st, aa);  \
        else hipLaunchKernelGGL((gemv_q4k_cu_kcut_any_kernel<KS_, NS_, 16>), grid, block, lds, st, aa);                   \
        break;
        switch (ks * 100 + any_steps) {
            CML_Q4K_KCUT_ANY(4, 3)
            CML_Q4K_KCUT_ANY(4, 4)
            CML_Q4K_KCUT_ANY(4, 5)
            CML_Q4K_KCUT_ANY(4, 6)
            CML_Q4K_KCUT_ANY(4, 7)
            CML_Q4K_KCUT_ANY(4, 8)
            CML_Q4K_KCUT_ANY(4, 9)
            CML_Q4K_KCUT_ANY(4, 10)
            CML_Q4K_KCUT_ANY(2, 3)
            CML_Q4K_KCUT_ANY(2, 4)
            CML_Q4K_KCUT_ANY(2, 5)
            CML_Q4K_KCUT_ANY(2, 6)
            CML_Q4K_KCUT_ANY(2, 7)
#define CML_Q4K_KCUT_ANY8(NS_)                                                                                      \
    case 8 * 100 + NS_:                                                                                             \
        if (waves == 8) hipLaunchKernelGGL((gemv_q4k_cu_kcut_any_kernel<8, NS_, 8>), grid, block, lds, st, aa);     \
        else hipLaunchKernelGGL((gemv_q4k_cu_kcut_any_kernel<8, NS_, 16>), grid, block, lds, st, aa);               \
        break;
            CML_Q4K_KCUT_ANY8(3)
            CML_Q4K_KCUT_ANY8(4)
            CML_Q4K_KCUT_ANY8(5)
            CML_Q4K_KCUT_ANY8(6)
#undef CML_Q4K_KCUT_ANY8
            default: return fail(CML_ERR_UNSUPPORTED, "no K-cut form for %d super-blocks cut %d ways", ka.n_sb, ks);
        }
#undef CML_Q4K_KCUT_ANY
        CML_COUNT_LAUNCH("q4k.dot.wg8.kcut.fused.uneven");
        return CML_OK;
    }
    if (ka.n_sb != 56) {
        if (ablate) return fail(CML_ERR_UNSUPPORTED, "the K-cut ablations exist for rows of 14336 values");
        const int ks = ka.ksplit, waves = q4k_cu_kcut_waves(ka, ks), tpw = waves / ks;  // half tiles per workgroup
        const dim3 grid(static_cast<unsigned>((2 * tiles16 + tpw - 1) / tpw)), block(64 * waves);
#define CML_Q4K_KCUT(KS_, NS_)                                                                              \
    case KS_ * 100 + NS_:                                                                                   \
        if (waves == 8) hipLaunchKernelGGL((gemv_q4k_cu_kcut_kernel<KS_, NS_>), grid, block, 0, st, ca);    \
        else if (waves == 12) hipLaunchKernelGGL((gemv_q4k_cu_kcut_kernel<KS_, NS_, 0, false, 12>), grid, block, 0, st, ca); \
        else hipLaunchKernelGGL((gemv_q4k_cu_kcut_kernel<KS_, NS_, 0, false, 16>), grid, block, 0, st, ca); \
        break;
        switch (ks * 100 + ka.n_sb / (2 * ks)) {
            CML_Q4K_KCUT(4, 2)
            CML_Q4K_KCUT(4, 3)
            CML_Q4K_KCUT(4, 4)
            CML_Q4K_KCUT(2, 2)
            CML_Q4K_KCUT(2, 3)
            CML_Q4K_KCUT(2, 4)
            CML_Q4K_KCUT(2, 5)
            CML_Q4K_KCUT(2, 6)
            CML_Q4K_KCUT(2, 8)
#define CML_Q4K_KCUT8(NS_)                                                                                \
    case 8 * 100 + NS_:                                                                                   \
        if (waves == 8) hipLaunchKernelGGL((gemv_q4k_cu_kcut_kernel<8, NS_>), grid, block, 0, st, ca);    \
        else hipLaunchKernelGGL((gemv_q4k_cu_kcut_kernel<8, NS_, 0, false, 16>), grid, block, 0, st, ca); \
        break;
            CML_Q4K_KCUT8(2)
            CML_Q4K_KCUT8(3)
            CML_Q4K_KCUT8(4)
#undef CML_Q4K_KCUT8
            default: return fail(CML_ERR_UNSUPPORTED, "no K-cut form for %d super-blocks cut %d ways", ka.n_sb, ks);
        }
#undef CML_Q4K_KCUT
        CML_COUNT_LAUNCH("q4k.dot.wg8.kcut.fused.short");
        return CML_OK;
    }
    const dim3 grid(static_cast<unsigned>((2 * tiles16 + 1) / 2)), block(512);  // two half tiles per workgroup
    switch (ablate) {
        case 0:
            // CAMELID_HIP_Q4K_KCUT_STAGED=0: the whole row quantized before the walk (7.63 us against 7.19 at 4096 x 14336)
            if (env_int("CAMELID_HIP_Q4K_KCUT_STAGED", 1)) {
                hipLaunchKernelGGL((gemv_q4k_cu_kcut_kernel<4, 7, 0, true>), grid, block, 0, st, ca);
                CML_COUNT_LAUNCH("q4k.dot.wg8.kcut.fused");
            } else {
                hipLaunchKernelGGL((gemv_q4k_cu_kcut_kernel<4, 7>), grid, block, 0, st, ca);
                CML_COUNT_LAUNCH("q4k.dot.wg8.kcut.fused.whole_row");
            }
            return CML_OK;
        case 1: hipLaunchKernelGGL((gemv_q4k_cu_kcut_kernel<4, 7, 1>), grid, block, 0, st, ca); break;
        case 4: hipLaunchKernelGGL((gemv_q4k_cu_kcut_kernel<4, 7, 4>), grid, block, 0, st, ca); break;
        case 7: hipLaunchKernelGGL((gemv_q4k_cu_kcut_kernel<4, 7, 7>), grid, block, 0, st, ca); break;
        default: return fail(CML_ERR_INVALID, "ablation mask must be 1, 4 or 7");
    }
    CML_COUNT_LAUNCH("q4k.calibrate.wg8.kcut");
    return CML_OK;
}

// Two to four tokens under a K cut: the general K-cut form replays each step's unpacked weight against the tokens
// (one launch, every cell the one-token bits).  Steps per part, 0 where it does not serve (the row lengths of the
// instantiations below; the tokens' staging must fit LDS; not below 96 workgroups).  Before: two tokens ran on
// 16-row waves that quantize both rows in every four-wave workgroup (or, beyond 8192 values, after a quantizing
// launch), three on the matrix cores -- 4096 x 14336: 10.7 / 15.2 us for two / three tokens, 4096 x 4096 5.1 / 7.7.
// CAMELID_HIP_Q4K_KCUT_TOKENS=0 keeps those.
static int q4k_cu_kcut_tokens_steps(const Q4KArgs &ka, int ksplit, int n_tokens) {
    if (n_tokens < 2 || n_tokens > 4 || !env_int("CAMELID_HIP_Q4K_KCUT_TOKENS", 1) || !env_int("CAMELID_HIP_Q4K_KCUT_SHORT", 1)) return 0;
    if (ka.sb_stride >= (int64_t(1) << 31) || env_int("CAMELID_HIP_Q4K_CU", 1) == 0 || env_int("CAMELID_HIP_Q4K_CLAMPED_LOADS", 0) ||
        env_int("CAMELID_HIP_Q4K_RING", 1) == 0)
        return 0;
    if (ksplit != 2 && ksplit != 4 && ksplit != 8) return 0;
    if (((ka.rows + ka.row_skip + 15) / 16 * 2 + 8 / ksplit - 1) / (8 / ksplit) < 96) return 0;
    const size_t lds = static_cast<size_t>(n_tokens) * ka.n_sb * (256 + 32) + ((static_cast<size_t>(n_tokens) * ka.n_sb + 3) & ~size_t(3)) * 4 + 16 * 4 * 8 * 4;
    if (lds > 64 * 1024) return 0;
    const int steps = ((ka.n_sb + ksplit - 1) / ksplit + 1) / 2;
    const bool served = ksplit == 4 ? (steps == 2 || steps == 3 || steps == 4 || steps == 6 || steps == 7 || steps == 10)
                      : ksplit == 2 ? (steps == 3 || steps == 4 || steps == 5 || steps == 7)
                                    : (steps == 2 || steps == 3 || steps == 4);
    // four tokens: parts of up to four steps (4096 x 4096 6.15 us against 7.76 on the matrix cores, 11008 x 4096 9.77 against 13.1,
    // 2048 x 8192 8.5 against 19.4; 4096 x 11008, six steps, 14.3 against 12.9)
    if (n_tokens == 4 && steps > 4) return 0;
    return served ? steps : 0;
}

static int launch_q4k_cu_kcut_tokens(const Q4KArgs &ka, int n_tokens, hipStream_t st) {
    if (!ka.x) return fail(CML_ERR_INVALID, "null activation");
    const int ks = ka.ksplit, steps = q4k_cu_kcut_tokens_steps(ka, ks, n_tokens);
    const int tiles16 = (ka.rows + ka.row_skip + 15) / 16;
    int waves = 8;
    if ((2 * tiles16 + 8 / ks - 1) / (8 / ks) > kComputeUnits) waves = ks == 8 ? 16 : 12;
    const int only = env_int("CAMELID_HIP_Q4K_KCUT_WAVES", 0);
    if (only == 8 || (only == 12 && ks != 8) || (only == 16 && ks == 8)) waves = only;
    const int tpw = waves / ks;
    const dim3 grid(static_cast<unsigned>((2 * tiles16 + tpw - 1) / tpw)), block(64 * waves);
    const size_t lds = static_cast<size_t>(n_tokens) * ka.n_sb * (256 + 32) + ((static_cast<size_t>(n_tokens) * ka.n_sb + 3) & ~size_t(3)) * 4 +
                       static_cast<size_t>(waves) * n_tokens * 8 * 4;
    const Q4KCuAnyArgs aa{Q4KCuArgs{ka.w, ka.x, ka.out, nullptr, static_cast<uint32_t>(ka.sb_stride), ka.rows, ka.row_skip, tiles16}, ka.n_sb};
#define CML_Q4K_KCUT_TOK(KS_, NS_, WIDE_)                                                                                                  \
    case KS_ * 100 + NS_:                                                                                                                  \
        if (n_tokens == 2) {                                                                                                               \
            if (waves == 8) hipLaunchKernelGGL((gemv_q4k_cu_kcut_any_kernel<KS_, NS_, 8, 2>), grid, block, lds, st, aa);                   \
            else hipLaunchKernelGGL((gemv_q4k_cu_kcut_any_kernel<KS_, NS_, WIDE_, 2>), grid, block, lds, st, aa);                          \
        } else if (n_tokens == 4) {                                                                                                        \
            if (waves == 8) hipLaunchKernelGGL((gemv_q4k_cu_kcut_any_kernel<KS_, NS_, 8, 4>), grid, block, lds, st, aa);                   \
            else hipLaunchKernelGGL((gemv_q4k_cu_kcut_any_kernel<KS_, NS_, WIDE_, 4>), grid, block, lds, st, aa);                          \
        } else {                                                                                                                           \
            if (waves == 8) hipLaunchKernelGGL((gemv_q4k_cu_kcut_any_kernel<KS_, NS_, 8, 3>), grid, block, lds, st, aa);                   \
            else hipLaunchKernelGGL((gemv_q4k_cu_kcut_any_kernel<KS_, NS_, WIDE_, 3>), grid, block, lds, st, aa);                          \
        }                                                                                                                                  \
        break;
    switch (ks * 100 + steps) {
        CML_Q4K_KCUT_TOK(4, 2, 12)
        CML_Q4K_KCUT_TOK(4, 3, 12)
        CML_Q4K_KCUT_TOK(4, 4, 12)
        CML_Q4K_KCUT_TOK(4, 6, 12)
        CML_Q4K_KCUT_TOK(4, 7, 12)
        CML_Q4K_KCUT_TOK(4, 10, 12)
        CML_Q4K_KCUT_TOK(2, 3, 12)
        CML_Q4K_KCUT_TOK(2, 4, 12)
        CML_Q4K_KCUT_TOK(2, 5, 12)
        CML_Q4K_KCUT_TOK(2, 7, 12)
        CML_Q4K_KCUT_TOK(8, 2, 16)
        CML_Q4K_KCUT_TOK(8, 3, 16)
        CML_Q4K_KCUT_TOK(8, 4, 16)
        default: return fail(CML_ERR_UNSUPPORTED, "no K-cut form for %d tokens on %d super-blocks cut %d ways", n_tokens, ka.n_sb, ks);
    }
#undef CML_Q4K_KCUT_TOK
    CML_COUNT_LAUNCH("q4k.dot.wg8.kcut.fused.tokens");
    return CML_OK;
}

// The short K-cut forms against two to four weights of one row length and one K cut in ONE launch (the q, k and v
// projections of an attention block): every output is its own call's bits.  -1 = not a set this launch serves.
// Against the four-wave multi launch: 4096 + 1024 + 1024 rows of 4096 values 4.96 us against 5.38, 6144 + 1024 + 1024
// of 6144 9.22 against 10.0, three times 4096 x 4096 6.83 against 6.84.  A pair of equal weights through it gains
// nothing (11008 x 4096 9.82 against 9.91, 4096 x 4096 5.38 against 5.25), so pairs stay on the four-wave pair launch.
// CAMELID_HIP_Q4K_KCUT_MULTI=0 keeps the four-wave multi launch.
static int launch_q4k_cu_kcut_multi(const cml_weight *const *ws, int n, const float *x, float *const *outs, int ksplit, hipStream_t st) {
    if (n < 2 || n > 4 || ws[0]->nb == 56) return -1;
    int64_t tiles16_all = 0;
    for (int j = 0; j < n; j++) tiles16_all += (ws[j]->rows + ws[j]->row_skip + 15) / 16;
    if (tiles16_all * 16 > INT32_MAX) return -1;
    Q4KArgs probe{};
    probe.n_sb = static_cast<int>(ws[0]->nb);
    probe.rows = static_cast<int>(tiles16_all * 16);
    for (int j = 0; j < n; j++) probe.sb_stride = std::max<int64_t>(probe.sb_stride, ws[j]->planes.row_stride[0]);
    if (!q4k_cu_kcut_waves(probe, ksplit) || q4k_cu_kcut_any_steps(probe, ksplit)) return -1;  // the whole-step forms only
    if (!x) return fail(CML_ERR_INVALID, "null activation");
    constexpr int waves = 8;         // twelve- and sixteen-wave workgroups are slower here at every set measured (q | k | v: 5.70 and 5.27 us against 4.96)
    const int tpw = waves / ksplit;  // half tiles per workgroup
    Q4KCuMultiArgs ma{};
    ma.x = x;
    int wg = 0;
    for (int j = 0; j < 4; j++) {
        const cml_weight *w = ws[std::min(j, n - 1)];
        ma.wm[j] = static_cast<const uint8_t *>(w->planes.p[0]);
        ma.outm[j] = outs[std::min(j, n - 1)];
        ma.stridem[j] = static_cast<uint32_t>(w->planes.row_stride[0]);
        ma.rowsm[j] = static_cast<int>(w->rows);
        ma.skipm[j] = w->row_skip;
        ma.tiles16m[j] = static_cast<int>((w->rows + w->row_skip + 15) / 16);
        if (j < n) wg += (2 * ma.tiles16m[j] + tpw - 1) / tpw;
        ma.wg_end[j] = j < n ? wg : INT32_MAX;
    }
    const dim3 grid(static_cast<unsigned>(wg)), block(64 * waves);
#define CML_Q4K_KCUT(KS_, NS_) \
    case KS_ * 100 + NS_: hipLaunchKernelGGL((gemv_q4k_cu_kcut_kernel<KS_, NS_, 0, false, 8, true>), grid, block, 0, st, ma); break;
    switch (ksplit * 100 + probe.n_sb / (2 * ksplit)) {
        CML_Q4K_KCUT(4, 2)
        CML_Q4K_KCUT(4, 3)
        CML_Q4K_KCUT(4, 4)
        CML_Q4K_KCUT(2, 2)
        CML_Q4K_KCUT(2, 3)
        CML_Q4K_KCUT(2, 4)
        CML_Q4K_KCUT(2, 5)
        CML_Q4K_KCUT(2, 6)
        CML_Q4K_KCUT(2, 8)
        CML_Q4K_KCUT(8, 2)
        CML_Q4K_KCUT(8, 3)
        CML_Q4K_KCUT(8, 4)
        default: return -1;
    }
#undef CML_Q4K_KCUT
    CML_COUNT_LAUNCH("q4k.dot.wg8.kcut.fused.multi");
    CML_HIP_TRY(hipGetLastError());
    return CML_OK;
}

// Whether the launch above serves this call: rows of 6 to 16 super-blocks (an even count: 1536 to 4096 values) or of
// 20, 24 or 32 (5120, 6144, 8192 values: two quantizer passes), no K cut (the shape policy gives that from 12288 rows
// on, i.e. at least 192 eight-wave workgroups), a stride the 32-bit lane offsets can hold.  One and two tokens only
// while the launch is at most one workgroup per compute unit (with more than 256 workgroups some units carry two:
// 18944 x 3584 with eight waves 9.33 us against 8.77 for the four-wave workgroups), which wider workgroups keep up to
// 24576 rows.  The longer rows, us per step against the four-wave / matrix-core launches that served them: 13824 x 5120
// 7.65 / 8.99 / 11.5 for one / two / three tokens against 8.62 / 10.66 / 17.2; 17920 x 5120 (ten waves) 9.45 against
// 10.74; 16384 x 6144 9.94 against 10.5; 14336 x 8192 11.27 against 12.2; 28672 x 8192, three tokens, 27.3 against 32.5.
// Seven waves per workgroup on 14336 x 4096 (256 workgroups instead of 224): 6.72 against 6.56.
// CAMELID_HIP_Q4K_CU=0 keeps the four-wave launch.
// Waves per workgroup of that launch, 0 when it does not serve the row count: the smallest of 8, 10 and 12 (three
// tokens: and 16) that keeps the launch within one workgroup per compute unit -- wider than eight for rows of 14 or 16
// super-blocks and up to three tokens; three tokens take eight waves at any row count beyond.  Measured, us per step,
// wide against what served the shape before: 18944 x 3584 (ten waves) 7.56 / 8.24 / 10.1 for one / two / three tokens
// against 8.68 / 11.07 / 13.27; 24576 x 4096 (twelve) 9.87 / 10.67 / 11.9 against 10.09 / 12.44 / 14.75; sixteen waves
// at 28672 and 32000 x 4096 lose to the 16-row waves for one and two tokens (11.7 against 11.25, 12.57 against 12.2,
// 13.6 against 13.1) and win for three (14.3 and 15.2 against 15.1 and 15.5 with eight waves, 18.2 and 18.6 before).
// CAMELID_HIP_Q4K_CU_WAVES considers that width only.
static int q4k_cu_waves(const Q4KArgs &ka, int n_tokens) {
    const int half_tiles = 2 * ((ka.rows + ka.row_skip + 15) / 16);
    const int only = env_int("CAMELID_HIP_Q4K_CU_WAVES", 0);
    for (int wv : {8, 10, 12, 16}) {
        if (only && wv != only) continue;
        if (wv > 8 && (ka.n_sb < 14 || ka.n_sb > 20 || n_tokens > 3)) break;
        if (wv == 16 && n_tokens < 3) break;
        if ((half_tiles + wv - 1) / wv <= kComputeUnits) return wv;
    }
    return n_tokens >= 3 ? 8 : 0;
}
static bool q4k_cu_serves(const Q4KArgs &ka, int ksplit, int n_tokens = 1) {
    const bool length = (ka.n_sb <= 16 && ka.n_sb >= 6 && (ka.n_sb & 1) == 0) || ka.n_sb == 20 || ka.n_sb == 24 || ka.n_sb == 32;
    return ksplit == 1 && length && q4k_cu_waves(ka, n_tokens) != 0 &&
           ka.sb_stride < (int64_t(1) << 31) && env_int("CAMELID_HIP_Q4K_CU", 1) != 0 && !env_int("CAMELID_HIP_Q4K_CLAMPED_LOADS", 0) &&
           env_int("CAMELID_HIP_Q4K_RING", 1) != 0;
}

// Most tokens the eight-wave launch replays per step (CAMELID_HIP_Q4K_CU_TOKENS, 1 to 4; four only on rows of 4096 values).
// Measured at 14336 x 4096, us per step against what served the call before: 2 tokens 7.0 (8.46, the 16-row-wave ring launch),
// 3 tokens 8.6 (9.71, the matrix-core launch with the quantizer inside), 4 tokens 10.4 (10.3: the vector work no longer hides
// behind the stream).  Default 3; 4 on rows of 3584 or 4096 values from 24576 rows on, where the matrix-core launch streams
// less well than this one (4 tokens on 128256 x 4096: 66.8 us against 75.2, 65536 x 4096 35.7 against 39.9, 32000 x 4096
// 19.3 against 20.7).
static int q4k_cu_max_tokens(int n_sb, int rows) {
    const int knob = env_int("CAMELID_HIP_Q4K_CU_TOKENS", 0);
    const int most = knob >= 1 ? knob : (rows >= 24576 ? 4 : 3);
    return std::min((n_sb == 16 || n_sb == 14) ? 4 : 3, most);
}

static int launch_q4k_cu(const Q4KArgs &ka, int ablate, hipStream_t st, int n_tokens = 1) {
    if (!(ablate & 1) && !ka.x) return fail(CML_ERR_INVALID, "null activation");  // every variant but the one without the activation reads it
    const int tiles16 = (ka.rows + ka.row_skip + 15) / 16;
    const dim3 grid(static_cast<unsigned>((2 * tiles16 + 7) / 8)), block(512);
    const Q4KCuArgs ca{ka.w, ka.x, ka.out, ka.residual, static_cast<uint32_t>(ka.sb_stride), ka.rows, ka.row_skip, tiles16};
    // rows of 2 * NSTEPS super-blocks: one instantiation per row length (1536 to 4096 values)
#define CML_Q4K_CU_STEPS(NT_)                                                                                 \
    switch (ka.n_sb) {                                                                                        \
        case 32: hipLaunchKernelGGL((gemv_q4k_cu_kernel<16, 0, NT_>), grid, block, 0, st, ca); break;         \
        case 24: hipLaunchKernelGGL((gemv_q4k_cu_kernel<12, 0, NT_>), grid, block, 0, st, ca); break;         \
        case 20: hipLaunchKernelGGL((gemv_q4k_cu_kernel<10, 0, NT_>), grid, block, 0, st, ca); break;         \
        case 16: hipLaunchKernelGGL((gemv_q4k_cu_kernel<8, 0, NT_>), grid, block, 0, st, ca); break;          \
        case 14: hipLaunchKernelGGL((gemv_q4k_cu_kernel<7, 0, NT_>), grid, block, 0, st, ca); break;          \
        case 12: hipLaunchKernelGGL((gemv_q4k_cu_kernel<6, 0, NT_>), grid, block, 0, st, ca); break;          \
        case 10: hipLaunchKernelGGL((gemv_q4k_cu_kernel<5, 0, NT_>), grid, block, 0, st, ca); break;          \
        case 8: hipLaunchKernelGGL((gemv_q4k_cu_kernel<4, 0, NT_>), grid, block, 0, st, ca); break;           \
        case 6: hipLaunchKernelGGL((gemv_q4k_cu_kernel<3, 0, NT_>), grid, block, 0, st, ca); break;           \
        default: return fail(CML_ERR_UNSUPPORTED, "the eight-wave launch takes rows of 6 to 16, 20, 24 or 32 super-blocks");  \
    }
    const int waves = ablate ? 8 : q4k_cu_waves(ka, n_tokens);
    if (waves > 8) {  // more than 256 eight-wave workgroups: wider ones, still one per compute unit
#define CML_Q4K_CU_WIDE(NS_, NT_, WV_) \
    hipLaunchKernelGGL((gemv_q4k_cu_kernel<NS_, 0, NT_, WV_>), dim3(static_cast<unsigned>((2 * tiles16 + WV_ - 1) / WV_)), dim3(WV_ * 64), 0, st, ca)
#define CML_Q4K_CU_WIDE_WAVES(NS_, NT_)                                                  \
    switch (waves) {                                                                     \
        case 10: CML_Q4K_CU_WIDE(NS_, NT_, 10); break;                                   \
        case 12: CML_Q4K_CU_WIDE(NS_, NT_, 12); break;                                   \
        default: CML_Q4K_CU_WIDE(NS_, NT_, 16); break;                                   \
    }
        if (ka.n_sb == 20 && n_tokens == 1) { CML_Q4K_CU_WIDE_WAVES(10, 1) }
        else if (ka.n_sb == 20 && n_tokens == 2) { CML_Q4K_CU_WIDE_WAVES(10, 2) }
        else if (ka.n_sb == 20) { CML_Q4K_CU_WIDE_WAVES(10, 3) }
        else if (ka.n_sb == 16 && n_tokens == 1) { CML_Q4K_CU_WIDE_WAVES(8, 1) }
        else if (ka.n_sb == 16 && n_tokens == 2) { CML_Q4K_CU_WIDE_WAVES(8, 2) }
        else if (ka.n_sb == 16) { CML_Q4K_CU_WIDE_WAVES(8, 3) }
        else if (n_tokens == 1) { CML_Q4K_CU_WIDE_WAVES(7, 1) }
        else if (n_tokens == 2) { CML_Q4K_CU_WIDE_WAVES(7, 2) }
        else { CML_Q4K_CU_WIDE_WAVES(7, 3) }
#undef CML_Q4K_CU_WIDE_WAVES
#undef CML_Q4K_CU_WIDE
        if (n_tokens > 1) CML_COUNT_LAUNCH("q4k.dot.wg8.fused.tokens.wide");
        else CML_COUNT_LAUNCH("q4k.dot.wg8.fused.wide");
        return CML_OK;
    }
    if (n_tokens > 1) {
        if (ablate) return fail(CML_ERR_INVALID, "the ablations are one-token launches");
        switch (n_tokens) {
            case 2: CML_Q4K_CU_STEPS(2); break;
            case 3: CML_Q4K_CU_STEPS(3); break;
            case 4:
                if (ka.n_sb == 16) hipLaunchKernelGGL((gemv_q4k_cu_kernel<8, 0, 4>), grid, block, 0, st, ca);
                else if (ka.n_sb == 14) hipLaunchKernelGGL((gemv_q4k_cu_kernel<7, 0, 4>), grid, block, 0, st, ca);
                else return fail(CML_ERR_INVALID, "four tokens: rows of 14 or 16 super-blocks only");
                break;
            default: return fail(CML_ERR_INVALID, "the eight-wave launch takes up to four tokens");
        }
        CML_COUNT_LAUNCH("q4k.dot.wg8.fused.tokens");
        return CML_OK;
    }
    if (ablate && ka.n_sb != 16) return fail(CML_ERR_UNSUPPORTED, "the ablations exist for rows of 4096 values");
#define CML_Q4K_CU(A_) hipLaunchKernelGGL((gemv_q4k_cu_kernel<8, A_>), grid, block, 0, st, ca)
    switch (ablate) {
        case 0: CML_Q4K_CU_STEPS(1); break;
        case 1: CML_Q4K_CU(1); break;
        case 4: CML_Q4K_CU(4); break;
        case 7: CML_Q4K_CU(7); break;
        default: return fail(CML_ERR_INVALID, "ablation mask must be 1, 4 or 7");
    }
#undef CML_Q4K_CU
#undef CML_Q4K_CU_STEPS
    if (ablate) CML_COUNT_LAUNCH("q4k.calibrate.wg8");
    else CML_COUNT_LAUNCH("q4k.dot.wg8.fused");
    return CML_OK;
}

// Launch shape.  `ksplit` depends on the weight shape only, so gemv and gemm
// give every cell the same association; 1 (the reference's own) whenever the
// row count alone yields about one wave per SIMD (1024 on this chip).
struct Q4KShape {
    int ksplit, tiles_per_wg;
};

static Q4KShape pick_shape(int64_t rows, int64_t n_sb) {
    Q4KShape s;
    const int64_t tiles = (rows + 15) / 16;
    int ks = 1;
    const int forced = env_int("CAMELID_HIP_Q4K_KSPLIT", 0);
    if ((forced == 1 || forced == 2 || forced == 4 || forced == 8) && forced <= n_sb) {
        ks = forced;
    } else if (!env_int("CAMELID_HIP_EXACT_ORDER", 0)) {
        // At most four parts: the matrix-core kernels run a cut of two or four as that many waves per row tile, but walk
        // an eight-way cut inside the lane, one wave per row tile -- 128 waves for 2048 rows (2048 x 8192, 64 tokens:
        // 38.9 us with eight parts, 13.9 with four; 16 tokens on 2560 x 10240 23.2 against 12.2).  A single token pays
        // 0.3 to 0.4 us for it on those shapes (2048 x 8192: 3.88 -> 4.21 us).  CAMELID_HIP_Q4K_MAX_KSPLIT=8 restores eight.
        const int most = env_int("CAMELID_HIP_Q4K_MAX_KSPLIT", 4) == 8 ? 8 : 4;
        while (ks < most && tiles * ks < 768 && n_sb / (ks * 2) >= 4) ks *= 2;
    }
    s.ksplit = ks;
    int tpw = env_int("CAMELID_HIP_Q4K_TILES_PER_WG", 0);
    if (tpw < 1 || tpw * ks > 8) {
        tpw = 1;
        while (tpw < 4 && tpw * 2 * ks <= 8 && tiles >= 2048 * tpw) tpw *= 2;
    }
    s.tiles_per_wg = tpw;
    return s;
}

// The K-split the matvec kernel applies to a weight of this shape (the
// matrix-core kernel reproduces the same association).
int q4k_ksplit_for(int64_t rows, int64_t n_sb) { return pick_shape(rows, n_sb).ksplit; }

// Rows per wave of a single-token launch: 8 (two groups per row) when 16-row tiles would leave at
// most one wave per SIMD of the 256 compute units -- measured on the 14336 x 4096 matvec: twice
// the waves hide each other's instruction latency as long as the bytes in flight stay the same
// (8.7 against 9.1 us cache-cold, 6.7 against 7.5 us cache-warm; 4096 x 14336: 9.2 against 9.5).
// The choice never changes a result bit.
static int q4k_rows_per_wave(int64_t tiles16, int ksplit, int64_t slots) {
    const int forced = env_int("CAMELID_HIP_Q4K_ROWS_PER_WAVE", 0);
    if (forced == 8 || forced == 16) return forced;
    const int64_t waves16 = tiles16 * ksplit * slots;
    if (waves16 <= 1024) return 8;
    // Taller matrices: 16-row waves, unless their workgroups (four waves) fall unevenly on the 256
    // compute units and the 8-row ones clearly less so -- 20000 x 4096 is 313 workgroups, 1.2 per
    // unit, so some units carry two: 11.5 us against 9.9 with 625 half-size workgroups.
    auto imbalance = [](int64_t waves) {
        const double per_cu = static_cast<double>((waves + 3) / 4) / 256.0;
        return std::ceil(per_cu) / per_cu;
    };
    return imbalance(2 * waves16) + 0.1 < imbalance(waves16) ? 8 : 16;
}

// A single f32 token on this weight runs as ONE launch although its rows are longer than the in-kernel quantizer of
// the four-wave launches takes (the caller's decision between one launch and quantize-then-matvec).
bool gemv_q4k_long_rows_fuse(const cml_weight *w, int n_tokens) {
    if (w->fmt != CML_Q4_K || w->rows <= 0) return false;
    if (n_tokens >= 2 && n_tokens <= 4) {
        Q4KArgs ka{};
        ka.n_sb = static_cast<int>(w->nb);
        ka.sb_stride = w->planes.row_stride[0];
        ka.rows = static_cast<int>(w->rows);
        ka.row_skip = w->row_skip;
        return q4k_cu_kcut_tokens_steps(ka, pick_shape(w->rows, ka.n_sb).ksplit, n_tokens) != 0 && !env_int("CAMELID_HIP_Q4K_GENERAL_ENTRY", 0);
    }
    if (n_tokens != 1) return false;
    Q4KArgs ka{};
    ka.n_sb = static_cast<int>(w->nb);
    ka.sb_stride = w->planes.row_stride[0];
    ka.rows = static_cast<int>(w->rows);
    ka.row_skip = w->row_skip;
    const int64_t tiles16 = (w->rows + w->row_skip + 15) / 16;
    const int ks = pick_shape(w->rows, ka.n_sb).ksplit;
    return q4k_cu_kcut_serves(ka, ks) && q4k_rows_per_wave(tiles16, ks, 1) == 8 && !env_int("CAMELID_HIP_Q4K_GENERAL_ENTRY", 0);
}

// Every K part a whole number of 4-super-block buffers and a stride of less than 2 GiB: the
// kernel variant whose loads need no clamping applies.
static bool q4k_whole_buffers(const Q4KArgs &ka, int ksplit) {
    if (env_int("CAMELID_HIP_Q4K_CLAMPED_LOADS", 0)) return false;
    return ka.n_sb % (4 * ksplit) == 0 && ka.sb_stride < (int64_t(1) << 31);
}

// The ring of small register buffers applies (plain calls): 8-row waves (spr = 2) walk a K part in
// steps of two super-blocks through three slots, 16-row waves (spr = 1) in steps of one through
// four; the part must hold at least one full ring of whole steps, the stride less than 2 GiB.
static bool q4k_ring(const Q4KArgs &ka, int ksplit, int spr = 2) {
    if (!env_int("CAMELID_HIP_Q4K_RING", 1) || env_int("CAMELID_HIP_Q4K_CLAMPED_LOADS", 0)) return false;
    const int slots = spr == 2 ? 3 : 4;
    return ka.n_sb % (spr * ksplit) == 0 && ka.n_sb / (spr * ksplit) >= slots && ka.sb_stride < (int64_t(1) << 31);
}

// A plain ring launch.  Part lengths that common models have get the walk unrolled (NSTEPS known
// at compile time: no loop, no per-remainder tails -- the two-token call on rows of 4096 values
// 8.87 -> 8.44 us, the single-token one 6.89 -> 6.81); every other length runs the loop.
// 8-row waves (SPR = 2, three slots) step two super-blocks at a time: rows / K parts of 3072, 3584
// and 4096 values are 6, 7 and 8 steps; 16-row waves (SPR = 1, four slots) step one: 12, 14, 16.
template <int NT, bool FUSEQ, int SPR, bool LOADONLY = false, bool PAIR = false, bool MULTI = false>
static void launch_q4k_ring(const Q4KArgs &ka, int ksplit, dim3 grid, dim3 block, size_t lds, hipStream_t st) {
    constexpr int SLOTS = SPR == 2 ? 3 : 4;
    const int steps = ka.n_sb / (SPR * ksplit);
#define CML_Q4K_RING(N_) hipLaunchKernelGGL((gemv_q4k_kernel<NT, false, FUSEQ, SPR, true, true, LOADONLY, false, SLOTS, N_, false, PAIR, MULTI>), grid, block, lds, st, ka)
    if constexpr (MULTI) {
        if (steps == 8) CML_Q4K_RING(8);
        else CML_Q4K_RING(0);
    } else if constexpr (LOADONLY && SPR == 2) {
        if (steps == 8) CML_Q4K_RING(8);
        else CML_Q4K_RING(0);
    } else if constexpr (LOADONLY) {
        CML_Q4K_RING(0);
    } else if constexpr (SPR == 2) {
        switch (steps) {
            case 6: CML_Q4K_RING(6); break;
            case 7: CML_Q4K_RING(7); break;
            case 8: CML_Q4K_RING(8); break;
            default: CML_Q4K_RING(0); break;
        }
    } else if constexpr (NT == 2 && FUSEQ) {
        switch (steps) {
            case 12: CML_Q4K_RING(12); break;
            case 14: CML_Q4K_RING(14); break;
            case 16: CML_Q4K_RING(16); break;
            default: CML_Q4K_RING(0); break;
        }
    } else {
        if (steps == 16) CML_Q4K_RING(16);
        else CML_Q4K_RING(0);
    }
#undef CML_Q4K_RING
    if constexpr (LOADONLY) CML_COUNT_LAUNCH("q4k.calibrate.ring");
    else if constexpr (MULTI) CML_COUNT_LAUNCH("q4k.dot.ring.fused.multi");
    else if constexpr (PAIR) CML_COUNT_LAUNCH("q4k.dot.ring.fused.pair");
    else if constexpr (FUSEQ) CML_COUNT_LAUNCH("q4k.dot.ring.fused");
    else CML_COUNT_LAUNCH("q4k.dot.ring");
}

template <int NT>
static int launch_q4k_nt(Q4KArgs ka, const Q4KShape &shape, int n_groups, bool ints, hipStream_t st) {
    const int waves = shape.ksplit * shape.tiles_per_wg;
    const int64_t tiles16 = (ka.rows + ka.row_skip + 15) / 16;
    const bool half_tiles = NT == 1 && !ints && q4k_rows_per_wave(tiles16, shape.ksplit, n_groups) == 8;
    const int64_t tiles = half_tiles ? 2 * tiles16 : tiles16;
    const unsigned gx = static_cast<unsigned>((tiles + shape.tiles_per_wg - 1) / shape.tiles_per_wg);
    const size_t lds = static_cast<size_t>(NT) * ka.n_sb * (256 + 32) + ((static_cast<size_t>(NT) * ka.n_sb + 3) & ~size_t(3)) * 4 +
                       static_cast<size_t>(waves) * NT * 16 * 4;
    if (lds > 64 * 1024) return fail(CML_ERR_UNSUPPORTED, "Q4_K activation of %d super-blocks x %d tokens exceeds the LDS staging limit", ka.n_sb, NT);
    ka.ksplit = shape.ksplit;
    ka.ksplit_log2 = shape.ksplit >= 8 ? 3 : (shape.ksplit >= 4 ? 2 : (shape.ksplit >= 2 ? 1 : 0));
    ka.tiles_per_wg = shape.tiles_per_wg;
    const bool plain = !ka.group_offsets && !ka.group_ids && !env_int("CAMELID_HIP_Q4K_GENERAL_ENTRY", 0);
    const dim3 grid(gx, n_groups), block(64 * waves);
    const bool grouped_call = ka.group_offsets || ka.group_ids;
    if (ints && NT == 1) {
        hipLaunchKernelGGL((gemv_q4k_kernel<1, true>), grid, block, lds, st, ka);
        CML_COUNT_LAUNCH("q4k.dot.ints");
    } else if (NT <= 2) {
        // one or two tokens: 8-row waves, unclamped loads and the short entry where they apply
        constexpr int NTS = NT <= 2 ? NT : 1;
        const bool whole = q4k_whole_buffers(ka, shape.ksplit);
#define CML_Q4K_LAUNCH(SPR_, WHOLE_, PLAIN_) hipLaunchKernelGGL((gemv_q4k_kernel<NTS, false, false, SPR_, WHOLE_, PLAIN_>), grid, block, lds, st, ka)
        if (half_tiles && plain && q4k_ring(ka, shape.ksplit)) {
            launch_q4k_ring<1, false, 2>(ka, shape.ksplit, grid, block, lds, st);
        } else if (!half_tiles && plain && q4k_ring(ka, shape.ksplit, 1)) {
            launch_q4k_ring<NTS, false, 1>(ka, shape.ksplit, grid, block, lds, st);
        } else if (half_tiles) {
            if (whole) { if (plain) CML_Q4K_LAUNCH(2, true, true); else CML_Q4K_LAUNCH(2, true, false); }
            else { if (plain) CML_Q4K_LAUNCH(2, false, true); else CML_Q4K_LAUNCH(2, false, false); }
            if (grouped_call) CML_COUNT_LAUNCH("q4k.dot.buffers.grouped"); else CML_COUNT_LAUNCH("q4k.dot.buffers");
        } else {
            if (whole) { if (plain) CML_Q4K_LAUNCH(1, true, true); else CML_Q4K_LAUNCH(1, true, false); }
            else { if (plain) CML_Q4K_LAUNCH(1, false, true); else CML_Q4K_LAUNCH(1, false, false); }
            if (grouped_call) CML_COUNT_LAUNCH("q4k.dot.buffers.grouped"); else CML_COUNT_LAUNCH("q4k.dot.buffers");
        }
#undef CML_Q4K_LAUNCH
    } else {
        hipLaunchKernelGGL((gemv_q4k_kernel<NT, false>), grid, block, lds, st, ka);
        if (grouped_call) CML_COUNT_LAUNCH("q4k.dot.buffers.grouped"); else CML_COUNT_LAUNCH("q4k.dot.buffers");
    }
    CML_HIP_TRY(hipGetLastError());
    return CML_OK;
}

// Largest token count per pass (8, 4, 2 or 1) whose LDS staging fits 64 KB.
static int cap_nt(int64_t want, int n_sb, int waves) {
    int nt = want >= 8 ? 8 : (want >= 4 ? 4 : (want >= 2 ? 2 : 1));
    while (nt > 1 && static_cast<size_t>(nt) * n_sb * (256 + 32) + ((static_cast<size_t>(nt) * n_sb + 3) & ~size_t(3)) * 4 +
                             static_cast<size_t>(waves) * nt * 16 * 4 > 64 * 1024)
        nt >>= 1;
    return nt;
}

static int launch_q4k_pick_nt(const Q4KArgs &ka, const Q4KShape &shape, int n_groups, int nt, bool ints, hipStream_t st) {
    switch (nt) {
        case 8: return launch_q4k_nt<8>(ka, shape, n_groups, false, st);
        case 4: return launch_q4k_nt<4>(ka, shape, n_groups, false, st);
        case 2: return launch_q4k_nt<2>(ka, shape, n_groups, false, st);
        default: return launch_q4k_nt<1>(ka, shape, n_groups, ints, st);
    }
}

// Single token per group, f32 activation in: quantize + matvec in one launch.  The K-split is
// the matvec's own (same association); waves of a workgroup share the quantizing, so a workgroup
// holds 4 waves where the split alone gives fewer.  Plain call: `a.w` against activation row 0.
// Grouped call (group_offsets set): every group dots its assignments' activation rows
// (group_rows) one at a time.  `w2`/`out2` non-null: a second weight of the same shape in the
// same launch (grid.z = 2).
// ablate: 0 = the real launch; 7 = its weight requests alone (x may be null); 1 / 4 = without the activation / without the
// store (the eight-wave launch only) -- the calibration entries' timing experiments.
static int launch_q4k_f32(const MatArgs &a, const cml_weight *w2, float *out2, const float *x, hipStream_t st, int ablate = 0) {
    const bool loads_only = ablate != 0;
    const cml_weight *w = a.w;
    const bool grouped = a.group_offsets != nullptr || a.group_ids != nullptr;
    if (w->rows == 0) return CML_OK;
    Q4KArgs ka{};
    ka.w = w->planes.p[0];
    ka.sb_stride = w->planes.row_stride[0];
    ka.rows = static_cast<int>(grouped ? a.band_rows : w->rows);
    if (grouped && ((ka.rows % 16) != 0 || w->row_skip != 0))
        return fail(CML_ERR_UNSUPPORTED, "Q4_K expert bands must be whole 16-row tiles (%d rows, first tile offset %d)", ka.rows, w->row_skip);
    ka.row_skip = grouped ? 0 : w->row_skip;
    ka.n_sb = static_cast<int>(w->nb);
    ka.x = x;
    ka.out = a.out;
    ka.group_offsets = a.group_offsets;
    ka.group_rows = a.group_rows;
    ka.group_ids = a.group_ids;
    ka.n_groups = a.n_groups;
    ka.shared_act = grouped && !a.group_offsets;  // direct call: the one f32 token
    ka.route_logits = a.route_logits;
    ka.route_k = a.route_k;
    ka.route_idx = a.route_idx;
    ka.route_w = a.route_w;
    if (w2) {
        if (w2->fmt != w->fmt || w2->rows != w->rows || w2->nb != w->nb || w2->row_skip != w->row_skip ||
            w2->planes.row_stride[0] != w->planes.row_stride[0])
            return fail(CML_ERR_SHAPE, "the two weights of a pair launch differ in shape");
        ka.w2 = w2->planes.p[0];
        ka.out2 = out2;
    }
    Q4KShape shape = pick_shape(ka.rows, ka.n_sb);
    const int64_t tiles16 = (ka.rows + ka.row_skip + 15) / 16;
    const int64_t slots = static_cast<int64_t>(grouped ? (a.group_ids ? a.max_active : a.n_groups) : 1) * (w2 ? 2 : 1);
    const bool two = !grouped && !w2 && a.n_tokens == 2;  // plain call with two contiguous f32 rows
    const bool half_tiles = !two && q4k_rows_per_wave(tiles16, shape.ksplit, slots) == 8;
    const int64_t tiles = half_tiles ? 2 * tiles16 : tiles16;
    int tpw = env_int("CAMELID_HIP_Q4K_FUSED_TILES_PER_WG", 0);
    // 4 waves share the quantizing.  Measured with 8-row tiles at 14336 x 4096 (1792 tiles): 2 waves
    // 9.6 us, 4 waves 8.7, 8 waves 9.1; 7 waves -- one workgroup for each of the 256 compute units
    // on paper -- 9.1, and 5 or 6 waves 12.7 / 13.2: workgroups do not land one per unit.
    if (tpw < 1 || tpw * shape.ksplit > 8) {
        tpw = std::max(1, 4 / shape.ksplit);
        // The decode launch of an expert layer (routed slots x gate and up in one grid): seven-wave workgroups where
        // they divide the half tiles -- 14336 rows are 256 of them per matrix, and the 1024 workgroups of the
        // Mixtral-shaped layer are four per compute unit, all resident (38.9 -> 38.1 us per token).
        if (ka.shared_act && a.group_ids && half_tiles && shape.ksplit == 1 && tiles % 7 == 0 && env_int("CAMELID_HIP_Q4K_DIRECT_SEVEN_WAVES", 1)) tpw = 7;
    }
    shape.tiles_per_wg = tpw;
    const int waves = shape.ksplit * shape.tiles_per_wg;
    const unsigned gx = static_cast<unsigned>((tiles + shape.tiles_per_wg - 1) / shape.tiles_per_wg);
    const size_t nt = two ? 2 : 1;
    const size_t lds = nt * ka.n_sb * (256 + 32) + ((nt * ka.n_sb + 3) & ~size_t(3)) * 4 + static_cast<size_t>(waves) * nt * 16 * 4;
    if (lds > 64 * 1024) return fail(CML_ERR_UNSUPPORTED, "Q4_K activation of %d super-blocks exceeds the LDS staging limit", ka.n_sb);
    ka.ksplit = shape.ksplit;
    ka.ksplit_log2 = shape.ksplit >= 8 ? 3 : (shape.ksplit >= 4 ? 2 : (shape.ksplit >= 2 ? 1 : 0));
    ka.tiles_per_wg = shape.tiles_per_wg;
    const dim3 grid(gx, grouped ? (a.group_ids ? a.max_active : a.n_groups) : 1, w2 ? 2 : 1);
    {
        const bool whole = q4k_whole_buffers(ka, shape.ksplit);
        const bool ring = q4k_ring(ka, shape.ksplit);
        const bool plain = !grouped && !w2 && !env_int("CAMELID_HIP_Q4K_GENERAL_ENTRY", 0);
        const dim3 block(64 * waves);
#define CML_Q4K_LAUNCH(SPR_, WHOLE_, PLAIN_) hipLaunchKernelGGL((gemv_q4k_kernel<1, false, true, SPR_, WHOLE_, PLAIN_>), grid, block, lds, st, ka)
        if (loads_only && half_tiles && ring && plain && q4k_cu_serves(ka, shape.ksplit) && ka.n_sb == 16) {
            if (int rc = launch_q4k_cu(ka, ablate, st)) return rc;
        } else if (loads_only && half_tiles && plain && q4k_cu_kcut_serves(ka, shape.ksplit) && ka.n_sb == 56 && !q4k_cu_kcut_any_steps(ka, shape.ksplit)) {
            if (int rc = launch_q4k_cu_kcut(ka, st, ablate)) return rc;
        } else if (loads_only && ablate != 7) {
            return fail(CML_ERR_UNSUPPORTED, "this ablation exists for the eight-wave single-token launch (rows of 4096 values, no K cut)");
        } else if (loads_only) {
            // calibration: the plain single-token launch with its loads and nothing else
#define CML_Q4K_LOADS(SPR_, WHOLE_) hipLaunchKernelGGL((gemv_q4k_kernel<1, false, true, SPR_, WHOLE_, true, true>), grid, block, lds, st, ka)
            if (half_tiles && ring) launch_q4k_ring<1, true, 2, true>(ka, shape.ksplit, grid, block, lds, st);
            else if (!half_tiles && q4k_ring(ka, shape.ksplit, 1)) launch_q4k_ring<1, true, 1, true>(ka, shape.ksplit, grid, block, lds, st);
            else if (half_tiles) { if (whole) CML_Q4K_LOADS(2, true); else CML_Q4K_LOADS(2, false); CML_COUNT_LAUNCH("q4k.calibrate.buffers"); }
            else { if (whole) CML_Q4K_LOADS(1, true); else CML_Q4K_LOADS(1, false); CML_COUNT_LAUNCH("q4k.calibrate.buffers"); }
#undef CML_Q4K_LOADS
        } else if (plain && a.n_tokens >= 2 && a.n_tokens <= q4k_cu_max_tokens(ka.n_sb, ka.rows) &&
                   (a.n_tokens >= 3 || q4k_rows_per_wave(tiles16, shape.ksplit, 1) == 8) &&  // three tokens: at any row count (128256 x 4096: 55.0 us against 66.7)
                   q4k_ring(ka, shape.ksplit) && q4k_cu_serves(ka, shape.ksplit, static_cast<int>(a.n_tokens))) {
            if (int rc = launch_q4k_cu(ka, 0, st, static_cast<int>(a.n_tokens))) return rc;  // a few tokens replayed against each step's weight
        } else if (plain && a.n_tokens >= 2 && a.n_tokens <= 4 && q4k_cu_kcut_tokens_steps(ka, shape.ksplit, static_cast<int>(a.n_tokens))) {
            if (int rc = launch_q4k_cu_kcut_tokens(ka, static_cast<int>(a.n_tokens), st)) return rc;  // two or three tokens under a K cut
        } else if (!grouped && !w2 && a.n_tokens > 2) {
            return -1;  // more than two tokens of a plain call: only the eight-wave launches above take them
        } else if (two) {
            // both tokens in one pass over the weight, 16-row waves as in the two-token matvec
            if (q4k_ring(ka, shape.ksplit, 1)) launch_q4k_ring<2, true, 1>(ka, shape.ksplit, grid, block, lds, st);
            else {
                if (whole) hipLaunchKernelGGL((gemv_q4k_kernel<2, false, true, 1, true, true>), grid, block, lds, st, ka);
                else hipLaunchKernelGGL((gemv_q4k_kernel<2, false, true, 1, false, true>), grid, block, lds, st, ka);
                CML_COUNT_LAUNCH("q4k.dot.buffers.fused");
            }
        } else if (!plain && ka.shared_act && ka.group_ids && !env_int("CAMELID_HIP_Q4K_GENERAL_ENTRY", 0)) {
            // the decode launch of an expert layer: its own entry
#define CML_Q4K_DIRECT(SPR_, WHOLE_) hipLaunchKernelGGL((gemv_q4k_kernel<1, false, true, SPR_, WHOLE_, false, false, true>), grid, block, lds, st, ka)
            if (ka.route_logits) {
                if (!(half_tiles && ring && ka.n_sb == 16 * shape.ksplit)) return fail(CML_ERR_UNSUPPORTED, "the routing launch serves rows of 4096 values under 8-row waves");
                hipLaunchKernelGGL((gemv_q4k_kernel<1, false, true, 2, true, false, false, true, 3, 8, true>), grid, block, lds, st, ka);
                CML_COUNT_LAUNCH("q4k.dot.direct.ring.route");
            } else if (half_tiles && ring && ka.n_sb == 16 * shape.ksplit && env_int("CAMELID_HIP_Q4K_DIRECT_RING", 1)) {
                hipLaunchKernelGGL((gemv_q4k_kernel<1, false, true, 2, true, false, false, true, 3, 8>), grid, block, lds, st, ka);
                CML_COUNT_LAUNCH("q4k.dot.direct.ring");
            } else if (half_tiles) { if (whole) CML_Q4K_DIRECT(2, true); else CML_Q4K_DIRECT(2, false); CML_COUNT_LAUNCH("q4k.dot.direct.buffers"); }
            else { if (whole) CML_Q4K_DIRECT(1, true); else CML_Q4K_DIRECT(1, false); CML_COUNT_LAUNCH("q4k.dot.direct.buffers"); }
#undef CML_Q4K_DIRECT
        } else if (!grouped && w2 && half_tiles && ring && !env_int("CAMELID_HIP_Q4K_GENERAL_ENTRY", 0)) {
            launch_q4k_ring<1, true, 2, false, true>(ka, shape.ksplit, grid, block, lds, st);  // a plain pair: grid.z = 2
        } else if (!grouped && w2 && !half_tiles && q4k_ring(ka, shape.ksplit, 1) && !env_int("CAMELID_HIP_Q4K_GENERAL_ENTRY", 0)) {
            launch_q4k_ring<1, true, 1, false, true>(ka, shape.ksplit, grid, block, lds, st);
        } else if (half_tiles && plain && !two && q4k_cu_kcut_serves(ka, shape.ksplit)) {
            if (int rc = launch_q4k_cu_kcut(ka, st)) return rc;  // rows of 14336 values cut four ways: eight-wave workgroups, the row quantized once each
        } else if (half_tiles && ring && plain && q4k_cu_serves(ka, shape.ksplit)) {
            if (int rc = launch_q4k_cu(ka, 0, st)) return rc;  // rows of 4096 values, no K cut: eight-wave workgroups
        } else if (half_tiles && ring && plain) {
            launch_q4k_ring<1, true, 2>(ka, shape.ksplit, grid, block, lds, st);
        } else if (!half_tiles && plain && q4k_ring(ka, shape.ksplit, 1)) {
            launch_q4k_ring<1, true, 1>(ka, shape.ksplit, grid, block, lds, st);
        } else if (half_tiles) {
            if (whole) { if (plain) CML_Q4K_LAUNCH(2, true, true); else CML_Q4K_LAUNCH(2, true, false); }
            else { if (plain) CML_Q4K_LAUNCH(2, false, true); else CML_Q4K_LAUNCH(2, false, false); }
            if (plain) CML_COUNT_LAUNCH("q4k.dot.buffers.fused"); else if (w2) CML_COUNT_LAUNCH("q4k.dot.buffers.fused.pair"); else CML_COUNT_LAUNCH("q4k.dot.buffers.fused.grouped");
        } else {
            if (whole) { if (plain) CML_Q4K_LAUNCH(1, true, true); else CML_Q4K_LAUNCH(1, true, false); }
            else { if (plain) CML_Q4K_LAUNCH(1, false, true); else CML_Q4K_LAUNCH(1, false, false); }
            if (plain) CML_COUNT_LAUNCH("q4k.dot.buffers.fused"); else if (w2) CML_COUNT_LAUNCH("q4k.dot.buffers.fused.pair"); else CML_COUNT_LAUNCH("q4k.dot.buffers.fused.grouped");
        }
#undef CML_Q4K_LAUNCH
    }
    CML_HIP_TRY(hipGetLastError());
    return CML_OK;
}

// The conditions under which the direct launch above takes the routing variant, for the caller
// that has to decide between it and a routing launch of its own.
bool gemv_q4k_direct_can_route(const cml_weight *w, int64_t band_rows, int n_slots, bool pair) {
    if (w->fmt != CML_Q4_K || band_rows <= 0 || band_rows % 16 != 0 || w->row_skip != 0 || n_slots < 1 || n_slots > 64) return false;
    if (env_int("CAMELID_HIP_Q4K_GENERAL_ENTRY", 0)) return false;
    Q4KArgs ka{};
    ka.n_sb = static_cast<int>(w->nb);
    ka.sb_stride = w->planes.row_stride[0];
    const Q4KShape shape = pick_shape(band_rows, ka.n_sb);
    const int64_t tiles16 = (band_rows + 15) / 16;
    const bool half_tiles = q4k_rows_per_wave(tiles16, shape.ksplit, static_cast<int64_t>(n_slots) * (pair ? 2 : 1)) == 8;
    return half_tiles && q4k_ring(ka, shape.ksplit) && ka.n_sb == 16 * shape.ksplit;
}

// Calibration: the launch of a plain single-token Q4_K matvec (same grid, same lanes, same
// register buffers) reduced to its weight loads.
int launch_gemv_q4k_loads_only(const cml_weight *w, float *out, hipStream_t st) {
    if (w->rows == 0) return CML_OK;
    MatArgs a{};
    a.w = w;
    a.out = out;
    a.n_tokens = 1;
    a.n_groups = 1;
    return launch_q4k_f32(a, nullptr, nullptr, nullptr, st, 7);
}

// Calibration: the eight-wave single-token launch with parts taken out (mask 1 = no activation, 4 = no store,
// 7 = the weight requests alone).  `out` must hold the weight's rows; its contents are meaningless afterwards.
int launch_gemv_q4k_ablated(const cml_weight *w, const float *x, float *out, int mask, hipStream_t st) {
    if (w->rows == 0) return CML_OK;
    if (mask != 1 && mask != 4 && mask != 7) return fail(CML_ERR_INVALID, "ablation mask must be 1, 4 or 7");
    MatArgs a{};
    a.w = w;
    a.out = out;
    a.n_tokens = 1;
    a.n_groups = 1;
    return launch_q4k_f32(a, nullptr, nullptr, x, st, mask);
}

// One f32 token against two weights of one shape (the gate and up projections of a dense FFN) in one launch.
int launch_gemv_q4k_f32_pair(const cml_weight *w, const cml_weight *w2, const float *x, float *out, float *out2, hipStream_t st) {
    MatArgs a{};
    a.w = w;
    a.out = out;
    a.n_tokens = 1;
    a.n_groups = 1;
    return launch_q4k_f32(a, w2, out2, x, st);
}

// One f32 token against up to four Q4_K weights of one row length (any row counts) in ONE launch: the workgroups of the
// weights lie end to end along grid.x, every workgroup quantizes the token once, and each weight keeps the K cut its
// shape has in a call of its own -- so every output is that call's bits.  -1 = not a set this launch serves (formats,
// row lengths or K cuts differ, rows too long to quantize in the kernel): the caller makes the calls one by one.
int launch_gemv_q4k_f32_multi(const cml_weight *const *ws, int n, const float *x, float *const *outs, hipStream_t st) {
    if (n < 2 || n > 4) return -1;
    if (env_int("CAMELID_HIP_Q4K_GENERAL_ENTRY", 0) || !env_int("CAMELID_HIP_MULTI_LAUNCH", 1)) return -1;
    const int n_sb = static_cast<int>(ws[0]->nb);
    int ksplit = 0;
    int64_t tiles16_all = 0;
    for (int j = 0; j < n; j++) {
        if (ws[j]->fmt != CML_Q4_K || ws[j]->nb != ws[0]->nb || ws[j]->rows <= 0 || ws[j]->planes.row_stride[0] >= (int64_t(1) << 31)) return -1;
        const int ks = pick_shape(ws[j]->rows, n_sb).ksplit;
        if (j && ks != ksplit) return -1;
        ksplit = ks;
        tiles16_all += (ws[j]->rows + ws[j]->row_skip + 15) / 16;
    }
    if (env_int("CAMELID_HIP_Q4K_KCUT_MULTI", 1)) {
        const int rc = launch_q4k_cu_kcut_multi(ws, n, x, outs, ksplit, st);
        if (rc != -1) return rc;
    }
    Q4KArgs ka{};
    ka.n_sb = n_sb;
    ka.x = x;
    ka.ksplit = ksplit;
    ka.ksplit_log2 = ksplit >= 8 ? 3 : (ksplit >= 4 ? 2 : (ksplit >= 2 ? 1 : 0));
    ka.tiles_per_wg = std::max(1, 4 / ksplit);
    const int waves = ksplit * ka.tiles_per_wg;
    // 8-row waves (two lane groups per row) unless the launch is tall enough for 16-row ones; the choice changes no bit
    const bool half_tiles = q4k_rows_per_wave(tiles16_all, ksplit, 1) == 8;
    int wg = 0;
    for (int j = 0; j < 4; j++) {
        const cml_weight *w = ws[std::min(j, n - 1)];
        ka.wm[j] = w->planes.p[0];
        ka.outm[j] = outs[std::min(j, n - 1)];
        ka.stridem[j] = w->planes.row_stride[0];
        ka.rowsm[j] = static_cast<int>(w->rows);
        ka.skipm[j] = w->row_skip;
        if (j < n) {
            const int64_t tiles16 = (w->rows + w->row_skip + 15) / 16;
            const int64_t tiles = half_tiles ? 2 * tiles16 : tiles16;
            wg += static_cast<int>((tiles + ka.tiles_per_wg - 1) / ka.tiles_per_wg);
        }
        ka.wg_end[j] = j < n ? wg : INT32_MAX;
    }
    ka.sb_stride = ka.stridem[0];  // the shape helpers below read these two; every weight passes the same checks
    ka.rows = ka.rowsm[0];
    const size_t lds = static_cast<size_t>(n_sb) * (256 + 32) + ((static_cast<size_t>(n_sb) + 3) & ~size_t(3)) * 4 + static_cast<size_t>(waves) * 16 * 4;
    if (lds > 64 * 1024) return -1;
    const dim3 grid(static_cast<unsigned>(wg)), block(64 * waves);
    const bool whole = q4k_whole_buffers(ka, ksplit);
    if (half_tiles && q4k_ring(ka, ksplit)) {
        launch_q4k_ring<1, true, 2, false, false, true>(ka, ksplit, grid, block, lds, st);
    } else if (!half_tiles && q4k_ring(ka, ksplit, 1)) {
        launch_q4k_ring<1, true, 1, false, false, true>(ka, ksplit, grid, block, lds, st);
    } else {
#define CML_Q4K_MULTI(SPR_, WHOLE_) hipLaunchKernelGGL((gemv_q4k_kernel<1, false, true, SPR_, WHOLE_, true, false, false, 0, 0, false, false, true>), grid, block, lds, st, ka)
        if (half_tiles) { if (whole) CML_Q4K_MULTI(2, true); else CML_Q4K_MULTI(2, false); }
        else { if (whole) CML_Q4K_MULTI(1, true); else CML_Q4K_MULTI(1, false); }
#undef CML_Q4K_MULTI
        CML_COUNT_LAUNCH("q4k.dot.buffers.fused.multi");
    }
    CML_HIP_TRY(hipGetLastError());
    return CML_OK;
}

int launch_gemv_q4k_f32(const cml_weight *w, const float *x, float *out, hipStream_t st, int n_tokens) {
    MatArgs a{};
    a.w = w;
    a.out = out;
    a.n_tokens = n_tokens;  // 1, or 2 (3, 4: -1 where the eight-wave launch does not serve the shape) contiguous rows of x -> out[n][rows]
    a.n_groups = 1;
    return launch_q4k_f32(a, nullptr, nullptr, x, st);
}

// Expert-grouped pair (gate and up of a mixture-of-experts layer), one assignment at a time.
int launch_gemv_q4k_f32_grouped_pair(const MatArgs &a, const cml_weight *w2, float *out2, const float *x, hipStream_t st) {
    return launch_q4k_f32(a, w2, out2, x, st);
}

// ---- mixture-of-experts decode: down projection of the routed experts + weighted sum, one launch ----
//
// One token, k routed experts, Q4_K down matrices stacked by expert.  The separate path is a launch
// with grid.y = routed slot that writes y[slot][row], then a launch that mixes
// out[row] = ((0 + y[0][row] * w[0]) + y[1][row] * w[1]) + ...  (reference src/inference.rs:14255-14257).
// Here a workgroup owns one 16-row tile for ALL slots: its waves are slot x K part (the K cut of
// the shape policy, as in the kernel above), every wave computes what its twin in the separate
// launch computes, and after the one barrier the first 16 threads add each slot's partial chains
// left to right and mix the slots in routed order -- the same operations in the same order,
// without the second launch and without y going through memory.  Same number of waves per
// launch as before (slots x parts x tiles); a slot whose expert id is out of range takes no part.
struct MoeDownSumArgs {
    const uint8_t *w;         // stacked experts, tiled layout
    int64_t sb_stride;
    int rows;                 // rows of one expert (a multiple of 16)
    int n_sb, n_experts, n_slots;
    int ksplit, ksplit_log2;
    const int32_t *idx;       // [n_slots] routed expert of each slot
    const float *weight;      // [n_slots]
    const int8_t *q;          // [n_slots][n_sb*256]: every slot's own activation
    const float *yd;          // [n_slots][n_sb]
    float *out;               // [rows]
};

// OWN (parts of at most 16 super-blocks): every wave stages the activation of its own (slot, K part) and nothing else --
// four 16-byte loads per lane, all requested ahead of the first weight requests, written to the wave's own stretch of
// LDS -- so no workgroup barrier stands before the walk (the shared staging loop made three dependent trips to
// memory, then a barrier for the slowest of eight waves).
template <bool RING, int NSTEPS = 0, bool OWN = false>
__global__ __launch_bounds__(512) void moe_down_sum_q4k_kernel(MoeDownSumArgs a) {
    static_assert(!OWN || RING, "own staging rides with the ring walk");
    // RING: three 2-super-block buffers instead of two 4-super-block ones, as in the matvec above
    // (every K part an even number of super-blocks, at least six: the launcher checks)
    constexpr int U = RING ? 2 : 4;
    constexpr int NB = 3;
    using Regs = Q4KRegs<U>;
    extern __shared__ uint4 smem[];
    const int n_sb = a.n_sb, S = a.n_slots, W = a.ksplit;
    int8_t *ys = reinterpret_cast<int8_t *>(smem);                     // [S][n_sb*256]
    int *bsum = reinterpret_cast<int *>(ys + S * n_sb * 256);          // [S][n_sb*8]
    float *yds = reinterpret_cast<float *>(bsum + S * n_sb * 8);       // [S][n_sb]
    float *part = yds + ((S * n_sb + 3) & ~3);                         // [S][W][16]

    const int tid = threadIdx.x, nthreads = blockDim.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
    const int slot = wave >> a.ksplit_log2, kpart = wave & (W - 1);
    const int expert = a.idx[slot];
    const bool served = expert >= 0 && expert < a.n_experts;   // wave-uniform
    const int tile = blockIdx.x;
    const int s0 = (kpart * n_sb) >> a.ksplit_log2, s1 = ((kpart + 1) * n_sb) >> a.ksplit_log2;
    const int r = lane / LPS, l = lane - r * LPS;
    const uint8_t *wtile = a.w + (static_cast<int64_t>(served ? expert : 0) * (a.rows / 16) + tile) * kQ4KChunk;
    const int piece = r * LPS + l;
    Q4KLane ln;
    ln.c = l;
    ln.sh = (ln.c & 1) * 16;
    ln.upper = ln.c >= 2;
    auto load_buffer = [&](Regs &dst, int sb) __attribute__((always_inline)) {
        if constexpr (RING)
            q4k_load_whole<U, 1>(dst, wtile + static_cast<int64_t>(sb) * a.sb_stride, a.sb_stride, static_cast<uint32_t>(r) * 16, static_cast<uint32_t>(piece) * 16);
        else
            q4k_load<U, 1>(dst, wtile, a.sb_stride, r, piece, sb, s1);
    };

    // every slot's activation row into LDS, with the 32-value sums; the first weight buffer goes out
    // behind the first activation loads
    Regs ra, rb;
    Regs ring[RING ? NB : 1];
    const int c16 = n_sb * 16, n16 = S * c16;
    uint4 *dst = reinterpret_cast<uint4 *>(ys);
    const uint4 *src = reinterpret_cast<const uint4 *>(a.q);
    if constexpr (OWN) {
        const int base16 = (slot * n_sb + s0) * 16, n_loc16 = (s1 - s0) * 16;  // this wave's stretch: at most 256 pieces
        uint4 v[4];
#pragma unroll
        for (int k = 0; k < 4; k++) v[k] = src[base16 + min(lane + 64 * k, n_loc16 - 1)];
        const float yd_mine = a.yd[slot * n_sb + s0 + min(lane, s1 - s0 - 1)];
        __builtin_amdgcn_sched_barrier(0);
        if (served) {
            load_buffer(ring[0], s0);
            load_buffer(ring[1], s0 + U);
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int k = 0; k < 4; k++) {
            const int i = lane + 64 * k;  // lanes 2j, 2j+1 hold the halves of a 32-value group
            int sum = bytesum16(v[k]);
            sum += row_shr_i32<1>(sum);
            if (i < n_loc16) {
                dst[base16 + i] = v[k];
                if (i & 1) bsum[(base16 + i) >> 1] = sum;
            }
        }
        if (lane < s1 - s0) yds[slot * n_sb + s0 + lane] = yd_mine;
        // written and read by this wave alone
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    } else {
    uint4 first = src[min(tid, n16 - 1)];
    __builtin_amdgcn_sched_barrier(0);
    if (served) {
        if constexpr (RING) {
            load_buffer(ring[0], s0);
            load_buffer(ring[1], s0 + U);
        } else {
            load_buffer(ra, s0);
        }
    }
    __builtin_amdgcn_sched_barrier(0);
    for (int i = tid; i < n16 + (n16 & 1); i += nthreads) {  // lanes 2k, 2k+1 stay together for the pair sum
        const uint4 v = i == tid ? first : src[min(i, n16 - 1)];
        int sum = bytesum16(v);
        sum += row_shr_i32<1>(sum);
        if (i < n16) {
            dst[i] = v;
            if (i & 1) bsum[i >> 1] = sum;
        }
    }
    for (int i = tid; i < S * n_sb; i += nthreads) yds[i] = a.yd[i];
    __syncthreads();
    }

    float acc[1] = {0.0f};
    if (served) {
        const int8_t *ys_s = ys + slot * n_sb * 256;
        const int *bsum_s = bsum + slot * n_sb * 8;
        const float *yds_s = yds + slot * n_sb;
        if constexpr (RING) {
            auto compute = [&](const Regs &b, int step) __attribute__((always_inline)) {
                q4k_compute<1, false, U, 1, true>(b, ln, s0 + step * U, s1, ys_s, bsum_s, yds_s, n_sb, acc, nullptr);
                __builtin_amdgcn_sched_barrier(0);
            };
            auto request = [&](Regs &b, int step) __attribute__((always_inline)) {
                load_buffer(b, s0 + step * U);
                __builtin_amdgcn_sched_barrier(0);
            };
            request(ring[2], 2);
            if constexpr (NSTEPS > 0) {  // the part's length known at compile time: the walk unrolled
                static_assert(NSTEPS >= NB, "a part holds at least one full ring");
#pragma unroll
                for (int i = 0; i < NSTEPS; i++) {
                    compute(ring[i % NB], i);
                    if (i + NB < NSTEPS) request(ring[i % NB], i + NB);
                }
            } else {
            const int n = (s1 - s0) / U;
            int k = 0;
            for (; k + 2 * NB <= n; k += NB) {
#pragma unroll
                for (int j = 0; j < NB; j++) {
                    compute(ring[j], k + j);
                    request(ring[j], k + NB + j);
                }
            }
            auto tail = [&](auto extra) __attribute__((always_inline)) {  // `extra` steps are not requested yet
                constexpr int E = decltype(extra)::value;
#pragma unroll
                for (int j = 0; j < NB; j++) {
                    compute(ring[j], k + j);
                    if (j < E) request(ring[j], k + NB + j);
                }
#pragma unroll
                for (int j = 0; j < E; j++) compute(ring[j], k + NB + j);
            };
            switch (n - k - NB) {
                case 0: tail(std::integral_constant<int, 0>{}); break;
                case 1: tail(std::integral_constant<int, 1>{}); break;
                default: tail(std::integral_constant<int, 2>{}); break;
            }
            }
        } else
        for (int sb = s0;;) {
            if (sb + U >= s1) {
                q4k_compute<1, false, U, 1>(ra, ln, sb, s1, ys_s, bsum_s, yds_s, n_sb, acc, nullptr);
                break;
            }
            load_buffer(rb, sb + U);
            __builtin_amdgcn_sched_barrier(0);
            q4k_compute<1, false, U, 1>(ra, ln, sb, s1, ys_s, bsum_s, yds_s, n_sb, acc, nullptr);
            __builtin_amdgcn_sched_barrier(0);
            sb += U;
            if (sb + U >= s1) {
                q4k_compute<1, false, U, 1>(rb, ln, sb, s1, ys_s, bsum_s, yds_s, n_sb, acc, nullptr);
                break;
            }
            load_buffer(ra, sb + U);
            __builtin_amdgcn_sched_barrier(0);
            q4k_compute<1, false, U, 1>(rb, ln, sb, s1, ys_s, bsum_s, yds_s, n_sb, acc, nullptr);
            __builtin_amdgcn_sched_barrier(0);
            sb += U;
        }
    }
    if (l == LPS - 1) part[wave * 16 + r] = acc[0];
    __syncthreads();
    if (tid < 16) {
        const int row = tile * 16 + tid;
        float mix = 0.0f;
        for (int s = 0; s < S; s++) {
            const int e = a.idx[s];
            if (e < 0 || e >= a.n_experts) continue;  // nobody served this slot
            float v = part[(s * W) * 16 + tid];
            for (int k = 1; k < W; k++) v = v + part[(s * W + k) * 16 + tid];
            mix = mix + v * a.weight[s];
        }
        if (row < a.rows) a.out[row] = mix;
    }
}

int q4k_moe_down_sum_waves(int64_t rows_per_expert, int64_t n_sb, int n_slots) { return pick_shape(rows_per_expert, n_sb).ksplit * n_slots; }

// -1: the shape is not one this launch serves (the caller runs the separate launches).
int launch_moe_down_sum_q4k(const cml_weight *down, int n_experts, int n_slots, const int32_t *idx, const float *weight, const int8_t *q,
                            const float *yd, float *out, hipStream_t st) {
    const int64_t rows = down->rows / n_experts;
    if (rows % 16 != 0 || down->row_skip != 0 || n_slots < 1) return -1;
    const Q4KShape shape = pick_shape(rows, down->nb);
    const int waves = shape.ksplit * n_slots;
    const int n_sb = static_cast<int>(down->nb);
    const size_t lds = static_cast<size_t>(n_slots) * n_sb * (256 + 32) + ((static_cast<size_t>(n_slots) * n_sb + 3) & ~size_t(3)) * 4 +
                       static_cast<size_t>(waves) * 16 * 4;
    if (waves > 8 || lds > 64 * 1024) return -1;  // eight waves: the register budget of the two buffers without spills
    MoeDownSumArgs a{};
    a.w = down->planes.p[0];
    a.sb_stride = down->planes.row_stride[0];
    a.rows = static_cast<int>(rows);
    a.n_sb = n_sb;
    a.n_experts = n_experts;
    a.n_slots = n_slots;
    a.ksplit = shape.ksplit;
    a.ksplit_log2 = shape.ksplit >= 8 ? 3 : (shape.ksplit >= 4 ? 2 : (shape.ksplit >= 2 ? 1 : 0));
    a.idx = idx;
    a.weight = weight;
    a.q = q;
    a.yd = yd;
    a.out = out;
    const bool ring = env_int("CAMELID_HIP_Q4K_RING", 1) && !env_int("CAMELID_HIP_Q4K_CLAMPED_LOADS", 0) && n_sb % (2 * shape.ksplit) == 0 &&
                      n_sb / (2 * shape.ksplit) >= 3 && a.sb_stride < (int64_t(1) << 31);
    if (ring && n_sb == 14 * shape.ksplit && env_int("CAMELID_HIP_MOE_DOWN_OWN_STAGING", 1))  // K parts of 3584 values (Mixtral's 14336 cut four ways): seven steps
        hipLaunchKernelGGL((moe_down_sum_q4k_kernel<true, 7, true>), dim3(static_cast<unsigned>(rows / 16)), dim3(64 * waves), lds, st, a);
    else if (ring && n_sb == 14 * shape.ksplit)
        hipLaunchKernelGGL((moe_down_sum_q4k_kernel<true, 7>), dim3(static_cast<unsigned>(rows / 16)), dim3(64 * waves), lds, st, a);
    else if (ring) hipLaunchKernelGGL(moe_down_sum_q4k_kernel<true>, dim3(static_cast<unsigned>(rows / 16)), dim3(64 * waves), lds, st, a);
    else hipLaunchKernelGGL(moe_down_sum_q4k_kernel<false>, dim3(static_cast<unsigned>(rows / 16)), dim3(64 * waves), lds, st, a);
    if (ring) CML_COUNT_LAUNCH("q4k.down_sum.ring"); else CML_COUNT_LAUNCH("q4k.down_sum.buffers");
    CML_HIP_TRY(hipGetLastError());
    return CML_OK;
}

// ---- the generic 8-lane order of the reference's wire row dot, bit for bit ----------------------
//
// q4_k_wire_row_dot (src/inference.rs:25806-25889, the Q4_K row dot of the Gemma-4 wire lane and
// the oracle of the reference's CUDA matvec) is not the fused chain the kernels above keep: per
// super-block it takes eight integer lanes by value index modulo 8
// (aux32[l] += scale_j * y * a), sums[l] += (d * yd) * (float)aux32[l] with multiply and add
// rounded separately, sumf -= (dmin * yd) * (float)sumi for the mins, and returns
// sumf + (((0 + sums[0]) + sums[1]) + ...).  The kernels above match it to 1e-5; this one
// reproduces it exactly and serves every plain Q4_K call under CAMELID_HIP_Q4K_LANE_ORDER=1
// (speed is secondary: byte loads from the tiled layout, one wave per row).  Lane = 8 * g + l:
// eight super-blocks g per pass, their integers independent; the f32 sums are then advanced in
// super-block order by the lanes of g = 0 through LDS.
__device__ __forceinline__ void q4k_wave_lds_sync() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

__global__ __launch_bounds__(256) void gemv_q4k_lanes_kernel(const uint8_t *__restrict__ wbase, int64_t sb_stride, int rows, int row_skip,
                                                             int n_sb, const int8_t *__restrict__ q, const float *__restrict__ yd,
                                                             float *__restrict__ out, const float *__restrict__ residual) {
    extern __shared__ uint4 smem[];
    int8_t *ys = reinterpret_cast<int8_t *>(smem);                        // [n_sb*256]
    float *yds = reinterpret_cast<float *>(ys + n_sb * 256);              // [n_sb]
    float *xch = yds + ((n_sb + 3) & ~3);                                 // [4 waves][64 lane terms + 8 mins terms]
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int token = blockIdx.y;
    const int8_t *qt = q + static_cast<int64_t>(token) * n_sb * 256;
    for (int i = tid; i < n_sb * 16; i += 256) reinterpret_cast<uint4 *>(ys)[i] = reinterpret_cast<const uint4 *>(qt)[i];
    for (int i = tid; i < n_sb; i += 256) yds[i] = yd[static_cast<int64_t>(token) * n_sb + i];
    __syncthreads();
    const int row = blockIdx.x * 4 + wave;
    if (row >= rows) return;  // whole waves leave; no workgroup barrier follows
    const int g = lane >> 3, l = lane & 7;
    const int lrow = row + row_skip;  // row in the tiled layout
    const uint8_t *tile = wbase + static_cast<int64_t>(lrow >> 4) * kQ4KChunk;
    const int rl = lrow & 15;
    float *mine = xch + wave * 72;
    float sum_l = 0.0f;   // lanes of g == 0: sums[l]
    float sumf = 0.0f;    // lane 0: the mins chain
    for (int sb0 = 0; sb0 < n_sb; sb0 += 8) {
        const int sb = sb0 + g;
        float term = 0.0f, mterm = 0.0f;
        if (sb < n_sb) {
            const uint8_t *chunk = tile + static_cast<int64_t>(sb) * sb_stride;
            const uint4 hdr = *reinterpret_cast<const uint4 *>(chunk + rl * 16);
            uint32_t sc03, sc47, m03, m47;
            q4k_unpack_scales(hdr.y, hdr.z, hdr.w, sc03, sc47, m03, m47);
            const int8_t *y = ys + sb * 256;
            int aux = 0;
#pragma unroll
            for (int j = 0; j < 8; j++) {  // sub-block j: chunk j / 2, low (even j) or high nibbles
                const int scale = static_cast<int>(((j < 4 ? sc03 : sc47) >> (8 * (j & 3))) & 0xff);
                int part = 0;
#pragma unroll
                for (int k = 0; k < 4; k++) {
                    const int jj = 8 * k + l;  // byte of the chunk
                    const uint8_t byte = chunk[(jj < 16 ? 256 : 1280) + rl * 64 + (j >> 1) * 16 + (jj & 15)];
                    const int a4 = (j & 1) ? (byte >> 4) : (byte & 15);
                    part += static_cast<int>(y[32 * j + jj]) * a4;
                }
                aux += scale * part;
            }
            // the mins: lane l takes the 16-value sums j = l and l + 8, the eight lanes' parts are added (exact integers)
            int sumi = 0;
#pragma unroll
            for (int h = 0; h < 2; h++) {
                const int j = l + 8 * h;
                int bs = 0;
#pragma unroll
                for (int t = 0; t < 16; t++) bs += y[16 * j + t];
                const int g8 = j >> 1;
                sumi += bs * static_cast<int>(((g8 < 4 ? m03 : m47) >> (8 * (g8 & 3))) & 0xff);
            }
            sumi += __shfl_xor(sumi, 1);
            sumi += __shfl_xor(sumi, 2);
            sumi += __shfl_xor(sumi, 4);
            const float d = f16_bits_to_f32(hdr.x & 0xffffu), dmin = f16_bits_to_f32(hdr.x >> 16);
            const float ydv = yds[sb];
            const float dd = d * ydv;
            term = dd * static_cast<float>(aux);
            mterm = (dmin * ydv) * static_cast<float>(sumi);
        }
        mine[lane] = term;
        if (l == 0) mine[64 + g] = mterm;
        q4k_wave_lds_sync();
        if (g == 0) {
            const int n = min(8, n_sb - sb0);
            for (int k = 0; k < n; k++) {
                sum_l = sum_l + mine[8 * k + l];
                sumf = sumf - mine[64 + k];  // only lane 0's copy is used
            }
        }
        q4k_wave_lds_sync();
    }
    if (g == 0) mine[l] = sum_l;
    q4k_wave_lds_sync();
    if (lane == 0) {
        float lanes = 0.0f;
        for (int k = 0; k < 8; k++) lanes = lanes + mine[k];
        float total = sumf + lanes;
        if (residual) total = total + residual[row];
        out[static_cast<int64_t>(token) * rows + row] = total;
    }
}

bool q4k_lane_order() { return env_int("CAMELID_HIP_Q4K_LANE_ORDER", 0) != 0; }

static int launch_gemv_q4k_lanes(const MatArgs &a, hipStream_t st) {
    const cml_weight *w = a.w;
    const int n_sb = static_cast<int>(w->nb);
    const size_t lds = static_cast<size_t>(n_sb) * 256 + ((static_cast<size_t>(n_sb) + 3) & ~size_t(3)) * 4 + 4 * 72 * 4;
    if (lds > 64 * 1024) return fail(CML_ERR_UNSUPPORTED, "Q4_K activation of %d super-blocks exceeds the LDS staging limit", n_sb);
    if (a.n_tokens > 65535) return fail(CML_ERR_UNSUPPORTED, "at most 65535 tokens per call in the lane-order mode");
    hipLaunchKernelGGL(gemv_q4k_lanes_kernel, dim3(static_cast<unsigned>((w->rows + 3) / 4), static_cast<unsigned>(a.n_tokens)), dim3(256), lds, st,
                       w->planes.p[0], w->planes.row_stride[0], static_cast<int>(w->rows), w->row_skip, n_sb, a.q, a.scales, a.out, a.residual);
    CML_COUNT_LAUNCH("q4k.lanes");
    CML_HIP_TRY(hipGetLastError());
    return CML_OK;
}

int launch_gemv_q4k(const MatArgs &a, hipStream_t st) {
    const cml_weight *w = a.w;
    if (w->rows == 0 || a.n_tokens == 0) return CML_OK;
    const bool grouped = a.group_offsets != nullptr || a.group_ids != nullptr;
    if (!grouped && !a.ints && q4k_lane_order()) return launch_gemv_q4k_lanes(a, st);
    Q4KArgs ka{};
    ka.w = w->planes.p[0];
    ka.sb_stride = w->planes.row_stride[0];
    ka.rows = static_cast<int>(grouped ? a.band_rows : w->rows);
    if (grouped && ((ka.rows % 16) != 0 || w->row_skip != 0))
        return fail(CML_ERR_UNSUPPORTED, "Q4_K expert bands must be whole 16-row tiles (%d rows, first tile offset %d)", ka.rows, w->row_skip);
    ka.row_skip = grouped ? 0 : w->row_skip;
    ka.n_sb = static_cast<int>(w->nb);
    ka.residual = a.residual;
    ka.ints = a.ints;
    ka.group_offsets = a.group_offsets;
    ka.group_rows = a.group_rows;
    ka.group_ids = a.group_ids;
    ka.n_groups = a.n_groups;
    const Q4KShape shape = pick_shape(ka.rows, ka.n_sb);
    if (grouped) {
        // One launch: every group walks its own assignments in passes of NT
        // (NT sized for the most a single group can hold).
        ka.q = a.q;
        ka.yd = a.scales;
        ka.out = a.out;
        const int nt = cap_nt(a.n_tokens, ka.n_sb, shape.ksplit * shape.tiles_per_wg);
        return launch_q4k_pick_nt(ka, shape, a.group_ids ? a.max_active : a.n_groups, nt, false, st);
    }
    // Plain call: tokens are served in launches of up to 8 activation rows.
    int64_t t0 = 0;
    while (t0 < a.n_tokens) {
        const int nt = cap_nt(a.n_tokens - t0, ka.n_sb, shape.ksplit * shape.tiles_per_wg);
        ka.q = a.q + t0 * w->cols;
        ka.yd = a.scales + t0 * w->nb;
        ka.out = a.out + t0 * ka.rows;
        if (int rc = launch_q4k_pick_nt(ka, shape, 1, nt, a.ints != nullptr, st)) return rc;
        t0 += nt;
    }
    return CML_OK;
}

int launch_gemm_q4k(const MatArgs &a, hipStream_t st) { return launch_gemv_q4k(a, st); }

}  // namespace cml
