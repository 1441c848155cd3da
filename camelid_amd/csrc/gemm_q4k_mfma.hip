// Q4_K x Q8_K small-batch matmul on the int8 matrix cores (gfx950), for
// batches of 4 tokens and more: speculative-verify chunks and short prefill.
//
// Arithmetic: identical, cell by cell, to the matvec kernel (gemv_q4k.hip;
// reference q4_k_dot_scalar, src/diffusion_gemma/refmath.rs:504-562):
//     per super-block:  acc = fma(-(yd*dmin), (float)P, acc);  acc = fma(yd*d, (float)S, acc)
//     S = sum_g sc_g * sum_{t<32} q*y      P = sum_g m_g * sum_{t<32} y
//
// Every 32-value sub-block has its own 6-bit scale, and sc*q (up to 945) does
// not fit an int8 operand -- but the scale splits into two 3-bit digits,
// sc = 8*sc_hi + sc_lo, and q*sc_lo, q*sc_hi (at most 15*7 = 105) do fit.  So
//     S = sum_k (q_k*sc_lo[g(k)]) * y_k  +  8 * sum_k (q_k*sc_hi[g(k)]) * y_k
// is two int8 contractions that run across sub-block boundaries and accumulate
// over the whole super-block inside the matrix core; a third one whose weight
// operand is the 6-bit min replicated gives P.  All three are exact integers,
// so every cell equals the packed-dot result.  The digit products cost one
// packed 16-bit multiply per four weights (a byte pair times a digit never
// carries into its neighbour), independent of the token count.
//
// Instruction: v_mfma_i32_16x16x64_i8.  One instruction contracts 64 values of ONE nibble plane
// (low nibbles = the even sub-block of a 32-byte chunk, high nibbles = the odd one) taken from two
// chunks, ch = 2q + half for q = 0, 1 -- the contraction index may be assigned freely as long as
// both operands agree, and the sum is an exact integer:
//     A[t][k]  = y_t[64ch + 32plane + 16p + j]         16 tokens, from LDS
//     B[k][n]  = digit-scaled nibble `plane` of byte j of piece p of chunk ch of row n
//     D[t][n] += ...                                   over the 4 steps (q, plane) of a super-block
// Lane L supplies A-row t = L%16 and B-column n = L%16 at k = 16*(L/16)..+15, where L/16 = 2*half + p:
// piece p (a or b) of chunk ch -- so a lane loads the 16 bytes of ONE piece of TWO chunks, both
// nibbles of every byte are its own (one sub-block per lane and step, hence one scale digit pair),
// and the 64 lanes of a load cover 1024 distinct bytes.  It receives D[4*(L/16)+v][L%16], v < 4:
// four tokens of one weight row, whose f32 chains live in that lane, in super-block order.
//
// A workgroup is 4 waves: 4/TB consecutive 16-row tiles x TB token blocks of
// 16*GPW tokens, sharing the staged activations of NTOK = 16*GPW*TB tokens.  K is
// walked in phases of KC = 128/NTOK super-blocks: a phase's activations (rows
// padded by 16 B against bank conflicts) sit in one of two LDS buffers; the next
// phase's loads are issued at the start of the current phase, ahead of the
// weight loads, and stored at its end, so the only barriers are the phase
// boundaries.  Weights (tile-interleaved layout, layout.hip) are double-buffered
// in registers.  When the matvec kernel would split K for this weight shape (few
// row tiles, long rows: an FFN down projection), the same split is reproduced, so
// every cell equals the matvec result bit for bit: with KS = 2 or 4 waves per row
// tile, each walking one part of K and the partial chains added left to right
// through LDS at the end -- which is also what fills the chip when there are
// fewer row tiles than SIMDs -- or, for other split factors, inside the lane (the
// chain restarts at the split points).
//
// Staged-once mode (ONCE): where the whole activation of a workgroup's tokens fits the LDS -- 16 tokens x up to 32
// super-blocks, or 32 tokens x up to 16 -- it is staged in the prologue and the walk has no barrier.  Such a launch
// is sized to be resident at once (two workgroups per compute unit for expert groups with 16 tokens per wave, one
// otherwise) and each workgroup walks every gridDim.x-th group of four row tiles, the register ring refilled across
// the groups: the staging and the start of the weight stream are paid once per workgroup, and the launch sweeps the
// weight as one contiguous front.  It serves expert-grouped gate|up launches and plain calls of up to 32 tokens on
// weights of more than 16384 rows (up to 16 tokens: any uncut weight with rows of 5120 / 6144 / 8192 values).
#include <type_traits>

#include <atomic>
#include <string>

#include "cml_device.hpp"
#include "cml_host.hpp"

#pragma clang fp contract(off)

namespace cml {

typedef int v4i __attribute__((ext_vector_type(4)));

constexpr int kSlabRow = 256 + 16;  // bytes of one token's super-block in LDS (padded)

struct Q4KMfmaArgs {
    const uint8_t *w;   // tiled layout [super-block][tile][2304 B]
    int64_t sb_stride;
    int rows, n_sb;
    int row_skip;       // leading rows of the first tile that precede this weight view (0..15)
    const int8_t *q;    // [n_tokens][n_sb*256]
    const float *yd;    // [n_tokens][n_sb]
    float *out;         // [n_tokens][rows]
    int n_tokens;       // plain: activation rows; grouped: the most assignments one group can hold
    int ksplit;         // association to reproduce (see gemv_q4k.hip)
    // Grouped call (mixture of experts): blockIdx.z = group e, which owns the weight band of rows
    // [e*rows, (e+1)*rows) and the assignments [group_offsets[e], group_offsets[e+1]); assignment j
    // reads activation row group_rows[j] (j itself when null) and writes output row j.
    const int32_t *group_offsets;
    const int32_t *group_rows;
    const int32_t *group_ids;  // z-slot -> group (-1: unused slot), or null (the z-slot is the group)
    // Pair launch (grouped calls only): a second stacked weight of the same shape against the same activations,
    // written to out2 (gate and up of an expert layer in ONE launch: blockIdx.z = 2 * slot + which, so the two
    // kernels' last, partly filled rounds of workgroups become one).
    const uint8_t *w2;
    float *out2;
    // Rows whose whole activation fits the LDS are staged in the prologue, once.  A workgroup of such a launch walks
    // every gridDim.x-th group of row tiles (of both weights of a pair launch, the second weight's groups following
    // the first's) against the activation it staged, the weight ring running on across the group boundaries;
    // blockIdx.z is then the group slot alone.
    int stage_once;
};

struct MfmaWeights {
    uint4 hdr;
    uint4 piece[2];  // this lane's 16 nibble bytes of the two chunks it contracts (both nibbles of every byte are its own)
};

// hdr_ptr / piece_ptr already include the lane's offsets inside a tile entry; `off` = sb * sb_stride.
// STREAM: non-temporal loads, for launches that read every weight byte once (staged-once mode: one token column
// per weight, or per expert; the 32-token Mixtral-shaped layer 173 -> 165 us).  Launches with several token columns
// read the weight once per column and want the later columns served by the caches (4096 x 14336, 64 tokens:
// 30.8 us with plain loads, 32.4 non-temporal).
template <bool STREAM = false>
__device__ __forceinline__ void mfma_load_weights(MfmaWeights &r, const uint8_t *hdr_ptr, const uint8_t *piece_ptr,
                                                  int64_t off) {
    if constexpr (STREAM) {
        r.hdr = ldg16_stream(hdr_ptr + off);
        r.piece[0] = ldg16_stream(piece_ptr + off);
        r.piece[1] = ldg16_stream(piece_ptr + off + 32);
    } else {
        r.hdr = ldg16(hdr_ptr + off);
        r.piece[0] = ldg16(piece_ptr + off);
        r.piece[1] = ldg16(piece_ptr + off + 32);
    }
}

__device__ __forceinline__ v4i as_v4i(const uint4 &v) {
    v4i r = {static_cast<int>(v.x), static_cast<int>(v.y), static_cast<int>(v.z), static_cast<int>(v.w)};
    return r;
}

typedef unsigned short us2 __attribute__((ext_vector_type(2)));
typedef _Float16 v4h __attribute__((ext_vector_type(4)));
typedef float v4f __attribute__((ext_vector_type(4)));

// P = sum_g m_g * sum_{t<32} y[32g+t] on the matrix cores without an int8 operand of replicated
// mins: the sums of the activation's sixteen 16-value runs (at most 16 * 127 = 2032 in magnitude:
// exact in f16) are staged beside the activation, the 6-bit mins are exact in f16, so ONE
// v_mfma_f32_16x16x16_f16 over k = run index gives P in f32 -- every product and every partial sum
// an integer below 2^24, hence exact whatever the order -- where four int8 instructions and
// their four replicated operands were needed, and the int -> float conversion falls away.
// Lane (n, kq) supplies runs 4 * kq .. + 3: the mins of sub-blocks 2 * kq and 2 * kq + 1, twice each.
__device__ __forceinline__ v4h q4k_min_operand(uint32_t m03, uint32_t m47, int kq) {
    const uint32_t mw = ((kq & 2) ? m47 : m03) >> (16 * (kq & 1));
    const _Float16 ma = static_cast<_Float16>(static_cast<float>(mw & 0xffu));
    const _Float16 mb = static_cast<_Float16>(static_cast<float>((mw >> 8) & 0xffu));
    return v4h{ma, ma, mb, mb};
}

// The sum of a 16-byte piece of int8 activation as f16 (exact).
__device__ __forceinline__ _Float16 run_sum_f16(const uint4 &piece) { return static_cast<_Float16>(static_cast<float>(bytesum16(piece))); }

// The two 3-bit digits of the scales in bytes 0 and 1 of `scw`, each replicated into both 16-bit halves of a word
// (operands of scale_bytes): lo2[plane], hi2[plane].
__device__ __forceinline__ void q4k_digit_words(uint32_t scw, uint32_t (&lo2)[2], uint32_t (&hi2)[2]) {
    const uint32_t lo = scw & 0x07070707u, hi = (scw >> 3) & 0x07070707u;
    lo2[0] = __builtin_amdgcn_perm(lo, lo, 0x0c000c00u);
    lo2[1] = __builtin_amdgcn_perm(lo, lo, 0x0c010c01u);
    hi2[0] = __builtin_amdgcn_perm(hi, hi, 0x0c000c00u);
    hi2[1] = __builtin_amdgcn_perm(hi, hi, 0x0c010c01u);
}

// Four bytes (each < 16) times one digit (< 8, replicated in both 16-bit halves of `digit2`).
__device__ __forceinline__ int scale_bytes(uint32_t bytes, uint32_t digit2) {
    const us2 p = __builtin_bit_cast(us2, bytes) * __builtin_bit_cast(us2, digit2);
    return __builtin_bit_cast(int, p);
}

template <int GPW, int TB, bool SPLIT, int KS = 1, bool PLAIN = false, bool ONCE = false, int NSB = 0>
__global__ __launch_bounds__(256) void gemm_q4k_mfma_kernel(Q4KMfmaArgs a) {
    static_assert(!(SPLIT && KS > 1), "K is split across waves or inside the lane, not both");
    constexpr int NTOK = 16 * GPW * TB;              // tokens staged per workgroup
    // super-blocks per phase and K part (a buffer holds up to 128 token-super-blocks)
    constexpr int KC = (128 / (NTOK * KS)) > 0 ? 128 / (NTOK * KS) : 1;
    constexpr int RT = 4 / (TB * KS);                // row tiles per workgroup
    // P through one f16 matrix instruction on staged run sums (q4k_min_operand) where it pays: two token groups per
    // wave, no K parts (14336 x 4096, 32 tokens: 13.8 -> 13.0 us).  Elsewhere the staging costs what the instructions
    // save or more (64 tokens 19.1 -> 20.1 us, expert groups 194.7 -> 196.7 us per layer), and with K parts the 32
    // bytes per token and slab are the difference between two workgroups per compute unit and one (27.4 -> 37.8 us).
    constexpr bool kF16P = (GPW == 2 && KS == 1) || ONCE;  // (staged once, the run sums cost one pass in the prologue)
    constexpr int kActBytes = KS * KC * NTOK * kSlabRow;  // activation slabs of one phase
    constexpr int kBufBytes = kActBytes + (kF16P ? KS * KC * NTOK * 32 : 0);  // + the sums of their 16-value runs, f16 [slab][token][16]
    constexpr int nthreads = 256;
    constexpr int kPieces = NTOK * 16;               // 16-byte pieces of one super-block of all tokens
    constexpr int kPer = kPieces / nthreads;         // 1, 2 or 4
    // weight super-blocks a wave keeps in flight (register ring): a 16-token step is short, so it
    // takes 8 to cover the HBM latency; steps over more tokens are longer and 4 are enough
    // (staged-once mode with the whole row of 16 requested in the prologue: the 32-token expert layer 174 -> 179 us)
    // (staged-once mode with two token groups per wave: one workgroup per compute unit, one wave per SIMD -- eight slots fit)
    // (rows of 12 / 14 super-blocks known at compile time: six / seven slots, so that a row is two rounds of the ring)
    constexpr int RING = NSB == 12 ? 6 : NSB == 14 ? 7 : NSB == 20 ? 10 : ((GPW == 1 && KS == 1) || ONCE) ? 8 : 4;
    static_assert((ONCE || RING % KC == 0) && kPer >= 1 && RT >= 1, "phase / staging shape");
    // staged-once mode holds a row of up to 16 super-blocks as kOnceChunks chunks of KC slabs, each laid out like a phase buffer
    // (one token group per wave: also rows of 20 / 24 / 32 super-blocks -- 32 x 16 tokens fill a compute unit's LDS like 16 x 32)
    constexpr int kOnceChunks = (NSB > 16 ? 32 : 16) / KC;
    // NSB: the row length in super-blocks where the launcher knows it at compile time (staged-once mode; 0 = any)
    static_assert(NSB == 0 || (ONCE && NSB % RING == 0 && (NSB <= 16 || (NSB <= 32 && GPW == 1))), "row length known at compile time: whole rounds of the ring");
    extern __shared__ uint4 smem[];
    uint8_t *buf0 = reinterpret_cast<uint8_t *>(smem);  // [KC][NTOK][kSlabRow], then [KC][NTOK][16] f16
    uint8_t *buf1 = buf0 + kBufBytes;
    float *yds = reinterpret_cast<float *>(buf0 + (ONCE ? kOnceChunks : 2) * kBufBytes);  // [n_sb][NTOK]

    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
    const int n_sb = a.n_sb;
    const int n = lane & 15, kq = lane >> 4;         // B/D column (weight row in tile) and k-quarter / A-row quad
    const int half = kq >> 1;                        // which sub-block of a chunk this lane's B bytes belong to
    const int ks = wave % KS, w2 = wave / KS;        // K part of this wave; its (row tile, token block)
    const int rt = w2 / TB, tb = w2 - rt * TB;
    // this wave's part of K (the matvec kernel's split points) and the longest part
    const int s_begin = KS > 1 ? ks * n_sb / KS : 0, s_end = KS > 1 ? (ks + 1) * n_sb / KS : n_sb;
    const int n_loc = s_end - s_begin, n_max = (n_sb + KS - 1) / KS;
    const int n_tiles = (a.rows + a.row_skip + 15) / 16;
    const bool grouped = !PLAIN && a.group_offsets != nullptr;
    const bool pair = !PLAIN && a.w2 != nullptr;
    // Staged-once mode: this workgroup's units are u0, u0 + ustride, ... of the launch's list -- the groups of RT
    // row tiles of the weight, then (pair launch) those of the second weight; strided by the grid, so that at any
    // moment neighbouring workgroups read neighbouring tile entries and the launch sweeps the weight as one front.
    // Otherwise one unit, and a pair launch keeps the weight in the low bit of blockIdx.z.
    const int units_per_w = (n_tiles + RT - 1) / RT;
    const int u0 = static_cast<int>(blockIdx.x), ustride = static_cast<int>(gridDim.x);
    const int n_units = ONCE ? ((pair ? 2 * units_per_w : units_per_w) - 1 - u0) / ustride + 1 : 1;
    const int zslot = (pair && !ONCE) ? static_cast<int>(blockIdx.z >> 1) : static_cast<int>(blockIdx.z);
    // the unit being consumed: its weight, row tile and this lane's output row
    bool second = ONCE ? (pair && u0 >= units_per_w) : (pair && (blockIdx.z & 1));
    int tile = (u0 - (ONCE && second ? units_per_w : 0)) * RT + rt;
    int row = tile * 16 + n - a.row_skip;
    const int64_t band = grouped ? (a.group_ids ? a.group_ids[zslot] : zslot) : 0;
    if (band < 0) return;  // a z-slot past the groups in use
    const int a0 = grouped ? a.group_offsets[band] : 0;                      // first assignment of this group
    const int n_assign = grouped ? a.group_offsets[band + 1] - a0 : a.n_tokens;
    const int tok0 = blockIdx.y * NTOK;                    // first token (assignment of the group) of this workgroup
    if (tok0 >= n_assign) return;                          // nothing routed here: the whole workgroup leaves
    const int n_here = min(NTOK, n_assign - tok0);
    // tile entry of super-block 0 of row tile `t` of this group's band (tiles past the end read the last one; their cells are not stored)
    auto tile_entry = [&](bool of_second, int t) __attribute__((always_inline)) -> const uint8_t * {
        return (of_second ? a.w2 : a.w) + (band * (a.rows / 16) + min(t, n_tiles - 1)) * 2304;
    };
    const uint8_t *wtile = tile_entry(second, tile);
    // activation row of local token t (tokens past the end repeat the last one; their cells are not stored)
    auto act_row = [&](int t) __attribute__((always_inline)) -> int64_t {
        const int j = a0 + tok0 + min(t, n_here - 1);
        if (PLAIN) return j;
        return a.group_rows ? a.group_rows[j] : j;
    };

    // activation scales: yds[sb][token] (tokens past the end repeat the last one; their cells are not stored)
    for (int i = tid; i < n_sb * NTOK; i += nthreads) {
        const int sb = i / NTOK, t = i - sb * NTOK;
        yds[i] = a.yd[act_row(t) * n_sb + sb];
    }

    // Staging: each thread owns kPer fixed (token, piece) pairs; only the super-block moves.
    // (native vector type on purpose: assigning the HIP uint4 struct between address spaces
    // becomes a memcpy that pins the staging array in scratch memory)
    const v4i *stage_src[kPer];
    int stage_dst[kPer];
#pragma unroll
    for (int k = 0; k < kPer; k++) {
        const int i = tid + k * nthreads;
        const int t = i >> 4, piece = i & 15;
        stage_src[k] = reinterpret_cast<const v4i *>(a.q + act_row(t) * n_sb * 256) + piece;
        stage_dst[k] = t * kSlabRow + piece * 16;
    }
    typedef v4i StageRegs[KS * KC][kPer];
    StageRegs sreg;
    auto stage_load_to = [&](StageRegs &sreg, int p0) __attribute__((always_inline)) {  // of every K part, the KC super-blocks starting at its p0-th
#pragma unroll
        for (int kp = 0; kp < KS; kp++)
#pragma unroll
            for (int s = 0; s < KC; s++) {
                const int off = min((KS > 1 ? kp * n_sb / KS : 0) + p0 + s, n_sb - 1) * 16;  // in uint4 units
#pragma unroll
                for (int k = 0; k < kPer; k++) sreg[kp * KC + s][k] = stage_src[k][off];
            }
    };
    auto stage_load = [&](int p0) __attribute__((always_inline)) { stage_load_to(sreg, p0); };
    auto stage_store_from = [&](const StageRegs &sreg, uint8_t *buf) __attribute__((always_inline)) {
#pragma unroll
        for (int s = 0; s < KS * KC; s++)
#pragma unroll
            for (int k = 0; k < kPer; k++) {
                *reinterpret_cast<v4i *>(buf + s * (NTOK * kSlabRow) + stage_dst[k]) = sreg[s][k];
                // thread tid + k * nthreads holds piece (token, piece) = that index: run sums are [slab][token][piece]
                if constexpr (kF16P)
                    reinterpret_cast<_Float16 *>(buf + kActBytes)[s * (NTOK * 16) + tid + k * nthreads] =
                        run_sum_f16(make_uint4(sreg[s][k][0], sreg[s][k][1], sreg[s][k][2], sreg[s][k][3]));
            }
    };
    auto stage_store = [&](uint8_t *buf) __attribute__((always_inline)) { stage_store_from(sreg, buf); };

    // Lane constants.
    const int hdr_off = n * 16;
    // A matrix instruction contracts 64 values of ONE nibble plane of two 32-byte chunks, ch = 2 * q + half
    // (q = 0, 1): the lane needs piece a (values 0..15) or b (16..31) of those two chunks only, and the 64
    // lanes of a load cover 1024 distinct bytes of the tile entry.
    const int piece_off = ((kq & 1) ? 1280 : 256) + n * 64 + half * 16;
    // (staged-once mode: the unit being REQUESTED, which runs ahead of the one being consumed)
    const uint8_t *w_hdr = wtile + hdr_off;
    const uint8_t *w_piece = wtile + piece_off;
    // A operand: this lane is token (lane & 15) of a group; step (q, plane) takes bytes 128q + 64half + 32plane + 16(kq&1) .. +15.
    const int a_off = (lane & 15) * kSlabRow + 64 * half + 16 * (kq & 1);  // + 128q + 32plane, + token-group and slot offsets
    // D values v = 0..3 of this lane: tokens 4*kq + v of the group, weight row n.
    const int cell_tok = 4 * kq;
    const int sc_shift = 16 * half;                 // scales of sub-blocks 2*half, 2*half+1 (and +4) within their words

    // A wave streams its tile through a ring of RING register slots: slot i is
    // refilled with super-block sb + RING right after super-block sb has been
    // consumed from it, so RING - 1 super-blocks (about 18 KB per wave) are in
    // flight under the arithmetic -- with one wave per SIMD that depth, not the
    // occupancy, is what covers the HBM latency.
    MfmaWeights ring[RING];
    // `loc` counts super-blocks inside this wave's part of K
    auto load_slot = [&](MfmaWeights &r, int loc) __attribute__((always_inline)) {
        mfma_load_weights<false>(r, w_hdr, w_piece, min(s_begin + loc, s_end - 1) * a.sb_stride);
    };
    // Staged-once mode: the next super-block of the walk over this workgroup's units.  The request itself is
    // unconditional (past the end of the walk the last super-block is requested again: a cache hit, at most
    // RING - 1 times per wave and only for walks that are no whole number of rounds), so the ring's loads stay
    // straight-line code and the waits on them exact; only the bookkeeping, uniform over the wave, branches.
    int pf_sb = 0, pf_unit = 0;
    auto request_next = [&](MfmaWeights &r) __attribute__((always_inline)) {
        mfma_load_weights<true>(r, w_hdr, w_piece, pf_sb * a.sb_stride);
        if (pf_sb + 1 < n_sb) {
            ++pf_sb;
        } else if (pf_unit + 1 < n_units) {
            pf_sb = 0;
            ++pf_unit;
            const int u = u0 + pf_unit * ustride;
            const bool s2 = pair && u >= units_per_w;
            const uint8_t *wt = tile_entry(s2, (u - (s2 ? units_per_w : 0)) * RT + rt);
            w_hdr = wt + hdr_off;
            w_piece = wt + piece_off;
        }
    };
    // ONCE (the launcher's choice for rows of up to 16 super-blocks; one or two 16-token groups per wave, no K parts): the LDS holds the
    // whole activation, so it is staged ONCE -- no barrier in the middle of the walk (0.9 us per workgroup waiting
    // for its slowest wave, per-wave time stamps) and no re-read of clamped slabs in the last phase.  The chunks of
    // KC slabs follow one another, so slab s of the row sits where phase s / KC would have put it.
    static_assert(!ONCE || (GPW <= 2 && KS == 1 && TB == 1), "staged-once mode: one or two token groups per wave, no K parts");
    if constexpr (ONCE) {
        // (half of the weight ring is requested behind the first two chunks of the activation, the other half once the staging registers are free)
        StageRegs sreg2;
        stage_load(0);
        stage_load_to(sreg2, KC);
        auto request_first = [&](MfmaWeights &r, int i) __attribute__((always_inline)) {
            if constexpr (NSB > 0) mfma_load_weights<true>(r, w_hdr, w_piece, i * a.sb_stride);
            else request_next(r);
        };
#pragma unroll
        for (int i = 0; i < RING / 2; i++) request_first(ring[i], i);
        __builtin_amdgcn_sched_barrier(0);
        stage_store(buf0);
        stage_store_from(sreg2, buf1);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int i = RING / 2; i < RING; i++) request_first(ring[i], i);
        // the chunks past the first two (32 tokens: chunks of four slabs), where the row has them
#pragma unroll
        for (int c = 2; c < kOnceChunks; c += 2) {
            if (c * KC < n_sb) {
                stage_load(c * KC);
                stage_load_to(sreg2, (c + 1) * KC);
                stage_store(buf0 + c * kBufBytes);
                stage_store_from(sreg2, buf0 + (c + 1) * kBufBytes);
            }
        }
    } else {
        stage_load(0);
#pragma unroll
        for (int i = 0; i < RING; i++) load_slot(ring[i], i);
        stage_store(buf0);
    }
    __syncthreads();

    float acc[GPW][4], total[GPW][4];
#pragma unroll
    for (int g = 0; g < GPW; g++)
#pragma unroll
        for (int j = 0; j < 4; j++) acc[g][j] = total[g][j] = 0.0f;
    int part = 0;                                            // index of the K-split part being accumulated
    int next_cut = a.ksplit <= 1 ? n_sb : n_sb / a.ksplit;  // first super-block of part 1

    // One super-block of this wave's tile against its token block.
    auto step = [&](const MfmaWeights &w0, int sb, const uint8_t *buf, int slab) __attribute__((always_inline)) {
        const uint8_t *slot = buf + slab * (NTOK * kSlabRow);
        // run sums of this wave's first token group: token n's runs 4 * kq .. + 3
        const _Float16 *runs = reinterpret_cast<const _Float16 *>(buf + kActBytes) + (slab * NTOK + tb * (16 * GPW) + n) * 16 + 4 * kq;
        if (SPLIT && sb == next_cut) {  // the matvec kernel's K-split point: close the partial chain
#pragma unroll
            for (int g = 0; g < GPW; g++)
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    total[g][j] = (part == 0) ? acc[g][j] : total[g][j] + acc[g][j];
                    acc[g][j] = 0.0f;
                }
            part++;
            next_cut = (part + 1) * n_sb / a.ksplit;
        }
        // Several token groups per wave (see below): the first group's activation operands are requested
        // from LDS before the nibbles are unpacked.
        constexpr bool kPipelined = GPW == 2;  // four groups per wave: measured slower than the compiler's own order (19.1 -> 20.6 us at 64 tokens)
        v4i av[kPipelined ? 2 : 1][4];
        auto load_a = [&](v4i (&dst)[4], int g) __attribute__((always_inline)) {
            const uint8_t *ybase = slot + (tb * GPW + g) * (16 * kSlabRow) + a_off;
#pragma unroll
            for (int c = 0; c < 4; c++) dst[c] = *reinterpret_cast<const v4i *>(ybase + 128 * (c >> 1) + 32 * (c & 1));
        };
        if constexpr (kPipelined) {
            load_a(av[0], 0);
            __builtin_amdgcn_sched_barrier(0);
        }
        // this row's scales and mins of the sub-blocks {2half, 2half+1, 4+2half, 5+2half}
        // (reference q4_k_scale_min, src/tensor/mod.rs:5997-6006)
        uint32_t sc03, sc47, m03, m47;
        q4k_unpack_scales(w0.hdr.y, w0.hdr.z, w0.hdr.w, sc03, sc47, m03, m47);
        const float dw = f16_bits_to_f32(w0.hdr.x & 0xffffu);
        const float dminw = f16_bits_to_f32(w0.hdr.x >> 16);
        v4i blo[4], bhi[4], bm[kF16P ? 1 : 4];  // step c = 2 * q + plane
        const v4h bp = q4k_min_operand(m03, m47, kq);
#pragma unroll
        for (int q = 0; q < 2; q++) {
            uint32_t lo2[2], hi2[2];
            q4k_digit_words((q ? sc47 : sc03) >> sc_shift, lo2, hi2);
            const uint4 &pc = w0.piece[q];
#pragma unroll
            for (int plane = 0; plane < 2; plane++) {  // low nibbles = sub-block 2 * ch, high = 2 * ch + 1
                const int c = 2 * q + plane;
                const uint32_t n0 = (pc.x >> (4 * plane)) & 0x0f0f0f0fu, n1 = (pc.y >> (4 * plane)) & 0x0f0f0f0fu;
                const uint32_t n2 = (pc.z >> (4 * plane)) & 0x0f0f0f0fu, n3 = (pc.w >> (4 * plane)) & 0x0f0f0f0fu;
                blo[c] = v4i{scale_bytes(n0, lo2[plane]), scale_bytes(n1, lo2[plane]), scale_bytes(n2, lo2[plane]), scale_bytes(n3, lo2[plane])};
                bhi[c] = v4i{scale_bytes(n0, hi2[plane]), scale_bytes(n1, hi2[plane]), scale_bytes(n2, hi2[plane]), scale_bytes(n3, hi2[plane])};
                if constexpr (!kF16P) {  // the sub-block's min in all 16 bytes: P as a third int8 contraction
                    const uint32_t m = (((q ? m47 : m03) >> sc_shift) >> (8 * plane)) & 0xff;
                    const int m4 = static_cast<int>(__builtin_amdgcn_perm(m, m, 0u));
                    bm[c] = v4i{m4, m4, m4, m4};
                }
            }
        }
        auto min_sums = [&](int g) __attribute__((always_inline)) -> v4f {  // P of token group g, exact (see q4k_min_operand)
            return __builtin_amdgcn_mfma_f32_16x16x16f16(*reinterpret_cast<const v4h *>(runs + g * (16 * 16)), bp, v4f{0.0f, 0.0f, 0.0f, 0.0f}, 0, 0, 0);
        };
        const float *ydp = yds + sb * NTOK + tb * (16 * GPW) + cell_tok;
        if constexpr (kPipelined) {
            // Several token groups per wave, and nothing else on the SIMD to cover a wait: the group loop
            // is pipelined by hand.  The activation operands of group g + 1 are read from LDS before the
            // matrix instructions of group g are issued, and the f32 chains of group g run behind the
            // matrix instructions of group g + 1 -- so an LDS round trip or a matrix result is never
            // waited for with an idle wave.  Two groups per wave: 14336 x 4096, 32 tokens 14.5 -> 13.8 us; 4096 x 14336, 32 tokens
            // 20.1 -> 19.2 us, 64 tokens 27.8 -> 27.4 us.
            v4i Slo[2], Shi[2];
            v4f P[2];
            auto chain = [&](int g) __attribute__((always_inline)) {
                const float4 ydv = *reinterpret_cast<const float4 *>(ydp + 16 * g);
                const float yv[4] = {ydv.x, ydv.y, ydv.z, ydv.w};
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    const int s_cell = Slo[g & 1][j] + 8 * Shi[g & 1][j];
                    const float Dd = yv[j] * dw;
                    const float Mm = yv[j] * dminw;
                    acc[g][j] = __builtin_fmaf(-Mm, P[g & 1][j], acc[g][j]);
                    acc[g][j] = __builtin_fmaf(Dd, static_cast<float>(s_cell), acc[g][j]);
                }
            };
#pragma unroll
            for (int g = 0; g < GPW; g++) {
                if (g + 1 < GPW) load_a(av[(g + 1) & 1], g + 1);
                __builtin_amdgcn_sched_barrier(0);
                Slo[g & 1] = v4i{0, 0, 0, 0};
                Shi[g & 1] = v4i{0, 0, 0, 0};
                v4i Pi = {0, 0, 0, 0};
                if constexpr (kF16P) P[g & 1] = min_sums(g);
#pragma unroll
                for (int c = 0; c < 4; c++) {
                    Slo[g & 1] = __builtin_amdgcn_mfma_i32_16x16x64_i8(av[g & 1][c], blo[c], Slo[g & 1], 0, 0, 0);
                    Shi[g & 1] = __builtin_amdgcn_mfma_i32_16x16x64_i8(av[g & 1][c], bhi[c], Shi[g & 1], 0, 0, 0);
                    if constexpr (!kF16P) Pi = __builtin_amdgcn_mfma_i32_16x16x64_i8(av[g & 1][c], bm[c], Pi, 0, 0, 0);
                }
                if constexpr (!kF16P) P[g & 1] = v4f{static_cast<float>(Pi[0]), static_cast<float>(Pi[1]), static_cast<float>(Pi[2]), static_cast<float>(Pi[3])};
                if (g > 0) chain(g - 1);
                __builtin_amdgcn_sched_barrier(0);
            }
            chain(GPW - 1);
        } else {
#pragma unroll
            for (int g = 0; g < GPW; g++) {
                load_a(av[0], g);
                v4i Slo = {0, 0, 0, 0}, Shi = {0, 0, 0, 0}, Pi = {0, 0, 0, 0};
                v4f P;
                if constexpr (kF16P) P = min_sums(g);
#pragma unroll
                for (int c = 0; c < 4; c++) {
                    Slo = __builtin_amdgcn_mfma_i32_16x16x64_i8(av[0][c], blo[c], Slo, 0, 0, 0);
                    Shi = __builtin_amdgcn_mfma_i32_16x16x64_i8(av[0][c], bhi[c], Shi, 0, 0, 0);
                    if constexpr (!kF16P) Pi = __builtin_amdgcn_mfma_i32_16x16x64_i8(av[0][c], bm[c], Pi, 0, 0, 0);
                }
                if constexpr (!kF16P) P = v4f{static_cast<float>(Pi[0]), static_cast<float>(Pi[1]), static_cast<float>(Pi[2]), static_cast<float>(Pi[3])};
                const float4 ydv = *reinterpret_cast<const float4 *>(ydp + 16 * g);
                const float yv[4] = {ydv.x, ydv.y, ydv.z, ydv.w};
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    const int s_cell = Slo[j] + 8 * Shi[j];
                    const float Dd = yv[j] * dw;
                    const float Mm = yv[j] * dminw;
                    acc[g][j] = __builtin_fmaf(-Mm, P[j], acc[g][j]);
                    acc[g][j] = __builtin_fmaf(Dd, static_cast<float>(s_cell), acc[g][j]);
                }
            }
        }
    };

    // Rounds of RING super-blocks, phases of KC inside them.  Order of issue at a
    // phase start: the next phase's activation loads (L2 hits) first, so that the
    // stores closing the phase never wait behind younger weight loads (vmcnt is in
    // order).  They are unconditional -- the last phase re-reads clamped
    // super-blocks into the idle buffer -- which keeps everything straight-line.
    // Every round but the last refills the ring; the last one only drains it, so
    // no weight is fetched twice when the row length is a multiple of RING.
    uint8_t *cur = buf0, *nxt = buf1;
    auto round = [&](int l0, auto refill) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < RING; i++) {
            const int loc = l0 + i;
            if (i % KC == 0) {
                stage_load(loc + KC);
                __builtin_amdgcn_sched_barrier(0);
            }
            if (loc < n_loc) step(ring[i], s_begin + loc, cur, ks * KC + i % KC);
            // many-token steps fill the register file on their own: keep the scheduler from
            // overlapping two of them (measured: it spills and loses more than it hides)
            if constexpr (GPW > 1) __builtin_amdgcn_sched_barrier(0);
            if constexpr (decltype(refill)::value) load_slot(ring[i], loc + RING);
            if (i % KC == KC - 1) {
                stage_store(nxt);
                __syncthreads();  // next phase complete in `nxt`, everyone done with `cur`
                uint8_t *t = cur;
                cur = nxt;
                nxt = t;
            }
        }
    };
    // the cells of the unit just walked: tokens cell_tok .. + 3 of each group, weight row `row`
    auto store_cells = [&]() __attribute__((always_inline)) {
        if (tile < n_tiles && row >= 0 && row < a.rows) {
#pragma unroll
            for (int g = 0; g < GPW; g++)
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    const int t = tb * (16 * GPW) + 16 * g + cell_tok + j;
                    if (t < n_here) {
                        const float v = (part == 0) ? acc[g][j] : total[g][j] + acc[g][j];
                        (second ? a.out2 : a.out)[static_cast<int64_t>(a0 + tok0 + t) * a.rows + row] = v;
                    }
                }
        }
    };
    if constexpr (ONCE) {
        // One walk over the super-blocks of all of this workgroup's units: the ring is refilled across the unit
        // boundaries, so the activation is staged and the stream started once per workgroup, not once per unit.
        // Slab s of the row sits in chunk s / KC.
        const int walk = n_units * n_sb;
        int sb = 0, unit = 0;
        // The chains advance inside their step: their only reader is the conditional store that closes a unit, and
        // without this the compiler sinks the fused steps of a whole round into that block -- every step's integers
        // stay live (spilled to the accumulation registers) and the dependent chains run where nothing overlaps them.
        auto pin_chains = [&]() __attribute__((always_inline)) {
#pragma unroll
            for (int g = 0; g < GPW; g++)
#pragma unroll
                for (int j = 0; j < 4; j++) asm volatile("" : "+v"(acc[g][j]));
        };
        auto walk_step = [&](const MfmaWeights &w0) __attribute__((always_inline)) {
            step(w0, sb, buf0 + (sb / KC) * kBufBytes, sb % KC);
            pin_chains();
            // (no barrier between steps here: without this fence the scheduler interleaves several steps
            // and needs more registers than two waves per SIMD leave)
            __builtin_amdgcn_sched_barrier(0);
        };
        auto close_unit = [&]() __attribute__((always_inline)) {
            if (++sb == n_sb) {  // the unit's rows are complete
                store_cells();
                sb = 0;
                ++unit;
                const int u = u0 + unit * ustride;
                second = pair && u >= units_per_w;
                tile = (u - (second ? units_per_w : 0)) * RT + rt;
                row = tile * 16 + n - a.row_skip;
                part = 0;
                next_cut = a.ksplit <= 1 ? n_sb : n_sb / a.ksplit;
#pragma unroll
                for (int g = 0; g < GPW; g++)
#pragma unroll
                    for (int j = 0; j < 4; j++) acc[g][j] = total[g][j] = 0.0f;
            }
        };
        if constexpr (NSB > 0) {
            // Rows of NSB super-blocks: the walk of a unit is straight-line code (slab addresses and ring slots known
            // at compile time); step s requests step s + RING, which for the last RING steps lies in the next unit.
            for (int k = 0; k < n_units; ++k) {
                auto fixed_step = [&](int s0) __attribute__((always_inline)) {
                    step(ring[s0 % RING], s0, buf0 + (s0 / KC) * kBufBytes, s0 % KC);
                    pin_chains();
                    __builtin_amdgcn_sched_barrier(0);
                };
#pragma unroll
                for (int s0 = 0; s0 < NSB - RING; s0++) {
                    fixed_step(s0);
                    mfma_load_weights<true>(ring[s0 % RING], w_hdr, w_piece, (s0 + RING) * a.sb_stride);
                }
                // The last RING steps request the next unit's first super-blocks.  After the last unit the requests
                // still go out -- every lane to the weight's first bytes, one cache line -- rather than sit in a
                // branch of their own: two arms with the same steps are merged above the branch by the compiler,
                // and with them the waits for all of the arm's ring slots (four steps' data awaited at once).
                const bool more = k + 1 < n_units;
                int64_t next_stride = 0;
                if (more) {
                    const int u = u0 + (k + 1) * ustride;
                    const bool s2 = pair && u >= units_per_w;
                    const uint8_t *wt = tile_entry(s2, (u - (s2 ? units_per_w : 0)) * RT + rt);
                    w_hdr = wt + hdr_off;
                    w_piece = wt + piece_off;
                    next_stride = a.sb_stride;
                } else {
                    w_hdr = w_piece = a.w;
                }
#pragma unroll
                for (int s0 = NSB - RING; s0 < NSB; s0++) {
                    fixed_step(s0);
                    mfma_load_weights<true>(ring[s0 % RING], w_hdr, w_piece, (s0 + RING - NSB) * next_stride);
                }
                sb = NSB - 1;
                close_unit();
            }
            return;
        }
        // Every round but the last refills the ring, all of its steps lie inside the walk; the last one only drains it.
        int l0 = 0;
        for (; l0 + RING < walk; l0 += RING) {
#pragma unroll
            for (int i = 0; i < RING; i++) {
                walk_step(ring[i]);
                request_next(ring[i]);
                close_unit();
            }
        }
#pragma unroll
        for (int i = 0; i < RING; i++) {
            if (l0 + i < walk) {
                walk_step(ring[i]);
                close_unit();
            }
        }
        return;
    }
    int l0 = 0;
    for (; l0 + RING < n_max; l0 += RING) round(l0, std::true_type{});
    round(l0, std::false_type{});

    if constexpr (KS > 1) {
        // The partial chains of a tile's KS waves, added left to right as the matvec kernel adds
        // them.  Every wave has passed the barrier that closed the last phase: the buffers are free.
        float *red = reinterpret_cast<float *>(buf0);  // [wave][g][j][lane]
#pragma unroll
        for (int g = 0; g < GPW; g++)
#pragma unroll
            for (int j = 0; j < 4; j++) red[((wave * GPW + g) * 4 + j) * 64 + lane] = acc[g][j];
        __syncthreads();
        if (ks != 0) return;
#pragma unroll
        for (int g = 0; g < GPW; g++)
#pragma unroll
            for (int j = 0; j < 4; j++) {
                float v = acc[g][j];
#pragma unroll
                for (int kp = 1; kp < KS; kp++) v = v + red[(((wave + kp) * GPW + g) * 4 + j) * 64 + lane];
                acc[g][j] = v;
            }
    }

    store_cells();
}

int q4k_ksplit_for(int64_t rows, int64_t n_sb);  // gemv_q4k.hip: the matvec kernel's K-split policy

// ---- up to 16 tokens, rows of up to 16 super-blocks: two waves per row tile ------------------------
//
// With one wave per row tile a 14336 x 4096 weight is 896 waves -- fewer than the chip has SIMDs,
// each alone on its SIMD, so nothing runs while a wave waits for memory or for its own matrix-core
// results.  Here two waves share a row tile and split K at `s_mid`; the reference's chain over the
// super-blocks of a row stays ONE chain, in order.  The first wave chains its super-blocks as the
// kernel above does.  The second cannot start its chain before the first has ended, but
// everything of a step that does not depend on the running sum it does at once: the exact
// integers (P, S) from the matrix cores, their conversion, the products yd * d and yd * dmin --
// the four operands of the two fused steps per super-block and cell, kept in registers.  After
// one barrier it takes the first wave's sums from LDS and runs the chain itself: sixteen dependent
// operations per cell.  Same integers, same f32 operations in the same order as the kernel
// above: bit for bit.
// The whole quantized activation (16 tokens x 4096 values) is staged once, before the only other
// barrier; a workgroup is 8 waves = 4 row tiles, one per compute unit.  Each lane loads only the
// nibble bytes it contracts itself (3 KB of requests per 2304-byte tile entry instead of 5 KB).
// Measured at 14336 x 4096, cache-cold, us per launch: 16 tokens 11.7 -> 10.3, 4 tokens 11.4 -> 9.9.
// Where the time goes (per-wave time stamps, medians): activation staged and first weights in at
// 2.7 us, eight steps of 0.5-1.0 us (the first four wait for memory: all of a wave's first half
// is requested at once), 0.9 us at the barrier for the slowest wave of the workgroup, then the
// chain, the store and the end of the launch.  (Parking the second wave's integers in LDS and
// splitting the rest of the chain between both waves measured the same 10.3 us with more code.)
struct Q4KMfmaPairArgs {
    const uint8_t *w;   // tiled layout [super-block][tile][2304 B]
    int64_t sb_stride;
    int rows, n_sb, row_skip;
    const int8_t *q;    // [n_tokens][n_sb*256]
    const float *yd;    // [n_tokens][n_sb]
    const float *x;     // FUSEQ: the f32 activation rows [n_tokens][n_sb*256] instead of q / yd
    float *out;         // [n_tokens][rows]
    int n_tokens;
    int s_mid;          // the first wave of a tile walks super-blocks [0, s_mid), the second [s_mid, n_sb); both at most 8
};

constexpr int kPairSb = 16;    // most super-blocks per row
constexpr int kPairPart = 8;   // most super-blocks per wave
constexpr int kPairTiles = 4;  // row tiles per workgroup
constexpr size_t kPairLds = static_cast<size_t>(kPairSb) * 16 * kSlabRow + kPairSb * 16 * 4 + kPairTiles * 64 * 16 + kPairSb * 16 * 32;

// FUSEQ (a few tokens): the f32 activation is quantized to Q8_K by the workgroup itself, a 16-lane
// row per (token, super-block) with the device function the quantizer launch uses -- the same bytes
// and scales, one launch fewer.  All f32 loads go out before the weight requests.  Every workgroup
// repeats the work, about 0.45 us per token, against 2.4 us for the launch it replaces (14336 x 4096,
// us per step: 3 tokens 12.3 -> 10.5, 4 tokens 12.4 -> 11.0, 8 tokens 12.6 -> 12.9): used up to 6.
template <bool FUSEQ>
__global__ __launch_bounds__(512) void gemm_q4k_mfma_pair_kernel(Q4KMfmaPairArgs a) {
    extern __shared__ uint4 smem[];
    uint8_t *act = reinterpret_cast<uint8_t *>(smem);                            // [kPairSb][16 tokens][kSlabRow]
    float *yds = reinterpret_cast<float *>(act + kPairSb * 16 * kSlabRow);        // [kPairSb][16 tokens]
    float4 *handoff = reinterpret_cast<float4 *>(yds + kPairSb * 16);             // [tile][lane]: the first wave's four chains
    _Float16 *runs = reinterpret_cast<_Float16 *>(handoff + kPairTiles * 64);     // [kPairSb][16 tokens][16]: sums of the 16-value runs

    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
    const int rt = wave >> 1, kd = wave & 1;
    const int n_sb = a.n_sb;
    const int n = lane & 15, kq = lane >> 4, half = kq >> 1;
    const int s_begin = kd ? a.s_mid : 0;
    const int n_loc = kd ? n_sb - a.s_mid : a.s_mid;
    const int n_tiles = (a.rows + a.row_skip + 15) / 16;
    const int tile = blockIdx.x * kPairTiles + rt;
    const int row = tile * 16 + n - a.row_skip;
    const int tok0 = blockIdx.y * 16;
    const int n_here = min(16, a.n_tokens - tok0);
    const uint8_t *wtile = a.w + static_cast<int64_t>(min(tile, n_tiles - 1)) * 2304;
    auto act_row = [&](int t) __attribute__((always_inline)) -> int64_t { return tok0 + min(t, n_here - 1); };

    // The activation first (cache hits, and the stores below then never wait behind a weight load:
    // loads return in order), then the first four super-blocks of this wave's weight.  (Holding three
    // of the four back until the activation is stored gains nothing: the weights then leave later.)
    v4i sreg[8];
    float yd_mine = 0.0f;
    // FUSEQ: block b = 16 * token + super-block; pass p of wave w quantizes blocks 4 * (w + 8 * p) .. + 3
    constexpr int kQuantPasses = 4;
    float4 xv[FUSEQ ? kQuantPasses : 1][4];
    const int qrow = lane >> 4, ql = lane & 15;
    const int n_blk = 16 * n_here;
    if constexpr (FUSEQ) {
        const float4 *x4 = reinterpret_cast<const float4 *>(a.x);
#pragma unroll
        for (int p = 0; p < kQuantPasses; p++) {
            if (4 * (wave + 8 * p) < n_blk) {  // wave-uniform
                const int b = 4 * (wave + 8 * p) + qrow;
                const int64_t t = tok0 + min(b >> 4, n_here - 1);
                const int sb = min(b & 15, n_sb - 1);
#pragma unroll
                for (int k = 0; k < 4; k++) xv[p][k] = x4[(t * n_sb + sb) * 64 + ql * 4 + k];
            }
        }
    } else {
#pragma unroll
        for (int k = 0; k < 8; k++) {
            const int i = tid + k * 512;
            const int sb = min(i >> 8, n_sb - 1), t = (i >> 4) & 15, piece = i & 15;
            sreg[k] = *reinterpret_cast<const v4i *>(a.q + (act_row(t) * n_sb + sb) * 256 + piece * 16);
        }
        if (tid < 256) yd_mine = a.yd[act_row(tid & 15) * n_sb + min(tid >> 4, n_sb - 1)];
    }

    // Lane (n, kq) supplies row n of the tile at k = 16 * kq .. + 15 of every matrix-core step.  A
    // step contracts 64 values of ONE nibble plane: the low (or the high) nibbles of two 32-byte
    // chunks, ch = 2 * q + half for q = 0, 1 -- so the lane needs the 16 bytes of piece (kq & 1) of
    // those two chunks only, both nibbles of every byte it loads are its own, and the 64 lanes of a
    // load cover 1024 distinct bytes of the tile.
    const uint8_t *w_hdr = wtile + n * 16;
    const uint8_t *w_piece = wtile + ((kq & 1) ? 1280 : 256) + n * 64 + half * 16;
    const int sc_shift = 16 * half;                       // scales of sub-blocks 2 * half, 2 * half + 1 (and + 4) within their words
    const int a_off = n * kSlabRow + 64 * half + 16 * (kq & 1);  // + 128 * q + 32 * nibble plane
    const int cell_tok = 4 * kq;
    struct Slot {
        uint4 hdr, piece[2];
    };
    Slot ring[4];
    auto load_slot = [&](Slot &r, int loc) __attribute__((always_inline)) {
        const int64_t off = min(s_begin + loc, n_sb - 1) * a.sb_stride;
        r.hdr = ldg16(w_hdr + off);
        r.piece[0] = ldg16(w_piece + off);
        r.piece[1] = ldg16(w_piece + off + 32);
    };
#pragma unroll
    for (int i = 0; i < 4; i++) load_slot(ring[i], i);
    __builtin_amdgcn_sched_barrier(0);
    if constexpr (FUSEQ) {
        // rows of tokens past n_here stay unwritten: their cells are never stored
#pragma unroll
        for (int p = 0; p < kQuantPasses; p++) {
            if (4 * (wave + 8 * p) < n_blk) {
                const int b = 4 * (wave + 8 * p) + qrow;
                float dv;
                int bs;
                const uint4 packed = q8k_quantize_row16(xv[p], lane, dv, bs);
                const int t = b >> 4, sb = b & 15;
                if (t < n_here && sb < n_sb) {
                    *reinterpret_cast<uint4 *>(act + (sb * 16 + t) * kSlabRow + ql * 16) = packed;
                    runs[(sb * 16 + t) * 16 + ql] = run_sum_f16(packed);
                    if (ql == 0) yds[sb * 16 + t] = dv;
                }
            }
        }
    } else {
#pragma unroll
        for (int k = 0; k < 8; k++) {
            const int i = tid + k * 512;  // slots past n_sb receive a copy of the last super-block; nobody reads them
            *reinterpret_cast<v4i *>(act + ((i >> 8) * 16 + ((i >> 4) & 15)) * kSlabRow + (i & 15) * 16) = sreg[k];
            runs[i] = run_sum_f16(make_uint4(sreg[k][0], sreg[k][1], sreg[k][2], sreg[k][3]));  // i = (sb * 16 + token) * 16 + piece
        }
        if (tid < 256) yds[tid] = yd_mine;
    }
    __syncthreads();

    // Cell j of this lane: token 4 * kq + j of the tile's row n.
    float acc[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    // The second wave cannot chain yet (its chain starts where the first wave's ends), but everything
    // of a step that does not depend on the running sum can be done now: it keeps, per super-block
    // and cell, the four operands of the two fused steps.  What is left for after the barrier is
    // the chain itself, sixteen dependent operations per cell.
    float keep[kPairPart][4][4];  // {-(yd * dmin), float(P), yd * d, float(S)}

#pragma unroll
    for (int i = 0; i < kPairPart; i++) {
        if (i < n_loc) {
            const Slot &w0 = ring[i & 3];
            const int sb = s_begin + i;
            uint32_t sc03, sc47, m03, m47;
            q4k_unpack_scales(w0.hdr.y, w0.hdr.z, w0.hdr.w, sc03, sc47, m03, m47);
            const float dw = f16_bits_to_f32(w0.hdr.x & 0xffffu);
            const float dminw = f16_bits_to_f32(w0.hdr.x >> 16);
            const uint8_t *ybase = act + sb * (16 * kSlabRow) + a_off;
            v4i Slo = {0, 0, 0, 0}, Shi = {0, 0, 0, 0};
            const v4f P = __builtin_amdgcn_mfma_f32_16x16x16f16(*reinterpret_cast<const v4h *>(runs + (sb * 16 + n) * 16 + 4 * kq),
                                                                q4k_min_operand(m03, m47, kq), v4f{0.0f, 0.0f, 0.0f, 0.0f}, 0, 0, 0);
#pragma unroll
            for (int q = 0; q < 2; q++) {
                uint32_t lo2[2], hi2[2];
                q4k_digit_words((q ? sc47 : sc03) >> sc_shift, lo2, hi2);
                const uint4 &pc = w0.piece[q];
#pragma unroll
                for (int plane = 0; plane < 2; plane++) {  // low nibbles = sub-block 2 * ch, high = 2 * ch + 1
                    const uint32_t n0 = (pc.x >> (4 * plane)) & 0x0f0f0f0fu, n1 = (pc.y >> (4 * plane)) & 0x0f0f0f0fu;
                    const uint32_t n2 = (pc.z >> (4 * plane)) & 0x0f0f0f0fu, n3 = (pc.w >> (4 * plane)) & 0x0f0f0f0fu;
                    const v4i blo = {scale_bytes(n0, lo2[plane]), scale_bytes(n1, lo2[plane]), scale_bytes(n2, lo2[plane]), scale_bytes(n3, lo2[plane])};
                    const v4i bhi = {scale_bytes(n0, hi2[plane]), scale_bytes(n1, hi2[plane]), scale_bytes(n2, hi2[plane]), scale_bytes(n3, hi2[plane])};
                    const v4i av = *reinterpret_cast<const v4i *>(ybase + 128 * q + 32 * plane);
                    Slo = __builtin_amdgcn_mfma_i32_16x16x64_i8(av, blo, Slo, 0, 0, 0);
                    Shi = __builtin_amdgcn_mfma_i32_16x16x64_i8(av, bhi, Shi, 0, 0, 0);
                }
            }
            const v4i S = Slo + Shi * 8;
            const float4 ydv = *reinterpret_cast<const float4 *>(yds + sb * 16 + cell_tok);
            const float yv[4] = {ydv.x, ydv.y, ydv.z, ydv.w};
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const float Dd = yv[j] * dw;
                const float Mm = yv[j] * dminw;
                if (kd == 0) {
                    acc[j] = __builtin_fmaf(-Mm, P[j], acc[j]);
                    acc[j] = __builtin_fmaf(Dd, static_cast<float>(S[j]), acc[j]);
                } else {
                    keep[i][j][0] = -Mm;
                    keep[i][j][1] = P[j];
                    keep[i][j][2] = Dd;
                    keep[i][j][3] = static_cast<float>(S[j]);
                }
            }
        }
        if (i + 4 < kPairPart) load_slot(ring[i & 3], i + 4);
    }
    // the first wave hands its chains to the second and is done
    if (kd == 0) handoff[rt * 64 + lane] = make_float4(acc[0], acc[1], acc[2], acc[3]);
    __syncthreads();
    if (kd == 0) return;
    {
        const float4 h = handoff[rt * 64 + lane];
        acc[0] = h.x;
        acc[1] = h.y;
        acc[2] = h.z;
        acc[3] = h.w;
    }
#pragma unroll
    for (int i = 0; i < kPairPart; i++) {
        if (i < n_loc) {
#pragma unroll
            for (int j = 0; j < 4; j++) {
                acc[j] = __builtin_fmaf(keep[i][j][0], keep[i][j][1], acc[j]);
                acc[j] = __builtin_fmaf(keep[i][j][2], keep[i][j][3], acc[j]);
            }
        }
    }
    if (tile < n_tiles && row >= 0 && row < a.rows) {
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const int t = cell_tok + j;
            if (t < n_here) a.out[static_cast<int64_t>(tok0 + t) * a.rows + row] = acc[j];
        }
    }
}

template <bool FUSEQ>
static int launch_mfma_pair(const Q4KMfmaArgs &ka, const float *x, hipStream_t st) {
    Q4KMfmaPairArgs pa{};
    pa.w = ka.w;
    pa.sb_stride = ka.sb_stride;
    pa.rows = ka.rows;
    pa.n_sb = ka.n_sb;
    pa.row_skip = ka.row_skip;
    pa.q = ka.q;
    pa.yd = ka.yd;
    pa.x = x;
    pa.out = ka.out;
    pa.n_tokens = ka.n_tokens;
    pa.s_mid = (ka.n_sb + 1) / 2;
    const int n_tiles = (ka.rows + ka.row_skip + 15) / 16;
    static std::atomic<bool> raised{false};  // setting the attribute twice from two threads is harmless
    if (!raised.load(std::memory_order_acquire)) {
        CML_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(&gemm_q4k_mfma_pair_kernel<FUSEQ>),
                                        hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
        raised.store(true, std::memory_order_release);
    }
    const dim3 grid(static_cast<unsigned>((n_tiles + kPairTiles - 1) / kPairTiles), static_cast<unsigned>((ka.n_tokens + 15) / 16));
    hipLaunchKernelGGL(gemm_q4k_mfma_pair_kernel<FUSEQ>, grid, dim3(512), kPairLds, st, pa);
    if constexpr (FUSEQ) CML_COUNT_LAUNCH("q4k.mfma.pair.fused"); else CML_COUNT_LAUNCH("q4k.mfma.pair");
    CML_HIP_TRY(hipGetLastError());
    return CML_OK;
}

// Which plain calls the pair kernel serves: one column of up to 16 tokens against rows of 2..16
// super-blocks that the shape policy does not cut, on weights of up to 16384 rows -- about one of its workgroups
// per compute unit.  A taller weight queues several of them per unit, each staging the whole activation again and
// filling its ring from nothing; there the staged-once kernel walks the weight with one resident workgroup per
// unit (16 tokens, us per step: 24576 x 4096 20.7 -> 17.5, 32000 x 4096 22.4 -> 19.0, 65536 x 4096 41.2 -> 31.5,
// 128256 x 4096 76.4 -> 59.0, 128256 x 2048 51.6 -> 33.5, 151936 x 3584 82.8 -> 71.9; 14336 x 4096 12.4 either way).
static bool mfma_pair_serves(int64_t rows, int64_t n_sb, int64_t n_tokens) {
    return n_tokens <= 16 && n_sb <= kPairSb && n_sb >= 2 && q4k_ksplit_for(rows, n_sb) == 1 &&
           rows <= env_int("CAMELID_HIP_Q4K_MFMA_PAIR_MAX_ROWS", 16384) &&
           env_int("CAMELID_HIP_Q4K_MFMA_SHAPE", 0) == 0 && env_int("CAMELID_HIP_Q4K_MFMA_PAIR", 1);
}

// f32 activations in, 3 to 6 tokens (8 at most by construction): quantize inside the pair kernel.
// Returns -1 when the call is not one this launch serves (the caller then quantizes in a launch of its own).
int launch_gemm_q4k_mfma_f32(const cml_weight *w, const float *x, int64_t n_tokens, float *out, hipStream_t st) {
    const int most = std::min(8, env_int("CAMELID_HIP_FUSED_QUANT_BATCH_MAX", 6));
    if (n_tokens < env_int("CAMELID_HIP_Q4K_MFMA_MIN_TOKENS", 3) || n_tokens > most || w->rows == 0) return -1;
    if (!mfma_pair_serves(w->rows, w->nb, n_tokens)) return -1;
    Q4KMfmaArgs ka{};
    ka.w = w->planes.p[0];
    ka.sb_stride = w->planes.row_stride[0];
    ka.rows = static_cast<int>(w->rows);
    ka.row_skip = w->row_skip;
    ka.n_sb = static_cast<int>(w->nb);
    ka.out = out;
    ka.n_tokens = static_cast<int>(n_tokens);
    return launch_mfma_pair<true>(ka, x, st);
}

// Counter name of a general-kernel instantiation: "q4k.mfma.tile" (one wave per row tile), ".ksplit<KS>" (K parts of a
// tile on KS waves) or ".serial_split" (the K cut walked inside the lane), then the workgroup shape g<token groups per
// wave>t<waves over tokens>, ".grouped" for expert-grouped calls and ".once" where the activation is staged once
// (then ".k<super-blocks per row>" where the walk knows the row length at compile time, ".units" where a workgroup
// walks more than one group of row tiles).
static std::string q4k_mfma_name(int gpw, int tb, bool split, int ks, bool plain, bool once) {
    std::string n = "q4k.mfma.";
    n += ks > 1 ? "ksplit" + std::to_string(ks) : (split ? "serial_split" : "tile");
    n += ".g" + std::to_string(gpw) + "t" + std::to_string(tb);
    if (!plain) n += ".grouped";
    if (once) n += ".once";
    return n;
}

// Staged-once mode (one 16-token group per wave, rows of up to 16 super-blocks): a unit is four row tiles, a
// workgroup walks every gridDim.x-th unit.  Units per workgroup: enough that the whole launch is resident at once,
// two workgroups per compute unit (what the LDS lets a unit hold) -- the staging and the start of the stream are
// paid once per workgroup's share of the weight, and there is no partly filled last round of workgroups (the
// 32-token Mixtral-shaped layer, gate and up in one launch: 3584 workgroups of one unit 178 us per layer, 1792 of
// two 170, 896 of four 178, 512 of seven 165).
template <bool SPLIT, bool PLAIN, int NSB, int GPW = 1>
static int launch_mfma_once(const Q4KMfmaArgs &ka, int n_tiles, int pair_f, int slots, unsigned gy, int64_t columns, size_t lds, hipStream_t st) {
    static std::atomic<bool> raised{false};  // per instantiation: allow more than 64 KB of dynamic LDS once
    if (!raised.load(std::memory_order_acquire)) {
        CML_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(&gemm_q4k_mfma_kernel<GPW, 1, SPLIT, 1, PLAIN, true, NSB>),
                                        hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
        raised.store(true, std::memory_order_release);
    }
    const int64_t units_all = static_cast<int64_t>((n_tiles + 3) / 4) * pair_f;
    int units = env_int("CAMELID_HIP_Q4K_MFMA_UNITS", 0);
    if (units <= 0) {
        // expert groups: two workgroups per compute unit; a plain call: one (128256 x 4096, 16 tokens, 2004 units:
        // 1 / 2 / 4 / 8 / 16 per workgroup 68.5 / 64.8 / 61.4 / 59.0 / 89.6 us; 65536 x 4096: 35.3 / 33.3 / 31.5 / 47.7 / 85.6)
        // (two token groups per wave fill a compute unit's LDS with one workgroup)
        const int64_t resident = (ka.group_offsets && GPW == 1 && NSB <= 16) ? 512 : 256;
        units = static_cast<int>(std::min<int64_t>(16, std::max<int64_t>(1, (units_all * slots * columns + resident - 1) / resident)));
        // the walk that does not know the row length at compile time pays for its bookkeeping beyond two units
        // (151936 x 3584, 16 tokens: 75.2 / 71.9 / 74.2 / 88.7 us for 1 / 2 / 4 / 8)
        if (NSB == 0 && !ka.group_offsets) units = std::min(units, 2);
    }
    units = static_cast<int>(std::min<int64_t>(units, units_all));
    const unsigned gxu = static_cast<unsigned>((units_all + units - 1) / units);
    hipLaunchKernelGGL((gemm_q4k_mfma_kernel<GPW, 1, SPLIT, 1, PLAIN, true, NSB>), dim3(gxu, gy, slots), dim3(256), lds, st, ka);
    // (a counter's name is built once per site: one site per name)
    if (units > 1) CML_COUNT_LAUNCH(q4k_mfma_name(GPW, 1, SPLIT, 1, PLAIN, true) + (NSB ? ".k" + std::to_string(NSB) : "") + ".units");
    else CML_COUNT_LAUNCH(q4k_mfma_name(GPW, 1, SPLIT, 1, PLAIN, true) + (NSB ? ".k" + std::to_string(NSB) : ""));
    CML_HIP_TRY(hipGetLastError());
    return CML_OK;
}

template <int GPW, int TB, bool SPLIT, int KS = 1, bool PLAIN = false>
static int launch_mfma_split(const Q4KMfmaArgs &ka, int n_groups, hipStream_t st) {
    constexpr int NTOK = 16 * GPW * TB, RT = 4 / (TB * KS);
    constexpr int KC = (128 / (NTOK * KS)) > 0 ? 128 / (NTOK * KS) : 1;
    const int n_tiles = (ka.rows + ka.row_skip + 15) / 16;
    const unsigned gx = static_cast<unsigned>((n_tiles + RT - 1) / RT);
    const unsigned gy = static_cast<unsigned>((ka.n_tokens + NTOK - 1) / NTOK);
    const size_t lds = 2 * static_cast<size_t>(KS * KC * NTOK) * (kSlabRow + ((GPW == 2 && KS == 1) ? 32 : 0)) + static_cast<size_t>(ka.n_sb) * NTOK * 4;
    if (lds > 160 * 1024) return fail(CML_ERR_UNSUPPORTED, "Q4_K matrix-core path: %d super-blocks exceed the LDS budget", ka.n_sb);
    if constexpr ((GPW == 1 || GPW == 2) && TB == 1 && KS == 1) {
        // Rows of up to 16 super-blocks: the whole activation fits the LDS and is staged once.  One token group per
        // wave: always.  Two (17 to 32 tokens; 155 KB, one workgroup per compute unit): expert groups, and plain calls
        // on weights of more than 16384 rows, where the launch walks the weight with resident workgroups.
        const bool two_groups_pay = ka.group_offsets != nullptr || n_tiles > env_int("CAMELID_HIP_Q4K_MFMA_ONCE_TWO_GROUPS_MIN_TILES", 1024);
        if (ka.n_sb <= 16 && ka.stage_once && (GPW == 1 || (two_groups_pay && env_int("CAMELID_HIP_Q4K_MFMA_ONCE_TWO_GROUPS", 1)))) {
            const size_t lds_once = static_cast<size_t>(16) * NTOK * (kSlabRow + 32) + static_cast<size_t>(ka.n_sb) * NTOK * 4;  // slabs + run sums, scales
            const int pair_f = ka.w2 ? 2 : 1, slots = n_groups / pair_f;
            const int64_t columns = ka.group_offsets ? 1 : gy;  // (a grouped call counts one token column per group: the others leave at once)
            // rows of 2048, 3072, 3584 or 4096 values: the walk of a unit as straight-line code
            const bool fixed = env_int("CAMELID_HIP_Q4K_MFMA_FIXED_ROWS", 1);
            if (fixed && ka.n_sb == 16) return launch_mfma_once<SPLIT, PLAIN, 16, GPW>(ka, n_tiles, pair_f, slots, gy, columns, lds_once, st);
            if (fixed && ka.n_sb == 14) return launch_mfma_once<SPLIT, PLAIN, 14, GPW>(ka, n_tiles, pair_f, slots, gy, columns, lds_once, st);
            if (fixed && ka.n_sb == 12) return launch_mfma_once<SPLIT, PLAIN, 12, GPW>(ka, n_tiles, pair_f, slots, gy, columns, lds_once, st);
            if (fixed && ka.n_sb == 8) return launch_mfma_once<SPLIT, PLAIN, 8, GPW>(ka, n_tiles, pair_f, slots, gy, columns, lds_once, st);
            return launch_mfma_once<SPLIT, PLAIN, 0, GPW>(ka, n_tiles, pair_f, slots, gy, columns, lds_once, st);
        }
        // Rows of 5120 / 6144 / 8192 values, up to 16 tokens: the same walk with 32 slabs of LDS
        // (one workgroup per compute unit); 128256 x 8192 at 16 tokens 132.9 -> 110.4 us, 152064 x 5120 108.0 -> 88.2, 32000 x 5120 26.9 -> 23.7.
        // (expert groups with such rows as well: gate and up of a Mixtral-8x22B-shaped layer, hidden 6144)
        if constexpr (GPW == 1) {
            // (plain calls: at any row count the shape policy leaves uncut -- 13824 x 5120 at 16 tokens 17.8 -> 15.8 us, 14336 x 8192 24.8 -> 19.6)
            const bool tall_or_grouped = ka.group_offsets != nullptr || n_tiles > env_int("CAMELID_HIP_Q4K_MFMA_ONCE_LONG_MIN_TILES", 0);
            if (ka.stage_once && tall_or_grouped && (ka.n_sb == 20 || ka.n_sb == 24 || ka.n_sb == 32) && env_int("CAMELID_HIP_Q4K_MFMA_ONCE_LONG_ROWS", 1)) {
                const size_t lds_long = static_cast<size_t>(32) * NTOK * (kSlabRow + 32) + static_cast<size_t>(ka.n_sb) * NTOK * 4;
                const int pair_f = ka.w2 ? 2 : 1, slots = n_groups / pair_f;
                const int64_t columns = ka.group_offsets ? 1 : gy;
                if (ka.n_sb == 20) return launch_mfma_once<SPLIT, PLAIN, 20, 1>(ka, n_tiles, pair_f, slots, gy, columns, lds_long, st);
                if (ka.n_sb == 24) return launch_mfma_once<SPLIT, PLAIN, 24, 1>(ka, n_tiles, pair_f, slots, gy, columns, lds_long, st);
                return launch_mfma_once<SPLIT, PLAIN, 32, 1>(ka, n_tiles, pair_f, slots, gy, columns, lds_long, st);
            }
        }
    }
    static std::atomic<bool> raised{false};  // per instantiation: allow more than 64 KB of dynamic LDS once
    if (!raised.load(std::memory_order_acquire)) {
        CML_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(&gemm_q4k_mfma_kernel<GPW, TB, SPLIT, KS, PLAIN>),
                                        hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
        raised.store(true, std::memory_order_release);
    }
    hipLaunchKernelGGL((gemm_q4k_mfma_kernel<GPW, TB, SPLIT, KS, PLAIN>), dim3(gx, gy, n_groups), dim3(256), lds, st, ka);
    CML_COUNT_LAUNCH(q4k_mfma_name(GPW, TB, SPLIT, KS, PLAIN, false));
    CML_HIP_TRY(hipGetLastError());
    return CML_OK;
}

// The K-split bookkeeping inside the lane costs a branch per super-block, so it is compiled in
// only where the matvec kernel splits K for this weight shape and the split is not 2 or 4 (those
// run as 2 or 4 waves per row tile).
// Plain calls (no expert groups) take the kernel entry without the group tables (PLAIN): three
// dependent scalar-load rounds fewer before the first request (14336 x 4096, 16 tokens: 12.2 -> 11.7 us).
template <int GPW, int TB, bool SPLIT, int KS>
static int launch_mfma_entry(const Q4KMfmaArgs &ka, int n_groups, hipStream_t st) {
    if (ka.group_offsets == nullptr && !env_int("CAMELID_HIP_Q4K_MFMA_GENERAL_ENTRY", 0)) return launch_mfma_split<GPW, TB, SPLIT, KS, true>(ka, n_groups, st);
    return launch_mfma_split<GPW, TB, SPLIT, KS, false>(ka, n_groups, st);
}

template <int GPW, int TB>
static int launch_mfma(const Q4KMfmaArgs &ka, int n_groups, hipStream_t st) {
    return ka.ksplit > 1 ? launch_mfma_entry<GPW, TB, true, 1>(ka, n_groups, st) : launch_mfma_entry<GPW, TB, false, 1>(ka, n_groups, st);
}

// Q4_K matmul on the matrix cores: plain calls, or grouped by expert (mixture of experts).
int launch_gemm_q4k_mfma(const MatArgs &a, hipStream_t st) {
    const cml_weight *w = a.w;
    const bool grouped = a.group_offsets != nullptr;
    if (w->rows == 0 || a.n_tokens == 0) return CML_OK;
    Q4KMfmaArgs ka{};
    ka.w = w->planes.p[0];
    ka.sb_stride = w->planes.row_stride[0];
    ka.rows = static_cast<int>(grouped ? a.band_rows : w->rows);
    if (grouped && ((ka.rows % 16) != 0 || w->row_skip != 0))
        return fail(CML_ERR_UNSUPPORTED, "Q4_K expert bands must be whole 16-row tiles (%d rows, first tile offset %d)", ka.rows, w->row_skip);
    ka.row_skip = grouped ? 0 : w->row_skip;
    ka.n_sb = static_cast<int>(w->nb);
    ka.ksplit = q4k_ksplit_for(ka.rows, w->nb);
    ka.q = a.q;
    ka.yd = a.scales;
    ka.out = a.out;
    ka.n_tokens = static_cast<int>(a.n_tokens);
    ka.group_offsets = a.group_offsets;
    ka.group_rows = a.group_rows;
    ka.group_ids = a.group_ids;
    ka.stage_once = env_int("CAMELID_HIP_Q4K_MFMA_STAGE_ONCE", 1);
    if (a.w2) {
        if (!grouped || a.w2->fmt != w->fmt || a.w2->rows != w->rows || a.w2->nb != w->nb || a.w2->row_skip != 0 ||
            a.w2->planes.row_stride[0] != w->planes.row_stride[0])
            return fail(CML_ERR_SHAPE, "the two weights of a pair launch differ in shape");
        ka.w2 = a.w2->planes.p[0];
        ka.out2 = a.out2;
    }
    const int ng = (grouped ? (a.group_ids ? a.max_active : a.n_groups) : 1) * (a.w2 ? 2 : 1);
    // Workgroup shape: tokens staged per workgroup x how they are split over waves.  Default: one
    // wave per row tile, 16 / 32 / 64 tokens per workgroup by batch size; more tokens = more
    // workgroup columns (grid.y), each a pass over the weight.  The other shapes stay selectable
    // for tuning.
    const int shape = env_int("CAMELID_HIP_Q4K_MFMA_SHAPE", 0);
    // One column of up to 16 tokens against rows of up to 16 super-blocks that the shape policy
    // does not cut: two waves per row tile, one chain.
    if (!grouped && mfma_pair_serves(ka.rows, ka.n_sb, a.n_tokens)) return launch_mfma_pair<false>(ka, nullptr, st);
    // K split across waves: 16 or 32 tokens per workgroup, more tokens = more workgroup columns
    // (worth it when the launch has fewer row tiles than the chip has SIMDs; a grouped call with
    // many experts in use fills the chip without it)
    const int64_t launch_tiles = static_cast<int64_t>((ka.rows + ka.row_skip + 15) / 16) * ng;
    if (shape == 0 && launch_tiles < 1024 && !env_int("CAMELID_HIP_Q4K_MFMA_SERIAL_SPLIT", 0)) {
        if (ka.ksplit == 4) return (grouped || a.n_tokens <= 16) ? launch_mfma_entry<1, 1, false, 4>(ka, ng, st) : launch_mfma_entry<2, 1, false, 4>(ka, ng, st);
        if (ka.ksplit == 2) return (grouped || a.n_tokens <= 16) ? launch_mfma_entry<1, 1, false, 2>(ka, ng, st) : launch_mfma_entry<2, 1, false, 2>(ka, ng, st);
    }
    switch (shape) {
        case 1: return launch_mfma<1, 1>(ka, ng, st);   // 16 tokens, 1 wave per row tile
        case 2: return launch_mfma<2, 1>(ka, ng, st);   // 32 tokens, 1 wave per row tile
        case 3: return launch_mfma<4, 1>(ka, ng, st);   // 64 tokens, 1 wave per row tile
        case 4: return launch_mfma<1, 2>(ka, ng, st);   // 32 tokens, 2 waves per row tile
        case 5: return launch_mfma<2, 2>(ka, ng, st);   // 64 tokens, 2 waves per row tile
        case 6: return launch_mfma<1, 4>(ka, ng, st);   // 64 tokens, 4 waves per row tile
        default: break;
    }
    if (grouped) {
        // assignments per expert are few and uneven: the smallest tile wastes least -- until most experts hold more
        // than 16 and a second token column would read their weights a second time
        const int slots = std::max(1, ng / (a.w2 ? 2 : 1));
        if (ka.n_sb <= 16 && a.n_tokens > 16 && a.n_assign_total > 12 * static_cast<int64_t>(slots) && env_int("CAMELID_HIP_Q4K_MFMA_ONCE_TWO_GROUPS", 1))
            return launch_mfma<2, 1>(ka, ng, st);
        return launch_mfma<1, 1>(ka, ng, st);
    }
    if (a.n_tokens > 32) return launch_mfma<4, 1>(ka, ng, st);
    if (a.n_tokens > 16) return launch_mfma<2, 1>(ka, ng, st);
    return launch_mfma<1, 1>(ka, ng, st);
}

}  // namespace cml
