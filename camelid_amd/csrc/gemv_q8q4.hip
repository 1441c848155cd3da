// Q8_0 x Q8_0 and Q4_0 x Q8_0 fused dequantize + matvec / small-batch matmul
// for gfx950.
//
// Arithmetic (reference q8_0_wire_row_dot_scalar, src/inference.rs:22729-22745;
// q4_0_wire_row_dot_scalar, :22778-22798): per 32-value block, in block order,
//     isum = sum_j w_j * x_j                (exact i32; Q4_0 weights are nibble - 8)
//     total = total + ((float)isum * d_w) * d_x
// The kernels keep exactly that association: one f32 chain per row, blocks
// added left to right.
//
// Mapping.  Weights are in the plane layout (quants | f16 scales).  P lanes (8, 16, 32 or 64)
// share a row and take P consecutive blocks per step with aligned 128-bit loads -- Q4_0 one block
// per lane, Q8_0 with P >= 16 two lanes per block (see kB32Paired), Q8_0 with 8 lanes one block per
// lane in two loads -- and the block's scale with a 16-bit load.  The per-block terms are folded
// into the row's accumulator in block order with DPP row_shr reads (the last lane of a 16-lane DPP
// row owns the chain; rows of 32 / 64 lanes hand it from one DPP row to the next).  A wave covers
// 64/P rows, a workgroup 2, 4, 8 or 16 waves.  Activations (int8 + per-block f32 scale, and for
// Q4_0 the per-block sums that carry the -8 bias) are staged once per workgroup in LDS, or
// quantized there from f32 by the workgroup itself (FUSEQ: one or two tokens).
#include <string>

#include "cml_device.hpp"
#include "cml_host.hpp"

#include <algorithm>
#include <type_traits>

#pragma clang fp contract(off)

namespace cml {

struct B32Args {
    const uint8_t *quants;  // plane 0
    int64_t q_stride;       // bytes per row
    const uint8_t *scales;  // plane 1 (f16)
    int64_t s_stride;
    int rows;  // rows of one band
    int nb;    // blocks per row
    const int8_t *q;  // [slot][NT][nb*32]
    const float *xs;  // [slot][NT][nb]
    const float *x;   // f32 activation row [nb*32]: only for the kernel that quantizes it itself
    float *out;
    const float *residual;
    int32_t *ints;  // [rows][nb] or null
    const int32_t *band_ids;
    int64_t act_slot_stride;
    int64_t out_slot_stride;
    int early_loads;  // issue the first weight loads ahead of the fused quantizer
    // PAIR (grid.z = 2): blockIdx.z = 1 works on a second weight of the same shape against the same token
    const uint8_t *quants2;
    const uint8_t *scales2;
    float *out2;
};

// One f32 token against up to four weights of one format and row length (any row counts) in one launch: their
// workgroups lie end to end along grid.x, every workgroup quantizes the token once.
struct B32MultiArgs {
    B32Args base;             // everything the weights share (nb, x, early_loads)
    const uint8_t *quantsm[4];
    const uint8_t *scalesm[4];
    int64_t q_stridem[4], s_stridem[4];
    float *outm[4];
    int rowsm[4];
    int wg_end[4];            // workgroups of weights 0 .. j (INT32_MAX beyond the last weight)
};

template <int FMT, int UU = 2>
struct B32Regs {
    static constexpr int U = UU;  // steps in flight per buffer
    uint4 qa[U];
    uint4 qb[U];  // Q8_0 only
    uint32_t d[U];
};

// Q8_0 rows of P >= 16 lanes ("paired" mapping; written out for P = 16): a step is 16 blocks = 512
// contiguous bytes of the row, and each of the two load instructions takes 256 contiguous bytes of
// it -- lane l the 16 bytes at l*16 and at 256 + l*16 -- so every instruction consumes whole 128-byte lines exactly once (two
// lanes share a block: lanes 2j, 2j+1 hold the halves of block j, then of block 8+j).  The two
// half-block integer sums meet by one lane swap (exact integers: the order inside a block is free);
// the even lane then carries block j's term, the odd lane block 8+j's, and the ordered fold visits
// even lanes first.  The one-block-per-lane mapping had each instruction touch half of every line.
template <int FMT, int P>
inline constexpr bool kB32Paired = (FMT == CML_Q8_0 && P >= 16);

__device__ __forceinline__ int quad_swap1_i32(int v) {  // lanes 2j <-> 2j+1
    return __builtin_amdgcn_update_dpp(0, v, 0xB1, 0xf, 0xf, true);
}

// The block whose term lane l carries in step `s` of a paired row, and the two blocks it loads halves of.
template <int P>
__device__ __forceinline__ int paired_block(int s, int l, int which) { return s * P + which * (P / 2) + (l >> 1); }

// Ordered fold for the paired mapping: terms of lanes 0, 2, .., 14 (blocks 0..7 of the step), then
// of lanes 1, 3, .., 15 (blocks 8..15); lane 15 returns the chain.
template <int K = 0>
__device__ __forceinline__ float paired_fold_ordered(float acc, float term) {
    if constexpr (K == 15) {
        return acc + term;
    } else {
        constexpr int src = (K < 8) ? 2 * K : 2 * (K - 8) + 1;  // lane whose term is the K-th block's
        acc = acc + row_shr_f32<15 - src>(term);
        return paired_fold_ordered<K + 1>(acc, term);
    }
}


// ---- rows wider than one 16-lane DPP row (P = 32 or 64 lanes per matrix row) ----
// For matrices with few, long rows: the block terms are independent, only the chain is ordered, so
// more lanes per row multiply the waves without touching a bit.  The chain runs through the R =
// P / 16 DPP rows of a group one after the other: every DPP row folds its sixteen terms onto the
// running sum (only the row whose turn it is holds the right one), and that row's last lane hands
// the sum to the whole group.  After the last hand-over every lane of the group holds the chain.
template <int P>
__device__ __forceinline__ float wide_carry(float t, int rho) {
    static_assert(P == 32 || P == 64, "lanes per row");
    const int ti = __builtin_bit_cast(int, t);
    if constexpr (P == 64) {
        return __builtin_bit_cast(float, __builtin_amdgcn_readlane(ti, 16 * rho + 15));
    } else {
        const int lo = __builtin_amdgcn_readlane(ti, 16 * rho + 15), hi = __builtin_amdgcn_readlane(ti, 32 + 16 * rho + 15);
        return __builtin_bit_cast(float, (threadIdx.x & 32) ? hi : lo);
    }
}
template <int P>
__device__ __forceinline__ float wide_fold_ordered(float acc, float term) {  // lane l carries block l of the step
#pragma unroll
    for (int rho = 0; rho < P / 16; rho++) acc = wide_carry<P>(group_fold_ordered<16>(acc, term), rho);
    return acc;
}
template <int ODD, int K = 0>
__device__ __forceinline__ float paired_half_fold(float acc, float term) {  // lanes ODD, ODD + 2, .., ODD + 14 of a DPP row
    if constexpr (K == 8) {
        return acc;
    } else {
        constexpr int shift = 15 - (2 * K + ODD);
        if constexpr (shift == 0) acc = acc + term;
        else acc = acc + row_shr_f32<shift>(term);
        return paired_half_fold<ODD, K + 1>(acc, term);
    }
}
template <int P>
__device__ __forceinline__ float wide_paired_fold_ordered(float acc, float term) {  // even lanes: blocks 0..P/2-1, odd lanes: the rest
#pragma unroll
    for (int rho = 0; rho < P / 16; rho++) acc = wide_carry<P>(paired_half_fold<0>(acc, term), rho);
#pragma unroll
    for (int rho = 0; rho < P / 16; rho++) acc = wide_carry<P>(paired_half_fold<1>(acc, term), rho);
    return acc;
}

template <int FMT, int P, int U>
__device__ __forceinline__ void b32_load(B32Regs<FMT, U> &r, const uint8_t *qrow, const uint8_t *srow, int l,
                                         int step, int n_steps, int nb) {
    // Unconditional, clamped loads: steps or lanes past the row end re-read the
    // last block and their term is dropped by the caller.  Straight-line code
    // keeps the next buffer's loads in flight under the current arithmetic.
#pragma unroll
    for (int u = 0; u < U; u++) {
        if constexpr (kB32Paired<FMT, P>) {
            const int s = min(step + u, n_steps - 1);
            const int ba = min(paired_block<P>(s, l, 0), nb - 1), bb = min(paired_block<P>(s, l, 1), nb - 1);
            const int half = (l & 1) * 16;
            r.qa[u] = ldg16_stream(qrow + static_cast<int64_t>(ba) * 32 + half);
            r.qb[u] = ldg16_stream(qrow + static_cast<int64_t>(bb) * 32 + half);
            r.d[u] = ldg2(srow + static_cast<int64_t>((l & 1) ? bb : ba) * 2);
            continue;
        }
        const int b = min(min(step + u, n_steps - 1) * P + l, nb - 1);
        if constexpr (FMT == CML_Q8_0) {
            // two loads per 32-byte block: each touches half of every line, so the lines must
            // stay cached between them (the streaming hint cost 0.25 us at 8192 x 2048)
            r.qa[u] = ldg16(qrow + static_cast<int64_t>(b) * 32);
            r.qb[u] = ldg16(qrow + static_cast<int64_t>(b) * 32 + 16);
        } else if constexpr (P >= 8) {
            // a row's lanes read whole 128-byte lines per step: read-once data
            // (128256 x 3072: 36.9 -> 32.8 us)
            r.qa[u] = ldg16_stream(qrow + static_cast<int64_t>(b) * 16);
        } else {
            r.qa[u] = ldg16(qrow + static_cast<int64_t>(b) * 16);  // 4 lanes: a line lasts two steps
        }
        r.d[u] = ldg2(srow + static_cast<int64_t>(b) * 2);
    }
}

template <int FMT, int P, int NT, bool INTS, int U>
__device__ __forceinline__ void b32_compute(const B32Regs<FMT, U> &r, int l, int step, int n_steps, int nb,
                                            const int8_t *ys, const int *bsum, const float *xss, float (&acc)[NT],
                                            int32_t *ints_row) {
#pragma unroll
    for (int u = 0; u < U; u++) {
        if constexpr (kB32Paired<FMT, P>) {
            const int s = min(step + u, n_steps - 1);
            const int ba = min(paired_block<P>(s, l, 0), nb - 1), bb = min(paired_block<P>(s, l, 1), nb - 1);
            const int odd = l & 1;
            const int b_raw = paired_block<P>(step + u, l, odd);
            const bool valid = (step + u < n_steps) && (b_raw < nb);
            const int b = odd ? bb : ba;
            const float dw = f16_bits_to_f32(r.d[u]);
#pragma unroll
            for (int t = 0; t < NT; t++) {
                const int8_t *y = ys + static_cast<int64_t>(t) * nb * 32 + odd * 16;
                const uint4 ya = *reinterpret_cast<const uint4 *>(y + ba * 32);
                const uint4 yb = *reinterpret_cast<const uint4 *>(y + bb * 32);
                int pa = dot16(r.qa[u], ya, 0), pb = dot16(r.qb[u], yb, 0);
                pa += quad_swap1_i32(pa);
                pb += quad_swap1_i32(pb);
                const int isum = odd ? pb : pa;
                float term = (static_cast<float>(isum) * dw) * xss[t * nb + b];
                term = valid ? term : 0.0f;
                if constexpr (P > 16) acc[t] = wide_paired_fold_ordered<P>(acc[t], term);
                else acc[t] = paired_fold_ordered(acc[t], term);
                if constexpr (INTS) {
                    if (ints_row != nullptr && valid) ints_row[b] = isum;
                }
            }
            continue;
        }
        const int b_raw = (step + u) * P + l;
        const bool valid = (step + u < n_steps) && (b_raw < nb);
        const int b = min(min(step + u, n_steps - 1) * P + l, nb - 1);
        const float dw = f16_bits_to_f32(r.d[u]);
        uint4 w0, w1;
        if constexpr (FMT == CML_Q8_0) {
            w0 = r.qa[u];
            w1 = r.qb[u];
        } else {
            // byte j: low nibble = value j, high nibble = value j+16
            w0 = make_uint4(r.qa[u].x & 0x0f0f0f0fu, r.qa[u].y & 0x0f0f0f0fu, r.qa[u].z & 0x0f0f0f0fu,
                            r.qa[u].w & 0x0f0f0f0fu);
            w1 = make_uint4((r.qa[u].x >> 4) & 0x0f0f0f0fu, (r.qa[u].y >> 4) & 0x0f0f0f0fu,
                            (r.qa[u].z >> 4) & 0x0f0f0f0fu, (r.qa[u].w >> 4) & 0x0f0f0f0fu);
        }
#pragma unroll
        for (int t = 0; t < NT; t++) {
            const int8_t *y = ys + (static_cast<int64_t>(t) * nb + b) * 32;
            const uint4 y0 = *reinterpret_cast<const uint4 *>(y);
            const uint4 y1 = *reinterpret_cast<const uint4 *>(y + 16);
            int isum = dot16(w1, y1, dot16(w0, y0, 0));
            if constexpr (FMT == CML_Q4_0) isum -= 8 * bsum[t * nb + b];
            float term = (static_cast<float>(isum) * dw) * xss[t * nb + b];
            term = valid ? term : 0.0f;
            if constexpr (P > 16) acc[t] = wide_fold_ordered<P>(acc[t], term);
            else acc[t] = group_fold_ordered<P>(acc[t], term);
            if constexpr (INTS) {
                if (ints_row != nullptr && valid) ints_row[b] = isum;
            }
        }
    }
}

// `ra` arrives loaded with steps 0..U-1 (b32_load) -- the caller may have issued those loads well
// before, e.g. ahead of its prologue.
template <int FMT, int P, int NT, bool INTS, int U = 2>
__device__ __forceinline__ void b32_row_pass_from(B32Regs<FMT, U> &ra, const uint8_t *qrow, const uint8_t *srow, int l, int nb,
                                                  const int8_t *ys, const int *bsum, const float *xss, float (&acc)[NT],
                                                  int32_t *ints_row) {
    const int n_steps = (nb + P - 1) / P;
    B32Regs<FMT, U> rb;
    for (int step = 0;;) {
        if (step + U >= n_steps) {
            b32_compute<FMT, P, NT, INTS, U>(ra, l, step, n_steps, nb, ys, bsum, xss, acc, ints_row);
            break;
        }
        b32_load<FMT, P, U>(rb, qrow, srow, l, step + U, n_steps, nb);
        __builtin_amdgcn_sched_barrier(0);
        b32_compute<FMT, P, NT, INTS, U>(ra, l, step, n_steps, nb, ys, bsum, xss, acc, ints_row);
        __builtin_amdgcn_sched_barrier(0);
        step += U;
        if (step + U >= n_steps) {
            b32_compute<FMT, P, NT, INTS, U>(rb, l, step, n_steps, nb, ys, bsum, xss, acc, ints_row);
            break;
        }
        b32_load<FMT, P, U>(ra, qrow, srow, l, step + U, n_steps, nb);
        __builtin_amdgcn_sched_barrier(0);
        b32_compute<FMT, P, NT, INTS, U>(rb, l, step, n_steps, nb, ys, bsum, xss, acc, ints_row);
        __builtin_amdgcn_sched_barrier(0);
        step += U;
    }
}

// One pass over a row's blocks for NT staged activation rows: two register buffers alternate,
// the last one is consumed without issuing further loads.
template <int FMT, int P, int NT, bool INTS, int U = 2>
__device__ __forceinline__ void b32_row_pass(const uint8_t *qrow, const uint8_t *srow, int l, int nb, const int8_t *ys,
                                             const int *bsum, const float *xss, float (&acc)[NT], int32_t *ints_row) {
    const int n_steps = (nb + P - 1) / P;
    B32Regs<FMT, U> ra;
    b32_load<FMT, P, U>(ra, qrow, srow, l, 0, n_steps, nb);
    __builtin_amdgcn_sched_barrier(0);
    b32_row_pass_from<FMT, P, NT, INTS, U>(ra, qrow, srow, l, nb, ys, bsum, xss, acc, ints_row);
}

// The same pass through a ring of NB one-step buffers: a slot is requested again after ONE step's
// arithmetic, so the wave's requests in flight never drop to half as they do between two U-step
// buffers.  `ring[0..PRE-1]` arrive loaded with steps 0..PRE-1; n_steps >= NB (the launcher checks).
// Whole turns run in a loop, the last NB..2NB-1 steps are straight-line code per remainder so
// that every wait counts exactly the loads behind the buffer it needs.
template <int FMT, int P, int NT, int NB, int PRE>
__device__ __forceinline__ void b32_row_pass_ring(B32Regs<FMT, 1> (&ring)[NB], const uint8_t *qrow, const uint8_t *srow, int l, int nb,
                                                  const int8_t *ys, const int *bsum, const float *xss, float (&acc)[NT]) {
    const int n = (nb + P - 1) / P;
    auto compute = [&](const B32Regs<FMT, 1> &b, int step) __attribute__((always_inline)) {
        b32_compute<FMT, P, NT, false, 1>(b, l, step, n, nb, ys, bsum, xss, acc, nullptr);
        __builtin_amdgcn_sched_barrier(0);
    };
    auto request = [&](B32Regs<FMT, 1> &b, int step) __attribute__((always_inline)) {
        b32_load<FMT, P, 1>(b, qrow, srow, l, step, n, nb);
        __builtin_amdgcn_sched_barrier(0);
    };
#pragma unroll
    for (int j = PRE; j < NB; j++) request(ring[j], j);
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

// FUSEQ (single token): the activation arrives as f32 and every workgroup quantizes it to Q8_0
// itself, eight lanes per block, straight into the LDS staging area -- the arithmetic of
// quantize_q8_0_kernel without the launch and the round trip through memory.
template <int FMT, int P, int NT, bool INTS, bool FUSEQ = false, int WAVES = 4, int NXQ = 0, int U = 2, int RING = 0, bool PAIR = false, bool MULTI = false>
__global__ __launch_bounds__(WAVES * 64) void gemv_b32_kernel(std::conditional_t<MULTI, B32MultiArgs, B32Args> a_in) {
    static_assert(!PAIR || (FUSEQ && NT == 1 && !INTS), "a pair: one f32 token against two weights of one shape");
    static_assert(!MULTI || (FUSEQ && NT == 1 && !INTS && !PAIR), "a multi launch: one f32 token against several weights");
    B32Args a_sel;        // MULTI: the shared arguments with this workgroup's weight filled in
    int bx = blockIdx.x;  // workgroup index within its weight
    if constexpr (MULTI) {
        B32Args &a = a_sel;
        a = a_in.base;
        // which weight this workgroup belongs to (wave-uniform selects: no indexed access to the argument block)
        const int j = (bx >= a_in.wg_end[0]) + (bx >= a_in.wg_end[1]) + (bx >= a_in.wg_end[2]);
        auto pick = [&](auto v0, auto v1, auto v2, auto v3) { return j == 0 ? v0 : (j == 1 ? v1 : (j == 2 ? v2 : v3)); };
        a.quants = pick(a_in.quantsm[0], a_in.quantsm[1], a_in.quantsm[2], a_in.quantsm[3]);
        a.scales = pick(a_in.scalesm[0], a_in.scalesm[1], a_in.scalesm[2], a_in.scalesm[3]);
        a.q_stride = pick(a_in.q_stridem[0], a_in.q_stridem[1], a_in.q_stridem[2], a_in.q_stridem[3]);
        a.s_stride = pick(a_in.s_stridem[0], a_in.s_stridem[1], a_in.s_stridem[2], a_in.s_stridem[3]);
        a.out = pick(a_in.outm[0], a_in.outm[1], a_in.outm[2], a_in.outm[3]);
        a.rows = pick(a_in.rowsm[0], a_in.rowsm[1], a_in.rowsm[2], a_in.rowsm[3]);
        bx -= pick(0, a_in.wg_end[0], a_in.wg_end[1], a_in.wg_end[2]);
    }
    const B32Args &a = [&]() -> const B32Args & {
        if constexpr (MULTI) return a_sel;
        else return a_in;
    }();
    static_assert(RING == 0 || (RING == 3 && FUSEQ && NXQ > 0 && !INTS), "the ring serves the fused single-launch calls with the activation in registers");
    constexpr int NB = RING ? RING : 1, PRE = RING ? 2 : 1;
    constexpr int T = WAVES * 64;  // threads of a workgroup; its activation prologue is shared by WAVES * (64 / P) rows
    static_assert(!FUSEQ || (NT <= 2 && !INTS), "the fused quantizer serves one token, or two contiguous f32 rows");
    constexpr int RPW = kWave / P;
    extern __shared__ uint4 smem[];
    const int nb = a.nb;
    int8_t *ys = reinterpret_cast<int8_t *>(smem);                 // [NT][nb*32]
    float *xss = reinterpret_cast<float *>(ys + NT * nb * 32);     // [NT][nb]
    int *bsum = reinterpret_cast<int *>(xss + NT * nb);            // [NT][nb] (Q4_0)

    const int tid = threadIdx.x;
    const int slot = blockIdx.y;
    const int64_t band = a.band_ids ? a.band_ids[slot] : 0;
    const int8_t *q = a.q + static_cast<int64_t>(slot) * a.act_slot_stride * nb * 32;
    const float *xs = a.xs + static_cast<int64_t>(slot) * a.act_slot_stride * nb;
    float *out = (PAIR && blockIdx.z == 1 ? a.out2 : a.out) + static_cast<int64_t>(slot) * a.out_slot_stride;

    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
    const int r = lane / P, l = lane - r * P;
    const int row = (bx * WAVES + wave) * RPW + r;
    const bool live = row < a.rows;
    const int64_t arow = band * a.rows + (live ? row : a.rows - 1);
    const bool second = PAIR && blockIdx.z == 1;
    const uint8_t *qrow = (second ? a.quants2 : a.quants) + arow * a.q_stride;
    const uint8_t *srow = (second ? a.scales2 : a.scales) + arow * a.s_stride;
    const bool leader = (l == P - 1);
    const int n_steps = (nb + P - 1) / P;
    constexpr int UE = U;  // steps per register buffer, also loaded ahead of the prologue
    B32Regs<FMT, UE> ra;
    B32Regs<FMT, 1> ring[NB];
    bool preloaded = false;

    if constexpr (FUSEQ) {
        const float4 *x4 = reinterpret_cast<const float4 *>(a.x);
        // NXQ > 0 (the launcher's promise that nb * 8 <= T * NXQ): the thread holds NXQ float4 of
        // the activation in registers -- rows of up to 128 blocks
        constexpr int NX = NXQ > 0 ? NXQ : 1;
        if constexpr (NXQ > 0) {
            // The token's f32 loads go out first, the row's first weight steps right behind them, and
            // the quantizer then waits for the f32 values only (a wave's loads return in order).
            const int n4 = NT * nb * 8;  // two tokens: contiguous rows, contiguous staging areas
            float4 xv[NX];
#pragma unroll
            for (int j = 0; j < NX; j++) xv[j] = x4[min(tid + T * j, n4 - 1)];
            __builtin_amdgcn_sched_barrier(0);
            if constexpr (RING) {
#pragma unroll
                for (int j = 0; j < PRE; j++) b32_load<FMT, P, 1>(ring[j], qrow, srow, l, j, n_steps, nb);
            } else {
                b32_load<FMT, P, UE>(ra, qrow, srow, l, 0, n_steps, nb);
            }
            preloaded = true;
            __builtin_amdgcn_sched_barrier(0);
            uint32_t *ys32 = reinterpret_cast<uint32_t *>(ys);
            // straight-line: the four blocks of a thread are independent chains the scheduler can
            // interleave; only the LDS stores are predicated (whole blocks of eight lanes are in or
            // out together, and a clamped load duplicates the last block's values)
            uint32_t packed[NX];
            float scale[NX];
#pragma unroll
            for (int j = 0; j < NX; j++) packed[j] = q8_0_quantize_lane8(xv[j], scale[j]);
#pragma unroll
            for (int j = 0; j < NX; j++) {
                const int i = tid + T * j;
                int sum = 0;
                if constexpr (FMT == CML_Q4_0) sum = group_sum_to_last<8>(sdot4(packed[j], 0x01010101u, 0));
                if (i < n4) {
                    ys32[i] = packed[j];
                    if ((i & 7) == 0) xss[i >> 3] = scale[j];
                    if constexpr (FMT == CML_Q4_0) {
                        if ((i & 7) == 7) bsum[i >> 3] = sum;
                    }
                }
            }
        } else {
            b32_stage_quantized_from<FMT, T>([&](int i) { return x4[i]; }, NT * nb, tid, ys, xss, bsum);
        }
    } else {
        const uint4 *src = reinterpret_cast<const uint4 *>(q);
        uint4 *dst = reinterpret_cast<uint4 *>(ys);
        const int n16 = NT * nb * 2;  // even: lanes 2k, 2k+1 are in or out together
        if (NT == 1 && n16 <= T && a.early_loads) {  // uniform: one 16-byte piece and one scale per thread at most
            // the same order of issue for a quantized activation: its loads, the first weight steps, then the staging
            const uint4 v = src[min(tid, n16 - 1)];
            const float sc = xs[min(tid, nb - 1)];
            __builtin_amdgcn_sched_barrier(0);
            b32_load<FMT, P, UE>(ra, qrow, srow, l, 0, n_steps, nb);
            preloaded = true;
            __builtin_amdgcn_sched_barrier(0);
            if (tid < n16) {
                dst[tid] = v;
                if constexpr (FMT == CML_Q4_0) {
                    int s = bytesum16(v);
                    s += row_shr_i32<1>(s);
                    if (tid & 1) bsum[tid >> 1] = s;
                }
            }
            if (tid < nb) xss[tid] = sc;
        } else {
            for (int i = tid; i < n16; i += T) {
                const uint4 v = src[i];
                dst[i] = v;
                if constexpr (FMT == CML_Q4_0) {
                    int s = bytesum16(v);
                    s += row_shr_i32<1>(s);
                    if (i & 1) bsum[i >> 1] = s;
                }
            }
            for (int i = tid; i < NT * nb; i += T) xss[i] = xs[i];
        }
    }
    __syncthreads();

    int32_t *ints_row = nullptr;
    if constexpr (INTS) {
        if (a.ints && live) ints_row = a.ints + arow * static_cast<int64_t>(nb);
    }

    float acc[NT];
#pragma unroll
    for (int t = 0; t < NT; t++) acc[t] = 0.0f;

    if constexpr (RING) {
        b32_row_pass_ring<FMT, P, NT, NB, PRE>(ring, qrow, srow, l, nb, ys, bsum, xss, acc);
    } else if (preloaded) {
        b32_row_pass_from<FMT, P, NT, INTS, UE>(ra, qrow, srow, l, nb, ys, bsum, xss, acc, ints_row);
    } else {
        b32_row_pass<FMT, P, NT, INTS, U>(qrow, srow, l, nb, ys, bsum, xss, acc, ints_row);
    }

    if (leader && live) {
#pragma unroll
        for (int t = 0; t < NT; t++) {
            float v = acc[t];
            if (NT == 1 && a.residual) v = v + a.residual[row];
            out[static_cast<int64_t>(t) * a.rows + row] = v;
        }
    }
}

// Lanes per matrix row of a single-token matvec: 16 (8 for very short rows); 32 where 16 would
// leave at most 1024 waves (matrices of up to 4096 rows), 64 at most 512 (up to 2048 rows of at
// least 4096 values).  Measured over rows 1024..5632 x values 2048..14336, both formats: e.g.
// Q8_0 2048 x 8192 9.4 / 7.8 / 7.2 us with 16 / 32 / 64 lanes, Q4_0 4096 x 4096 4.8 / 4.2 / 5.3,
// Q4_0 5632 x 4096 4.9 / 5.9 / 6.7.
static int b32_lanes(int fmt, int64_t rows, int64_t nb) {
    int p = env_int(fmt == CML_Q8_0 ? "CAMELID_HIP_Q8_0_LANES" : "CAMELID_HIP_Q4_0_LANES", 0);
    if (p == 8 || p == 16 || p == 32 || p == 64) return p;
    p = nb <= 8 ? 8 : 16;
    if (p == 16 && env_int("CAMELID_HIP_B32_WIDE_ROWS", 1)) {
        const int64_t waves16 = (rows + 3) / 4;
        if (waves16 <= 512 && nb >= 128) p = 64;
        else if (fmt == CML_Q8_0 && nb == 128 && rows > 3584 && rows <= 4096) p = 64;  // Q8_0 4096 x 4096: 6.26 -> 5.66 us (3200 x 4096, 4096 x 5120 ... 8192 lose with 64)
        else if (waves16 <= 1024 && nb >= 64) p = 32;
    }
    return p;
}

// Steps per register buffer.  Long rows of a matrix with few of them leave one or two waves per
// SIMD, and then the bytes each wave keeps in flight decide the rate: four steps per buffer
// instead of two (Q4_0 4096 x 14336: 10.5 -> 9.5 us).  With more waves the deeper buffers only
// cost registers (14336 x 4096: 15.3 -> 16.4 us).
static int b32_depth(int rows, int lanes_per_row, int nb) {
    const int u = env_int("CAMELID_HIP_B32_DEPTH", 0);
    if (u == 2 || u == 4) return u;
    const int waves = (rows + 64 / lanes_per_row - 1) / (64 / lanes_per_row);
    const int n_steps = (nb + lanes_per_row - 1) / lanes_per_row;
    return (waves <= 2048 && n_steps >= 16) ? 4 : 2;
}


// Counter names of this file: "<format>.dot.p<lanes per row>.<variant>" (launch-counter registry, cml_kernel_launches).
template <int FMT, int P>
static std::string b32_counter(const char *variant) {
    return std::string(FMT == CML_Q8_0 ? "q8_0" : "q4_0") + ".dot.p" + std::to_string(P) + "." + variant;
}

template <int FMT, int P, int NT>
static int launch_b32_nt(const B32Args &ba, int n_bands, bool ints, hipStream_t st) {
    const int rows_per_wg = 4 * (64 / P);
    const unsigned gx = static_cast<unsigned>((ba.rows + rows_per_wg - 1) / rows_per_wg);
    const size_t lds = static_cast<size_t>(NT) * ba.nb * (32 + 4 + 4);
    if (lds > 64 * 1024) return fail(CML_ERR_UNSUPPORTED, "activation of %d blocks x %d tokens exceeds the LDS staging limit", ba.nb, NT);
    if (ints && NT == 1) {
        hipLaunchKernelGGL((gemv_b32_kernel<FMT, P, 1, true>), dim3(gx, n_bands), dim3(256), lds, st, ba);
        CML_COUNT_LAUNCH((b32_counter<FMT, P>("ints")));
    } else if (NT <= 2 && n_bands == 1 && b32_depth(ba.rows, P, ba.nb) == 4) {
        hipLaunchKernelGGL((gemv_b32_kernel<FMT, P, (NT <= 2 ? NT : 1), false, false, 4, 0, 4>), dim3(gx, n_bands), dim3(256), lds, st, ba);
        CML_COUNT_LAUNCH((b32_counter<FMT, P>("w4.deep")));
    } else if (NT <= 2 && n_bands == 1 && env_int("CAMELID_HIP_B32_WAVES", ba.rows >= 384 * 8 * (64 / P) ? 8 : 4) == 8) {
        // eight-wave workgroups where they still come to 1.5 per compute unit (Q8_0 14336 x 4096: 14.0 -> 12.5 us;
        // 11008 x 4096, 1.3 per compute unit: 6.1 -> 6.9)
        hipLaunchKernelGGL((gemv_b32_kernel<FMT, P, (NT <= 2 ? NT : 1), false, false, 8, 0, 2>), dim3((gx + 1) / 2, n_bands), dim3(512), lds, st, ba);
        CML_COUNT_LAUNCH((b32_counter<FMT, P>("w8")));
    } else {
        hipLaunchKernelGGL((gemv_b32_kernel<FMT, P, NT, false>), dim3(gx, n_bands), dim3(256), lds, st, ba);
        CML_COUNT_LAUNCH((b32_counter<FMT, P>("w4")));
    }
    CML_HIP_TRY(hipGetLastError());
    return CML_OK;
}

template <int FMT, int P>
static int launch_b32_p(const MatArgs &a, hipStream_t st) {
    const cml_weight *w = a.w;
    B32Args ba;
    ba.quants = w->planes.p[0];
    ba.q_stride = w->planes.row_stride[0];
    ba.scales = w->planes.p[1];
    ba.s_stride = w->planes.row_stride[1];
    ba.rows = static_cast<int>(w->rows);
    ba.nb = static_cast<int>(w->nb);
    ba.residual = a.residual;
    ba.ints = a.ints;
    ba.band_ids = nullptr;
    ba.early_loads = env_int("CAMELID_HIP_B32_EARLY_LOADS", 1);
    ba.act_slot_stride = 0;
    ba.out_slot_stride = a.n_tokens * static_cast<int64_t>(ba.rows);
    const int n_bands = 1;
    int64_t t0 = 0;
    while (t0 < a.n_tokens) {
        const int64_t left = a.n_tokens - t0;
        int nt = left >= 8 ? 8 : (left >= 4 ? 4 : (left >= 2 ? 2 : 1));
        while (nt > 1 && static_cast<size_t>(nt) * ba.nb * (32 + 4 + 4) > 64 * 1024) nt /= 2;  // long rows: fewer tokens per pass
        ba.q = a.q + t0 * w->cols;
        ba.xs = a.scales + t0 * w->nb;
        ba.out = a.out + t0 * ba.rows;
        int rc;
        switch (nt) {
            case 8: rc = launch_b32_nt<FMT, P, 8>(ba, n_bands, false, st); break;
            case 4: rc = launch_b32_nt<FMT, P, 4>(ba, n_bands, false, st); break;
            case 2: rc = launch_b32_nt<FMT, P, 2>(ba, n_bands, false, st); break;
            default: rc = launch_b32_nt<FMT, P, 1>(ba, n_bands, a.ints != nullptr, st); break;
        }
        if (rc != CML_OK) return rc;
        t0 += nt;
    }
    return CML_OK;
}

// Workgroup width of the fused (f32 token in) launch, how many float4 of the token a thread holds in registers
// (0 = the token is staged through a loop) and whether the two-step buffers are kept where the depth rule would take four.
struct B32FusedShape {
    int waves, nxq;
    bool shallow;
};
static B32FusedShape b32_fused_shape(int fmt, int P, int rows, int nb, bool two, bool pair, bool early_loads) {
    // Every workgroup quantizes the whole activation for itself; with eight waves twice the rows
    // share that prologue.  Worth it while the matrix still gives every compute unit a workgroup.
    int waves = env_int("CAMELID_HIP_B32_FUSED_WAVES", 0);
    if (waves != 2 && waves != 4 && waves != 8 && waves != 16) {
        waves = (rows >= 128 * 8 * (64 / P)) ? 8 : 4;
        // Q8_0 rows of 4096 values (the longest the register prologue takes) on tall matrices: sixteen
        // waves (16384 x 4096: 14.2 -> 12.7 us, 32000 x 4096: 24.7 -> 22.3); slower for Q4_0 and shorter rows
        if (fmt == CML_Q8_0 && nb == 128 && rows >= 224 * 16 * (64 / P)) waves = 16;
        // Q4_0 on a vocabulary-sized matrix: sixteen waves halve the number of workgroups that each quantize the
        // token (128256 x 3072: 34.1 -> 33.3 us; Q8_0 there is the same 59.2 us with 4, 8 or 16)
        if (fmt == CML_Q4_0 && nb <= 128 && rows >= 65536) waves = 16;
    }
    // Rows of more than 4096 values (the token is staged through LDS by every workgroup), one token, 16 lanes per row:
    // sixteen waves once eight-wave workgroups would outnumber the compute units (Q8_0 14336 x 8192: 30.0 -> 23.3 us,
    // 28672 x 8192 52.4 -> 42.2, 10240 x 8192 25.6 -> 18.4; Q4_0 14336 x 8192 15.9 -> 14.5, 9216 x 5120 9.23 -> 8.49);
    // Q8_0 rows of 8192 values on up to 8192 rows: four waves and two-step buffers (8192 x 8192: 19.3 -> 16.2 us,
    // 6144 x 8192 15.6 -> 13.5; shorter rows and Q4_0 keep eight: 8192 x 6144 11.1 against 11.9, Q4_0 8192 x 8192 10.95 against 12.6)
    bool shallow = false;
    if (P == 16 && !two && !pair && nb > 128 && !env_int("CAMELID_HIP_B32_FUSED_WAVES", 0) && env_int("CAMELID_HIP_B32_LONG_ROW_WAVES", 1)) {
        if (rows > 256 * 8 * (64 / P)) {
            if (fmt == CML_Q4_0 || nb >= 256 || rows < 16384) waves = 16;  // (Q8_0 16384 x 6144 and 32000 x 5120: 1 % slower with sixteen)
        } else if (fmt == CML_Q8_0 && nb >= 256) {
            waves = 4, shallow = true;
        }
    }
    if (two && waves != 4) waves = 8;  // the two-token variants: four or eight waves
    if (P > 16) waves = 8;
    // float4 of the activation per thread: 1, 2 or 4 in registers; longer rows (or the knob) take the staged path
    const int n4 = (two ? 2 : 1) * nb * 8, threads = waves * 64;
    int nxq = !early_loads ? 0 : n4 <= threads ? 1 : n4 <= 2 * threads ? 2 : n4 <= 4 * threads ? 4 : n4 <= 8 * threads ? 8 : 0;
    // (the token held in registers -- its requests out ahead of the first weight requests -- instead of staged through a loop
    // that the weight requests wait behind: Q8_0 2048 x 8192 7.14 -> 6.29 us, 4096 x 8192 9.86 -> 8.58; Q4_0 8192 x 8192 11.2 -> 9.8)
    const int nxq_most = env_int("CAMELID_HIP_B32_NXQ_MOST", 8);
    if (nxq > nxq_most) nxq = 0;
    if (two && nxq == 8) nxq = 0;
    if (waves == 16 && nxq > 2) nxq = 0;
    if (waves == 2) nxq = (nxq >= 1 && nxq <= 4) ? 4 : 0;  // one register variant for the short workgroup
    return B32FusedShape{waves, nxq, shallow};
}

// A single f32 token on this weight runs as ONE launch although its rows are longer than 8192 values: where the
// launch holds the token in registers (rows of up to 16384 values on eight-wave workgroups).  Against a quantizing
// launch followed by the matvec: Q8_0 4096 x 14336 13.5 us against 14.65, 4096 x 11008 12.96 against 14.92, 2048 x 11008
// 8.67 against 10.09; Q4_0 8192 x 14336 14.66 against 17.0, 5120 x 13824 13.0 against 14.4, 4096 x 14336 10.57 against 11.09.
// Where the token would be staged through a loop the two launches are as fast or faster (Q8_0 8192 x 14336 24.8 against 23.9,
// 8192 x 28672 47.9 against 44.4).
bool gemv_b32_long_rows_fuse(const cml_weight *w) {
    if ((w->fmt != CML_Q8_0 && w->fmt != CML_Q4_0) || w->rows <= 0 || !env_int("CAMELID_HIP_B32_LONG_ROWS_FUSE", 1)) return false;
    if (static_cast<size_t>(w->nb) * (32 + 4 + 4) > 64 * 1024) return false;
    const int p = b32_lanes(w->fmt, w->rows, w->nb);
    return b32_fused_shape(w->fmt, p, static_cast<int>(w->rows), static_cast<int>(w->nb), false, false, env_int("CAMELID_HIP_B32_EARLY_LOADS", 1) != 0).nxq > 0;
}

// Single token, f32 activation in: quantize + matvec in one launch.
template <int FMT, int P>
static int launch_b32_f32_p(const cml_weight *w, const float *x, float *out, hipStream_t st, int n_tokens, const cml_weight *w2 = nullptr,
                            float *out2 = nullptr) {
    B32Args ba{};
    if (w2) {
        ba.quants2 = w2->planes.p[0];
        ba.scales2 = w2->planes.p[1];
        ba.out2 = out2;
    }
    ba.quants = w->planes.p[0];
    ba.q_stride = w->planes.row_stride[0];
    ba.scales = w->planes.p[1];
    ba.s_stride = w->planes.row_stride[1];
    ba.rows = static_cast<int>(w->rows);
    ba.nb = static_cast<int>(w->nb);
    ba.x = x;
    ba.out = out;
    ba.early_loads = env_int("CAMELID_HIP_B32_EARLY_LOADS", 1);
    const bool two = n_tokens == 2;
    const size_t lds = static_cast<size_t>(two ? 2 : 1) * ba.nb * (32 + 4 + 4);
    if (lds > 64 * 1024) return fail(CML_ERR_UNSUPPORTED, "activation of %d blocks exceeds the LDS staging limit", ba.nb);
    const B32FusedShape fs = b32_fused_shape(FMT, P, ba.rows, ba.nb, two, w2 != nullptr, ba.early_loads != 0);
    const int waves = fs.waves, nxq = fs.nxq;
    const bool shallow = fs.shallow;
    const int rows_per_wg = waves * (64 / P);
    const unsigned gx = static_cast<unsigned>((ba.rows + rows_per_wg - 1) / rows_per_wg);
    if (w2) {
        // one token, two weights (grid.z = 2): the 16-lane, eight-wave launches with the token in registers; -1 = not served
        if constexpr (P == 16) {
            if (two || waves != 8 || (nxq != 1 && nxq != 2)) return -1;
            const bool ring = FMT == CML_Q8_0 && (ba.nb + P - 1) / P >= 3 && env_int("CAMELID_HIP_B32_RING", 1);
            const dim3 grid2(gx, 1, 2);
            if (ring && nxq == 1) hipLaunchKernelGGL((gemv_b32_kernel<FMT, P, 1, false, true, 8, 1, 2, 3, true>), grid2, dim3(512), lds, st, ba);
            else if (ring) hipLaunchKernelGGL((gemv_b32_kernel<FMT, P, 1, false, true, 8, 2, 2, 3, true>), grid2, dim3(512), lds, st, ba);
            else if (nxq == 1) hipLaunchKernelGGL((gemv_b32_kernel<FMT, P, 1, false, true, 8, 1, 2, 0, true>), grid2, dim3(512), lds, st, ba);
            else hipLaunchKernelGGL((gemv_b32_kernel<FMT, P, 1, false, true, 8, 2, 2, 0, true>), grid2, dim3(512), lds, st, ba);
            if (ring) CML_COUNT_LAUNCH((b32_counter<FMT, P>("w8.ring.fused.pair"))); else CML_COUNT_LAUNCH((b32_counter<FMT, P>("w8.fused.pair")));
            CML_HIP_TRY(hipGetLastError());
            return CML_OK;
        } else {
            return -1;
        }
    }
#define CML_B32_FUSED(W_, N_) \
    hipLaunchKernelGGL((gemv_b32_kernel<FMT, P, 1, false, true, W_, N_>), dim3(gx, 1), dim3(W_ * 64), lds, st, ba)
    const bool deep = !two && nxq == 0 && !shallow && b32_depth(ba.rows, P, ba.nb) == 4;
    if constexpr (P > 16) {
        // wide rows: eight-wave workgroups only (the launcher below sets them), single token
        if (two || waves != 8) return fail(CML_ERR_UNSUPPORTED, "rows of %d lanes take one token and eight-wave workgroups", P);
        if (deep) hipLaunchKernelGGL((gemv_b32_kernel<FMT, P, 1, false, true, 8, 0, 4>), dim3(gx, 1), dim3(512), lds, st, ba);
        else if (nxq == 1) CML_B32_FUSED(8, 1);
        else if (nxq == 2) CML_B32_FUSED(8, 2);
        else if (nxq == 4) CML_B32_FUSED(8, 4);
        else if (nxq == 8) CML_B32_FUSED(8, 8);
        else CML_B32_FUSED(8, 0);
    } else
    if (two) {
#define CML_B32_FUSED2(W_, N_) \
    hipLaunchKernelGGL((gemv_b32_kernel<FMT, P, 2, false, true, W_, N_>), dim3(gx, 1), dim3(W_ * 64), lds, st, ba)
        if (waves == 8) {
            if (nxq == 1 || nxq == 2) CML_B32_FUSED2(8, 2);
            else if (nxq == 4) CML_B32_FUSED2(8, 4);
            else CML_B32_FUSED2(8, 0);
        } else {
            if (nxq == 1 || nxq == 2) CML_B32_FUSED2(4, 2);
            else if (nxq == 4) CML_B32_FUSED2(4, 4);
            else CML_B32_FUSED2(4, 0);
        }
#undef CML_B32_FUSED2
    } else if (deep) {
        if (waves == 2) hipLaunchKernelGGL((gemv_b32_kernel<FMT, P, 1, false, true, 2, 0, 4>), dim3(gx, 1), dim3(128), lds, st, ba);
        else if (waves == 8) hipLaunchKernelGGL((gemv_b32_kernel<FMT, P, 1, false, true, 8, 0, 4>), dim3(gx, 1), dim3(512), lds, st, ba);
        else if (waves == 16) hipLaunchKernelGGL((gemv_b32_kernel<FMT, P, 1, false, true, 16, 0, 4>), dim3(gx, 1), dim3(1024), lds, st, ba);
        else hipLaunchKernelGGL((gemv_b32_kernel<FMT, P, 1, false, true, 4, 0, 4>), dim3(gx, 1), dim3(256), lds, st, ba);
    } else if (waves == 16) {
        if (nxq == 1) CML_B32_FUSED(16, 1);
        else if (nxq == 2) CML_B32_FUSED(16, 2);
        else CML_B32_FUSED(16, 0);
    } else if (waves == 2) {
        if (nxq == 4) CML_B32_FUSED(2, 4);
        else CML_B32_FUSED(2, 0);
    } else if (waves == 8) {
        // Q8_0 rows of 16 lanes: a ring of three one-step buffers instead of two two-step ones
        // (8192 x 2048: 4.80 -> 4.61 us; four slots 5.2; Q4_0 14336 x 4096 7.22 / 7.20 / 7.8 with
        // none / three / four, so Q4_0 keeps the two buffers; sixteen-wave workgroups gain nothing)
        const bool ring = FMT == CML_Q8_0 && P == 16 && (ba.nb + P - 1) / P >= 3 && env_int("CAMELID_HIP_B32_RING", 1);
        if (ring && nxq == 1) hipLaunchKernelGGL((gemv_b32_kernel<FMT, P, 1, false, true, 8, 1, 2, 3>), dim3(gx, 1), dim3(512), lds, st, ba);
        else if (ring && nxq == 2) hipLaunchKernelGGL((gemv_b32_kernel<FMT, P, 1, false, true, 8, 2, 2, 3>), dim3(gx, 1), dim3(512), lds, st, ba);
        else if (nxq == 1) CML_B32_FUSED(8, 1);
        else if (nxq == 2) CML_B32_FUSED(8, 2);
        else if (nxq == 4) CML_B32_FUSED(8, 4);
        else if (nxq == 8) CML_B32_FUSED(8, 8);
        else CML_B32_FUSED(8, 0);
    } else {
        if (nxq == 1) CML_B32_FUSED(4, 1);
        else if (nxq == 2) CML_B32_FUSED(4, 2);
        else if (nxq == 4) CML_B32_FUSED(4, 4);
        else if (nxq == 8) CML_B32_FUSED(4, 8);
        else CML_B32_FUSED(4, 0);
    }
#undef CML_B32_FUSED
    {
        const bool ring_taken = !two && !deep && waves == 8 && FMT == CML_Q8_0 && P == 16 && (ba.nb + P - 1) / P >= 3 && env_int("CAMELID_HIP_B32_RING", 1) &&
                                (nxq == 1 || nxq == 2);
        if (two) { if (waves == 8) CML_COUNT_LAUNCH((b32_counter<FMT, P>("w8.fused.two"))); else CML_COUNT_LAUNCH((b32_counter<FMT, P>("w4.fused.two"))); }
        else if (ring_taken) CML_COUNT_LAUNCH((b32_counter<FMT, P>("w8.ring.fused")));
        else if (deep) { if (waves == 2) CML_COUNT_LAUNCH((b32_counter<FMT, P>("w2.deep.fused"))); else if (waves == 8) CML_COUNT_LAUNCH((b32_counter<FMT, P>("w8.deep.fused"))); else if (waves == 16) CML_COUNT_LAUNCH((b32_counter<FMT, P>("w16.deep.fused"))); else CML_COUNT_LAUNCH((b32_counter<FMT, P>("w4.deep.fused"))); }
        else if (waves == 16) CML_COUNT_LAUNCH((b32_counter<FMT, P>("w16.fused")));
        else if (waves == 8) CML_COUNT_LAUNCH((b32_counter<FMT, P>("w8.fused")));
        else if (waves == 2) CML_COUNT_LAUNCH((b32_counter<FMT, P>("w2.fused")));
        else CML_COUNT_LAUNCH((b32_counter<FMT, P>("w4.fused")));
    }
    CML_HIP_TRY(hipGetLastError());
    return CML_OK;
}

// One f32 token against two weights of one shape in one launch; -1 = a shape that launch does not serve.
int launch_gemv_b32_f32_pair(const cml_weight *w, const cml_weight *w2, const float *x, float *out, float *out2, hipStream_t st) {
    if (w->rows == 0) return CML_OK;
    if (b32_lanes(w->fmt, w->rows, w->nb) != 16) return -1;
    return w->fmt == CML_Q8_0 ? launch_b32_f32_p<CML_Q8_0, 16>(w, x, out, st, 1, w2, out2) : launch_b32_f32_p<CML_Q4_0, 16>(w, x, out, st, 1, w2, out2);
}

// One f32 token against two to four Q8_0 or Q4_0 weights of one row length in ONE launch (the q, k and v projections of
// an attention block): the eight-wave launches with the token in registers; every output is its own call's bits
// (the row chain does not depend on the launch shape).  -1 = not a set this launch serves.
// CAMELID_HIP_B32_MULTI=0: the caller makes the calls one by one.
template <int FMT, int P>
static int launch_b32_multi_p(const cml_weight *const *ws, int n, const float *x, float *const *outs, int nxq, hipStream_t st) {
    B32MultiArgs ma{};
    ma.base.nb = static_cast<int>(ws[0]->nb);
    ma.base.x = x;
    ma.base.early_loads = 1;
    constexpr int rows_per_wg = 8 * (64 / P);
    int wg = 0;
    for (int j = 0; j < 4; j++) {
        const cml_weight *w = ws[std::min(j, n - 1)];
        ma.quantsm[j] = w->planes.p[0];
        ma.q_stridem[j] = w->planes.row_stride[0];
        ma.scalesm[j] = w->planes.p[1];
        ma.s_stridem[j] = w->planes.row_stride[1];
        ma.outm[j] = outs[std::min(j, n - 1)];
        ma.rowsm[j] = static_cast<int>(w->rows);
        if (j < n) wg += (ma.rowsm[j] + rows_per_wg - 1) / rows_per_wg;
        ma.wg_end[j] = j < n ? wg : INT32_MAX;
    }
    const size_t lds = static_cast<size_t>(ma.base.nb) * (32 + 4 + 4);
    const dim3 grid(static_cast<unsigned>(wg)), block(512);
#define CML_B32_MULTI(N_) hipLaunchKernelGGL((gemv_b32_kernel<FMT, P, 1, false, true, 8, N_, 2, 0, false, true>), grid, block, lds, st, ma)
    switch (nxq) {
        case 1: CML_B32_MULTI(1); break;
        case 2: CML_B32_MULTI(2); break;
        case 4: CML_B32_MULTI(4); break;
        case 8: CML_B32_MULTI(8); break;
        default: return -1;
    }
#undef CML_B32_MULTI
    CML_COUNT_LAUNCH((b32_counter<FMT, P>("w8.fused.multi")));
    CML_HIP_TRY(hipGetLastError());
    return CML_OK;
}

int launch_gemv_b32_f32_multi(const cml_weight *const *ws, int n, const float *x, float *const *outs, hipStream_t st) {
    if (n < 2 || n > 4 || !env_int("CAMELID_HIP_B32_MULTI", 1) || !env_int("CAMELID_HIP_MULTI_LAUNCH", 1)) return -1;
    const int fmt = ws[0]->fmt;
    if (fmt != CML_Q8_0 && fmt != CML_Q4_0) return -1;
    int64_t rows_all = 0;
    for (int j = 0; j < n; j++) {
        if (ws[j]->fmt != fmt || ws[j]->nb != ws[0]->nb || ws[j]->rows <= 0) return -1;
        rows_all += ws[j]->rows;
    }
    if (rows_all > INT32_MAX || static_cast<size_t>(ws[0]->nb) * (32 + 4 + 4) > 64 * 1024) return -1;
    if (!x) return fail(CML_ERR_INVALID, "null activation");
    const int p = b32_lanes(fmt, rows_all, ws[0]->nb);
    const B32FusedShape fs = b32_fused_shape(fmt, p, static_cast<int>(rows_all), static_cast<int>(ws[0]->nb), false, false, true);
    // the eight-wave launches with the token in registers (a set whose total shape takes another launch: single calls)
    int nxq = fs.nxq;
    if (fs.waves != 8) {
        const int n4 = static_cast<int>(ws[0]->nb) * 8;
        nxq = n4 <= 512 ? 1 : n4 <= 1024 ? 2 : n4 <= 2048 ? 4 : n4 <= 4096 ? 8 : 0;
    }
    if (nxq == 0) return -1;
    const bool q8 = fmt == CML_Q8_0;
    switch (p) {
        case 8: return q8 ? launch_b32_multi_p<CML_Q8_0, 8>(ws, n, x, outs, nxq, st) : launch_b32_multi_p<CML_Q4_0, 8>(ws, n, x, outs, nxq, st);
        case 32: return q8 ? launch_b32_multi_p<CML_Q8_0, 32>(ws, n, x, outs, nxq, st) : launch_b32_multi_p<CML_Q4_0, 32>(ws, n, x, outs, nxq, st);
        case 64: return q8 ? launch_b32_multi_p<CML_Q8_0, 64>(ws, n, x, outs, nxq, st) : launch_b32_multi_p<CML_Q4_0, 64>(ws, n, x, outs, nxq, st);
        default: return q8 ? launch_b32_multi_p<CML_Q8_0, 16>(ws, n, x, outs, nxq, st) : launch_b32_multi_p<CML_Q4_0, 16>(ws, n, x, outs, nxq, st);
    }
}

int launch_gemv_b32_f32(const cml_weight *w, const float *x, float *out, hipStream_t st, int n_tokens) {
    if (w->rows == 0) return CML_OK;
    const bool q8 = w->fmt == CML_Q8_0;
    int p = b32_lanes(w->fmt, w->rows, w->nb);
    if (n_tokens != 1 && p > 16) p = 16;
    switch (p) {
        case 8: return q8 ? launch_b32_f32_p<CML_Q8_0, 8>(w, x, out, st, n_tokens) : launch_b32_f32_p<CML_Q4_0, 8>(w, x, out, st, n_tokens);
        case 32: return q8 ? launch_b32_f32_p<CML_Q8_0, 32>(w, x, out, st, n_tokens) : launch_b32_f32_p<CML_Q4_0, 32>(w, x, out, st, n_tokens);
        case 64: return q8 ? launch_b32_f32_p<CML_Q8_0, 64>(w, x, out, st, n_tokens) : launch_b32_f32_p<CML_Q4_0, 64>(w, x, out, st, n_tokens);
        default: return q8 ? launch_b32_f32_p<CML_Q8_0, 16>(w, x, out, st, n_tokens) : launch_b32_f32_p<CML_Q4_0, 16>(w, x, out, st, n_tokens);
    }
}

// ---- grouped (mixture-of-experts) dispatch ------------------------------------------------------
// blockIdx.y = y-slot.  With group_offsets: the slot serves group (expert) e = group_ids[y] (y
// itself when group_ids is null; -1 = unused slot): the band of rows [e*rows, (e+1)*rows) of the
// stacked weight dotted with the activation rows of the assignments [group_offsets[e],
// group_offsets[e+1]).  Without group_offsets (single-token decode): y-slot y IS assignment y and
// group_ids[y] its expert; ids outside [0, n_groups) are skipped.
// A group's assignments are staged NTMAX at a time; a chunk of 1, 2 or 3-4 runs the 1-, 2- or
// 4-token row pass (slots past the chunk repeat its last row and are not written).  Every cell is
// the single-row chain of the plain kernel: bit-identical to it.
// PRO selects where the staged activation comes from:
//   0  quantized rows q / xs (row group_rows[j], or j)
//   1  ONE f32 token x, quantized to Q8_0 inside every workgroup; every assignment reads it
//   2  assignment j's row is silu(x[j]) * u[j] (f32 rows x_stride apart), quantized in the workgroup
//   3  the same with gelu_tanh
struct B32GroupArgs {
    const uint8_t *quants;
    int64_t q_stride;
    const uint8_t *scales;
    int64_t s_stride;
    int rows;  // rows of one band
    int nb;
    int n_groups;
    const int8_t *q;  // [activation rows][nb*32]
    const float *xs;  // [activation rows][nb]
    const float *x;   // PRO 1: the f32 token; PRO 2, 3: gate rows
    const float *u;   // PRO 2, 3: up rows
    int64_t x_stride;
    float *out;       // [assignments][rows]
    const int32_t *group_offsets;
    const int32_t *group_rows;  // assignment -> activation row, or null (the assignment itself)
    const int32_t *group_ids;
};

// Quantize one row of nb blocks to Q8_0 straight into the LDS staging area, eight lanes per block;
// value4(i) yields the row's i-th float4.
template <int FMT, int T = 256, typename F>
__device__ __forceinline__ void b32_stage_quantized_from(F value4, int nb, int tid, int8_t *ys, float *xss, int *bsum) {
    uint32_t *ys32 = reinterpret_cast<uint32_t *>(ys);
    const int n4 = nb * 8;  // a multiple of 8: the eight lanes of a block enter and leave together
    for (int i = tid; i < n4; i += T) {
        float scale;
        const uint32_t packed = q8_0_quantize_lane8(value4(i), scale);
        ys32[i] = packed;
        if ((i & 7) == 0) xss[i >> 3] = scale;
        if constexpr (FMT == CML_Q4_0) {
            const int s = group_sum_to_last<8>(sdot4(packed, 0x01010101u, 0));
            if ((i & 7) == 7) bsum[i >> 3] = s;
        }
    }
}

template <int FMT, int P, int NTMAX, int PRO, int U>
__global__ __launch_bounds__(256) void gemv_b32_grouped_kernel(B32GroupArgs a) {
    static_assert(PRO == 0 || NTMAX == 1, "the fused prologues stage one activation row at a time");
    constexpr int RPW = kWave / P;
    extern __shared__ uint4 smem[];
    const int nb = a.nb;
    int8_t *ys = reinterpret_cast<int8_t *>(smem);                 // [NTMAX][nb*32]
    float *xss = reinterpret_cast<float *>(ys + NTMAX * nb * 32);  // [NTMAX][nb]
    int *bsum = reinterpret_cast<int *>(xss + NTMAX * nb);         // [NTMAX][nb] (Q4_0)

    const int tid = threadIdx.x;
    int g, a0, cnt;
    if (a.group_offsets) {
        g = a.group_ids ? a.group_ids[blockIdx.y] : static_cast<int>(blockIdx.y);
        if (g < 0 || g >= a.n_groups) return;  // the whole workgroup leaves together
        a0 = a.group_offsets[g];
        cnt = a.group_offsets[g + 1] - a0;
    } else {
        g = a.group_ids[blockIdx.y];
        a0 = blockIdx.y;
        cnt = 1;
    }
    if (g < 0 || g >= a.n_groups || cnt <= 0) return;

    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
    const int r = lane / P, l = lane - r * P;
    const int row = (blockIdx.x * 4 + wave) * RPW + r;
    const bool live = row < a.rows;
    const int64_t arow = static_cast<int64_t>(g) * a.rows + (live ? row : a.rows - 1);
    const uint8_t *qrow = a.quants + arow * a.q_stride;
    const uint8_t *srow = a.scales + arow * a.s_stride;
    const bool leader = (l == P - 1);

    // Stage the activation rows of assignments a0+c0 .. (nt of them, `staged` slots filled).
    auto stage = [&](int c0, int nt, int staged) {
        if constexpr (PRO == 1) {
            if (c0 == 0) {
                const float4 *x4 = reinterpret_cast<const float4 *>(a.x);
                b32_stage_quantized_from<FMT>([&](int i) { return x4[i]; }, nb, tid, ys, xss, bsum);
            }
        } else if constexpr (PRO >= 2) {
            const float4 *g4 = reinterpret_cast<const float4 *>(a.x + static_cast<int64_t>(a0 + c0) * a.x_stride);
            const float4 *u4 = reinterpret_cast<const float4 *>(a.u + static_cast<int64_t>(a0 + c0) * a.x_stride);
            b32_stage_quantized_from<FMT>([&](int i) { return glu4<PRO - 2>(g4[i], u4[i]); }, nb, tid, ys, xss, bsum);
        } else {
            const int per_t = nb * 2;  // 16-byte pieces per activation row (even)
            uint4 *dst = reinterpret_cast<uint4 *>(ys);
            for (int i = tid; i < staged * per_t; i += 256) {
                const int t = i / per_t, j = i - t * per_t;
                const int slot = a0 + c0 + min(t, nt - 1);
                const int64_t src_row = a.group_rows ? a.group_rows[slot] : slot;
                const uint4 v = reinterpret_cast<const uint4 *>(a.q + src_row * nb * 32)[j];
                dst[i] = v;
                if constexpr (FMT == CML_Q4_0) {
                    int s = bytesum16(v);
                    s += row_shr_i32<1>(s);
                    if (i & 1) bsum[i >> 1] = s;
                }
            }
            for (int i = tid; i < staged * nb; i += 256) {
                const int t = i / nb, j = i - t * nb;
                const int slot = a0 + c0 + min(t, nt - 1);
                const int64_t src_row = a.group_rows ? a.group_rows[slot] : slot;
                xss[i] = a.xs[src_row * nb + j];
            }
        }
    };

    for (int c0 = 0; c0 < cnt; c0 += NTMAX) {
        const int nt = min(NTMAX, cnt - c0);
        if (c0 > 0 && PRO != 1) __syncthreads();  // the previous chunk's readers are done
        stage(c0, nt, nt <= 1 ? 1 : (nt <= 2 ? 2 : 4));
        __syncthreads();
        float *out = a.out + static_cast<int64_t>(a0 + c0) * a.rows + row;
        auto run = [&](auto nt_tag) {
            constexpr int NT = decltype(nt_tag)::value;
            float acc[NT];
#pragma unroll
            for (int t = 0; t < NT; t++) acc[t] = 0.0f;
            b32_row_pass<FMT, P, NT, false, U>(qrow, srow, l, nb, ys, bsum, xss, acc, nullptr);
            if (leader && live) {
#pragma unroll
                for (int t = 0; t < NT; t++)
                    if (t < nt) out[static_cast<int64_t>(t) * a.rows] = acc[t];
            }
        };
        if constexpr (NTMAX == 1) {
            run(std::integral_constant<int, 1>{});
        } else {
            static_assert(NTMAX == 4, "chunk sizes 1, 2, 4");
            if (nt <= 1) run(std::integral_constant<int, 1>{});
            else if (nt <= 2) run(std::integral_constant<int, 2>{});
            else run(std::integral_constant<int, 4>{});
        }
    }
}

template <int FMT, int P, int U>
static int launch_b32_grouped_u(const MatArgs &a, const GroupedPrologue &pro, hipStream_t st) {
    const cml_weight *w = a.w;
    B32GroupArgs ga{};
    ga.quants = w->planes.p[0];
    ga.q_stride = w->planes.row_stride[0];
    ga.scales = w->planes.p[1];
    ga.s_stride = w->planes.row_stride[1];
    ga.rows = static_cast<int>(a.band_rows);
    ga.nb = static_cast<int>(w->nb);
    ga.n_groups = a.n_groups;
    ga.q = a.q;
    ga.xs = a.scales;
    ga.x = pro.x;
    ga.u = pro.u;
    ga.x_stride = pro.stride;
    ga.out = a.out;
    ga.group_offsets = a.group_offsets;
    ga.group_rows = a.group_rows;
    ga.group_ids = a.group_ids;
    const int rows_per_wg = 4 * (64 / P);
    const int slots = a.group_ids ? a.max_active : a.n_groups;
    const dim3 grid(static_cast<unsigned>((ga.rows + rows_per_wg - 1) / rows_per_wg), static_cast<unsigned>(slots));
    // one activation row per pass: single-token calls, and rows too long to stage four at a time
    const bool one = pro.kind != 0 || a.n_tokens <= 1 || static_cast<size_t>(4) * ga.nb * (32 + 4 + 4) > 64 * 1024;
    const size_t lds = static_cast<size_t>(one ? 1 : 4) * ga.nb * (32 + 4 + 4);
    if (lds > 64 * 1024) return fail(CML_ERR_UNSUPPORTED, "activation of %d blocks exceeds the LDS staging limit", ga.nb);
    switch (pro.kind) {
        case 1: hipLaunchKernelGGL((gemv_b32_grouped_kernel<FMT, P, 1, 1, U>), grid, dim3(256), lds, st, ga); break;
        case 2: hipLaunchKernelGGL((gemv_b32_grouped_kernel<FMT, P, 1, 2, U>), grid, dim3(256), lds, st, ga); break;
        case 3: hipLaunchKernelGGL((gemv_b32_grouped_kernel<FMT, P, 1, 3, U>), grid, dim3(256), lds, st, ga); break;
        default:
            if (one) hipLaunchKernelGGL((gemv_b32_grouped_kernel<FMT, P, 1, 0, U>), grid, dim3(256), lds, st, ga);
            else hipLaunchKernelGGL((gemv_b32_grouped_kernel<FMT, P, 4, 0, U>), grid, dim3(256), lds, st, ga);
            break;
    }
    switch (pro.kind) {  // "<format>.dot.p<lanes>.grouped[.token | .silu | .gelu | .one]": the prologue a grouped launch ran
        case 1: CML_COUNT_LAUNCH((b32_counter<FMT, P>("grouped.token"))); break;
        case 2: CML_COUNT_LAUNCH((b32_counter<FMT, P>("grouped.silu"))); break;
        case 3: CML_COUNT_LAUNCH((b32_counter<FMT, P>("grouped.gelu"))); break;
        default:
            if (one) CML_COUNT_LAUNCH((b32_counter<FMT, P>("grouped.one"))); else CML_COUNT_LAUNCH((b32_counter<FMT, P>("grouped")));
            break;
    }
    CML_HIP_TRY(hipGetLastError());
    return CML_OK;
}

template <int FMT, int P>
static int launch_b32_grouped_p(const MatArgs &a, const GroupedPrologue &pro, hipStream_t st) {
    return launch_b32_grouped_u<FMT, P, 2>(a, pro, st);  // 2 steps in flight per register buffer (4 measured slower)
}

int launch_gemv_b32_grouped(const MatArgs &a, const GroupedPrologue &pro, hipStream_t st) {
    const cml_weight *w = a.w;
    if (a.band_rows <= 0 || a.n_groups <= 0 || a.n_tokens <= 0) return CML_OK;
    if (w->fmt != CML_Q8_0 && w->fmt != CML_Q4_0) return fail(CML_ERR_UNSUPPORTED, "not a 32-value block format");
    if (a.band_rows * a.n_groups != w->rows) return fail(CML_ERR_SHAPE, "%d bands of %lld rows do not cover %lld rows", a.n_groups, (long long)a.band_rows, (long long)w->rows);
    if (!a.group_offsets && !a.group_ids) return fail(CML_ERR_INVALID, "grouped call without groups");
    if (pro.kind < 0 || pro.kind > 3 || (pro.kind != 0 && !pro.x) || (pro.kind >= 2 && !pro.u)) return fail(CML_ERR_INVALID, "bad prologue");
    const bool q8 = w->fmt == CML_Q8_0;
    // Lanes per row.  Batched calls: 4, so that a workgroup covers 64 rows -- the per-workgroup
    // chain (group lookup, activation staging, barrier) is then paid once per 64 rows instead of
    // once per 16, which is what bounds many small expert bands.  Single-token calls: 16, or 8 for
    // rows of up to 32 blocks so that a step's lanes are not mostly idle.
    int p = env_int(q8 ? "CAMELID_HIP_Q8_0_GROUPED_LANES" : "CAMELID_HIP_Q4_0_GROUPED_LANES", 0);
    const bool single = pro.kind != 0 || a.n_tokens <= 1;
    if (p != 4 && p != 8 && p != 16) p = !single ? 4 : (w->nb <= 8 ? 4 : (w->nb <= 32 ? 8 : 16));
    if (q8) {
        if (p == 4) return launch_b32_grouped_p<CML_Q8_0, 4>(a, pro, st);
        return p == 8 ? launch_b32_grouped_p<CML_Q8_0, 8>(a, pro, st) : launch_b32_grouped_p<CML_Q8_0, 16>(a, pro, st);
    }
    if (p == 4) return launch_b32_grouped_p<CML_Q4_0, 4>(a, pro, st);
    return p == 8 ? launch_b32_grouped_p<CML_Q4_0, 8>(a, pro, st) : launch_b32_grouped_p<CML_Q4_0, 16>(a, pro, st);
}

// One token, quantized activation in, rows of 32 or 64 lanes: eight-wave workgroups.
template <int FMT, int P>
static int launch_b32_wide(const MatArgs &a, hipStream_t st) {
    const cml_weight *w = a.w;
    B32Args ba{};
    ba.quants = w->planes.p[0];
    ba.q_stride = w->planes.row_stride[0];
    ba.scales = w->planes.p[1];
    ba.s_stride = w->planes.row_stride[1];
    ba.rows = static_cast<int>(w->rows);
    ba.nb = static_cast<int>(w->nb);
    ba.residual = a.residual;
    ba.q = a.q;
    ba.xs = a.scales;
    ba.out = a.out;
    ba.early_loads = env_int("CAMELID_HIP_B32_EARLY_LOADS", 1);
    ba.out_slot_stride = ba.rows;
    const int rows_per_wg = 8 * (64 / P);
    const unsigned gx = static_cast<unsigned>((ba.rows + rows_per_wg - 1) / rows_per_wg);
    const size_t lds = static_cast<size_t>(ba.nb) * (32 + 4 + 4);
    if (lds > 64 * 1024) return fail(CML_ERR_UNSUPPORTED, "activation of %d blocks exceeds the LDS staging limit", ba.nb);
    if (b32_depth(ba.rows, P, ba.nb) == 4)
        hipLaunchKernelGGL((gemv_b32_kernel<FMT, P, 1, false, false, 8, 0, 4>), dim3(gx, 1), dim3(512), lds, st, ba);
    else
        hipLaunchKernelGGL((gemv_b32_kernel<FMT, P, 1, false, false, 8, 0, 2>), dim3(gx, 1), dim3(512), lds, st, ba);
    CML_COUNT_LAUNCH((b32_counter<FMT, P>("w8.wide")));
    CML_HIP_TRY(hipGetLastError());
    return CML_OK;
}

template <int FMT>
static int launch_b32(const MatArgs &a, hipStream_t st) {
    if (a.w->rows == 0 || a.n_tokens == 0) return CML_OK;
    if (a.group_offsets) return launch_gemv_b32_grouped(a, GroupedPrologue{}, st);
    // 16 lanes per row by default; 8 when rows are short enough that half the lanes would idle;
    // 32 or 64 for a single token on a matrix of few, long rows.
    int p = b32_lanes(FMT, a.w->rows, a.w->nb);
    if (p > 16 && (a.n_tokens != 1 || a.ints != nullptr)) p = 16;
    if (p == 32) return launch_b32_wide<FMT, 32>(a, st);
    if (p == 64) return launch_b32_wide<FMT, 64>(a, st);
    return p == 8 ? launch_b32_p<FMT, 8>(a, st) : launch_b32_p<FMT, 16>(a, st);
}

int launch_gemv_q8_0(const MatArgs &a, hipStream_t st) { return launch_b32<CML_Q8_0>(a, st); }
int launch_gemv_q4_0(const MatArgs &a, hipStream_t st) { return launch_b32<CML_Q4_0>(a, st); }
int launch_gemm_q8_0(const MatArgs &a, hipStream_t st) { return launch_b32<CML_Q8_0>(a, st); }
int launch_gemm_q4_0(const MatArgs &a, hipStream_t st) { return launch_b32<CML_Q4_0>(a, st); }

}  // namespace cml
