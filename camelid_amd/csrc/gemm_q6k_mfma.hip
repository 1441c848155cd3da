// Q6_K x Q8_K small-batch matmul on the int8 matrix cores (gfx950), for batches
// of several tokens: speculative-verify chunks and short prefill against a Q6_K
// matrix (typically the LM head).
//
// Arithmetic: identical, cell by cell, to the matvec kernel (gemv_q6k.hip;
// reference q6_k_dot_scalar, src/diffusion_gemma/refmath.rs:678-721; the 8-lane
// form q6_k_wire_row_dot, src/inference.rs:25535-25581, differs by f32
// association only): per 256-value super-block the exact integer
//     T = sum_{j<16} sc_j * sum_{k<16} a[16j+k] * y[16j+k],   a = 6-bit code - 32
// then  acc = fma(d_w * yd, (float)T, acc),  super-blocks in order.
//
// Every 16-value sub-block has its own int8 scale, and a*sc does not fit an
// int8 operand, so the sub-block sums are taken one at a time and scaled in
// integer registers: one v_mfma_i32_16x16x32_i8 per sub-block, half of whose K
// range carries the sub-block and the other half zeros,
//     A[t][k]  = y_t[...]            16 tokens, from LDS (one 8-byte operand serves two sub-blocks)
//     B[k][n]  = a_n[...] or 0       16 rows, rebuilt in registers as signed bytes
//     T[t][n] += sc_j[n] * D[t][n]   v_mad_i32_i24 per cell
// Lane L supplies A-row t = L%16 and B-column n = L%16 at k-octet kq = L/16 and
// receives D[4*kq+v][L%16], v < 4: four tokens of one weight row.
//
// Weights stay in the plane layout (ql | qh | scales | d).  Lane kq = (h, s) of a
// row loads the 16-byte pieces ql[64h+16s..], ql[64h+32+16s..] and qh[32h+16s..]:
// four whole sub-blocks (8h+s, 8h+2+s, 8h+4+s, 8h+6+s) of 16 signed bytes each.
// Four 4x4 lane transposes (v_permlane32_swap, v_permlane16_swap) then hand lane
// kq the bytes 4kq..4kq+3 of sixteen sub-blocks, i.e. a quarter of K of every
// matrix instruction of the super-block.  Activations are staged in LDS in the
// matching order: [group of 4 sub-blocks][lane octet][sub-block][4 bytes].
//
// Workgroup, phases and register ring as in the Q4_K / 32-value-block
// matrix-core kernels.  When the matvec kernel would split K for this weight
// shape the same split is reproduced inside the lane, so that every cell equals
// the matvec result bit for bit.
#include <type_traits>

#include <atomic>
#include <string>

#include "cml_device.hpp"
#include "cml_host.hpp"

#pragma clang fp contract(off)

namespace cml {

typedef int v4i_q6 __attribute__((ext_vector_type(4)));
typedef unsigned v2u_q6 __attribute__((ext_vector_type(2)));

constexpr int kQ6SlabRow = 256 + 16;  // bytes of one token's super-block in LDS (padded)

struct Q6KMfmaArgs {
    const uint8_t *ql, *qh, *sc, *d;
    int64_t ql_stride, qh_stride, sc_stride, d_stride;
    int rows, n_sb;
    const int8_t *q;   // [n_tokens][n_sb*256]
    const float *yd;   // [n_tokens][n_sb]
    float *out;        // [n_tokens][rows]
    int n_tokens;      // plain: activation rows; grouped: the most assignments one group can hold
    int ksplit;        // association to reproduce (see gemv_q6k.hip)
    // Grouped call (mixture of experts): blockIdx.z -> group e (through group_ids when set; -1 =
    // unused slot), which owns the band of rows [e*rows, (e+1)*rows) and the assignments
    // [group_offsets[e], group_offsets[e+1]); assignment j reads activation row group_rows[j] (j
    // itself when null) and writes output row j.
    const int32_t *group_offsets;
    const int32_t *group_rows;
    const int32_t *group_ids;
};

struct Q6KMfmaWeights {
    uint4 ql0, ql1;  // pieces (h, p = 0, s) and (h, p = 1, s)
    uint4 qh;        // piece (h, s)
    uint4 sc;        // the super-block's 16 int8 scales
    uint32_t d;      // f16
};

// qlp / qhp already include the lane's (h, s) offsets inside a super-block.
__device__ __forceinline__ void q6k_mfma_load(Q6KMfmaWeights &r, const uint8_t *qlp, const uint8_t *qhp, const uint8_t *scp,
                                              const uint8_t *dp, int64_t sb) {
    r.ql0 = ldg16(qlp + sb * 128);
    r.ql1 = ldg16(qlp + sb * 128 + 32);
    r.qh = ldg16(qhp + sb * 64);
    r.sc = ldg16(scp + sb * 16);
    r.d = ldg2(dp + sb * 2);
}

// vdst's lanes 32..63 trade places with src's lanes 0..31
__device__ __forceinline__ void q6_swap32(uint32_t &vdst, uint32_t &src) {
    const v2u_q6 r = __builtin_amdgcn_permlane32_swap(vdst, src, false, false);
    vdst = r.x;
    src = r.y;
}
// vdst's odd 16-lane rows trade places with src's even rows
__device__ __forceinline__ void q6_swap16(uint32_t &vdst, uint32_t &src) {
    const v2u_q6 r = __builtin_amdgcn_permlane16_swap(vdst, src, false, false);
    vdst = r.x;
    src = r.y;
}
// In: word m of the sub-block this lane owns.  Out: w[r] = word kq of the sub-block lane r owns.
__device__ __forceinline__ void q6_transpose4(uint32_t (&w)[4]) {
    q6_swap32(w[0], w[2]);
    q6_swap32(w[1], w[3]);
    q6_swap16(w[0], w[1]);
    q6_swap16(w[2], w[3]);
}
// Four 6-bit codes (one per byte, 0..63) -> signed bytes code - 32: force bit 7 so that the
// byte-wise subtraction never borrows from its neighbour, then take it out again.
__device__ __forceinline__ uint32_t q6_center(uint32_t codes) {
    return ((codes | 0x80808080u) - 0x20202020u) ^ 0x80808080u;
}

// KS > 1: KS waves per row tile, each walking one part of K (the matvec kernel's split points);
// their partial chains are added left to right through LDS at the end.  SPLIT: the same split
// reproduced inside one lane (for split factors that are not run as waves).
// PLAIN: the entry of a call without expert groups (no group tables to read before the first request).
template <int GPW, int TB, bool SPLIT, int KC, int RING, int KS = 1, bool PLAIN = false>
__global__ __launch_bounds__(256) void gemm_q6k_mfma_kernel(Q6KMfmaArgs a) {
    static_assert(!(SPLIT && KS > 1), "K is split across waves or inside the lane, not both");
    constexpr int NTOK = 16 * GPW * TB;              // tokens staged per workgroup
    constexpr int RT = 4 / (TB * KS);                // row tiles per workgroup
    constexpr int kBufBytes = KS * KC * NTOK * kQ6SlabRow;
    constexpr int nthreads = 256;
    constexpr int kPer = NTOK * 16 / nthreads;       // 16-byte pieces of one super-block of all tokens, per thread
    static_assert(RING % KC == 0 && kPer >= 1 && RT >= 1, "phase / staging shape");
    extern __shared__ uint4 smem[];
    uint8_t *buf0 = reinterpret_cast<uint8_t *>(smem);  // [KS][KC][NTOK][kQ6SlabRow]
    uint8_t *buf1 = buf0 + kBufBytes;
    float *yds = reinterpret_cast<float *>(buf1 + kBufBytes);  // [n_sb][NTOK]

    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
    const int n_sb = a.n_sb;
    const int n = lane & 15, kq = lane >> 4;  // B/D column (weight row in tile) and k-octet / A-row quad
    const int n_tiles = (a.rows + 15) / 16;
    const int ks = wave % KS, w2 = wave / KS;  // K part of this wave; its (row tile, token block)
    const int rt = w2 / TB, tb = w2 - rt * TB;
    // this wave's part of K and the longest part
    const int s_begin = KS > 1 ? ks * n_sb / KS : 0, s_end = KS > 1 ? (ks + 1) * n_sb / KS : n_sb;
    const int n_loc = s_end - s_begin, n_max = (n_sb + KS - 1) / KS;
    const int tile = blockIdx.x * RT + rt;
    const int row = tile * 16 + n;
    const bool grouped = !PLAIN && a.group_offsets != nullptr;
    const int64_t band = grouped ? (a.group_ids ? a.group_ids[blockIdx.z] : static_cast<int>(blockIdx.z)) : 0;
    if (band < 0) return;  // a z-slot past the groups in use
    const int a0 = grouped ? a.group_offsets[band] : 0;  // first assignment of this group
    const int n_assign = grouped ? a.group_offsets[band + 1] - a0 : a.n_tokens;
    const int tok0 = blockIdx.y * NTOK;  // first token (assignment of the group) of this workgroup
    if (tok0 >= n_assign) return;        // nothing routed here: the whole workgroup leaves
    const int n_here = min(NTOK, n_assign - tok0);
    // activation row of local token t (tokens past the end repeat the last one; their cells are not stored)
    auto act_row = [&](int t) __attribute__((always_inline)) -> int64_t {
        const int j = a0 + tok0 + min(t, n_here - 1);
        if (PLAIN) return j;
        return a.group_rows ? a.group_rows[j] : j;
    };

    // activation scales: yds[sb][token]
    for (int i = tid; i < n_sb * NTOK; i += nthreads) {
        const int sb = i / NTOK, t = i - sb * NTOK;
        yds[i] = a.yd[act_row(t) * n_sb + sb];
    }

    // Staging: each thread owns kPer fixed (token, piece) pairs; only the super-block moves.  Piece
    // j = sub-block j = values 16j..16j+15.  Sub-block j = 8h + s + off belongs to the transpose
    // group of `off` (0, 4, 2, 6 -> group 0..3) and to owner lane r = 2h + s; its word m goes to
    // lane octet m:  [group][lane octet m][r][4 bytes].
    const v4i_q6 *stage_src[kPer];
    int stage_dst[kPer];
#pragma unroll
    for (int k = 0; k < kPer; k++) {
        const int i = tid + k * nthreads;
        const int t = i >> 4, j = i & 15;
        const int h = j >> 3, s = j & 1, off = j & 6;
        const int gidx = (off == 0) ? 0 : (off == 4) ? 1 : (off == 2) ? 2 : 3;
        stage_src[k] = reinterpret_cast<const v4i_q6 *>(a.q + act_row(t) * n_sb * 256) + j;
        stage_dst[k] = t * kQ6SlabRow + gidx * 64 + (2 * h + s) * 4;
    }
    v4i_q6 sreg[KS * KC][kPer];
    auto stage_load = [&](int p0) __attribute__((always_inline)) {  // of every K part, the KC super-blocks starting at its p0-th
#pragma unroll
        for (int kp = 0; kp < KS; kp++)
#pragma unroll
            for (int s = 0; s < KC; s++) {
                const int off = min((KS > 1 ? kp * n_sb / KS : 0) + p0 + s, n_sb - 1) * 16;  // in 16-byte units
#pragma unroll
                for (int k = 0; k < kPer; k++) sreg[kp * KC + s][k] = stage_src[k][off];
            }
    };
    auto stage_store = [&](uint8_t *buf) __attribute__((always_inline)) {
#pragma unroll
        for (int s = 0; s < KS * KC; s++)
#pragma unroll
            for (int k = 0; k < kPer; k++) {
                uint8_t *dst = buf + s * (NTOK * kQ6SlabRow) + stage_dst[k];
                const v4i_q6 v = sreg[s][k];
                *reinterpret_cast<int *>(dst) = v.x;
                *reinterpret_cast<int *>(dst + 16) = v.y;
                *reinterpret_cast<int *>(dst + 32) = v.z;
                *reinterpret_cast<int *>(dst + 48) = v.w;
            }
    };

    // Lane constants: this lane owns (h, s) = (kq >> 1, kq & 1) of its weight row.
    const int64_t arow = band * a.rows + min(row, a.rows - 1);
    const int h = kq >> 1, s = kq & 1;
    const uint8_t *qlp = a.ql + arow * a.ql_stride + 64 * h + 16 * s;
    const uint8_t *qhp = a.qh + arow * a.qh_stride + 32 * h + 16 * s;
    const uint8_t *scp = a.sc + arow * a.sc_stride;
    const uint8_t *dp = a.d + arow * a.d_stride;
    // A operand: this lane is token (lane & 15) of a group, octet kq: 16 bytes per transpose group.
    const int a_off = (lane & 15) * kQ6SlabRow + 16 * kq;
    const int cell_tok = 4 * kq;  // D values v = 0..3 of this lane: tokens 4*kq + v of the group, weight row n

    Q6KMfmaWeights ring[RING];
    // `loc` counts super-blocks inside this wave's part of K
    auto load_slot = [&](Q6KMfmaWeights &r, int loc) __attribute__((always_inline)) { q6k_mfma_load(r, qlp, qhp, scp, dp, min(s_begin + loc, s_end - 1)); };

    stage_load(0);
#pragma unroll
    for (int i = 0; i < RING; i++) load_slot(ring[i], i);
    stage_store(buf0);
    __syncthreads();

    float acc[GPW][4], total[GPW][4];
#pragma unroll
    for (int g = 0; g < GPW; g++)
#pragma unroll
        for (int j = 0; j < 4; j++) acc[g][j] = total[g][j] = 0.0f;
    int part = 0;                                            // index of the K-split part being accumulated
    int next_cut = a.ksplit <= 1 ? n_sb : n_sb / a.ksplit;  // first super-block of part 1

    // One super-block of this wave's tile against its token block.
    auto step = [&](const Q6KMfmaWeights &w0, int sb, const uint8_t *act) __attribute__((always_inline)) {
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
        // Rebuild this lane's four sub-blocks as signed bytes, in transpose-group order
        // off = 0 (low nibbles, p = 0), 4 (high, p = 0), 2 (low, p = 1), 6 (high, p = 1).
        const uint32_t ql[2][4] = {{w0.ql0.x, w0.ql0.y, w0.ql0.z, w0.ql0.w}, {w0.ql1.x, w0.ql1.y, w0.ql1.z, w0.ql1.w}};
        const uint32_t qh[4] = {w0.qh.x, w0.qh.y, w0.qh.z, w0.qh.w};
        uint32_t wq[4][4];  // [group][word of the sub-block]
#pragma unroll
        for (int p = 0; p < 2; p++)
#pragma unroll
            for (int m = 0; m < 4; m++) {
                const uint32_t hp = qh[m] >> (2 * p);  // p = 0: bits 0-1 / 4-5; p = 1: bits 2-3 / 6-7
                wq[2 * p][m] = q6_center((ql[p][m] & 0x0f0f0f0fu) | ((hp << 4) & 0x30303030u));
                wq[2 * p + 1][m] = q6_center(((ql[p][m] >> 4) & 0x0f0f0f0fu) | (hp & 0x30303030u));
            }
        // after the transposes: wq[gidx][r] = bytes 4kq..4kq+3 of sub-block 8*(r>>1) + (r&1) + off(gidx)
#pragma unroll
        for (int gi = 0; gi < 4; gi++) q6_transpose4(wq[gi]);
        const uint32_t scw[4] = {w0.sc.x, w0.sc.y, w0.sc.z, w0.sc.w};
        const float dw = f16_bits_to_f32(w0.d);
        const float *ydp = yds + sb * NTOK + tb * (16 * GPW) + cell_tok;
#pragma unroll
        for (int g = 0; g < GPW; g++) {
            const uint8_t *ybase = act + (tb * GPW + g) * (16 * kQ6SlabRow) + a_off;
            v4i_q6 T = {0, 0, 0, 0};
#pragma unroll
            for (int gi = 0; gi < 4; gi++) {
                constexpr int kOff[4] = {0, 4, 2, 6};
                const v4i_q6 av = *reinterpret_cast<const v4i_q6 *>(ybase + 64 * gi);
                const uint32_t aw[4] = {static_cast<uint32_t>(av.x), static_cast<uint32_t>(av.y), static_cast<uint32_t>(av.z),
                                        static_cast<uint32_t>(av.w)};
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    const int j = 8 * (r >> 1) + (r & 1) + kOff[gi];  // the sub-block of this instruction
                    // sub-blocks r = 0, 2 ride in the low half of their operand pair, r = 1, 3 in the high half
                    const unsigned long long a64 = static_cast<unsigned long long>(aw[r & ~1]) | (static_cast<unsigned long long>(aw[r | 1]) << 32);
                    const unsigned long long b64 = (r & 1) ? static_cast<unsigned long long>(wq[gi][r]) << 32 : static_cast<unsigned long long>(wq[gi][r]);
                    const v4i_q6 zero = {0, 0, 0, 0};
                    const v4i_q6 d = __builtin_amdgcn_mfma_i32_16x16x32_i8(static_cast<long>(a64), static_cast<long>(b64), zero, 0, 0, 0);
                    const int scj = static_cast<int>(static_cast<int8_t>((scw[j >> 2] >> (8 * (j & 3))) & 0xff));
                    T[0] = __mul24(scj, d[0]) + T[0];
                    T[1] = __mul24(scj, d[1]) + T[1];
                    T[2] = __mul24(scj, d[2]) + T[2];
                    T[3] = __mul24(scj, d[3]) + T[3];
                }
            }
            const float4 ydv = *reinterpret_cast<const float4 *>(ydp + 16 * g);
            acc[g][0] = __builtin_fmaf(dw * ydv.x, static_cast<float>(T[0]), acc[g][0]);
            acc[g][1] = __builtin_fmaf(dw * ydv.y, static_cast<float>(T[1]), acc[g][1]);
            acc[g][2] = __builtin_fmaf(dw * ydv.z, static_cast<float>(T[2]), acc[g][2]);
            acc[g][3] = __builtin_fmaf(dw * ydv.w, static_cast<float>(T[3]), acc[g][3]);
        }
    };

    // Rounds of RING super-blocks, phases of KC inside them: the next phase's activation loads are
    // issued at a phase start, ahead of younger weight loads, and stored at its end; the only
    // barriers are the phase boundaries.
    uint8_t *cur = buf0, *nxt = buf1;
    auto round = [&](int l0, auto refill) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < RING; i++) {
            const int loc = l0 + i;
            if (i % KC == 0) {
                stage_load(loc + KC);
                __builtin_amdgcn_sched_barrier(0);
            }
            if (loc < n_loc) step(ring[i], s_begin + loc, cur + (ks * KC + i % KC) * (NTOK * kQ6SlabRow));
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

    if (tile < n_tiles && row < a.rows) {
#pragma unroll
        for (int g = 0; g < GPW; g++)
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const int t = 16 * (tb * GPW + g) + cell_tok + j;
                if (t < n_here) {
                    const float v = (part == 0) ? acc[g][j] : total[g][j] + acc[g][j];
                    a.out[static_cast<int64_t>(a0 + tok0 + t) * a.rows + row] = v;
                }
            }
    }
}

int q6k_ksplit_for(int64_t rows, int64_t n_sb);  // gemv_q6k.hip: the matvec kernel's K-split policy

template <int GPW, int TB, bool SPLIT, int KC, int RING, int KS, bool PLAIN>
static int launch_q6k_mfma_gp(const Q6KMfmaArgs &ka, int n_groups, hipStream_t st) {
    constexpr int NTOK = 16 * GPW * TB, RT = 4 / (TB * KS);
    const int n_tiles = (ka.rows + 15) / 16;
    const unsigned gx = static_cast<unsigned>((n_tiles + RT - 1) / RT);
    const unsigned gy = static_cast<unsigned>((ka.n_tokens + NTOK - 1) / NTOK);
    const size_t lds = 2 * static_cast<size_t>(KS * KC * NTOK) * kQ6SlabRow + static_cast<size_t>(ka.n_sb) * NTOK * 4;
    if (lds > 160 * 1024) return fail(CML_ERR_UNSUPPORTED, "Q6_K matrix-core path: %d super-blocks exceed the LDS budget", ka.n_sb);
    static std::atomic<bool> raised{false};  // per instantiation: allow more than 64 KB of dynamic LDS once
    if (!raised.load(std::memory_order_acquire)) {
        CML_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(&gemm_q6k_mfma_kernel<GPW, TB, SPLIT, KC, RING, KS, PLAIN>),
                                        hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
        raised.store(true, std::memory_order_release);
    }
    hipLaunchKernelGGL((gemm_q6k_mfma_kernel<GPW, TB, SPLIT, KC, RING, KS, PLAIN>), dim3(gx, gy, n_groups), dim3(256), lds, st, ka);
    // "q6k.mfma.<tile | ksplit<KS> | serial_split>.g<token groups per wave>t<waves over tokens>.r<ring depth>[.grouped]"
    CML_COUNT_LAUNCH(std::string("q6k.mfma.") + (KS > 1 ? "ksplit" + std::to_string(KS) : std::string(SPLIT ? "serial_split" : "tile")) + ".g" +
                     std::to_string(GPW) + "t" + std::to_string(TB) + ".r" + std::to_string(RING) + (PLAIN ? "" : ".grouped"));
    CML_HIP_TRY(hipGetLastError());
    return CML_OK;
}

template <int GPW, int TB, bool SPLIT, int KC, int RING, int KS = 1>
static int launch_q6k_mfma_g(const Q6KMfmaArgs &ka, int n_groups, hipStream_t st) {
    return (ka.group_offsets == nullptr && !env_int("CAMELID_HIP_MFMA_GENERAL_ENTRY", 0)) ? launch_q6k_mfma_gp<GPW, TB, SPLIT, KC, RING, KS, true>(ka, n_groups, st)
                                       : launch_q6k_mfma_gp<GPW, TB, SPLIT, KC, RING, KS, false>(ka, n_groups, st);
}

// Phase length and ring depth: short phases and a shallow ring let several workgroups share a
// compute unit (what a large matrix wants); a matrix with few workgroups prefers the deep ring.
template <int GPW, int TB, bool SPLIT>
static int launch_q6k_mfma_p(const Q6KMfmaArgs &ka, int n_groups, hipStream_t st) {
    constexpr int NTOK = 16 * GPW * TB;
    int deep = env_int("CAMELID_HIP_Q6K_MFMA_DEEP", -1);
    if (deep != 0 && deep != 1) deep = (ka.rows + 15) / 16 < 2048 ? 1 : 0;
    if constexpr (NTOK == 16) {
        return deep ? launch_q6k_mfma_g<GPW, TB, SPLIT, 4, 4>(ka, n_groups, st) : launch_q6k_mfma_g<GPW, TB, SPLIT, 2, 2>(ka, n_groups, st);
    } else if constexpr (NTOK == 32) {
        return deep ? launch_q6k_mfma_g<GPW, TB, SPLIT, 4, 4>(ka, n_groups, st) : launch_q6k_mfma_g<GPW, TB, SPLIT, 2, 2>(ka, n_groups, st);
    } else {
        return deep ? launch_q6k_mfma_g<GPW, TB, SPLIT, 1, 4>(ka, n_groups, st) : launch_q6k_mfma_g<GPW, TB, SPLIT, 1, 2>(ka, n_groups, st);
    }
}

template <int GPW, int TB>
static int launch_q6k_mfma_s(const Q6KMfmaArgs &ka, int n_groups, hipStream_t st) {
    return ka.ksplit > 1 ? launch_q6k_mfma_p<GPW, TB, true>(ka, n_groups, st) : launch_q6k_mfma_p<GPW, TB, false>(ka, n_groups, st);
}

// Batch size from which the matrix-core kernel beats the packed-dot kernel.  Measured on MI355X:
// 128256x3072, 4 / 8 tokens: 70 / 102 us packed dot against 74 / 76 us; 4096x14336 (K split over
// four waves): 26 / 50 us against 19 us.
int q6k_mfma_min_tokens(int64_t rows, int64_t n_sb) {
    const int forced = env_int("CAMELID_HIP_Q6K_MFMA_MIN_TOKENS", 0);
    if (forced > 0) return forced;
    if ((rows + 15) / 16 >= 2048) return 5;
    const int ks = q6k_ksplit_for(rows, n_sb);
    return (ks == 2 || ks == 4) ? 4 : 7;
}

// Q6_K matmul on the matrix cores: plain calls, or grouped by expert (mixture of experts).
int launch_gemm_q6k_mfma(const MatArgs &a, hipStream_t st) {
    const cml_weight *w = a.w;
    const bool grouped = a.group_offsets != nullptr;
    if (w->rows == 0 || a.n_tokens == 0) return CML_OK;
    Q6KMfmaArgs ka{};
    ka.ql = w->planes.p[0]; ka.ql_stride = w->planes.row_stride[0];
    ka.qh = w->planes.p[1]; ka.qh_stride = w->planes.row_stride[1];
    ka.sc = w->planes.p[2]; ka.sc_stride = w->planes.row_stride[2];
    ka.d = w->planes.p[3];  ka.d_stride = w->planes.row_stride[3];
    ka.rows = static_cast<int>(grouped ? a.band_rows : w->rows);
    ka.n_sb = static_cast<int>(w->nb);
    ka.ksplit = q6k_ksplit_for(ka.rows, w->nb);
    ka.q = a.q;
    ka.yd = a.scales;
    ka.out = a.out;
    ka.n_tokens = static_cast<int>(a.n_tokens);
    ka.group_offsets = a.group_offsets;
    ka.group_rows = a.group_rows;
    ka.group_ids = a.group_ids;
    const int ng = grouped ? (a.group_ids ? a.max_active : a.n_groups) : 1;
    const int shape = env_int("CAMELID_HIP_Q6K_MFMA_SHAPE", 0);
    // K split across waves where the matvec kernel splits K two or four ways and the launch has
    // fewer row tiles than the chip has SIMDs: 16 or 32 tokens per workgroup, more tokens = more
    // workgroup columns.
    const int64_t launch_tiles = static_cast<int64_t>((ka.rows + 15) / 16) * ng;
    if (shape == 0 && launch_tiles < 1024 && !env_int("CAMELID_HIP_Q6K_MFMA_SERIAL_SPLIT", 0)) {
        const bool small = grouped || a.n_tokens <= 16;
        if (ka.ksplit == 4) return small ? launch_q6k_mfma_g<1, 1, false, 2, 4, 4>(ka, ng, st) : launch_q6k_mfma_g<2, 1, false, 1, 4, 4>(ka, ng, st);
        if (ka.ksplit == 2) return small ? launch_q6k_mfma_g<1, 1, false, 4, 4, 2>(ka, ng, st) : launch_q6k_mfma_g<2, 1, false, 2, 4, 2>(ka, ng, st);
    }
    switch (shape) {
        case 1: return launch_q6k_mfma_s<1, 1>(ka, ng, st);   // 16 tokens, 1 wave per row tile
        case 2: return launch_q6k_mfma_s<2, 1>(ka, ng, st);   // 32 tokens, 1 wave per row tile
        case 3: return launch_q6k_mfma_s<4, 1>(ka, ng, st);   // 64 tokens, 1 wave per row tile
        case 4: return launch_q6k_mfma_s<1, 2>(ka, ng, st);   // 32 tokens, 2 waves per row tile
        case 6: return launch_q6k_mfma_s<1, 4>(ka, ng, st);   // 64 tokens, 4 waves per row tile
        default: break;
    }
    if (grouped || a.n_tokens <= 16) return launch_q6k_mfma_s<1, 1>(ka, ng, st);
    const bool few_tiles = (ka.rows + 15) / 16 < 1024;
    if (a.n_tokens <= 32) return few_tiles ? launch_q6k_mfma_s<1, 2>(ka, ng, st) : launch_q6k_mfma_s<2, 1>(ka, ng, st);
    return few_tiles ? launch_q6k_mfma_s<1, 4>(ka, ng, st) : launch_q6k_mfma_s<4, 1>(ka, ng, st);
}

}  // namespace cml
