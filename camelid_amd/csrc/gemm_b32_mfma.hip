// Q8_0 x Q8_0 and Q4_0 x Q8_0 small-batch matmul on the int8 matrix cores
// (gfx950), for batches of several tokens: speculative-verify chunks and short
// prefill on the 32-value-block formats.
//
// Arithmetic: identical, cell by cell, to the matvec kernel (gemv_q8q4.hip;
// reference q8_0_wire_row_dot_scalar, src/inference.rs:22729-22745;
// q4_0_wire_row_dot_scalar, :22778-22798): per 32-value block, in block order,
//     isum = sum_j w_j * x_j                  (exact i32; Q4_0 weights are nibble - 8)
//     acc  = acc + ((float)isum * d_w) * d_x
// Every block has its own f32 step, so one matrix instruction covers exactly one
// block: v_mfma_i32_16x16x32_i8, K = 32.
//     A[t][k]  = x_t[32b + k]          16 tokens, from LDS
//     B[k][n]  = w_n[32b + k]          16 rows, straight from the weight plane
//     D[t][n]  = isum                  (Q4_0: C[t][n] = -8 * sum_k x_t[32b+k] carries the bias)
// Lane L supplies A-row t = L%16 and B-column n = L%16 at k-octet L/16, and
// receives D[4*(L/16)+v][L%16], v < 4: four tokens of one weight row, whose f32
// chains live in that lane, in block order.  The contraction index inside a
// block may be permuted freely (the sum is an exact integer), which is what makes
// the plain row-major weight plane usable without a re-layout.  The four lanes of
// a weight row load 64 contiguous bytes (16 each; narrower loads per lane were
// measured at a fraction of the bandwidth) and trade pieces with lane-swap
// instructions so that each ends up with its k-octet of every block:
//   Q8_0: 64 bytes = 2 blocks.  v_permlane32_swap hands each lane one 8-byte
//         octet of either block; lane octet kq supplies bytes 8*p..8*p+7 of a
//         block, p = {0, 2, 1, 3}[kq].
//   Q4_0: 64 bytes = 4 blocks, one per lane.  A 4x4 transpose (v_permlane32_swap,
//         v_permlane16_swap) leaves lane kq with bytes 4kq..4kq+3 of each block:
//         its low nibbles are values 4kq..4kq+3, its high nibbles 16+4kq..16+4kq+3.
// The activations are staged in LDS in the matching order, the two octets a lane
// needs of a pair of blocks side by side (one 16-byte LDS read per pair).
//
// A workgroup is 4 waves: 4/TB consecutive 16-row tiles x TB token blocks of
// 16*GPW tokens, sharing the staged activations of NTOK = 16*GPW*TB tokens.  K is
// walked in slabs of 256 values (8 blocks; rows must be whole slabs -- other
// lengths take the packed-dot kernel), phases of KC slabs double-buffered in LDS
// as in the Q4_K matrix-core kernel; weights stream through a register ring of
// RING slabs per wave.
#include <type_traits>

#include <atomic>
#include <string>

#include "cml_device.hpp"
#include "cml_host.hpp"

#pragma clang fp contract(off)

namespace cml {

typedef int v4i_b32 __attribute__((ext_vector_type(4)));
typedef int v2i_b32 __attribute__((ext_vector_type(2)));

constexpr int kB32SlabRow = 256 + 16;  // bytes of one token's 256-value slab in LDS (padded)

struct B32MfmaArgs {
    const uint8_t *quants;  // plane 0, row-major
    int64_t q_stride;
    const uint8_t *scales;  // plane 1: f16 per block, row-major
    int64_t s_stride;
    int rows, n_slabs;      // rows of one band; 256-value slabs per row
    const int8_t *q;        // [n_tokens][n_slabs*256]
    const float *xs;        // [n_tokens][n_slabs*8]
    float *out;             // [n_tokens][rows]
    int n_tokens;           // plain: activation rows; grouped: the most assignments one group can hold
    // Grouped call (mixture of experts): blockIdx.z -> group e (through group_ids when set; -1 =
    // unused slot), which owns the band of rows [e*rows, (e+1)*rows) and the assignments
    // [group_offsets[e], group_offsets[e+1]); assignment j reads activation row group_rows[j] (j
    // itself when null) and writes output row j.
    const int32_t *group_offsets;
    const int32_t *group_rows;
    const int32_t *group_ids;
};

template <int FMT>
struct B32SlabWeights {
    static constexpr int kPieces = FMT == CML_Q8_0 ? 4 : 2;  // 16-byte loads per slab and lane
    uint4 piece[kPieces];
    uint4 d;  // the slab's eight f16 block scales
};

// qlane already includes the lane's 16 * kq.
template <int FMT>
__device__ __forceinline__ void b32_mfma_load(B32SlabWeights<FMT> &r, const uint8_t *qlane, const uint8_t *srow, int64_t slab) {
    constexpr int slab_bytes = FMT == CML_Q8_0 ? 256 : 128;
#pragma unroll
    for (int i = 0; i < B32SlabWeights<FMT>::kPieces; i++) r.piece[i] = ldg16(qlane + slab * slab_bytes + i * 64);
    r.d = ldg16(srow + slab * 16);
}

typedef unsigned v2u_b32 __attribute__((ext_vector_type(2)));
// vdst's lanes 32..63 trade places with src's lanes 0..31
__device__ __forceinline__ void swap32(uint32_t &vdst, uint32_t &src) {
    const v2u_b32 r = __builtin_amdgcn_permlane32_swap(vdst, src, false, false);
    vdst = r.x;
    src = r.y;
}
// vdst's odd 16-lane rows trade places with src's even rows
__device__ __forceinline__ void swap16(uint32_t &vdst, uint32_t &src) {
    const v2u_b32 r = __builtin_amdgcn_permlane16_swap(vdst, src, false, false);
    vdst = r.x;
    src = r.y;
}

// The eight B operands (one per block of the slab) of this lane.
template <int FMT>
__device__ __forceinline__ void b32_mfma_operands(const B32SlabWeights<FMT> &r, long (&bw)[8]) {
    auto pack = [](uint32_t lo, uint32_t hi) __attribute__((always_inline)) {
        return static_cast<long>(static_cast<unsigned long long>(lo) | (static_cast<unsigned long long>(hi) << 32));
    };
    if constexpr (FMT == CML_Q8_0) {
        // piece i: lanes kq = 0, 1 hold block 2i (its halves), lanes 2, 3 block 2i+1
#pragma unroll
        for (int i = 0; i < 4; i++) {
            uint32_t a0 = r.piece[i].x, a1 = r.piece[i].y, b0 = r.piece[i].z, b1 = r.piece[i].w;
            swap32(a0, b0);
            swap32(a1, b1);
            bw[2 * i] = pack(a0, a1);      // an octet of block 2i
            bw[2 * i + 1] = pack(b0, b1);  // an octet of block 2i+1
        }
    } else {
        // piece i: lane kq holds block 4i + kq; transpose so that it holds word kq of blocks 4i..4i+3
#pragma unroll
        for (int i = 0; i < 2; i++) {
            uint32_t r0 = r.piece[i].x, r1 = r.piece[i].y, r2 = r.piece[i].z, r3 = r.piece[i].w;
            swap32(r0, r2);
            swap32(r1, r3);
            swap16(r0, r1);
            swap16(r2, r3);
            const uint32_t w[4] = {r0, r1, r2, r3};
#pragma unroll
            for (int j = 0; j < 4; j++) bw[4 * i + j] = pack(w[j] & 0x0f0f0f0fu, (w[j] >> 4) & 0x0f0f0f0fu);
        }
    }
}

// KC = slabs per phase (LDS holds two phases of NTOK tokens), RING = weight slabs a wave keeps in
// flight in registers.
// A workgroup's 4 waves are 4/TB consecutive row tiles x TB token blocks of 16*GPW tokens.
// PLAIN: the entry of a call without expert groups (no group tables to read before the first request).
template <int FMT, int GPW, int TB, int KC, int RING, bool PLAIN = false, int WAVES = 4>
__global__ __launch_bounds__(64 * WAVES) void gemm_b32_mfma_kernel(B32MfmaArgs a) {
    constexpr int NTOK = 16 * GPW * TB;              // tokens staged per workgroup
    constexpr int RT = WAVES / TB;                   // row tiles per workgroup
    constexpr int kBufBytes = KC * NTOK * kB32SlabRow;
    constexpr int kBsInts = KC * 8 * NTOK;           // per buffer: -8 * block sums, [slab][block][token]
    constexpr int nthreads = 64 * WAVES;
    constexpr int kPer = NTOK * 16 / nthreads;       // 16-byte pieces of one slab of all tokens, per thread
    static_assert(RING % KC == 0 && kPer >= 1, "phase / staging shape");
    extern __shared__ uint4 smem[];
    uint8_t *buf0 = reinterpret_cast<uint8_t *>(smem);  // [KC][NTOK][kB32SlabRow]
    uint8_t *buf1 = buf0 + kBufBytes;
    int *bs0 = reinterpret_cast<int *>(buf1 + kBufBytes);  // Q4_0 only
    int *bs1 = bs0 + (FMT == CML_Q4_0 ? kBsInts : 0);
    float *xss = reinterpret_cast<float *>(bs1 + (FMT == CML_Q4_0 ? kBsInts : 0));  // [n_slabs*8][NTOK]

    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
    const int n_slabs = a.n_slabs;
    const int n = lane & 15, kq = lane >> 4;  // B/D column (weight row in tile) and k-octet / A-row quad
    const int n_tiles = (a.rows + 15) / 16;
    const int rt = wave / TB, tb = wave - rt * TB;
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

    // activation scales: xss[block][token]
    const int nb = n_slabs * 8;
    // The first values per thread go to registers now and to LDS after the weight and activation
    // loads below have been issued: storing them here would put a whole memory round trip in front
    // of the first weight request.
    constexpr int kScaleRegs = 4;
    float scale_reg[kScaleRegs];
    const int n_scales = nb * NTOK;
#pragma unroll
    for (int k = 0; k < kScaleRegs; k++) {
        const int i = min(tid + k * nthreads, n_scales - 1);
        { const int b = i / NTOK, t = i - b * NTOK; scale_reg[k] = a.xs[act_row(t) * nb + b]; }
    }
    auto store_scales = [&]() __attribute__((always_inline)) {
#pragma unroll
        for (int k = 0; k < kScaleRegs; k++) {
            const int i = tid + k * nthreads;
            if (i < n_scales) xss[i] = scale_reg[k];
        }
        for (int i = tid + kScaleRegs * nthreads; i < n_scales; i += nthreads) {
        { const int b = i / NTOK, t = i - b * NTOK; xss[i] = a.xs[act_row(t) * nb + b]; }
        }
    };

    // Staging: each thread owns kPer fixed (token, piece) pairs; only the slab moves.  Piece pc =
    // half h = pc & 1 of block pc >> 1.  Destination order inside a slab: [pair of blocks][octet
    // lane 0..3][block of the pair][8 bytes], so that a lane reads its octets of both blocks of a
    // pair with one 16-byte load.
    const v4i_b32 *stage_src[kPer];
    int stage_dst[kPer], stage_tok[kPer], stage_blk[kPer];
#pragma unroll
    for (int k = 0; k < kPer; k++) {
        const int i = tid + k * nthreads;
        const int t = i >> 4, pc = i & 15;
        const int blk = pc >> 1, h = pc & 1;
        stage_src[k] = reinterpret_cast<const v4i_b32 *>(a.q + act_row(t) * n_slabs * 256) + pc;
        stage_tok[k] = t;
        stage_blk[k] = blk;
        if constexpr (FMT == CML_Q8_0)  // bytes 16h..16h+15 = octets 2h and 2h+1, which go to lane octets h and h + 2
            stage_dst[k] = t * kB32SlabRow + (blk >> 1) * 64 + h * 16 + (blk & 1) * 8;
        else  // values 16h..16h+15: dword o of the piece joins octet o at byte 4h
            stage_dst[k] = t * kB32SlabRow + (blk >> 1) * 64 + (blk & 1) * 8 + h * 4;
    }
    v4i_b32 sreg[KC][kPer];
    auto stage_load = [&](int p0) __attribute__((always_inline)) {  // the KC slabs starting at p0
#pragma unroll
        for (int s = 0; s < KC; s++) {
            const int off = min(p0 + s, n_slabs - 1) * 16;  // in 16-byte units
#pragma unroll
            for (int k = 0; k < kPer; k++) sreg[s][k] = stage_src[k][off];
        }
    };
    auto stage_store = [&](uint8_t *buf, int *bs) __attribute__((always_inline)) {
#pragma unroll
        for (int s = 0; s < KC; s++)
#pragma unroll
            for (int k = 0; k < kPer; k++) {
                uint8_t *dst = buf + s * (NTOK * kB32SlabRow) + stage_dst[k];
                const v4i_b32 v = sreg[s][k];
                if constexpr (FMT == CML_Q8_0) {
                    *reinterpret_cast<v2i_b32 *>(dst) = v2i_b32{v.x, v.y};
                    *reinterpret_cast<v2i_b32 *>(dst + 32) = v2i_b32{v.z, v.w};
                } else {
                    *reinterpret_cast<int *>(dst) = v.x;
                    *reinterpret_cast<int *>(dst + 16) = v.y;
                    *reinterpret_cast<int *>(dst + 32) = v.z;
                    *reinterpret_cast<int *>(dst + 48) = v.w;
                    // the block's -8 * sum of activations: the two halves sit in adjacent lanes, which
                    // swap partial sums and both store the total (a store under a lane condition here
                    // breaks the straight-line schedule and spills)
                    int sum = sdot4(static_cast<uint32_t>(v.x), 0x01010101u, 0);
                    sum = sdot4(static_cast<uint32_t>(v.y), 0x01010101u, sum);
                    sum = sdot4(static_cast<uint32_t>(v.z), 0x01010101u, sum);
                    sum = sdot4(static_cast<uint32_t>(v.w), 0x01010101u, sum);
                    sum += __builtin_amdgcn_update_dpp(0, sum, 0xB1 /* quad_perm [1,0,3,2] */, 0xf, 0xf, false);
                    bs[(s * 8 + stage_blk[k]) * NTOK + stage_tok[k]] = -8 * sum;
                }
            }
    };

    // Lane constants.
    const int64_t arow = band * a.rows + min(row, a.rows - 1);
    const uint8_t *qlane = a.quants + arow * a.q_stride + 16 * kq;
    const uint8_t *srow = a.scales + arow * a.s_stride;
    // A operand: this lane is token (lane & 15) of a group, octet kq: 16 bytes per pair of blocks.
    const int a_off = (lane & 15) * kB32SlabRow + 16 * kq;
    const int cell_tok = 4 * kq;  // D values v = 0..3 of this lane: tokens 4*kq + v of the group, weight row n

    B32SlabWeights<FMT> ring[RING];
    auto load_slot = [&](B32SlabWeights<FMT> &r, int slab) __attribute__((always_inline)) { b32_mfma_load<FMT>(r, qlane, srow, min(slab, n_slabs - 1)); };

    stage_load(0);
#pragma unroll
    for (int i = 0; i < RING; i++) load_slot(ring[i], i);
    store_scales();
    stage_store(buf0, bs0);
    __syncthreads();

    float acc[GPW][4];
#pragma unroll
    for (int g = 0; g < GPW; g++)
#pragma unroll
        for (int j = 0; j < 4; j++) acc[g][j] = 0.0f;

    // One slab (8 blocks) of this wave's tile against its tokens.
    auto step = [&](const B32SlabWeights<FMT> &w0, int slab, const uint8_t *act, const int *bs) __attribute__((always_inline)) {
        const uint32_t dwords[4] = {w0.d.x, w0.d.y, w0.d.z, w0.d.w};
        long bw8[8];
        b32_mfma_operands<FMT>(w0, bw8);
        {
            // Per token group: the slab's eight matrix instructions go out back to back (they do not depend on one
            // another), then the eight f32 steps run in block order -- the same operations in the same order per
            // cell, without a wait on the matrix core in front of every step (16 tokens: Q4_0 128256 x 3072
            // 61.7 -> 60.9 us, 32000 x 4096 39.7 -> 37.8, 14336 x 4096 21.7 -> 20.8; Q8_0 128256 x 3072 97.8 -> 95.0;
            // Q4_0 128256 x 3072 at 32 / 64 tokens 97.9 -> 85.2 / 181.5 -> 158.6).
#pragma unroll
            for (int g = 0; g < GPW; g++) {
                v4i_b32 d8[8];
#pragma unroll
                for (int pr = 0; pr < 4; pr++) {
                    const v4i_b32 av = *reinterpret_cast<const v4i_b32 *>(act + (tb * GPW + g) * (16 * kB32SlabRow) + a_off + 64 * pr);
                    const long a2[2] = {
                        static_cast<long>(static_cast<unsigned long long>(static_cast<uint32_t>(av.x)) | (static_cast<unsigned long long>(static_cast<uint32_t>(av.y)) << 32)),
                        static_cast<long>(static_cast<unsigned long long>(static_cast<uint32_t>(av.z)) | (static_cast<unsigned long long>(static_cast<uint32_t>(av.w)) << 32))};
#pragma unroll
                    for (int e = 0; e < 2; e++) {
                        const int b = 2 * pr + e;
                        v4i_b32 c = {0, 0, 0, 0};
                        if constexpr (FMT == CML_Q4_0) c = *reinterpret_cast<const v4i_b32 *>(bs + b * NTOK + 16 * (tb * GPW + g) + cell_tok);
                        d8[b] = __builtin_amdgcn_mfma_i32_16x16x32_i8(a2[e], bw8[b], c, 0, 0, 0);
                    }
                }
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int b = 0; b < 8; b++) {
                    const float dwb = f16_bits_to_f32((dwords[b >> 1] >> (16 * (b & 1))) & 0xffffu);
                    const float4 xv = *reinterpret_cast<const float4 *>(xss + (slab * 8 + b) * NTOK + 16 * (tb * GPW + g) + cell_tok);
                    acc[g][0] = acc[g][0] + (static_cast<float>(d8[b][0]) * dwb) * xv.x;
                    acc[g][1] = acc[g][1] + (static_cast<float>(d8[b][1]) * dwb) * xv.y;
                    acc[g][2] = acc[g][2] + (static_cast<float>(d8[b][2]) * dwb) * xv.z;
                    acc[g][3] = acc[g][3] + (static_cast<float>(d8[b][3]) * dwb) * xv.w;
                }
            }
        }
    };

    // Rounds of RING slabs, phases of KC inside them (the schedule of the Q4_K matrix-core
    // kernel): the next phase's activation loads are issued at a phase start, ahead of younger
    // weight loads, and stored at its end; the only barriers are the phase boundaries.
    uint8_t *cur = buf0, *nxt = buf1;
    int *bcur = bs0, *bnxt = bs1;
    auto round = [&](int s0, auto refill) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < RING; i++) {
            const int slab = s0 + i;
            if (i % KC == 0) {
                stage_load(slab + KC);
                __builtin_amdgcn_sched_barrier(0);
            }
            if (slab < n_slabs) step(ring[i], slab, cur + (i % KC) * (NTOK * kB32SlabRow), bcur + (i % KC) * (8 * NTOK));
            if constexpr (GPW > 1) __builtin_amdgcn_sched_barrier(0);
            if constexpr (decltype(refill)::value) load_slot(ring[i], slab + RING);
            if (i % KC == KC - 1) {
                stage_store(nxt, bnxt);
                __syncthreads();  // next phase complete in `nxt`, everyone done with `cur`
                uint8_t *t = cur;
                cur = nxt;
                nxt = t;
                int *tb = bcur;
                bcur = bnxt;
                bnxt = tb;
            }
        }
    };
    int s0 = 0;
    for (; s0 + RING < n_slabs; s0 += RING) round(s0, std::true_type{});
    round(s0, std::false_type{});

    if (tile < n_tiles && row < a.rows) {
#pragma unroll
        for (int g = 0; g < GPW; g++)
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const int t = 16 * (tb * GPW + g) + cell_tok + j;
                if (t < n_here) a.out[static_cast<int64_t>(a0 + tok0 + t) * a.rows + row] = acc[g][j];
            }
    }
}

// ---- up to 16 tokens, short rows, few row tiles: KD waves per row tile ------------------------------
//
// A matrix of 512 row tiles is 512 waves for the kernel above, each walking its tile's blocks alone
// on its SIMD: 24 thousand cycles per wave of which the vector and matrix instructions are a
// third -- the rest is one instruction waiting for the one before it (counters: 1561 vector
// instructions, 64 matrix instructions, 4900 cycles of s_waitcnt in 24461).  What is ordered in
// the reference's sum is only the chain  acc = acc + term_b  over the blocks of a row; a block's
// term  (float(isum) * d_w) * d_x  does not depend on the running sum.  So KD waves share a row
// tile, each taking one run of the row's 256-value slabs (all of them requested at entry): wave 0
// chains its terms as it goes, the others keep theirs in registers, and the running sums are
// handed from wave to wave through LDS behind KD - 1 barriers, each wave adding its terms in
// block order -- the reference's association bit for bit, with KD times the waves.
// SPW = most slabs per wave (rows of up to KD * SPW slabs), TPW = row tiles per workgroup (they share the staged activation).
template <int FMT, int KD, int SPW, int TPW>
__global__ __launch_bounds__(64 * KD * TPW) void gemm_b32_mfma_kpar_kernel(B32MfmaArgs a) {
    constexpr int nthreads = 64 * KD * TPW;
    constexpr int kStage = 256 * KD * SPW / nthreads;  // 16-byte activation pieces per thread for the longest row
    static_assert(kStage >= 1 && kStage * nthreads == 256 * KD * SPW, "the threads of a workgroup stage the longest row in whole passes");
    extern __shared__ uint4 smem[];
    const int n_slabs = a.n_slabs, nb = n_slabs * 8;
    uint8_t *act = reinterpret_cast<uint8_t *>(smem);                                   // [n_slabs][16 tokens][kB32SlabRow]
    int *bs = reinterpret_cast<int *>(act + n_slabs * 16 * kB32SlabRow);                // Q4_0: [nb][16 tokens] -8 * block sums
    float *xss = reinterpret_cast<float *>(bs + (FMT == CML_Q4_0 ? nb * 16 : 0));       // [nb][16 tokens]
    float4 *handoff_all = reinterpret_cast<float4 *>(xss + nb * 16);                    // [TPW][64 lanes]

    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
    const int kd = wave % KD, tw = wave / KD;
    float4 *handoff = handoff_all + tw * 64;
    const int n = lane & 15, kq = lane >> 4;
    const int n_tiles = (a.rows + 15) / 16;
    const int tile = blockIdx.x * TPW + tw;
    const int row = tile * 16 + n;
    const int tok0 = blockIdx.y * 16;
    const int n_here = min(16, a.n_tokens - tok0);
    auto act_row = [&](int t) __attribute__((always_inline)) -> int64_t { return tok0 + min(t, n_here - 1); };
    // this wave's slabs: [s_begin, s_begin + n_loc), at most SPW
    const int s_begin = kd * n_slabs / KD, n_loc = (kd + 1) * n_slabs / KD - s_begin;

    // activation pieces first (cache hits; the stores below then never wait behind a weight load)
    v4i_b32 sreg[kStage];
#pragma unroll
    for (int k = 0; k < kStage; k++) {
        const int i = tid + k * nthreads;  // piece (slab, token, pc)
        if (i < n_slabs * 256) {
            const int slab = i >> 8, t = (i >> 4) & 15, pc = i & 15;
            sreg[k] = reinterpret_cast<const v4i_b32 *>(a.q + (act_row(t) * n_slabs + slab) * 256)[pc];
        }
    }
    const int64_t arow = min(row, a.rows - 1);
    const uint8_t *qlane = a.quants + arow * a.q_stride + 16 * kq;
    const uint8_t *srow = a.scales + arow * a.s_stride;
    B32SlabWeights<FMT> ring[SPW];
#pragma unroll
    for (int i = 0; i < SPW; i++)
        if (i < n_loc) b32_mfma_load<FMT>(ring[i], qlane, srow, s_begin + i);  // wave-uniform
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int k = 0; k < kStage; k++) {
        const int i = tid + k * nthreads;
        const int slab = i >> 8, t = (i >> 4) & 15, pc = i & 15, blk = pc >> 1, h = pc & 1;
        if (i >= n_slabs * 256) continue;
        if (slab < n_slabs) {
            uint8_t *dst = act + (slab * 16 + t) * kB32SlabRow;
            const v4i_b32 v = sreg[k];
            if constexpr (FMT == CML_Q8_0) {
                dst += (blk >> 1) * 64 + h * 16 + (blk & 1) * 8;
                *reinterpret_cast<v2i_b32 *>(dst) = v2i_b32{v.x, v.y};
                *reinterpret_cast<v2i_b32 *>(dst + 32) = v2i_b32{v.z, v.w};
            } else {
                dst += (blk >> 1) * 64 + (blk & 1) * 8 + h * 4;
                *reinterpret_cast<int *>(dst) = v.x;
                *reinterpret_cast<int *>(dst + 16) = v.y;
                *reinterpret_cast<int *>(dst + 32) = v.z;
                *reinterpret_cast<int *>(dst + 48) = v.w;
            }
        }
        if constexpr (FMT == CML_Q4_0) {
            // the block's -8 * sum of activations: the two halves sit in adjacent lanes, which swap partial sums
            const v4i_b32 v = sreg[k];
            int sum = sdot4(static_cast<uint32_t>(v.x), 0x01010101u, 0);
            sum = sdot4(static_cast<uint32_t>(v.y), 0x01010101u, sum);
            sum = sdot4(static_cast<uint32_t>(v.z), 0x01010101u, sum);
            sum = sdot4(static_cast<uint32_t>(v.w), 0x01010101u, sum);
            sum += __builtin_amdgcn_update_dpp(0, sum, 0xB1 /* quad_perm [1,0,3,2] */, 0xf, 0xf, false);
            if (slab < n_slabs) bs[(slab * 8 + blk) * 16 + t] = -8 * sum;
        }
    }
    for (int i = tid; i < nb * 16; i += nthreads) {
        const int b = i >> 4, t = i & 15;
        xss[i] = a.xs[act_row(t) * nb + b];
    }
    __syncthreads();

    const int a_off = n * kB32SlabRow + 16 * kq;
    const int cell_tok = 4 * kq;
    float acc[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    float keep[SPW][8][4];
#pragma unroll
    for (int i = 0; i < SPW; i++) {
        if (i < n_loc) {
            const int slab = s_begin + i;
            const B32SlabWeights<FMT> &w0 = ring[i];
            const uint32_t dwords[4] = {w0.d.x, w0.d.y, w0.d.z, w0.d.w};
            long bw8[8];
            b32_mfma_operands<FMT>(w0, bw8);
            const uint8_t *abase = act + slab * (16 * kB32SlabRow) + a_off;
#pragma unroll
            for (int pr = 0; pr < 4; pr++) {
                const v4i_b32 av = *reinterpret_cast<const v4i_b32 *>(abase + 64 * pr);
                const long a2[2] = {
                    static_cast<long>(static_cast<unsigned long long>(static_cast<uint32_t>(av.x)) | (static_cast<unsigned long long>(static_cast<uint32_t>(av.y)) << 32)),
                    static_cast<long>(static_cast<unsigned long long>(static_cast<uint32_t>(av.z)) | (static_cast<unsigned long long>(static_cast<uint32_t>(av.w)) << 32))};
                const float dw[2] = {f16_bits_to_f32(dwords[pr] & 0xffffu), f16_bits_to_f32(dwords[pr] >> 16)};
#pragma unroll
                for (int e = 0; e < 2; e++) {
                    const int b = 2 * pr + e;
                    v4i_b32 c = {0, 0, 0, 0};
                    if constexpr (FMT == CML_Q4_0) c = *reinterpret_cast<const v4i_b32 *>(bs + (slab * 8 + b) * 16 + cell_tok);
                    const v4i_b32 d = __builtin_amdgcn_mfma_i32_16x16x32_i8(a2[e], bw8[b], c, 0, 0, 0);
                    const float4 xv = *reinterpret_cast<const float4 *>(xss + (slab * 8 + b) * 16 + cell_tok);
                    const float t4[4] = {(static_cast<float>(d[0]) * dw[e]) * xv.x, (static_cast<float>(d[1]) * dw[e]) * xv.y,
                                         (static_cast<float>(d[2]) * dw[e]) * xv.z, (static_cast<float>(d[3]) * dw[e]) * xv.w};
#pragma unroll
                    for (int j = 0; j < 4; j++) {
                        if (kd == 0) acc[j] = acc[j] + t4[j];
                        else keep[i][b][j] = t4[j];
                    }
                }
            }
        }
    }
    // the running sums go from wave to wave, each adding its blocks in order
#pragma unroll
    for (int stage = 1; stage < KD; stage++) {
        if (kd == stage - 1) handoff[lane] = make_float4(acc[0], acc[1], acc[2], acc[3]);
        __syncthreads();
        if (kd == stage) {
            const float4 h = handoff[lane];
            acc[0] = h.x;
            acc[1] = h.y;
            acc[2] = h.z;
            acc[3] = h.w;
#pragma unroll
            for (int i = 0; i < SPW; i++) {
                if (i < n_loc) {
#pragma unroll
                    for (int b = 0; b < 8; b++)
#pragma unroll
                        for (int j = 0; j < 4; j++) acc[j] = acc[j] + keep[i][b][j];
                }
            }
        }
        // (the next stage's writer is the wave that has just read the slot: no second barrier)
    }
    if (kd == KD - 1 && tile < n_tiles && row < a.rows) {
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const int t = cell_tok + j;
            if (t < n_here) a.out[static_cast<int64_t>(tok0 + t) * a.rows + row] = acc[j];
        }
    }
}

template <int FMT, int KD, int SPW, int TPW>
static int launch_b32_mfma_kpar(const B32MfmaArgs &ka, hipStream_t st) {
    const int n_tiles = (ka.rows + 15) / 16;
    const int nb = ka.n_slabs * 8;
    const size_t lds = static_cast<size_t>(ka.n_slabs) * 16 * kB32SlabRow + (FMT == CML_Q4_0 ? static_cast<size_t>(nb) * 16 * 4 : 0) +
                       static_cast<size_t>(nb) * 16 * 4 + TPW * 64 * 16;
    static std::atomic<bool> raised{false};  // setting the attribute twice from two threads is harmless
    if (!raised.load(std::memory_order_acquire)) {
        CML_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(&gemm_b32_mfma_kpar_kernel<FMT, KD, SPW, TPW>),
                                        hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
        raised.store(true, std::memory_order_release);
    }
    hipLaunchKernelGGL((gemm_b32_mfma_kpar_kernel<FMT, KD, SPW, TPW>),
                       dim3(static_cast<unsigned>((n_tiles + TPW - 1) / TPW), static_cast<unsigned>((ka.n_tokens + 15) / 16)), dim3(64 * KD * TPW), lds, st, ka);
    // "<format>.mfma.kpar.k<waves per row tile>s<slabs per wave>t<tiles per workgroup>"
    CML_COUNT_LAUNCH(std::string(FMT == CML_Q8_0 ? "q8_0" : "q4_0") + ".mfma.kpar.k" + std::to_string(KD) + "s" + std::to_string(SPW) + "t" + std::to_string(TPW));
    CML_HIP_TRY(hipGetLastError());
    return CML_OK;
}

template <int FMT, int GPW, int TB, int KC, int RING, bool PLAIN, int WAVES = 4>
static int launch_b32_mfma_gp(const B32MfmaArgs &ka, int n_groups, hipStream_t st) {
    constexpr int NTOK = 16 * GPW * TB, RT = WAVES / TB;
    const int n_tiles = (ka.rows + 15) / 16;
    const unsigned gx = static_cast<unsigned>((n_tiles + RT - 1) / RT);
    const unsigned gy = static_cast<unsigned>((ka.n_tokens + NTOK - 1) / NTOK);
    const size_t lds = 2 * static_cast<size_t>(KC * NTOK) * kB32SlabRow + (FMT == CML_Q4_0 ? 2 * static_cast<size_t>(KC * NTOK) * 8 * 4 : 0) +
                       static_cast<size_t>(ka.n_slabs) * 8 * NTOK * 4;
    if (lds > 160 * 1024) return fail(CML_ERR_UNSUPPORTED, "matrix-core path: %d blocks per row exceed the LDS budget", ka.n_slabs * 8);
    static std::atomic<bool> raised{false};  // per instantiation: allow more than 64 KB of dynamic LDS once
    if (!raised.load(std::memory_order_acquire)) {
        CML_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(&gemm_b32_mfma_kernel<FMT, GPW, TB, KC, RING, PLAIN, WAVES>),
                                        hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
        raised.store(true, std::memory_order_release);
    }
    hipLaunchKernelGGL((gemm_b32_mfma_kernel<FMT, GPW, TB, KC, RING, PLAIN, WAVES>), dim3(gx, gy, n_groups), dim3(64 * WAVES), lds, st, ka);
    // "<format>.mfma.tile.g<token groups per wave>t<waves over tokens>.w<waves>.r<ring depth>[.grouped]"
    CML_COUNT_LAUNCH(std::string(FMT == CML_Q8_0 ? "q8_0" : "q4_0") + ".mfma.tile.g" + std::to_string(GPW) + "t" + std::to_string(TB) + ".w" +
                     std::to_string(WAVES) + ".r" + std::to_string(RING) + (PLAIN ? "" : ".grouped"));
    CML_HIP_TRY(hipGetLastError());
    return CML_OK;
}

template <int FMT, int GPW, int TB, int KC, int RING>
static int launch_b32_mfma_g(const B32MfmaArgs &ka, int n_groups, hipStream_t st) {
    // Measured per variant, same box, alternating runs: the plain entry gains 0.5-2 % everywhere
    // (Q4_K 4 %) except the 16-token Q8_0 shape, which it slows from 11.3 to 11.9 us -- same
    // register count, a different schedule; that one keeps the general entry.
    constexpr bool kPlainPays = !(FMT == CML_Q8_0 && GPW == 1 && TB == 1);
    return (kPlainPays && ka.group_offsets == nullptr && !env_int("CAMELID_HIP_MFMA_GENERAL_ENTRY", 0)) ? launch_b32_mfma_gp<FMT, GPW, TB, KC, RING, true>(ka, n_groups, st)
                                       : launch_b32_mfma_gp<FMT, GPW, TB, KC, RING, false>(ka, n_groups, st);
}

// Phase length and ring depth.  Short phases keep the LDS footprint small, so that several
// workgroups share a compute unit and cover each other's barriers and load latency: what a large
// matrix wants (measured at 128256x3072, 8 tokens: 130 us with 128 token-slabs per phase, 60 us with
// 32).  A matrix with fewer workgroups than compute units gains nothing from that and prefers the
// deep ring.
template <int FMT, int GPW, int TB>
static int launch_b32_mfma_p(const B32MfmaArgs &ka, int n_groups, hipStream_t st) {
    constexpr int NTOK = 16 * GPW * TB;
    int deep = env_int("CAMELID_HIP_B32_MFMA_DEEP", -1);
    if (deep != 0 && deep != 1) deep = (ka.rows + 15) / 16 < 2048 ? 1 : 0;
    if constexpr (NTOK == 16) {
        // Q8_0 with at most 512 row tiles: workgroups of two waves instead of four, so that every compute
        // unit gets one (measured, 16 tokens: 8192 x 2048 11.4 -> 10.6 us, 4096 x 4096 17.5 -> 15.6; Q4_0
        // 4096 x 4096 18.6 -> 19.9, so Q4_0 keeps four).  A wave still walks a whole row tile alone: the
        // serial chain of one f32 step per 32-value block is what bounds these launches.
        const int two = env_int("CAMELID_HIP_B32_MFMA_TWO_WAVES", -1);
        if (deep && ka.group_offsets == nullptr && (two == 1 || (two != 0 && FMT == CML_Q8_0 && (ka.rows + 15) / 16 <= 512)))
            return launch_b32_mfma_gp<FMT, GPW, TB, 8, 8, true, 2>(ka, n_groups, st);
        return deep ? launch_b32_mfma_g<FMT, GPW, TB, 8, 8>(ka, n_groups, st) : launch_b32_mfma_g<FMT, GPW, TB, 2, 2>(ka, n_groups, st);
    } else if constexpr (NTOK == 32) {
        return deep ? launch_b32_mfma_g<FMT, GPW, TB, 4, 4>(ka, n_groups, st) : launch_b32_mfma_g<FMT, GPW, TB, 2, 2>(ka, n_groups, st);
    } else {  // 64 tokens: one slab per phase either way, so that two or three workgroups fit a compute unit
        return deep ? launch_b32_mfma_g<FMT, GPW, TB, 1, 4>(ka, n_groups, st) : launch_b32_mfma_g<FMT, GPW, TB, 1, 2>(ka, n_groups, st);
    }
}

template <int FMT>
static int launch_b32_mfma_fmt(const B32MfmaArgs &ka, int n_groups, bool grouped, hipStream_t st) {
    // Workgroup shape: token groups per wave x token blocks across waves.  Default: one wave per
    // row tile with 16 / 32 / 64 tokens; a matrix with fewer row tiles than the chip has SIMDs
    // spreads the tokens of a tile over 2 or 4 waves instead.
    // Up to 16 tokens, rows of at most 16 slabs, few row tiles: several waves per row tile, one chain.
    // Workgroup shapes by measurement (16 tokens, kernel us cache-cold, against the kernel below):
    //   rows of <= 8 slabs:  <= 256 tiles: 8 waves per tile (4096 x 2048 Q8_0 10.0 -> 6.0);
    //                        <= 768 tiles: 4 waves per tile, 2 tiles per workgroup (8192 x 2048 Q8_0 10.6 -> 8.0, Q4_0 11.8 -> 7.0);
    //                        more tiles: no gain (16384 x 2048 12.3 -> 12.2), the kernel below stays;
    //   rows of 9..16 slabs: the staged activation fills half of a compute unit's LDS, one workgroup per unit:
    //                        <= 256 tiles: 8 waves per tile (4096 x 4096 Q8_0 15.6 -> 10.8, Q4_0 18.6 -> 8.8);
    //                        <= 512 tiles: the same, 2 tiles per workgroup (8192 x 4096 Q8_0 16.9 -> 14.3, Q4_0 19.1 -> 11.1);
    //                        896 tiles lose (14336 x 4096 20.6 -> 26.0).
    const int kpar = env_int("CAMELID_HIP_B32_MFMA_KPAR", -1);
    const int tiles = (ka.rows + 15) / 16;
    if (!grouped && ka.n_tokens <= 16 && env_int("CAMELID_HIP_B32_MFMA_SHAPE", 0) == 0 && kpar != 0) {
        if (ka.n_slabs >= 4 && ka.n_slabs <= 8) {
            if (kpar == 1) return launch_b32_mfma_kpar<FMT, 4, 2, 1>(ka, st);
            if (kpar == 2) return launch_b32_mfma_kpar<FMT, 4, 2, 2>(ka, st);
            if (kpar == 3) return launch_b32_mfma_kpar<FMT, 8, 1, 1>(ka, st);
            if (kpar == 4) return launch_b32_mfma_kpar<FMT, 8, 1, 2>(ka, st);
            if (tiles <= 256) return launch_b32_mfma_kpar<FMT, 8, 1, 1>(ka, st);
            if (tiles <= 768) return launch_b32_mfma_kpar<FMT, 4, 2, 2>(ka, st);
        } else if (ka.n_slabs > 8 && ka.n_slabs <= 16) {
            if (kpar == 1) return launch_b32_mfma_kpar<FMT, 4, 4, 1>(ka, st);
            if (kpar == 2) return launch_b32_mfma_kpar<FMT, 8, 2, 1>(ka, st);
            if (kpar == 3) return launch_b32_mfma_kpar<FMT, 8, 2, 2>(ka, st);
            if (tiles <= 256) return launch_b32_mfma_kpar<FMT, 8, 2, 1>(ka, st);
            if (tiles <= 512) return launch_b32_mfma_kpar<FMT, 8, 2, 2>(ka, st);
        } else if (ka.n_slabs >= 2 && ka.n_slabs < 4 && (kpar > 0 || tiles <= 768)) {
            return launch_b32_mfma_kpar<FMT, 2, 2, 1>(ka, st);
        }
    }
    switch (env_int("CAMELID_HIP_B32_MFMA_SHAPE", 0)) {
        case 1: return launch_b32_mfma_p<FMT, 1, 1>(ka, n_groups, st);   // 16 tokens, 1 wave per row tile
        case 2: return launch_b32_mfma_p<FMT, 2, 1>(ka, n_groups, st);   // 32 tokens, 1 wave per row tile
        case 3: return launch_b32_mfma_p<FMT, 4, 1>(ka, n_groups, st);   // 64 tokens, 1 wave per row tile
        case 4: return launch_b32_mfma_p<FMT, 1, 2>(ka, n_groups, st);   // 32 tokens, 2 waves per row tile
        case 5: return launch_b32_mfma_p<FMT, 2, 2>(ka, n_groups, st);   // 64 tokens, 2 waves per row tile
        case 6: return launch_b32_mfma_p<FMT, 1, 4>(ka, n_groups, st);   // 64 tokens, 4 waves per row tile
        default: break;
    }
    if (grouped || ka.n_tokens <= 16) return launch_b32_mfma_p<FMT, 1, 1>(ka, n_groups, st);
    const bool few_tiles = (ka.rows + 15) / 16 < 1024;
    if (ka.n_tokens <= 32) return few_tiles ? launch_b32_mfma_p<FMT, 1, 2>(ka, n_groups, st) : launch_b32_mfma_p<FMT, 2, 1>(ka, n_groups, st);
    return few_tiles ? launch_b32_mfma_p<FMT, 1, 4>(ka, n_groups, st) : launch_b32_mfma_p<FMT, 4, 1>(ka, n_groups, st);
}

// Rows must be whole 256-value slabs whose scale octets can be read with one aligned 16-byte load.
bool b32_mfma_usable(const cml_weight *w) {
    return (w->fmt == CML_Q8_0 || w->fmt == CML_Q4_0) && w->nb > 0 && w->nb % 8 == 0 &&
           (reinterpret_cast<uintptr_t>(w->planes.p[1]) % 16 == 0) && (w->planes.row_stride[1] % 16 == 0);
}

// Batch size from which the matrix-core kernel beats the packed-dot kernel (which serves up to 8
// tokens per pass over the weight).  Measured on MI355X: 8192x2048 Q8_0, 4 / 8 tokens: 7.0 / 10.0 us
// packed dot against 10.9 us; 128256x3072 Q4_0: 62 / 105 us against 59 / 61 us.
int b32_mfma_min_tokens(int64_t rows) {
    const int forced = env_int("CAMELID_HIP_B32_MFMA_MIN_TOKENS", 0);
    if (forced > 0) return forced;
    return (rows + 15) / 16 >= 2048 ? 4 : 9;  // 128256 x 3072 Q4_0, 4 tokens: 54.6 us against 61.8 us for the packed dot
}

// Q8_0 / Q4_0 matmul on the matrix cores: plain calls, or grouped by expert (mixture of experts).
int launch_gemm_b32_mfma(const MatArgs &a, hipStream_t st) {
    const cml_weight *w = a.w;
    const bool grouped = a.group_offsets != nullptr;
    if (w->rows == 0 || a.n_tokens == 0) return CML_OK;
    if (!b32_mfma_usable(w)) return fail(CML_ERR_UNSUPPORTED, "matrix-core path needs rows of whole 256-value slabs");
    B32MfmaArgs ka{};
    ka.quants = w->planes.p[0];
    ka.q_stride = w->planes.row_stride[0];
    ka.scales = w->planes.p[1];
    ka.s_stride = w->planes.row_stride[1];
    ka.rows = static_cast<int>(grouped ? a.band_rows : w->rows);
    ka.n_slabs = static_cast<int>(w->nb / 8);
    ka.q = a.q;
    ka.xs = a.scales;
    ka.out = a.out;
    ka.n_tokens = static_cast<int>(a.n_tokens);
    ka.group_offsets = a.group_offsets;
    ka.group_rows = a.group_rows;
    ka.group_ids = a.group_ids;
    const int ng = grouped ? (a.group_ids ? a.max_active : a.n_groups) : 1;
    if (w->fmt == CML_Q8_0) return launch_b32_mfma_fmt<CML_Q8_0>(ka, ng, grouped, st);
    return launch_b32_mfma_fmt<CML_Q4_0>(ka, ng, grouped, st);
}

}  // namespace cml
