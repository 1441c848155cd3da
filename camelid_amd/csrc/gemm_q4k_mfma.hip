// Q4_K x Q8_K small-batch matmul on the int8 matrix cores (gfx950), for
// 16 <= n tokens: speculative-verify chunks and short prefill.
//
// Arithmetic: identical, cell by cell, to the matvec kernel (gemv_q4k.hip;
// reference q4_k_dot_scalar, src/diffusion_gemma/refmath.rs:504-562):
//     per super-block:  acc = fma(-(yd*dmin), (float)P, acc);  acc = fma(yd*d, (float)S, acc)
//     S = sum_g sc_g * sum_{t<32} q*y      P = sum_g m_g * sum_{t<32} y
//
// Every 32-value sub-block has its own 6-bit scale and sc*q (up to 945) does
// not fit an int8 operand, so a matrix-core contraction must not run across a
// sub-block boundary (the reference's tensor-core precedent obeys the same
// rule for Q4_0: one K=32 MMA per block into a zeroed accumulator,
// src/cuda_resident.rs:2641-2654).  gfx950's full-rate int8 instruction is
// v_mfma_i32_16x16x64_i8 (K = 64 = TWO sub-blocks: the low and the high nibbles
// of one 32-byte chunk of the block).  The two sub-blocks are kept apart on
// the M side instead: the 16 A-rows are 8 tokens x 2 halves, and A-row
// (token t, half h) carries y only in the 32 k's of half h and zeros in the
// others,
//     A[(t,h)][(h',j)] = (h == h') ? y_t[32(2c+h)+j] : 0      (from LDS)
//     B[(h',j)][n]     = nibble j of sub-block 2c+h' of row n   (registers)
//     D[(t,h)][n]      = dot of sub-block 2c+h, token t, row n
// Lane L of D holds row n = L%16 and four A-rows 4*(L/16)..+3, i.e. ONE weight
// row, ONE half and four tokens: scaling by sc_{2c+h} is four integer
// multiply-adds per instruction, the two halves of a cell meet through one
// v_permlane32_swap per pair of values, and the f32 chain of each cell then
// stays inside one lane, in super-block order.  The mins side rides the same A
// operand: a second MFMA per chunk whose B operand is the sub-block's 6-bit min
// replicated gives m_g * sum(y), accumulated over the four chunks in the matrix
// core.
//
// A workgroup is 4 waves: 4/TB consecutive 16-row tiles x TB token blocks of
// 8*GPW tokens, sharing the staged activations of NTOK = 8*GPW*TB tokens.  K is
// walked in phases of KC = 128/NTOK super-blocks: a phase's activations (rows
// padded by 16 B against bank conflicts) sit in one of two LDS buffers; the next
// phase's loads are issued at the start of the current phase, ahead of the
// weight loads, and stored at its end, so the only barriers are the phase
// boundaries.  Weights (tile-interleaved layout, layout.hip) are double-buffered
// in registers two super-blocks at a time.  When the matvec kernel would split K
// for this weight shape, the same split is reproduced inside the lane (the
// chain restarts at the split points and the partial chains are added left to
// right), so every cell equals the matvec result bit for bit.
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
    const int8_t *q;    // [n_tokens][n_sb*256]
    const float *yd;    // [n_tokens][n_sb]
    float *out;         // [n_tokens][rows]
    int n_tokens;
    int ksplit;         // association to reproduce (see gemv_q4k.hip)
};

struct MfmaWeights {
    uint4 hdr;
    uint4 piece[4];  // this lane's 16 nibble bytes of each of the 4 chunks
};

// hdr_ptr / piece_ptr already include the lane's offsets inside a chunk; `off` = sb * sb_stride.
__device__ __forceinline__ void mfma_load_weights(MfmaWeights &r, const uint8_t *hdr_ptr, const uint8_t *piece_ptr,
                                                  int64_t off) {
    r.hdr = ldg16(hdr_ptr + off);
#pragma unroll
    for (int c = 0; c < 4; c++) r.piece[c] = ldg16(piece_ptr + off + c * 16);
}

__device__ __forceinline__ v4i as_v4i(const uint4 &v) {
    v4i r = {static_cast<int>(v.x), static_cast<int>(v.y), static_cast<int>(v.z), static_cast<int>(v.w)};
    return r;
}

// Exchange the upper 32 lanes of `a` with the lower 32 lanes of `b`.
__device__ __forceinline__ void swap_halves(int &a, int &b) {
    const auto r = __builtin_amdgcn_permlane32_swap(a, b, false, false);
    a = r[0];
    b = r[1];
}

template <int GPW, int TB>
__global__ __launch_bounds__(256) void gemm_q4k_mfma_kernel(Q4KMfmaArgs a) {
    constexpr int NTOK = 8 * GPW * TB;               // tokens staged per workgroup
    constexpr int KC = 128 / NTOK;                   // super-blocks per phase (a buffer is always 128 token-super-blocks)
    constexpr int RT = 4 / TB;                       // row tiles per workgroup
    constexpr int kBufBytes = KC * NTOK * kSlabRow;
    constexpr int nthreads = 256;
    constexpr int kPieces = NTOK * 16;               // 16-byte pieces of one super-block of all tokens
    constexpr int kPer = kPieces / nthreads;         // 1, 2 or 4
    constexpr int U = KC >= 4 ? 2 : 1;               // weight super-blocks per register buffer (a phase is a whole number of buffer pairs)
    static_assert(KC % (2 * U) == 0 && kPer >= 1, "phase / staging shape");
    extern __shared__ uint4 smem[];
    uint8_t *buf0 = reinterpret_cast<uint8_t *>(smem);  // [KC][NTOK][kSlabRow]
    uint8_t *buf1 = buf0 + kBufBytes;
    uint8_t *zeros = buf1 + kBufBytes;                   // kSlabRow bytes of zeros: the A operand's "other half"
    float *yds = reinterpret_cast<float *>(zeros + kSlabRow);  // [n_sb][NTOK]

    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
    const int n_sb = a.n_sb;
    const int n = lane & 15, kq = lane >> 4;         // B/D column (weight row in tile) and k-quarter / A-row quad
    const int half = kq >> 1;                        // which sub-block of a chunk this lane's B bytes and D values belong to
    const int rt = wave / TB, tb = wave - rt * TB;
    const int n_tiles = (a.rows + 15) / 16;
    const int tile = blockIdx.x * RT + rt;
    const int row = tile * 16 + n;
    const uint8_t *wtile = a.w + static_cast<int64_t>(min(tile, n_tiles - 1)) * 2304;
    const int tok0 = blockIdx.y * NTOK;                    // first token of this workgroup
    const int n_here = min(NTOK, a.n_tokens - tok0);       // >= 1 by construction of the grid
    const int8_t *q = a.q + static_cast<int64_t>(tok0) * n_sb * 256;
    const float *yd = a.yd + static_cast<int64_t>(tok0) * n_sb;

    for (int i = tid; i < kSlabRow / 4; i += nthreads) reinterpret_cast<uint32_t *>(zeros)[i] = 0u;
    // activation scales: yds[sb][token] (tokens past the end repeat the last one; their cells are not stored)
    for (int i = tid; i < n_sb * NTOK; i += nthreads) {
        const int sb = i / NTOK, t = i - sb * NTOK;
        yds[i] = yd[min(t, n_here - 1) * n_sb + sb];
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
        stage_src[k] = reinterpret_cast<const v4i *>(q + static_cast<int64_t>(min(t, n_here - 1)) * n_sb * 256) + piece;
        stage_dst[k] = t * kSlabRow + piece * 16;
    }
    v4i sreg[KC][kPer];
    auto stage_load = [&](int p0) {  // the KC super-blocks starting at p0
#pragma unroll
        for (int s = 0; s < KC; s++) {
            const int off = min(p0 + s, n_sb - 1) * 16;  // in uint4 units
#pragma unroll
            for (int k = 0; k < kPer; k++) sreg[s][k] = stage_src[k][off];
        }
    };
    auto stage_store = [&](uint8_t *buf) {
#pragma unroll
        for (int s = 0; s < KC; s++)
#pragma unroll
            for (int k = 0; k < kPer; k++) *reinterpret_cast<v4i *>(buf + s * (NTOK * kSlabRow) + stage_dst[k]) = sreg[s][k];
    };

    // Lane constants.
    const uint8_t *w_hdr = wtile + n * 16;
    const uint8_t *w_piece = wtile + ((kq & 1) ? 1280 : 256) + n * 64;   // piece a (values 0..15) or b (16..31) of chunk 0
    const int nib_shift = 4 * half;                                       // low nibbles = sub-block 2c, high = 2c+1
    // A operand: this lane is A-row m = lane & 15 = (token t = m & 7, half hm = m >> 3), k-quarter kq.
    const int am = lane & 15, at = am & 7, ahm = am >> 3;
    const bool a_live = (kq >> 1) == ahm;
    const int a_off = at * kSlabRow + 32 * ahm + 16 * (kq & 1);  // + 64c, + token-group and slot offsets
    // D values v = 0..3 of this lane: tokens 4*(kq & 1) + v of the group, sub-block half `half`.
    // After the halves are exchanged a lane finishes two cells: lower half-wave v = 0,1; upper v = 2,3.
    const int cell_tok = 4 * (kq & 1) + 2 * half;  // + {0,1}
    const int sc_shift = 8 * half;                  // byte `half` / `2+half` of the scale words

    MfmaWeights wa[U], wb[U];
    auto loadU = [&](MfmaWeights (&w)[U], int sb0) {
#pragma unroll
        for (int u = 0; u < U; u++) mfma_load_weights(w[u], w_hdr, w_piece, min(sb0 + u, n_sb - 1) * a.sb_stride);
    };

    stage_load(0);
    loadU(wa, 0);
    stage_store(buf0);
    __syncthreads();

    float acc[GPW][2], total[GPW][2];
#pragma unroll
    for (int g = 0; g < GPW; g++) { acc[g][0] = acc[g][1] = 0.0f; total[g][0] = total[g][1] = 0.0f; }
    int part = 0;                                            // index of the K-split part being accumulated
    int next_cut = a.ksplit <= 1 ? n_sb : n_sb / a.ksplit;  // first super-block of part 1

    // One super-block of this wave's tile against its token block.
    auto step = [&](const MfmaWeights &w0, int sb, const uint8_t *slot) {
        if (sb == next_cut) {  // the matvec kernel's K-split point: close the partial chain
#pragma unroll
            for (int g = 0; g < GPW; g++)
#pragma unroll
                for (int j = 0; j < 2; j++) {
                    total[g][j] = (part == 0) ? acc[g][j] : total[g][j] + acc[g][j];
                    acc[g][j] = 0.0f;
                }
            part++;
            next_cut = (part + 1) * n_sb / a.ksplit;
        }
        // this row's scales and mins of the sub-blocks {half, 2+half, 4+half, 6+half}
        // (reference q4_k_scale_min, src/tensor/mod.rs:5997-6006)
        uint32_t sc03, sc47, m03, m47;
        q4k_unpack_scales(w0.hdr.y, w0.hdr.z, w0.hdr.w, sc03, sc47, m03, m47);
        const float dw = f16_bits_to_f32(w0.hdr.x & 0xffffu);
        const float dminw = f16_bits_to_f32(w0.hdr.x >> 16);
        int sc[4];
        v4i bq[4], bm[4];
#pragma unroll
        for (int c = 0; c < 4; c++) {
            const uint32_t scw = (c < 2) ? sc03 : sc47, mw = (c < 2) ? m03 : m47;
            const int sh = sc_shift + 16 * (c & 1);
            sc[c] = (scw >> sh) & 0xff;
            const uint32_t m = (mw >> sh) & 0xff;
            const uint32_t m2 = m | (m << 8);
            const int m4 = static_cast<int>(m2 | (m2 << 16));
            bm[c] = v4i{m4, m4, m4, m4};
            const uint4 &pc = w0.piece[c];
            bq[c] = v4i{static_cast<int>((pc.x >> nib_shift) & 0x0f0f0f0fu), static_cast<int>((pc.y >> nib_shift) & 0x0f0f0f0fu),
                        static_cast<int>((pc.z >> nib_shift) & 0x0f0f0f0fu), static_cast<int>((pc.w >> nib_shift) & 0x0f0f0f0fu)};
        }
        const float *ydp = yds + sb * NTOK + tb * (8 * GPW) + cell_tok;
#pragma unroll
        for (int g = 0; g < GPW; g++) {
            const uint8_t *ybase = slot + (tb * GPW + g) * (8 * kSlabRow) + a_off;
            int S[4] = {0, 0, 0, 0};
            v4i P = {0, 0, 0, 0};
#pragma unroll
            for (int c = 0; c < 4; c++) {
                const uint8_t *ap = a_live ? ybase + 64 * c : zeros;
                const v4i av = as_v4i(*reinterpret_cast<const uint4 *>(ap));
                const v4i zero = {0, 0, 0, 0};
                const v4i D = __builtin_amdgcn_mfma_i32_16x16x64_i8(av, bq[c], zero, 0, 0, 0);
                P = __builtin_amdgcn_mfma_i32_16x16x64_i8(av, bm[c], P, 0, 0, 0);
#pragma unroll
                for (int v = 0; v < 4; v++) S[v] += __mul24(D[v], sc[c]);
            }
            // bring the two halves of each cell together: lower lanes end with cells v = 0,1, upper with v = 2,3
            int p0 = P[0], p1 = P[1], p2 = P[2], p3 = P[3];
            swap_halves(S[0], S[2]);
            swap_halves(S[1], S[3]);
            swap_halves(p0, p2);
            swap_halves(p1, p3);
            const int s_cell[2] = {S[0] + S[2], S[1] + S[3]};
            const int p_cell[2] = {p0 + p2, p1 + p3};
            const float2 ydv = *reinterpret_cast<const float2 *>(ydp + 8 * g);
            const float yv[2] = {ydv.x, ydv.y};
#pragma unroll
            for (int j = 0; j < 2; j++) {
                const float Dd = yv[j] * dw;
                const float Mm = yv[j] * dminw;
                acc[g][j] = __builtin_fmaf(-Mm, static_cast<float>(p_cell[j]), acc[g][j]);
                acc[g][j] = __builtin_fmaf(Dd, static_cast<float>(s_cell[j]), acc[g][j]);
            }
        }
    };

    // Phases of KC super-blocks.  Order of issue at a phase start: the next
    // phase's activation loads (L2 hits) first, so that the stores closing the
    // phase never wait behind the long-latency weight loads (vmcnt is in order).
    for (int p0 = 0, ph = 0; p0 < n_sb; p0 += KC, ph++) {
        uint8_t *cur = (ph & 1) ? buf1 : buf0;
        uint8_t *nxt = (ph & 1) ? buf0 : buf1;
        // unconditional (the last phase re-reads clamped super-blocks into the idle buffer): keeps
        // the staging values in registers and the loads in straight-line code
        stage_load(p0 + KC);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int s0 = 0; s0 < KC; s0 += 2 * U) {
            if (p0 + s0 < n_sb) {
                if (p0 + s0 + U < n_sb) loadU(wb, p0 + s0 + U);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int u = 0; u < U; u++)
                    if (p0 + s0 + u < n_sb) step(wa[u], p0 + s0 + u, cur + (s0 + u) * (NTOK * kSlabRow));
            }
            if (p0 + s0 + U < n_sb) {
                if (p0 + s0 + 2 * U < n_sb) loadU(wa, p0 + s0 + 2 * U);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int u = 0; u < U; u++)
                    if (p0 + s0 + U + u < n_sb) step(wb[u], p0 + s0 + U + u, cur + (s0 + U + u) * (NTOK * kSlabRow));
            }
        }
        stage_store(nxt);
        __syncthreads();  // next phase complete in `nxt`, everyone done with `cur`
    }

    if (tile < n_tiles && row < a.rows) {
#pragma unroll
        for (int g = 0; g < GPW; g++)
#pragma unroll
            for (int j = 0; j < 2; j++) {
                const int t = tb * (8 * GPW) + 8 * g + cell_tok + j;
                if (t < n_here) {
                    const float v = (part == 0) ? acc[g][j] : total[g][j] + acc[g][j];
                    a.out[static_cast<int64_t>(tok0 + t) * a.rows + row] = v;
                }
            }
    }
}

int q4k_ksplit_for(int64_t rows, int64_t n_sb);  // gemv_q4k.hip: the matvec kernel's K-split policy

template <int GPW, int TB>
static int launch_mfma(const Q4KMfmaArgs &ka, hipStream_t st) {
    constexpr int NTOK = 8 * GPW * TB, RT = 4 / TB;
    const int n_tiles = (ka.rows + 15) / 16;
    const unsigned gx = static_cast<unsigned>((n_tiles + RT - 1) / RT);
    const unsigned gy = static_cast<unsigned>((ka.n_tokens + NTOK - 1) / NTOK);
    const size_t lds = 2 * static_cast<size_t>(128) * kSlabRow + kSlabRow + static_cast<size_t>(ka.n_sb) * NTOK * 4;
    if (lds > 160 * 1024) return fail(CML_ERR_UNSUPPORTED, "Q4_K matrix-core path: %d super-blocks exceed the LDS budget", ka.n_sb);
    static bool raised = false;  // per instantiation: allow more than 64 KB of dynamic LDS once
    if (!raised) {
        CML_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(&gemm_q4k_mfma_kernel<GPW, TB>),
                                        hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
        raised = true;
    }
    hipLaunchKernelGGL((gemm_q4k_mfma_kernel<GPW, TB>), dim3(gx, gy), dim3(256), lds, st, ka);
    CML_HIP_TRY(hipGetLastError());
    return CML_OK;
}

// Plain (ungrouped) Q4_K matmul for n_tokens >= 16 on the matrix cores.
int launch_gemm_q4k_mfma(const MatArgs &a, hipStream_t st) {
    const cml_weight *w = a.w;
    Q4KMfmaArgs ka;
    ka.w = w->planes.p[0];
    ka.sb_stride = w->planes.row_stride[0];
    ka.rows = static_cast<int>(w->rows);
    ka.n_sb = static_cast<int>(w->nb);
    ka.ksplit = q4k_ksplit_for(w->rows, w->nb);
    ka.q = a.q;
    ka.yd = a.scales;
    ka.out = a.out;
    ka.n_tokens = static_cast<int>(a.n_tokens);
    // Workgroup shape: tokens staged per workgroup x how they are split over waves.
    // Default: 16 tokens (n <= 16) or 32 tokens per workgroup, one wave per row tile; more
    // tokens = more workgroup columns (grid.y), each a pass over the weight.  The other
    // shapes stay selectable for tuning.
    const int shape = env_int("CAMELID_HIP_Q4K_MFMA_SHAPE", 0);
    switch (shape) {
        case 1: return launch_mfma<2, 1>(ka, st);   // 16 tokens, 1 wave per row tile
        case 2: return launch_mfma<1, 2>(ka, st);   // 16 tokens, 2 waves per row tile
        case 3: return launch_mfma<4, 1>(ka, st);   // 32 tokens, 1 wave per row tile
        case 4: return launch_mfma<2, 2>(ka, st);   // 32 tokens, 2 waves per row tile
        case 5: return launch_mfma<4, 2>(ka, st);   // 64 tokens, 2 waves per row tile
        case 6: return launch_mfma<2, 4>(ka, st);   // 64 tokens, 4 waves per row tile
        case 7: return launch_mfma<1, 4>(ka, st);   // 32 tokens, 4 waves per row tile
        default: break;
    }
    // measured on MI355X at 14336x4096: one wave per row tile is fastest at both sizes
    if (a.n_tokens > 16) return launch_mfma<4, 1>(ka, st);
    return launch_mfma<2, 1>(ka, st);
}

}  // namespace cml
