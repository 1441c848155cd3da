// Load-time re-layout (wire blocks <-> per-field planes) and the bit-exact
// dequantizers.
//
// Device layouts.  Q4_K (144 B = 9 x 16 B pieces per super-block) is
// tile-interleaved: rows are grouped in tiles of 16 (the last tile zero-padded)
// and for every (super-block, tile) -- in that order, super-block major --
// there is one contiguous 2304-byte chunk
//     [16 rows x 16 B header][16 rows x 4 x 16 B piece a][16 rows x 4 x 16 B piece b]
// where piece a / b of lane c holds nibble bytes [32c, 32c+16) / [32c+16, 32c+32)
// of that row's block -- so the three 128-bit loads of a wave that owns the
// tile each read whole consecutive cache lines.  Q8_0 (34 B), Q4_0 (18 B) and
// Q6_K (210 B) blocks are not 16-byte periodic; their fields are split into
// planes, each plane row-major by (row, block):
//   Q8_0: quants int8[rows][nb*32]            | d f16[rows][nb]
//   Q4_0: nibbles u8[rows][nb*16]             | d f16[rows][nb]
//   Q6_K: ql u8[rows][nb*128] | qh u8[rows][nb*64] | scales i8[rows][nb*16] | d f16[rows][nb]
// The split moves bytes and changes none: plane sizes add up to the wire size
// and planes_to_wire is the exact inverse (the reference keeps the same
// discipline for its own load-time re-layouts, src/cuda_resident.rs:9681-9753).
#include "cml_device.hpp"
#include "cml_host.hpp"

#pragma clang fp contract(off)

namespace cml {

Geometry geometry(int fmt) {
    switch (fmt) {
        case CML_Q8_0: return {32, 34};
        case CML_Q4_0: return {32, 18};
        case CML_Q4_K: return {256, 144};
        case CML_Q6_K: return {256, 210};
        default: return {0, 0};
    }
}

int plane_layout(int fmt, int64_t rows, int64_t nb, int64_t stride[4], size_t offset[4], size_t *total) {
    int n = 0;
    switch (fmt) {
        case CML_Q4_K: stride[0] = ((rows + 15) / 16) * 2304; n = 1; break;  // bytes between super-blocks (all tiles)
        case CML_Q8_0: stride[0] = nb * 32; stride[1] = nb * 2; n = 2; break;
        case CML_Q4_0: stride[0] = nb * 16; stride[1] = nb * 2; n = 2; break;
        case CML_Q6_K: stride[0] = nb * 128; stride[1] = nb * 64; stride[2] = nb * 16; stride[3] = nb * 2; n = 4; break;
        default: return 0;
    }
    size_t at = 0;
    for (int i = 0; i < n; i++) {
        offset[i] = at;
        const size_t units = fmt == CML_Q4_K ? static_cast<size_t>(nb) : static_cast<size_t>(rows);
        at += static_cast<size_t>(stride[i]) * units;
        at = (at + 255) & ~static_cast<size_t>(255);  // every plane starts 256-byte aligned
    }
    for (int i = n; i < 4; i++) { stride[i] = 0; offset[i] = 0; }
    *total = at;
    return n;
}

// Where the 2-byte unit at byte `off` of block (row, b) lives in the planes.
__device__ __forceinline__ void locate(int fmt, int64_t row, int64_t b, int off, const int64_t *stride,
                                       int &plane, int64_t &pos) {
    if (fmt == CML_Q6_K) {
        if (off < 128) { plane = 0; pos = row * stride[0] + b * 128 + off; }
        else if (off < 192) { plane = 1; pos = row * stride[1] + b * 64 + (off - 128); }
        else if (off < 208) { plane = 2; pos = row * stride[2] + b * 16 + (off - 192); }
        else { plane = 3; pos = row * stride[3] + b * 2; }
    } else {  // Q8_0 / Q4_0: [f16 d][payload]
        const int payload = fmt == CML_Q8_0 ? 32 : 16;
        if (off < 2) { plane = 1; pos = row * stride[1] + b * 2; }
        else { plane = 0; pos = row * stride[0] + b * payload + (off - 2); }
    }
}

struct PlanePtrs {
    uint8_t *p[4];
    int64_t stride[4];
};

// One thread per 2-byte unit of the wire image (all three block sizes are even).
template <bool TO_PLANES>
__global__ __launch_bounds__(256) void relayout_kernel(int fmt, uint8_t *wire, PlanePtrs planes, int64_t nb,
                                                       int block_bytes, int64_t n_units) {
    const int64_t u = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (u >= n_units) return;
    const int units_per_block = block_bytes / 2;
    const int64_t g = u / units_per_block;
    const int off = static_cast<int>(u - g * units_per_block) * 2;
    const int64_t row = g / nb, b = g - row * nb;
    int plane;
    int64_t pos;
    locate(fmt, row, b, off, planes.stride, plane, pos);
    uint16_t *w = reinterpret_cast<uint16_t *>(wire + u * 2);
    uint16_t *p = reinterpret_cast<uint16_t *>(planes.p[plane] + pos);
    if (TO_PLANES) *p = *w; else *w = *p;
}

// Q4_K: one thread per 16-byte piece of the wire image (9 per super-block).
template <bool TO_TILED>
__global__ __launch_bounds__(256) void q4k_tile_kernel(uint4 *wire, uint8_t *tiled, int64_t sb_stride, int64_t nb,
                                                       int64_t n_pieces, int row_skip) {
    const int64_t g = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (g >= n_pieces) return;
    const int64_t blk = g / 9;
    const int piece = static_cast<int>(g - blk * 9);
    const int64_t wire_row = blk / nb, sb = blk - wire_row * nb;
    const int64_t row = wire_row + row_skip;  // position in the tiled image (`tiled` points at the view's first tile)
    const int r = static_cast<int>(row & 15);
    uint8_t *chunk = tiled + sb * sb_stride + (row >> 4) * 2304;
    uint8_t *p;
    if (piece == 0) {
        p = chunk + r * 16;
    } else {
        const int c = (piece - 1) >> 1, half = (piece - 1) & 1;
        p = chunk + (half ? 1280 : 256) + (4 * r + c) * 16;
    }
    if (TO_TILED) *reinterpret_cast<uint4 *>(p) = wire[g]; else wire[g] = *reinterpret_cast<const uint4 *>(p);
}

static int relayout(bool to_planes, int fmt, uint8_t *wire, const Planes &pl, int64_t rows, int64_t nb, int row_skip, hipStream_t st) {
    const Geometry g = geometry(fmt);
    const int64_t nbytes = rows * nb * g.block_bytes;
    if (nbytes == 0) return CML_OK;
    if (fmt == CML_Q4_K) {
        if (reinterpret_cast<uintptr_t>(wire) & 15u) return fail(CML_ERR_INVALID, "Q4_K wire bytes must be 16-byte aligned on the device");
        const int64_t n_pieces = rows * nb * 9;
        const unsigned grid = static_cast<unsigned>((n_pieces + 255) / 256);
        uint8_t *tiled = const_cast<uint8_t *>(pl.p[0]);
        if (to_planes) {
            if (rows % 16) {  // zero the padding rows of the last tile (one chunk per super-block)
                const int64_t last = rows / 16;
                CML_HIP_TRY(hipMemset2DAsync(tiled + last * 2304, static_cast<size_t>(pl.row_stride[0]), 0, 2304, static_cast<size_t>(nb), st));
            }
            hipLaunchKernelGGL(q4k_tile_kernel<true>, dim3(grid), dim3(256), 0, st, reinterpret_cast<uint4 *>(wire), tiled, pl.row_stride[0], nb, n_pieces, 0);
        } else {
            hipLaunchKernelGGL(q4k_tile_kernel<false>, dim3(grid), dim3(256), 0, st, reinterpret_cast<uint4 *>(wire), tiled, pl.row_stride[0], nb, n_pieces, row_skip);
        }
        CML_HIP_TRY(hipGetLastError());
        return CML_OK;
    }
    PlanePtrs pp;
    for (int i = 0; i < 4; i++) { pp.p[i] = const_cast<uint8_t *>(pl.p[i]); pp.stride[i] = pl.row_stride[i]; }
    const int64_t n_units = nbytes / 2;
    const unsigned grid = static_cast<unsigned>((n_units + 255) / 256);
    if (to_planes) hipLaunchKernelGGL(relayout_kernel<true>, dim3(grid), dim3(256), 0, st, fmt, wire, pp, nb, g.block_bytes, n_units);
    else hipLaunchKernelGGL(relayout_kernel<false>, dim3(grid), dim3(256), 0, st, fmt, wire, pp, nb, g.block_bytes, n_units);
    CML_HIP_TRY(hipGetLastError());
    return CML_OK;
}

int launch_wire_to_planes(int fmt, const uint8_t *wire, int64_t rows, int64_t nb, const Planes &dst, hipStream_t st) {
    return relayout(true, fmt, const_cast<uint8_t *>(wire), dst, rows, nb, 0, st);
}

int launch_planes_to_wire(int fmt, const Planes &src, int64_t rows, int64_t nb, int row_skip, uint8_t *wire, hipStream_t st) {
    return relayout(false, fmt, wire, src, rows, nb, row_skip, st);
}

// ---- dequantize -----------------------------------------------------------------------------------
// One thread per output value; the float operations and their order are the
// reference decoders' (each product and difference rounds on its own).

// Output row -> weight row.  With `row_ids` (embedding gather) output row r decodes weight row
// row_ids[r]; an id outside the table yields -1 and the caller writes NaN instead of reading.
struct RowMap {
    const uint32_t *row_ids;  // device, or null: identity
    int64_t table_rows;
};
__device__ __forceinline__ int64_t map_row(const RowMap &m, int64_t out_row) {
    if (!m.row_ids) return out_row;
    const uint32_t id = m.row_ids[out_row];
    return id < static_cast<uint64_t>(m.table_rows) ? static_cast<int64_t>(id) : -1;
}
__device__ __forceinline__ float quiet_nan() { return __builtin_bit_cast(float, 0x7fc00000u); }

// Q8_0: scale * q (reference src/tensor/mod.rs:5365-5378).
// Q4_0: (nibble - 8) * scale (reference src/inference.rs:25698-25708).
__global__ __launch_bounds__(256) void dequant_q8q4_kernel(int fmt, Planes pl, int64_t nb, int64_t n_values, RowMap rm,
                                                           float *__restrict__ out) {
    const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i >= n_values) return;
    const int64_t g = i >> 5;
    const int j = static_cast<int>(i & 31);
    const int64_t out_row = g / nb, b = g - out_row * nb;
    const int64_t row = map_row(rm, out_row);
    if (row < 0) {
        out[i] = quiet_nan();
        return;
    }
    const float d = f16_bits_to_f32(ldg2(pl.p[1] + row * pl.row_stride[1] + b * 2));
    if (fmt == CML_Q8_0) {
        const int q = static_cast<int8_t>(pl.p[0][row * pl.row_stride[0] + b * 32 + j]);
        out[i] = d * static_cast<float>(q);
    } else {
        const uint8_t byte = pl.p[0][row * pl.row_stride[0] + b * 16 + (j & 15)];
        const int nib = (j < 16) ? (byte & 0x0f) : (byte >> 4);
        out[i] = static_cast<float>(nib - 8) * d;
    }
}

// Q4_K: (d*sc)*q - (dmin*m) (reference Q4KBlock::dequantize, src/tensor/mod.rs:5903-5924;
// q4_k_scale_min, :5997-6006).
__global__ __launch_bounds__(256) void dequant_q4k_kernel(const uint8_t *__restrict__ tiled, int64_t sb_stride,
                                                          int64_t nb, int64_t n_values, int row_skip, RowMap rm,
                                                          float *__restrict__ out) {
    const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i >= n_values) return;
    const int64_t blk = i >> 8;
    const int64_t out_row = blk / nb, sb = blk - out_row * nb;
    const int64_t mapped = map_row(rm, out_row);
    if (mapped < 0) {
        out[i] = quiet_nan();
        return;
    }
    const int64_t row = mapped + row_skip;
    const int rr = static_cast<int>(row & 15);
    const uint8_t *chunk = tiled + sb * sb_stride + (row >> 4) * 2304;
    const uint8_t *hdr = chunk + rr * 16;
    const int v = static_cast<int>(i & 255);
    const int g = v >> 5, t = v & 31;
    const float d = f16_bits_to_f32(ldg2(hdr));
    const float dmin = f16_bits_to_f32(ldg2(hdr + 2));
    const uint8_t *s = hdr + 4;
    int sc, m;
    if (g < 4) {
        sc = s[g] & 63;
        m = s[g + 4] & 63;
    } else {
        sc = (s[g + 4] & 0x0f) | ((s[g - 4] >> 6) << 4);
        m = (s[g + 4] >> 4) | ((s[g] >> 6) << 4);
    }
    // nibble byte t of chunk c = g/2: piece a holds bytes 0..15, piece b bytes 16..31
    const uint8_t byte = chunk[((t & 16) ? 1280 : 256) + (4 * rr + (g >> 1)) * 16 + (t & 15)];
    const int q = (g & 1) ? (byte >> 4) : (byte & 0x0f);
    const float scale = d * static_cast<float>(sc);
    const float min = dmin * static_cast<float>(m);
    out[i] = scale * static_cast<float>(q) - min;
}

// Q6_K: (d*sc)*q (reference Q6KBlock::dequantize, src/tensor/mod.rs:6039-6066).
__global__ __launch_bounds__(256) void dequant_q6k_kernel(Planes pl, int64_t nb, int64_t n_values, RowMap rm,
                                                          float *__restrict__ out) {
    const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i >= n_values) return;
    const int64_t g = i >> 8;
    const int v = static_cast<int>(i & 255);
    const int64_t out_row = g / nb, b = g - out_row * nb;
    const int64_t row = map_row(rm, out_row);
    if (row < 0) {
        out[i] = quiet_nan();
        return;
    }
    const int half = v >> 7, r = v & 127, quarter = r >> 5, l = r & 31;
    const uint8_t qlb = pl.p[0][row * pl.row_stride[0] + b * 128 + 64 * half + l + ((quarter & 1) ? 32 : 0)];
    const uint8_t qhb = pl.p[1][row * pl.row_stride[1] + b * 64 + 32 * half + l];
    const int nib = (quarter >= 2) ? (qlb >> 4) : (qlb & 0x0f);
    const int q = (nib | (((qhb >> (2 * quarter)) & 3) << 4)) - 32;
    const int sc = static_cast<int8_t>(pl.p[2][row * pl.row_stride[2] + b * 16 + (v >> 4)]);
    const float d = f16_bits_to_f32(ldg2(pl.p[3] + row * pl.row_stride[3] + b * 2));
    out[i] = d * static_cast<float>(sc) * static_cast<float>(q);
}

// Decodes `n_rows` rows: the weight's own rows in order (row_ids null), or the rows row_ids[0..n_rows).
static int dequantize_rows(const cml_weight *w, const uint32_t *row_ids, int64_t n_rows, float *out, hipStream_t st) {
    const int64_t n_values = n_rows * w->cols;
    if (n_values == 0) return CML_OK;
    const unsigned grid = static_cast<unsigned>((n_values + 255) / 256);
    const RowMap rm{row_ids, w->rows};
    switch (w->fmt) {
        case CML_Q8_0:
        case CML_Q4_0:
            hipLaunchKernelGGL(dequant_q8q4_kernel, dim3(grid), dim3(256), 0, st, w->fmt, w->planes, w->nb, n_values, rm, out);
            break;
        case CML_Q4_K:
            hipLaunchKernelGGL(dequant_q4k_kernel, dim3(grid), dim3(256), 0, st, w->planes.p[0], w->planes.row_stride[0], w->nb, n_values, w->row_skip, rm, out);
            break;
        case CML_Q6_K:
            hipLaunchKernelGGL(dequant_q6k_kernel, dim3(grid), dim3(256), 0, st, w->planes, w->nb, n_values, rm, out);
            break;
        default:
            return fail(CML_ERR_INVALID, "unknown format %d", w->fmt);
    }
    CML_HIP_TRY(hipGetLastError());
    return CML_OK;
}

int launch_dequantize(const cml_weight *w, float *out, hipStream_t st) { return dequantize_rows(w, nullptr, w->rows, out, st); }

int launch_embed_gather(const cml_weight *table, const uint32_t *token_ids, int64_t n_tokens, float *out, hipStream_t st) {
    return dequantize_rows(table, token_ids, n_tokens, out, st);
}

// Greedy argmax of each row: strict >, the first index wins ties, starting from (-3.4e38, index 0)
// like the reference's scan (argmax_f32, src/cuda_resident.rs:6391-6417) -- values that are not
// greater than -3.4e38 (and NaNs) never win.  One workgroup of 1024 threads per row.
__global__ __launch_bounds__(1024) void argmax_f32_kernel(const float *__restrict__ logits, int64_t n, uint32_t *__restrict__ out_idx) {
    __shared__ float sval[16];
    __shared__ int sidx[16];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const float *row = logits + static_cast<int64_t>(blockIdx.x) * n;
    float best = -3.4e38f;
    int besti = 0;
    // pairs meet keeping the greater value, the lower index on equal values
    auto meet = [](float &bv, int &bi, float ov, int oi) __attribute__((always_inline)) {
        if (ov > bv || (ov == bv && oi < bi)) {
            bv = ov;
            bi = oi;
        }
    };
    // The row is read as 16-byte pieces, four of them in flight per thread: up to three leading
    // values before the first aligned address and the values after the last whole piece are taken
    // one by one.  Every thread meets ascending indices in the body, so strict > keeps its first
    // maximum; the odd ends go through meet(), which orders equal values by index.
    const int64_t head = min<int64_t>(n, static_cast<int64_t>((16 - (reinterpret_cast<uintptr_t>(row) & 15)) & 15) >> 2);
    const int64_t n4 = (n - head) >> 2;
    const float4 *row4 = reinterpret_cast<const float4 *>(row + head);
    if (tid < head) meet(best, besti, row[tid], tid);
    auto take4 = [&](const float4 &v, int64_t p) __attribute__((always_inline)) {
        const int i0 = static_cast<int>(head + 4 * p);
        if (v.x > best) { best = v.x; besti = i0; }
        if (v.y > best) { best = v.y; besti = i0 + 1; }
        if (v.z > best) { best = v.z; besti = i0 + 2; }
        if (v.w > best) { best = v.w; besti = i0 + 3; }
    };
    int64_t p = tid;
    for (; p + 3 * 1024 < n4; p += 4 * 1024) {
        const float4 a = row4[p], b = row4[p + 1024], c = row4[p + 2048], d = row4[p + 3072];
        take4(a, p);
        take4(b, p + 1024);
        take4(c, p + 2048);
        take4(d, p + 3072);
    }
    for (; p < n4; p += 1024) take4(row4[p], p);
    for (int64_t i = head + 4 * n4 + tid; i < n; i += 1024) meet(best, besti, row[i], static_cast<int>(i));
    for (int m = 1; m < 64; m <<= 1) meet(best, besti, __shfl_xor(best, m), __shfl_xor(besti, m));
    if (lane == 0) {
        sval[wave] = best;
        sidx[wave] = besti;
    }
    __syncthreads();
    if (tid == 0) {
        for (int k = 1; k < 16; k++) meet(best, besti, sval[k], sidx[k]);
        out_idx[blockIdx.x] = static_cast<uint32_t>(besti);
    }
}

int launch_argmax_f32(const float *logits, int64_t n_rows, int64_t n, uint32_t *out_idx, hipStream_t st) {
    if (n_rows == 0) return CML_OK;
    hipLaunchKernelGGL(argmax_f32_kernel, dim3(static_cast<unsigned>(n_rows)), dim3(1024), 0, st, logits, n, out_idx);
    CML_HIP_TRY(hipGetLastError());
    return CML_OK;
}

}  // namespace cml
