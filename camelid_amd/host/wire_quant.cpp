// WireQuant, SharedActivation and SharedActivationBatch over the C ABI
// (reference src/gemma4_runtime.rs:660-1150, :1288-1340).  Every arithmetic
// step happens on the device; this file only moves buffers and checks shapes.
#include <cstring>

#include "../../include/camelid_hip.h"
#include "camelid_host.hpp"

namespace camelid {

namespace {

[[noreturn]] void device_error(const char *what) {
    throw BackendError(BackendError::Kind::Device, std::string(what) + ": " + cml_last_error());
}
void dev(int rc, const char *what) {
    if (rc != CML_OK) device_error(what);
}
void ensure_device() {
    if (cml_available() != 1) device_error("no usable gfx950 device");
    dev(cml_init(-1), "cml_init");
}

}  // namespace

size_t values_per_block(WireFormat f) { return (f == WireFormat::Q8_0 || f == WireFormat::Q4_0) ? 32 : 256; }
size_t bytes_per_block(WireFormat f) {
    switch (f) {
        case WireFormat::Q8_0: return 34;
        case WireFormat::Q4_0: return 18;
        case WireFormat::Q4K: return 144;
        default: return 210;
    }
}
int ggml_type_id(WireFormat f) {
    switch (f) {
        case WireFormat::Q8_0: return CML_Q8_0;
        case WireFormat::Q4_0: return CML_Q4_0;
        case WireFormat::Q4K: return CML_Q4_K;
        default: return CML_Q6_K;
    }
}

// ---- DeviceScratch ------------------------------------------------------------------------------------

DeviceScratch::~DeviceScratch() {
    if (ptr_) cml_dev_free(ptr_);
}

void *DeviceScratch::reserve(size_t nbytes) {
    if (nbytes <= cap_ && ptr_) return ptr_;
    if (ptr_) {
        cml_dev_free(ptr_);
        ptr_ = nullptr;
        cap_ = 0;
    }
    dev(cml_dev_alloc(nbytes, &ptr_), "cml_dev_alloc");
    cap_ = nbytes;
    return ptr_;
}

// ---- SharedActivation -----------------------------------------------------------------------------------

SharedActivation::SharedActivation(const float *x, size_t len) : x_(x), len_(len) {}

const float *SharedActivation::x_dev() const {
    if (!have_x_) {
        ensure_device();
        const size_t n = rows_ * len_ * sizeof(float);
        xd_.reserve(n ? n : 16);
        dev(cml_memcpy_h2d(xd_.get(), x_, n, nullptr), "cml_memcpy_h2d");
        have_x_ = true;
    }
    return static_cast<const float *>(xd_.get());
}

std::pair<const int8_t *, const float *> SharedActivation::q8_0_dev() const {
    if (!have_q0_) {
        if (len_ % 32 != 0) throw BackendError(BackendError::Kind::InvalidTensorData, "activation length is not whole Q8_0 blocks");
        const float *xd = x_dev();
        q0_.reserve(rows_ * len_ + 16);
        s0_.reserve(rows_ * (len_ / 32) * sizeof(float) + 16);
        dev(cml_quantize_q8_0(xd, static_cast<int64_t>(rows_), static_cast<int64_t>(len_), static_cast<int8_t *>(q0_.get()),
                              static_cast<float *>(s0_.get()), nullptr),
            "cml_quantize_q8_0");
        have_q0_ = true;
    }
    return {static_cast<const int8_t *>(q0_.get()), static_cast<const float *>(s0_.get())};
}

std::pair<const int8_t *, const float *> SharedActivation::q8_k_dev() const {
    if (!have_qk_) {
        if (len_ % 256 != 0) throw BackendError(BackendError::Kind::InvalidTensorData, "activation length is not whole Q8_K super-blocks");
        const float *xd = x_dev();
        qk_.reserve(rows_ * len_ + 16);
        sk_.reserve(rows_ * (len_ / 256) * sizeof(float) + 16);
        dev(cml_quantize_q8_k(xd, static_cast<int64_t>(rows_), static_cast<int64_t>(len_), static_cast<int8_t *>(qk_.get()),
                              static_cast<float *>(sk_.get()), nullptr),
            "cml_quantize_q8_k");
        have_qk_ = true;
    }
    return {static_cast<const int8_t *>(qk_.get()), static_cast<const float *>(sk_.get())};
}

std::vector<Q8_0Block> SharedActivation::q8_0() const {
    const auto [q, s] = q8_0_dev();
    const size_t nb = rows_ * len_ / 32;
    std::vector<int8_t> hq(nb * 32);
    std::vector<float> hs(nb);
    dev(cml_memcpy_d2h(hq.data(), q, hq.size(), nullptr), "cml_memcpy_d2h");
    dev(cml_memcpy_d2h(hs.data(), s, hs.size() * sizeof(float), nullptr), "cml_memcpy_d2h");
    std::vector<Q8_0Block> out(nb);
    for (size_t b = 0; b < nb; b++) {
        out[b].scale = hs[b];
        std::memcpy(out[b].quants, hq.data() + b * 32, 32);
    }
    return out;
}

std::vector<Q8KBlock> SharedActivation::q8_k() const {
    const auto [q, s] = q8_k_dev();
    const size_t nb = rows_ * len_ / 256;
    std::vector<int8_t> hq(nb * 256);
    std::vector<float> hs(nb);
    dev(cml_memcpy_d2h(hq.data(), q, hq.size(), nullptr), "cml_memcpy_d2h");
    dev(cml_memcpy_d2h(hs.data(), s, hs.size() * sizeof(float), nullptr), "cml_memcpy_d2h");
    std::vector<Q8KBlock> out(nb);
    for (size_t b = 0; b < nb; b++) {
        out[b].d = hs[b];
        std::memcpy(out[b].qs, hq.data() + b * 256, 256);
    }
    return out;
}

namespace {
std::vector<float> flatten(const std::vector<std::vector<float>> &xs) {
    std::vector<float> flat;
    const size_t len = xs.empty() ? 0 : xs[0].size();
    flat.reserve(xs.size() * len);
    for (const auto &x : xs) {
        if (x.size() != len) throw BackendError(BackendError::Kind::InvalidTensorData, "activation rows of a batch differ in length");
        flat.insert(flat.end(), x.begin(), x.end());
    }
    return flat;
}
}  // namespace

SharedActivationBatch::SharedActivationBatch(const std::vector<std::vector<float>> &xs)
    : flat_(flatten(xs)), rows_(xs.size()), len_(xs.empty() ? 0 : xs[0].size()), inner_(flat_.data(), len_) {
    inner_.rows_ = rows_;
}

// ---- WireQuant --------------------------------------------------------------------------------------------

WireQuant WireQuant::from_gguf(const GgufFile &file, const GgufWireMmap &mmap, const std::string &name) {
    const GgufTensorDescriptor *t = file.tensor(name);
    if (!t) throw BackendError(BackendError::Kind::InvalidTensorData, "tensor " + name + " is not in " + file.path);
    WireFormat format;
    switch (t->tensor_type) {
        case CML_Q8_0: format = WireFormat::Q8_0; break;
        case CML_Q4_0: format = WireFormat::Q4_0; break;
        case CML_Q4_K: format = WireFormat::Q4K; break;
        case CML_Q6_K: format = WireFormat::Q6K; break;
        default:
            throw BackendError(BackendError::Kind::UnsupportedTensorType,
                               "tensor " + name + " has GGML type " + std::to_string(t->tensor_type) +
                                   "; the quantized matvec path serves Q8_0, Q4_0, Q4_K and Q6_K");
    }
    size_t elements = 1;
    for (uint64_t d : t->dimensions) elements *= static_cast<size_t>(d);
    const uint8_t *bytes = mmap.bytes(t->absolute_offset, t->n_bytes);
    if (!bytes) throw BackendError(BackendError::Kind::InvalidTensorData, "tensor " + name + " lies outside the mapped file");
    WireQuant w = from_wire(format, bytes, static_cast<size_t>(t->n_bytes), elements, name);
    // the directory already fixes the row length: upload now and drop the host copy
    w.rows_for(static_cast<size_t>(t->dimensions[0]));
    return w;
}

WireQuant WireQuant::from_wire(WireFormat format, const uint8_t *bytes, size_t n_bytes, size_t element_count, const std::string &name) {
    if (element_count % values_per_block(format) != 0)
        throw BackendError(BackendError::Kind::InvalidTensorData,
                           "tensor " + name + " element count " + std::to_string(element_count) + " is not block-aligned");
    const size_t expected = element_count / values_per_block(format) * bytes_per_block(format);
    if (n_bytes != expected)
        throw BackendError(BackendError::Kind::InvalidTensorData,
                           "tensor " + name + " has " + std::to_string(n_bytes) + " wire bytes; expected " + std::to_string(expected));
    WireQuant w;
    w.format_ = format;
    w.element_count_ = element_count;
    w.name_ = name;
    w.wire_.assign(bytes, bytes + n_bytes);
    return w;
}

WireQuant::WireQuant(WireQuant &&o) noexcept { *this = std::move(o); }

void WireQuant::release() {
    for (auto &b : bands_) cml_weight_free(b.second);
    bands_.clear();
    if (weight_) cml_weight_free(weight_);
    weight_ = nullptr;
    if (block_view_) cml_weight_free(block_view_);
    block_view_ = nullptr;
}

WireQuant &WireQuant::operator=(WireQuant &&o) noexcept {
    if (this != &o) {
        release();
        format_ = o.format_;
        element_count_ = o.element_count_;
        name_ = std::move(o.name_);
        wire_ = std::move(o.wire_);
        weight_ = o.weight_;
        block_view_ = o.block_view_;
        cols_ = o.cols_;
        bands_ = std::move(o.bands_);
        o.weight_ = nullptr;
        o.block_view_ = nullptr;
        o.bands_.clear();
    }
    return *this;
}

WireQuant::~WireQuant() { release(); }

// Uploads on first use (the reference's WireQuant learns the row length from its callers too)
// and returns the row count for that row length.
size_t WireQuant::rows_for(size_t in_dim) const {
    if (in_dim == 0 || in_dim % values_per_block(format_) != 0 || element_count_ % in_dim != 0)
        throw BackendError(BackendError::Kind::InvalidTensorData,
                           "tensor " + name_ + ": rows of " + std::to_string(in_dim) + " values do not tile " + std::to_string(element_count_) + " elements in whole blocks");
    if (!weight_) {
        ensure_device();
        const size_t rows = element_count_ / in_dim;
        dev(cml_weight_upload(ggml_type_id(format_), static_cast<int64_t>(rows), static_cast<int64_t>(in_dim), wire_.data(), wire_.size(), &weight_),
            "cml_weight_upload");
        cols_ = in_dim;
        if (block_view_) cml_weight_free(block_view_);  // the row layout serves dequantize_elements from here on
        block_view_ = nullptr;
        auto *self = const_cast<WireQuant *>(this);
        self->wire_.clear();
        self->wire_.shrink_to_fit();
    } else if (cols_ != in_dim) {
        throw BackendError(BackendError::Kind::InvalidTensorData,
                           "tensor " + name_ + " is resident with rows of " + std::to_string(cols_) + " values; asked for " + std::to_string(in_dim));
    }
    return element_count_ / in_dim;
}

const cml_weight *WireQuant::band(size_t in_dim, size_t row_start, size_t count) const {
    const size_t rows = rows_for(in_dim);
    if (row_start + count > rows)
        throw BackendError(BackendError::Kind::InvalidTensorData,
                           "tensor " + name_ + ": rows [" + std::to_string(row_start) + ", " + std::to_string(row_start + count) + ") leave the " + std::to_string(rows) + " rows");
    if (row_start == 0 && count == rows) return weight_;
    const auto key = std::make_pair(row_start, count);
    const auto it = bands_.find(key);
    if (it != bands_.end()) return it->second;
    cml_weight *view = nullptr;
    dev(cml_weight_slice(weight_, static_cast<int64_t>(row_start), static_cast<int64_t>(count), &view), "cml_weight_slice");
    bands_.emplace(key, view);
    return view;
}

std::vector<float> WireQuant::run(const cml_weight *w, const int8_t *q, const float *s, size_t n_tokens, size_t rows) const {
    std::vector<float> out(n_tokens * rows);
    if (out.empty()) return out;
    float *od = static_cast<float *>(out_.reserve(out.size() * sizeof(float)));
    dev(cml_gemm(w, q, s, static_cast<int64_t>(n_tokens), od, nullptr), "cml_gemm");
    dev(cml_memcpy_d2h(out.data(), od, out.size() * sizeof(float), nullptr), "cml_memcpy_d2h");
    return out;
}

std::vector<float> WireQuant::matvec(size_t in_dim, size_t out_dim, const float *x) const {
    const cml_weight *w = band(in_dim, 0, out_dim);
    std::vector<float> out(out_dim);
    if (out_dim == 0) return out;
    // f32 in, f32 out: one call quantizes and multiplies (a single launch for Q4_K rows up to 4096 values)
    SharedActivation sa(x, in_dim);
    const size_t ws_bytes = cml_matmul_workspace_bytes(ggml_type_id(format_), static_cast<int64_t>(in_dim), 1);
    void *ws = q_.reserve(ws_bytes ? ws_bytes : 16);
    float *od = static_cast<float *>(out_.reserve(out_dim * sizeof(float)));
    dev(cml_matmul_f32(w, sa.x_dev(), 1, od, ws, ws_bytes, nullptr), "cml_matmul_f32");
    dev(cml_memcpy_d2h(out.data(), od, out_dim * sizeof(float), nullptr), "cml_memcpy_d2h");
    return out;
}

std::vector<float> WireQuant::matvec_proj(size_t out_dim, const SharedActivation &x) const {
    const cml_weight *w = band(x.len(), 0, out_dim);
    const auto qs = is_k_family() ? x.q8_k_dev() : x.q8_0_dev();
    return run(w, qs.first, qs.second, 1, out_dim);
}

std::vector<std::vector<float>> WireQuant::matmul_proj(size_t out_dim, const SharedActivationBatch &xs) const {
    std::vector<std::vector<float>> out(xs.rows());
    if (xs.rows() == 0) return out;
    const cml_weight *w = band(xs.len(), 0, out_dim);
    const auto qs = is_k_family() ? xs.q8_k_dev() : xs.q8_0_dev();
    const std::vector<float> flat = run(w, qs.first, qs.second, xs.rows(), out_dim);
    for (size_t k = 0; k < xs.rows(); k++) out[k].assign(flat.begin() + k * out_dim, flat.begin() + (k + 1) * out_dim);
    return out;
}

std::vector<float> WireQuant::matvec_rows_proj(size_t row_start, size_t out_count, const SharedActivation &x) const {
    const cml_weight *w = band(x.len(), row_start, out_count);
    const auto qs = is_k_family() ? x.q8_k_dev() : x.q8_0_dev();
    return run(w, qs.first, qs.second, 1, out_count);
}

namespace {
// Host block structs -> the device layout (quants then scales), one or many activation rows.
template <typename Block, int N>
void upload_blocks(const std::vector<const std::vector<Block> *> &rows, DeviceScratch &qd, DeviceScratch &sd, size_t &len) {
    const size_t nb = rows.empty() ? 0 : rows[0]->size();
    len = nb * N;
    std::vector<int8_t> q(rows.size() * nb * N);
    std::vector<float> s(rows.size() * nb);
    for (size_t r = 0; r < rows.size(); r++) {
        if (rows[r]->size() != nb) throw BackendError(BackendError::Kind::InvalidTensorData, "quantized activation rows differ in length");
        for (size_t b = 0; b < nb; b++) {
            const Block &blk = (*rows[r])[b];
            if constexpr (N == 32) {
                s[r * nb + b] = blk.scale;
                std::memcpy(q.data() + (r * nb + b) * N, blk.quants, N);
            } else {
                s[r * nb + b] = blk.d;
                std::memcpy(q.data() + (r * nb + b) * N, blk.qs, N);
            }
        }
    }
    ensure_device();
    qd.reserve(q.size() + 16);
    sd.reserve(s.size() * sizeof(float) + 16);
    dev(cml_memcpy_h2d(qd.get(), q.data(), q.size(), nullptr), "cml_memcpy_h2d");
    dev(cml_memcpy_h2d(sd.get(), s.data(), s.size() * sizeof(float), nullptr), "cml_memcpy_h2d");
}

[[noreturn]] void wrong_family(const char *method, const char *needs) {
    throw BackendError(BackendError::Kind::UnsupportedTensorType, std::string(method) + " serves " + needs + " weights only");
}
}  // namespace

std::vector<float> WireQuant::matvec_q(size_t out_dim, const std::vector<Q8_0Block> &xq) const { return matvec_q_rows(0, out_dim, xq); }

std::vector<float> WireQuant::matvec_q_rows(size_t row_start, size_t out_count, const std::vector<Q8_0Block> &xq) const {
    if (is_k_family()) wrong_family("matvec_q", "Q8_0 / Q4_0");
    size_t len;
    upload_blocks<Q8_0Block, 32>({&xq}, q_, s_, len);
    const cml_weight *w = band(len, row_start, out_count);
    return run(w, static_cast<const int8_t *>(q_.get()), static_cast<const float *>(s_.get()), 1, out_count);
}

std::vector<std::vector<float>> WireQuant::matmul_q(size_t out_dim, const std::vector<std::vector<Q8_0Block>> &xqs) const {
    if (is_k_family()) wrong_family("matmul_q", "Q8_0 / Q4_0");
    std::vector<std::vector<float>> out(xqs.size());
    if (xqs.empty()) return out;
    std::vector<const std::vector<Q8_0Block> *> rows;
    for (const auto &r : xqs) rows.push_back(&r);
    size_t len;
    upload_blocks<Q8_0Block, 32>(rows, q_, s_, len);
    const cml_weight *w = band(len, 0, out_dim);
    const std::vector<float> flat = run(w, static_cast<const int8_t *>(q_.get()), static_cast<const float *>(s_.get()), xqs.size(), out_dim);
    for (size_t k = 0; k < xqs.size(); k++) out[k].assign(flat.begin() + k * out_dim, flat.begin() + (k + 1) * out_dim);
    return out;
}

std::vector<float> WireQuant::matvec_q8k(size_t out_dim, const std::vector<Q8KBlock> &xq) const { return matvec_q8k_rows(0, out_dim, xq); }

std::vector<float> WireQuant::matvec_q8k_rows(size_t row_start, size_t out_count, const std::vector<Q8KBlock> &xq) const {
    if (!is_k_family()) wrong_family("matvec_q8k", "Q4_K / Q6_K");
    size_t len;
    upload_blocks<Q8KBlock, 256>({&xq}, q_, s_, len);
    const cml_weight *w = band(len, row_start, out_count);
    return run(w, static_cast<const int8_t *>(q_.get()), static_cast<const float *>(s_.get()), 1, out_count);
}

std::vector<std::vector<float>> WireQuant::matmul_q8k(size_t out_dim, const std::vector<std::vector<Q8KBlock>> &xqs) const {
    if (!is_k_family()) wrong_family("matmul_q8k", "Q4_K / Q6_K");
    std::vector<std::vector<float>> out(xqs.size());
    if (xqs.empty()) return out;
    std::vector<const std::vector<Q8KBlock> *> rows;
    for (const auto &r : xqs) rows.push_back(&r);
    size_t len;
    upload_blocks<Q8KBlock, 256>(rows, q_, s_, len);
    const cml_weight *w = band(len, 0, out_dim);
    const std::vector<float> flat = run(w, static_cast<const int8_t *>(q_.get()), static_cast<const float *>(s_.get()), xqs.size(), out_dim);
    for (size_t k = 0; k < xqs.size(); k++) out[k].assign(flat.begin() + k * out_dim, flat.begin() + (k + 1) * out_dim);
    return out;
}

std::vector<float> WireQuant::dequantize_elements(size_t start, size_t len) const {
    if (start + len > element_count_)
        throw BackendError(BackendError::Kind::InvalidTensorData,
                           "tensor " + name_ + ": elements [" + std::to_string(start) + ", " + std::to_string(start + len) + ") leave the tensor");
    std::vector<float> out(len);
    if (len == 0) return out;
    if (!weight_) {
        // The row length is not known yet (it is fixed by the first matvec) and this call must not fix it (the
        // reference's dequantize_elements has no side effect either, src/gemma4_runtime.rs:1154).  The tensor goes to
        // the device ONCE, seen as rows of one block each, and stays there: a token's embedding row is then a row
        // band of that view -- no allocation, upload or free per call (an embedding table is read this way for every
        // token and never gets a matvec).
        const size_t bv = values_per_block(format_), bb = bytes_per_block(format_);
        const size_t b0 = start / bv, b1 = (start + len + bv - 1) / bv;
        ensure_device();
        if (!block_view_)
            dev(cml_weight_upload(ggml_type_id(format_), static_cast<int64_t>(wire_.size() / bb), static_cast<int64_t>(bv), wire_.data(),
                                  wire_.size(), &block_view_),
                "cml_weight_upload");
        cml_weight *raw = nullptr;
        dev(cml_weight_slice(block_view_, static_cast<int64_t>(b0), static_cast<int64_t>(b1 - b0), &raw), "cml_weight_slice");
        // the view handle is released on every way out of this block, an exception from reserve() or dev() included
        const std::unique_ptr<cml_weight, void (*)(cml_weight *)> tmp(raw, cml_weight_free);
        float *od = static_cast<float *>(out_.reserve((b1 - b0) * bv * sizeof(float)));
        dev(cml_dequantize(tmp.get(), od, nullptr), "cml_dequantize");
        dev(cml_stream_sync(nullptr), "cml_stream_sync");
        dev(cml_memcpy_d2h(out.data(), od + (start - b0 * bv), len * sizeof(float), nullptr), "cml_memcpy_d2h");
        return out;
    }
    // decode the rows that cover the range
    const size_t in_dim = cols_;
    const size_t r0 = start / in_dim, r1 = (start + len + in_dim - 1) / in_dim;
    const cml_weight *w = band(in_dim, r0, r1 - r0);
    float *od = static_cast<float *>(out_.reserve((r1 - r0) * in_dim * sizeof(float)));
    dev(cml_dequantize(w, od, nullptr), "cml_dequantize");
    dev(cml_stream_sync(nullptr), "cml_stream_sync");
    dev(cml_memcpy_d2h(out.data(), od + (start - r0 * in_dim), len * sizeof(float), nullptr), "cml_memcpy_d2h");
    return out;
}

}  // namespace camelid
