// Host side of the quantized matvec path, above the C ABI (include/camelid_hip.h):
// a GGUF reader that hands tensor wire bytes to the device, and the operator
// object the reference engine calls its quantized projections through.
//
// The shapes follow the reference so that a caller written against it reads the
// same here:
//   read_metadata / GgufFile / GgufTensorDescriptor   src/gguf/reader.rs:186-560
//   GgufWireMmap                                      src/gemma4_runtime.rs (memory-mapped wire bytes)
//   WireFormat, WireQuant                             src/gemma4_runtime.rs:590-1150
//   SharedActivation, SharedActivationBatch           src/gemma4_runtime.rs:1288-1340
//   Q8_0Block                                         src/tensor/mod.rs:105-110
//   Q8KBlock                                          src/inference.rs:23102-23105
// What differs is where things live: a WireQuant owns a device-resident copy of
// the weight (uploaded once, re-laid for the kernels), activations are quantized
// on the device, and every method is one or two kernel launches plus the copies
// in and out.  Results are the reference CPU path's, bit for bit where the
// kernels keep its accumulation order (see the C header).
//
// Errors: the reference returns Result<_, BackendError>; here the same kinds
// are thrown as camelid::BackendError.  Nothing in this layer falls back to a
// CPU implementation.
#pragma once

#include <cstddef>
#include <cstdint>
#include <map>
#include <memory>
#include <optional>
#include <stdexcept>
#include <string>
#include <utility>
#include <variant>
#include <vector>

struct cml_weight;

namespace camelid {

// ---- errors (reference BackendError, src/error.rs) ------------------------------------------------
class BackendError : public std::runtime_error {
public:
    enum class Kind { Io, InvalidGguf, UnsupportedGguf, UnsupportedTensorType, InvalidTensorData, Device };
    BackendError(Kind kind, const std::string &message) : std::runtime_error(message), kind_(kind) {}
    Kind kind() const { return kind_; }

private:
    Kind kind_;
};

// ---- GGUF (reference src/gguf/reader.rs) ----------------------------------------------------------

// GGML tensor type ids as stored in the file (reference GgufTensorType::from_id, :71-106).
enum class GgufTensorType : int32_t {
    F32 = 0, F16 = 1, Q4_0 = 2, Q4_1 = 3, Q5_0 = 6, Q5_1 = 7, Q8_0 = 8, Q8_1 = 9,
    Q2K = 10, Q3K = 11, Q4K = 12, Q5K = 13, Q6K = 14, Q8K = 15, IQ4NL = 20, IQ4XS = 23,
    I8 = 24, I16 = 25, I32 = 26, I64 = 27, F64 = 28, BF16 = 30, Tq1_0 = 34, Tq2_0 = 35,
    NVFP4 = 40, Q1_0 = 41,
};
// (values per block, bytes per block), or nullopt for a type this reader cannot size
// (reference GgufTensorType::layout, :108-185).
std::optional<std::pair<uint64_t, uint64_t>> tensor_type_layout(int32_t type_id);

struct GgufMetadataValue;
using GgufArray = std::vector<GgufMetadataValue>;
struct GgufMetadataValue {
    std::variant<uint8_t, int8_t, uint16_t, int16_t, uint32_t, int32_t, float, bool, std::string, GgufArray, uint64_t,
                 int64_t, double>
        value;
};

struct GgufTensorDescriptor {
    std::string name;
    std::vector<uint64_t> dimensions;  // innermost (contraction) first, as stored
    int32_t tensor_type = 0;           // raw GGML id
    uint64_t relative_offset = 0;
    uint64_t absolute_offset = 0;
    uint64_t n_bytes = 0;
};

struct GgufFile {
    std::string path;
    uint32_t version = 0;
    int64_t tensor_count = 0;
    int64_t metadata_count = 0;
    uint64_t alignment = 32;
    uint64_t data_start_offset = 0;
    std::map<std::string, GgufMetadataValue> metadata;
    std::vector<GgufTensorDescriptor> tensors;

    const GgufTensorDescriptor *tensor(const std::string &name) const;
    std::optional<std::string> metadata_string(const std::string &key) const;
    std::optional<std::string> architecture() const { return metadata_string("general.architecture"); }
};

// Parses header, metadata and the tensor directory with the reference's checks
// (magic, version 2..3, counts, duplicate keys/names, power-of-two alignment,
// name length, 1..4 dimensions, contiguous aligned offsets, ranges inside the
// file).  No tensor data is read.
GgufFile read_metadata(const std::string &path);
// Same, validating ranges against `declared_len` instead of the file's size
// (reference read_metadata_with_len: a header prefix of a larger file).
GgufFile read_metadata_with_len(const std::string &path, uint64_t declared_len);

// Read-only memory map of a GGUF file: tensor wire bytes are handed to the
// device straight from the page cache.
class GgufWireMmap {
public:
    explicit GgufWireMmap(const std::string &path);
    ~GgufWireMmap();
    GgufWireMmap(const GgufWireMmap &) = delete;
    GgufWireMmap &operator=(const GgufWireMmap &) = delete;
    // Pointer to [offset, offset+len) or nullptr when the range leaves the file.
    const uint8_t *bytes(uint64_t offset, uint64_t len) const;
    uint64_t size() const { return size_; }

private:
    void *base_ = nullptr;
    uint64_t size_ = 0;
};

// ---- quantized operator -----------------------------------------------------------------------------

// The wire formats this path serves (a subset of the reference's WireFormat).
enum class WireFormat { Q8_0, Q4_0, Q4K, Q6K };
size_t values_per_block(WireFormat f);
size_t bytes_per_block(WireFormat f);
int ggml_type_id(WireFormat f);

// Host images of quantized activation blocks, laid out as the reference's structs.
struct Q8_0Block {
    float scale;
    int8_t quants[32];
};
struct Q8KBlock {
    float d;
    int8_t qs[256];
};
static_assert(sizeof(Q8_0Block) == 36 && sizeof(Q8KBlock) == 260, "block images are packed like the reference's repr(C) structs");

// A device buffer that grows on demand and is freed with its owner.
class DeviceScratch {
public:
    DeviceScratch() = default;
    ~DeviceScratch();
    DeviceScratch(const DeviceScratch &) = delete;
    DeviceScratch &operator=(const DeviceScratch &) = delete;
    void *reserve(size_t nbytes);
    void *get() const { return ptr_; }

private:
    void *ptr_ = nullptr;
    size_t cap_ = 0;
};

// One activation row shared by several projections: each quantized family is
// produced lazily, at most once (on the device), however many projections
// consume it (reference SharedActivation).
class SharedActivation {
public:
    SharedActivation(const float *x, size_t len);
    size_t len() const { return len_; }
    // Device-resident quantized forms (quants, scales); created on first use.
    std::pair<const int8_t *, const float *> q8_0_dev() const;
    std::pair<const int8_t *, const float *> q8_k_dev() const;
    // Host copies of the same, in the reference's block structs (for callers and tests that inspect them).
    std::vector<Q8_0Block> q8_0() const;
    std::vector<Q8KBlock> q8_k() const;
    const float *x_dev() const;

private:
    friend class SharedActivationBatch;
    const float *x_;
    size_t len_, rows_ = 1;
    mutable DeviceScratch xd_, q0_, s0_, qk_, sk_;
    mutable bool have_x_ = false, have_q0_ = false, have_qk_ = false;
};

// K activation rows (speculative-verify chunk), same laziness (reference SharedActivationBatch).
class SharedActivationBatch {
public:
    explicit SharedActivationBatch(const std::vector<std::vector<float>> &xs);
    size_t rows() const { return rows_; }
    size_t len() const { return len_; }
    std::pair<const int8_t *, const float *> q8_0_dev() const { return inner_.q8_0_dev(); }
    std::pair<const int8_t *, const float *> q8_k_dev() const { return inner_.q8_k_dev(); }

private:
    std::vector<float> flat_;
    size_t rows_, len_;
    SharedActivation inner_;
};

// A quantized weight resident on the device (reference WireQuant: there a view
// of the memory-mapped file, here an uploaded copy of exactly those bytes).
class WireQuant {
public:
    // Binds tensor `name` of a parsed GGUF: the type must be one this path serves
    // (else UnsupportedTensorType), the element count whole blocks and the byte
    // range the expected size (else InvalidTensorData) -- reference WireQuant::new.
    static WireQuant from_gguf(const GgufFile &file, const GgufWireMmap &mmap, const std::string &name);
    // From wire bytes in host memory (reference WireQuant::from_owned_range, the ghost-expert loader).
    static WireQuant from_wire(WireFormat format, const uint8_t *bytes, size_t n_bytes, size_t element_count,
                               const std::string &name = "<owned>");
    WireQuant(WireQuant &&) noexcept;
    WireQuant &operator=(WireQuant &&) noexcept;
    ~WireQuant();

    WireFormat format() const { return format_; }
    size_t element_count() const { return element_count_; }

    // y[o] = sum_i dequant(W[o*in_dim + i]) * x[i], o < out_dim: the activation is quantized once
    // (Q8_0 for Q8_0/Q4_0 weights, Q8_K for the K-quants) and dotted against every row.
    std::vector<float> matvec(size_t in_dim, size_t out_dim, const float *x) const;
    // One projection off a shared activation, routed by the weight's family.
    std::vector<float> matvec_proj(size_t out_dim, const SharedActivation &x) const;
    // Batched sibling: out[k][o], each row bit-identical to matvec_proj of activation k.
    std::vector<std::vector<float>> matmul_proj(size_t out_dim, const SharedActivationBatch &xs) const;
    // Rows [row_start, row_start + out_count) only: the expert band of a stacked tensor; bitwise
    // the corresponding rows of the full matvec.
    std::vector<float> matvec_rows_proj(size_t row_start, size_t out_count, const SharedActivation &x) const;

    // The same against activations the caller has already quantized.
    std::vector<float> matvec_q(size_t out_dim, const std::vector<Q8_0Block> &xq) const;
    std::vector<float> matvec_q_rows(size_t row_start, size_t out_count, const std::vector<Q8_0Block> &xq) const;
    std::vector<std::vector<float>> matmul_q(size_t out_dim, const std::vector<std::vector<Q8_0Block>> &xqs) const;
    std::vector<float> matvec_q8k(size_t out_dim, const std::vector<Q8KBlock> &xq) const;
    std::vector<float> matvec_q8k_rows(size_t row_start, size_t out_count, const std::vector<Q8KBlock> &xq) const;
    std::vector<std::vector<float>> matmul_q8k(size_t out_dim, const std::vector<std::vector<Q8KBlock>> &xqs) const;

    // Decoded values [start, start + len) of the tensor (reference dequantize_elements).
    std::vector<float> dequantize_elements(size_t start, size_t len) const;

    // The device handle, for callers that drive the C ABI themselves (graphs, streams).
    const cml_weight *device_weight() const { return weight_; }

private:
    WireQuant() = default;
    void release();
    bool is_k_family() const { return format_ == WireFormat::Q4K || format_ == WireFormat::Q6K; }
    size_t rows_for(size_t in_dim) const;
    // rows [row_start, row_start+count) as a device view (cached), for a weight of `in_dim` columns
    const cml_weight *band(size_t in_dim, size_t row_start, size_t count) const;
    std::vector<float> run(const cml_weight *w, const int8_t *q, const float *s, size_t n_tokens, size_t rows) const;

    WireFormat format_ = WireFormat::Q8_0;
    size_t element_count_ = 0;
    std::string name_;
    std::vector<uint8_t> wire_;  // kept until the first use fixes the column count
    mutable cml_weight *weight_ = nullptr;
    // before the row length is known: the tensor resident as rows of ONE block each, for dequantize_elements
    // (an embedding table is only ever read that way); released when a matvec fixes the row length
    mutable cml_weight *block_view_ = nullptr;
    mutable size_t cols_ = 0;
    mutable std::map<std::pair<size_t, size_t>, cml_weight *> bands_;
    mutable DeviceScratch out_, q_, s_;
};

}  // namespace camelid
