// GGUF header / metadata / tensor-directory reader and a read-only memory map
// of the file (reference src/gguf/reader.rs:378-555 for the parse and its
// checks, :654-698 for metadata values, :700-741 for tensor byte sizes,
// :839-849 for strings).  Little-endian hosts only, like the format.
#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <cstring>
#include <fstream>
#include <set>

#include "camelid_host.hpp"

namespace camelid {

namespace {

constexpr uint64_t kDefaultAlignment = 32;  // reference DEFAULT_ALIGNMENT
constexpr uint32_t kMaxDims = 4;            // GGML_MAX_DIMS
constexpr size_t kMaxName = 64;             // GGML_MAX_NAME

[[noreturn]] void invalid(const std::string &m) { throw BackendError(BackendError::Kind::InvalidGguf, "invalid GGUF: " + m); }
[[noreturn]] void unsupported(const std::string &m) { throw BackendError(BackendError::Kind::UnsupportedGguf, "unsupported GGUF: " + m); }

class Cursor {
public:
    Cursor(const std::string &path) : path_(path), in_(path, std::ios::binary) {
        if (!in_) throw BackendError(BackendError::Kind::Io, "cannot open " + path);
    }
    void read(void *dst, size_t n) {
        in_.read(static_cast<char *>(dst), static_cast<std::streamsize>(n));
        if (static_cast<size_t>(in_.gcount()) != n) invalid("unexpected end of file in " + path_);
        pos_ += n;
    }
    template <typename T>
    T scalar() {
        T v;
        read(&v, sizeof(T));
        return v;
    }
    std::string string() {
        const uint64_t len = scalar<uint64_t>();
        if (len > 16ull * 1024 * 1024) invalid("string too large: " + std::to_string(len));
        std::string s(static_cast<size_t>(len), '\0');
        if (len) read(s.data(), static_cast<size_t>(len));
        return s;
    }
    uint64_t position() const { return pos_; }

private:
    std::string path_;
    std::ifstream in_;
    uint64_t pos_ = 0;
};

GgufMetadataValue read_value_of_type(Cursor &c, int32_t ty) {
    GgufMetadataValue v;
    switch (ty) {
        case 0: v.value = c.scalar<uint8_t>(); break;
        case 1: v.value = c.scalar<int8_t>(); break;
        case 2: v.value = c.scalar<uint16_t>(); break;
        case 3: v.value = c.scalar<int16_t>(); break;
        case 4: v.value = c.scalar<uint32_t>(); break;
        case 5: v.value = c.scalar<int32_t>(); break;
        case 6: v.value = c.scalar<float>(); break;
        case 7: v.value = (c.scalar<uint8_t>() != 0); break;
        case 8: v.value = c.string(); break;
        case 9: {
            const int32_t element_ty = c.scalar<int32_t>();
            if (element_ty == 9) unsupported("nested metadata arrays");
            const uint64_t len = c.scalar<uint64_t>();
            if (len > 1000000) invalid("metadata array too large: " + std::to_string(len));
            GgufArray values;
            values.reserve(static_cast<size_t>(len));
            for (uint64_t i = 0; i < len; i++) values.push_back(read_value_of_type(c, element_ty));
            v.value = std::move(values);
            break;
        }
        case 10: v.value = c.scalar<uint64_t>(); break;
        case 11: v.value = c.scalar<int64_t>(); break;
        case 12: v.value = c.scalar<double>(); break;
        default: unsupported("metadata value type " + std::to_string(ty));
    }
    return v;
}

uint64_t checked_mul(uint64_t a, uint64_t b, const std::string &what) {
    uint64_t r;
    if (__builtin_mul_overflow(a, b, &r)) invalid(what + " overflow");
    return r;
}
uint64_t checked_add(uint64_t a, uint64_t b, const std::string &what) {
    uint64_t r;
    if (__builtin_add_overflow(a, b, &r)) invalid(what + " overflow");
    return r;
}
uint64_t align_to(uint64_t v, uint64_t alignment) {
    const uint64_t r = v % alignment;
    return r == 0 ? v : checked_add(v, alignment - r, "aligned offset");
}

uint64_t tensor_nbytes(const std::string &name, const std::vector<uint64_t> &dims, int32_t type_id) {
    const auto layout = tensor_type_layout(type_id);
    if (!layout) unsupported("tensor " + name + " has unknown or removed GGML type Unknown(" + std::to_string(type_id) + ")");
    const uint64_t block = layout->first, type_size = layout->second;
    const uint64_t first = dims.empty() ? 1 : dims[0];
    if (first % block != 0)
        invalid("tensor " + name + " first dimension " + std::to_string(first) + " is not divisible by block size " + std::to_string(block));
    uint64_t elements = 1;
    for (uint64_t d : dims) elements = checked_mul(elements, d, "tensor " + name + " element count");
    return checked_mul(elements / block, type_size, "tensor " + name + " byte size");
}

}  // namespace

std::optional<std::pair<uint64_t, uint64_t>> tensor_type_layout(int32_t id) {
    using P = std::pair<uint64_t, uint64_t>;
    switch (id) {
        case 0: return P{1, 4};       // F32
        case 1: return P{1, 2};       // F16
        case 2: return P{32, 18};     // Q4_0
        case 3: return P{32, 20};     // Q4_1
        case 6: return P{32, 22};     // Q5_0
        case 7: return P{32, 24};     // Q5_1
        case 8: return P{32, 34};     // Q8_0
        case 9: return P{32, 36};     // Q8_1
        case 10: return P{256, 84};   // Q2_K
        case 11: return P{256, 110};  // Q3_K
        case 12: return P{256, 144};  // Q4_K
        case 13: return P{256, 176};  // Q5_K
        case 14: return P{256, 210};  // Q6_K
        case 15: return P{256, 292};  // Q8_K
        case 20: return P{32, 18};    // IQ4_NL
        case 23: return P{256, 136};  // IQ4_XS
        case 24: return P{1, 1};      // I8
        case 25: return P{1, 2};      // I16
        case 26: return P{1, 4};      // I32
        case 27: return P{1, 8};      // I64
        case 28: return P{1, 8};      // F64
        case 30: return P{1, 2};      // BF16
        case 34: return P{256, 54};   // TQ1_0
        case 35: return P{256, 66};   // TQ2_0
        case 40: return P{64, 36};    // NVFP4
        case 41: return P{128, 18};   // Q1_0
        default: return std::nullopt; // I2_S and the two type-42 dialects need whole-directory resolution: not served here
    }
}

const GgufTensorDescriptor *GgufFile::tensor(const std::string &name) const {
    for (const auto &t : tensors)
        if (t.name == name) return &t;
    return nullptr;
}

std::optional<std::string> GgufFile::metadata_string(const std::string &key) const {
    const auto it = metadata.find(key);
    if (it == metadata.end()) return std::nullopt;
    if (const auto *s = std::get_if<std::string>(&it->second.value)) return *s;
    return std::nullopt;
}

GgufFile read_metadata(const std::string &path) {
    struct stat st;
    if (::stat(path.c_str(), &st) != 0) throw BackendError(BackendError::Kind::Io, "cannot stat " + path);
    return read_metadata_with_len(path, static_cast<uint64_t>(st.st_size));
}

GgufFile read_metadata_with_len(const std::string &path, uint64_t file_len) {
    Cursor c(path);
    char magic[4];
    c.read(magic, 4);
    if (std::memcmp(magic, "GGUF", 4) != 0) invalid("bad magic; expected GGUF");

    GgufFile f;
    f.path = path;
    f.version = c.scalar<uint32_t>();
    if (f.version < 2 || f.version > 3) unsupported("version " + std::to_string(f.version) + "; expected v2 or v3");
    f.tensor_count = c.scalar<int64_t>();
    f.metadata_count = c.scalar<int64_t>();
    if (f.tensor_count < 0 || f.metadata_count < 0) invalid("negative tensor or metadata count");

    for (int64_t i = 0; i < f.metadata_count; i++) {
        std::string key = c.string();
        const int32_t ty = c.scalar<int32_t>();
        GgufMetadataValue v = read_value_of_type(c, ty);
        if (!f.metadata.emplace(key, std::move(v)).second) invalid("duplicate metadata key " + key);
    }

    f.alignment = kDefaultAlignment;
    if (const auto it = f.metadata.find("general.alignment"); it != f.metadata.end()) {
        if (const auto *u32 = std::get_if<uint32_t>(&it->second.value)) f.alignment = *u32;
        else if (const auto *u64 = std::get_if<uint64_t>(&it->second.value)) f.alignment = *u64;
        else invalid("general.alignment has non-integer type");
    }
    if (f.alignment == 0 || (f.alignment & (f.alignment - 1)) != 0) invalid("invalid alignment " + std::to_string(f.alignment));

    struct Raw {
        std::string name;
        std::vector<uint64_t> dims;
        int32_t type;
        uint64_t offset;
    };
    std::vector<Raw> raw;
    // no reserve from the file's own count: a crafted header must fail as InvalidGguf when the
    // entries run out, not as a length_error (the reference pushes one by one, src/gguf/reader.rs:444-470)
    for (int64_t i = 0; i < f.tensor_count; i++) {
        Raw r;
        r.name = c.string();
        if (r.name.size() >= kMaxName) invalid("tensor name " + r.name + " exceeds GGML_MAX_NAME");
        const uint32_t nd = c.scalar<uint32_t>();
        if (nd == 0 || nd > kMaxDims) invalid("tensor " + r.name + " has invalid dimension count " + std::to_string(nd));
        for (uint32_t d = 0; d < nd; d++) {
            const int64_t dim = c.scalar<int64_t>();
            if (dim < 0) invalid("tensor " + r.name + " has negative dimension " + std::to_string(dim));
            r.dims.push_back(static_cast<uint64_t>(dim));
        }
        r.type = c.scalar<int32_t>();
        r.offset = c.scalar<uint64_t>();
        raw.push_back(std::move(r));
    }

    f.data_start_offset = align_to(c.position(), f.alignment);
    if (f.data_start_offset > file_len) invalid("aligned tensor data start is beyond end of file");

    std::set<std::string> seen;
    uint64_t expected = 0;
    for (auto &r : raw) {
        if (!seen.insert(r.name).second) invalid("duplicate tensor name " + r.name);
        if (r.offset != expected)
            invalid("tensor " + r.name + " offset " + std::to_string(r.offset) + " is not contiguous; expected " + std::to_string(expected));
        GgufTensorDescriptor d;
        d.n_bytes = tensor_nbytes(r.name, r.dims, r.type);
        d.absolute_offset = checked_add(f.data_start_offset, r.offset, "tensor " + r.name + " absolute offset");
        const uint64_t end = checked_add(d.absolute_offset, d.n_bytes, "tensor " + r.name + " byte range");
        if (end > file_len) invalid("tensor " + r.name + " data extends beyond end of file");
        d.name = std::move(r.name);
        d.dimensions = std::move(r.dims);
        d.tensor_type = r.type;
        d.relative_offset = r.offset;
        expected = align_to(checked_add(r.offset, d.n_bytes, "tensor offset"), f.alignment);
        f.tensors.push_back(std::move(d));
    }
    return f;
}

GgufWireMmap::GgufWireMmap(const std::string &path) {
    const int fd = ::open(path.c_str(), O_RDONLY);
    if (fd < 0) throw BackendError(BackendError::Kind::Io, "cannot open " + path);
    struct stat st;
    if (::fstat(fd, &st) != 0) {
        ::close(fd);
        throw BackendError(BackendError::Kind::Io, "cannot stat " + path);
    }
    size_ = static_cast<uint64_t>(st.st_size);
    if (size_ > 0) {
        void *p = ::mmap(nullptr, static_cast<size_t>(size_), PROT_READ, MAP_PRIVATE, fd, 0);
        if (p == MAP_FAILED) {
            ::close(fd);
            throw BackendError(BackendError::Kind::Io, "cannot map " + path);
        }
        base_ = p;
    }
    ::close(fd);
}

GgufWireMmap::~GgufWireMmap() {
    if (base_) ::munmap(base_, static_cast<size_t>(size_));
}

const uint8_t *GgufWireMmap::bytes(uint64_t offset, uint64_t len) const {
    uint64_t end;
    if (__builtin_add_overflow(offset, len, &end) || end > size_) return nullptr;
    return static_cast<const uint8_t *>(base_) + offset;
}

}  // namespace camelid
