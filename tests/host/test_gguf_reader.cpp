// GGUF reader against the reference's own committed files (tests/golden/gguf, byte-for-byte
// the reference's tests/fixtures/gguf) and against files written here.  No GPU needed.
// Expectations follow the reference's tests: tests/nvfp4_wire_lane_refusals.rs:60-80 (sidecar
// file parses: v3, gemma4, three named tensors, NVFP4 first), tests/invariant_matrix_binding.rs:
// 561-610 (type id 99 and a first dimension of 48 refuse at parse, with those messages).
#include <cstring>
#include <cstdint>
#include <fstream>
#include <vector>

#include "../../camelid_amd/host/camelid_host.hpp"
#include "check.hpp"

using namespace camelid;

namespace {

struct Writer {
    std::vector<uint8_t> b;
    template <typename T>
    void put(T v) {
        const auto *p = reinterpret_cast<const uint8_t *>(&v);
        b.insert(b.end(), p, p + sizeof(T));
    }
    void str(const std::string &s) {
        put<uint64_t>(s.size());
        b.insert(b.end(), s.begin(), s.end());
    }
    void pad(uint64_t alignment) {
        while (b.size() % alignment) b.push_back(0);
    }
};

struct TensorSpec {
    std::string name;
    std::vector<int64_t> dims;
    int32_t type;
    std::vector<uint8_t> data;
};

// A GGUF v3 file with one string, one u32 and one array key, and the given tensors.
std::vector<uint8_t> build(const std::vector<TensorSpec> &tensors, uint32_t alignment, bool contiguous = true, uint32_t version = 3) {
    Writer w;
    w.b = {'G', 'G', 'U', 'F'};
    w.put<uint32_t>(version);
    w.put<int64_t>(static_cast<int64_t>(tensors.size()));
    w.put<int64_t>(alignment == 32 ? 2 : 3);
    w.str("general.architecture");
    w.put<int32_t>(8);
    w.str("llama");
    w.str("test.array");
    w.put<int32_t>(9);
    w.put<int32_t>(5);
    w.put<uint64_t>(3);
    for (int i = 0; i < 3; i++) w.put<int32_t>(10 * i - 7);
    if (alignment != 32) {
        w.str("general.alignment");
        w.put<int32_t>(4);
        w.put<uint32_t>(alignment);
    }
    uint64_t off = 0;
    for (const auto &t : tensors) {
        w.str(t.name);
        w.put<uint32_t>(static_cast<uint32_t>(t.dims.size()));
        for (int64_t d : t.dims) w.put<int64_t>(d);
        w.put<int32_t>(t.type);
        w.put<uint64_t>(contiguous ? off : off + alignment);
        off += t.data.size();
        off = (off + alignment - 1) / alignment * alignment;
    }
    w.pad(alignment);
    for (const auto &t : tensors) {
        w.b.insert(w.b.end(), t.data.begin(), t.data.end());
        w.pad(alignment);
    }
    return w.b;
}

void write_file(const std::string &path, const std::vector<uint8_t> &bytes) {
    std::ofstream f(path, std::ios::binary);
    f.write(reinterpret_cast<const char *>(bytes.data()), static_cast<std::streamsize>(bytes.size()));
}

template <typename F>
std::string error_of(F &&f, BackendError::Kind want) {
    try {
        f();
    } catch (const BackendError &e) {
        CHECK_MSG(e.kind() == want, "wrong error kind for: %s", e.what());
        return e.what();
    }
    CHECK_MSG(false, "expected a BackendError");
    return "";
}

}  // namespace

int main(int argc, char **argv) {
    CHECK(argc == 3);
    const std::string fixtures = argv[1], tmp = argv[2];

    say("reference file nvfp4_sidecar_trip.gguf parses");
    {
        const GgufFile g = read_metadata(fixtures + "/nvfp4_sidecar_trip.gguf");
        CHECK(g.version == 3);
        CHECK(g.architecture() && *g.architecture() == "gemma4");
        CHECK(g.tensors.size() == 3 && g.tensor_count == 3);
        CHECK(g.tensors[0].name == "blk.0.ffn_down.weight");
        CHECK(g.tensors[1].name == "blk.0.ffn_down.weight.scale");
        CHECK(g.tensors[2].name == "blk.0.ffn_down.weight.input_scale");
        CHECK(g.tensors[0].tensor_type == 40);  // NVFP4
        CHECK(g.tensors[0].relative_offset == 0);
        CHECK(g.data_start_offset % g.alignment == 0);
        const GgufWireMmap m(g.path);
        for (const auto &t : g.tensors) {
            CHECK(t.absolute_offset == g.data_start_offset + t.relative_offset);
            CHECK(m.bytes(t.absolute_offset, t.n_bytes) != nullptr);
        }
        CHECK(m.bytes(m.size(), 1) == nullptr);
        // the quantized matvec path does not serve NVFP4: typed refusal, no device needed to say so
        const std::string msg = error_of([&] { WireQuant::from_gguf(g, m, "blk.0.ffn_down.weight"); }, BackendError::Kind::UnsupportedTensorType);
        CHECK(msg.find("blk.0.ffn_down.weight") != std::string::npos);
    }
    const std::pair<const char *, const char *> parsing[] = {{"nvfp4_nan_sentinel_trip.gguf", "blk.0.ffn_up.weight"},
                                                             {"nvfp4_sidecar_admit_trip.gguf", "blk.0.ffn_down.weight"},
                                                             {"nvfp4_pilot_admit.gguf", "blk.0.ffn_down.weight"}};
    for (const auto &[name, tensor] : parsing) {
        say(std::string("reference file ") + name + " parses");
        const GgufFile g = read_metadata(fixtures + "/" + name);
        CHECK(g.version == 3 && !g.tensors.empty());
        CHECK(g.architecture() && *g.architecture() == "gemma4");
        CHECK(g.tensor(tensor) != nullptr);
        CHECK(g.tensor(tensor)->tensor_type == 40);
        uint64_t elements = 1;
        for (uint64_t d : g.tensor(tensor)->dimensions) elements *= d;
        CHECK(g.tensor(tensor)->n_bytes == elements / 64 * 36);
    }

    say("reference file with GGML type 99 refuses at parse");
    {
        const std::string msg = error_of([&] { read_metadata(fixtures + "/nvfp4_unknown_type_trip.gguf"); }, BackendError::Kind::UnsupportedGguf);
        CHECK(msg.find("unknown or removed GGML type") != std::string::npos);
        CHECK(msg.find("Unknown(99)") != std::string::npos);
        CHECK(msg.find("blk.0.mystery.weight") != std::string::npos);
    }
    say("reference file with a first dimension of 48 refuses at parse");
    {
        const std::string msg = error_of([&] { read_metadata(fixtures + "/nvfp4_k_div_trip.gguf"); }, BackendError::Kind::InvalidGguf);
        CHECK(msg.find("first dimension 48 is not divisible by block size 64") != std::string::npos);
        CHECK(msg.find("blk.0.ffn_down.weight") != std::string::npos);
    }

    say("files written here: offsets, alignment, sizes");
    for (uint32_t alignment : {32u, 64u, 256u}) {
        std::vector<TensorSpec> ts;
        ts.push_back({"blk.0.ffn_up.weight", {256, 6}, 12, std::vector<uint8_t>(6 * 144, 0x5a)});        // Q4_K
        ts.push_back({"output.weight", {512, 3}, 14, std::vector<uint8_t>(3 * 2 * 210, 0x17)});           // Q6_K
        ts.push_back({"blk.0.attn_q.weight", {64, 5}, 8, std::vector<uint8_t>(5 * 2 * 34, 0x33)});        // Q8_0
        ts.push_back({"blk.0.attn_k.weight", {32, 4, 2}, 2, std::vector<uint8_t>(8 * 18, 0x44)});         // Q4_0, rank 3
        ts.push_back({"norm.weight", {7}, 0, std::vector<uint8_t>(28, 1)});                               // F32
        const std::string path = tmp + "/ok_" + std::to_string(alignment) + ".gguf";
        write_file(path, build(ts, alignment));
        const GgufFile g = read_metadata(path);
        CHECK(g.alignment == alignment && g.tensors.size() == ts.size());
        CHECK(g.architecture() && *g.architecture() == "llama");
        const auto &arr = std::get<GgufArray>(g.metadata.at("test.array").value);
        CHECK(arr.size() == 3 && std::get<int32_t>(arr[2].value) == 13);
        const GgufWireMmap m(path);
        uint64_t expected = 0;
        for (size_t i = 0; i < ts.size(); i++) {
            const auto &t = g.tensors[i];
            CHECK(t.name == ts[i].name && t.n_bytes == ts[i].data.size() && t.relative_offset == expected);
            const uint8_t *p = m.bytes(t.absolute_offset, t.n_bytes);
            CHECK(p && p[0] == ts[i].data[0] && p[t.n_bytes - 1] == ts[i].data[0]);
            expected = (expected + t.n_bytes + alignment - 1) / alignment * alignment;
        }
        // a header prefix validates against the declared full length
        CHECK(read_metadata_with_len(path, 1u << 30).tensors.size() == ts.size());
        error_of([&] { read_metadata_with_len(path, g.data_start_offset + 10); }, BackendError::Kind::InvalidGguf);
    }

    say("refusals");
    {
        std::vector<TensorSpec> one = {{"w", {32, 2}, 8, std::vector<uint8_t>(68, 0)}};
        auto bytes = build(one, 32);
        auto bad = bytes;
        bad[0] = 'X';
        write_file(tmp + "/bad_magic.gguf", bad);
        CHECK(error_of([&] { read_metadata(tmp + "/bad_magic.gguf"); }, BackendError::Kind::InvalidGguf).find("bad magic") != std::string::npos);
        write_file(tmp + "/v1.gguf", build(one, 32, true, 1));
        CHECK(error_of([&] { read_metadata(tmp + "/v1.gguf"); }, BackendError::Kind::UnsupportedGguf).find("version 1") != std::string::npos);
        write_file(tmp + "/gap.gguf", build(one, 32, false));
        CHECK(error_of([&] { read_metadata(tmp + "/gap.gguf"); }, BackendError::Kind::InvalidGguf).find("not contiguous") != std::string::npos);
        write_file(tmp + "/align3.gguf", build(one, 48));
        CHECK(error_of([&] { read_metadata(tmp + "/align3.gguf"); }, BackendError::Kind::InvalidGguf).find("invalid alignment") != std::string::npos);
        auto cut = bytes;
        cut.resize(cut.size() - 40);
        write_file(tmp + "/cut.gguf", cut);
        CHECK(error_of([&] { read_metadata(tmp + "/cut.gguf"); }, BackendError::Kind::InvalidGguf).find("beyond end of file") != std::string::npos);
        // a header that claims 2^62 tensors: refused as an invalid file when the entries run out
        auto huge = bytes;
        const uint64_t claimed = uint64_t(1) << 62;
        std::memcpy(huge.data() + 8, &claimed, 8);   // magic (4) + version (4), then the tensor count
        write_file(tmp + "/huge_count.gguf", huge);
        error_of([&] { read_metadata(tmp + "/huge_count.gguf"); }, BackendError::Kind::InvalidGguf);
        std::vector<TensorSpec> dup = {{"w", {32}, 8, std::vector<uint8_t>(34, 0)}, {"w", {32}, 8, std::vector<uint8_t>(34, 0)}};
        write_file(tmp + "/dup.gguf", build(dup, 32));
        CHECK(error_of([&] { read_metadata(tmp + "/dup.gguf"); }, BackendError::Kind::InvalidGguf).find("duplicate tensor name") != std::string::npos);
        std::vector<TensorSpec> dims5 = {{"w", {32, 1, 1, 1, 1}, 8, std::vector<uint8_t>(34, 0)}};
        write_file(tmp + "/dims5.gguf", build(dims5, 32));
        CHECK(error_of([&] { read_metadata(tmp + "/dims5.gguf"); }, BackendError::Kind::InvalidGguf).find("invalid dimension count") != std::string::npos);
        error_of([&] { read_metadata(tmp + "/does_not_exist.gguf"); }, BackendError::Kind::Io);
    }

    say("WireQuant shape refusals that need no device");
    {
        std::vector<uint8_t> wire(144 * 6, 0);
        error_of([&] { WireQuant::from_wire(WireFormat::Q4K, wire.data(), wire.size(), 6 * 256 + 32); }, BackendError::Kind::InvalidTensorData);
        const std::string msg = error_of([&] { WireQuant::from_wire(WireFormat::Q4K, wire.data(), wire.size() - 1, 6 * 256); }, BackendError::Kind::InvalidTensorData);
        CHECK(msg.find("expected 864") != std::string::npos);
    }

    std::printf("gguf reader: %d checks passed\n", g_checks);
    return 0;
}
