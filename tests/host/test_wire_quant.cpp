// WireQuant / SharedActivation on the device, written like the reference's own tests of that
// API (src/gemma4_runtime.rs:22551-22760): the same closed-form wires ((i*131+17)%256 with
// d = 0.0173, dmin = 0.0049) and sin activations, and the same claims -- projection dispatch
// equals the top-level matvec and the raw row dot, batched equals single, a row band equals the
// rows of the full matvec, all bitwise.  The row dots come from the CPU oracle.  Needs a GPU.
#include <cmath>
#include <cstdint>
#include <fstream>
#include <vector>

#include "../../camelid_amd/host/camelid_host.hpp"
#include "../../oracle/camelid_oracle.h"
#include "check.hpp"

using namespace camelid;

namespace {

uint16_t f16_bits(float v) { return orc_f32_to_f16_bits(v); }

std::vector<uint8_t> synth_wire(size_t blocks, size_t bytes_per_block, const std::vector<size_t> &f16_offs) {
    std::vector<uint8_t> wire(blocks * bytes_per_block);
    for (size_t i = 0; i < wire.size(); i++) wire[i] = static_cast<uint8_t>((i * 131 + 17) % 256);
    for (size_t b = 0; b < blocks; b++)
        for (size_t j = 0; j < f16_offs.size(); j++) {
            const uint16_t h = f16_bits(j == 0 ? 0.0173f : 0.0049f);
            wire[b * bytes_per_block + f16_offs[j]] = static_cast<uint8_t>(h & 0xff);
            wire[b * bytes_per_block + f16_offs[j] + 1] = static_cast<uint8_t>(h >> 8);
        }
    return wire;
}

std::vector<float> activation(size_t n, float seed) {
    std::vector<float> x(n);
    for (size_t i = 0; i < n; i++) x[i] = std::sin(static_cast<float>(i) * 0.37f + seed) * 3.0f;
    return x;
}

struct Case {
    WireFormat format;
    int fmt;  // oracle / GGML id
    size_t block_values, block_bytes;
    std::vector<size_t> f16_offs;
    const char *name;
};

const std::vector<Case> kCases = {
    {WireFormat::Q4K, ORC_Q4_K, 256, 144, {0, 2}, "Q4_K"},
    {WireFormat::Q6K, ORC_Q6_K, 256, 210, {208}, "Q6_K"},
    {WireFormat::Q8_0, ORC_Q8_0, 32, 34, {0}, "Q8_0"},
    {WireFormat::Q4_0, ORC_Q4_0, 32, 18, {0}, "Q4_0"},
};

// The order the kernels keep bit for bit (Q4_K: fused chain; Q6_K: fused chain; block order otherwise).
int exact_order(int fmt) { return fmt == ORC_Q6_K ? ORC_ORDER_ALT : ORC_ORDER_PRIMARY; }
int other_order(int fmt) { return fmt == ORC_Q6_K ? ORC_ORDER_PRIMARY : ORC_ORDER_ALT; }

std::vector<float> oracle_rows(const Case &c, const std::vector<uint8_t> &wire, size_t in_dim, size_t row_start, size_t rows,
                               const std::vector<float> &x, int order) {
    std::vector<float> out(rows);
    CHECK(orc_matmul(c.fmt, order, wire.data(), in_dim, row_start, rows, x.data(), 1, out.data(), 1) == 0);
    return out;
}

void put_str(std::vector<uint8_t> &b, const std::string &s) {
    const uint64_t n = s.size();
    b.insert(b.end(), reinterpret_cast<const uint8_t *>(&n), reinterpret_cast<const uint8_t *>(&n) + 8);
    b.insert(b.end(), s.begin(), s.end());
}
template <typename T>
void put(std::vector<uint8_t> &b, T v) {
    b.insert(b.end(), reinterpret_cast<const uint8_t *>(&v), reinterpret_cast<const uint8_t *>(&v) + sizeof(T));
}

// One-tensor GGUF v3 file around `wire`.
void write_gguf(const std::string &path, const std::string &name, int type, size_t in_dim, size_t out_dim, const std::vector<uint8_t> &wire) {
    std::vector<uint8_t> b = {'G', 'G', 'U', 'F'};
    put<uint32_t>(b, 3);
    put<int64_t>(b, 1);
    put<int64_t>(b, 1);
    put_str(b, "general.architecture");
    put<int32_t>(b, 8);
    put_str(b, "gemma4");
    put_str(b, name);
    put<uint32_t>(b, 2);
    put<int64_t>(b, static_cast<int64_t>(in_dim));
    put<int64_t>(b, static_cast<int64_t>(out_dim));
    put<int32_t>(b, type);
    put<uint64_t>(b, 0);
    while (b.size() % 32) b.push_back(0);
    b.insert(b.end(), wire.begin(), wire.end());
    std::ofstream f(path, std::ios::binary);
    f.write(reinterpret_cast<const char *>(b.data()), static_cast<std::streamsize>(b.size()));
}

float max_rel(const std::vector<float> &a, const std::vector<float> &b) {
    float m = 0.0f;
    for (size_t i = 0; i < a.size(); i++) m = std::fmax(m, std::fabs(a[i] - b[i]) / std::fmax(std::fabs(b[i]), 1.0f));
    return m;
}

}  // namespace

int main(int argc, char **argv) {
    CHECK(argc == 2);
    const std::string tmp = argv[1];
    // keep the reference's accumulation order at every shape, so that bitwise claims hold
    setenv("CAMELID_HIP_EXACT_ORDER", "1", 1);

    for (const Case &c : kCases) {
        // ---- projection dispatch == top-level matvec == raw row dot (reference :22571-22624) ----
        {
            const size_t in_dim = 2 * 256, out_dim = 5;
            say(std::string(c.name) + ": matvec_proj equals matvec and the wire row dot");
            const auto wire = synth_wire(out_dim * in_dim / c.block_values, c.block_bytes, c.f16_offs);
            const std::string path = tmp + "/" + c.name + ".gguf";
            write_gguf(path, "blk.0.ffn_up.weight", c.fmt, in_dim, out_dim, wire);
            const GgufFile file = read_metadata(path);
            const GgufWireMmap mmap(path);
            const WireQuant wq = WireQuant::from_gguf(file, mmap, "blk.0.ffn_up.weight");
            CHECK(wq.element_count() == in_dim * out_dim);
            const auto x = activation(in_dim, 0.25f);
            const auto top = wq.matvec(in_dim, out_dim, x.data());
            const SharedActivation sa(x.data(), in_dim);
            const auto got = wq.matvec_proj(out_dim, sa);
            const auto dot = oracle_rows(c, wire, in_dim, 0, out_dim, x, exact_order(c.fmt));
            const auto alt = oracle_rows(c, wire, in_dim, 0, out_dim, x, other_order(c.fmt));
            for (size_t o = 0; o < out_dim; o++) {
                CHECK_MSG(bits_of(got[o]) == bits_of(top[o]), "%s matvec_proj row %zu != top-level matvec", c.name, o);
                CHECK_MSG(bits_of(got[o]) == bits_of(dot[o]), "%s matvec_proj row %zu != wire row dot (%a vs %a)", c.name, o, got[o], dot[o]);
            }
            CHECK_MSG(max_rel(got, alt) <= 1e-5f, "%s: the reference's other accumulation order differs by %g", c.name, max_rel(got, alt));
            // the shared activation's quantized image is the oracle's, bit for bit
            if (c.block_values == 256) {
                const auto blocks = sa.q8_k();
                std::vector<float> d(in_dim / 256);
                std::vector<int8_t> q(in_dim);
                orc_quantize_q8_k(x.data(), in_dim, d.data(), q.data());
                for (size_t b = 0; b < blocks.size(); b++) {
                    CHECK(bits_of(blocks[b].d) == bits_of(d[b]));
                    CHECK(std::memcmp(blocks[b].qs, q.data() + 256 * b, 256) == 0);
                }
                const auto again = wq.matvec_q8k(out_dim, blocks);
                for (size_t o = 0; o < out_dim; o++) CHECK(bits_of(again[o]) == bits_of(got[o]));
            } else {
                const auto blocks = sa.q8_0();
                std::vector<float> s(in_dim / 32);
                std::vector<int8_t> q(in_dim);
                orc_quantize_q8_0(x.data(), in_dim, s.data(), q.data());
                for (size_t b = 0; b < blocks.size(); b++) {
                    CHECK(bits_of(blocks[b].scale) == bits_of(s[b]));
                    CHECK(std::memcmp(blocks[b].quants, q.data() + 32 * b, 32) == 0);
                }
                const auto again = wq.matvec_q(out_dim, blocks);
                for (size_t o = 0; o < out_dim; o++) CHECK(bits_of(again[o]) == bits_of(got[o]));
            }
            // decoded values are the oracle's
            const auto deq = wq.dequantize_elements(in_dim + 7, in_dim + 100);
            std::vector<float> ref(in_dim * out_dim);
            orc_dequant(c.fmt, wire.data(), ref.size() / c.block_values, ref.data());
            for (size_t i = 0; i < deq.size(); i++) CHECK(bits_of(deq[i]) == bits_of(ref[in_dim + 7 + i]));
        }
        // ---- decode before the first matvec (an embedding lookup, then the tied output head):
        //      decoding must not fix the row length or drop the host bytes ----
        {
            const size_t in_dim = 512, out_dim = 9;
            say(std::string(c.name) + ": from_wire, dequantize_elements, then matvec with the real row length");
            const auto wire = synth_wire(out_dim * in_dim / c.block_values, c.block_bytes, c.f16_offs);
            const WireQuant wq = WireQuant::from_wire(c.format, wire.data(), wire.size(), in_dim * out_dim, "token_embd.weight");
            std::vector<float> ref(in_dim * out_dim);
            orc_dequant(c.fmt, wire.data(), ref.size() / c.block_values, ref.data());
            const auto row3 = wq.dequantize_elements(3 * in_dim, in_dim);   // one embedding row
            for (size_t i = 0; i < row3.size(); i++) CHECK(bits_of(row3[i]) == bits_of(ref[3 * in_dim + i]));
            const auto odd = wq.dequantize_elements(in_dim - 5, 300);       // a range that straddles blocks and rows
            for (size_t i = 0; i < odd.size(); i++) CHECK(bits_of(odd[i]) == bits_of(ref[in_dim - 5 + i]));
            const auto x = activation(in_dim, 0.5f);
            const auto got = wq.matvec(in_dim, out_dim, x.data());
            const auto dot = oracle_rows(c, wire, in_dim, 0, out_dim, x, exact_order(c.fmt));
            for (size_t o = 0; o < out_dim; o++) CHECK_MSG(bits_of(got[o]) == bits_of(dot[o]), "%s matvec after a decode, row %zu", c.name, o);
            const auto again = wq.dequantize_elements(3 * in_dim, in_dim);  // and from the resident weight afterwards
            for (size_t i = 0; i < again.size(); i++) CHECK(bits_of(again[i]) == bits_of(ref[3 * in_dim + i]));
        }
        // ---- batched == single, row band == rows of the full matvec (reference :22626-22677) ----
        {
            const size_t in_dim = 256, out_dim = 6;
            say(std::string(c.name) + ": matmul_proj equals matvec_proj per activation; matvec_rows_proj(2, 3) equals rows 2..4");
            const auto wire = synth_wire(out_dim * in_dim / c.block_values, c.block_bytes, c.f16_offs);
            const WireQuant wq = WireQuant::from_wire(c.format, wire.data(), wire.size(), in_dim * out_dim, "blk.0.ffn_up.weight");
            std::vector<std::vector<float>> xs;
            for (int k = 0; k < 3; k++) xs.push_back(activation(in_dim, static_cast<float>(k) * 0.7f));
            const SharedActivationBatch xb(xs);
            const auto batched = wq.matmul_proj(out_dim, xb);
            CHECK(batched.size() == 3);
            for (size_t k = 0; k < xs.size(); k++) {
                const SharedActivation sa(xs[k].data(), in_dim);
                const auto single = wq.matvec_proj(out_dim, sa);
                for (size_t o = 0; o < out_dim; o++)
                    CHECK_MSG(bits_of(batched[k][o]) == bits_of(single[o]), "%s matmul_proj[%zu][%zu] != matvec_proj", c.name, k, o);
            }
            const SharedActivation sa(xs[0].data(), in_dim);
            const auto full = wq.matvec_proj(out_dim, sa);
            const auto band = wq.matvec_rows_proj(2, 3, sa);
            CHECK(band.size() == 3);
            for (size_t i = 0; i < 3; i++) CHECK_MSG(bits_of(band[i]) == bits_of(full[2 + i]), "%s row band offset %zu", c.name, 2 + i);
            const auto band_dot = oracle_rows(c, wire, in_dim, 2, 3, xs[0], exact_order(c.fmt));
            for (size_t i = 0; i < 3; i++) CHECK(bits_of(band[i]) == bits_of(band_dot[i]));
        }
        // ---- a speculative-verify sized chunk on a decode-sized weight ----
        {
            const size_t in_dim = 4096, out_dim = 200, k_tokens = 16;
            say(std::string(c.name) + ": 16-token matmul_proj on 200 x 4096");
            const auto wire = synth_wire(out_dim * in_dim / c.block_values, c.block_bytes, c.f16_offs);
            const WireQuant wq = WireQuant::from_wire(c.format, wire.data(), wire.size(), in_dim * out_dim);
            std::vector<std::vector<float>> xs;
            for (size_t k = 0; k < k_tokens; k++) xs.push_back(activation(in_dim, 0.1f * static_cast<float>(k)));
            const SharedActivationBatch xb(xs);
            const auto batched = wq.matmul_proj(out_dim, xb);
            for (size_t k = 0; k < k_tokens; k++) {
                const auto dot = oracle_rows(c, wire, in_dim, 0, out_dim, xs[k], exact_order(c.fmt));
                for (size_t o = 0; o < out_dim; o++)
                    CHECK_MSG(bits_of(batched[k][o]) == bits_of(dot[o]), "%s chunk cell [%zu][%zu]", c.name, k, o);
            }
        }
    }

    say("family and shape refusals");
    {
        const auto wire = synth_wire(6, 144, {0, 2});
        const WireQuant wq = WireQuant::from_wire(WireFormat::Q4K, wire.data(), wire.size(), 6 * 256);
        bool threw = false;
        try {
            wq.matvec_q(6, std::vector<Q8_0Block>(8));
        } catch (const BackendError &e) {
            threw = e.kind() == BackendError::Kind::UnsupportedTensorType;
        }
        CHECK(threw);
        threw = false;
        const auto x = activation(256, 0.0f);
        const SharedActivation sa(x.data(), 256);
        try {
            wq.matvec_rows_proj(4, 3, sa);  // rows 4..6 of a 6-row tensor
        } catch (const BackendError &e) {
            threw = e.kind() == BackendError::Kind::InvalidTensorData;
        }
        CHECK(threw);
    }

    std::printf("wire quant: %d checks passed\n", g_checks);
    return 0;
}
