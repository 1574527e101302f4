// Mutation fuzz of the GGUF reader, meant to be built with -fsanitize=address,undefined
// (tests/test_gguf.py compiles and runs it).  A valid file is written with GgufWriter, then
// mutated by a seeded generator -- byte flips, truncations, counts and lengths overwritten with
// extreme values -- and parsed; every outcome must be "nullptr + error text" or a file whose
// tensors and metadata can be walked without touching memory outside the buffer.
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <string>
#include <vector>

#include "cera_host.h"
#include "gguf.h"

using namespace cera;

static uint64_t lcg(uint64_t& s) {
    s = s * 6364136223846793005ull + 1442695040888963407ull;
    return s >> 17;
}

static std::vector<uint8_t> valid_file() {
    GgufWriter w(32);
    w.add_metadata("general.architecture", GgufValue::str("llama"));
    w.add_metadata("llama.block_count", GgufValue::u32(2));
    w.add_metadata("llama.rope.freq_base", GgufValue::f32(10000.0f));
    w.add_metadata("flag", GgufValue::boolean(true));
    GgufValue arr;
    arr.type = GGUF_ARRAY;
    arr.elem_type = GGUF_STRING;
    for (int i = 0; i < 5; ++i) arr.arr.push_back(GgufValue::str("tok" + std::to_string(i)));
    w.add_metadata("tokenizer.ggml.tokens", arr);
    w.add_tensor("a.weight", {64, 4}, 0, 64 * 4 * 4);          // F32
    w.add_tensor("b.weight", {256, 2}, 12, 2 * 144);          // Q4_K
    w.add_tensor("c.weight", {32, 3}, 8, 3 * 34);             // Q8_0
    w.add_tensor("norm.weight", {64}, 1, 64 * 2);             // F16
    std::vector<uint8_t> f = w.header_bytes();
    // payloads with their alignment padding, as write_file lays them out
    const uint64_t sizes[4] = {64 * 4 * 4, 2 * 144, 3 * 34, 64 * 2};
    for (int i = 0; i < 4; ++i) {
        for (uint64_t j = 0; j < sizes[i]; ++j) f.push_back(static_cast<uint8_t>(31 * i + j));
        while (f.size() % 32) f.push_back(0);
    }
    return f;
}

static unsigned walk(const GgufFile& g) {
    unsigned sum = 0;
    for (const auto& kv : g.metadata()) sum += static_cast<unsigned>(kv.first.size() + kv.second.s.size() + kv.second.arr.size());
    (void)g.get_u32("llama.block_count");
    (void)g.get_f32("llama.rope.freq_base");
    (void)g.get_str("general.architecture");
    (void)g.get_bool("flag");
    for (const auto& t : g.tensors()) {
        const uint8_t* p = g.tensor_data(t.second);
        if (p)
            for (uint64_t i = 0; i < t.second.size_bytes; i += 17) sum += p[i];   // inside the buffer, or the sanitizer says so
        if (p && t.second.size_bytes) sum += p[t.second.size_bytes - 1];
        std::vector<float> f32;
        std::string err;
        (void)g.tensor_to_f32(t.first, &f32, &err);
        WeightRef ref;
        (void)resolve_weight(g, t.first, &ref, &err);
    }
    return sum;
}

int main(int argc, char** argv) {
    const unsigned iters = argc > 1 ? static_cast<unsigned>(std::stoul(argv[1])) : 20000;
    const std::vector<uint8_t> base = valid_file();
    std::string err;
    auto ok = GgufFile::from_bytes(base, &err);
    if (!ok) {
        std::fprintf(stderr, "the unmutated file does not parse: %s\n", err.c_str());
        return 2;
    }
    if (ok->tensors().size() != 4) return 3;
    unsigned sink = walk(*ok), parsed = 0, refused = 0;
    const uint64_t extremes[] = {0, 1, 0x7F, 0xFF, 0xFFFF, 0x7FFFFFFFull, 0xFFFFFFFFull, 0x100000000ull, 0x7FFFFFFFFFFFFFFFull,
                                 0xFFFFFFFFFFFFFFFFull, 0x8000000000000000ull, base.size(), base.size() - 1, base.size() + 1};
    uint64_t s = 0x9E3779B97F4A7C15ull;
    const size_t header = static_cast<size_t>(ok->data_offset());
    for (unsigned it = 0; it < iters; ++it) {
        std::vector<uint8_t> f = base;
        const unsigned kind = lcg(s) % 5;
        if (kind == 0) {   // flip a few header bytes
            const unsigned n = 1 + lcg(s) % 4;
            for (unsigned i = 0; i < n; ++i) f[lcg(s) % header] ^= static_cast<uint8_t>(1u << (lcg(s) % 8));
        } else if (kind == 1) {   // truncate
            f.resize(lcg(s) % f.size());
        } else if (kind == 2) {   // overwrite an aligned 8-byte field with an extreme value
            const size_t at = (lcg(s) % (header / 4)) * 4;
            const uint64_t v = extremes[lcg(s) % (sizeof(extremes) / sizeof(extremes[0]))];
            std::memcpy(f.data() + at, &v, std::min<size_t>(8, f.size() - at));
        } else if (kind == 3) {   // overwrite a 4-byte field
            const size_t at = lcg(s) % (header - 4);
            const uint32_t v = static_cast<uint32_t>(extremes[lcg(s) % (sizeof(extremes) / sizeof(extremes[0]))]);
            std::memcpy(f.data() + at, &v, 4);
        } else {   // random bytes over a short run
            const size_t at = lcg(s) % header, n = 1 + lcg(s) % 16;
            for (size_t i = 0; i < n && at + i < f.size(); ++i) f[at + i] = static_cast<uint8_t>(lcg(s));
        }
        err.clear();
        auto g = GgufFile::from_bytes(std::move(f), &err);
        if (g) {
            sink += walk(*g);
            ++parsed;
        } else {
            if (err.empty()) {
                std::fprintf(stderr, "iteration %u: refused without an error text\n", it);
                return 4;
            }
            ++refused;
        }
    }
    // the quantizers on hostile values (NaN, infinities, denormals, huge magnitudes): no
    // undefined conversion or shift, no write past the block buffer
    {
        const uint32_t types[] = {2, 8, 12, 13, 14};   // the types the host quantizer writes
        std::vector<float> x(512);
        for (unsigned round = 0; round < 200; ++round) {
            for (size_t i = 0; i < x.size(); ++i) {
                const uint64_t r = lcg(s);
                float v;
                switch (r % 9) {
                    case 0: v = __builtin_nanf(""); break;
                    case 1: v = __builtin_inff(); break;
                    case 2: v = -__builtin_inff(); break;
                    case 3: v = 3.0e38f; break;
                    case 4: v = -3.0e38f; break;
                    case 5: v = 1.0e-42f; break;
                    case 6: v = 0.0f; break;
                    default: v = static_cast<float>(static_cast<int64_t>(lcg(s) % 2001) - 1000) * 0.01f; break;
                }
                x[i] = round < 20 ? static_cast<float>(static_cast<int64_t>(r % 2001) - 1000) * 0.01f : v;
            }
            for (uint32_t t : types) {
                std::vector<uint8_t> out(cera_tensor_bytes(t, x.size()));
                if (cera_quantize(t, x.data(), x.size(), out.data(), out.size()) != 0 && round < 20) {
                    std::fprintf(stderr, "quantize type %u refused finite input\n", t);
                    return 5;
                }
                for (uint8_t b : out) sink += b;
            }
        }
    }
    std::printf("gguf fuzz: %u mutations, %u parsed, %u refused (checksum %u)\n", iters, parsed, refused, sink);
    return 0;
}
