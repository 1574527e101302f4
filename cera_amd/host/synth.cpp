// Seeded random-init llama-architecture GGUF files (the synthetic stand-in for a
// checkpoint): matrices w ~ N(0, sigma) pushed through the GGUF quantizers of
// quantize.cpp, norm vectors 1.0 (+ optional jitter), metadata keys as
// LlamaModel::from_gguf reads them (cera/src/model/llama.rs:166-265).
//
// Random numbers are counter-based, so a tensor's values depend only on
// (seed, tensor name, element index) and not on thread count or order:
// splitmix64 of the counter -> two 53-bit uniforms -> Box-Muller in f64 -> f32.
#include <algorithm>
#include <atomic>
#include <cmath>
#include <cstring>
#include <string>
#include <thread>
#include <vector>

#include "cera_host.h"
#include "gguf.h"

namespace {

inline uint64_t splitmix64(uint64_t x) {
    x += 0x9E3779B97F4A7C15ull;
    x = (x ^ (x >> 30)) * 0xBF58476D1CE4E5B9ull;
    x = (x ^ (x >> 27)) * 0x94D049BB133111EBull;
    return x ^ (x >> 31);
}

uint64_t name_stream(uint64_t seed, const std::string& name) {
    uint64_t h = 0xcbf29ce484222325ull;  // FNV-1a over the tensor name
    for (unsigned char c : name) h = (h ^ c) * 0x100000001b3ull;
    return splitmix64(seed ^ splitmix64(h));
}

// elements [2*pair, 2*pair+1] of a stream
inline void normal_pair(uint64_t stream, uint64_t pair, double* z0, double* z1) {
    uint64_t a = splitmix64(stream + 2 * pair), b = splitmix64(stream + 2 * pair + 1);
    double u1 = (static_cast<double>(a >> 11) + 1.0) * (1.0 / 9007199254740992.0);  // (0, 1]
    double u2 = static_cast<double>(b >> 11) * (1.0 / 9007199254740992.0);          // [0, 1)
    double r = std::sqrt(-2.0 * std::log(u1)), t = 6.283185307179586476925 * u2;
    *z0 = r * std::cos(t);
    *z1 = r * std::sin(t);
}

void fill_normal(uint64_t stream, uint64_t first, uint64_t n, float sigma, float mean, float* out) {
    // first and n are even at every call site except a vector's odd tail
    for (uint64_t i = 0; i < n; i += 2) {
        double z0, z1;
        normal_pair(stream, (first + i) / 2, &z0, &z1);
        out[i] = mean + sigma * static_cast<float>(z0);
        if (i + 1 < n) out[i + 1] = mean + sigma * static_cast<float>(z1);
    }
}

struct Matrix { std::string name; uint64_t m, k; uint32_t type; };

}  // namespace

extern "C" int cera_synth_llama_gguf(const char* path, const cera_synth_config* c, uint64_t seed, int n_threads,
                                     char* err, uint64_t err_len) {
    auto fail = [&](const std::string& m) {
        if (err && err_len) {
            std::strncpy(err, m.c_str(), err_len - 1);
            err[err_len - 1] = 0;
        }
        return -1;
    };
    if (!path || !c) return fail("null argument");
    if (!c->n_layers || !c->hidden || !c->ffn || !c->n_heads || !c->n_kv_heads || !c->vocab)
        return fail("zero dimension in config");
    const uint32_t head_dim = c->head_dim ? c->head_dim : c->hidden / c->n_heads;
    const uint64_t q_dim = uint64_t(c->n_heads) * head_dim, kv_dim = uint64_t(c->n_kv_heads) * head_dim;
    const std::string arch = c->architecture ? c->architecture : "llama";
    if (n_threads <= 0) n_threads = 1;

    std::vector<Matrix> mats;
    mats.push_back({"token_embd.weight", c->vocab, c->hidden, c->type_token_embd});
    if (!c->tied_output) mats.push_back({"output.weight", c->vocab, c->hidden, c->type_output});
    for (uint32_t i = 0; i < c->n_layers; ++i) {
        std::string p = "blk." + std::to_string(i) + ".";
        mats.push_back({p + "attn_q.weight", q_dim, c->hidden, c->type_attn_q});
        mats.push_back({p + "attn_k.weight", kv_dim, c->hidden, c->type_attn_k});
        mats.push_back({p + "attn_v.weight", kv_dim, c->hidden, c->type_attn_v});
        mats.push_back({p + "attn_output.weight", c->hidden, q_dim, c->type_attn_output});
        mats.push_back({p + "ffn_gate.weight", c->ffn, c->hidden, c->type_ffn_gate});
        mats.push_back({p + "ffn_up.weight", c->ffn, c->hidden, c->type_ffn_up});
        mats.push_back({p + "ffn_down.weight", c->hidden, c->ffn, c->type_ffn_down});
    }
    for (const Matrix& m : mats)
        if (!cera_tensor_bytes(m.type, m.k))
            return fail(m.name + ": row length " + std::to_string(m.k) + " is not a whole number of type-" +
                        std::to_string(m.type) + " blocks");

    cera::GgufWriter w(32);
    using V = cera::GgufValue;
    w.add_metadata("general.architecture", V::str(arch));
    w.add_metadata("general.name", V::str("synthetic random-init " + arch));
    w.add_metadata("general.alignment", V::u32(32));
    w.add_metadata(arch + ".block_count", V::u32(c->n_layers));
    w.add_metadata(arch + ".embedding_length", V::u32(c->hidden));
    w.add_metadata(arch + ".feed_forward_length", V::u32(c->ffn));
    w.add_metadata(arch + ".attention.head_count", V::u32(c->n_heads));
    w.add_metadata(arch + ".attention.head_count_kv", V::u32(c->n_kv_heads));
    if (c->head_dim) w.add_metadata(arch + ".attention.key_length", V::u32(c->head_dim));
    w.add_metadata(arch + ".vocab_size", V::u32(c->vocab));
    w.add_metadata(arch + ".context_length", V::u32(c->context_length));
    w.add_metadata(arch + ".rope.freq_base", V::f32(c->rope_theta));
    w.add_metadata(arch + ".attention.layer_norm_rms_epsilon", V::f32(c->rms_eps));

    // tensor table: matrices first, then the f32 vectors
    struct Vec { std::string name; uint64_t n; };
    std::vector<Vec> vecs;
    vecs.push_back({"output_norm.weight", c->hidden});
    for (uint32_t i = 0; i < c->n_layers; ++i) {
        std::string p = "blk." + std::to_string(i) + ".";
        vecs.push_back({p + "attn_norm.weight", c->hidden});
        vecs.push_back({p + "ffn_norm.weight", c->hidden});
        if (c->qkv_bias) {
            vecs.push_back({p + "attn_q.bias", q_dim});
            vecs.push_back({p + "attn_k.bias", kv_dim});
            vecs.push_back({p + "attn_v.bias", kv_dim});
        }
        if (c->qk_norm) {
            vecs.push_back({p + "attn_q_norm.weight", head_dim});
            vecs.push_back({p + "attn_k_norm.weight", head_dim});
        }
    }
    for (const Matrix& m : mats) w.add_tensor(m.name, {m.k, m.m}, m.type, cera_tensor_bytes(m.type, m.m * m.k));
    for (const Vec& v : vecs) w.add_tensor(v.name, {v.n}, CERA_TYPE_F32, v.n * 4);

    std::vector<uint8_t> blocks;
    std::vector<float> vecbuf;
    std::string werr;
    auto payload = [&](size_t idx) -> const void* {
        if (idx >= mats.size()) {
            const Vec& v = vecs[idx - mats.size()];
            vecbuf.assign(v.n, 0.0f);
            bool is_bias = v.name.size() > 5 && v.name.compare(v.name.size() - 5, 5, ".bias") == 0;
            if (is_bias)
                fill_normal(name_stream(seed, v.name), 0, v.n, c->weight_sigma, 0.0f, vecbuf.data());
            else if (c->norm_jitter != 0.0f)
                fill_normal(name_stream(seed, v.name), 0, v.n, c->norm_jitter, 1.0f, vecbuf.data());
            else
                std::fill(vecbuf.begin(), vecbuf.end(), 1.0f);
            return vecbuf.data();
        }
        const Matrix& m = mats[idx];
        const uint64_t row_bytes = cera_tensor_bytes(m.type, m.k);
        blocks.resize(row_bytes * m.m);
        const uint64_t stream = name_stream(seed, m.name);
        // workers take strips of rows: generate f32, quantize in place into the tensor
        const uint64_t strip = std::max<uint64_t>(1, (1u << 18) / m.k);
        std::atomic<uint64_t> next{0};
        std::atomic<int> bad{0};
        auto worker = [&]() {
            std::vector<float> rows(strip * m.k);
            for (;;) {
                uint64_t r0 = next.fetch_add(strip);
                if (r0 >= m.m) break;
                uint64_t nr = std::min<uint64_t>(strip, m.m - r0);
                fill_normal(stream, r0 * m.k, nr * m.k, c->weight_sigma, 0.0f, rows.data());
                if (cera_quantize(m.type, rows.data(), nr * m.k, blocks.data() + r0 * row_bytes, nr * row_bytes) != 0)
                    bad.store(1);
            }
        };
        std::vector<std::thread> pool;
        for (int t = 1; t < n_threads; ++t) pool.emplace_back(worker);
        worker();
        for (auto& t : pool) t.join();
        return bad.load() ? nullptr : blocks.data();
    };
    if (!w.write_file(path, payload, &werr)) return fail(werr.empty() ? "write failed" : werr);
    return 0;
}
