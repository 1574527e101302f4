// cera-hip: command-line driver of the hip backend.
//
//   cera-hip gen     --out m.gguf [--preset llama3-8b|tiny] [--seed S] [--threads T] [--ctx N]
//   cera-hip inspect --model m.gguf
//   cera-hip run     --model m.gguf [--prompt-len 512] [--n-predict 256] [--seed S]
//                    [--ubatch 512] [--ctx 1024] [--device 0] [--tokens-out FILE] [--per-token-prefill]
//                    [--kv f32|f16]
//
// `run` is the workload `cera bench` times (cera-cli/src/main.rs:932-938 for the
// protocol): a prompt of uniform random token ids is prefilled in `ubatch`
// chunks, then tokens are decoded greedily; prefill and decode rates are
// reported separately as one JSON line on stdout.
#include <chrono>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <fstream>
#include <map>
#include <string>
#include <thread>

#include "cera_host.h"
#include "hip_llama.h"

namespace {

struct Args {
    std::map<std::string, std::string> kv;
    bool has(const std::string& k) const { return kv.count(k) != 0; }
    std::string str(const std::string& k, const std::string& d) const { return has(k) ? kv.at(k) : d; }
    uint64_t num(const std::string& k, uint64_t d) const { return has(k) ? std::strtoull(kv.at(k).c_str(), nullptr, 0) : d; }
};

Args parse(int argc, char** argv, int first) {
    Args a;
    for (int i = first; i < argc; ++i) {
        std::string k = argv[i];
        if (k.rfind("--", 0) != 0) {
            std::fprintf(stderr, "unexpected argument: %s\n", argv[i]);
            std::exit(2);
        }
        k = k.substr(2);
        if (i + 1 < argc && std::strncmp(argv[i + 1], "--", 2) != 0) a.kv[k] = argv[++i];
        else a.kv[k] = "1";
    }
    return a;
}

double now_s() { return std::chrono::duration<double>(std::chrono::steady_clock::now().time_since_epoch()).count(); }

uint64_t splitmix64(uint64_t& s) {
    s += 0x9E3779B97F4A7C15ull;
    uint64_t x = s;
    x = (x ^ (x >> 30)) * 0xBF58476D1CE4E5B9ull;
    x = (x ^ (x >> 27)) * 0x94D049BB133111EBull;
    return x ^ (x >> 31);
}

int cmd_gen(const Args& a) {
    if (!a.has("out")) { std::fprintf(stderr, "gen: --out is required\n"); return 2; }
    cera_synth_config c{};
    std::string preset = a.str("preset", "llama3-8b");
    if (preset == "llama3-8b") {
        c.n_layers = 32; c.hidden = 4096; c.ffn = 14336; c.n_heads = 32; c.n_kv_heads = 8; c.vocab = 128256;
        c.context_length = 8192; c.rope_theta = 500000.0f;
    } else if (preset == "tiny") {
        c.n_layers = 2; c.hidden = 256; c.ffn = 512; c.n_heads = 4; c.n_kv_heads = 2; c.head_dim = 128; c.vocab = 512;
        c.context_length = 256; c.rope_theta = 10000.0f;
    } else {
        std::fprintf(stderr, "gen: unknown preset %s\n", preset.c_str());
        return 2;
    }
    c.context_length = static_cast<uint32_t>(a.num("ctx", c.context_length));
    c.rms_eps = 1e-5f;
    c.weight_sigma = 0.02f;
    // Q4_K_M-style mix: attn_v, ffn_down and the output head in Q6_K, the rest in Q4_K
    c.type_token_embd = CERA_TYPE_Q4_K; c.type_output = CERA_TYPE_Q6_K;
    c.type_attn_q = c.type_attn_k = c.type_attn_output = c.type_ffn_gate = c.type_ffn_up = CERA_TYPE_Q4_K;
    c.type_attn_v = c.type_ffn_down = CERA_TYPE_Q6_K;
    // --quant q5_k_m: Q5_K in place of Q4_K; q4_0 | q8_0: every matrix in that 32-block type (the head stays Q6_K as
    // llama.cpp's converters leave it for q4_0, and follows for q8_0)
    const std::string quant = a.str("quant", "q4_k_m");
    if (quant == "q5_k_m") {   // Q5_K where Q4_K_M has Q4_K
        c.type_token_embd = c.type_attn_q = c.type_attn_k = c.type_attn_output = c.type_ffn_gate = c.type_ffn_up = CERA_TYPE_Q5_K;
    } else if (quant != "q4_k_m") {
        int t;
        if (quant == "q4_0") t = CERA_TYPE_Q4_0;
        else if (quant == "q8_0") t = CERA_TYPE_Q8_0;
        else { std::fprintf(stderr, "gen: --quant must be q4_k_m, q5_k_m, q4_0 or q8_0\n"); return 2; }
        c.type_token_embd = c.type_attn_q = c.type_attn_k = c.type_attn_v = c.type_attn_output = t;
        c.type_ffn_gate = c.type_ffn_up = c.type_ffn_down = t;
        if (quant == "q8_0") c.type_output = t;
    }
    char err[512] = {0};
    int threads = static_cast<int>(a.num("threads", std::max(1u, std::thread::hardware_concurrency())));
    double t0 = now_s();
    if (cera_synth_llama_gguf(a.str("out", "").c_str(), &c, a.num("seed", 1), threads, err, sizeof err) != 0) {
        std::fprintf(stderr, "gen failed: %s\n", err);
        return 1;
    }
    std::fprintf(stderr, "wrote %s in %.1f s\n", a.str("out", "").c_str(), now_s() - t0);
    return 0;
}

int cmd_inspect(const Args& a) {
    std::string err;
    auto g = cera::GgufFile::open(a.str("model", ""), &err);
    if (!g) { std::fprintf(stderr, "%s\n", err.c_str()); return 1; }
    for (const auto& kv : g->metadata()) {
        const cera::GgufValue& v = kv.second;
        if (v.type == cera::GGUF_STRING) std::printf("%s = \"%s\"\n", kv.first.c_str(), v.s.c_str());
        else if (v.type == cera::GGUF_F32 || v.type == cera::GGUF_F64) std::printf("%s = %g\n", kv.first.c_str(), v.f);
        else if (v.type == cera::GGUF_ARRAY) std::printf("%s = [%zu values]\n", kv.first.c_str(), v.arr.size());
        else if (v.type == cera::GGUF_I8 || v.type == cera::GGUF_I16 || v.type == cera::GGUF_I32 || v.type == cera::GGUF_I64)
            std::printf("%s = %lld\n", kv.first.c_str(), static_cast<long long>(v.i));
        else std::printf("%s = %llu\n", kv.first.c_str(), static_cast<unsigned long long>(v.u));
    }
    for (const auto& kv : g->tensors()) {
        std::printf("%-32s type %2u  [", kv.first.c_str(), kv.second.ggml_type);
        for (size_t i = 0; i < kv.second.shape.size(); ++i)
            std::printf("%s%llu", i ? ", " : "", static_cast<unsigned long long>(kv.second.shape[i]));
        std::printf("]  %llu bytes\n", static_cast<unsigned long long>(kv.second.size_bytes));
    }
    return 0;
}

int cmd_run(const Args& a) {
    std::string err;
    auto g = cera::GgufFile::open(a.str("model", ""), &err);
    if (!g) { std::fprintf(stderr, "%s\n", err.c_str()); return 1; }
    const size_t n_prompt = a.num("prompt-len", 512), n_predict = a.num("n-predict", 256), ubatch = a.num("ubatch", 512);
    const size_t ctx = a.num("ctx", std::max<size_t>(1024, n_prompt + n_predict));
    double t0 = now_s();
    std::unique_ptr<cera::Model> model;
    try {
        model = cera::load_model_hip(*g, ctx, static_cast<int>(a.num("device", 0)));
    } catch (const std::exception& e) {
        std::fprintf(stderr, "load failed: %s\n", e.what());
        return 1;
    }
    const std::string kv = a.str("kv", "f32");
    if (kv != "f32" && kv != "f16") { std::fprintf(stderr, "--kv must be f32 or f16\n"); return 1; }
    try {
        if (kv == "f16") {
            if (!model->f16_kv_supported()) { std::fprintf(stderr, "this backend has no f16 KV cache\n"); return 1; }
            model->configure_kv_compression(cera::KvCompression::F16);
        }
    } catch (const std::exception& e) {
        std::fprintf(stderr, "configure failed: %s\n", e.what());
        return 1;
    }
    double load_s = now_s() - t0;
    const cera::ModelConfig& c = model->config();
    std::vector<uint32_t> prompt(n_prompt);
    uint64_t s = a.num("seed", 1);
    for (auto& t : prompt) t = static_cast<uint32_t>(splitmix64(s) % c.vocab_size);

    std::vector<uint32_t> out;
    double prefill_s = 0, decode_s = 0;
    try {
        cera::InferenceState st;
        std::atomic<bool> cancel{false};
        double t1 = now_s();
        std::vector<float> logits;
        if (a.has("per-token-prefill")) {
            for (size_t i = 0; i < n_prompt; ++i) logits = model->forward(&prompt[i], 1, i, st);
        } else {
            auto r = model->forward_prefill_chunked(prompt.data(), n_prompt, 0, st, ubatch, cancel);
            logits = std::move(*r.second);
        }
        uint32_t next = 0;
        for (size_t i = 1; i < logits.size(); ++i)
            if (logits[i] > logits[next]) next = static_cast<uint32_t>(i);
        double t2 = now_s();
        out.push_back(next);
        while (out.size() < n_predict) out.push_back(model->forward_greedy(&out.back(), 1, st.seq_len, st));
        double t3 = now_s();
        prefill_s = t2 - t1;
        decode_s = t3 - t2;
    } catch (const std::exception& e) {
        std::fprintf(stderr, "inference failed: %s\n", e.what());
        return 1;
    }
    if (a.has("tokens-out")) {
        std::ofstream f(a.str("tokens-out", ""));
        for (uint32_t t : prompt) f << t << ' ';
        f << '\n';
        for (uint32_t t : out) f << t << ' ';
        f << '\n';
    }
    const double decode_steps = n_predict > 1 ? double(n_predict - 1) : 0.0;
    std::printf("{\"arch\": \"%s\", \"n_layers\": %zu, \"hidden\": %zu, \"vocab\": %zu, \"prompt_len\": %zu, "
                "\"n_predict\": %zu, \"ubatch\": %zu, \"kv\": \"%s\", \"load_s\": %.3f, \"gpu_memory_bytes\": %llu, "
                "\"prefill_s\": %.6f, \"prefill_tok_s\": %.2f, \"decode_s\": %.6f, \"decode_tok_s\": %.2f, "
                "\"first_tokens\": [%u, %u, %u, %u]}\n",
                c.architecture.c_str(), c.n_layers, c.hidden_size, c.vocab_size, n_prompt, n_predict, ubatch, kv.c_str(), load_s,
                static_cast<unsigned long long>(model->gpu_memory_bytes()), prefill_s, n_prompt / prefill_s, decode_s,
                decode_s > 0 ? decode_steps / decode_s : 0.0, out.size() > 0 ? out[0] : 0, out.size() > 1 ? out[1] : 0,
                out.size() > 2 ? out[2] : 0, out.size() > 3 ? out[3] : 0);
    return 0;
}

}  // namespace

int main(int argc, char** argv) {
    if (argc < 2) {
        std::fprintf(stderr, "usage: cera-hip gen|inspect|run [options]\n");
        return 2;
    }
    std::string cmd = argv[1];
    Args a = parse(argc, argv, 2);
    if (cmd == "gen") return cmd_gen(a);
    if (cmd == "inspect") return cmd_inspect(a);
    if (cmd == "run") return cmd_run(a);
    std::fprintf(stderr, "unknown command: %s\n", cmd.c_str());
    return 2;
}
