// HipLlamaModel over the C-ABI of cera_hip.h.  Reference lines: see hip_llama.h.
#include "hip_llama.h"

#include "cera_host.h"

#include <algorithm>
#include <cmath>
#include <cstring>

namespace cera {
namespace {

[[noreturn]] void bail(const std::string& m) { throw BackendError(m); }

uint32_t need_u32(const GgufFile& g, const std::string& key) {
    auto v = g.get_u32(key);
    if (!v) bail("missing " + key);
    return *v;
}

std::vector<float> need_f32_tensor(const GgufFile& g, const std::string& name) {
    std::vector<float> v;
    std::string e;
    if (!g.tensor_to_f32(name, &v, &e)) bail(e);
    return v;
}

cera_hip_tensor as_tensor(const GgufFile& g, const std::string& name) {
    WeightRef r;
    std::string e;
    if (!resolve_weight(g, name, &r, &e)) bail(e);
    const TensorInfo* info = g.tensor(name);
    cera_hip_tensor t{};
    t.ggml_type = r.ggml_type;
    t.m = r.m;
    t.k = r.k;
    t.data = g.tensor_data(*info);
    t.nbytes = r.size;
    return t;
}

size_t argmax(const std::vector<float>& v) {  // cera/src/sampler.rs:20-30
    size_t best = 0;
    float bv = -INFINITY;
    for (size_t i = 0; i < v.size(); ++i)
        if (v[i] > bv) { bv = v[i]; best = i; }
    return best;
}

}  // namespace

// ---- trait defaults (cera/src/model/mod.rs:207-220, 303-332, 494-497) ----

std::vector<float> Model::forward_prefill(const uint32_t* tokens, size_t n, size_t start_pos, InferenceState& state) {
    std::vector<float> logits;
    for (size_t i = 0; i < n; ++i) logits = forward(tokens + i, 1, start_pos + i, state);
    return logits;
}

uint32_t Model::forward_greedy(const uint32_t* tokens, size_t n, size_t pos, InferenceState& state) {
    return static_cast<uint32_t>(argmax(forward(tokens, n, pos, state)));
}

std::pair<size_t, std::optional<std::vector<float>>> Model::forward_prefill_chunked(
    const uint32_t* tokens, size_t n, size_t start_pos, InferenceState& state, size_t ubatch,
    const std::atomic<bool>& cancel) {
    if (ubatch == 0) ubatch = std::max<size_t>(n, 1);
    size_t consumed = 0;
    std::optional<std::vector<float>> last;
    while (consumed < n) {
        size_t len = std::min(ubatch, n - consumed);
        last = forward_prefill(tokens + consumed, len, start_pos + consumed, state);
        consumed += len;
        // polled after the chunk, so a cancel raised before the call still advances by one chunk
        if (cancel.load(std::memory_order_relaxed) && consumed < n) break;
    }
    return {consumed, std::move(last)};
}

// ---- HipLlamaModel ----

std::unique_ptr<HipLlamaModel> HipLlamaModel::from_gguf(const GgufFile& g, size_t context_size, int device) {
    if (context_size == 0) bail("context_size must be > 0");
    auto arch_opt = g.get_str("general.architecture");
    if (!arch_opt) bail("missing general.architecture");
    const std::string p = *arch_opt;

    std::unique_ptr<HipLlamaModel> self(new HipLlamaModel());
    if (p == "qwen2" || p == "qwen3") self->rope_type_ = RopeType::Neox;
    else if (p == "llama" || p == "granite") self->rope_type_ = RopeType::Norm;
    else bail("HipLlamaModel: no RoPE layout mapping for arch \"" + p + "\"");

    ModelConfig& c = self->config_;
    c.architecture = p;
    c.scalars.embedding = g.get_f32(p + ".embedding_scale").value_or(1.0f);
    c.scalars.residual = g.get_f32(p + ".residual_scale").value_or(1.0f);
    if (auto a = g.get_f32(p + ".attention.scale"); a && *a != 0.0f) c.scalars.attn = *a;
    c.scalars.logit = g.get_f32(p + ".logit_scale").value_or(1.0f);
    if (c.scalars.logit == 0.0f) bail(p + ".logit_scale must be non-zero");

    c.n_layers = need_u32(g, p + ".block_count");
    c.hidden_size = need_u32(g, p + ".embedding_length");
    c.intermediate_size = need_u32(g, p + ".feed_forward_length");
    c.n_heads = need_u32(g, p + ".attention.head_count");
    c.n_kv_heads = need_u32(g, p + ".attention.head_count_kv");
    if (c.n_heads == 0 || c.n_kv_heads == 0 || c.n_heads % c.n_kv_heads)
        bail("n_heads (" + std::to_string(c.n_heads) + ") must be a positive multiple of n_kv_heads (" +
             std::to_string(c.n_kv_heads) + ")");
    if (auto v = g.get_u32(p + ".vocab_size")) {
        c.vocab_size = *v;
    } else {
        const TensorInfo* e = g.tensor("token_embd.weight");
        if (!e) bail("missing token_embd.weight (cannot derive vocab_size)");
        if (e->shape.size() < 2) bail("token_embd.weight has unexpected shape");
        c.vocab_size = e->shape[1];
    }
    size_t gguf_ctx = g.get_u32(p + ".context_length").value_or(128000);
    c.max_seq_len = std::min(context_size, gguf_ctx);
    c.rope_theta = g.get_f32(p + ".rope.freq_base").value_or(1000000.0f);
    c.rms_norm_eps = g.get_f32(p + ".attention.layer_norm_rms_epsilon").value_or(1e-6f);
    if (auto kl = g.get_u32(p + ".attention.key_length")) c.head_dim = *kl;
    else c.head_dim = c.hidden_size / c.n_heads;
    if (c.head_dim == 0) bail("head_dim must be > 0");

    // host-side vectors stay alive until model_create has copied them
    std::vector<float> output_norm = need_f32_tensor(g, "output_norm.weight");
    struct LayerVecs { std::vector<float> attn_norm, ffn_norm, q_norm, k_norm, q_bias, k_bias, v_bias; };
    std::vector<LayerVecs> vecs(c.n_layers);
    std::vector<cera_hip_layer> layers(c.n_layers);
    auto expect_len = [](const std::vector<float>& v, size_t n, const std::string& name) {
        if (v.size() != n) bail(name + " has " + std::to_string(v.size()) + " entries, expected " + std::to_string(n));
    };
    expect_len(output_norm, c.hidden_size, "output_norm.weight");
    const size_t q_dim = c.n_heads * c.head_dim, kv_dim = c.n_kv_heads * c.head_dim;
    for (size_t i = 0; i < c.n_layers; ++i) {
        const std::string b = "blk." + std::to_string(i) + ".";
        LayerVecs& v = vecs[i];
        cera_hip_layer& L = layers[i];
        std::memset(&L, 0, sizeof L);
        v.attn_norm = need_f32_tensor(g, b + "attn_norm.weight");
        v.ffn_norm = need_f32_tensor(g, b + "ffn_norm.weight");
        expect_len(v.attn_norm, c.hidden_size, b + "attn_norm.weight");
        expect_len(v.ffn_norm, c.hidden_size, b + "ffn_norm.weight");
        L.attn_norm = v.attn_norm.data();
        L.ffn_norm = v.ffn_norm.data();
        if (g.tensor(b + "attn_q_norm.weight")) {  // Qwen3 QK-norm, gated on presence
            v.q_norm = need_f32_tensor(g, b + "attn_q_norm.weight");
            v.k_norm = need_f32_tensor(g, b + "attn_k_norm.weight");
            expect_len(v.q_norm, c.head_dim, b + "attn_q_norm.weight");
            expect_len(v.k_norm, c.head_dim, b + "attn_k_norm.weight");
            L.q_norm = v.q_norm.data();
            L.k_norm = v.k_norm.data();
        }
        if (g.tensor(b + "attn_q.bias")) {  // Qwen2 biases, gated on presence
            v.q_bias = need_f32_tensor(g, b + "attn_q.bias");
            v.k_bias = need_f32_tensor(g, b + "attn_k.bias");
            v.v_bias = need_f32_tensor(g, b + "attn_v.bias");
            expect_len(v.q_bias, q_dim, b + "attn_q.bias");
            expect_len(v.k_bias, kv_dim, b + "attn_k.bias");
            expect_len(v.v_bias, kv_dim, b + "attn_v.bias");
            L.q_bias = v.q_bias.data();
            L.k_bias = v.k_bias.data();
            L.v_bias = v.v_bias.data();
        }
        L.attn_q = as_tensor(g, b + "attn_q.weight");
        L.attn_k = as_tensor(g, b + "attn_k.weight");
        L.attn_v = as_tensor(g, b + "attn_v.weight");
        L.attn_output = as_tensor(g, b + "attn_output.weight");
        L.ffn_gate = as_tensor(g, b + "ffn_gate.weight");
        L.ffn_up = as_tensor(g, b + "ffn_up.weight");
        L.ffn_down = as_tensor(g, b + "ffn_down.weight");
    }
    cera_hip_tensor embd = as_tensor(g, "token_embd.weight");
    cera_hip_tensor output{};
    const bool untied = g.tensor("output.weight") != nullptr;
    if (untied) output = as_tensor(g, "output.weight");
    {
        const cera_hip_tensor& head = untied ? output : embd;
        const char* head_name = untied ? "output.weight" : "token_embd.weight";
        if (head.k != c.hidden_size)
            bail(std::string("LM head `") + head_name + "` has k=" + std::to_string(head.k) + " but hidden_size is " +
                 std::to_string(c.hidden_size));
        if (head.m < c.vocab_size)
            bail(std::string("LM head `") + head_name + "` has " + std::to_string(head.m) +
                 " rows, fewer than vocab_size " + std::to_string(c.vocab_size));
        if (c.hidden_size % 32)
            bail("hidden_size " + std::to_string(c.hidden_size) +
                 " is not a multiple of 32, which the Q8_0 activation quantization requires");
    }
    std::vector<float> rope_freqs;
    if (g.tensor("rope_freqs.weight")) {
        rope_freqs = need_f32_tensor(g, "rope_freqs.weight");
        expect_len(rope_freqs, c.head_dim / 2, "rope_freqs.weight");
    }

    cera_hip_config hc{};
    hc.n_layers = static_cast<uint32_t>(c.n_layers);
    hc.hidden = static_cast<uint32_t>(c.hidden_size);
    hc.ffn = static_cast<uint32_t>(c.intermediate_size);
    hc.n_heads = static_cast<uint32_t>(c.n_heads);
    hc.n_kv_heads = static_cast<uint32_t>(c.n_kv_heads);
    hc.head_dim = static_cast<uint32_t>(c.head_dim);
    hc.vocab = static_cast<uint32_t>(c.vocab_size);
    hc.max_seq_len = static_cast<uint32_t>(c.max_seq_len);
    hc.rope_type = self->rope_type_ == RopeType::Norm ? 1u : 0u;
    hc.rope_theta = c.rope_theta;
    hc.rms_eps = c.rms_norm_eps;
    hc.embed_scale = c.scalars.embedding;
    hc.residual_scale = c.scalars.residual;
    hc.attn_scale = c.scalars.attn.value_or(0.0f);
    hc.logit_scale = c.scalars.logit;
    hc.rope_freqs = rope_freqs.empty() ? nullptr : rope_freqs.data();

    if (cera_hip_ctx_create(device, nullptr, &self->ctx_) != CERA_HIP_OK)
        bail(std::string("hip context: ") + cera_hip_last_error(nullptr));
    if (cera_hip_model_create(self->ctx_, &hc, &embd, untied ? &output : nullptr, output_norm.data(), layers.data(),
                              &self->model_) != CERA_HIP_OK)
        bail(std::string("hip model: ") + cera_hip_last_error(self->ctx_));
    return self;
}

HipLlamaModel::~HipLlamaModel() {
    if (model_) cera_hip_model_destroy(model_);
    if (ctx_) cera_hip_ctx_destroy(ctx_);
}

void HipLlamaModel::device_panic(const char* what) const {
    throw BackendError(std::string(what) + ": " + cera_hip_last_error(ctx_));
}

std::vector<float> HipLlamaModel::forward(const uint32_t* tokens, size_t n, size_t pos, InferenceState& state) {
    if (n != 1) bail("HipLlamaModel forward expects single token");
    if (tokens[0] >= config_.vocab_size)
        bail("token_id " + std::to_string(tokens[0]) + " out of range (vocab_size=" + std::to_string(config_.vocab_size) + ")");
    std::vector<float> logits(config_.vocab_size);
    if (cera_hip_forward(model_, tokens[0], static_cast<uint32_t>(pos), logits.data()) != CERA_HIP_OK)
        device_panic("forward");
    state.seq_len = cera_hip_seq_len(model_);
    return logits;
}

std::vector<float> HipLlamaModel::forward_prefill(const uint32_t* tokens, size_t n, size_t start_pos,
                                                  InferenceState& state) {
    if (n == 0) bail("forward_prefill requires at least one token");
    if (start_pos != state.seq_len)
        bail("forward_prefill: start_pos (" + std::to_string(start_pos) + ") must equal state.seq_len (" +
             std::to_string(state.seq_len) + ")");
    std::vector<float> logits(config_.vocab_size);
    if (cera_hip_forward_prefill(model_, tokens, static_cast<uint32_t>(n), static_cast<uint32_t>(start_pos),
                                 logits.data()) != CERA_HIP_OK)
        device_panic("forward_prefill");
    state.seq_len = cera_hip_seq_len(model_);
    return logits;
}

std::vector<float> HipLlamaModel::forward_prefill_logits_all(const uint32_t* tokens, size_t n, size_t start_pos,
                                                             InferenceState& state) {
    if (n == 0) bail("forward_prefill_logits_all requires at least one token");
    if (start_pos != state.seq_len)
        bail("forward_prefill_logits_all: start_pos (" + std::to_string(start_pos) + ") must equal state.seq_len (" +
             std::to_string(state.seq_len) + ")");
    std::vector<float> logits(n * config_.vocab_size);
    if (cera_hip_forward_prefill_logits_all(model_, tokens, static_cast<uint32_t>(n), static_cast<uint32_t>(start_pos),
                                            logits.data()) != CERA_HIP_OK)
        device_panic("forward_prefill_logits_all");
    state.seq_len = cera_hip_seq_len(model_);
    return logits;
}

uint32_t HipLlamaModel::forward_greedy(const uint32_t* tokens, size_t n, size_t pos, InferenceState& state) {
    if (n != 1) bail("HipLlamaModel forward_greedy expects single token");
    uint32_t next = 0;
    if (cera_hip_forward_greedy(model_, tokens[0], static_cast<uint32_t>(pos), &next) != CERA_HIP_OK)
        device_panic("forward_greedy");
    state.seq_len = cera_hip_seq_len(model_);
    return next;
}

void HipLlamaModel::truncate_kv(InferenceState& state, size_t len) {
    if (len > state.seq_len)
        bail("truncate_kv: len (" + std::to_string(len) + ") exceeds seq_len (" + std::to_string(state.seq_len) + ")");
    if (cera_hip_truncate_kv(model_, static_cast<uint32_t>(len)) != CERA_HIP_OK) device_panic("truncate_kv");
    state.seq_len = len;
}

// The trait defaults panic with unimplemented!(): a backend without device-resident state has
// nothing to snapshot (cera/src/model/mod.rs:521-533).
StateSnapshot Model::snapshot_state() { throw BackendError("snapshot_state not supported by this backend"); }
void Model::restore_state(const StateSnapshot&) { throw BackendError("restore_state not supported by this backend"); }

void HipLlamaModel::shift_kv(InferenceState& state, size_t n_keep, size_t shift) {
    // the reference asserts these in all builds (cera/src/kv_cache.rs:1110-1116)
    if (shift == 0) bail("shift_kv: shift must be > 0");
    if (n_keep + shift > state.seq_len)
        bail("shift range out of bounds: n_keep=" + std::to_string(n_keep) + " + shift=" + std::to_string(shift) +
             " > seq_len=" + std::to_string(state.seq_len));
    if (cera_hip_shift_kv(model_, static_cast<uint32_t>(n_keep), static_cast<uint32_t>(shift)) != CERA_HIP_OK)
        device_panic("shift_kv");
    state.seq_len = cera_hip_seq_len(model_);
}

void HipLlamaModel::configure_kv_compression(KvCompression mode) {
    // a second call with a different mode is CeraError::KvCompressionConflict in the reference
    if (cera_hip_configure_kv(model_, mode == KvCompression::F16 ? CERA_HIP_KV_F16 : CERA_HIP_KV_F32) != CERA_HIP_OK)
        bail(std::string("configure_kv_compression: ") + cera_hip_last_error(ctx_));
}
KvCompression HipLlamaModel::kv_compression() const {
    return cera_hip_kv_type(model_) == CERA_HIP_KV_F16 ? KvCompression::F16 : KvCompression::None;
}

// the integer-only converters of the host library (the reference's, cera/src/quant.rs:48-164)
static uint16_t half_bits(float v) { return cera_f32_to_f16(v); }
static float half_value(uint16_t b) { return cera_f16_to_f32(b); }

StateSnapshot HipLlamaModel::snapshot_state() {
    StateSnapshot snap;
    snap.seq_len = cera_hip_seq_len(model_);
    const bool f16 = kv_compression() == KvCompression::F16;
    const size_t elems = snap.seq_len * config_.n_kv_heads * config_.head_dim;
    std::vector<float> k(elems), v(elems);
    snap.layers.resize(config_.n_layers);
    for (size_t l = 0; l < config_.n_layers; ++l) {
        LayerSnapshot& L = snap.layers[l];
        L.f16 = f16;
        if (elems && cera_hip_read_kv(model_, static_cast<uint32_t>(l), k.data(), v.data()) != CERA_HIP_OK)
            device_panic("snapshot_state");
        if (!f16) {
            L.k_data.assign(reinterpret_cast<uint8_t*>(k.data()), reinterpret_cast<uint8_t*>(k.data() + elems));
            L.v_data.assign(reinterpret_cast<uint8_t*>(v.data()), reinterpret_cast<uint8_t*>(v.data() + elems));
        } else {  // the cache's own half bits: read_kv widened them exactly
            L.k_data.resize(elems * 2);
            L.v_data.resize(elems * 2);
            for (size_t i = 0; i < elems; ++i) {
                const uint16_t kb = half_bits(k[i]), vb = half_bits(v[i]);
                std::memcpy(L.k_data.data() + 2 * i, &kb, 2);
                std::memcpy(L.v_data.data() + 2 * i, &vb, 2);
            }
        }
    }
    return snap;
}

void HipLlamaModel::restore_state(const StateSnapshot& snap) {
    const bool f16 = kv_compression() == KvCompression::F16;
    const size_t elems = snap.seq_len * config_.n_kv_heads * config_.head_dim;
    const size_t bytes = elems * (f16 ? 2 : 4);
    if (snap.layers.size() != config_.n_layers) bail("restore_state: snapshot has " + std::to_string(snap.layers.size()) +
                                                     " layers, model has " + std::to_string(config_.n_layers));
    if (snap.seq_len > config_.max_seq_len) bail("restore_state: snapshot is longer than the context");
    for (const LayerSnapshot& L : snap.layers) {
        // the cross-mode gate: an f16 snapshot never loads into an f32 cache or the reverse
        if (L.f16 != f16) bail("restore_state: snapshot and model disagree on the KV cache element type");
        if (L.k_data.size() != bytes || L.v_data.size() != bytes)
            bail("restore_state: layer byte length does not match seq_len * kv_dim * element size");
    }
    std::vector<float> k(elems), v(elems);
    for (size_t l = 0; l < config_.n_layers; ++l) {
        const LayerSnapshot& L = snap.layers[l];
        if (!f16) {
            std::memcpy(k.data(), L.k_data.data(), bytes);
            std::memcpy(v.data(), L.v_data.data(), bytes);
        } else {
            for (size_t i = 0; i < elems; ++i) {
                uint16_t kb, vb;
                std::memcpy(&kb, L.k_data.data() + 2 * i, 2);
                std::memcpy(&vb, L.v_data.data() + 2 * i, 2);
                k[i] = half_value(kb);
                v[i] = half_value(vb);
            }
        }
        if (cera_hip_write_kv(model_, static_cast<uint32_t>(l), k.data(), v.data(), static_cast<uint32_t>(snap.seq_len)) !=
            CERA_HIP_OK)
            device_panic("restore_state");
    }
    if (cera_hip_set_seq_len(model_, static_cast<uint32_t>(snap.seq_len)) != CERA_HIP_OK) device_panic("restore_state");
}

void HipLlamaModel::set_reference_order(uint32_t mode) {
    if (cera_hip_set_reference_order(model_, mode) != CERA_HIP_OK)
        bail(std::string("set_reference_order: ") + cera_hip_last_error(ctx_));
}

uint64_t HipLlamaModel::gpu_memory_bytes() const { return cera_hip_memory_bytes(model_); }

std::string HipLlamaModel::device_name() const {
    char name[256] = {0};
    uint32_t cu = 0;
    uint64_t hbm = 0;
    if (cera_hip_device_info(ctx_, name, &cu, &hbm) != CERA_HIP_OK) return "unknown";
    return std::string(name) + " (" + std::to_string(cu) + " CUs, " + std::to_string(hbm >> 30) + " GiB)";
}

std::unique_ptr<Model> load_model_hip(const GgufFile& gguf, size_t context_size, int device) {
    std::string arch = gguf.get_str("general.architecture").value_or("unknown");
    if (arch == "qwen2" || arch == "qwen3" || arch == "llama" || arch == "granite")
        return HipLlamaModel::from_gguf(gguf, context_size, device);
    bail("unsupported architecture for hip: " + arch);
}

}  // namespace cera
