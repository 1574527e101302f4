// HipLlamaModel: the `Model`-trait implementation a `--device hip` backend adds
// to cera, written against the C-ABI of cera_hip.h only (the same calls a Rust
// `impl Model for HipLlamaModel` over a -sys crate would make).
//
// Reference surface mirrored here:
//   * trait Model                      cera/src/model/mod.rs:200-606
//   * LlamaModel::from_gguf_with_id    cera/src/model/llama.rs:158-450 (metadata keys, defaults,
//                                      load-time checks, optional tensors)
//   * the device-resident-KV contract  cera/src/model/mod.rs:176-199, 251-283: the backend keeps its
//                                      own position counter and keeps InferenceState::seq_len equal to it
//   * forward_prefill_chunked default  cera/src/model/mod.rs:303-332
//
// Rust's forward methods are infallible by signature and the reference GPU
// backends panic on a device error; here such an error throws
// cera::BackendError, which the C face in hip_llama_capi.cpp turns into a
// status code so nothing unwinds across a C boundary.
#pragma once
#include <atomic>
#include <cstdint>
#include <memory>
#include <optional>
#include <stdexcept>
#include <string>
#include <utility>
#include <vector>

#include "cera_hip.h"
#include "gguf.h"

namespace cera {

struct BackendError : std::runtime_error {
    using std::runtime_error::runtime_error;
};

enum class RopeType { Neox = 0, Norm = 1 };

// cera/src/model/mod.rs:52-113
struct ScalarMultipliers {
    float embedding = 1.0f, residual = 1.0f;
    std::optional<float> attn;  // absent (or stored 0.0) => 1/sqrt(head_dim)
    float logit = 1.0f;
};

// cera/src/model/mod.rs:117-145 (the fields a dense transformer uses)
struct ModelConfig {
    std::string architecture;
    size_t n_layers = 0, hidden_size = 0, intermediate_size = 0, n_heads = 0, n_kv_heads = 0, head_dim = 0,
           vocab_size = 0, max_seq_len = 0;
    float rope_theta = 1000000.0f, rms_norm_eps = 1e-6f;
    ScalarMultipliers scalars;
};

// The KV cache lives in HBM inside the model; only the position counter is
// mirrored on the caller's side (InferenceState::seq_len in cera).
struct InferenceState {
    size_t seq_len = 0;
};

// cera/src/kv_cache.rs:1382-1396: per attention layer the raw f32 K and V bytes of rows
// [0, seq_len), time-major [pos][kv_dim] (LayerSnapshot::Attention).
// With an f16 cache the bytes are the raw little-endian half bits (LayerSnapshot::AttentionF16,
// cera/src/kv_cache.rs:1411-1421); `f16` is the variant tag restore checks.
struct LayerSnapshot {
    std::vector<uint8_t> k_data, v_data;
    bool f16 = false;
};
struct StateSnapshot {
    std::vector<LayerSnapshot> layers;
    size_t seq_len = 0;
};

// cera/src/kv_cache.rs:88-110, the modes a dense transformer on this backend honours
enum class KvCompression { None = 0, F16 = 1 };

// The subset of `trait Model` a text backend implements.
class Model {
public:
    virtual ~Model() = default;
    virtual std::vector<float> forward(const uint32_t* tokens, size_t n_tokens, size_t pos, InferenceState& state) = 0;
    virtual std::vector<float> forward_prefill(const uint32_t* tokens, size_t n_tokens, size_t start_pos,
                                               InferenceState& state);
    virtual uint32_t forward_greedy(const uint32_t* tokens, size_t n_tokens, size_t pos, InferenceState& state);
    // logits of every position, row-major [n_tokens * vocab]; empty unless supports_all_logits()
    virtual std::vector<float> forward_prefill_logits_all(const uint32_t*, size_t, size_t, InferenceState&) { return {}; }
    virtual void truncate_kv(InferenceState& state, size_t len) = 0;
    // n_keep context shift (cera/src/model/mod.rs:336-365): callers check supports_kv_shift() first
    virtual void shift_kv(InferenceState&, size_t /*n_keep*/, size_t /*shift*/) {}
    // prefix-cache snapshots (cera/src/model/mod.rs:507-533)
    virtual struct StateSnapshot snapshot_state();
    virtual void restore_state(const struct StateSnapshot&);
    // (tokens consumed, logits of the last processed chunk); chunks of `ubatch` (0 = one chunk),
    // `cancel` polled after each chunk.
    std::pair<size_t, std::optional<std::vector<float>>> forward_prefill_chunked(const uint32_t* tokens, size_t n_tokens,
                                                                                 size_t start_pos, InferenceState& state,
                                                                                 size_t ubatch,
                                                                                 const std::atomic<bool>& cancel);
    virtual const ModelConfig& config() const = 0;
    virtual uint64_t gpu_memory_bytes() const { return 0; }
    virtual bool supports_all_logits() const { return false; }
    virtual bool supports_kv_shift() const { return false; }
    virtual bool supports_embedding_input() const { return false; }
    virtual bool supports_hidden_states() const { return false; }
    virtual bool turboquant_supported() const { return false; }
    virtual bool f16_kv_supported() const { return false; }
    // cera/src/model/mod.rs:557-592: called before any forward pass; first call wins
    virtual void configure_kv_compression(KvCompression) {}
};

class HipLlamaModel final : public Model {
public:
    // Parses metadata, resolves every tensor in the mapping and uploads it to HBM in
    // its native block layout.  Throws BackendError with the reason on any failure
    // (missing key/tensor, unsupported arch or tensor type, shape mismatch, device error).
    static std::unique_ptr<HipLlamaModel> from_gguf(const GgufFile& gguf, size_t context_size, int device = 0);
    ~HipLlamaModel() override;

    std::vector<float> forward(const uint32_t* tokens, size_t n_tokens, size_t pos, InferenceState& state) override;
    std::vector<float> forward_prefill(const uint32_t* tokens, size_t n_tokens, size_t start_pos,
                                       InferenceState& state) override;
    uint32_t forward_greedy(const uint32_t* tokens, size_t n_tokens, size_t pos, InferenceState& state) override;
    std::vector<float> forward_prefill_logits_all(const uint32_t* tokens, size_t n_tokens, size_t start_pos,
                                                  InferenceState& state) override;
    bool supports_all_logits() const override { return true; }
    void truncate_kv(InferenceState& state, size_t len) override;
    // the shift kernel is instantiated for the head sizes models use
    bool supports_kv_shift() const override {
        const size_t hd = config_.head_dim;
        return hd == 32 || hd == 64 || hd == 80 || hd == 96 || hd == 128 || hd == 256;
    }
    bool f16_kv_supported() const override { return true; }
    void configure_kv_compression(KvCompression mode) override;
    KvCompression kv_compression() const;
    void shift_kv(InferenceState& state, size_t n_keep, size_t shift) override;
    StateSnapshot snapshot_state() override;
    void restore_state(const StateSnapshot& snapshot) override;
    const ModelConfig& config() const override { return config_; }
    uint64_t gpu_memory_bytes() const override;

    // verification hook: run every forward on the reference-order kernels (bit-identical to the
    // CPU AVX2 path, many times slower); only with an empty cache
    // 0 off, 1 reference order with per-token prefill, 2 with the x86 host's batched prefill (cera_hip.h)
    void set_reference_order(uint32_t mode);
    RopeType rope_type() const { return rope_type_; }
    std::string device_name() const;

private:
    HipLlamaModel() = default;
    [[noreturn]] void device_panic(const char* what) const;
    ModelConfig config_;
    RopeType rope_type_ = RopeType::Norm;
    cera_hip_ctx* ctx_ = nullptr;
    cera_hip_model* model_ = nullptr;
};

// load_model_gpu's twin (cera/src/model/mod.rs:672-703): arch allow-list, then the model.
std::unique_ptr<Model> load_model_hip(const GgufFile& gguf, size_t context_size, int device = 0);

}  // namespace cera
