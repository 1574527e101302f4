// Device-resident model state shared by model.hip and prefill.hip.
#pragma once
#include <mutex>
#include <vector>

#include "host_common.h"

struct LayerDev {
    cera_hip_dtensor *q = nullptr, *k = nullptr, *v = nullptr, *o = nullptr, *gate = nullptr, *up = nullptr,
                     *down = nullptr;
    // q|k (and |v when all three share a type) stored back to back so decode runs them as one
    // GEMV; then q, k (, v) above are row-range views into it
    cera_hip_dtensor* qkv = nullptr;
    uint32_t qkv_rows = 0;  // rows covered by the fused launch (0: not fused)
    float *attn_norm = nullptr, *ffn_norm = nullptr;
    float *q_bias = nullptr, *k_bias = nullptr, *v_bias = nullptr, *q_norm = nullptr, *k_norm = nullptr;
    void *kc = nullptr, *vc = nullptr;  // [n_kv_heads][max_seq_len][head_dim], f32 or half (model->kv_f16)
};

struct cera_hip_model {
    cera_hip_ctx* ctx = nullptr;
    cera_hip_config cfg{};
    cera_hip_dtensor *embd = nullptr, *output = nullptr;
    float* output_norm = nullptr;
    std::vector<LayerDev> layers;
    float* rope_table = nullptr;  // [max_seq_len][head_dim/2] (cos, sin)
    std::vector<float> rope_ff;   // host copy of the per-pair frequency factors (empty: none)
    float* shift_cs = nullptr;    // [head_dim/2] (cos, sin) of the last context shift's delta rotation
    // single-token activations
    float *hidden = nullptr, *normed = nullptr, *q = nullptr, *k = nullptr, *v = nullptr, *attn_out = nullptr,
          *proj = nullptr, *act = nullptr, *up = nullptr, *xs = nullptr, *logits = nullptr;
    int8_t* xq = nullptr;
    uint32_t* scalars = nullptr;  // device: [token, pos, argmax result, spare]
    std::vector<void*> owned;     // plain device allocations freed with the model
    // batched-prefill activations, token-major [n][dim], allocated on first use
    uint32_t pf_cap = 0;
    uint64_t pf_bytes = 0;        // bytes held by pf_owned (part of `bytes`)
    float *pf_hidden = nullptr, *pf_normed = nullptr, *pf_q = nullptr, *pf_k = nullptr, *pf_v = nullptr,
          *pf_attn = nullptr, *pf_gate = nullptr, *pf_up = nullptr, *pf_xs = nullptr, *pf_bsum = nullptr;
    int8_t* pf_xq = nullptr;
    void* pf_x8 = nullptr;   // the same activations as the fragment-ordered fp8 split copy (Q4_K GEMMs)
    void* pf_xh = nullptr;   // the same quants as f16 (Q6_K GEMMs run their dots on the f16 matrix cores)
    uint32_t* pf_tokens = nullptr;
    float* pf_logits = nullptr;   // [pf_cap][head rows], allocated on the first all-logits call
    uint32_t pf_logits_cap = 0;
    std::vector<void*> pf_owned;
    uint32_t seq_len = 0;
    // reference-order verification route (reforder.hip): every f32 operation in the CPU path's
    // order, bit-identical logits; slow, never the default
    uint32_t ref_order = 0;   // 0 fast route; 1 reference order, per-token prefill; 2 reference order, the x86 host's batched prefill
    float* ref_scores = nullptr;  // [n_heads][max_seq_len] attention scores of that route
    bool kv_f16 = false;          // KV caches hold IEEE half instead of f32
    bool kv_configured = false;   // cera_hip_configure_kv was called: a different mode is a conflict
    bool kv_broken = false;       // a cache re-allocation failed part-way: every later call fails
    uint64_t bytes = 0;
    // every trait call is serialised, like the reference GPU backends' infer_lock
    // (cera/src/model/mod.rs:184-199)
    std::mutex infer_lock;
};

// Held for the length of a model-level call: the model's own lock, then the lock of the context
// whose stream and workspaces (scratch slots, attention partials) the call uses -- two models on
// one context may be driven from two threads.
struct ModelLock {
    std::lock_guard<std::mutex> model;
    std::lock_guard<std::recursive_mutex> ctx;
    explicit ModelLock(cera_hip_model* m) : model(m->infer_lock), ctx(m->ctx->op_mu) {}
};

cera_hip_status cera_attn_step(cera_hip_ctx* ctx, float* q, float* k_new, const float* v_new, void* kc, void* vc,
                               const float* rope_table, const uint32_t* pos_dev, uint32_t pos, uint32_t n_heads,
                               uint32_t n_kv_heads, uint32_t head_dim, uint32_t max_seq, uint32_t rope_type, float scale,
                               bool kv_f16, float* out, float* out_scales, int8_t* out_quants);
void cera_build_rope_table(uint32_t max_seq, uint32_t head_dim, float base, const float* ff, std::vector<float>& out);
cera_hip_status cera_model_prefill_per_token(cera_hip_model* m, const uint32_t* tokens, uint32_t n, uint32_t start_pos,
                                             float* last_logits);
// batched route (prefill.hip); falls back to the per-token route when a weight
// type has no int8 GEMM
cera_hip_status cera_model_prefill(cera_hip_model* m, const uint32_t* tokens, uint32_t n, uint32_t start_pos,
                                   float* last_logits);
// same, logits of every position into logits_all[n][vocab] (host)
cera_hip_status cera_model_prefill_logits_all(cera_hip_model* m, const uint32_t* tokens, uint32_t n, uint32_t start_pos,
                                              float* logits_all);
// one token through the reference-order kernels (reforder.hip)
cera_hip_status cera_model_decode_step_ref(cera_hip_model* m, uint32_t pos, bool want_logits);
// n tokens in one pass in the order of the x86 host's forward_prefill_batched (reforder.hip); the
// last row's logits are left in m->logits when want_logits
cera_hip_status cera_model_prefill_ref_batched(cera_hip_model* m, const uint32_t* tokens, uint32_t n, uint32_t start_pos,
                                               bool want_logits);
// (re)allocates the prefill pass buffers for n tokens (at most one pass's capacity, m->pf_cap)
cera_hip_status cera_model_ensure_prefill_buffers(cera_hip_model* m, uint32_t n);
// hipMalloc for allocations made after model creation: out of memory -> the decode copies are
// freed and the allocation is tried once more
cera_hip_status cera_model_malloc(cera_hip_model* m, void** out, uint64_t bytes, const char* what);
uint64_t cera_model_drop_decode_copies(cera_hip_model* m);
bool cera_model_ref_order_supported(const cera_hip_model* m, std::string* why);
cera_hip_status cera_model_decode_logits(cera_hip_model* m, uint32_t token, uint32_t pos, float* logits);
