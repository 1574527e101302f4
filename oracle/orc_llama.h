// CPU oracle (test infrastructure only): model-level twin of cera's LlamaModel.
#pragma once
#include "orc_common.h"

struct OrcTensor {
    uint32_t dtype;
    uint32_t _pad;
    uint64_t m, k;      // m output rows, k inner dimension (GGUF shape is [k, m])
    const void* data;   // row-major blocks, GGUF byte layout
};

struct OrcLlamaLayer {
    const float* attn_norm;
    const float* ffn_norm;
    OrcTensor attn_q, attn_k, attn_v, attn_output, ffn_gate, ffn_up, ffn_down;
    const float *q_bias, *k_bias, *v_bias;  // nullable (Qwen2)
    const float *q_norm, *k_norm;           // nullable (Qwen3)
};

struct OrcLlamaConfig {
    uint32_t n_layers, hidden, ffn, n_heads, n_kv_heads, head_dim, vocab, max_seq_len;
    uint32_t rope_type;  // 0 neox, 1 norm
    float rope_theta, rms_eps, embed_scale, residual_scale, attn_scale /*0 => 1/sqrt(hd)*/, logit_scale;
    const float* rope_freqs;  // nullable, head_dim/2
};

struct OrcLlama;

ORC_API OrcLlama* orc_llama_create(const OrcLlamaConfig* cfg, const OrcTensor* embd,
                                   const OrcTensor* output /*nullable => tied*/,
                                   const float* output_norm, const OrcLlamaLayer* layers, int variant);
ORC_API void     orc_llama_destroy(OrcLlama*);
ORC_API void     orc_llama_set_pool(OrcLlama*, void* pool);
ORC_API void     orc_llama_set_kv_f16(OrcLlama*, int on);  // KvCompression::F16; set before the first forward
// batched prefill through the x86 route of transformer::gemm_preq (repacked Q4_0 / Q4_K weights)
ORC_API void     orc_llama_set_x86_repack(OrcLlama*, int on);
ORC_API uint32_t orc_llama_seq_len(const OrcLlama*);
ORC_API void     orc_llama_truncate(OrcLlama*, uint32_t len);
ORC_API int      orc_llama_forward(OrcLlama*, uint32_t token, uint32_t pos, float* logits /*nullable*/,
                                   float* hidden_out /*nullable*/);
ORC_API int      orc_llama_forward_prefill_per_token(OrcLlama*, const uint32_t* tokens, uint32_t n,
                                                     uint32_t start_pos, float* last_logits);
// LlamaModel::forward_prefill_batched (llama.rs:738-1523): all n tokens through
// each layer together; logits of the last token.  all_hidden (nullable)
// receives the per-token final-normed hidden states [n][hidden].
ORC_API int      orc_llama_forward_prefill_batched(OrcLlama*, const uint32_t* tokens, uint32_t n,
                                                   uint32_t start_pos, float* last_logits, float* all_hidden);
ORC_API int      orc_llama_shift_kv(OrcLlama*, uint32_t n_keep, uint32_t shift);
ORC_API int      orc_llama_restore_kv(OrcLlama*, uint32_t layer, const float* k, const float* v, uint32_t n_pos);
ORC_API void     orc_llama_set_seq_len(OrcLlama*, uint32_t len);
ORC_API const float* orc_llama_kcache(const OrcLlama*, uint32_t layer);
ORC_API const float* orc_llama_vcache(const OrcLlama*, uint32_t layer);
