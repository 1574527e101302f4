/* C face of HipLlamaModel (hip_llama.h) for callers without C++: the ctypes
 * tests and the bench driver.  One handle = one loaded model + its
 * InferenceState + a cancel flag.  Every call returns 0 on success and -1 on
 * failure with the reason readable through cera_llama_last_error (the C++
 * layer's BackendError never crosses this boundary). */
#pragma once
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define CERA_LLAMA_API __attribute__((visibility("default")))

typedef struct cera_llama cera_llama;

typedef struct {
    uint64_t n_layers, hidden_size, intermediate_size, n_heads, n_kv_heads, head_dim, vocab_size, max_seq_len;
    float rope_theta, rms_norm_eps;
    uint32_t rope_type; /* 0 NEOX, 1 NORM */
} cera_llama_config;

CERA_LLAMA_API cera_llama* cera_llama_open(const char* gguf_path, uint64_t context_size, int device, char* err,
                                           uint64_t err_len);
CERA_LLAMA_API void cera_llama_close(cera_llama*);
CERA_LLAMA_API const char* cera_llama_last_error(const cera_llama*);
CERA_LLAMA_API int cera_llama_get_config(const cera_llama*, cera_llama_config* out);
CERA_LLAMA_API uint64_t cera_llama_seq_len(const cera_llama*);
CERA_LLAMA_API uint64_t cera_llama_gpu_memory_bytes(const cera_llama*);
CERA_LLAMA_API int cera_llama_forward(cera_llama*, uint32_t token, uint64_t pos, float* logits);
CERA_LLAMA_API int cera_llama_forward_greedy(cera_llama*, uint32_t token, uint64_t pos, uint32_t* next);
CERA_LLAMA_API int cera_llama_forward_prefill(cera_llama*, const uint32_t* tokens, uint64_t n, uint64_t start_pos,
                                              float* last_logits);
/* Model::forward_prefill_logits_all: logits_all[n][vocab] */
CERA_LLAMA_API int cera_llama_forward_prefill_logits_all(cera_llama*, const uint32_t* tokens, uint64_t n,
                                                         uint64_t start_pos, float* logits_all);
/* Model::forward_prefill_chunked: *consumed tokens went into the KV cache; last_logits is
 * written when at least one chunk ran.  The cancel flag is the one set by cera_llama_set_cancel. */
CERA_LLAMA_API int cera_llama_forward_prefill_chunked(cera_llama*, const uint32_t* tokens, uint64_t n,
                                                      uint64_t start_pos, uint64_t ubatch, uint64_t* consumed,
                                                      float* last_logits);
CERA_LLAMA_API void cera_llama_set_cancel(cera_llama*, int cancel);
CERA_LLAMA_API int cera_llama_truncate_kv(cera_llama*, uint64_t len);
/* Model::f16_kv_supported / configure_kv_compression: kind 0 = KvCompression::None (f32 cache),
 * 1 = KvCompression::F16.  Before the first forward pass; the first call wins. */
CERA_LLAMA_API int cera_llama_f16_kv_supported(const cera_llama*);
CERA_LLAMA_API int cera_llama_configure_kv_compression(cera_llama*, int kind);
/* Model::supports_kv_shift / shift_kv */
CERA_LLAMA_API int cera_llama_supports_kv_shift(const cera_llama*);
CERA_LLAMA_API int cera_llama_shift_kv(cera_llama*, uint64_t n_keep, uint64_t shift);
/* Model::snapshot_state / restore_state.  A snapshot is an opaque handle owned by the caller
 * (free it with cera_llama_snapshot_free); it can be restored into any model of the same shape.
 * restore also sets the session's seq_len, as the trait method sets the model's. */
typedef struct cera_llama_snapshot cera_llama_snapshot;
CERA_LLAMA_API cera_llama_snapshot* cera_llama_snapshot_state(cera_llama*);
CERA_LLAMA_API uint64_t cera_llama_snapshot_seq_len(const cera_llama_snapshot*);
CERA_LLAMA_API uint64_t cera_llama_snapshot_bytes(const cera_llama_snapshot*);
CERA_LLAMA_API int cera_llama_restore_state(cera_llama*, const cera_llama_snapshot*);
CERA_LLAMA_API void cera_llama_snapshot_free(cera_llama_snapshot*);
/* Greedy generation as Session drives it for temperature 0: prefill the prompt in `ubatch`
 * chunks, take argmax of its last logits as the first new token, then n_new-1
 * forward_greedy steps.  out_tokens[n_new]; timings in seconds (nullable). */
CERA_LLAMA_API int cera_llama_generate_greedy(cera_llama*, const uint32_t* prompt, uint64_t n_prompt, uint64_t n_new,
                                              uint64_t ubatch, uint32_t* out_tokens, double* prefill_s,
                                              double* decode_s);

/* Verification hook (no counterpart in the trait): switches the model to the reference-order
 * route of cera_hip_set_reference_order (logits bit-identical to the CPU AVX2 path, many times
 * slower); the session must be empty. */
CERA_LLAMA_API int cera_llama_set_reference_order(cera_llama*, int on);

#ifdef __cplusplus
}
#endif
