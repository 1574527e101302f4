// Host-side (CPU) half of the `hip` backend, above the C-ABI of cera_hip.h:
// the pieces of cera's Rust host code that a HIP backend still needs on the
// CPU -- f16 conversion, the GGUF weight quantizers used to build models, a
// GGUF v3 reader/writer, and HipLlamaModel (the `Model`-trait twin).
//
// cera is Rust and no Rust toolchain is available to this build, so this
// layer is C++17 with a C-ABI face for ctypes-based tests.
#pragma once
#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#if defined(__GNUC__)
#define CERA_HOST_API __attribute__((visibility("default")))
#else
#define CERA_HOST_API
#endif

/* GGML tensor type ids, cera/src/gguf.rs:259-278 */
enum {
    CERA_TYPE_F32 = 0, CERA_TYPE_F16 = 1, CERA_TYPE_Q4_0 = 2, CERA_TYPE_Q4_1 = 3,
    CERA_TYPE_Q8_0 = 8, CERA_TYPE_Q4_K = 12, CERA_TYPE_Q5_K = 13, CERA_TYPE_Q6_K = 14,
    CERA_TYPE_BF16 = 30
};

/* cera/src/quant.rs:48-164 */
CERA_HOST_API float    cera_f16_to_f32(uint16_t bits);
CERA_HOST_API uint16_t cera_f32_to_f16(float v);

/* Bytes of n elements stored as `ggml_type` (0 if n is not a whole number of
 * blocks or the type is unknown).  cera/src/convert/quantize.rs:118-140. */
CERA_HOST_API uint64_t cera_tensor_bytes(uint32_t ggml_type, uint64_t n_elements);

/* f32 -> GGUF blocks, cera/src/convert/quantize.rs: quantize_q8_0 (:344),
 * quantize_q4_0 (:523), quantize_q4_k (:719), quantize_q5_k (:851),
 * quantize_q6_k (:993).  Returns 0, or -1 on a bad length / type / buffer. */
CERA_HOST_API int cera_quantize(uint32_t ggml_type, const float* input, uint64_t n,
                                void* output, uint64_t output_bytes);
/* Same, split over `n_threads` workers by whole blocks (n_threads <= 0: 1). */
CERA_HOST_API int cera_quantize_mt(uint32_t ggml_type, const float* input, uint64_t n,
                                   void* output, uint64_t output_bytes, int n_threads);

/* ---- GGUF v3 container (C face of gguf.h; cera/src/gguf.rs, convert/writer.rs) ---- */
typedef struct cera_gguf cera_gguf;
/* NULL on failure with the reason in err (NUL-terminated, truncated to err_len). */
CERA_HOST_API cera_gguf* cera_gguf_open(const char* path, char* err, uint64_t err_len);
CERA_HOST_API cera_gguf* cera_gguf_from_bytes(const void* bytes, uint64_t n, char* err, uint64_t err_len);
CERA_HOST_API void cera_gguf_close(cera_gguf*);
/* typed getters: 1 if the key holds exactly that value type, else 0 (gguf.rs:578-600) */
CERA_HOST_API int cera_gguf_get_u32(const cera_gguf*, const char* key, uint32_t* out);
CERA_HOST_API int cera_gguf_get_f32(const cera_gguf*, const char* key, float* out);
/* copies at most out_len-1 bytes; returns the full length, or -1 if absent / not a string */
CERA_HOST_API int64_t cera_gguf_get_str(const cera_gguf*, const char* key, char* out, uint64_t out_len);
CERA_HOST_API uint64_t cera_gguf_data_offset(const cera_gguf*);
CERA_HOST_API uint64_t cera_gguf_n_tensors(const cera_gguf*);
/* i-th tensor name in sorted order (NULL past the end); valid while the file is open */
CERA_HOST_API const char* cera_gguf_tensor_name(const cera_gguf*, uint64_t i);
typedef struct {
    uint32_t ggml_type, n_dims;
    uint64_t dims[8];      /* GGUF order: dims[0] is the row length */
    uint64_t offset;       /* absolute file offset */
    uint64_t size_bytes;   /* 0: unsupported type */
    const void* data;      /* into the mapping; NULL when size_bytes == 0 */
} cera_gguf_tensor_info;
CERA_HOST_API int cera_gguf_tensor(const cera_gguf*, const char* name, cera_gguf_tensor_info* out);

typedef struct cera_gguf_writer cera_gguf_writer;
CERA_HOST_API cera_gguf_writer* cera_gguf_writer_new(uint32_t alignment);
CERA_HOST_API void cera_gguf_writer_free(cera_gguf_writer*);
CERA_HOST_API void cera_gguf_writer_add_u32(cera_gguf_writer*, const char* key, uint32_t v);
CERA_HOST_API void cera_gguf_writer_add_f32(cera_gguf_writer*, const char* key, float v);
CERA_HOST_API void cera_gguf_writer_add_str(cera_gguf_writer*, const char* key, const char* v);
/* data is borrowed until cera_gguf_writer_write returns */
CERA_HOST_API void cera_gguf_writer_add_tensor(cera_gguf_writer*, const char* name, const uint64_t* dims, uint32_t n_dims,
                                               uint32_t ggml_type, const void* data, uint64_t size_bytes);
CERA_HOST_API int cera_gguf_writer_write(cera_gguf_writer*, const char* path, char* err, uint64_t err_len);

/* ---- seeded random-init llama-architecture GGUF (synth.cpp) ---- */
typedef struct {
    const char* architecture;      /* NULL => "llama" */
    uint32_t n_layers, hidden, ffn, n_heads, n_kv_heads;
    uint32_t head_dim;             /* 0 => hidden / n_heads and no key_length key */
    uint32_t vocab, context_length;
    float rope_theta, rms_eps;
    float weight_sigma;            /* matrices ~ N(0, sigma) before quantization */
    float norm_jitter;             /* norm vectors 1 + jitter * N(0,1); 0 => exactly 1 */
    uint32_t type_token_embd, type_output, type_attn_q, type_attn_k, type_attn_v, type_attn_output,
             type_ffn_gate, type_ffn_up, type_ffn_down;   /* CERA_TYPE_* of the five quantizable types */
    uint32_t tied_output;          /* 1: no output.weight (head = token_embd) */
    uint32_t qkv_bias, qk_norm;    /* 1: emit Qwen2-style biases / Qwen3-style per-head norms */
} cera_synth_config;
CERA_HOST_API int cera_synth_llama_gguf(const char* path, const cera_synth_config* cfg, uint64_t seed, int n_threads,
                                        char* err, uint64_t err_len);

#ifdef __cplusplus
}
#endif
