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

#ifdef __cplusplus
}
#endif
