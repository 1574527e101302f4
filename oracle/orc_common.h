// CPU oracle for the cera `hip` hot path -- TEST INFRASTRUCTURE ONLY.
//
// This directory is a CPU restatement of the arithmetic of hyeons-lab/cera's
// x86 AVX2-tier int8 decode/prefill path.  It exists to check the HIP kernels
// and to be timed as the "restated cera AVX2 path" CPU baseline.  Nothing in
// the shipped library links, loads or calls it.
//
// Every function cites the reference file:line (relative to the cera tree)
// whose arithmetic it restates.  Float code is compiled with
// -ffp-contract=off because Rust never contracts a*b+c into an FMA; FMAs
// appear only where the reference spells `_mm256_fmadd_ps` (here: fmaf).
#pragma once
#include <cstddef>
#include <cstdint>

#if defined(__GNUC__)
#define ORC_API extern "C" __attribute__((visibility("default")))
#else
#define ORC_API extern "C"
#endif

// GGML type ids as cera maps them (cera/src/gguf.rs:259-278).
enum OrcDType : uint32_t {
    ORC_F32 = 0,
    ORC_F16 = 1,
    ORC_Q4_0 = 2,
    ORC_Q4_1 = 3,
    ORC_Q8_0 = 8,
    ORC_Q4_K = 12,
    ORC_Q5_K = 13,
    ORC_Q6_K = 14,
    ORC_BF16 = 30,
};

// Block layouts, cera/src/quant.rs:173-293 (repr(C, packed), little endian).
#pragma pack(push, 1)
struct OrcBlockQ4_0 { uint16_t d; uint8_t qs[16]; };
struct OrcBlockQ4_1 { uint16_t d; uint16_t m; uint8_t qs[16]; };
struct OrcBlockQ8_0 { uint16_t d; int8_t qs[32]; };
struct OrcBlockQ4K  { uint16_t d; uint16_t dmin; uint8_t scales[12]; uint8_t qs[128]; };
struct OrcBlockQ5K  { uint16_t d; uint16_t dmin; uint8_t scales[12]; uint8_t qh[32]; uint8_t qs[128]; };
struct OrcBlockQ6K  { uint8_t ql[128]; uint8_t qh[64]; int8_t scales[16]; uint16_t d; };
#pragma pack(pop)
static_assert(sizeof(OrcBlockQ4_0) == 18, "Q4_0");
static_assert(sizeof(OrcBlockQ4_1) == 20, "Q4_1");
static_assert(sizeof(OrcBlockQ8_0) == 34, "Q8_0");
static_assert(sizeof(OrcBlockQ4K) == 144, "Q4_K");
static_assert(sizeof(OrcBlockQ5K) == 176, "Q5_K");
static_assert(sizeof(OrcBlockQ6K) == 210, "Q6_K");

// elements per block / bytes per block for a dtype; 0 when unknown.
ORC_API uint32_t orc_block_elems(uint32_t dtype);
ORC_API uint32_t orc_block_bytes(uint32_t dtype);
ORC_API uint64_t orc_row_bytes(uint32_t dtype, uint64_t k);

// ---- quant.rs -------------------------------------------------------------
ORC_API float    orc_f16_to_f32(uint16_t bits);
ORC_API uint16_t orc_f32_to_f16(float v);
ORC_API float    orc_bf16_to_f32(uint16_t bits);
ORC_API void     orc_decode_q4km_scales(const uint8_t* scales12, uint8_t* sc8, uint8_t* mn8);
ORC_API int      orc_dequantize_row(uint32_t dtype, const void* src, uint64_t k, float* dst);
// f32 activations x quantized row (quant.rs vec_dot_*_f32*): one row, k elements.
ORC_API float    orc_vec_dot_row_f32(uint32_t dtype, const void* row, const float* x, uint64_t k);

// ---- Q8_0 activation quantizer (cpu.rs:942-958) ---------------------------
ORC_API void orc_quantize_q8_0(const float* x, uint64_t k, float* scales, int8_t* quants);

// ---- integer specification of the int8 kernels ----------------------------
// dots: Q4_0 [m][k/32] sum (q-8)*a ; Q8_0 [m][k/32] sum w*a ; Q4_1/Q4_K [m][k/32]
// sum q*a (q in 0..15) ; Q6_K [m][k/16] sum q*a (q in 0..63).
// asums: Q4_1/Q4_K [k/32] sum a ; Q6_K [k/16] sum a ; unused otherwise.
ORC_API int orc_block_dots(uint32_t dtype, const void* w, uint64_t m, uint64_t k,
                           const int8_t* xq, int32_t* dots, int32_t* asums);

// ---- int8 GEMV / GEMM, AVX2-tier float order (simd.rs:4543-6249 @ 6359) ---
// variant 0: scalar 8-lane emulation; variant 1: AVX2 intrinsics twin.
// out is [m][n] row-major (out[i*n + j]); b_scales [n][k/32], b_quants [n][k].
ORC_API int orc_gemm_preq(uint32_t dtype, const void* w, const float* b_scales,
                          const int8_t* b_quants, float* out, uint64_t m, uint64_t n,
                          uint64_t k, int variant);
// The x86 prefill route for repacked weights (orc_repack.cpp): repack_q4_0_8x8 / repack_q4_k_8x8
// (cpu.rs:1145-1196, 1282-1358), gemm_q4_0_8x8_q8_0 / gemm_q4_k_8x8_q8_0 (simd.rs:5215-5518), and
// transformer::gemm_preq's choice between them and the standard layout (transformer.rs:758-775).
ORC_API int orc_repack_q4_0_8x8(const uint8_t* src, uint64_t m, uint64_t k, uint8_t* packed, float* scales);
ORC_API int orc_repack_q4_k_8x8(const uint8_t* src, uint64_t m, uint64_t k, uint8_t* packed, float* dsc, float* dmn);
ORC_API int orc_gemm_q4_0_8x8_q8_0(const uint8_t* packed, const float* scales, const float* b_scales, const int8_t* b_quants,
                                   float* out, uint64_t m, uint64_t n, uint64_t k);
ORC_API int orc_gemm_q4_k_8x8_q8_0(const uint8_t* packed, const float* dsc, const float* dmn, const float* b_scales,
                                   const int8_t* b_quants, float* out, uint64_t m, uint64_t n, uint64_t k);
ORC_API int orc_gemm_preq_x86(uint32_t dtype, const void* w, const float* b_scales, const int8_t* b_quants, float* out,
                              uint64_t m, uint64_t n, uint64_t k, int variant);
// cpu::gemv_dispatch (cpu.rs:2360): quantizes x to Q8_0 then runs the int8
// kernel; Q5_K/F32/F16/BF16 take the scalar f32 route on unquantized x.
ORC_API int orc_gemv(uint32_t dtype, const void* w, const float* x, float* y, uint64_t m,
                     uint64_t k, int variant);
// f64 reference: sum_b xs*(...) with exact integer block dots (for tolerance pins).
ORC_API int orc_gemv_f64ref(uint32_t dtype, const void* w, const float* x, double* y,
                            uint64_t m, uint64_t k);
ORC_API int orc_have_avx2(void);

// ---- threaded baseline ----------------------------------------------------
ORC_API void* orc_pool_create(int n_threads);
ORC_API void  orc_pool_destroy(void* pool);
ORC_API int   orc_pool_threads(void* pool);
// fn(tid, n_threads, arg) on every worker of the pool (tid 0 = the caller); returns when all are done
ORC_API void  orc_pool_run(void* pool, void (*fn)(int, int, void*), void* arg);
// Row-parallel gemv on the pool (AVX2 variant when available): the timed
// "restated cera AVX2 path" baseline.  Quantizes x on the calling thread first.
ORC_API int orc_gemv_mt(void* pool, uint32_t dtype, const void* w, const float* x, float* y,
                        uint64_t m, uint64_t k);

// ---- glue ops (cpu.rs) ----------------------------------------------------
ORC_API void  orc_rmsnorm(float* x, const float* weight, uint64_t n, float eps);
ORC_API float orc_expf(float x);
ORC_API void  orc_silu_mul(float* gate, const float* up, uint64_t n);
ORC_API void  orc_softmax(float* x, uint64_t n);
ORC_API void  orc_add(float* a, const float* b, uint64_t n);
ORC_API void  orc_rope_norm(float* q, float* k, uint64_t pos, uint32_t n_heads,
                            uint32_t n_kv_heads, uint32_t head_dim, float freq_base,
                            const float* freq_factors);
ORC_API void  orc_rope_neox(float* q, float* k, uint64_t pos, uint32_t n_heads,
                            uint32_t n_kv_heads, uint32_t head_dim, float freq_base);
ORC_API void  orc_rope_delta_head(float* head, int32_t delta_pos, uint32_t head_dim, float freq_base,
                                  uint32_t rope_type /*0 neox, 1 norm*/, const float* freq_factors);
ORC_API uint32_t orc_argmax(const float* logits, uint64_t n);

// ---- attention ------------------------------------------------------------
// K/V caches are time-major [pos][kv_dim] (kv_cache.rs:201-212).
ORC_API void orc_attn_scores(const float* q_head, const float* k_cache, float* scores,
                             uint64_t kv_dim, uint64_t kv_h_offset, uint32_t head_dim,
                             float scale, uint64_t seq_len, int variant);
ORC_API void orc_attn_values(const float* scores, const float* v_cache, float* out,
                             uint64_t kv_dim, uint64_t kv_h_offset, uint32_t head_dim,
                             uint64_t seq_len, int variant);
ORC_API void orc_decode_attention(const float* q, const float* k_cache, const float* v_cache,
                                  uint32_t n_heads, uint32_t n_kv_heads, uint32_t head_dim,
                                  float scale, uint64_t seq_len, float* out, int variant);

// One head of flash_attention_gqa_cpu (scalar route): q, out are [n_queries][head_dim].
ORC_API void orc_flash_attention_head(const float* q, const float* k_cache, const float* v_cache, float* out,
                                      uint64_t n_queries, uint64_t kv_dim, uint64_t kv_h_offset,
                                      uint32_t head_dim, float scale, uint64_t start_pos);
// The same head through the kernel an AVX2 host takes (flash_attention_gqa_avx2, cpu.rs:4261-4412):
// variant 1 the intrinsics, 2 their lane algebra in plain C, 0 the scalar route above.
ORC_API void orc_flash_attention_head_v(const float* q, const float* k_cache, const float* v_cache, float* out,
                                        uint64_t n_queries, uint64_t kv_dim, uint64_t kv_h_offset,
                                        uint32_t head_dim, float scale, uint64_t start_pos, int variant);
