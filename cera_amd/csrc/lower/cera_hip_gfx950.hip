// The standalone gfx950 code object: the decode GEMV layer's kernels under fixed extern "C" names,
// for hosts that load it with hipModuleLoad and launch with hipModuleLaunchKernel
// (include/cera_hip_kernels.h documents names, argument structs and launch geometry).  Compiled
// with `hipcc --genco`; the bodies are the ones libcera_hip.so instantiates.
#include <cstddef>

#include "cera_hip_kernels.h"
#include "gemv.hip.h"
#include "gemv_rows.hip.h"
#include "glue.hip.h"
#include "quantize.hip.h"

// the header's structs are the kernels' argument layouts
static_assert(sizeof(cera_k_gemv_args) == sizeof(GemvArgs), "gemv args");
static_assert(offsetof(cera_k_gemv_args, resid) == offsetof(GemvArgs, resid) && offsetof(cera_k_gemv_args, m) == offsetof(GemvArgs, m) &&
                  offsetof(cera_k_gemv_args, rows_per_group) == offsetof(GemvArgs, rows_per_wave) &&
                  offsetof(cera_k_gemv_args, dbg_dots) == offsetof(GemvArgs, dbg_dots) &&
                  offsetof(cera_k_gemv_args, dbg_asums) == offsetof(GemvArgs, dbg_asums),
              "gemv args");

extern "C" __global__ __launch_bounds__(256) void cera_k_quantize_q8_0(cera_k_quantize_q8_0_args a) {
    quantize_q8_0_body(a.x, a.k, a.scales, a.quants, a.bsum);
}

extern "C" __global__ __launch_bounds__(1024) void cera_k_rmsnorm_q8_0(cera_k_rmsnorm_q8_0_args a) {
    __shared__ double part[16];
    rmsnorm_row_body<true>(a.x, a.w, a.n, a.eps, a.y, a.scales, a.quants, part);
}

#define CERA_K_GEMV(NAME, T, KS, EPI)                                                                    \
    extern "C" __global__ __launch_bounds__(64 * KS) void NAME(GemvArgs p) {                             \
        __shared__ float part[2][1][2][KS * 4];                                                          \
        gemv_body<T, 1, KS, 2, EPI, false>(p, blockIdx.x, threadIdx.x & 63, threadIdx.x >> 6, part);     \
    }
#define CERA_K_GEMV_TYPE(TN, T)                       \
    CERA_K_GEMV(cera_k_gemv_##TN##_ks1_store, T, 1, EPI_STORE) \
    CERA_K_GEMV(cera_k_gemv_##TN##_ks2_store, T, 2, EPI_STORE) \
    CERA_K_GEMV(cera_k_gemv_##TN##_ks4_store, T, 4, EPI_STORE) \
    CERA_K_GEMV(cera_k_gemv_##TN##_ks8_store, T, 8, EPI_STORE) \
    CERA_K_GEMV(cera_k_gemv_##TN##_ks1_add, T, 1, EPI_ADD)     \
    CERA_K_GEMV(cera_k_gemv_##TN##_ks2_add, T, 2, EPI_ADD)     \
    CERA_K_GEMV(cera_k_gemv_##TN##_ks4_add, T, 4, EPI_ADD)     \
    CERA_K_GEMV(cera_k_gemv_##TN##_ks8_add, T, 8, EPI_ADD)
CERA_K_GEMV_TYPE(q4_0, Q4_0)
CERA_K_GEMV_TYPE(q4_1, Q4_1)
CERA_K_GEMV_TYPE(q8_0, Q8_0)
CERA_K_GEMV_TYPE(q4_k, Q4K)
CERA_K_GEMV_TYPE(q6_k, Q6K)

// ---- the one-wavefront-per-row decode kernels and the decode copies ----------------------------
static_assert(sizeof(cera_k_row_gemv_args) == sizeof(RowGemvArgs) && offsetof(cera_k_row_gemv_args, row_bytes) == offsetof(RowGemvArgs, row_bytes) &&
                  offsetof(cera_k_row_gemv_args, xq) == offsetof(RowGemvArgs, xq) && offsetof(cera_k_row_gemv_args, x) == offsetof(RowGemvArgs, x) &&
                  offsetof(cera_k_row_gemv_args, eps) == offsetof(RowGemvArgs, eps) && offsetof(cera_k_row_gemv_args, y) == offsetof(RowGemvArgs, y) &&
                  offsetof(cera_k_row_gemv_args, resid) == offsetof(RowGemvArgs, resid) &&
                  offsetof(cera_k_row_gemv_args, out_q) == offsetof(RowGemvArgs, out_q) &&
                  offsetof(cera_k_row_gemv_args, out_s) == offsetof(RowGemvArgs, out_s),
              "row gemv args");
static_assert(sizeof(cera_k_row_gemv_pair_args) == sizeof(RowGemvPairArgs) &&
                  offsetof(cera_k_row_gemv_pair_args, b) == offsetof(RowGemvPairArgs, b) &&
                  offsetof(cera_k_row_gemv_pair_args, n_blocks_a) == offsetof(RowGemvPairArgs, n_blocks_a),
              "row gemv pair args");
#define CERA_K_COPY_BYTES_OK(GT, T, K) (CERA_K_DECODE_COPY_ROW_BYTES(GT, K) == T::stream_row_bytes(K))
static_assert(CERA_K_COPY_BYTES_OK(12, Q4K, 256) && CERA_K_COPY_BYTES_OK(12, Q4K, 4096) && CERA_K_COPY_BYTES_OK(12, Q4K, 14336), "Q4_K copy row bytes");
static_assert(CERA_K_COPY_BYTES_OK(14, Q6K, 256) && CERA_K_COPY_BYTES_OK(14, Q6K, 4096) && CERA_K_COPY_BYTES_OK(14, Q6K, 14336), "Q6_K copy row bytes");
static_assert(CERA_K_COPY_BYTES_OK(2, Q4_0, 32) && CERA_K_COPY_BYTES_OK(2, Q4_0, 4096) && CERA_K_COPY_BYTES_OK(2, Q4_0, 11008), "Q4_0 copy row bytes");
static_assert(CERA_K_COPY_BYTES_OK(3, Q4_1, 32) && CERA_K_COPY_BYTES_OK(3, Q4_1, 4096) && CERA_K_COPY_BYTES_OK(3, Q4_1, 11008), "Q4_1 copy row bytes");
static_assert(CERA_K_COPY_BYTES_OK(8, Q8_0, 32) && CERA_K_COPY_BYTES_OK(8, Q8_0, 4096) && CERA_K_COPY_BYTES_OK(8, Q8_0, 11008), "Q8_0 copy row bytes");

#define CERA_K_DECODE_COPY(TN, T)                                                                        \
    extern "C" __global__ __launch_bounds__(256) void cera_k_decode_copy_##TN(cera_k_decode_copy_args a) { \
        stream_rows_body<T>(a.src, a.dst, a.n_units, a.row_bytes, a.copy_row_bytes);                     \
    }
CERA_K_DECODE_COPY(q4_0, Q4_0)
CERA_K_DECODE_COPY(q4_1, Q4_1)
CERA_K_DECODE_COPY(q8_0, Q8_0)
CERA_K_DECODE_COPY(q4_k, Q4K)
CERA_K_DECODE_COPY(q6_k, Q6K)

// the launch bounds are those of the library's instances (gemv_rows.hip.h)
#define CERA_K_ROW(NAME, T, P, EPI)                                                              \
    extern "C" __global__ __launch_bounds__(256, 2) void NAME(RowGemvArgs p) {                   \
        __shared__ uint32_t s_xq[1];                                                             \
        __shared__ float s_xs[1];                                                                \
        __shared__ double s_part[4];                                                             \
        __shared__ __attribute__((aligned(16))) float s_out[4];                                  \
        row_gemv_body<T, 4, 2, false, EPI, true, P>(p, blockIdx.x, s_xq, s_xs, s_part, s_out);   \
    }
#define CERA_K_ROW_BOTH(TN, T, P)                                \
    CERA_K_ROW(cera_k_row_gemv_##TN##_p##P##_store, T, P, FEPI_STORE) \
    CERA_K_ROW(cera_k_row_gemv_##TN##_p##P##_add, T, P, FEPI_ADD)
CERA_K_ROW_BOTH(q4_k, Q4K, 1)
CERA_K_ROW_BOTH(q6_k, Q6K, 1)
CERA_K_ROW_BOTH(q4_0, Q4_0, 1)
CERA_K_ROW_BOTH(q4_0, Q4_0, 2)
CERA_K_ROW_BOTH(q4_1, Q4_1, 1)
CERA_K_ROW_BOTH(q4_1, Q4_1, 2)
CERA_K_ROW_BOTH(q8_0, Q8_0, 1)
CERA_K_ROW_BOTH(q8_0, Q8_0, 2)

#define CERA_K_ROW_LONG(TN, T, P)                                                                        \
    extern "C" __global__ __launch_bounds__(256) void cera_k_row_gemv_long_##TN##_p##P##_add(RowGemvArgs p) { \
        __shared__ __attribute__((aligned(16))) int8_t s_xq[P * 64 * T::ELEMS_PER_UNIT];                 \
        __shared__ __attribute__((aligned(16))) float s_xs[P * 64 * T::ELEMS_PER_UNIT / 32];             \
        row_gemv_long_body<T, 4, P, FEPI_ADD, true>(p, s_xq, s_xs);                                      \
    }
CERA_K_ROW_LONG(q4_k, Q4K, 2)
CERA_K_ROW_LONG(q4_k, Q4K, 3)
CERA_K_ROW_LONG(q4_k, Q4K, 4)
CERA_K_ROW_LONG(q6_k, Q6K, 2)
CERA_K_ROW_LONG(q6_k, Q6K, 3)
CERA_K_ROW_LONG(q6_k, Q6K, 4)
CERA_K_ROW_LONG(q4_0, Q4_0, 4)
CERA_K_ROW_LONG(q4_0, Q4_0, 8)
CERA_K_ROW_LONG(q4_1, Q4_1, 4)
CERA_K_ROW_LONG(q4_1, Q4_1, 8)
CERA_K_ROW_LONG(q8_0, Q8_0, 4)
CERA_K_ROW_LONG(q8_0, Q8_0, 8)

#define CERA_K_GATE_UP(TN, T, P)                                                                         \
    extern "C" __global__ __launch_bounds__(1024, 1) void cera_k_norm_gate_up_##TN##_p##P(RowGemvArgs p) { \
        __shared__ uint32_t s_xq[1024];                                                                  \
        __shared__ float s_xs[128];                                                                      \
        __shared__ double s_part[16];                                                                    \
        __shared__ __attribute__((aligned(16))) float s_out[64];                                         \
        row_gemv_body<T, 16, 4, true, FEPI_SILU_Q8, true, P>(p, blockIdx.x, s_xq, s_xs, s_part, s_out);  \
    }
CERA_K_GATE_UP(q4_k, Q4K, 1)
CERA_K_GATE_UP(q4_0, Q4_0, 1)
CERA_K_GATE_UP(q4_0, Q4_0, 2)
CERA_K_GATE_UP(q4_1, Q4_1, 1)
CERA_K_GATE_UP(q4_1, Q4_1, 2)
CERA_K_GATE_UP(q8_0, Q8_0, 1)
CERA_K_GATE_UP(q8_0, Q8_0, 2)

#define CERA_K_QKV(TNA, TNB, TA, TB, P, R)                                                                                  \
    extern "C" __global__ __launch_bounds__(512, 2) void cera_k_norm_qkv_##TNA##_##TNB##_p##P##_r##R(RowGemvPairArgs p) {     \
        __shared__ uint32_t s_xq[1024];                                                                                     \
        __shared__ float s_xs[128];                                                                                         \
        __shared__ double s_part[8];                                                                                        \
        if (blockIdx.x < p.n_blocks_a) row_gemv_body<TA, 8, R, true, FEPI_STORE, true, P>(p.a, blockIdx.x, s_xq, s_xs, s_part, nullptr); \
        else row_gemv_body<TB, 8, R, true, FEPI_STORE, true, P>(p.b, blockIdx.x - p.n_blocks_a, s_xq, s_xs, s_part, nullptr); \
    }
#define CERA_K_QKV_R(TNA, TNB, TA, TB, P) CERA_K_QKV(TNA, TNB, TA, TB, P, 1) CERA_K_QKV(TNA, TNB, TA, TB, P, 2)
CERA_K_QKV_R(q4_k, q4_k, Q4K, Q4K, 1)
CERA_K_QKV_R(q4_k, q6_k, Q4K, Q6K, 1)
CERA_K_QKV_R(q6_k, q4_k, Q6K, Q4K, 1)
CERA_K_QKV_R(q6_k, q6_k, Q6K, Q6K, 1)
CERA_K_QKV_R(q4_0, q4_0, Q4_0, Q4_0, 1)
CERA_K_QKV_R(q4_0, q4_0, Q4_0, Q4_0, 2)
CERA_K_QKV_R(q4_1, q4_1, Q4_1, Q4_1, 1)
CERA_K_QKV_R(q4_1, q4_1, Q4_1, Q4_1, 2)
CERA_K_QKV_R(q8_0, q8_0, Q8_0, Q8_0, 1)
CERA_K_QKV_R(q8_0, q8_0, Q8_0, Q8_0, 2)

// ==== the rest of a forward pass: embedding, norms over rows, RoPE + cache append, attention,
// ==== SwiGLU, argmax, context shift, and the batched (prefill) GEMMs ============================
#include "attention.hip.h"
#include "gemm_fp8.hip.h"
#include "gemm_q6k_f16.hip.h"

static_assert(sizeof(cera_k_gemm_args) == sizeof(GemmArgs) && offsetof(cera_k_gemm_args, bh) == offsetof(GemmArgs, bh) &&
                  offsetof(cera_k_gemm_args, out) == offsetof(GemmArgs, out) && offsetof(cera_k_gemm_args, row_bytes) == offsetof(GemmArgs, row_bytes) &&
                  offsetof(cera_k_gemm_args, ld_n) == offsetof(GemmArgs, ld_n) && offsetof(cera_k_gemm_args, resid_scale) == offsetof(GemmArgs, resid_scale) &&
                  offsetof(cera_k_gemm_args, k_chunk) == offsetof(GemmArgs, k_chunk) && offsetof(cera_k_gemm_args, part_stride) == offsetof(GemmArgs, part_stride) &&
                  offsetof(cera_k_gemm_args, w2) == offsetof(GemmArgs, w2) && offsetof(cera_k_gemm_args, tiles1) == offsetof(GemmArgs, tiles1) &&
                  offsetof(cera_k_gemm_args, ld_n2) == offsetof(GemmArgs, ld_n2) && offsetof(cera_k_gemm_args, hq) == offsetof(GemmArgs, hq) &&
                  offsetof(cera_k_gemm_args, hbsum) == offsetof(GemmArgs, hbsum) && offsetof(cera_k_gemm_args, dbg_dots) == offsetof(GemmArgs, dbg_dots) &&
                  offsetof(cera_k_gemm_args, bf8) == offsetof(GemmArgs, bf8),
              "gemm args");
static_assert(CERA_K_GEMM_FP8_ACT_BYTES(64, 256) == G8_REC * 2 && CERA_K_GEMM_FP8_ACT_BYTES(65, 512) == G8_REC * 2 * 2 * 2 && G8_BN == 64 && G8_BM == 128,
              "fp8 activation record geometry");
static_assert(GEMM_BM == 128 && GEMM_BN == 64, "int8 / f16 GEMM tile");

extern "C" __global__ __launch_bounds__(256) void cera_k_embed_token(cera_k_embed_token_args a) {
    embed_token_body(a.ggml_type, a.w, a.row_bytes, a.token, a.pos, a.scalars, a.k, a.scale, a.out);
}
extern "C" __global__ __launch_bounds__(256) void cera_k_embed_rows(cera_k_embed_rows_args a) {
    embed_row_body(a.ggml_type, a.w, a.row_bytes, a.tokens, a.k, a.scale, a.out);
}
extern "C" __global__ __launch_bounds__(256) void cera_k_rmsnorm_rows(cera_k_rmsnorm_rows_args a) {
    rmsnorm_body<false>(a.x, a.w, a.n, a.eps, a.y, nullptr, nullptr, nullptr);
}
extern "C" __global__ __launch_bounds__(256) void cera_k_rmsnorm_rows_q8_0(cera_k_rmsnorm_rows_args a) {
    rmsnorm_body<true>(a.x, a.w, a.n, a.eps, a.y, a.scales, a.quants, a.bsum);
}
extern "C" __global__ void cera_k_rope_kv_f32(cera_k_rope_kv_args a) {
    rope_kv_body<float>(a.q, a.k, a.v, a.cs_table, a.pos, a.n_heads, a.n_kv_heads, a.head_dim, a.rope_type,
                        static_cast<float*>(a.k_cache), static_cast<float*>(a.v_cache), a.max_seq);
}
extern "C" __global__ void cera_k_rope_kv_f16(cera_k_rope_kv_args a) {
    rope_kv_body<kv_half>(a.q, a.k, a.v, a.cs_table, a.pos, a.n_heads, a.n_kv_heads, a.head_dim, a.rope_type,
                          static_cast<kv_half*>(a.k_cache), static_cast<kv_half*>(a.v_cache), a.max_seq);
}
extern "C" __global__ __launch_bounds__(256) void cera_k_silu_mul(cera_k_silu_mul_args a) {
    silu_mul_body<false>(a.gate, a.up, a.n, a.out, nullptr, nullptr, nullptr);
}
extern "C" __global__ __launch_bounds__(256) void cera_k_silu_mul_q8_0(cera_k_silu_mul_args a) {
    silu_mul_body<true>(a.gate, a.up, a.n, a.out, a.scales, a.quants, a.bsum);
}
extern "C" __global__ __launch_bounds__(256) void cera_k_add(cera_k_add_args a) { add_body(a.a, a.b, a.b_scale, a.n, a.out); }
extern "C" __global__ __launch_bounds__(256) void cera_k_bias(cera_k_bias_args a) { bias_body(a.x, a.b, a.n); }
extern "C" __global__ __launch_bounds__(256) void cera_k_scale(cera_k_scale_args a) { scale_body(a.x, a.s, a.n); }
extern "C" __global__ __launch_bounds__(256) void cera_k_argmax_partial(cera_k_argmax_partial_args a) {
    argmax_partial_body(a.x, a.n, a.pv, a.pi);
}
extern "C" __global__ __launch_bounds__(256) void cera_k_argmax_final(cera_k_argmax_final_args a) {
    argmax_final_body(a.pv, a.pi, a.np, a.out, a.out2);
}

#define CERA_K_KV_SHIFT(KN, KV, HD)                                                                            \
    extern "C" __global__ __launch_bounds__(256) void cera_k_kv_shift_##KN##_hd##HD(cera_k_kv_shift_args a) {    \
        kv_shift_body<KV, HD>(static_cast<const KV*>(a.src), static_cast<KV*>(a.dst), a.src_row, a.dst_row, a.n_rows, \
                              a.src_head_stride, a.dst_head_stride, a.delta_cs, a.rope_type);                   \
    }
CERA_K_KV_SHIFT(f32, float, 64)
CERA_K_KV_SHIFT(f32, float, 128)
CERA_K_KV_SHIFT(f16, kv_half, 64)
CERA_K_KV_SHIFT(f16, kv_half, 128)

// ---- attention ---------------------------------------------------------------------------------
#define CERA_K_ATTN_DEC(KN, KV, HD, G, S)                                                                              \
    extern "C" __global__ __launch_bounds__(256) void cera_k_attn_decode_partial_##KN##_hd##HD##_g##G##_s##S(cera_k_attn_decode_args a) { \
        attn_decode_partial_body<G, S, false, KV, HD, false>(a.q, static_cast<const KV*>(a.kc), static_cast<const KV*>(a.vc), a.seq_len, \
                                                             a.max_seq, a.scale, a.chunks_per_part, a.n_parts, a.q_stride, a.g_total,   \
                                                             a.n_kv, a.n_queries, a.part_acc, a.part_ml, AttnNewKV{});                 \
    }
#define CERA_K_ATTN_DEC_GS(KN, KV, HD) \
    CERA_K_ATTN_DEC(KN, KV, HD, 1, 1) CERA_K_ATTN_DEC(KN, KV, HD, 2, 1) CERA_K_ATTN_DEC(KN, KV, HD, 4, 1) \
    CERA_K_ATTN_DEC(KN, KV, HD, 1, 4) CERA_K_ATTN_DEC(KN, KV, HD, 2, 4) CERA_K_ATTN_DEC(KN, KV, HD, 4, 4)
CERA_K_ATTN_DEC_GS(f32, float, 64)
CERA_K_ATTN_DEC_GS(f32, float, 128)
CERA_K_ATTN_DEC_GS(f16, kv_half, 64)
CERA_K_ATTN_DEC_GS(f16, kv_half, 128)

#define CERA_K_ATTN_MERGE(HD)                                                                                      \
    extern "C" __global__ __launch_bounds__(256) void cera_k_attn_decode_merge_hd##HD(cera_k_attn_merge_args a) {   \
        attn_decode_merge_body<false, HD>(a.part_acc, a.part_ml, a.n_parts, a.g_total, a.n_heads, a.out, nullptr, nullptr, nullptr); \
    }                                                                                                              \
    extern "C" __global__ __launch_bounds__(256) void cera_k_attn_decode_merge_hd##HD##_q8_0(cera_k_attn_merge_args a) { \
        attn_decode_merge_body<true, HD>(a.part_acc, a.part_ml, a.n_parts, a.g_total, a.n_heads, a.out, a.scales, a.quants, a.bsum); \
    }                                                                                                              \
    extern "C" __global__ __launch_bounds__(256) void cera_k_attn_prefill_merge_hd##HD(cera_k_attn_merge_args a) {  \
        attn_prefill_merge_body<false, HD>(a.part_acc, a.part_ml, a.n_parts, a.g_total, a.n_heads, a.n_pairs, a.out, nullptr, nullptr, nullptr); \
    }                                                                                                              \
    extern "C" __global__ __launch_bounds__(256) void cera_k_attn_prefill_merge_hd##HD##_q8_0(cera_k_attn_merge_args a) { \
        attn_prefill_merge_body<true, HD>(a.part_acc, a.part_ml, a.n_parts, a.g_total, a.n_heads, a.n_pairs, a.out, a.scales, a.quants, a.bsum); \
    }
CERA_K_ATTN_MERGE(64)
CERA_K_ATTN_MERGE(128)

#define CERA_K_ATTN_PF(KN, KV, HD, G)                                                                                   \
    extern "C" __global__ __launch_bounds__(64 * G) void cera_k_attn_prefill_partial_##KN##_hd##HD##_g##G(cera_k_attn_prefill_args a) { \
        attn_prefill_partial_body<KV, HD, G>(a.q, static_cast<const KV*>(a.kc), static_cast<const KV*>(a.vc), a.first_len, a.n_queries, \
                                             a.max_seq, a.scale, a.part_keys, a.n_parts, a.q_stride, a.part_acc, a.part_ml);     \
    }
#define CERA_K_ATTN_PF_G(KN, KV, HD) CERA_K_ATTN_PF(KN, KV, HD, 1) CERA_K_ATTN_PF(KN, KV, HD, 2) CERA_K_ATTN_PF(KN, KV, HD, 4) CERA_K_ATTN_PF(KN, KV, HD, 8)
CERA_K_ATTN_PF_G(f32, float, 64)
CERA_K_ATTN_PF_G(f32, float, 128)
CERA_K_ATTN_PF_G(f16, kv_half, 64)
CERA_K_ATTN_PF_G(f16, kv_half, 128)

// ---- batched GEMMs -------------------------------------------------------------------------------
extern "C" __global__ __launch_bounds__(256) void cera_k_gemm_act_fp8(cera_k_gemm_act_fp8_args a) {
    gemm_act_fp8_body(a.quants, a.scales, a.bsum, a.out, a.n, a.k, static_cast<uint4*>(a.halves));
}
extern "C" __global__ __launch_bounds__(256) void cera_k_gemm_act_f16(cera_k_gemm_act_f16_args a) {
    gemm_act_f16_body(reinterpret_cast<const uint4*>(a.quants), reinterpret_cast<uint4*>(a.out), a.n_words);
}
extern "C" __global__ __launch_bounds__(64 * G8_NW, 8 / G8_NW) void cera_k_gemm_q4_k(GemmArgs p) { gemm_q4k_fp8_body<false, false, G8_NW>(p); }
extern "C" __global__ __launch_bounds__(64 * G8_NW, 8 / G8_NW) void cera_k_gemm_q4_k_swiglu(GemmArgs p) { gemm_q4k_fp8_body<true, false, G8_NW>(p); }
extern "C" __global__ __launch_bounds__(256, 2) void cera_k_gemm_q6_k(GemmArgs p) { gemm_q6k_f16_body<false>(p); }
extern "C" __global__ __launch_bounds__(256, GemmQ4_0::WAVES_PER_SIMD) void cera_k_gemm_q4_0(GemmArgs p) { gemm_body<GemmQ4_0, false, false>(p); }
extern "C" __global__ __launch_bounds__(256, GemmQ4_1::WAVES_PER_SIMD) void cera_k_gemm_q4_1(GemmArgs p) { gemm_body<GemmQ4_1, false, false>(p); }
extern "C" __global__ __launch_bounds__(256, GemmQ8_0::WAVES_PER_SIMD) void cera_k_gemm_q8_0(GemmArgs p) { gemm_body<GemmQ8_0, false, false>(p); }
extern "C" __global__ __launch_bounds__(256) void cera_k_gemm_reduce(cera_k_gemm_reduce_args a) {
    gemm_reduce_body(a.part, a.n_split, a.part_stride, a.n4, a.out, a.resid, a.resid_scale, a.n4_first, a.out2);
}
