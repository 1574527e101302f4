/* cera_hip_kernels.h -- the LOWER ABI of the `hip` backend: the kernels inside the standalone gfx950
 * code object `cera_hip_gfx950.hsaco` (built next to libcera_hip.so), for a host that wants to
 * drive the GPU itself with nothing but hipMalloc / hipMemcpyAsync / hipModuleLoad /
 * hipModuleLaunchKernel -- e.g. a pure-Rust `hip-sys` host inside cera -- instead of linking
 * libcera_hip.so (include/cera_hip.h, the primary boundary).
 *
 * Every kernel takes ONE argument: a struct of this header passed by value, i.e. the kernarg
 * segment is exactly the struct's bytes in natural C layout (`#[repr(C)]` in Rust).  Launch with
 *   void* params[] = { &args };  hipModuleLaunchKernel(f, gx, 1, 1, bx, 1, 1, 0, stream, params, NULL);
 * All pointers are device pointers.  The arithmetic is that of the same-named operations of
 * cera_hip.h: these are the very kernels libcera_hip.so launches (cera_hip_ctx_create with an
 * `hsaco_path` makes the library itself launch them from the code object).
 *
 * Weight matrices are rows of native GGML blocks, byte for byte as in a GGUF file
 * (cera/src/quant.rs:37-78), row r at w + r * row_bytes.
 */
#ifndef CERA_HIP_KERNELS_H
#define CERA_HIP_KERNELS_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define CERA_HIP_HSACO_NAME "cera_hip_gfx950.hsaco"

/* ---- cera_k_quantize_q8_0 --------------------------------------------------------------------
 * quantize_f32_to_q8_0 (cera/src/backend/cpu.rs:942-958): quants[k] int8, scales[k/32] f32 (each
 * an exact f16 value).  k % 32 == 0.  bsum nullable: per-block scale * sum(quants).
 * grid = ceil(k / 4 / 256) workgroups of 256 threads. */
typedef struct {
    const float* x;
    uint64_t k;
    float* scales;
    int8_t* quants;
    float* bsum;
} cera_k_quantize_q8_0_args;

/* ---- cera_k_rmsnorm_q8_0 ---------------------------------------------------------------------
 * cpu::rmsnorm (cera/src/backend/cpu.rs:2479-2496) of one row followed by its Q8_0 quantization:
 * y[n] f32, scales[n/32], quants[n].  n % 32 == 0, n <= 16384.  grid = 1 workgroup of 1024 threads. */
typedef struct {
    const float* x;
    const float* w;
    uint32_t n;
    float eps;
    float* y;
    float* scales;
    int8_t* quants;
} cera_k_rmsnorm_q8_0_args;

/* ---- cera_k_gemv_<type>_ks<KS>_<store|add> ---------------------------------------------------
 * The batch-1 int8 GEMV of transformer::gemv_preq (cera/src/model/transformer.rs:455-533) on
 * already-quantized activations: y[m] = W . (xs, xq)  (`add`: y = resid + W . x).
 *   <type>  q4_0 | q4_1 | q8_0 | q4_k | q6_k
 *   <KS>    1 | 2 | 4 | 8: wavefronts that split a row's K.  A lane owns one unit of
 *           CERA_K_UNIT_ELEMS(type) weights, so pick the smallest KS with k / unit <= 64 * KS
 *           (k up to 16384 for 32-weight units, 32768 for the K-quants).
 *   n_units        = k / CERA_K_UNIT_ELEMS(type)
 *   row_bytes      = k / block_elems * block_bytes of the type
 *   rows_per_group = rows one workgroup walks, two at a time: any positive even number; the
 *                    library uses ceil(m / (n_cu * 24 / KS)) rounded up to even
 *   grid  = ceil(m / rows_per_group) workgroups of 64 * KS threads.
 * w2, dbg_dots, dbg_stride and dbg_asums are unused by these instances: pass zero. */
#define CERA_K_UNIT_ELEMS(ggml_type) (((ggml_type) == 12 || (ggml_type) == 14) ? 64u : 32u)
typedef struct {
    const uint8_t* w;
    const uint8_t* w2;
    const int8_t* xq;      /* [k] */
    const float* xs;       /* [k/32] */
    float* y;              /* [m] */
    const float* resid;    /* [m], `add` instances only */
    uint32_t m;
    uint32_t n_units;
    uint32_t row_bytes;
    uint32_t rows_per_group;
    int32_t* dbg_dots;
    uint32_t dbg_stride;
    int32_t* dbg_asums;
} cera_k_gemv_args;

/* ==== the one-wavefront-per-row decode kernels and the decode copies they read ====================
 * What libcera_hip.so launches for a decode step on matrices with k <= 16384: a wavefront owns
 * whole rows, so there is no K split, no LDS combine and no barrier in the row loop, and the
 * matrix is read from its DECODE COPY -- a per-row permutation of the native blocks into planes
 * padded to 128 bytes, so that every load instruction of a wavefront covers whole 128-byte lines
 * and can carry the non-temporal hint (a load-time re-layout for the kernel that reads it, as
 * cera's x86 path does with repack_q4_k_8x8, cera/src/backend/cpu.rs:1282-1358).  Results have
 * the bits of the cera_k_gemv_* kernels on the native bytes.
 *
 * "passes" P below: a lane holds one unit (CERA_K_UNIT_ELEMS weights) per pass of 64 units, so
 * P = ceil(k / CERA_K_UNIT_ELEMS / 64).  k must be whole blocks of the type (256 for the K-quants,
 * 32 otherwise). */

/* bytes of one row of the decode copy (rows are contiguous at this stride) */
#define CERA_K_UP128(b) ((((uint32_t)(b)) + 127u) & ~127u)
#define CERA_K_DECODE_COPY_ROW_BYTES(ggml_type, k)                                                              \
    ((ggml_type) == 12   ? CERA_K_UP128(4 * ((k) / 64)) + 2 * CERA_K_UP128(16 * ((k) / 64))                      \
     : (ggml_type) == 14 ? 3 * CERA_K_UP128(16 * ((k) / 64)) + CERA_K_UP128(4 * ((k) / 64)) + CERA_K_UP128((k) / 128) \
     : (ggml_type) == 2  ? CERA_K_UP128(2 * ((k) / 32)) + CERA_K_UP128(16 * ((k) / 32))                          \
     : (ggml_type) == 3  ? CERA_K_UP128(4 * ((k) / 32)) + CERA_K_UP128(16 * ((k) / 32))                          \
                         : CERA_K_UP128(2 * ((k) / 32)) + 2 * CERA_K_UP128(16 * ((k) / 32)))

/* ---- cera_k_decode_copy_<type> ---------------------------------------------------------------
 * Builds the decode copy of m rows: dst row r at dst + r * copy_row_bytes, copy_row_bytes =
 * CERA_K_DECODE_COPY_ROW_BYTES(type, k).  src must be 16-byte aligned, k <= 16384.
 * grid = m workgroups of 256 threads. */
typedef struct {
    const uint8_t* src;        /* native rows, row r at src + r * row_bytes */
    uint8_t* dst;
    uint32_t n_units;          /* k / CERA_K_UNIT_ELEMS(type) */
    uint32_t row_bytes;
    uint32_t copy_row_bytes;
} cera_k_decode_copy_args;

/* Arguments of every row kernel.  w / w2 point at DECODE COPIES and row_bytes is their stride. */
typedef struct {
    const uint8_t* w;          /* [m] rows */
    const uint8_t* w2;         /* norm_gate_up: the up matrix (w = gate), same shape; else NULL */
    uint32_t m;
    uint32_t k;
    uint32_t row_bytes;
    uint32_t rows_per_wave;    /* the instance's fixed value (below): informational */
    const int8_t* xq;          /* row_gemv / row_gemv_long: Q8_0 activations [k], scales [k/32] */
    const float* xs;
    const float* x;            /* norm_* kernels: the f32 vector [k] and the norm weights [k] */
    const float* norm_w;
    float eps;
    float* y;                  /* store / add / norm_qkv: [m] */
    const float* resid;        /* add: [m] */
    int8_t* out_q;             /* norm_gate_up: Q8_0 of silu(gate.n) * (up.n): [m] codes, [m/32] scales */
    float* out_s;
} cera_k_row_gemv_args;

/* ---- cera_k_row_gemv_<type>_p<P>_<store|add> -------------------------------------------------
 * y = W . (xs, xq)  (add: + resid), k <= 4096: the O projection and the vocabulary head.
 *   <type> q4_k | q6_k with P = 1;  q4_0 | q4_1 | q8_0 with P = 1 (k <= 2048) or 2.
 * Two rows per wavefront, four wavefronts per workgroup: grid = ceil(m / 8) workgroups of 256.
 *
 * ---- cera_k_row_gemv_long_<type>_p<P>_add ----------------------------------------------------
 * y = resid + W . (xs, xq), 4096 < k <= 16384: the down projection.  One row per wavefront, the
 * activations staged in LDS.  <type> q4_k | q6_k with P = 2 | 3 | 4;  q4_0 | q4_1 | q8_0 with P = 4
 * (k <= 8192) or 8.  grid = ceil(m / 4) workgroups of 256.
 *
 * ---- cera_k_norm_gate_up_<type>_p<P> ---------------------------------------------------------
 * out = Q8_0(silu(gate . n) * (up . n)) with n = Q8_0(rmsnorm(x, norm_w, eps)): the first half of
 * the feed-forward block in one launch (cpu::rmsnorm cera/src/backend/cpu.rs:2479-2496,
 * quantize_f32_to_q8_0 :942-958, silu_mul_inplace :2570-2575).  k <= 4096, m % 32 == 0.
 *   <type> q4_k with P = 1;  q4_0 | q4_1 | q8_0 with P = 1 | 2.
 * Four row pairs per wavefront, sixteen wavefronts: grid = ceil(m / 64) workgroups of 1024. */

/* ---- cera_k_norm_qkv_<ta>_<tb>_p<P>_r<R> -----------------------------------------------------
 * ya = A . n and yb = B . n with n = Q8_0(rmsnorm(x, norm_w, eps)): the attention projections in
 * one launch (A = the fused Q|K|V matrix or Q|K, B = V; pass b = a and n_blocks_a = the whole grid
 * for a single matrix).  Same k (<= 4096) and x / norm_w / eps in a and b.
 *   <ta>_<tb>  q4_k_q4_k | q4_k_q6_k | q6_k_q4_k | q6_k_q6_k with P = 1;
 *              q4_0_q4_0 | q4_1_q4_1 | q8_0_q8_0 with P = 1 | 2
 *   <R>        rows per wavefront, 1 | 2 (the library uses 2 when the two matrices have at
 *              least 8 rows per CU together)
 * Eight wavefronts per workgroup: n_blocks_a = ceil(a.m / (8 R)), grid = n_blocks_a +
 * ceil(b.m / (8 R)) workgroups of 512; workgroups [0, n_blocks_a) take a. */
typedef struct {
    cera_k_row_gemv_args a, b;
    uint32_t n_blocks_a;
} cera_k_row_gemv_pair_args;

/* ==== the rest of a forward pass ===================================================================
 * With the kernels below a host runs LlamaModel::forward and ::forward_prefill
 * (cera/src/model/llama.rs:468-597, 738-1523) from the code object alone; cera_amd/hsaco_api.py does,
 * and tests/test_gpu_hsaco.py compares its logits with the library's.  KV caches are head-major,
 * [n_kv_heads][max_seq][head_dim], f32 (`f32` instances) or IEEE half (`f16`); head_dim 64 or 128. */

/* ---- cera_k_embed_token / cera_k_embed_rows ---------------------------------------------------
 * One row of the embedding table dequantized (dequantize_*_row, cera/src/quant.rs:318-539) and
 * multiplied by `scale` when that is not 1.  ggml_type: 0 F32, 1 F16, 30 BF16, 2, 3, 8, 12, 13, 14.
 * embed_token also writes scalars[0] = token, scalars[1] = pos (the position word rope_kv reads).
 * grid = ceil(k / 256) workgroups of 256;  embed_rows: grid = (ceil(k / 256), n_tokens), out [n][k]. */
typedef struct {
    const uint8_t* w;
    uint64_t row_bytes;
    uint32_t ggml_type, token, pos, k;
    uint32_t* scalars;
    float scale;
    float* out;
} cera_k_embed_token_args;
typedef struct {
    const uint8_t* w;
    uint64_t row_bytes;
    const uint32_t* tokens;
    uint32_t ggml_type, k;
    float scale;
    float* out;
} cera_k_embed_rows_args;

/* ---- cera_k_rmsnorm_rows / cera_k_rmsnorm_rows_q8_0 -------------------------------------------
 * cpu::rmsnorm (cera/src/backend/cpu.rs:2479-2496) of `rows` rows of n elements (x and y may be
 * the same buffer); _q8_0 also writes each row's Q8_0 quantization: scales [rows][n/32], quants
 * [rows][n], bsum [rows][n/32] = scale * sum(quants) (nullable).  n % 32 == 0 for _q8_0.
 * grid = rows workgroups of 256. */
typedef struct {
    const float* x;
    const float* w;
    uint32_t n;
    float eps;
    float* y;
    float* scales;
    int8_t* quants;
    float* bsum;
} cera_k_rmsnorm_rows_args;

/* ---- cera_k_rope_kv_<f32|f16> -----------------------------------------------------------------
 * RoPE on q and k in place and the append of k, v to the caches (rope_type 1: interleaved pairs,
 * cera/src/backend/cpu.rs:5161-5180; 0: split halves, :5031-5045).  cs_table [max_seq][head_dim/2]
 * of (cos, sin) built by the host with the reference's recurrence: theta_0 = pos as f32,
 * theta_{i+1} = theta_i * base^(-2/head_dim) in f32, angle = theta_i (/ freq_factor_i for rope_type
 * 1), libm cosf / sinf.  Token t of the batch sits at position *pos + t; q [n][n_heads*head_dim],
 * k, v [n][n_kv_heads*head_dim].  grid = (n_heads + 2 n_kv_heads, n_tokens) of head_dim / 2 threads. */
typedef struct {
    float* q;
    float* k;
    const float* v;
    const float* cs_table;
    const uint32_t* pos;
    uint32_t n_heads, n_kv_heads, head_dim, rope_type;
    void* k_cache;
    void* v_cache;
    uint32_t max_seq;
} cera_k_rope_kv_args;

/* ---- cera_k_attn_decode_partial_<f32|f16>_hd<64|128>_g<1|2|4>_s<1|4> ---------------------------
 * GQA flash-decode, split over the keys (decode_attention, cera/src/model/transformer.rs:1249-1305):
 * wavefront (query, kv head, sub-group, part) scans chunks_per_part chunks of 8 S keys with an
 * online softmax for g query heads and leaves an unnormalised partial.
 *   g        query heads one wavefront serves; g_total = n_heads / n_kv_heads must be a multiple
 *            (the library takes g = g_total / 2 for groups of 4 and 8 below 16k keys)
 *   S        8 S keys per chunk (the library: 1 below 1024 keys, 4 beyond with split groups)
 *   n_parts  = ceil(ceil(seq_len / (8 S)) / chunks_per_part), at most 1024; the library aims at
 *            4 wavefronts per CU: chunks_per_part = max(1, ceil(chunks / (4 n_cu / n_kv)))
 *   seq_len  keys visible to query 0; query i (n_queries > 1, q rows q_stride floats apart) sees
 *            seq_len + i
 *   part_acc [n_queries][n_kv][n_parts][g_total][head_dim], part_ml [...][g_total][2]
 * grid = ceil(ceil(n_parts / 4) * n_kv / 8) * 8 * (g_total / g) * n_queries workgroups of 256
 * (four consecutive parts per workgroup; the kernel maps launch indices to key ranges XCD by XCD
 * and ignores the padding).
 * ---- cera_k_attn_decode_merge_hd<64|128>[_q8_0] ------------------------------------------------
 * out[head] = sum_p e^(m_p - M) acc_p / sum_p e^(m_p - M) l_p; _q8_0 also writes the Q8_0
 * quantization of the n_heads * head_dim outputs (scales, quants, bsum nullable).
 * grid = (n_heads, n_queries) workgroups of 256; out [n_queries][n_heads * head_dim]. */
typedef struct {
    const float* q;
    const void* kc;
    const void* vc;
    uint32_t seq_len, max_seq;
    float scale;
    uint32_t chunks_per_part, n_parts, q_stride, g_total, n_kv, n_queries;
    float* part_acc;
    float* part_ml;
} cera_k_attn_decode_args;
typedef struct {
    const float* part_acc;
    const float* part_ml;
    uint32_t n_parts, g_total, n_heads;
    uint32_t n_pairs;          /* prefill merge: n_heads * n_queries; decode merge: unused */
    float* out;
    float* scales;
    int8_t* quants;
    float* bsum;
} cera_k_attn_merge_args;

/* ---- cera_k_attn_prefill_partial_<f32|f16>_hd<64|128>_g<1|2|4|8> ------------------------------
 * Causal attention of a batch of queries (>= 16; fewer go through the decode kernel with
 * n_queries) on the f16 matrix cores: a workgroup = 32 queries x one kv head x one key part,
 * g = n_heads / n_kv_heads wavefronts.  The batch's own keys are already in the cache (rope_kv).
 *   first_len  keys visible to query 0; query i sees first_len + i
 *   part_keys  keys per part, a multiple of 32 (the library: 128 up to 1024 keys, else about an
 *              eighth of the keys); n_parts = ceil((first_len + n_queries - 1) / part_keys) <= 1024
 *   q rows 16-byte aligned, q_stride floats apart
 * grid = (ceil(n_queries / 32), n_kv, n_parts) workgroups of 64 g.
 * ---- cera_k_attn_prefill_merge_hd<64|128>[_q8_0] -----------------------------------------------
 * The merge for a batch: eight (query, head) pairs per workgroup.  grid = ceil(n_pairs / 8) of 256. */
typedef struct {
    const float* q;
    const void* kc;
    const void* vc;
    uint32_t first_len, n_queries, max_seq;
    float scale;
    uint32_t part_keys, n_parts, q_stride;
    float* part_acc;
    float* part_ml;
} cera_k_attn_prefill_args;

/* ---- cera_k_silu_mul[_q8_0], cera_k_add, cera_k_bias, cera_k_scale ----------------------------
 * silu_mul: out = gate / (1 + expf(-gate)) * up (silu_mul_inplace, cera/src/backend/cpu.rs:2570-2575),
 * n % 4 == 0 (_q8_0: n % 32 == 0, plus the Q8_0 quantization of out in rows of any length that
 * is a multiple of 32); grid = ceil(n / 4 / 256) of 256.  add: out = a + b_scale * b.  bias: x += b.
 * scale: x *= s.  grid = ceil(n / 256) of 256. */
typedef struct {
    const float* gate;
    const float* up;
    uint64_t n;
    float* out;
    float* scales;
    int8_t* quants;
    float* bsum;
} cera_k_silu_mul_args;
typedef struct { const float* a; const float* b; float b_scale; uint32_t n; float* out; } cera_k_add_args;
typedef struct { float* x; const float* b; uint32_t n; } cera_k_bias_args;
typedef struct { float* x; float s; uint32_t n; } cera_k_scale_args;

/* ---- cera_k_argmax_partial / cera_k_argmax_final ----------------------------------------------
 * Greedy sampling (cera/src/sampler.rs:20-30: strict >, lowest index on ties).  partial: workgroup
 * b reduces its slice of x[0, n) to (pv[b], pi[b]); grid = np workgroups of 256 (the library:
 * np = min(1024, ceil(n / 1024))).  final: one workgroup of 256 reduces the np candidates into
 * *out (and *out2 when not null, e.g. a device view of pinned host memory). */
typedef struct { const float* x; uint32_t n; float* pv; uint32_t* pi; } cera_k_argmax_partial_args;
typedef struct { const float* pv; const uint32_t* pi; uint32_t np; uint32_t* out; uint32_t* out2; } cera_k_argmax_final_args;

/* ---- cera_k_kv_shift_<f32|f16>_hd<64|128> -----------------------------------------------------
 * The n_keep context shift (InferenceState::shift_kv_with_rope, cera/src/kv_cache.rs:1091-1310):
 * rows [src_row, src_row + n_rows) of every kv head move to [dst_row, ...) of dst, K rows rotated
 * on the way by R(-shift) whose head_dim / 2 (cos, sin) pairs the host builds with the recurrence
 * above (theta_0 = -shift); delta_cs NULL = plain copy (V, and the copy back from staging when
 * source and destination rows overlap).  head strides in elements.
 * grid = (ceil(n_rows * head_dim / 8 / 256), n_kv_heads) of 256. */
typedef struct {
    const void* src;
    void* dst;
    uint32_t src_row, dst_row, n_rows;
    uint64_t src_head_stride, dst_head_stride;
    const float* delta_cs;
    uint32_t rope_type;
} cera_k_kv_shift_args;

/* ==== batched (prefill) GEMMs: transformer::gemm_preq (cera/src/model/transformer.rs:710-788) =====
 * out[i * ld_m + j * ld_n] = sum over k of W[i][k] * B[j][k] (+ resid), B = n token rows quantized
 * to Q8_0 by cera_k_quantize_q8_0 / cera_k_rmsnorm_rows_q8_0 / a _q8_0 merge: bq [n][k], bs
 * [n][k/32], bsum [n][k/32] (needed by q4_k and q4_1).  Exact integer block dots, then the
 * reference's per-block float scales.  k % 256 == 0 for q4_k / q6_k, k % 128 == 0 otherwise.
 *   cera_k_gemm_q4_k          fp8 matrix cores; reads bf8, the split copy cera_k_gemm_act_fp8 makes
 *                             of (bq, bs, bsum): CERA_K_GEMM_FP8_ACT_BYTES(n, k) bytes,
 *                             grid = ceil(n / 64) * 2 * (k / 256) workgroups of 256; its halves (nullable) also
 *                             receives what cera_k_gemm_act_f16 would write for the same quants ([n][k] f16)
 *   cera_k_gemm_q4_k_swiglu   w = gate, w2 = up (both m x k, m % 32 == 0): nothing goes to out; hq [n][m], hs and
 *                             hbsum [n][m/32] receive Q8_0(silu(gate.x) * (up.x)); a workgroup takes 64 gate and the
 *                             same 64 up rows: grid = (ceil(n / 64), ceil(m / 64)), k_chunk = k; hh (nullable) also
 *                             receives the quants as f16 [n][m] in cera_k_gemm_act_f16's order, for a q6_k GEMM that
 *                             follows (NULL in every other kernel of this family)
 *   cera_k_gemm_q6_k          f16 matrix cores; reads bh, the quants as f16 made by
 *                             cera_k_gemm_act_f16 (n * k * 2 bytes; n_words = n * k / 16,
 *                             grid = ceil(n_words / 256) of 256)
 *   cera_k_gemm_q4_0 | q4_1 | q8_0   int8 matrix cores
 * grid = (ceil(n / 64), ceil(m / 128) [+ ceil(m2 / 128) for a pair], split) workgroups of 256.
 * One matrix, no split: k_chunk = k, part_stride = 0, w2 = out2 = NULL, m2 = 0, tiles1 =
 * ceil(m / 128), hq = hs = hbsum = dbg_dots = NULL.  Split K (grid.z = split, k_chunk = k / split
 * a multiple of 512): every slice writes its partial to out + z * part_stride (out is then a
 * scratch buffer, ld_m = 1, ld_n = m) and cera_k_gemm_reduce adds them in order.
 * The library's results for a token-major output are ld_m = 1, ld_n = m. */
#define CERA_K_GEMM_FP8_ACT_BYTES(n, k) ((uint64_t)(((n) + 63) / 64) * 2 * ((k) / 256) * 21504u)
typedef struct {
    const uint8_t* w;
    const int8_t* bq;
    const float* bs;
    const float* bsum;
    const void* bh;
    float* out;
    uint32_t m, n, k;
    uint32_t row_bytes;
    uint64_t ld_m, ld_n;
    const float* resid;
    float resid_scale;
    uint32_t k_chunk;
    uint64_t part_stride;
    const uint8_t* w2;
    float* out2;
    uint32_t m2, tiles1;
    uint64_t ld_n2;
    int8_t* hq;
    float* hs;
    float* hbsum;
    int32_t* dbg_dots;
    const uint8_t* bf8;
    uint16_t* hh;
} cera_k_gemm_args;
typedef struct { const int8_t* quants; const float* scales; const float* bsum; uint8_t* out; uint32_t n, k; void* halves; } cera_k_gemm_act_fp8_args;
typedef struct { const void* quants; void* out; uint64_t n_words; } cera_k_gemm_act_f16_args;
/* out[e] = (resid[e] + resid_scale *) sum_z part[z * part_stride + e] over n4 float4s; for a pair
 * float4s from n4_first on go to out2 (no pair: n4_first = n4, out2 = NULL).
 * grid = ceil(n4 / 256) of 256. */
typedef struct {
    const float* part;
    uint32_t n_split;
    uint64_t part_stride, n4;
    float* out;
    const float* resid;
    float resid_scale;
    uint64_t n4_first;
    float* out2;
} cera_k_gemm_reduce_args;

#ifdef __cplusplus
}
#endif
#endif /* CERA_HIP_KERNELS_H */
