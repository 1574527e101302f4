/* cera_hip.h -- C ABI of the MI355X `hip` compute backend for cera's dense
 * transformer decode/prefill hot path.
 *
 * This is the boundary a `cera-hip-sys` Rust crate binds (plain pointers and
 * sizes, no C++ types).  Each entry point names the cera interface it stands
 * in for (paths relative to the cera source tree).
 *
 * Conventions
 *  - every function that can fail returns a cera_hip_status; the message for
 *    the last failure on a context is returned by cera_hip_last_error();
 *  - nothing aborts or throws across this boundary;
 *  - "host" pointers are ordinary CPU memory owned by the caller and only
 *    borrowed for the duration of the call; "dev" pointers come from
 *    cera_hip_malloc() on the same context;
 *  - all work of a context runs on that context's single HIP stream; calls on one context are
 *    serialised by the library (a model is additionally serialised by its own lock), so models
 *    sharing a context may be driven from different threads, one call at a time;
 *  - weights stay in their native GGUF block layout in device memory.
 */
#ifndef CERA_HIP_H
#define CERA_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#if defined(__GNUC__)
#define CERA_HIP_API __attribute__((visibility("default")))
#else
#define CERA_HIP_API
#endif

typedef struct cera_hip_ctx cera_hip_ctx;         /* device, stream, scratch            */
typedef struct cera_hip_model cera_hip_model;     /* device weights, KV cache, seq_len   */
typedef struct cera_hip_dtensor cera_hip_dtensor; /* one weight matrix resident in HBM   */
typedef struct cera_hip_event cera_hip_event;     /* HIP event on the context's stream   */

typedef enum {
    CERA_HIP_OK = 0,
    CERA_HIP_ERR_DEVICE = 1,            /* HIP runtime error (message has the HIP string)  */
    CERA_HIP_ERR_OOM = 2,               /* device or host allocation failed                */
    CERA_HIP_ERR_UNSUPPORTED_DTYPE = 3, /* no kernel for this GGML type: refuse, never skip */
    CERA_HIP_ERR_SHAPE = 4,             /* size/shape/alignment does not fit the kernel    */
    CERA_HIP_ERR_POSITION = 5,          /* pos/start_pos != current sequence length        */
    CERA_HIP_ERR_ARGUMENT = 6           /* null pointer or out-of-range scalar             */
} cera_hip_status;

/* GGML type ids as cera maps them: cera/src/gguf.rs:259-278. */
enum {
    CERA_HIP_F32 = 0, CERA_HIP_F16 = 1, CERA_HIP_Q4_0 = 2, CERA_HIP_Q4_1 = 3, CERA_HIP_Q8_0 = 8,
    CERA_HIP_Q4_K = 12, CERA_HIP_Q5_K = 13, CERA_HIP_Q6_K = 14, CERA_HIP_BF16 = 30
};

/* A weight matrix as cera resolves it from a GGUF: `WeightRef` {dtype, m, k}
 * plus the mmap slice (cera/src/model/transformer.rs:127-139, 187-231).
 * m = output rows, k = inner dimension; data is m rows of k/block_elems blocks. */
typedef struct {
    uint32_t ggml_type;
    uint32_t _reserved;
    uint64_t m, k;
    const void* data; /* host */
    uint64_t nbytes;
} cera_hip_tensor;

/* Per-layer weights: the fields of `LayerRefs` + norm/bias vectors that
 * LlamaModel::from_gguf_with_id resolves (cera/src/model/llama.rs:158-450). */
typedef struct {
    const float *attn_norm, *ffn_norm; /* f32[hidden] */
    cera_hip_tensor attn_q, attn_k, attn_v, attn_output, ffn_gate, ffn_up, ffn_down;
    const float *q_bias, *k_bias, *v_bias; /* nullable (Qwen2) */
    const float *q_norm, *k_norm;          /* nullable, f32[head_dim] (Qwen3) */
} cera_hip_layer;

/* `ModelConfig` + `AttnDims` (cera/src/model/mod.rs:117-145, llama.rs:450-466). */
typedef struct {
    uint32_t n_layers, hidden, ffn, n_heads, n_kv_heads, head_dim, vocab, max_seq_len;
    uint32_t rope_type; /* 0 = NEOX (split halves), 1 = NORM (interleaved pairs) */
    float rope_theta, rms_eps, embed_scale, residual_scale;
    float attn_scale;  /* 0 => 1/sqrt(head_dim) */
    float logit_scale; /* logits are divided by this; 1 = off */
    const float* rope_freqs; /* nullable, f32[head_dim/2] */
} cera_hip_config;

/* ---- context ------------------------------------------------------------ */

/* Create a context on HIP device `device`.  Stands where a GPU backend's context constructor
 * does (cera/src/model/mod.rs:672-703 builds one per load).  hsaco_path NULL: every kernel comes
 * from the gfx950 code object embedded in this library.  hsaco_path = path of the standalone
 * code object cera_hip_gfx950.hsaco (built beside this library; include/cera_hip_kernels.h): it
 * is loaded with hipModuleLoad and the Q8_0 quantizer and the GEMV instances it exports are
 * launched from it with hipModuleLaunchKernel -- the same code, results bit-identical; kernels
 * it does not export still come from the embedded object.  A file that cannot be loaded or is
 * not that code object fails the call. */
CERA_HIP_API cera_hip_status cera_hip_ctx_create(int device, const char* hsaco_path, cera_hip_ctx** out);
CERA_HIP_API void cera_hip_ctx_destroy(cera_hip_ctx*);
/* Message of the most recent failure on `ctx` (ctx may be NULL for a failed
 * cera_hip_ctx_create: then the process-wide last message).  Valid until the
 * next call on the same context. */
CERA_HIP_API const char* cera_hip_last_error(const cera_hip_ctx*);
CERA_HIP_API cera_hip_status cera_hip_sync(cera_hip_ctx*);
/* Decode copies (on by default).  When on, cera_hip_model_create and cera_hip_decode_ops_dev give
 * every Q4_K / Q6_K / Q4_0 / Q4_1 / Q8_0 projection matrix (k at most 32768; 16384 for the 32-weight blocks) a second copy of
 * about the same size in which each row's bytes are permuted so that the decode GEMV kernels read
 * it in whole 128-byte lines with non-temporal loads (+6 % decode rate on the 8B model for about
 * twice those matrices' memory); every other reader keeps the native GGUF bytes.  Results are
 * bit-identical either way; a copy that does not fit in device memory is skipped.  Applies to
 * matrices prepared after the call.  A load-time re-layout
 * for one kernel, as the reference's x86 path does with repack_q4_k_8x8
 * (cera/src/backend/cpu.rs:1282-1358); it has no switch there. */
CERA_HIP_API cera_hip_status cera_hip_ctx_set_decode_copies(cera_hip_ctx* ctx, int enabled);
/* The rule by which cera_hip_model_create hands out decode copies, as plain arithmetic (no device
 * is touched; callable without a GPU).  A model's copies are built last -- after every native
 * upload, the KV caches and the single-token buffers -- and only while the device keeps
 * cera_hip_decode_copy_reserve_bytes(cfg) free: the buffers of the largest batched prefill pass
 * (2048 tokens, fewer when max_seq_len is shorter), that pass's all-positions logits, and 512 MiB
 * for the context's workspaces.  Candidates are walked in priority order (the vocabulary head, then
 * layer by layer); copy_bytes[i] == 0 marks a matrix that gets none; one that does not fit is
 * skipped and later, smaller ones are still tried.  take[i] (nullable) receives 1 for each copy
 * built; the return value is the bytes they take.  A model that loads and prefills with copies off
 * therefore does so with copies on, with all, some or none of its matrices copied.  No counterpart
 * in the reference (its repack replaces the native bytes instead of adding to them). */
CERA_HIP_API uint64_t cera_hip_decode_copy_reserve_bytes(const cera_hip_config* cfg);
CERA_HIP_API uint64_t cera_hip_decode_copy_plan(const uint64_t* copy_bytes, uint32_t n, uint64_t free_bytes,
                                                uint64_t reserve_bytes, uint8_t* take);
/* Device properties for reporting: name (<= 255 chars), CU count, bytes of HBM. */
CERA_HIP_API cera_hip_status cera_hip_device_info(cera_hip_ctx*, char* name256, uint32_t* n_cu,
                                                  uint64_t* hbm_bytes);

/* ---- device memory and events (benchmark / timing plumbing) ------------- */
CERA_HIP_API cera_hip_status cera_hip_malloc(cera_hip_ctx*, uint64_t nbytes, void** dev_out);
CERA_HIP_API cera_hip_status cera_hip_free(cera_hip_ctx*, void* dev);
CERA_HIP_API cera_hip_status cera_hip_upload(cera_hip_ctx*, void* dev_dst, const void* host_src, uint64_t nbytes);
CERA_HIP_API cera_hip_status cera_hip_download(cera_hip_ctx*, void* host_dst, const void* dev_src, uint64_t nbytes);
CERA_HIP_API cera_hip_status cera_hip_copy_dev(cera_hip_ctx*, void* dev_dst, const void* dev_src, uint64_t nbytes);
/* Device-to-device copy done by a plain streaming kernel of this library (not the runtime's
 * copy engine): exactly nbytes read + nbytes written, the known-traffic kernel used to
 * calibrate hardware byte counters.  nbytes and both pointers must be multiples of 16.
 * Measurement aid; no counterpart in the reference. */
CERA_HIP_API cera_hip_status cera_hip_copy_kernel(cera_hip_ctx*, void* dev_dst, const void* dev_src, uint64_t nbytes);
CERA_HIP_API cera_hip_status cera_hip_event_create(cera_hip_ctx*, cera_hip_event** out);
CERA_HIP_API void cera_hip_event_destroy(cera_hip_event*);
CERA_HIP_API cera_hip_status cera_hip_event_record(cera_hip_ctx*, cera_hip_event*);
/* Waits for `stop`, then returns milliseconds between the two events. */
CERA_HIP_API cera_hip_status cera_hip_event_elapsed_ms(cera_hip_ctx*, cera_hip_event* start,
                                                       cera_hip_event* stop, float* ms);

/* ---- weights in HBM, native GGUF block layout --------------------------- */
/* Copies `t->data` to device memory unchanged (the GPU loaders' upload step,
 * cera/src/model/gpu_weight_source.rs:40-118 consumers).  Refuses types
 * without a kernel and k that is not a whole number of blocks. */
CERA_HIP_API cera_hip_status cera_hip_tensor_upload(cera_hip_ctx*, const cera_hip_tensor* t, cera_hip_dtensor** out);
/* A second handle of the same shape whose bytes are a device-side copy of
 * `src` (distinct addresses: lets a benchmark rotate its working set past the
 * last-level cache without re-uploading). */
CERA_HIP_API cera_hip_status cera_hip_tensor_clone(cera_hip_ctx*, const cera_hip_dtensor* src, cera_hip_dtensor** out);
CERA_HIP_API void cera_hip_tensor_free(cera_hip_ctx*, cera_hip_dtensor*);
CERA_HIP_API uint64_t cera_hip_tensor_nbytes(const cera_hip_dtensor*);

/* ---- kernel-level entry points, host buffers (parity tests) ------------- */

/* cpu::quantize_f32_to_q8_0_into (cera/src/backend/cpu.rs:969-1041; arithmetic
 * at :942-958).  x f32[k], k % 32 == 0 -> scales f32[k/32], quants i8[k]. */
CERA_HIP_API cera_hip_status cera_hip_quantize_q8_0(cera_hip_ctx*, const float* x, uint64_t k, float* scales,
                                                    int8_t* quants);

/* cpu::gemv_dispatch (cera/src/backend/cpu.rs:2360-2474): y[m] = W[m,k] . x[k].
 * Q4_0/Q4_1/Q8_0/Q4_K/Q6_K quantize x to Q8_0 and run the int8 kernel; Q5_K
 * dots against the unquantized f32 x, as the CPU path does.
 * dbg_block_dots / dbg_block_asums (nullable) receive the integer block dots
 * the kernel formed: Q4_0 [m][k/32] sum (q-8)a; Q8_0 [m][k/32] sum w a;
 * Q4_1, Q4_K [m][k/32] sum q a with asums [k/32] = sum a; Q6_K [m][k/16]
 * sum q a (q unsigned 0..63) with asums [k/16]. */
CERA_HIP_API cera_hip_status cera_hip_gemv(cera_hip_ctx*, const cera_hip_tensor* w, const float* x, float* y,
                                           int32_t* dbg_block_dots, int32_t* dbg_block_asums);

/* The same product for a short batch of n activation vectors (x f32 [n][k], y f32 [n][m]) with
 * the weights streamed once per 8 vectors: what the prefill path runs instead of the int8 GEMM
 * while a batch is at most 16 tokens (a few new tokens of a chat turn, the verification pass of
 * speculative decoding, cera/src/model/mod.rs:221-249).  Row t of y is bit-identical to
 * cera_hip_gemv on x[t].  A matrix of 8192 rows or more is given its decode copy first and read
 * through the one-wavefront-per-row form, as a model's gate / up / head matrices are (same bits).
 * CERA_HIP_ERR_UNSUPPORTED_DTYPE for Q5_K and for k beyond one unit per
 * lane (k > 16384; Q4_K and Q6_K 32768). */
CERA_HIP_API cera_hip_status cera_hip_gemv_nb(cera_hip_ctx*, const cera_hip_tensor* w, const float* x, uint32_t n,
                                              float* y);

/* Two projections of the same activation vector in one launch: what the decode step does for a
 * layer whose attn_q|attn_k (Q4_K, stored back to back) and attn_v (Q6_K) differ in block type
 * (the Q4_K_M mix, cera/src/convert/quantize.rs:102-113); each result is exactly that of
 * cera_hip_gemv on its own matrix (same kernel body, same row grouping).  Kernel instances
 * exist for a Q4_K matrix with k <= 4096 next to a Q6_K one; any other combination is
 * CERA_HIP_ERR_UNSUPPORTED_DTYPE (the model then launches the two one after the other). */
CERA_HIP_API cera_hip_status cera_hip_gemv_pair(cera_hip_ctx*, const cera_hip_tensor* a, const cera_hip_tensor* b,
                                                const float* x, float* ya, float* yb);

/* transformer::gemm_preq over quantize_columns (cera/src/model/transformer.rs:
 * 710-788, 865-946; kernels cera/src/backend/cpu.rs:1437-1557).
 * x is [n][k] row-major f32 (one activation row per token), each row is
 * quantized to Q8_0; out is [m][n] row-major -- the reference's
 * out[m_out_features][n_tokens] layout (cera/src/backend/simd.rs:5130-5148).
 * A Q5_K matrix (k a multiple of 256) is multiplied with the f32 rows as they are, to f32
 * accuracy: the reference never quantizes the input of a Q5_K projection
 * (gemv_q5km_f32, cera/src/backend/cpu.rs:1830-1854), it only has no batched form of it. */
CERA_HIP_API cera_hip_status cera_hip_gemm(cera_hip_ctx*, const cera_hip_tensor* w, const float* x, uint64_t n,
                                           float* out);

/* cera_hip_gemm with the integer block dots its matrix-core instructions produced, from debug
 * instances of the same kernels (the integer quantities cera's own test reference defines,
 * cera/src/backend/simd.rs:6609-6629): dots [m][n][k/32] int32 -- Q4_0 sum (q-8)a, Q8_0 sum w a,
 * Q4_1 / Q4_K sum q a, q in 0..15.  Q6_K forms its dots per 16-element scale group on the f16
 * matrix cores: dots [m][n][k/16], each the f32 bit pattern of that instruction's result,
 * sum (q-32)a -- an exact integer, which a test can check because it sees the float.  out
 * (nullable) receives the [m][n] result of the same launch.  At most 64 Mi dots per call. */
CERA_HIP_API cera_hip_status cera_hip_gemm_block_dots(cera_hip_ctx*, const cera_hip_tensor* w, const float* x, uint64_t n,
                                                      int32_t* dots, float* out);

/* Two gemm_preq calls on the same quantized activations in one launch, the way the prefill pass
 * issues attn_q | attn_k and ffn_gate | ffn_up (LlamaModel::forward_prefill_batched,
 * cera/src/model/llama.rs:738-1523, multiplies them one after the other): one grid over both
 * matrices' row tiles, split-K partials side by side when the tiles are few.  The matrices must
 * share a type that has an int8 GEMM and k.  Outputs are token-major, out_a[n][m_a] and
 * out_b[n][m_b] (the layout the batched forward pass keeps), each equal to cera_hip_gemm on its
 * own matrix up to the order of the split-K partial sums. */
CERA_HIP_API cera_hip_status cera_hip_gemm_pair(cera_hip_ctx*, const cera_hip_tensor* a, const cera_hip_tensor* b,
                                                const float* x, uint64_t n, float* out_a, float* out_b);

/* The first half of the FFN of the batched forward pass in one launch (LlamaModel::
 * forward_prefill_batched, cera/src/model/llama.rs:738-1523: gemm_preq on ffn_gate and ffn_up,
 * cpu::silu_mul_inplace, cera/src/backend/cpu.rs:2570-2575, then quantize_columns for the down
 * projection, cera/src/model/transformer.rs:865-946): quants[n][m] / scales[n][m/32] =
 * Q8_0(silu(gate.x) * (up.x)) per token row, quantized in the GEMM's epilogue.  gate and up must
 * share a type with an int8 GEMM (not Q6_K), k and m, m a multiple of 32.  Small batches, which
 * need a K split to fill the chip, take the two GEMMs and the SwiGLU kernel instead (*fused = 0,
 * nullable); both routes give identical bytes. */
CERA_HIP_API cera_hip_status cera_hip_gemm_swiglu(cera_hip_ctx*, const cera_hip_tensor* gate, const cera_hip_tensor* up,
                                                  const float* x, uint64_t n, int8_t* quants, float* scales, int* fused);

/* The same, and halves[n][m] (uint16) receive the quants once more in the form the batched Q6_K GEMM
 * reads its activations: IEEE half words of the integer values, the four of every group of four in
 * the order 0, 2, 1, 3 (n * m a multiple of 16).  The forward pass takes them straight from the
 * epilogue of a Q4_K gate | up launch when the down projection is Q6_K (the Q4_K_M mix) instead of
 * converting the quants in a launch of its own; every other route converts afterwards, and both
 * give the same words.  No counterpart in the reference, whose CPU kernels read the int8 quants
 * directly (cera/src/model/transformer.rs:865-946). */
CERA_HIP_API cera_hip_status cera_hip_gemm_swiglu_f16(cera_hip_ctx*, const cera_hip_tensor* gate, const cera_hip_tensor* up,
                                                      const float* x, uint64_t n, int8_t* quants, float* scales,
                                                      uint16_t* halves, int* fused);

/* transformer::decode_attention (cera/src/model/transformer.rs:1249-1305) with
 * cpu::attn_scores / softmax_inplace / attn_values (cera/src/backend/cpu.rs:
 * 3222-3363, 2617-2633).  q f32[n_heads*head_dim]; k, v f32 time-major
 * [seq_len][n_kv_heads*head_dim] (cera/src/kv_cache.rs:201-212);
 * out f32[n_heads*head_dim]; all seq_len positions visible.
 * n_splits = 0 lets the library choose the split-K factor.
 * n_heads a multiple of n_kv_heads.  The tuned kernels cover head_dim 64 and 128 with up to 8
 * query heads per kv head (any count: 28 / 4 and 12 / 2 included); every other head_dim that is
 * a multiple of 8 up to 256, and larger groups, run one launch per query of a generic kernel
 * (the reference takes any shape: transformer.rs:1249-1305, cpu.rs:7075-7088) -- correct, not
 * tuned, n_splits ignored.  Anything else is CERA_HIP_ERR_SHAPE.  The same holds for every
 * attention entry below except the fused decode step and the allocation-free entry, which take
 * the tuned shapes only. */
CERA_HIP_API cera_hip_status cera_hip_attn_decode(cera_hip_ctx*, const float* q, const float* k, const float* v,
                                                  uint32_t n_heads, uint32_t n_kv_heads, uint32_t head_dim,
                                                  uint64_t seq_len, float scale, uint32_t n_splits, float* out);

/* Causal attention of a batch of n_queries new tokens, the attention step of
 * LlamaModel::forward_prefill_batched (cera/src/model/llama.rs:845-1010; flash route
 * cera/src/backend/cpu.rs:4028-4241, per-query route transformer.rs:1249-1305).
 * q f32 [n_queries][n_heads*head_dim]; k, v f32 time-major [start_pos + n_queries][n_kv_heads*head_dim]
 * already containing the batch's own keys/values; query i sees positions 0 .. start_pos + i.
 * out f32 [n_queries][n_heads*head_dim]. */
CERA_HIP_API cera_hip_status cera_hip_attn_prefill(cera_hip_ctx*, const float* q, const float* k, const float* v,
                                                   uint32_t n_heads, uint32_t n_kv_heads, uint32_t head_dim,
                                                   uint64_t start_pos, uint32_t n_queries, float scale, float* out);

/* The same two operations over an f16 KV cache (KvCompression::F16; the kernels
 * cpu::attn_scores_f16 / attn_values_f16 widen on read, cera/src/model/transformer.rs:1170-1196):
 * k and v arrive as f32 in the layout above and are narrowed to IEEE half (round to nearest
 * even, as the cache append does, transformer.rs:1435-1446) before the upload.  n_queries = 1 is
 * the decode step with start_pos + 1 visible keys; n_splits as in cera_hip_attn_decode. */
CERA_HIP_API cera_hip_status cera_hip_attn_f16kv(cera_hip_ctx*, const float* q, const float* k, const float* v,
                                                 uint32_t n_heads, uint32_t n_kv_heads, uint32_t head_dim,
                                                 uint64_t start_pos, uint32_t n_queries, float scale,
                                                 uint32_t n_splits, float* out);

/* cpu::rmsnorm (cera/src/backend/cpu.rs:2479-2496), out of place: y = x*inv_rms*w. */
CERA_HIP_API cera_hip_status cera_hip_rmsnorm(cera_hip_ctx*, const float* x, const float* weight, uint64_t n,
                                              float eps, float* y);
/* cpu::silu_mul_inplace (cera/src/backend/cpu.rs:2570-2575): out = silu(gate)*up. */
CERA_HIP_API cera_hip_status cera_hip_silu_mul(cera_hip_ctx*, const float* gate, const float* up, uint64_t n,
                                               float* out);
/* cpu::rope / cpu::rope_norm (cera/src/backend/cpu.rs:5008-5180), in place on
 * host copies of q [n_heads*head_dim] and k [n_kv_heads*head_dim]. */
CERA_HIP_API cera_hip_status cera_hip_rope(cera_hip_ctx*, float* q, float* k, uint32_t pos, uint32_t n_heads,
                                           uint32_t n_kv_heads, uint32_t head_dim, float freq_base,
                                           uint32_t rope_type, const float* freq_factors);
/* sampler::argmax (cera/src/sampler.rs:20-30). */
CERA_HIP_API cera_hip_status cera_hip_argmax(cera_hip_ctx*, const float* logits, uint64_t n, uint32_t* index);
/* transformer::dequantize_row_into (cera/src/model/transformer.rs:949-1017). */
CERA_HIP_API cera_hip_status cera_hip_dequantize_row(cera_hip_ctx*, const cera_hip_tensor* w, uint64_t row,
                                                     float* out);

/* ---- the decode step's fused kernels, host buffers (parity tests) -------- */
/* cpu::rmsnorm followed by quantize_f32_to_q8_0 of its result (cera/src/backend/cpu.rs:2479-2496,
 * 942-958), as ONE launch: what the decode step runs before the Q/K/V and gate/up projections.
 * n % 32 == 0.  y f32[n], scales f32[n/32], quants i8[n]. */
CERA_HIP_API cera_hip_status cera_hip_rmsnorm_q8_0(cera_hip_ctx*, const float* x, const float* weight, uint64_t n,
                                                   float eps, float* y, float* scales, int8_t* quants);
/* The attention step of one decode layer exactly as the model's decode step issues it
 * (transformer::forward_attn_block from the RoPE on, cera/src/model/transformer.rs:1399-1470, with
 * cpu::rope / rope_norm, cera/src/backend/cpu.rs:5008-5180, and decode_attention,
 * transformer.rs:1249-1305): q [n_heads*head_dim] and k_new [n_kv_heads*head_dim] arrive unrotated,
 * v_new [n_kv_heads*head_dim]; k_cache / v_cache hold positions [0, pos) time-major
 * [pos][n_kv_heads*head_dim] f32 (narrowed to half first when kv_type is CERA_HIP_KV_F16).  Below
 * 1024 keys one attention launch rotates q, rotates and appends the new K/V rows and attends;
 * beyond, a RoPE/append launch precedes it.  Returns the attention output out [n_heads*head_dim],
 * its Q8_0 quantization (the O projection's input, written by the merge kernel) and the rows the
 * step appended to the cache at `pos` (k_row rotated; widened exactly from a half cache). */
CERA_HIP_API cera_hip_status cera_hip_attn_decode_step(cera_hip_ctx*, const float* q, const float* k_new,
                                                       const float* v_new, const float* k_cache, const float* v_cache,
                                                       uint32_t n_heads, uint32_t n_kv_heads, uint32_t head_dim,
                                                       uint32_t pos, float rope_base, uint32_t rope_type,
                                                       const float* freq_factors, float scale, uint32_t kv_type,
                                                       float* out, float* out_scales, int8_t* out_quants, float* k_row,
                                                       float* v_row);

/* The two fused launches of the decode step, for parity tests.  gate | up: cpu::rmsnorm(x, norm_w),
 * its Q8_0 quantization, the two projections of transformer::forward_ffn_block
 * (cera/src/model/transformer.rs:1541), cpu::silu_mul_inplace (cera/src/backend/cpu.rs:2570-2575)
 * and the Q8_0 quantization of the result for the down projection (cpu.rs:942-958) in ONE launch:
 * quants i8[m], scales f32[m/32].  Two Q4_K matrices of one shape, k <= 8192 in whole
 * 256-element super-blocks (or two Q4_0 / Q4_1 / Q8_0 matrices, k <= 4096), m a multiple of 32; anything else is CERA_HIP_ERR_UNSUPPORTED_DTYPE
 * (the decode step then issues the separate launches). */
CERA_HIP_API cera_hip_status cera_hip_ffn_gate_up_fused(cera_hip_ctx*, const cera_hip_tensor* gate,
                                                        const cera_hip_tensor* up, const float* x, const float* norm_w,
                                                        float eps, int8_t* quants, float* scales);
/* q | k | v: cpu::rmsnorm(x, norm_w), its Q8_0 quantization and the projections of
 * transformer::forward_attn_block (cera/src/model/transformer.rs:1340-1373) in one launch:
 * ya = A . n, yb = B . n (b / yb nullable).  Q4_K or Q6_K matrices with k <= 8192 in whole
 * super-blocks, or two matrices of one 32-weight-block type with k <= 4096. */
CERA_HIP_API cera_hip_status cera_hip_qkv_fused(cera_hip_ctx*, const cera_hip_tensor* a, const cera_hip_tensor* b,
                                                const float* x, const float* norm_w, float eps, float* ya, float* yb);

/* ---- reference-order verification route (never the default, never timed) -- */
/* The same three operations with every f32 operation performed exactly as the CPU AVX2 path
 * performs it, in its order, so the results are bit-identical to that path (not merely within
 * the float tolerance): gemm_q4_k_q8_0 / gemm_q6_k_q8_0 at n == 1 with their eight-lane
 * four-accumulator FMA chains, tree add and hsum256_ps (cera/src/backend/simd.rs:5742-5795,
 * 6025-6093, 4546-4554), row_dot_q4_0 / row_dot_q8_0 (:4593-4637), gemm_q4_1_q8_0 (:5893-5976);
 * attn_scores / softmax_inplace / attn_values of the AVX2 tier (cera/src/backend/cpu.rs:3503-3589,
 * 2617-2633); cpu::rmsnorm with its serial f64 sum (:2479-2496).  A Q5_K matrix is dotted with the
 * f32 activations themselves in the scalar order of vec_dot_q5_k_f32_scalar (cera/src/quant.rs:892-937,
 * cera/src/backend/cpu.rs:1830-1854): per 64-weight pair four sequential 32-step chains with
 * separate multiply and add.  Arguments as the fast entry points of the same name. */
CERA_HIP_API cera_hip_status cera_hip_gemv_reference_order(cera_hip_ctx*, const cera_hip_tensor* w, const float* x,
                                                           float* y);
CERA_HIP_API cera_hip_status cera_hip_attn_decode_reference_order(cera_hip_ctx*, const float* q, const float* k,
                                                                  const float* v, uint32_t n_heads, uint32_t n_kv_heads,
                                                                  uint32_t head_dim, uint64_t seq_len, float scale,
                                                                  float* out);
CERA_HIP_API cera_hip_status cera_hip_rmsnorm_reference_order(cera_hip_ctx*, const float* x, const float* weight,
                                                              uint64_t n, float eps, float* y);
/* The batched prefill's two kernels in the order of an x86 host (transformer::gemm_preq,
 * cera/src/model/transformer.rs:710-788): out[m][n] = W . Q8_0(x[n][k]) with every element's f32
 * chain that of gemm_q4_k_8x8_q8_0 / gemm_q4_0_8x8_q8_0 (cera/src/backend/simd.rs:5392-5518,
 * 5215-5366) for a weight cera repacks at load (x86_repack != 0, m % 8 == 0), of the KQ_COLS-tiled
 * K-quant kernels (:5796-5851, :6094-6168) and the strip kernels otherwise; and
 * flash_attention_gqa_avx2 (cera/src/backend/cpu.rs:4261-4412) for n_queries queries at positions
 * start_pos .., q / out [n_queries][n_heads * head_dim], k / v time-major
 * [start_pos + n_queries][n_kv_heads * head_dim].  Bit-identical to the CPU kernels. */
CERA_HIP_API cera_hip_status cera_hip_gemm_reference_order(cera_hip_ctx*, const cera_hip_tensor* w, const float* x, uint64_t n,
                                                           uint32_t x86_repack, float* out);
CERA_HIP_API cera_hip_status cera_hip_flash_attn_reference_order(cera_hip_ctx*, const float* q, const float* k,
                                                                 const float* v, uint32_t n_queries, uint32_t n_heads,
                                                                 uint32_t n_kv_heads, uint32_t head_dim, uint32_t start_pos,
                                                                 float scale, float* out);

/* ---- kernel-level entry points, device buffers (timing) ----------------- */
CERA_HIP_API cera_hip_status cera_hip_quantize_q8_0_dev(cera_hip_ctx*, const float* x, uint64_t k, float* scales,
                                                        int8_t* quants);
/* int8 GEMV on already-quantized activations (transformer::gemv_preq shape,
 * cera/src/model/transformer.rs:455-533): y[m] = W . (xs, xq). */
CERA_HIP_API cera_hip_status cera_hip_gemv_q8_dev(cera_hip_ctx*, const cera_hip_dtensor* w, const float* xs,
                                                  const int8_t* xq, float* y);
typedef struct {
    const cera_hip_dtensor* w;
    const cera_hip_dtensor* w2; /* nullable; when set (same type and shape as w) the launch is
                                   the fused FFN pair: y = silu(w.x) * (w2.x), the gate/up step of
                                   transformer::forward_ffn_block (cera/src/model/transformer.rs:1541) */
    const float* xs;  /* dev f32[k/32] */
    const int8_t* xq; /* dev i8[k]     */
    float* y;         /* dev f32[m]    */
} cera_hip_gemv_op;
/* Launches ops[0..n) back to back on the context's stream (one decode token's
 * worth of GEMVs without per-call host overhead). */
CERA_HIP_API cera_hip_status cera_hip_gemv_seq_dev(cera_hip_ctx*, const cera_hip_gemv_op* ops, uint32_t n);
/* One decode token's projection launches on device-resident operands, issued back to back on the
 * context's stream exactly as cera_hip_forward issues them (benchmarks and profiling; the
 * operations are those of LlamaModel::forward, cera/src/model/llama.rs:468-597):
 *   CERA_HIP_OP_GEMV           y = w . (xs, xq) [+ resid]                  (O and down projections, head)
 *   CERA_HIP_OP_NORM_GEMV      y = w . Q8_0(rmsnorm(x, norm_w)), y2 = w2 . same (w2 / y2 nullable)
 *                              (the Q|K|V launch; refused with CERA_HIP_ERR_UNSUPPORTED_DTYPE where
 *                              cera_hip_qkv_fused is)
 *   CERA_HIP_OP_NORM_GATE_UP   (out_q, out_s) = Q8_0(silu(w . n) * (w2 . n)), n = Q8_0(rmsnorm(x, norm_w))
 *   CERA_HIP_OP_NORM_QUANT     y = rmsnorm(x, norm_w), (out_q, out_s) = Q8_0(y), n elements (before the head)
 *   CERA_HIP_OP_QUANT          (out_q, out_s) = Q8_0(x), n elements (quantize_f32_to_q8_0,
 *                              cera/src/backend/cpu.rs:942-958)
 * All pointers are device pointers; fields an op does not use are ignored.  With decode copies on
 * (cera_hip_ctx_set_decode_copies), a matrix's first use here allocates and builds its copy, as
 * cera_hip_model_create does for a model's: time the second call, not the first. */
enum { CERA_HIP_OP_GEMV = 0, CERA_HIP_OP_NORM_GEMV = 1, CERA_HIP_OP_NORM_GATE_UP = 2, CERA_HIP_OP_NORM_QUANT = 3,
       CERA_HIP_OP_QUANT = 4 };
typedef struct {
    uint32_t kind;
    uint32_t n;               /* NORM_QUANT / QUANT: element count (multiple of 32) */
    const cera_hip_dtensor* w;
    const cera_hip_dtensor* w2;
    const float* x;           /* f32 input of the NORM_* and QUANT kinds */
    const float* norm_w;
    float eps;
    const float* xs;          /* GEMV: Q8_0 scales f32[k/32] */
    const int8_t* xq;         /* GEMV: Q8_0 quants i8[k] */
    const float* resid;       /* GEMV: nullable residual f32[m] */
    float* y;
    float* y2;
    float* out_s;
    int8_t* out_q;
} cera_hip_decode_op;
CERA_HIP_API cera_hip_status cera_hip_decode_ops_dev(cera_hip_ctx*, const cera_hip_decode_op* ops, uint32_t n);
CERA_HIP_API cera_hip_status cera_hip_attn_decode_dev(cera_hip_ctx*, const float* q, const float* k_headmajor,
                                                      const float* v_headmajor, uint32_t n_heads,
                                                      uint32_t n_kv_heads, uint32_t head_dim, uint64_t seq_len,
                                                      uint64_t max_seq, float scale, uint32_t n_splits, float* out);
/* cera_hip_attn_decode_dev for callers that cannot allocate device memory (code under HIP graph
 * capture, tight serving loops, harnesses that forbid it).  No counterpart in the reference.  The
 * split-K partials go to a fixed CERA_HIP_NOALLOC_WORKSPACE_BYTES array inside the library (one
 * per GPU, held until the process ends) instead of the context's grow-on-demand workspace, and
 * the call allocates and frees nothing.  Same arguments and the same result, bit for bit, as
 * cera_hip_attn_decode_dev.  A shape whose partials do not fit -- n_heads * parts * head_dim * 4
 * bytes beyond the array less 128 KiB, parts being n_splits or the library's choice (about
 * 4 * CUs / n_kv_heads, at most one per 8 keys) -- is CERA_HIP_ERR_SHAPE.  Every call on a GPU
 * shares that GPU's array: calls that overlap on one GPU (two contexts, two streams) race. */
#define CERA_HIP_NOALLOC_WORKSPACE_BYTES (4u << 20)
CERA_HIP_API cera_hip_status cera_hip_attn_decode_dev_noalloc(cera_hip_ctx*, const float* q, const float* k_headmajor,
                                                              const float* v_headmajor, uint32_t n_heads,
                                                              uint32_t n_kv_heads, uint32_t head_dim, uint64_t seq_len,
                                                              uint64_t max_seq, float scale, uint32_t n_splits,
                                                              float* out);
/* k, v: device, head-major IEEE half [n_kv_heads][max_seq][head_dim] */
CERA_HIP_API cera_hip_status cera_hip_attn_decode_f16_dev(cera_hip_ctx*, const float* q, const void* k_headmajor_f16,
                                                          const void* v_headmajor_f16, uint32_t n_heads,
                                                          uint32_t n_kv_heads, uint32_t head_dim, uint64_t seq_len,
                                                          uint64_t max_seq, float scale, uint32_t n_splits,
                                                          float* out);
/* out[m][n] = W . quantize(x[n][k]) with x, out on the device. */
CERA_HIP_API cera_hip_status cera_hip_gemm_dev(cera_hip_ctx*, const cera_hip_dtensor* w, const float* x, uint64_t n,
                                               float* out);

/* ---- model level: the `Model` trait surface ------------------------------ */

/* load_model_gpu-style construction from resolved weights
 * (cera/src/model/mod.rs:672-703; cera/src/model/llama.rs:158-450).  Host
 * pointers are borrowed for the call only; everything is copied to HBM. */
CERA_HIP_API cera_hip_status cera_hip_model_create(cera_hip_ctx*, const cera_hip_config*,
                                                   const cera_hip_tensor* token_embd,
                                                   const cera_hip_tensor* output /* nullable => tied */,
                                                   const float* output_norm, const cera_hip_layer* layers,
                                                   cera_hip_model** out);
CERA_HIP_API void cera_hip_model_destroy(cera_hip_model*);
/* Model::forward (cera/src/model/mod.rs:200-606; LlamaModel::forward,
 * cera/src/model/llama.rs:1585-1605): one token at `pos` -> vocab logits.
 * pos must equal cera_hip_seq_len, except that pos == 0 always starts a fresh sequence (the
 * device-side counter is reset, as the reference's device-resident backends do when a caller
 * arrives with a new InferenceState, cera/src/model/metal_lfm2.rs:4091-4096); the same holds
 * for start_pos of the prefill calls. */
CERA_HIP_API cera_hip_status cera_hip_forward(cera_hip_model*, uint32_t token, uint32_t pos, float* logits);
/* Model::forward_greedy (cera/src/model/mod.rs:494-497): forward + argmax on
 * the device, 4-byte readback. */
CERA_HIP_API cera_hip_status cera_hip_forward_greedy(cera_hip_model*, uint32_t token, uint32_t pos, uint32_t* next);
/* Model::forward_prefill (cera/src/model/llama.rs:1607-1649): n tokens from
 * start_pos, logits of the last one. */
CERA_HIP_API cera_hip_status cera_hip_forward_prefill(cera_hip_model*, const uint32_t* tokens, uint32_t n,
                                                      uint32_t start_pos, float* last_logits);
/* Model::forward_prefill_logits_all (cera/src/model/llama.rs:1655-1722; the projection is
 * project_logits_batched, :645-722): like forward_prefill, but returns the logits of EVERY
 * position, row-major [n][vocab] -- the verification primitive of speculative decoding
 * (cera/src/model/mod.rs:221-249).  The LM head is read once for all n positions. */
CERA_HIP_API cera_hip_status cera_hip_forward_prefill_logits_all(cera_hip_model*, const uint32_t* tokens, uint32_t n,
                                                                 uint32_t start_pos, float* logits_all);
/* Model::configure_kv_compression for KvCompression::None / ::F16 (cera/src/model/mod.rs:557-592,
 * cera/src/kv_cache.rs:88-98; f16_kv_supported, mod.rs:594-603): an f16 cache stores K and V as
 * IEEE half (round to nearest even on append, exact widening on read, f32 accumulation --
 * cera/src/model/transformer.rs:1424-1447, 1170-1196), halving the bytes decode attention
 * streams.  Call before the first forward pass: the first call wins, the same mode again is a
 * no-op, a different mode is CERA_HIP_ERR_ARGUMENT, a non-empty cache CERA_HIP_ERR_POSITION. */
#define CERA_HIP_KV_F32 0u
#define CERA_HIP_KV_F16 1u
CERA_HIP_API cera_hip_status cera_hip_configure_kv(cera_hip_model*, uint32_t kv_type);
CERA_HIP_API uint32_t cera_hip_kv_type(const cera_hip_model*);
/* Switches a model to the reference-order verification route (on != 0) or back: forward,
 * forward_greedy and forward_prefill then run LlamaModel::forward's operations one by one
 * (cera/src/model/llama.rs:468-597, 1585-1649) on the reference-order kernels above, and logits
 * are bit-identical to the CPU AVX2 path's -- the harness of
 * cera/tests/gpu_transformer_parity.rs:75-103 then sees the identical greedy token stream.
 *   CERA_HIP_REF_ORDER_PER_TOKEN   forward_prefill runs token by token (llama.rs:1643-1648);
 *   CERA_HIP_REF_ORDER_X86_BATCHED a prompt of more than one token takes
 *       LlamaModel::forward_prefill_batched as an x86 host runs it (llama.rs:1639-1641, 738-1523):
 *       quantize_columns, the repacked gemm_q4_k_8x8_q8_0 / gemm_q4_0_8x8_q8_0 for the weights
 *       cera repacks at load and the tiled kernels for the rest (cera/src/backend/simd.rs:5392-5518,
 *       5215-5366, 5796-5851, 6094-6168), flash_attention_gqa_avx2 from 256 tokens on
 *       (cera/src/backend/cpu.rs:4261-4412), per-token attention below; one call = one batch, as
 *       one call of the reference is (callers split prompts at their ubatch).
 *       A model with a Q5_K layer projection prefills token by token in this mode too: the
 *       reference's batched route hands such a model to its per-token path (llama.rs:762-795).
 * Many times slower than the default route; meant for verification only.  Only with an
 * empty cache (CERA_HIP_ERR_POSITION otherwise). */
#define CERA_HIP_REF_ORDER_OFF 0u
#define CERA_HIP_REF_ORDER_PER_TOKEN 1u
#define CERA_HIP_REF_ORDER_X86_BATCHED 2u
CERA_HIP_API cera_hip_status cera_hip_set_reference_order(cera_hip_model*, uint32_t on);
CERA_HIP_API uint32_t cera_hip_reference_order(const cera_hip_model*);
/* Model::truncate_kv (cera/src/model/mod.rs:251-283). */
CERA_HIP_API cera_hip_status cera_hip_truncate_kv(cera_hip_model*, uint32_t len);
CERA_HIP_API uint32_t cera_hip_seq_len(const cera_hip_model*);
/* Model::gpu_memory_bytes. */
CERA_HIP_API uint64_t cera_hip_memory_bytes(const cera_hip_model*);
/* Frees every decode copy of the model (second line of defence of the rule above: the library
 * calls this itself and retries once when a prefill buffer does not fit).  Decode then reads the
 * native bytes, with bit-identical results; *freed_bytes (nullable) receives what was given back,
 * and cera_hip_memory_bytes drops by as much.  The copies are not rebuilt. */
CERA_HIP_API cera_hip_status cera_hip_drop_decode_copies(cera_hip_model*, uint64_t* freed_bytes);
/* Model::shift_kv for a RoPE model (cera/src/model/llama.rs:1727-1738 ->
 * InferenceState::shift_kv_with_rope, cera/src/kv_cache.rs:1091-1310): drops cache cells
 * [n_keep, n_keep + shift), moves the tail down and re-rotates its K rows by R(-shift)
 * (cera/src/backend/cpu.rs:5065-5086, 5145-5180); V rows only move.  seq_len -= shift.
 * shift == 0 -> CERA_HIP_ERR_ARGUMENT, n_keep + shift > seq_len -> CERA_HIP_ERR_POSITION
 * (the reference asserts both). */
CERA_HIP_API cera_hip_status cera_hip_shift_kv(cera_hip_model*, uint32_t n_keep, uint32_t shift);
/* Model::snapshot_state, one layer (cera/src/model/mod.rs:507-524; LayerSnapshot::Attention,
 * cera/src/kv_cache.rs:1382-1396): K and V cache rows [0, seq_len) to host in the reference's
 * time-major [pos][kv_dim] f32 order.  Also the parity tests' view of the cache. */
CERA_HIP_API cera_hip_status cera_hip_read_kv(cera_hip_model*, uint32_t layer, float* k_out, float* v_out);
/* Model::restore_state, one layer (cera/src/model/mod.rs:526-533): the inverse of
 * cera_hip_read_kv for rows [0, n_pos).  After the last layer call cera_hip_set_seq_len(n_pos),
 * which "sets internal seq_len" as the trait method does. */
CERA_HIP_API cera_hip_status cera_hip_write_kv(cera_hip_model*, uint32_t layer, const float* k, const float* v,
                                               uint32_t n_pos);
CERA_HIP_API cera_hip_status cera_hip_set_seq_len(cera_hip_model*, uint32_t len);
/* Test hook: final normed hidden state of the last forward (f32[hidden]). */
CERA_HIP_API cera_hip_status cera_hip_read_hidden(cera_hip_model*, float* hidden_out);

#ifdef __cplusplus
}
#endif
#endif /* CERA_HIP_H */
