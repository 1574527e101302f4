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

#ifdef __cplusplus
}
#endif
#endif /* CERA_HIP_KERNELS_H */
