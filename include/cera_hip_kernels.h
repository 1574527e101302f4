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

#ifdef __cplusplus
}
#endif
#endif /* CERA_HIP_KERNELS_H */
