// The standalone gfx950 code object: the decode GEMV layer's kernels under fixed extern "C" names,
// for hosts that load it with hipModuleLoad and launch with hipModuleLaunchKernel
// (include/cera_hip_kernels.h documents names, argument structs and launch geometry).  Compiled
// with `hipcc --genco`; the bodies are the ones libcera_hip.so instantiates.
#include <cstddef>

#include "cera_hip_kernels.h"
#include "gemv.hip.h"
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
