// Prefill: batched int8 GEMM over Q8_0-quantized activation rows and the
// batched forward pass built on it.
#include "model.h"

cera_hip_status cera_model_prefill(cera_hip_model* m, const uint32_t* tokens, uint32_t n, uint32_t start_pos,
                                   float* last_logits) {
    return cera_model_prefill_per_token(m, tokens, n, start_pos, last_logits);
}

extern "C" cera_hip_status cera_hip_gemm_dev(cera_hip_ctx* ctx, const cera_hip_dtensor* w, const float* x, uint64_t n,
                                             float* out) {
    (void)w; (void)x; (void)n; (void)out;
    return cera_fail(ctx, CERA_HIP_ERR_UNSUPPORTED_DTYPE, "gemm: not built yet");
}
extern "C" cera_hip_status cera_hip_gemm(cera_hip_ctx* ctx, const cera_hip_tensor* w, const float* x, uint64_t n,
                                         float* out) {
    (void)w; (void)x; (void)n; (void)out;
    return cera_fail(ctx, CERA_HIP_ERR_UNSUPPORTED_DTYPE, "gemm: not built yet");
}
