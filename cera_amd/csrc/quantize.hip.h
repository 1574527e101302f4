// Q8_0 dynamic activation quantizer (cera/src/backend/cpu.rs:942-958).
//
// Per 32-element block: amax = max|x| (NaN lanes ignored), d = amax/127,
// id = 1/d unless d == 0 or 1/d is not finite, scale = f16 round trip of d,
// q = clamp(round_half_even(x*id), -128, 127), NaN -> 0.  Every operation is a
// correctly rounded IEEE f32 op, so the output is bit-identical to the CPU's.
//
// Eight lanes own one block (a float4 each): loads and stores are fully
// coalesced, the block maximum is a three-step DPP reduction.
#pragma once
#include "common.hip.h"

__device__ __forceinline__ int q8_round(float v, float id) {
    float r = rintf(__fmul_rn(v, id));  // v_rndne_f32
    // Rust's saturating `as i8` after clamp(-128, 127); NaN -> 0.
    if (r != r) return 0;
    r = fminf(fmaxf(r, -128.0f), 127.0f);
    return static_cast<int>(r);
}

// Quantizes one 32-block spread over 8 consecutive lanes; returns this lane's
// four quants packed little-endian and the block scale (same in all 8 lanes).
__device__ __forceinline__ uint32_t q8_quantize_quad(float4 v, float& scale_out) {
    float amax = fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w)));
    // fmaxf ignores a NaN operand, like f32::max in the reference's fold; a NaN
    // lane must not poison the other lanes, so canonicalise NaN partials to 0.
    if (amax != amax) amax = 0.0f;
    amax = fmaxf(amax, dpp_f<0xB1>(amax));
    amax = fmaxf(amax, dpp_f<0x4E>(amax));
    amax = fmaxf(amax, dpp_f<0x141>(amax));
    float d = __fdiv_rn(amax, 127.0f);
    float r = __fdiv_rn(1.0f, d);
    float id = (d != 0.0f && fabsf(r) != __builtin_inff() && r == r) ? r : 0.0f;
    scale_out = h2f(f2h(d));
    uint32_t q0 = static_cast<uint32_t>(q8_round(v.x, id)) & 0xFF;
    uint32_t q1 = static_cast<uint32_t>(q8_round(v.y, id)) & 0xFF;
    uint32_t q2 = static_cast<uint32_t>(q8_round(v.z, id)) & 0xFF;
    uint32_t q3 = static_cast<uint32_t>(q8_round(v.w, id)) & 0xFF;
    return q0 | (q1 << 8) | (q2 << 16) | (q3 << 24);
}

// scale * (sum of the 32 quants of the block this lane belongs to): the
// activation-side factor of the Q4_K / Q4_1 min terms.  |sum| <= 32*128 and the
// scale has an 11-bit significand, so the product is exact in f32.
__device__ __forceinline__ float q8_block_scaled_sum(uint32_t packed, float scale) {
    int s = sum4(packed, 0);
    s += __builtin_amdgcn_update_dpp(0, s, 0xB1, 0xF, 0xF, true);
    s += __builtin_amdgcn_update_dpp(0, s, 0x4E, 0xF, 0xF, true);
    s += __builtin_amdgcn_update_dpp(0, s, 0x141, 0xF, 0xF, true);
    return scale * static_cast<float>(s);
}

// grid: ceil(k/4 / 256) blocks of 256 threads; thread t owns x[4t .. 4t+3].
// bsum (nullable): per-block scale * sum(quants), consumed by the prefill GEMM.
__device__ __forceinline__ void quantize_q8_0_body(const float* __restrict__ x, uint64_t k, float* __restrict__ scales,
                                                   int8_t* __restrict__ quants, float* __restrict__ bsum) {
    uint64_t t = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    bool live = 4 * t < k;
    // k % 32 == 0, so a whole 8-lane group is live or dead together.
    float4 v = live ? reinterpret_cast<const float4*>(x)[t] : make_float4(0.f, 0.f, 0.f, 0.f);
    float scale;
    uint32_t packed = q8_quantize_quad(v, scale);
    float ssum = bsum ? q8_block_scaled_sum(packed, scale) : 0.0f;
    if (live) {
        reinterpret_cast<uint32_t*>(quants)[t] = packed;
        if ((t & 7) == 0) {
            scales[t >> 3] = scale;
            if (bsum) bsum[t >> 3] = ssum;
        }
    }
}
static __global__ __launch_bounds__(256) void quantize_q8_0_kernel(const float* __restrict__ x, uint64_t k,
                                                            float* __restrict__ scales,
                                                            int8_t* __restrict__ quants,
                                                            float* __restrict__ bsum) {
    quantize_q8_0_body(x, k, scales, quants, bsum);
}
