// Q5_K decode GEMV.  cera's CPU path dots Q5_K rows against the *unquantized* f32 activations
// (cera/src/backend/cpu.rs:1830-1854, cera/src/quant.rs:892-937: acc += (d*sc*q - dmin*mn) * x per
// element), so there are no integer block dots here and the bar is the float one.  Same shape as
// the int8 kernels (gemv.hip.h): a lane owns one 64-weight unit of K -- a 32-byte chunk of `qs`,
// i.e. sub-block 2j in the low nibbles and 2j+1 in the high ones, plus the fifth bits of both from
// `qh` -- keeps its 64 f32 activations and their two sub-block sums in registers for the whole
// kernel, and streams weights only; KS wavefronts split longer rows and meet in LDS.  Per unit
//   d * (sc1 * sum q1 x + sc2 * sum q2 x) - dmin * (mn1 * sum x_lo + mn2 * sum x_hi),
// the reference's sum with the block scales factored out (fewer roundings than its per-element
// form: closer to the exact value, well inside 1e-3 * rms).
#include "gemv.hip.h"
#include "host_common.h"

struct Q5KF {
    static constexpr int ELEMS_PER_UNIT = 64;
    struct Act { float x[64]; float s0, s1; };
    struct Wt { uint4 h, qh0, qh1, q0, q1; };
    __device__ static void dbg_asum(const Act&, uint32_t, int32_t*) {}
    // `xs` carries the f32 activations [k]; there is no quantized copy
    __device__ static void load_act(Act& a, const int8_t*, const float* xs, uint32_t u, bool live) {
        const float4* p = reinterpret_cast<const float4*>(xs + u * 64);
        float s0 = 0.0f, s1 = 0.0f;
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            float4 v = p[i];
            if (!live) v = make_float4(0.f, 0.f, 0.f, 0.f);
            a.x[4 * i] = v.x; a.x[4 * i + 1] = v.y; a.x[4 * i + 2] = v.z; a.x[4 * i + 3] = v.w;
            const float t = (v.x + v.y) + (v.z + v.w);
            if (i < 8) s0 += t; else s1 += t;
        }
        a.s0 = s0; a.s1 = s1;
    }
    __device__ static void load_w(Wt& w, const uint8_t* row, uint32_t u) {
        const uint8_t* blk = row + (u >> 2) * 176;
        w.h = ld_u128(blk);
        w.qh0 = ld_u128(blk + 16);
        w.qh1 = ld_u128(blk + 32);
        w.q0 = ld_u128(blk + 48 + (u & 3) * 32);
        w.q1 = ld_u128(blk + 64 + (u & 3) * 32);
    }
    __device__ static float dot(const Wt& w, const Act& a, uint32_t u, int32_t*) {
        const uint32_t g = u & 3;
        // 6-bit scales / mins of sub-blocks 2g, 2g+1 (decode_q4km_scales, cera/src/quant.rs:591)
        const uint32_t sh = 16 * (g & 1);
        const bool low = g < 2;
        const uint32_t sh_a = low ? sh : sh + 2, m_a = low ? 0x3F3Fu : 0x3030u, m_b = low ? 0u : 0x0F0Fu;
        const uint32_t sc2 = ((w.h.y >> sh_a) & m_a) | ((w.h.w >> sh) & m_b);
        const uint32_t mn2 = ((w.h.z >> sh_a) & m_a) | ((w.h.w >> (sh + 4)) & m_b);
        const float d = h2f(w.h.x & 0xFFFF), dmin = h2f(w.h.x >> 16);
        const uint32_t q[8] = {w.q0.x, w.q0.y, w.q0.z, w.q0.w, w.q1.x, w.q1.y, w.q1.z, w.q1.w};
        const uint32_t hb[8] = {w.qh0.x, w.qh0.y, w.qh0.z, w.qh0.w, w.qh1.x, w.qh1.y, w.qh1.z, w.qh1.w};
        float t1 = 0.0f, t2 = 0.0f;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            // bytes l = 4i .. 4i+3: code = nibble + 16 * (bit 2g (low) / 2g+1 (high) of qh[l])
            const uint32_t v1 = (q[i] & 0x0F0F0F0Fu) | (((hb[i] >> (2 * g)) & 0x01010101u) << 4);
            const uint32_t v2 = ((q[i] >> 4) & 0x0F0F0F0Fu) | (((hb[i] >> (2 * g + 1)) & 0x01010101u) << 4);
#pragma unroll
            for (int b = 0; b < 4; ++b) {
                t1 = fmaf(static_cast<float>((v1 >> (8 * b)) & 0xFF), a.x[4 * i + b], t1);
                t2 = fmaf(static_cast<float>((v2 >> (8 * b)) & 0xFF), a.x[32 + 4 * i + b], t2);
            }
        }
        float s = static_cast<float>(sc2 & 0xFF) * t1;
        s = fmaf(static_cast<float>(sc2 >> 8), t2, s);
        float mm = static_cast<float>(mn2 & 0xFF) * a.s0;
        mm = fmaf(static_cast<float>(mn2 >> 8), a.s1, mm);
        return fmaf(d, s, -(dmin * mm));
    }
};

// y = W . x for a Q5_K matrix and f32 x (KS = 1, 2 or 4 wavefronts per row group up to k = 16384).
cera_hip_status cera_launch_gemv_q5k_f32(cera_hip_ctx* ctx, const cera_hip_dtensor* w, const float* x, float* y) {
    if (w->k % 256 || w->k == 0) return cera_fail(ctx, CERA_HIP_ERR_SHAPE, "Q5_K gemv: k must be a multiple of 256");
    if (w->k > 16384) {   // longer rows than four wavefronts of units: the one-wavefront-per-row loop over blocks
        hipLaunchKernelGGL(gemv_q5k_f32_kernel, dim3(static_cast<uint32_t>((w->m + 3) / 4)), dim3(256), 0, ctx->stream, w->dev, x, y,
                           static_cast<uint32_t>(w->m), static_cast<uint32_t>(w->k));
        HIP_TRY(ctx, hipGetLastError());
        return CERA_HIP_OK;
    }
    GemvArgs a{};
    a.w = w->dev; a.xs = x; a.y = y;
    a.m = static_cast<uint32_t>(w->m);
    a.n_units = static_cast<uint32_t>(w->k / 64);
    a.row_bytes = static_cast<uint32_t>(w->row_bytes);
    const uint32_t ks = a.n_units <= 64 ? 1 : (a.n_units <= 128 ? 2 : 4);
    // about 4 wavefronts per CU: a wavefront's 64 f32 activations per lane are 16 KB from L2, so it
    // has to own several rows to pay for them (16 per CU: 318 tok/s on a Q5_K_M-style 8B model, 8: 359,
    // 4: 377, 2: 330); two rows in flight per workgroup step where there are rows enough
    const uint32_t target_blocks = std::max(1u, ctx->n_cu * 4 / ks);
    uint32_t rpb = (a.m + target_blocks - 1) / target_blocks;
    const int rb = rpb >= 2 ? 2 : 1;
    rpb = (rpb + rb - 1) / rb * rb;
    a.rows_per_wave = rpb;
    const dim3 grid((a.m + rpb - 1) / rpb), block(64 * ks);
#define Q5K_LAUNCH(KS_)                                                                                             \
    do {                                                                                                            \
        if (rb == 2) hipLaunchKernelGGL((gemv_kernel<Q5KF, 1, KS_, 2, EPI_STORE, false>), grid, block, 0, ctx->stream, a); \
        else hipLaunchKernelGGL((gemv_kernel<Q5KF, 1, KS_, 1, EPI_STORE, false>), grid, block, 0, ctx->stream, a);    \
    } while (0)
    if (ks == 1) Q5K_LAUNCH(1);
    else if (ks == 2) Q5K_LAUNCH(2);
    else Q5K_LAUNCH(4);
#undef Q5K_LAUNCH
    HIP_TRY(ctx, hipGetLastError());
    return CERA_HIP_OK;
}
