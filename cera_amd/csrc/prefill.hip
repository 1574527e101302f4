// Prefill: batched int8-MFMA GEMM over Q8_0-quantized activation rows
// (transformer::gemm_preq over quantize_columns, cera/src/model/transformer.rs:
// 710-788, 865-946) and the batched forward pass built on it
// (LlamaModel::forward_prefill_batched, cera/src/model/llama.rs:738-1523).
#include <cmath>
#include <cstring>

#include "copy_budget.h"
#include "gemm_q5k_f16.hip.h"
#include "gemm_q6k_f16.hip.h"
#include "gemm_fp8.hip.h"
#include "glue.hip.h"
#include "model.h"

static bool gemm_type_ok(uint32_t t) {
    return t == CERA_HIP_Q4_0 || t == CERA_HIP_Q4_1 || t == CERA_HIP_Q8_0 || t == CERA_HIP_Q4_K || t == CERA_HIP_Q6_K;
}

// batched_gemm_supports (cera/src/model/transformer.rs:536-565): the int8 GEMM
// takes K in whole 256-element steps.
bool cera_gemm_supports(uint32_t dtype, uint64_t k) { return gemm_type_ok(dtype) && k % GEMM_KSUPER == 0 && k > 0; }
// Q5_K has a batched kernel of its own that reads the f32 activations (gemm_q5k_f16.hip.h), as its
// GEMV does: the reference never quantizes the input of a Q5_K projection (cera/src/backend/cpu.rs:1830-1854).
static bool gemm_f32_supports(uint32_t dtype, uint64_t k) { return dtype == CERA_HIP_Q5_K && k % GEMM_KSUPER == 0 && k > 0; }
static bool gemm_batched(uint32_t dtype, uint64_t k) { return cera_gemm_supports(dtype, k) || gemm_f32_supports(dtype, k); }

// bytes of the fragment-ordered fp8 split copy of n activation rows of k elements
static_assert(G8_BN == 64 && G8_REC == 21504, "cera_fp8_split_bytes (copy_budget.h) restates this record geometry");
uint64_t cera_gemm_fp8_ws_bytes(uint64_t n, uint64_t k) { return cera_fp8_split_bytes(n, k); }

// out[i*ld_m + j*ld_n] = (W . B)[i][j] (+ resid)
// w2 / out2 (nullable): a second matrix of the same type and k multiplied by the same activations
// in the same launch, out2[i*ld_m + j*ld_n2]; *paired says whether that happened (if not, the
// caller launches the second matrix on its own)
cera_hip_status cera_launch_gemm(cera_hip_ctx* ctx, const cera_hip_dtensor* w, const float* bs, const int8_t* bq,
                                 const float* bsum, uint32_t n, float* out, uint64_t ld_m, uint64_t ld_n,
                                 const float* resid, float resid_scale, const cera_hip_dtensor* w2 = nullptr,
                                 float* out2 = nullptr, uint64_t ld_n2 = 0, bool* paired = nullptr, void* bh_ws = nullptr,
                                 bool* staged = nullptr, int32_t* dbg_dots = nullptr, const float* x_f32 = nullptr,
                                 bool* staged_f32 = nullptr, void* b8_ws = nullptr, bool* staged8 = nullptr,
                                 RowsPending* pending = nullptr, int part_slot = 9) {
    // pending (nullable): a caller whose next launch can add split-K partial sums itself (the row norm or the
    // RoPE kernel of a prefill); when K is split, the reduction launch is left out and *pending says what to
    // add (n_split = 0: nothing, out is complete).  A pair's partial sums lie side by side: the second
    // matrix's start m * n floats into every slice.  part_slot: the scratch slot the partial sums go to (a
    // caller that keeps two sets pending gives the second one a slot of its own).
    if (pending) *pending = RowsPending{};
    // Q5_K: x_f32 [n][k] are the activations (bs / bq / bsum are not read); *staged_f32 (nullable)
    // says whether the context's split copy still holds exactly these activations
    const bool q5 = gemm_f32_supports(w->dtype, w->k);
    if (!q5 && !cera_gemm_supports(w->dtype, w->k))
        return cera_fail(ctx, CERA_HIP_ERR_UNSUPPORTED_DTYPE,
                         "gemm: no batched kernel for ggml type " + std::to_string(w->dtype) + " with k=" + std::to_string(w->k));
    if (q5 && (!x_f32 || dbg_dots || (reinterpret_cast<uintptr_t>(w->dev) & 15) || (reinterpret_cast<uintptr_t>(x_f32) & 15)))
        return cera_fail(ctx, CERA_HIP_ERR_ARGUMENT, "gemm: a Q5_K matrix takes 16-byte aligned f32 activations and has no integer block dots");
    if (n == 0) return cera_fail(ctx, CERA_HIP_ERR_SHAPE, "gemm: n must be positive");
    GemmArgs a;
    a.w = w->dev; a.bq = bq; a.bs = bs; a.bsum = bsum; a.out = out;
    a.m = static_cast<uint32_t>(w->m); a.n = n; a.k = static_cast<uint32_t>(w->k);
    a.row_bytes = static_cast<uint32_t>(w->row_bytes);
    a.ld_m = ld_m; a.ld_n = ld_n; a.resid = resid; a.resid_scale = resid_scale;
    a.hq = nullptr; a.hs = nullptr; a.hbsum = nullptr; a.hh = nullptr; a.dbg_dots = dbg_dots;
    // Q6_K runs its block dots on the f16 matrix cores and reads the quants as f16: converted here
    // unless the caller says its workspace (bh_ws) still holds these activations (*staged)
    a.bh = nullptr;
    if (w->dtype == CERA_HIP_Q6_K) {
        if (!bh_ws) {
            CERA_TRY(cera_scratch(ctx, 10, static_cast<uint64_t>(n) * a.k * 2, &bh_ws));
            staged = nullptr;
        }
        if (!staged || !*staged) {
            const uint64_t words = static_cast<uint64_t>(n) * a.k / 16;
            hipLaunchKernelGGL(gemm_act_f16_kernel, dim3(static_cast<uint32_t>((words + 255) / 256)), dim3(256), 0,
                               ctx->stream, reinterpret_cast<const uint4*>(bq), static_cast<uint4*>(bh_ws), words);
            if (staged) *staged = true;
        }
        a.bh = bh_ws;
    }
    // Q4_K runs its block dots on the fp8 matrix cores and reads the activations from their
    // fragment-ordered split copy (gemm_fp8.hip.h): built here unless the caller says its workspace
    // (b8_ws) still holds these activations (*staged8)
    const bool fp8 = w->dtype == CERA_HIP_Q4_K;
    a.bf8 = nullptr;
    if (fp8) {
        const uint32_t tiles = (n + G8_BN - 1) / G8_BN * 2, nsb = a.k / 256;
        if (!b8_ws) {
            CERA_TRY(cera_scratch(ctx, 12, cera_gemm_fp8_ws_bytes(n, a.k), &b8_ws));
            staged8 = nullptr;
        }
        if (!staged8 || !*staged8) {
            hipLaunchKernelGGL(gemm_act_fp8_kernel, dim3(tiles * nsb), dim3(256), 0, ctx->stream, bq, bs, bsum,
                               static_cast<uint8_t*>(b8_ws), n, a.k, static_cast<uint4*>(nullptr));
            if (staged8) *staged8 = true;
        }
        a.bf8 = static_cast<const uint8_t*>(b8_ws);
    }
    // Q6_K: 128-token tiles (eight wavefronts) once there is more than one 64-token tile, where they round the
    // token count up by at most a tenth more than 64-token tiles do (down projection of the 8B shapes: 71 -> 62 us
    // at 128 tokens, 243 -> 207 at 512, 828 -> 727 at 2048)
    const bool q6_wide = w->dtype == CERA_HIP_Q6_K && !dbg_dots && n > 64 &&
                         (n + 127) / 128 * 128 * 10 <= (n + 63) / 64 * 64 * 11;
    const uint32_t BM = fp8 ? G8_BM : GEMM_BM, BN = fp8 ? G8_BN : (q6_wide ? 2 * GEMM_BN : GEMM_BN);
    if (q5) {
        // hi | lo f16 halves of x and its f32 block sums, in one scratch allocation
        const uint64_t nk = static_cast<uint64_t>(n) * a.k;
        void* ws;
        CERA_TRY(cera_scratch(ctx, 11, nk * 4 + nk / 32 * 4 + static_cast<uint64_t>(n) * 4, &ws));
        uint8_t* base = static_cast<uint8_t*>(ws);
        float* xsum = reinterpret_cast<float*>(base + nk * 4);
        float* unscale = xsum + nk / 32;   // 2^-e per token
        if (!staged_f32 || !*staged_f32) {
            hipLaunchKernelGGL(gemm_act_split_kernel, dim3(n), dim3(256), 0, ctx->stream, x_f32, reinterpret_cast<uint4*>(base),
                               reinterpret_cast<uint4*>(base + nk * 2), xsum, unscale, a.k);
            if (staged_f32) *staged_f32 = true;
        }
        a.bh = base;
        a.bq = reinterpret_cast<const int8_t*>(base + nk * 2);
        a.bs = unscale;
        a.bsum = xsum;
    }
    dim3 grid((n + BN - 1) / BN, (a.m + BM - 1) / BM);
    a.w2 = nullptr; a.out2 = nullptr; a.m2 = 0; a.tiles1 = grid.y; a.ld_n2 = 0;
    if (paired) *paired = false;
    // a pair is taken when both outputs are token-major and dense (what the split-K reduction needs)
    if (w2 && !resid && w2->dtype == w->dtype && w2->k == w->k && w2->row_bytes == w->row_bytes && ld_m == 1 &&
        ld_n == w->m && ld_n2 == w2->m && (w->m * n) % 4 == 0 && (w2->m * n) % 4 == 0) {
        a.w2 = w2->dev; a.out2 = out2; a.m2 = static_cast<uint32_t>(w2->m); a.ld_n2 = ld_n2;
        grid.y += static_cast<uint32_t>((w2->m + BM - 1) / BM);
        if (paired) *paired = true;
    }
    // Few output tiles and a long K (the down projection at a few hundred tokens): split K over
    // grid.z so the chip is filled, partial sums to scratch, then one fixed-order reduction.
    // The outputs must be dense in m*n floats for the elementwise reduction.
    uint32_t split = 1;
    const uint32_t wgs = grid.x * grid.y, nsb = a.k / GEMM_KSUPER;
    const bool dense = (ld_m == 1 && ld_n == a.m) || (ld_n == 1 && ld_m == n);
    const uint32_t per_cu = q6_wide ? 1 : 2;   // workgroups a CU holds at once
    if (!dbg_dots && wgs < per_cu * ctx->n_cu && nsb >= 8 && dense && (static_cast<uint64_t>(a.m) * n) % 4 == 0) {
        // smallest divisor of the super-block count that fills every CU
        const uint32_t want = std::min<uint32_t>(8, (per_cu * ctx->n_cu + wgs - 1) / wgs);
        // (a slice keeps at least two super-blocks: below that the tile's prologue outweighs its K loop)
        for (uint32_t d = 2; d <= 8 && split < want; ++d)
            if (nsb % d == 0 && nsb / d >= 2) split = d;
    }
    a.k_chunk = a.k / split;
    a.part_stride = 0;
    // a pair's partials lie side by side: [split][m*n | m2*n]
    const uint64_t mn = static_cast<uint64_t>(a.m) * n, mn2 = static_cast<uint64_t>(a.m2) * n;
    if (split > 1) {
        void* part;
        CERA_TRY(cera_scratch(ctx, part_slot, split * (mn + mn2) * sizeof(float), &part));
        a.out = static_cast<float*>(part);
        if (a.w2) a.out2 = a.out + mn;
        a.part_stride = mn + mn2;
        a.resid = nullptr;
        grid.z = split;
    }
    if (dbg_dots) {
        // the same kernels, compiled to also store every block's integer tile (no K split, no pair)
        switch (w->dtype) {
            case CERA_HIP_Q4_K: hipLaunchKernelGGL((gemm_q4k_fp8_kernel<false, true>), grid, dim3(256), 0, ctx->stream, a); break;
            case CERA_HIP_Q6_K: hipLaunchKernelGGL(gemm_q6k_f16_kernel<true>, grid, dim3(256), 0, ctx->stream, a); break;
            case CERA_HIP_Q4_0: hipLaunchKernelGGL((gemm_kernel<GemmQ4_0, false, true>), grid, dim3(256), 0, ctx->stream, a); break;
            case CERA_HIP_Q4_1: hipLaunchKernelGGL((gemm_kernel<GemmQ4_1, false, true>), grid, dim3(256), 0, ctx->stream, a); break;
            default: hipLaunchKernelGGL((gemm_kernel<GemmQ8_0, false, true>), grid, dim3(256), 0, ctx->stream, a); break;
        }
        HIP_TRY(ctx, hipGetLastError());
        return CERA_HIP_OK;
    }
    switch (w->dtype) {
        case CERA_HIP_Q4_K: hipLaunchKernelGGL((gemm_q4k_fp8_kernel<false, false>), grid, dim3(256), 0, ctx->stream, a); break;
        case CERA_HIP_Q6_K:
            if (q6_wide) hipLaunchKernelGGL((gemm_q6k_f16_kernel<false, 2>), grid, dim3(512), 0, ctx->stream, a);
            else hipLaunchKernelGGL(gemm_q6k_f16_kernel<false>, grid, dim3(256), 0, ctx->stream, a);
            break;
        case CERA_HIP_Q5_K: hipLaunchKernelGGL(gemm_q5k_f16_kernel, grid, dim3(256), 0, ctx->stream, a); break;
        case CERA_HIP_Q4_0: hipLaunchKernelGGL((gemm_kernel<GemmQ4_0>), grid, dim3(256), 0, ctx->stream, a); break;
        case CERA_HIP_Q4_1: hipLaunchKernelGGL((gemm_kernel<GemmQ4_1>), grid, dim3(256), 0, ctx->stream, a); break;
        default: hipLaunchKernelGGL((gemm_kernel<GemmQ8_0>), grid, dim3(256), 0, ctx->stream, a); break;
    }
    if (split > 1 && pending && ld_m == 1 && ld_n == a.m && (!a.w2 || ld_n2 == a.m2))
        *pending = RowsPending{a.out, split, a.part_stride, resid, resid_scale, out};
    else if (split > 1)   // one launch reduces both matrices of a pair
        hipLaunchKernelGGL(gemm_reduce_kernel, dim3(static_cast<uint32_t>(((mn + mn2) / 4 + 255) / 256)), dim3(256), 0,
                           ctx->stream, a.out, split, a.part_stride, (mn + mn2) / 4, out, resid, resid_scale, mn / 4, out2);
    HIP_TRY(ctx, hipGetLastError());
    return CERA_HIP_OK;
}

// First half of the FFN in one launch: hq/hs/hbsum [n][m] = Q8_0(silu(gate.B) * (up.B)), the
// activation of the down projection, quantized in the GEMM's epilogue.  *fused = false (nothing
// launched) when the pair is not two int8-GEMM matrices of one shape or when the launch would
// need a K split to fill the chip; the caller then takes the GEMM pair and the SwiGLU kernel.
cera_hip_status cera_launch_gemm_swiglu(cera_hip_ctx* ctx, const cera_hip_dtensor* gate, const cera_hip_dtensor* up,
                                        const float* bs, const int8_t* bq, const float* bsum, uint32_t n, int8_t* hq,
                                        float* hs, float* hbsum, bool* fused, void* b8_ws = nullptr, bool* staged8 = nullptr,
                                        void* hh_ws = nullptr) {
    // hh_ws (nullable, Q4_K pairs only): also receives the quants as f16 [n][m] in gemm_act_f16_kernel's order
    *fused = false;
    if (!cera_gemm_supports(gate->dtype, gate->k) || gate->dtype == CERA_HIP_Q6_K || up->dtype != gate->dtype ||
        up->k != gate->k || up->m != gate->m || up->row_bytes != gate->row_bytes || gate->m % 32 || n == 0)
        return CERA_HIP_OK;
    GemmArgs a{};
    a.w = gate->dev; a.w2 = up->dev; a.bq = bq; a.bs = bs; a.bsum = bsum;
    a.m = static_cast<uint32_t>(gate->m); a.n = n; a.k = static_cast<uint32_t>(gate->k);
    a.row_bytes = static_cast<uint32_t>(gate->row_bytes);
    a.k_chunk = a.k;
    a.hq = hq; a.hs = hs; a.hbsum = hbsum;
    const bool fp8 = gate->dtype == CERA_HIP_Q4_K;
    a.hh = fp8 ? static_cast<uint16_t*>(hh_ws) : nullptr;
    const uint32_t BM = fp8 ? G8_BM : GEMM_BM, BN = fp8 ? G8_BN : GEMM_BN;
    const dim3 grid((n + BN - 1) / BN, (a.m + BM / 2 - 1) / (BM / 2));
    if (grid.x * grid.y < 2 * ctx->n_cu) return CERA_HIP_OK;
    if (fp8) {
        if (!b8_ws) {
            CERA_TRY(cera_scratch(ctx, 12, cera_gemm_fp8_ws_bytes(n, a.k), &b8_ws));
            staged8 = nullptr;
        }
        if (!staged8 || !*staged8) {
            hipLaunchKernelGGL(gemm_act_fp8_kernel, dim3((n + G8_BN - 1) / G8_BN * 2 * (a.k / 256)), dim3(256), 0, ctx->stream, bq, bs,
                               bsum, static_cast<uint8_t*>(b8_ws), n, a.k, static_cast<uint4*>(nullptr));
            if (staged8) *staged8 = true;
        }
        a.bf8 = static_cast<const uint8_t*>(b8_ws);
    }
    switch (gate->dtype) {
        case CERA_HIP_Q4_K: hipLaunchKernelGGL((gemm_q4k_fp8_kernel<true, false>), grid, dim3(256), 0, ctx->stream, a); break;
        case CERA_HIP_Q4_0: hipLaunchKernelGGL((gemm_kernel<GemmQ4_0, true>), grid, dim3(256), 0, ctx->stream, a); break;
        case CERA_HIP_Q4_1: hipLaunchKernelGGL((gemm_kernel<GemmQ4_1, true>), grid, dim3(256), 0, ctx->stream, a); break;
        default: hipLaunchKernelGGL((gemm_kernel<GemmQ8_0, true>), grid, dim3(256), 0, ctx->stream, a); break;
    }
    HIP_TRY(ctx, hipGetLastError());
    *fused = true;
    return CERA_HIP_OK;
}

// quantize n rows of k floats: quants [n][k], scales and bsum [n][k/32]
static cera_hip_status quantize_rows(cera_hip_ctx* ctx, const float* x, uint64_t n, uint64_t k, float* scales,
                                     int8_t* quants, float* bsum) {
    return cera_launch_quantize(ctx, x, n * k, scales, quants, bsum);
}

extern "C" cera_hip_status cera_hip_gemm_dev(cera_hip_ctx* ctx, const cera_hip_dtensor* w, const float* x, uint64_t n,
                                             float* out) {
    if (!ctx || !w || !x || !out) return CERA_HIP_ERR_ARGUMENT;
    std::lock_guard<std::recursive_mutex> op_lk(ctx->op_mu);
    if (n == 0 || n > 0x7FFFFFFFull) return cera_fail(ctx, CERA_HIP_ERR_SHAPE, "gemm: bad n");
    if (gemm_f32_supports(w->dtype, w->k))   // f32 activations, no quantization (the reference's Q5_K semantics)
        return cera_launch_gemm(ctx, w, nullptr, nullptr, nullptr, static_cast<uint32_t>(n), out, n, 1, nullptr, 1.0f, nullptr,
                                nullptr, 0, nullptr, nullptr, nullptr, nullptr, x);
    if (!cera_gemm_supports(w->dtype, w->k))
        return cera_fail(ctx, CERA_HIP_ERR_UNSUPPORTED_DTYPE,
                         "gemm: no batched kernel for ggml type " + std::to_string(w->dtype) + " with k=" + std::to_string(w->k));
    void *ds, *dq, *db;
    CERA_TRY(cera_scratch(ctx, 1, n * (w->k / 32) * 4, &ds));
    CERA_TRY(cera_scratch(ctx, 2, n * w->k, &dq));
    CERA_TRY(cera_scratch(ctx, 7, n * (w->k / 32) * 4, &db));
    CERA_TRY(quantize_rows(ctx, x, n, w->k, static_cast<float*>(ds), static_cast<int8_t*>(dq), static_cast<float*>(db)));
    // reference layout: out[m][n]
    return cera_launch_gemm(ctx, w, static_cast<float*>(ds), static_cast<int8_t*>(dq), static_cast<float*>(db),
                            static_cast<uint32_t>(n), out, n, 1, nullptr, 1.0f);
}

extern "C" cera_hip_status cera_hip_gemm(cera_hip_ctx* ctx, const cera_hip_tensor* t, const float* x, uint64_t n,
                                         float* out) {
    if (!ctx || !x || !out) return CERA_HIP_ERR_ARGUMENT;
    std::lock_guard<std::recursive_mutex> op_lk(ctx->op_mu);
    if (n == 0 || n > 0x7FFFFFFFull) return cera_fail(ctx, CERA_HIP_ERR_SHAPE, "gemm: bad n");
    cera_hip_dtensor* w = nullptr;
    CERA_TRY(cera_hip_tensor_upload(ctx, t, &w));
    auto run = [&]() -> cera_hip_status {
        void *dx, *dy;
        CERA_TRY(cera_scratch(ctx, 0, n * w->k * 4, &dx));
        CERA_TRY(cera_scratch(ctx, 3, n * w->m * 4, &dy));
        CERA_TRY(cera_hip_upload(ctx, dx, x, n * w->k * 4));
        CERA_TRY(cera_hip_gemm_dev(ctx, w, static_cast<float*>(dx), n, static_cast<float*>(dy)));
        return cera_hip_download(ctx, out, dy, n * w->m * 4);
    };
    cera_hip_status st = run();
    cera_hip_tensor_free(ctx, w);
    return st;
}

// The GEMM's integer block dots as the matrix cores deliver them (debug instances of the same
// kernels): dots [m][n][k/32] int32 -- Q4_0 sum (q-8)a, Q8_0 sum w a, Q4_1 / Q4_K sum q a -- and
// for Q6_K [m][n][k/16], each the f32 result of the f16 MFMA for one 16-element scale group,
// sum (q-32)a, returned as f32 so that a test can see it is an exact integer.  out (nullable)
// receives the float result of the same launch.
extern "C" cera_hip_status cera_hip_gemm_block_dots(cera_hip_ctx* ctx, const cera_hip_tensor* t, const float* x, uint64_t n,
                                                    int32_t* dots, float* out) {
    if (!ctx || !t || !x || !dots) return CERA_HIP_ERR_ARGUMENT;
    std::lock_guard<std::recursive_mutex> op_lk(ctx->op_mu);
    if (n == 0 || n > 0x7FFFFFFFull) return cera_fail(ctx, CERA_HIP_ERR_SHAPE, "gemm_block_dots: bad n");
    const uint64_t per = t->ggml_type == CERA_HIP_Q6_K ? t->k / 16 : t->k / 32;
    if (t->m * n * per > (64ull << 20)) return cera_fail(ctx, CERA_HIP_ERR_SHAPE, "gemm_block_dots: more than 64 Mi block dots; use a smaller shape");
    cera_hip_dtensor* w = nullptr;
    CERA_TRY(cera_hip_tensor_upload(ctx, t, &w));
    auto run = [&]() -> cera_hip_status {
        if (!cera_gemm_supports(w->dtype, w->k))
            return cera_fail(ctx, CERA_HIP_ERR_UNSUPPORTED_DTYPE, "gemm_block_dots: no int8 GEMM for this type / k");
        void *dx, *dy, *ds, *dq, *db, *dd;
        CERA_TRY(cera_scratch(ctx, 0, n * w->k * 4, &dx));
        CERA_TRY(cera_scratch(ctx, 3, n * w->m * 4, &dy));
        CERA_TRY(cera_scratch(ctx, 1, n * (w->k / 32) * 4, &ds));
        CERA_TRY(cera_scratch(ctx, 2, n * w->k, &dq));
        CERA_TRY(cera_scratch(ctx, 7, n * (w->k / 32) * 4, &db));
        CERA_TRY(cera_scratch(ctx, 4, w->m * n * per * 4, &dd));
        CERA_TRY(cera_hip_upload(ctx, dx, x, n * w->k * 4));
        CERA_TRY(quantize_rows(ctx, static_cast<float*>(dx), n, w->k, static_cast<float*>(ds), static_cast<int8_t*>(dq), static_cast<float*>(db)));
        CERA_TRY(cera_launch_gemm(ctx, w, static_cast<float*>(ds), static_cast<int8_t*>(dq), static_cast<float*>(db),
                                  static_cast<uint32_t>(n), static_cast<float*>(dy), n, 1, nullptr, 1.0f, nullptr, nullptr, 0,
                                  nullptr, nullptr, nullptr, static_cast<int32_t*>(dd)));
        CERA_TRY(cera_hip_download(ctx, dots, dd, w->m * n * per * 4));
        if (out) CERA_TRY(cera_hip_download(ctx, out, dy, n * w->m * 4));
        return CERA_HIP_OK;
    };
    cera_hip_status st = run();
    cera_hip_tensor_free(ctx, w);
    return st;
}

extern "C" cera_hip_status cera_hip_gemm_pair(cera_hip_ctx* ctx, const cera_hip_tensor* ta, const cera_hip_tensor* tb,
                                              const float* x, uint64_t n, float* out_a, float* out_b) {
    if (!ctx || !ta || !tb || !x || !out_a || !out_b) return CERA_HIP_ERR_ARGUMENT;
    std::lock_guard<std::recursive_mutex> op_lk(ctx->op_mu);
    if (n == 0 || n > 0x7FFFFFFFull) return cera_fail(ctx, CERA_HIP_ERR_SHAPE, "gemm_pair: bad n");
    cera_hip_dtensor *wa = nullptr, *wb = nullptr;
    CERA_TRY(cera_hip_tensor_upload(ctx, ta, &wa));
    cera_hip_status st = cera_hip_tensor_upload(ctx, tb, &wb);
    if (st != CERA_HIP_OK) { cera_hip_tensor_free(ctx, wa); return st; }
    auto run = [&]() -> cera_hip_status {
        if (!cera_gemm_supports(wa->dtype, wa->k) || wa->dtype != wb->dtype || wa->k != wb->k)
            return cera_fail(ctx, CERA_HIP_ERR_UNSUPPORTED_DTYPE,
                             "gemm_pair: the matrices must share a type with an int8 GEMM and k");
        const uint64_t k = wa->k;
        void *dx, *ds, *dq, *db, *dya, *dyb;
        CERA_TRY(cera_scratch(ctx, 0, n * k * 4, &dx));
        CERA_TRY(cera_scratch(ctx, 1, n * (k / 32) * 4, &ds));
        CERA_TRY(cera_scratch(ctx, 2, n * k, &dq));
        CERA_TRY(cera_scratch(ctx, 7, n * (k / 32) * 4, &db));
        CERA_TRY(cera_scratch(ctx, 3, n * wa->m * 4, &dya));
        CERA_TRY(cera_scratch(ctx, 4, n * wb->m * 4, &dyb));
        CERA_TRY(cera_hip_upload(ctx, dx, x, n * k * 4));
        CERA_TRY(quantize_rows(ctx, static_cast<float*>(dx), n, k, static_cast<float*>(ds), static_cast<int8_t*>(dq),
                               static_cast<float*>(db)));
        bool paired = false;
        CERA_TRY(cera_launch_gemm(ctx, wa, static_cast<float*>(ds), static_cast<int8_t*>(dq), static_cast<float*>(db),
                                  static_cast<uint32_t>(n), static_cast<float*>(dya), 1, wa->m, nullptr, 1.0f, wb,
                                  static_cast<float*>(dyb), wb->m, &paired));
        if (!paired)   // rows x tokens not a multiple of 4: one after the other, as the forward pass does
            CERA_TRY(cera_launch_gemm(ctx, wb, static_cast<float*>(ds), static_cast<int8_t*>(dq), static_cast<float*>(db),
                                      static_cast<uint32_t>(n), static_cast<float*>(dyb), 1, wb->m, nullptr, 1.0f));
        CERA_TRY(cera_hip_download(ctx, out_a, dya, n * wa->m * 4));
        return cera_hip_download(ctx, out_b, dyb, n * wb->m * 4);
    };
    st = run();
    cera_hip_tensor_free(ctx, wa);
    cera_hip_tensor_free(ctx, wb);
    return st;
}

// halves (nullable, host [n][m] uint16): the quants once more as the f16 words a Q6_K down projection reads
static cera_hip_status gemm_swiglu_host(cera_hip_ctx* ctx, const cera_hip_tensor* tg, const cera_hip_tensor* tu,
                                        const float* x, uint64_t n, int8_t* quants, float* scales, uint16_t* halves,
                                        int* fused_out) {
    if (!ctx || !tg || !tu || !x || !quants || !scales) return CERA_HIP_ERR_ARGUMENT;
    std::lock_guard<std::recursive_mutex> op_lk(ctx->op_mu);
    if (n == 0 || n > 0x7FFFFFFFull) return cera_fail(ctx, CERA_HIP_ERR_SHAPE, "gemm_swiglu: bad n");
    cera_hip_dtensor *wg = nullptr, *wu = nullptr;
    CERA_TRY(cera_hip_tensor_upload(ctx, tg, &wg));
    cera_hip_status st = cera_hip_tensor_upload(ctx, tu, &wu);
    if (st != CERA_HIP_OK) { cera_hip_tensor_free(ctx, wg); return st; }
    auto run = [&]() -> cera_hip_status {
        if (!cera_gemm_supports(wg->dtype, wg->k) || wg->dtype != wu->dtype || wg->k != wu->k || wg->m != wu->m || wg->m % 32)
            return cera_fail(ctx, CERA_HIP_ERR_UNSUPPORTED_DTYPE,
                             "gemm_swiglu: gate and up must share a type with an int8 GEMM, k and m (a multiple of 32)");
        const uint64_t k = wg->k, mm = wg->m;
        void *dx, *ds, *dq, *db, *dg, *du, *hq, *hs, *hb;
        CERA_TRY(cera_scratch(ctx, 0, n * k * 4, &dx));
        CERA_TRY(cera_scratch(ctx, 1, n * (k / 32) * 4, &ds));
        CERA_TRY(cera_scratch(ctx, 2, n * k, &dq));
        CERA_TRY(cera_scratch(ctx, 7, n * (k / 32) * 4, &db));
        CERA_TRY(cera_scratch(ctx, 3, n * mm * 4, &dg));
        CERA_TRY(cera_scratch(ctx, 4, n * mm * 4, &du));
        CERA_TRY(cera_scratch(ctx, 5, n * mm, &hq));
        CERA_TRY(cera_scratch(ctx, 6, n * (mm / 32) * 4, &hs));
        CERA_TRY(cera_scratch(ctx, 8, n * (mm / 32) * 4, &hb));
        CERA_TRY(cera_hip_upload(ctx, dx, x, n * k * 4));
        CERA_TRY(quantize_rows(ctx, static_cast<float*>(dx), n, k, static_cast<float*>(ds), static_cast<int8_t*>(dq),
                               static_cast<float*>(db)));
        bool fused = false;
        void* hh = nullptr;
        if (halves) CERA_TRY(cera_scratch(ctx, 10, n * mm * 2, &hh));
        // (a Q4_K pair's epilogue writes the f16 words itself; every other route converts the quants afterwards)
        const bool hh_in_epilogue = halves && wg->dtype == CERA_HIP_Q4_K;
        CERA_TRY(cera_launch_gemm_swiglu(ctx, wg, wu, static_cast<float*>(ds), static_cast<int8_t*>(dq), static_cast<float*>(db),
                                         static_cast<uint32_t>(n), static_cast<int8_t*>(hq), static_cast<float*>(hs),
                                         static_cast<float*>(hb), &fused, nullptr, nullptr, hh_in_epilogue ? hh : nullptr));
        if (!fused) {   // the forward pass's other route: the two GEMMs, then the SwiGLU + quantize kernel
            CERA_TRY(cera_launch_gemm(ctx, wg, static_cast<float*>(ds), static_cast<int8_t*>(dq), static_cast<float*>(db),
                                      static_cast<uint32_t>(n), static_cast<float*>(dg), 1, mm, nullptr, 1.0f));
            CERA_TRY(cera_launch_gemm(ctx, wu, static_cast<float*>(ds), static_cast<int8_t*>(dq), static_cast<float*>(db),
                                      static_cast<uint32_t>(n), static_cast<float*>(du), 1, mm, nullptr, 1.0f));
            const uint64_t tot = n * mm;
            hipLaunchKernelGGL((silu_mul_kernel<true>), dim3(static_cast<uint32_t>((tot / 4 + 255) / 256)), dim3(256), 0,
                               ctx->stream, static_cast<float*>(dg), static_cast<float*>(du), tot, static_cast<float*>(nullptr),
                               static_cast<float*>(hs), static_cast<int8_t*>(hq), static_cast<float*>(hb));
            HIP_TRY(ctx, hipGetLastError());
        }
        if (fused_out) *fused_out = fused ? 1 : 0;
        if (halves) {
            if (!(fused && hh_in_epilogue)) {
                if ((n * mm) % 16) return cera_fail(ctx, CERA_HIP_ERR_SHAPE, "gemm_swiglu: n * m must be a multiple of 16 for the f16 form");
                const uint64_t words = n * mm / 16;
                hipLaunchKernelGGL(gemm_act_f16_kernel, dim3(static_cast<uint32_t>((words + 255) / 256)), dim3(256), 0, ctx->stream,
                                   static_cast<const uint4*>(hq), static_cast<uint4*>(hh), words);
                HIP_TRY(ctx, hipGetLastError());
            }
            CERA_TRY(cera_hip_download(ctx, halves, hh, n * mm * 2));
        }
        CERA_TRY(cera_hip_download(ctx, quants, hq, n * mm));
        return cera_hip_download(ctx, scales, hs, n * (mm / 32) * 4);
    };
    st = run();
    cera_hip_tensor_free(ctx, wg);
    cera_hip_tensor_free(ctx, wu);
    return st;
}

extern "C" cera_hip_status cera_hip_gemm_swiglu(cera_hip_ctx* ctx, const cera_hip_tensor* tg, const cera_hip_tensor* tu,
                                                const float* x, uint64_t n, int8_t* quants, float* scales, int* fused_out) {
    return gemm_swiglu_host(ctx, tg, tu, x, n, quants, scales, nullptr, fused_out);
}

extern "C" cera_hip_status cera_hip_gemm_swiglu_f16(cera_hip_ctx* ctx, const cera_hip_tensor* tg, const cera_hip_tensor* tu,
                                                    const float* x, uint64_t n, int8_t* quants, float* scales,
                                                    uint16_t* halves, int* fused_out) {
    if (!halves) return CERA_HIP_ERR_ARGUMENT;
    return gemm_swiglu_host(ctx, tg, tu, x, n, quants, scales, halves, fused_out);
}

// ---------------------------------------------------------------------------
// Batched prefill of one chunk of n <= CHUNK tokens.
// Largest batch one pass takes; longer prompts are cut into passes of this size.  A caller that
// wants the reference Session's default ubatch of 512 (cera/src/model/mod.rs:303-332) gets it
// through forward_prefill_chunked; given the whole prompt, 2048-token passes amortise the weight
// staging of the GEMM better (+15 % tokens/s on an 8k prompt).
static constexpr uint32_t PREFILL_CHUNK = CERA_PREFILL_CHUNK;
// batches up to this many tokens run their projections on the multi-token GEMV instead of the GEMM
// (measured on the 8B shapes: 2 tokens 2.8 ms against 7.7 ms, 8 tokens 5.4 against 7.9, 16 tokens
// 10.7 against 9.4 -- the per-token dots grow with the batch while the GEMM's tile fills up)
static constexpr uint32_t PREFILL_SMALL_BATCH = 8;

cera_hip_status cera_model_ensure_prefill_buffers(cera_hip_model* m, uint32_t n) {
    if (m->pf_cap >= n) return CERA_HIP_OK;
    cera_hip_ctx* ctx = m->ctx;
    const cera_hip_config& c = m->cfg;
    HIP_TRY(ctx, hipStreamSynchronize(ctx->stream));
    for (void* p : m->pf_owned) (void)hipFree(p);
    m->pf_owned.clear();
    m->bytes -= m->pf_bytes;
    m->pf_bytes = 0;
    m->pf_cap = 0;
    const uint32_t cap = cera_prefill_cap(n);
    const CeraPrefillSizes sz = cera_prefill_sizes(c, cap);
    auto alloc = [&](uint64_t bytes, void** p) -> cera_hip_status {
        CERA_TRY(cera_model_malloc(m, p, bytes, "prefill buffer"));
        m->pf_owned.push_back(*p);
        m->bytes += bytes;
        m->pf_bytes += bytes;
        return CERA_HIP_OK;
    };
    CERA_TRY(alloc(sz.hidden, reinterpret_cast<void**>(&m->pf_hidden)));
    CERA_TRY(alloc(sz.normed, reinterpret_cast<void**>(&m->pf_normed)));
    CERA_TRY(alloc(sz.q, reinterpret_cast<void**>(&m->pf_q)));
    CERA_TRY(alloc(sz.k, reinterpret_cast<void**>(&m->pf_k)));
    CERA_TRY(alloc(sz.v, reinterpret_cast<void**>(&m->pf_v)));
    CERA_TRY(alloc(sz.attn, reinterpret_cast<void**>(&m->pf_attn)));
    CERA_TRY(alloc(sz.gate, reinterpret_cast<void**>(&m->pf_gate)));
    CERA_TRY(alloc(sz.up, reinterpret_cast<void**>(&m->pf_up)));
    CERA_TRY(alloc(sz.xq, reinterpret_cast<void**>(&m->pf_xq)));
    CERA_TRY(alloc(sz.xh, &m->pf_xh));
    CERA_TRY(alloc(sz.x8, &m->pf_x8));
    CERA_TRY(alloc(sz.xs, reinterpret_cast<void**>(&m->pf_xs)));
    CERA_TRY(alloc(sz.bsum, reinterpret_cast<void**>(&m->pf_bsum)));
    CERA_TRY(alloc(sz.tokens, reinterpret_cast<void**>(&m->pf_tokens)));
    m->pf_cap = cap;
    return CERA_HIP_OK;
}

static __global__ void set_pos_kernel(uint32_t* scalars, uint32_t pos) { scalars[1] = pos; }

// all_logits (host, [n][vocab]): when set, every position is projected through the LM head in one
// GEMM (project_logits_batched, cera/src/model/llama.rs:645-722) instead of the last one only.
static cera_hip_status prefill_chunk(cera_hip_model* m, const uint32_t* tokens, uint32_t n, uint32_t start_pos,
                                     bool want_logits, float* all_logits = nullptr) {
    cera_hip_ctx* ctx = m->ctx;
    const cera_hip_config& c = m->cfg;
    hipStream_t s = ctx->stream;
    const uint32_t hs = c.hidden, q_dim = c.n_heads * c.head_dim, kv_dim = c.n_kv_heads * c.head_dim;
    const float scale = c.attn_scale != 0.0f ? c.attn_scale : 1.0f / std::sqrt(static_cast<float>(c.head_dim));
    CERA_TRY(cera_model_ensure_prefill_buffers(m, n));
    CERA_TRY(cera_hip_upload(ctx, m->pf_tokens, tokens, n * 4ull));
    hipLaunchKernelGGL(set_pos_kernel, dim3(1), dim3(1), 0, s, m->scalars, start_pos);
    hipLaunchKernelGGL(embed_row_kernel, dim3((hs + 255) / 256, n), dim3(256), 0, s, m->embd->dtype, m->embd->dev,
                       m->embd->row_bytes, m->pf_tokens, hs, c.embed_scale, m->pf_hidden);
    HIP_TRY(ctx, hipGetLastError());

    // whether pf_xh holds the f16 form of the quants now in pf_xq; cleared wherever those are rewritten
    bool staged = false;
    // the same for pf_x8, the fp8 split copy the Q4_K GEMMs read
    bool staged8 = false;
    // the f32 activations whose hi / lo split (Q5_K GEMMs) the context's workspace holds now
    const float* split_of = nullptr;
    // split-K partial sums of pf_hidden that the next row norm adds up (n_split = 0: none).  From 128 rows on:
    // the norm runs one workgroup per row, and a few dozen workgroups adding up partial sums take longer than
    // the reduction launch they save (12.8 against 4.8 + 5.7 us at 16 rows, 11.3 against 6.3 + 7.4 at 512).
    RowsPending pend{};
    const bool norm_adds = n >= 128;
    auto norm_rows = [&](const float* x, const float* w, float* y) -> cera_hip_status {
        staged = false;
        staged8 = false;
        split_of = nullptr;
        if (pend.n_split && pend.x_out == x)
            hipLaunchKernelGGL(rmsnorm_pending_kernel, dim3(n), dim3(256), 0, s, x, w, hs, c.rms_eps, y, m->pf_xs, m->pf_xq,
                               m->pf_bsum, pend);
        else
            hipLaunchKernelGGL((rmsnorm_kernel<true>), dim3(n), dim3(256), 0, s, x, w, hs, c.rms_eps, y, m->pf_xs, m->pf_xq,
                               m->pf_bsum);
        pend = RowsPending{};
        HIP_TRY(ctx, hipGetLastError());
        return CERA_HIP_OK;
    };
    // out[n][w->m] (token-major rows) = B . W^T, optionally added onto resid
    // xf: the f32 activations the quantized ones in pf_xs / pf_xq were made from (what a Q5_K matrix reads)
    auto gemm = [&](const cera_hip_dtensor* w, float* out, const float* resid, const float* xf,
                    RowsPending* pending = nullptr, int part_slot = 9) -> cera_hip_status {
        // a short batch streams the weights once per 8 tokens through the multi-token GEMV (an
        // int8-MFMA tile would be mostly empty); its residual add is unscaled
        if ((n <= PREFILL_SMALL_BATCH || !gemm_batched(w->dtype, w->k)) && (!resid || c.residual_scale == 1.0f)) {
            bool launched = false;
            CERA_TRY(cera_launch_gemv_nb(ctx, w, m->pf_xs, m->pf_xq, static_cast<uint32_t>(w->k / 32),
                                         static_cast<uint32_t>(w->k), n, out, static_cast<uint32_t>(w->m), resid, &launched));
            if (launched) return CERA_HIP_OK;
        }
        bool split_held = split_of == xf;
        CERA_TRY(cera_launch_gemm(ctx, w, m->pf_xs, m->pf_xq, m->pf_bsum, n, out, 1, w->m, resid, c.residual_scale, nullptr,
                                  nullptr, 0, nullptr, m->pf_xh, &staged, nullptr, xf, &split_held, m->pf_x8, &staged8, pending,
                                  part_slot));
        if (w->dtype == CERA_HIP_Q5_K) split_of = xf;
        return CERA_HIP_OK;
    };

    // two projections of the same activations: one launch when both have an int8 GEMM of the same
    // type (the tail of one matrix's workgroups then overlaps the other's, and a short K-split
    // matrix like K shares Q's launch), else one after the other
    // pending (nullable): filled when the two went out as one launch whose split-K partial sums the caller adds up
    auto gemm2 = [&](const cera_hip_dtensor* wa, float* outa, const cera_hip_dtensor* wb, float* outb, const float* xf,
                     RowsPending* pending = nullptr) -> cera_hip_status {
        if (n > PREFILL_SMALL_BATCH && gemm_batched(wa->dtype, wa->k) && gemm_batched(wb->dtype, wb->k)) {
            bool paired = false;
            bool split_held = split_of == xf;
            CERA_TRY(cera_launch_gemm(ctx, wa, m->pf_xs, m->pf_xq, m->pf_bsum, n, outa, 1, wa->m, nullptr, 1.0f, wb, outb,
                                      wb->m, &paired, m->pf_xh, &staged, nullptr, xf, &split_held, m->pf_x8, &staged8, pending));
            if (wa->dtype == CERA_HIP_Q5_K) split_of = xf;
            if (paired) return CERA_HIP_OK;
            if (pending && pending->n_split) {
                // the first matrix went out alone and left its partial sums pending: the second one's launch reuses
                // their scratch, so they are added up now
                const uint64_t n4 = static_cast<uint64_t>(wa->m) * n / 4;
                hipLaunchKernelGGL(gemm_reduce_kernel, dim3(static_cast<uint32_t>((n4 + 255) / 256)), dim3(256), 0, s, pending->part,
                                   pending->n_split, pending->stride, n4, outa, static_cast<const float*>(nullptr), 1.0f, n4,
                                   static_cast<float*>(nullptr));
                HIP_TRY(ctx, hipGetLastError());
                *pending = RowsPending{};
            }
            return gemm(wb, outb, nullptr, xf);
        }
        CERA_TRY(gemm(wa, outa, nullptr, xf));
        return gemm(wb, outb, nullptr, xf);
    };

    for (uint32_t i = 0; i < c.n_layers; ++i) {
        LayerDev& L = m->layers[i];
        CERA_TRY(norm_rows(m->pf_hidden, L.attn_norm, m->pf_normed));
        // Q4_K Q and K next to a Q6_K V (the Q4_K_M mix): both re-laid copies of the activations in one launch
        if (n > PREFILL_SMALL_BATCH && L.q->dtype == CERA_HIP_Q4_K && L.k->dtype == CERA_HIP_Q4_K && L.v->dtype == CERA_HIP_Q6_K &&
            gemm_batched(CERA_HIP_Q4_K, hs) && gemm_batched(CERA_HIP_Q6_K, hs)) {
            hipLaunchKernelGGL(gemm_act_fp8_kernel, dim3((n + G8_BN - 1) / G8_BN * 2 * (hs / 256)), dim3(256), 0, s, m->pf_xq, m->pf_xs,
                               m->pf_bsum, static_cast<uint8_t*>(m->pf_x8), n, hs, static_cast<uint4*>(m->pf_xh));
            HIP_TRY(ctx, hipGetLastError());
            staged = true;
            staged8 = true;
        }
        // With nothing between the projections and RoPE (no biases, no QK norm) the RoPE / append kernel adds up
        // the split-K partial sums of Q | K and of V itself: two reduction launches less.
        RowsPending pqk{}, pvv{};
        const bool rope_adds = !L.q_bias && !L.q_norm;
        CERA_TRY(gemm2(L.q, m->pf_q, L.k, m->pf_k, m->pf_normed, rope_adds ? &pqk : nullptr));
        CERA_TRY(gemm(L.v, m->pf_v, nullptr, m->pf_normed, rope_adds ? &pvv : nullptr, 14));
        if (L.q_bias) {
            // bias rows: one launch per token keeps the kernel trivial; models with biases are rare here
            for (uint32_t t = 0; t < n; ++t) {
                hipLaunchKernelGGL(bias_kernel, dim3((q_dim + 255) / 256), dim3(256), 0, s, m->pf_q + static_cast<uint64_t>(t) * q_dim, L.q_bias, q_dim);
                hipLaunchKernelGGL(bias_kernel, dim3((kv_dim + 255) / 256), dim3(256), 0, s, m->pf_k + static_cast<uint64_t>(t) * kv_dim, L.k_bias, kv_dim);
                hipLaunchKernelGGL(bias_kernel, dim3((kv_dim + 255) / 256), dim3(256), 0, s, m->pf_v + static_cast<uint64_t>(t) * kv_dim, L.v_bias, kv_dim);
            }
        }
        if (L.q_norm) {
            hipLaunchKernelGGL((rmsnorm_kernel<false>), dim3(n * c.n_heads), dim3(256), 0, s, m->pf_q, L.q_norm, c.head_dim,
                               c.rms_eps, m->pf_q, nullptr, nullptr, nullptr);
            hipLaunchKernelGGL((rmsnorm_kernel<false>), dim3(n * c.n_kv_heads), dim3(256), 0, s, m->pf_k, L.k_norm, c.head_dim,
                               c.rms_eps, m->pf_k, nullptr, nullptr, nullptr);
        }
        if (pqk.n_split || pvv.n_split) {
            const RopePending rq{pqk.part, pqk.n_split, pqk.stride};
            const RopePending rk{pqk.n_split ? pqk.part + static_cast<uint64_t>(n) * q_dim : nullptr, pqk.n_split, pqk.stride};
            const RopePending rv{pvv.part, pvv.n_split, pvv.stride};
            if (m->kv_f16)
                hipLaunchKernelGGL(rope_kv_pending_kernel<kv_half>, dim3(c.n_heads + 2 * c.n_kv_heads, n), dim3(c.head_dim / 2), 0, s,
                                   m->pf_q, m->pf_k, m->pf_v, m->rope_table, m->scalars + 1, c.n_heads, c.n_kv_heads, c.head_dim,
                                   c.rope_type, static_cast<kv_half*>(L.kc), static_cast<kv_half*>(L.vc), c.max_seq_len, rq, rk, rv);
            else
                hipLaunchKernelGGL(rope_kv_pending_kernel<float>, dim3(c.n_heads + 2 * c.n_kv_heads, n), dim3(c.head_dim / 2), 0, s,
                                   m->pf_q, m->pf_k, m->pf_v, m->rope_table, m->scalars + 1, c.n_heads, c.n_kv_heads, c.head_dim,
                                   c.rope_type, static_cast<float*>(L.kc), static_cast<float*>(L.vc), c.max_seq_len, rq, rk, rv);
        } else if (m->kv_f16)
            hipLaunchKernelGGL(rope_kv_kernel<kv_half>, dim3(c.n_heads + 2 * c.n_kv_heads, n), dim3(c.head_dim / 2), 0, s,
                               m->pf_q, m->pf_k, m->pf_v, m->rope_table, m->scalars + 1, c.n_heads, c.n_kv_heads, c.head_dim,
                               c.rope_type, static_cast<kv_half*>(L.kc), static_cast<kv_half*>(L.vc), c.max_seq_len);
        else
            hipLaunchKernelGGL(rope_kv_kernel<float>, dim3(c.n_heads + 2 * c.n_kv_heads, n), dim3(c.head_dim / 2), 0, s,
                               m->pf_q, m->pf_k, m->pf_v, m->rope_table, m->scalars + 1, c.n_heads, c.n_kv_heads, c.head_dim,
                               c.rope_type, static_cast<float*>(L.kc), static_cast<float*>(L.vc), c.max_seq_len);
        HIP_TRY(ctx, hipGetLastError());
        // causal attention: query t sees positions 0 .. start_pos + t
        CERA_TRY(cera_launch_attn(ctx, m->pf_q, L.kc, L.vc, c.n_heads, c.n_kv_heads, c.head_dim, start_pos + 1ull,
                                  c.max_seq_len, scale, 0, n, m->pf_attn, m->pf_xs, m->pf_xq, m->pf_bsum, nullptr, m->kv_f16));
        staged = false;   // the attention merge rewrote the quants
        staged8 = false;
        split_of = nullptr;
        // (the row norm that follows adds the O projection's split-K partial sums itself)
        CERA_TRY(gemm(L.o, m->pf_hidden, m->pf_hidden, m->pf_attn, norm_adds ? &pend : nullptr));

        CERA_TRY(norm_rows(m->pf_hidden, L.ffn_norm, m->pf_normed));
        // gate, up, SwiGLU and the quantization for the down projection in one launch where the
        // batch fills the chip; the quantized activations then lie in the (otherwise unused) gate
        // and up buffers, since the launch still reads its own input from pf_xq
        bool fused = false;
        int8_t* const hq = reinterpret_cast<int8_t*>(m->pf_gate);
        float *const hs = m->pf_up, *const hb = m->pf_up + static_cast<uint64_t>(n) * (c.ffn / 32);
        // a Q6_K down projection reads its activations as f16: the SwiGLU epilogue of the fp8 kernel writes them too
        const bool hh = L.gate->dtype == CERA_HIP_Q4_K && L.down->dtype == CERA_HIP_Q6_K;
        if (n > PREFILL_SMALL_BATCH && L.down->dtype != CERA_HIP_Q5_K)   // a Q5_K down projection reads the f32 SwiGLU output
            CERA_TRY(cera_launch_gemm_swiglu(ctx, L.gate, L.up, m->pf_xs, m->pf_xq, m->pf_bsum, n, hq, hs, hb, &fused, m->pf_x8, &staged8,
                                             hh ? m->pf_xh : nullptr));
        staged = fused && hh;   // pf_xh: the down projection's activations, or stale
        if (fused) staged8 = false;
        if (fused && cera_gemm_supports(L.down->dtype, L.down->k)) {
            // (all layers but the last: the next layer's first row norm adds the partial sums)
            CERA_TRY(cera_launch_gemm(ctx, L.down, hs, hq, hb, n, m->pf_hidden, 1, L.down->m, m->pf_hidden, c.residual_scale,
                                      nullptr, nullptr, 0, nullptr, m->pf_xh, &staged, nullptr, nullptr, nullptr, m->pf_x8, &staged8,
                                      norm_adds && i + 1 < c.n_layers ? &pend : nullptr));
            staged = false;   // pf_xh / pf_x8 now mirror hq, not pf_xq
            staged8 = false;
            continue;
        }
        if (fused) {   // a down projection without a GEMM reads pf_xq: move the quantized activations there
            HIP_TRY(ctx, hipMemcpyAsync(m->pf_xq, hq, static_cast<uint64_t>(n) * c.ffn, hipMemcpyDeviceToDevice, s));
            HIP_TRY(ctx, hipMemcpyAsync(m->pf_xs, hs, static_cast<uint64_t>(n) * (c.ffn / 32) * 4, hipMemcpyDeviceToDevice, s));
            HIP_TRY(ctx, hipMemcpyAsync(m->pf_bsum, hb, static_cast<uint64_t>(n) * (c.ffn / 32) * 4, hipMemcpyDeviceToDevice, s));
        } else {
            CERA_TRY(gemm2(L.gate, m->pf_gate, L.up, m->pf_up, m->pf_normed));
            const uint64_t tot = static_cast<uint64_t>(n) * c.ffn;
            hipLaunchKernelGGL((silu_mul_kernel<true>), dim3(static_cast<uint32_t>((tot / 4 + 255) / 256)), dim3(256), 0, s,
                               m->pf_gate, m->pf_up, tot, m->pf_gate, m->pf_xs, m->pf_xq, m->pf_bsum);
            HIP_TRY(ctx, hipGetLastError());
            split_of = nullptr;
        }
        staged8 = false;   // pf_xq holds the SwiGLU output now
        CERA_TRY(gemm(L.down, m->pf_hidden, m->pf_hidden, m->pf_gate, norm_adds && i + 1 < c.n_layers ? &pend : nullptr));
    }
    m->seq_len = start_pos + n;
    if (all_logits) {
        const cera_hip_dtensor* o = m->output ? m->output : m->embd;
        const uint64_t rows = o->m;   // == vocab: pad rows of a table are cut off at load
        if (m->pf_logits_cap < n) {
            HIP_TRY(ctx, hipStreamSynchronize(s));
            if (m->pf_logits) {
                (void)hipFree(m->pf_logits);
                m->bytes -= static_cast<uint64_t>(m->pf_logits_cap) * rows * 4;
                m->pf_logits = nullptr;
                m->pf_logits_cap = 0;
            }
            CERA_TRY(cera_model_malloc(m, reinterpret_cast<void**>(&m->pf_logits), static_cast<uint64_t>(m->pf_cap) * rows * 4,
                                       "all-positions logits"));
            m->pf_logits_cap = m->pf_cap;
            m->bytes += static_cast<uint64_t>(m->pf_cap) * rows * 4;
        }
        // final norm of every row (+ Q8_0), then logits[n][rows] = normed . head^T
        CERA_TRY(norm_rows(m->pf_hidden, m->output_norm, m->pf_normed));
        CERA_TRY(gemm(o, m->pf_logits, nullptr, m->pf_normed));
        if (c.logit_scale != 1.0f) {
            const uint64_t tot = static_cast<uint64_t>(n) * rows;
            hipLaunchKernelGGL(scale_kernel, dim3(static_cast<uint32_t>((tot + 255) / 256)), dim3(256), 0, s, m->pf_logits,
                               1.0f / c.logit_scale, static_cast<uint32_t>(tot));
            HIP_TRY(ctx, hipGetLastError());
        }
        return cera_hip_download(ctx, all_logits, m->pf_logits, static_cast<uint64_t>(n) * rows * 4);
    }
    if (want_logits) {
        // last token: final norm then the decode-style GEMV (project_logits)
        const float* last = m->pf_hidden + static_cast<uint64_t>(n - 1) * hs;
        hipLaunchKernelGGL((rmsnorm_kernel<true>), dim3(1), dim3(256), 0, s, last, m->output_norm, hs, c.rms_eps, m->hidden,
                           m->xs, m->xq, static_cast<float*>(nullptr));
        HIP_TRY(ctx, hipGetLastError());
        const cera_hip_dtensor* o = m->output ? m->output : m->embd;
        if (o->dtype == CERA_HIP_Q5_K) CERA_TRY(cera_launch_gemv_q5k_f32(ctx, o, m->hidden, m->logits));
        else CERA_TRY(cera_launch_gemv(ctx, o, nullptr, m->xs, m->xq, m->logits, nullptr, CERA_EPI_STORE));
        if (c.logit_scale != 1.0f) {
            hipLaunchKernelGGL(scale_kernel, dim3((c.vocab + 255) / 256), dim3(256), 0, s, m->logits, 1.0f / c.logit_scale, c.vocab);
            HIP_TRY(ctx, hipGetLastError());
        }
    }
    return CERA_HIP_OK;
}

// A matrix can take a batch of tokens either through the int8 GEMM (K in whole 256-element
// steps) or, any int8 type with one unit per lane, through the multi-token GEMV in passes of 8
// tokens (unscaled residual add only) -- e.g. the Q4_0 / Q8_0 files of small models whose hidden
// size is not a multiple of 256.
static bool batched_supports(const cera_hip_model* m, const cera_hip_dtensor* w) {
    if (gemm_batched(w->dtype, w->k)) return true;
    const bool int8_type = w->dtype == CERA_HIP_Q4_0 || w->dtype == CERA_HIP_Q4_1 || w->dtype == CERA_HIP_Q8_0 ||
                           w->dtype == CERA_HIP_Q4_K || w->dtype == CERA_HIP_Q6_K;
    const uint64_t unit = w->dtype == CERA_HIP_Q6_K ? 64 : 32;
    return int8_type && w->k % unit == 0 && w->k / unit <= 512 && m->cfg.residual_scale == 1.0f;
}
static bool prefill_batchable(const cera_hip_model* m) {
    if (m->ref_order) return false;   // the verification route prefills token by token, as its CPU twin does
    for (const LayerDev& L : m->layers)
        for (const cera_hip_dtensor* w : {L.q, L.k, L.v, L.o, L.gate, L.up, L.down})
            if (!batched_supports(m, w)) return false;
    return true;
}

cera_hip_status cera_model_prefill_logits_all(cera_hip_model* m, const uint32_t* tokens, uint32_t n, uint32_t start_pos,
                                              float* logits_all) {
    const cera_hip_dtensor* head = m->output ? m->output : m->embd;
    const uint64_t vocab = m->cfg.vocab;
    // single token, or a weight / head type without an int8 GEMM: each forward returns that
    // position's logits (the reference's fallback, cera/src/model/llama.rs:1712-1720)
    if (n == 1 || !prefill_batchable(m) || !batched_supports(m, head)) {
        for (uint32_t i = 0; i < n; ++i)
            CERA_TRY(cera_model_decode_logits(m, tokens[i], start_pos + i, logits_all + i * vocab));
        return CERA_HIP_OK;
    }
    for (uint32_t off = 0; off < n; off += PREFILL_CHUNK) {
        uint32_t len = std::min(PREFILL_CHUNK, n - off);
        CERA_TRY(prefill_chunk(m, tokens + off, len, start_pos + off, false, logits_all + off * vocab));
    }
    return CERA_HIP_OK;
}

cera_hip_status cera_model_prefill(cera_hip_model* m, const uint32_t* tokens, uint32_t n, uint32_t start_pos,
                                   float* last_logits) {
    // A single token, or a weight shape with no batched kernel, takes the per-token
    // route -- the same decision LlamaModel::forward_prefill makes (llama.rs:1643,
    // 762-795); it is still the HIP path, only slower.  (Q5_K, which sends the reference down
    // that route, has a batched kernel here.)
    // a layer projection the reference's batched GEMM cannot take (Q5_K) sends its whole prefill
    // down the per-token route (cera/src/model/llama.rs:762-795); so does the verification route
    bool ref_gemmable = true;
    for (const LayerDev& L : m->layers)
        for (const cera_hip_dtensor* w : {L.q, L.k, L.v, L.o, L.gate, L.up, L.down})
            if (w->dtype == CERA_HIP_Q5_K) ref_gemmable = false;
    if (m->ref_order == 2 && n > 1 && ref_gemmable) {
        // the verification route in the x86 host's batched order (forward_prefill takes
        // forward_prefill_batched for n > 1, cera/src/model/llama.rs:1639-1641); one pass holds
        // PREFILL_CHUNK tokens, the reference's callers split at ubatch = 512 (model/mod.rs:303-332)
        for (uint32_t off = 0; off < n; off += PREFILL_CHUNK) {
            uint32_t len = std::min(PREFILL_CHUNK, n - off);
            CERA_TRY(cera_model_prefill_ref_batched(m, tokens + off, len, start_pos + off, off + len == n));
        }
        return cera_hip_download(m->ctx, last_logits, m->logits, static_cast<uint64_t>(m->cfg.vocab) * 4);
    }
    if (n == 1 || !prefill_batchable(m)) return cera_model_prefill_per_token(m, tokens, n, start_pos, last_logits);
    for (uint32_t off = 0; off < n; off += PREFILL_CHUNK) {
        uint32_t len = std::min(PREFILL_CHUNK, n - off);
        CERA_TRY(prefill_chunk(m, tokens + off, len, start_pos + off, off + len == n));
    }
    return cera_hip_download(m->ctx, last_logits, m->logits, static_cast<uint64_t>(m->cfg.vocab) * 4);
}
