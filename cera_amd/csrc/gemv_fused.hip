// Launch rules of the one-wavefront-per-row decode GEMVs (gemv_rows.hip.h): which instance a
// matrix's type and shape get, the decode copies they stream, and the host-buffer entry points.
#include "gemv_rows.hip.h"
#include "host_common.h"

// ---------------------------------------------------------------------------
static constexpr int FUSED_NW = 8;

static bool kquant_type(uint32_t t) { return t == CERA_HIP_Q4_K || t == CERA_HIP_Q6_K; }
static bool block32_type(uint32_t t) { return t == CERA_HIP_Q4_0 || t == CERA_HIP_Q4_1 || t == CERA_HIP_Q8_0; }
static bool fused_type(uint32_t t) { return kquant_type(t) || block32_type(t); }
static uint32_t unit_elems(uint32_t t) { return kquant_type(t) ? 64 : 32; }
// Passes of 64 units a row of k weights of this type takes in the one-wavefront-per-row kernels
// (0: the type or the row length has no such kernel).
static uint32_t row_tiles(uint32_t type, uint64_t k) {
    if (!fused_type(type) || k == 0 || k % (kquant_type(type) ? 256 : 32)) return 0;
    return static_cast<uint32_t>((k / unit_elems(type) + 63) / 64);
}
// rows short enough for the kernels that keep a row's activations in registers
// (one or two passes per lane: k <= 8192 for the K-quants' 64-weight units, k <= 4096 for 32-weight blocks)
static uint32_t short_tiles(uint32_t type, uint64_t k) {
    const uint32_t t = k <= (kquant_type(type) ? 8192u : 4096u) ? row_tiles(type, k) : 0;
    return t <= 2u ? t : 0;
}

static void fill(RowGemvArgs& a, const cera_hip_dtensor* w, const cera_hip_dtensor* w2, uint32_t rows_per_wave, bool stream = false) {
    a = RowGemvArgs{};
    a.w = stream ? w->dev_stream : w->dev;
    a.w2 = w2 ? (stream ? w2->dev_stream : w2->dev) : nullptr;
    a.m = static_cast<uint32_t>(w->m);
    a.k = static_cast<uint32_t>(w->k);
    a.row_bytes = static_cast<uint32_t>(stream ? w->stream_row_bytes : w->row_bytes);
    a.rows_per_wave = rows_per_wave;
}

// ---- decode copies ------------------------------------------------------------------------------
// Gives a Q4_K / Q6_K / Q4_0 / Q4_1 / Q8_0 matrix its decode copy (a second allocation of about the same size, kept
// until the tensor is freed): the per-row permutation that lets the one-wavefront-per-row
// kernels stream it with non-temporal loads.  A load-time re-layout for the kernel that reads
// it, as the reference's own x86 path does with repack_q4_k_8x8 (cera/src/backend/cpu.rs:1282-1358);
// the native bytes stay for every other reader (prefill GEMM, embedding lookup, verification
// route).  Other types and views are left alone.
static uint64_t stream_row_bytes_of(const cera_hip_ctx* ctx, const cera_hip_dtensor* w) {
    if (!ctx->decode_copies) return 0;
    if (!w || !w->owns || w->k > 32768 || w->m == 0 || w->m > 0x7FFFFFFFull) return 0;
    if (row_tiles(w->dtype, w->k) == 0 || (reinterpret_cast<uintptr_t>(w->dev) & 15)) return 0;
    const uint32_t k = static_cast<uint32_t>(w->k);
    switch (w->dtype) {
        case CERA_HIP_Q4_K: return Q4K::stream_row_bytes(k);
        case CERA_HIP_Q6_K: return Q6K::stream_row_bytes(k);
        case CERA_HIP_Q4_0: return Q4_0::stream_row_bytes(k);
        case CERA_HIP_Q4_1: return Q4_1::stream_row_bytes(k);
        default: return Q8_0::stream_row_bytes(k);
    }
}
// bytes a decode copy of w would take; 0 when w gets none (copies off, a view, a type or shape
// without a streaming kernel) or already has one
uint64_t cera_tensor_stream_bytes(const cera_hip_ctx* ctx, const cera_hip_dtensor* w) {
    return (w && w->dev_stream) ? 0 : stream_row_bytes_of(ctx, w) * (w ? w->m : 0);
}
void cera_tensor_drop_stream(cera_hip_dtensor* w) {
    if (!w || !w->dev_stream) return;
    (void)hipFree(w->dev_stream);
    w->dev_stream = nullptr;
    w->stream_row_bytes = 0;
}
cera_hip_status cera_tensor_prepare_stream(cera_hip_ctx* ctx, cera_hip_dtensor* w) {
    if (!w || w->dev_stream) return CERA_HIP_OK;
    const uint64_t srb = stream_row_bytes_of(ctx, w);
    if (srb == 0) return CERA_HIP_OK;
    const uint32_t k = static_cast<uint32_t>(w->k);
    void* p = nullptr;
    const hipError_t e = hipMalloc(&p, srb * w->m);
    if (e != hipSuccess) {
        (void)hipGetLastError();
        // an optimisation only: without room for the copy the kernels read the native bytes
        if (e == hipErrorOutOfMemory) return CERA_HIP_OK;
        return cera_fail(ctx, CERA_HIP_ERR_DEVICE, std::string("hipMalloc(decode copy): ") + hipGetErrorString(e));
    }
    const dim3 grid(static_cast<uint32_t>(w->m)), block(256);
    const uint32_t n_units = k / unit_elems(w->dtype), rb = static_cast<uint32_t>(w->row_bytes);
    uint8_t* dst = static_cast<uint8_t*>(p);
    switch (w->dtype) {
        case CERA_HIP_Q4_K: hipLaunchKernelGGL(stream_rows_kernel<Q4K>, grid, block, 0, ctx->stream, w->dev, dst, grid.x, n_units, rb, static_cast<uint32_t>(srb)); break;
        case CERA_HIP_Q6_K: hipLaunchKernelGGL(stream_rows_kernel<Q6K>, grid, block, 0, ctx->stream, w->dev, dst, grid.x, n_units, rb, static_cast<uint32_t>(srb)); break;
        case CERA_HIP_Q4_0: hipLaunchKernelGGL(stream_rows_kernel<Q4_0>, grid, block, 0, ctx->stream, w->dev, dst, grid.x, n_units, rb, static_cast<uint32_t>(srb)); break;
        case CERA_HIP_Q4_1: hipLaunchKernelGGL(stream_rows_kernel<Q4_1>, grid, block, 0, ctx->stream, w->dev, dst, grid.x, n_units, rb, static_cast<uint32_t>(srb)); break;
        default: hipLaunchKernelGGL(stream_rows_kernel<Q8_0>, grid, block, 0, ctx->stream, w->dev, dst, grid.x, n_units, rb, static_cast<uint32_t>(srb)); break;
    }
    const hipError_t le = hipGetLastError();
    if (le != hipSuccess) {
        (void)hipFree(p);
        return cera_fail(ctx, CERA_HIP_ERR_DEVICE, std::string("decode copy: ") + hipGetErrorString(le));
    }
    w->dev_stream = static_cast<uint8_t*>(p);
    w->stream_row_bytes = srb;
    return CERA_HIP_OK;
}
static uint32_t blocks_for(uint64_t m, uint32_t rows_per_wave) {
    const uint64_t per = static_cast<uint64_t>(FUSED_NW) * rows_per_wave;
    return static_cast<uint32_t>((m + per - 1) / per);
}

// ffn first half: Q8_0(silu(gate . n) * (up . n)) with n = Q8_0(rmsnorm(x, norm_w)); out_q [m], out_s [m/32].
// *launched = false (nothing done) when the shapes / types have no fused instance.
cera_hip_status cera_launch_ffn_gate_up_fused(cera_hip_ctx* ctx, const cera_hip_dtensor* gate, const cera_hip_dtensor* up,
                                              const float* x, const float* norm_w, float eps, int8_t* out_q, float* out_s,
                                              bool* launched) {
    *launched = false;
    const uint32_t tiles = short_tiles(gate->dtype, gate->k);
    if (tiles == 0 || gate->dtype == CERA_HIP_Q6_K || up->dtype != gate->dtype || gate->m != up->m || gate->k != up->k || gate->m % 32)
        return CERA_HIP_OK;
    RowGemvArgs a;
    // 16 wavefronts x 4 rows: a workgroup owns two Q8_0 blocks of the output, and 14336 rows make
    // 224 workgroups -- one per CU in a single wave of the launch (448 eight-wavefront workgroups
    // leave a quarter of the CUs with half the others' share: 1 % slower end to end).  A CU runs
    // one of these workgroups at a time, so a matrix of more than 64 n_cu rows takes 6 or 8 rows per
    // wavefront rather than a second round (Q4_K 18944 x 3584: 296 workgroups 23.0 us; 17408 rows
    // the same, 16384 rows 13.8).  Q4_K rows of two passes per lane (4096 < k <= 8192) hold twice
    // the weights and activations per lane and take 8 wavefronts of 8 rows.
    constexpr int GATE_UP_NW = 16, WIDE_NW = 8, WIDE_ROWS = 8;
    const bool stream = gate->dev_stream && up->dev_stream;
    const bool wide = gate->dtype == CERA_HIP_Q4_K && tiles == 2;
    uint32_t rows = 4;
    if (!wide) {   // the instance with the fewest rows per wavefront x rounds
        uint64_t best = ~0ull;
        for (uint32_t r : {4u, 6u, 8u}) {
            const uint64_t wgs = (gate->m + GATE_UP_NW * r - 1) / (GATE_UP_NW * r);
            const uint64_t cost = r * ((wgs + ctx->n_cu - 1) / ctx->n_cu);
            if (cost <= best) { best = cost; rows = r; }   // of equals the one with fewer rounds
        }
    }
    if (wide) rows = WIDE_ROWS;
    fill(a, gate, up, rows, stream);
    a.x = x; a.norm_w = norm_w; a.eps = eps; a.out_q = out_q; a.out_s = out_s;
    const uint32_t nw = wide ? WIDE_NW : GATE_UP_NW, per_wg = nw * rows;
    const dim3 grid((a.m + per_wg - 1) / per_wg), block(64 * nw);
#define GATE_UP_LAUNCH_R(TT, TL, RR)                                                                                                    \
    do {                                                                                                                                \
        if (stream) hipLaunchKernelGGL((row_gemv_kernel<TT, GATE_UP_NW, RR, true, FEPI_SILU_Q8, true, TL>), grid, block, 0, ctx->stream, a); \
        else hipLaunchKernelGGL((row_gemv_kernel<TT, GATE_UP_NW, RR, true, FEPI_SILU_Q8, false, TL>), grid, block, 0, ctx->stream, a);   \
    } while (0)
#define GATE_UP_LAUNCH(TT, TL)                     \
    do {                                           \
        if (rows == 4) GATE_UP_LAUNCH_R(TT, TL, 4); \
        else if (rows == 6) GATE_UP_LAUNCH_R(TT, TL, 6); \
        else GATE_UP_LAUNCH_R(TT, TL, 8);          \
    } while (0)
#define GATE_UP_LAUNCH_B32(TT)            \
    do {                                  \
        if (tiles == 1) GATE_UP_LAUNCH(TT, 1); \
        else GATE_UP_LAUNCH(TT, 2);       \
    } while (0)
    if (wide) {
        if (stream) hipLaunchKernelGGL((row_gemv_kernel<Q4K, WIDE_NW, WIDE_ROWS, true, FEPI_SILU_Q8, true, 2, 8192>), grid, block, 0, ctx->stream, a);
        else hipLaunchKernelGGL((row_gemv_kernel<Q4K, WIDE_NW, WIDE_ROWS, true, FEPI_SILU_Q8, false, 2, 8192>), grid, block, 0, ctx->stream, a);
    } else if (gate->dtype == CERA_HIP_Q4_K) GATE_UP_LAUNCH(Q4K, 1);
    else if (gate->dtype == CERA_HIP_Q4_0) GATE_UP_LAUNCH_B32(Q4_0);
    else if (gate->dtype == CERA_HIP_Q4_1) GATE_UP_LAUNCH_B32(Q4_1);
    else GATE_UP_LAUNCH_B32(Q8_0);
#undef GATE_UP_LAUNCH_R
#undef GATE_UP_LAUNCH_B32
#undef GATE_UP_LAUNCH
    HIP_TRY(ctx, hipGetLastError());
    *launched = true;
    return CERA_HIP_OK;
}

// attention projections: ya = A . n, yb = B . n (b nullable) with n = Q8_0(rmsnorm(x, norm_w)).
cera_hip_status cera_launch_qkv_fused(cera_hip_ctx* ctx, const cera_hip_dtensor* wa, const cera_hip_dtensor* wb, const float* x,
                                      const float* norm_w, float eps, float* ya, float* yb, bool* launched) {
    *launched = false;
    const uint32_t tiles = short_tiles(wa->dtype, wa->k);
    if (tiles == 0 || (wb && (wb->k != wa->k || short_tiles(wb->dtype, wb->k) != tiles))) return CERA_HIP_OK;
    // the 32-weight-block types pair with their own kind only
    if (wb && block32_type(wa->dtype) != block32_type(wb->dtype)) return CERA_HIP_OK;
    if (wb && block32_type(wa->dtype) && wb->dtype != wa->dtype) return CERA_HIP_OK;
    // two rows per wavefront (12 wavefronts per CU on the 8B shapes), one for short matrices
    // (four for the 10240 x 8192 matrix of a 70B-class layer, to fit one round: no faster)
    const uint64_t rows = wa->m + (wb ? wb->m : 0);
    const uint32_t rpw = rows >= static_cast<uint64_t>(ctx->n_cu) * 8 ? 2 : 1;
    RowGemvPairArgs p;
    const bool stream = wa->dev_stream && (!wb || wb->dev_stream);
    fill(p.a, wa, nullptr, rpw, stream);
    p.a.x = x; p.a.norm_w = norm_w; p.a.eps = eps; p.a.y = ya;
    p.n_blocks_a = blocks_for(wa->m, rpw);
    uint32_t n_blocks = p.n_blocks_a;
    if (wb) {
        fill(p.b, wb, nullptr, rpw, stream);
        p.b.x = x; p.b.norm_w = norm_w; p.b.eps = eps; p.b.y = yb;
        n_blocks += blocks_for(wb->m, rpw);
    } else {
        p.b = p.a;
    }
    const dim3 grid(n_blocks), block(64 * FUSED_NW);
    const uint32_t ta = wa->dtype, tb = wb ? wb->dtype : wa->dtype;
#define QKV_LAUNCH_S(TA_, TB_, ST_, TL_)                                                                                                \
    do {                                                                                                                                \
        if (rpw == 2) hipLaunchKernelGGL((row_gemv_pair_kernel<TA_, TB_, FUSED_NW, 2, true, ST_, TL_, 4096 * TL_>), grid, block, 0, ctx->stream, p); \
        else hipLaunchKernelGGL((row_gemv_pair_kernel<TA_, TB_, FUSED_NW, 1, true, ST_, TL_, 4096 * TL_>), grid, block, 0, ctx->stream, p);          \
    } while (0)
#define QKV_LAUNCH(TA_, TB_, TL_)                    \
    do {                                             \
        if (stream) QKV_LAUNCH_S(TA_, TB_, true, TL_); \
        else QKV_LAUNCH_S(TA_, TB_, false, TL_);     \
    } while (0)
#define QKV_LAUNCH_B32(TT)                  \
    do {                                    \
        if (tiles == 1) QKV_LAUNCH(TT, TT, 1); \
        else QKV_LAUNCH(TT, TT, 2);         \
    } while (0)
    if (ta == CERA_HIP_Q4_0) QKV_LAUNCH_B32(Q4_0);
    else if (ta == CERA_HIP_Q4_1) QKV_LAUNCH_B32(Q4_1);
    else if (ta == CERA_HIP_Q8_0) QKV_LAUNCH_B32(Q8_0);
#define QKV_LAUNCH_KQ(TA_, TB_)                \
    do {                                       \
        if (tiles == 1) QKV_LAUNCH(TA_, TB_, 1); \
        else QKV_LAUNCH(TA_, TB_, 2);          \
    } while (0)
    else if (ta == CERA_HIP_Q4_K && tb == CERA_HIP_Q6_K) QKV_LAUNCH_KQ(Q4K, Q6K);
    else if (ta == CERA_HIP_Q4_K && tb == CERA_HIP_Q4_K) QKV_LAUNCH_KQ(Q4K, Q4K);
    else if (ta == CERA_HIP_Q6_K && tb == CERA_HIP_Q6_K) QKV_LAUNCH_KQ(Q6K, Q6K);
    else QKV_LAUNCH_KQ(Q6K, Q4K);
#undef QKV_LAUNCH_KQ
#undef QKV_LAUNCH_B32
#undef QKV_LAUNCH
#undef QKV_LAUNCH_S
    HIP_TRY(ctx, hipGetLastError());
    *launched = true;
    return CERA_HIP_OK;
}

// y = resid + W . (xs, xq) with a wavefront per row (k <= 4096: no K split, no LDS combine, no
// barrier): the O projection.  Same per-row arithmetic as gemv_kernel, so the same bits; 4.4 -> 4.0 us
// on the 4096 x 4096 Q4_K matrix inside the model (588 -> 595 tok/s).
cera_hip_status cera_launch_row_gemv_add(cera_hip_ctx* ctx, const cera_hip_dtensor* w, const float* xs, const int8_t* xq,
                                         float* y, const float* resid, bool* launched) {
    *launched = false;
    const uint32_t tiles = short_tiles(w->dtype, w->k);
    if (tiles == 0 || !resid || w->m > 65535) return CERA_HIP_OK;
    constexpr int NW = 4, ROWS = 2;
    RowGemvArgs a;
    const bool stream = w->dev_stream != nullptr;
    fill(a, w, nullptr, ROWS, stream);
    a.xq = xq; a.xs = xs; a.y = y; a.resid = resid;
    const dim3 grid((a.m + NW * ROWS - 1) / (NW * ROWS)), block(64 * NW);
#define ADD_LAUNCH(TT, TL)                                                                                                     \
    do {                                                                                                                       \
        if (stream) hipLaunchKernelGGL((row_gemv_kernel<TT, NW, ROWS, false, FEPI_ADD, true, TL>), grid, block, 0, ctx->stream, a); \
        else hipLaunchKernelGGL((row_gemv_kernel<TT, NW, ROWS, false, FEPI_ADD, false, TL>), grid, block, 0, ctx->stream, a);    \
    } while (0)
#define ADD_LAUNCH_B32(TT)            \
    do {                              \
        if (tiles == 1) ADD_LAUNCH(TT, 1); \
        else ADD_LAUNCH(TT, 2);       \
    } while (0)
    if (w->dtype == CERA_HIP_Q4_K) ADD_LAUNCH_B32(Q4K);
    else if (w->dtype == CERA_HIP_Q6_K) ADD_LAUNCH_B32(Q6K);
    else if (w->dtype == CERA_HIP_Q4_0) ADD_LAUNCH_B32(Q4_0);
    else if (w->dtype == CERA_HIP_Q4_1) ADD_LAUNCH_B32(Q4_1);
    else ADD_LAUNCH_B32(Q8_0);
#undef ADD_LAUNCH_B32
#undef ADD_LAUNCH
    HIP_TRY(ctx, hipGetLastError());
    *launched = true;
    return CERA_HIP_OK;
}

// y = W . (xs, xq) from a decode copy with a wavefront per row (k <= 4096): the vocabulary head.
// Only taken when the matrix has a decode copy -- from the native bytes the K-split kernel is as
// fast.  Same per-row arithmetic, same bits; 73.6 -> 62.3 us on the 128256 x 4096 Q6_K head
// (6.9 TB/s).
cera_hip_status cera_launch_row_gemv_store(cera_hip_ctx* ctx, const cera_hip_dtensor* w, const float* xs, const int8_t* xq,
                                           float* y, bool* launched) {
    *launched = false;
    const uint32_t tiles = short_tiles(w->dtype, w->k);
    if (tiles == 0 || !w->dev_stream || w->m > (1u << 24)) return CERA_HIP_OK;
    constexpr int NW = 4, ROWS = 2;   // four rows per wavefront measured the same
    RowGemvArgs a;
    fill(a, w, nullptr, ROWS, true);
    a.xq = xq; a.xs = xs; a.y = y;
    const dim3 grid((a.m + NW * ROWS - 1) / (NW * ROWS)), block(64 * NW);
#define STORE_LAUNCH(TT, TL) hipLaunchKernelGGL((row_gemv_kernel<TT, NW, ROWS, false, FEPI_STORE, true, TL>), grid, block, 0, ctx->stream, a)
    if (w->dtype == CERA_HIP_Q4_K && tiles == 1) STORE_LAUNCH(Q4K, 1);
    else if (w->dtype == CERA_HIP_Q4_K) STORE_LAUNCH(Q4K, 2);
    else if (w->dtype == CERA_HIP_Q6_K && tiles == 1) STORE_LAUNCH(Q6K, 1);
    else if (w->dtype == CERA_HIP_Q6_K) STORE_LAUNCH(Q6K, 2);
    else if (w->dtype == CERA_HIP_Q4_0 && tiles == 1) STORE_LAUNCH(Q4_0, 1);
    else if (w->dtype == CERA_HIP_Q4_0) STORE_LAUNCH(Q4_0, 2);
    else if (w->dtype == CERA_HIP_Q4_1 && tiles == 1) STORE_LAUNCH(Q4_1, 1);
    else if (w->dtype == CERA_HIP_Q4_1) STORE_LAUNCH(Q4_1, 2);
    else if (tiles == 1) STORE_LAUNCH(Q8_0, 1);
    else STORE_LAUNCH(Q8_0, 2);
#undef STORE_LAUNCH
    HIP_TRY(ctx, hipGetLastError());
    *launched = true;
    return CERA_HIP_OK;
}

// y = resid + W . (xs, xq) for long rows (see row_gemv_long_kernel); *launched = false when the
// shape has no instance.
cera_hip_status cera_launch_row_gemv_long_add(cera_hip_ctx* ctx, const cera_hip_dtensor* w, const float* xs, const int8_t* xq,
                                              float* y, const float* resid, bool* launched) {
    *launched = false;
    const uint32_t tiles = row_tiles(w->dtype, w->k);
    const bool b32 = block32_type(w->dtype);
    if (tiles == 0 || short_tiles(w->dtype, w->k) != 0 || tiles > 8u || !resid || w->m > (1u << 20)) return CERA_HIP_OK;
    // four rows per workgroup: small workgroups start and retire independently, which measured
    // faster end to end than 8 or 16 rows sharing one staged copy of the activations
    constexpr int NW = 4;
    RowGemvArgs a;
    const bool stream = w->dev_stream != nullptr;
    fill(a, w, nullptr, 1, stream);
    a.xq = xq; a.xs = xs; a.y = y; a.resid = resid;
    const dim3 grid((a.m + NW - 1) / NW), block(64 * NW);
    // K-quant rows: 3 or 4 passes as they come (the 8B / 7B down projections), longer rows in 6 or 8
    // (a surplus pass re-reads unit 0 against zeroed activations)
#define LONG_LAUNCH_S(TT, ST_)                                                                                                 \
    do {                                                                                                                       \
        if (tiles <= 3) hipLaunchKernelGGL((row_gemv_long_kernel<TT, NW, 3, FEPI_ADD, ST_>), grid, block, 0, ctx->stream, a);   \
        else if (tiles == 4) hipLaunchKernelGGL((row_gemv_long_kernel<TT, NW, 4, FEPI_ADD, ST_>), grid, block, 0, ctx->stream, a); \
        else if (tiles <= 6) hipLaunchKernelGGL((row_gemv_long_kernel<TT, NW, 6, FEPI_ADD, ST_>), grid, block, 0, ctx->stream, a); \
        else hipLaunchKernelGGL((row_gemv_long_kernel<TT, NW, 8, FEPI_ADD, ST_>), grid, block, 0, ctx->stream, a);              \
    } while (0)
#define LONG_LAUNCH(TT)                      \
    do {                                     \
        if (stream) LONG_LAUNCH_S(TT, true); \
        else LONG_LAUNCH_S(TT, false);       \
    } while (0)
    // the 32-weight-block types take 4 or 8 passes (a surplus pass re-reads unit 0 against zeroed activations)
#define LONG_LAUNCH_B32(TT)                                                                                                     \
    do {                                                                                                                        \
        if (tiles <= 4 && stream) hipLaunchKernelGGL((row_gemv_long_kernel<TT, NW, 4, FEPI_ADD, true>), grid, block, 0, ctx->stream, a);  \
        else if (tiles <= 4) hipLaunchKernelGGL((row_gemv_long_kernel<TT, NW, 4, FEPI_ADD, false>), grid, block, 0, ctx->stream, a);      \
        else if (stream) hipLaunchKernelGGL((row_gemv_long_kernel<TT, NW, 8, FEPI_ADD, true>), grid, block, 0, ctx->stream, a);           \
        else hipLaunchKernelGGL((row_gemv_long_kernel<TT, NW, 8, FEPI_ADD, false>), grid, block, 0, ctx->stream, a);                      \
    } while (0)
    if (w->dtype == CERA_HIP_Q4_K) LONG_LAUNCH(Q4K);
    else if (w->dtype == CERA_HIP_Q6_K) LONG_LAUNCH(Q6K);
    else if (w->dtype == CERA_HIP_Q4_0) LONG_LAUNCH_B32(Q4_0);
    else if (w->dtype == CERA_HIP_Q4_1) LONG_LAUNCH_B32(Q4_1);
    else LONG_LAUNCH_B32(Q8_0);
#undef LONG_LAUNCH_B32
#undef LONG_LAUNCH
#undef LONG_LAUNCH_S
    HIP_TRY(ctx, hipGetLastError());
    *launched = true;
    return CERA_HIP_OK;
}

// y[t][row] (row stride 1, token stride y_stride) = W . x_t (+ resid, same layout) for a few tokens at
// once from the decode copy: the weights are streamed once per 8 tokens by the one-wavefront-per-row
// kernel (row_gemv_nb_kernel).  *launched = false when the matrix has no decode copy or its rows take
// more than one pass per lane: the caller then takes the K-split multi-token kernel on the native bytes.
cera_hip_status cera_launch_row_gemv_nb(cera_hip_ctx* ctx, const cera_hip_dtensor* w, const float* xs, const int8_t* xq,
                                        uint32_t xs_stride, uint32_t xq_stride, uint32_t n_tok, float* y, uint32_t y_stride,
                                        const float* resid, bool* launched) {
    *launched = false;
    if (!w->dev_stream || short_tiles(w->dtype, w->k) != 1 || n_tok == 0 || w->m > (1u << 24)) return CERA_HIP_OK;
    // Measured on the 8B shapes at 8 tokens against the K-split kernel: gate / up 14336 x 4096 23.1 -> 17.3 us, the
    // 128256 x 4096 head 157 -> 115 us; the 4096- and 1024-row matrices are too few workgroups of 32 rows to gain
    // (O 13.2 -> 11.8 us, V 6.4 -> 12.2 us).  Both are bound by the vector ALU's work per (row, token) pair
    // (this kernel: 1073 vector instructions per wavefront for 16 pairs, 16 of each pair's ~55 the v_dot4).
    // (no residual form: the matrices that gain are projections out of the hidden size, not into it)
    if (w->m < 8192 || resid) return CERA_HIP_OK;
    constexpr int NW = 8, ROWS = 4;   // two rows per wavefront measured the same
    RowGemvNbArgs a{};
    a.w = w->dev_stream;
    a.m = static_cast<uint32_t>(w->m);
    a.k = static_cast<uint32_t>(w->k);
    a.row_bytes = static_cast<uint32_t>(w->stream_row_bytes);
    a.xq_stride = xq_stride;
    a.xs_stride = xs_stride;
    a.y_stride = y_stride;
    const dim3 grid((a.m + NW * ROWS - 1) / (NW * ROWS)), block(64 * NW);
    for (uint32_t t0 = 0; t0 < n_tok; t0 += 8) {
        const uint32_t nt = std::min(8u, n_tok - t0);
        a.n_tok = nt;
        a.xq = xq + static_cast<uint64_t>(t0) * xq_stride;
        a.xs = xs + static_cast<uint64_t>(t0) * xs_stride;
        a.y = y + static_cast<uint64_t>(t0) * y_stride;
        a.resid = nullptr;
#define NB_LAUNCH_N(TT, NBV) hipLaunchKernelGGL((row_gemv_nb_kernel<TT, NW, ROWS, FEPI_STORE, true, NBV>), grid, block, 0, ctx->stream, a)
#define NB_LAUNCH(TT)                       \
    do {                                    \
        if (nt <= 2) NB_LAUNCH_N(TT, 2);    \
        else if (nt <= 4) NB_LAUNCH_N(TT, 4); \
        else NB_LAUNCH_N(TT, 8);            \
    } while (0)
        if (w->dtype == CERA_HIP_Q4_K) NB_LAUNCH(Q4K);
        else if (w->dtype == CERA_HIP_Q6_K) NB_LAUNCH(Q6K);
        else if (w->dtype == CERA_HIP_Q4_0) NB_LAUNCH(Q4_0);
        else if (w->dtype == CERA_HIP_Q4_1) NB_LAUNCH(Q4_1);
        else NB_LAUNCH(Q8_0);
#undef NB_LAUNCH
#undef NB_LAUNCH_N
        HIP_TRY(ctx, hipGetLastError());
    }
    *launched = true;
    return CERA_HIP_OK;
}

// ---- kernel-level entry points (host buffers) --------------------------------------------------
extern "C" cera_hip_status cera_hip_ffn_gate_up_fused(cera_hip_ctx* ctx, const cera_hip_tensor* gate, const cera_hip_tensor* up,
                                                      const float* x, const float* norm_w, float eps, int8_t* quants,
                                                      float* scales) {
    if (!ctx || !gate || !up || !x || !norm_w || !quants || !scales) return CERA_HIP_ERR_ARGUMENT;
    std::lock_guard<std::recursive_mutex> lk(ctx->op_mu);
    cera_hip_dtensor *wg = nullptr, *wu = nullptr;
    CERA_TRY(cera_hip_tensor_upload(ctx, gate, &wg));
    cera_hip_status st = cera_hip_tensor_upload(ctx, up, &wu);
    if (st != CERA_HIP_OK) { cera_hip_tensor_free(ctx, wg); return st; }
    auto run = [&]() -> cera_hip_status {
        CERA_TRY(cera_tensor_prepare_stream(ctx, wg));
        CERA_TRY(cera_tensor_prepare_stream(ctx, wu));
        const uint64_t k = wg->k, m = wg->m;
        void *dx, *dw, *dq, *ds;
        CERA_TRY(cera_scratch(ctx, 0, k * 4, &dx));
        CERA_TRY(cera_scratch(ctx, 1, k * 4, &dw));
        CERA_TRY(cera_scratch(ctx, 2, m, &dq));
        CERA_TRY(cera_scratch(ctx, 3, m / 32 * 4 + 4, &ds));
        CERA_TRY(cera_hip_upload(ctx, dx, x, k * 4));
        CERA_TRY(cera_hip_upload(ctx, dw, norm_w, k * 4));
        bool launched = false;
        CERA_TRY(cera_launch_ffn_gate_up_fused(ctx, wg, wu, static_cast<float*>(dx), static_cast<float*>(dw), eps,
                                               static_cast<int8_t*>(dq), static_cast<float*>(ds), &launched));
        if (!launched) return cera_fail(ctx, CERA_HIP_ERR_UNSUPPORTED_DTYPE, "ffn_gate_up_fused: needs two matrices of one fused type and shape, k <= 8192 (Q4_K) or 4096 in whole blocks, m a multiple of 32");
        CERA_TRY(cera_hip_download(ctx, quants, dq, m));
        return cera_hip_download(ctx, scales, ds, m / 32 * 4);
    };
    st = run();
    cera_hip_tensor_free(ctx, wg);
    cera_hip_tensor_free(ctx, wu);
    return st;
}

extern "C" cera_hip_status cera_hip_qkv_fused(cera_hip_ctx* ctx, const cera_hip_tensor* a, const cera_hip_tensor* b, const float* x,
                                              const float* norm_w, float eps, float* ya, float* yb) {
    if (!ctx || !a || !x || !norm_w || !ya || (b && !yb)) return CERA_HIP_ERR_ARGUMENT;
    std::lock_guard<std::recursive_mutex> lk(ctx->op_mu);
    cera_hip_dtensor *wa = nullptr, *wb = nullptr;
    CERA_TRY(cera_hip_tensor_upload(ctx, a, &wa));
    cera_hip_status st = b ? cera_hip_tensor_upload(ctx, b, &wb) : CERA_HIP_OK;
    if (st != CERA_HIP_OK) { cera_hip_tensor_free(ctx, wa); return st; }
    auto run = [&]() -> cera_hip_status {
        CERA_TRY(cera_tensor_prepare_stream(ctx, wa));
        if (wb) CERA_TRY(cera_tensor_prepare_stream(ctx, wb));
        const uint64_t k = wa->k;
        void *dx, *dw, *dy;
        CERA_TRY(cera_scratch(ctx, 0, k * 4, &dx));
        CERA_TRY(cera_scratch(ctx, 1, k * 4, &dw));
        CERA_TRY(cera_scratch(ctx, 3, (wa->m + (wb ? wb->m : 0)) * 4, &dy));
        CERA_TRY(cera_hip_upload(ctx, dx, x, k * 4));
        CERA_TRY(cera_hip_upload(ctx, dw, norm_w, k * 4));
        float *da = static_cast<float*>(dy), *db = da + wa->m;
        bool launched = false;
        CERA_TRY(cera_launch_qkv_fused(ctx, wa, wb, static_cast<float*>(dx), static_cast<float*>(dw), eps, da, db, &launched));
        if (!launched) return cera_fail(ctx, CERA_HIP_ERR_UNSUPPORTED_DTYPE, "qkv_fused: needs Q4_K / Q6_K matrices with k <= 8192 in whole super-blocks (or 32-block types of one kind, k <= 4096)");
        CERA_TRY(cera_hip_download(ctx, ya, da, wa->m * 4));
        if (wb) CERA_TRY(cera_hip_download(ctx, yb, db, wb->m * 4));
        return CERA_HIP_OK;
    };
    st = run();
    cera_hip_tensor_free(ctx, wa);
    if (wb) cera_hip_tensor_free(ctx, wb);
    return st;
}
