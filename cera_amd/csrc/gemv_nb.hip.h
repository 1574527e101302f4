// Decode GEMV for a handful of tokens at once (2..8 activation vectors): the weights are
// streamed once and every row is dotted with each token's Q8_0 activations.  Same lanes, same
// units, same per-row arithmetic and reduction order as gemv_kernel with one unit per lane, so
// column b of the result is bit-identical to the single-vector kernel run on token b.  Used by
// the prefill path for short batches (a few new tokens, speculative-decoding verification),
// where an int8-MFMA tile would be mostly empty and one GEMV per token would re-read the weights.
#pragma once
#include "gemv.hip.h"

struct GemvNbArgs {
    const uint8_t* w;     // [m] rows of native blocks
    const int8_t* xq;     // [n_tok][xq_stride]
    const float* xs;      // [n_tok][xs_stride]
    float* y;             // y[b * y_stride + row]
    const float* resid;   // ADD: y = resid + W.x, same layout as y
    uint32_t m, n_units, row_bytes, rows_per_block;
    uint32_t n_tok;       // live tokens, 1 <= n_tok <= NB
    uint32_t xq_stride, xs_stride, y_stride;
};

template <class T, int KS, int RB, int NB, bool ADD>
static __global__ __launch_bounds__(64 * KS) void gemv_nb_kernel(GemvNbArgs p) {
    __shared__ float part[2][RB][NB][KS * 4];
    const uint32_t lane = threadIdx.x & 63, kw = threadIdx.x >> 6;
    uint32_t r = blockIdx.x * p.rows_per_block;
    if (r >= p.m) return;
    const uint32_t r1 = min(p.m, r + p.rows_per_block);
    const uint32_t u0 = kw * 64 + lane;
    const bool live1 = u0 < p.n_units;
    const uint32_t unit[1] = {live1 ? u0 : 0};   // dead lanes re-read unit 0 with zeroed activations

    GemvArgs g{};                                // what GemvTile::load reads
    g.w = p.w;
    g.row_bytes = p.row_bytes;
    GemvTile<T, 1, RB, 1> ta, tb;
    ta.load(g, unit, r, r1);

    typename T::Act act[NB];
#pragma unroll
    for (int b = 0; b < NB; ++b) {
        const uint32_t tok = min(static_cast<uint32_t>(b), p.n_tok - 1);   // surplus columns repeat the last token
        T::load_act(act[b], p.xq + static_cast<uint64_t>(tok) * p.xq_stride, p.xs + static_cast<uint64_t>(tok) * p.xs_stride,
                    unit[0], live1);
    }

    auto store = [&](uint32_t row, uint32_t b, float v) {
        const uint64_t at = static_cast<uint64_t>(b) * p.y_stride + row;
        if (ADD) v = p.resid[at] + v;
        p.y[at] = v;
    };
    auto compute = [&](const GemvTile<T, 1, RB, 1>& t, uint32_t rr, float (*pt)[NB][KS * 4]) {
#pragma unroll
        for (int rb = 0; rb < RB; ++rb) {
            const uint32_t row = rr + rb;
#pragma unroll
            for (int b = 0; b < NB; ++b) {
                float acc = 0.0f;
                acc += T::dot(t.w[0][rb][0], act[b], unit[0], nullptr);
                const float tot = KS == 1 ? wave_sum(acc) : wave_row_sum(acc);
                if (KS == 1) {
                    if (lane == 0 && row < r1 && static_cast<uint32_t>(b) < p.n_tok) store(row, b, tot);
                } else if ((lane & 15) == 0) {
                    pt[rb][b][kw * 4 + (lane >> 4)] = tot;
                }
            }
        }
        if (KS > 1) {
            lds_barrier();
            if (threadIdx.x < RB * NB) {
                const uint32_t rb = threadIdx.x / NB, b = threadIdx.x % NB;
                if (rr + rb < r1 && b < p.n_tok) {
                    float s = 0.0f;
#pragma unroll
                    for (int w = 0; w < KS; ++w) {   // wavefront order, rows paired as wave_sum pairs them
                        const float* q4 = &pt[rb][b][4 * w];
                        s += (q4[0] + q4[1]) + (q4[2] + q4[3]);
                    }
                    store(rr + rb, b, s);
                }
            }
        }
    };
    float (*part0)[NB][KS * 4] = KS == 1 ? nullptr : part[0];
    float (*part1)[NB][KS * 4] = KS == 1 ? nullptr : part[1];
    for (;;) {
        if (r + RB >= r1) {
            compute(ta, r, part0);
            break;
        }
        tb.load(g, unit, r + RB, r1);
        compute(ta, r, part0);
        r += RB;
        if (r + RB >= r1) {
            compute(tb, r, part1);
            break;
        }
        ta.load(g, unit, r + RB, r1);
        compute(tb, r, part1);
        r += RB;
    }
}

// Host-side dispatch over (KS, RB, NB, ADD) for one weight type.
template <class T, int KS, int RB>
static bool gemv_nb_launch_nb(const GemvNbArgs& a, int NB, bool add, dim3 grid, hipStream_t s) {
    const dim3 block(64 * KS);
#define NBCASE(N)                                                                                              \
    if (NB == N) {                                                                                             \
        if (add) hipLaunchKernelGGL((gemv_nb_kernel<T, KS, RB, N, true>), grid, block, 0, s, a);               \
        else hipLaunchKernelGGL((gemv_nb_kernel<T, KS, RB, N, false>), grid, block, 0, s, a);                  \
        return true;                                                                                           \
    }
    NBCASE(2) NBCASE(4) NBCASE(8)
#undef NBCASE
    return false;
}
template <class T>
static bool gemv_nb_launch_t(const GemvNbArgs& a, int KS, int RB, int NB, bool add, uint32_t n_blocks, hipStream_t s) {
    const dim3 grid(n_blocks);
#define KCASE(K)                                                                         \
    if (KS == K) {                                                                       \
        if (RB == 1) return gemv_nb_launch_nb<T, K, 1>(a, NB, add, grid, s);             \
        return gemv_nb_launch_nb<T, K, 2>(a, NB, add, grid, s);                          \
    }
    KCASE(1) KCASE(2) KCASE(4) KCASE(8)
#undef KCASE
    return false;
}
