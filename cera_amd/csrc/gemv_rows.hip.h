// Decode GEMVs with the neighbouring small operations folded in, for rows that fit one wavefront
// (k <= 4096 with 64-weight units in one pass per lane: the hidden size of the 7-8B models; k <= 8192 in two).
//
// A decode step is a chain of dependent launches, and on this hardware a launch costs about 3 us
// before its first byte arrives, whatever it does.  rmsnorm + Q8_0 quantization of a 4096-vector
// and the Q8_0 quantization of the SwiGLU output are such launches: 16 KB of work each.  Here
//   * the consumer does the norm: every workgroup of the Q|K|V and gate|up projections reads the
//     f32 hidden vector and the norm weights itself (32 KB from L2), reduces the sum of squares,
//     normalizes and quantizes into LDS -- exactly rmsnorm_row_kernel's arithmetic
//     (cpu::rmsnorm + quantize_f32_to_q8_0, cera/src/backend/cpu.rs:2479-2496, 942-958) -- while its
//     first weight rows are already in flight, and its wavefronts take their activations from LDS;
//   * the producer does the SwiGLU quantization: a workgroup owns 32 consecutive rows of gate and
//     up, i.e. one whole Q8_0 block of the down projection's input, and writes its int8 codes and
//     scale (silu_mul_inplace cpu.rs:2570-2575, then cpu.rs:942-958); the f32 vector is never stored.
// A wavefront owns whole rows (one 64-weight unit per lane), walks its rows one at a time with
// the next row's loads in flight, and reduces with DPP only: no LDS combine, no barrier in the
// row loop.  Per-row arithmetic is gemv.hip.h's (T::dot), so results meet the same bars.
//
// This header holds the kernels; gemv_fused.hip holds the launch rules of the library, and the
// standalone code object (lower/cera_hip_gfx950.hip) exports the same bodies under extern "C" names.
#pragma once
#include "gemv.hip.h"
#include "quantize.hip.h"

enum { FEPI_STORE = 0, FEPI_ADD = 1, FEPI_SILU_Q8 = 2 };

struct RowGemvArgs {
    const uint8_t* w;       // [m] rows
    const uint8_t* w2;      // second matrix, same shape (SILU_Q8: w = gate, w2 = up)
    uint32_t m, k, row_bytes, rows_per_wave;
    const int8_t* xq;       // NORM == false: quantized activations
    const float* xs;
    const float* x;         // NORM == true: f32 vector [k] and norm weights [k]
    const float* norm_w;
    float eps;
    float* y;               // STORE / ADD
    const float* resid;
    int8_t* out_q;          // SILU_Q8: [m] int8, [m/32] scales
    float* out_s;
};
struct RowGemvPairArgs {
    RowGemvArgs a, b;       // two matrices over the same activations: workgroups [0, n_blocks_a) take a
    uint32_t n_blocks_a;
};

// rmsnorm + Q8_0 of x[0, k) into LDS by all 64 * NW threads (k % 32 == 0, k <= MAXK), in two steps:
// load() issues the loads of x and the norm weights, finish() does the rest.  The caller issues
// its weight-row loads between the two: the hardware counts outstanding loads in order, so a wait
// for x placed behind the weight loads would wait for every weight row as well.
template <int NW, int MAXK = 4096>
struct NormQuant {
    static constexpr int NT = 64 * NW, MAXIT = (MAXK / 4 + NT - 1) / NT;
    float4 v[MAXIT], g[MAXIT];
    __device__ __forceinline__ void load(const float* __restrict__ x, const float* __restrict__ w, uint32_t k) {
#pragma unroll
        for (int it = 0; it < MAXIT; ++it) {
            const uint32_t i = (threadIdx.x + NT * it) * 4;
            v[it] = make_float4(0.f, 0.f, 0.f, 0.f);
            g[it] = v[it];
            if (i < k) {
                v[it] = *reinterpret_cast<const float4*>(x + i);
                g[it] = *reinterpret_cast<const float4*>(w + i);
            }
        }
    }
    __device__ __forceinline__ void finish(uint32_t k, float eps, uint32_t* s_xq, float* s_xs, double* s_part) {
        double s = 0.0;
#pragma unroll
        for (int it = 0; it < MAXIT; ++it) {   // elements past k are zero
            s += static_cast<double>(v[it].x) * v[it].x;
            s += static_cast<double>(v[it].y) * v[it].y;
            s += static_cast<double>(v[it].z) * v[it].z;
            s += static_cast<double>(v[it].w) * v[it].w;
        }
        s = wave_sum_f64(s);
        if ((threadIdx.x & 63) == 0) s_part[threadIdx.x >> 6] = s;
        lds_barrier();
        double tot = 0.0;
#pragma unroll
        for (int i = 0; i < NW; ++i) tot += s_part[i];
        const float inv = static_cast<float>(1.0 / sqrt(tot / static_cast<double>(k) + static_cast<double>(eps)));
#pragma unroll
        for (int it = 0; it < MAXIT; ++it) {
            const uint32_t i = (threadIdx.x + NT * it) * 4;
            if (i < k) {   // k % 32 == 0: the eight lanes of a block are live together
                float4 o;
                o.x = __fmul_rn(__fmul_rn(v[it].x, inv), g[it].x);
                o.y = __fmul_rn(__fmul_rn(v[it].y, inv), g[it].y);
                o.z = __fmul_rn(__fmul_rn(v[it].z, inv), g[it].z);
                o.w = __fmul_rn(__fmul_rn(v[it].w, inv), g[it].w);
                float sc;
                const uint32_t packed = q8_quantize_quad(o, sc);
                s_xq[i >> 2] = packed;
                if ((threadIdx.x & 7) == 0) s_xs[i >> 5] = sc;
            }
        }
        lds_barrier();
    }
};

// STREAM: p.w / p.w2 point at the matrices' decode copies (T::load_w_stream), p.row_bytes is
// their row stride.
template <class T, int NM, bool STREAM, int TILES>
struct RowTile {
    typename T::Wt w[NM][TILES];
    __device__ __forceinline__ void load_one(const RowGemvArgs& p, int mi, const uint32_t (&unit)[TILES], uint32_t row) {
        const uint8_t* r = (mi == 0 ? p.w : p.w2) + static_cast<uint64_t>(row) * p.row_bytes;
#pragma unroll
        for (int tt = 0; tt < TILES; ++tt) {
            if (STREAM) T::load_w_stream(w[mi][tt], r, unit[tt], p.k / T::ELEMS_PER_UNIT);
            else T::load_w(w[mi][tt], r, unit[tt]);
        }
    }
    __device__ __forceinline__ void load(const RowGemvArgs& p, const uint32_t (&unit)[TILES], uint32_t row) {
#pragma unroll
        for (int mi = 0; mi < NM; ++mi) load_one(p, mi, unit, row);
    }
};

// The work of workgroup `block` on matrix p: wavefront w owns rows (block * NW + w) * ROWS .. + ROWS.
// The first two rows' weight loads are issued before the activations are prepared (NORM: a memory
// round trip for x and the norm weights, an f64 reduction, two barriers), every buffer is
// refilled as soon as its dot product is formed, and the per-row epilogue runs once per
// wavefront with lane i finishing row i.  Every thread of the workgroup must call this (it contains barriers when NORM or
// SILU_Q8), including wavefronts whose row range is empty.
// TILES: units per lane (a row is TILES passes of 64 units: 1 for the K-quants' 64-weight units up
// to k = 4096, 2 for the 32-weight blocks of Q4_0 / Q8_0 beyond k = 2048).  Pass t holds the units
// wavefront t of the K-split kernel holds and the pass totals are added in that order: same bits.
template <class T, int NW, int ROWS, bool NORM, int EPI, bool STREAM, int TILES, int MAXK = 4096>
__device__ __forceinline__ void row_gemv_body(const RowGemvArgs& p, uint32_t block, uint32_t* s_xq, float* s_xs, double* s_part,
                                              float* s_out) {
    constexpr int NM = EPI == FEPI_SILU_Q8 ? 2 : 1;
    const uint32_t lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint32_t n_units = p.k / T::ELEMS_PER_UNIT;
    bool live[TILES];
    uint32_t unit[TILES];
#pragma unroll
    for (int tt = 0; tt < TILES; ++tt) {
        live[tt] = 64 * tt + lane < n_units;
        unit[tt] = live[tt] ? 64 * tt + lane : 0;   // dead lanes re-read unit 0 with zeroed activations
    }
    constexpr int DEPTH = ROWS < 2 ? ROWS : 2;
    const uint32_t r0 = (block * NW + wave) * ROWS;
    auto row_of = [&](int i) -> uint32_t { return r0 + i; };

    NormQuant<NW, MAXK> nq;
    if (NORM) {
        nq.load(p.x, p.norm_w, p.k);
        __builtin_amdgcn_sched_barrier(0);   // x and the norm weights first: they are waited for first
    }
    // DEPTH rows in flight per wavefront: their loads are issued before the activations are
    // prepared, and each finished row's buffer is refilled with the row DEPTH further on
    RowTile<T, NM, STREAM, TILES> t[DEPTH];
#pragma unroll
    for (int i = 0; i < DEPTH; ++i) t[i].load(p, unit, min(row_of(i), p.m - 1));   // rows past the end re-read the last row
    __builtin_amdgcn_sched_barrier(0);   // the loads are issued here, not wherever their first use would pull them

    typename T::Act act[TILES];
    if (NORM) nq.finish(p.k, p.eps, s_xq, s_xs, s_part);
#pragma unroll
    for (int tt = 0; tt < TILES; ++tt) {
        if (NORM) T::load_act(act[tt], reinterpret_cast<const int8_t*>(s_xq), s_xs, unit[tt], live[tt]);
        else T::load_act(act[tt], p.xq, p.xs, unit[tt], live[tt]);
    }

    float tot[ROWS][NM];   // wave-uniform row totals
#pragma unroll
    for (int i = 0; i < ROWS; ++i) {
#pragma unroll
        for (int mi = 0; mi < NM; ++mi) {
            float part[TILES];
#pragma unroll
            for (int tt = 0; tt < TILES; ++tt) part[tt] = T::dot(t[i % DEPTH].w[mi][tt], act[tt], unit[tt], nullptr);
            // the buffer is free as soon as its dots are formed: refill it before the reduction
            if (i + DEPTH < ROWS) {
                __builtin_amdgcn_sched_barrier(0);
                t[i % DEPTH].load_one(p, mi, unit, min(row_of(i + DEPTH), p.m - 1));
                __builtin_amdgcn_sched_barrier(0);
            }
            if (TILES == 1) {
                tot[i][mi] = wave_sum(part[0]);
            } else {
                float sum = 0.0f;
#pragma unroll
                for (int tt = 0; tt < TILES; ++tt) sum += wave_sum(part[tt]);
                tot[i][mi] = sum;
            }
        }
    }
    // epilogue once per wavefront: lane i finishes row i
    {
        float mine[NM];
        uint32_t row = row_of(0);
#pragma unroll
        for (int mi = 0; mi < NM; ++mi) mine[mi] = tot[0][mi];
#pragma unroll
        for (int i = 1; i < ROWS; ++i) {
            if (lane == i) {
                row = row_of(i);
#pragma unroll
                for (int mi = 0; mi < NM; ++mi) mine[mi] = tot[i][mi];
            }
        }
        if (lane < ROWS && row < p.m) {
            if (EPI == FEPI_SILU_Q8) {
                // cera/src/backend/cpu.rs:2570-2575: g / (1 + expf(-g)) * u
                const float g = mine[0];
                s_out[wave * ROWS + lane] = __fmul_rn(__fdiv_rn(g, __fadd_rn(1.0f, cera_expf(-g))), mine[NM - 1]);
            } else {
                p.y[row] = EPI == FEPI_ADD ? p.resid[row] + mine[0] : mine[0];
            }
        }
    }
    if (EPI == FEPI_SILU_Q8) {
        // the workgroup's NW * ROWS rows are whole Q8_0 blocks of the next projection's input
        static_assert(EPI != FEPI_SILU_Q8 || (NW * ROWS) % 32 == 0, "a workgroup must own whole Q8_0 blocks of output rows");
        lds_barrier();
        if (wave == 0) {
            constexpr uint32_t NQ = NW * ROWS / 4;   // float4 groups of the workgroup's rows, 8 per Q8_0 block
            const uint32_t row0 = block * NW * ROWS;
            const bool q_live = lane < NQ && row0 + 4 * lane < p.m;   // m % 32 == 0: a block is whole or absent
            const float4 h = q_live ? reinterpret_cast<const float4*>(s_out)[lane] : make_float4(0.f, 0.f, 0.f, 0.f);
            float sc;
            const uint32_t packed = q8_quantize_quad(h, sc);
            if (q_live) {
                reinterpret_cast<uint32_t*>(p.out_q + row0)[lane] = packed;
                if ((lane & 7) == 0) p.out_s[(row0 + 4 * lane) >> 5] = sc;
            }
        }
    }
}

// MAXK: the longest row the NORM form stages (LDS for its quantized activations)
template <class T, int NW, int ROWS, bool NORM, int EPI, bool STREAM, int TILES = 1, int MAXK = 4096>
static __global__ __launch_bounds__(64 * NW, NW <= 8 ? 2 : 1) void row_gemv_kernel(RowGemvArgs p) {
    __shared__ uint32_t s_xq[NORM ? MAXK / 4 : 1];
    __shared__ float s_xs[NORM ? MAXK / 32 : 1];
    __shared__ double s_part[NW];
    __shared__ __attribute__((aligned(16))) float s_out[EPI == FEPI_SILU_Q8 ? NW * ROWS : 4];
    row_gemv_body<T, NW, ROWS, NORM, EPI, STREAM, TILES, MAXK>(p, blockIdx.x, s_xq, s_xs, s_part, s_out);
}

template <class TA, class TB, int NW, int ROWS, bool NORM, bool STREAM, int TILES = 1, int MAXK = 4096>
static __global__ __launch_bounds__(64 * NW, 2) void row_gemv_pair_kernel(RowGemvPairArgs p) {
    __shared__ uint32_t s_xq[NORM ? MAXK / 4 : 1];
    __shared__ float s_xs[NORM ? MAXK / 32 : 1];
    __shared__ double s_part[NW];
    if (blockIdx.x < p.n_blocks_a) row_gemv_body<TA, NW, ROWS, NORM, FEPI_STORE, STREAM, TILES, MAXK>(p.a, blockIdx.x, s_xq, s_xs, s_part, nullptr);
    else row_gemv_body<TB, NW, ROWS, NORM, FEPI_STORE, STREAM, TILES, MAXK>(p.b, blockIdx.x - p.n_blocks_a, s_xq, s_xs, s_part, nullptr);
}

// Long rows (beyond the short kernels, k <= 32768 for the K-quants: the down projection): still one wavefront per row, walking the
// row in TILES passes of 64 units with every pass's weights requested up front and the activations
// read from LDS pass by pass (a lane cannot keep four passes' activations in registers).  There is
// no K split across wavefronts, so no combine and no barrier after the activations are staged:
// a wavefront's only dependencies are its own loads.  The K-split kernel's workgroup meets at a
// barrier per row group, which costs it most when the weights come from HBM (12.3 us against
// 9.6 us from the last-level cache).  Pass t sees exactly the units wavefront t of the K-split
// kernel sees, and the pass totals are added in wavefront order, so the result has the same bits.
template <class T, int NW, int TILES, int EPI, bool STREAM>
__device__ __forceinline__ void row_gemv_long_body(const RowGemvArgs& p, int8_t* s_xq, float* s_xs) {
    constexpr uint32_t MAX_K = TILES * 64 * T::ELEMS_PER_UNIT;
    const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const uint32_t n_units = p.k / T::ELEMS_PER_UNIT;
    const uint32_t row = blockIdx.x * NW + wave;
    const uint8_t* rp = p.w + static_cast<uint64_t>(min(row, p.m - 1)) * p.row_bytes;
    // activations first (they are waited for first: the load counter is in order), then all weights
    constexpr int XI = (MAX_K / 16 + 64 * NW - 1) / (64 * NW);
    uint4 xv[XI];
#pragma unroll
    for (int i = 0; i < XI; ++i) {
        const uint32_t o = (tid + 64 * NW * i) * 16;
        xv[i] = o < p.k ? *reinterpret_cast<const uint4*>(p.xq + o) : make_uint4(0, 0, 0, 0);
    }
    const uint32_t n_sc = p.k / 32;
    constexpr int SI = (MAX_K / 32 + 64 * NW - 1) / (64 * NW);
    float sv[SI];
#pragma unroll
    for (int i = 0; i < SI; ++i) sv[i] = tid + 64 * NW * i < n_sc ? p.xs[tid + 64 * NW * i] : 0.0f;
    __builtin_amdgcn_sched_barrier(0);
    typename T::Wt w[TILES];
    bool live[TILES];
    uint32_t unit[TILES];
#pragma unroll
    for (int t = 0; t < TILES; ++t) {
        const uint32_t u = 64 * t + lane;
        live[t] = u < n_units;
        unit[t] = live[t] ? u : 0;   // dead lanes re-read unit 0 with zeroed activations
        if (STREAM) T::load_w_stream(w[t], rp, unit[t], n_units);
        else T::load_w(w[t], rp, unit[t]);
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int i = 0; i < XI; ++i) {
        const uint32_t o = (tid + 64 * NW * i) * 16;
        if (o < MAX_K) *reinterpret_cast<uint4*>(s_xq + o) = xv[i];
    }
#pragma unroll
    for (int i = 0; i < SI; ++i)
        if (tid + 64 * NW * i < MAX_K / 32) s_xs[tid + 64 * NW * i] = sv[i];
    lds_barrier();
    float s = 0.0f;
#pragma unroll
    for (int t = 0; t < TILES; ++t) {
        typename T::Act act;
        T::load_act(act, s_xq, s_xs, unit[t], live[t]);
        s += wave_sum(T::dot(w[t], act, unit[t], nullptr));
    }
    if (lane == 0 && row < p.m) p.y[row] = EPI == FEPI_ADD ? p.resid[row] + s : s;
}

template <class T, int NW, int TILES, int EPI, bool STREAM>
static __global__ __launch_bounds__(64 * NW) void row_gemv_long_kernel(RowGemvArgs p) {
    constexpr uint32_t MAX_K = TILES * 64 * T::ELEMS_PER_UNIT;
    __shared__ __attribute__((aligned(16))) int8_t s_xq[MAX_K];
    __shared__ __attribute__((aligned(16))) float s_xs[MAX_K / 32];
    row_gemv_long_body<T, NW, TILES, EPI, STREAM>(p, s_xq, s_xs);
}

// ---- a few tokens per weight pass ---------------------------------------------------------------
// The row kernel above for 2..NB activation vectors at once (short batches: a few new tokens,
// speculative-decoding verification): a wavefront streams its rows once and dots each with every
// token's activations.  Eight tokens' prepared activations (T::Act, 22-24 registers each) do not
// fit a lane's registers at an occupancy that keeps the vector ALU busy, so the workgroup prepares
// them once -- wavefront w the tokens w, w + NW, ... -- and parks them in LDS as 16-byte planes
// [token][quad][lane]; a lane reads its own unit's copy back for every (row, token) pair with
// ds_read_b128, conflict-free (as dword planes the kernel was bound by the LDS instruction rate).  Same units per lane, same T::load_act, T::dot and wave_sum as the single-vector
// kernels, so column b of the result has the bits of a single-vector launch on token b.  One pass
// per lane (k <= 64 units).
struct RowGemvNbArgs {
    const uint8_t* w;       // [m] rows (STREAM: of the decode copy)
    uint32_t m, k, row_bytes;
    const int8_t* xq;       // [n_tok][xq_stride]
    const float* xs;        // [n_tok][xs_stride]
    uint32_t xq_stride, xs_stride;
    uint32_t n_tok;         // live tokens, 1 <= n_tok <= NB (surplus columns repeat the last token and are not stored)
    float* y;               // y[b * y_stride + row]
    const float* resid;     // ADD: same layout as y
    uint32_t y_stride;
};

template <class T, int NW, int ROWS, int EPI, bool STREAM, int NB>
__device__ __forceinline__ void row_gemv_nb_body(const RowGemvNbArgs& p, uint4* s_act) {
    static_assert(ROWS * NB <= 64, "lane i of a wavefront finishes (row, token) pair i");
    constexpr int NA = sizeof(typename T::Act) / 4, NQ = (NA + 3) / 4;   // dwords, 16-byte quads (the last one padded)
    static_assert(sizeof(typename T::Act) % 4 == 0, "the prepared activations are parked as dwords");
    const uint32_t lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint32_t n_units = p.k / T::ELEMS_PER_UNIT;
    const bool live = lane < n_units;
    const uint32_t unit[1] = {live ? lane : 0};   // dead lanes re-read unit 0 with zeroed activations
    constexpr int DEPTH = ROWS < 2 ? ROWS : 2;
    const uint32_t r0 = (blockIdx.x * NW + wave) * ROWS;
    RowGemvArgs g{};
    g.w = p.w; g.m = p.m; g.k = p.k; g.row_bytes = p.row_bytes;
    RowTile<T, 1, STREAM, 1> t[DEPTH];
#pragma unroll
    for (int i = 0; i < DEPTH; ++i) t[i].load(g, unit, min(r0 + i, p.m - 1));   // rows past the end re-read the last row
    __builtin_amdgcn_sched_barrier(0);
    for (uint32_t b = wave; b < NB; b += NW) {   // wavefront-uniform
        const uint32_t tok = min(b, p.n_tok - 1);
        typename T::Act a;
        T::load_act(a, p.xq + static_cast<uint64_t>(tok) * p.xq_stride, p.xs + static_cast<uint64_t>(tok) * p.xs_stride, unit[0], live);
        uint32_t raw[4 * NQ] = {};
        __builtin_memcpy(raw, &a, sizeof(a));
#pragma unroll
        for (int q = 0; q < NQ; ++q) s_act[(b * NQ + q) * 64 + lane] = make_uint4(raw[4 * q], raw[4 * q + 1], raw[4 * q + 2], raw[4 * q + 3]);
    }
    lds_barrier();
    float mine = 0.0f;   // lane i: the total of row i / NB, token i % NB
#pragma unroll
    for (int i = 0; i < ROWS; ++i) {
        float part[NB];
#pragma unroll
        for (int b = 0; b < NB; ++b) {
            uint32_t raw[4 * NQ];
#pragma unroll
            for (int q = 0; q < NQ; ++q) {
                const uint4 v = s_act[(b * NQ + q) * 64 + lane];
                raw[4 * q] = v.x; raw[4 * q + 1] = v.y; raw[4 * q + 2] = v.z; raw[4 * q + 3] = v.w;
            }
            typename T::Act a;
            __builtin_memcpy(&a, raw, sizeof(a));
            part[b] = T::dot(t[i % DEPTH].w[0][0], a, unit[0], nullptr);
            // two tokens' activations in registers at a time: left alone, the scheduler requests all NB
            // tokens' LDS reads first (200+ registers, or spills under a cap)
            if (NB >= 4 && (b & 1)) __builtin_amdgcn_sched_barrier(0);
        }
        if (i + DEPTH < ROWS) {   // the buffer is free as soon as its dots are formed
            __builtin_amdgcn_sched_barrier(0);
            t[i % DEPTH].load_one(g, 0, unit, min(r0 + i + DEPTH, p.m - 1));
            __builtin_amdgcn_sched_barrier(0);
        }
#pragma unroll
        for (int b = 0; b < NB; ++b) {
            const float tot = wave_sum(part[b]);
            if (lane == static_cast<uint32_t>(i * NB + b)) mine = tot;
        }
    }
    const uint32_t row = r0 + lane / NB, b = lane % NB;
    if (lane < ROWS * NB && row < p.m && b < p.n_tok) {
        const uint64_t at = static_cast<uint64_t>(b) * p.y_stride + row;
        p.y[at] = EPI == FEPI_ADD ? p.resid[at] + mine : mine;
    }
}

template <class T, int NW, int ROWS, int EPI, bool STREAM, int NB>
static __global__ __launch_bounds__(64 * NW, 4) void row_gemv_nb_kernel(RowGemvNbArgs p) {
    __shared__ __attribute__((aligned(16))) uint4 s_act[NB * ((sizeof(typename T::Act) / 4 + 3) / 4) * 64];
    row_gemv_nb_body<T, NW, ROWS, EPI, STREAM, NB>(p, s_act);
}

// ---- decode copies ------------------------------------------------------------------------------
// One thread per unit of a row: the unit's bytes from the native block layout to their places in
// the decode copy (T::to_stream).  grid = m workgroups of 256 threads.
template <class T>
__device__ __forceinline__ void stream_rows_body(const uint8_t* __restrict__ src, uint8_t* __restrict__ dst, uint32_t n_units,
                                                 uint32_t row_bytes, uint32_t stream_row_bytes) {
    const uint32_t row = blockIdx.x;
    for (uint32_t u = threadIdx.x; u < n_units; u += blockDim.x)
        T::to_stream(src + static_cast<uint64_t>(row) * row_bytes, dst + static_cast<uint64_t>(row) * stream_row_bytes, u, n_units);
}

template <class T>
static __global__ __launch_bounds__(256) void stream_rows_kernel(const uint8_t* __restrict__ src, uint8_t* __restrict__ dst, uint32_t m,
                                                                 uint32_t n_units, uint32_t row_bytes, uint32_t stream_row_bytes) {
    (void)m;
    stream_rows_body<T>(src, dst, n_units, row_bytes, stream_row_bytes);
}
