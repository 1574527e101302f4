// Decode GEMV kernels, one per GGUF weight type, for gfx950.
//
//   y[m] = W[m, k] . x[k],  W in native GGUF blocks, x pre-quantized to Q8_0.
//
// Arithmetic contract (cera's CPU int8 path, cera/src/backend/simd.rs:
// 4593-4637 Q4_0/Q8_0, :5693-5878 Q4_K, :5893-5976 Q4_1, :5988-6195 Q6_K):
// integer dot of weight codes with int8 activations per 32-element block (16
// for Q6_K), then an f32 epilogue  sum_b xs[b] * (d*sc * dot - dmin*mn * sum a).
// The integer part is exact; only the order of the f32 additions differs from
// the CPU's eight-lane FMA chains.
//
// Design: "activation-stationary lanes".  The K dimension is cut into
// fixed-size *units* (16 B of Q4_K nibbles, 24 B of Q6_K codes, one Q4_0 /
// Q4_1 / Q8_0 block).  Unit u of every row belongs to lane u % 64, so a lane
// keeps the int8 activations, activation scales and activation sums of its
// units in registers for the whole kernel and only streams weights.  A
// wavefront walks a contiguous range of rows, RB rows at a time; for each row
// its 64 lanes read one contiguous span of the row (coalesced 16/8-byte
// loads), so HBM sees pure sequential streams.  Per row the 64 partial sums
// are combined with a DPP reduction.  No LDS, no atomics.
#pragma once
#include "common.cuh"

struct GemvArgs {
    const uint8_t* w;    // [m] rows of native blocks
    const uint8_t* w2;   // second matrix (DUAL: gate/up pair), same shape
    const int8_t* xq;    // [k]
    const float* xs;     // [k/32]
    float* y;            // [m]
    const float* resid;  // EPI_ADD: y = resid + W.x
    uint32_t m;
    uint32_t n_units;        // units per row
    uint32_t row_bytes;
    uint32_t rows_per_wave;
    int32_t* dbg_dots;   // nullable: integer block dots, layout per type
    uint32_t dbg_stride; // ints per row in dbg_dots
    int32_t* dbg_asums;  // nullable: integer activation sums per 32 (Q6_K: per 16)
};

enum { EPI_STORE = 0, EPI_ADD = 1, EPI_SILU_MUL = 2 };

// ---------------------------------------------------------------------------
// Q4_K: unit = 16 bytes of qs (32 nibbles): 16 codes of sub-block 2g (low
// nibbles) and 16 of sub-block 2g+1 (high nibbles); 8 units per 144-byte block.
struct Q4K {
    static constexpr int UNITS_PER_BLOCK = 8;
    struct Act { uint32_t lo[4], hi[4]; float xs0, xs1, c0, c1; int s0, s1; };
    struct Wt { uint4 q; uint4 h; };
    __device__ static void dbg_asum(const Act& a, uint32_t u, int32_t* out) {
        atomicAdd(out + (u >> 3) * 8 + ((u >> 1) & 3) * 2, a.s0);
        atomicAdd(out + (u >> 3) * 8 + ((u >> 1) & 3) * 2 + 1, a.s1);
    }
    __device__ static void load_act(Act& a, const int8_t* xq, const float* xs, uint32_t u, bool live) {
        uint32_t b = u >> 3, w8 = u & 7, g = w8 >> 1, h = w8 & 1;
        const uint32_t* p = reinterpret_cast<const uint32_t*>(xq + b * 256 + g * 64 + h * 16);
        int s0 = 0, s1 = 0;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            a.lo[i] = live ? p[i] : 0u;
            a.hi[i] = live ? p[8 + i] : 0u;
            s0 = sum4(a.lo[i], s0);
            s1 = sum4(a.hi[i], s1);
        }
        a.xs0 = live ? xs[b * 8 + 2 * g] : 0.0f;
        a.xs1 = live ? xs[b * 8 + 2 * g + 1] : 0.0f;
        // xs has an 11-bit significand and |s| <= 16*127: the products are exact.
        a.c0 = a.xs0 * static_cast<float>(s0);
        a.c1 = a.xs1 * static_cast<float>(s1);
        a.s0 = s0;
        a.s1 = s1;
    }
    __device__ static void load_w(Wt& w, const uint8_t* row, uint32_t u) {
        const uint8_t* blk = row + (u >> 3) * 144;
        w.h = ld_u128(blk);
        w.q = ld_u128(blk + 16 + (u & 7) * 16);
    }
    __device__ static float dot(const Wt& w, const Act& a, uint32_t u, int32_t* dbg) {
        uint32_t g = (u >> 1) & 3;
        // 6-bit scales/mins of sub-blocks 2g, 2g+1 (get_scale_min_k4)
        uint32_t sh = 16 * (g & 1);
        uint32_t y2 = (w.h.y >> sh) & 0xFFFF, z2 = (w.h.z >> sh) & 0xFFFF, w2 = (w.h.w >> sh) & 0xFFFF;
        uint32_t sc2 = g < 2 ? (y2 & 0x3F3F) : ((w2 & 0x0F0F) | ((y2 >> 2) & 0x3030));
        uint32_t mn2 = g < 2 ? (z2 & 0x3F3F) : (((w2 >> 4) & 0x0F0F) | ((z2 >> 2) & 0x3030));
        float d = h2f(w.h.x & 0xFFFF), dmin = h2f(w.h.x >> 16);
        int dl = 0, dh = 0;
        const uint32_t q[4] = {w.q.x, w.q.y, w.q.z, w.q.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            dl = dot4(q[i] & 0x0F0F0F0Fu, a.lo[i], dl);
            dh = dot4((q[i] >> 4) & 0x0F0F0F0Fu, a.hi[i], dh);
        }
        if (dbg) {
            atomicAdd(dbg + (u >> 3) * 8 + 2 * g, dl);
            atomicAdd(dbg + (u >> 3) * 8 + 2 * g + 1, dh);
        }
        float s = (static_cast<float>(sc2 & 0xFF) * a.xs0) * static_cast<float>(dl);
        s = fmaf(static_cast<float>(sc2 >> 8) * a.xs1, static_cast<float>(dh), s);
        float mm = static_cast<float>(mn2 & 0xFF) * a.c0;
        mm = fmaf(static_cast<float>(mn2 >> 8), a.c1, mm);
        return fmaf(d, s, -(dmin * mm));
    }
};

// ---------------------------------------------------------------------------
// Q6_K: unit = 8 consecutive positions l0..l0+7 of one 128-element half:
// 8 B of ql (low half), 8 B of ql (+32), 8 B of qh -> 32 six-bit codes in four
// runs of 8 (elements +0, +32, +64, +96); 8 units per 210-byte block.
struct Q6K {
    static constexpr int UNITS_PER_BLOCK = 8;
    struct Act { uint32_t a[4][2]; float xs[4]; int init[4]; };
    struct Wt { uint2 qa, qb, qh, sc; uint32_t d; };
    __device__ static void dbg_asum(const Act& a, uint32_t u, int32_t* out) {
        uint32_t base = (u >> 3) * 16 + ((u >> 2) & 1) * 8 + ((u >> 1) & 1);
#pragma unroll
        for (int t = 0; t < 4; ++t) atomicAdd(out + base + 2 * t, a.init[t] / -32);
    }
    __device__ static void load_act(Act& a, const int8_t* xq, const float* xs, uint32_t u, bool live) {
        uint32_t b = u >> 3, nh = (u >> 2) & 1, j = u & 3;
        const int8_t* base = xq + b * 256 + nh * 128 + j * 8;
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            const uint32_t* p = reinterpret_cast<const uint32_t*>(base + 32 * t);
            a.a[t][0] = live ? p[0] : 0u;
            a.a[t][1] = live ? p[1] : 0u;
            a.xs[t] = live ? xs[b * 8 + nh * 4 + t] : 0.0f;
            // codes are stored +32: start each dot at -32 * sum(a)
            a.init[t] = -32 * sum4(a.a[t][1], sum4(a.a[t][0], 0));
        }
    }
    __device__ static void load_w(Wt& w, const uint8_t* row, uint32_t u) {
        const uint8_t* blk = row + (u >> 3) * 210;
        uint32_t nh = (u >> 2) & 1, j = u & 3;
        w.qa = ld_u64_a2(blk + nh * 64 + j * 8);
        w.qb = ld_u64_a2(blk + nh * 64 + 32 + j * 8);
        w.qh = ld_u64_a2(blk + 128 + nh * 32 + j * 8);
        w.sc = ld_u64_a2(blk + 192 + nh * 8);
        w.d = ld_u16(blk + 208);
    }
    __device__ static float dot(const Wt& w, const Act& a, uint32_t u, int32_t* dbg) {
        uint32_t is = (u >> 1) & 1;  // (l0 / 16) with l0 = 8 * (u & 3)
        int acc[4] = {a.init[0], a.init[1], a.init[2], a.init[3]};
        const uint32_t qa[2] = {w.qa.x, w.qa.y}, qb[2] = {w.qb.x, w.qb.y}, qh[2] = {w.qh.x, w.qh.y};
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            uint32_t q0 = (qa[i] & 0x0F0F0F0Fu) | ((qh[i] << 4) & 0x30303030u);
            uint32_t q1 = (qb[i] & 0x0F0F0F0Fu) | ((qh[i] << 2) & 0x30303030u);
            uint32_t q2 = ((qa[i] >> 4) & 0x0F0F0F0Fu) | (qh[i] & 0x30303030u);
            uint32_t q3 = ((qb[i] >> 4) & 0x0F0F0F0Fu) | ((qh[i] >> 2) & 0x30303030u);
            acc[0] = dot4(q0, a.a[0][i], acc[0]);
            acc[1] = dot4(q1, a.a[1][i], acc[1]);
            acc[2] = dot4(q2, a.a[2][i], acc[2]);
            acc[3] = dot4(q3, a.a[3][i], acc[3]);
        }
        if (dbg) {
            // report the unsigned dot (sum q*a, q in 0..63) per 16-element run
            uint32_t base = (u >> 3) * 16 + ((u >> 2) & 1) * 8 + is;
#pragma unroll
            for (int t = 0; t < 4; ++t) atomicAdd(dbg + base + 2 * t, acc[t] - a.init[t]);
        }
        // scales nh*8 + is + {0, 2, 4, 6}: bytes is, is+2 of each dword
        uint32_t slo = w.sc.x >> (8 * is), shi = w.sc.y >> (8 * is);
        float s0 = static_cast<float>(static_cast<int8_t>(slo & 0xFF));
        float s1 = static_cast<float>(static_cast<int8_t>((slo >> 16) & 0xFF));
        float s2 = static_cast<float>(static_cast<int8_t>(shi & 0xFF));
        float s3 = static_cast<float>(static_cast<int8_t>((shi >> 16) & 0xFF));
        float s = (s0 * a.xs[0]) * static_cast<float>(acc[0]);
        s = fmaf(s1 * a.xs[1], static_cast<float>(acc[1]), s);
        s = fmaf(s2 * a.xs[2], static_cast<float>(acc[2]), s);
        s = fmaf(s3 * a.xs[3], static_cast<float>(acc[3]), s);
        return h2f(w.d) * s;
    }
};

// ---------------------------------------------------------------------------
// 32-element block formats: unit = one block.
struct ActB32 { uint32_t a[8]; float xs; int asum; };
__device__ __forceinline__ void dbg_asum_b32(const ActB32& a, uint32_t u, int32_t* out) { out[u] = a.asum; }
__device__ __forceinline__ void load_act_b32(ActB32& a, const int8_t* xq, const float* xs, uint32_t u, bool live) {
    const uint32_t* p = reinterpret_cast<const uint32_t*>(xq + u * 32);
    int s = 0;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        a.a[i] = live ? p[i] : 0u;
        s = sum4(a.a[i], s);
    }
    a.xs = live ? xs[u] : 0.0f;
    a.asum = s;
}

struct Q4_0 {  // 18 B: d, qs[16]; byte i = element i (low nibble), element i+16 (high); code - 8
    static constexpr int UNITS_PER_BLOCK = 1;
    using Act = ActB32;
    __device__ static void dbg_asum(const Act& a, uint32_t u, int32_t* out) { dbg_asum_b32(a, u, out); }
    struct Wt { uint4 q; uint32_t d; };
    __device__ static void load_act(Act& a, const int8_t* xq, const float* xs, uint32_t u, bool live) {
        load_act_b32(a, xq, xs, u, live);
    }
    __device__ static void load_w(Wt& w, const uint8_t* row, uint32_t u) {
        const uint8_t* blk = row + u * 18;
        w.d = ld_u16(blk);
        w.q = ld_u128_a2(blk + 2);
    }
    __device__ static float dot(const Wt& w, const Act& a, uint32_t u, int32_t* dbg) {
        int acc = -8 * a.asum;
        const uint32_t q[4] = {w.q.x, w.q.y, w.q.z, w.q.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            acc = dot4(q[i] & 0x0F0F0F0Fu, a.a[i], acc);
            acc = dot4((q[i] >> 4) & 0x0F0F0F0Fu, a.a[4 + i], acc);
        }
        if (dbg) dbg[u] = acc;
        return (h2f(w.d) * a.xs) * static_cast<float>(acc);
    }
};

struct Q4_1 {  // 20 B: d, m, qs[16]; value = q*d + m
    static constexpr int UNITS_PER_BLOCK = 1;
    using Act = ActB32;
    __device__ static void dbg_asum(const Act& a, uint32_t u, int32_t* out) { dbg_asum_b32(a, u, out); }
    struct Wt { uint4 q; uint32_t dm; };
    __device__ static void load_act(Act& a, const int8_t* xq, const float* xs, uint32_t u, bool live) {
        load_act_b32(a, xq, xs, u, live);
    }
    __device__ static void load_w(Wt& w, const uint8_t* row, uint32_t u) {
        const uint8_t* blk = row + u * 20;
        w.dm = *reinterpret_cast<const uint32_t*>(blk);
        w.q = ld_u128_a4(blk + 4);
    }
    __device__ static float dot(const Wt& w, const Act& a, uint32_t u, int32_t* dbg) {
        int acc = 0;
        const uint32_t q[4] = {w.q.x, w.q.y, w.q.z, w.q.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            acc = dot4(q[i] & 0x0F0F0F0Fu, a.a[i], acc);
            acc = dot4((q[i] >> 4) & 0x0F0F0F0Fu, a.a[4 + i], acc);
        }
        if (dbg) dbg[u] = acc;
        float d = h2f(w.dm & 0xFFFF), mn = h2f(w.dm >> 16);
        return a.xs * fmaf(d, static_cast<float>(acc), mn * static_cast<float>(a.asum));
    }
};

struct Q8_0 {  // 34 B: d, int8[32]
    static constexpr int UNITS_PER_BLOCK = 1;
    using Act = ActB32;
    __device__ static void dbg_asum(const Act& a, uint32_t u, int32_t* out) { dbg_asum_b32(a, u, out); }
    struct Wt { uint4 q0, q1; uint32_t d; };
    __device__ static void load_act(Act& a, const int8_t* xq, const float* xs, uint32_t u, bool live) {
        load_act_b32(a, xq, xs, u, live);
    }
    __device__ static void load_w(Wt& w, const uint8_t* row, uint32_t u) {
        const uint8_t* blk = row + u * 34;
        w.d = ld_u16(blk);
        w.q0 = ld_u128_a2(blk + 2);
        w.q1 = ld_u128_a2(blk + 18);
    }
    __device__ static float dot(const Wt& w, const Act& a, uint32_t u, int32_t* dbg) {
        int acc = 0;
        const uint32_t q[8] = {w.q0.x, w.q0.y, w.q0.z, w.q0.w, w.q1.x, w.q1.y, w.q1.z, w.q1.w};
#pragma unroll
        for (int i = 0; i < 8; ++i) acc = dot4(q[i], a.a[i], acc);
        if (dbg) dbg[u] = acc;
        return (h2f(w.d) * a.xs) * static_cast<float>(acc);
    }
};

// ---------------------------------------------------------------------------
// The kernel.  U = units per lane held in registers (ceil(n_units / 64)),
// RB = rows in flight per wavefront, EPI = epilogue.
template <class T, int U, int RB, int EPI, bool DBG>
static __global__ __launch_bounds__(256) void gemv_kernel(GemvArgs p) {
    const uint32_t lane = threadIdx.x & 63;
    const uint32_t wave = (blockIdx.x * blockDim.x + threadIdx.x) >> 6;
    uint32_t r0 = wave * p.rows_per_wave;
    if (r0 >= p.m) return;
    uint32_t r1 = min(p.m, r0 + p.rows_per_wave);

    typename T::Act act[U];
    uint32_t unit[U];
#pragma unroll
    for (int i = 0; i < U; ++i) {
        uint32_t u = lane + 64 * i;
        bool live = u < p.n_units;
        unit[i] = live ? u : 0;  // dead lanes re-read unit 0 with zeroed activations
        T::load_act(act[i], p.xq, p.xs, unit[i], live);
        if (DBG && wave == 0 && live && p.dbg_asums) T::dbg_asum(act[i], u, p.dbg_asums);
    }

    constexpr int NM = EPI == EPI_SILU_MUL ? 2 : 1;
    for (uint32_t r = r0; r < r1; r += RB) {
        typename T::Wt wt[NM][RB][U];
#pragma unroll
        for (int mi = 0; mi < NM; ++mi) {
            const uint8_t* base = mi == 0 ? p.w : p.w2;
#pragma unroll
            for (int rb = 0; rb < RB; ++rb) {
                uint32_t row = min(r + rb, r1 - 1);
                const uint8_t* rp = base + static_cast<uint64_t>(row) * p.row_bytes;
#pragma unroll
                for (int i = 0; i < U; ++i) T::load_w(wt[mi][rb][i], rp, unit[i]);
            }
        }
#pragma unroll
        for (int rb = 0; rb < RB; ++rb) {
            uint32_t row = r + rb;
            float tot[NM];
#pragma unroll
            for (int mi = 0; mi < NM; ++mi) {
                float acc = 0.0f;
#pragma unroll
                for (int i = 0; i < U; ++i) {
                    int32_t* dbg = nullptr;
                    if (DBG) dbg = (lane + 64 * i < p.n_units && row < r1)
                                       ? p.dbg_dots + static_cast<uint64_t>(row) * p.dbg_stride : nullptr;
                    acc += T::dot(wt[mi][rb][i], act[i], unit[i], dbg);
                }
                tot[mi] = wave_sum(acc);
            }
            if (lane == 0 && row < r1) {
                float v = tot[0];
                if (EPI == EPI_ADD) v = p.resid[row] + v;
                if (EPI == EPI_SILU_MUL) {
                    // cera/src/backend/cpu.rs:2570-2575: g / (1 + expf(-g)) * u
                    float g = tot[0], up = tot[NM - 1];
                    v = __fmul_rn(__fdiv_rn(g, __fadd_rn(1.0f, cera_expf(-g))), up);
                }
                p.y[row] = v;
            }
        }
    }
}

// ---------------------------------------------------------------------------
// Q5_K: cera's CPU path dots Q5_K rows against the *unquantized* f32
// activations (cera/src/backend/cpu.rs:1830-1854, cera/src/quant.rs:892-937),
// so this kernel does too: dequantize in registers, f32 FMA.  One wavefront
// per row; lane l owns bytes 2l, 2l+1 of each 32-byte qs chunk.
static __global__ __launch_bounds__(256) void gemv_q5k_f32_kernel(const uint8_t* __restrict__ w,
                                                           const float* __restrict__ x,
                                                           float* __restrict__ y, uint32_t m, uint32_t k) {
    const uint32_t lane = threadIdx.x & 63;
    const uint32_t row = (blockIdx.x * blockDim.x + threadIdx.x) >> 6;
    if (row >= m) return;
    const uint32_t nb = k / 256;
    const uint8_t* rp = w + static_cast<uint64_t>(row) * nb * 176;
    float acc = 0.0f;
    // lane -> (chunk j = lane / 16, byte pair p = lane % 16) of each block
    const uint32_t j = lane >> 4, l0 = (lane & 15) * 2;
    for (uint32_t b = 0; b < nb; ++b) {
        const uint8_t* blk = rp + b * 176;
        uint32_t dd = *reinterpret_cast<const uint32_t*>(blk);
        float d = h2f(dd & 0xFFFF), dmin = h2f(dd >> 16);
        const uint8_t* s = blk + 4;
        uint32_t sc[2], mn[2];
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            uint32_t idx = 2 * j + h;
            if (idx < 4) {
                sc[h] = s[idx] & 63;
                mn[h] = s[idx + 4] & 63;
            } else {
                sc[h] = (s[idx + 4] & 0xF) | ((s[idx - 4] >> 6) << 4);
                mn[h] = (s[idx + 4] >> 4) | ((s[idx] >> 6) << 4);
            }
        }
        uint32_t qh = *reinterpret_cast<const uint16_t*>(blk + 16 + l0);
        uint32_t qs = *reinterpret_cast<const uint16_t*>(blk + 48 + 32 * j + l0);
        const float* xb = x + b * 256 + 64 * j + l0;
        float d1 = d * static_cast<float>(sc[0]), m1 = dmin * static_cast<float>(mn[0]);
        float d2 = d * static_cast<float>(sc[1]), m2 = dmin * static_cast<float>(mn[1]);
#pragma unroll
        for (int e = 0; e < 2; ++e) {
            uint32_t qb = (qs >> (8 * e)) & 0xFF, hb = (qh >> (8 * e)) & 0xFF;
            float q1 = static_cast<float>((qb & 0xF) + (((hb >> (2 * j)) & 1) << 4));
            float q2 = static_cast<float>((qb >> 4) + (((hb >> (2 * j + 1)) & 1) << 4));
            acc = fmaf(fmaf(d1, q1, -m1), xb[e], acc);
            acc = fmaf(fmaf(d2, q2, -m2), xb[32 + e], acc);
        }
    }
    acc = wave_sum(acc);
    if (lane == 0) y[row] = acc;
}
