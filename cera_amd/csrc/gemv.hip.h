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
// fixed-size *units* (32 B of Q4_K nibbles, 48 B of Q6_K codes, one Q4_0 /
// Q4_1 / Q8_0 block).  A workgroup is KS wavefronts that split K between them:
// wavefront kw owns units kw*64 .. kw*64+63 (+ 64*KS*i for i < U), one per
// lane, so a lane keeps the int8 activations, activation scales and activation
// sums of its units in registers for the whole kernel and only streams weights.
// The workgroup walks a contiguous range of rows, RB rows at a time; for each
// row its lanes read one contiguous span of the row (coalesced 16/8-byte
// loads), so HBM sees pure sequential streams.  Per row each wavefront reduces
// its 64 partial sums with DPP; the KS per-wavefront sums meet in LDS and are
// added in wavefront order (deterministic, no atomics).
#pragma once
#include "common.hip.h"

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
    uint32_t rows_per_wave;  // rows per workgroup
    int32_t* dbg_dots;   // nullable: integer block dots, layout per type
    uint32_t dbg_stride; // ints per row in dbg_dots
    int32_t* dbg_asums;  // nullable: integer activation sums per 32 (Q6_K: per 16)
};

enum { EPI_STORE = 0, EPI_ADD = 1, EPI_SILU_MUL = 2 };

// ---------------------------------------------------------------------------
// Q4_K: unit = 32 bytes of qs -- one whole chunk g of a 144-byte block, i.e. ALL 32 codes of
// sub-block 2g (low nibbles) and all 32 of sub-block 2g+1 (high nibbles); 4 units per block.
// The per-sub-block work (6-bit scale/min decode, the f32 scale algebra, the row reduction and
// the header load) is paid once per 64 weights: a unit of 16 bytes (half of each sub-block, the
// two halves in neighbouring lanes) needed about half as many VALU instructions again per byte
// and streamed 8 % slower (5.3 against 5.8 TB/s on long matrices).  A 4096-wide row is exactly
// one wavefront: no LDS combine, no barrier.
struct Q4K {
    static constexpr int ELEMS_PER_UNIT = 64;
    struct Act { uint32_t lo[8], hi[8]; float xs0, xs1, c0, c1; int s0, s1; };
    struct Wt { uint4 q0, q1; uint4 h; };
    __device__ static void dbg_asum(const Act& a, uint32_t u, int32_t* out) {
        out[(u >> 2) * 8 + (u & 3) * 2] = a.s0;
        out[(u >> 2) * 8 + (u & 3) * 2 + 1] = a.s1;
    }
    __device__ static void load_act(Act& a, const int8_t* xq, const float* xs, uint32_t u, bool live) {
        const uint32_t b = u >> 2, g = u & 3;
        const uint4* p = reinterpret_cast<const uint4*>(xq + b * 256 + g * 64);
        const uint4 l0 = p[0], l1 = p[1], h0 = p[2], h1 = p[3];
        const float2 sc = *reinterpret_cast<const float2*>(xs + b * 8 + 2 * g);
        const uint32_t keep = live ? 0xFFFFFFFFu : 0u;
        const uint32_t lv[8] = {l0.x, l0.y, l0.z, l0.w, l1.x, l1.y, l1.z, l1.w};
        const uint32_t hv[8] = {h0.x, h0.y, h0.z, h0.w, h1.x, h1.y, h1.z, h1.w};
        int s0 = 0, s1 = 0;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            a.lo[i] = lv[i] & keep;
            a.hi[i] = hv[i] & keep;
            s0 = sum4(a.lo[i], s0);
            s1 = sum4(a.hi[i], s1);
        }
        a.xs0 = live ? sc.x : 0.0f;
        a.xs1 = live ? sc.y : 0.0f;
        a.c0 = a.xs0 * static_cast<float>(s0);   // exact: 11-bit significand x |s| <= 32*127
        a.c1 = a.xs1 * static_cast<float>(s1);
        a.s0 = s0;
        a.s1 = s1;
    }
    __device__ static void load_w(Wt& w, const uint8_t* row, uint32_t u) {
        const uint8_t* blk = row + (u >> 2) * 144;
        w.h = ld_u128(blk);
        w.q0 = ld_u128(blk + 16 + (u & 3) * 32);
        w.q1 = ld_u128(blk + 32 + (u & 3) * 32);
    }
    // The decode copy of a row (see stream_rows_kernel): the row's bytes permuted into planes --
    // every block's 16-byte header, then every unit's first 16 quant bytes, then every unit's
    // second 16, each plane padded to whole 128-byte lines -- so that each of the three loads of a
    // wavefront reads consecutive bytes, whole lines, once: the shape the non-temporal hint needs.
    static constexpr uint32_t up128(uint32_t b) { return (b + 127u) & ~127u; }
    static constexpr uint32_t stream_q0(uint32_t n_units) { return up128(4 * n_units); }
    static constexpr uint32_t stream_q1(uint32_t n_units) { return stream_q0(n_units) + up128(16 * n_units); }
    static constexpr uint32_t stream_row_bytes(uint32_t k) { return stream_q1(k / 64) + up128(16 * (k / 64)); }
    __device__ static void load_w_stream(Wt& w, const uint8_t* row, uint32_t u, uint32_t n_units) {
        w.h = ld_u128_nt(row + (u >> 2) * 16);
        w.q0 = ld_u128_nt(row + stream_q0(n_units) + u * 16);
        w.q1 = ld_u128_nt(row + stream_q1(n_units) + u * 16);
    }
    __device__ static void to_stream(const uint8_t* row, uint8_t* dst, uint32_t u, uint32_t n_units) {
        const uint8_t* blk = row + (u >> 2) * 144;
        if ((u & 3) == 0) *reinterpret_cast<uint4*>(dst + (u >> 2) * 16) = ld_u128(blk);
        *reinterpret_cast<uint4*>(dst + stream_q0(n_units) + u * 16) = ld_u128(blk + 16 + (u & 3) * 32);
        *reinterpret_cast<uint4*>(dst + stream_q1(n_units) + u * 16) = ld_u128(blk + 32 + (u & 3) * 32);
    }
    __device__ static float dot(const Wt& w, const Act& a, uint32_t u, int32_t* dbg) {
        const uint32_t g = u & 3;
        const uint32_t sh = 16 * (g & 1);
        const bool low = g < 2;
        const uint32_t sh_a = low ? sh : sh + 2, m_a = low ? 0x3F3Fu : 0x3030u, m_b = low ? 0u : 0x0F0Fu;
        const uint32_t sc2 = ((w.h.y >> sh_a) & m_a) | ((w.h.w >> sh) & m_b);
        const uint32_t mn2 = ((w.h.z >> sh_a) & m_a) | ((w.h.w >> (sh + 4)) & m_b);
        const float d = h2f(w.h.x & 0xFFFF), dmin = h2f(w.h.x >> 16);
        int dl = 0, dh = 0;
        const uint32_t q[8] = {w.q0.x, w.q0.y, w.q0.z, w.q0.w, w.q1.x, w.q1.y, w.q1.z, w.q1.w};
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            dl = dot4(q[i] & 0x0F0F0F0Fu, a.lo[i], dl);
            dh = dot4((q[i] >> 4) & 0x0F0F0F0Fu, a.hi[i], dh);
        }
        if (dbg) {
            dbg[(u >> 2) * 8 + 2 * g] = dl;
            dbg[(u >> 2) * 8 + 2 * g + 1] = dh;
        }
        float s = (static_cast<float>(sc2 & 0xFF) * a.xs0) * static_cast<float>(dl);
        s = fmaf(static_cast<float>(sc2 >> 8) * a.xs1, static_cast<float>(dh), s);
        float mm = static_cast<float>(mn2 & 0xFF) * a.c0;
        mm = fmaf(static_cast<float>(mn2 >> 8), a.c1, mm);
        return fmaf(d, s, -(dmin * mm));
    }
};

// ---------------------------------------------------------------------------
// Q6_K: unit = 16 consecutive positions l0..l0+15 of one 128-element half:
// 16 B of ql (low half), 16 B of ql (+32), 16 B of qh -> 64 six-bit codes in
// four runs of 16 (elements +0, +32, +64, +96), each run with its own int8
// scale; 4 units per 210-byte block.  Blocks are only 2-byte aligned.
struct Q6K {
    static constexpr int ELEMS_PER_UNIT = 64;
    struct Act { uint32_t a[4][4]; float xs[4]; int init[4]; };
    struct Wt { uint4 qa, qb, qh; uint2 sc; uint32_t d; };
    __device__ static void dbg_asum(const Act& a, uint32_t u, int32_t* out) {
        uint32_t base = (u >> 2) * 16 + ((u >> 1) & 1) * 8 + (u & 1);
#pragma unroll
        for (int t = 0; t < 4; ++t) out[base + 2 * t] = a.init[t] / -32;
    }
    __device__ static void load_act(Act& a, const int8_t* xq, const float* xs, uint32_t u, bool live) {
        uint32_t b = u >> 2, nh = (u >> 1) & 1, j = u & 1;
        const int8_t* base = xq + b * 256 + nh * 128 + j * 16;
        const float4 sc = *reinterpret_cast<const float4*>(xs + b * 8 + nh * 4);
        const float scv[4] = {sc.x, sc.y, sc.z, sc.w};
        const uint32_t keep = live ? 0xFFFFFFFFu : 0u;
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            const uint4 v = *reinterpret_cast<const uint4*>(base + 32 * t);
            a.a[t][0] = v.x & keep; a.a[t][1] = v.y & keep; a.a[t][2] = v.z & keep; a.a[t][3] = v.w & keep;
            a.xs[t] = live ? scv[t] : 0.0f;
            // codes are stored +32: start each dot at -32 * sum(a)
            a.init[t] = -32 * sum4(a.a[t][3], sum4(a.a[t][2], sum4(a.a[t][1], sum4(a.a[t][0], 0))));
        }
    }
    __device__ static void load_w(Wt& w, const uint8_t* row, uint32_t u) {
        const uint8_t* blk = row + (u >> 2) * 210;
        uint32_t nh = (u >> 1) & 1, j = u & 1;
        w.qa = ld_u128_a2(blk + nh * 64 + j * 16);
        w.qb = ld_u128_a2(blk + nh * 64 + 32 + j * 16);
        w.qh = ld_u128_a2(blk + 128 + nh * 32 + j * 16);
        w.sc = ld_u64_a2(blk + 192 + nh * 8);
        w.d = ld_u16(blk + 208);
    }
    // The decode copy of a row: planes of the units' three 16-byte runs (ql low, ql + 32, qh),
    // then the scales (8 bytes per half block) and the block scales d, every plane padded to
    // whole 128-byte lines.  The three big planes are read once, non-temporally; the small ones
    // are shared by neighbouring lanes and passes and stay ordinary loads.
    static constexpr uint32_t up128(uint32_t b) { return (b + 127u) & ~127u; }
    static constexpr uint32_t stream_sc(uint32_t n_units) { return 3 * up128(16 * n_units); }
    static constexpr uint32_t stream_d(uint32_t n_units) { return stream_sc(n_units) + up128(4 * n_units); }
    static constexpr uint32_t stream_row_bytes(uint32_t k) { return stream_d(k / 64) + up128(k / 64 / 2); }
    __device__ static void load_w_stream(Wt& w, const uint8_t* row, uint32_t u, uint32_t n_units) {
        const uint32_t plane = up128(16 * n_units);
        w.qa = ld_u128_nt(row + u * 16);
        w.qb = ld_u128_nt(row + plane + u * 16);
        w.qh = ld_u128_nt(row + 2 * plane + u * 16);
        w.sc = *reinterpret_cast<const uint2*>(row + stream_sc(n_units) + (u >> 1) * 8);
        w.d = ld_u16(row + stream_d(n_units) + (u >> 2) * 2);
    }
    __device__ static void to_stream(const uint8_t* row, uint8_t* dst, uint32_t u, uint32_t n_units) {
        const uint8_t* blk = row + (u >> 2) * 210;
        const uint32_t nh = (u >> 1) & 1, j = u & 1, plane = up128(16 * n_units);
        *reinterpret_cast<uint4*>(dst + u * 16) = ld_u128_a2(blk + nh * 64 + j * 16);
        *reinterpret_cast<uint4*>(dst + plane + u * 16) = ld_u128_a2(blk + nh * 64 + 32 + j * 16);
        *reinterpret_cast<uint4*>(dst + 2 * plane + u * 16) = ld_u128_a2(blk + 128 + nh * 32 + j * 16);
        if (j == 0) *reinterpret_cast<uint2*>(dst + stream_sc(n_units) + (u >> 1) * 8) = ld_u64_a2(blk + 192 + nh * 8);
        if ((u & 3) == 0) *reinterpret_cast<uint16_t*>(dst + stream_d(n_units) + (u >> 2) * 2) = static_cast<uint16_t>(ld_u16(blk + 208));
    }
    __device__ static float dot(const Wt& w, const Act& a, uint32_t u, int32_t* dbg) {
        uint32_t is = u & 1;  // l0 / 16
        int acc[4] = {a.init[0], a.init[1], a.init[2], a.init[3]};
        const uint32_t qa[4] = {w.qa.x, w.qa.y, w.qa.z, w.qa.w}, qb[4] = {w.qb.x, w.qb.y, w.qb.z, w.qb.w},
                       qh[4] = {w.qh.x, w.qh.y, w.qh.z, w.qh.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
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
            uint32_t base = (u >> 2) * 16 + ((u >> 1) & 1) * 8 + is;
#pragma unroll
            for (int t = 0; t < 4; ++t) dbg[base + 2 * t] = acc[t] - a.init[t];
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
    const uint4 v0 = *reinterpret_cast<const uint4*>(xq + u * 32);
    const uint4 v1 = *reinterpret_cast<const uint4*>(xq + u * 32 + 16);
    const uint32_t keep = live ? 0xFFFFFFFFu : 0u;
    const uint32_t v[8] = {v0.x, v0.y, v0.z, v0.w, v1.x, v1.y, v1.z, v1.w};
    int s = 0;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        a.a[i] = v[i] & keep;
        s = sum4(a.a[i], s);
    }
    const float t = xs[u];
    a.xs = live ? t : 0.0f;
    a.asum = s;
}

struct Q4_0 {  // 18 B: d, qs[16]; byte i = element i (low nibble), element i+16 (high); code - 8
    static constexpr int ELEMS_PER_UNIT = 32;
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
    // decode copy of a row: every block's scale, then every block's 16 quant bytes, each plane
    // padded to whole 128-byte lines (see Q4K::load_w_stream)
    static constexpr uint32_t up128(uint32_t b) { return (b + 127u) & ~127u; }
    static constexpr uint32_t stream_q(uint32_t n_units) { return up128(2 * n_units); }
    static constexpr uint32_t stream_row_bytes(uint32_t k) { return stream_q(k / 32) + up128(16 * (k / 32)); }
    __device__ static void load_w_stream(Wt& w, const uint8_t* row, uint32_t u, uint32_t n_units) {
        w.d = *reinterpret_cast<const uint16_t*>(row + 2 * u);
        w.q = ld_u128_nt(row + stream_q(n_units) + u * 16);
    }
    __device__ static void to_stream(const uint8_t* row, uint8_t* dst, uint32_t u, uint32_t n_units) {
        const uint8_t* blk = row + u * 18;
        *reinterpret_cast<uint16_t*>(dst + 2 * u) = static_cast<uint16_t>(ld_u16(blk));
        *reinterpret_cast<uint4*>(dst + stream_q(n_units) + u * 16) = ld_u128_a2(blk + 2);
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
    static constexpr int ELEMS_PER_UNIT = 32;
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
    // decode copy of a row: every block's (d, m), then every block's 16 quant bytes
    static constexpr uint32_t up128(uint32_t b) { return (b + 127u) & ~127u; }
    static constexpr uint32_t stream_q(uint32_t n_units) { return up128(4 * n_units); }
    static constexpr uint32_t stream_row_bytes(uint32_t k) { return stream_q(k / 32) + up128(16 * (k / 32)); }
    __device__ static void load_w_stream(Wt& w, const uint8_t* row, uint32_t u, uint32_t n_units) {
        w.dm = *reinterpret_cast<const uint32_t*>(row + 4 * u);
        w.q = ld_u128_nt(row + stream_q(n_units) + u * 16);
    }
    __device__ static void to_stream(const uint8_t* row, uint8_t* dst, uint32_t u, uint32_t n_units) {
        const uint8_t* blk = row + u * 20;
        *reinterpret_cast<uint32_t*>(dst + 4 * u) = *reinterpret_cast<const uint32_t*>(blk);
        *reinterpret_cast<uint4*>(dst + stream_q(n_units) + u * 16) = ld_u128_a4(blk + 4);
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
    static constexpr int ELEMS_PER_UNIT = 32;
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
    // decode copy of a row: every block's scale, then every block's first and second 16 codes
    static constexpr uint32_t up128(uint32_t b) { return (b + 127u) & ~127u; }
    static constexpr uint32_t stream_q(uint32_t n_units) { return up128(2 * n_units); }
    static constexpr uint32_t stream_row_bytes(uint32_t k) { return stream_q(k / 32) + 2 * up128(16 * (k / 32)); }
    __device__ static void load_w_stream(Wt& w, const uint8_t* row, uint32_t u, uint32_t n_units) {
        w.d = *reinterpret_cast<const uint16_t*>(row + 2 * u);
        w.q0 = ld_u128_nt(row + stream_q(n_units) + u * 16);
        w.q1 = ld_u128_nt(row + stream_q(n_units) + up128(16 * n_units) + u * 16);
    }
    __device__ static void to_stream(const uint8_t* row, uint8_t* dst, uint32_t u, uint32_t n_units) {
        const uint8_t* blk = row + u * 34;
        *reinterpret_cast<uint16_t*>(dst + 2 * u) = static_cast<uint16_t>(ld_u16(blk));
        *reinterpret_cast<uint4*>(dst + stream_q(n_units) + u * 16) = ld_u128_a2(blk + 2);
        *reinterpret_cast<uint4*>(dst + stream_q(n_units) + up128(16 * n_units) + u * 16) = ld_u128_a2(blk + 18);
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
// The kernel.  U = units per lane, KS = wavefronts per workgroup (K split),
// RB = rows in flight per workgroup, EPI = epilogue.
//
// Latency structure: a wavefront first issues the weight loads of its first row
// group, then loads its activations (so the two memory round trips overlap),
// and from then on keeps the next row group's loads in flight while it computes
// the current one (two register buffers, loop unrolled by two so no copies).
template <class T, int U, int RB, int NM>
struct GemvTile {
    typename T::Wt w[NM][RB][U];
    __device__ __forceinline__ void load(const GemvArgs& p, const uint32_t (&unit)[U], uint32_t r, uint32_t r1) {
#pragma unroll
        for (int mi = 0; mi < NM; ++mi) {
            const uint8_t* base = mi == 0 ? p.w : p.w2;
#pragma unroll
            for (int rb = 0; rb < RB; ++rb) {
                uint32_t row = min(r + rb, r1 - 1);  // rows past the range re-read the last row; results unused
                const uint8_t* rp = base + static_cast<uint64_t>(row) * p.row_bytes;
#pragma unroll
                for (int i = 0; i < U; ++i) T::load_w(w[mi][rb][i], rp, unit[i]);
            }
        }
    }
};

template <int EPI>
__device__ __forceinline__ void gemv_store(const GemvArgs& p, uint32_t row, float v0, float v1) {
    float v = v0;
    if (EPI == EPI_ADD) v = p.resid[row] + v;
    if (EPI == EPI_SILU_MUL) {
        // cera/src/backend/cpu.rs:2570-2575: g / (1 + expf(-g)) * u
        v = __fmul_rn(__fdiv_rn(v0, __fadd_rn(1.0f, cera_expf(-v0))), v1);
    }
    p.y[row] = v;
}

template <class T, int U, int KS, int RB, int EPI, bool DBG>
__device__ __forceinline__ void gemv_compute(const GemvArgs& p, const GemvTile<T, U, RB, (EPI == EPI_SILU_MUL ? 2 : 1)>& t,
                                             const typename T::Act (&act)[U], const uint32_t (&unit)[U],
                                             const bool (&live)[U], uint32_t lane, uint32_t kw, uint32_t r,
                                             uint32_t r1, float (*part)[RB][KS * 4]) {
    constexpr int NM = EPI == EPI_SILU_MUL ? 2 : 1;
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
                if (DBG) dbg = (live[i] && row < r1) ? p.dbg_dots + static_cast<uint64_t>(row) * p.dbg_stride : nullptr;
                acc += T::dot(t.w[mi][rb][i], act[i], unit[i], dbg);
            }
            // K-split workgroups leave the four 16-lane row sums of each wavefront to the LDS
            // combine below instead of folding them with cross-lane reads here
            tot[mi] = KS == 1 ? wave_sum(acc) : wave_row_sum(acc);
        }
        if (KS == 1) {
            if (lane == 0 && row < r1) gemv_store<EPI>(p, row, tot[0], tot[NM - 1]);
        } else if ((lane & 15) == 0) {
#pragma unroll
            for (int mi = 0; mi < NM; ++mi) part[mi][rb][kw * 4 + (lane >> 4)] = tot[mi];
        }
    }
    if (KS > 1) {
        lds_barrier();
        if (threadIdx.x < RB && r + threadIdx.x < r1) {
            float v[NM];
#pragma unroll
            for (int mi = 0; mi < NM; ++mi) {
                float s = 0.0f;
#pragma unroll
                for (int w = 0; w < KS; ++w) {   // wavefront order, rows paired as wave_sum pairs them
                    const float* q4 = &part[mi][threadIdx.x][4 * w];
                    s += (q4[0] + q4[1]) + (q4[2] + q4[3]);
                }
                v[mi] = s;
            }
            gemv_store<EPI>(p, r + threadIdx.x, v[0], v[NM - 1]);
        }
    }
}

// The work of workgroup `block` (KS wavefronts; this wavefront is number kw, this lane `lane`).
// `part` is the workgroup's LDS combine buffer (unused when KS == 1, which also has no barrier).
template <class T, int U, int KS, int RB, int EPI, bool DBG>
__device__ __forceinline__ void gemv_body(const GemvArgs& p, uint32_t block, uint32_t lane, uint32_t kw,
                                          float (*part)[EPI == EPI_SILU_MUL ? 2 : 1][RB][KS * 4]) {
    constexpr int NM = EPI == EPI_SILU_MUL ? 2 : 1;
    uint32_t r = block * p.rows_per_wave;  // rows per workgroup
    if (r >= p.m) return;
    const uint32_t r1 = min(p.m, r + p.rows_per_wave);

    uint32_t unit[U];
    bool live[U];
#pragma unroll
    for (int i = 0; i < U; ++i) {
        uint32_t u = kw * 64 + lane + 64 * KS * i;
        live[i] = u < p.n_units;
        unit[i] = live[i] ? u : 0;  // dead lanes re-read unit 0 with zeroed activations
    }
    GemvTile<T, U, RB, NM> ta, tb;
    ta.load(p, unit, r, r1);

    typename T::Act act[U];
#pragma unroll
    for (int i = 0; i < U; ++i) {
        T::load_act(act[i], p.xq, p.xs, unit[i], live[i]);
        if (DBG && block == 0 && live[i] && p.dbg_asums) T::dbg_asum(act[i], unit[i], p.dbg_asums);
    }

    // Each prefetch sits in the same straight-line block as the compute it overlaps, so the
    // compiler can wait for exactly the older tile's loads (a prefetch under its own
    // condition would force a wait for everything at the join).
    float (*part0)[RB][KS * 4] = KS == 1 ? nullptr : part[0];
    float (*part1)[RB][KS * 4] = KS == 1 ? nullptr : part[1];
    for (;;) {
        if (r + RB >= r1) {
            gemv_compute<T, U, KS, RB, EPI, DBG>(p, ta, act, unit, live, lane, kw, r, r1, part0);
            break;
        }
        tb.load(p, unit, r + RB, r1);
        gemv_compute<T, U, KS, RB, EPI, DBG>(p, ta, act, unit, live, lane, kw, r, r1, part0);
        r += RB;
        if (r + RB >= r1) {
            gemv_compute<T, U, KS, RB, EPI, DBG>(p, tb, act, unit, live, lane, kw, r, r1, part1);
            break;
        }
        ta.load(p, unit, r + RB, r1);
        gemv_compute<T, U, KS, RB, EPI, DBG>(p, tb, act, unit, live, lane, kw, r, r1, part1);
        r += RB;
    }
}

template <class T, int U, int KS, int RB, int EPI, bool DBG>
static __global__ __launch_bounds__(64 * KS) void gemv_kernel(GemvArgs p) {
    constexpr int NM = EPI == EPI_SILU_MUL ? 2 : 1;
    // two LDS buffers: a buffer is rewritten two row groups later, after another barrier
    __shared__ float part[2][NM][RB][KS * 4];
    gemv_body<T, U, KS, RB, EPI, DBG>(p, blockIdx.x, threadIdx.x & 63, threadIdx.x >> 6, part);
}

// Two independent GEMVs over the same activations in one launch: workgroups [0, n_blocks_a) run
// matrix A (KSA wavefronts split its K), the rest run matrix B, whose K fits one wavefront, so each
// of their KSA wavefronts is a workgroup of B on its own (no LDS, no barrier on that side).
// For a layer whose V projection has another block type than Q and K: one launch instead of two.
struct GemvPairArgs {
    GemvArgs a, b;
    uint32_t n_blocks_a;
};
template <class TA, int KSA, int RBA, class TB, int RBB>
static __global__ __launch_bounds__(64 * KSA) void gemv_pair_kernel(GemvPairArgs p) {
    __shared__ float part[2][1][RBA][KSA * 4];
    const uint32_t lane = threadIdx.x & 63, kw = threadIdx.x >> 6;
    if (blockIdx.x < p.n_blocks_a) {
        gemv_body<TA, 1, KSA, RBA, EPI_STORE, false>(p.a, blockIdx.x, lane, kw, part);
    } else {
        gemv_body<TB, 1, 1, RBB, EPI_STORE, false>(p.b, (blockIdx.x - p.n_blocks_a) * KSA + kw, lane, 0,
                                                   static_cast<float(*)[1][RBB][4]>(nullptr));
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
