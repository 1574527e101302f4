// Prefill GEMM for Q6_K with the block dots on the f16 matrix cores.
//
// Same arithmetic contract as gemm.hip.h (cera's batched int8 path for Q6_K,
// cera/src/backend/simd.rs:5988-6195): exact integer dots of the 6-bit codes (minus 32) with
// the int8 activations per 16-element scale group, then  sum_g (sc[g]*d) * xs[b] * dot[g].
// The int8 kernel is VALU-bound for this type: two groups per 32-block, each needing a convert
// and an FMA per output, on top of an unpack that sign-extends every code.  Here the codes and
// the activation quants are staged as f16 (both exact: |code| <= 32, |a| <= 127), one
// v_mfma_f32_32x32x16_f16 is exactly one scale group (K = 16), and its f32 result IS the
// integer dot (|dot| <= 16*32*127, far below 2^24): no convert, and no sign extension (the
// -32 is one packed f16 add on the 1024 + q form the unpack produces anyway).  The per-output
// scales (sc*d)[row] x xs[token] of the two groups of a block come from one two-block
// outer-product MFMA as in gemm.hip.h.  VALU work per output per 32-block: two FMAs.
//
// 6-bit codes become f16 without a convert: the low nibble and the two high bits are OR-ed into
// the mantissa of 1024.0 (ulp 1), giving 1024 + q.  That pairs bytes (0, 2) and (1, 3) of each
// 32-bit word, so K is stored in the order 0, 2, 1, 3 within every four; the activations are
// staged in the same order (gemm_act_f16_kernel) -- the order inside a scale group does not
// matter to its dot product.
//
// Tiles as gemm.hip.h: 256 threads = 2 x 2 wavefronts, 128 rows x 64 tokens, K in steps of 128
// (one half of a super-block); LDS rows are 256 B + 16 B pad (57 KB a workgroup, two per CU: an
// unpadded, XOR-swizzled layout that fits three was tried and spilled on its sixteen distinct
// fragment addresses).
#pragma once
#include "gemm.hip.h"

typedef _Float16 gq_v8h __attribute__((ext_vector_type(8)));
typedef _Float16 gq_h2 __attribute__((ext_vector_type(2)));
typedef uint32_t gq_u4 __attribute__((ext_vector_type(4)));

#define GQ_LD 272   // bytes per staged row: 128 f16 + 16 pad

// 16 int8 quants -> 16 f16 words in the 0,2,1,3 order
__device__ __forceinline__ void gemm_act_f16_words(const uint4 v, uint4& out0, uint4& out1) {
    const uint32_t x[4] = {v.x, v.y, v.z, v.w};
    uint32_t o[8];
    const _Float16 mh = static_cast<_Float16>(-1152.0f);
    const gq_h2 off = {mh, mh};
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        // a + 128 as an unsigned byte in the mantissa of 1024.0, then minus (1024 + 128): exact
        const uint32_t y = x[j] ^ 0x80808080u;
        o[2 * j] = __builtin_bit_cast(uint32_t, __builtin_bit_cast(gq_h2, (y & 0x00FF00FFu) | 0x64006400u) + off);
        o[2 * j + 1] = __builtin_bit_cast(uint32_t, __builtin_bit_cast(gq_h2, ((y >> 8) & 0x00FF00FFu) | 0x64006400u) + off);
    }
    out0 = make_uint4(o[0], o[1], o[2], o[3]);
    out1 = make_uint4(o[4], o[5], o[6], o[7]);
}
// int8 quants [n_words * 16] -> f16 in the 0,2,1,3 order, 16 per thread
__device__ __forceinline__ void gemm_act_f16_body(const uint4* __restrict__ q, uint4* __restrict__ out,
                                                                  uint64_t n_words) {
    const uint64_t i = static_cast<uint64_t>(blockIdx.x) * 256 + threadIdx.x;
    if (i >= n_words) return;
    gemm_act_f16_words(q[i], out[2 * i], out[2 * i + 1]);
}
static __global__ __launch_bounds__(256) void gemm_act_f16_kernel(const uint4* __restrict__ q, uint4* __restrict__ out,
                                                                  uint64_t n_words) {
    gemm_act_f16_body(q, out, n_words);
}

// byte offset of 16-byte chunk `chunk` of staged row `row`
__device__ __forceinline__ uint32_t gq_off(uint32_t row, uint32_t chunk) { return row * GQ_LD + (chunk << 4); }

// WIDE = 1: the tile above.  WIDE = 2: 512 threads = 2 x 4 wavefronts on 128 rows x 128 tokens, every
// wavefront the same 64 x 32 share as before: the weight unpack (a quarter of the narrow tile's vector
// instructions) is spread over twice the threads for twice the outputs, and a SIMD holds four
// wavefronts instead of two.  76 KB of LDS a workgroup, still two per CU.
template <bool DBG = false, int WIDE = 1>
__device__ __forceinline__ void gemm_q6k_f16_body(GemmArgs p) {
    constexpr int NB = GEMM_KT / 32;
    constexpr uint32_t BN = GEMM_BN * WIDE, NT = 256 * WIDE;   // tokens per workgroup, threads
    constexpr int AW = 4 / WIDE;                               // 32-bit words of each code run a thread unpacks
    // the wide tile has the CU to itself and stages K steps alternately into two buffers: one barrier per
    // step (a buffer is rewritten two steps later, behind the barrier of the step between)
    constexpr int NBUF = WIDE;
    __shared__ __attribute__((aligned(16))) uint8_t sA_[NBUF][GEMM_BM * GQ_LD];
    __shared__ __attribute__((aligned(16))) uint8_t sB_[NBUF][BN * GQ_LD];
    __shared__ __attribute__((aligned(16))) float sRS_[NBUF][2 * NB * GEMM_BM];   // (sc * d) per 16-group per row
    __shared__ __attribute__((aligned(16))) float sCS_[NBUF][NB * BN];

    const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const uint32_t wm = wave / (2 * WIDE), wn = wave % (2 * WIDE);
    const bool second = p.w2 != nullptr && blockIdx.y >= p.tiles1;
    const uint8_t* const wmat = second ? p.w2 : p.w;
    float* const omat = second ? p.out2 : p.out;
    const uint32_t mrows = second ? p.m2 : p.m;
    const uint64_t ldn = second ? p.ld_n2 : p.ld_n;
    const uint32_t m0 = (second ? blockIdx.y - p.tiles1 : blockIdx.y) * GEMM_BM, n0 = blockIdx.x * BN;
    const uint32_t col = lane & 31, half = lane >> 5;
    const uint32_t nb32 = p.k / 32;

    v16f acc[2];
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[t][r] = 0.0f;

    // staging assignments, fixed for the whole K loop.  Weight item (row, j): positions 4 AW j ..
    // 4 AW (j + 1) - 1 of each 32 of the 128-element half (AW words of ql[l], ql[32 + l] and qh[l]);
    // threads 0..127 also decode their row's scales.
    // Rows and tokens past the edge are clamped: their products are computed and never stored.
    const uint32_t a_row = tid / (2 * WIDE), a_j = tid % (2 * WIDE);
    const uint8_t* a_src = wmat + static_cast<uint64_t>(min(m0 + a_row, mrows - 1)) * p.row_bytes;
    const uint8_t* s_src = wmat + static_cast<uint64_t>(min(m0 + (tid & (GEMM_BM - 1)), mrows - 1)) * p.row_bytes;
    const uint8_t* b_src[4];
    uint32_t b_dst[4];   // byte offset in sB
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const uint32_t it = tid + NT * i, c = it >> 4, wi = it & 15;
        b_src[i] = static_cast<const uint8_t*>(p.bh) + static_cast<uint64_t>(min(n0 + c, p.n - 1)) * p.k * 2 + wi * 16;
        b_dst[i] = gq_off(c, wi);
    }
    const uint32_t c_tok = tid >> 2, c_b = tid & 3;
    const uint64_t c_off = static_cast<uint64_t>(min(n0 + c_tok, p.n - 1)) * nb32 + c_b;

    uint32_t qa[AW], qb[AW], qh[AW];   // prefetched codes of the item
    uint2 rsc;          // the half's eight int8 group scales (threads 0..127)
    uint32_t rd;
    gq_u4 rb[4];
    float rcs;
    auto fetch = [&](uint32_t k0) __attribute__((always_inline)) {
        const uint32_t nh = (k0 / GEMM_KT) & 1;
        const uint8_t* blk = a_src + (k0 / 256) * 210;
        if (WIDE == 1) {
            const uint4 va = ld_u128_a2(blk + nh * 64 + a_j * 16), vb = ld_u128_a2(blk + nh * 64 + 32 + a_j * 16),
                        vh = ld_u128_a2(blk + 128 + nh * 32 + a_j * 16);
            qa[0] = va.x; qa[1] = va.y; qa[AW - 2] = va.z; qa[AW - 1] = va.w;
            qb[0] = vb.x; qb[1] = vb.y; qb[AW - 2] = vb.z; qb[AW - 1] = vb.w;
            qh[0] = vh.x; qh[1] = vh.y; qh[AW - 2] = vh.z; qh[AW - 1] = vh.w;
        } else {
            const uint2 va = ld_u64_a2(blk + nh * 64 + a_j * 8), vb = ld_u64_a2(blk + nh * 64 + 32 + a_j * 8),
                        vh = ld_u64_a2(blk + 128 + nh * 32 + a_j * 8);
            qa[0] = va.x; qa[1] = va.y;
            qb[0] = vb.x; qb[1] = vb.y;
            qh[0] = vh.x; qh[1] = vh.y;
        }
        if (tid < GEMM_BM) {
            const uint8_t* sblk = s_src + (k0 / 256) * 210;
            rsc = ld_u64_a2(sblk + 192 + nh * 8);
            rd = ld_u16(sblk + 208);
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) rb[i] = *reinterpret_cast<const gq_u4*>(b_src[i] + static_cast<uint64_t>(k0) * 2);
        rcs = p.bs[c_off + k0 / 32];
    };
    const _Float16 m1056 = static_cast<_Float16>(-1056.0f);
    const gq_h2 recentre = {m1056, m1056};   // (1024 + q) - 1056 = q - 32
    const uint32_t k_begin = blockIdx.z * p.k_chunk, k_end = k_begin + p.k_chunk;
    fetch(k_begin);
    for (uint32_t k0 = k_begin; k0 < k_end; k0 += GEMM_KT) {
        const uint32_t buf = NBUF == 2 ? ((k0 - k_begin) / GEMM_KT) & 1 : 0;
        uint8_t* const sA = sA_[buf];
        uint8_t* const sB = sB_[buf];
        float* const sRS = sRS_[buf];
        float* const sCS = sCS_[buf];
        // ---- registers -> LDS.  Element 32t + l of the half: low nibble of ql[l] (t = 0), of ql[32 + l]
        // (t = 1), high nibbles of the same (t = 2, 3); bits 2t, 2t+1 of qh[l] are its bits 4, 5.
        {
            const uint32_t *a = qa, *b = qb, *h = qh;
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                uint32_t o[2 * AW];
#pragma unroll
                for (int i = 0; i < AW; ++i) {
                    const uint32_t ql = (t & 1) ? b[i] : a[i];
                    const uint32_t lo = t >= 2 ? ql >> 4 : ql;          // the nibble of bytes 0, 2 at bits 0..3, 16..19
                    const uint32_t n02 = lo & 0x000F000Fu, n13 = (lo >> 8) & 0x000F000Fu;
                    // field t of bytes 0, 2 sits at bits 2t, 16 + 2t; of bytes 1, 3 at 8 + 2t, 24 + 2t: both to bits 4, 5
                    const uint32_t h02 = (t <= 2 ? h[i] << (4 - 2 * t) : h[i] >> (2 * t - 4)) & 0x00300030u;
                    const uint32_t h13 = (h[i] >> (4 + 2 * t)) & 0x00300030u;
                    o[2 * i] = __builtin_bit_cast(uint32_t, __builtin_bit_cast(gq_h2, n02 | h02 | 0x64006400u) + recentre);
                    o[2 * i + 1] = __builtin_bit_cast(uint32_t, __builtin_bit_cast(gq_h2, n13 | h13 | 0x64006400u) + recentre);
                }
                if (WIDE == 1) {
                    *reinterpret_cast<gq_u4*>(sA + gq_off(a_row, 4 * t + 2 * a_j)) = gq_u4{o[0], o[1], o[2], o[3]};
                    *reinterpret_cast<gq_u4*>(sA + gq_off(a_row, 4 * t + 2 * a_j + 1)) = gq_u4{o[2 * AW - 4], o[2 * AW - 3], o[2 * AW - 2], o[2 * AW - 1]};
                } else {
                    *reinterpret_cast<gq_u4*>(sA + gq_off(a_row, 4 * t + a_j)) = gq_u4{o[0], o[1], o[2], o[3]};
                }
            }
        }
        if (tid < GEMM_BM) {
            // (sc * d): an 8-bit integer times an f16 value, exact in f32
            const float d = h2f(rd);
            const uint32_t s[2] = {rsc.x, rsc.y};
#pragma unroll
            for (int g = 0; g < 8; ++g)
                sRS[g * GEMM_BM + tid] = d * static_cast<float>(static_cast<int>(static_cast<int8_t>((s[g >> 2] >> (8 * (g & 3))) & 0xFF)));
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) *reinterpret_cast<gq_u4*>(sB + b_dst[i]) = rb[i];
        sCS[c_b * BN + c_tok] = rcs;
        __syncthreads();
        if (k0 + GEMM_KT < k_end) fetch(k0 + GEMM_KT);

        // ---- per 32-block: the two groups' scale tiles from one outer product, then one f16 MFMA per group
        const uint32_t bR = wn * 32 + col;
#pragma unroll
        for (int b = 0; b < NB; ++b) {
            const float xs = sCS[b * BN + wn * 32 + col];
            const gq_v8h bf0 = *reinterpret_cast<const gq_v8h*>(sB + gq_off(bR, 4 * b + half));
            const gq_v8h bf1 = *reinterpret_cast<const gq_v8h*>(sB + gq_off(bR, 4 * b + 2 + half));
#pragma unroll
            for (int t = 0; t < 2; ++t) {
                const float rsl = sRS[(2 * b + half) * GEMM_BM + wm * 64 + t * 32 + col];
                v32f z32;
#pragma unroll
                for (int e = 0; e < 32; ++e) z32[e] = 0.0f;
                const v32f sc = __builtin_amdgcn_mfma_f32_32x32x1f32(rsl, xs, z32, 0, 0, 0);
                const uint32_t aR = wm * 64 + t * 32 + col;
                const gq_v8h af0 = *reinterpret_cast<const gq_v8h*>(sA + gq_off(aR, 4 * b + half));
                const gq_v8h af1 = *reinterpret_cast<const gq_v8h*>(sA + gq_off(aR, 4 * b + 2 + half));
                v16f z = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
                const v16f c0 = __builtin_amdgcn_mfma_f32_32x32x16_f16(af0, bf0, z, 0, 0, 0);
                const v16f c1 = __builtin_amdgcn_mfma_f32_32x32x16_f16(af1, bf1, z, 0, 0, 0);
                if (DBG) {
                    const uint32_t dtok = n0 + wn * 32 + col, dgrp = 2 * (k0 / 32 + b);
#pragma unroll
                    for (int e = 0; e < 16; ++e) {
                        const uint32_t drow = m0 + wm * 64 + t * 32 + (e >> 2) * 8 + half * 4 + (e & 3);
                        if (drow < mrows && dtok < p.n) {
                            int32_t* d = p.dbg_dots + (static_cast<uint64_t>(drow) * p.n + dtok) * (2 * nb32) + dgrp;
                            const float v0 = c0[e], v1 = c1[e];   // (a bit_cast of the element expression itself reads element 0)
                            d[0] = __float_as_int(v0);
                            d[1] = __float_as_int(v1);
                        }
                    }
                }
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    acc[t][e] = fmaf(c0[e], sc[e], acc[t][e]);
                    acc[t][e] = fmaf(c1[e], sc[16 + e], acc[t][e]);
                }
            }
        }
        if (NBUF == 1) __syncthreads();
    }
    // ---- store: lane holds token n0 + wn*32 + col, rows 8*blk + 4*half + r of each row tile
    const uint32_t tok = n0 + wn * 32 + col;
    if (tok < p.n) {
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int blk = 0; blk < 4; ++blk)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    uint32_t row = m0 + wm * 64 + t * 32 + blk * 8 + half * 4 + r;
                    if (row < mrows) {
                        float v = acc[t][blk * 4 + r];
                        uint64_t idx = row * p.ld_m + tok * ldn;
                        if (p.resid) v = p.resid[idx] + (p.resid_scale != 1.0f ? v * p.resid_scale : v);
                        omat[idx + blockIdx.z * p.part_stride] = v;
                    }
                }
    }
}
template <bool DBG = false, int WIDE = 1>
static __global__ __launch_bounds__(256 * WIDE, 2) void gemm_q6k_f16_kernel(GemmArgs p) {
    gemm_q6k_f16_body<DBG, WIDE>(p);
}
