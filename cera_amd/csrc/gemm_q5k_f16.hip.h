// Prefill GEMM for Q5_K: f32-class activations on the f16 matrix cores.
//
// cera dots Q5_K weights with the UNQUANTIZED f32 activations (gemv_q5km_f32,
// cera/src/backend/cpu.rs:1830-1854 over vec_dot_q5km_f32, cera/src/quant.rs:892-937):
//   y = sum_b ( d*sc[b] * sum_{i in b} q_i x_i  -  dmin*mn[b] * sum_{i in b} x_i ),   q_i in 0..31,
// so a batched kernel has no int8 route.  Here the 5-bit codes are staged as f16 (exact) and an
// activation as an f16 pair x = hi + lo (hi = x rounded to f16, lo = the rounded remainder:
// 2^-22 relative), so that two pairs of v_mfma_f32_32x32x16_f16 per 32-block give
// sum q_i x_i with f32 accumulation -- the three-product split of the prefill attention with the
// weight side exact.  The per-output factors come from ONE two-block outer-product MFMA per
// block and row tile: block 0 = (d*sc)[row] x 2^-e[token] (e: the split's per-token power of two), block 1 = (dmin*mn)[row] x (sum_b x)[token];
// VALU work per output per block: one FMA and one subtract.  The block sums of x are f32 sums
// made once per activation matrix by the kernel that splits it.  Results differ from the
// reference's sequential f32 FMA chain by rounding order only (tested to 1e-3 rms, measured ~1e-6).
//
// Tiles, K steps, K order (0, 2, 1, 3 within every four, from the OR-into-the-mantissa unpack)
// and LDS rows are those of gemm_q6k_f16.hip.h; LDS is 75 KB a workgroup, two per CU.
#pragma once
#include "gemm_q6k_f16.hip.h"

// One workgroup per token row: x [k] f32 -> hi / lo f16 of x * 2^e in the 0,2,1,3 order, the f32 sums of
// x per 32-block, and 2^-e.  e puts the row's largest magnitude in [2^13, 2^14): the f16 pair then
// resolves every element that matters to the dot product to 2^-22 of itself (unscaled, the lo halves
// of small activations fall on the f16 subnormal grid: 1.5e-4 rms at |x| ~ 1e-3), and a power of
// two changes no mantissa.  k % 32 == 0.
static __global__ __launch_bounds__(256) void gemm_act_split_kernel(const float* __restrict__ x, uint4* __restrict__ hi,
                                                                     uint4* __restrict__ lo, float* __restrict__ bsum,
                                                                     float* __restrict__ inv_scale, uint32_t k) {
    __shared__ float s_max[4];
    const uint32_t tid = threadIdx.x;
    const float4* xr = reinterpret_cast<const float4*>(x + static_cast<uint64_t>(blockIdx.x) * k);
    float mx = 0.0f;
    for (uint32_t i = tid; i < k / 4; i += 256) {
        const float4 v = xr[i];
        mx = fmaxf(fmaxf(mx, fmaxf(fabsf(v.x), fabsf(v.y))), fmaxf(fabsf(v.z), fabsf(v.w)));
    }
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o));
    if ((tid & 63) == 0) s_max[tid >> 6] = mx;
    __syncthreads();
    mx = fmaxf(fmaxf(s_max[0], s_max[1]), fmaxf(s_max[2], s_max[3]));
    int e = 0;
    if (mx > 0.0f && mx < __builtin_inff()) {
        (void)frexpf(mx, &e);              // mx = f * 2^e, f in [0.5, 1)
        e = min(max(14 - e, -100), 100);   // x * 2^e has its maximum in [2^13, 2^14)
    }
    const float scale = ldexpf(1.0f, e);
    if (tid == 0) inv_scale[blockIdx.x] = ldexpf(1.0f, -e);
    const uint64_t row_oct = static_cast<uint64_t>(blockIdx.x) * (k / 8);
    for (uint32_t i = tid; i < k / 8; i += 256) {   // k / 8 is a multiple of 4: the four lanes of a block stay together
        const float4 a = xr[2 * i], b = xr[2 * i + 1];
        const float v[8] = {a.x, a.z, a.y, a.w, b.x, b.z, b.y, b.w};
        uint32_t oh[4], ol[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            gq_h2 h, l;
#pragma unroll
            for (int c = 0; c < 2; ++c) {
                const float xs = v[2 * j + c] * scale;
                // A NaN or an infinity goes through as itself (hi = the f16 NaN / infinity, lo = 0), so
                // the token's outputs come out non-finite as the reference's f32 dot gives them
                // (vec_dot_q5km_f32, cera/src/backend/cpu.rs:1830-1854).  The clamp only matters beside
                // an infinity, where the row maximum gives no scale and a finite value may pass 65504.
                const bool finite = (xs - xs) == 0.0f;
                const _Float16 hh = static_cast<_Float16>(finite ? fminf(fmaxf(xs, -65504.0f), 65504.0f) : xs);
                h[c] = hh;
                l[c] = finite ? static_cast<_Float16>(xs - static_cast<float>(hh)) : static_cast<_Float16>(0.0f);
            }
            oh[j] = __builtin_bit_cast(uint32_t, h);
            ol[j] = __builtin_bit_cast(uint32_t, l);
        }
        float s = ((a.x + a.y) + (a.z + a.w)) + ((b.x + b.y) + (b.z + b.w));
        s += __shfl_xor(s, 1);
        s += __shfl_xor(s, 2);
        hi[row_oct + i] = make_uint4(oh[0], oh[1], oh[2], oh[3]);
        lo[row_oct + i] = make_uint4(ol[0], ol[1], ol[2], ol[3]);
        if ((tid & 3) == 0) bsum[(row_oct + i) >> 2] = s;
    }
}

// p.bh = hi, p.bq = lo (both [n][k] f16, of x * 2^e), p.bsum = block sums of x [n][k/32], p.bs = 2^-e per token [n].
static __global__ __launch_bounds__(256, 2) void gemm_q5k_f16_kernel(GemmArgs p) {
    constexpr int NB = GEMM_KT / 32;
    __shared__ __attribute__((aligned(16))) uint8_t sA[GEMM_BM * GQ_LD];
    __shared__ __attribute__((aligned(16))) uint8_t sBh[GEMM_BN * GQ_LD];
    __shared__ __attribute__((aligned(16))) uint8_t sBl[GEMM_BN * GQ_LD];
    __shared__ __attribute__((aligned(16))) float sRS[NB * GEMM_BM];   // d * sc per block per row
    __shared__ __attribute__((aligned(16))) float sRM[NB * GEMM_BM];   // dmin * mn
    __shared__ __attribute__((aligned(16))) float sCS[NB * GEMM_BN];   // sum of x per block per token

    const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const uint32_t wm = wave >> 1, wn = wave & 1;
    const bool second = p.w2 != nullptr && blockIdx.y >= p.tiles1;
    const uint8_t* const wmat = second ? p.w2 : p.w;
    float* const omat = second ? p.out2 : p.out;
    const uint32_t mrows = second ? p.m2 : p.m;
    const uint64_t ldn = second ? p.ld_n2 : p.ld_n;
    const uint32_t m0 = (second ? blockIdx.y - p.tiles1 : blockIdx.y) * GEMM_BM, n0 = blockIdx.x * GEMM_BN;
    const uint32_t col = lane & 31, half = lane >> 5;
    const uint32_t nb32 = p.k / 32;

    v16f acc[2];
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[t][r] = 0.0f;

    // staging assignments, fixed for the whole K loop.  Weight item (row, j): byte positions
    // 16j .. 16j+15 of the half's two 32-byte code chunks and of the high-bit bytes; threads 0..127
    // also decode their row's scales.  Rows and tokens past the edge are clamped: their products
    // are computed and never stored.
    const uint32_t a_row = tid >> 1, a_j = tid & 1;
    const uint8_t* a_src = wmat + static_cast<uint64_t>(min(m0 + a_row, mrows - 1)) * p.row_bytes;
    const uint8_t* s_src = wmat + static_cast<uint64_t>(min(m0 + (tid & (GEMM_BM - 1)), mrows - 1)) * p.row_bytes;
    uint64_t b_off[4];
    uint32_t b_dst[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const uint32_t it = tid + 256 * i, c = it >> 4, wi = it & 15;
        b_off[i] = static_cast<uint64_t>(min(n0 + c, p.n - 1)) * p.k * 2 + wi * 16;
        b_dst[i] = gq_off(c, wi);
    }
    const uint8_t* const bh = static_cast<const uint8_t*>(p.bh);
    const uint8_t* const bl = reinterpret_cast<const uint8_t*>(p.bq);
    const uint32_t c_tok = tid >> 2, c_b = tid & 3;
    const uint64_t c_off = static_cast<uint64_t>(min(n0 + c_tok, p.n - 1)) * nb32 + c_b;
    const float unscale = p.bs[min(n0 + wn * 32 + col, p.n - 1)];   // 2^-e of this lane's token

    uint4 qa, qb, qh;        // prefetched codes of the item: two nibble chunks and the high bits
    GemmQ4K::RawS rsc;       // d, dmin and the twelve scale bytes: the header Q5_K shares with Q4_K
    gq_u4 rbh[4], rbl[4];
    float rcs;
    auto fetch = [&](uint32_t k0) __attribute__((always_inline)) {
        const uint32_t nh = (k0 / GEMM_KT) & 1;
        const uint8_t* blk = a_src + (k0 / 256) * 176;
        qa = *reinterpret_cast<const uint4*>(blk + 48 + nh * 64 + a_j * 16);
        qb = *reinterpret_cast<const uint4*>(blk + 48 + nh * 64 + 32 + a_j * 16);
        qh = *reinterpret_cast<const uint4*>(blk + 16 + a_j * 16);
        if (tid < GEMM_BM) rsc.h = *reinterpret_cast<const uint4*>(s_src + (k0 / 256) * 176);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            rbh[i] = *reinterpret_cast<const gq_u4*>(bh + b_off[i] + static_cast<uint64_t>(k0) * 2);
            rbl[i] = *reinterpret_cast<const gq_u4*>(bl + b_off[i] + static_cast<uint64_t>(k0) * 2);
        }
        rcs = p.bsum[c_off + k0 / 32];
    };
    const _Float16 m1024 = static_cast<_Float16>(-1024.0f);
    const gq_h2 unbias = {m1024, m1024};   // (1024 + q) - 1024 = q
    const uint32_t k_begin = blockIdx.z * p.k_chunk, k_end = k_begin + p.k_chunk;
    fetch(k_begin);
    for (uint32_t k0 = k_begin; k0 < k_end; k0 += GEMM_KT) {
        // ---- registers -> LDS.  Sub-block t of the half (t = 0..3): element l is the low (t even) or
        // high (t odd) nibble of byte l of code chunk t / 2, plus 16 x bit (4 nh + t) of high-bit byte l.
        {
            const uint32_t nh = (k0 / GEMM_KT) & 1;
            const uint32_t a[4] = {qa.x, qa.y, qa.z, qa.w}, b[4] = {qb.x, qb.y, qb.z, qb.w}, h[4] = {qh.x, qh.y, qh.z, qh.w};
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                uint32_t o[8];
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const uint32_t qs = (t >> 1) ? b[i] : a[i];
                    const uint32_t nib = (t & 1) ? qs >> 4 : qs;
                    const uint32_t hb = h[i] >> (4 * nh + t);   // this sub-block's bit of bytes 0..3 at bits 0, 8, 16, 24
                    const uint32_t c02 = (nib & 0x000F000Fu) | ((hb & 0x00010001u) << 4);
                    const uint32_t c13 = ((nib >> 8) & 0x000F000Fu) | (((hb >> 8) & 0x00010001u) << 4);
                    o[2 * i] = __builtin_bit_cast(uint32_t, __builtin_bit_cast(gq_h2, c02 | 0x64006400u) + unbias);
                    o[2 * i + 1] = __builtin_bit_cast(uint32_t, __builtin_bit_cast(gq_h2, c13 | 0x64006400u) + unbias);
                }
                *reinterpret_cast<gq_u4*>(sA + gq_off(a_row, 4 * t + 2 * a_j)) = gq_u4{o[0], o[1], o[2], o[3]};
                *reinterpret_cast<gq_u4*>(sA + gq_off(a_row, 4 * t + 2 * a_j + 1)) = gq_u4{o[4], o[5], o[6], o[7]};
            }
            if (tid < GEMM_BM) GemmQ4K::scales(rsc, nh, sRS + tid, sRM + tid, GEMM_BM);
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            *reinterpret_cast<gq_u4*>(sBh + b_dst[i]) = rbh[i];
            *reinterpret_cast<gq_u4*>(sBl + b_dst[i]) = rbl[i];
        }
        sCS[c_b * GEMM_BN + c_tok] = rcs;
        __syncthreads();
        if (k0 + GEMM_KT < k_end) fetch(k0 + GEMM_KT);

        // ---- per 32-block: the scale and min tiles from one outer product, then hi and lo dots
        const uint32_t bR = wn * 32 + col;
#pragma unroll 1
        for (int b = 0; b < NB; ++b) {   // not unrolled: two blocks' fragments and scale tiles at once already spill (190 VGPRs as it is)
            // B operand of the outer product: block 0 (lanes 0..31) undoes the token's 2^e, block 1 is sum(x)
            const float xsum = half ? sCS[b * GEMM_BN + wn * 32 + col] : unscale;
            const gq_v8h bh0 = *reinterpret_cast<const gq_v8h*>(sBh + gq_off(bR, 4 * b + half));
            const gq_v8h bh1 = *reinterpret_cast<const gq_v8h*>(sBh + gq_off(bR, 4 * b + 2 + half));
            const gq_v8h bl0 = *reinterpret_cast<const gq_v8h*>(sBl + gq_off(bR, 4 * b + half));
            const gq_v8h bl1 = *reinterpret_cast<const gq_v8h*>(sBl + gq_off(bR, 4 * b + 2 + half));
#pragma unroll
            for (int t = 0; t < 2; ++t) {
                const uint32_t aR = wm * 64 + t * 32 + col;
                const float rsl = (half ? sRM : sRS)[b * GEMM_BM + aR];
                v32f z32;
#pragma unroll
                for (int e = 0; e < 32; ++e) z32[e] = 0.0f;
                const v32f sc = __builtin_amdgcn_mfma_f32_32x32x1f32(rsl, xsum, z32, 0, 0, 0);
                const gq_v8h af0 = *reinterpret_cast<const gq_v8h*>(sA + gq_off(aR, 4 * b + half));
                const gq_v8h af1 = *reinterpret_cast<const gq_v8h*>(sA + gq_off(aR, 4 * b + 2 + half));
                v16f c = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
                c = __builtin_amdgcn_mfma_f32_32x32x16_f16(af0, bl0, c, 0, 0, 0);   // the small terms first
                c = __builtin_amdgcn_mfma_f32_32x32x16_f16(af1, bl1, c, 0, 0, 0);
                c = __builtin_amdgcn_mfma_f32_32x32x16_f16(af0, bh0, c, 0, 0, 0);
                c = __builtin_amdgcn_mfma_f32_32x32x16_f16(af1, bh1, c, 0, 0, 0);
#pragma unroll
                for (int e = 0; e < 16; ++e) acc[t][e] = fmaf(c[e], sc[e], acc[t][e] - sc[16 + e]);
            }
        }
        __syncthreads();
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
