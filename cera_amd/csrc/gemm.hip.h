// Prefill GEMM: out[m][n] = W[m, k] . B[k, n] with W in native GGUF blocks and
// B the Q8_0-quantized activations of n tokens, on the int8 matrix cores
// (Q4_K, Q4_0, Q4_1, Q8_0; Q6_K has a kernel of its own in gemm_q6k_f16.hip.h).
//
// Arithmetic contract (cera's batched int8 path, cera/src/backend/simd.rs:
// 5693-5878 Q4_K, :5893-5976 Q4_1, :4718-5010 Q4_0/Q8_0;
// cera/src/model/transformer.rs:710-788, 865-946): exact int32 dots of weight
// codes with int8 activations per 32-element block, then an f32
// epilogue  sum_b xs[j][b] * (d*sc * dot - dmin*mn * sum a).
//
// Mapping to gfx950: one v_mfma_i32_32x32x32_i8 computes the 32x32 int32 dots
// of one 32-element block for 32 weight rows x 32 tokens.  Every block carries its own
// pair of scales (weight side x activation side), so the int32 tile is folded
// into f32 accumulators after each block: a convert and an FMA per output per block
// on the VALU.  Everything else about the scales runs on the matrix core:
//   * the per-output scale  rs[row][b] * xs[token][b]  is a rank-1 matrix per block;
//     one v_mfma_f32_32x32x1_2b_f32 produces it for two blocks from ONE scalar LDS
//     read per lane per operand, already in the accumulator layout.  Reading the
//     sixteen row scales a lane needs straight from LDS costs a full-width read for
//     data every lane of a half shares, and that broadcast traffic, not the fragments,
//     was what kept the LDS busy;
//   * the min terms  dmin*mn[row][b] * (xs*sum a)[tok][b]  (Q4_K, Q4_1) are a small
//     f32 contraction over blocks of their own: v_mfma_f32_32x32x2_f32, two blocks
//     per instruction, accumulated (negated) into the same f32 tile as the dots.
//
// Workgroup: 256 threads = 4 wavefronts as 2 (M) x 2 (N); block tile 128 rows x
// 64 tokens; each wavefront owns 64 x 32 (two MFMA row tiles).  K advances in
// steps of 128 elements (half a K-quant super-block): the LDS footprint stays
// near 32 KB, so several workgroups share a CU and one's global loads and
// unpacking overlap another's MFMA/VALU phase.  Per step the workgroup stages
//   A: 128 rows x 128 weight codes unpacked to int8 (Q4_0 re-centred to
//      signed so no activation-sum correction is needed), row stride 144 B so
//      16-byte fragment reads of 16 consecutive rows fall in distinct banks;
//   rs/rm: per-row scale (d*sc) and min (dmin*mn) per
//      sub-block, stored [sub][row];
//   B: 64 tokens x 128 int8 activations, cs/cm: activation scale and
//      scale*sum(a) per 32-block.
#pragma once
#include "common.hip.h"
#include "quantize.hip.h"

#define GEMM_BM 128
#define GEMM_BN 64
#define GEMM_KT 128      // K elements per staged tile
#define GEMM_KSUPER 256  // K must be a whole number of these (the K-quant super-block)
#define GEMM_LDA 144     // bytes per staged row (128 + 16 pad)

typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef float v32f __attribute__((ext_vector_type(32)));
typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v2i __attribute__((ext_vector_type(2)));

struct GemmArgs {
    const uint8_t* w;   // [m] rows of native blocks
    const int8_t* bq;   // [n][k] int8 activations
    const float* bs;    // [n][k/32] activation scales
    const float* bsum;  // [n][k/32] scale * sum(a) per block (exact product)
    const void* bh;     // [n][k] the quants as f16, K in 0,2,1,3 order within fours (Q6_K kernel only)
    float* out;
    uint32_t m, n, k;
    uint32_t row_bytes;
    uint64_t ld_m, ld_n;  // out[i*ld_m + j*ld_n]
    const float* resid;   // nullable: out = resid + W.B (same strides)
    float resid_scale;
    // split-K: workgroup z covers k in [z*k_chunk, (z+1)*k_chunk) and writes its partial
    // sums to out + z*part_stride (k_chunk == k, part_stride == 0 when not split)
    uint32_t k_chunk;
    uint64_t part_stride;
    // optional second matrix of the same type and k sharing the launch (and the activations):
    // row tiles [tiles1, gridDim.y) belong to it.  No residual, no split-K for a pair.
    const uint8_t* w2;
    float* out2;
    uint32_t m2, tiles1;
    uint64_t ld_n2;
    // SwiGLU form of the kernel (w = gate, w2 = up, both m x k): nothing goes to out; the Q8_0
    // quantization of silu(gate.x) * (up.x) goes to hq [n][m], hs and hbsum [n][m/32]
    int8_t* hq;
    float* hs;
    float* hbsum;
    // debug instances only: the integer dot of every (row, token, block) as the matrix core
    // delivered it, [m][n][k/32] int32 (Q6_K: [m][n][k/16], f32 bit patterns of the f16 MFMA's result)
    int32_t* dbg_dots;
    // fp8 kernel (gemm_fp8.hip.h) only: the activations' fragment-ordered split copy
    const uint8_t* bf8;
    // SwiGLU form of the fp8 kernel, nullable: the same quants also as f16 [n][m] in the order
    // gemm_act_f16_kernel writes them (what a Q6_K down projection reads: saves that launch)
    uint16_t* hh;
};

// ---- per-type staging of one 128-element K tile of one row -------------------
// `blk` points at the row's 256-element super-block (or run of eight 32-blocks)
// containing the tile, `hs` says which half.  unpack() handles one 16-byte word
// `w` of the tile's packed codes and writes int8 codes to `dst` (the LDS row);
// scales() writes the row's per-sub-block scales.  NSUB = MFMA steps per tile,
// KSTEP = elements per MFMA.
struct GemmQ4K {
    static constexpr int WAVES_PER_SIMD = 3;   // register budget the kernel is compiled for
    static constexpr int NSUB = 4, KSTEP = 32;
    static constexpr bool HAS_MIN = true;
    static constexpr int BLOCK_BYTES = 144;
    static constexpr int WORDS = 4;
    struct Raw { uint4 q; };
    struct RawS { uint4 h; };
    __device__ static void load(Raw& r, const uint8_t* blk, uint32_t hs, uint32_t w) { r.q = ld_u128(blk + 16 + (4 * hs + w) * 16); }
    __device__ static void load_scales(RawS& r, const uint8_t* blk, uint32_t) { r.h = ld_u128(blk); }
    __device__ static void unpack(const Raw& raw, uint32_t w, int8_t* dst) {
        const uint4 q = raw.q;
        uint32_t g = w >> 1, h = w & 1;   // sub-block pair within the tile, half of it
        uint4 lo, hi;
        lo.x = q.x & 0x0F0F0F0Fu; lo.y = q.y & 0x0F0F0F0Fu; lo.z = q.z & 0x0F0F0F0Fu; lo.w = q.w & 0x0F0F0F0Fu;
        hi.x = (q.x >> 4) & 0x0F0F0F0Fu; hi.y = (q.y >> 4) & 0x0F0F0F0Fu;
        hi.z = (q.z >> 4) & 0x0F0F0F0Fu; hi.w = (q.w >> 4) & 0x0F0F0F0Fu;
        *reinterpret_cast<uint4*>(dst + 64 * g + 16 * h) = lo;
        *reinterpret_cast<uint4*>(dst + 64 * g + 32 + 16 * h) = hi;
    }
    __device__ static void scales(const RawS& raw, uint32_t hs, float* rs, float* rm, uint32_t ld) {
        const uint4 h = raw.h;
        float d = h2f(h.x & 0xFFFF), dmin = h2f(h.x >> 16);
        const uint32_t s[3] = {h.y, h.z, h.w};
#pragma unroll
        for (int jj = 0; jj < 4; ++jj) {
            uint32_t sc, mn;
            if (hs == 0) {
                sc = (s[0] >> (8 * jj)) & 63;
                mn = (s[1] >> (8 * jj)) & 63;
            } else {
                uint32_t b8 = (s[2] >> (8 * jj)) & 0xFF;
                sc = (b8 & 0xF) | ((((s[0] >> (8 * jj)) & 0xFF) >> 6) << 4);
                mn = (b8 >> 4) | ((((s[1] >> (8 * jj)) & 0xFF) >> 6) << 4);
            }
            rs[jj * ld] = d * static_cast<float>(sc);
            rm[jj * ld] = dmin * static_cast<float>(mn);
        }
    }
};

// 32-element block formats: a tile is 4 blocks; word w = block index within the tile.
struct GemmQ4_0 {
    static constexpr int WAVES_PER_SIMD = 3;   // register budget the kernel is compiled for
    static constexpr int NSUB = 4, KSTEP = 32;
    static constexpr bool HAS_MIN = false;
    static constexpr int BLOCK_BYTES = 18 * 8;  // bytes per 256 elements
    static constexpr int WORDS = 4;
    struct Raw { uint4 q; };
    struct RawS { uint32_t d[4]; };
    __device__ static void load(Raw& r, const uint8_t* blk, uint32_t hs, uint32_t w) { r.q = ld_u128_a2(blk + (4 * hs + w) * 18 + 2); }
    __device__ static void load_scales(RawS& r, const uint8_t* blk, uint32_t hs) {
#pragma unroll
        for (int b = 0; b < 4; ++b) r.d[b] = ld_u16(blk + 18 * (4 * hs + b));
    }
    __device__ static void unpack(const Raw& raw, uint32_t w, int8_t* dst) {
        const uint4 q = raw.q;
        uint4 lo, hi;  // code - 8, per byte: codes 0..15 -> flip bit 3, sign-extend the nibble
        const uint32_t v[4] = {q.x, q.y, q.z, q.w};
        uint32_t l[4], h[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            uint32_t a = (v[i] & 0x0F0F0F0Fu) ^ 0x08080808u, b = ((v[i] >> 4) & 0x0F0F0F0Fu) ^ 0x08080808u;
            l[i] = a | ((a & 0x08080808u) * 0x1E);  // bits 4..7 = bit 3
            h[i] = b | ((b & 0x08080808u) * 0x1E);
        }
        lo = make_uint4(l[0], l[1], l[2], l[3]);
        hi = make_uint4(h[0], h[1], h[2], h[3]);
        *reinterpret_cast<uint4*>(dst + 32 * w) = lo;
        *reinterpret_cast<uint4*>(dst + 32 * w + 16) = hi;
    }
    __device__ static void scales(const RawS& raw, uint32_t, float* rs, float* rm, uint32_t ld) {
#pragma unroll
        for (int b = 0; b < 4; ++b) rs[b * ld] = h2f(raw.d[b]);
        (void)rm;
    }
};
struct GemmQ4_1 {
    static constexpr int WAVES_PER_SIMD = 3;   // register budget the kernel is compiled for
    static constexpr int NSUB = 4, KSTEP = 32;
    static constexpr bool HAS_MIN = true;   // rm holds -m so that out = rs*dot - rm*sum(a) covers q*d + m
    static constexpr int BLOCK_BYTES = 20 * 8;
    static constexpr int WORDS = 4;
    struct Raw { uint4 q; };
    struct RawS { uint32_t dm[4]; };
    __device__ static void load(Raw& r, const uint8_t* blk, uint32_t hs, uint32_t w) { r.q = ld_u128_a4(blk + (4 * hs + w) * 20 + 4); }
    __device__ static void load_scales(RawS& r, const uint8_t* blk, uint32_t hs) {
#pragma unroll
        for (int b = 0; b < 4; ++b) r.dm[b] = *reinterpret_cast<const uint32_t*>(blk + 20 * (4 * hs + b));
    }
    __device__ static void unpack(const Raw& raw, uint32_t w, int8_t* dst) {
        const uint4 q = raw.q;
        uint4 lo, hi;
        lo.x = q.x & 0x0F0F0F0Fu; lo.y = q.y & 0x0F0F0F0Fu; lo.z = q.z & 0x0F0F0F0Fu; lo.w = q.w & 0x0F0F0F0Fu;
        hi.x = (q.x >> 4) & 0x0F0F0F0Fu; hi.y = (q.y >> 4) & 0x0F0F0F0Fu;
        hi.z = (q.z >> 4) & 0x0F0F0F0Fu; hi.w = (q.w >> 4) & 0x0F0F0F0Fu;
        *reinterpret_cast<uint4*>(dst + 32 * w) = lo;
        *reinterpret_cast<uint4*>(dst + 32 * w + 16) = hi;
    }
    __device__ static void scales(const RawS& raw, uint32_t, float* rs, float* rm, uint32_t ld) {
#pragma unroll
        for (int b = 0; b < 4; ++b) {
            uint32_t dm = raw.dm[b];
            rs[b * ld] = h2f(dm & 0xFFFF);
            rm[b * ld] = -h2f(dm >> 16);
        }
    }
};
struct GemmQ8_0 {
    static constexpr int WAVES_PER_SIMD = 2;   // register budget the kernel is compiled for
    static constexpr int NSUB = 4, KSTEP = 32;
    static constexpr bool HAS_MIN = false;
    static constexpr int BLOCK_BYTES = 34 * 8;
    static constexpr int WORDS = 4;
    struct Raw { uint4 q0, q1; };
    struct RawS { uint32_t d[4]; };
    __device__ static void load(Raw& r, const uint8_t* blk, uint32_t hs, uint32_t w) {
        const uint8_t* b = blk + (4 * hs + w) * 34;
        r.q0 = ld_u128_a2(b + 2);
        r.q1 = ld_u128_a2(b + 18);
    }
    __device__ static void load_scales(RawS& r, const uint8_t* blk, uint32_t hs) {
#pragma unroll
        for (int b = 0; b < 4; ++b) r.d[b] = ld_u16(blk + 34 * (4 * hs + b));
    }
    __device__ static void unpack(const Raw& raw, uint32_t w, int8_t* dst) {
        *reinterpret_cast<uint4*>(dst + 32 * w) = raw.q0;
        *reinterpret_cast<uint4*>(dst + 32 * w + 16) = raw.q1;
    }
    __device__ static void scales(const RawS& raw, uint32_t, float* rs, float* rm, uint32_t ld) {
#pragma unroll
        for (int b = 0; b < 4; ++b) rs[b * ld] = h2f(raw.d[b]);
        (void)rm;
    }
};

// SWIGLU: the workgroup's 128 staged rows are 64 rows of the gate matrix and the same 64 rows of
// the up matrix, and a wavefront's two row tiles are 32 gate rows and the same 32 up rows: both
// factors of an output of the FFN's first half then sit in the same lane and register index, a
// 32-row Q8_0 block of one token in the two lanes of a column, and the activation of the down
// projection is quantized straight from the accumulators.
template <class T, bool SWIGLU = false, bool DBG = false>
__device__ __forceinline__ void gemm_body(GemmArgs p) {
    constexpr int NB = GEMM_KT / 32;  // 32-blocks per tile
    __shared__ __attribute__((aligned(16))) int8_t sA[GEMM_BM * GEMM_LDA];
    __shared__ __attribute__((aligned(16))) int8_t sB[GEMM_BN * GEMM_LDA];
    __shared__ __attribute__((aligned(16))) float sRS[T::NSUB * GEMM_BM];
    __shared__ __attribute__((aligned(16))) float sRM[T::HAS_MIN ? NB * GEMM_BM : 4];
    __shared__ __attribute__((aligned(16))) float sCS[NB * GEMM_BN];
    __shared__ __attribute__((aligned(16))) float sCM[T::HAS_MIN ? NB * GEMM_BN : 4];

    const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const uint32_t wm = wave >> 1, wn = wave & 1;           // wavefront position in the 2 x 2 grid
    const bool second = !SWIGLU && p.w2 != nullptr && blockIdx.y >= p.tiles1;
    const uint8_t* const wmat = second ? p.w2 : p.w;
    float* const omat = second ? p.out2 : p.out;
    const uint32_t mrows = second ? p.m2 : p.m;
    const uint64_t ldn = second ? p.ld_n2 : p.ld_n;
    const uint32_t m0 = (second ? blockIdx.y - p.tiles1 : blockIdx.y) * (SWIGLU ? GEMM_BM / 2 : GEMM_BM), n0 = blockIdx.x * GEMM_BN;
    // staged row r of the tile -> matrix and row; row tile t of wavefront row wm -> first staged row
    auto row_ptr = [&](uint32_t r) __attribute__((always_inline)) {
        if (SWIGLU) return (r < GEMM_BM / 2 ? p.w : p.w2) + static_cast<uint64_t>(min(m0 + (r & (GEMM_BM / 2 - 1)), mrows - 1)) * p.row_bytes;
        return wmat + static_cast<uint64_t>(min(m0 + r, mrows - 1)) * p.row_bytes;
    };
    const uint32_t arow0 = SWIGLU ? wm * 32 : wm * 64, arow_step = SWIGLU ? GEMM_BM / 2 : 32;
    const uint32_t col = lane & 31, half = lane >> 5;
    const uint32_t nb32 = p.k / 32;

    // acc takes the scaled block dots (VALU) and, negated, the min terms (matrix core)
    v16f acc[2];
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[t][r] = 0.0f;

    // per-thread staging assignments, fixed for the whole K loop: AI weight words, one row's
    // scales (threads 0..127), two activation words, one activation scale
    constexpr int AI = GEMM_BM * T::WORDS / 256;
    const uint8_t* a_src[AI];
    int8_t* a_dst[AI];
    uint32_t a_w[AI];
#pragma unroll
    for (int i = 0; i < AI; ++i) {
        const uint32_t it = tid + 256 * i, r = it / T::WORDS;
        a_w[i] = it % T::WORDS;
        a_src[i] = row_ptr(r);
        a_dst[i] = sA + r * GEMM_LDA;
    }
    const uint8_t* s_src = row_ptr(tid & (GEMM_BM - 1));
    const int8_t* b_src[2];
    int8_t* b_dst[2];
    bool b_live[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const uint32_t it = tid + 256 * i, c = it >> 3, wi = it & 7;
        b_live[i] = n0 + c < p.n;
        b_src[i] = p.bq + static_cast<uint64_t>(min(n0 + c, p.n - 1)) * p.k + wi * 16;
        b_dst[i] = sB + c * GEMM_LDA + wi * 16;
    }
    const uint32_t c_tok = tid >> 2, c_b = tid & 3;   // 64 tokens x 4 blocks = 256 threads
    const bool c_live = n0 + c_tok < p.n;
    const uint64_t c_off = static_cast<uint64_t>(min(n0 + c_tok, p.n - 1)) * nb32 + c_b;

    // Register prefetch: the global loads of tile k+1 are issued right after tile k has been
    // written to LDS and stay in flight while tile k is multiplied.
    typename T::Raw ra[AI];
    typename T::RawS rsc;
    uint4 rb[2];
    float rcs, rcm;
    auto fetch = [&](uint32_t k0) {
        const uint32_t hs = (k0 / GEMM_KT) & 1;
        const uint32_t sb_off = (k0 / 256) * T::BLOCK_BYTES;
#pragma unroll
        for (int i = 0; i < AI; ++i) T::load(ra[i], a_src[i] + sb_off, hs, a_w[i]);
        if (tid < GEMM_BM) T::load_scales(rsc, s_src + sb_off, hs);
#pragma unroll
        for (int i = 0; i < 2; ++i) rb[i] = *reinterpret_cast<const uint4*>(b_src[i] + k0);
        rcs = p.bs[c_off + k0 / 32];
        rcm = T::HAS_MIN ? p.bsum[c_off + k0 / 32] : 0.0f;
    };
    const uint32_t k_begin = blockIdx.z * p.k_chunk, k_end = k_begin + p.k_chunk;
    fetch(k_begin);
    for (uint32_t k0 = k_begin; k0 < k_end; k0 += GEMM_KT) {
        const uint32_t hs = (k0 / GEMM_KT) & 1;
        // ---- registers -> LDS: A 128 rows x WORDS words (unpacked), B 64 tokens x 8 words
#pragma unroll
        for (int i = 0; i < AI; ++i) T::unpack(ra[i], a_w[i], a_dst[i]);
        if (tid < GEMM_BM) T::scales(rsc, hs, sRS + tid, sRM + tid, GEMM_BM);
#pragma unroll
        for (int i = 0; i < 2; ++i) *reinterpret_cast<uint4*>(b_dst[i]) = b_live[i] ? rb[i] : make_uint4(0, 0, 0, 0);
        sCS[c_b * GEMM_BN + c_tok] = c_live ? rcs : 0.0f;
        if (T::HAS_MIN) sCM[c_b * GEMM_BN + c_tok] = c_live ? rcm : 0.0f;
        __syncthreads();
        if (k0 + GEMM_KT < k_end) fetch(k0 + GEMM_KT);

        // ---- MFMA over the K tile
        const int8_t* bRow = sB + (wn * 32 + col) * GEMM_LDA;
        {
            // Blocks in pairs.  The per-output scale  rs[row][b] * xs[token][b]  of both blocks of a
            // pair is one two-block outer product on the matrix core (each lane supplies the scale
            // of row `col` and of token `col` for the block of its half): one scalar LDS read per
            // lane per operand instead of the same sixteen row scales re-read by every lane of a
            // half, which made the LDS the limit of this kernel, and no multiply on the VALU.
#pragma unroll
            for (int pr = 0; pr < NB / 2; ++pr) {
                v4i bf[2];
#pragma unroll
                for (int jb = 0; jb < 2; ++jb) bf[jb] = *reinterpret_cast<const v4i*>(bRow + (2 * pr + jb) * 32 + half * 16);
                const float xsl = sCS[(2 * pr + half) * GEMM_BN + wn * 32 + col];
#pragma unroll
                for (int t = 0; t < 2; ++t) {
                    const float rsl = sRS[(2 * pr + half) * GEMM_BM + arow0 + t * arow_step + col];
                    v32f z32;
#pragma unroll
                    for (int e = 0; e < 32; ++e) z32[e] = 0.0f;
                    const v32f sc = __builtin_amdgcn_mfma_f32_32x32x1f32(rsl, xsl, z32, 0, 0, 0);
                    const int8_t* aRow = sA + (arow0 + t * arow_step + col) * GEMM_LDA;
#pragma unroll
                    for (int jb = 0; jb < 2; ++jb) {
                        const v4i af = *reinterpret_cast<const v4i*>(aRow + (2 * pr + jb) * 32 + half * 16);
                        v16i c = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
                        c = __builtin_amdgcn_mfma_i32_32x32x32_i8(af, bf[jb], c, 0, 0, 0);
                        // rows held by this lane: 8*blk + 4*half + r, blk = 0..3, r = 0..3
                        if (DBG) {
                            const uint32_t dtok = n0 + wn * 32 + col, dblk = k0 / 32 + 2 * pr + jb;
#pragma unroll
                            for (int e = 0; e < 16; ++e) {
                                const uint32_t drow = m0 + arow0 + t * arow_step + (e >> 2) * 8 + half * 4 + (e & 3);
                                if (drow < mrows && dtok < p.n)
                                    p.dbg_dots[(static_cast<uint64_t>(drow) * p.n + dtok) * nb32 + dblk] = c[e];
                            }
                        }
#pragma unroll
                        for (int e = 0; e < 16; ++e) acc[t][e] = fmaf(static_cast<float>(c[e]), sc[16 * jb + e], acc[t][e]);
                    }
                }
                if (T::HAS_MIN) {
                    // min terms of the pair's blocks: a rank-2 f32 update on the matrix core
                    const float xm = sCM[(2 * pr + half) * GEMM_BN + wn * 32 + col];
#pragma unroll
                    for (int t = 0; t < 2; ++t) {
                        const float rm = -sRM[(2 * pr + half) * GEMM_BM + arow0 + t * arow_step + col];
                        acc[t] = __builtin_amdgcn_mfma_f32_32x32x2f32(rm, xm, acc[t], 0, 0, 0);
                    }
                }
            }
        }
        __syncthreads();
    }
    // ---- store: lane holds token n0 + wn*32 + col, 32 rows
    const uint32_t tok = n0 + wn * 32 + col;
    if (SWIGLU) {
        // h = silu(gate) * up (cera/src/backend/cpu.rs:2570-2575), then the Q8_0 block of this token's
        // rows m0 + 32 wm .. +31 (cpu.rs:942-958): this lane holds 16 of them, lane ^ 32 the others
        float h[16];
        float amax = 0.0f;
#pragma unroll
        for (int e = 0; e < 16; ++e) {
            const float g = acc[0][e];
            h[e] = __fmul_rn(__fdiv_rn(g, __fadd_rn(1.0f, cera_expf(-g))), acc[1][e]);
            amax = fmaxf(amax, fabsf(h[e]));   // fmaxf drops a NaN operand, as f32::max does
        }
        amax = fmaxf(amax, __shfl_xor(amax, 32, 64));
        const float d = __fdiv_rn(amax, 127.0f), r = __fdiv_rn(1.0f, d);
        const float id = (d != 0.0f && fabsf(r) != __builtin_inff() && r == r) ? r : 0.0f;
        const float scale = h2f(f2h(d));
        uint32_t packed[4];
        int sum = 0;
#pragma unroll
        for (int blk = 0; blk < 4; ++blk) {
            packed[blk] = 0;
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int v = q8_round(h[4 * blk + q], id);
                sum += v;
                packed[blk] |= (static_cast<uint32_t>(v) & 0xFF) << (8 * q);
            }
        }
        sum += __shfl_xor(sum, 32, 64);
        const uint32_t row0 = m0 + wm * 32;   // m % 32 == 0: the block is whole or absent
        if (tok < p.n && row0 < mrows) {
#pragma unroll
            for (int blk = 0; blk < 4; ++blk)
                *reinterpret_cast<uint32_t*>(p.hq + static_cast<uint64_t>(tok) * mrows + row0 + 8 * blk + 4 * half) = packed[blk];
            if (half == 0) {
                const uint64_t b = static_cast<uint64_t>(tok) * (mrows / 32) + row0 / 32;
                p.hs[b] = scale;
                p.hbsum[b] = scale * static_cast<float>(sum);
            }
        }
        return;
    }
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
template <class T, bool SWIGLU = false, bool DBG = false>
static __global__ __launch_bounds__(256, T::WAVES_PER_SIMD) void gemm_kernel(GemmArgs p) {
    gemm_body<T, SWIGLU, DBG>(p);
}


// Sums the split-K partials in a fixed order: out[e] = (resid[e] +) sum_z part[z][e].
__device__ __forceinline__ void gemm_reduce_body(const float* __restrict__ part, uint32_t n_split,
                                                          uint64_t stride, uint64_t n4, float* __restrict__ out,
                                                          const float* resid, float resid_scale, uint64_t n4_first,
                                                          float* __restrict__ out2) {
    const uint64_t e = static_cast<uint64_t>(blockIdx.x) * 256 + threadIdx.x;
    if (e >= n4) return;
    float4 s = reinterpret_cast<const float4*>(part)[e];
    for (uint32_t z = 1; z < n_split; ++z) {
        const float4 v = reinterpret_cast<const float4*>(part + z * stride)[e];
        s.x += v.x; s.y += v.y; s.z += v.z; s.w += v.w;
    }
    // a pair's partials lie side by side; the second matrix's sums go to its own output
    if (e >= n4_first) { reinterpret_cast<float4*>(out2)[e - n4_first] = s; return; }
    if (resid) {
        const float4 r = reinterpret_cast<const float4*>(resid)[e];
        if (resid_scale != 1.0f) { s.x *= resid_scale; s.y *= resid_scale; s.z *= resid_scale; s.w *= resid_scale; }
        s.x = r.x + s.x; s.y = r.y + s.y; s.z = r.z + s.z; s.w = r.w + s.w;
    }
    reinterpret_cast<float4*>(out)[e] = s;
}
static __global__ __launch_bounds__(256) void gemm_reduce_kernel(const float* __restrict__ part, uint32_t n_split,
                                                          uint64_t stride, uint64_t n4, float* __restrict__ out,
                                                          const float* resid, float resid_scale, uint64_t n4_first,
                                                          float* __restrict__ out2) {
    gemm_reduce_body(part, n_split, stride, n4, out, resid, resid_scale, n4_first, out2);
}
