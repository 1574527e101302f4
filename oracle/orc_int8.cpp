// CPU oracle (test infrastructure only): Q8_0 activation quantizer and the
// int8 GEMV/GEMM kernels of cera's x86 AVX2 tier, restated twice:
//   variant 0 -- portable scalar code that emulates the eight f32 lanes of a
//                ymm register one by one (defines the float order);
//   variant 1 -- an AVX2+FMA intrinsics twin (same operations on real ymm
//                registers; also the timed CPU baseline).
// The two must agree bit for bit; tests check that.
#include "orc_common.h"

#include <cmath>
#include <cstring>
#include <vector>

#if defined(__x86_64__)
#include <immintrin.h>
#define ORC_X86 1
#else
#define ORC_X86 0
#endif

// ---------------------------------------------------------------------------
// Q8_0 activation quantizer -- cpu.rs:942-958.
//   amax via f32::max (NaN lanes ignored), d = amax/127,
//   id = 1/d unless d == 0 or 1/d is not finite (then 0),
//   scale = f16 round trip of d, q = clamp(round_ties_even(v*id), -128, 127)
//   with Rust's saturating `as i8` (NaN -> 0).
void orc_quantize_q8_0(const float* x, uint64_t k, float* scales, int8_t* quants) {
    for (uint64_t bi = 0; bi < k / 32; ++bi) {
        const float* blk = x + 32 * bi;
        float amax = 0.0f;
        for (int t = 0; t < 32; ++t) amax = fmaxf(amax, fabsf(blk[t]));
        float d = amax / 127.0f;
        float r = 1.0f / d;
        float id = (d != 0.0f && std::isfinite(r)) ? r : 0.0f;
        scales[bi] = orc_f16_to_f32(orc_f32_to_f16(d));
        for (int t = 0; t < 32; ++t) {
            float v = nearbyintf(blk[t] * id);  // default rounding mode: ties to even
            int8_t q;
            if (std::isnan(v)) q = 0;
            else if (v <= -128.0f) q = -128;
            else if (v >= 127.0f) q = 127;
            else q = int8_t(int(v));
            quants[32 * bi + t] = q;
        }
    }
}

// ---------------------------------------------------------------------------
// Weight unpacking shared by the integer spec and the scalar kernels.
// Each helper writes the 32 weights of one 32-element group in activation order.

// simd.rs:4563-4571 (unpack_q4_0): lo nibbles = elements 0..15, hi = 16..31, minus 8.
static inline void unpack_q4_0(const uint8_t* qs, int8_t* w) {
    for (int i = 0; i < 16; ++i) {
        w[i] = int8_t(int(qs[i] & 0xF) - 8);
        w[i + 16] = int8_t(int(qs[i] >> 4) - 8);
    }
}
// simd.rs:5931-5934 (Q4_1: same nibble order, unbiased).
static inline void unpack_q4_1(const uint8_t* qs, int8_t* w) {
    for (int i = 0; i < 16; ++i) {
        w[i] = int8_t(qs[i] & 0xF);
        w[i + 16] = int8_t(qs[i] >> 4);
    }
}
// simd.rs:5757-5760: chunk g of 32 bytes; lo nibbles = sub-block 2g, hi = 2g+1.
static inline void unpack_q4_k(const uint8_t* qs, int s, int8_t* w) {
    const uint8_t* c = qs + 32 * (s >> 1);
    if (s & 1) for (int i = 0; i < 32; ++i) w[i] = int8_t(c[i] >> 4);
    else       for (int i = 0; i < 32; ++i) w[i] = int8_t(c[i] & 0xF);
}
// simd.rs:6039-6053: group (nh, g) of a Q6_K block, unsigned 0..63.
static inline void unpack_q6_k(const OrcBlockQ6K* b, int nh, int g, int8_t* w) {
    const uint8_t* ql = b->ql + nh * 64 + (g & 1) * 32;
    const uint8_t* qh = b->qh + nh * 32;
    for (int i = 0; i < 32; ++i) {
        int l4 = (g < 2) ? (ql[i] & 0xF) : (ql[i] >> 4);
        int h2 = (qh[i] >> (2 * g)) & 3;
        w[i] = int8_t(l4 | (h2 << 4));
    }
}

static inline int32_t dot_n(const int8_t* w, const int8_t* a, int n) {
    int32_t s = 0;
    for (int i = 0; i < n; ++i) s += int32_t(w[i]) * int32_t(a[i]);
    return s;
}
static inline int32_t sum_n(const int8_t* a, int n) {
    int32_t s = 0;
    for (int i = 0; i < n; ++i) s += a[i];
    return s;
}

// The integer quantities the kernels are built from (brute force; mirrors the
// reference's own integer test reference, simd.rs:6609-6629, and the lane
// algebra at simd.rs:5772-5774, 6070-6073).
int orc_block_dots(uint32_t dtype, const void* wv, uint64_t m, uint64_t k, const int8_t* xq,
                   int32_t* dots, int32_t* asums) {
    const uint8_t* w = static_cast<const uint8_t*>(wv);
    uint64_t rb = orc_row_bytes(dtype, k);
    if (rb == 0) return -1;
    int8_t wq[32];
    switch (dtype) {
        case ORC_Q4_0:
            for (uint64_t i = 0; i < m; ++i)
                for (uint64_t b = 0; b < k / 32; ++b) {
                    auto* blk = reinterpret_cast<const OrcBlockQ4_0*>(w + i * rb + 18 * b);
                    unpack_q4_0(blk->qs, wq);
                    dots[i * (k / 32) + b] = dot_n(wq, xq + 32 * b, 32);
                }
            return 0;
        case ORC_Q8_0:
            for (uint64_t i = 0; i < m; ++i)
                for (uint64_t b = 0; b < k / 32; ++b) {
                    auto* blk = reinterpret_cast<const OrcBlockQ8_0*>(w + i * rb + 34 * b);
                    dots[i * (k / 32) + b] = dot_n(blk->qs, xq + 32 * b, 32);
                }
            return 0;
        case ORC_Q4_1:
            if (asums) for (uint64_t b = 0; b < k / 32; ++b) asums[b] = sum_n(xq + 32 * b, 32);
            for (uint64_t i = 0; i < m; ++i)
                for (uint64_t b = 0; b < k / 32; ++b) {
                    auto* blk = reinterpret_cast<const OrcBlockQ4_1*>(w + i * rb + 20 * b);
                    unpack_q4_1(blk->qs, wq);
                    dots[i * (k / 32) + b] = dot_n(wq, xq + 32 * b, 32);
                }
            return 0;
        case ORC_Q4_K:
            if (asums) for (uint64_t b = 0; b < k / 32; ++b) asums[b] = sum_n(xq + 32 * b, 32);
            for (uint64_t i = 0; i < m; ++i)
                for (uint64_t bi = 0; bi < k / 256; ++bi) {
                    auto* blk = reinterpret_cast<const OrcBlockQ4K*>(w + i * rb + 144 * bi);
                    for (int s = 0; s < 8; ++s) {
                        unpack_q4_k(blk->qs, s, wq);
                        dots[i * (k / 32) + bi * 8 + s] = dot_n(wq, xq + 256 * bi + 32 * s, 32);
                    }
                }
            return 0;
        case ORC_Q6_K:
            if (asums) for (uint64_t h = 0; h < k / 16; ++h) asums[h] = sum_n(xq + 16 * h, 16);
            for (uint64_t i = 0; i < m; ++i)
                for (uint64_t bi = 0; bi < k / 256; ++bi) {
                    auto* blk = reinterpret_cast<const OrcBlockQ6K*>(w + i * rb + 210 * bi);
                    for (int nh = 0; nh < 2; ++nh)
                        for (int g = 0; g < 4; ++g) {
                            unpack_q6_k(blk, nh, g, wq);
                            uint64_t xb = bi * 8 + nh * 4 + g;
                            dots[i * (k / 16) + 2 * xb] = dot_n(wq, xq + 32 * xb, 16);
                            dots[i * (k / 16) + 2 * xb + 1] = dot_n(wq + 16, xq + 32 * xb + 16, 16);
                        }
                }
            return 0;
        default:
            return -1;
    }
}

// ---------------------------------------------------------------------------
// variant 0: scalar emulation of the ymm lanes.

// dot32 / dot32u (simd.rs:6319-6341): maddubs pairs then madd with ones gives
// eight i32 lanes, lane j = sum of products of elements 4j..4j+3.  The i16
// intermediate of maddubs cannot saturate for these operand ranges
// (simd.rs:6265-6273), so plain integer arithmetic is the same function.
static inline void lanes8(const int8_t* w, const int8_t* a, float* lanes) {
    for (int j = 0; j < 8; ++j) {
        int32_t s = 0;
        for (int i = 0; i < 4; ++i) s += int32_t(w[4 * j + i]) * int32_t(a[4 * j + i]);
        lanes[j] = float(s);  // _mm256_cvtepi32_ps
    }
}
// hsum256_ps (simd.rs:4546-4554): (v0+v4 + v2+v6) + (v1+v5 + v3+v7).
static inline float hsum8(const float* v) {
    float s0 = v[4] + v[0], s1 = v[5] + v[1], s2 = v[6] + v[2], s3 = v[7] + v[3];
    float t0 = s0 + s2, t1 = s1 + s3;
    return t0 + t1;
}
static inline void fma8(float* acc, const float* lanes, float scale) {
    for (int j = 0; j < 8; ++j) acc[j] = fmaf(lanes[j], scale, acc[j]);
}

// row_dot_q4_0 / row_dot_q8_0 (simd.rs:4593-4637); also every (row, col) of
// gemm_q4_0_q8_0 / gemm_q8_0_q8_0 (strip and row kernels, simd.rs:4718-5010),
// whose per-element arithmetic is the same single-accumulator chain.
static float s_row_q4_0(const uint8_t* row, const float* xs, const int8_t* xq, uint64_t nb) {
    float acc[8] = {0}, lanes[8];
    int8_t w[32];
    for (uint64_t b = 0; b < nb; ++b) {
        auto* blk = reinterpret_cast<const OrcBlockQ4_0*>(row + 18 * b);
        unpack_q4_0(blk->qs, w);
        lanes8(w, xq + 32 * b, lanes);
        fma8(acc, lanes, orc_f16_to_f32(blk->d) * xs[b]);
    }
    return hsum8(acc);
}
static float s_row_q8_0(const uint8_t* row, const float* xs, const int8_t* xq, uint64_t nb) {
    float acc[8] = {0}, lanes[8];
    for (uint64_t b = 0; b < nb; ++b) {
        auto* blk = reinterpret_cast<const OrcBlockQ8_0*>(row + 34 * b);
        lanes8(blk->qs, xq + 32 * b, lanes);
        fma8(acc, lanes, orc_f16_to_f32(blk->d) * xs[b]);
    }
    return hsum8(acc);
}
// gemm_q4_1_q8_0 (simd.rs:5893-5976): one accumulator, macc added.
static float s_row_q4_1(const uint8_t* row, const float* xs, const int8_t* xq, const int32_t* cs,
                        uint64_t nb) {
    float acc[8] = {0}, lanes[8], macc = 0.0f;
    int8_t w[32];
    for (uint64_t b = 0; b < nb; ++b) {
        auto* blk = reinterpret_cast<const OrcBlockQ4_1*>(row + 20 * b);
        float d = orc_f16_to_f32(blk->d), mmin = orc_f16_to_f32(blk->m);
        unpack_q4_1(blk->qs, w);
        lanes8(w, xq + 32 * b, lanes);
        fma8(acc, lanes, xs[b] * d);
        macc += xs[b] * mmin * float(cs[b]);
    }
    return hsum8(acc) + macc;
}
// gemm_q4_k_q8_0 (simd.rs:5693-5878).  nacc = 4 is the n == 1 decode branch
// (:5742-5795), nacc = 1 the KQ_COLS-tiled branch (:5796-5851).
static float s_row_q4_k(const uint8_t* row, const float* xs, const int8_t* xq, const int32_t* cs,
                        uint64_t sb, int nacc) {
    float facc[4][8] = {{0}}, lanes[8], macc = 0.0f;
    int8_t w[32];
    int slot = 0;
    for (uint64_t bi = 0; bi < sb; ++bi) {
        auto* blk = reinterpret_cast<const OrcBlockQ4K*>(row + 144 * bi);
        float d = orc_f16_to_f32(blk->d), dmin = orc_f16_to_f32(blk->dmin);
        uint8_t sc[8], mn[8];
        orc_decode_q4km_scales(blk->scales, sc, mn);
        for (int s = 0; s < 8; ++s) {
            uint64_t xb = bi * 8 + s;
            float dsc = d * float(sc[s]);
            float dmn = dmin * float(mn[s]);
            unpack_q4_k(blk->qs, s, w);
            lanes8(w, xq + 32 * xb, lanes);
            fma8(facc[slot], lanes, xs[xb] * dsc);
            macc += xs[xb] * dmn * float(cs[xb]);
            slot = (slot + 1) & (nacc - 1);
        }
    }
    if (nacc == 4) {
        float f[8];
        for (int j = 0; j < 8; ++j) f[j] = (facc[0][j] + facc[1][j]) + (facc[2][j] + facc[3][j]);
        return hsum8(f) - macc;
    }
    return hsum8(facc[0]) - macc;
}
// gemm_q6_k_q8_0 (simd.rs:5988-6195); nacc as above (:6025-6093 / :6094-6168).
static float s_row_q6_k(const uint8_t* row, const float* xs, const int8_t* xq, const int32_t* cs16,
                        uint64_t sb, int nacc) {
    float facc[4][8] = {{0}}, lanes[8], macc = 0.0f;
    int8_t w[32];
    int slot = 0;
    for (uint64_t bi = 0; bi < sb; ++bi) {
        auto* blk = reinterpret_cast<const OrcBlockQ6K*>(row + 210 * bi);
        float d = orc_f16_to_f32(blk->d);
        float d32 = d * 32.0f;
        for (int nh = 0; nh < 2; ++nh)
            for (int g = 0; g < 4; ++g) {
                unpack_q6_k(blk, nh, g, w);
                float sc0 = float(blk->scales[nh * 8 + 2 * g]);
                float sc1 = float(blk->scales[nh * 8 + 2 * g + 1]);
                uint64_t xb = bi * 8 + nh * 4 + g;
                float x = xs[xb];
                float s0 = (sc0 * d) * x, s1 = (sc1 * d) * x;  // _mm256_mul_ps(sc_split_d, xs)
                lanes8(w, xq + 32 * xb, lanes);
                float* acc = facc[slot];
                for (int j = 0; j < 4; ++j) acc[j] = fmaf(lanes[j], s0, acc[j]);
                for (int j = 4; j < 8; ++j) acc[j] = fmaf(lanes[j], s1, acc[j]);
                float sx0 = float(cs16[2 * xb]), sx1 = float(cs16[2 * xb + 1]);
                macc += x * d32 * (sc0 * sx0 + sc1 * sx1);
                slot = (slot + 1) & (nacc - 1);
            }
    }
    if (nacc == 4) {
        float f[8];
        for (int j = 0; j < 8; ++j) f[j] = (facc[0][j] + facc[1][j]) + (facc[2][j] + facc[3][j]);
        return hsum8(f) - macc;
    }
    return hsum8(facc[0]) - macc;
}

// ---------------------------------------------------------------------------
// variant 1: AVX2 + FMA intrinsics twin (operation for operation).
#if ORC_X86
#define ORC_AVX2 __attribute__((target("avx2,fma")))

ORC_AVX2 static inline __m256i v_dot32u(__m256i w, __m256i a) {  // simd.rs:6319
    return _mm256_madd_epi16(_mm256_maddubs_epi16(w, a), _mm256_set1_epi16(1));
}
ORC_AVX2 static inline __m128i v_dot16u(__m128i w, __m128i a) {  // simd.rs:6328
    return _mm_madd_epi16(_mm_maddubs_epi16(w, a), _mm_set1_epi16(1));
}
ORC_AVX2 static inline __m256i v_dot32(__m256i w, __m256i a) {  // simd.rs:6339
    return v_dot32u(_mm256_sign_epi8(w, w), _mm256_sign_epi8(a, w));
}
ORC_AVX2 static inline float v_hsum256_ps(__m256 v) {  // simd.rs:4546
    __m128 hi = _mm256_extractf128_ps(v, 1);
    __m128 lo = _mm256_castps256_ps128(v);
    __m128 sum = _mm_add_ps(hi, lo);
    __m128 shuf = _mm_movehl_ps(sum, sum);
    sum = _mm_add_ps(sum, shuf);
    shuf = _mm_shuffle_ps(sum, sum, 0x55);
    return _mm_cvtss_f32(_mm_add_ss(sum, shuf));
}
ORC_AVX2 static inline int32_t v_hsum256_epi32(__m256i v) {
    __m128i s = _mm_add_epi32(_mm256_castsi256_si128(v), _mm256_extracti128_si256(v, 1));
    s = _mm_add_epi32(s, _mm_srli_si128(s, 8));
    s = _mm_add_epi32(s, _mm_srli_si128(s, 4));
    return _mm_cvtsi128_si32(s);
}
ORC_AVX2 static inline int32_t v_hsum128_epi32(__m128i v) {  // simd.rs:5641
    __m128i s = _mm_add_epi32(v, _mm_srli_si128(v, 8));
    s = _mm_add_epi32(s, _mm_srli_si128(s, 4));
    return _mm_cvtsi128_si32(s);
}
ORC_AVX2 static inline __m256i v_unpack_q4_0(const uint8_t* qs) {  // simd.rs:4563
    __m128i qb = _mm_loadu_si128(reinterpret_cast<const __m128i*>(qs));
    __m128i mask = _mm_set1_epi8(0x0F);
    __m128i lo = _mm_and_si128(qb, mask);
    __m128i hi = _mm_and_si128(_mm_srli_epi16(qb, 4), mask);
    return _mm256_sub_epi8(_mm256_set_m128i(hi, lo), _mm256_set1_epi8(8));
}
ORC_AVX2 static void v_col_sums(const int8_t* q, uint64_t k, int32_t* sums) {  // simd.rs:5651
    __m256i ones = _mm256_set1_epi8(1);
    for (uint64_t b = 0; b < k / 32; ++b) {
        __m256i x = _mm256_loadu_si256(reinterpret_cast<const __m256i*>(q + 32 * b));
        sums[b] = v_hsum256_epi32(v_dot32u(ones, x));
    }
}
ORC_AVX2 static void v_col_sums16(const int8_t* q, uint64_t k, int32_t* sums) {  // simd.rs:5670
    __m128i ones = _mm_set1_epi8(1);
    for (uint64_t h = 0; h < k / 16; ++h) {
        __m128i x = _mm_loadu_si128(reinterpret_cast<const __m128i*>(q + 16 * h));
        sums[h] = v_hsum128_epi32(v_dot16u(ones, x));
    }
}
ORC_AVX2 static float v_row_q4_0(const uint8_t* row, const float* xs, const int8_t* xq, uint64_t nb) {
    __m256 acc = _mm256_setzero_ps();
    for (uint64_t b = 0; b < nb; ++b) {
        auto* blk = reinterpret_cast<const OrcBlockQ4_0*>(row + 18 * b);
        __m256i w = v_unpack_q4_0(blk->qs);
        __m256i a = _mm256_loadu_si256(reinterpret_cast<const __m256i*>(xq + 32 * b));
        __m256 scale = _mm256_set1_ps(orc_f16_to_f32(blk->d) * xs[b]);
        acc = _mm256_fmadd_ps(_mm256_cvtepi32_ps(v_dot32(w, a)), scale, acc);
    }
    return v_hsum256_ps(acc);
}
ORC_AVX2 static float v_row_q8_0(const uint8_t* row, const float* xs, const int8_t* xq, uint64_t nb) {
    __m256 acc = _mm256_setzero_ps();
    for (uint64_t b = 0; b < nb; ++b) {
        auto* blk = reinterpret_cast<const OrcBlockQ8_0*>(row + 34 * b);
        __m256i w = _mm256_loadu_si256(reinterpret_cast<const __m256i*>(blk->qs));
        __m256i a = _mm256_loadu_si256(reinterpret_cast<const __m256i*>(xq + 32 * b));
        __m256 scale = _mm256_set1_ps(orc_f16_to_f32(blk->d) * xs[b]);
        acc = _mm256_fmadd_ps(_mm256_cvtepi32_ps(v_dot32(w, a)), scale, acc);
    }
    return v_hsum256_ps(acc);
}
ORC_AVX2 static float v_row_q4_1(const uint8_t* row, const float* xs, const int8_t* xq,
                                 const int32_t* cs, uint64_t nb) {
    __m128i mask128 = _mm_set1_epi8(0x0F);
    __m256 facc = _mm256_setzero_ps();
    float macc = 0.0f;
    for (uint64_t b = 0; b < nb; ++b) {
        auto* blk = reinterpret_cast<const OrcBlockQ4_1*>(row + 20 * b);
        float d = orc_f16_to_f32(blk->d), mmin = orc_f16_to_f32(blk->m);
        __m128i qb = _mm_loadu_si128(reinterpret_cast<const __m128i*>(blk->qs));
        __m128i lo = _mm_and_si128(qb, mask128);
        __m128i hi = _mm_and_si128(_mm_srli_epi16(qb, 4), mask128);
        __m256i w = _mm256_inserti128_si256(_mm256_castsi128_si256(lo), hi, 1);
        __m256i x = _mm256_loadu_si256(reinterpret_cast<const __m256i*>(xq + 32 * b));
        __m256 lanes = _mm256_cvtepi32_ps(v_dot32u(w, x));
        facc = _mm256_fmadd_ps(lanes, _mm256_set1_ps(xs[b] * d), facc);
        macc += xs[b] * mmin * float(cs[b]);
    }
    return v_hsum256_ps(facc) + macc;
}
ORC_AVX2 static float v_row_q4_k(const uint8_t* row, const float* xs, const int8_t* xq,
                                 const int32_t* cs, uint64_t sb, int nacc) {
    __m256i mask_0f = _mm256_set1_epi8(0x0F);
    __m256 facc[4] = {_mm256_setzero_ps(), _mm256_setzero_ps(), _mm256_setzero_ps(), _mm256_setzero_ps()};
    float macc = 0.0f;
    int slot = 0;
    for (uint64_t bi = 0; bi < sb; ++bi) {
        auto* blk = reinterpret_cast<const OrcBlockQ4K*>(row + 144 * bi);
        float d = orc_f16_to_f32(blk->d), dmin = orc_f16_to_f32(blk->dmin);
        uint8_t sc[8], mn[8];
        orc_decode_q4km_scales(blk->scales, sc, mn);
        for (int g = 0; g < 4; ++g) {
            __m256i qb = _mm256_loadu_si256(reinterpret_cast<const __m256i*>(blk->qs + 32 * g));
            __m256i wv[2] = {_mm256_and_si256(qb, mask_0f),
                             _mm256_and_si256(_mm256_srli_epi16(qb, 4), mask_0f)};
            for (int h = 0; h < 2; ++h) {
                int s = 2 * g + h;
                uint64_t xb = bi * 8 + s;
                float dsc = d * float(sc[s]);
                float dmn = dmin * float(mn[s]);
                __m256i x = _mm256_loadu_si256(reinterpret_cast<const __m256i*>(xq + 32 * xb));
                __m256 lanes = _mm256_cvtepi32_ps(v_dot32u(wv[h], x));
                facc[slot] = _mm256_fmadd_ps(lanes, _mm256_set1_ps(xs[xb] * dsc), facc[slot]);
                macc += xs[xb] * dmn * float(cs[xb]);
                slot = (slot + 1) & (nacc - 1);
            }
        }
    }
    if (nacc == 4) {
        __m256 f = _mm256_add_ps(_mm256_add_ps(facc[0], facc[1]), _mm256_add_ps(facc[2], facc[3]));
        return v_hsum256_ps(f) - macc;
    }
    return v_hsum256_ps(facc[0]) - macc;
}
ORC_AVX2 static float v_row_q6_k(const uint8_t* row, const float* xs, const int8_t* xq,
                                 const int32_t* cs16, uint64_t sb, int nacc) {
    __m256i mask_0f = _mm256_set1_epi8(0x0F), mask_03 = _mm256_set1_epi8(0x03);
    __m256 facc[4] = {_mm256_setzero_ps(), _mm256_setzero_ps(), _mm256_setzero_ps(), _mm256_setzero_ps()};
    float macc = 0.0f;
    int slot = 0;
    for (uint64_t bi = 0; bi < sb; ++bi) {
        auto* blk = reinterpret_cast<const OrcBlockQ6K*>(row + 210 * bi);
        float d = orc_f16_to_f32(blk->d);
        float d32 = d * 32.0f;
        for (int nh = 0; nh < 2; ++nh) {
            __m256i qhb = _mm256_loadu_si256(reinterpret_cast<const __m256i*>(blk->qh + 32 * nh));
            for (int g = 0; g < 4; ++g) {
                __m256i qlb = _mm256_loadu_si256(
                    reinterpret_cast<const __m256i*>(blk->ql + nh * 64 + (g & 1) * 32));
                __m256i l4 = g < 2 ? _mm256_and_si256(qlb, mask_0f)
                                   : _mm256_and_si256(_mm256_srli_epi16(qlb, 4), mask_0f);
                __m256i h2 = _mm256_and_si256(_mm256_srl_epi16(qhb, _mm_cvtsi32_si128(2 * g)), mask_03);
                __m256i w = _mm256_or_si256(l4, _mm256_slli_epi16(h2, 4));
                float sc0 = float(blk->scales[nh * 8 + 2 * g]);
                float sc1 = float(blk->scales[nh * 8 + 2 * g + 1]);
                uint64_t xb = bi * 8 + nh * 4 + g;
                __m256 sc_split_d = _mm256_set_m128(_mm_set1_ps(sc1 * d), _mm_set1_ps(sc0 * d));
                __m256i x = _mm256_loadu_si256(reinterpret_cast<const __m256i*>(xq + 32 * xb));
                __m256 lanes = _mm256_cvtepi32_ps(v_dot32u(w, x));
                float xsv = xs[xb];
                __m256 scale = _mm256_mul_ps(sc_split_d, _mm256_set1_ps(xsv));
                facc[slot] = _mm256_fmadd_ps(lanes, scale, facc[slot]);
                macc += xsv * d32 * (sc0 * float(cs16[2 * xb]) + sc1 * float(cs16[2 * xb + 1]));
                slot = (slot + 1) & (nacc - 1);
            }
        }
    }
    if (nacc == 4) {
        __m256 f = _mm256_add_ps(_mm256_add_ps(facc[0], facc[1]), _mm256_add_ps(facc[2], facc[3]));
        return v_hsum256_ps(f) - macc;
    }
    return v_hsum256_ps(facc[0]) - macc;
}
int orc_have_avx2(void) { return __builtin_cpu_supports("avx2") && __builtin_cpu_supports("fma"); }
#else
int orc_have_avx2(void) { return 0; }
#endif

// ---------------------------------------------------------------------------
static void col_sums_scalar(const int8_t* q, uint64_t k, int width, int32_t* sums) {
    for (uint64_t b = 0; b < k / width; ++b) sums[b] = sum_n(q + width * b, width);
}

// One output element.  cs = per-32 (Q4_1/Q4_K) or per-16 (Q6_K) activation sums.
static inline float row_col(uint32_t dtype, const uint8_t* row, const float* xs, const int8_t* xq,
                            const int32_t* cs, uint64_t k, int nacc, int variant) {
#if ORC_X86
    if (variant == 1) {
        switch (dtype) {
            case ORC_Q4_0: return v_row_q4_0(row, xs, xq, k / 32);
            case ORC_Q8_0: return v_row_q8_0(row, xs, xq, k / 32);
            case ORC_Q4_1: return v_row_q4_1(row, xs, xq, cs, k / 32);
            case ORC_Q4_K: return v_row_q4_k(row, xs, xq, cs, k / 256, nacc);
            default:       return v_row_q6_k(row, xs, xq, cs, k / 256, nacc);
        }
    }
#endif
    (void)variant;
    switch (dtype) {
        case ORC_Q4_0: return s_row_q4_0(row, xs, xq, k / 32);
        case ORC_Q8_0: return s_row_q8_0(row, xs, xq, k / 32);
        case ORC_Q4_1: return s_row_q4_1(row, xs, xq, cs, k / 32);
        case ORC_Q4_K: return s_row_q4_k(row, xs, xq, cs, k / 256, nacc);
        default:       return s_row_q6_k(row, xs, xq, cs, k / 256, nacc);
    }
}

static bool int8_dtype(uint32_t dtype) {
    return dtype == ORC_Q4_0 || dtype == ORC_Q8_0 || dtype == ORC_Q4_1 || dtype == ORC_Q4_K ||
           dtype == ORC_Q6_K;
}

static void make_col_sums(uint32_t dtype, const int8_t* bq, uint64_t n, uint64_t k, int variant,
                          std::vector<int32_t>& cs, uint64_t& per_col) {
    per_col = 0;
    if (dtype == ORC_Q4_1 || dtype == ORC_Q4_K) per_col = k / 32;
    else if (dtype == ORC_Q6_K) per_col = k / 16;
    cs.assign(n * per_col + 1, 0);
    for (uint64_t j = 0; j < n && per_col; ++j) {
#if ORC_X86
        if (variant == 1) {
            if (dtype == ORC_Q6_K) v_col_sums16(bq + j * k, k, cs.data() + j * per_col);
            else v_col_sums(bq + j * k, k, cs.data() + j * per_col);
            continue;
        }
#endif
        col_sums_scalar(bq + j * k, k, dtype == ORC_Q6_K ? 16 : 32, cs.data() + j * per_col);
    }
}

// gemm_preq_dispatch (cpu.rs:1437-1557), standard (non-repacked) layout.
int orc_gemm_preq(uint32_t dtype, const void* wv, const float* b_scales, const int8_t* b_quants,
                  float* out, uint64_t m, uint64_t n, uint64_t k, int variant) {
    if (!int8_dtype(dtype)) return -1;
    uint64_t rb = orc_row_bytes(dtype, k);
    if (rb == 0) return -1;
    if (variant == 1 && !orc_have_avx2()) return -2;
    const uint8_t* w = static_cast<const uint8_t*>(wv);
    std::vector<int32_t> cs;
    uint64_t per_col;
    make_col_sums(dtype, b_quants, n, k, variant, cs, per_col);
    // K-quants take the four-accumulator branch only when n == 1.
    int nacc = (n == 1 && (dtype == ORC_Q4_K || dtype == ORC_Q6_K)) ? 4 : 1;
    for (uint64_t i = 0; i < m; ++i)
        for (uint64_t j = 0; j < n; ++j)
            out[i * n + j] = row_col(dtype, w + i * rb, b_scales + j * (k / 32), b_quants + j * k,
                                     cs.data() + j * per_col, k, nacc, variant);
    return 0;
}

int orc_gemv(uint32_t dtype, const void* wv, const float* x, float* y, uint64_t m, uint64_t k,
             int variant) {
    uint64_t rb = orc_row_bytes(dtype, k);
    if (rb == 0) return -1;
    const uint8_t* w = static_cast<const uint8_t*>(wv);
    if (int8_dtype(dtype)) {
        std::vector<float> xs(k / 32);
        std::vector<int8_t> xq(k);
        orc_quantize_q8_0(x, k, xs.data(), xq.data());
        return orc_gemm_preq(dtype, wv, xs.data(), xq.data(), y, m, 1, k, variant);
    }
    if (dtype == ORC_Q5_K) {  // cpu.rs:1830-1854: scalar f32 dot on unquantized x
        for (uint64_t i = 0; i < m; ++i) y[i] = orc_vec_dot_row_f32(dtype, w + i * rb, x, k);
        return 0;
    }
    return -1;
}

// f64 reference built from exact integer block dots (test pin, not a kernel).
int orc_gemv_f64ref(uint32_t dtype, const void* wv, const float* x, double* y, uint64_t m,
                    uint64_t k) {
    if (!int8_dtype(dtype)) return -1;
    uint64_t rb = orc_row_bytes(dtype, k);
    if (rb == 0) return -1;
    const uint8_t* w = static_cast<const uint8_t*>(wv);
    std::vector<float> xs(k / 32);
    std::vector<int8_t> xq(k);
    orc_quantize_q8_0(x, k, xs.data(), xq.data());
    uint64_t nd = dtype == ORC_Q6_K ? k / 16 : k / 32;
    std::vector<int32_t> dots(m * nd), as(nd);
    orc_block_dots(dtype, wv, m, k, xq.data(), dots.data(), as.data());
    for (uint64_t i = 0; i < m; ++i) {
        const uint8_t* row = w + i * rb;
        double acc = 0.0;
        const int32_t* dr = dots.data() + i * nd;
        if (dtype == ORC_Q4_0) {
            for (uint64_t b = 0; b < k / 32; ++b)
                acc += double(orc_f16_to_f32(reinterpret_cast<const OrcBlockQ4_0*>(row + 18 * b)->d)) * xs[b] * dr[b];
        } else if (dtype == ORC_Q8_0) {
            for (uint64_t b = 0; b < k / 32; ++b)
                acc += double(orc_f16_to_f32(reinterpret_cast<const OrcBlockQ8_0*>(row + 34 * b)->d)) * xs[b] * dr[b];
        } else if (dtype == ORC_Q4_1) {
            for (uint64_t b = 0; b < k / 32; ++b) {
                auto* blk = reinterpret_cast<const OrcBlockQ4_1*>(row + 20 * b);
                acc += double(xs[b]) * (double(orc_f16_to_f32(blk->d)) * dr[b] + double(orc_f16_to_f32(blk->m)) * as[b]);
            }
        } else if (dtype == ORC_Q4_K) {
            for (uint64_t bi = 0; bi < k / 256; ++bi) {
                auto* blk = reinterpret_cast<const OrcBlockQ4K*>(row + 144 * bi);
                double d = orc_f16_to_f32(blk->d), dmin = orc_f16_to_f32(blk->dmin);
                uint8_t sc[8], mn[8];
                orc_decode_q4km_scales(blk->scales, sc, mn);
                for (int s = 0; s < 8; ++s) {
                    uint64_t xb = bi * 8 + s;
                    acc += double(xs[xb]) * (d * sc[s] * dr[xb] - dmin * mn[s] * as[xb]);
                }
            }
        } else {
            for (uint64_t bi = 0; bi < k / 256; ++bi) {
                auto* blk = reinterpret_cast<const OrcBlockQ6K*>(row + 210 * bi);
                double d = orc_f16_to_f32(blk->d);
                for (int h = 0; h < 16; ++h) {
                    uint64_t hb = bi * 16 + h;
                    // group (nh, g) covers scales nh*8 + 2g, +1 == 16-element run index h
                    acc += double(xs[hb / 2]) * d * double(blk->scales[h]) * (double(dr[hb]) - 32.0 * as[hb]);
                }
            }
        }
        y[i] = acc;
    }
    return 0;
}
