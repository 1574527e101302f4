// CPU oracle (test infrastructure only): the x86 prefill route cera actually runs for Q4_0 and
// Q4_K weights -- the 8-row-interleaved repack built once at load and the "8x8" GEMM kernels
// that consume it:
//   repack_q4_0_8x8 / repack_q4_k_8x8          cera/src/backend/cpu.rs:1145-1196, 1282-1358
//   gemm_q4_0_8x8_q8_0 / gemm_q4_k_8x8_q8_0    cera/src/backend/simd.rs:5215-5366, 5392-5518
//   which weights take it (transformer::gemm_preq, *_repack_supported)
//                                              cera/src/model/transformer.rs:758-775,
//                                              cera/src/backend/cpu.rs:1204-1206, 1364-1366
// In those kernels the eight dpbusd/maddubs lanes of a k-group are eight output ROWS of one
// column, so every output element has an f32 chain of its own (no horizontal sum): one FMA per
// 32-block (Q4_K: an FMA and an FNMADD).  The column tiling (TILE_N) only amortises weight
// decode; it does not change any element's arithmetic, so plain loops restate it exactly.
#include <cmath>
#include <cstring>
#include <vector>
#if defined(__x86_64__)
#include <immintrin.h>
#endif

#include "orc_common.h"

// packed[(sr*nb + b)*128 + g*16 + i] = row 8sr + i/4 (low nibble) | row 8sr + 4 + i/4 (high
// nibble) at element 4g + i%4 of 32-block b.
static inline uint8_t nib_q4_0(const uint8_t* src, uint64_t nb, uint64_t row, uint64_t b, uint32_t e) {
    const uint8_t* qs = src + (row * nb + b) * 18 + 2;
    return e < 16 ? (qs[e] & 0x0F) : (qs[e - 16] >> 4);
}
static inline uint8_t nib_q4_k(const uint8_t* src, uint64_t sb, uint64_t row, uint64_t block, uint32_t e) {
    const uint64_t bi = block / 8, s = block % 8;
    const uint8_t byte = src[(row * sb + bi) * 144 + 16 + (s / 2) * 32 + e];
    return (s % 2 == 0) ? (byte & 0x0F) : (byte >> 4);
}

// cpu.rs:1145-1196.  packed: (m/8)*(k/32)*128 bytes; scales: (m/8)*(k/32)*8 floats.
ORC_API int orc_repack_q4_0_8x8(const uint8_t* src, uint64_t m, uint64_t k, uint8_t* packed, float* scales) {
    if (m % 8 || k % 32) return -1;
    const uint64_t nb = k / 32;
    for (uint64_t sr = 0; sr < m / 8; ++sr)
        for (uint64_t b = 0; b < nb; ++b) {
            for (uint32_t r = 0; r < 8; ++r) {
                uint16_t d;
                std::memcpy(&d, src + ((8 * sr + r) * nb + b) * 18, 2);
                scales[(sr * nb + b) * 8 + r] = orc_f16_to_f32(d);
            }
            for (uint32_t g = 0; g < 8; ++g)
                for (uint32_t i = 0; i < 16; ++i) {
                    const uint32_t e = 4 * g + (i % 4);
                    const uint8_t lo = nib_q4_0(src, nb, 8 * sr + i / 4, b, e), hi = nib_q4_0(src, nb, 8 * sr + 4 + i / 4, b, e);
                    packed[(sr * nb + b) * 128 + g * 16 + i] = uint8_t(lo | (hi << 4));
                }
        }
    return 0;
}

// cpu.rs:1282-1358.  dsc / dmn: (m/8)*(k/32)*8 floats, the baked d*sc[s] and dmin*mn[s].
ORC_API int orc_repack_q4_k_8x8(const uint8_t* src, uint64_t m, uint64_t k, uint8_t* packed, float* dsc, float* dmn) {
    if (m % 8 || k % 256) return -1;
    const uint64_t sb = k / 256, nb32 = k / 32;
    for (uint64_t sr = 0; sr < m / 8; ++sr)
        for (uint64_t bi = 0; bi < sb; ++bi) {
            for (uint32_t r = 0; r < 8; ++r) {
                const OrcBlockQ4K* blk = reinterpret_cast<const OrcBlockQ4K*>(src + ((8 * sr + r) * sb + bi) * 144);
                const float d = orc_f16_to_f32(blk->d), dmin = orc_f16_to_f32(blk->dmin);
                uint8_t sc[8], mn[8];
                orc_decode_q4km_scales(blk->scales, sc, mn);
                for (uint32_t s = 0; s < 8; ++s) {
                    const uint64_t block = bi * 8 + s;
                    dsc[(sr * nb32 + block) * 8 + r] = d * float(sc[s]);
                    dmn[(sr * nb32 + block) * 8 + r] = dmin * float(mn[s]);
                }
            }
            for (uint32_t s = 0; s < 8; ++s) {
                const uint64_t block = bi * 8 + s;
                for (uint32_t g = 0; g < 8; ++g)
                    for (uint32_t i = 0; i < 16; ++i) {
                        const uint32_t e = 4 * g + (i % 4);
                        const uint8_t lo = nib_q4_k(src, sb, 8 * sr + i / 4, block, e), hi = nib_q4_k(src, sb, 8 * sr + 4 + i / 4, block, e);
                        packed[(sr * nb32 + block) * 128 + g * 16 + i] = uint8_t(lo | (hi << 4));
                    }
            }
        }
    return 0;
}

// The integer part both kernels share: acc[r] = sum over the 32 elements of block `b` of
// q[row 8sr + r][e] * a[e], read back out of the packed layout the way `unpack` + dot32u +
// _mm256_add_epi32 over the eight k-groups do (simd.rs:5273-5283, 5297-5306).
static inline void block_acc8(const uint8_t* pk /*128 bytes*/, const int8_t* a /*32*/, int32_t acc[8]) {
    for (int r = 0; r < 8; ++r) acc[r] = 0;
    for (int g = 0; g < 8; ++g)
        for (int i = 0; i < 16; ++i) {
            const uint8_t byte = pk[g * 16 + i];
            const int32_t av = a[4 * g + (i % 4)];
            acc[i / 4] += int32_t(byte & 0x0F) * av;
            acc[4 + i / 4] += int32_t(byte >> 4) * av;
        }
}
#if defined(__x86_64__)
// The same eight sums with AVX2 (integer sums are order-free, so this is an exact twin, used when the
// host has AVX2 only to make the checker fast): group g holds rows 0..3 in the low nibbles and rows
// 4..7 in the high nibbles of 16 bytes, four elements per row; maddubs + madd leave one sum per row.
__attribute__((target("avx2"))) static void block_acc8_avx2(const uint8_t* pk, const int8_t* a, int32_t acc[8]) {
    const __m256i m4 = _mm256_set1_epi8(0x0F), ones = _mm256_set1_epi16(1);
    __m256i s = _mm256_setzero_si256();
    for (int g = 0; g < 8; ++g) {
        const __m128i p = _mm_loadu_si128(reinterpret_cast<const __m128i*>(pk + 16 * g));
        const __m256i both = _mm256_and_si256(_mm256_set_m128i(_mm_srli_epi16(p, 4), p), m4);
        int32_t a4;
        std::memcpy(&a4, a + 4 * g, 4);
        s = _mm256_add_epi32(s, _mm256_madd_epi16(_mm256_maddubs_epi16(both, _mm256_set1_epi32(a4)), ones));
    }
    _mm256_storeu_si256(reinterpret_cast<__m256i*>(acc), s);
}
#endif
typedef void (*BlockAcc8)(const uint8_t*, const int8_t*, int32_t*);
static BlockAcc8 pick_block_acc8() {
#if defined(__x86_64__)
    if (orc_have_avx2()) return block_acc8_avx2;
#endif
    return block_acc8;
}
static void col_sums32(const int8_t* q, uint64_t k, int32_t* sums) {   // q8_0_col_sums, simd.rs:5651-5665
    for (uint64_t b = 0; b < k / 32; ++b) {
        int32_t s = 0;
        for (int t = 0; t < 32; ++t) s += q[32 * b + t];
        sums[b] = s;
    }
}

// simd.rs:5215-5366: per block  eff = cvt(acc) - 8*sum_a ; facc = fma(eff, d_row*d_a, facc).
ORC_API int orc_gemm_q4_0_8x8_q8_0(const uint8_t* packed, const float* scales, const float* b_scales, const int8_t* b_quants,
                                   float* out, uint64_t m, uint64_t n, uint64_t k) {
    if (m % 8 || k % 32) return -1;
    const uint64_t nb = k / 32;
    std::vector<int32_t> cs(nb);
    const BlockAcc8 block_acc8 = pick_block_acc8();
    for (uint64_t j = 0; j < n; ++j) {
        col_sums32(b_quants + j * k, k, cs.data());
        for (uint64_t sr = 0; sr < m / 8; ++sr) {
            float facc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
            for (uint64_t b = 0; b < nb; ++b) {
                int32_t acc[8];
                block_acc8(packed + (sr * nb + b) * 128, b_quants + j * k + 32 * b, acc);
                const float d_a = b_scales[j * nb + b];
                const float sub = 8.0f * float(cs[b]);
                for (int r = 0; r < 8; ++r) {
                    const float scale = scales[(sr * nb + b) * 8 + r] * d_a;
                    const float eff = float(acc[r]) - sub;
                    facc[r] = fmaf(eff, scale, facc[r]);
                }
            }
            for (int r = 0; r < 8; ++r) out[(8 * sr + r) * n + j] = facc[r];
        }
    }
    return 0;
}

// simd.rs:5392-5518: per block  facc = fma(cvt(acc), dsc*xs, facc); facc = fnmadd(dmn, xs*sx, facc).
ORC_API int orc_gemm_q4_k_8x8_q8_0(const uint8_t* packed, const float* dsc, const float* dmn, const float* b_scales,
                                   const int8_t* b_quants, float* out, uint64_t m, uint64_t n, uint64_t k) {
    if (m % 8 || k % 256) return -1;
    const uint64_t nb32 = k / 32;
    std::vector<int32_t> cs(nb32);
    const BlockAcc8 block_acc8 = pick_block_acc8();
    for (uint64_t j = 0; j < n; ++j) {
        col_sums32(b_quants + j * k, k, cs.data());
        for (uint64_t sr = 0; sr < m / 8; ++sr) {
            float facc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
            for (uint64_t block = 0; block < nb32; ++block) {
                int32_t acc[8];
                block_acc8(packed + (sr * nb32 + block) * 128, b_quants + j * k + 32 * block, acc);
                const float xs = b_scales[j * nb32 + block];
                const float xsum = xs * float(cs[block]);
                const uint64_t sbase = (sr * nb32 + block) * 8;
                for (int r = 0; r < 8; ++r) {
                    const float eff = dsc[sbase + r] * xs;
                    facc[r] = fmaf(float(acc[r]), eff, facc[r]);
                    facc[r] = fmaf(-dmn[sbase + r], xsum, facc[r]);   // _mm256_fnmadd_ps: -(a*b) + c, one rounding
                }
            }
            for (int r = 0; r < 8; ++r) out[(8 * sr + r) * n + j] = facc[r];
        }
    }
    return 0;
}

// transformer::gemm_preq on an x86 host without `blas` (transformer.rs:710-788): a weight that was
// repacked at load (Q4_0 with m % 8 == 0; Q4_K with m % 8 == 0 and k % 256 == 0) takes its 8x8
// kernel, everything else gemm_preq_dispatch in the standard layout.  Repacks on the fly (the
// reference keeps the repacked copy from load; same bytes).
ORC_API int orc_gemm_preq_x86(uint32_t dtype, const void* wv, const float* b_scales, const int8_t* b_quants, float* out,
                              uint64_t m, uint64_t n, uint64_t k, int variant) {
    const uint8_t* w = static_cast<const uint8_t*>(wv);
    if (dtype == ORC_Q4_0 && m % 8 == 0 && k % 32 == 0) {
        std::vector<uint8_t> packed((m / 8) * (k / 32) * 128);
        std::vector<float> scales((m / 8) * (k / 32) * 8);
        if (orc_repack_q4_0_8x8(w, m, k, packed.data(), scales.data())) return -1;
        return orc_gemm_q4_0_8x8_q8_0(packed.data(), scales.data(), b_scales, b_quants, out, m, n, k);
    }
    if (dtype == ORC_Q4_K && m % 8 == 0 && k % 256 == 0) {
        std::vector<uint8_t> packed((m / 8) * (k / 32) * 128);
        std::vector<float> dsc((m / 8) * (k / 32) * 8), dmn(dsc.size());
        if (orc_repack_q4_k_8x8(w, m, k, packed.data(), dsc.data(), dmn.data())) return -1;
        return orc_gemm_q4_k_8x8_q8_0(packed.data(), dsc.data(), dmn.data(), b_scales, b_quants, out, m, n, k);
    }
    return orc_gemm_preq(dtype, wv, b_scales, b_quants, out, m, n, k, variant);
}
