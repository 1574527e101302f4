// CPU oracle (test infrastructure only): glue ops and decode attention,
// restating cera/src/backend/cpu.rs and cera/src/model/transformer.rs.
#include "orc_common.h"

#include <cmath>
#include <cstring>
#include <vector>

#if defined(__x86_64__)
#include <immintrin.h>
#define ORC_X86 1
#define ORC_AVX2 __attribute__((target("avx2,fma")))
#else
#define ORC_X86 0
#endif

static inline float bits_f32(uint32_t b) { float f; std::memcpy(&f, &b, 4); return f; }
static inline uint32_t f32_bits(float f) { uint32_t b; std::memcpy(&b, &f, 4); return b; }

// cpu.rs:2479-2496 -- f64 sum of squares, inv_rms narrowed to f32.
void orc_rmsnorm(float* x, const float* weight, uint64_t n, float eps) {
    double sum_sq = 0.0;
    for (uint64_t i = 0; i < n; ++i) sum_sq += double(x[i]) * double(x[i]);
    double mean = sum_sq / double(n);
    double rms = std::sqrt(mean + double(eps));
    float inv_rms = float(1.0 / rms);
    for (uint64_t i = 0; i < n; ++i) x[i] = x[i] * inv_rms * weight[i];
}

// cpu.rs:2504-2544 -- ggml's polynomial expf, no FMA contraction.
float orc_expf(float x) {
    const float R = bits_f32(0x4B400000u);
    const float LOG2E = bits_f32(0x3FB8AA3Bu);
    const float LN2_HI = bits_f32(0x3F317200u);
    const float LN2_LO = bits_f32(0x35BFBE8Eu);
    const float C1 = bits_f32(0x3F7FFFF6u);
    const float C2 = bits_f32(0x3EFFFEDBu);
    const float C3 = bits_f32(0x3E2AAF33u);
    const float C4 = bits_f32(0x3D2B9F17u);
    const float C5 = bits_f32(0x3C072010u);

    float z = R + x * LOG2E;
    float n = z - R;
    float b = x - n * LN2_HI - n * LN2_LO;
    uint32_t e = f32_bits(z) << 23;
    float k = bits_f32(e + f32_bits(1.0f));
    float u = b * b;
    float j = C1 * b + (C2 + C3 * b + (C4 + C5 * b) * u) * u;
    float abs_n = bits_f32(f32_bits(n) & 0x7FFFFFFFu);
    if (abs_n <= 126.0f) {
        return k + j * k;
    } else if (abs_n > 192.0f) {
        return n > 0.0f ? INFINITY : 0.0f;
    } else {
        uint32_t d = n <= 0.0f ? 0x82000000u : 0u;
        float s1 = bits_f32(d + 0x7f000000u);
        float s2 = bits_f32(e - d);
        return (s2 + s2 * j) * s1;
    }
}

// cpu.rs:2570-2575
void orc_silu_mul(float* gate, const float* up, uint64_t n) {
    for (uint64_t i = 0; i < n; ++i) gate[i] = gate[i] / (1.0f + orc_expf(-gate[i])) * up[i];
}

// cpu.rs:2617-2633 -- max via f32::max, f64 sum, f32 inverse.
void orc_softmax(float* x, uint64_t n) {
    float mx = -INFINITY;
    for (uint64_t i = 0; i < n; ++i) mx = fmaxf(mx, x[i]);
    double sum = 0.0;
    for (uint64_t i = 0; i < n; ++i) {
        x[i] = orc_expf(x[i] - mx);
        sum += double(x[i]);
    }
    float inv_sum = float(1.0 / sum);
    for (uint64_t i = 0; i < n; ++i) x[i] *= inv_sum;
}

// cpu.rs:5223-5228
void orc_add(float* a, const float* b, uint64_t n) {
    for (uint64_t i = 0; i < n; ++i) a[i] += b[i];
}

// cpu.rs:5161-5180 (rope_norm_pairs): interleaved pairs, theta iterated in f32,
// libm sincos.
static void rope_norm_head(float* head, float theta_start, uint32_t head_dim, float freq_base,
                           const float* ff) {
    float theta_scale = powf(freq_base, -2.0f / float(head_dim));
    float theta_base = theta_start;
    for (uint32_t i = 0; i < head_dim / 2; ++i) {
        float f = ff ? ff[i] : 1.0f;
        float theta = theta_base / f;
        float s = sinf(theta), c = cosf(theta);
        float x0 = head[2 * i], x1 = head[2 * i + 1];
        head[2 * i] = x0 * c - x1 * s;
        head[2 * i + 1] = x0 * s + x1 * c;
        theta_base *= theta_scale;
    }
}
// cpu.rs:5091-5125
void orc_rope_norm(float* q, float* k, uint64_t pos, uint32_t n_heads, uint32_t n_kv_heads,
                   uint32_t head_dim, float freq_base, const float* freq_factors) {
    for (uint32_t h = 0; h < n_heads; ++h) rope_norm_head(q + h * head_dim, float(pos), head_dim, freq_base, freq_factors);
    for (uint32_t h = 0; h < n_kv_heads; ++h) rope_norm_head(k + h * head_dim, float(pos), head_dim, freq_base, freq_factors);
}
// cpu.rs:5031-5045 (apply_rope_to_head): split-half (NEOX) pairing.
static void rope_neox_head(float* head, float theta_start, uint32_t head_dim, float freq_base) {
    uint32_t half = head_dim / 2;
    float theta_scale = powf(freq_base, -2.0f / float(head_dim));
    float theta = theta_start;
    for (uint32_t i = 0; i < half; ++i) {
        float s = sinf(theta), c = cosf(theta);
        float x0 = head[i], x1 = head[i + half];
        head[i] = x0 * c - x1 * s;
        head[i + half] = x0 * s + x1 * c;
        theta *= theta_scale;
    }
}
void orc_rope_neox(float* q, float* k, uint64_t pos, uint32_t n_heads, uint32_t n_kv_heads,
                   uint32_t head_dim, float freq_base) {
    for (uint32_t h = 0; h < n_heads; ++h) rope_neox_head(q + h * head_dim, float(pos), head_dim, freq_base);
    for (uint32_t h = 0; h < n_kv_heads; ++h) rope_neox_head(k + h * head_dim, float(pos), head_dim, freq_base);
}

// cpu.rs:5065-5086 (apply_rope_delta_to_head, NEOX) and :5145-5153
// (apply_rope_norm_delta_to_head): compose a further rotation of delta_pos onto an
// already-rotated head; the same recurrences with theta_start = delta_pos as f32.
// NEOX takes no frequency factors.
void orc_rope_delta_head(float* head, int32_t delta_pos, uint32_t head_dim, float freq_base, uint32_t rope_type,
                         const float* freq_factors) {
    if (rope_type == 0) rope_neox_head(head, float(delta_pos), head_dim, freq_base);
    else rope_norm_head(head, float(delta_pos), head_dim, freq_base, freq_factors);
}

// sampler.rs:20-30 -- strict >, lowest index on ties, NaN never wins.
uint32_t orc_argmax(const float* logits, uint64_t n) {
    uint32_t best_i = 0;
    float best_v = -INFINITY;
    for (uint64_t i = 0; i < n; ++i)
        if (logits[i] > best_v) { best_v = logits[i]; best_i = uint32_t(i); }
    return best_i;
}

// ---------------------------------------------------------------------------
// Decode attention.  variant 0: the scalar loops (cpu.rs:3275-3282, 3352-3362);
// variant 1: the AVX2 twins (cpu.rs:3503-3553, 3555-3589).  They differ in
// float summation order, as in the reference.
#if ORC_X86
ORC_AVX2 static inline float v_hsum256(__m256 v) {  // cpu.rs:3489
    __m128 hi = _mm256_extractf128_ps(v, 1);
    __m128 lo = _mm256_castps256_ps128(v);
    __m128 s128 = _mm_add_ps(lo, hi);
    __m128 s64 = _mm_add_ps(s128, _mm_movehl_ps(s128, s128));
    __m128 s32 = _mm_add_ss(s64, _mm_shuffle_ps(s64, s64, 1));
    return _mm_cvtss_f32(s32);
}
ORC_AVX2 static void v_attn_scores(const float* q, const float* kc, float* scores, uint64_t kv_dim,
                                   uint64_t off, uint32_t hd, float scale, uint64_t L) {
    __m256 qv[32];
    uint32_t nq = hd / 8;
    for (uint32_t i = 0; i < nq; ++i) qv[i] = _mm256_loadu_ps(q + 8 * i);
    for (uint64_t t = 0; t < L; ++t) {
        const float* kp = kc + t * kv_dim + off;
        __m256 s0 = _mm256_setzero_ps(), s1 = _mm256_setzero_ps();
        uint32_t i = 0;
        while (i + 2 <= nq) {
            s0 = _mm256_fmadd_ps(qv[i], _mm256_loadu_ps(kp + 8 * i), s0);
            s1 = _mm256_fmadd_ps(qv[i + 1], _mm256_loadu_ps(kp + 8 * (i + 1)), s1);
            i += 2;
        }
        if (i < nq) s0 = _mm256_fmadd_ps(qv[i], _mm256_loadu_ps(kp + 8 * i), s0);
        scores[t] = v_hsum256(_mm256_add_ps(s0, s1)) * scale;
    }
}
ORC_AVX2 static void v_attn_values(const float* scores, const float* vc, float* out, uint64_t kv_dim,
                                   uint64_t off, uint32_t hd, uint64_t L) {
    __m256 acc[32];
    uint32_t nv = hd / 8;
    for (uint32_t i = 0; i < nv; ++i) acc[i] = _mm256_setzero_ps();
    for (uint64_t t = 0; t < L; ++t) {
        __m256 s = _mm256_set1_ps(scores[t]);
        const float* vp = vc + t * kv_dim + off;
        for (uint32_t i = 0; i < nv; ++i) acc[i] = _mm256_fmadd_ps(s, _mm256_loadu_ps(vp + 8 * i), acc[i]);
    }
    for (uint32_t i = 0; i < nv; ++i) _mm256_storeu_ps(out + 8 * i, acc[i]);
}
static bool avx2_ok() { return __builtin_cpu_supports("avx2") && __builtin_cpu_supports("fma"); }
#else
static bool avx2_ok() { return false; }
#endif

void orc_attn_scores(const float* q, const float* kc, float* scores, uint64_t kv_dim, uint64_t off,
                     uint32_t hd, float scale, uint64_t L, int variant) {
#if ORC_X86
    if (variant == 1 && hd % 8 == 0 && hd <= 256 && avx2_ok()) {
        v_attn_scores(q, kc, scores, kv_dim, off, hd, scale, L);
        return;
    }
#endif
    (void)variant;
    for (uint64_t t = 0; t < L; ++t) {
        float dot = 0.0f;
        const float* kp = kc + t * kv_dim + off;
        for (uint32_t d = 0; d < hd; ++d) dot += q[d] * kp[d];
        scores[t] = dot * scale;
    }
}
void orc_attn_values(const float* scores, const float* vc, float* out, uint64_t kv_dim, uint64_t off,
                     uint32_t hd, uint64_t L, int variant) {
#if ORC_X86
    if (variant == 1 && hd % 8 == 0 && hd <= 256 && avx2_ok()) {
        v_attn_values(scores, vc, out, kv_dim, off, hd, L);
        return;
    }
#endif
    (void)variant;
    for (uint32_t d = 0; d < hd; ++d) out[d] = 0.0f;
    for (uint64_t t = 0; t < L; ++t) {
        float s = scores[t];
        const float* vp = vc + t * kv_dim + off;
        for (uint32_t d = 0; d < hd; ++d) out[d] += s * vp[d];
    }
}

// transformer.rs:1164-1220 (decode_attn_head) over all heads (:1249-1305);
// query head h reads kv head h / (n_heads / n_kv_heads).
void orc_decode_attention(const float* q, const float* kc, const float* vc, uint32_t n_heads,
                          uint32_t n_kv_heads, uint32_t hd, float scale, uint64_t L, float* out,
                          int variant) {
    std::vector<float> scores(L);
    uint64_t kv_dim = uint64_t(n_kv_heads) * hd;
    uint32_t group = n_heads / n_kv_heads;
    for (uint32_t h = 0; h < n_heads; ++h) {
        uint64_t off = uint64_t(h / group) * hd;
        orc_attn_scores(q + h * hd, kc, scores.data(), kv_dim, off, hd, scale, L, variant);
        orc_softmax(scores.data(), L);
        orc_attn_values(scores.data(), vc, out + h * hd, kv_dim, off, hd, L, variant);
    }
}

// ---------------------------------------------------------------------------
// Causal prefill attention, tiled online softmax -- the scalar route of
// flash_attention_gqa_cpu (cpu.rs:4028-4241, FLASH_TILE_KV = 32): per query j
// (absolute position start_pos + j) scores over positions 0..=start_pos+j in
// tiles of 32, running max, f64 running sum, ggml expf.  The reference's AVX2
// twin (cpu.rs:4261-4412) differs only in f32 summation order.
// q is [n_queries][head_dim] for ONE head (row-major); out likewise.
void orc_flash_attention_head(const float* q, const float* k_cache, const float* v_cache, float* out,
                              uint64_t n_queries, uint64_t kv_dim, uint64_t kv_h_offset,
                              uint32_t head_dim, float scale, uint64_t start_pos) {
    const int TILE = 32;
    std::vector<float> acc(head_dim);
    float tile_scores[TILE];
    for (uint64_t j = 0; j < n_queries; ++j) {
        uint64_t max_kv = start_pos + j + 1;
        const float* ql = q + j * head_dim;
        float running_max = -INFINITY;
        double running_sum = 0.0;
        for (auto& a : acc) a = 0.0f;
        for (uint64_t kv_start = 0; kv_start < max_kv; kv_start += TILE) {
            uint64_t kv_end = kv_start + TILE < max_kv ? kv_start + TILE : max_kv;
            int tile_len = int(kv_end - kv_start);
            for (int ti = 0; ti < tile_len; ++ti) {
                const float* kp = k_cache + (kv_start + ti) * kv_dim + kv_h_offset;
                float dot = 0.0f;
                for (uint32_t d = 0; d < head_dim; ++d) dot += ql[d] * kp[d];
                tile_scores[ti] = dot * scale;
            }
            float tile_max = -INFINITY;
            for (int ti = 0; ti < tile_len; ++ti) tile_max = fmaxf(tile_max, tile_scores[ti]);
            float new_max = fmaxf(running_max, tile_max);
            float rescale = running_max > -INFINITY ? orc_expf(running_max - new_max) : 0.0f;
            double tile_sum = 0.0;
            for (int ti = 0; ti < tile_len; ++ti) {
                tile_scores[ti] = orc_expf(tile_scores[ti] - new_max);
                tile_sum += double(tile_scores[ti]);
            }
            for (uint32_t d = 0; d < head_dim; ++d) acc[d] *= rescale;
            for (int ti = 0; ti < tile_len; ++ti) {
                float s = tile_scores[ti];
                const float* vp = v_cache + (kv_start + ti) * kv_dim + kv_h_offset;
                for (uint32_t d = 0; d < head_dim; ++d) acc[d] += s * vp[d];
            }
            running_sum = running_sum * double(rescale) + tile_sum;
            running_max = new_max;
        }
        float inv_sum = float(1.0 / running_sum);
        for (uint32_t d = 0; d < head_dim; ++d) out[j * head_dim + d] = acc[d] * inv_sum;
    }
}

// ---------------------------------------------------------------------------
// flash_attention_gqa_avx2 (cpu.rs:4261-4412), what flash_attention_gqa_cpu dispatches to on an
// AVX2 host without AVX-512 (:4028-4140).  Same tiles and the same scalar online-softmax
// bookkeeping as the scalar route; the QK dot is two 8-lane FMA chains over the even / odd
// 8-wide slices of the head, added, folded by hsum256 (cpu.rs:3489) and scaled; the weighted-V
// accumulate is one FMA per (key, column), keys in order.  The tile maximum uses `>`
// (NaN never wins), the running maximum f32::max.
//   variant 1: the intrinsics, operation for operation;
//   variant 2: the same lane algebra in plain C (any host) -- bit-identical to variant 1;
//   variant 0: the scalar route above.
static void flash_head_avx2_order(const float* q, const float* k_cache, const float* v_cache, float* out,
                                  uint64_t n_queries, uint64_t kv_dim, uint64_t kv_h_offset, uint32_t head_dim,
                                  float scale, uint64_t start_pos) {
    const int TILE = 32;
    const uint32_t n_vecs = head_dim / 8;
    std::vector<float> acc(head_dim);
    float tile_scores[TILE];
    for (uint64_t j = 0; j < n_queries; ++j) {
        const uint64_t max_kv = start_pos + j + 1;
        const float* ql = q + j * head_dim;
        for (auto& a : acc) a = 0.0f;
        float running_max = -INFINITY;
        double running_sum = 0.0;
        for (uint64_t kv_start = 0; kv_start < max_kv; kv_start += TILE) {
            const uint64_t kv_end = kv_start + TILE < max_kv ? kv_start + TILE : max_kv;
            const int tile_len = int(kv_end - kv_start);
            for (int ti = 0; ti < tile_len; ++ti) {
                const float* kp = k_cache + (kv_start + ti) * kv_dim + kv_h_offset;
                float s0[8] = {0}, s1[8] = {0};
                uint32_t i = 0;
                while (i + 2 <= n_vecs) {
                    for (int l = 0; l < 8; ++l) s0[l] = fmaf(ql[8 * i + l], kp[8 * i + l], s0[l]);
                    for (int l = 0; l < 8; ++l) s1[l] = fmaf(ql[8 * (i + 1) + l], kp[8 * (i + 1) + l], s1[l]);
                    i += 2;
                }
                if (i < n_vecs)
                    for (int l = 0; l < 8; ++l) s0[l] = fmaf(ql[8 * i + l], kp[8 * i + l], s0[l]);
                float v[8];
                for (int l = 0; l < 8; ++l) v[l] = s0[l] + s1[l];
                // hsum256: lo + hi, then movehl add, then lane 0 + lane 1
                const float a0 = v[0] + v[4], a1 = v[1] + v[5], a2 = v[2] + v[6], a3 = v[3] + v[7];
                const float b0 = a0 + a2, b1 = a1 + a3;
                tile_scores[ti] = (b0 + b1) * scale;
            }
            float tile_max = -INFINITY;
            for (int ti = 0; ti < tile_len; ++ti)
                if (tile_scores[ti] > tile_max) tile_max = tile_scores[ti];
            const float new_max = fmaxf(running_max, tile_max);
            const float rescale = running_max > -INFINITY ? orc_expf(running_max - new_max) : 0.0f;
            double tile_sum = 0.0;
            for (int ti = 0; ti < tile_len; ++ti) {
                tile_scores[ti] = orc_expf(tile_scores[ti] - new_max);
                tile_sum += double(tile_scores[ti]);
            }
            for (uint32_t d = 0; d < head_dim; ++d) acc[d] = acc[d] * rescale;
            for (int ti = 0; ti < tile_len; ++ti) {
                const float sv = tile_scores[ti];
                const float* vp = v_cache + (kv_start + ti) * kv_dim + kv_h_offset;
                for (uint32_t d = 0; d < head_dim; ++d) acc[d] = fmaf(sv, vp[d], acc[d]);
            }
            running_sum = running_sum * double(rescale) + tile_sum;
            running_max = new_max;
        }
        const float inv_sum = float(1.0 / running_sum);
        for (uint32_t d = 0; d < head_dim; ++d) out[j * head_dim + d] = acc[d] * inv_sum;
    }
}
#if ORC_X86
ORC_AVX2 static void v_flash_head(const float* q, const float* k_cache, const float* v_cache, float* out,
                                  uint64_t n_queries, uint64_t kv_dim, uint64_t kv_h_offset, uint32_t head_dim,
                                  float scale, uint64_t start_pos) {
    const int TILE = 32;
    const uint32_t n_vecs = head_dim / 8;
    __m256 q_vecs[32], acc_vecs[32];
    float tile_scores[TILE];
    for (uint64_t j = 0; j < n_queries; ++j) {
        const uint64_t max_kv = start_pos + j + 1;
        for (uint32_t i = 0; i < n_vecs; ++i) {
            q_vecs[i] = _mm256_loadu_ps(q + j * head_dim + 8 * i);
            acc_vecs[i] = _mm256_setzero_ps();
        }
        float running_max = -INFINITY;
        double running_sum = 0.0;
        for (uint64_t kv_start = 0; kv_start < max_kv; kv_start += TILE) {
            const uint64_t kv_end = kv_start + TILE < max_kv ? kv_start + TILE : max_kv;
            const int tile_len = int(kv_end - kv_start);
            for (int ti = 0; ti < tile_len; ++ti) {
                const float* kp = k_cache + (kv_start + ti) * kv_dim + kv_h_offset;
                __m256 s0 = _mm256_setzero_ps(), s1 = _mm256_setzero_ps();
                uint32_t i = 0;
                while (i + 2 <= n_vecs) {
                    s0 = _mm256_fmadd_ps(q_vecs[i], _mm256_loadu_ps(kp + 8 * i), s0);
                    s1 = _mm256_fmadd_ps(q_vecs[i + 1], _mm256_loadu_ps(kp + 8 * i + 8), s1);
                    i += 2;
                }
                if (i < n_vecs) s0 = _mm256_fmadd_ps(q_vecs[i], _mm256_loadu_ps(kp + 8 * i), s0);
                tile_scores[ti] = v_hsum256(_mm256_add_ps(s0, s1)) * scale;
            }
            float tile_max = -INFINITY;
            for (int ti = 0; ti < tile_len; ++ti)
                if (tile_scores[ti] > tile_max) tile_max = tile_scores[ti];
            const float new_max = fmaxf(running_max, tile_max);
            const float rescale = running_max > -INFINITY ? orc_expf(running_max - new_max) : 0.0f;
            double tile_sum = 0.0;
            for (int ti = 0; ti < tile_len; ++ti) {
                tile_scores[ti] = orc_expf(tile_scores[ti] - new_max);
                tile_sum += double(tile_scores[ti]);
            }
            const __m256 rescale_v = _mm256_set1_ps(rescale);
            for (uint32_t i = 0; i < n_vecs; ++i) acc_vecs[i] = _mm256_mul_ps(acc_vecs[i], rescale_v);
            for (int ti = 0; ti < tile_len; ++ti) {
                const __m256 sv = _mm256_set1_ps(tile_scores[ti]);
                const float* vp = v_cache + (kv_start + ti) * kv_dim + kv_h_offset;
                for (uint32_t i = 0; i < n_vecs; ++i) acc_vecs[i] = _mm256_fmadd_ps(sv, _mm256_loadu_ps(vp + 8 * i), acc_vecs[i]);
            }
            running_sum = running_sum * double(rescale) + tile_sum;
            running_max = new_max;
        }
        const __m256 inv_sum_v = _mm256_set1_ps(float(1.0 / running_sum));
        for (uint32_t i = 0; i < n_vecs; ++i) _mm256_storeu_ps(out + j * head_dim + 8 * i, _mm256_mul_ps(acc_vecs[i], inv_sum_v));
    }
}
#endif
void orc_flash_attention_head_v(const float* q, const float* k_cache, const float* v_cache, float* out,
                                uint64_t n_queries, uint64_t kv_dim, uint64_t kv_h_offset, uint32_t head_dim,
                                float scale, uint64_t start_pos, int variant) {
    // the dispatcher takes the vector kernels only for head_dim % 8 == 0 and head_dim <= 256 (cpu.rs:4060-4140)
    if (variant == 0 || head_dim % 8 != 0 || head_dim > 256) {
        orc_flash_attention_head(q, k_cache, v_cache, out, n_queries, kv_dim, kv_h_offset, head_dim, scale, start_pos);
        return;
    }
#if ORC_X86
    if (variant == 1 && avx2_ok()) {
        v_flash_head(q, k_cache, v_cache, out, n_queries, kv_dim, kv_h_offset, head_dim, scale, start_pos);
        return;
    }
#endif
    flash_head_avx2_order(q, k_cache, v_cache, out, n_queries, kv_dim, kv_h_offset, head_dim, scale, start_pos);
}
