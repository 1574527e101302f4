// CPU oracle (test infrastructure only): block formats, f16 conversion and
// scalar dequantisation, restating cera/src/quant.rs.
#include "orc_common.h"

#include <cstring>

static inline float bits_f32(uint32_t b) { float f; std::memcpy(&f, &b, 4); return f; }
static inline uint32_t f32_bits(float f) { uint32_t b; std::memcpy(&b, &f, 4); return b; }

uint32_t orc_block_elems(uint32_t dtype) {
    switch (dtype) {
        case ORC_F32: case ORC_F16: case ORC_BF16: return 1;
        case ORC_Q4_0: case ORC_Q4_1: case ORC_Q8_0: return 32;
        case ORC_Q4_K: case ORC_Q5_K: case ORC_Q6_K: return 256;
        default: return 0;
    }
}
uint32_t orc_block_bytes(uint32_t dtype) {
    switch (dtype) {
        case ORC_F32: return 4;
        case ORC_F16: case ORC_BF16: return 2;
        case ORC_Q4_0: return 18;
        case ORC_Q4_1: return 20;
        case ORC_Q8_0: return 34;
        case ORC_Q4_K: return 144;
        case ORC_Q5_K: return 176;
        case ORC_Q6_K: return 210;
        default: return 0;
    }
}
uint64_t orc_row_bytes(uint32_t dtype, uint64_t k) {
    uint32_t e = orc_block_elems(dtype);
    if (e == 0 || k % e) return 0;
    return k / e * orc_block_bytes(dtype);
}

// quant.rs:48-73 -- integer-only widen; subnormals renormalised, sNaN quieted.
float orc_f16_to_f32(uint16_t bits) {
    uint32_t sign = (uint32_t(bits) & 0x8000u) << 16;
    uint32_t exp = (uint32_t(bits) >> 10) & 0x1Fu;
    uint32_t mant = uint32_t(bits) & 0x03FFu;
    uint32_t rest;
    if (exp == 0) {
        if (mant == 0) {
            rest = 0;
        } else {
            uint32_t shift = uint32_t(__builtin_clz(mant)) - 21;
            rest = ((113 - shift) << 23) | ((mant << (shift + 13)) & 0x007FFFFFu);
        }
    } else if (exp == 0x1F) {
        rest = mant == 0 ? 0x7F800000u : (0x7FC00000u | (mant << 13));
    } else {
        rest = ((exp + 112) << 23) | (mant << 13);
    }
    return bits_f32(sign | rest);
}

// quant.rs:91-100
float orc_bf16_to_f32(uint16_t bits) {
    uint32_t quiet = ((bits & 0x7FFF) > 0x7F80) ? 0x00400000u : 0u;
    return bits_f32((uint32_t(bits) << 16) | quiet);
}

// quant.rs:117-164 -- narrow, round to nearest even.
uint16_t orc_f32_to_f16(float v) {
    uint32_t b = f32_bits(v);
    uint16_t sign = uint16_t((b >> 16) & 0x8000u);
    int32_t exp = int32_t((b >> 23) & 0xFFu);
    uint32_t mant = b & 0x007FFFFFu;
    if (exp == 0xFF) {
        if (mant == 0) return sign | 0x7C00;
        return uint16_t(sign | 0x7E00 | (uint16_t(mant >> 13) & 0x03FF));
    }
    int32_t e = exp - 127 + 15;
    if (e >= 0x1F) return sign | 0x7C00;
    if (e <= 0) {
        if (e < -10) return sign;
        uint32_t m = mant | 0x00800000u;
        uint32_t shift = uint32_t(14 - e);
        uint32_t round = ((m >> (shift - 1)) & 1u) &
                         (uint32_t((m & ((1u << (shift - 1)) - 1)) != 0) | ((m >> shift) & 1u));
        return uint16_t(sign | uint16_t((m >> shift) + round));
    }
    uint32_t lsb = (mant >> 13) & 1u;
    uint32_t rounded = mant + 0x0FFFu + lsb;
    uint32_t carry = rounded >> 23;
    uint32_t ee = uint32_t(e) + carry;
    if (ee >= 0x1F) return sign | 0x7C00;
    return uint16_t(sign | uint16_t(ee << 10) | uint16_t((rounded >> 13) & 0x03FF));
}

// quant.rs:591-605 (get_scale_min_k4)
void orc_decode_q4km_scales(const uint8_t* s, uint8_t* sc, uint8_t* mn) {
    for (int j = 0; j < 4; ++j) {
        sc[j] = s[j] & 63;
        mn[j] = s[j + 4] & 63;
    }
    for (int j = 4; j < 8; ++j) {
        sc[j] = uint8_t((s[j + 4] & 0xF) | ((s[j - 4] >> 6) << 4));
        mn[j] = uint8_t((s[j + 4] >> 4) | ((s[j] >> 6) << 4));
    }
}

// quant.rs:364-376
static void dequant_q4_0(const OrcBlockQ4_0* b, float* out) {
    float d = orc_f16_to_f32(b->d);
    for (int i = 0; i < 16; ++i) {
        int lo = int(b->qs[i] & 0xF) - 8;
        int hi = int(b->qs[i] >> 4) - 8;
        out[i] = float(lo) * d;
        out[i + 16] = float(hi) * d;
    }
}
// quant.rs:423-437
static void dequant_q4_1(const OrcBlockQ4_1* b, float* out) {
    float d = orc_f16_to_f32(b->d), m = orc_f16_to_f32(b->m);
    for (int i = 0; i < 16; ++i) {
        int lo = int(b->qs[i] & 0xF);
        int hi = int(b->qs[i] >> 4);
        out[i] = float(lo) * d + m;
        out[i + 16] = float(hi) * d + m;
    }
}
// quant.rs:496-503
static void dequant_q8_0(const OrcBlockQ8_0* b, float* out) {
    float d = orc_f16_to_f32(b->d);
    for (int i = 0; i < 32; ++i) out[i] = float(b->qs[i]) * d;
}
// quant.rs:607-642
static void dequant_q4_k(const OrcBlockQ4K* b, float* out) {
    float d = orc_f16_to_f32(b->d), dmin = orc_f16_to_f32(b->dmin);
    uint8_t sc[8], mn[8];
    orc_decode_q4km_scales(b->scales, sc, mn);
    for (int j = 0; j < 4; ++j) {
        float d1 = d * float(sc[2 * j]), m1 = dmin * float(mn[2 * j]);
        float d2 = d * float(sc[2 * j + 1]), m2 = dmin * float(mn[2 * j + 1]);
        for (int l = 0; l < 32; ++l) {
            uint8_t q = b->qs[32 * j + l];
            out[64 * j + l] = d1 * float(q & 0xF) - m1;
            out[64 * j + l + 32] = d2 * float(q >> 4) - m2;
        }
    }
}
// quant.rs:796-832
static void dequant_q5_k(const OrcBlockQ5K* b, float* out) {
    float d = orc_f16_to_f32(b->d), dmin = orc_f16_to_f32(b->dmin);
    uint8_t sc[8], mn[8];
    orc_decode_q4km_scales(b->scales, sc, mn);
    uint8_t u1 = 1, u2 = 2;
    for (int j = 0; j < 4; ++j) {
        float d1 = d * float(sc[2 * j]), m1 = dmin * float(mn[2 * j]);
        float d2 = d * float(sc[2 * j + 1]), m2 = dmin * float(mn[2 * j + 1]);
        for (int l = 0; l < 32; ++l) {
            float hi = (b->qh[l] & u1) ? 16.0f : 0.0f;
            out[64 * j + l] = d1 * (float(b->qs[32 * j + l] & 0xF) + hi) - m1;
        }
        for (int l = 0; l < 32; ++l) {
            float hi = (b->qh[l] & u2) ? 16.0f : 0.0f;
            out[64 * j + l + 32] = d2 * (float(b->qs[32 * j + l] >> 4) + hi) - m2;
        }
        u1 = uint8_t(u1 << 2);
        u2 = uint8_t(u2 << 2);
    }
}
// quant.rs:703-737
static void dequant_q6_k(const OrcBlockQ6K* b, float* out) {
    float d = orc_f16_to_f32(b->d);
    for (int n = 0; n < 2; ++n) {
        const uint8_t* ql = b->ql + 64 * n;
        const uint8_t* qh = b->qh + 32 * n;
        const int8_t* sc = b->scales + 8 * n;
        float* y = out + 128 * n;
        for (int l = 0; l < 32; ++l) {
            int is = l / 16;
            int8_t q1 = int8_t(int((ql[l] & 0xF) | ((qh[l] & 3) << 4)) - 32);
            int8_t q2 = int8_t(int((ql[l + 32] & 0xF) | (((qh[l] >> 2) & 3) << 4)) - 32);
            int8_t q3 = int8_t(int((ql[l] >> 4) | (((qh[l] >> 4) & 3) << 4)) - 32);
            int8_t q4 = int8_t(int((ql[l + 32] >> 4) | (((qh[l] >> 6) & 3) << 4)) - 32);
            y[l] = d * float(sc[is]) * float(q1);
            y[l + 32] = d * float(sc[is + 2]) * float(q2);
            y[l + 64] = d * float(sc[is + 4]) * float(q3);
            y[l + 96] = d * float(sc[is + 6]) * float(q4);
        }
    }
}

// transformer.rs:949-1017 (embedding row lookup) / quant.rs *_row helpers.
int orc_dequantize_row(uint32_t dtype, const void* src, uint64_t k, float* dst) {
    uint32_t be = orc_block_elems(dtype);
    if (be == 0 || k % be) return -1;
    const uint8_t* p = static_cast<const uint8_t*>(src);
    uint64_t nb = k / be;
    switch (dtype) {
        case ORC_F32: std::memcpy(dst, src, k * 4); return 0;
        case ORC_F16:
            for (uint64_t i = 0; i < k; ++i) { uint16_t h; std::memcpy(&h, p + 2 * i, 2); dst[i] = orc_f16_to_f32(h); }
            return 0;
        case ORC_BF16:
            for (uint64_t i = 0; i < k; ++i) { uint16_t h; std::memcpy(&h, p + 2 * i, 2); dst[i] = orc_bf16_to_f32(h); }
            return 0;
        case ORC_Q4_0: for (uint64_t i = 0; i < nb; ++i) dequant_q4_0(reinterpret_cast<const OrcBlockQ4_0*>(p + 18 * i), dst + 32 * i); return 0;
        case ORC_Q4_1: for (uint64_t i = 0; i < nb; ++i) dequant_q4_1(reinterpret_cast<const OrcBlockQ4_1*>(p + 20 * i), dst + 32 * i); return 0;
        case ORC_Q8_0: for (uint64_t i = 0; i < nb; ++i) dequant_q8_0(reinterpret_cast<const OrcBlockQ8_0*>(p + 34 * i), dst + 32 * i); return 0;
        case ORC_Q4_K: for (uint64_t i = 0; i < nb; ++i) dequant_q4_k(reinterpret_cast<const OrcBlockQ4K*>(p + 144 * i), dst + 256 * i); return 0;
        case ORC_Q5_K: for (uint64_t i = 0; i < nb; ++i) dequant_q5_k(reinterpret_cast<const OrcBlockQ5K*>(p + 176 * i), dst + 256 * i); return 0;
        case ORC_Q6_K: for (uint64_t i = 0; i < nb; ++i) dequant_q6_k(reinterpret_cast<const OrcBlockQ6K*>(p + 210 * i), dst + 256 * i); return 0;
        default: return -1;
    }
}

// ---- f32 vec_dot (quant.rs) -- per block, then summed over the row in block
// order exactly as the scalar gemv fallbacks do (cpu.rs:1830-1854 for Q5_K).

// quant.rs:397-411
static float vdot_q4_0(const OrcBlockQ4_0* b, const float* y) {
    float d = orc_f16_to_f32(b->d), sum = 0.0f;
    for (int i = 0; i < 16; ++i) {
        int lo = int(b->qs[i] & 0xF) - 8, hi = int(b->qs[i] >> 4) - 8;
        sum += float(lo) * y[i];
        sum += float(hi) * y[i + 16];
    }
    return sum * d;
}
// quant.rs:464-481
static float vdot_q4_1(const OrcBlockQ4_1* b, const float* y) {
    float d = orc_f16_to_f32(b->d), m = orc_f16_to_f32(b->m), qsum = 0.0f, ysum = 0.0f;
    for (int i = 0; i < 16; ++i) {
        int lo = int(b->qs[i] & 0xF), hi = int(b->qs[i] >> 4);
        qsum += float(lo) * y[i];
        qsum += float(hi) * y[i + 16];
        ysum += y[i] + y[i + 16];
    }
    return qsum * d + m * ysum;
}
// quant.rs:566-577
static float vdot_q8_0(const OrcBlockQ8_0* b, const float* y) {
    float d = orc_f16_to_f32(b->d), sum = 0.0f;
    for (int i = 0; i < 32; ++i) sum += float(b->qs[i]) * y[i];
    return sum * d;
}
// quant.rs:658-697
static float vdot_q4_k(const OrcBlockQ4K* b, const float* y) {
    float d = orc_f16_to_f32(b->d), dmin = orc_f16_to_f32(b->dmin);
    uint8_t sc[8], mn[8];
    orc_decode_q4km_scales(b->scales, sc, mn);
    float sumf = 0.0f;
    for (int j = 0; j < 4; ++j) {
        float sc1 = float(sc[2 * j]), mn1 = float(mn[2 * j]);
        float sc2 = float(sc[2 * j + 1]), mn2 = float(mn[2 * j + 1]);
        float sum1 = 0, sum2 = 0, smn1 = 0, smn2 = 0;
        for (int l = 0; l < 32; ++l) {
            uint8_t q = b->qs[32 * j + l];
            sum1 += float(q & 0xF) * y[64 * j + l];
            sum2 += float(q >> 4) * y[64 * j + l + 32];
            smn1 += y[64 * j + l];
            smn2 += y[64 * j + l + 32];
        }
        sumf += d * (sc1 * sum1 + sc2 * sum2) - dmin * (mn1 * smn1 + mn2 * smn2);
    }
    return sumf;
}
// quant.rs:892-937
static float vdot_q5_k(const OrcBlockQ5K* b, const float* y) {
    float d = orc_f16_to_f32(b->d), dmin = orc_f16_to_f32(b->dmin);
    uint8_t sc[8], mn[8];
    orc_decode_q4km_scales(b->scales, sc, mn);
    float sumf = 0.0f;
    uint8_t u1 = 1, u2 = 2;
    for (int j = 0; j < 4; ++j) {
        float sc1 = float(sc[2 * j]), mn1 = float(mn[2 * j]);
        float sc2 = float(sc[2 * j + 1]), mn2 = float(mn[2 * j + 1]);
        float sum1 = 0, sum2 = 0, smn1 = 0, smn2 = 0;
        for (int l = 0; l < 32; ++l) {
            float hi1 = (b->qh[l] & u1) ? 16.0f : 0.0f;
            float hi2 = (b->qh[l] & u2) ? 16.0f : 0.0f;
            float q1 = float(b->qs[32 * j + l] & 0xF) + hi1;
            float q2 = float(b->qs[32 * j + l] >> 4) + hi2;
            sum1 += q1 * y[64 * j + l];
            sum2 += q2 * y[64 * j + l + 32];
            smn1 += y[64 * j + l];
            smn2 += y[64 * j + l + 32];
        }
        sumf += d * (sc1 * sum1 + sc2 * sum2) - dmin * (mn1 * smn1 + mn2 * smn2);
        u1 = uint8_t(u1 << 2);
        u2 = uint8_t(u2 << 2);
    }
    return sumf;
}
// quant.rs:753-788
static float vdot_q6_k(const OrcBlockQ6K* b, const float* y) {
    float d = orc_f16_to_f32(b->d), sumf = 0.0f;
    for (int n = 0; n < 2; ++n) {
        const uint8_t* ql = b->ql + 64 * n;
        const uint8_t* qh = b->qh + 32 * n;
        const int8_t* sc = b->scales + 8 * n;
        const float* yy = y + 128 * n;
        for (int l = 0; l < 32; ++l) {
            int is = l / 16;
            int8_t q1 = int8_t(int((ql[l] & 0xF) | ((qh[l] & 3) << 4)) - 32);
            int8_t q2 = int8_t(int((ql[l + 32] & 0xF) | (((qh[l] >> 2) & 3) << 4)) - 32);
            int8_t q3 = int8_t(int((ql[l] >> 4) | (((qh[l] >> 4) & 3) << 4)) - 32);
            int8_t q4 = int8_t(int((ql[l + 32] >> 4) | (((qh[l] >> 6) & 3) << 4)) - 32);
            sumf += float(sc[is]) * float(q1) * yy[l];
            sumf += float(sc[is + 2]) * float(q2) * yy[l + 32];
            sumf += float(sc[is + 4]) * float(q3) * yy[l + 64];
            sumf += float(sc[is + 6]) * float(q4) * yy[l + 96];
        }
    }
    return sumf * d;
}

float orc_vec_dot_row_f32(uint32_t dtype, const void* row, const float* x, uint64_t k) {
    const uint8_t* p = static_cast<const uint8_t*>(row);
    float sum = 0.0f;
    switch (dtype) {
        case ORC_Q4_0: for (uint64_t b = 0; b < k / 32; ++b) sum += vdot_q4_0(reinterpret_cast<const OrcBlockQ4_0*>(p + 18 * b), x + 32 * b); break;
        case ORC_Q4_1: for (uint64_t b = 0; b < k / 32; ++b) sum += vdot_q4_1(reinterpret_cast<const OrcBlockQ4_1*>(p + 20 * b), x + 32 * b); break;
        case ORC_Q8_0: for (uint64_t b = 0; b < k / 32; ++b) sum += vdot_q8_0(reinterpret_cast<const OrcBlockQ8_0*>(p + 34 * b), x + 32 * b); break;
        case ORC_Q4_K: for (uint64_t b = 0; b < k / 256; ++b) sum += vdot_q4_k(reinterpret_cast<const OrcBlockQ4K*>(p + 144 * b), x + 256 * b); break;
        case ORC_Q5_K: for (uint64_t b = 0; b < k / 256; ++b) sum += vdot_q5_k(reinterpret_cast<const OrcBlockQ5K*>(p + 176 * b), x + 256 * b); break;
        case ORC_Q6_K: for (uint64_t b = 0; b < k / 256; ++b) sum += vdot_q6_k(reinterpret_cast<const OrcBlockQ6K*>(p + 210 * b), x + 256 * b); break;
        default: return 0.0f;
    }
    return sum;
}
