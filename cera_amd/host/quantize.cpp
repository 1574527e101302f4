// f32 -> GGUF block quantizers and f16 conversion for the host side of the
// `hip` backend.  These follow cera/src/convert/quantize.rs and
// cera/src/quant.rs so that synthetic models built here are byte-compatible
// with what cera's own converter would write.
#include "cera_host.h"

#include <cmath>
#include <cstring>
#include <thread>
#include <vector>

namespace {

inline float from_bits(uint32_t b) { float f; std::memcpy(&f, &b, 4); return f; }
inline uint32_t to_bits(float f) { uint32_t b; std::memcpy(&b, &f, 4); return b; }

// convert/quantize.rs:12-20 -- NaN maps to the lower bound.
inline float safe_clamp(float v, float lo, float hi) {
    if (std::isnan(v) || v < lo) return lo;
    if (v > hi) return hi;
    return v;
}
inline void put_u16(uint8_t* p, uint16_t v) { p[0] = uint8_t(v & 0xFF); p[1] = uint8_t(v >> 8); }

// convert/quantize.rs:344-388
void q8_0_block(const float* in, uint8_t* out) {
    float amax = 0.0f;
    for (int i = 0; i < 32; ++i) { float a = std::fabs(in[i]); if (a > amax) amax = a; }
    uint16_t dh = cera_f32_to_f16(amax / 127.0f);
    put_u16(out, dh);
    float d = cera_f16_to_f32(dh);
    float id = d != 0.0f ? 1.0f / d : 0.0f;
    for (int i = 0; i < 32; ++i)
        out[2 + i] = uint8_t(int8_t(safe_clamp(std::round(in[i] * id), -127.0f, 127.0f)));
}

// convert/quantize.rs:523-570 -- d = amax/8, q = floor(x/d + 8.5) in 0..15,
// element i in the low nibble of byte i, element i+16 in the high nibble.
void q4_0_block(const float* in, uint8_t* out) {
    float amax = 0.0f;
    for (int i = 0; i < 32; ++i) { float a = std::fabs(in[i]); if (a > amax) amax = a; }
    uint16_t dh = cera_f32_to_f16(amax / 8.0f);
    put_u16(out, dh);
    float d = cera_f16_to_f32(dh);
    float id = d != 0.0f ? 1.0f / d : 0.0f;
    for (int i = 0; i < 16; ++i) {
        uint8_t q0 = uint8_t(safe_clamp(std::floor(in[i] * id + 8.5f), 0.0f, 15.0f));
        uint8_t q1 = uint8_t(safe_clamp(std::floor(in[i + 16] * id + 8.5f), 0.0f, 15.0f));
        out[2 + i] = uint8_t((q0 & 0x0F) | ((q1 & 0x0F) << 4));
    }
}

// Shared front half of Q4_K / Q5_K (convert/quantize.rs:737-816, 869-947):
// per-32 min/max, super-scales d and dmin, 6-bit sub-scales, 12-byte packing.
struct KHeader { float d, dmin; uint8_t sc[8], mn[8]; };
KHeader k_header(const float* in, float qmax, uint8_t* out16) {
    float mins[8], maxs[8];
    for (int sb = 0; sb < 8; ++sb) {
        const float* s = in + 32 * sb;
        float lo = s[0], hi = s[0];
        for (int i = 1; i < 32; ++i) { if (s[i] < lo) lo = s[i]; if (s[i] > hi) hi = s[i]; }
        mins[sb] = lo; maxs[sb] = hi;
    }
    float max_range = 0.0f, max_min_abs = 0.0f;
    for (int sb = 0; sb < 8; ++sb) {
        float eff_min = std::fmin(mins[sb], 0.0f);
        float range = maxs[sb] - eff_min;
        if (range > max_range) max_range = range;
        if (-eff_min > max_min_abs) max_min_abs = -eff_min;
    }
    uint16_t dh = cera_f32_to_f16((max_range / 63.0f) / qmax);
    uint16_t mh = cera_f32_to_f16(max_min_abs / 63.0f);
    put_u16(out16, dh);
    put_u16(out16 + 2, mh);
    KHeader h;
    h.d = cera_f16_to_f32(dh);
    h.dmin = cera_f16_to_f32(mh);
    for (int sb = 0; sb < 8; ++sb) {
        float eff_min = std::fmin(mins[sb], 0.0f);
        float range = maxs[sb] - eff_min;
        h.sc[sb] = h.d > 0.0f ? uint8_t(safe_clamp(std::round((range / qmax) / h.d), 0.0f, 63.0f)) : 0;
        h.mn[sb] = h.dmin > 0.0f ? uint8_t(safe_clamp(std::round((-eff_min) / h.dmin), 0.0f, 63.0f)) : 0;
    }
    uint8_t* sb = out16 + 4;
    for (int j = 0; j < 4; ++j) {
        sb[j] = uint8_t((h.sc[j] & 0x3F) | (((h.sc[j + 4] & 0x30) >> 4) << 6));
        sb[j + 4] = uint8_t((h.mn[j] & 0x3F) | (((h.mn[j + 4] & 0x30) >> 4) << 6));
        sb[j + 8] = uint8_t((h.sc[j + 4] & 0x0F) | ((h.mn[j + 4] & 0x0F) << 4));
    }
    return h;
}

// convert/quantize.rs:719-846
void q4_k_block(const float* in, uint8_t* out) {
    KHeader h = k_header(in, 15.0f, out);
    for (int j = 0; j < 4; ++j) {
        float sc0 = float(h.sc[2 * j]) * h.d, sc1 = float(h.sc[2 * j + 1]) * h.d;
        float m0 = float(h.mn[2 * j]) * h.dmin, m1 = float(h.mn[2 * j + 1]) * h.dmin;
        const float* s0 = in + 64 * j;
        const float* s1 = s0 + 32;
        uint8_t* qs = out + 16 + 32 * j;
        for (int l = 0; l < 32; ++l) {
            uint8_t q0 = sc0 > 0.0f ? uint8_t(safe_clamp(std::round((s0[l] + m0) / sc0), 0.0f, 15.0f)) : 0;
            uint8_t q1 = sc1 > 0.0f ? uint8_t(safe_clamp(std::round((s1[l] + m1) / sc1), 0.0f, 15.0f)) : 0;
            qs[l] = uint8_t((q0 & 0x0F) | ((q1 & 0x0F) << 4));
        }
    }
}

// convert/quantize.rs:851-987 -- as Q4_K with 5-bit quants; bit 4 goes to qh.
void q5_k_block(const float* in, uint8_t* out) {
    KHeader h = k_header(in, 31.0f, out);
    uint8_t* qh = out + 16;
    uint8_t* qs = out + 48;
    std::memset(qh, 0, 32);
    for (int j = 0; j < 4; ++j) {
        float sc0 = float(h.sc[2 * j]) * h.d, sc1 = float(h.sc[2 * j + 1]) * h.d;
        float m0 = float(h.mn[2 * j]) * h.dmin, m1 = float(h.mn[2 * j + 1]) * h.dmin;
        const float* s0 = in + 64 * j;
        const float* s1 = s0 + 32;
        for (int l = 0; l < 32; ++l) {
            uint8_t q0 = sc0 > 0.0f ? uint8_t(safe_clamp(std::round((s0[l] + m0) / sc0), 0.0f, 31.0f)) : 0;
            uint8_t q1 = sc1 > 0.0f ? uint8_t(safe_clamp(std::round((s1[l] + m1) / sc1), 0.0f, 31.0f)) : 0;
            qs[32 * j + l] = uint8_t((q0 & 0x0F) | ((q1 & 0x0F) << 4));
            qh[l] = uint8_t(qh[l] | (((q0 >> 4) & 1) << (2 * j)) | (((q1 >> 4) & 1) << (2 * j + 1)));
        }
    }
}

// convert/quantize.rs:993-1094 -- d = max|x| / 4096, int8 per-16 scales,
// q = floor(x/(sc*d) + 32.5) in 0..63 split into ql nibbles and qh bit pairs.
void q6_k_block(const float* in, uint8_t* out) {
    float sub_max[16], max_all = 0.0f;
    for (int sb = 0; sb < 16; ++sb) {
        float amax = 0.0f;
        for (int i = 0; i < 16; ++i) { float a = std::fabs(in[16 * sb + i]); if (a > amax) amax = a; }
        sub_max[sb] = amax;
        if (amax > max_all) max_all = amax;
    }
    uint16_t dh = cera_f32_to_f16(max_all / (128.0f * 32.0f));
    put_u16(out + 208, dh);
    float d = cera_f16_to_f32(dh);
    float id = d != 0.0f ? 1.0f / d : 0.0f;
    int8_t qsc[16];
    for (int sb = 0; sb < 16; ++sb) {
        qsc[sb] = int8_t(safe_clamp(std::round(sub_max[sb] * id / 32.0f), -128.0f, 127.0f));
        out[192 + sb] = uint8_t(qsc[sb]);
    }
    std::memset(out, 0, 192);
    for (int pass = 0; pass < 2; ++pass) {
        const float* y = in + 128 * pass;
        uint8_t* ql = out + 64 * pass;
        uint8_t* qh = out + 128 + 32 * pass;
        const int8_t* sc = qsc + 8 * pass;
        for (int l = 0; l < 32; ++l) {
            int is = l / 16;
            uint8_t q[4];
            for (int t = 0; t < 4; ++t) {
                float s = float(sc[is + 2 * t]) * d;
                float isc = s != 0.0f ? 1.0f / s : 0.0f;
                q[t] = uint8_t(safe_clamp(std::floor(y[l + 32 * t] * isc + 32.5f), 0.0f, 63.0f));
            }
            ql[l] = uint8_t((q[0] & 0x0F) | ((q[2] & 0x0F) << 4));
            ql[l + 32] = uint8_t((q[1] & 0x0F) | ((q[3] & 0x0F) << 4));
            qh[l] = uint8_t(((q[0] >> 4) & 3) | (((q[1] >> 4) & 3) << 2) | (((q[2] >> 4) & 3) << 4) |
                            (((q[3] >> 4) & 3) << 6));
        }
    }
}

struct TypeInfo { uint32_t elems, bytes; void (*fn)(const float*, uint8_t*); };
bool type_info(uint32_t t, TypeInfo* ti) {
    switch (t) {
        case CERA_TYPE_Q8_0: *ti = {32, 34, q8_0_block}; return true;
        case CERA_TYPE_Q4_0: *ti = {32, 18, q4_0_block}; return true;
        case CERA_TYPE_Q4_K: *ti = {256, 144, q4_k_block}; return true;
        case CERA_TYPE_Q5_K: *ti = {256, 176, q5_k_block}; return true;
        case CERA_TYPE_Q6_K: *ti = {256, 210, q6_k_block}; return true;
        default: return false;
    }
}

}  // namespace

extern "C" {

// quant.rs:48-73
float cera_f16_to_f32(uint16_t bits) {
    uint32_t sign = (uint32_t(bits) & 0x8000u) << 16;
    uint32_t exp = (bits >> 10) & 0x1Fu, mant = bits & 0x3FFu, rest;
    if (exp == 0) {
        if (mant == 0) rest = 0;
        else {
            uint32_t shift = uint32_t(__builtin_clz(mant)) - 21;
            rest = ((113 - shift) << 23) | ((mant << (shift + 13)) & 0x007FFFFFu);
        }
    } else if (exp == 0x1F) {
        rest = mant ? (0x7FC00000u | (mant << 13)) : 0x7F800000u;
    } else {
        rest = ((exp + 112) << 23) | (mant << 13);
    }
    return from_bits(sign | rest);
}

// quant.rs:117-164 (round to nearest even)
uint16_t cera_f32_to_f16(float v) {
    uint32_t b = to_bits(v);
    uint16_t sign = uint16_t((b >> 16) & 0x8000u);
    int32_t exp = int32_t((b >> 23) & 0xFF);
    uint32_t mant = b & 0x007FFFFFu;
    if (exp == 0xFF) return mant ? uint16_t(sign | 0x7E00 | ((mant >> 13) & 0x3FF)) : uint16_t(sign | 0x7C00);
    int32_t e = exp - 112;
    if (e >= 0x1F) return sign | 0x7C00;
    if (e <= 0) {
        if (e < -10) return sign;
        uint32_t m = mant | 0x00800000u, shift = uint32_t(14 - e);
        uint32_t half = (m >> (shift - 1)) & 1u;
        uint32_t sticky = (m & ((1u << (shift - 1)) - 1)) != 0;
        uint32_t odd = (m >> shift) & 1u;
        return uint16_t(sign | uint16_t((m >> shift) + (half & (sticky | odd))));
    }
    uint32_t rounded = mant + 0x0FFFu + ((mant >> 13) & 1u);
    uint32_t ee = uint32_t(e) + (rounded >> 23);
    if (ee >= 0x1F) return sign | 0x7C00;
    return uint16_t(sign | (ee << 10) | ((rounded >> 13) & 0x3FF));
}

uint64_t cera_tensor_bytes(uint32_t t, uint64_t n) {
    switch (t) {
        case CERA_TYPE_F32: return n * 4;
        case CERA_TYPE_F16: case CERA_TYPE_BF16: return n * 2;
        case CERA_TYPE_Q4_1: return n % 32 ? 0 : n / 32 * 20;
        default: break;
    }
    TypeInfo ti;
    if (!type_info(t, &ti) || n % ti.elems) return 0;
    return n / ti.elems * ti.bytes;
}

int cera_quantize_mt(uint32_t t, const float* in, uint64_t n, void* out, uint64_t out_bytes, int n_threads) {
    TypeInfo ti;
    if (!type_info(t, &ti) || n % ti.elems) return -1;
    uint64_t nb = n / ti.elems;
    if (out_bytes < nb * ti.bytes) return -1;
    uint8_t* o = static_cast<uint8_t*>(out);
    auto work = [&](uint64_t b0, uint64_t b1) {
        for (uint64_t b = b0; b < b1; ++b) ti.fn(in + b * ti.elems, o + b * ti.bytes);
    };
    if (n_threads <= 1 || nb < 1024) { work(0, nb); return 0; }
    std::vector<std::thread> th;
    for (int i = 0; i < n_threads; ++i)
        th.emplace_back(work, nb * uint64_t(i) / uint64_t(n_threads), nb * uint64_t(i + 1) / uint64_t(n_threads));
    for (auto& x : th) x.join();
    return 0;
}

int cera_quantize(uint32_t t, const float* in, uint64_t n, void* out, uint64_t out_bytes) {
    return cera_quantize_mt(t, in, n, out, out_bytes, 1);
}

}  // extern "C"
