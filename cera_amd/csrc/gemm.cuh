// Prefill GEMM: out[m][n] = W[m, k] . B[k, n] with W in native GGUF blocks and
// B the Q8_0-quantized activations of n tokens, on the int8 matrix cores.
//
// Arithmetic contract (cera's batched int8 path, cera/src/backend/simd.rs:
// 5693-5878 Q4_K, :5988-6195 Q6_K, :5893-5976 Q4_1, :4718-5010 Q4_0/Q8_0;
// cera/src/model/transformer.rs:710-788, 865-946): exact int32 dots of weight
// codes with int8 activations per 32-element block (16 for Q6_K), then an f32
// epilogue  sum_b xs[j][b] * (d*sc * dot - dmin*mn * sum a).
//
// Mapping to gfx950: one v_mfma_i32_32x32x32_i8 computes the 32x32 int32 dots
// of one 32-element block for 32 weight rows x 32 tokens (Q6_K uses the
// 32x32x16 form, one per 16-element scale run).  Because every block carries
// its own pair of f32 scales (weight side x activation side), the int32 tile
// is converted and folded into f32 accumulators after each MFMA; that VALU
// epilogue (cvt, mul, fma per output) is the throughput limit of this kernel,
// not the matrix core.
//
// Workgroup: 256 threads = 4 wavefronts as 2 (M) x 2 (N); block tile 128 rows x
// 64 tokens; each wavefront owns 64 x 32 (two MFMA row tiles).  K advances in
// steps of 256 elements.  Per step the workgroup stages into LDS
//   A: 128 rows x 256 weight codes unpacked to int8 (Q6_K/Q4_0 re-centred to
//      signed so no activation-sum correction is needed), row stride 272 B so
//      16-byte fragment reads do not collide on banks;
//   rs/rm: per-row scale (d*sc) and min (dmin*mn) per sub-block, stored
//      [sub][row] so a lane fetches its four consecutive rows with one b128;
//   B: 64 tokens x 256 int8 activations, cs/cm: activation scale and
//      scale*sum(a) per 32-block.
#pragma once
#include "common.cuh"

#define GEMM_BM 128
#define GEMM_BN 64
#define GEMM_KT 256
#define GEMM_LDA 272  // bytes per staged row (256 + 16 pad)

typedef int v16i __attribute__((ext_vector_type(16)));
typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v2i __attribute__((ext_vector_type(2)));

struct GemmArgs {
    const uint8_t* w;   // [m] rows of native blocks
    const int8_t* bq;   // [n][k] int8 activations
    const float* bs;    // [n][k/32] activation scales
    const float* bsum;  // [n][k/32] scale * sum(a) per block (exact product)
    float* out;
    uint32_t m, n, k;
    uint32_t row_bytes;
    uint64_t ld_m, ld_n;  // out[i*ld_m + j*ld_n]
    const float* resid;   // nullable: out = resid + W.B (same strides)
    float resid_scale;
};

// ---- per-type staging of one 256-element K step of one row ------------------
// Each type writes 256 int8 codes to `dst` (LDS row) and its per-sub-block row
// scales.  NSUB = MFMA steps per K tile, KSTEP = elements per MFMA.
struct GemmQ4K {
    static constexpr int NSUB = 8, KSTEP = 32;
    static constexpr bool HAS_MIN = true;
    static constexpr int BLOCK_BYTES = 144;
    // thread handles one 16-byte packed word `wi` (0..7) of the row's block
    __device__ static void unpack(const uint8_t* blk, uint32_t wi, int8_t* dst) {
        uint4 q = ld_u128(blk + 16 + wi * 16);
        uint32_t g = wi >> 1, h = wi & 1;
        uint4 lo, hi;
        lo.x = q.x & 0x0F0F0F0Fu; lo.y = q.y & 0x0F0F0F0Fu; lo.z = q.z & 0x0F0F0F0Fu; lo.w = q.w & 0x0F0F0F0Fu;
        hi.x = (q.x >> 4) & 0x0F0F0F0Fu; hi.y = (q.y >> 4) & 0x0F0F0F0Fu;
        hi.z = (q.z >> 4) & 0x0F0F0F0Fu; hi.w = (q.w >> 4) & 0x0F0F0F0Fu;
        *reinterpret_cast<uint4*>(dst + 64 * g + 16 * h) = lo;
        *reinterpret_cast<uint4*>(dst + 64 * g + 32 + 16 * h) = hi;
    }
    static constexpr int WORDS = 8;
    __device__ static void scales(const uint8_t* blk, float* rs, float* rm, uint32_t ld) {
        uint4 h = ld_u128(blk);
        float d = h2f(h.x & 0xFFFF), dmin = h2f(h.x >> 16);
        const uint32_t s[3] = {h.y, h.z, h.w};
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            uint32_t sc, mn;
            if (j < 4) {
                sc = (s[0] >> (8 * j)) & 63;
                mn = (s[1] >> (8 * j)) & 63;
            } else {
                uint32_t b8 = (s[2] >> (8 * (j - 4))) & 0xFF;
                sc = (b8 & 0xF) | ((((s[0] >> (8 * (j - 4))) & 0xFF) >> 6) << 4);
                mn = (b8 >> 4) | ((((s[1] >> (8 * (j - 4))) & 0xFF) >> 6) << 4);
            }
            rs[j * ld] = d * static_cast<float>(sc);
            rm[j * ld] = dmin * static_cast<float>(mn);
        }
    }
};

struct GemmQ6K {
    static constexpr int NSUB = 16, KSTEP = 16;
    static constexpr bool HAS_MIN = false;
    static constexpr int BLOCK_BYTES = 210;
    static constexpr int WORDS = 4;  // (nh, j): 16 positions l0..l0+15 -> 64 codes
    __device__ static void unpack(const uint8_t* blk, uint32_t wi, int8_t* dst) {
        uint32_t nh = wi >> 1, j = wi & 1;
        uint4 qa = ld_u128_a2(blk + nh * 64 + j * 16);
        uint4 qb = ld_u128_a2(blk + nh * 64 + 32 + j * 16);
        uint4 qh = ld_u128_a2(blk + 128 + nh * 32 + j * 16);
        const uint32_t a[4] = {qa.x, qa.y, qa.z, qa.w}, b[4] = {qb.x, qb.y, qb.z, qb.w}, h[4] = {qh.x, qh.y, qh.z, qh.w};
        uint32_t o[4][4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            uint32_t q0 = (a[i] & 0x0F0F0F0Fu) | ((h[i] << 4) & 0x30303030u);
            uint32_t q1 = (b[i] & 0x0F0F0F0Fu) | ((h[i] << 2) & 0x30303030u);
            uint32_t q2 = ((a[i] >> 4) & 0x0F0F0F0Fu) | (h[i] & 0x30303030u);
            uint32_t q3 = ((b[i] >> 4) & 0x0F0F0F0Fu) | ((h[i] >> 2) & 0x30303030u);
            // q - 32 per byte: codes are 0..63, so flipping bit 5 gives the 6-bit two's
            // complement; replicate it into bits 6 and 7 to sign-extend to int8
            uint32_t s;
            s = q0 ^ 0x20202020u; o[0][i] = s | ((s & 0x20202020u) << 1) | ((s & 0x20202020u) << 2);
            s = q1 ^ 0x20202020u; o[1][i] = s | ((s & 0x20202020u) << 1) | ((s & 0x20202020u) << 2);
            s = q2 ^ 0x20202020u; o[2][i] = s | ((s & 0x20202020u) << 1) | ((s & 0x20202020u) << 2);
            s = q3 ^ 0x20202020u; o[3][i] = s | ((s & 0x20202020u) << 1) | ((s & 0x20202020u) << 2);
        }
#pragma unroll
        for (int t = 0; t < 4; ++t)
            *reinterpret_cast<uint4*>(dst + nh * 128 + 32 * t + 16 * j) = make_uint4(o[t][0], o[t][1], o[t][2], o[t][3]);
    }
    __device__ static void scales(const uint8_t* blk, float* rs, float* rm, uint32_t ld) {
        float d = h2f(ld_u16(blk + 208));
        uint4 sc = ld_u128_a2(blk + 192);
        const uint32_t s[4] = {sc.x, sc.y, sc.z, sc.w};
#pragma unroll
        for (int h = 0; h < 16; ++h)
            rs[h * ld] = d * static_cast<float>(static_cast<int8_t>((s[h >> 2] >> (8 * (h & 3))) & 0xFF));
        (void)rm;
    }
};

// 32-element block formats: a K tile is 8 blocks; word wi = block index.
struct GemmQ4_0 {
    static constexpr int NSUB = 8, KSTEP = 32;
    static constexpr bool HAS_MIN = false;
    static constexpr int BLOCK_BYTES = 18 * 8;  // bytes per 256 elements
    static constexpr int WORDS = 8;
    __device__ static void unpack(const uint8_t* blk, uint32_t wi, int8_t* dst) {
        uint4 q = ld_u128_a2(blk + wi * 18 + 2);
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
        *reinterpret_cast<uint4*>(dst + 32 * wi) = lo;
        *reinterpret_cast<uint4*>(dst + 32 * wi + 16) = hi;
    }
    __device__ static void scales(const uint8_t* blk, float* rs, float* rm, uint32_t ld) {
#pragma unroll
        for (int b = 0; b < 8; ++b) rs[b * ld] = h2f(ld_u16(blk + 18 * b));
        (void)rm;
    }
};
struct GemmQ4_1 {
    static constexpr int NSUB = 8, KSTEP = 32;
    static constexpr bool HAS_MIN = true;   // rm holds -m so that out = rs*dot - rm*sum(a) covers q*d + m
    static constexpr int BLOCK_BYTES = 20 * 8;
    static constexpr int WORDS = 8;
    __device__ static void unpack(const uint8_t* blk, uint32_t wi, int8_t* dst) {
        uint4 q = ld_u128_a4(blk + wi * 20 + 4);
        uint4 lo, hi;
        lo.x = q.x & 0x0F0F0F0Fu; lo.y = q.y & 0x0F0F0F0Fu; lo.z = q.z & 0x0F0F0F0Fu; lo.w = q.w & 0x0F0F0F0Fu;
        hi.x = (q.x >> 4) & 0x0F0F0F0Fu; hi.y = (q.y >> 4) & 0x0F0F0F0Fu;
        hi.z = (q.z >> 4) & 0x0F0F0F0Fu; hi.w = (q.w >> 4) & 0x0F0F0F0Fu;
        *reinterpret_cast<uint4*>(dst + 32 * wi) = lo;
        *reinterpret_cast<uint4*>(dst + 32 * wi + 16) = hi;
    }
    __device__ static void scales(const uint8_t* blk, float* rs, float* rm, uint32_t ld) {
#pragma unroll
        for (int b = 0; b < 8; ++b) {
            uint32_t dm = *reinterpret_cast<const uint32_t*>(blk + 20 * b);
            rs[b * ld] = h2f(dm & 0xFFFF);
            rm[b * ld] = -h2f(dm >> 16);
        }
    }
};
struct GemmQ8_0 {
    static constexpr int NSUB = 8, KSTEP = 32;
    static constexpr bool HAS_MIN = false;
    static constexpr int BLOCK_BYTES = 34 * 8;
    static constexpr int WORDS = 8;
    __device__ static void unpack(const uint8_t* blk, uint32_t wi, int8_t* dst) {
        *reinterpret_cast<uint4*>(dst + 32 * wi) = ld_u128_a2(blk + wi * 34 + 2);
        *reinterpret_cast<uint4*>(dst + 32 * wi + 16) = ld_u128_a2(blk + wi * 34 + 18);
    }
    __device__ static void scales(const uint8_t* blk, float* rs, float* rm, uint32_t ld) {
#pragma unroll
        for (int b = 0; b < 8; ++b) rs[b * ld] = h2f(ld_u16(blk + 34 * b));
        (void)rm;
    }
};

template <class T>
static __global__ __launch_bounds__(256) void gemm_kernel(GemmArgs p) {
    __shared__ __attribute__((aligned(16))) int8_t sA[GEMM_BM * GEMM_LDA];
    __shared__ __attribute__((aligned(16))) int8_t sB[GEMM_BN * GEMM_LDA];
    __shared__ __attribute__((aligned(16))) float sRS[T::NSUB * GEMM_BM];
    // the min arrays exist only for formats with a per-block minimum (keeps the
    // workgroup under 64 KB of LDS)
    __shared__ __attribute__((aligned(16))) float sRM[T::HAS_MIN ? 8 * GEMM_BM : 4];
    __shared__ __attribute__((aligned(16))) float sCS[8 * GEMM_BN];
    __shared__ __attribute__((aligned(16))) float sCM[T::HAS_MIN ? 8 * GEMM_BN : 4];

    const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const uint32_t wm = wave >> 1, wn = wave & 1;           // wavefront position in the 2 x 2 grid
    const uint32_t m0 = blockIdx.y * GEMM_BM, n0 = blockIdx.x * GEMM_BN;
    const uint32_t col = lane & 31, half = lane >> 5;
    const uint32_t nb32 = p.k / 32;

    float acc[2][16], macc[2][16];
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int r = 0; r < 16; ++r) { acc[t][r] = 0.0f; macc[t][r] = 0.0f; }

    for (uint32_t k0 = 0; k0 < p.k; k0 += GEMM_KT) {
        // ---- stage A: 128 rows x WORDS words; B: 64 tokens x 16 words of 16 B
        for (uint32_t it = tid; it < GEMM_BM * T::WORDS; it += 256) {
            uint32_t r = it / T::WORDS, wi = it % T::WORDS;
            uint32_t row = min(m0 + r, p.m - 1);
            const uint8_t* blk = p.w + static_cast<uint64_t>(row) * p.row_bytes + static_cast<uint64_t>(k0 / 256) * T::BLOCK_BYTES;
            T::unpack(blk, wi, sA + r * GEMM_LDA);
        }
        if (tid < GEMM_BM) {
            uint32_t row = min(m0 + tid, p.m - 1);
            const uint8_t* blk = p.w + static_cast<uint64_t>(row) * p.row_bytes + static_cast<uint64_t>(k0 / 256) * T::BLOCK_BYTES;
            T::scales(blk, sRS + tid, sRM + tid, GEMM_BM);
        }
        for (uint32_t it = tid; it < GEMM_BN * 16; it += 256) {
            uint32_t c = it >> 4, wi = it & 15;
            uint32_t tok = n0 + c;
            uint4 v = make_uint4(0, 0, 0, 0);
            if (tok < p.n) v = *reinterpret_cast<const uint4*>(p.bq + static_cast<uint64_t>(tok) * p.k + k0 + wi * 16);
            *reinterpret_cast<uint4*>(sB + c * GEMM_LDA + wi * 16) = v;
        }
        for (uint32_t it = tid; it < GEMM_BN * 8; it += 256) {
            uint32_t c = it >> 3, b = it & 7;
            uint32_t tok = n0 + c;
            float s = 0.0f, sm = 0.0f;
            if (tok < p.n) {
                s = p.bs[static_cast<uint64_t>(tok) * nb32 + k0 / 32 + b];
                if (T::HAS_MIN) sm = p.bsum[static_cast<uint64_t>(tok) * nb32 + k0 / 32 + b];
            }
            sCS[b * GEMM_BN + c] = s;
            if (T::HAS_MIN) sCM[b * GEMM_BN + c] = sm;
        }
        __syncthreads();

        // ---- MFMA over the K tile
        const int8_t* bRow = sB + (wn * 32 + col) * GEMM_LDA;
#pragma unroll
        for (int sub = 0; sub < T::NSUB; ++sub) {
            const int b32 = sub * T::KSTEP / 32;  // 32-block index of this step
            const float xs = sCS[b32 * GEMM_BN + wn * 32 + col];
            const float xm = T::HAS_MIN ? sCM[b32 * GEMM_BN + wn * 32 + col] : 0.0f;
#pragma unroll
            for (int t = 0; t < 2; ++t) {
                const int8_t* aRow = sA + (wm * 64 + t * 32 + col) * GEMM_LDA;
                v16i c = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
                if (T::KSTEP == 32) {
                    v4i a = *reinterpret_cast<const v4i*>(aRow + sub * 32 + half * 16);
                    v4i b = *reinterpret_cast<const v4i*>(bRow + sub * 32 + half * 16);
                    c = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, c, 0, 0, 0);
                } else {
                    long a = *reinterpret_cast<const long*>(aRow + sub * 16 + half * 8);
                    long b = *reinterpret_cast<const long*>(bRow + sub * 16 + half * 8);
                    c = __builtin_amdgcn_mfma_i32_32x32x16_i8(a, b, c, 0, 0, 0);
                }
                // rows held by this lane: 8*blk + 4*half + r, blk = 0..3, r = 0..3
#pragma unroll
                for (int blk = 0; blk < 4; ++blk) {
                    const uint32_t rbase = wm * 64 + t * 32 + blk * 8 + half * 4;
                    const float4 rs = *reinterpret_cast<const float4*>(sRS + sub * GEMM_BM + rbase);
                    const float rsv[4] = {rs.x, rs.y, rs.z, rs.w};
#pragma unroll
                    for (int r = 0; r < 4; ++r)
                        acc[t][blk * 4 + r] = fmaf(static_cast<float>(c[blk * 4 + r]), rsv[r] * xs, acc[t][blk * 4 + r]);
                    if (T::HAS_MIN) {
                        const float4 rm = *reinterpret_cast<const float4*>(sRM + b32 * GEMM_BM + rbase);
                        const float rmv[4] = {rm.x, rm.y, rm.z, rm.w};
#pragma unroll
                        for (int r = 0; r < 4; ++r) macc[t][blk * 4 + r] = fmaf(rmv[r], xm, macc[t][blk * 4 + r]);
                    }
                }
            }
        }
        __syncthreads();
    }

    // ---- store: lane holds token n0 + wn*32 + col, 32 rows
    const uint32_t tok = n0 + wn * 32 + col;
    if (tok < p.n) {
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int blk = 0; blk < 4; ++blk)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    uint32_t row = m0 + wm * 64 + t * 32 + blk * 8 + half * 4 + r;
                    if (row < p.m) {
                        float v = acc[t][blk * 4 + r] - macc[t][blk * 4 + r];
                        uint64_t idx = row * p.ld_m + tok * p.ld_n;
                        if (p.resid) v = p.resid[idx] + (p.resid_scale != 1.0f ? v * p.resid_scale : v);
                        p.out[idx] = v;
                    }
                }
    }
}

