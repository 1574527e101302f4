// Reference-order verification route.
//
// The fast kernels sum the f32 partial products of a row in an order chosen for the GPU, so
// their outputs differ from cera's CPU AVX2 path in the last bits -- and every projection
// re-quantizes its input, which amplifies last-bit differences into whole int8 steps.  The
// kernels in this file instead perform exactly the f32 operations of the CPU path, in its
// order, so a whole forward pass is bit-identical to it and greedy decoding yields the same
// token stream.  They are slow (one 8-lane group plays the eight lanes of a ymm register, the
// serial f64 sums are serial here too), opt-in per model (cera_hip_set_reference_order) and
// never timed; the fast route is what ships, this one is what it is checked against.
//
//   GEMV   gemm_q4_k_q8_0 / gemm_q6_k_q8_0 at n == 1 (cera/src/backend/simd.rs:5742-5795,
//          6025-6093): dot32u per 32-block gives eight i32 lanes (lane j = elements 4j..4j+3,
//          i.e. exactly one v_dot4_i32_i8), converted and FMA'd into four round-robin
//          accumulators, scalar min-term chain, tree add, hsum256_ps (:4546-4554);
//          row_dot_q4_0 / row_dot_q8_0 (:4593-4637) and gemm_q4_1_q8_0 (:5893-5976) with one
//          accumulator.
//   norm   cpu::rmsnorm (cera/src/backend/cpu.rs:2479-2496) with the serial f64 sum.
//   attn   cpu::attn_scores / softmax_inplace / attn_values, AVX2 tier
//          (cera/src/backend/cpu.rs:3503-3589, 2617-2633): two 8-lane FMA chains per key,
//          f64 softmax sum in key order, one FMA chain per output column in key order.
#include <cmath>

#include "glue.hip.h"
#include "host_common.h"
#include "model.h"

namespace {

// ---- 8-lane groups: lane j of a group is lane j of the CPU's ymm register -------------
__device__ __forceinline__ float grp_hsum(float v) {
    // hsum256_ps: (v0+v4 + v2+v6) + (v1+v5 + v3+v7); f32 addition is commutative, so every lane
    // of the group ends up with the same bits
    v = __fadd_rn(v, __shfl_xor(v, 4, 64));
    v = __fadd_rn(v, __shfl_xor(v, 2, 64));
    v = __fadd_rn(v, __shfl_xor(v, 1, 64));
    return v;
}
__device__ __forceinline__ int grp_isum(int v) {
    v += __shfl_xor(v, 4, 64);
    v += __shfl_xor(v, 2, 64);
    v += __shfl_xor(v, 1, 64);
    return v;
}

struct RefGemvArgs {
    const uint8_t* w;
    const int8_t* xq;
    const float* xs;
    float* y;
    uint32_t m, k, row_bytes;
};

// One row, one lane of its group.  Every lane carries the scalar chains (macc) redundantly.
// NACC = 4: the n == 1 (decode) branch with its four round-robin accumulators; NACC = 1: the
// KQ_COLS-tiled branch every column of a batch (n > 1) takes (cera/src/backend/simd.rs:5796-5851,
// 6094-6168), one accumulator.
template <int NACC = 4>
__device__ __forceinline__ float ref_row_q4_k(const uint8_t* row, const int8_t* xq, const float* xs, uint32_t k, uint32_t j) {
    float facc[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    float macc = 0.0f;
    int slot = 0;
    for (uint32_t bi = 0; bi < k / 256; ++bi) {
        const uint8_t* blk = row + 144 * bi;
        const float d = h2f(ld_u16(blk)), dmin = h2f(ld_u16(blk + 2));
        const uint8_t* s12 = blk + 4;
#pragma unroll
        for (int s = 0; s < 8; ++s) {
            uint32_t sc, mn;   // get_scale_min_k4 (cera/src/quant.rs:591-605)
            if (s < 4) {
                sc = s12[s] & 63;
                mn = s12[s + 4] & 63;
            } else {
                sc = (s12[s + 4] & 0xF) | ((s12[s - 4] >> 6) << 4);
                mn = (s12[s + 4] >> 4) | ((s12[s] >> 6) << 4);
            }
            const uint32_t xb = bi * 8 + s;
            const uint32_t wq = *reinterpret_cast<const uint32_t*>(blk + 16 + 32 * (s >> 1) + 4 * j);
            const uint32_t w4 = (s & 1) ? ((wq >> 4) & 0x0F0F0F0Fu) : (wq & 0x0F0F0F0Fu);
            const uint32_t a4 = *reinterpret_cast<const uint32_t*>(xq + 32 * xb + 4 * j);
            const float lanes = static_cast<float>(dot4(w4, a4, 0));
            const int sx = grp_isum(sum4(a4, 0));
            const float x = xs[xb];
            const float dsc = __fmul_rn(d, static_cast<float>(sc));
            const float dmn = __fmul_rn(dmin, static_cast<float>(mn));
            facc[slot] = fmaf(lanes, __fmul_rn(x, dsc), facc[slot]);
            macc = __fadd_rn(macc, __fmul_rn(__fmul_rn(x, dmn), static_cast<float>(sx)));
            slot = (slot + 1) & (NACC - 1);
        }
    }
    const float f = NACC == 4 ? __fadd_rn(__fadd_rn(facc[0], facc[1]), __fadd_rn(facc[2], facc[3])) : facc[0];
    return __fsub_rn(grp_hsum(f), macc);
}

template <int NACC = 4>
__device__ __forceinline__ float ref_row_q6_k(const uint8_t* row, const int8_t* xq, const float* xs, uint32_t k, uint32_t j) {
    float facc[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    float macc = 0.0f;
    int slot = 0;
    for (uint32_t bi = 0; bi < k / 256; ++bi) {
        const uint8_t* blk = row + 210 * bi;
        const float d = h2f(ld_u16(blk + 208));
        const float d32 = __fmul_rn(d, 32.0f);
        for (int nh = 0; nh < 2; ++nh) {
            const uint32_t qh = ld_u32_a2(blk + 128 + 32 * nh + 4 * j);
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const uint32_t ql = ld_u32_a2(blk + 64 * nh + (g & 1) * 32 + 4 * j);
                const uint32_t l4 = g < 2 ? (ql & 0x0F0F0F0Fu) : ((ql >> 4) & 0x0F0F0F0Fu);
                const uint32_t h2 = (qh >> (2 * g)) & 0x03030303u;
                const uint32_t w4 = l4 | (h2 << 4);
                const float sc0 = static_cast<float>(static_cast<int8_t>(blk[192 + nh * 8 + 2 * g]));
                const float sc1 = static_cast<float>(static_cast<int8_t>(blk[192 + nh * 8 + 2 * g + 1]));
                const uint32_t xb = bi * 8 + nh * 4 + g;
                const uint32_t a4 = *reinterpret_cast<const uint32_t*>(xq + 32 * xb + 4 * j);
                const float lanes = static_cast<float>(dot4(w4, a4, 0));
                const float x = xs[xb];
                // lanes 0..3 hold the first 16 elements (scale sc0), lanes 4..7 the second 16
                const float scale = __fmul_rn(__fmul_rn(j < 4 ? sc0 : sc1, d), x);
                facc[slot] = fmaf(lanes, scale, facc[slot]);
                int s16 = sum4(a4, 0);
                s16 += __shfl_xor(s16, 1, 64);
                s16 += __shfl_xor(s16, 2, 64);
                const int other = __shfl_xor(s16, 4, 64);
                const float sx0 = static_cast<float>(j < 4 ? s16 : other), sx1 = static_cast<float>(j < 4 ? other : s16);
                const float mins = __fadd_rn(__fmul_rn(sc0, sx0), __fmul_rn(sc1, sx1));
                macc = __fadd_rn(macc, __fmul_rn(__fmul_rn(x, d32), mins));
                slot = (slot + 1) & (NACC - 1);
            }
        }
    }
    const float f = NACC == 4 ? __fadd_rn(__fadd_rn(facc[0], facc[1]), __fadd_rn(facc[2], facc[3])) : facc[0];
    return __fsub_rn(grp_hsum(f), macc);
}

// 32-element block formats: one accumulator.  TYPE: 2 Q4_0, 3 Q4_1, 8 Q8_0.
template <int TYPE>
__device__ __forceinline__ float ref_row_b32(const uint8_t* row, const int8_t* xq, const float* xs, uint32_t k, uint32_t j) {
    float acc = 0.0f, macc = 0.0f;
    for (uint32_t b = 0; b < k / 32; ++b) {
        const uint32_t a4 = *reinterpret_cast<const uint32_t*>(xq + 32 * b + 4 * j);
        const float x = xs[b];
        if (TYPE == 8) {
            const uint8_t* blk = row + 34 * b;
            const float lanes = static_cast<float>(dot4(ld_u32_a2(blk + 2 + 4 * j), a4, 0));
            acc = fmaf(lanes, __fmul_rn(h2f(ld_u16(blk)), x), acc);
        } else {
            const uint8_t* blk = row + (TYPE == 2 ? 18 : 20) * b;
            // element i = low nibble of byte i, element i + 16 = high nibble: lanes 4..7 take the high nibbles
            const uint32_t wq = ld_u32_a2(blk + (TYPE == 2 ? 2 : 4) + 4 * (j & 3));
            const uint32_t w4 = j < 4 ? (wq & 0x0F0F0F0Fu) : ((wq >> 4) & 0x0F0F0F0Fu);
            if (TYPE == 2) {
                const float lanes = static_cast<float>(dot4(w4, a4, -8 * sum4(a4, 0)));   // sum (q - 8) a, exact
                acc = fmaf(lanes, __fmul_rn(h2f(ld_u16(blk)), x), acc);
            } else {
                const float d = h2f(ld_u16(blk)), mmin = h2f(ld_u16(blk + 2));
                const int sx = grp_isum(sum4(a4, 0));
                acc = fmaf(static_cast<float>(dot4(w4, a4, 0)), __fmul_rn(x, d), acc);
                macc = __fadd_rn(macc, __fmul_rn(__fmul_rn(x, mmin), static_cast<float>(sx)));
            }
        }
    }
    return TYPE == 3 ? __fadd_rn(grp_hsum(acc), macc) : grp_hsum(acc);
}

template <int TYPE>
__global__ __launch_bounds__(256) void gemv_ref_kernel(RefGemvArgs p) {
    const uint32_t row = blockIdx.x * 32 + (threadIdx.x >> 3), j = threadIdx.x & 7;
    // rows past the end recompute the last row (the group's lanes must stay together for the
    // cross-lane sums) and drop the result
    const uint8_t* rp = p.w + static_cast<uint64_t>(min(row, p.m - 1)) * p.row_bytes;
    float v;
    if (TYPE == 12) v = ref_row_q4_k(rp, p.xq, p.xs, p.k, j);
    else if (TYPE == 14) v = ref_row_q6_k(rp, p.xq, p.xs, p.k, j);
    else v = ref_row_b32<TYPE>(rp, p.xq, p.xs, p.k, j);
    if (j == 0 && row < p.m) p.y[row] = v;
}

// ---- Q5_K: f32 activations, scalar chains ----------------------------------------------------
// gemv_q5km_f32 -> vec_dot_q5_k_f32_scalar (cera/src/backend/cpu.rs:1830-1854,
// cera/src/quant.rs:892-937): the reference never quantizes the input of a Q5_K matrix; each
// 256-weight block runs, per 64-weight pair j, four sequential 32-step chains with separate
// multiply and add -- sum1 += q1*y, sum2 += q2*y', smn1 += y, smn2 += y' -- then
// sumf += d*(sc1*sum1 + sc2*sum2) - dmin*(mn1*smn1 + mn2*smn2), and the row adds the block
// results in order.  One wavefront per row: its 64 lanes are the 4 x 4 x 4 chains of four
// consecutive blocks; the combination steps then run in the reference's order on one lane.
struct RefGemvF32Args {
    const uint8_t* w;
    const float* x;
    float* y;
    uint32_t m, k, row_bytes;
};
__global__ __launch_bounds__(256) void gemv_q5k_ref_kernel(RefGemvF32Args p) {
    const uint32_t lane = threadIdx.x & 63;
    const uint32_t row = blockIdx.x * 4 + (threadIdx.x >> 6);
    // a wavefront past the last row recomputes it and drops the result (lanes stay together for the shuffles)
    const uint8_t* rp = p.w + static_cast<uint64_t>(min(row, p.m - 1)) * p.row_bytes;
    const uint32_t nb = p.k / 256;
    const uint32_t bsel = lane >> 4, j = (lane >> 2) & 3, which = lane & 3;
    float sum = 0.0f;
    for (uint32_t b0 = 0; b0 < nb; b0 += 4) {
        const uint32_t b = min(b0 + bsel, nb - 1);
        const uint8_t* blk = rp + 176 * b;   // d, dmin, scales[12], qh[32], qs[128]
        const uint8_t* qh = blk + 16;
        const uint8_t* qs = blk + 48 + 32 * j;
        const float* y = p.x + 256 * b + 64 * j + ((which & 1) ? 32 : 0);
        const uint32_t bit = 1u << (2 * j + (which & 1));
        float acc = 0.0f;
        if (which < 2) {
            for (int l = 0; l < 32; ++l) {
                const uint32_t nib = (which & 1) ? (qs[l] >> 4) : (qs[l] & 0xF);
                const float q = __fadd_rn(static_cast<float>(nib), (qh[l] & bit) ? 16.0f : 0.0f);
                acc = __fadd_rn(acc, __fmul_rn(q, y[l]));
            }
        } else {
            for (int l = 0; l < 32; ++l) acc = __fadd_rn(acc, y[l]);
        }
        // lanes 4q .. 4q+3 hold sum1, sum2, smn1, smn2 of one (block, j)
        const uint32_t base = lane & ~3u;
        const float sum1 = __shfl(acc, base), sum2 = __shfl(acc, base + 1), smn1 = __shfl(acc, base + 2), smn2 = __shfl(acc, base + 3);
        const float d = h2f(ld_u16(blk)), dmin = h2f(ld_u16(blk + 2));
        const uint8_t* s12 = blk + 4;
        uint32_t sc[2], mn[2];
#pragma unroll
        for (int e = 0; e < 2; ++e) {
            const uint32_t s = 2 * j + e;
            if (s < 4) {
                sc[e] = s12[s] & 63;
                mn[e] = s12[s + 4] & 63;
            } else {
                sc[e] = (s12[s + 4] & 0xF) | ((s12[s - 4] >> 6) << 4);
                mn[e] = (s12[s + 4] >> 4) | ((s12[s] >> 6) << 4);
            }
        }
        const float pos = __fmul_rn(d, __fadd_rn(__fmul_rn(static_cast<float>(sc[0]), sum1), __fmul_rn(static_cast<float>(sc[1]), sum2)));
        const float neg = __fmul_rn(dmin, __fadd_rn(__fmul_rn(static_cast<float>(mn[0]), smn1), __fmul_rn(static_cast<float>(mn[1]), smn2)));
        const float term = __fsub_rn(pos, neg);
        // block result: sumf = 0; sumf += term_j for j = 0..3 (lanes 16*bsel + 4*j hold term_j)
        const uint32_t bl = lane & ~15u;
        float sumf = 0.0f;
#pragma unroll
        for (int jj = 0; jj < 4; ++jj) sumf = __fadd_rn(sumf, __shfl(term, bl + 4 * jj));
        // row: sum += block result, blocks in order (lanes 0, 16, 32, 48 hold them)
#pragma unroll
        for (int bb = 0; bb < 4; ++bb) {
            const float v = __shfl(sumf, 16 * bb);
            if (b0 + bb < nb) sum = __fadd_rn(sum, v);
        }
    }
    if (lane == 0 && row < p.m) p.y[row] = sum;
}

// ---- batched prefill in the order of cera's x86 host ---------------------------------------
// transformer::gemm_preq (cera/src/model/transformer.rs:710-788) sends a Q4_K / Q4_0 weight
// that was repacked at load (m % 8 == 0; cpu.rs:1204-1206, 1364-1366) to the 8-row-interleaved
// kernels gemm_q4_k_8x8_q8_0 / gemm_q4_0_8x8_q8_0 (cera/src/backend/simd.rs:5392-5518, 5215-5366).
// There the eight lanes of a vector are eight output ROWS of one column, so every output
// element has an f32 chain of its own: per 32-block one FMA with the exact integer block dot
// (Q4_K: and one FNMADD with the exact activation sum).  Integer sums are order-free, so the
// eight lanes of a group only share the integer work; the float chain is the same in each.
__device__ __forceinline__ float ref_elem_q4_k_8x8(const uint8_t* row, const int8_t* xq, const float* xs, uint32_t k, uint32_t j) {
    float facc = 0.0f;
    for (uint32_t bi = 0; bi < k / 256; ++bi) {
        const uint8_t* blk = row + 144 * bi;
        const float d = h2f(ld_u16(blk)), dmin = h2f(ld_u16(blk + 2));
        const uint8_t* s12 = blk + 4;
#pragma unroll
        for (int s = 0; s < 8; ++s) {
            uint32_t sc, mn;
            if (s < 4) {
                sc = s12[s] & 63;
                mn = s12[s + 4] & 63;
            } else {
                sc = (s12[s + 4] & 0xF) | ((s12[s - 4] >> 6) << 4);
                mn = (s12[s + 4] >> 4) | ((s12[s] >> 6) << 4);
            }
            const uint32_t xb = bi * 8 + s;
            const uint32_t wq = *reinterpret_cast<const uint32_t*>(blk + 16 + 32 * (s >> 1) + 4 * j);
            const uint32_t w4 = (s & 1) ? ((wq >> 4) & 0x0F0F0F0Fu) : (wq & 0x0F0F0F0Fu);
            const uint32_t a4 = *reinterpret_cast<const uint32_t*>(xq + 32 * xb + 4 * j);
            const int acc = grp_isum(dot4(w4, a4, 0));
            const int sx = grp_isum(sum4(a4, 0));
            const float x = xs[xb];
            const float dsc = __fmul_rn(d, static_cast<float>(sc));     // baked at repack time (cpu.rs:1282-1358)
            const float dmn = __fmul_rn(dmin, static_cast<float>(mn));
            facc = fmaf(static_cast<float>(acc), __fmul_rn(dsc, x), facc);
            facc = fmaf(-dmn, __fmul_rn(x, static_cast<float>(sx)), facc);   // _mm256_fnmadd_ps
        }
    }
    return facc;
}
__device__ __forceinline__ float ref_elem_q4_0_8x8(const uint8_t* row, const int8_t* xq, const float* xs, uint32_t k, uint32_t j) {
    float facc = 0.0f;
    for (uint32_t b = 0; b < k / 32; ++b) {
        const uint8_t* blk = row + 18 * b;
        const uint32_t wq = ld_u32_a2(blk + 2 + 4 * (j & 3));
        const uint32_t w4 = j < 4 ? (wq & 0x0F0F0F0Fu) : ((wq >> 4) & 0x0F0F0F0Fu);   // raw codes 0..15
        const uint32_t a4 = *reinterpret_cast<const uint32_t*>(xq + 32 * b + 4 * j);
        const int acc = grp_isum(dot4(w4, a4, 0));
        const int cs = grp_isum(sum4(a4, 0));
        const float eff = __fsub_rn(static_cast<float>(acc), __fmul_rn(8.0f, static_cast<float>(cs)));
        facc = fmaf(eff, __fmul_rn(h2f(ld_u16(blk)), xs[b]), facc);
    }
    return facc;
}

struct RefGemmArgs {
    const uint8_t* w;
    const int8_t* xq;   // [n][k]
    const float* xs;    // [n][k/32]
    float* out;         // out[j * ld_n + i * ld_m]
    uint32_t m, n, k, row_bytes;
    uint64_t ld_m, ld_n;
};
// One 8-lane group per (row, token): grid = (ceil(m / 32), n).  REPACK: the 8x8 kernels' order.
template <int TYPE, bool REPACK>
__global__ __launch_bounds__(256) void gemm_ref_kernel(RefGemmArgs p) {
    const uint32_t row = blockIdx.x * 32 + (threadIdx.x >> 3), j = threadIdx.x & 7, tok = blockIdx.y;
    const uint8_t* rp = p.w + static_cast<uint64_t>(min(row, p.m - 1)) * p.row_bytes;
    const int8_t* xq = p.xq + static_cast<uint64_t>(tok) * p.k;
    const float* xs = p.xs + static_cast<uint64_t>(tok) * (p.k / 32);
    float v;
    if (TYPE == 12) v = REPACK ? ref_elem_q4_k_8x8(rp, xq, xs, p.k, j) : ref_row_q4_k<1>(rp, xq, xs, p.k, j);
    else if (TYPE == 14) v = ref_row_q6_k<1>(rp, xq, xs, p.k, j);
    else if (TYPE == 2 && REPACK) v = ref_elem_q4_0_8x8(rp, xq, xs, p.k, j);
    else v = ref_row_b32<TYPE>(rp, xq, xs, p.k, j);
    if (j == 0 && row < p.m) p.out[tok * p.ld_n + row * p.ld_m] = v;
}

// flash_attention_gqa_avx2 (cera/src/backend/cpu.rs:4261-4412), one wavefront per (query, head):
// keys in tiles of 32; a score is two 8-lane FMA chains over the even / odd 8-wide slices of the
// head, added, folded with hsum256 (cpu.rs:3489) and scaled; the online softmax is the scalar
// bookkeeping of the CPU kernel (tile maximum with `>`, ggml expf, f64 tile sum in key order,
// running sum in f64); every output column is one FMA chain over the keys in order.
// q: [n][n_heads * hd] rotated queries; out the same shape.  Caches head-major.
template <typename KV>
__global__ __launch_bounds__(64) void flash_ref_kernel(const float* __restrict__ q, const KV* __restrict__ kc,
                                                       const KV* __restrict__ vc, uint32_t n_heads, uint32_t group, uint32_t hd,
                                                       uint32_t max_seq, uint32_t start_pos, float scale, float* __restrict__ out) {
    __shared__ float sc_sh[32];
    const uint32_t jq = blockIdx.x, h = blockIdx.y, kvh = h / group, lane = threadIdx.x;
    const uint32_t grp = lane >> 3, j = lane & 7, nq = hd / 8;
    const float* qh = q + (static_cast<uint64_t>(jq) * n_heads + h) * hd;
    const KV* kbase = kc + static_cast<uint64_t>(kvh) * max_seq * hd;
    const KV* vbase = vc + static_cast<uint64_t>(kvh) * max_seq * hd;
    const uint32_t max_kv = start_pos + jq + 1;
    float acc[4] = {0.0f, 0.0f, 0.0f, 0.0f};   // columns lane + 64 c, hd <= 256
    float running_max = -__builtin_inff();
    double running_sum = 0.0;
    for (uint32_t kv_start = 0; kv_start < max_kv; kv_start += 32) {
        const uint32_t tile_len = min(32u, max_kv - kv_start);
        // scores: group grp takes keys grp, grp + 8, grp + 16, grp + 24 of the tile
        for (uint32_t r = 0; r < 4; ++r) {
            const uint32_t ti = grp + 8 * r;
            const KV* kp = kbase + static_cast<uint64_t>(kv_start + min(ti, tile_len - 1)) * hd;
            float s0 = 0.0f, s1 = 0.0f;
            uint32_t i = 0;
            for (; i + 2 <= nq; i += 2) {
                s0 = fmaf(qh[8 * i + j], KvOps<KV>::ld1(kp + 8 * i + j), s0);
                s1 = fmaf(qh[8 * (i + 1) + j], KvOps<KV>::ld1(kp + 8 * (i + 1) + j), s1);
            }
            if (i < nq) s0 = fmaf(qh[8 * i + j], KvOps<KV>::ld1(kp + 8 * i + j), s0);
            const float v = grp_hsum(__fadd_rn(s0, s1));
            if (j == 0 && ti < tile_len) sc_sh[ti] = __fmul_rn(v, scale);
        }
        __syncthreads();
        float tile_max = -__builtin_inff();
        for (uint32_t ti = 0; ti < tile_len; ++ti)
            if (sc_sh[ti] > tile_max) tile_max = sc_sh[ti];
        const float new_max = fmaxf(running_max, tile_max);   // f32::max
        const float rescale = running_max > -__builtin_inff() ? cera_expf(__fsub_rn(running_max, new_max)) : 0.0f;
        // every lane keeps the whole bookkeeping (identical values in all lanes); lane ti < 32 makes p[ti]
        float p_mine = 0.0f;
        if (lane < tile_len) p_mine = cera_expf(__fsub_rn(sc_sh[lane], new_max));
        __syncthreads();
        if (lane < tile_len) sc_sh[lane] = p_mine;
        __syncthreads();
        double tile_sum = 0.0;
        for (uint32_t ti = 0; ti < tile_len; ++ti) tile_sum += static_cast<double>(sc_sh[ti]);
#pragma unroll
        for (int c = 0; c < 4; ++c) acc[c] = __fmul_rn(acc[c], rescale);
        for (uint32_t ti = 0; ti < tile_len; ++ti) {
            const float pv = sc_sh[ti];
            const KV* vp = vbase + static_cast<uint64_t>(kv_start + ti) * hd;
#pragma unroll
            for (int c = 0; c < 4; ++c)
                if (lane + 64 * c < hd) acc[c] = fmaf(pv, KvOps<KV>::ld1(vp + lane + 64 * c), acc[c]);
        }
        running_sum = running_sum * static_cast<double>(rescale) + tile_sum;
        running_max = new_max;
        __syncthreads();
    }
    const float inv_sum = static_cast<float>(1.0 / running_sum);
    float* oh = out + (static_cast<uint64_t>(jq) * n_heads + h) * hd;
#pragma unroll
    for (int c = 0; c < 4; ++c)
        if (lane + 64 * c < hd) oh[lane + 64 * c] = __fmul_rn(acc[c], inv_sum);
}

__global__ void ref_set_pos_kernel(uint32_t* scalars, uint32_t pos) { scalars[1] = pos; }

// cpu::rmsnorm with the CPU's serial f64 chain: squares are formed in parallel (exact in f64),
// staged through LDS 256 at a time and added by one thread in index order.  In place is fine
// (y == x): every element is read and written by the same thread.
__global__ __launch_bounds__(256) void rmsnorm_ref_kernel(const float* x, const float* __restrict__ w, uint32_t n, float eps,
                                                          float* y) {
    __shared__ double sq[256];
    __shared__ float inv_sh;
    const float* xr = x + static_cast<uint64_t>(blockIdx.x) * n;
    float* yr = y + static_cast<uint64_t>(blockIdx.x) * n;
    double sum = 0.0;
    for (uint32_t base = 0; base < n; base += 256) {
        const uint32_t i = base + threadIdx.x;
        const double v = i < n ? static_cast<double>(xr[i]) : 0.0;
        sq[threadIdx.x] = v * v;
        __syncthreads();
        if (threadIdx.x == 0) {
            const uint32_t cnt = min(256u, n - base);
            for (uint32_t t = 0; t < cnt; ++t) sum += sq[t];
        }
        __syncthreads();
    }
    if (threadIdx.x == 0) {
        const double mean = sum / static_cast<double>(n);
        inv_sh = static_cast<float>(1.0 / sqrt(mean + static_cast<double>(eps)));
    }
    __syncthreads();
    const float inv = inv_sh;
    for (uint32_t i = threadIdx.x; i < n; i += 256) yr[i] = __fmul_rn(__fmul_rn(xr[i], inv), w[i]);
}

// One workgroup per query head.  scores: [n_heads][max_seq] scratch.
template <typename KV>
__global__ __launch_bounds__(256) void attn_ref_kernel(const float* __restrict__ q, const KV* __restrict__ kc,
                                                       const KV* __restrict__ vc, uint32_t L, uint32_t max_seq, uint32_t hd,
                                                       uint32_t group, float scale, float* scores_all, float* __restrict__ out) {
    __shared__ float red[256];
    __shared__ float inv_sh;
    const uint32_t h = blockIdx.x, kvh = h / group;
    const float* qh = q + h * hd;
    const KV* kbase = kc + static_cast<uint64_t>(kvh) * max_seq * hd;
    const KV* vbase = vc + static_cast<uint64_t>(kvh) * max_seq * hd;
    float* scores = scores_all + static_cast<uint64_t>(h) * max_seq;
    const uint32_t grp = threadIdx.x >> 3, j = threadIdx.x & 7, nq = hd / 8;
    // attn_scores_avx2: s0 takes the even 8-wide slices, s1 the odd ones
    for (uint32_t t0 = 0; t0 < L; t0 += 32) {
        const uint32_t t = min(t0 + grp, L - 1);   // surplus groups redo the last key
        const KV* kp = kbase + static_cast<uint64_t>(t) * hd;
        float s0 = 0.0f, s1 = 0.0f;
        uint32_t i = 0;
        for (; i + 2 <= nq; i += 2) {
            s0 = fmaf(qh[8 * i + j], KvOps<KV>::ld1(kp + 8 * i + j), s0);
            s1 = fmaf(qh[8 * (i + 1) + j], KvOps<KV>::ld1(kp + 8 * (i + 1) + j), s1);
        }
        if (i < nq) s0 = fmaf(qh[8 * i + j], KvOps<KV>::ld1(kp + 8 * i + j), s0);
        const float v = grp_hsum(__fadd_rn(s0, s1));
        if (j == 0 && t0 + grp < L) scores[t] = __fmul_rn(v, scale);
    }
    __syncthreads();
    // softmax_inplace: max (order-free), exp, f64 sum in key order, f32 inverse
    float mx = -__builtin_inff();
    for (uint32_t t = threadIdx.x; t < L; t += 256) mx = fmaxf(mx, scores[t]);
    red[threadIdx.x] = mx;
    __syncthreads();
    for (uint32_t s = 128; s > 0; s >>= 1) {
        if (threadIdx.x < s) red[threadIdx.x] = fmaxf(red[threadIdx.x], red[threadIdx.x + s]);
        __syncthreads();
    }
    mx = red[0];
    __syncthreads();
    double sum = 0.0;
    for (uint32_t base = 0; base < L; base += 256) {
        const uint32_t t = base + threadIdx.x;
        if (t < L) {
            const float e = cera_expf(__fsub_rn(scores[t], mx));
            scores[t] = e;
            red[threadIdx.x] = e;
        }
        __syncthreads();
        if (threadIdx.x == 0) {
            const uint32_t cnt = min(256u, L - base);
            for (uint32_t u = 0; u < cnt; ++u) sum += static_cast<double>(red[u]);
        }
        __syncthreads();
    }
    if (threadIdx.x == 0) inv_sh = static_cast<float>(1.0 / sum);
    __syncthreads();
    const float inv = inv_sh;
    for (uint32_t t = threadIdx.x; t < L; t += 256) scores[t] = __fmul_rn(scores[t], inv);
    __syncthreads();
    // attn_values_avx2: one FMA chain per output column, keys in order
    if (threadIdx.x < hd) {
        float acc = 0.0f;
        for (uint32_t t = 0; t < L; ++t) acc = fmaf(scores[t], KvOps<KV>::ld1(vbase + static_cast<uint64_t>(t) * hd + threadIdx.x), acc);
        out[h * hd + threadIdx.x] = acc;
    }
}

bool ref_type_ok(uint32_t t) {
    return t == CERA_HIP_Q4_0 || t == CERA_HIP_Q4_1 || t == CERA_HIP_Q8_0 || t == CERA_HIP_Q4_K || t == CERA_HIP_Q6_K;
}

// Q5_K reads the f32 activations themselves (no Q8_0 step on the reference's route)
cera_hip_status launch_gemv_q5k_ref(cera_hip_ctx* ctx, const cera_hip_dtensor* w, const float* x_f32, float* y) {
    if (w->dtype != CERA_HIP_Q5_K || w->k % 256 || w->k == 0)
        return cera_fail(ctx, CERA_HIP_ERR_SHAPE, "reference-order Q5_K gemv: k must be a positive multiple of 256");
    RefGemvF32Args a{w->dev, x_f32, y, static_cast<uint32_t>(w->m), static_cast<uint32_t>(w->k), static_cast<uint32_t>(w->row_bytes)};
    hipLaunchKernelGGL(gemv_q5k_ref_kernel, dim3(static_cast<uint32_t>((w->m + 3) / 4)), dim3(256), 0, ctx->stream, a);
    HIP_TRY(ctx, hipGetLastError());
    return CERA_HIP_OK;
}

cera_hip_status launch_gemv_ref(cera_hip_ctx* ctx, const cera_hip_dtensor* w, const float* xs, const int8_t* xq, float* y) {
    if (!ref_type_ok(w->dtype))
        return cera_fail(ctx, CERA_HIP_ERR_UNSUPPORTED_DTYPE,
                         "reference-order gemv: no kernel for ggml type " + std::to_string(w->dtype));
    RefGemvArgs a{w->dev, xq, xs, y, static_cast<uint32_t>(w->m), static_cast<uint32_t>(w->k), static_cast<uint32_t>(w->row_bytes)};
    const dim3 grid(static_cast<uint32_t>((w->m + 31) / 32)), block(256);
    switch (w->dtype) {
        case CERA_HIP_Q4_K: hipLaunchKernelGGL(gemv_ref_kernel<12>, grid, block, 0, ctx->stream, a); break;
        case CERA_HIP_Q6_K: hipLaunchKernelGGL(gemv_ref_kernel<14>, grid, block, 0, ctx->stream, a); break;
        case CERA_HIP_Q4_0: hipLaunchKernelGGL(gemv_ref_kernel<2>, grid, block, 0, ctx->stream, a); break;
        case CERA_HIP_Q4_1: hipLaunchKernelGGL(gemv_ref_kernel<3>, grid, block, 0, ctx->stream, a); break;
        default: hipLaunchKernelGGL(gemv_ref_kernel<8>, grid, block, 0, ctx->stream, a); break;
    }
    HIP_TRY(ctx, hipGetLastError());
    return CERA_HIP_OK;
}

cera_hip_status launch_rmsnorm_ref(cera_hip_ctx* ctx, const float* x, const float* w, uint32_t n, uint32_t rows, float eps, float* y) {
    hipLaunchKernelGGL(rmsnorm_ref_kernel, dim3(rows), dim3(256), 0, ctx->stream, x, w, n, eps, y);
    HIP_TRY(ctx, hipGetLastError());
    return CERA_HIP_OK;
}

cera_hip_status launch_attn_ref(cera_hip_ctx* ctx, const float* q, const void* kc, const void* vc, uint32_t n_heads,
                                uint32_t n_kv_heads, uint32_t head_dim, uint32_t seq_len, uint32_t max_seq, float scale,
                                float* scores, float* out, bool kv_f16) {
    if (head_dim % 8 || head_dim > 256 || seq_len == 0 || seq_len > max_seq || n_kv_heads == 0 || n_heads % n_kv_heads)
        return cera_fail(ctx, CERA_HIP_ERR_SHAPE, "reference-order attention: bad shape");
    const uint32_t group = n_heads / n_kv_heads;
    if (kv_f16)
        hipLaunchKernelGGL(attn_ref_kernel<kv_half>, dim3(n_heads), dim3(256), 0, ctx->stream, q, static_cast<const kv_half*>(kc),
                           static_cast<const kv_half*>(vc), seq_len, max_seq, head_dim, group, scale, scores, out);
    else
        hipLaunchKernelGGL(attn_ref_kernel<float>, dim3(n_heads), dim3(256), 0, ctx->stream, q, static_cast<const float*>(kc),
                           static_cast<const float*>(vc), seq_len, max_seq, head_dim, group, scale, scores, out);
    HIP_TRY(ctx, hipGetLastError());
    return CERA_HIP_OK;
}

// out[j * ld_n + i * ld_m] = (W . B)[i][j] for n quantized activation rows, every element in the
// order of the x86 host's batched route: the 8x8 kernels for a weight cera repacks at load when
// x86_repack is set, the KQ_COLS-tiled / strip kernels otherwise.
cera_hip_status launch_gemm_ref(cera_hip_ctx* ctx, const cera_hip_dtensor* w, const float* xs, const int8_t* xq, uint32_t n,
                                bool x86_repack, float* out, uint64_t ld_m, uint64_t ld_n) {
    if (!ref_type_ok(w->dtype))
        return cera_fail(ctx, CERA_HIP_ERR_UNSUPPORTED_DTYPE,
                         "reference-order gemm: no kernel for ggml type " + std::to_string(w->dtype));
    if (n == 0 || n > 65535) return cera_fail(ctx, CERA_HIP_ERR_SHAPE, "reference-order gemm: 1 .. 65535 activation rows");
    RefGemmArgs a{w->dev, xq, xs, out, static_cast<uint32_t>(w->m), n, static_cast<uint32_t>(w->k),
                  static_cast<uint32_t>(w->row_bytes), ld_m, ld_n};
    const dim3 grid(static_cast<uint32_t>((w->m + 31) / 32), n), block(256);
    // repack_supported: Q4_0 with m % 8 == 0, Q4_K with m % 8 == 0 and whole super-blocks
    const bool rp = x86_repack && w->m % 8 == 0 && (w->dtype == CERA_HIP_Q4_0 || (w->dtype == CERA_HIP_Q4_K && w->k % 256 == 0));
    switch (w->dtype) {
        case CERA_HIP_Q4_K:
            if (rp) hipLaunchKernelGGL((gemm_ref_kernel<12, true>), grid, block, 0, ctx->stream, a);
            else hipLaunchKernelGGL((gemm_ref_kernel<12, false>), grid, block, 0, ctx->stream, a);
            break;
        case CERA_HIP_Q6_K: hipLaunchKernelGGL((gemm_ref_kernel<14, false>), grid, block, 0, ctx->stream, a); break;
        case CERA_HIP_Q4_0:
            if (rp) hipLaunchKernelGGL((gemm_ref_kernel<2, true>), grid, block, 0, ctx->stream, a);
            else hipLaunchKernelGGL((gemm_ref_kernel<2, false>), grid, block, 0, ctx->stream, a);
            break;
        case CERA_HIP_Q4_1: hipLaunchKernelGGL((gemm_ref_kernel<3, false>), grid, block, 0, ctx->stream, a); break;
        default: hipLaunchKernelGGL((gemm_ref_kernel<8, false>), grid, block, 0, ctx->stream, a); break;
    }
    HIP_TRY(ctx, hipGetLastError());
    return CERA_HIP_OK;
}

cera_hip_status launch_flash_ref(cera_hip_ctx* ctx, const float* q, const void* kc, const void* vc, uint32_t n_queries,
                                 uint32_t n_heads, uint32_t n_kv_heads, uint32_t head_dim, uint32_t max_seq, uint32_t start_pos,
                                 float scale, float* out, bool kv_f16) {
    if (head_dim % 8 || head_dim > 256 || n_queries == 0 || n_queries > 65535 || start_pos + n_queries > max_seq ||
        n_kv_heads == 0 || n_heads % n_kv_heads)
        return cera_fail(ctx, CERA_HIP_ERR_SHAPE, "reference-order flash attention: bad shape");
    const dim3 grid(n_queries, n_heads);
    const uint32_t group = n_heads / n_kv_heads;
    if (kv_f16)
        hipLaunchKernelGGL(flash_ref_kernel<kv_half>, grid, dim3(64), 0, ctx->stream, q, static_cast<const kv_half*>(kc),
                           static_cast<const kv_half*>(vc), n_heads, group, head_dim, max_seq, start_pos, scale, out);
    else
        hipLaunchKernelGGL(flash_ref_kernel<float>, grid, dim3(64), 0, ctx->stream, q, static_cast<const float*>(kc),
                           static_cast<const float*>(vc), n_heads, group, head_dim, max_seq, start_pos, scale, out);
    HIP_TRY(ctx, hipGetLastError());
    return CERA_HIP_OK;
}

}  // namespace

// Attention of one query for any head_dim that is a multiple of 8 (at most 256) and any number of
// query heads per kv head: the kernel of the verification route, which is what the default route
// runs for shapes its tuned kernels (head_dim 64 / 128, groups of at most 8) do not cover.
cera_hip_status cera_launch_attn_generic(cera_hip_ctx* ctx, const float* q, const void* kc, const void* vc, uint32_t n_heads,
                                         uint32_t n_kv_heads, uint32_t head_dim, uint32_t seq_len, uint32_t max_seq, float scale,
                                         float* scores, float* out, bool kv_f16) {
    return launch_attn_ref(ctx, q, kc, vc, n_heads, n_kv_heads, head_dim, seq_len, max_seq, scale, scores, out, kv_f16);
}

// ---------------------------------------------------------------------------
// LlamaModel::run_layers + project_logits (cera/src/model/llama.rs:468-597) with every
// operation a launch of its own, in the CPU path's order.
cera_hip_status cera_model_decode_step_ref(cera_hip_model* m, uint32_t pos, bool want_logits) {
    cera_hip_ctx* ctx = m->ctx;
    const cera_hip_config& c = m->cfg;
    hipStream_t s = ctx->stream;
    const uint32_t q_dim = c.n_heads * c.head_dim, kv_dim = c.n_kv_heads * c.head_dim;
    const float scale = c.attn_scale != 0.0f ? c.attn_scale : 1.0f / std::sqrt(static_cast<float>(c.head_dim));
    if (!m->ref_scores) {
        const uint64_t bytes = static_cast<uint64_t>(c.n_heads) * c.max_seq_len * sizeof(float);
        HIP_TRY(ctx, hipMalloc(reinterpret_cast<void**>(&m->ref_scores), bytes));
        m->owned.push_back(m->ref_scores);
        m->bytes += bytes;
    }
    auto gemv = [&](const cera_hip_dtensor* w, const float* x_f32, uint32_t k, float* y) -> cera_hip_status {
        if (w->dtype == CERA_HIP_Q5_K) return launch_gemv_q5k_ref(ctx, w, x_f32, y);
        // gemv_dispatch quantizes its input on every call (cera/src/backend/cpu.rs:787-790)
        CERA_TRY(cera_launch_quantize(ctx, x_f32, k, m->xs, m->xq));
        return launch_gemv_ref(ctx, w, m->xs, m->xq, y);
    };
    auto add_scaled = [&](const float* block_out) -> cera_hip_status {
        hipLaunchKernelGGL(add_kernel, dim3((c.hidden + 255) / 256), dim3(256), 0, s, m->hidden, block_out, c.residual_scale,
                           c.hidden, m->hidden);
        HIP_TRY(ctx, hipGetLastError());
        return CERA_HIP_OK;
    };

    hipLaunchKernelGGL(embed_row_kernel, dim3((c.hidden + 255) / 256), dim3(256), 0, s, m->embd->dtype, m->embd->dev,
                       m->embd->row_bytes, m->scalars, c.hidden, c.embed_scale, m->hidden);
    HIP_TRY(ctx, hipGetLastError());
    for (uint32_t i = 0; i < c.n_layers; ++i) {
        LayerDev& L = m->layers[i];
        CERA_TRY(launch_rmsnorm_ref(ctx, m->hidden, L.attn_norm, c.hidden, 1, c.rms_eps, m->normed));
        CERA_TRY(gemv(L.q, m->normed, c.hidden, m->q));
        CERA_TRY(gemv(L.k, m->normed, c.hidden, m->k));
        CERA_TRY(gemv(L.v, m->normed, c.hidden, m->v));
        if (L.q_bias) {
            hipLaunchKernelGGL(bias_kernel, dim3((q_dim + 255) / 256), dim3(256), 0, s, m->q, L.q_bias, q_dim);
            hipLaunchKernelGGL(bias_kernel, dim3((kv_dim + 255) / 256), dim3(256), 0, s, m->k, L.k_bias, kv_dim);
            hipLaunchKernelGGL(bias_kernel, dim3((kv_dim + 255) / 256), dim3(256), 0, s, m->v, L.v_bias, kv_dim);
        }
        if (L.q_norm) {
            CERA_TRY(launch_rmsnorm_ref(ctx, m->q, L.q_norm, c.head_dim, c.n_heads, c.rms_eps, m->q));
            CERA_TRY(launch_rmsnorm_ref(ctx, m->k, L.k_norm, c.head_dim, c.n_kv_heads, c.rms_eps, m->k));
        }
        const dim3 rgrid(c.n_heads + 2 * c.n_kv_heads, 1), rblock(c.head_dim / 2);
        if (m->kv_f16)
            hipLaunchKernelGGL(rope_kv_kernel<kv_half>, rgrid, rblock, 0, s, m->q, m->k, m->v, m->rope_table, m->scalars + 1,
                               c.n_heads, c.n_kv_heads, c.head_dim, c.rope_type, static_cast<kv_half*>(L.kc),
                               static_cast<kv_half*>(L.vc), c.max_seq_len);
        else
            hipLaunchKernelGGL(rope_kv_kernel<float>, rgrid, rblock, 0, s, m->q, m->k, m->v, m->rope_table, m->scalars + 1,
                               c.n_heads, c.n_kv_heads, c.head_dim, c.rope_type, static_cast<float*>(L.kc),
                               static_cast<float*>(L.vc), c.max_seq_len);
        HIP_TRY(ctx, hipGetLastError());
        CERA_TRY(launch_attn_ref(ctx, m->q, L.kc, L.vc, c.n_heads, c.n_kv_heads, c.head_dim, pos + 1, c.max_seq_len, scale,
                                 m->ref_scores, m->attn_out, m->kv_f16));
        CERA_TRY(gemv(L.o, m->attn_out, q_dim, m->proj));
        CERA_TRY(add_scaled(m->proj));

        CERA_TRY(launch_rmsnorm_ref(ctx, m->hidden, L.ffn_norm, c.hidden, 1, c.rms_eps, m->normed));
        CERA_TRY(gemv(L.gate, m->normed, c.hidden, m->act));
        CERA_TRY(gemv(L.up, m->normed, c.hidden, m->up));
        hipLaunchKernelGGL((silu_mul_kernel<false>), dim3((c.ffn / 4 + 255) / 256), dim3(256), 0, s, m->act, m->up,
                           static_cast<uint64_t>(c.ffn), m->act, static_cast<float*>(nullptr), static_cast<int8_t*>(nullptr),
                           static_cast<float*>(nullptr));
        HIP_TRY(ctx, hipGetLastError());
        CERA_TRY(gemv(L.down, m->act, c.ffn, m->proj));
        CERA_TRY(add_scaled(m->proj));
    }
    CERA_TRY(launch_rmsnorm_ref(ctx, m->hidden, m->output_norm, c.hidden, 1, c.rms_eps, m->hidden));
    if (want_logits) {
        const cera_hip_dtensor* o = m->output ? m->output : m->embd;
        CERA_TRY(gemv(o, m->hidden, c.hidden, m->logits));
        if (c.logit_scale != 1.0f) {
            hipLaunchKernelGGL(scale_kernel, dim3((c.vocab + 255) / 256), dim3(256), 0, s, m->logits, 1.0f / c.logit_scale,
                               c.vocab);
            HIP_TRY(ctx, hipGetLastError());
        }
    }
    return CERA_HIP_OK;
}

// LlamaModel::forward_prefill_batched (cera/src/model/llama.rs:738-1523) as an x86 host without
// `blas` runs it, every operation a launch of its own in the CPU path's order: rmsnorm per row,
// quantize_columns (transformer.rs:865-946), gemm_preq with the repacked 8x8 kernels where cera
// repacks (transformer.rs:710-788), RoPE + cache append per token, flash_attention_gqa_avx2 from
// 256 tokens on (llama.rs:885) and the per-token attn_scores / softmax / attn_values below that,
// SwiGLU, residual adds; then project_logits of the last row through the n == 1 GEMV branch.
// n tokens in one pass (n <= the prefill buffers' capacity; the caller splits longer prompts).
cera_hip_status cera_model_prefill_ref_batched(cera_hip_model* m, const uint32_t* tokens, uint32_t n, uint32_t start_pos,
                                               bool want_logits) {
    cera_hip_ctx* ctx = m->ctx;
    const cera_hip_config& c = m->cfg;
    hipStream_t s = ctx->stream;
    const uint32_t hs = c.hidden, q_dim = c.n_heads * c.head_dim, kv_dim = c.n_kv_heads * c.head_dim;
    const float scale = c.attn_scale != 0.0f ? c.attn_scale : 1.0f / std::sqrt(static_cast<float>(c.head_dim));
    CERA_TRY(cera_model_ensure_prefill_buffers(m, n));
    if (n > m->pf_cap) return cera_fail(ctx, CERA_HIP_ERR_SHAPE, "reference-order prefill: more tokens than one pass holds");
    if (!m->ref_scores) {
        const uint64_t bytes = static_cast<uint64_t>(c.n_heads) * c.max_seq_len * sizeof(float);
        HIP_TRY(ctx, hipMalloc(reinterpret_cast<void**>(&m->ref_scores), bytes));
        m->owned.push_back(m->ref_scores);
        m->bytes += bytes;
    }
    CERA_TRY(cera_hip_upload(ctx, m->pf_tokens, tokens, n * 4ull));
    hipLaunchKernelGGL(ref_set_pos_kernel, dim3(1), dim3(1), 0, s, m->scalars, start_pos);
    hipLaunchKernelGGL(embed_row_kernel, dim3((hs + 255) / 256, n), dim3(256), 0, s, m->embd->dtype, m->embd->dev,
                       m->embd->row_bytes, m->pf_tokens, hs, c.embed_scale, m->pf_hidden);
    HIP_TRY(ctx, hipGetLastError());
    const bool repack = m->ref_order == 2;
    // quantize_columns + gemm_preq: out[n][w->m]
    auto gemm = [&](const cera_hip_dtensor* w, const float* x_f32, float* out) -> cera_hip_status {
        CERA_TRY(cera_launch_quantize(ctx, x_f32, static_cast<uint64_t>(n) * w->k, m->pf_xs, m->pf_xq));
        return launch_gemm_ref(ctx, w, m->pf_xs, m->pf_xq, n, repack, out, 1, w->m);
    };
    auto add_rows = [&](const float* block_out) -> cera_hip_status {
        const uint32_t tot = n * hs;
        hipLaunchKernelGGL(add_kernel, dim3((tot + 255) / 256), dim3(256), 0, s, m->pf_hidden, block_out, c.residual_scale, tot,
                           m->pf_hidden);
        HIP_TRY(ctx, hipGetLastError());
        return CERA_HIP_OK;
    };
    for (uint32_t i = 0; i < c.n_layers; ++i) {
        LayerDev& L = m->layers[i];
        CERA_TRY(launch_rmsnorm_ref(ctx, m->pf_hidden, L.attn_norm, hs, n, c.rms_eps, m->pf_normed));
        CERA_TRY(gemm(L.q, m->pf_normed, m->pf_q));
        CERA_TRY(launch_gemm_ref(ctx, L.k, m->pf_xs, m->pf_xq, n, repack, m->pf_k, 1, L.k->m));   // the same quantized columns
        CERA_TRY(launch_gemm_ref(ctx, L.v, m->pf_xs, m->pf_xq, n, repack, m->pf_v, 1, L.v->m));
        if (L.q_bias) {
            for (uint32_t t = 0; t < n; ++t) {
                hipLaunchKernelGGL(bias_kernel, dim3((q_dim + 255) / 256), dim3(256), 0, s, m->pf_q + static_cast<uint64_t>(t) * q_dim, L.q_bias, q_dim);
                hipLaunchKernelGGL(bias_kernel, dim3((kv_dim + 255) / 256), dim3(256), 0, s, m->pf_k + static_cast<uint64_t>(t) * kv_dim, L.k_bias, kv_dim);
                hipLaunchKernelGGL(bias_kernel, dim3((kv_dim + 255) / 256), dim3(256), 0, s, m->pf_v + static_cast<uint64_t>(t) * kv_dim, L.v_bias, kv_dim);
            }
        }
        if (L.q_norm) {
            CERA_TRY(launch_rmsnorm_ref(ctx, m->pf_q, L.q_norm, c.head_dim, n * c.n_heads, c.rms_eps, m->pf_q));
            CERA_TRY(launch_rmsnorm_ref(ctx, m->pf_k, L.k_norm, c.head_dim, n * c.n_kv_heads, c.rms_eps, m->pf_k));
        }
        const dim3 rgrid(c.n_heads + 2 * c.n_kv_heads, n), rblock(c.head_dim / 2);
        if (m->kv_f16)
            hipLaunchKernelGGL(rope_kv_kernel<kv_half>, rgrid, rblock, 0, s, m->pf_q, m->pf_k, m->pf_v, m->rope_table, m->scalars + 1,
                               c.n_heads, c.n_kv_heads, c.head_dim, c.rope_type, static_cast<kv_half*>(L.kc),
                               static_cast<kv_half*>(L.vc), c.max_seq_len);
        else
            hipLaunchKernelGGL(rope_kv_kernel<float>, rgrid, rblock, 0, s, m->pf_q, m->pf_k, m->pf_v, m->rope_table, m->scalars + 1,
                               c.n_heads, c.n_kv_heads, c.head_dim, c.rope_type, static_cast<float*>(L.kc),
                               static_cast<float*>(L.vc), c.max_seq_len);
        HIP_TRY(ctx, hipGetLastError());
        if (n >= 256) {   // FLASH_ATTN_THRESHOLD
            CERA_TRY(launch_flash_ref(ctx, m->pf_q, L.kc, L.vc, n, c.n_heads, c.n_kv_heads, c.head_dim, c.max_seq_len, start_pos,
                                      scale, m->pf_attn, m->kv_f16));
        } else {
            for (uint32_t t = 0; t < n; ++t)
                CERA_TRY(launch_attn_ref(ctx, m->pf_q + static_cast<uint64_t>(t) * q_dim, L.kc, L.vc, c.n_heads, c.n_kv_heads,
                                         c.head_dim, start_pos + t + 1, c.max_seq_len, scale, m->ref_scores,
                                         m->pf_attn + static_cast<uint64_t>(t) * q_dim, m->kv_f16));
        }
        CERA_TRY(gemm(L.o, m->pf_attn, m->pf_normed));   // pf_normed is free here: block_out
        CERA_TRY(add_rows(m->pf_normed));

        CERA_TRY(launch_rmsnorm_ref(ctx, m->pf_hidden, L.ffn_norm, hs, n, c.rms_eps, m->pf_normed));
        CERA_TRY(gemm(L.gate, m->pf_normed, m->pf_gate));
        CERA_TRY(launch_gemm_ref(ctx, L.up, m->pf_xs, m->pf_xq, n, repack, m->pf_up, 1, L.up->m));
        const uint64_t tot = static_cast<uint64_t>(n) * c.ffn;
        hipLaunchKernelGGL((silu_mul_kernel<false>), dim3(static_cast<uint32_t>((tot / 4 + 255) / 256)), dim3(256), 0, s, m->pf_gate,
                           m->pf_up, tot, m->pf_gate, static_cast<float*>(nullptr), static_cast<int8_t*>(nullptr),
                           static_cast<float*>(nullptr));
        HIP_TRY(ctx, hipGetLastError());
        CERA_TRY(gemm(L.down, m->pf_gate, m->pf_normed));
        CERA_TRY(add_rows(m->pf_normed));
    }
    m->seq_len = start_pos + n;
    if (want_logits) {
        // project_logits on the last row: the per-token path's norm and n == 1 GEMV
        const float* last = m->pf_hidden + static_cast<uint64_t>(n - 1) * hs;
        CERA_TRY(launch_rmsnorm_ref(ctx, last, m->output_norm, hs, 1, c.rms_eps, m->hidden));
        const cera_hip_dtensor* o = m->output ? m->output : m->embd;
        if (o->dtype == CERA_HIP_Q5_K) {
            CERA_TRY(launch_gemv_q5k_ref(ctx, o, m->hidden, m->logits));
        } else {
            CERA_TRY(cera_launch_quantize(ctx, m->hidden, hs, m->xs, m->xq));
            CERA_TRY(launch_gemv_ref(ctx, o, m->xs, m->xq, m->logits));
        }
        if (c.logit_scale != 1.0f) {
            hipLaunchKernelGGL(scale_kernel, dim3((c.vocab + 255) / 256), dim3(256), 0, s, m->logits, 1.0f / c.logit_scale, c.vocab);
            HIP_TRY(ctx, hipGetLastError());
        }
    }
    return CERA_HIP_OK;
}

bool cera_model_ref_order_supported(const cera_hip_model* m, std::string* why) {
    auto ok = [&](const cera_hip_dtensor* w, const char* name) {
        if (w && !ref_type_ok(w->dtype) && w->dtype != CERA_HIP_Q5_K) {
            *why = std::string(name) + " has ggml type " + std::to_string(w->dtype) + " (no reference-order kernel)";
            return false;
        }
        return true;
    };
    for (const LayerDev& L : m->layers)
        if (!ok(L.q, "attn_q") || !ok(L.k, "attn_k") || !ok(L.v, "attn_v") || !ok(L.o, "attn_output") || !ok(L.gate, "ffn_gate") ||
            !ok(L.up, "ffn_up") || !ok(L.down, "ffn_down"))
            return false;
    return ok(m->output ? m->output : m->embd, "output");
}

// ---- kernel-level entry points (host buffers) ------------------------------------------------
extern "C" cera_hip_status cera_hip_gemv_reference_order(cera_hip_ctx* ctx, const cera_hip_tensor* t, const float* x, float* y) {
    if (!ctx || !t || !x || !y) return CERA_HIP_ERR_ARGUMENT;
    std::lock_guard<std::recursive_mutex> lk(ctx->op_mu);
    cera_hip_dtensor* w = nullptr;
    CERA_TRY(cera_hip_tensor_upload(ctx, t, &w));
    auto run = [&]() -> cera_hip_status {
        const uint64_t k = w->k, mm = w->m;
        void *dx, *ds, *dq, *dy;
        CERA_TRY(cera_scratch(ctx, 0, k * 4, &dx));
        CERA_TRY(cera_scratch(ctx, 1, k / 32 * 4, &ds));
        CERA_TRY(cera_scratch(ctx, 2, k, &dq));
        CERA_TRY(cera_scratch(ctx, 3, mm * 4, &dy));
        CERA_TRY(cera_hip_upload(ctx, dx, x, k * 4));
        if (w->dtype == CERA_HIP_Q5_K) {
            CERA_TRY(launch_gemv_q5k_ref(ctx, w, static_cast<float*>(dx), static_cast<float*>(dy)));
            return cera_hip_download(ctx, y, dy, mm * 4);
        }
        CERA_TRY(cera_launch_quantize(ctx, static_cast<float*>(dx), k, static_cast<float*>(ds), static_cast<int8_t*>(dq)));
        CERA_TRY(launch_gemv_ref(ctx, w, static_cast<float*>(ds), static_cast<int8_t*>(dq), static_cast<float*>(dy)));
        return cera_hip_download(ctx, y, dy, mm * 4);
    };
    cera_hip_status st = run();
    cera_hip_tensor_free(ctx, w);
    return st;
}

extern "C" cera_hip_status cera_hip_attn_decode_reference_order(cera_hip_ctx* ctx, const float* q, const float* k, const float* v,
                                                                uint32_t n_heads, uint32_t n_kv_heads, uint32_t head_dim,
                                                                uint64_t seq_len, float scale, float* out) {
    if (!ctx || !q || !k || !v || !out) return CERA_HIP_ERR_ARGUMENT;
    if (seq_len == 0 || seq_len > 0x7FFFFFFFull || n_kv_heads == 0 || head_dim == 0)
        return cera_fail(ctx, CERA_HIP_ERR_SHAPE, "attn_decode_reference_order: empty input");
    std::lock_guard<std::recursive_mutex> lk(ctx->op_mu);
    const uint64_t kv_dim = static_cast<uint64_t>(n_kv_heads) * head_dim, q_bytes = static_cast<uint64_t>(n_heads) * head_dim * 4;
    std::vector<float> hk(seq_len * kv_dim), hv(seq_len * kv_dim);   // time-major -> head-major
    for (uint64_t t = 0; t < seq_len; ++t)
        for (uint32_t h = 0; h < n_kv_heads; ++h)
            for (uint32_t d = 0; d < head_dim; ++d) {
                hk[(h * seq_len + t) * head_dim + d] = k[t * kv_dim + h * head_dim + d];
                hv[(h * seq_len + t) * head_dim + d] = v[t * kv_dim + h * head_dim + d];
            }
    void *dq, *dk, *dv, *dout, *dsc;
    CERA_TRY(cera_scratch(ctx, 0, q_bytes, &dq));
    CERA_TRY(cera_scratch(ctx, 5, hk.size() * 4, &dk));
    CERA_TRY(cera_scratch(ctx, 6, hv.size() * 4, &dv));
    CERA_TRY(cera_scratch(ctx, 3, q_bytes, &dout));
    CERA_TRY(cera_scratch(ctx, 4, n_heads * seq_len * 4, &dsc));
    CERA_TRY(cera_hip_upload(ctx, dq, q, q_bytes));
    CERA_TRY(cera_hip_upload(ctx, dk, hk.data(), hk.size() * 4));
    CERA_TRY(cera_hip_upload(ctx, dv, hv.data(), hv.size() * 4));
    CERA_TRY(launch_attn_ref(ctx, static_cast<float*>(dq), dk, dv, n_heads, n_kv_heads, head_dim, static_cast<uint32_t>(seq_len),
                             static_cast<uint32_t>(seq_len), scale, static_cast<float*>(dsc), static_cast<float*>(dout), false));
    return cera_hip_download(ctx, out, dout, q_bytes);
}

extern "C" cera_hip_status cera_hip_rmsnorm_reference_order(cera_hip_ctx* ctx, const float* x, const float* weight, uint64_t n,
                                                            float eps, float* y) {
    if (!ctx || !x || !weight || !y) return CERA_HIP_ERR_ARGUMENT;
    if (n == 0 || n > 0xFFFFFFFFull) return cera_fail(ctx, CERA_HIP_ERR_SHAPE, "rmsnorm_reference_order: bad n");
    std::lock_guard<std::recursive_mutex> lk(ctx->op_mu);
    void *dx, *dw, *dy;
    CERA_TRY(cera_scratch(ctx, 0, n * 4, &dx));
    CERA_TRY(cera_scratch(ctx, 1, n * 4, &dw));
    CERA_TRY(cera_scratch(ctx, 3, n * 4, &dy));
    CERA_TRY(cera_hip_upload(ctx, dx, x, n * 4));
    CERA_TRY(cera_hip_upload(ctx, dw, weight, n * 4));
    CERA_TRY(launch_rmsnorm_ref(ctx, static_cast<float*>(dx), static_cast<float*>(dw), static_cast<uint32_t>(n), 1, eps,
                                static_cast<float*>(dy)));
    return cera_hip_download(ctx, y, dy, n * 4);
}

// out[m][n] (the reference's layout, simd.rs:5130-5148) = W . Q8_0(x[n][k]) in the order of the x86
// host's batched route; x86_repack != 0: the 8x8 kernels for the weights cera repacks at load.
extern "C" cera_hip_status cera_hip_gemm_reference_order(cera_hip_ctx* ctx, const cera_hip_tensor* t, const float* x, uint64_t n,
                                                         uint32_t x86_repack, float* out) {
    if (!ctx || !t || !x || !out) return CERA_HIP_ERR_ARGUMENT;
    if (n == 0 || n > 65535) return cera_fail(ctx, CERA_HIP_ERR_SHAPE, "gemm_reference_order: 1 .. 65535 activation rows");
    std::lock_guard<std::recursive_mutex> lk(ctx->op_mu);
    cera_hip_dtensor* w = nullptr;
    CERA_TRY(cera_hip_tensor_upload(ctx, t, &w));
    auto run = [&]() -> cera_hip_status {
        const uint64_t k = w->k, mm = w->m;
        void *dx, *ds, *dq, *dy;
        CERA_TRY(cera_scratch(ctx, 0, n * k * 4, &dx));
        CERA_TRY(cera_scratch(ctx, 1, n * (k / 32) * 4, &ds));
        CERA_TRY(cera_scratch(ctx, 2, n * k, &dq));
        CERA_TRY(cera_scratch(ctx, 3, mm * n * 4, &dy));
        CERA_TRY(cera_hip_upload(ctx, dx, x, n * k * 4));
        CERA_TRY(cera_launch_quantize(ctx, static_cast<float*>(dx), n * k, static_cast<float*>(ds), static_cast<int8_t*>(dq)));
        CERA_TRY(launch_gemm_ref(ctx, w, static_cast<float*>(ds), static_cast<int8_t*>(dq), static_cast<uint32_t>(n), x86_repack != 0,
                                 static_cast<float*>(dy), n, 1));
        return cera_hip_download(ctx, out, dy, mm * n * 4);
    };
    cera_hip_status st = run();
    cera_hip_tensor_free(ctx, w);
    return st;
}

// flash_attention_gqa_avx2 for n_queries queries at positions start_pos .. start_pos + n_queries - 1:
// q, out [n_queries][n_heads * head_dim]; k, v the reference's time-major caches
// [start_pos + n_queries][n_kv_heads * head_dim].
extern "C" cera_hip_status cera_hip_flash_attn_reference_order(cera_hip_ctx* ctx, const float* q, const float* k, const float* v,
                                                               uint32_t n_queries, uint32_t n_heads, uint32_t n_kv_heads,
                                                               uint32_t head_dim, uint32_t start_pos, float scale, float* out) {
    if (!ctx || !q || !k || !v || !out) return CERA_HIP_ERR_ARGUMENT;
    if (n_queries == 0 || n_kv_heads == 0 || head_dim == 0)
        return cera_fail(ctx, CERA_HIP_ERR_SHAPE, "flash_attn_reference_order: empty input");
    std::lock_guard<std::recursive_mutex> lk(ctx->op_mu);
    const uint64_t seq = static_cast<uint64_t>(start_pos) + n_queries, kv_dim = static_cast<uint64_t>(n_kv_heads) * head_dim;
    const uint64_t q_bytes = static_cast<uint64_t>(n_queries) * n_heads * head_dim * 4;
    std::vector<float> hk(seq * kv_dim), hv(seq * kv_dim);   // time-major -> head-major
    for (uint64_t t = 0; t < seq; ++t)
        for (uint32_t h = 0; h < n_kv_heads; ++h)
            for (uint32_t d = 0; d < head_dim; ++d) {
                hk[(h * seq + t) * head_dim + d] = k[t * kv_dim + h * head_dim + d];
                hv[(h * seq + t) * head_dim + d] = v[t * kv_dim + h * head_dim + d];
            }
    void *dq, *dk, *dv, *dout;
    CERA_TRY(cera_scratch(ctx, 0, q_bytes, &dq));
    CERA_TRY(cera_scratch(ctx, 5, hk.size() * 4, &dk));
    CERA_TRY(cera_scratch(ctx, 6, hv.size() * 4, &dv));
    CERA_TRY(cera_scratch(ctx, 3, q_bytes, &dout));
    CERA_TRY(cera_hip_upload(ctx, dq, q, q_bytes));
    CERA_TRY(cera_hip_upload(ctx, dk, hk.data(), hk.size() * 4));
    CERA_TRY(cera_hip_upload(ctx, dv, hv.data(), hv.size() * 4));
    CERA_TRY(launch_flash_ref(ctx, static_cast<float*>(dq), dk, dv, n_queries, n_heads, n_kv_heads, head_dim,
                              static_cast<uint32_t>(seq), start_pos, scale, static_cast<float*>(dout), false));
    return cera_hip_download(ctx, out, dout, q_bytes);
}
