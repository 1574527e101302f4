// Small per-token kernels between the GEMVs: embedding row lookup, RMSNorm
// (+ Q8_0 quantize), RoPE + KV-cache append, SiLU*mul (+ quantize), argmax.
// All of them mirror cera's scalar CPU code operation by operation
// (cera/src/backend/cpu.rs) so that their f32 outputs match it bit for bit
// wherever the CPU order is a plain elementwise expression.
#pragma once
#include "common.hip.h"
#include "quantize.hip.h"

// ---------------------------------------------------------------------------
// Row dequantisation (cera/src/quant.rs:364-886 via
// cera/src/model/transformer.rs:949-1017): out[k] = dequant(row).  One thread
// per element; runs once per token for the embedding lookup.
__device__ __forceinline__ float dequant_elem(uint32_t dtype, const uint8_t* row, uint32_t e) {
    switch (dtype) {
        case 0: return reinterpret_cast<const float*>(row)[e];
        case 1: return h2f(reinterpret_cast<const uint16_t*>(row)[e]);
        case 30: {
            uint32_t b = reinterpret_cast<const uint16_t*>(row)[e];
            uint32_t quiet = ((b & 0x7FFF) > 0x7F80) ? 0x00400000u : 0u;
            return __builtin_bit_cast(float, (b << 16) | quiet);
        }
        case 2: {  // Q4_0
            const uint8_t* blk = row + (e >> 5) * 18;
            uint32_t i = e & 31, byte = blk[2 + (i & 15)];
            int q = static_cast<int>(i < 16 ? (byte & 0xF) : (byte >> 4)) - 8;
            return static_cast<float>(q) * h2f(ld_u16(blk));
        }
        case 3: {  // Q4_1
            const uint8_t* blk = row + (e >> 5) * 20;
            uint32_t i = e & 31, byte = blk[4 + (i & 15)];
            uint32_t q = i < 16 ? (byte & 0xF) : (byte >> 4);
            return __fadd_rn(__fmul_rn(static_cast<float>(q), h2f(ld_u16(blk))), h2f(ld_u16(blk + 2)));
        }
        case 8: {  // Q8_0
            const uint8_t* blk = row + (e >> 5) * 34;
            return static_cast<float>(static_cast<int8_t>(blk[2 + (e & 31)])) * h2f(ld_u16(blk));
        }
        case 12:
        case 13: {  // Q4_K / Q5_K
            const bool q5 = dtype == 13;
            const uint8_t* blk = row + (e >> 8) * (q5 ? 176 : 144);
            uint32_t i = e & 255, s = i >> 5, l = i & 31, j = s >> 1;
            const uint8_t* sc12 = blk + 4;
            uint32_t sc, mn;
            if (s < 4) {
                sc = sc12[s] & 63;
                mn = sc12[s + 4] & 63;
            } else {
                sc = (sc12[s + 4] & 0xF) | ((sc12[s - 4] >> 6) << 4);
                mn = (sc12[s + 4] >> 4) | ((sc12[s] >> 6) << 4);
            }
            uint32_t byte = blk[(q5 ? 48 : 16) + 32 * j + l];
            float q = static_cast<float>((s & 1) ? (byte >> 4) : (byte & 0xF));
            if (q5 && ((blk[16 + l] >> s) & 1)) q = __fadd_rn(q, 16.0f);
            float d = h2f(ld_u16(blk)), dmin = h2f(ld_u16(blk + 2));
            return __fsub_rn(__fmul_rn(__fmul_rn(d, static_cast<float>(sc)), q),
                             __fmul_rn(dmin, static_cast<float>(mn)));
        }
        case 14: {  // Q6_K
            const uint8_t* blk = row + (e >> 8) * 210;
            uint32_t i = e & 255, n = i >> 7, r = i & 127, t = r >> 5, l = r & 31;
            uint32_t ql = blk[64 * n + (t & 1) * 32 + l];
            uint32_t nib = t < 2 ? (ql & 0xF) : (ql >> 4);
            uint32_t h2 = (blk[128 + 32 * n + l] >> (2 * t)) & 3;
            int q = static_cast<int>(nib | (h2 << 4)) - 32;
            float sc = static_cast<float>(static_cast<int8_t>(blk[192 + 8 * n + (l >> 4) + 2 * t]));
            return __fmul_rn(__fmul_rn(h2f(ld_u16(blk + 208)), sc), static_cast<float>(q));
        }
        default: return 0.0f;
    }
}

// token comes from device memory so a graph-captured decode step can chain on
// the previous step's argmax without a host round trip.
// grid.y = number of tokens (prefill looks up a batch of rows: out is [n][k]).
__device__ __forceinline__ void embed_row_body(uint32_t dtype, const uint8_t* __restrict__ w, uint64_t row_bytes,
                                 const uint32_t* __restrict__ token, uint32_t k, float scale,
                                 float* __restrict__ out) {
    uint32_t e = blockIdx.x * blockDim.x + threadIdx.x;
    if (e >= k) return;
    float v = dequant_elem(dtype, w + static_cast<uint64_t>(token[blockIdx.y]) * row_bytes, e);
    out[static_cast<uint64_t>(blockIdx.y) * k + e] = scale != 1.0f ? __fmul_rn(v, scale) : v;
}
static __global__ void embed_row_kernel(uint32_t dtype, const uint8_t* __restrict__ w, uint64_t row_bytes,
                                 const uint32_t* __restrict__ token, uint32_t k, float scale,
                                 float* __restrict__ out) {
    embed_row_body(dtype, w, row_bytes, token, k, scale, out);
}

// The decode step's first launch: the token's embedding row, and the token id and position into
// scalars[0..1] for the kernels behind it (one launch instead of a one-thread kernel plus the lookup).
__device__ __forceinline__ void embed_token_body(uint32_t dtype, const uint8_t* __restrict__ w, uint64_t row_bytes, uint32_t token,
                                          uint32_t pos, uint32_t* __restrict__ scalars, uint32_t k, float scale,
                                          float* __restrict__ out) {
    uint32_t e = blockIdx.x * blockDim.x + threadIdx.x;
    if (e == 0) {
        scalars[0] = token;
        scalars[1] = pos;
    }
    if (e >= k) return;
    float v = dequant_elem(dtype, w + static_cast<uint64_t>(token) * row_bytes, e);
    out[e] = scale != 1.0f ? __fmul_rn(v, scale) : v;
}
static __global__ void embed_token_kernel(uint32_t dtype, const uint8_t* __restrict__ w, uint64_t row_bytes, uint32_t token,
                                          uint32_t pos, uint32_t* __restrict__ scalars, uint32_t k, float scale,
                                          float* __restrict__ out) {
    embed_token_body(dtype, w, row_bytes, token, pos, scalars, k, scale, out);
}

// ---------------------------------------------------------------------------
// RMSNorm (cera/src/backend/cpu.rs:2479-2496): f64 sum of squares,
// inv = (1/sqrt(mean + eps)) as f32, y = (x*inv)*w.  One 256-thread block per
// row of n elements; optionally also emits the Q8_0 quantisation of y.
// The f64 sum is a tree instead of the CPU's serial chain: f64 rounding
// differences (~1e-16 relative) vanish when inv is narrowed to f32 except in
// astronomically rare double-rounding cases.
// Split-K partial sums that the consumer of the rows adds up itself (PENDING): x_out[e] = (resid[e] +
// resid_scale *) sum_z part[z * stride + e], e over [rows][n]
struct RowsPending {
    const float* part;
    uint32_t n_split;
    uint64_t stride;
    const float* resid;
    float resid_scale;
    float* x_out;
};
template <bool QUANT, bool PENDING = false>
__device__ __forceinline__ void rmsnorm_body(const float* x, const float* __restrict__ w,
                                                      uint32_t n, float eps, float* __restrict__ y,
                                                      float* __restrict__ scales, int8_t* __restrict__ quants,
                                                      float* __restrict__ bsum, RowsPending pd = RowsPending{}) {
    __shared__ double part[4];
    const float* xr = x + static_cast<uint64_t>(blockIdx.x) * n;
    float* yr = y + static_cast<uint64_t>(blockIdx.x) * n;
    double s = 0.0;
    for (uint32_t i = threadIdx.x * 4; i < n; i += 1024) {
        float4 v;
        if (PENDING) {
            // the rows are not summed yet: x = (resid +) sum_z part[z], in gemm_reduce_kernel's order, stored to
            // x on the way (the second pass below re-reads what this thread wrote)
            const uint64_t e = static_cast<uint64_t>(blockIdx.x) * n + i;
            v = *reinterpret_cast<const float4*>(pd.part + e);
            for (uint32_t z = 1; z < pd.n_split; ++z) {
                const float4 a = *reinterpret_cast<const float4*>(pd.part + z * pd.stride + e);
                v.x += a.x; v.y += a.y; v.z += a.z; v.w += a.w;
            }
            if (pd.resid) {
                const float4 r = *reinterpret_cast<const float4*>(pd.resid + e);
                if (pd.resid_scale != 1.0f) { v.x *= pd.resid_scale; v.y *= pd.resid_scale; v.z *= pd.resid_scale; v.w *= pd.resid_scale; }
                v.x = r.x + v.x; v.y = r.y + v.y; v.z = r.z + v.z; v.w = r.w + v.w;
            }
            *reinterpret_cast<float4*>(pd.x_out + e) = v;
        } else {
            v = *reinterpret_cast<const float4*>(xr + i);
        }
        s += static_cast<double>(v.x) * v.x;
        s += static_cast<double>(v.y) * v.y;
        s += static_cast<double>(v.z) * v.z;
        s += static_cast<double>(v.w) * v.w;
    }
    s = wave_sum_f64(s);
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = s;
    __syncthreads();
    double tot = (part[0] + part[1]) + (part[2] + part[3]);
    double mean = tot / static_cast<double>(n);
    float inv = static_cast<float>(1.0 / sqrt(mean + static_cast<double>(eps)));
    for (uint32_t i = threadIdx.x * 4; i < n; i += 1024) {
        float4 v = *reinterpret_cast<const float4*>(xr + i);
        float4 g = *reinterpret_cast<const float4*>(w + i);
        float4 o;
        o.x = __fmul_rn(__fmul_rn(v.x, inv), g.x);
        o.y = __fmul_rn(__fmul_rn(v.y, inv), g.y);
        o.z = __fmul_rn(__fmul_rn(v.z, inv), g.z);
        o.w = __fmul_rn(__fmul_rn(v.w, inv), g.w);
        *reinterpret_cast<float4*>(yr + i) = o;
        if (QUANT) {
            // n % 32 == 0 and i advances in float4 steps: the 8 lanes of a block stay together
            float sc;
            uint32_t packed = q8_quantize_quad(o, sc);
            uint64_t e = static_cast<uint64_t>(blockIdx.x) * n + i;
            float ssum = bsum ? q8_block_scaled_sum(packed, sc) : 0.0f;
            reinterpret_cast<uint32_t*>(quants)[e >> 2] = packed;
            if ((threadIdx.x & 7) == 0) {
                scales[e >> 5] = sc;
                if (bsum) bsum[e >> 5] = ssum;
            }
        }
    }
}
template <bool QUANT>
static __global__ __launch_bounds__(256) void rmsnorm_kernel(const float* __restrict__ x, const float* __restrict__ w,
                                                      uint32_t n, float eps, float* __restrict__ y,
                                                      float* __restrict__ scales, int8_t* __restrict__ quants,
                                                      float* __restrict__ bsum) {
    rmsnorm_body<QUANT>(x, w, n, eps, y, scales, quants, bsum);
}
// The same over rows whose split-K partial sums are still pending (pd.x_out == x): one launch instead of the
// reduction and the norm.
static __global__ __launch_bounds__(256) void rmsnorm_pending_kernel(const float* x, const float* __restrict__ w, uint32_t n,
                                                                     float eps, float* __restrict__ y,
                                                                     float* __restrict__ scales, int8_t* __restrict__ quants,
                                                                     float* __restrict__ bsum, RowsPending pd) {
    rmsnorm_body<true, true>(x, w, n, eps, y, scales, quants, bsum, pd);
}

// Single-pass variant for the decode step (one row, n <= 16384): 1024 threads
// keep the row in registers, so the row is read once and the whole kernel is
// one memory round trip plus the reduction.  Same arithmetic as rmsnorm_kernel.
template <bool QUANT>
__device__ __forceinline__ void rmsnorm_row_body(const float* __restrict__ x, const float* __restrict__ w, uint32_t n, float eps,
                                                 float* __restrict__ y, float* __restrict__ scales, int8_t* __restrict__ quants,
                                                 double* part /* LDS, 16 */) {
    float4 v[4], g[4];
    double s = 0.0;
#pragma unroll
    for (int it = 0; it < 4; ++it) {
        uint32_t i = threadIdx.x * 4 + 4096 * it;
        if (i < n) {
            v[it] = *reinterpret_cast<const float4*>(x + i);
            g[it] = *reinterpret_cast<const float4*>(w + i);
            s += static_cast<double>(v[it].x) * v[it].x;
            s += static_cast<double>(v[it].y) * v[it].y;
            s += static_cast<double>(v[it].z) * v[it].z;
            s += static_cast<double>(v[it].w) * v[it].w;
        }
    }
    s = wave_sum_f64(s);
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = s;
    __syncthreads();
    double tot = 0.0;
#pragma unroll
    for (int i = 0; i < 16; ++i) tot += part[i];
    float inv = static_cast<float>(1.0 / sqrt(tot / static_cast<double>(n) + static_cast<double>(eps)));
#pragma unroll
    for (int it = 0; it < 4; ++it) {
        uint32_t i = threadIdx.x * 4 + 4096 * it;
        if (i < n) {
            float4 o;
            o.x = __fmul_rn(__fmul_rn(v[it].x, inv), g[it].x);
            o.y = __fmul_rn(__fmul_rn(v[it].y, inv), g[it].y);
            o.z = __fmul_rn(__fmul_rn(v[it].z, inv), g[it].z);
            o.w = __fmul_rn(__fmul_rn(v[it].w, inv), g[it].w);
            *reinterpret_cast<float4*>(y + i) = o;
            if (QUANT) {
                float sc;
                uint32_t packed = q8_quantize_quad(o, sc);
                reinterpret_cast<uint32_t*>(quants)[i >> 2] = packed;
                if ((threadIdx.x & 7) == 0) scales[i >> 5] = sc;
            }
        }
    }
}
template <bool QUANT>
static __global__ __launch_bounds__(1024) void rmsnorm_row_kernel(const float* __restrict__ x, const float* __restrict__ w,
                                                                  uint32_t n, float eps, float* __restrict__ y,
                                                                  float* __restrict__ scales, int8_t* __restrict__ quants) {
    __shared__ double part[16];
    rmsnorm_row_body<QUANT>(x, w, n, eps, y, scales, quants, part);
}

// ---------------------------------------------------------------------------
// RoPE on q and k in place + append k, v to the head-major KV cache.
// cos/sin come from a host-built table [max_seq][head_dim/2] computed with the
// same libm calls and the same iterated f32 theta as the CPU path
// (cera/src/backend/cpu.rs:5031-5045 NEOX, :5161-5180 NORM), so rotated values
// are bit-identical to it.  grid = n_heads + 2*n_kv_heads blocks of head_dim/2
// threads: blocks [0, n_heads) rotate q; the next n_kv_heads rotate k and
// store it; the last n_kv_heads copy v.
// KV cache layout: [kv_head][max_seq][head_dim] f32.
// Split-K partial sums of q, k or v that this kernel adds up itself instead of a reduction launch in front
// of it: value e = sum_z part[z * stride + e] in that order (n_split = 0: the rows are complete as they are).
struct RopePending {
    const float* part;
    uint32_t n_split;
    uint64_t stride;
};
__device__ __forceinline__ float rope_pending_ld(const float* rows, const RopePending& pd, uint64_t e) {
    if (pd.n_split == 0) return rows[e];
    float s = pd.part[e];
    for (uint32_t z = 1; z < pd.n_split; ++z) s += pd.part[z * pd.stride + e];
    return s;
}
template <typename KV>
__device__ __forceinline__ void rope_kv_body(float* __restrict__ q, float* __restrict__ k, const float* v,
                               const float* __restrict__ cs_table, const uint32_t* __restrict__ pos_ptr,
                               uint32_t n_heads, uint32_t n_kv_heads, uint32_t head_dim, uint32_t rope_type,
                               KV* __restrict__ k_cache, KV* __restrict__ v_cache, uint32_t max_seq,
                               RopePending pq = RopePending{}, RopePending pk = RopePending{}, RopePending pv = RopePending{}) {
    // grid.y = tokens of a prefill batch: token t sits at position *pos_ptr + t and its
    // q/k/v rows follow each other ([n][n_heads*head_dim], [n][n_kv_heads*head_dim])
    const uint32_t pos = *pos_ptr + blockIdx.y;
    const uint64_t q_row = static_cast<uint64_t>(blockIdx.y) * n_heads * head_dim, kv_row = static_cast<uint64_t>(blockIdx.y) * n_kv_heads * head_dim;
    const uint32_t half = head_dim / 2, i = threadIdx.x, b = blockIdx.x;
    if (b < n_heads + n_kv_heads) {
        const bool is_q = b < n_heads;
        float* const rows = is_q ? q : k;
        const uint64_t at = is_q ? q_row + b * head_dim : kv_row + (b - n_heads) * head_dim;
        float* head = rows + at;
        float2 cs = reinterpret_cast<const float2*>(cs_table)[static_cast<uint64_t>(pos) * half + i];
        uint32_t i0 = rope_type == 1 ? 2 * i : i, i1 = rope_type == 1 ? 2 * i + 1 : i + half;
        const RopePending& pd = is_q ? pq : pk;
        float x0 = rope_pending_ld(rows, pd, at + i0), x1 = rope_pending_ld(rows, pd, at + i1);
        float r0 = __fsub_rn(__fmul_rn(x0, cs.x), __fmul_rn(x1, cs.y));
        float r1 = __fadd_rn(__fmul_rn(x0, cs.y), __fmul_rn(x1, cs.x));
        head[i0] = r0;
        head[i1] = r1;
        if (b >= n_heads && k_cache) {
            KV* dst = k_cache + (static_cast<uint64_t>(b - n_heads) * max_seq + pos) * head_dim;
            dst[i0] = static_cast<KV>(r0);   // half cache: round to nearest even
            dst[i1] = static_cast<KV>(r1);
        }
    } else if (v_cache) {
        uint32_t h = b - n_heads - n_kv_heads;
        KV* dst = v_cache + (static_cast<uint64_t>(h) * max_seq + pos) * head_dim;
        dst[2 * i] = static_cast<KV>(rope_pending_ld(v, pv, kv_row + h * head_dim + 2 * i));
        dst[2 * i + 1] = static_cast<KV>(rope_pending_ld(v, pv, kv_row + h * head_dim + 2 * i + 1));
    }
}
template <typename KV>
static __global__ void rope_kv_kernel(float* __restrict__ q, float* __restrict__ k, const float* v,
                               const float* __restrict__ cs_table, const uint32_t* __restrict__ pos_ptr,
                               uint32_t n_heads, uint32_t n_kv_heads, uint32_t head_dim, uint32_t rope_type,
                               KV* __restrict__ k_cache, KV* __restrict__ v_cache, uint32_t max_seq) {
    rope_kv_body<KV>(q, k, v, cs_table, pos_ptr, n_heads, n_kv_heads, head_dim, rope_type, k_cache, v_cache, max_seq);
}
// The same over q / k / v rows whose split-K partial sums are still pending.
template <typename KV>
static __global__ void rope_kv_pending_kernel(float* __restrict__ q, float* __restrict__ k, const float* v,
                               const float* __restrict__ cs_table, const uint32_t* __restrict__ pos_ptr,
                               uint32_t n_heads, uint32_t n_kv_heads, uint32_t head_dim, uint32_t rope_type,
                               KV* __restrict__ k_cache, KV* __restrict__ v_cache, uint32_t max_seq,
                               RopePending pq, RopePending pk, RopePending pv) {
    rope_kv_body<KV>(q, k, v, cs_table, pos_ptr, n_heads, n_kv_heads, head_dim, rope_type, k_cache, v_cache, max_seq, pq, pk, pv);
}

// n_keep context shift (cera/src/kv_cache.rs:1091-1310): rows [src_row, src_row + n_rows) of every
// kv head move to [dst_row, ...) of `dst` (the cache itself when the two ranges do not overlap,
// a staging buffer otherwise), and K rows are rotated on the way by the constant delta rotation
// R(-shift) -- `delta_cs` holds its head_dim/2 (cos, sin) pairs, built on the host with the
// reference's recurrence (cera/src/backend/cpu.rs:5065-5086 NEOX, :5145-5180 NORM); null = plain
// copy (V, and the copy back from staging).  HD / 8 threads per row, each owning float4 j and
// float4 j + HD / 8 (its NEOX partner).  grid = (ceil(n_rows * HD / 8 / 256), n_kv_heads).
template <typename KV, int HD>
__device__ __forceinline__ void kv_shift_body(const KV* __restrict__ src, KV* __restrict__ dst,
                                                              uint32_t src_row, uint32_t dst_row, uint32_t n_rows,
                                                              uint64_t src_head_stride, uint64_t dst_head_stride,
                                                              const float* __restrict__ delta_cs, uint32_t rope_type) {
    constexpr uint32_t TPR = HD / 8;
    const uint32_t gi = blockIdx.x * 256 + threadIdx.x, t = gi / TPR, j = gi % TPR;   // TPR need not divide 256
    if (t >= n_rows) return;
    const KV* sp = src + blockIdx.y * src_head_stride + static_cast<uint64_t>(src_row + t) * HD;
    KV* dp = dst + blockIdx.y * dst_head_stride + static_cast<uint64_t>(dst_row + t) * HD;
    // a half cache is widened, rotated in f32 and narrowed again (cera/src/kv_cache.rs:1196-1230)
    float4 a = KvOps<KV>::ld4(sp, j), b = KvOps<KV>::ld4(sp, j + TPR);
    if (delta_cs) {
        const float4* cs = reinterpret_cast<const float4*>(delta_cs);
        if (rope_type == 1) {   // NORM: pairs (2i, 2i+1): pair i uses cs[i]; float4 j holds pairs 2j, 2j+1
            const float4 ca = cs[j], cb = cs[j + TPR];
            float4 r;
            r.x = __fsub_rn(__fmul_rn(a.x, ca.x), __fmul_rn(a.y, ca.y));
            r.y = __fadd_rn(__fmul_rn(a.x, ca.y), __fmul_rn(a.y, ca.x));
            r.z = __fsub_rn(__fmul_rn(a.z, ca.z), __fmul_rn(a.w, ca.w));
            r.w = __fadd_rn(__fmul_rn(a.z, ca.w), __fmul_rn(a.w, ca.z));
            a = r;
            r.x = __fsub_rn(__fmul_rn(b.x, cb.x), __fmul_rn(b.y, cb.y));
            r.y = __fadd_rn(__fmul_rn(b.x, cb.y), __fmul_rn(b.y, cb.x));
            r.z = __fsub_rn(__fmul_rn(b.z, cb.z), __fmul_rn(b.w, cb.w));
            r.w = __fadd_rn(__fmul_rn(b.z, cb.w), __fmul_rn(b.w, cb.z));
            b = r;
        } else {                // NEOX: pairs (i, i + HD/2): element 4j + e of a with the same of b, cs[4j + e]
            const float4 c01 = cs[2 * j], c23 = cs[2 * j + 1];
            float4 ra, rb;
            ra.x = __fsub_rn(__fmul_rn(a.x, c01.x), __fmul_rn(b.x, c01.y));
            rb.x = __fadd_rn(__fmul_rn(a.x, c01.y), __fmul_rn(b.x, c01.x));
            ra.y = __fsub_rn(__fmul_rn(a.y, c01.z), __fmul_rn(b.y, c01.w));
            rb.y = __fadd_rn(__fmul_rn(a.y, c01.w), __fmul_rn(b.y, c01.z));
            ra.z = __fsub_rn(__fmul_rn(a.z, c23.x), __fmul_rn(b.z, c23.y));
            rb.z = __fadd_rn(__fmul_rn(a.z, c23.y), __fmul_rn(b.z, c23.x));
            ra.w = __fsub_rn(__fmul_rn(a.w, c23.z), __fmul_rn(b.w, c23.w));
            rb.w = __fadd_rn(__fmul_rn(a.w, c23.w), __fmul_rn(b.w, c23.z));
            a = ra; b = rb;
        }
    }
    KvOps<KV>::st4(dp, j, a);
    KvOps<KV>::st4(dp, j + TPR, b);
}
template <typename KV, int HD>
static __global__ __launch_bounds__(256) void kv_shift_kernel(const KV* __restrict__ src, KV* __restrict__ dst,
                                                              uint32_t src_row, uint32_t dst_row, uint32_t n_rows,
                                                              uint64_t src_head_stride, uint64_t dst_head_stride,
                                                              const float* __restrict__ delta_cs, uint32_t rope_type) {
    kv_shift_body<KV, HD>(src, dst, src_row, dst_row, n_rows, src_head_stride, dst_head_stride, delta_cs, rope_type);
}

// out = a + b (cera/src/backend/cpu.rs:5223-5228), optional scale on b first.
__device__ __forceinline__ void add_body(const float* __restrict__ a, const float* __restrict__ b, float bscale, uint32_t n,
                           float* __restrict__ out) {
    uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    float t = bscale != 1.0f ? __fmul_rn(b[i], bscale) : b[i];
    out[i] = __fadd_rn(a[i], t);
}
static __global__ void add_kernel(const float* __restrict__ a, const float* __restrict__ b, float bscale, uint32_t n,
                           float* __restrict__ out) {
    add_body(a, b, bscale, n, out);
}

// bias add in place: x[i] += b[i]
__device__ __forceinline__ void bias_body(float* __restrict__ x, const float* __restrict__ b, uint32_t n) {
    uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) x[i] = __fadd_rn(x[i], b[i]);
}
static __global__ void bias_kernel(float* __restrict__ x, const float* __restrict__ b, uint32_t n) {
    bias_body(x, b, n);
}
__device__ __forceinline__ void scale_body(float* __restrict__ x, float s, uint32_t n) {
    uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) x[i] = __fmul_rn(x[i], s);
}
static __global__ void scale_kernel(float* __restrict__ x, float s, uint32_t n) {
    scale_body(x, s, n);
}

// SiLU(gate)*up (cera/src/backend/cpu.rs:2570-2575) with optional Q8_0
// quantisation of the result (the activation of the down projection).
template <bool QUANT>
__device__ __forceinline__ void silu_mul_body(const float* __restrict__ gate, const float* __restrict__ up,
                                                       uint64_t n, float* __restrict__ out,
                                                       float* __restrict__ scales, int8_t* __restrict__ quants,
                                                       float* __restrict__ bsum) {
    uint64_t t = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    bool live = 4 * t < n;
    float4 g = live ? reinterpret_cast<const float4*>(gate)[t] : make_float4(0, 0, 0, 0);
    float4 u = live ? reinterpret_cast<const float4*>(up)[t] : make_float4(0, 0, 0, 0);
    float4 o;
    o.x = __fmul_rn(__fdiv_rn(g.x, __fadd_rn(1.0f, cera_expf(-g.x))), u.x);
    o.y = __fmul_rn(__fdiv_rn(g.y, __fadd_rn(1.0f, cera_expf(-g.y))), u.y);
    o.z = __fmul_rn(__fdiv_rn(g.z, __fadd_rn(1.0f, cera_expf(-g.z))), u.z);
    o.w = __fmul_rn(__fdiv_rn(g.w, __fadd_rn(1.0f, cera_expf(-g.w))), u.w);
    if (QUANT) {
        float sc;
        uint32_t packed = q8_quantize_quad(o, sc);
        float ssum = bsum ? q8_block_scaled_sum(packed, sc) : 0.0f;
        if (live) {
            reinterpret_cast<uint32_t*>(quants)[t] = packed;
            if ((t & 7) == 0) {
                scales[t >> 3] = sc;
                if (bsum) bsum[t >> 3] = ssum;
            }
        }
    }
    if (live && out) reinterpret_cast<float4*>(out)[t] = o;
}
template <bool QUANT>
static __global__ __launch_bounds__(256) void silu_mul_kernel(const float* __restrict__ gate, const float* __restrict__ up,
                                                       uint64_t n, float* __restrict__ out,
                                                       float* __restrict__ scales, int8_t* __restrict__ quants,
                                                       float* __restrict__ bsum) {
    silu_mul_body<QUANT>(gate, up, n, out, scales, quants, bsum);
}

// ---------------------------------------------------------------------------
// argmax (cera/src/sampler.rs:20-30): strict >, lowest index on ties, NaN never
// wins, index 0 when nothing beats -inf.  Two stages: ARGMAX_PARTS workgroups each
// scan a contiguous slice keeping (best value, lowest index) and leave one
// candidate; a single workgroup merges the candidates with the same tie rule.
#define ARGMAX_PARTS 256
__device__ __forceinline__ void argmax_merge(float& bv, uint32_t& bi, float ov, uint32_t oi) {
    if (ov > bv || (ov == bv && oi < bi)) { bv = ov; bi = oi; }
}
// reduces the workgroup's (bv, bi) candidates into thread 0
__device__ __forceinline__ void argmax_block_reduce(float& bv, uint32_t& bi, float* sv, uint32_t* si) {
    for (int off = 32; off > 0; off >>= 1) {
        float ov = __shfl_xor(bv, off, 64);
        uint32_t oi = __shfl_xor(bi, off, 64);
        argmax_merge(bv, bi, ov, oi);
    }
    if ((threadIdx.x & 63) == 0) { sv[threadIdx.x >> 6] = bv; si[threadIdx.x >> 6] = bi; }
    __syncthreads();
    if (threadIdx.x == 0)
        for (uint32_t w = 1; w < blockDim.x / 64; ++w) argmax_merge(bv, bi, sv[w], si[w]);
}
__device__ __forceinline__ void argmax_partial_body(const float* __restrict__ x, uint32_t n,
                                                             float* __restrict__ pv, uint32_t* __restrict__ pi) {
    __shared__ float sv[4];
    __shared__ uint32_t si[4];
    const uint32_t chunk = (n + gridDim.x - 1) / gridDim.x;
    const uint32_t lo = blockIdx.x * chunk, hi = min(n, lo + chunk);
    float bv = -__builtin_inff();
    uint32_t bi = 0xFFFFFFFFu;  // "no candidate yet": loses every tie
    for (uint32_t i = lo + threadIdx.x; i < hi; i += 256) {
        float v = x[i];
        if (v > bv) { bv = v; bi = i; }
    }
    argmax_block_reduce(bv, bi, sv, si);
    if (threadIdx.x == 0) { pv[blockIdx.x] = bv; pi[blockIdx.x] = bi; }
}
static __global__ __launch_bounds__(256) void argmax_partial_kernel(const float* __restrict__ x, uint32_t n,
                                                             float* __restrict__ pv, uint32_t* __restrict__ pi) {
    argmax_partial_body(x, n, pv, pi);
}
// out2 (nullable): a second place for the index -- host memory the device can write, so that the
// greedy step needs no copy launch after this one
__device__ __forceinline__ void argmax_final_body(const float* __restrict__ pv, const uint32_t* __restrict__ pi,
                                                           uint32_t np, uint32_t* __restrict__ out, uint32_t* __restrict__ out2) {
    __shared__ float sv[4];
    __shared__ uint32_t si[4];
    float bv = -__builtin_inff();
    uint32_t bi = 0xFFFFFFFFu;
    for (uint32_t i = threadIdx.x; i < np; i += 256) argmax_merge(bv, bi, pv[i], pi[i]);
    argmax_block_reduce(bv, bi, sv, si);
    if (threadIdx.x == 0) {
        const uint32_t v = bi == 0xFFFFFFFFu ? 0u : bi;
        *out = v;
        if (out2) *out2 = v;
    }
}
static __global__ __launch_bounds__(256) void argmax_final_kernel(const float* __restrict__ pv, const uint32_t* __restrict__ pi,
                                                           uint32_t np, uint32_t* __restrict__ out, uint32_t* __restrict__ out2) {
    argmax_final_body(pv, pi, np, out, out2);
}
