// GQA flash-decode attention for one new query token, split-K over context.
//
// Semantics (cera/src/model/transformer.rs:1164-1305, cera/src/backend/cpu.rs:
// 3222-3363, 2617-2633): per query head h, s[t] = (q_h . K[t]) * scale over all
// cached positions of kv head h / group, p = softmax(s), out_h = sum_t p[t] V[t].
// The CPU computes a global max and a single softmax; this kernel computes the
// same quantity with the online-softmax recurrence over chunks of 64 positions
// and merges partial (max, sum, acc) triples, which agrees to f32 rounding.
//
// KV cache layout in HBM: [kv_head][max_seq][head_dim] f32 (head-major), so a
// wavefront streams one contiguous region.  head_dim is 128 and the group
// size G = n_heads / n_kv_heads is a template parameter: all G query heads of
// a kv head are served by one pass over its K/V (4x fewer bytes than per-head
// passes for Llama-3's 32/8 heads).
//
// Work split: part = one wavefront = `chunks_per_part` chunks of 64 positions.
// Eight lanes share a position (16 values each: of an f32 row four float4 spaced
// 128 B apart, of a half row two 16-byte runs spaced 128 B apart, so every load
// instruction covers whole 128-byte lines); a wavefront
// covers 8 positions per step and 64 per chunk.  The P.V accumulation keeps
// positions lane-local (lane group g accumulates positions == g mod 8), so the
// only cross-lane traffic is the 3-step reduction of the q.k partials and one
// reduction at the end of the part.
#pragma once
#include "common.hip.h"
#include "attn_types.h"
#include "quantize.hip.h"

#define ATTN_MAX_PARTS 1024  // the merge kernel keeps one weight per part in LDS
#define ATTN_MERGE_PF 16      // parts per lane group the merge kernel requests per round trip (x8 groups: 128 parts, every short-context split)

struct AttnPart {  // per (part, query head): running max, sum and unnormalised output
    float m, l;
};

// Which columns of a head_dim-wide row a lane of an 8-lane position group holds, and how it loads
// them.  A lane keeps NQ = head_dim / 32 register quads; quad c is float4 column col4(j, c).  The
// mapping is chosen per (element type, head_dim) so that loads are as wide as possible, the 8
// lanes of a load cover whole 128-byte lines, and the NEOX partner of quad c (head_dim / 2
// columns on) is quad c + NQ / 2 of the same lane.
template <typename KV, int HD> struct AttnLay {   // f32 rows, and half rows of 64
    static constexpr int NQ = HD / 32;
    __device__ static __forceinline__ uint32_t col4(uint32_t j, int c) { return j + 8 * c; }
    template <bool NT = false>
    __device__ static __forceinline__ void ld(const KV* row, uint32_t j, float4 (&v)[NQ]) {
#pragma unroll
        for (int c = 0; c < NQ; ++c) v[c] = NT ? KvOps<KV>::ld4nt(row, j + 8 * c) : KvOps<KV>::ld4(row, j + 8 * c);
    }
};
template <> struct AttnLay<kv_half, 128> {         // two 16-byte loads per row: quads 2c', 2c'+1 together
    static constexpr int NQ = 4;
    __device__ static __forceinline__ uint32_t col4(uint32_t j, int c) { return 2 * (j + 8 * (c >> 1)) + (c & 1); }
    template <bool NT = false>
    __device__ static __forceinline__ void ld(const kv_half* row, uint32_t j, float4 (&v)[4]) {
#pragma unroll
        for (int cc = 0; cc < 2; ++cc) {
            const uint4 r = NT ? ld_u128_nt(reinterpret_cast<const uint4*>(row) + j + 8 * cc) : reinterpret_cast<const uint4*>(row)[j + 8 * cc];
            v[2 * cc] = KvOps<kv_half>::cvt4(r.x, r.y);
            v[2 * cc + 1] = KvOps<kv_half>::cvt4(r.z, r.w);
        }
    }
};

// S = steps of 8 positions per chunk.  Short contexts use small chunks so that
// every wavefront has a single memory round trip (all its K and V loads in
// flight at once) and there are enough wavefronts to cover the chip; long
// contexts use 64-position chunks to amortise the softmax bookkeeping.
// RoPE of the values a lane holds of one head (register quad c is float4 column Lay::col4(j, c)),
// same arithmetic as rope_kv_kernel.  The lane's (cos, sin) values are loaded once
// (attn_rope_load: NQ float4 of the position's head_dim / 2 pairs) and applied to as many heads
// as needed.  NORM rotates pairs (2i, 2i+1) = (x, y) and (z, w) of each float4 with the float4 of
// the table at the same column; NEOX rotates pairs (i, i + head_dim / 2) = quad c with quad
// c + NQ / 2, whose four pairs take two float4 of the table.
template <typename Lay>
__device__ __forceinline__ void attn_rope_load(float4 (&cs)[Lay::NQ], const float* __restrict__ rope_row, uint32_t j,
                                               uint32_t rope_type) {
#pragma unroll
    for (int i = 0; i < Lay::NQ; ++i) {
        const uint32_t idx = rope_type == 1 ? Lay::col4(j, i) : 2 * Lay::col4(j, i >> 1) + (i & 1);
        cs[i] = reinterpret_cast<const float4*>(rope_row)[idx];
    }
}
template <typename Lay>
__device__ __forceinline__ void attn_rope_apply(float4 (&x)[Lay::NQ], const float4 (&cs)[Lay::NQ], uint32_t rope_type) {
    constexpr int NQ = Lay::NQ;
    if (rope_type == 1) {
#pragma unroll
        for (int c = 0; c < NQ; ++c) {
            const float4 v = x[c], t = cs[c];
            x[c].x = __fsub_rn(__fmul_rn(v.x, t.x), __fmul_rn(v.y, t.y));
            x[c].y = __fadd_rn(__fmul_rn(v.x, t.y), __fmul_rn(v.y, t.x));
            x[c].z = __fsub_rn(__fmul_rn(v.z, t.z), __fmul_rn(v.w, t.w));
            x[c].w = __fadd_rn(__fmul_rn(v.z, t.w), __fmul_rn(v.w, t.z));
        }
    } else {
        constexpr int H2 = NQ / 2;
#pragma unroll
        for (int c = 0; c < H2; ++c) {
            const float4 c01 = cs[2 * c], c23 = cs[2 * c + 1];
            const float4 a = x[c], b = x[c + H2];
            x[c].x = __fsub_rn(__fmul_rn(a.x, c01.x), __fmul_rn(b.x, c01.y));
            x[c + H2].x = __fadd_rn(__fmul_rn(a.x, c01.y), __fmul_rn(b.x, c01.x));
            x[c].y = __fsub_rn(__fmul_rn(a.y, c01.z), __fmul_rn(b.y, c01.w));
            x[c + H2].y = __fadd_rn(__fmul_rn(a.y, c01.w), __fmul_rn(b.y, c01.z));
            x[c].z = __fsub_rn(__fmul_rn(a.z, c23.x), __fmul_rn(b.z, c23.y));
            x[c + H2].z = __fadd_rn(__fmul_rn(a.z, c23.y), __fmul_rn(b.z, c23.x));
            x[c].w = __fsub_rn(__fmul_rn(a.w, c23.z), __fmul_rn(b.w, c23.w));
            x[c + H2].w = __fadd_rn(__fmul_rn(a.w, c23.w), __fmul_rn(b.w, c23.z));
        }
    }
}

// The token's own K or V row, not in the cache yet: its loads (raw projection output, this lane's
// columns) are issued first; once they are in, the row is rotated (K only), narrowed like a
// cached row and stored into the cache if this caller owns the append.
template <typename KV, int HD>
__device__ __forceinline__ void attn_new_row_load(float4 (&r)[HD / 32], const float* fresh, uint32_t kvh, uint32_t j) {
    using Lay = AttnLay<KV, HD>;
    const float4* p = reinterpret_cast<const float4*>(fresh + kvh * HD);
#pragma unroll
    for (int c = 0; c < Lay::NQ; ++c) r[c] = p[Lay::col4(j, c)];
}
template <bool ROTATE, typename KV, int HD>
__device__ __forceinline__ void attn_new_row_finish(float4 (&r)[HD / 32], const float4 (&cs)[HD / 32], uint32_t rope_type,
                                                    void* cache, uint64_t row, uint32_t j, bool store) {
    using Lay = AttnLay<KV, HD>;
    if (ROTATE) attn_rope_apply<Lay>(r, cs, rope_type);
#pragma unroll
    for (int c = 0; c < Lay::NQ; ++c) r[c] = KvOps<KV>::rnd4(r[c]);
    if (store) {
        KV* dst = static_cast<KV*>(cache) + row * HD;
#pragma unroll
        for (int c = 0; c < Lay::NQ; ++c) KvOps<KV>::st4(dst, Lay::col4(j, c), r[c]);
    }
}

// One wavefront's share of the keys: chunks of 8*S positions at t_begin, t_begin + t_step, ...
// below t_end, for the G query heads of one kv head.  Returns the online-softmax state with
// the eight position groups folded: the wavefront-wide m and l in every lane, and of the
// unnormalised output each lane's head_dim / 64 consecutive columns from attn_fold_column.  `q` points at the first of the G heads; `write_new` says whether
// this caller stores the new position's K/V row into the cache (NEWKV only).
template <int G, int S, bool NEWKV, typename KV, int HD, bool NT>
__device__ __forceinline__ void attn_decode_range(const float* __restrict__ q, const KV* __restrict__ kbase,
                                                  const KV* __restrict__ vbase, uint32_t kvh, uint32_t max_seq,
                                                  uint32_t seq_len, uint32_t t_begin, uint32_t t_end, uint32_t t_step,
                                                  float scale, const AttnNewKV& nk, bool write_new, uint32_t lane,
                                                  float (&out)[G][HD / 64], float (&m)[G], float (&l)[G]) {
    using Lay = AttnLay<KV, HD>;
    constexpr int NQ = Lay::NQ;
    const uint32_t j = lane & 7, pg = lane >> 3;  // float4 column group, position group
    float4 acc[G][NQ];

    // NEWKV: the last position's K/V are not in the cache yet.  The chunk loop below only walks
    // cached positions, so it is the same straight-line code with or without NEWKV; the wavefront
    // whose range holds the new position takes it as one extra step afterwards.
    const uint32_t new_pos = seq_len - 1;
    const bool own_new = NEWKV && t_begin <= new_pos && new_pos < t_end;   // wavefront-uniform
    if (NEWKV) t_end = min(t_end, new_pos);
    constexpr bool PREFETCH_V = S <= 2;  // small chunks: V loads issued together with K
    // Short chunks are latency-bound, so their first chunk's K/V loads go out before anything
    // else: one memory round trip covers the cache rows, q and the RoPE row together.
    float4 kbuf[PREFETCH_V ? S : 1][NQ], vpre[PREFETCH_V ? S : 1][NQ];
    // a lane past t_end re-reads the range's first position and gets a dead score
    auto issue_chunk = [&](uint32_t t0) {
#pragma unroll
        for (int s = 0; s < S; ++s) {
            const uint32_t t = t0 + 8 * s + pg, tt = t < t_end ? t : t_begin;
            Lay::ld(kbase + static_cast<uint64_t>(tt) * HD, j, kbuf[s]);
            Lay::ld(vbase + static_cast<uint64_t>(tt) * HD, j, vpre[s]);
        }
    };
    if (PREFETCH_V && t_begin < t_end) issue_chunk(t_begin);
    float4 kn[NQ], vn[NQ];
    if (own_new) {
        attn_new_row_load<KV, HD>(kn, nk.k_new, kvh, j);
        attn_new_row_load<KV, HD>(vn, nk.v_new, kvh, j);
    }

    // this lane's 16 q values for each of the G heads, and its part of the position's RoPE row
    float4 qv[G][NQ], cs[NQ];
    if (NEWKV) attn_rope_load<Lay>(cs, nk.rope_row, j, nk.rope_type);
#pragma unroll
    for (int h = 0; h < G; ++h)
#pragma unroll
        for (int c = 0; c < NQ; ++c)
            qv[h][c] = reinterpret_cast<const float4*>(q + h * HD)[Lay::col4(j, c)];
    if (NEWKV) {
#pragma unroll
        for (int h = 0; h < G; ++h) attn_rope_apply<Lay>(qv[h], cs, nk.rope_type);
    }

#pragma unroll
    for (int h = 0; h < G; ++h) {
        m[h] = -__builtin_inff();
        l[h] = 0.0f;
#pragma unroll
        for (int c = 0; c < NQ; ++c) acc[h][c] = make_float4(0.f, 0.f, 0.f, 0.f);
    }

    for (uint32_t t0 = t_begin; t0 < t_end; t0 += t_step) {
        if (PREFETCH_V && t0 != t_begin) issue_chunk(t0);
        // ---- scores: step s covers positions t0 + 8s + pg
        float sc[G][S];
#pragma unroll
        for (int s = 0; s < S; ++s) {
            const uint32_t t = t0 + 8 * s + pg;
            const bool live = t < t_end;
            float4 kv[NQ];
            if (PREFETCH_V) {
#pragma unroll
                for (int c = 0; c < NQ; ++c) kv[c] = kbuf[s][c];
            } else {
                Lay::template ld<NT>(kbase + static_cast<uint64_t>(live ? t : t_begin) * HD, j, kv);
            }
#pragma unroll
            for (int h = 0; h < G; ++h) {
                float d = 0.0f;
#pragma unroll
                for (int c = 0; c < NQ; ++c) {
                    d = fmaf(qv[h][c].x, kv[c].x, d);
                    d = fmaf(qv[h][c].y, kv[c].y, d);
                    d = fmaf(qv[h][c].z, kv[c].z, d);
                    d = fmaf(qv[h][c].w, kv[c].w, d);
                }
                d += dpp_f<0xB1>(d);
                d += dpp_f<0x4E>(d);
                d += dpp_f<0x141>(d);
                sc[h][s] = live ? d * scale : -__builtin_inff();
            }
        }
        // ---- online softmax update per head
        float corr[G];
#pragma unroll
        for (int h = 0; h < G; ++h) {
            float mx = sc[h][0];
#pragma unroll
            for (int s = 1; s < S; ++s) mx = fmaxf(mx, sc[h][s]);
            mx = wave_max(mx);
            // short chunks (latency-bound, usually one per wavefront): nothing is accumulated yet on
            // the first one, so skip the rescale; long chunks keep straight-line code for the scheduler
            if (PREFETCH_V && t0 == t_begin) {
                m[h] = mx;
                continue;
            }
            float m_new = fmaxf(m[h], mx);
            corr[h] = cera_expf(m[h] - m_new);  // 0 on the first chunk (m = -inf)
            m[h] = m_new;
            l[h] *= corr[h];
#pragma unroll
            for (int c = 0; c < NQ; ++c) {
                acc[h][c].x *= corr[h]; acc[h][c].y *= corr[h];
                acc[h][c].z *= corr[h]; acc[h][c].w *= corr[h];
            }
        }
        // ---- P.V: this lane's positions, its 16 columns
#pragma unroll
        for (int s = 0; s < S; ++s) {
            float4 vv[NQ];
            if (PREFETCH_V) {
#pragma unroll
                for (int c = 0; c < NQ; ++c) vv[c] = vpre[s][c];
            } else {
                const uint32_t t = t0 + 8 * s + pg;
                Lay::template ld<NT>(vbase + static_cast<uint64_t>(t < t_end ? t : t_begin) * HD, j, vv);
            }
#pragma unroll
            for (int h = 0; h < G; ++h) {
                float p = cera_expf(sc[h][s] - m[h]);  // -inf score -> 0
                // all 8 lanes of a position add the same p; count it once (lane j == 0)
                l[h] += (j == 0) ? p : 0.0f;
#pragma unroll
                for (int c = 0; c < NQ; ++c) {
                    acc[h][c].x = fmaf(p, vv[c].x, acc[h][c].x);
                    acc[h][c].y = fmaf(p, vv[c].y, acc[h][c].y);
                    acc[h][c].z = fmaf(p, vv[c].z, acc[h][c].z);
                    acc[h][c].w = fmaf(p, vv[c].w, acc[h][c].w);
                }
            }
        }
    }

    // ---- the token's own position: every position group holds the same row, so the score is the
    // same in all lanes; group 0 alone accumulates it and (if this caller owns the append) stores
    // the row into the cache
    if (own_new) {
        const uint64_t row = static_cast<uint64_t>(kvh) * max_seq + new_pos;
        attn_new_row_finish<true, KV, HD>(kn, cs, nk.rope_type, nk.kc_w, row, j, write_new && pg == 0);
        attn_new_row_finish<false, KV, HD>(vn, cs, 0, nk.vc_w, row, j, write_new && pg == 0);
#pragma unroll
        for (int h = 0; h < G; ++h) {
            float d = 0.0f;
#pragma unroll
            for (int c = 0; c < NQ; ++c) {
                d = fmaf(qv[h][c].x, kn[c].x, d);
                d = fmaf(qv[h][c].y, kn[c].y, d);
                d = fmaf(qv[h][c].z, kn[c].z, d);
                d = fmaf(qv[h][c].w, kn[c].w, d);
            }
            d += dpp_f<0xB1>(d);
            d += dpp_f<0x4E>(d);
            d += dpp_f<0x141>(d);
            const float sn = d * scale;
            const float m_new = fmaxf(m[h], sn);
            const float corr = cera_expf(m[h] - m_new);   // 0 when nothing came before (m = -inf)
            m[h] = m_new;
            l[h] *= corr;
            const float p = pg == 0 ? cera_expf(sn - m_new) : 0.0f;
            l[h] += (j == 0) ? p : 0.0f;
#pragma unroll
            for (int c = 0; c < NQ; ++c) {
                acc[h][c].x = fmaf(p, vn[c].x, acc[h][c].x * corr);
                acc[h][c].y = fmaf(p, vn[c].y, acc[h][c].y * corr);
                acc[h][c].z = fmaf(p, vn[c].z, acc[h][c].z * corr);
                acc[h][c].w = fmaf(p, vn[c].w, acc[h][c].w * corr);
            }
        }
    }

    // ---- fold the 8 position groups (lanes differing in bits 3..5) together: a reduce-scatter.
    // Each exchange halves what a lane keeps (half its quads with the lane 32 away, half of those
    // with the lane 16 away, half of that with the lane 8 away), so a lane ends with
    // 4 * NQ / 8 consecutive floats of the sum: out[h][e], columns attn_fold_column(lane) + e.
    const bool b5 = lane & 32, b4 = lane & 16, b3 = lane & 8;
#pragma unroll
    for (int h = 0; h < G; ++h) {
        l[h] = wave_sum(l[h]);
        float v[4 * NQ];
#pragma unroll
        for (int c = 0; c < NQ; ++c) {
            v[4 * c] = acc[h][c].x; v[4 * c + 1] = acc[h][c].y; v[4 * c + 2] = acc[h][c].z; v[4 * c + 3] = acc[h][c].w;
        }
        constexpr int N1 = 2 * NQ, N2 = NQ, N3 = NQ / 2;
        float w1[N1], w2[N2];
#pragma unroll
        for (int i = 0; i < N1; ++i) {
            const float keep = b5 ? v[N1 + i] : v[i], send = b5 ? v[i] : v[N1 + i];
            w1[i] = keep + __shfl_xor(send, 32, 64);
        }
#pragma unroll
        for (int i = 0; i < N2; ++i) {
            const float keep = b4 ? w1[N2 + i] : w1[i], send = b4 ? w1[i] : w1[N2 + i];
            w2[i] = keep + __shfl_xor(send, 16, 64);
        }
#pragma unroll
        for (int i = 0; i < N3; ++i) {
            const float keep = b3 ? w2[N3 + i] : w2[i], send = b3 ? w2[i] : w2[N3 + i];
            out[h][i] = keep + __shfl_xor(send, 8, 64);
        }
    }
}

// First float column (of head_dim) of the NQ / 2 a lane holds after the fold above.
template <typename Lay>
__device__ __forceinline__ uint32_t attn_fold_column(uint32_t lane) {
    constexpr int NQ = Lay::NQ;
    const uint32_t j = lane & 7, b5 = (lane >> 5) & 1, b4 = (lane >> 4) & 1, b3 = (lane >> 3) & 1;
    // floats kept: index range [f0, f0 + NQ/2) of the lane's 4*NQ values, f0 = b5*2NQ + b4*NQ + b3*NQ/2
    const uint32_t f0 = b5 * 2 * NQ + b4 * NQ + b3 * (NQ / 2);
    return 4 * Lay::col4(j, f0 >> 2) + (f0 & 3);
}

// G = query heads one wavefront serves (all of a kv head's group, or -- short contexts, where the
// kernel is bound by a wavefront's own instruction stream, not by bytes -- half of it: grid.y is
// then n_kv * 2 and the two halves of a group run as separate wavefronts, re-reading the same few
// K/V rows from cache).  g_total = heads per kv head, the stride of the partials.
// NT: every K/V row is read once, by this wavefront only (one query, the group not split):
// non-temporal loads.
template <int G, int S, bool NEWKV, typename KV, int HD, bool NT = false>
__device__ __forceinline__ void attn_decode_partial_body(
    const float* __restrict__ q,       // [n_heads][128]
    const KV* __restrict__ kc,         // [n_kv][max_seq][128]
    const KV* __restrict__ vc,
    uint32_t seq_len, uint32_t max_seq, float scale, uint32_t chunks_per_part, uint32_t n_parts,
    uint32_t q_stride,                 // floats between consecutive queries (prefill batches queries on grid.z)
    uint32_t g_total,                  // query heads per kv head (a multiple of G)
    uint32_t n_kv, uint32_t n_queries,
    float* __restrict__ part_acc,      // [n_queries][n_kv][n_parts][g_total][128]
    float* __restrict__ part_ml,       // [n_queries][n_kv][n_parts][g_total][2]
    AttnNewKV nk) {
    const uint32_t lane = threadIdx.x & 63;
    // Workgroups are handed to the eight XCDs round-robin in launch order and every XCD has an L2 of
    // its own.  The workgroups that read the same K/V rows (the sub-groups of a kv head's query heads,
    // the queries of a small batch) therefore take launch indices 8 apart: same XCD, consecutive
    // there, so all but the first find the rows in that L2 whatever the number of parts is.
    // Launch index = (slot * reps + rep) * 8 + xcd, key-range group = slot * 8 + xcd; the launcher
    // (attn_launch_decode_g) rounds the groups up to whole eights.
    const uint32_t subs = g_total / G, reps = subs * n_queries;
    const uint32_t xcd = blockIdx.x & 7, t = blockIdx.x >> 3;
    const uint32_t group = (t / reps) * 8 + xcd, rep = t % reps;
    const uint32_t part_groups = (n_parts + 3) >> 2;
    if (group >= part_groups * n_kv) return;
    const uint32_t kvh = group / part_groups, sub = rep % subs, qi = rep / subs;
    const uint32_t part = (group % part_groups) * 4 + (threadIdx.x >> 6);
    if (part >= n_parts) return;
    // causal prefill: query qi sits at position seq_len - 1 + qi and sees seq_len + qi keys
    seq_len += qi;
    q += static_cast<uint64_t>(qi) * q_stride + (kvh * g_total + sub * G) * HD;
    using Lay = AttnLay<KV, HD>;
    constexpr int NQ = Lay::NQ;
    constexpr uint32_t CHUNK = 8 * S;
    const uint32_t t_begin = part * chunks_per_part * CHUNK;
    const uint32_t t_end = min(seq_len, t_begin + chunks_per_part * CHUNK);
    float out[G][NQ / 2];
    float m[G], l[G];
    // the first sub-group's wavefront appends the token's K/V rows to the cache
    attn_decode_range<G, S, NEWKV, KV, HD, NT>(q, kc + static_cast<uint64_t>(kvh) * max_seq * HD,
                                   vc + static_cast<uint64_t>(kvh) * max_seq * HD, kvh, max_seq, seq_len, t_begin,
                                   t_end, CHUNK, scale, nk, sub == 0, lane, out, m, l);
    const uint64_t base = ((static_cast<uint64_t>(qi) * n_kv + kvh) * n_parts + part) * g_total + sub * G;
    const uint32_t col = attn_fold_column<Lay>(lane);
#pragma unroll
    for (int h = 0; h < G; ++h) {
        float* dst = part_acc + (base + h) * HD + col;
        if (NQ == 4) *reinterpret_cast<float2*>(dst) = make_float2(out[h][0], out[h][NQ / 2 - 1]);
        else dst[0] = out[h][0];
        if (lane == 0) {
            part_ml[(base + h) * 2] = m[h];
            part_ml[(base + h) * 2 + 1] = l[h];
        }
    }
}
template <int G, int S, bool NEWKV, typename KV, int HD, bool NT = false>
__global__ __launch_bounds__(256) void attn_decode_partial_kernel(
    const float* __restrict__ q,       // [n_heads][128]
    const KV* __restrict__ kc,         // [n_kv][max_seq][128]
    const KV* __restrict__ vc,
    uint32_t seq_len, uint32_t max_seq, float scale, uint32_t chunks_per_part, uint32_t n_parts,
    uint32_t q_stride,                 // floats between consecutive queries (prefill batches queries on grid.z)
    uint32_t g_total,                  // query heads per kv head (a multiple of G)
    uint32_t n_kv, uint32_t n_queries,
    float* __restrict__ part_acc,      // [n_queries][n_kv][n_parts][g_total][128]
    float* __restrict__ part_ml,       // [n_queries][n_kv][n_parts][g_total][2]
    AttnNewKV nk) {
    attn_decode_partial_body<G, S, NEWKV, KV, HD, NT>(q, kc, vc, seq_len, max_seq, scale, chunks_per_part, n_parts, q_stride, g_total, n_kv, n_queries, part_acc, part_ml, nk);
}

// ---------------------------------------------------------------------------
// Causal attention for a batch of queries (prefill) on the f16 matrix cores, at f32
// accuracy.
//
// The decode kernel above reads the whole visible K/V range once per query; for a
// prompt of n tokens that is n passes over the cache.  Here one wavefront owns a
// block of 32 consecutive queries of one head and walks the keys in tiles of 32, so
// a K/V tile is read once per 32 queries.  Both contractions run as
// v_mfma_f32_32x32x16_f16 on operands split in two: every f32 value x is staged as
// the f16 pair (hi, lo), hi = x truncated to f16 and lo = (x - hi) truncated, so
// x = hi + lo up to 2^-21 |x|, and a product x.y is the three MFMAs hi.hi + hi.lo + lo.hi
// (each f16 product is exact in the f32 accumulator; the dropped lo.lo term is below
// 2^-22 |x.y|; the low parts of Q and K are carried times 2^11 and their two cross products
// collect in an accumulator of their own, so that they stay in f16's normal range and a
// large Q element cannot magnify a subnormal's absolute rounding).  That keeps the arithmetic class of the reference's f32 dot products
// (cera/src/backend/cpu.rs:4028-4241) at a fifth of the f32 MFMA's cycles.  A half
// cache has no low parts and takes two MFMAs per product.
//
//   S^T = K . Q^T   A = K tile (row = key; the lane of key `col` reads 8 consecutive
//                   dims of its half from LDS), B = the lane's query (registers, the
//                   same dims).  A lane ends up with 16 keys of ONE query, so the
//                   softmax reduction over keys is over registers plus one exchange
//                   between the wavefront halves.
//   O  += P . V     A = P straight from those registers: the lanes of half h hold keys
//                   8blk + 4h + r, and the MFMA over keys 16kk .. 16kk+15 takes its
//                   eight K slots of half h from blk = 2kk, 2kk+1.  B = the V tile,
//                   staged TRANSPOSED in LDS with the keys of each 16 in that slot order
//                   (position 8h + 4(blk&1) + r), so a lane reads its eight keys of one
//                   output column as one 16-byte word.
//
// Online softmax per key tile in the base-2 domain (v_exp_f32 on scores pre-multiplied by
// log2 e; the reference's polynomial expf agrees with it to a few ulp, far inside this
// kernel's tolerance) with an f64 running sum.  The key range is cut into parts of `part_keys`; a workgroup
// produces the (m, l, acc) partial of one (query block, head, part) in the layout
// the merge kernel below consumes, so long prompts spread over the chip and the
// merge (and its fused Q8_0 quantisation) is shared with the decode path.
// A workgroup is the G query heads of one KV head, one wavefront each: the K and V
// tiles are split and staged in LDS once, by all G wavefronts together, and every
// head of the group reads them from there.
// grid = (query blocks, KV heads, parts), 64 * G threads.
typedef float attn_v16f __attribute__((ext_vector_type(16)));
typedef _Float16 attn_v8h __attribute__((ext_vector_type(8)));
typedef _Float16 attn_v2h __attribute__((ext_vector_type(2)));
#define ATTN_PF_KLD(HD) ((HD) + 8)   // halves per LDS row of the K tile: 16-byte reads of 16 rows cover all banks
#define ATTN_PF_VTLD 40              // halves per LDS row of the transposed V tile (32 keys + 8 pad), same property

// (a, b) -> packed f16 high parts and packed f16 low parts.  SCALED: the low parts times 2^11,
// which keeps them in the f16 normal range whenever the high part is (an unscaled low part of a
// value below 1/8 is subnormal, i.e. absolute instead of relative precision: harmless against
// an operand of ordinary size, not against a very large one).
#define ATTN_LO_SCALE 2048.0f
template <bool SCALED>
__device__ __forceinline__ void attn_split2(float a, float b, uint32_t& hi, uint32_t& lo) {
    const attn_v2h h = __builtin_bit_cast(attn_v2h, __builtin_amdgcn_cvt_pkrtz(a, b));
    hi = __builtin_bit_cast(uint32_t, h);
    float ra = a - static_cast<float>(h[0]), rb = b - static_cast<float>(h[1]);
    if (SCALED) { ra *= ATTN_LO_SCALE; rb *= ATTN_LO_SCALE; }
    lo = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(ra, rb));
}
__device__ __forceinline__ attn_v16f attn_mfma(const uint4& a, const uint4& b, attn_v16f c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(attn_v8h, a), __builtin_bit_cast(attn_v8h, b), c, 0, 0, 0);
}

template <typename KV, int HD, int G>
__device__ __forceinline__ void attn_prefill_partial_body(
    const float* __restrict__ q,       // [n_queries][q_stride], rows 16-byte aligned
    const KV* __restrict__ kc,         // [n_kv][max_seq][128], already holding the batch's keys
    const KV* __restrict__ vc,
    uint32_t first_len,                // keys visible to query 0; query i sees first_len + i
    uint32_t n_queries, uint32_t max_seq, float scale, uint32_t part_keys, uint32_t n_parts, uint32_t q_stride,
    float* __restrict__ part_acc,      // [n_queries][n_kv][n_parts][G][128]
    float* __restrict__ part_ml) {     // [n_queries][n_kv][n_parts][G][2]
    constexpr bool LOW = sizeof(KV) == 4;   // an f32 cache has low parts, a half cache is its own high part
    constexpr int KLD = ATTN_PF_KLD(HD), VTLD = ATTN_PF_VTLD;
    constexpr int NJ = HD / 16;    // MFMA steps over the head dimension
    constexpr int NDT = HD / 32;   // 32-column output tiles
    constexpr int NT = 64 * G;     // threads
    // staging items per thread: K quads (32 keys x HD/4), V quad pairs (16 key pairs x HD/4)
    constexpr int K_ITEMS = 32 * (HD / 4), V_ITEMS = 16 * (HD / 4);
    constexpr int KI = (K_ITEMS + NT - 1) / NT, VI = (V_ITEMS + NT - 1) / NT;
    // the next tile's global loads stay in flight (in registers) while this one is multiplied,
    // where a thread's share of a tile is small enough to hold
    constexpr bool PREFETCH = KI + 2 * VI <= 10;
    __shared__ __attribute__((aligned(16))) _Float16 sKh[32 * KLD];
    __shared__ __attribute__((aligned(16))) _Float16 sKl[LOW ? 32 * KLD : 8];
    __shared__ __attribute__((aligned(16))) _Float16 sVh[HD * VTLD];
    __shared__ __attribute__((aligned(16))) _Float16 sVl[LOW ? HD * VTLD : 8];
    __shared__ __attribute__((aligned(16))) float sXall[G * 32];
    const uint32_t tid = threadIdx.x, lane = tid & 63, col = lane & 31, half = lane >> 5;
    const uint32_t kvh = blockIdx.y, hg = tid >> 6, head = kvh * G + hg, n_kv = gridDim.y;
    float* sX = sXall + 32 * hg;
    const uint32_t part = blockIdx.z;
    const uint32_t q0 = blockIdx.x * 32, qidx = q0 + col;
    const bool q_live = qidx < n_queries;
    const uint32_t my_len = first_len + qidx;                             // keys this lane's query sees
    const uint32_t block_len = first_len + min(n_queries, q0 + 32) - 1;   // ... and the block's last query
    const uint32_t key_lo = part * part_keys;
    const uint32_t key_hi = min(key_lo + part_keys, block_len);

    const KV* kbase = kc + static_cast<uint64_t>(kvh) * max_seq * HD;
    const KV* vbase = vc + static_cast<uint64_t>(kvh) * max_seq * HD;

    // this lane's query, split: step j holds dims 16j + 8half .. +7
    uint4 qh[NJ], ql[NJ];
    {
        const float* qp = q + static_cast<uint64_t>(min(qidx, n_queries - 1)) * q_stride + head * HD + 8 * half;
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
            const float4 a = *reinterpret_cast<const float4*>(qp + 16 * j), b = *reinterpret_cast<const float4*>(qp + 16 * j + 4);
            attn_split2<true>(a.x, a.y, qh[j].x, ql[j].x);
            attn_split2<true>(a.z, a.w, qh[j].y, ql[j].y);
            attn_split2<true>(b.x, b.y, qh[j].z, ql[j].z);
            attn_split2<true>(b.z, b.w, qh[j].w, ql[j].w);
        }
    }
    attn_v16f acc[NDT];
#pragma unroll
    for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[dt][e] = 0.0f;
    float m = -__builtin_inff();   // running maximum, base-2 domain
    double l = 0.0;
    const float scale2 = scale * 1.44269504088896340736f;

    // ---- staging.  K tile -> LDS by rows, an item is one key x one quad of dims.  V tile -> LDS
    // transposed: an item is two neighbouring keys (neighbours in slot order too) x one quad of
    // dims; consecutive lanes take consecutive key pairs, so the 4-byte stores of a wavefront fall
    // in different banks.  Keys past the part's end are zeros (their weights are zero too).
    float4 kreg[KI], v0reg[VI], v1reg[VI];
    auto fetch = [&](uint32_t k0) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < KI; ++i) {
            const uint32_t f = tid + NT * i, key = f / (HD / 4), c4 = f % (HD / 4);
            kreg[i] = make_float4(0.f, 0.f, 0.f, 0.f);
            if (f < K_ITEMS && k0 + key < key_hi) kreg[i] = KvOps<KV>::ld4(kbase + static_cast<uint64_t>(k0 + key) * HD, c4);
        }
#pragma unroll
        for (int i = 0; i < VI; ++i) {
            const uint32_t f = tid + NT * i, key = 2 * (f & 15), c4 = f >> 4;
            v0reg[i] = v1reg[i] = make_float4(0.f, 0.f, 0.f, 0.f);
            if (f < V_ITEMS && k0 + key < key_hi) v0reg[i] = KvOps<KV>::ld4(vbase + static_cast<uint64_t>(k0 + key) * HD, c4);
            if (f < V_ITEMS && k0 + key + 1 < key_hi) v1reg[i] = KvOps<KV>::ld4(vbase + static_cast<uint64_t>(k0 + key + 1) * HD, c4);
        }
    };
    auto stage = [&]() __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < KI; ++i) {
            const uint32_t f = tid + NT * i, key = f / (HD / 4), c4 = f % (HD / 4);
            uint2 hi, lo;
            attn_split2<true>(kreg[i].x, kreg[i].y, hi.x, lo.x);
            attn_split2<true>(kreg[i].z, kreg[i].w, hi.y, lo.y);
            if (f < K_ITEMS) {
                *reinterpret_cast<uint2*>(sKh + key * KLD + 4 * c4) = hi;
                if (LOW) *reinterpret_cast<uint2*>(sKl + key * KLD + 4 * c4) = lo;
            }
        }
#pragma unroll
        for (int i = 0; i < VI; ++i) {
            const uint32_t f = tid + NT * i, key = 2 * (f & 15), c4 = f >> 4;
            // slot of key: 16 (key / 16) + 8 h + 4 (blk & 1) + r  with  key % 16 = 8 (blk & 1) + 4 h + r
            const uint32_t slot = (key & 16) + ((key & 4) << 1) + ((key & 8) >> 1) + (key & 3);
            const float a[4] = {v0reg[i].x, v0reg[i].y, v0reg[i].z, v0reg[i].w};
            const float b[4] = {v1reg[i].x, v1reg[i].y, v1reg[i].z, v1reg[i].w};
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                uint32_t hi, lo;
                attn_split2<false>(a[e], b[e], hi, lo);
                if (f < V_ITEMS) {
                    *reinterpret_cast<uint32_t*>(sVh + (4 * c4 + e) * VTLD + slot) = hi;
                    if (LOW) *reinterpret_cast<uint32_t*>(sVl + (4 * c4 + e) * VTLD + slot) = lo;
                }
            }
        }
    };

    if (PREFETCH && key_lo < key_hi) fetch(key_lo);
    for (uint32_t k0 = key_lo; k0 < key_hi; k0 += 32) {
        if (!PREFETCH) fetch(k0);
        stage();
        __syncthreads();
        if (PREFETCH && k0 + 32 < key_hi) fetch(k0 + 32);
        // ---- scores, transposed: c[4blk + r] = <K[k0 + 8blk + 4half + r], Q[qidx]>; the cross terms
        // (scaled low parts) collect in c2
        attn_v16f c, c2;
#pragma unroll
        for (int e = 0; e < 16; ++e) c[e] = c2[e] = 0.0f;
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
            const uint4 kh = *reinterpret_cast<const uint4*>(sKh + col * KLD + 16 * j + 8 * half);
            c = attn_mfma(kh, qh[j], c);
            c2 = attn_mfma(kh, ql[j], c2);
            if (LOW) {
                const uint4 kl = *reinterpret_cast<const uint4*>(sKl + col * KLD + 16 * j + 8 * half);
                c2 = attn_mfma(kl, qh[j], c2);
            }
        }
        // scores in the base-2 domain (scale * log2 e folded into one factor); a tile that every
        // query of the block sees whole skips the masking
        float mx = -__builtin_inff();
        if (k0 + 32 <= min(key_hi, first_len + q0)) {
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                c[e] = fmaf(c2[e], 1.0f / ATTN_LO_SCALE, c[e]) * scale2;
                mx = fmaxf(mx, c[e]);
            }
        } else {
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const uint32_t kg = k0 + 8 * (e >> 2) + 4 * half + (e & 3);
                const bool ok = q_live && kg < my_len && kg < key_hi;
                c[e] = ok ? fmaf(c2[e], 1.0f / ATTN_LO_SCALE, c[e]) * scale2 : -__builtin_inff();
                mx = fmaxf(mx, c[e]);
            }
        }
        mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
        const float m_new = fmaxf(m, mx);
        // a query with nothing visible yet keeps m = -inf: weights and correction are then 0 / 1
        const float corr = m_new == -__builtin_inff() ? 1.0f : __builtin_amdgcn_exp2f(m - m_new);
        float ps = 0.0f;
#pragma unroll
        for (int e = 0; e < 16; ++e) {
            c[e] = c[e] == -__builtin_inff() ? 0.0f : __builtin_amdgcn_exp2f(c[e] - m_new);
            ps += c[e];
        }
        ps += __shfl_xor(ps, 32, 64);
        l = l * static_cast<double>(corr) + static_cast<double>(ps);
        m = m_new;
        // ---- the correction factors, re-laid out by output row (query 8blk + 4half + r); once the
        // running maxima have settled they are all exactly 1
        if (__builtin_amdgcn_ballot_w64(corr != 1.0f) != 0) {
            if (half == 0) sX[col] = corr;
            __builtin_amdgcn_wave_barrier();   // sX is this wavefront's own: LDS operations of one wavefront complete in order
#pragma unroll
            for (int blk = 0; blk < 4; ++blk) {
                const float4 cr = *reinterpret_cast<const float4*>(sX + 8 * blk + 4 * half);
                const float crv[4] = {cr.x, cr.y, cr.z, cr.w};
#pragma unroll
                for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
                    for (int r = 0; r < 4; ++r) acc[dt][4 * blk + r] *= crv[r];
            }
        }
        // ---- O += P . V: the weights split like everything else; slot s of step kk is c[8kk + s]
        uint4 ph[2], pl[2];
#pragma unroll
        for (int kk = 0; kk < 2; ++kk) {
            attn_split2<false>(c[8 * kk + 0], c[8 * kk + 1], ph[kk].x, pl[kk].x);
            attn_split2<false>(c[8 * kk + 2], c[8 * kk + 3], ph[kk].y, pl[kk].y);
            attn_split2<false>(c[8 * kk + 4], c[8 * kk + 5], ph[kk].z, pl[kk].z);
            attn_split2<false>(c[8 * kk + 6], c[8 * kk + 7], ph[kk].w, pl[kk].w);
        }
#pragma unroll
        for (int kk = 0; kk < 2; ++kk)
#pragma unroll
            for (int dt = 0; dt < NDT; ++dt) {
                const uint4 vh = *reinterpret_cast<const uint4*>(sVh + (32 * dt + col) * VTLD + 16 * kk + 8 * half);
                acc[dt] = attn_mfma(ph[kk], vh, acc[dt]);
                acc[dt] = attn_mfma(pl[kk], vh, acc[dt]);
                if (LOW) {
                    const uint4 vl = *reinterpret_cast<const uint4*>(sVl + (32 * dt + col) * VTLD + 16 * kk + 8 * half);
                    acc[dt] = attn_mfma(ph[kk], vl, acc[dt]);
                }
            }
        __syncthreads();   // the K and V tiles are rewritten by the next tile
    }

    // ---- partial out: rows of acc are queries 8blk + 4half + r, columns 32dt + col
#pragma unroll
    for (int blk = 0; blk < 4; ++blk)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const uint32_t qi = q0 + 8 * blk + 4 * half + r;
            if (qi < n_queries) {
                float* dst = part_acc + (((static_cast<uint64_t>(qi) * n_kv + kvh) * n_parts + part) * G + hg) * HD + col;
#pragma unroll
                for (int dt = 0; dt < NDT; ++dt) dst[32 * dt] = acc[dt][4 * blk + r];
            }
        }
    if (half == 0 && q_live) {
        float* ml = part_ml + (((static_cast<uint64_t>(qidx) * n_kv + kvh) * n_parts + part) * G + hg) * 2;
        ml[0] = m * 0.69314718055994530942f;   // back to the natural-log domain the merge works in
        ml[1] = static_cast<float>(l);
    }
}
template <typename KV, int HD, int G>
__global__ __launch_bounds__(64 * G) void attn_prefill_partial_kernel(
    const float* __restrict__ q,       // [n_queries][q_stride], rows 16-byte aligned
    const KV* __restrict__ kc,         // [n_kv][max_seq][128], already holding the batch's keys
    const KV* __restrict__ vc,
    uint32_t first_len,                // keys visible to query 0; query i sees first_len + i
    uint32_t n_queries, uint32_t max_seq, float scale, uint32_t part_keys, uint32_t n_parts, uint32_t q_stride,
    float* __restrict__ part_acc,      // [n_queries][n_kv][n_parts][G][128]
    float* __restrict__ part_ml) {
    attn_prefill_partial_body<KV, HD, G>(q, kc, vc, first_len, n_queries, max_seq, scale, part_keys, n_parts, q_stride, part_acc, part_ml);
}

// Merge the parts of one query head: out = sum_p e^{m_p - M} acc_p / sum_p e^{m_p - M} l_p.
// One workgroup of 256 threads per (head, query): the maxima and weights are
// computed with the parts spread over all threads, the weighted accumulation
// with the parts spread over 8 groups of 32 lanes (a float4 of the head's columns
// per lane; half of each group idles when head_dim is 64), so the dependent-load chain is n_parts / 8 long.  Group 0 folds
// the groups together and optionally writes the Q8_0 quantisation of the
// result for the output projection.
template <bool QUANT, int HD>
__device__ __forceinline__ void attn_decode_merge_body(const float* __restrict__ part_acc,
                                                                const float* __restrict__ part_ml,
                                                                uint32_t n_parts, uint32_t G, uint32_t n_heads,
                                                                float* __restrict__ out,
                                                                float* __restrict__ scales,
                                                                int8_t* __restrict__ quants,
                                                                float* __restrict__ bsum) {
    __shared__ float wbuf[ATTN_MAX_PARTS];
    __shared__ float red[8];
    __shared__ float4 sacc[8][32];
    const uint32_t head = blockIdx.x, tid = threadIdx.x, c = tid & 31, grp = tid >> 5, wave = tid >> 6;
    const uint32_t kvh = head / G, hg = head % G, qi = blockIdx.y, n_kv = n_heads / G;
    const uint64_t pbase = (static_cast<uint64_t>(qi) * n_kv + kvh) * n_parts;
    constexpr uint32_t C4 = HD / 4;          // float4 columns of a head; lanes c >= C4 of a group idle
    const bool live = c < C4;
    // the first ATTN_MERGE_PF parts of this group are requested before anything depends on them
    float4 pre[ATTN_MERGE_PF];
#pragma unroll
    for (int i = 0; i < ATTN_MERGE_PF; ++i) {
        const uint32_t p = grp + 8 * i;
        pre[i] = make_float4(0.f, 0.f, 0.f, 0.f);
        if (p < n_parts && live) pre[i] = reinterpret_cast<const float4*>(part_acc + ((pbase + p) * G + hg) * HD)[c];
    }
    float M = -__builtin_inff();
    for (uint32_t p = tid; p < n_parts; p += 256) M = fmaxf(M, part_ml[((pbase + p) * G + hg) * 2]);
    M = wave_max(M);
    if ((tid & 63) == 0) red[wave] = M;
    __syncthreads();
    M = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
    float L = 0.0f;
    for (uint32_t p = tid; p < n_parts; p += 256) {
        const float2 ml = *reinterpret_cast<const float2*>(part_ml + ((pbase + p) * G + hg) * 2);
        float w = cera_expf(ml.x - M);
        wbuf[p] = w;
        L = fmaf(w, ml.y, L);
    }
    L = wave_sum(L);
    if ((tid & 63) == 0) red[4 + wave] = L;
    __syncthreads();
    L = (red[4] + red[5]) + (red[6] + red[7]);
    float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
    for (int i = 0; i < ATTN_MERGE_PF; ++i) {
        const uint32_t p = grp + 8 * i;
        const float w = p < n_parts ? wbuf[p] : 0.0f;
        acc.x = fmaf(w, pre[i].x, acc.x); acc.y = fmaf(w, pre[i].y, acc.y);
        acc.z = fmaf(w, pre[i].z, acc.z); acc.w = fmaf(w, pre[i].w, acc.w);
    }
    // further parts in batches of ATTN_MERGE_PF per group, each batch one memory round trip
    for (uint32_t base = 8 * ATTN_MERGE_PF; base < n_parts; base += 8 * ATTN_MERGE_PF) {
#pragma unroll
        for (int i = 0; i < ATTN_MERGE_PF; ++i) {
            const uint32_t p = base + grp + 8 * i;
            pre[i] = make_float4(0.f, 0.f, 0.f, 0.f);
            if (p < n_parts && live) pre[i] = reinterpret_cast<const float4*>(part_acc + ((pbase + p) * G + hg) * HD)[c];
        }
#pragma unroll
        for (int i = 0; i < ATTN_MERGE_PF; ++i) {
            const uint32_t p = base + grp + 8 * i;
            const float w = p < n_parts ? wbuf[p] : 0.0f;
            acc.x = fmaf(w, pre[i].x, acc.x); acc.y = fmaf(w, pre[i].y, acc.y);
            acc.z = fmaf(w, pre[i].z, acc.z); acc.w = fmaf(w, pre[i].w, acc.w);
        }
    }
    sacc[grp][c] = acc;
    __syncthreads();
    if (grp == 0) {
#pragma unroll
        for (int g = 1; g < 8; ++g) {
            const float4 a = sacc[g][c];
            acc.x += a.x; acc.y += a.y; acc.z += a.z; acc.w += a.w;
        }
        float inv = 1.0f / L;
        float4 o = make_float4(acc.x * inv, acc.y * inv, acc.z * inv, acc.w * inv);
        const uint64_t row = static_cast<uint64_t>(qi) * n_heads + head;  // outputs are [n_queries][n_heads][HD]
        if (live) reinterpret_cast<float4*>(out + row * HD)[c] = o;
        if (QUANT) {
            // every lane takes part in the 8-lane exchanges; whole groups of 8 are live or idle together
            float sc;
            uint32_t packed = q8_quantize_quad(o, sc);
            float ssum = bsum ? q8_block_scaled_sum(packed, sc) : 0.0f;
            if (live) {
                reinterpret_cast<uint32_t*>(quants)[row * C4 + c] = packed;
                if ((c & 7) == 0) {
                    scales[row * (HD / 32) + (c >> 3)] = sc;
                    if (bsum) bsum[row * (HD / 32) + (c >> 3)] = ssum;
                }
            }
        }
    }
}
template <bool QUANT, int HD>
__global__ __launch_bounds__(256) void attn_decode_merge_kernel(const float* __restrict__ part_acc,
                                                                const float* __restrict__ part_ml,
                                                                uint32_t n_parts, uint32_t G, uint32_t n_heads,
                                                                float* __restrict__ out,
                                                                float* __restrict__ scales,
                                                                int8_t* __restrict__ quants,
                                                                float* __restrict__ bsum) {
    attn_decode_merge_body<QUANT, HD>(part_acc, part_ml, n_parts, G, n_heads, out, scales, quants, bsum);
}

// Merge for a batch of queries (prefill): the same formula as above over the few parts a prefill
// pass makes (8 at most), but eight (query, head) pairs per workgroup, 32 lanes each (a float4 of
// the head's columns per lane), the parts walked in order by every lane.  The decode merge spends
// a 256-thread workgroup and two barriers on one pair, which for 512 queries x 32 heads x 4 parts
// cost more than the attention itself.
template <bool QUANT, int HD>
__device__ __forceinline__ void attn_prefill_merge_body(const float* __restrict__ part_acc,
                                                                 const float* __restrict__ part_ml,
                                                                 uint32_t n_parts, uint32_t G, uint32_t n_heads,
                                                                 uint32_t n_pairs, float* __restrict__ out,
                                                                 float* __restrict__ scales, int8_t* __restrict__ quants,
                                                                 float* __restrict__ bsum) {
    const uint32_t pair = blockIdx.x * 8 + (threadIdx.x >> 5), c = threadIdx.x & 31;
    if (pair >= n_pairs) return;   // whole 32-lane groups leave together
    const uint32_t qi = pair / n_heads, head = pair % n_heads;
    const uint32_t kvh = head / G, hg = head % G, n_kv = n_heads / G;
    const uint64_t pbase = (static_cast<uint64_t>(qi) * n_kv + kvh) * n_parts;
    constexpr uint32_t C4 = HD / 4;
    const bool live = c < C4;
    float M = -__builtin_inff();
    for (uint32_t p = 0; p < n_parts; ++p) M = fmaxf(M, part_ml[((pbase + p) * G + hg) * 2]);
    float L = 0.0f;
    float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
    for (uint32_t p = 0; p < n_parts; ++p) {
        const float2 ml = *reinterpret_cast<const float2*>(part_ml + ((pbase + p) * G + hg) * 2);
        const float w = cera_expf(ml.x - M);
        L = fmaf(w, ml.y, L);
        float4 a = make_float4(0.f, 0.f, 0.f, 0.f);
        if (live) a = reinterpret_cast<const float4*>(part_acc + ((pbase + p) * G + hg) * HD)[c];
        acc.x = fmaf(w, a.x, acc.x); acc.y = fmaf(w, a.y, acc.y);
        acc.z = fmaf(w, a.z, acc.z); acc.w = fmaf(w, a.w, acc.w);
    }
    const float inv = 1.0f / L;
    const float4 o = make_float4(acc.x * inv, acc.y * inv, acc.z * inv, acc.w * inv);
    const uint64_t row = static_cast<uint64_t>(qi) * n_heads + head;   // outputs are [n_queries][n_heads][HD]
    if (live) reinterpret_cast<float4*>(out + row * HD)[c] = o;
    if (QUANT) {
        // every lane of the pair takes part in the 8-lane exchanges; whole groups of 8 are live or idle together
        float sc;
        const uint32_t packed = q8_quantize_quad(o, sc);
        const float ssum = bsum ? q8_block_scaled_sum(packed, sc) : 0.0f;
        if (live) {
            reinterpret_cast<uint32_t*>(quants)[row * C4 + c] = packed;
            if ((c & 7) == 0) {
                scales[row * (HD / 32) + (c >> 3)] = sc;
                if (bsum) bsum[row * (HD / 32) + (c >> 3)] = ssum;
            }
        }
    }
}
template <bool QUANT, int HD>
__global__ __launch_bounds__(256) void attn_prefill_merge_kernel(const float* __restrict__ part_acc,
                                                                 const float* __restrict__ part_ml,
                                                                 uint32_t n_parts, uint32_t G, uint32_t n_heads,
                                                                 uint32_t n_pairs, float* __restrict__ out,
                                                                 float* __restrict__ scales, int8_t* __restrict__ quants,
                                                                 float* __restrict__ bsum) {
    attn_prefill_merge_body<QUANT, HD>(part_acc, part_ml, n_parts, G, n_heads, n_pairs, out, scales, quants, bsum);
}

