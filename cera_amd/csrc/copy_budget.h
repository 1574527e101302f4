// How much device memory a model's decode copies may take.  Host-only arithmetic, no device calls.
//
// A decode copy is a second, stream-ordered copy of a weight matrix; it speeds decode up and is
// never needed for correctness.  It must therefore never be the reason a model that fits without
// copies fails to load or to prefill: copies are built last, after every native upload, the KV
// caches and the single-token buffers, and only while the device keeps a reserve free for what a
// model allocates later (one prefill pass's buffers, the all-positions logits, and headroom for
// the context's workspaces).
#pragma once
#include <algorithm>
#include <cstddef>
#include <cstdint>

#include "cera_hip.h"

static constexpr uint32_t CERA_PREFILL_CHUNK = 2048;          // tokens one batched prefill pass takes
static constexpr uint64_t CERA_COPY_HEADROOM = 512ull << 20;  // left for scratch slots, attention partials, split-K

// bytes of the fragment-ordered fp8 split copy of n activation rows of k elements
// (64-token tiles in two halves, one 21504-byte record per half tile and 256-element super-block)
static inline uint64_t cera_fp8_split_bytes(uint64_t n, uint64_t k) { return (n + 63) / 64 * 2 * (k / 256) * 21504ull; }

// sizes of the buffers one batched prefill pass over `cap` tokens holds, in allocation order
struct CeraPrefillSizes {
    uint64_t hidden, normed, q, k, v, attn, gate, up, xq, xh, x8, xs, bsum, tokens;
    uint64_t total() const { return hidden + normed + q + k + v + attn + gate + up + xq + xh + x8 + xs + bsum + tokens; }
};
static inline CeraPrefillSizes cera_prefill_sizes(const cera_hip_config& c, uint32_t cap) {
    const uint64_t n = cap, q_dim = static_cast<uint64_t>(c.n_heads) * c.head_dim,
                   kv_dim = static_cast<uint64_t>(c.n_kv_heads) * c.head_dim;
    const uint64_t maxk = std::max<uint64_t>(std::max<uint64_t>(c.hidden, c.ffn), q_dim);
    CeraPrefillSizes s;
    s.hidden = s.normed = n * c.hidden * 4;
    s.q = s.attn = n * q_dim * 4;
    s.k = s.v = n * kv_dim * 4;
    s.gate = s.up = n * c.ffn * 4;
    s.xq = n * maxk;
    s.xh = n * maxk * 2;
    s.x8 = cera_fp8_split_bytes(n, maxk);
    s.xs = s.bsum = n * (maxk / 32) * 4;
    s.tokens = n * 4;
    return s;
}
// tokens the pass buffers are sized for when a prefill of n tokens asks for them
static inline uint32_t cera_prefill_cap(uint32_t n) { return std::min<uint32_t>(CERA_PREFILL_CHUNK, std::max<uint32_t>(n, 64)); }

// what stays free after the decode copies: the largest prefill pass this model can be asked for,
// its all-positions logits, and the headroom
static inline uint64_t cera_copy_reserve_bytes(const cera_hip_config& c) {
    const uint32_t cap = cera_prefill_cap(std::min<uint32_t>(c.max_seq_len, CERA_PREFILL_CHUNK));
    return cera_prefill_sizes(c, cap).total() + static_cast<uint64_t>(cap) * c.vocab * 4 + CERA_COPY_HEADROOM;
}

// Candidates in priority order (bytes[i] == 0: no copy possible for that matrix).  A candidate is
// taken when, after it, at least `reserve` bytes stay free; one that does not fit is skipped and
// later, smaller ones are still tried.  Returns the bytes taken.
static inline uint64_t cera_plan_decode_copies(const uint64_t* bytes, size_t n, uint64_t free_bytes, uint64_t reserve,
                                               uint8_t* take) {
    uint64_t used = 0;
    for (size_t i = 0; i < n; ++i) {
        const bool ok = bytes[i] != 0 && bytes[i] <= free_bytes && free_bytes - bytes[i] >= reserve;
        if (take) take[i] = ok ? 1 : 0;
        if (ok) { free_bytes -= bytes[i]; used += bytes[i]; }
    }
    return used;
}
