// CPU oracle (test infrastructure only): the dense-transformer forward pass of
// cera's LlamaModel on the CPU int8 path -- cera/src/model/llama.rs:468-597
// (run_layers, project_logits), :1585-1605 (forward) and
// cera/src/model/transformer.rs:1313-1652 (attention / FFN blocks).
#include "orc_llama.h"

#include <atomic>

#include <cmath>
#include <cstring>
#include <vector>

struct OrcLlama {
    OrcLlamaConfig cfg;
    OrcTensor embd, output;
    bool has_output = false;
    const float* output_norm = nullptr;
    std::vector<OrcLlamaLayer> layers;
    // state (kv_cache.rs:201-221): per layer time-major f32 K and V, [pos][kv_dim]
    std::vector<std::vector<float>> kc, vc;
    uint32_t seq_len = 0;
    // KvCompression::F16 (kv_cache.rs:93-98): rows are narrowed to half on append and widened on
    // every read (transformer.rs:1424-1447, llama.rs:1134-1170).  Widening is exact, so the
    // caches here keep the widened values: same numbers, one code path.
    bool kv_f16 = false;
    int variant = 0;
    // batched prefill GEMMs through transformer::gemm_preq's x86 route: Q4_0 / Q4_K weights that
    // cera repacks at load take the 8-row-interleaved kernels (orc_repack.cpp)
    bool x86_repack = false;
    void* pool = nullptr;  // optional worker pool for the GEMVs (timing only)
};

static void gemv(OrcLlama* m, const OrcTensor& t, const float* x, float* y) {
    if (m->pool) orc_gemv_mt(m->pool, t.dtype, t.data, x, y, t.m, t.k);
    else orc_gemv(t.dtype, t.data, x, y, t.m, t.k, m->variant);
}

OrcLlama* orc_llama_create(const OrcLlamaConfig* cfg, const OrcTensor* embd, const OrcTensor* output,
                           const float* output_norm, const OrcLlamaLayer* layers, int variant) {
    OrcLlama* m = new OrcLlama();
    m->cfg = *cfg;
    m->embd = *embd;
    if (output) { m->output = *output; m->has_output = true; }
    m->output_norm = output_norm;
    m->layers.assign(layers, layers + cfg->n_layers);
    m->kc.resize(cfg->n_layers);
    m->vc.resize(cfg->n_layers);
    m->variant = variant;
    return m;
}
void orc_llama_destroy(OrcLlama* m) { delete m; }
void orc_llama_set_pool(OrcLlama* m, void* pool) { m->pool = pool; }
void orc_llama_set_kv_f16(OrcLlama* m, int on) { m->kv_f16 = on != 0; }
void orc_llama_set_x86_repack(OrcLlama* m, int on) { m->x86_repack = on != 0; }
static void append_kv(const OrcLlama* m, std::vector<float>& cache, const float* row, uint64_t n) {
    if (!m->kv_f16) { cache.insert(cache.end(), row, row + n); return; }
    for (uint64_t i = 0; i < n; ++i) cache.push_back(orc_f16_to_f32(orc_f32_to_f16(row[i])));
}
uint32_t orc_llama_seq_len(const OrcLlama* m) { return m->seq_len; }
void orc_llama_truncate(OrcLlama* m, uint32_t len) {
    if (len >= m->seq_len) return;
    uint64_t kv_dim = uint64_t(m->cfg.n_kv_heads) * m->cfg.head_dim;
    for (auto& v : m->kc) v.resize(len * kv_dim);
    for (auto& v : m->vc) v.resize(len * kv_dim);
    m->seq_len = len;
}

// LlamaModel::shift_kv (llama.rs:1727-1738) -> InferenceState::shift_kv_with_rope, f32 path
// (kv_cache.rs:1091-1160, 1233-1310): drain rows [n_keep, n_keep + shift) of every layer's K and
// V, then delta-rotate the K heads of the rows now at [n_keep, new_seq_len) by -shift.
// Returns -1 where the reference asserts (shift == 0, range past seq_len).
int orc_llama_shift_kv(OrcLlama* m, uint32_t n_keep, uint32_t shift) {
    const OrcLlamaConfig& c = m->cfg;
    if (shift == 0 || uint64_t(n_keep) + shift > m->seq_len) return -1;
    const uint64_t kv_dim = uint64_t(c.n_kv_heads) * c.head_dim;
    const uint32_t new_len = m->seq_len - shift;
    for (uint32_t l = 0; l < c.n_layers; ++l) {
        auto& kc = m->kc[l];
        auto& vc = m->vc[l];
        if (kc.empty() && vc.empty()) continue;
        kc.erase(kc.begin() + n_keep * kv_dim, kc.begin() + (uint64_t(n_keep) + shift) * kv_dim);
        vc.erase(vc.begin() + n_keep * kv_dim, vc.begin() + (uint64_t(n_keep) + shift) * kv_dim);
        for (uint32_t t = n_keep; t < new_len; ++t)
            for (uint32_t h = 0; h < c.n_kv_heads; ++h)
            {
                float* head = kc.data() + t * kv_dim + h * c.head_dim;
                orc_rope_delta_head(head, -int32_t(shift), c.head_dim, c.rope_theta, c.rope_type, c.rope_freqs);
                // f16 cache: widened, rotated, narrowed back (kv_cache.rs:1196-1230)
                if (m->kv_f16)
                    for (uint32_t d = 0; d < c.head_dim; ++d) head[d] = orc_f16_to_f32(orc_f32_to_f16(head[d]));
            }
    }
    m->seq_len = new_len;
    return 0;
}

// Prefix-cache restore (InferenceState::restore, the CPU twin of Model::restore_state,
// mod.rs:526-533): replace every layer's K/V with n_pos rows and set seq_len.
int orc_llama_restore_kv(OrcLlama* m, uint32_t layer, const float* k, const float* v, uint32_t n_pos) {
    if (layer >= m->cfg.n_layers) return -1;
    const uint64_t n = uint64_t(n_pos) * m->cfg.n_kv_heads * m->cfg.head_dim;
    m->kc[layer].clear();
    m->vc[layer].clear();
    append_kv(m, m->kc[layer], k, n);
    append_kv(m, m->vc[layer], v, n);
    return 0;
}
void orc_llama_set_seq_len(OrcLlama* m, uint32_t len) { m->seq_len = len; }

// llama.rs:1585-1605 + :468-597.  Writes vocab logits; optionally the final
// normed hidden state (for intermediate-value checks).
int orc_llama_forward(OrcLlama* m, uint32_t token, uint32_t pos, float* logits, float* hidden_out) {
    const OrcLlamaConfig& c = m->cfg;
    if (token >= c.vocab || pos != m->seq_len) return -1;
    const uint32_t hs = c.hidden, hd = c.head_dim;
    const uint32_t q_dim = c.n_heads * hd, kv_dim = c.n_kv_heads * hd;
    std::vector<float> hidden(hs), normed(hs), ffn_in(hs), q(q_dim), k(kv_dim), v(kv_dim),
        attn_out(q_dim), out(hs), gate(c.ffn), up(c.ffn);

    const uint8_t* erow = static_cast<const uint8_t*>(m->embd.data) +
                          uint64_t(token) * orc_row_bytes(m->embd.dtype, m->embd.k);
    if (orc_dequantize_row(m->embd.dtype, erow, m->embd.k, hidden.data())) return -2;
    if (c.embed_scale != 1.0f) for (auto& x : hidden) x *= c.embed_scale;

    const float scale = c.attn_scale != 0.0f ? c.attn_scale : 1.0f / std::sqrt(float(hd));
    for (uint32_t l = 0; l < c.n_layers; ++l) {
        const OrcLlamaLayer& L = m->layers[l];
        normed = hidden;
        orc_rmsnorm(normed.data(), L.attn_norm, hs, c.rms_eps);
        gemv(m, L.attn_q, normed.data(), q.data());
        gemv(m, L.attn_k, normed.data(), k.data());
        gemv(m, L.attn_v, normed.data(), v.data());
        if (L.q_bias && L.k_bias && L.v_bias) {
            orc_add(q.data(), L.q_bias, q_dim);
            orc_add(k.data(), L.k_bias, kv_dim);
            orc_add(v.data(), L.v_bias, kv_dim);
        }
        if (L.q_norm && L.k_norm) {
            for (uint32_t h = 0; h < c.n_heads; ++h) orc_rmsnorm(q.data() + h * hd, L.q_norm, hd, c.rms_eps);
            for (uint32_t h = 0; h < c.n_kv_heads; ++h) orc_rmsnorm(k.data() + h * hd, L.k_norm, hd, c.rms_eps);
        }
        if (c.rope_type == 0) orc_rope_neox(q.data(), k.data(), pos, c.n_heads, c.n_kv_heads, hd, c.rope_theta);
        else orc_rope_norm(q.data(), k.data(), pos, c.n_heads, c.n_kv_heads, hd, c.rope_theta, c.rope_freqs);
        append_kv(m, m->kc[l], k.data(), k.size());
        append_kv(m, m->vc[l], v.data(), v.size());
        uint64_t L_ctx = m->kc[l].size() / kv_dim;
        orc_decode_attention(q.data(), m->kc[l].data(), m->vc[l].data(), c.n_heads, c.n_kv_heads, hd,
                             scale, L_ctx, attn_out.data(), m->variant);
        gemv(m, L.attn_output, attn_out.data(), out.data());
        if (c.residual_scale != 1.0f) for (auto& x : out) x *= c.residual_scale;
        orc_add(hidden.data(), out.data(), hs);

        ffn_in = hidden;
        orc_rmsnorm(ffn_in.data(), L.ffn_norm, hs, c.rms_eps);
        gemv(m, L.ffn_gate, ffn_in.data(), gate.data());
        gemv(m, L.ffn_up, ffn_in.data(), up.data());
        orc_silu_mul(gate.data(), up.data(), c.ffn);
        gemv(m, L.ffn_down, gate.data(), out.data());
        if (c.residual_scale != 1.0f) for (auto& x : out) x *= c.residual_scale;
        orc_add(hidden.data(), out.data(), hs);
    }
    orc_rmsnorm(hidden.data(), m->output_norm, hs, c.rms_eps);
    m->seq_len += 1;
    if (hidden_out) std::memcpy(hidden_out, hidden.data(), hs * sizeof(float));
    if (logits) {
        const OrcTensor& o = m->has_output ? m->output : m->embd;
        gemv(m, o, hidden.data(), logits);
        if (c.logit_scale != 1.0f) {
            float inv = 1.0f / c.logit_scale;
            for (uint32_t i = 0; i < c.vocab; ++i) logits[i] *= inv;
        }
    }
    return 0;
}

// llama.rs:1607-1649 per-token route (tokens.len() == 1 or oracle-dump mode);
// the batched route is orc_llama_forward_prefill_batched.
int orc_llama_forward_prefill_per_token(OrcLlama* m, const uint32_t* tokens, uint32_t n,
                                        uint32_t start_pos, float* last_logits) {
    if (n == 0 || start_pos != m->seq_len) return -1;
    for (uint32_t i = 0; i < n; ++i) {
        int rc = orc_llama_forward(m, tokens[i], start_pos + i, i + 1 == n ? last_logits : nullptr, nullptr);
        if (rc) return rc;
    }
    return 0;
}

const float* orc_llama_kcache(const OrcLlama* m, uint32_t layer) { return m->kc[layer].data(); }
const float* orc_llama_vcache(const OrcLlama* m, uint32_t layer) { return m->vc[layer].data(); }

// ---------------------------------------------------------------------------
// forward_prefill_batched (llama.rs:738-1523), no-`blas` int8 route.  The
// reference keeps activations column-major [dim][n]; here they are row-major
// [n][dim] -- the same numbers, and every per-element operation is in the
// reference's order.  GEMMs are gemm_preq over quantize_columns
// (transformer.rs:710-788, 865-946) with the tiled (n > 1) accumulator order.
static void quantize_rows(const std::vector<float>& x, uint32_t n, uint32_t dim, std::vector<float>& bs,
                          std::vector<int8_t>& bq) {
    bs.resize(size_t(n) * (dim / 32));
    bq.resize(size_t(n) * dim);
    for (uint32_t j = 0; j < n; ++j)
        orc_quantize_q8_0(x.data() + size_t(j) * dim, dim, bs.data() + size_t(j) * (dim / 32), bq.data() + size_t(j) * dim);
}
// out_rows[n][m] = (W . B)^T, B given as quantized rows.  With a pool the weight rows are
// split into contiguous ranges, one per worker; every output row is computed by the same
// code either way (the strip kernels are row-independent), so the result does not change.
static int gemm_rows(OrcLlama* m, const OrcTensor& t, const std::vector<float>& bs, const std::vector<int8_t>& bq,
                     uint32_t n, std::vector<float>& out_rows, std::vector<float>& tmp) {
    tmp.resize(size_t(t.m) * n);
    int rc = 0;
    if (m->pool) {
        struct Job { OrcLlama* m; const OrcTensor* t; const float* bs; const int8_t* bq; uint32_t n; float* tmp; uint64_t rb; std::atomic<int> rc; };
        Job job{m, &t, bs.data(), bq.data(), n, tmp.data(), orc_row_bytes(t.dtype, t.k), {0}};
        orc_pool_run(m->pool, [](int tid, int nt, void* a) {
            Job& j = *static_cast<Job*>(a);
            // ranges on multiples of 8 rows so a range never splits a row tile
            uint64_t tiles = (j.t->m + 7) / 8;
            uint64_t r0 = std::min<uint64_t>(j.t->m, tiles * uint64_t(tid) / uint64_t(nt) * 8);
            uint64_t r1 = std::min<uint64_t>(j.t->m, tiles * uint64_t(tid + 1) / uint64_t(nt) * 8);
            if (r1 <= r0) return;
            // a weight is repacked as a whole (m % 8 == 0); the ranges here are whole 8-row tiles
            auto fn = (j.m->x86_repack && j.t->m % 8 == 0) ? orc_gemm_preq_x86 : orc_gemm_preq;
            int e = fn(j.t->dtype, static_cast<const uint8_t*>(j.t->data) + r0 * j.rb, j.bs, j.bq,
                       j.tmp + r0 * j.n, r1 - r0, j.n, j.t->k, j.m->variant);
            if (e) j.rc = e;
        }, &job);
        rc = job.rc;
    } else {
        auto fn = m->x86_repack ? orc_gemm_preq_x86 : orc_gemm_preq;
        rc = fn(t.dtype, t.data, bs.data(), bq.data(), tmp.data(), t.m, n, t.k, m->variant);
    }
    if (rc) return rc;
    out_rows.resize(size_t(n) * t.m);
    for (uint64_t i = 0; i < t.m; ++i)
        for (uint32_t j = 0; j < n; ++j) out_rows[size_t(j) * t.m + i] = tmp[i * n + j];
    return 0;
}

int orc_llama_forward_prefill_batched(OrcLlama* m, const uint32_t* tokens, uint32_t n, uint32_t start_pos,
                                      float* last_logits, float* all_hidden) {
    const OrcLlamaConfig& c = m->cfg;
    if (n == 0 || start_pos != m->seq_len) return -1;
    const uint32_t hs = c.hidden, hd = c.head_dim, is = c.ffn;
    const uint32_t q_dim = c.n_heads * hd, kv_dim = c.n_kv_heads * hd, group = c.n_heads / c.n_kv_heads;
    const float scale = c.attn_scale != 0.0f ? c.attn_scale : 1.0f / std::sqrt(float(hd));
    std::vector<float> hidden(size_t(n) * hs), normed(size_t(n) * hs), qm, km, vm, attn(size_t(n) * q_dim), blk, gate, up, tmp;
    std::vector<float> bs;
    std::vector<int8_t> bq;
    for (uint32_t j = 0; j < n; ++j) {
        if (tokens[j] >= c.vocab) return -1;
        const uint8_t* erow = static_cast<const uint8_t*>(m->embd.data) + uint64_t(tokens[j]) * orc_row_bytes(m->embd.dtype, m->embd.k);
        if (orc_dequantize_row(m->embd.dtype, erow, m->embd.k, hidden.data() + size_t(j) * hs)) return -2;
        if (c.embed_scale != 1.0f) for (uint32_t i = 0; i < hs; ++i) hidden[size_t(j) * hs + i] *= c.embed_scale;
    }
    const bool use_flash = n >= 256;  // FLASH_ATTN_THRESHOLD, llama.rs:845
    for (uint32_t l = 0; l < c.n_layers; ++l) {
        const OrcLlamaLayer& L = m->layers[l];
        normed = hidden;
        for (uint32_t j = 0; j < n; ++j) orc_rmsnorm(normed.data() + size_t(j) * hs, L.attn_norm, hs, c.rms_eps);
        quantize_rows(normed, n, hs, bs, bq);
        if (gemm_rows(m, L.attn_q, bs, bq, n, qm, tmp) || gemm_rows(m, L.attn_k, bs, bq, n, km, tmp) ||
            gemm_rows(m, L.attn_v, bs, bq, n, vm, tmp))
            return -3;
        for (uint32_t j = 0; j < n; ++j) {
            float* q = qm.data() + size_t(j) * q_dim;
            float* k = km.data() + size_t(j) * kv_dim;
            float* v = vm.data() + size_t(j) * kv_dim;
            if (L.q_bias && L.k_bias && L.v_bias) {
                orc_add(q, L.q_bias, q_dim);
                orc_add(k, L.k_bias, kv_dim);
                orc_add(v, L.v_bias, kv_dim);
            }
            if (L.q_norm && L.k_norm) {
                for (uint32_t h = 0; h < c.n_heads; ++h) orc_rmsnorm(q + h * hd, L.q_norm, hd, c.rms_eps);
                for (uint32_t h = 0; h < c.n_kv_heads; ++h) orc_rmsnorm(k + h * hd, L.k_norm, hd, c.rms_eps);
            }
            if (c.rope_type == 0) orc_rope_neox(q, k, start_pos + j, c.n_heads, c.n_kv_heads, hd, c.rope_theta);
            else orc_rope_norm(q, k, start_pos + j, c.n_heads, c.n_kv_heads, hd, c.rope_theta, c.rope_freqs);
            append_kv(m, m->kc[l], k, kv_dim);
            append_kv(m, m->vc[l], v, kv_dim);
        }
        const float* kcache = m->kc[l].data();
        const float* vcache = m->vc[l].data();
        if (use_flash) {
            struct Job { const OrcLlamaConfig* c; const float *qm, *kc, *vc; float* attn; uint32_t n, start_pos, q_dim, kv_dim, group; float scale; int variant; };
            Job job{&c, qm.data(), kcache, vcache, attn.data(), n, start_pos, q_dim, kv_dim, group, scale, m->variant};
            auto heads = [](int tid, int nt, void* a) {   // heads are independent: one range per worker
                Job& j = *static_cast<Job*>(a);
                const uint32_t hd = j.c->head_dim;
                std::vector<float> qh(size_t(j.n) * hd), oh(size_t(j.n) * hd);
                for (uint32_t h = j.c->n_heads * uint32_t(tid) / uint32_t(nt); h < j.c->n_heads * uint32_t(tid + 1) / uint32_t(nt); ++h) {
                    for (uint32_t t = 0; t < j.n; ++t)
                        std::memcpy(qh.data() + size_t(t) * hd, j.qm + size_t(t) * j.q_dim + h * hd, hd * sizeof(float));
                    orc_flash_attention_head_v(qh.data(), j.kc, j.vc, oh.data(), j.n, j.kv_dim, uint64_t(h / j.group) * hd, hd, j.scale, j.start_pos, j.variant);
                    for (uint32_t t = 0; t < j.n; ++t)
                        std::memcpy(j.attn + size_t(t) * j.q_dim + h * hd, oh.data() + size_t(t) * hd, hd * sizeof(float));
                }
            };
            if (m->pool) orc_pool_run(m->pool, heads, &job);
            else heads(0, 1, &job);
        } else {
            for (uint32_t j = 0; j < n; ++j) {
                uint64_t L_ctx = uint64_t(start_pos) + j + 1;
                orc_decode_attention(qm.data() + size_t(j) * q_dim, kcache, vcache, c.n_heads, c.n_kv_heads, hd, scale, L_ctx,
                                     attn.data() + size_t(j) * q_dim, m->variant);
            }
        }
        quantize_rows(attn, n, q_dim, bs, bq);
        if (gemm_rows(m, L.attn_output, bs, bq, n, blk, tmp)) return -3;
        if (c.residual_scale != 1.0f) for (auto& x : blk) x *= c.residual_scale;
        orc_add(hidden.data(), blk.data(), size_t(n) * hs);

        normed = hidden;
        for (uint32_t j = 0; j < n; ++j) orc_rmsnorm(normed.data() + size_t(j) * hs, L.ffn_norm, hs, c.rms_eps);
        quantize_rows(normed, n, hs, bs, bq);
        if (gemm_rows(m, L.ffn_gate, bs, bq, n, gate, tmp) || gemm_rows(m, L.ffn_up, bs, bq, n, up, tmp)) return -3;
        orc_silu_mul(gate.data(), up.data(), size_t(n) * is);
        quantize_rows(gate, n, is, bs, bq);
        if (gemm_rows(m, L.ffn_down, bs, bq, n, blk, tmp)) return -3;
        if (c.residual_scale != 1.0f) for (auto& x : blk) x *= c.residual_scale;
        orc_add(hidden.data(), blk.data(), size_t(n) * hs);
    }
    m->seq_len = start_pos + n;
    if (all_hidden) {
        for (uint32_t j = 0; j < n; ++j) {
            std::memcpy(all_hidden + size_t(j) * hs, hidden.data() + size_t(j) * hs, hs * sizeof(float));
            orc_rmsnorm(all_hidden + size_t(j) * hs, m->output_norm, hs, c.rms_eps);
        }
    }
    if (last_logits) {
        std::vector<float> last(hidden.begin() + size_t(n - 1) * hs, hidden.end());
        orc_rmsnorm(last.data(), m->output_norm, hs, c.rms_eps);
        const OrcTensor& o = m->has_output ? m->output : m->embd;
        gemv(m, o, last.data(), last_logits);  // project_logits: the n == 1 GEMV branch
        if (c.logit_scale != 1.0f) {
            float inv = 1.0f / c.logit_scale;
            for (uint32_t i = 0; i < c.vocab; ++i) last_logits[i] *= inv;
        }
    }
    return 0;
}
