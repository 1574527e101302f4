// C ABI, model level: a device-resident dense transformer (llama architecture)
// driven through the `Model`-trait surface -- forward / forward_greedy /
// forward_prefill / truncate_kv (cera/src/model/mod.rs:200-606) -- with the
// layer graph of LlamaModel (cera/src/model/llama.rs:468-597, 1585-1649;
// cera/src/model/transformer.rs:1313-1652).
#include <cmath>
#include <cstdlib>
#include <cstring>
#include <new>

#include <type_traits>

#include "copy_budget.h"
#include "glue.hip.h"
#include "host_common.h"
#include "model.h"

// ---------------------------------------------------------------------------
static cera_hip_status dev_alloc(cera_hip_ctx* ctx, uint64_t bytes, void** out, uint64_t* total) {
    *out = nullptr;
    HIP_TRY(ctx, hipMalloc(out, bytes ? bytes : 256));
    if (total) *total += bytes;
    return CERA_HIP_OK;
}
template <class T>
static cera_hip_status dev_alloc_t(cera_hip_ctx* ctx, uint64_t n, T** out, uint64_t* total) {
    return dev_alloc(ctx, n * sizeof(T), reinterpret_cast<void**>(out), total);
}
static cera_hip_status upload_f32(cera_hip_ctx* ctx, const float* host, uint64_t n, float** out, uint64_t* total) {
    if (!host) { *out = nullptr; return CERA_HIP_OK; }
    CERA_TRY(dev_alloc_t(ctx, n, out, total));
    return cera_hip_upload(ctx, *out, host, n * 4);
}

// lanes past the end of a key range re-read a cached row with weight 0: keep every row finite
static cera_hip_status alloc_kv_cache(cera_hip_ctx* ctx, uint64_t bytes, void** out, uint64_t* total) {
    CERA_TRY(dev_alloc(ctx, bytes, out, total));
    HIP_TRY(ctx, hipMemsetAsync(*out, 0, bytes, ctx->stream));
    return CERA_HIP_OK;
}

// The matrices the one-wavefront-per-row decode kernels stream, in the order copies are handed
// out: the vocabulary head first (a tied head: the embedding table), then layer by layer.
static std::vector<cera_hip_dtensor*> decode_copy_candidates(cera_hip_model* m) {
    std::vector<cera_hip_dtensor*> v;
    v.push_back(m->output ? m->output : m->embd);
    for (LayerDev& D : m->layers)
        for (cera_hip_dtensor* w : {D.qkv, D.v, D.o, D.gate, D.up, D.down})
            if (w && w->owns) v.push_back(w);
    return v;
}

// Decode copies come last -- after every native upload, the KV caches and the single-token
// buffers -- and only from memory the model will not need later (copy_budget.h): a model that
// loads and prefills with copies off must do so with copies on.
static cera_hip_status build_decode_copies(cera_hip_model* m) {
    cera_hip_ctx* ctx = m->ctx;
    if (!ctx->decode_copies) return CERA_HIP_OK;
    std::vector<cera_hip_dtensor*> cand = decode_copy_candidates(m);
    std::vector<uint64_t> bytes(cand.size());
    for (size_t i = 0; i < cand.size(); ++i) bytes[i] = cera_tensor_stream_bytes(ctx, cand[i]);
    size_t free_b = 0, total_b = 0;
    HIP_TRY(ctx, hipMemGetInfo(&free_b, &total_b));
    std::vector<uint8_t> take(cand.size());
    cera_plan_decode_copies(bytes.data(), bytes.size(), free_b, cera_copy_reserve_bytes(m->cfg), take.data());
    for (size_t i = 0; i < cand.size(); ++i) {
        if (!take[i]) continue;
        CERA_TRY(cera_tensor_prepare_stream(ctx, cand[i]));
        if (cand[i]->dev_stream) m->bytes += cand[i]->stream_row_bytes * cand[i]->m;
    }
    return CERA_HIP_OK;
}

// Frees every decode copy of the model (the kernels then read the native bytes); returns the bytes
// given back.  The stream is drained first: a launched kernel may still be reading a copy.
uint64_t cera_model_drop_decode_copies(cera_hip_model* m) {
    uint64_t freed = 0;
    (void)hipStreamSynchronize(m->ctx->stream);
    for (cera_hip_dtensor* w : decode_copy_candidates(m)) {
        if (!w->dev_stream) continue;
        freed += w->stream_row_bytes * w->m;
        cera_tensor_drop_stream(w);
    }
    m->bytes -= std::min(m->bytes, freed);
    return freed;
}

// hipMalloc for a model's later allocations (prefill buffers, all-positions logits, re-typed KV
// caches): when the device is out of memory the decode copies are given up and the allocation is
// tried once more.
cera_hip_status cera_model_malloc(cera_hip_model* m, void** out, uint64_t bytes, const char* what) {
    *out = nullptr;
    hipError_t e = hipMalloc(out, bytes ? bytes : 256);
    if (e == hipErrorOutOfMemory) {
        (void)hipGetLastError();
        if (cera_model_drop_decode_copies(m) > 0) e = hipMalloc(out, bytes ? bytes : 256);
    }
    if (e != hipSuccess) {
        (void)hipGetLastError();
        *out = nullptr;
        return cera_fail(m->ctx, e == hipErrorOutOfMemory ? CERA_HIP_ERR_OOM : CERA_HIP_ERR_DEVICE,
                         std::string("hipMalloc(") + what + ", " + std::to_string(bytes) + " bytes): " + hipGetErrorString(e));
    }
    return CERA_HIP_OK;
}

// cos/sin table [max_seq][head_dim/2] built with the CPU path's own recurrence:
// theta_scale = base^(-2/hd); theta_0 = pos as f32; theta_{i+1} = theta_i *
// theta_scale (f32); angle = theta_i / freq_factor_i; libm sinf/cosf
// (cera/src/backend/cpu.rs:5031-5045, 5161-5180).
void cera_build_rope_table(uint32_t max_seq, uint32_t head_dim, float base, const float* ff, std::vector<float>& out) {
    const uint32_t half = head_dim / 2;
    out.resize(static_cast<size_t>(max_seq) * half * 2);
    const float theta_scale = powf(base, -2.0f / static_cast<float>(head_dim));
    for (uint32_t p = 0; p < max_seq; ++p) {
        float theta = static_cast<float>(p);
        float* row = out.data() + static_cast<size_t>(p) * half * 2;
        for (uint32_t i = 0; i < half; ++i) {
            float ang = ff ? theta / ff[i] : theta;
            row[2 * i] = cosf(ang);
            row[2 * i + 1] = sinf(ang);
            theta *= theta_scale;
        }
    }
}

static void free_model(cera_hip_model* m) {
    if (!m) return;
    cera_hip_ctx* ctx = m->ctx;
    std::lock_guard<std::recursive_mutex> op_lk(ctx->op_mu);
    (void)hipStreamSynchronize(ctx->stream);
    auto ft = [&](cera_hip_dtensor* t) { if (t) cera_hip_tensor_free(ctx, t); };
    for (auto& L : m->layers) {
        ft(L.q); ft(L.k); ft(L.v); ft(L.o); ft(L.gate); ft(L.up); ft(L.down); ft(L.qkv);
        for (float* p : {L.attn_norm, L.ffn_norm, L.q_bias, L.k_bias, L.v_bias, L.q_norm, L.k_norm})
            if (p) (void)hipFree(p);
        if (L.kc) (void)hipFree(L.kc);
        if (L.vc) (void)hipFree(L.vc);
    }
    ft(m->embd);
    ft(m->output);
    for (void* p : m->owned)
        if (p) (void)hipFree(p);
    for (void* p : m->pf_owned)
        if (p) (void)hipFree(p);
    if (m->pf_logits) (void)hipFree(m->pf_logits);
    delete m;
}

static bool gemv_type_ok(uint32_t t) {
    return t == CERA_HIP_Q4_0 || t == CERA_HIP_Q4_1 || t == CERA_HIP_Q8_0 || t == CERA_HIP_Q4_K ||
           t == CERA_HIP_Q5_K || t == CERA_HIP_Q6_K;
}

extern "C" cera_hip_status cera_hip_model_create(cera_hip_ctx* ctx, const cera_hip_config* cfg,
                                                 const cera_hip_tensor* token_embd, const cera_hip_tensor* output,
                                                 const float* output_norm, const cera_hip_layer* layers,
                                                 cera_hip_model** out) {
    if (!ctx || !cfg || !token_embd || !output_norm || !layers || !out) return CERA_HIP_ERR_ARGUMENT;
    std::lock_guard<std::recursive_mutex> op_lk(ctx->op_mu);
    *out = nullptr;
    const cera_hip_config& c = *cfg;
    if (c.n_layers == 0 || c.hidden == 0 || c.ffn == 0 || c.n_heads == 0 || c.n_kv_heads == 0 || c.vocab == 0 ||
        c.max_seq_len == 0)
        return cera_fail(ctx, CERA_HIP_ERR_ARGUMENT, "model_create: zero dimension in config");
    // head sizes other than 64 / 128 and more than 8 query heads per kv head run on a generic attention kernel
    if (c.head_dim == 0 || c.head_dim % 8 || c.head_dim > 256)
        return cera_fail(ctx, CERA_HIP_ERR_SHAPE, "model_create: head_dim must be a multiple of 8, at most 256");
    if (c.n_heads % c.n_kv_heads) return cera_fail(ctx, CERA_HIP_ERR_SHAPE, "model_create: n_heads % n_kv_heads != 0");
    if (c.hidden % 32 || c.ffn % 32) return cera_fail(ctx, CERA_HIP_ERR_SHAPE, "model_create: hidden and ffn must be multiples of 32");
    if (c.rope_type > 1) return cera_fail(ctx, CERA_HIP_ERR_ARGUMENT, "model_create: rope_type must be 0 (neox) or 1 (norm)");
    const uint32_t q_dim = c.n_heads * c.head_dim, kv_dim = c.n_kv_heads * c.head_dim;

    // shape checks before anything is uploaded: refuse, never silently skip a matmul
    auto expect = [&](const cera_hip_tensor& t, uint64_t m, uint64_t k, const char* name, bool matmul) -> cera_hip_status {
        if (t.m != m || t.k != k)
            return cera_fail(ctx, CERA_HIP_ERR_SHAPE, std::string(name) + ": expected [" + std::to_string(m) + " x " +
                                                          std::to_string(k) + "], got [" + std::to_string(t.m) + " x " +
                                                          std::to_string(t.k) + "]");
        if (matmul && !gemv_type_ok(t.ggml_type))
            return cera_fail(ctx, CERA_HIP_ERR_UNSUPPORTED_DTYPE,
                             std::string(name) + ": no hip GEMV kernel for ggml type " + std::to_string(t.ggml_type));
        return CERA_HIP_OK;
    };
    // The embedding / head tables may carry pad rows past vocab_size (the reference bounds token
    // ids and logits by vocab_size, not by the row count, cera/src/model/llama.rs:839-846): only
    // the first vocab rows are ever read, so only those are uploaded.
    auto vocab_rows = [&](const cera_hip_tensor& t, const char* name, bool matmul, cera_hip_tensor* cut) -> cera_hip_status {
        *cut = t;
        if (t.m > c.vocab && t.m != 0 && t.nbytes % t.m == 0) {
            cut->nbytes = t.nbytes / t.m * c.vocab;
            cut->m = c.vocab;
        }
        return expect(*cut, c.vocab, c.hidden, name, matmul);
    };
    cera_hip_tensor embd_cut, output_cut;
    CERA_TRY(vocab_rows(*token_embd, "token_embd", output == nullptr, &embd_cut));
    if (output) CERA_TRY(vocab_rows(*output, "output", true, &output_cut));
    for (uint32_t i = 0; i < c.n_layers; ++i) {
        const cera_hip_layer& L = layers[i];
        if (!L.attn_norm || !L.ffn_norm) return cera_fail(ctx, CERA_HIP_ERR_ARGUMENT, "layer norm weights missing");
        CERA_TRY(expect(L.attn_q, q_dim, c.hidden, "attn_q", true));
        CERA_TRY(expect(L.attn_k, kv_dim, c.hidden, "attn_k", true));
        CERA_TRY(expect(L.attn_v, kv_dim, c.hidden, "attn_v", true));
        CERA_TRY(expect(L.attn_output, c.hidden, q_dim, "attn_output", true));
        CERA_TRY(expect(L.ffn_gate, c.ffn, c.hidden, "ffn_gate", true));
        CERA_TRY(expect(L.ffn_up, c.ffn, c.hidden, "ffn_up", true));
        CERA_TRY(expect(L.ffn_down, c.hidden, c.ffn, "ffn_down", true));
    }

    cera_hip_model* m = new (std::nothrow) cera_hip_model();
    if (!m) return cera_fail(ctx, CERA_HIP_ERR_OOM, "host allocation failed");
    m->ctx = ctx;
    m->cfg = c;
    m->cfg.rope_freqs = nullptr;
    m->layers.resize(c.n_layers);
    uint64_t* tot = &m->bytes;
    auto build = [&]() -> cera_hip_status {
        CERA_TRY(cera_hip_tensor_upload(ctx, &embd_cut, &m->embd));
        *tot += m->embd->nbytes;
        if (output) {
            CERA_TRY(cera_hip_tensor_upload(ctx, &output_cut, &m->output));
            *tot += m->output->nbytes;
        }
        float* tmp;
        CERA_TRY(upload_f32(ctx, output_norm, c.hidden, &tmp, tot));
        m->output_norm = tmp; m->owned.push_back(tmp);
        const uint64_t kv_elems = static_cast<uint64_t>(c.n_kv_heads) * c.max_seq_len * c.head_dim;
        for (uint32_t i = 0; i < c.n_layers; ++i) {
            const cera_hip_layer& L = layers[i];
            LayerDev& D = m->layers[i];
            const cera_hip_tensor* src[7] = {&L.attn_q, &L.attn_k, &L.attn_v, &L.attn_output, &L.ffn_gate, &L.ffn_up, &L.ffn_down};
            cera_hip_dtensor** dst[7] = {&D.q, &D.k, &D.v, &D.o, &D.gate, &D.up, &D.down};
            // Q and K (and V) of one type and width share an allocation: one decode GEMV
            int fuse = 0;
            if (L.attn_q.ggml_type == L.attn_k.ggml_type && L.attn_q.ggml_type != CERA_HIP_Q5_K)
                fuse = (L.attn_v.ggml_type == L.attn_q.ggml_type) ? 3 : 2;
            if (fuse) {
                cera_hip_dtensor* views[3] = {nullptr, nullptr, nullptr};
                CERA_TRY(cera_tensor_upload_concat(ctx, src, fuse, &D.qkv, views));
                D.q = views[0]; D.k = views[1];
                if (fuse == 3) D.v = views[2];
                D.qkv_rows = static_cast<uint32_t>(D.qkv->m);
                *tot += D.qkv->nbytes;
            }
            for (int t = fuse; t < 7; ++t) {
                CERA_TRY(cera_hip_tensor_upload(ctx, src[t], dst[t]));
                *tot += (*dst[t])->nbytes;
            }
            CERA_TRY(upload_f32(ctx, L.attn_norm, c.hidden, &D.attn_norm, tot));
            CERA_TRY(upload_f32(ctx, L.ffn_norm, c.hidden, &D.ffn_norm, tot));
            if (L.q_bias && L.k_bias && L.v_bias) {
                CERA_TRY(upload_f32(ctx, L.q_bias, q_dim, &D.q_bias, tot));
                CERA_TRY(upload_f32(ctx, L.k_bias, kv_dim, &D.k_bias, tot));
                CERA_TRY(upload_f32(ctx, L.v_bias, kv_dim, &D.v_bias, tot));
            }
            if (L.q_norm && L.k_norm) {
                CERA_TRY(upload_f32(ctx, L.q_norm, c.head_dim, &D.q_norm, tot));
                CERA_TRY(upload_f32(ctx, L.k_norm, c.head_dim, &D.k_norm, tot));
            }
            CERA_TRY(alloc_kv_cache(ctx, kv_elems * sizeof(float), &D.kc, tot));
            CERA_TRY(alloc_kv_cache(ctx, kv_elems * sizeof(float), &D.vc, tot));
        }
        // frequency factors belong to the interleaved-pair layout only: the split-half rotation
        // never divides by them (cera/src/backend/cpu.rs:5031-5045, transformer.rs:1411)
        const float* ff = c.rope_type == 1 ? cfg->rope_freqs : nullptr;
        if (ff) m->rope_ff.assign(ff, ff + c.head_dim / 2);
        CERA_TRY(dev_alloc_t(ctx, c.head_dim, &tmp, tot));
        m->shift_cs = tmp; m->owned.push_back(tmp);
        std::vector<float> table;
        cera_build_rope_table(c.max_seq_len, c.head_dim, c.rope_theta, ff, table);
        CERA_TRY(upload_f32(ctx, table.data(), table.size(), &tmp, tot));
        m->rope_table = tmp; m->owned.push_back(tmp);

        const uint64_t maxk = std::max<uint64_t>(std::max(c.hidden, c.ffn), q_dim);
        auto af = [&](uint64_t n, float** p) -> cera_hip_status {
            CERA_TRY(dev_alloc_t(ctx, n, p, tot));
            m->owned.push_back(*p);
            return CERA_HIP_OK;
        };
        CERA_TRY(af(c.hidden, &m->hidden));
        CERA_TRY(af(c.hidden, &m->normed));
        CERA_TRY(af(q_dim + 2 * kv_dim, &m->q));  // q | k | v contiguous: the fused GEMV writes them in one go
        m->k = m->q + q_dim;
        m->v = m->k + kv_dim;
        CERA_TRY(af(q_dim, &m->attn_out));
        CERA_TRY(af(c.hidden, &m->proj));
        CERA_TRY(af(c.ffn, &m->act));
        CERA_TRY(af(c.ffn, &m->up));
        CERA_TRY(af(maxk / 32, &m->xs));
        CERA_TRY(af(c.vocab, &m->logits));
        CERA_TRY(dev_alloc_t(ctx, maxk, &m->xq, tot));
        m->owned.push_back(m->xq);
        CERA_TRY(dev_alloc_t(ctx, 4, &m->scalars, tot));  // [token, pos, argmax, spare]
        m->owned.push_back(m->scalars);
        // last, from what is left: the decode copies
        return build_decode_copies(m);
    };
    cera_hip_status st = build();
    if (st != CERA_HIP_OK) {
        std::string keep = ctx->err;
        free_model(m);
        ctx->err = keep;
        return st;
    }
    *out = m;
    return CERA_HIP_OK;
}

extern "C" void cera_hip_model_destroy(cera_hip_model* m) { free_model(m); }
extern "C" uint64_t cera_hip_decode_copy_reserve_bytes(const cera_hip_config* cfg) { return cfg ? cera_copy_reserve_bytes(*cfg) : 0; }
extern "C" uint64_t cera_hip_decode_copy_plan(const uint64_t* copy_bytes, uint32_t n, uint64_t free_bytes, uint64_t reserve_bytes,
                                              uint8_t* take) {
    return copy_bytes ? cera_plan_decode_copies(copy_bytes, n, free_bytes, reserve_bytes, take) : 0;
}
extern "C" cera_hip_status cera_hip_drop_decode_copies(cera_hip_model* m, uint64_t* freed_bytes) {
    if (!m) return CERA_HIP_ERR_ARGUMENT;
    ModelLock lk(m);
    const uint64_t f = cera_model_drop_decode_copies(m);
    if (freed_bytes) *freed_bytes = f;
    return CERA_HIP_OK;
}
extern "C" uint32_t cera_hip_seq_len(const cera_hip_model* m) { return m ? m->seq_len : 0; }
extern "C" uint64_t cera_hip_memory_bytes(const cera_hip_model* m) { return m ? m->bytes : 0; }

extern "C" cera_hip_status cera_hip_truncate_kv(cera_hip_model* m, uint32_t len) {
    if (!m) return CERA_HIP_ERR_ARGUMENT;
    ModelLock lk(m);
    if (len < m->seq_len) m->seq_len = len;  // rows past len are simply overwritten later
    return CERA_HIP_OK;
}

// LlamaModel::shift_kv -> InferenceState::shift_kv_with_rope (cera/src/model/llama.rs:1727-1738,
// cera/src/kv_cache.rs:1091-1310): drop cache cells [n_keep, n_keep + shift), move the tail down
// and re-rotate its K rows by R(-shift) so their encoded position matches their new index.
extern "C" cera_hip_status cera_hip_shift_kv(cera_hip_model* m, uint32_t n_keep, uint32_t shift) {
    if (!m) return CERA_HIP_ERR_ARGUMENT;
    ModelLock lk(m);
    cera_hip_ctx* ctx = m->ctx;
    const cera_hip_config& c = m->cfg;
    if (shift == 0) return cera_fail(ctx, CERA_HIP_ERR_ARGUMENT, "shift_kv: shift must be > 0");
    if (static_cast<uint64_t>(n_keep) + shift > m->seq_len)
        return cera_fail(ctx, CERA_HIP_ERR_POSITION, "shift_kv: n_keep=" + std::to_string(n_keep) + " + shift=" +
                                                         std::to_string(shift) + " > seq_len=" + std::to_string(m->seq_len));
    const uint32_t new_len = m->seq_len - shift, tail = new_len - n_keep, src_row = n_keep + shift;
    if (tail) {
        // delta rotation: theta_0 = -(shift) as f32, the forward pass's recurrence and factors
        std::vector<float> row;
        {
            const uint32_t half = c.head_dim / 2;
            row.resize(2 * half);
            const float theta_scale = powf(c.rope_theta, -2.0f / static_cast<float>(c.head_dim));
            float theta = static_cast<float>(-static_cast<int32_t>(shift));
            for (uint32_t i = 0; i < half; ++i) {
                // NEOX never divides by frequency factors (cera/src/backend/cpu.rs:5065-5086)
                const float ang = (c.rope_type == 1 && !m->rope_ff.empty()) ? theta / m->rope_ff[i] : theta;
                row[2 * i] = cosf(ang);
                row[2 * i + 1] = sinf(ang);
                theta *= theta_scale;
            }
        }
        CERA_TRY(cera_hip_upload(ctx, m->shift_cs, row.data(), row.size() * 4));
        const uint64_t head_stride = static_cast<uint64_t>(c.max_seq_len) * c.head_dim;
        const dim3 grid((tail * (c.head_dim / 8) + 255) / 256, c.n_kv_heads), block(256);
        const bool overlap = tail > shift;   // source and destination rows intersect: go through staging
        void* stage = nullptr;
        const uint64_t stage_stride = static_cast<uint64_t>(tail) * c.head_dim;
        if (overlap) {
            CERA_TRY(cera_scratch(ctx, 5, stage_stride * c.n_kv_heads * sizeof(float), &stage));
        }
        auto run = [&](auto* tag, auto hd_tag) {
            using KV = std::remove_pointer_t<decltype(tag)>;
            constexpr int HD = decltype(hd_tag)::value;
            for (LayerDev& L : m->layers) {
                for (int is_v = 0; is_v < 2; ++is_v) {
                    KV* cache = static_cast<KV*>(is_v ? L.vc : L.kc);
                    const float* cs = is_v ? nullptr : m->shift_cs;
                    if (!overlap) {
                        hipLaunchKernelGGL((kv_shift_kernel<KV, HD>), grid, block, 0, ctx->stream, cache, cache, src_row,
                                           n_keep, tail, head_stride, head_stride, cs, c.rope_type);
                    } else {
                        hipLaunchKernelGGL((kv_shift_kernel<KV, HD>), grid, block, 0, ctx->stream, cache,
                                           static_cast<KV*>(stage), src_row, 0u, tail, head_stride, stage_stride, cs,
                                           c.rope_type);
                        hipLaunchKernelGGL((kv_shift_kernel<KV, HD>), grid, block, 0, ctx->stream, static_cast<KV*>(stage),
                                           cache, 0u, n_keep, tail, stage_stride, head_stride,
                                           static_cast<const float*>(nullptr), c.rope_type);
                    }
                }
            }
        };
        auto run_hd = [&](auto hd_tag) {
            if (m->kv_f16) run(static_cast<kv_half*>(nullptr), hd_tag);
            else run(static_cast<float*>(nullptr), hd_tag);
        };
        switch (c.head_dim) {
            case 128: run_hd(std::integral_constant<int, 128>{}); break;
            case 64: run_hd(std::integral_constant<int, 64>{}); break;
            case 32: run_hd(std::integral_constant<int, 32>{}); break;
            case 80: run_hd(std::integral_constant<int, 80>{}); break;
            case 96: run_hd(std::integral_constant<int, 96>{}); break;
            case 256: run_hd(std::integral_constant<int, 256>{}); break;
            default: return cera_fail(ctx, CERA_HIP_ERR_SHAPE, "shift_kv: head_dim must be one of 32, 64, 80, 96, 128, 256");
        }
        HIP_TRY(ctx, hipGetLastError());
        HIP_TRY(ctx, hipStreamSynchronize(ctx->stream));
    }
    m->seq_len = new_len;
    return CERA_HIP_OK;
}

// Prefix-cache snapshots (Model::snapshot_state / restore_state, cera/src/model/mod.rs:507-533;
// layer layout LayerSnapshot::Attention, cera/src/kv_cache.rs:1382-1396): a layer's K and V as
// time-major [n_pos][kv_dim] f32, the CPU state's own layout.  cera_hip_read_kv is the snapshot
// side; this is the restore side.  Call it for every layer, then cera_hip_set_seq_len.
extern "C" cera_hip_status cera_hip_write_kv(cera_hip_model* m, uint32_t layer, const float* k, const float* v,
                                             uint32_t n_pos) {
    if (!m || (n_pos && (!k || !v)) || layer >= m->cfg.n_layers) return CERA_HIP_ERR_ARGUMENT;
    ModelLock lk(m);
    const cera_hip_config& c = m->cfg;
    if (n_pos > c.max_seq_len) return cera_fail(m->ctx, CERA_HIP_ERR_POSITION, "write_kv: more positions than max_seq_len");
    const uint64_t per_head = static_cast<uint64_t>(c.max_seq_len) * c.head_dim;
    const uint64_t kv_dim = static_cast<uint64_t>(c.n_kv_heads) * c.head_dim;
    std::vector<float> hk(static_cast<uint64_t>(n_pos) * c.head_dim), hv(hk.size());
    std::vector<kv_half> h16;
    const uint64_t esz = m->kv_f16 ? sizeof(kv_half) : sizeof(float);
    auto put = [&](void* cache, uint32_t h, const std::vector<float>& rows) -> cera_hip_status {
        char* dst = static_cast<char*>(cache) + h * per_head * esz;
        if (!m->kv_f16) return cera_hip_upload(m->ctx, dst, rows.data(), rows.size() * 4);
        h16.resize(rows.size());
        for (size_t i = 0; i < rows.size(); ++i) h16[i] = static_cast<kv_half>(rows[i]);   // round to nearest even
        return cera_hip_upload(m->ctx, dst, h16.data(), h16.size() * sizeof(kv_half));
    };
    for (uint32_t h = 0; h < c.n_kv_heads && n_pos; ++h) {
        for (uint32_t t = 0; t < n_pos; ++t) {
            std::memcpy(hk.data() + static_cast<uint64_t>(t) * c.head_dim, k + t * kv_dim + h * c.head_dim, c.head_dim * 4);
            std::memcpy(hv.data() + static_cast<uint64_t>(t) * c.head_dim, v + t * kv_dim + h * c.head_dim, c.head_dim * 4);
        }
        CERA_TRY(put(m->layers[layer].kc, h, hk));
        CERA_TRY(put(m->layers[layer].vc, h, hv));
    }
    return CERA_HIP_OK;
}

extern "C" cera_hip_status cera_hip_set_seq_len(cera_hip_model* m, uint32_t len) {
    if (!m) return CERA_HIP_ERR_ARGUMENT;
    ModelLock lk(m);
    if (len > m->cfg.max_seq_len) return cera_fail(m->ctx, CERA_HIP_ERR_POSITION, "set_seq_len: beyond max_seq_len");
    m->seq_len = len;
    return CERA_HIP_OK;
}

// Model::configure_kv_compression for the modes this backend has (cera/src/model/mod.rs:557-592,
// KvCompression::{None, F16}, cera/src/kv_cache.rs:88-98): called before the first forward pass;
// the first call wins, the same mode again is a no-op, a different one a conflict.  Switching
// re-allocates the (still empty) caches at the new element width.
extern "C" cera_hip_status cera_hip_configure_kv(cera_hip_model* m, uint32_t kv_type) {
    if (!m) return CERA_HIP_ERR_ARGUMENT;
    ModelLock lk(m);
    cera_hip_ctx* ctx = m->ctx;
    if (kv_type > CERA_HIP_KV_F16) return cera_fail(ctx, CERA_HIP_ERR_ARGUMENT, "configure_kv: unknown cache type");
    const bool want_f16 = kv_type == CERA_HIP_KV_F16;
    if (m->kv_broken) return cera_fail(ctx, CERA_HIP_ERR_DEVICE, "configure_kv: an earlier cache re-allocation failed; the model is unusable");
    if (m->kv_configured && want_f16 != m->kv_f16)
        return cera_fail(ctx, CERA_HIP_ERR_ARGUMENT, "configure_kv: the KV cache is already configured for another mode");
    if (want_f16 == m->kv_f16) { m->kv_configured = true; return CERA_HIP_OK; }
    if (m->seq_len != 0) return cera_fail(ctx, CERA_HIP_ERR_POSITION, "configure_kv: the cache already holds positions");
    const cera_hip_config& c = m->cfg;
    const uint64_t kv_elems = static_cast<uint64_t>(c.n_kv_heads) * c.max_seq_len * c.head_dim;
    const uint64_t old_bytes = kv_elems * (m->kv_f16 ? sizeof(kv_half) : sizeof(float));
    const uint64_t new_bytes = kv_elems * (want_f16 ? sizeof(kv_half) : sizeof(float));
    HIP_TRY(ctx, hipStreamSynchronize(ctx->stream));
    // A failure part-way leaves layers with caches of different widths: the model is then marked
    // unusable (every later forward / configure call fails) instead of running on them.
    auto swap_all = [&]() -> cera_hip_status {
        for (LayerDev& L : m->layers) {
            for (void** cache : {&L.kc, &L.vc}) {
                if (*cache) HIP_TRY(ctx, hipFree(*cache));
                *cache = nullptr;
                m->bytes -= old_bytes;
                CERA_TRY(alloc_kv_cache(ctx, new_bytes, cache, &m->bytes));
            }
        }
        return CERA_HIP_OK;
    };
    const cera_hip_status st = swap_all();
    if (st != CERA_HIP_OK) { m->kv_broken = true; return st; }
    m->kv_f16 = want_f16;
    m->kv_configured = true;
    return CERA_HIP_OK;
}

extern "C" cera_hip_status cera_hip_set_reference_order(cera_hip_model* m, uint32_t on) {
    if (!m) return CERA_HIP_ERR_ARGUMENT;
    ModelLock lk(m);
    if (m->seq_len != 0) return cera_fail(m->ctx, CERA_HIP_ERR_POSITION, "set_reference_order: the cache already holds positions");
    std::string why;
    if (on && !cera_model_ref_order_supported(m, &why))
        return cera_fail(m->ctx, CERA_HIP_ERR_UNSUPPORTED_DTYPE, "set_reference_order: " + why);
    m->ref_order = on >= 2 ? 2u : on;
    return CERA_HIP_OK;
}
extern "C" uint32_t cera_hip_reference_order(const cera_hip_model* m) { return m ? m->ref_order : 0u; }

extern "C" uint32_t cera_hip_kv_type(const cera_hip_model* m) { return m && m->kv_f16 ? CERA_HIP_KV_F16 : CERA_HIP_KV_F32; }

// ---------------------------------------------------------------------------
// One projection: int8 kernels read the quantized activations, Q5_K the f32 ones.
// y = resid + W . (xs, xq): one wavefront per row where a row fits one (the O projection) or a few
// passes of one (the down projection), the K-split kernel otherwise.  All three give the same bits.
static cera_hip_status launch_proj_add(cera_hip_ctx* ctx, const cera_hip_dtensor* w, const float* xs, const int8_t* xq, float* y,
                                       const float* resid) {
    bool done = false;
    CERA_TRY(cera_launch_row_gemv_add(ctx, w, xs, xq, y, resid, &done));
    if (!done) CERA_TRY(cera_launch_row_gemv_long_add(ctx, w, xs, xq, y, resid, &done));
    if (done) return CERA_HIP_OK;
    return cera_launch_gemv(ctx, w, nullptr, xs, xq, y, resid, CERA_EPI_ADD);
}

// y = W . (xs, xq): from the decode copy where the matrix has one, else the K-split kernel.
static cera_hip_status launch_proj_store(cera_hip_ctx* ctx, const cera_hip_dtensor* w, const float* xs, const int8_t* xq, float* y) {
    bool done = false;
    CERA_TRY(cera_launch_row_gemv_store(ctx, w, xs, xq, y, &done));
    if (done) return CERA_HIP_OK;
    return cera_launch_gemv(ctx, w, nullptr, xs, xq, y, nullptr, CERA_EPI_STORE);
}

static cera_hip_status project(cera_hip_model* m, const cera_hip_dtensor* w, const float* x_f32, float* y,
                               const float* resid) {
    cera_hip_ctx* ctx = m->ctx;
    const float rs = m->cfg.residual_scale;
    if (w->dtype == CERA_HIP_Q5_K) {
        float* dst = resid ? m->proj : y;
        CERA_TRY(cera_launch_gemv_q5k_f32(ctx, w, x_f32, dst));
        if (resid) {
            hipLaunchKernelGGL(add_kernel, dim3((w->m + 255) / 256), dim3(256), 0, ctx->stream, resid, dst, rs,
                               static_cast<uint32_t>(w->m), y);
            HIP_TRY(ctx, hipGetLastError());
        }
        return CERA_HIP_OK;
    }
    if (resid && rs != 1.0f) {
        CERA_TRY(cera_launch_gemv(ctx, w, nullptr, m->xs, m->xq, m->proj, nullptr, CERA_EPI_STORE));
        hipLaunchKernelGGL(add_kernel, dim3((w->m + 255) / 256), dim3(256), 0, ctx->stream, resid, m->proj, rs,
                           static_cast<uint32_t>(w->m), y);
        HIP_TRY(ctx, hipGetLastError());
        return CERA_HIP_OK;
    }
    if (resid) return launch_proj_add(ctx, w, m->xs, m->xq, y, resid);
    return launch_proj_store(ctx, w, m->xs, m->xq, y);
}

// rmsnorm of `rows` rows of n elements with the Q8_0 quantization of the result fused in
// (cpu::rmsnorm then quantize_f32_to_q8_0, cera/src/backend/cpu.rs:2479-2496, 942-958).  A single
// row of up to 16384 elements (the decode step) runs the register-resident one-pass kernel.
static cera_hip_status launch_norm_quant(cera_hip_ctx* ctx, const float* x, const float* w, uint32_t n, uint32_t rows,
                                         float eps, float* y, float* xs, int8_t* xq) {
    if (rows == 1 && n <= 16384)
        hipLaunchKernelGGL((rmsnorm_row_kernel<true>), dim3(1), dim3(1024), 0, ctx->stream, x, w, n, eps, y, xs, xq);
    else
        hipLaunchKernelGGL((rmsnorm_kernel<true>), dim3(rows), dim3(256), 0, ctx->stream, x, w, n, eps, y, xs, xq,
                           static_cast<float*>(nullptr));
    HIP_TRY(ctx, hipGetLastError());
    return CERA_HIP_OK;
}
static cera_hip_status norm_quant(cera_hip_model* m, const float* x, const float* w, uint32_t n, uint32_t rows, float* y) {
    return launch_norm_quant(m->ctx, x, w, n, rows, m->cfg.rms_eps, y, m->xs, m->xq);
}

// The attention step of one decode layer: RoPE on q and the new K row, append of the new K/V rows
// to the cache at `pos`, attention over positions [0, pos], and the Q8_0 quantization of the
// result for the O projection (the merge kernel writes both).  While the context is short the
// attention kernel rotates q on load, takes the new token's K/V rows from the projections
// (rotating K) and appends them to the cache itself; longer contexts run RoPE + append as their
// own launch, then plain attention.  q / k_new are rotated in place only on the second route.
cera_hip_status cera_attn_step(cera_hip_ctx* ctx, float* q, float* k_new, const float* v_new, void* kc, void* vc,
                               const float* rope_table, const uint32_t* pos_dev, uint32_t pos, uint32_t n_heads,
                               uint32_t n_kv_heads, uint32_t head_dim, uint32_t max_seq, uint32_t rope_type, float scale,
                               bool kv_f16, float* out, float* out_scales, int8_t* out_quants) {
    hipStream_t s = ctx->stream;
    if (pos + 1 < ATTN_FUSED_NEW_KV_MAX_KEYS && cera_attn_shape_tuned(n_heads, n_kv_heads, head_dim)) {
        AttnNewKV nk;
        nk.rope_row = rope_table + static_cast<uint64_t>(pos) * head_dim;
        nk.rope_type = rope_type;
        nk.k_new = k_new;
        nk.v_new = v_new;
        nk.kc_w = kc;
        nk.vc_w = vc;
        return cera_launch_attn_decode(ctx, q, kc, vc, n_heads, n_kv_heads, head_dim, pos + 1, max_seq, scale, 0, out,
                                       out_scales, out_quants, &nk, kv_f16);
    }
    const dim3 rgrid(n_heads + 2 * n_kv_heads, 1), rblock(head_dim / 2);
    if (kv_f16)
        hipLaunchKernelGGL(rope_kv_kernel<kv_half>, rgrid, rblock, 0, s, q, k_new, v_new, rope_table, pos_dev, n_heads,
                           n_kv_heads, head_dim, rope_type, static_cast<kv_half*>(kc), static_cast<kv_half*>(vc), max_seq);
    else
        hipLaunchKernelGGL(rope_kv_kernel<float>, rgrid, rblock, 0, s, q, k_new, v_new, rope_table, pos_dev, n_heads,
                           n_kv_heads, head_dim, rope_type, static_cast<float*>(kc), static_cast<float*>(vc), max_seq);
    HIP_TRY(ctx, hipGetLastError());
    return cera_launch_attn_decode(ctx, q, kc, vc, n_heads, n_kv_heads, head_dim, pos + 1, max_seq, scale, 0, out, out_scales,
                                   out_quants, nullptr, kv_f16);
}

// The per-token layer stack: LlamaModel::run_layers + project_logits.  The first launch puts the
// token id and position into m->scalars[0..1], where the kernels behind it read the position.
static cera_hip_status set_token_pos(cera_hip_model* m, uint32_t token, uint32_t pos);

static cera_hip_status decode_step(cera_hip_model* m, uint32_t token, uint32_t pos, bool want_logits) {
    if (m->ref_order) {
        CERA_TRY(set_token_pos(m, token, pos));
        return cera_model_decode_step_ref(m, pos, want_logits);
    }
    cera_hip_ctx* ctx = m->ctx;
    const cera_hip_config& c = m->cfg;
    hipStream_t s = ctx->stream;
    const uint32_t q_dim = c.n_heads * c.head_dim, kv_dim = c.n_kv_heads * c.head_dim;
    const float scale = c.attn_scale != 0.0f ? c.attn_scale : 1.0f / std::sqrt(static_cast<float>(c.head_dim));

    hipLaunchKernelGGL(embed_token_kernel, dim3((c.hidden + 255) / 256), dim3(256), 0, s, m->embd->dtype, m->embd->dev,
                       m->embd->row_bytes, token, pos, m->scalars, c.hidden, c.embed_scale, m->hidden);
    HIP_TRY(ctx, hipGetLastError());

    for (uint32_t i = 0; i < c.n_layers; ++i) {
        LayerDev& L = m->layers[i];
        // Q|K|V with the attention norm and its Q8_0 quantization done by the projection's own
        // workgroups (one launch instead of two), where the shapes allow
        bool qkv_done = false;
        if (L.qkv)
            CERA_TRY(cera_launch_qkv_fused(ctx, L.qkv, L.qkv_rows == q_dim + kv_dim ? L.v : nullptr, m->hidden, L.attn_norm,
                                           c.rms_eps, m->q, m->v, &qkv_done));
        if (qkv_done) {
        } else if (L.qkv) {
            CERA_TRY(norm_quant(m, m->hidden, L.attn_norm, c.hidden, 1, m->normed));
            bool paired = false;
            // Q|K in one block type and V in another (the Q4_K_M mix): still one launch where a
            // paired kernel instance exists
            if (L.qkv_rows == q_dim + kv_dim)
                CERA_TRY(cera_launch_gemv_pair(ctx, L.qkv, L.v, m->xs, m->xq, m->q, m->v, &paired));
            if (!paired) {
                CERA_TRY(project(m, L.qkv, m->normed, m->q, nullptr));
                if (L.qkv_rows == q_dim + kv_dim) CERA_TRY(project(m, L.v, m->normed, m->v, nullptr));
            }
        } else {
            CERA_TRY(norm_quant(m, m->hidden, L.attn_norm, c.hidden, 1, m->normed));
            CERA_TRY(project(m, L.q, m->normed, m->q, nullptr));
            CERA_TRY(project(m, L.k, m->normed, m->k, nullptr));
            CERA_TRY(project(m, L.v, m->normed, m->v, nullptr));
        }
        if (L.q_bias) {
            hipLaunchKernelGGL(bias_kernel, dim3((q_dim + 255) / 256), dim3(256), 0, s, m->q, L.q_bias, q_dim);
            hipLaunchKernelGGL(bias_kernel, dim3((kv_dim + 255) / 256), dim3(256), 0, s, m->k, L.k_bias, kv_dim);
            hipLaunchKernelGGL(bias_kernel, dim3((kv_dim + 255) / 256), dim3(256), 0, s, m->v, L.v_bias, kv_dim);
        }
        if (L.q_norm) {
            hipLaunchKernelGGL((rmsnorm_kernel<false>), dim3(c.n_heads), dim3(256), 0, s, m->q, L.q_norm, c.head_dim,
                               c.rms_eps, m->q, nullptr, nullptr, nullptr);
            hipLaunchKernelGGL((rmsnorm_kernel<false>), dim3(c.n_kv_heads), dim3(256), 0, s, m->k, L.k_norm, c.head_dim,
                               c.rms_eps, m->k, nullptr, nullptr, nullptr);
        }
        CERA_TRY(cera_attn_step(ctx, m->q, m->k, m->v, L.kc, L.vc, m->rope_table, m->scalars + 1, pos, c.n_heads, c.n_kv_heads,
                                c.head_dim, c.max_seq_len, c.rope_type, scale, m->kv_f16, m->attn_out, m->xs, m->xq));
        CERA_TRY(project(m, L.o, m->attn_out, m->hidden, m->hidden));

        // gate | up with the FFN norm in front and SwiGLU + the down projection's Q8_0 quantization
        // behind, all in one launch instead of three, where the shapes allow
        bool ffn_done = false;
        CERA_TRY(cera_launch_ffn_gate_up_fused(ctx, L.gate, L.up, m->hidden, L.ffn_norm, c.rms_eps, m->xq, m->xs, &ffn_done));
        const bool fuse = L.gate->dtype == L.up->dtype && L.gate->dtype != CERA_HIP_Q5_K;
        if (!ffn_done) CERA_TRY(norm_quant(m, m->hidden, L.ffn_norm, c.hidden, 1, m->normed));
        if (ffn_done) {
        } else if (fuse) {
            CERA_TRY(cera_launch_gemv(ctx, L.gate, L.up, m->xs, m->xq, m->act, nullptr, CERA_EPI_SILU_MUL));
            CERA_TRY(cera_launch_quantize(ctx, m->act, c.ffn, m->xs, m->xq));
        } else {
            CERA_TRY(project(m, L.gate, m->normed, m->act, nullptr));
            CERA_TRY(project(m, L.up, m->normed, m->up, nullptr));
            hipLaunchKernelGGL((silu_mul_kernel<true>), dim3((c.ffn / 4 + 255) / 256), dim3(256), 0, s, m->act, m->up,
                               static_cast<uint64_t>(c.ffn), m->act, m->xs, m->xq, static_cast<float*>(nullptr));
            HIP_TRY(ctx, hipGetLastError());
        }
        CERA_TRY(project(m, L.down, m->act, m->hidden, m->hidden));
    }
    // final norm in place (run_layers ends with rmsnorm(hidden, output_norm))
    CERA_TRY(norm_quant(m, m->hidden, m->output_norm, c.hidden, 1, m->hidden));
    if (want_logits) {
        const cera_hip_dtensor* o = m->output ? m->output : m->embd;
        CERA_TRY(project(m, o, m->hidden, m->logits, nullptr));
        if (c.logit_scale != 1.0f) {
            hipLaunchKernelGGL(scale_kernel, dim3((c.vocab + 255) / 256), dim3(256), 0, s, m->logits,
                               1.0f / c.logit_scale, c.vocab);
            HIP_TRY(ctx, hipGetLastError());
        }
    }
    return CERA_HIP_OK;
}

// A call at position 0 starts a fresh sequence: callers hand a new InferenceState to every
// generate(), and a device-resident backend resets its own counter then, as the reference's do
// (cera/src/model/metal_lfm2.rs:4091-4096, gpu_lfm2.rs:3755-3762).  Cached rows are simply
// overwritten.
static cera_hip_status begin_at(cera_hip_model* m, uint32_t pos) {
    if (m->kv_broken) return cera_fail(m->ctx, CERA_HIP_ERR_DEVICE, "the model's KV cache is unusable (a cache re-allocation failed)");
    if (pos == 0) m->seq_len = 0;
    return CERA_HIP_OK;
}

static cera_hip_status check_step(cera_hip_model* m, uint32_t token, uint32_t pos) {
    CERA_TRY(begin_at(m, pos));
    if (token >= m->cfg.vocab)
        return cera_fail(m->ctx, CERA_HIP_ERR_ARGUMENT, "token id " + std::to_string(token) + " out of range (vocab " + std::to_string(m->cfg.vocab) + ")");
    if (pos != m->seq_len)
        return cera_fail(m->ctx, CERA_HIP_ERR_POSITION, "pos " + std::to_string(pos) + " != seq_len " + std::to_string(m->seq_len));
    if (pos >= m->cfg.max_seq_len)
        return cera_fail(m->ctx, CERA_HIP_ERR_POSITION, "context full: pos " + std::to_string(pos) + " >= max_seq_len " + std::to_string(m->cfg.max_seq_len));
    return CERA_HIP_OK;
}

// Kernel arguments are captured at launch, so (unlike an async copy from a
// stack variable) the values cannot change under a launch that is still queued.
static __global__ void set_token_pos_kernel(uint32_t* scalars, uint32_t token, uint32_t pos) {
    scalars[0] = token;
    scalars[1] = pos;
}
static cera_hip_status set_token_pos(cera_hip_model* m, uint32_t token, uint32_t pos) {
    hipLaunchKernelGGL(set_token_pos_kernel, dim3(1), dim3(1), 0, m->ctx->stream, m->scalars, token, pos);
    HIP_TRY(m->ctx, hipGetLastError());
    return CERA_HIP_OK;
}

extern "C" cera_hip_status cera_hip_forward(cera_hip_model* m, uint32_t token, uint32_t pos, float* logits) {
    if (!m || !logits) return CERA_HIP_ERR_ARGUMENT;
    ModelLock lk(m);
    CERA_TRY(check_step(m, token, pos));
    CERA_TRY(decode_step(m, token, pos, true));
    CERA_TRY(cera_hip_download(m->ctx, logits, m->logits, static_cast<uint64_t>(m->cfg.vocab) * 4));
    m->seq_len = pos + 1;
    return CERA_HIP_OK;
}

extern "C" cera_hip_status cera_hip_forward_greedy(cera_hip_model* m, uint32_t token, uint32_t pos, uint32_t* next) {
    if (!m || !next) return CERA_HIP_ERR_ARGUMENT;
    ModelLock lk(m);
    CERA_TRY(check_step(m, token, pos));
    CERA_TRY(decode_step(m, token, pos, true));
    // the argmax kernel writes the token into pinned host memory itself: no copy launch behind it
    uint32_t *word_host, *word_dev;
    CERA_TRY(cera_pinned_word(m->ctx, &word_host, &word_dev));
    CERA_TRY(cera_launch_argmax(m->ctx, m->logits, m->cfg.vocab, m->scalars + 2, word_dev));
    HIP_TRY(m->ctx, hipStreamSynchronize(m->ctx->stream));
    *next = *static_cast<volatile uint32_t*>(word_host);
    m->seq_len = pos + 1;
    return CERA_HIP_OK;
}

extern "C" cera_hip_status cera_hip_forward_prefill(cera_hip_model* m, const uint32_t* tokens, uint32_t n,
                                                    uint32_t start_pos, float* last_logits) {
    if (!m || !tokens || !last_logits) return CERA_HIP_ERR_ARGUMENT;
    if (n == 0) return cera_fail(m->ctx, CERA_HIP_ERR_ARGUMENT, "forward_prefill requires at least one token");
    ModelLock lk(m);
    CERA_TRY(begin_at(m, start_pos));
    if (start_pos != m->seq_len)
        return cera_fail(m->ctx, CERA_HIP_ERR_POSITION, "forward_prefill: start_pos " + std::to_string(start_pos) +
                                                            " must equal seq_len " + std::to_string(m->seq_len));
    if (static_cast<uint64_t>(start_pos) + n > m->cfg.max_seq_len)
        return cera_fail(m->ctx, CERA_HIP_ERR_POSITION, "forward_prefill: prompt does not fit max_seq_len");
    for (uint32_t i = 0; i < n; ++i)
        if (tokens[i] >= m->cfg.vocab) return cera_fail(m->ctx, CERA_HIP_ERR_ARGUMENT, "token id out of range");
    return cera_model_prefill(m, tokens, n, start_pos, last_logits);
}

extern "C" cera_hip_status cera_hip_forward_prefill_logits_all(cera_hip_model* m, const uint32_t* tokens, uint32_t n,
                                                               uint32_t start_pos, float* logits_all) {
    if (!m || !tokens || !logits_all) return CERA_HIP_ERR_ARGUMENT;
    if (n == 0) return cera_fail(m->ctx, CERA_HIP_ERR_ARGUMENT, "forward_prefill_logits_all requires at least one token");
    ModelLock lk(m);
    CERA_TRY(begin_at(m, start_pos));
    if (start_pos != m->seq_len)
        return cera_fail(m->ctx, CERA_HIP_ERR_POSITION, "forward_prefill_logits_all: start_pos " + std::to_string(start_pos) +
                                                            " must equal seq_len " + std::to_string(m->seq_len));
    if (static_cast<uint64_t>(start_pos) + n > m->cfg.max_seq_len)
        return cera_fail(m->ctx, CERA_HIP_ERR_POSITION, "forward_prefill_logits_all: tokens do not fit max_seq_len");
    for (uint32_t i = 0; i < n; ++i)
        if (tokens[i] >= m->cfg.vocab) return cera_fail(m->ctx, CERA_HIP_ERR_ARGUMENT, "token id out of range");
    return cera_model_prefill_logits_all(m, tokens, n, start_pos, logits_all);
}

// one decode step with the logits copied out (the per-token route of the all-logits call)
cera_hip_status cera_model_decode_logits(cera_hip_model* m, uint32_t token, uint32_t pos, float* logits) {
    CERA_TRY(decode_step(m, token, pos, true));
    m->seq_len = pos + 1;
    return cera_hip_download(m->ctx, logits, m->logits, static_cast<uint64_t>(m->cfg.vocab) * 4);
}

// Token-at-a-time prefill (LlamaModel::forward_prefill's per-token route,
// cera/src/model/llama.rs:1643-1648); the batched route replaces it when the
// weight types support the int8 GEMM.
cera_hip_status cera_model_prefill_per_token(cera_hip_model* m, const uint32_t* tokens, uint32_t n,
                                             uint32_t start_pos, float* last_logits) {
    for (uint32_t i = 0; i < n; ++i) {
        CERA_TRY(decode_step(m, tokens[i], start_pos + i, i + 1 == n));
        m->seq_len = start_pos + i + 1;
    }
    return cera_hip_download(m->ctx, last_logits, m->logits, static_cast<uint64_t>(m->cfg.vocab) * 4);
}

extern "C" cera_hip_status cera_hip_read_kv(cera_hip_model* m, uint32_t layer, float* k_out, float* v_out) {
    if (!m || !k_out || !v_out || layer >= m->cfg.n_layers) return CERA_HIP_ERR_ARGUMENT;
    ModelLock lk(m);
    const cera_hip_config& c = m->cfg;
    const uint64_t per_head = static_cast<uint64_t>(c.max_seq_len) * c.head_dim;
    std::vector<float> hk(static_cast<uint64_t>(m->seq_len) * c.head_dim), hv(hk.size());
    const uint64_t kv_dim = static_cast<uint64_t>(c.n_kv_heads) * c.head_dim;
    std::vector<kv_half> h16;
    const uint64_t esz = m->kv_f16 ? sizeof(kv_half) : sizeof(float);
    // a half cache is widened (exactly) to the f32 the caller sees
    auto get = [&](const void* cache, uint32_t h, std::vector<float>& rows) -> cera_hip_status {
        const char* src = static_cast<const char*>(cache) + h * per_head * esz;
        if (!m->kv_f16) return cera_hip_download(m->ctx, rows.data(), src, rows.size() * 4);
        h16.resize(rows.size());
        CERA_TRY(cera_hip_download(m->ctx, h16.data(), src, h16.size() * sizeof(kv_half)));
        for (size_t i = 0; i < rows.size(); ++i) rows[i] = static_cast<float>(h16[i]);
        return CERA_HIP_OK;
    };
    for (uint32_t h = 0; h < c.n_kv_heads; ++h) {
        CERA_TRY(get(m->layers[layer].kc, h, hk));
        CERA_TRY(get(m->layers[layer].vc, h, hv));
        for (uint32_t t = 0; t < m->seq_len; ++t) {
            std::memcpy(k_out + t * kv_dim + h * c.head_dim, hk.data() + static_cast<uint64_t>(t) * c.head_dim, c.head_dim * 4);
            std::memcpy(v_out + t * kv_dim + h * c.head_dim, hv.data() + static_cast<uint64_t>(t) * c.head_dim, c.head_dim * 4);
        }
    }
    return CERA_HIP_OK;
}

extern "C" cera_hip_status cera_hip_read_hidden(cera_hip_model* m, float* hidden_out) {
    if (!m || !hidden_out) return CERA_HIP_ERR_ARGUMENT;
    ModelLock lk(m);
    return cera_hip_download(m->ctx, hidden_out, m->hidden, static_cast<uint64_t>(m->cfg.hidden) * 4);
}

// cpu::rope / cpu::rope_norm on host buffers (test entry point).
extern "C" cera_hip_status cera_hip_rope(cera_hip_ctx* ctx, float* q, float* k, uint32_t pos, uint32_t n_heads,
                                         uint32_t n_kv_heads, uint32_t head_dim, float freq_base, uint32_t rope_type,
                                         const float* freq_factors) {
    if (!ctx || !q || !k) return CERA_HIP_ERR_ARGUMENT;
    if (head_dim == 0 || head_dim % 2 || head_dim > 2048 || rope_type > 1) return cera_fail(ctx, CERA_HIP_ERR_SHAPE, "rope: bad head_dim or rope_type");
    std::lock_guard<std::recursive_mutex> lk(ctx->op_mu);
    std::vector<float> table;
    cera_build_rope_table(pos + 1, head_dim, freq_base, rope_type == 1 ? freq_factors : nullptr, table);
    const uint64_t half = head_dim / 2;
    void *dq, *dk, *dt, *dp;
    CERA_TRY(cera_scratch(ctx, 0, static_cast<uint64_t>(n_heads) * head_dim * 4, &dq));
    CERA_TRY(cera_scratch(ctx, 1, static_cast<uint64_t>(n_kv_heads) * head_dim * 4, &dk));
    CERA_TRY(cera_scratch(ctx, 2, half * 8, &dt));
    CERA_TRY(cera_scratch(ctx, 3, 4, &dp));
    uint32_t zero = 0;
    CERA_TRY(cera_hip_upload(ctx, dq, q, static_cast<uint64_t>(n_heads) * head_dim * 4));
    CERA_TRY(cera_hip_upload(ctx, dk, k, static_cast<uint64_t>(n_kv_heads) * head_dim * 4));
    CERA_TRY(cera_hip_upload(ctx, dt, table.data() + static_cast<uint64_t>(pos) * half * 2, half * 8));
    CERA_TRY(cera_hip_upload(ctx, dp, &zero, 4));
    hipLaunchKernelGGL(rope_kv_kernel<float>, dim3(n_heads + n_kv_heads), dim3(head_dim / 2), 0, ctx->stream,
                       static_cast<float*>(dq), static_cast<float*>(dk), static_cast<const float*>(nullptr),
                       static_cast<float*>(dt), static_cast<uint32_t*>(dp), n_heads, n_kv_heads, head_dim, rope_type,
                       static_cast<float*>(nullptr), static_cast<float*>(nullptr), 1u);
    HIP_TRY(ctx, hipGetLastError());
    CERA_TRY(cera_hip_download(ctx, q, dq, static_cast<uint64_t>(n_heads) * head_dim * 4));
    return cera_hip_download(ctx, k, dk, static_cast<uint64_t>(n_kv_heads) * head_dim * 4);
}

// ---- one token's projection launches on device operands (benchmarks, profiling) ---------------
extern "C" cera_hip_status cera_hip_decode_ops_dev(cera_hip_ctx* ctx, const cera_hip_decode_op* ops, uint32_t n) {
    if (!ctx || (!ops && n)) return CERA_HIP_ERR_ARGUMENT;
    std::lock_guard<std::recursive_mutex> lk(ctx->op_mu);
    // the launches below are the decode step's, so their matrices get decode copies as a model's do
    // (on first use; the handles are this library's own objects)
    for (uint32_t i = 0; i < n; ++i) {
        if (ops[i].kind > CERA_HIP_OP_NORM_GATE_UP) continue;
        CERA_TRY(cera_tensor_prepare_stream(ctx, const_cast<cera_hip_dtensor*>(ops[i].w)));
        CERA_TRY(cera_tensor_prepare_stream(ctx, const_cast<cera_hip_dtensor*>(ops[i].w2)));
    }
    for (uint32_t i = 0; i < n; ++i) {
        const cera_hip_decode_op& o = ops[i];
        auto bad = [&](const char* what) {
            return cera_fail(ctx, CERA_HIP_ERR_ARGUMENT, "decode_ops: op " + std::to_string(i) + ": " + what);
        };
        bool done = false;
        switch (o.kind) {
            case CERA_HIP_OP_GEMV:
                if (!o.w || !o.xs || !o.xq || !o.y) return bad("GEMV needs w, xs, xq, y");
                if (o.resid) CERA_TRY(launch_proj_add(ctx, o.w, o.xs, o.xq, o.y, o.resid));
                else CERA_TRY(launch_proj_store(ctx, o.w, o.xs, o.xq, o.y));
                break;
            case CERA_HIP_OP_NORM_GEMV:
                if (!o.w || !o.x || !o.norm_w || !o.y || (o.w2 && !o.y2)) return bad("NORM_GEMV needs w, x, norm_w, y (and y2 with w2)");
                CERA_TRY(cera_launch_qkv_fused(ctx, o.w, o.w2, o.x, o.norm_w, o.eps, o.y, o.y2, &done));
                if (!done) return cera_fail(ctx, CERA_HIP_ERR_UNSUPPORTED_DTYPE, "decode_ops: no fused norm + projection launch for this shape");
                break;
            case CERA_HIP_OP_NORM_GATE_UP:
                if (!o.w || !o.w2 || !o.x || !o.norm_w || !o.out_q || !o.out_s) return bad("NORM_GATE_UP needs w, w2, x, norm_w, out_q, out_s");
                CERA_TRY(cera_launch_ffn_gate_up_fused(ctx, o.w, o.w2, o.x, o.norm_w, o.eps, o.out_q, o.out_s, &done));
                if (!done) return cera_fail(ctx, CERA_HIP_ERR_UNSUPPORTED_DTYPE, "decode_ops: no fused gate | up launch for this shape");
                break;
            case CERA_HIP_OP_NORM_QUANT:
                if (!o.x || !o.norm_w || !o.y || !o.out_q || !o.out_s || o.n == 0 || o.n % 32) return bad("NORM_QUANT needs x, norm_w, y, out_q, out_s and n % 32 == 0");
                CERA_TRY(launch_norm_quant(ctx, o.x, o.norm_w, o.n, 1, o.eps, o.y, o.out_s, o.out_q));
                break;
            case CERA_HIP_OP_QUANT:
                if (!o.x || !o.out_q || !o.out_s || o.n == 0 || o.n % 32) return bad("QUANT needs x, out_q, out_s and n % 32 == 0");
                CERA_TRY(cera_launch_quantize(ctx, o.x, o.n, o.out_s, o.out_q));
                break;
            default: return bad("unknown kind");
        }
    }
    return CERA_HIP_OK;
}

// ---- kernel-level entry points for the decode step's fused kernels (host buffers) ------------
extern "C" cera_hip_status cera_hip_rmsnorm_q8_0(cera_hip_ctx* ctx, const float* x, const float* weight, uint64_t n, float eps,
                                                 float* y, float* scales, int8_t* quants) {
    if (!ctx || !x || !weight || !y || !scales || !quants) return CERA_HIP_ERR_ARGUMENT;
    if (n == 0 || n % 32 || n > 0xFFFFFFFFull) return cera_fail(ctx, CERA_HIP_ERR_SHAPE, "rmsnorm_q8_0: n must be a positive multiple of 32");
    std::lock_guard<std::recursive_mutex> lk(ctx->op_mu);
    void *dx, *dw, *dy, *ds, *dq;
    CERA_TRY(cera_scratch(ctx, 0, n * 4, &dx));
    CERA_TRY(cera_scratch(ctx, 1, n * 4, &dw));
    CERA_TRY(cera_scratch(ctx, 3, n * 4, &dy));
    CERA_TRY(cera_scratch(ctx, 4, n / 32 * 4, &ds));
    CERA_TRY(cera_scratch(ctx, 2, n, &dq));
    CERA_TRY(cera_hip_upload(ctx, dx, x, n * 4));
    CERA_TRY(cera_hip_upload(ctx, dw, weight, n * 4));
    CERA_TRY(launch_norm_quant(ctx, static_cast<float*>(dx), static_cast<float*>(dw), static_cast<uint32_t>(n), 1, eps,
                               static_cast<float*>(dy), static_cast<float*>(ds), static_cast<int8_t*>(dq)));
    CERA_TRY(cera_hip_download(ctx, y, dy, n * 4));
    CERA_TRY(cera_hip_download(ctx, scales, ds, n / 32 * 4));
    return cera_hip_download(ctx, quants, dq, n);
}

extern "C" cera_hip_status cera_hip_attn_decode_step(cera_hip_ctx* ctx, const float* q, const float* k_new, const float* v_new,
                                                     const float* k_cache, const float* v_cache, uint32_t n_heads,
                                                     uint32_t n_kv_heads, uint32_t head_dim, uint32_t pos, float rope_base,
                                                     uint32_t rope_type, const float* freq_factors, float scale,
                                                     uint32_t kv_type, float* out, float* out_scales, int8_t* out_quants,
                                                     float* k_row, float* v_row) {
    if (!ctx || !q || !k_new || !v_new || (pos && (!k_cache || !v_cache)) || !out || !out_scales || !out_quants || !k_row || !v_row)
        return CERA_HIP_ERR_ARGUMENT;
    if ((head_dim != 64 && head_dim != 128) || rope_type > 1 || kv_type > CERA_HIP_KV_F16 || n_kv_heads == 0 || n_heads % n_kv_heads)
        return cera_fail(ctx, CERA_HIP_ERR_SHAPE, "attn_decode_step: bad shape");
    std::lock_guard<std::recursive_mutex> lk(ctx->op_mu);
    const bool f16 = kv_type == CERA_HIP_KV_F16;
    const uint32_t max_seq = pos + 1;
    const uint64_t kv_dim = static_cast<uint64_t>(n_kv_heads) * head_dim, q_dim = static_cast<uint64_t>(n_heads) * head_dim;
    const uint64_t esz = f16 ? sizeof(kv_half) : sizeof(float), cache_bytes = kv_dim * max_seq * esz;
    // caches: head-major [kv_head][max_seq][head_dim], rows [0, pos) from the caller, row pos zero
    std::vector<char> hk(cache_bytes, 0), hv(cache_bytes, 0);
    for (uint64_t t = 0; t < pos; ++t)
        for (uint32_t h = 0; h < n_kv_heads; ++h)
            for (uint32_t d = 0; d < head_dim; ++d) {
                const uint64_t dst = (static_cast<uint64_t>(h) * max_seq + t) * head_dim + d, src = t * kv_dim + h * head_dim + d;
                if (f16) {
                    reinterpret_cast<kv_half*>(hk.data())[dst] = static_cast<kv_half>(k_cache[src]);
                    reinterpret_cast<kv_half*>(hv.data())[dst] = static_cast<kv_half>(v_cache[src]);
                } else {
                    reinterpret_cast<float*>(hk.data())[dst] = k_cache[src];
                    reinterpret_cast<float*>(hv.data())[dst] = v_cache[src];
                }
            }
    std::vector<float> table;
    cera_build_rope_table(max_seq, head_dim, rope_base, rope_type == 1 ? freq_factors : nullptr, table);
    void *dq, *dk, *dv, *dkc, *dvc, *dt, *dp, *dout, *dsc, *dqq;
    CERA_TRY(cera_scratch(ctx, 0, q_dim * 4, &dq));
    CERA_TRY(cera_scratch(ctx, 1, kv_dim * 4, &dk));
    CERA_TRY(cera_scratch(ctx, 2, kv_dim * 4, &dv));
    CERA_TRY(cera_scratch(ctx, 5, cache_bytes, &dkc));
    CERA_TRY(cera_scratch(ctx, 6, cache_bytes, &dvc));
    CERA_TRY(cera_scratch(ctx, 4, table.size() * 4, &dt));
    CERA_TRY(cera_scratch(ctx, 7, 4, &dp));
    CERA_TRY(cera_scratch(ctx, 3, q_dim * 4, &dout));
    CERA_TRY(cera_scratch(ctx, 9, q_dim / 32 * 4, &dsc));
    CERA_TRY(cera_scratch(ctx, 10, q_dim, &dqq));
    CERA_TRY(cera_hip_upload(ctx, dq, q, q_dim * 4));
    CERA_TRY(cera_hip_upload(ctx, dk, k_new, kv_dim * 4));
    CERA_TRY(cera_hip_upload(ctx, dv, v_new, kv_dim * 4));
    CERA_TRY(cera_hip_upload(ctx, dkc, hk.data(), cache_bytes));
    CERA_TRY(cera_hip_upload(ctx, dvc, hv.data(), cache_bytes));
    CERA_TRY(cera_hip_upload(ctx, dt, table.data(), table.size() * 4));
    CERA_TRY(cera_hip_upload(ctx, dp, &pos, 4));
    CERA_TRY(cera_attn_step(ctx, static_cast<float*>(dq), static_cast<float*>(dk), static_cast<float*>(dv), dkc, dvc,
                            static_cast<float*>(dt), static_cast<uint32_t*>(dp), pos, n_heads, n_kv_heads, head_dim, max_seq,
                            rope_type, scale, f16, static_cast<float*>(dout), static_cast<float*>(dsc), static_cast<int8_t*>(dqq)));
    CERA_TRY(cera_hip_download(ctx, out, dout, q_dim * 4));
    CERA_TRY(cera_hip_download(ctx, out_scales, dsc, q_dim / 32 * 4));
    CERA_TRY(cera_hip_download(ctx, out_quants, dqq, q_dim));
    // the rows the step appended at `pos`, widened exactly when the cache holds halves
    std::vector<char> row(head_dim * esz);
    for (int is_v = 0; is_v < 2; ++is_v)
        for (uint32_t h = 0; h < n_kv_heads; ++h) {
            const char* src = static_cast<const char*>(is_v ? dvc : dkc) + (static_cast<uint64_t>(h) * max_seq + pos) * head_dim * esz;
            CERA_TRY(cera_hip_download(ctx, row.data(), src, row.size()));
            float* dst = (is_v ? v_row : k_row) + h * head_dim;
            for (uint32_t d = 0; d < head_dim; ++d)
                dst[d] = f16 ? static_cast<float>(reinterpret_cast<const kv_half*>(row.data())[d]) : reinterpret_cast<const float*>(row.data())[d];
        }
    return CERA_HIP_OK;
}
