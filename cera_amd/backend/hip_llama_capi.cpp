#include "hip_llama_capi.h"

#include <algorithm>

#include <chrono>
#include <cmath>
#include <cstring>

#include "hip_llama.h"

struct cera_llama {
    std::unique_ptr<cera::GgufFile> gguf;
    std::unique_ptr<cera::HipLlamaModel> model;
    cera::InferenceState state;
    std::atomic<bool> cancel{false};
    std::string err;
};

namespace {
void set_err(char* err, uint64_t n, const std::string& m) {
    if (!err || !n) return;
    std::strncpy(err, m.c_str(), n - 1);
    err[n - 1] = 0;
}
template <class F>
int guarded(cera_llama* h, F&& f) {
    try {
        f();
        return 0;
    } catch (const std::exception& e) {
        h->err = e.what();
    } catch (...) {
        h->err = "unknown error";
    }
    return -1;
}
// The handle carries one InferenceState for the caller's convenience.  A call at position 0 is a
// caller arriving with a new state (every generate() in the reference makes one): start over.
void fresh_at(cera_llama* h, uint64_t pos) {
    if (pos == 0) h->state = cera::InferenceState{};
}
double now_s() {
    return std::chrono::duration<double>(std::chrono::steady_clock::now().time_since_epoch()).count();
}
}  // namespace

extern "C" {

cera_llama* cera_llama_open(const char* path, uint64_t context_size, int device, char* err, uint64_t err_len) {
    if (!path) {
        set_err(err, err_len, "null path");
        return nullptr;
    }
    std::unique_ptr<cera_llama> h(new cera_llama());
    std::string e;
    h->gguf = cera::GgufFile::open(path, &e);
    if (!h->gguf) {
        set_err(err, err_len, e);
        return nullptr;
    }
    try {
        h->model = cera::HipLlamaModel::from_gguf(*h->gguf, context_size, device);
    } catch (const std::exception& ex) {
        set_err(err, err_len, ex.what());
        return nullptr;
    }
    // the weights are in HBM now; the mapping is only needed for metadata afterwards
    return h.release();
}
void cera_llama_close(cera_llama* h) { delete h; }
const char* cera_llama_last_error(const cera_llama* h) { return h ? h->err.c_str() : ""; }

int cera_llama_get_config(const cera_llama* h, cera_llama_config* out) {
    if (!h || !out) return -1;
    const cera::ModelConfig& c = h->model->config();
    out->n_layers = c.n_layers;
    out->hidden_size = c.hidden_size;
    out->intermediate_size = c.intermediate_size;
    out->n_heads = c.n_heads;
    out->n_kv_heads = c.n_kv_heads;
    out->head_dim = c.head_dim;
    out->vocab_size = c.vocab_size;
    out->max_seq_len = c.max_seq_len;
    out->rope_theta = c.rope_theta;
    out->rms_norm_eps = c.rms_norm_eps;
    out->rope_type = h->model->rope_type() == cera::RopeType::Norm ? 1u : 0u;
    return 0;
}
uint64_t cera_llama_seq_len(const cera_llama* h) { return h->state.seq_len; }
uint64_t cera_llama_gpu_memory_bytes(const cera_llama* h) { return h->model->gpu_memory_bytes(); }

int cera_llama_forward(cera_llama* h, uint32_t token, uint64_t pos, float* logits) {
    return guarded(h, [&] {
        fresh_at(h, pos);
        std::vector<float> l = h->model->forward(&token, 1, pos, h->state);
        std::memcpy(logits, l.data(), l.size() * sizeof(float));
    });
}
int cera_llama_forward_greedy(cera_llama* h, uint32_t token, uint64_t pos, uint32_t* next) {
    return guarded(h, [&] {
        fresh_at(h, pos);
        *next = h->model->forward_greedy(&token, 1, pos, h->state);
    });
}
int cera_llama_forward_prefill(cera_llama* h, const uint32_t* tokens, uint64_t n, uint64_t start_pos, float* logits) {
    return guarded(h, [&] {
        fresh_at(h, start_pos);
        std::vector<float> l = h->model->forward_prefill(tokens, n, start_pos, h->state);
        std::memcpy(logits, l.data(), l.size() * sizeof(float));
    });
}
int cera_llama_forward_prefill_logits_all(cera_llama* h, const uint32_t* tokens, uint64_t n, uint64_t start_pos,
                                          float* logits) {
    return guarded(h, [&] {
        fresh_at(h, start_pos);
        std::vector<float> l = h->model->forward_prefill_logits_all(tokens, n, start_pos, h->state);
        std::memcpy(logits, l.data(), l.size() * sizeof(float));
    });
}
int cera_llama_forward_prefill_chunked(cera_llama* h, const uint32_t* tokens, uint64_t n, uint64_t start_pos,
                                       uint64_t ubatch, uint64_t* consumed, float* logits) {
    return guarded(h, [&] {
        fresh_at(h, start_pos);
        auto r = h->model->forward_prefill_chunked(tokens, n, start_pos, h->state, ubatch, h->cancel);
        if (consumed) *consumed = r.first;
        if (r.second && logits) std::memcpy(logits, r.second->data(), r.second->size() * sizeof(float));
    });
}
void cera_llama_set_cancel(cera_llama* h, int c) { h->cancel.store(c != 0); }
int cera_llama_truncate_kv(cera_llama* h, uint64_t len) {
    return guarded(h, [&] { h->model->truncate_kv(h->state, len); });
}
int cera_llama_f16_kv_supported(const cera_llama* h) { return h && h->model->f16_kv_supported() ? 1 : 0; }
int cera_llama_configure_kv_compression(cera_llama* h, int kind) {
    return guarded(h, [&] {
        if (kind != 0 && kind != 1) throw cera::BackendError("configure_kv_compression: kind must be 0 (none) or 1 (f16)");
        h->model->configure_kv_compression(kind == 1 ? cera::KvCompression::F16 : cera::KvCompression::None);
    });
}
int cera_llama_supports_kv_shift(const cera_llama* h) { return h && h->model->supports_kv_shift() ? 1 : 0; }
int cera_llama_shift_kv(cera_llama* h, uint64_t n_keep, uint64_t shift) {
    return guarded(h, [&] { h->model->shift_kv(h->state, n_keep, shift); });
}
struct cera_llama_snapshot {
    cera::StateSnapshot snap;
};
cera_llama_snapshot* cera_llama_snapshot_state(cera_llama* h) {
    cera_llama_snapshot* out = nullptr;
    if (guarded(h, [&] {
            out = new cera_llama_snapshot();
            out->snap = h->model->snapshot_state();
        }) != 0) {
        delete out;
        return nullptr;
    }
    return out;
}
uint64_t cera_llama_snapshot_seq_len(const cera_llama_snapshot* s) { return s ? s->snap.seq_len : 0; }
uint64_t cera_llama_snapshot_bytes(const cera_llama_snapshot* s) {
    uint64_t n = 0;
    if (s)
        for (const auto& L : s->snap.layers) n += L.k_data.size() + L.v_data.size();
    return n;
}
int cera_llama_restore_state(cera_llama* h, const cera_llama_snapshot* s) {
    if (!s) return -1;
    return guarded(h, [&] {
        h->model->restore_state(s->snap);
        h->state.seq_len = s->snap.seq_len;
    });
}
void cera_llama_snapshot_free(cera_llama_snapshot* s) { delete s; }

int cera_llama_generate_greedy(cera_llama* h, const uint32_t* prompt, uint64_t n_prompt, uint64_t n_new,
                               uint64_t ubatch, uint32_t* out, double* prefill_s, double* decode_s) {
    return guarded(h, [&] {
        if (!n_prompt || !n_new) throw cera::BackendError("generate_greedy needs a prompt and n_new > 0");
        std::atomic<bool> never{false};
        h->state = cera::InferenceState{};   // a generation starts with a new state, as Session::generate does
        double t0 = now_s();
        auto r = h->model->forward_prefill_chunked(prompt, n_prompt, 0, h->state, ubatch, never);
        const std::vector<float>& l = *r.second;
        size_t best = 0;
        float bv = -INFINITY;
        for (size_t i = 0; i < l.size(); ++i)
            if (l[i] > bv) { bv = l[i]; best = i; }
        out[0] = static_cast<uint32_t>(best);
        double t1 = now_s();
        for (uint64_t i = 1; i < n_new; ++i) out[i] = h->model->forward_greedy(&out[i - 1], 1, h->state.seq_len, h->state);
        double t2 = now_s();
        if (prefill_s) *prefill_s = t1 - t0;
        if (decode_s) *decode_s = t2 - t1;
    });
}

int cera_llama_set_reference_order(cera_llama* h, int on) {
    return guarded(h, [&] {
        auto* hm = dynamic_cast<cera::HipLlamaModel*>(h->model.get());
        if (!hm) throw cera::BackendError("set_reference_order: not a hip model");
        hm->set_reference_order(on < 0 ? 0u : static_cast<uint32_t>(on));
    });
}

}  // extern "C"
