#include "spec.h"

#include <algorithm>
#include <cmath>
#include <string>

namespace cera {

std::vector<uint32_t> prompt_lookup_draft(const uint32_t* tokens, size_t n, size_t ngram, size_t k) {
    if (ngram == 0 || k == 0 || n <= ngram) return {};
    const uint32_t* pattern = tokens + (n - ngram);
    // earlier start positions, most recent first
    for (size_t start = n - ngram; start-- > 0;) {
        if (std::equal(pattern, pattern + ngram, tokens + start)) {
            const size_t follow = start + ngram, end = std::min(follow + k, n);
            return std::vector<uint32_t>(tokens + follow, tokens + end);
        }
    }
    return {};
}

uint32_t argmax(const float* logits, size_t n) {
    uint32_t best = 0;
    float bv = -INFINITY;
    for (size_t i = 0; i < n; ++i)
        if (logits[i] > bv) {
            bv = logits[i];
            best = static_cast<uint32_t>(i);
        }
    return best;
}

VerifyResult verify_draft(Model& model, InferenceState& state, uint32_t guaranteed, const std::vector<uint32_t>& draft,
                          size_t vocab) {
    const size_t old = state.seq_len;
    std::vector<uint32_t> batch;
    batch.reserve(1 + draft.size());
    batch.push_back(guaranteed);
    batch.insert(batch.end(), draft.begin(), draft.end());
    const std::vector<float> all = model.forward_prefill_logits_all(batch.data(), batch.size(), old, state);
    if (all.size() != batch.size() * vocab)
        throw BackendError("forward_prefill_logits_all returned " + std::to_string(all.size()) + " logits for " +
                           std::to_string(batch.size()) + " positions x vocab " + std::to_string(vocab));
    // row j predicts the token that should follow batch[j]
    VerifyResult r;
    for (size_t j = 0; j < draft.size(); ++j) {
        if (argmax(all.data() + j * vocab, vocab) != draft[j]) break;
        r.accepted.push_back(draft[j]);
    }
    const size_t m = r.accepted.size();
    model.truncate_kv(state, old + 1 + m);   // through the model: its cache is device-resident
    r.follow_logits.assign(all.begin() + m * vocab, all.begin() + (m + 1) * vocab);
    return r;
}

std::vector<uint32_t> greedy_generate_spec(Model& model, InferenceState& state, const std::vector<uint32_t>& prompt,
                                           size_t max_new, const std::vector<uint32_t>& eos, size_t ngram, size_t k,
                                           SpecStats* stats_out) {
    std::vector<uint32_t> out;
    SpecStats stats;
    if (!model.supports_all_logits()) throw BackendError("greedy_generate_spec requires forward_prefill_logits_all support");
    if (state.seq_len != 0)
        throw BackendError("greedy_generate_spec requires a fresh InferenceState (seq_len == 0); this one holds " +
                           std::to_string(state.seq_len) + " positions");
    if (prompt.empty() || max_new == 0) {
        if (stats_out) *stats_out = stats;
        return out;
    }
    std::vector<float> next_logits = model.forward_prefill(prompt.data(), prompt.size(), 0, state);
    const size_t vocab = next_logits.size();
    std::vector<uint32_t> history = prompt;
    auto is_eos = [&](uint32_t t) { return std::find(eos.begin(), eos.end(), t) != eos.end(); };

    for (;;) {
        if (out.size() >= max_new) break;
        const uint32_t t = argmax(next_logits.data(), vocab);
        if (is_eos(t)) break;            // an EOS token is not emitted
        out.push_back(t);
        history.push_back(t);
        if (out.size() >= max_new) break;   // the budget cap emits the token and stops

        const std::vector<uint32_t> draft = prompt_lookup_draft(history.data(), history.size(), ngram, k);
        if (draft.empty()) {
            next_logits = model.forward(&t, 1, state.seq_len, state);
            continue;
        }
        const size_t old = state.seq_len;
        stats.rounds += 1;
        stats.drafted += draft.size();
        VerifyResult vr = verify_draft(model, state, t, draft, vocab);

        size_t kept = 0;
        bool stopped = false;
        for (uint32_t q : vr.accepted) {
            if (out.size() >= max_new || is_eos(q)) {
                stopped = true;
                break;
            }
            out.push_back(q);
            history.push_back(q);
            kept += 1;
            stats.accepted += 1;
        }
        if (kept < vr.accepted.size()) model.truncate_kv(state, old + 1 + kept);
        if (stopped) break;
        next_logits = std::move(vr.follow_logits);
    }
    if (stats_out) *stats_out = stats;
    return out;
}

}  // namespace cera
