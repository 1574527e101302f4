// Speculative decoding above the Model interface: prompt-lookup drafting, greedy verification of
// a draft in one forward, and the standalone greedy driver -- the callers of
// forward_prefill_logits_all / truncate_kv (cera/src/spec.rs).
#pragma once
#include <cstddef>
#include <cstdint>
#include <vector>

#include "hip_llama.h"

namespace cera {

// cera/src/spec.rs:23-40: the tokens (at most k) that followed the most recent earlier occurrence
// of the last `ngram` tokens; empty when there is none, or on degenerate arguments.
std::vector<uint32_t> prompt_lookup_draft(const uint32_t* tokens, size_t n, size_t ngram, size_t k);

// cera/src/spec.rs:43-61
struct SpecStats {
    size_t drafted = 0, accepted = 0, rounds = 0;
    float acceptance_rate() const { return drafted ? static_cast<float>(accepted) / static_cast<float>(drafted) : 0.0f; }
};

// cera/src/spec.rs:64-75
struct VerifyResult {
    std::vector<uint32_t> accepted;      // longest draft prefix equal to the target's greedy argmax
    std::vector<float> follow_logits;    // logits after the guaranteed token plus `accepted`
};

// sampler::argmax (cera/src/sampler.rs:20-30): strict >, lowest index on ties, NaN never wins
uint32_t argmax(const float* logits, size_t n);

// cera/src/spec.rs:91-143: feeds [guaranteed, draft...] at state.seq_len in one forward, keeps the
// guaranteed token plus the accepted drafts in the KV (the rest is truncated through the model).
VerifyResult verify_draft(Model& model, InferenceState& state, uint32_t guaranteed, const std::vector<uint32_t>& draft,
                          size_t vocab);

// cera/src/spec.rs:160-268.  `state` must be fresh; an EOS token is not emitted, the max_new cap
// emits the token and stops.  Throws BackendError where the reference asserts.
std::vector<uint32_t> greedy_generate_spec(Model& model, InferenceState& state, const std::vector<uint32_t>& prompt,
                                           size_t max_new, const std::vector<uint32_t>& eos, size_t ngram, size_t k,
                                           SpecStats* stats);

}  // namespace cera
