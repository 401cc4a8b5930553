// Greedy generation loops over LlamaRuntime: the plain incremental loop and the exact two-token
// draft/verify loop.
#pragma once

#include <vector>

#include "llama_runtime.h"

namespace esp {

struct GenerationTiming {
    double prefill_ms = 0, decode_ms = 0, first_token_latency_ms = 0;
    std::vector<double> token_latencies_ms;
};

// generateIncrementalExactCPULlama at temperature 0 (RealModelInferenceEngine.swift:6192-6431).
// effectiveMaxTokens = min(maxTokens, maxSeq - promptLen) (:1425-1426).
int generate_greedy(LlamaRuntime &rt, const uint32_t *prompt, int prompt_count, int max_tokens,
                    std::vector<uint32_t> *out, GenerationTiming *timing);

struct TwoTokenStats {
    // one pass = one batched verify of [current token, proposed future token] by the full model
    // (ExactTwoTokenGenerationHarness, Sources/Espresso/GenerationHarness.swift:599-687)
    int passes = 0, committed_total = 0, accepted_total = 0;
    // the reference CPU loop's accounting of the same token stream (:6109-6175)
    int reference_passes = 0, reference_committed_total = 0, reference_accepted_total = 0;
};

// Exact two-token draft/verify: the emitted stream equals generate_greedy(full) by construction.
// (generateIncrementalExactTwoTokenDraftLlama, :6014-6190; promotion rule of
// ExactTwoTokenBranchPromotionPlan.make, GenerationHarness.swift:156-180.)
int generate_two_token(LlamaRuntime &full, LlamaRuntime &draft, const uint32_t *prompt, int prompt_count,
                       int max_tokens, bool reference_accounting, std::vector<uint32_t> *out,
                       TwoTokenStats *stats, GenerationTiming *timing);

}  // namespace esp
