// Greedy generation loops over LlamaRuntime: the plain incremental loop and the exact two-token
// draft/verify loop.
#pragma once

#include <cstdint>
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

// sampleToken (RealModelInferenceEngine.swift:8036-8068).  `unit` in [0, 1) plays Double.random(in: 0..<total) / total.
int sample_token(const float *logits, int count, float temperature, double unit);
// SplitMix64 (the generator the reference's tests seed, Tests/CPUOpsTests/CPUOpsTests.swift:6-21) and the unit
// double Swift's BinaryFloatingPoint.random(in:using:) derives from one 64-bit draw: 53 high bits * 2^-53.
struct SplitMix64 {
    uint64_t state;
    uint64_t next() {
        state += 0x9E3779B97F4A7C15ull;
        uint64_t z = state;
        z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
        z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
        return z ^ (z >> 31);
    }
    double unit() { return (double)(next() >> 11) * (1.0 / 9007199254740992.0); }
};
// generate(prompt:maxTokens:temperature:) with temperature > 0 (:1405-1493 with :8070-8081): per token the full
// logits come back from the GPU and the reference's sampling runs on the host.
int generate_sampled(LlamaRuntime &rt, const uint32_t *prompt, int prompt_count, int max_tokens, float temperature,
                     uint64_t seed, std::vector<uint32_t> *out, GenerationTiming *timing);

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

// `n_seq` independent sequences in lock step (sequence s uses KV cache s), greedy, fixed budget: every
// sequence yields min(max_tokens, context left for the longest prompt) tokens.  Steps of more than two rows
// run on the matrix cores.  The closest reference notion is lane/stream packing (ane_interop.h:270-289).
int generate_greedy_batch(LlamaRuntime &rt, const uint32_t *const *prompts, const int *prompt_counts, int n_seq, int max_tokens,
                          std::vector<std::vector<uint32_t>> *out, double *decode_ms);
// The exact two-token loop over `n_seq` sequences: each target pass verifies (current, proposed) of every
// sequence at once.  Every sequence's stream equals its stream from generate_greedy_batch.
int generate_two_token_batch(LlamaRuntime &full, LlamaRuntime &draft, const uint32_t *const *prompts, const int *prompt_counts,
                             int n_seq, int max_tokens, std::vector<std::vector<uint32_t>> *out, TwoTokenStats *stats, double *decode_ms);

}  // namespace esp
