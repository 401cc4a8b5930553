// RealModelInferenceEngine for the llama decode path, GPU-resident.  Mirrors the reference's entry
// points (Sources/RealModelInference/RealModelInferenceEngine.swift): build(config:weightDir:tokenizerDir:)
// :1377, generate(...) :1405 in its token-id form, generateTokensExactCPUForTesting :1838, and the
// exact two-token draft selection through ESPRESSO_BUNDLE_DRAFT_* (:5324-5390).
#pragma once

#include <map>
#include <memory>
#include <string>
#include <vector>

#include "../llama_runtime.h"
#include "model_support.h"
#include "tokenizer.h"

namespace esp {

using Environment = std::map<std::string, std::string>;

// GenerationResult (:17-55); `text` is filled by the prompt-text entry point only
struct GenerationResult {
    std::string text;
    std::vector<TokenID> tokens, promptTokens;
    std::vector<double> tokenLatenciesMs;
    double tokensPerSecond = 0, compileTimeMs = 0, firstTokenLatencyMs = 0;
    std::string exactHeadBackend;
    bool hasTwoTokenStats = false;
    double committedExactTokensPerPass = 0, acceptedFutureTokensPerPass = 0;
};

class RealModelInferenceEngine {
  public:
    // Loads the weight directory (packed sidecar, else float32 sidecar, else fp16 BLOBFILE, per tensor) into HBM.
    // A non-empty tokenizerDir is searched in the reference's order (loadTokenizer, :7558-7613) and must hold a
    // tokenizer; an empty one leaves the engine with the token-id entry points only.
    static int build(const MultiModelConfig &config, const std::string &weightDir, const std::string &tokenizerDir,
                     const Environment &environment, std::unique_ptr<RealModelInferenceEngine> *out);
    // Greedy generation from token ids.  temperature must be 0 on this path.
    int generate(const std::vector<TokenID> &promptTokens, int maxTokens, float temperature, const Environment &environment,
                 GenerationResult *out);
    // generate(prompt:maxTokens:temperature:) (:1405-1437): encodePrompt (:5404-5418), the token-id path above,
    // text = decode(prompt tokens + generated tokens).  Needs a tokenizer.
    int generateText(const std::string &prompt, int maxTokens, float temperature, const Environment &environment, GenerationResult *out);
    const Tokenizer *tokenizer() const { return tokenizer_.get(); }
    static int generateTokensForTesting(const MultiModelConfig &config, const std::string &weightDir,
                                        const std::vector<TokenID> &promptTokens, int maxTokens, std::vector<TokenID> *out);
    const MultiModelConfig &config() const { return config_; }
    LlamaRuntime &runtime() { return *runtime_; }
    double buildTimeMs() const { return build_ms_; }

    // resolveExactTwoTokenDraft (:5324-5390): returns 0 and an empty draftWeightDir when no draft is configured
    static int resolveExactTwoTokenDraft(const MultiModelConfig &config, const std::string &weightDir, const Environment &environment,
                                         std::string *draftWeightDir, MultiModelConfig *draftConfig);

  private:
    RealModelInferenceEngine() = default;
    static int loadRuntime(const MultiModelConfig &config, const std::string &weightDir, const Environment &environment,
                           std::unique_ptr<LlamaRuntime> *out);
    MultiModelConfig config_;
    std::string weight_dir_;
    std::unique_ptr<LlamaRuntime> runtime_;
    std::unique_ptr<LlamaRuntime> draft_runtime_;
    std::unique_ptr<Tokenizer> tokenizer_;
    std::string draft_dir_loaded_;
    double build_ms_ = 0;
};

}  // namespace esp
