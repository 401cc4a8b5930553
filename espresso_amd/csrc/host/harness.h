// ExactTwoTokenGenerationHarness and its protocol (Sources/Espresso/GenerationHarness.swift:104-252,
// 599-687): the harness checks the invariants of every pass, the model does the work.  The model is an
// abstract class so that the GPU runtime pair and scripted test doubles both plug in.
#pragma once

#include <string>
#include <vector>

#include "../llama_runtime.h"
#include "model_support.h"

namespace esp {

struct ExactTwoTokenPassMetrics {   // :104-131
    double proposerLatencyMs = 0, verifierTrunkLatencyMs = 0, verifierLogitsLatencyMs = 0, stateAdvanceLatencyMs = 0;
    int acceptedFutureTokenCount = 0, committedExactTokenCount = 0;
};

struct ExactTwoTokenPassResult {    // :133-147
    std::vector<TokenID> committedTokens;
    TokenID nextCurrentToken = 0;
    ExactTwoTokenPassMetrics metrics;
};

// ExactTwoTokenBranchPromotionPlan.make (:149-180)
struct ExactTwoTokenBranchPromotionPlan {
    std::vector<TokenID> committedTokens;
    TokenID nextCurrentToken = 0;
    int committedExactTokenCount = 0, acceptedFutureTokenCount = 0, promotedStepCount = 0;
    static ExactTwoTokenBranchPromotionPlan make(TokenID currentToken, TokenID proposedFutureToken, TokenID exactNextToken,
                                                 TokenID exactFutureToken, int remainingTokenBudget);
};

struct ExactTwoTokenGenerationTrace {   // :182-237
    std::vector<TokenID> promptTokens, generatedTokens;
    double prefillLatencyMs = 0;
    std::vector<ExactTwoTokenPassMetrics> passMetrics;
    double committedExactTokensPerPass() const;
    double acceptedFutureTokensPerPass() const;
};

// ExactTwoTokenGeneratingLanguageModel (:239-252).  Methods return 0 or a negative ESP_ERR_* code with the
// thread's error text set.
class ExactTwoTokenGeneratingLanguageModel {
  public:
    virtual ~ExactTwoTokenGeneratingLanguageModel() = default;
    virtual int vocabSize() const = 0;
    virtual int reset() = 0;
    virtual int prefillSelectedToken(const std::vector<TokenID> &promptTokens, TokenID *selected) = 0;
    virtual int performExactTwoTokenPass(TokenID currentToken, int remainingTokenBudget, ExactTwoTokenPassResult *result) = 0;
};

// ExactTwoTokenGenerationHarness.generate (:612-686)
int exactTwoTokenHarnessGenerate(ExactTwoTokenGeneratingLanguageModel &model, const std::vector<TokenID> &promptTokens,
                                 int maxNewTokens, ExactTwoTokenGenerationTrace *trace);

// The GPU implementation: the target verifies [current, proposed] in one batched step, the draft proposes.
class HipExactTwoTokenModel : public ExactTwoTokenGeneratingLanguageModel {
  public:
    HipExactTwoTokenModel(LlamaRuntime &target, LlamaRuntime &draft) : target_(target), draft_(draft) {}
    int vocabSize() const override { return target_.config().vocab; }
    int reset() override;
    int prefillSelectedToken(const std::vector<TokenID> &promptTokens, TokenID *selected) override;
    int performExactTwoTokenPass(TokenID currentToken, int remainingTokenBudget, ExactTwoTokenPassResult *result) override;

  private:
    LlamaRuntime &target_, &draft_;
};

}  // namespace esp
