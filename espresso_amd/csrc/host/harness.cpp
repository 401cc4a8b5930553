#include "harness.h"

#include <chrono>

namespace esp {
namespace {
using Clock = std::chrono::steady_clock;
double ms_between(Clock::time_point a, Clock::time_point b) { return std::chrono::duration<double, std::milli>(b - a).count(); }
}  // namespace

ExactTwoTokenBranchPromotionPlan ExactTwoTokenBranchPromotionPlan::make(TokenID currentToken, TokenID proposedFutureToken,
                                                                       TokenID exactNextToken, TokenID exactFutureToken,
                                                                       int remainingTokenBudget) {
    ExactTwoTokenBranchPromotionPlan p;
    if (remainingTokenBudget > 1 && proposedFutureToken == exactNextToken) {
        p.committedTokens = {currentToken, exactNextToken};
        p.nextCurrentToken = exactFutureToken;
        p.committedExactTokenCount = 2;
        p.acceptedFutureTokenCount = 1;
        p.promotedStepCount = 2;
    } else {
        p.committedTokens = {currentToken};
        p.nextCurrentToken = exactNextToken;
        p.committedExactTokenCount = 1;
        p.acceptedFutureTokenCount = 0;
        p.promotedStepCount = 1;
    }
    return p;
}

double ExactTwoTokenGenerationTrace::committedExactTokensPerPass() const {
    if (passMetrics.empty()) return 0;
    double total = 0;
    for (const auto &m : passMetrics) total += m.committedExactTokenCount;
    return total / (double)passMetrics.size();
}
double ExactTwoTokenGenerationTrace::acceptedFutureTokensPerPass() const {
    if (passMetrics.empty()) return 0;
    double total = 0;
    for (const auto &m : passMetrics) total += m.acceptedFutureTokenCount;
    return total / (double)passMetrics.size();
}

int exactTwoTokenHarnessGenerate(ExactTwoTokenGeneratingLanguageModel &model, const std::vector<TokenID> &promptTokens,
                                 int maxNewTokens, ExactTwoTokenGenerationTrace *trace) {
    *trace = ExactTwoTokenGenerationTrace{};
    if (promptTokens.empty()) return fail(ESP_ERR_INVALID_ARGUMENT, "promptTokens must not be empty");
    if (maxNewTokens <= 0) return fail(ESP_ERR_INVALID_ARGUMENT, "maxNewTokens must be > 0");
    int rc = model.reset();
    if (rc != ESP_OK) return rc;
    const auto t0 = Clock::now();
    TokenID current = 0;
    if ((rc = model.prefillSelectedToken(promptTokens, &current)) != ESP_OK) return rc;
    trace->prefillLatencyMs = ms_between(t0, Clock::now());
    trace->promptTokens = promptTokens;
    while ((int)trace->generatedTokens.size() < maxNewTokens) {
        const int budget = maxNewTokens - (int)trace->generatedTokens.size();
        ExactTwoTokenPassResult r;
        if ((rc = model.performExactTwoTokenPass(current, budget, &r)) != ESP_OK) return rc;
        const int n = (int)r.committedTokens.size();
        if (n == 0) return fail(ESP_ERR_LAUNCH_FAILED, "exact two-token pass must commit at least one token");
        if (r.committedTokens[0] != current) return fail(ESP_ERR_LAUNCH_FAILED, "exact two-token pass must commit current token first");
        if (n < 1 || n > (budget < 2 ? budget : 2))
            return fail(ESP_ERR_LAUNCH_FAILED, "exact two-token pass committed %d tokens with remaining budget %d", n, budget);
        if (r.metrics.acceptedFutureTokenCount < 0 || r.metrics.acceptedFutureTokenCount > 1)
            return fail(ESP_ERR_LAUNCH_FAILED, "acceptedFutureTokenCount %d must be in 0...1", r.metrics.acceptedFutureTokenCount);
        if (r.metrics.committedExactTokenCount != n)
            return fail(ESP_ERR_LAUNCH_FAILED, "committedExactTokenCount %d must equal committed token count %d", r.metrics.committedExactTokenCount, n);
        if (r.metrics.acceptedFutureTokenCount == 1) {
            if (n != 2) return fail(ESP_ERR_LAUNCH_FAILED, "accepted future token requires exactly two committed tokens");
            if (budget <= 1) return fail(ESP_ERR_LAUNCH_FAILED, "accepted future token requires remaining token budget > 1");
        } else if (r.metrics.stateAdvanceLatencyMs != 0) {
            return fail(ESP_ERR_LAUNCH_FAILED, "stateAdvanceLatencyMs must be zero when no future token is accepted");
        }
        trace->generatedTokens.insert(trace->generatedTokens.end(), r.committedTokens.begin(), r.committedTokens.end());
        trace->passMetrics.push_back(r.metrics);
        current = r.nextCurrentToken;
    }
    return ESP_OK;
}

int HipExactTwoTokenModel::reset() {
    int rc = target_.reset();
    return rc != ESP_OK ? rc : draft_.reset();
}

int HipExactTwoTokenModel::prefillSelectedToken(const std::vector<TokenID> &promptTokens, TokenID *selected) {
    int rc = target_.prefill(0, promptTokens.data(), (int)promptTokens.size());
    if (rc != ESP_OK) return rc;
    if ((rc = draft_.prefill(0, promptTokens.data(), (int)promptTokens.size())) != ESP_OK) return rc;
    return target_.select_greedy(0, selected);
}

int HipExactTwoTokenModel::performExactTwoTokenPass(TokenID currentToken, int remainingTokenBudget, ExactTwoTokenPassResult *result) {
    const auto t0 = Clock::now();
    TokenID proposed = 0;
    int rc = draft_.advance(0, currentToken);
    if (rc != ESP_OK) return rc;
    if ((rc = draft_.select_greedy(0, &proposed)) != ESP_OK) return rc;
    const auto t1 = Clock::now();
    const int pos = target_.visible(0);
    const bool two = remainingTokenBudget > 1 && pos + 1 < target_.config().max_seq;
    StepRows rows{};
    rows.count = two ? 2 : 1;
    rows.token[0] = (int)currentToken; rows.pos[0] = pos; rows.seq[0] = 0;
    rows.token[1] = (int)proposed; rows.pos[1] = pos + 1; rows.seq[1] = 0;
    if ((rc = target_.forward_rows(rows)) != ESP_OK) return rc;
    const auto t2 = Clock::now();
    uint32_t exact[2] = {0, 0};
    if ((rc = target_.head_rows(rows.count, exact)) != ESP_OK) return rc;
    const auto t3 = Clock::now();
    const ExactTwoTokenBranchPromotionPlan plan =
        ExactTwoTokenBranchPromotionPlan::make(currentToken, proposed, exact[0], exact[1], two ? remainingTokenBudget : 1);
    // promotion: keep 1 or 2 of the freshly written KV columns by moving the visible length
    target_.set_visible(0, pos + plan.promotedStepCount);
    if ((rc = target_.keep_row(plan.promotedStepCount - 1, 0)) != ESP_OK) return rc;
    double advance_ms = 0;
    if (plan.promotedStepCount == 2) {
        const auto t4 = Clock::now();
        if ((rc = draft_.advance(0, proposed)) != ESP_OK) return rc;
        advance_ms = ms_between(t4, Clock::now());
        if (advance_ms <= 0) advance_ms = 1e-6;
    }
    result->committedTokens = plan.committedTokens;
    result->nextCurrentToken = plan.nextCurrentToken;
    result->metrics.proposerLatencyMs = ms_between(t0, t1);
    result->metrics.verifierTrunkLatencyMs = ms_between(t1, t2);
    result->metrics.verifierLogitsLatencyMs = ms_between(t2, t3);
    result->metrics.stateAdvanceLatencyMs = advance_ms;
    result->metrics.acceptedFutureTokenCount = plan.acceptedFutureTokenCount;
    result->metrics.committedExactTokenCount = plan.committedExactTokenCount;
    return ESP_OK;
}

}  // namespace esp
