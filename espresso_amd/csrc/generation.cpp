#include "generation.h"

#include <cmath>

#include <chrono>

namespace esp {
namespace {
using Clock = std::chrono::steady_clock;
double ms_since(Clock::time_point t0) { return std::chrono::duration<double, std::milli>(Clock::now() - t0).count(); }
}  // namespace

int generate_greedy(LlamaRuntime &rt, const uint32_t *prompt, int prompt_count, int max_tokens,
                    std::vector<uint32_t> *out, GenerationTiming *timing) {
    out->clear();
    const LlamaConfig &c = rt.config();
    if (prompt_count <= 0 || !prompt) return fail(ESP_ERR_INVALID_ARGUMENT, "Prompt tokens must not be empty");       // (:6200-6202)
    if (max_tokens < 0) return fail(ESP_ERR_INVALID_ARGUMENT, "maxTokens must be >= 0");                               // (:1411-1413)
    if (prompt_count >= c.max_seq) return fail(ESP_ERR_OUT_OF_RANGE, "prompt of %d tokens does not fit context %d", prompt_count, c.max_seq);
    const int eff = max_tokens < c.max_seq - prompt_count ? max_tokens : c.max_seq - prompt_count;
    auto t_prefill = Clock::now();
    int rc = rt.prefill(0, prompt, prompt_count);
    if (rc != ESP_OK) return rc;
    if (timing) timing->prefill_ms = ms_since(t_prefill);

    auto t_start = Clock::now(), t_emit = t_start;
    int all = prompt_count;
    if (c.eos_token < 0 && eff > 1) {
        // No stop token: the first eff-1 tokens need no host decision, so they run as graph replays with
        // one synchronisation; the last token is selected but not advanced, as in the loop below.
        out->resize(eff - 1);
        if ((rc = rt.continue_greedy(0, eff - 1, out->data())) != ESP_OK) return rc;
        all += eff - 1;
        if (timing) {
            const double per_token = ms_since(t_start) / (eff - 1);
            timing->first_token_latency_ms = per_token;
            timing->token_latencies_ms.assign(eff - 1, per_token);   // one measurement for the whole run
        }
        t_emit = Clock::now();
    }
    while ((int)out->size() < eff) {
        uint32_t next = 0;
        if ((rc = rt.select_greedy(0, &next)) != ESP_OK) return rc;
        auto now = Clock::now();
        if (timing) {
            if (out->empty()) timing->first_token_latency_ms = std::chrono::duration<double, std::milli>(now - t_start).count();
            timing->token_latencies_ms.push_back(std::chrono::duration<double, std::milli>(now - t_emit).count());
        }
        out->push_back(next);
        if (c.eos_token >= 0 && next == (uint32_t)c.eos_token) break;   // EOS is appended, then the loop ends (:6385-6388)
        all++;
        if ((int)out->size() >= eff || all >= c.max_seq) break;         // (:6407)
        if ((rc = rt.advance(0, next)) != ESP_OK) return rc;            // position all - 1 (:6411)
        t_emit = now;
    }
    if (timing) timing->decode_ms = ms_since(t_start);
    return ESP_OK;
}

int generate_two_token(LlamaRuntime &full, LlamaRuntime &draft, const uint32_t *prompt, int prompt_count,
                       int max_tokens, bool reference_accounting, std::vector<uint32_t> *out,
                       TwoTokenStats *stats, GenerationTiming *timing) {
    out->clear();
    TwoTokenStats st;
    const LlamaConfig &c = full.config();
    if (prompt_count <= 0 || !prompt) return fail(ESP_ERR_INVALID_ARGUMENT, "Prompt tokens must not be empty");   // (:6021-6023)
    if (max_tokens < 0) return fail(ESP_ERR_INVALID_ARGUMENT, "maxTokens must be >= 0");
    if (draft.config().vocab != c.vocab)
        return fail(ESP_ERR_INVALID_ARGUMENT, "draft vocab %d does not match target vocab %d", draft.config().vocab, c.vocab);  // (:5375-5379)
    if (prompt_count >= c.max_seq || prompt_count >= draft.config().max_seq)
        return fail(ESP_ERR_OUT_OF_RANGE, "prompt of %d tokens does not fit the context", prompt_count);
    const int max_seq = c.max_seq < draft.config().max_seq ? c.max_seq : draft.config().max_seq;
    const int eff = max_tokens < max_seq - prompt_count ? max_tokens : max_seq - prompt_count;
    const int eos = c.eos_token;

    auto t_prefill = Clock::now();
    int rc;
    if ((rc = full.prefill(0, prompt, prompt_count)) != ESP_OK) return rc;
    if ((rc = draft.prefill(0, prompt, prompt_count)) != ESP_OK) return rc;
    if (timing) timing->prefill_ms = ms_since(t_prefill);
    auto t_start = Clock::now(), t_emit = t_start;
    auto emit = [&](uint32_t tok) {
        auto now = Clock::now();
        if (timing) {
            if (out->empty()) timing->first_token_latency_ms = std::chrono::duration<double, std::milli>(now - t_start).count();
            timing->token_latencies_ms.push_back(std::chrono::duration<double, std::milli>(now - t_emit).count());
        }
        t_emit = now;
        out->push_back(tok);
    };
    auto finish = [&]() {
        const int after_first = (int)out->size() - 1;
        if (after_first > 0) {
            st.reference_passes = (after_first + 1) / 2;
            st.reference_committed_total = after_first;
        }
        if (!reference_accounting) st.reference_accepted_total = -1;
        if (stats) *stats = st;
        if (timing) timing->decode_ms = ms_since(t_start);
        return ESP_OK;
    };
    if (eff <= 0) return finish();

    // the first token comes from the prefilled state (:6069-6087)
    uint32_t current = 0;
    if ((rc = full.select_greedy(0, &current)) != ESP_OK) return rc;
    emit(current);
    int all = prompt_count + 1;
    if ((eos >= 0 && current == (uint32_t)eos) || (int)out->size() >= eff || all >= max_seq) return finish();

    // Invariant: `current` is the last emitted token; neither model has consumed it yet.
    while ((int)out->size() < eff && all < max_seq) {
        st.passes++;
        uint32_t proposed = 0;
        if ((rc = draft.advance(0, current)) != ESP_OK) return rc;
        if ((rc = draft.select_greedy(0, &proposed)) != ESP_OK) return rc;

        const int pos = full.visible(0);                       // == all - 1
        const bool can_two = eff - (int)out->size() >= 2 && all + 1 < max_seq;
        StepRows rows{};
        rows.count = can_two ? 2 : 1;
        rows.token[0] = (int)current; rows.pos[0] = pos; rows.seq[0] = 0;
        rows.token[1] = (int)proposed; rows.pos[1] = pos + 1; rows.seq[1] = 0;
        uint32_t exact[2] = {0, 0};
        if ((rc = full.forward_rows(rows)) != ESP_OK) return rc;
        if ((rc = full.head_rows(rows.count, exact)) != ESP_OK) return rc;

        // row 0 is always exact: keep its KV column and emit the token that follows it
        full.set_visible(0, pos + 1);
        emit(exact[0]);
        all++;
        st.committed_total++;
        if (reference_accounting && proposed == exact[0]) st.reference_accepted_total++;
        const bool accepted = can_two && proposed == exact[0];
        if ((eos >= 0 && exact[0] == (uint32_t)eos) || (int)out->size() >= eff || all >= max_seq) {
            if ((rc = full.keep_row(0, 0)) != ESP_OK) return rc;
            break;
        }
        if (!accepted) {
            if ((rc = full.keep_row(0, 0)) != ESP_OK) return rc;
            current = exact[0];
            continue;
        }
        // the proposal was right: row 1 ran on the exact token, so its column and its successor stand
        st.accepted_total++;
        st.committed_total++;
        full.set_visible(0, pos + 2);
        if ((rc = full.keep_row(1, 0)) != ESP_OK) return rc;
        if ((rc = draft.advance(0, proposed)) != ESP_OK) return rc;
        if (reference_accounting) {
            uint32_t p1 = 0;
            if ((rc = draft.select_greedy(0, &p1)) != ESP_OK) return rc;
            if (p1 == exact[1]) st.reference_accepted_total++;
        }
        emit(exact[1]);
        all++;
        current = exact[1];
        if (eos >= 0 && exact[1] == (uint32_t)eos) break;
    }
    return finish();
}

int sample_token(const float *logits, int count, float temperature, double unit) {
    if (count <= 0) return 0;
    auto first_max = [&]() { int b = 0; for (int i = 1; i < count; i++) if (logits[b] < logits[i]) b = i; return b; };
    if (temperature <= 0.0f) return first_max();
    float max_logit = logits[0];
    for (int i = 1; i < count; i++) if (logits[i] > max_logit) max_logit = logits[i];
    std::vector<double> scaled(count);
    double total = 0.0;
    for (int i = 0; i < count; i++) {
        scaled[i] = std::exp((double)((logits[i] - max_logit) / temperature));
        total += scaled[i];
    }
    if (!std::isfinite(total) || total <= 0.0) return first_max();
    double threshold = unit * total;
    for (int i = 0; i < count; i++) {
        threshold -= scaled[i];
        if (threshold <= 0.0) return i;
    }
    return count - 1;
}

int generate_sampled(LlamaRuntime &rt, const uint32_t *prompt, int prompt_count, int max_tokens, float temperature,
                     uint64_t seed, std::vector<uint32_t> *out, GenerationTiming *timing) {
    out->clear();
    const LlamaConfig &c = rt.config();
    if (prompt_count <= 0 || !prompt) return fail(ESP_ERR_INVALID_ARGUMENT, "Prompt tokens must not be empty");
    if (max_tokens < 0) return fail(ESP_ERR_INVALID_ARGUMENT, "maxTokens must be >= 0");
    if (prompt_count >= c.max_seq) return fail(ESP_ERR_OUT_OF_RANGE, "prompt of %d tokens does not fit the context", prompt_count);
    const int eff = max_tokens < c.max_seq - prompt_count ? max_tokens : c.max_seq - prompt_count;
    auto t_prefill = Clock::now();
    int rc = rt.prefill(0, prompt, prompt_count);
    if (rc != ESP_OK) return rc;
    if (timing) timing->prefill_ms = ms_since(t_prefill);
    auto t_start = Clock::now(), t_emit = t_start;
    SplitMix64 rng{seed};
    std::vector<float> logits(c.vocab);
    int all = prompt_count;
    while ((int)out->size() < eff && all < c.max_seq) {
        if ((rc = rt.read_logits(0, logits.data())) != ESP_OK) return rc;
        const uint32_t tok = (uint32_t)sample_token(logits.data(), c.vocab, temperature, rng.unit());
        auto now = Clock::now();
        if (timing) {
            if (out->empty()) timing->first_token_latency_ms = std::chrono::duration<double, std::milli>(now - t_start).count();
            timing->token_latencies_ms.push_back(std::chrono::duration<double, std::milli>(now - t_emit).count());
        }
        t_emit = now;
        out->push_back(tok);
        all++;
        if (c.eos_token >= 0 && tok == (uint32_t)c.eos_token) break;        // appended, then stop (:6385-6388)
        if ((int)out->size() >= eff || all >= c.max_seq) break;
        if ((rc = rt.advance(0, tok)) != ESP_OK) return rc;
    }
    if (timing) timing->decode_ms = ms_since(t_start);
    return ESP_OK;
}

// ---- lock-step batches of independent sequences ---------------------------------------------------
// Sequence s of `n_seq` uses KV cache s of both runtimes.  Greedy, no EOS handling (the batched configs
// decode a fixed budget); every sequence produces exactly `eff` tokens.
static int batch_budget(const LlamaRuntime &a, const LlamaRuntime *b, const int *prompt_counts, int n_seq, int max_tokens, int *eff) {
    if (n_seq < 1 || n_seq > a.config().max_sequences || (b && n_seq > b->config().max_sequences) || 2 * n_seq > kMaxStepRows)
        return fail(ESP_ERR_INVALID_ARGUMENT, "batch of %d sequences does not fit the runtime", n_seq);
    int max_seq = a.config().max_seq;
    if (b && b->config().max_seq < max_seq) max_seq = b->config().max_seq;
    int budget = max_tokens;
    for (int s = 0; s < n_seq; s++) {
        if (prompt_counts[s] <= 0) return fail(ESP_ERR_INVALID_ARGUMENT, "Prompt tokens must not be empty");
        if (prompt_counts[s] >= max_seq) return fail(ESP_ERR_OUT_OF_RANGE, "prompt of %d tokens does not fit the context", prompt_counts[s]);
        if (max_seq - prompt_counts[s] < budget) budget = max_seq - prompt_counts[s];
    }
    *eff = budget < 0 ? 0 : budget;
    return ESP_OK;
}

int generate_greedy_batch(LlamaRuntime &rt, const uint32_t *const *prompts, const int *prompt_counts, int n_seq, int max_tokens,
                          std::vector<std::vector<uint32_t>> *out, double *decode_ms) {
    out->assign(n_seq, {});
    int eff = 0, rc = batch_budget(rt, nullptr, prompt_counts, n_seq, max_tokens, &eff);
    if (rc != ESP_OK) return rc;
    for (int s = 0; s < n_seq; s++)
        if ((rc = rt.prefill(s, prompts[s], prompt_counts[s])) != ESP_OK) return rc;
    auto t0 = Clock::now();
    if (eff > 0) {
        std::vector<uint32_t> current(n_seq);
        for (int s = 0; s < n_seq; s++) {
            if ((rc = rt.select_greedy(s, &current[s])) != ESP_OK) return rc;
            (*out)[s].push_back(current[s]);
        }
        for (int step = 1; step < eff; step++) {
            StepRows rows{};
            rows.count = n_seq;
            for (int s = 0; s < n_seq; s++) { rows.token[s] = (int)current[s]; rows.pos[s] = rt.visible(s); rows.seq[s] = s; }
            uint32_t next[kMaxStepRows];
            if ((rc = rt.forward_rows(rows)) != ESP_OK) return rc;
            if ((rc = rt.head_rows(n_seq, next)) != ESP_OK) return rc;
            for (int s = 0; s < n_seq; s++) {
                rt.set_visible(s, rows.pos[s] + 1);
                current[s] = next[s];
                (*out)[s].push_back(next[s]);
            }
        }
    }
    if (decode_ms) *decode_ms = ms_since(t0);
    return ESP_OK;
}

// The exact two-token loop over `n_seq` sequences in lock step: one draft pass over the sequences' current
// tokens, one target pass over (current, proposed) of every sequence (2 * n_seq rows sharing one read of the
// weights), a second draft pass over the sequences whose proposal was right.  Per sequence the rule is the
// single-sequence loop's: row 0 is always exact; row 1 stands iff the proposal equals the exact successor.
int generate_two_token_batch(LlamaRuntime &full, LlamaRuntime &draft, const uint32_t *const *prompts, const int *prompt_counts,
                             int n_seq, int max_tokens, std::vector<std::vector<uint32_t>> *out, TwoTokenStats *stats, double *decode_ms) {
    out->assign(n_seq, {});
    TwoTokenStats st;
    if (draft.config().vocab != full.config().vocab)
        return fail(ESP_ERR_INVALID_ARGUMENT, "draft vocab %d does not match target vocab %d", draft.config().vocab, full.config().vocab);
    int eff = 0, rc = batch_budget(full, &draft, prompt_counts, n_seq, max_tokens, &eff);
    if (rc != ESP_OK) return rc;
    for (int s = 0; s < n_seq; s++) {
        if ((rc = full.prefill(s, prompts[s], prompt_counts[s])) != ESP_OK) return rc;
        if ((rc = draft.prefill(s, prompts[s], prompt_counts[s])) != ESP_OK) return rc;
    }
    auto t0 = Clock::now();
    std::vector<uint32_t> current(n_seq);
    if (eff > 0) {
        for (int s = 0; s < n_seq; s++) {
            if ((rc = full.select_greedy(s, &current[s])) != ESP_OK) return rc;
            (*out)[s].push_back(current[s]);
        }
    }
    auto active = [&](int s) { return (int)(*out)[s].size() < eff; };
    for (;;) {
        std::vector<int> live;
        for (int s = 0; s < n_seq; s++) if (active(s)) live.push_back(s);
        if (live.empty()) break;
        st.passes++;
        // draft: consume every live sequence's current token, propose its successor
        StepRows dr{};
        dr.count = (int)live.size();
        for (int i = 0; i < dr.count; i++) { const int s = live[i]; dr.token[i] = (int)current[s]; dr.pos[i] = draft.visible(s); dr.seq[i] = s; }
        uint32_t proposed[kMaxStepRows];
        if ((rc = draft.forward_rows(dr)) != ESP_OK) return rc;
        if ((rc = draft.head_rows(dr.count, proposed)) != ESP_OK) return rc;
        for (int i = 0; i < dr.count; i++) draft.set_visible(live[i], dr.pos[i] + 1);
        // target: (current, proposed) of every live sequence; the second row only where two tokens still fit
        StepRows vr{};
        std::vector<int> row0(live.size()), row1(live.size(), -1);
        for (size_t i = 0; i < live.size(); i++) {
            const int s = live[i], pos = full.visible(s);
            row0[i] = vr.count;
            vr.token[vr.count] = (int)current[s]; vr.pos[vr.count] = pos; vr.seq[vr.count] = s; vr.count++;
            if (eff - (int)(*out)[s].size() >= 2) {
                row1[i] = vr.count;
                vr.token[vr.count] = (int)proposed[i]; vr.pos[vr.count] = pos + 1; vr.seq[vr.count] = s; vr.count++;
            }
        }
        uint32_t exact[kMaxStepRows];
        if ((rc = full.forward_rows(vr)) != ESP_OK) return rc;
        if ((rc = full.head_rows(vr.count, exact)) != ESP_OK) return rc;
        StepRows ar{};   // accepted sequences: the draft consumes the proposal as well
        for (size_t i = 0; i < live.size(); i++) {
            const int s = live[i], pos = vr.pos[row0[i]];
            const uint32_t e0 = exact[row0[i]];
            (*out)[s].push_back(e0);
            st.committed_total++;
            const bool accepted = row1[i] >= 0 && proposed[i] == e0;
            if (!accepted) {
                full.set_visible(s, pos + 1);
                if ((rc = full.keep_row(row0[i], s)) != ESP_OK) return rc;
                current[s] = e0;
                continue;
            }
            st.accepted_total++;
            st.committed_total++;
            full.set_visible(s, pos + 2);
            if ((rc = full.keep_row(row1[i], s)) != ESP_OK) return rc;
            (*out)[s].push_back(exact[row1[i]]);
            current[s] = exact[row1[i]];
            ar.token[ar.count] = (int)proposed[i]; ar.pos[ar.count] = draft.visible(s); ar.seq[ar.count] = s; ar.count++;
        }
        if (ar.count > 0) {
            if ((rc = draft.forward_rows(ar)) != ESP_OK) return rc;
            for (int i = 0; i < ar.count; i++) draft.set_visible(ar.seq[i], ar.pos[i] + 1);
        }
    }
    if (stats) *stats = st;
    if (decode_ms) *decode_ms = ms_since(t0);
    return ESP_OK;
}

}  // namespace esp
