#include "generation.h"

#include <cmath>

#include <chrono>

namespace esp {
namespace {
using Clock = std::chrono::steady_clock;
double ms_since(Clock::time_point t0) { return std::chrono::duration<double, std::milli>(Clock::now() - t0).count(); }

// A pass of a generation loop as a captured graph: the first pass runs as plain launches (whatever a kernel configures on its first
// use happens outside the capture), later ones replay.
struct PassGraph {
    hipGraphExec_t exec = nullptr;
    ~PassGraph() { if (exec) (void)hipGraphExecDestroy(exec); }
    template <class Enqueue>
    int capture(Enqueue enqueue) {
        hipStream_t s = context().stream;
        hipGraph_t graph = nullptr;
        hipError_t e = hipStreamBeginCapture(s, hipStreamCaptureModeThreadLocal);
        if (e != hipSuccess) return fail_hip(e, "hipStreamBeginCapture");
        int rc = enqueue();
        e = hipStreamEndCapture(s, &graph);
        if (rc == ESP_OK && e != hipSuccess) rc = fail_hip(e, "hipStreamEndCapture");
        if (rc == ESP_OK && (e = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0)) != hipSuccess) rc = fail_hip(e, "hipGraphInstantiate");
        if (graph) (void)hipGraphDestroy(graph);
        return rc;
    }
    int launch(int times) {
        for (int i = 0; i < times; i++) {
            const hipError_t e = hipGraphLaunch(exec, context().stream);
            if (e != hipSuccess) return fail_hip(e, "hipGraphLaunch");
        }
        return ESP_OK;
    }
};
template <class T>
struct DeviceArray {
    T *p = nullptr;
    ~DeviceArray() { if (p) (void)hipFree(p); }
    int alloc(size_t count) { return device_alloc(&p, count); }
};
int hip_ok(hipError_t e, const char *what) { return e == hipSuccess ? ESP_OK : fail_hip(e, what); }

// One pass of the exact two-token loop with every decision on the device (TwoTokenState): the draft runs two rows (the row
// it owes after an accepted pass and the current token, or the current token twice) and proposes; the target verifies
// (current, proposed); the accept kernel emits, keeps the hidden row and writes the next pass's rows.  No host decision, so
// the pass replays as a captured graph.
// draft_rows_embedded: the pass before this one left the embeddings of the draft's two rows in its hidden rows (its accept kernel
// does); the first pass after the host set the rows has to fetch them itself.
int enqueue_two_token_pass(LlamaRuntime &full, LlamaRuntime &draft, TwoTokenState *state, int *log, int log_capacity, bool draft_rows_embedded) {
    hipStream_t s = context().stream;
    int rc;
    if ((rc = draft.enqueue_device_rows(2, draft_rows_embedded)) != ESP_OK) return rc;
    if ((rc = draft.enqueue_device_head(2)) != ESP_OK) return rc;
    // the two small kernels between the models also fetch the embedding rows of the model that runs next: two launches fewer per pass
    ESP_HIP_TRY(launch_two_token_verify_rows(state, draft.device_head_tokens(), full.device_row_tokens(), full.device_row_positions(),
                                             full.device_embed_target(), s));
    if ((rc = full.enqueue_device_rows(2, true)) != ESP_OK) return rc;
    if ((rc = full.enqueue_device_head(2)) != ESP_OK) return rc;
    EmbedTarget draft_rows = draft.device_embed_target();
    draft_rows.keep_row1 = draft.device_last_hidden(0);   // the draft's last output row, before the embeddings replace it
    ESP_HIP_TRY(launch_two_token_accept(state, full.device_head_tokens(), log, log_capacity, full.device_hidden_rows(), full.device_last_hidden(0),
                                        full.config().d_model, draft.device_row_tokens(), draft.device_row_positions(), draft_rows, s));
    return ESP_OK;
}

// Runs passes on the device until the loop ends or a pass would need a host decision (fewer than two tokens of budget or two
// positions of context left).  `state` comes in with the host loop's variables and goes out with them; log receives the
// emitted tokens at their output indices.
int run_two_token_passes_on_device(LlamaRuntime &full, LlamaRuntime &draft, TwoTokenState *state, std::vector<int> *log) {
    hipStream_t s = context().stream;
    constexpr int kPassesPerGraph = 4;   // a boundary between two graph launches costs ~3.5 us on the device
    const int capacity = state->budget + 2;
    log->assign(capacity, 0);
    auto hip = [&](hipError_t e, const char *what) { return e == hipSuccess ? ESP_OK : fail_hip(e, what); };
    // State, log and the captured passes live in the target's session from call to call (a call costs neither an allocation
    // nor a capture after the first); the session is rebuilt when the partner or either runtime's kernels changed.
    DeviceLoopSession &ss = full.loop_session();
    if (ss.partner_id != draft.id() || ss.epoch != full.graph_epoch() || ss.partner_epoch != draft.graph_epoch() || ss.log_capacity < capacity) {
        full.release_loop_session();
        TwoTokenState *fresh_state = nullptr;
        int *fresh_log = nullptr;
        const int log_capacity = full.config().max_seq + 2 > capacity ? full.config().max_seq + 2 : capacity;
        int rc = device_alloc(&fresh_state, (size_t)1);
        if (rc == ESP_OK) rc = device_alloc(&fresh_log, (size_t)log_capacity);
        if (rc != ESP_OK) { if (fresh_state) (void)hipFree(fresh_state); return rc; }
        ss.state = fresh_state; ss.log = fresh_log; ss.log_capacity = log_capacity;
        ss.partner_id = draft.id(); ss.epoch = full.graph_epoch(); ss.partner_epoch = draft.graph_epoch();
    }
    TwoTokenState *d_state = static_cast<TwoTokenState *>(ss.state);
    int *d_log = ss.log;
    int rc;
    auto fetch = [&]() {
        int r = hip(hipMemcpyAsync(state, d_state, sizeof(TwoTokenState), hipMemcpyDeviceToHost, s), "two-token state");
        if (r == ESP_OK) r = hip(hipStreamSynchronize(s), "two-token pass");
        return r;
    };
    StepRows rows{};
    rows.count = 2;
    rows.token[0] = rows.token[1] = state->current;
    rows.pos[0] = rows.pos[1] = state->full_pos;
    rows.seq[0] = rows.seq[1] = 0;
    if ((rc = hip(hipMemcpyAsync(d_state, state, sizeof(TwoTokenState), hipMemcpyHostToDevice, s), "two-token state")) != ESP_OK) return rc;
    if ((rc = hip(launch_set_rows(rows, draft.device_row_tokens(), draft.device_row_positions(), draft.device_row_sequences(), s), "rows")) != ESP_OK) return rc;
    if ((rc = hip(launch_set_rows(rows, full.device_row_tokens(), full.device_row_positions(), full.device_row_sequences(), s), "rows")) != ESP_OK) return rc;
    // the first pass runs as plain launches: whatever a kernel configures on its first use happens outside the capture, and
    // the draft's rows are embedded by the pass itself (later passes find them embedded by the pass before)
    if ((rc = enqueue_two_token_pass(full, draft, d_state, d_log, ss.log_capacity, false)) != ESP_OK) return rc;
    if ((rc = fetch()) != ESP_OK) return rc;
    auto capture = [&](int passes, hipGraphExec_t *out) {
        hipGraph_t graph = nullptr;
        int r = hip(hipStreamBeginCapture(s, hipStreamCaptureModeThreadLocal), "hipStreamBeginCapture");
        if (r != ESP_OK) return r;
        for (int p = 0; p < passes && r == ESP_OK; p++) r = enqueue_two_token_pass(full, draft, d_state, d_log, ss.log_capacity, true);
        const hipError_t e = hipStreamEndCapture(s, &graph);
        if (r == ESP_OK) r = hip(e, "hipStreamEndCapture");
        if (r == ESP_OK) r = hip(hipGraphInstantiate(out, graph, nullptr, nullptr, 0), "hipGraphInstantiate");
        if (graph) (void)hipGraphDestroy(graph);
        return r;
    };
    while (!state->done) {
        if (!ss.one && (rc = capture(1, &ss.one)) != ESP_OK) return rc;
        // a pass emits one or two tokens: half of what is left can never overrun, and passes after the end change nothing
        const int left = state->budget - state->emitted, chunk = left / 2 > 1 ? left / 2 : 1;
        if (!ss.many && chunk >= kPassesPerGraph && (rc = capture(kPassesPerGraph, &ss.many)) != ESP_OK) return rc;
        int i = 0;
        if (ss.many)
            for (; i + kPassesPerGraph <= chunk; i += kPassesPerGraph)
                if ((rc = hip(hipGraphLaunch(ss.many, s), "hipGraphLaunch")) != ESP_OK) return rc;
        for (; i < chunk; i++)
            if ((rc = hip(hipGraphLaunch(ss.one, s), "hipGraphLaunch")) != ESP_OK) return rc;
        if ((rc = fetch()) != ESP_OK) return rc;
    }
    rc = hip(hipMemcpyAsync(log->data(), d_log, sizeof(int) * capacity, hipMemcpyDeviceToHost, s), "two-token log");
    if (rc == ESP_OK) rc = hip(hipStreamSynchronize(s), "two-token log");
    return rc;
}
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
    if (eff > 1) {
        // The first eff-1 tokens need no host decision (the step graph notices a stop token by itself), so they run as graph
        // replays with a synchronisation at the end or every 32 tokens; the last token is selected but not advanced, as in the
        // loop below.
        out->resize(eff - 1);
        int produced = eff - 1;
        if (c.eos_token < 0) rc = rt.continue_greedy(0, eff - 1, out->data());
        else rc = rt.continue_greedy_until_stop(0, eff - 1, out->data(), &produced);
        if (rc != ESP_OK) return rc;
        out->resize(produced);
        all += produced;
        if (timing && produced > 0) {
            const double per_token = ms_since(t_start) / produced;
            timing->first_token_latency_ms = per_token;
            timing->token_latencies_ms.assign(produced, per_token);   // one measurement for the whole run
        }
        t_emit = Clock::now();
        if (produced > 0 && c.eos_token >= 0 && out->back() == (uint32_t)c.eos_token) {   // EOS is appended, then the loop ends (:6385-6388)
            if (timing) timing->decode_ms = ms_since(t_start);
            return ESP_OK;
        }
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

    // Full passes (two tokens of budget and two positions of context left) run on the device, one captured graph per pass and
    // no host decision in between; what is left afterwards (at most one pass) takes the loop below.
    if (full.graph_replay_enabled() && draft.graph_replay_enabled() && &full != &draft && eff - (int)out->size() >= 2 && all + 1 < max_seq) {
        TwoTokenState ds{};
        ds.current = (int)current; ds.full_pos = full.visible(0); ds.emitted = (int)out->size(); ds.budget = eff; ds.all = all;
        ds.max_seq = max_seq; ds.eos = eos; ds.reference_accounting = reference_accounting ? 1 : 0;
        std::vector<int> log;
        const auto t_device = Clock::now();
        const int first = ds.emitted;
        if ((rc = run_two_token_passes_on_device(full, draft, &ds, &log)) != ESP_OK) return rc;
        const double per_token = ms_since(t_device) / (ds.emitted - first > 0 ? ds.emitted - first : 1);
        for (int i = first; i < ds.emitted; i++) {
            out->push_back((uint32_t)log[i]);
            if (timing) timing->token_latencies_ms.push_back(per_token);   // one measurement for all of them
        }
        t_emit = Clock::now();
        st.passes += ds.passes; st.committed_total += ds.committed_total; st.accepted_total += ds.accepted_total;
        st.reference_accepted_total += ds.reference_accepted_total;
        all = ds.all;
        current = (uint32_t)ds.current;
        // both models as the host loop would have left them: the draft has consumed what the target has, less the row it owes
        if ((rc = full.set_visible(0, ds.full_pos)) != ESP_OK) return rc;
        if ((rc = draft.set_visible(0, ds.full_pos - (ds.accepted_prev ? 1 : 0))) != ESP_OK) return rc;
        // (the draft's last output row was kept by the pass's last kernel, which then put the next rows' embeddings in its place)
        if (ds.accepted_prev) {
            if ((rc = draft.advance(0, (uint32_t)ds.proposed_prev)) != ESP_OK) return rc;
            if (reference_accounting) {
                uint32_t p1 = 0;
                if ((rc = draft.select_greedy(0, &p1)) != ESP_OK) return rc;
                if (p1 == (uint32_t)ds.exact1_prev) st.reference_accepted_total++;
            }
        }
        if (ds.stopped) return finish();
    }

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
        int first_host_step = 1;
        if (rt.graph_replay_enabled() && eff > 2) {
            // every step but none of the decisions needs the host: rows feed themselves on the device, one graph per step
            hipStream_t st = context().stream;
            const int steps = eff - 1;
            DeviceArray<int> d_log, d_step;
            if ((rc = d_log.alloc((size_t)steps * n_seq)) != ESP_OK || (rc = d_step.alloc(1)) != ESP_OK) return rc;
            StepRows rows{};
            rows.count = n_seq;
            for (int s = 0; s < n_seq; s++) { rows.token[s] = (int)current[s]; rows.pos[s] = rt.visible(s); rows.seq[s] = s; }
            if ((rc = hip_ok(launch_set_rows(rows, rt.device_row_tokens(), rt.device_row_positions(), rt.device_row_sequences(), st), "rows")) != ESP_OK) return rc;
            if ((rc = hip_ok(launch_set_ints(d_step.p, 0, nullptr, 0, st), "step")) != ESP_OK) return rc;
            auto pass = [&]() {
                int r = rt.enqueue_device_rows(n_seq);
                if (r == ESP_OK) r = rt.enqueue_device_head(n_seq);
                if (r == ESP_OK) r = hip_ok(launch_batch_greedy_feed(rt.device_head_tokens(), n_seq, rt.device_row_tokens(), rt.device_row_positions(), d_log.p,
                                                                     d_step.p, steps, st), "feed");
                return r;
            };
            PassGraph graph;
            if ((rc = pass()) != ESP_OK) return rc;
            if ((rc = graph.capture(pass)) != ESP_OK) return rc;
            if ((rc = graph.launch(steps - 1)) != ESP_OK) return rc;
            std::vector<int> log((size_t)steps * n_seq);
            if ((rc = hip_ok(hipMemcpyAsync(log.data(), d_log.p, sizeof(int) * log.size(), hipMemcpyDeviceToHost, st), "log")) != ESP_OK) return rc;
            if ((rc = hip_ok(hipStreamSynchronize(st), "greedy batch")) != ESP_OK) return rc;
            for (int s = 0; s < n_seq; s++) {
                for (int i = 0; i < steps; i++) (*out)[s].push_back((uint32_t)log[(size_t)i * n_seq + s]);
                rt.set_visible(s, rt.visible(s) + steps);
            }
            first_host_step = eff;
        }
        for (int step = first_host_step; step < eff; step++) {
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
    if (full.graph_replay_enabled() && draft.graph_replay_enabled() && &full != &draft && eff > 2 && n_seq <= kMaxLoopSequences) {
        // the passes run on the device: per-sequence variables in TwoTokenBatchState, rows 2 s and 2 s + 1 of both models belong to
        // sequence s, a sequence whose budget is spent keeps replaying its last rows (which rewrite the same values)
        hipStream_t strm = context().stream;
        TwoTokenBatchState h{};
        h.n_seq = n_seq; h.budget = eff;
        StepRows rows{};
        rows.count = 2 * n_seq;
        for (int s = 0; s < n_seq; s++) {
            h.current[s] = (int)current[s]; h.full_pos[s] = full.visible(s); h.emitted[s] = 1;
            for (int k = 0; k < 2; k++) { rows.token[2 * s + k] = (int)current[s]; rows.pos[2 * s + k] = full.visible(s); rows.seq[2 * s + k] = s; }
        }
        DeviceArray<TwoTokenBatchState> d_state;
        DeviceArray<int> d_log;
        if ((rc = d_state.alloc(1)) != ESP_OK || (rc = d_log.alloc((size_t)n_seq * eff)) != ESP_OK) return rc;
        if ((rc = hip_ok(hipMemcpyAsync(d_state.p, &h, sizeof(h), hipMemcpyHostToDevice, strm), "state")) != ESP_OK) return rc;
        if ((rc = hip_ok(launch_set_rows(rows, draft.device_row_tokens(), draft.device_row_positions(), draft.device_row_sequences(), strm), "rows")) != ESP_OK) return rc;
        if ((rc = hip_ok(launch_set_rows(rows, full.device_row_tokens(), full.device_row_positions(), full.device_row_sequences(), strm), "rows")) != ESP_OK) return rc;
        auto pass = [&]() {
            int r = draft.enqueue_device_rows(2 * n_seq);
            if (r == ESP_OK) r = draft.enqueue_device_head(2 * n_seq);
            if (r == ESP_OK) r = hip_ok(launch_two_token_batch_verify_rows(d_state.p, draft.device_head_tokens(), full.device_row_tokens(), full.device_row_positions(), strm), "verify rows");
            if (r == ESP_OK) r = full.enqueue_device_rows(2 * n_seq);
            if (r == ESP_OK) r = full.enqueue_device_head(2 * n_seq);
            if (r == ESP_OK) r = hip_ok(launch_two_token_batch_accept(d_state.p, n_seq, full.device_head_tokens(), d_log.p, full.device_hidden_rows(), full.device_last_hidden(0),
                                                                      full.config().d_model, draft.device_row_tokens(), draft.device_row_positions(), strm), "accept");
            return r;
        };
        auto fetch = [&]() {
            int r = hip_ok(hipMemcpyAsync(&h, d_state.p, sizeof(h), hipMemcpyDeviceToHost, strm), "state");
            if (r == ESP_OK) r = hip_ok(hipStreamSynchronize(strm), "two-token batch pass");
            return r;
        };
        auto fewest = [&]() { int m = h.emitted[0]; for (int s = 1; s < n_seq; s++) m = h.emitted[s] < m ? h.emitted[s] : m; return m; };
        PassGraph graph;
        if ((rc = pass()) != ESP_OK || (rc = fetch()) != ESP_OK) return rc;
        while (fewest() < eff) {
            if (!graph.exec && (rc = graph.capture(pass)) != ESP_OK) return rc;
            const int left = eff - fewest();
            if ((rc = graph.launch(left / 2 > 1 ? left / 2 : 1)) != ESP_OK || (rc = fetch()) != ESP_OK) return rc;
        }
        std::vector<int> log((size_t)n_seq * eff);
        if ((rc = hip_ok(hipMemcpyAsync(log.data(), d_log.p, sizeof(int) * log.size(), hipMemcpyDeviceToHost, strm), "log")) != ESP_OK) return rc;
        if ((rc = hip_ok(hipStreamSynchronize(strm), "two-token batch log")) != ESP_OK) return rc;
        StepRows owed{};
        for (int s = 0; s < n_seq; s++) {
            for (int i = 1; i < eff; i++) (*out)[s].push_back((uint32_t)log[(size_t)s * eff + i]);
            st.committed_total += h.committed[s]; st.accepted_total += h.accepted[s];
            if ((rc = full.set_visible(s, h.full_pos[s])) != ESP_OK) return rc;
            if ((rc = draft.set_visible(s, h.full_pos[s] - (h.accepted_prev[s] ? 1 : 0))) != ESP_OK) return rc;
            if (h.accepted_prev[s]) {   // the row the draft still owes, as the host loop runs it at the end of an accepting pass
                owed.token[owed.count] = h.proposed_prev[s]; owed.pos[owed.count] = draft.visible(s); owed.seq[owed.count] = s; owed.count++;
            }
        }
        st.passes += h.passes;
        if (owed.count > 0) {
            if ((rc = draft.forward_rows(owed)) != ESP_OK) return rc;
            for (int i = 0; i < owed.count; i++) draft.set_visible(owed.seq[i], owed.pos[i] + 1);
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
