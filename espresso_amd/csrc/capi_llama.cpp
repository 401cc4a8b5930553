// C ABI: the GPU-resident llama runtime and its generation loops.
#include "generation.h"

using namespace esp;

namespace {
int bad_handle() { return fail(ESP_ERR_INVALID_ARGUMENT, "null runtime handle"); }
void fill_stats(ESPGenerationStats *stats, const GenerationTiming &t, size_t generated) {
    if (!stats) return;
    stats->generated = (int32_t)generated;
    stats->prefill_ms = t.prefill_ms;
    stats->decode_ms = t.decode_ms;
    stats->first_token_latency_ms = t.first_token_latency_ms;
    stats->tokens_per_second = generated ? (double)generated / (t.decode_ms > 1e-9 ? t.decode_ms / 1e3 : 1e-9) : 0.0;
}
}  // namespace

extern "C" {

ESPLlamaRuntime *esp_llama_create(const ESPLlamaConfig *config) {
    if (!config) { fail(ESP_ERR_INVALID_ARGUMENT, "null config"); return nullptr; }
    LlamaConfig c;
    c.n_layer = config->n_layer; c.n_head = config->n_head; c.n_kv_head = config->n_kv_head;
    c.d_model = config->d_model; c.head_dim = config->head_dim; c.hidden_dim = config->hidden_dim;
    c.vocab = config->vocab; c.max_seq = config->max_seq; c.norm_eps = config->norm_eps;
    c.rope_theta = config->rope_theta; c.eos_token = config->eos_token; c.kv_format = config->kv_format;
    c.max_sequences = config->max_sequences;
    LlamaRuntime *rt = nullptr;
    if (LlamaRuntime::create(c, &rt) != ESP_OK) return nullptr;
    ESPLlamaRuntime *h = new ESPLlamaRuntime();
    h->rt = rt;
    return h;
}

void esp_llama_free(ESPLlamaRuntime *runtime) {
    if (!runtime) return;
    delete runtime->rt;
    delete runtime;
}

int esp_llama_set_weight(ESPLlamaRuntime *runtime, int layer, int slot, int format, const void *data, size_t bytes) {
    return runtime ? runtime->rt->set_weight(layer, slot, format, data, bytes) : bad_handle();
}
int esp_llama_finalize(ESPLlamaRuntime *runtime) { return runtime ? runtime->rt->finalize() : bad_handle(); }
size_t esp_llama_weight_bytes(const ESPLlamaRuntime *runtime) { return runtime ? runtime->rt->weight_bytes_per_token() : 0; }
size_t esp_llama_resident_weight_bytes(const ESPLlamaRuntime *runtime) { return runtime ? runtime->rt->resident_weight_bytes() : 0; }
int esp_llama_reset(ESPLlamaRuntime *runtime) { return runtime ? runtime->rt->reset() : bad_handle(); }
int esp_llama_prefill(ESPLlamaRuntime *runtime, int sequence, const uint32_t *tokens, int count) {
    if (!runtime) return bad_handle();
    if (!runtime->rt->finalized()) return fail(ESP_ERR_INVALID_ARGUMENT, "runtime is not finalized");
    return runtime->rt->prefill(sequence, tokens, count);
}
int esp_llama_advance(ESPLlamaRuntime *runtime, int sequence, uint32_t token) {
    if (!runtime) return bad_handle();
    if (!runtime->rt->finalized()) return fail(ESP_ERR_INVALID_ARGUMENT, "runtime is not finalized");
    return runtime->rt->advance(sequence, token);
}
int esp_llama_select_greedy_token(ESPLlamaRuntime *runtime, int sequence, uint32_t *token) {
    return runtime ? runtime->rt->select_greedy(sequence, token) : bad_handle();
}
int esp_llama_visible_token_count(const ESPLlamaRuntime *runtime, int sequence) {
    return runtime ? runtime->rt->visible(sequence) : -1;
}
int esp_llama_set_visible_token_count(ESPLlamaRuntime *runtime, int sequence, int count) {
    return runtime ? runtime->rt->set_visible(sequence, count) : bad_handle();
}
int esp_llama_read_last_hidden(ESPLlamaRuntime *runtime, int sequence, float *out) {
    return runtime ? runtime->rt->read_last_hidden(sequence, out) : bad_handle();
}
int esp_llama_read_logits(ESPLlamaRuntime *runtime, int sequence, float *out) {
    return runtime ? runtime->rt->read_logits(sequence, out) : bad_handle();
}

int esp_llama_generate(ESPLlamaRuntime *runtime, const uint32_t *prompt, int prompt_count, int max_tokens,
                       uint32_t *out_tokens, int *out_count, ESPGenerationStats *stats, double *token_latencies_ms) {
    if (!runtime) return bad_handle();
    if (!runtime->rt->finalized()) return fail(ESP_ERR_INVALID_ARGUMENT, "runtime is not finalized");
    if (out_count) *out_count = 0;
    std::vector<uint32_t> toks;
    GenerationTiming timing;
    int rc = generate_greedy(*runtime->rt, prompt, prompt_count, max_tokens, &toks, &timing);
    if (rc != ESP_OK) return rc;
    for (size_t i = 0; i < toks.size(); i++) {
        if (out_tokens) out_tokens[i] = toks[i];
        if (token_latencies_ms) token_latencies_ms[i] = timing.token_latencies_ms[i];
    }
    if (out_count) *out_count = (int)toks.size();
    fill_stats(stats, timing, toks.size());
    return ESP_OK;
}

int esp_llama_generate_two_token(ESPLlamaRuntime *target, ESPLlamaRuntime *draft, const uint32_t *prompt,
                                 int prompt_count, int max_tokens, int reference_accounting,
                                 uint32_t *out_tokens, int *out_count, ESPGenerationStats *stats,
                                 ESPTwoTokenStats *two_token_stats) {
    if (!target || !draft) return bad_handle();
    if (!target->rt->finalized() || !draft->rt->finalized()) return fail(ESP_ERR_INVALID_ARGUMENT, "runtime is not finalized");
    if (out_count) *out_count = 0;
    std::vector<uint32_t> toks;
    GenerationTiming timing;
    TwoTokenStats st;
    int rc = generate_two_token(*target->rt, *draft->rt, prompt, prompt_count, max_tokens, reference_accounting != 0,
                                &toks, &st, &timing);
    if (rc != ESP_OK) return rc;
    for (size_t i = 0; i < toks.size(); i++) if (out_tokens) out_tokens[i] = toks[i];
    if (out_count) *out_count = (int)toks.size();
    fill_stats(stats, timing, toks.size());
    if (two_token_stats) {
        two_token_stats->passes = st.passes;
        two_token_stats->committed_total = st.committed_total;
        two_token_stats->accepted_total = st.accepted_total;
        two_token_stats->reference_passes = st.reference_passes;
        two_token_stats->reference_committed_total = st.reference_committed_total;
        two_token_stats->reference_accepted_total = st.reference_accepted_total;
    }
    return ESP_OK;
}

int esp_llama_generate_batch(ESPLlamaRuntime *target, ESPLlamaRuntime *draft_or_null, const uint32_t *const *prompts,
                             const int *prompt_counts, int n_seq, int max_tokens, uint32_t *out_tokens, int *out_counts,
                             ESPTwoTokenStats *two_token_stats, double *decode_ms) {
    if (!target) return bad_handle();
    if (!target->rt->finalized() || (draft_or_null && !draft_or_null->rt->finalized())) return fail(ESP_ERR_INVALID_ARGUMENT, "runtime is not finalized");
    if (!prompts || !prompt_counts || n_seq < 1 || max_tokens < 0) return fail(ESP_ERR_INVALID_ARGUMENT, "generate_batch: bad argument");
    std::vector<std::vector<uint32_t>> toks;
    TwoTokenStats st;
    int rc = draft_or_null ? generate_two_token_batch(*target->rt, *draft_or_null->rt, prompts, prompt_counts, n_seq, max_tokens, &toks, &st, decode_ms)
                           : generate_greedy_batch(*target->rt, prompts, prompt_counts, n_seq, max_tokens, &toks, decode_ms);
    if (rc != ESP_OK) return rc;
    for (int s = 0; s < n_seq; s++) {
        if (out_counts) out_counts[s] = (int)toks[s].size();
        if (out_tokens) for (size_t i = 0; i < toks[s].size(); i++) out_tokens[(size_t)s * max_tokens + i] = toks[s][i];
    }
    if (two_token_stats) {
        two_token_stats->passes = st.passes;
        two_token_stats->committed_total = st.committed_total;
        two_token_stats->accepted_total = st.accepted_total;
        two_token_stats->reference_passes = 0;
        two_token_stats->reference_committed_total = 0;
        two_token_stats->reference_accepted_total = -1;
    }
    return ESP_OK;
}

int esp_llama_continue_greedy(ESPLlamaRuntime *runtime, int sequence, int steps, uint32_t *out_tokens) {
    if (!runtime) return bad_handle();
    if (!runtime->rt->finalized()) return fail(ESP_ERR_INVALID_ARGUMENT, "runtime is not finalized");
    return runtime->rt->continue_greedy(sequence, steps, out_tokens);
}

int esp_llama_set_graph_replay(ESPLlamaRuntime *runtime, int enabled) {
    if (!runtime) return bad_handle();
    runtime->rt->set_use_graph(enabled != 0);
    return ESP_OK;
}

int esp_llama_set_merged_attention(ESPLlamaRuntime *runtime, int enabled) {
    if (!runtime || !runtime->rt) return fail(ESP_ERR_INVALID_ARGUMENT, "set_merged_attention: null runtime");
    runtime->rt->set_merged_attention(enabled != 0);
    return runtime->rt->merged_attention_in_use() ? 1 : 0;
}

int esp_llama_set_split_activations(ESPLlamaRuntime *runtime, int enabled) {
    if (!runtime || !runtime->rt) return fail(ESP_ERR_INVALID_ARGUMENT, "set_split_activations: null runtime");
    runtime->rt->set_split_activations(enabled != 0);
    return ESP_OK;
}

int esp_llama_set_matrix_prefill(ESPLlamaRuntime *runtime, int enabled) {
    if (!runtime || !runtime->rt) return fail(ESP_ERR_INVALID_ARGUMENT, "set_matrix_prefill: null runtime");
    runtime->rt->set_matrix_prefill(enabled != 0);
    return ESP_OK;
}

int esp_llama_set_kernel_timing(ESPLlamaRuntime *runtime, int enabled) {
    if (!runtime) return bad_handle();
    runtime->rt->set_kernel_timing(enabled != 0);
    return ESP_OK;
}

int esp_llama_kernel_times(ESPLlamaRuntime *runtime, double *total_us, int64_t *launches, uint64_t *bytes_per_launch,
                           int reset) {
    if (!runtime) return bad_handle();
    double t[LlamaRuntime::K_CLASS_COUNT];
    long n[LlamaRuntime::K_CLASS_COUNT];
    int rc = runtime->rt->collect_kernel_times(t, n, reset != 0);
    if (rc != ESP_OK) return rc;
    for (int k = 0; k < LlamaRuntime::K_CLASS_COUNT; k++) {
        if (total_us) total_us[k] = t[k];
        if (launches) launches[k] = n[k];
        if (bytes_per_launch) bytes_per_launch[k] = runtime->rt->kernel_bytes(k);
    }
    return ESP_OK;
}

int esp_llama_time_kernel(ESPLlamaRuntime *runtime, int kernel_class, int iters, double *mean_us) {
    if (!runtime) return bad_handle();
    return runtime->rt->time_kernel_class(kernel_class, iters, mean_us);
}

int esp_llama_time_kernel_dispatch(ESPLlamaRuntime *runtime, int kernel_class, int iters, double *back_to_back_us, double *kernel_us) {
    if (!runtime) return bad_handle();
    return runtime->rt->time_kernel_class(kernel_class, iters, back_to_back_us, kernel_us);
}

int esp_synth_weights(int format, uint64_t seed, float std_dev, size_t elements, void *out_blocks) {
    if (!out_blocks || elements == 0 || elements % 256 != 0)
        return fail(ESP_ERR_INVALID_ARGUMENT, "synth_weights: elements must be a positive multiple of 256");
    if (!(format == FMT_F16 || format == FMT_Q8_0 || format == FMT_Q4_0 || format == FMT_Q4_K))
        return fail(ESP_ERR_UNSUPPORTED, "synth_weights: format %d", format);
    int rc = ensure_init();
    if (rc != ESP_OK) return rc;
    const size_t bytes = format_bytes(format, elements);
    uint8_t *d = nullptr;
    if ((rc = device_alloc(&d, bytes)) != ESP_OK) return rc;
    hipError_t e = launch_synth(format, seed, std_dev, elements, d, context().stream);
    if (e == hipSuccess) e = hipMemcpyAsync(out_blocks, d, bytes, hipMemcpyDeviceToHost, context().stream);
    if (e == hipSuccess) e = hipStreamSynchronize(context().stream);
    (void)hipFree(d);
    return e == hipSuccess ? ESP_OK : fail_hip(e, "synth_weights");
}

}  // extern "C"
