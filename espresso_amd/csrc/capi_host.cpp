// C ABI: weight files, metadata, the GGUF front door, the engine and the exact two-token harness.
#include <algorithm>
#include <chrono>
#include <cstring>

#include "generation.h"
#include "host/engine.h"
#include "host/gguf.h"
#include "host/bundle.h"
#include "host/harness.h"
#include "host/tokenizer.h"

using namespace esp;

struct ESPEngine {
    std::unique_ptr<RealModelInferenceEngine> engine;
    ESPLlamaRuntime runtime_handle{nullptr};
};

namespace {

MultiModelConfig from_c(const ESPModelConfig &c) {
    MultiModelConfig m;
    m.name = std::string(c.name, strnlen(c.name, sizeof(c.name)));
    m.nLayer = c.n_layer; m.nHead = c.n_head; m.nKVHead = c.n_kv_head; m.dModel = c.d_model; m.headDim = c.head_dim;
    m.hiddenDim = c.hidden_dim; m.vocab = c.vocab; m.maxSeq = c.max_seq; m.normEps = c.norm_eps; m.ropeTheta = c.rope_theta;
    m.hasEosToken = c.eos_token >= 0;
    m.eosToken = c.eos_token >= 0 ? (TokenID)c.eos_token : 0;
    m.architecture = c.architecture == 0 ? MultiModelConfig::Architecture::gpt2 : MultiModelConfig::Architecture::llama;
    return m;
}

void to_c(const MultiModelConfig &m, ESPModelConfig *c) {
    std::memset(c, 0, sizeof(*c));
    std::strncpy(c->name, m.name.c_str(), sizeof(c->name) - 1);
    c->n_layer = m.nLayer; c->n_head = m.nHead; c->n_kv_head = m.nKVHead; c->d_model = m.dModel; c->head_dim = m.headDim;
    c->hidden_dim = m.hiddenDim; c->vocab = m.vocab; c->max_seq = m.maxSeq; c->norm_eps = m.normEps; c->rope_theta = m.ropeTheta;
    c->eos_token = m.hasEosToken ? (int32_t)m.eosToken : -1;
    c->architecture = m.architecture == MultiModelConfig::Architecture::gpt2 ? 0 : 1;
}

Environment env_from(const char *const *keys, const char *const *values, int count) {
    Environment e;
    for (int i = 0; i < count; i++) if (keys && values && keys[i] && values[i]) e[keys[i]] = values[i];
    return e;
}

// adapts the C callback table to the C++ protocol
class CallbackModel : public ExactTwoTokenGeneratingLanguageModel {
  public:
    explicit CallbackModel(const ESPExactTwoTokenModel &m) : m_(m) {}
    int vocabSize() const override { return 0; }
    int reset() override { return check(m_.reset(m_.context), "reset"); }
    int prefillSelectedToken(const std::vector<TokenID> &p, TokenID *sel) override {
        return check(m_.prefill_selected_token(m_.context, p.data(), (int)p.size(), sel), "prefillSelectedToken");
    }
    int performExactTwoTokenPass(TokenID cur, int budget, ExactTwoTokenPassResult *r) override {
        ESPPassResult c{};
        int rc = check(m_.perform_exact_two_token_pass(m_.context, cur, budget, &c), "performExactTwoTokenPass");
        if (rc != ESP_OK) return rc;
        const int n = c.committed_count < 0 ? 0 : (c.committed_count > 2 ? 3 : c.committed_count);
        r->committedTokens.clear();
        for (int i = 0; i < n && i < 2; i++) r->committedTokens.push_back(c.committed_tokens[i]);
        if (n == 3) r->committedTokens.push_back(0);   // too many: let the harness reject it
        r->nextCurrentToken = c.next_current_token;
        r->metrics.proposerLatencyMs = c.proposer_latency_ms;
        r->metrics.verifierTrunkLatencyMs = c.verifier_trunk_latency_ms;
        r->metrics.verifierLogitsLatencyMs = c.verifier_logits_latency_ms;
        r->metrics.stateAdvanceLatencyMs = c.state_advance_latency_ms;
        r->metrics.acceptedFutureTokenCount = c.accepted_future_token_count;
        r->metrics.committedExactTokenCount = c.committed_exact_token_count;
        return ESP_OK;
    }

  private:
    static int check(int rc, const char *what) { return rc == 0 ? ESP_OK : fail(ESP_ERR_LAUNCH_FAILED, "model callback %s failed (%d)", what, rc); }
    ESPExactTwoTokenModel m_;
};

}  // namespace

extern "C" {

size_t esp_weight_blob_bytes(size_t element_count) { return 128 + element_count * 2; }

int esp_weight_blob_build(const float *weights, size_t element_count, uint8_t *out) {
    if ((!weights && element_count) || !out) return fail(ESP_ERR_INVALID_ARGUMENT, "weight_blob_build: null pointer");
    const std::vector<uint8_t> b = WeightBlob::build(weights, element_count);
    std::memcpy(out, b.data(), b.size());
    return ESP_OK;
}

long esp_blob_weight_load(const char *path, float *out, size_t capacity) {
    if (!path) return -6;
    std::vector<float> v;
    const BlobWeightLoaderError e = BlobWeightLoader::load(path, &v);
    if (e != BlobWeightLoaderError::none) return -(long)e;
    if (out) std::memcpy(out, v.data(), sizeof(float) * (v.size() < capacity ? v.size() : capacity));
    return (long)v.size();
}

int esp_layer_weight_path(int layer, const char *blob_dir, int slot, char *out, size_t capacity) {
    if (!blob_dir || !out || capacity == 0) return fail(ESP_ERR_INVALID_ARGUMENT, "layer_weight_path: null pointer");
    const LayerWeightPaths p = LayerWeightPaths::forLayer(layer, MultiModelConfig{}, blob_dir);
    const std::string *s = nullptr;
    switch (slot) {
    case SLOT_RMS_ATT: s = &p.rmsAtt; break;
    case SLOT_WQ: s = &p.wq; break;
    case SLOT_WK: s = &p.wk; break;
    case SLOT_WV: s = &p.wv; break;
    case SLOT_WO: s = &p.wo; break;
    case SLOT_RMS_FFN: s = &p.rmsFfn; break;
    case SLOT_W1: s = &p.w1; break;
    case SLOT_W2: s = &p.w2; break;
    case SLOT_W3: s = &p.w3; break;
    case SLOT_Q_NORM: s = &p.qNorm; break;
    case SLOT_K_NORM: s = &p.kNorm; break;
    default: return fail(ESP_ERR_INVALID_ARGUMENT, "layer_weight_path: slot %d is not a layer slot", slot);
    }
    if (s->size() + 1 > capacity) return fail(ESP_ERR_OUT_OF_RANGE, "layer_weight_path: buffer too small");
    std::memcpy(out, s->c_str(), s->size() + 1);
    return (int)s->size();
}

int esp_model_config_load_metadata(const char *path, ESPModelConfig *out) {
    if (!path || !out) return fail(ESP_ERR_INVALID_ARGUMENT, "null pointer");
    MultiModelConfig m;
    std::string err;
    if (!loadConfigFromMetadataFile(path, &m, &err)) return fail(ESP_ERR_IO, "%s", err.c_str());
    to_c(m, out);
    return ESP_OK;
}

int esp_model_config_write_metadata(const ESPModelConfig *config, const char *path) {
    if (!path || !config) return fail(ESP_ERR_INVALID_ARGUMENT, "null pointer");
    const std::string j = metadataJSON(from_c(*config));
    return writeFile(path, j.data(), j.size()) ? ESP_OK : fail(ESP_ERR_IO, "cannot write %s", path);
}

int esp_model_registry_count(void) { return (int)ModelRegistry::all().size(); }
int esp_model_registry_at(int index, ESPModelConfig *out) {
    if (!out || index < 0 || index >= (int)ModelRegistry::all().size()) return fail(ESP_ERR_INVALID_ARGUMENT, "model registry: index %d", index);
    to_c(ModelRegistry::all()[(size_t)index], out);
    return ESP_OK;
}
int esp_model_registry_config(const char *name, ESPModelConfig *out) {
    if (!name || !out) return fail(ESP_ERR_INVALID_ARGUMENT, "model registry: null argument");
    const MultiModelConfig *c = ModelRegistry::config(name);
    if (!c) return fail(ESP_ERR_INVALID_ARGUMENT, "model registry: no configuration named %s", name);
    to_c(*c, out);
    return ESP_OK;
}
int esp_classifier_strategy_select(const ESPModelConfig *config, int has_exact_float32_lm_head, char *out_label, size_t label_bytes) {
    if (!config) return fail(ESP_ERR_INVALID_ARGUMENT, "classifier strategy: null config");
    const ClassifierStrategy s = selectClassifierStrategy(from_c(*config), has_exact_float32_lm_head != 0);
    if (out_label && label_bytes) { std::strncpy(out_label, exactHeadBackendLabel(s), label_bytes - 1); out_label[label_bytes - 1] = 0; }
    return (int)s;
}

int esp_gguf_prepare(const char *gguf_path, const char *output_dir, const ESPPrepareOptions *o, ESPModelConfig *out_config,
                     int *out_tensor_count) {
    if (!gguf_path || !output_dir) return fail(ESP_ERR_INVALID_ARGUMENT, "null path");
    PrepareOptions opt;
    if (o) { opt.emitDequantizedBlobs = o->emit_dequantized_blobs != 0; opt.emitFloat32Sidecars = o->emit_float32_sidecars != 0; opt.qkLayout = o->qk_layout; }
    PreparedModel pm;
    int rc = GGUFModelLoader::prepare(gguf_path, output_dir, opt, &pm);
    if (rc != ESP_OK) return rc;
    if (out_config) to_c(pm.config, out_config);
    if (out_tensor_count) *out_tensor_count = pm.tensorCount;
    return ESP_OK;
}

namespace {
std::map<std::string, std::string> env_map(const char *const *keys, const char *const *values, int n) {
    std::map<std::string, std::string> m;
    for (int i = 0; i < n; i++) if (keys && values && keys[i] && values[i]) m[keys[i]] = values[i];
    return m;
}
PrepareOptions from_c(const ESPPrepareCacheOptions &c, const ESPPrepareOptions *convert) {
    PrepareOptions o;
    if (convert) { o.emitDequantizedBlobs = convert->emit_dequantized_blobs != 0; o.emitFloat32Sidecars = convert->emit_float32_sidecars != 0; o.qkLayout = convert->qk_layout; }
    o.artifactCacheEnabled = c.cache_enabled != 0;
    o.cacheRoot = std::string(c.cache_root, strnlen(c.cache_root, sizeof(c.cache_root)));
    o.exactFloat32SidecarMode = c.sidecar_mode == ESP_SIDECAR_NONE ? ExactFloat32SidecarMode::none
                              : c.sidecar_mode == ESP_SIDECAR_ESSENTIAL ? ExactFloat32SidecarMode::essential
                              : c.sidecar_mode == ESP_SIDECAR_SELECTED ? ExactFloat32SidecarMode::selected
                              : c.sidecar_mode == ESP_SIDECAR_FULL ? ExactFloat32SidecarMode::full : ExactFloat32SidecarMode::automatic;
    const std::string names(c.selected_sidecars, strnlen(c.selected_sidecars, sizeof(c.selected_sidecars)));
    for (size_t at = 0; at <= names.size();) {
        const size_t comma = names.find(',', at);
        const std::string n = names.substr(at, comma == std::string::npos ? std::string::npos : comma - at);
        if (!n.empty()) o.selectedSidecars.insert(n);
        if (comma == std::string::npos) break;
        at = comma + 1;
    }
    return o;
}
int copy_out(const std::string &v, char *out, size_t bytes, const char *what) {
    if (!out || bytes < v.size() + 1) return fail(ESP_ERR_INVALID_ARGUMENT, "%s: buffer of %zu bytes is too small", what, bytes);
    std::memcpy(out, v.c_str(), v.size() + 1);
    return ESP_OK;
}
}  // namespace

int esp_gguf_prepare_options_from_environment(const char *const *env_keys, const char *const *env_values, int env_count,
                                              ESPPrepareCacheOptions *out) {
    if (!out || env_count < 0) return fail(ESP_ERR_INVALID_ARGUMENT, "prepare options: bad argument");
    const PrepareOptions o = PrepareOptions::environment(env_map(env_keys, env_values, env_count));
    std::memset(out, 0, sizeof(*out));
    out->cache_enabled = o.artifactCacheEnabled ? 1 : 0;
    out->sidecar_mode = (int32_t)o.exactFloat32SidecarMode;
    std::string names;
    for (const std::string &n : o.selectedSidecars) names += (names.empty() ? "" : ",") + n;
    if (o.cacheRoot.size() >= sizeof(out->cache_root) || names.size() >= sizeof(out->selected_sidecars))
        return fail(ESP_ERR_INVALID_ARGUMENT, "prepare options: cache root or sidecar list too long");
    std::memcpy(out->cache_root, o.cacheRoot.c_str(), o.cacheRoot.size());
    std::memcpy(out->selected_sidecars, names.c_str(), names.size());
    return ESP_OK;
}

int esp_gguf_artifact_cache_key(const char *gguf_path, const ESPPrepareCacheOptions *options, const char *const *env_keys,
                                const char *const *env_values, int env_count, char *out_key, size_t out_key_bytes) {
    if (!gguf_path || !options) return fail(ESP_ERR_INVALID_ARGUMENT, "cache key: null argument");
    std::string key;
    const int rc = GGUFModelLoader::artifactCacheKey(gguf_path, from_c(*options, nullptr), env_map(env_keys, env_values, env_count), &key);
    return rc != ESP_OK ? rc : copy_out(key, out_key, out_key_bytes, "cache key");
}

int esp_gguf_prepare_cached(const char *gguf_path, const ESPPrepareCacheOptions *options, const ESPPrepareOptions *convert,
                            const char *const *env_keys, const char *const *env_values, int env_count, ESPModelConfig *out_config,
                            int *out_tensor_count, char *out_weight_dir, size_t out_weight_dir_bytes) {
    if (!gguf_path || !options) return fail(ESP_ERR_INVALID_ARGUMENT, "prepare: null argument");
    PreparedModel pm;
    int rc = GGUFModelLoader::prepare(gguf_path, from_c(*options, convert), env_map(env_keys, env_values, env_count), &pm);
    if (rc != ESP_OK) return rc;
    if (out_config) to_c(pm.config, out_config);
    if (out_tensor_count) *out_tensor_count = pm.tensorCount;
    return out_weight_dir ? copy_out(pm.weightDir, out_weight_dir, out_weight_dir_bytes, "weight directory") : ESP_OK;
}

int esp_gguf_cleanup(const char *weight_dir) {
    if (!weight_dir) return fail(ESP_ERR_INVALID_ARGUMENT, "cleanup: null path");
    GGUFModelLoader::cleanup(weight_dir);
    return ESP_OK;
}

int esp_gguf_default_cache_root(char *out, size_t out_bytes) { return copy_out(GGUFModelLoader::defaultPreparedArtifactCacheRoot(), out, out_bytes, "cache root"); }

namespace {
void fill_result(const GenerationResult &r, ESPGenerationResult *result) {
    std::memset(result, 0, sizeof(*result));
    result->token_count = (int32_t)r.tokens.size();
    result->tokens_per_second = r.tokensPerSecond;
    result->compile_time_ms = r.compileTimeMs;
    result->first_token_latency_ms = r.firstTokenLatencyMs;
    result->has_two_token_stats = r.hasTwoTokenStats ? 1 : 0;
    result->committed_exact_tokens_per_pass = r.committedExactTokensPerPass;
    result->accepted_future_tokens_per_pass = r.acceptedFutureTokensPerPass;
    std::strncpy(result->exact_head_backend, r.exactHeadBackend.c_str(), sizeof(result->exact_head_backend) - 1);
}
}  // namespace

ESPEngine *esp_engine_build(const ESPModelConfig *config, const char *weight_dir, const char *tokenizer_dir,
                            const char *const *env_keys, const char *const *env_values, int env_count) {
    if (!config || !weight_dir) { fail(ESP_ERR_INVALID_ARGUMENT, "null config or weight directory"); return nullptr; }
    std::unique_ptr<RealModelInferenceEngine> e;
    if (RealModelInferenceEngine::build(from_c(*config), weight_dir, tokenizer_dir ? tokenizer_dir : "",
                                        env_from(env_keys, env_values, env_count), &e) != ESP_OK)
        return nullptr;
    ESPEngine *h = new ESPEngine();
    h->engine = std::move(e);
    h->runtime_handle.rt = &h->engine->runtime();
    return h;
}

void esp_engine_free(ESPEngine *engine) { delete engine; }

ESPLlamaRuntime *esp_engine_runtime(ESPEngine *engine) { return engine ? &engine->runtime_handle : nullptr; }

int esp_engine_generate(ESPEngine *engine, const uint32_t *prompt_tokens, int prompt_count, int max_tokens, float temperature,
                        const char *const *env_keys, const char *const *env_values, int env_count, uint32_t *out_tokens,
                        ESPGenerationResult *result) {
    if (!engine) return fail(ESP_ERR_INVALID_ARGUMENT, "null engine");
    std::vector<TokenID> prompt;
    if (prompt_tokens && prompt_count > 0) prompt.assign(prompt_tokens, prompt_tokens + prompt_count);
    GenerationResult r;
    int rc = engine->engine->generate(prompt, max_tokens, temperature, env_from(env_keys, env_values, env_count), &r);
    if (rc != ESP_OK) return rc;
    if (out_tokens) for (size_t i = 0; i < r.tokens.size(); i++) out_tokens[i] = r.tokens[i];
    if (result) fill_result(r, result);
    return ESP_OK;
}

int esp_engine_generate_text(ESPEngine *engine, const char *prompt_utf8, size_t prompt_bytes, int max_tokens, float temperature,
                             const char *const *env_keys, const char *const *env_values, int env_count, uint32_t *out_tokens,
                             char *out_text, size_t text_capacity, size_t *out_text_bytes, ESPGenerationResult *result) {
    if (!engine || (!prompt_utf8 && prompt_bytes)) return fail(ESP_ERR_INVALID_ARGUMENT, "null engine or prompt");
    GenerationResult r;
    int rc = engine->engine->generateText(std::string(prompt_utf8 ? prompt_utf8 : "", prompt_bytes), max_tokens, temperature,
                                          env_from(env_keys, env_values, env_count), &r);
    if (rc != ESP_OK) return rc;
    if (out_tokens) for (size_t i = 0; i < r.tokens.size(); i++) out_tokens[i] = r.tokens[i];
    if (out_text_bytes) *out_text_bytes = r.text.size();
    if (out_text && text_capacity) std::memcpy(out_text, r.text.data(), std::min(text_capacity, r.text.size()));
    if (result) fill_result(r, result);
    return ESP_OK;
}

int esp_run_gguf(const char *gguf_path, const char *tokenizer_dir, const char *prompt_utf8, size_t prompt_bytes, int max_tokens,
                 const char *const *env_keys, const char *const *env_values, int env_count, uint32_t *out_tokens, char *out_text,
                 size_t text_capacity, size_t *out_text_bytes, ESPGenerationResult *result, ESPRunGGUFInfo *info) {
    if (!gguf_path || !tokenizer_dir || (!prompt_utf8 && prompt_bytes)) return fail(ESP_ERR_INVALID_ARGUMENT, "run_gguf: null argument");
    const Environment env = env_from(env_keys, env_values, env_count);
    auto now_ms = [] { return std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now().time_since_epoch()).count(); };
    const double t0 = now_ms();
    PreparedModel pm;
    int rc = GGUFModelLoader::prepare(gguf_path, PrepareOptions::environment(env), env, &pm);
    if (rc != ESP_OK) return rc;
    const double t1 = now_ms();
    auto env_it = env.find("ESPRESSO_GGUF_KEEP_WEIGHT_DIR");
    const bool keep = env_it != env.end() && env_it->second == "1";
    auto finish = [&](int code) {
        if (!keep) GGUFModelLoader::cleanup(pm.weightDir);
        if (info) info->kept_weight_dir = directoryExists(pm.weightDir) ? 1 : 0;
        return code;
    };
    if (info) {
        std::memset(info, 0, sizeof(*info));
        to_c(pm.config, &info->config);
        info->tensor_count = pm.tensorCount;
        info->prepare_ms = t1 - t0;
        std::strncpy(info->weight_dir, pm.weightDir.c_str(), sizeof(info->weight_dir) - 1);
    }
    std::unique_ptr<RealModelInferenceEngine> engine;
    if ((rc = RealModelInferenceEngine::build(pm.config, pm.weightDir, tokenizer_dir, env, &engine)) != ESP_OK) return finish(rc);
    if (info) info->build_ms = now_ms() - t1;
    GenerationResult r;
    rc = engine->generateText(std::string(prompt_utf8 ? prompt_utf8 : "", prompt_bytes), max_tokens, 0.0f, env, &r);
    engine.reset();
    if (rc != ESP_OK) return finish(rc);
    if (out_tokens) for (size_t i = 0; i < r.tokens.size(); i++) out_tokens[i] = r.tokens[i];
    if (out_text_bytes) *out_text_bytes = r.text.size();
    if (out_text && text_capacity) std::memcpy(out_text, r.text.data(), std::min(text_capacity, r.text.size()));
    if (result) fill_result(r, result);
    return finish(ESP_OK);
}

// ---- tokenizers ----------------------------------------------------------------------------------------
struct ESPTokenizer { std::unique_ptr<Tokenizer> impl; };

namespace {
thread_local ESPTokenizerError g_tokenizer_error = {};

ESPTokenizer *finish_tokenizer(const TokenizerStatus &st, std::unique_ptr<Tokenizer> t) {
    g_tokenizer_error = ESPTokenizerError{};
    g_tokenizer_error.code = (int32_t)st.error;
    g_tokenizer_error.detail = st.detail;
    g_tokenizer_error.detail2 = st.detail2;
    std::strncpy(g_tokenizer_error.text, st.text.c_str(), sizeof(g_tokenizer_error.text) - 1);
    if (!st.ok()) { fail(ESP_ERR_INVALID_ARGUMENT, "tokenizer load failed: error %d %s", (int)st.error, st.text.c_str()); return nullptr; }
    ESPTokenizer *h = new ESPTokenizer();
    h->impl = std::move(t);
    return h;
}
}  // namespace

ESPTokenizer *esp_tokenizer_load_sentencepiece(const char *model_path) {
    if (!model_path) { fail(ESP_ERR_INVALID_ARGUMENT, "null path"); return nullptr; }
    std::unique_ptr<SentencePieceTokenizer> t;
    const TokenizerStatus st = SentencePieceTokenizer::load(model_path, &t);
    return finish_tokenizer(st, std::move(t));
}

ESPTokenizer *esp_tokenizer_load_gpt2(const char *vocab_json_path, const char *merges_txt_path) {
    if (!vocab_json_path || !merges_txt_path) { fail(ESP_ERR_INVALID_ARGUMENT, "null path"); return nullptr; }
    std::unique_ptr<GPT2BPETokenizer> t;
    const TokenizerStatus st = GPT2BPETokenizer::load(vocab_json_path, merges_txt_path, &t);
    return finish_tokenizer(st, std::move(t));
}

ESPTokenizer *esp_tokenizer_load_tokenizer_json(const char *tokenizer_json_path) {
    if (!tokenizer_json_path) { fail(ESP_ERR_INVALID_ARGUMENT, "null path"); return nullptr; }
    std::unique_ptr<GPT2BPETokenizer> t;
    const TokenizerStatus st = GPT2BPETokenizer::loadTokenizerJSON(tokenizer_json_path, &t);
    return finish_tokenizer(st, std::move(t));
}

ESPTokenizer *esp_tokenizer_load_dir(const ESPModelConfig *config, const char *tokenizer_dir) {
    if (!config || !tokenizer_dir) { fail(ESP_ERR_INVALID_ARGUMENT, "null config or directory"); return nullptr; }
    std::unique_ptr<Tokenizer> t;
    const TokenizerStatus st = loadTokenizer(from_c(*config), tokenizer_dir, &t);
    return finish_tokenizer(st, std::move(t));
}

void esp_tokenizer_last_error(ESPTokenizerError *out) { if (out) *out = g_tokenizer_error; }
void esp_tokenizer_free(ESPTokenizer *tokenizer) { delete tokenizer; }
int esp_tokenizer_vocab_size(const ESPTokenizer *tokenizer) { return tokenizer ? tokenizer->impl->vocabSize() : 0; }
const char *esp_tokenizer_kind(const ESPTokenizer *tokenizer) { return tokenizer ? tokenizer->impl->kind() : ""; }

long esp_tokenizer_encode(const ESPTokenizer *tokenizer, const char *text_utf8, size_t text_bytes, int32_t *out_tokens, size_t capacity) {
    if (!tokenizer || (!text_utf8 && text_bytes)) return fail(ESP_ERR_INVALID_ARGUMENT, "null tokenizer or text");
    const std::vector<int> tokens = tokenizer->impl->encode(std::string(text_utf8 ? text_utf8 : "", text_bytes));
    if (out_tokens) for (size_t i = 0; i < tokens.size() && i < capacity; i++) out_tokens[i] = tokens[i];
    return (long)tokens.size();
}

long esp_pretokenize(const char *pattern_utf8, const char *text_utf8, size_t text_bytes, int64_t *out_ranges, size_t capacity_pairs) {
    if (!text_utf8 && text_bytes) return fail(ESP_ERR_INVALID_ARGUMENT, "null text");
    Regex re;
    std::string err;
    if (!re.compile(pattern_utf8 ? pattern_utf8 : GPT2BPETokenizer::defaultPreTokenizerPattern(), &err))
        return fail(ESP_ERR_INVALID_ARGUMENT, "invalid pre-tokenizer pattern: %s", err.c_str());
    const std::vector<uint32_t> cps = utf8_to_code_points(std::string(text_utf8 ? text_utf8 : "", text_bytes));
    std::vector<size_t> byte_offset(cps.size() + 1, 0);   // of the re-encoded text, equal to the input's when that is valid UTF-8
    for (size_t i = 0; i < cps.size(); i++) {
        std::string one;
        append_utf8(cps[i], &one);
        byte_offset[i + 1] = byte_offset[i] + one.size();
    }
    const auto ms = re.matches(cps);
    for (size_t i = 0; i < ms.size() && i < capacity_pairs && out_ranges; i++) {
        out_ranges[2 * i] = (int64_t)byte_offset[ms[i].first];
        out_ranges[2 * i + 1] = (int64_t)byte_offset[ms[i].second];
    }
    return (long)ms.size();
}

long esp_tokenizer_decode(const ESPTokenizer *tokenizer, const int32_t *tokens, size_t count, char *out_utf8, size_t capacity) {
    if (!tokenizer || (!tokens && count)) return fail(ESP_ERR_INVALID_ARGUMENT, "null tokenizer or tokens");
    const std::string text = tokenizer->impl->decode(std::vector<int>(tokens, tokens + count));
    if (out_utf8 && capacity) std::memcpy(out_utf8, text.data(), std::min(capacity, text.size()));
    return (long)text.size();
}

// ---- bundles ---------------------------------------------------------------------------------------------
struct ESPBundle { ESPRuntimeBundle bundle; };

namespace {
thread_local ESPBundleError g_bundle_error = {};

int bundle_status(const BundleStatus &st) {
    g_bundle_error = ESPBundleError{};
    g_bundle_error.code = (int32_t)st.error;
    g_bundle_error.detail = st.detail;
    g_bundle_error.detail2 = st.detail2;
    std::strncpy(g_bundle_error.text, st.text.c_str(), sizeof(g_bundle_error.text) - 1);
    if (st.ok()) return ESP_OK;
    return fail(ESP_ERR_INVALID_ARGUMENT, "bundle error %d (%ld, %ld) %s", (int)st.error, st.detail, st.detail2, st.text.c_str());
}

void fill_selection(const ESPRuntimeSelection &s, ESPRuntimeSelectionInfo *out) {
    std::memset(out, 0, sizeof(*out));
    std::strncpy(out->backend, s.backend.c_str(), sizeof(out->backend) - 1);
    std::strncpy(out->profile, s.profile.c_str(), sizeof(out->profile) - 1);
    std::strncpy(out->reason, s.reason.c_str(), sizeof(out->reason) - 1);
    out->context_target_tokens = s.contextTargetTokens;
    out->has_output_head = s.hasOutputHead ? 1 : 0;
    out->has_draft = s.hasDraft ? 1 : 0;
}
}  // namespace

void esp_bundle_last_error(ESPBundleError *out) { if (out) *out = g_bundle_error; }

int esp_manifest_parse_toml(const char *text, size_t text_bytes, char *out_toml, size_t capacity, size_t *out_bytes) {
    if (!text && text_bytes) return fail(ESP_ERR_INVALID_ARGUMENT, "null manifest text");
    ESPManifest m;
    int rc = bundle_status(ESPManifest::parseTOML(std::string(text ? text : "", text_bytes), &m));
    if (rc != ESP_OK) return rc;
    const std::string rendered = m.renderTOML();
    if (out_bytes) *out_bytes = rendered.size();
    if (out_toml && capacity) std::memcpy(out_toml, rendered.data(), std::min(capacity, rendered.size()));
    return ESP_OK;
}

int esp_bundle_write_signature_catalog(const char *bundle_dir) {
    if (!bundle_dir) return fail(ESP_ERR_INVALID_ARGUMENT, "null bundle directory");
    ESPBundleArchive a;
    a.bundleDir = bundle_dir;
    return bundle_status(a.writeSignatureCatalog());
}

ESPBundle *esp_bundle_open(const char *bundle_dir, int verify_signatures) {
    if (!bundle_dir) { fail(ESP_ERR_INVALID_ARGUMENT, "null bundle directory"); return nullptr; }
    std::unique_ptr<ESPBundle> b(new ESPBundle());
    if (bundle_status(ESPRuntimeBundle::open(bundle_dir, verify_signatures != 0, &b->bundle)) != ESP_OK) return nullptr;
    return b.release();
}

void esp_bundle_free(ESPBundle *bundle) { delete bundle; }

int esp_bundle_model_config(const ESPBundle *bundle, ESPModelConfig *out) {
    if (!bundle || !out) return fail(ESP_ERR_INVALID_ARGUMENT, "null bundle or config");
    to_c(bundle->bundle.config, out);
    return ESP_OK;
}

int esp_bundle_resolve(const ESPBundle *bundle, long requested_context_tokens, int supports_ane_private, ESPRuntimeSelectionInfo *out) {
    if (!bundle || !out) return fail(ESP_ERR_INVALID_ARGUMENT, "null bundle or selection");
    ESPRuntimeSelection s;
    int rc = bundle_status(selectBackend(supports_ane_private != 0, bundle->bundle.archive.manifest, requested_context_tokens, &s));
    if (rc != ESP_OK) return rc;
    fill_selection(s, out);
    return ESP_OK;
}

long esp_bundle_environment_overrides(const ESPBundle *bundle, long requested_context_tokens, int supports_ane_private, char *out,
                                      size_t capacity) {
    if (!bundle) return fail(ESP_ERR_INVALID_ARGUMENT, "null bundle");
    ESPRuntimeSelection s;
    int rc = bundle_status(selectBackend(supports_ane_private != 0, bundle->bundle.archive.manifest, requested_context_tokens, &s));
    if (rc != ESP_OK) return rc;
    std::string text;
    for (const auto &kv : environmentOverrides(s)) text += kv.first + "=" + kv.second + "\n";
    if (out && capacity) std::memcpy(out, text.data(), std::min(capacity, text.size()));
    return (long)text.size();
}

int esp_bundle_generate(const ESPBundle *bundle, const char *prompt_utf8, size_t prompt_bytes, int max_tokens, float temperature,
                        const char *const *env_keys, const char *const *env_values, int env_count, uint32_t *out_tokens,
                        char *out_text, size_t text_capacity, size_t *out_text_bytes, ESPGenerationResult *result,
                        ESPRuntimeSelectionInfo *selection) {
    if (!bundle || (!prompt_utf8 && prompt_bytes)) return fail(ESP_ERR_INVALID_ARGUMENT, "null bundle or prompt");
    GenerationResult r;
    ESPRuntimeSelection sel;
    BundleStatus st;
    int rc = bundle->bundle.generate(std::string(prompt_utf8 ? prompt_utf8 : "", prompt_bytes), max_tokens, temperature,
                                     env_from(env_keys, env_values, env_count), &r, &sel, &st);
    if (!st.ok()) return bundle_status(st);
    if (rc != ESP_OK) return rc;
    if (selection) fill_selection(sel, selection);
    if (out_tokens) for (size_t i = 0; i < r.tokens.size(); i++) out_tokens[i] = r.tokens[i];
    if (out_text_bytes) *out_text_bytes = r.text.size();
    if (out_text && text_capacity) std::memcpy(out_text, r.text.data(), std::min(text_capacity, r.text.size()));
    if (result) fill_result(r, result);
    return ESP_OK;
}

void esp_exact_two_token_promotion_plan(uint32_t current_token, uint32_t proposed_future_token, uint32_t exact_next_token,
                                        uint32_t exact_future_token, int remaining_token_budget, ESPPromotionPlan *out) {
    if (!out) return;
    const ExactTwoTokenBranchPromotionPlan p =
        ExactTwoTokenBranchPromotionPlan::make(current_token, proposed_future_token, exact_next_token, exact_future_token, remaining_token_budget);
    std::memset(out, 0, sizeof(*out));
    for (size_t i = 0; i < p.committedTokens.size(); i++) out->committed_tokens[i] = p.committedTokens[i];
    out->committed_exact_token_count = p.committedExactTokenCount;
    out->accepted_future_token_count = p.acceptedFutureTokenCount;
    out->promoted_step_count = p.promotedStepCount;
    out->next_current_token = p.nextCurrentToken;
}

int esp_exact_two_token_harness_generate(const ESPExactTwoTokenModel *model, ESPLlamaRuntime *target, ESPLlamaRuntime *draft,
                                         const uint32_t *prompt_tokens, int prompt_count, int max_new_tokens,
                                         uint32_t *out_tokens, int *out_token_count, int32_t *out_committed_per_pass,
                                         int32_t *out_accepted_per_pass, int *out_pass_count) {
    std::vector<TokenID> prompt;
    if (prompt_tokens && prompt_count > 0) prompt.assign(prompt_tokens, prompt_tokens + prompt_count);
    ExactTwoTokenGenerationTrace trace;
    int rc;
    if (model) {
        if (!model->reset || !model->prefill_selected_token || !model->perform_exact_two_token_pass)
            return fail(ESP_ERR_INVALID_ARGUMENT, "model callback table is incomplete");
        CallbackModel m(*model);
        rc = exactTwoTokenHarnessGenerate(m, prompt, max_new_tokens, &trace);
    } else {
        if (!target || !draft) return fail(ESP_ERR_INVALID_ARGUMENT, "no model given");
        if (!target->rt->finalized() || !draft->rt->finalized()) return fail(ESP_ERR_INVALID_ARGUMENT, "runtime is not finalized");
        if (!prompt.empty() && (int)prompt.size() + max_new_tokens + 1 > target->rt->config().max_seq)
            return fail(ESP_ERR_OUT_OF_RANGE, "prompt %zu + %d new tokens exceed context %d", prompt.size(), max_new_tokens, target->rt->config().max_seq);
        HipExactTwoTokenModel m(*target->rt, *draft->rt);
        rc = exactTwoTokenHarnessGenerate(m, prompt, max_new_tokens, &trace);
    }
    if (rc != ESP_OK) return rc;
    if (out_tokens) for (size_t i = 0; i < trace.generatedTokens.size(); i++) out_tokens[i] = trace.generatedTokens[i];
    if (out_token_count) *out_token_count = (int)trace.generatedTokens.size();
    for (size_t i = 0; i < trace.passMetrics.size(); i++) {
        if (out_committed_per_pass) out_committed_per_pass[i] = trace.passMetrics[i].committedExactTokenCount;
        if (out_accepted_per_pass) out_accepted_per_pass[i] = trace.passMetrics[i].acceptedFutureTokenCount;
    }
    if (out_pass_count) *out_pass_count = (int)trace.passMetrics.size();
    return ESP_OK;
}

int esp_sample_token(const float *logits, int count, float temperature, double unit) {
    if (!logits || count <= 0) return fail(ESP_ERR_INVALID_ARGUMENT, "sample_token: bad argument");
    return sample_token(logits, count, temperature, unit);
}

double esp_splitmix64_unit(uint64_t *state) {
    if (!state) return 0.0;
    SplitMix64 g{*state};
    const double u = g.unit();
    *state = g.state;
    return u;
}

}  // extern "C"
