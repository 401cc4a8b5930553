#include "engine.h"

#include <algorithm>
#include <chrono>
#include <cmath>

#include "../generation.h"
#include "json_min.h"

namespace esp {
namespace {

const int kPackedFormats[] = {FMT_Q4_K, FMT_Q8_0, FMT_Q4_0};

LlamaConfig to_runtime_config(const MultiModelConfig &c, const Environment &env) {
    LlamaConfig r;
    r.n_layer = c.nLayer; r.n_head = c.nHead; r.n_kv_head = c.nKVHead; r.d_model = c.dModel; r.head_dim = c.headDim;
    r.hidden_dim = c.hiddenDim; r.vocab = c.vocab; r.max_seq = c.maxSeq; r.norm_eps = c.normEps; r.rope_theta = c.ropeTheta;
    r.eos_token = c.hasEosToken ? (int)c.eosToken : -1;
    auto it = env.find("ESPRESSO_HIP_KV_CACHE");   // "f16" halves KV traffic; default keeps the reference's fp32 caches
    r.kv_format = (it != env.end() && it->second == "f16") ? FMT_F16 : FMT_F32;
    r.max_sequences = 1;
    return r;
}

// One tensor: packed GGUF blocks if a packed sidecar exists, else the exact float32 sidecar
// (loadWeightTablePreferringFloat32Sidecar, :7830-7879), else the fp16 BLOBFILE payload.
int load_tensor(LlamaRuntime &rt, int layer, int slot, const std::string &path, size_t elements, bool matrix, bool optional,
                bool *present) {
    if (present) *present = false;
    std::vector<uint8_t> raw;
    if (matrix) {
        for (int fmt : kPackedFormats) {
            const std::string p = packedSidecarPath(path, fmt);
            if (!fileExists(p)) continue;
            if (!readFile(p, &raw)) return fail(ESP_ERR_IO, "Failed to read %s", p.c_str());
            if (present) *present = true;
            return rt.set_weight(layer, slot, fmt, raw.data(), raw.size());
        }
    }
    const std::string sidecar = exactFloat32SidecarPath(path);
    if (fileExists(sidecar)) {
        if (!readFile(sidecar, &raw)) return fail(ESP_ERR_IO, "Failed to read float32 sidecar %s", sidecar.c_str());
        if (raw.size() != elements * 4)
            return fail(ESP_ERR_INVALID_ARGUMENT, "invalid weight count in %s: expected %zu, got %zu", sidecar.c_str(), elements, raw.size() / 4);
        if (present) *present = true;
        return rt.set_weight(layer, slot, FMT_F32, raw.data(), raw.size());
    }
    if (!fileExists(path)) {
        if (optional) return ESP_OK;
        return fail(ESP_ERR_IO, "missing weight file %s", path.c_str());
    }
    std::vector<uint16_t> half;
    BlobWeightLoaderError e = BlobWeightLoader::loadFP16(path, &half);
    if (e != BlobWeightLoaderError::none) return fail(ESP_ERR_IO, "BlobWeightLoader error %d for %s", (int)e, path.c_str());
    if (half.size() != elements)
        return fail(ESP_ERR_INVALID_ARGUMENT, "invalid weight count in %s: expected %zu, got %zu", path.c_str(), elements, half.size());
    if (present) *present = true;
    return rt.set_weight(layer, slot, FMT_F16, half.data(), half.size() * 2);
}

}  // namespace

int RealModelInferenceEngine::loadRuntime(const MultiModelConfig &config, const std::string &weightDir, const Environment &env,
                                          std::unique_ptr<LlamaRuntime> *out) {
    const std::string bad = validateRuntimeConfig(config);
    if (!bad.empty()) return fail(ESP_ERR_INVALID_ARGUMENT, "%s", bad.c_str());
    if (config.architecture != MultiModelConfig::Architecture::llama)
        return fail(ESP_ERR_UNSUPPORTED, "this engine runs llama-family artifacts only");
    if (!directoryExists(weightDir)) return fail(ESP_ERR_IO, "missing path: %s", weightDir.c_str());
    const std::string meta = validateMetadataIfPresent(config, weightDir);
    if (!meta.empty()) return fail(ESP_ERR_INVALID_ARGUMENT, "%s", meta.c_str());
    LlamaTopLevelWeightPaths top;
    std::string err;
    if (!resolveLlamaTopLevelWeightPaths(weightDir, &top, &err)) return fail(ESP_ERR_IO, "%s", err.c_str());

    LlamaRuntime *raw = nullptr;
    int rc = LlamaRuntime::create(to_runtime_config(config, env), &raw);
    if (rc != ESP_OK) return rc;
    std::unique_ptr<LlamaRuntime> rt(raw);
    const size_t d = config.dModel, ad = config.attentionDim(), kd = config.kvDim(), hd = config.hiddenDim, v = config.vocab;
    if ((rc = load_tensor(*rt, 0, SLOT_TOKEN_EMBEDDING, top.tokenEmbedding, v * d, false, false, nullptr)) != ESP_OK) return rc;
    if ((rc = load_tensor(*rt, 0, SLOT_FINAL_NORM, top.finalNormGamma, d, false, false, nullptr)) != ESP_OK) return rc;
    if ((rc = load_tensor(*rt, 0, SLOT_LM_HEAD, top.lmHead, v * d, true, false, nullptr)) != ESP_OK) return rc;
    for (int l = 0; l < config.nLayer; l++) {
        const LayerWeightPaths p = LayerWeightPaths::forLayer(l, config, weightDir);
        struct Item { int slot; const std::string *path; size_t n; bool matrix; };
        const Item items[] = {{SLOT_RMS_ATT, &p.rmsAtt, d, false}, {SLOT_WQ, &p.wq, ad * d, true}, {SLOT_WK, &p.wk, kd * d, true},
                              {SLOT_WV, &p.wv, kd * d, true}, {SLOT_WO, &p.wo, d * ad, true}, {SLOT_RMS_FFN, &p.rmsFfn, d, false},
                              {SLOT_W1, &p.w1, hd * d, true}, {SLOT_W2, &p.w2, d * hd, true}, {SLOT_W3, &p.w3, hd * d, true}};
        for (const Item &it : items)
            if ((rc = load_tensor(*rt, l, it.slot, *it.path, it.n, it.matrix, false, nullptr)) != ESP_OK) return rc;
        // q_norm / k_norm are used only when both files exist (:6585-6607)
        if (fileExists(p.qNorm) && fileExists(p.kNorm)) {
            if ((rc = load_tensor(*rt, l, SLOT_Q_NORM, p.qNorm, config.headDim, false, false, nullptr)) != ESP_OK) return rc;
            if ((rc = load_tensor(*rt, l, SLOT_K_NORM, p.kNorm, config.headDim, false, false, nullptr)) != ESP_OK) return rc;
        }
    }
    if ((rc = rt->finalize()) != ESP_OK) return rc;
    *out = std::move(rt);
    return ESP_OK;
}

int RealModelInferenceEngine::build(const MultiModelConfig &config, const std::string &weightDir, const std::string &tokenizerDir,
                                    const Environment &environment, std::unique_ptr<RealModelInferenceEngine> *out) {
    auto t0 = std::chrono::steady_clock::now();
    std::unique_ptr<RealModelInferenceEngine> e(new RealModelInferenceEngine());
    e->config_ = config;
    e->weight_dir_ = weightDir;
    if (!tokenizerDir.empty()) {
        if (!directoryExists(tokenizerDir)) return fail(ESP_ERR_IO, "missing path: %s", tokenizerDir.c_str());
        const TokenizerStatus st = loadTokenizer(config, tokenizerDir, &e->tokenizer_);
        if (st.error == TokenizerError::MissingPath) return fail(ESP_ERR_IO, "missing path: %s", st.text.c_str());
        if (!st.ok()) return fail(ESP_ERR_INVALID_ARGUMENT, "Failed to load tokenizer from %s: error %d (%ld, %ld) %s", tokenizerDir.c_str(),
                                  (int)st.error, st.detail, st.detail2, st.text.c_str());
    }
    int rc = loadRuntime(config, weightDir, environment, &e->runtime_);
    if (rc != ESP_OK) return rc;
    e->build_ms_ = std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - t0).count();
    *out = std::move(e);
    return ESP_OK;
}

int RealModelInferenceEngine::resolveExactTwoTokenDraft(const MultiModelConfig &config, const std::string &weightDir,
                                                        const Environment &env, std::string *draftWeightDir,
                                                        MultiModelConfig *draftConfig) {
    draftWeightDir->clear();
    auto get = [&](const char *k) { auto it = env.find(k); return it == env.end() ? std::string() : it->second; };
    if (get("ESPRESSO_BUNDLE_DRAFT_KIND") != "exact_two_token") return ESP_OK;
    const std::string horizon = get("ESPRESSO_BUNDLE_DRAFT_HORIZON");
    if (!horizon.empty() && std::atoi(horizon.c_str()) != 2)
        return fail(ESP_ERR_INVALID_ARGUMENT, "exact two-token draft requires horizon == 2, got %s", horizon.c_str());
    const std::string ref = get("ESPRESSO_BUNDLE_DRAFT_ARTIFACT_REF");
    if (ref.empty()) return fail(ESP_ERR_INVALID_ARGUMENT, "exact two-token draft requires ESPRESSO_BUNDLE_DRAFT_ARTIFACT_REF");
    const std::string weightRoot = normalizePath(weightDir);
    const std::string bundleRoot = normalizePath(joinPath(weightRoot, ".."));
    const std::string descriptorPath = normalizePath(joinPath(bundleRoot, ref));
    if (descriptorPath != bundleRoot && descriptorPath.compare(0, bundleRoot.size() + 1, bundleRoot + "/") != 0)
        return fail(ESP_ERR_INVALID_ARGUMENT, "Draft artifact ref escapes bundle root: %s", ref.c_str());
    if (!fileExists(descriptorPath)) return fail(ESP_ERR_IO, "Draft artifact file is missing: %s", descriptorPath.c_str());
    std::vector<uint8_t> raw;
    JsonObject obj;
    std::string perr;
    if (!readFile(descriptorPath, &raw) || !json_parse_object(std::string(raw.begin(), raw.end()), &obj, &perr))
        return fail(ESP_ERR_INVALID_ARGUMENT, "Failed to decode draft descriptor %s: %s", descriptorPath.c_str(), perr.c_str());
    const std::string modelDir = obj.count("model_dir") ? obj["model_dir"].text : "";
    if (modelDir.empty()) return fail(ESP_ERR_INVALID_ARGUMENT, "Draft descriptor is missing model_dir");
    const std::string draftDir = normalizePath(joinPath(weightRoot, modelDir));
    if (draftDir != weightRoot && draftDir.compare(0, weightRoot.size() + 1, weightRoot + "/") != 0)
        return fail(ESP_ERR_INVALID_ARGUMENT, "Draft model_dir escapes weights root: %s", modelDir.c_str());
    if (!directoryExists(draftDir)) return fail(ESP_ERR_IO, "missing path: %s", draftDir.c_str());
    std::string err;
    if (!loadConfigFromMetadataFile(joinPath(draftDir, "metadata.json"), draftConfig, &err))
        return fail(ESP_ERR_INVALID_ARGUMENT, "%s", err.c_str());
    if (draftConfig->architecture != MultiModelConfig::Architecture::llama)
        return fail(ESP_ERR_UNSUPPORTED, "exact two-token draft currently supports llama draft models only");
    if (draftConfig->vocab != config.vocab)
        return fail(ESP_ERR_INVALID_ARGUMENT, "draft/full vocab mismatch: draft=%d full=%d", draftConfig->vocab, config.vocab);
    *draftWeightDir = draftDir;
    return ESP_OK;
}

int RealModelInferenceEngine::generate(const std::vector<TokenID> &promptTokens, int maxTokens, float temperature,
                                       const Environment &environment, GenerationResult *out) {
    *out = GenerationResult{};
    // argument contract of generate() (:1411-1437)
    if (maxTokens < 0) return fail(ESP_ERR_INVALID_ARGUMENT, "maxTokens must be >= 0");
    if (!std::isfinite(temperature) || temperature < 0) return fail(ESP_ERR_INVALID_ARGUMENT, "temperature must be finite and >= 0");
    if (promptTokens.empty()) return fail(ESP_ERR_INVALID_ARGUMENT, "Prompt tokens must not be empty");
    if ((int)promptTokens.size() >= config_.maxSeq)
        return fail(ESP_ERR_OUT_OF_RANGE, "Prompt of %zu tokens does not fit context %d", promptTokens.size(), config_.maxSeq);
    out->promptTokens = promptTokens;
    out->compileTimeMs = build_ms_;

    std::string draftDir;
    MultiModelConfig draftConfig;
    int rc = resolveExactTwoTokenDraft(config_, weight_dir_, environment, &draftDir, &draftConfig);
    if (rc != ESP_OK) return rc;
    GenerationTiming timing;
    if (temperature > 0) {
        // sampling needs the full logits of every step: plain loop, never the two-token path (:8070-8081)
        uint64_t seed = 0x5EED5EED5EEDull;
        auto it = environment.find("ESPRESSO_HIP_SAMPLING_SEED");
        if (it != environment.end()) seed = std::strtoull(it->second.c_str(), nullptr, 0);
        if ((rc = generate_sampled(*runtime_, promptTokens.data(), (int)promptTokens.size(), maxTokens, temperature, seed, &out->tokens, &timing)) != ESP_OK)
            return rc;
        out->exactHeadBackend = "hip_gemv_logits_host_sampling";
    } else if (!draftDir.empty()) {
        if (!draft_runtime_ || draft_dir_loaded_ != draftDir) {
            if ((rc = loadRuntime(draftConfig, draftDir, environment, &draft_runtime_)) != ESP_OK) return rc;
            draft_dir_loaded_ = draftDir;
        }
        TwoTokenStats st;
        if ((rc = generate_two_token(*runtime_, *draft_runtime_, promptTokens.data(), (int)promptTokens.size(), maxTokens, true,
                                     &out->tokens, &st, &timing)) != ESP_OK)
            return rc;
        out->exactHeadBackend = "hip_exact_two_token_draft";
        if (st.reference_passes > 0) {   // nil when no speculative pass ran (:6170-6175)
            out->hasTwoTokenStats = true;
            out->committedExactTokensPerPass = (double)st.reference_committed_total / st.reference_passes;
            out->acceptedFutureTokensPerPass = (double)st.reference_accepted_total / st.reference_passes;
        }
    } else {
        if ((rc = generate_greedy(*runtime_, promptTokens.data(), (int)promptTokens.size(), maxTokens, &out->tokens, &timing)) != ESP_OK)
            return rc;
        out->exactHeadBackend = "hip_gemv_argmax";
    }
    out->tokenLatenciesMs = timing.token_latencies_ms;
    out->firstTokenLatencyMs = timing.first_token_latency_ms;
    out->tokensPerSecond = out->tokens.empty() ? 0.0 : (double)out->tokens.size() / std::max(timing.decode_ms / 1e3, 1e-9);
    return ESP_OK;
}

int RealModelInferenceEngine::generateText(const std::string &prompt, int maxTokens, float temperature, const Environment &environment,
                                           GenerationResult *out) {
    *out = GenerationResult{};
    if (!tokenizer_) return fail(ESP_ERR_INVALID_ARGUMENT, "the engine was built without a tokenizer directory");
    if (maxTokens < 0) return fail(ESP_ERR_INVALID_ARGUMENT, "maxTokens must be >= 0");
    if (!std::isfinite(temperature) || temperature < 0) return fail(ESP_ERR_INVALID_ARGUMENT, "temperature must be finite and >= 0");
    // encodePrompt (:5404-5418)
    const std::vector<int> raw = tokenizer_->encode(prompt);
    if (raw.empty()) return fail(ESP_ERR_INVALID_ARGUMENT, "Prompt produced no tokens");
    std::vector<TokenID> promptTokens;
    for (int t : raw) {
        if (t < 0) return fail(ESP_ERR_INVALID_ARGUMENT, "Token %d does not fit TokenID", t);
        promptTokens.push_back((TokenID)t);
    }
    if ((int)promptTokens.size() >= config_.maxSeq)
        return fail(ESP_ERR_OUT_OF_RANGE, "Prompt token count %zu exceeds model context %d", promptTokens.size(), config_.maxSeq - 1);
    std::vector<int> all(raw);
    if (std::min(maxTokens, config_.maxSeq - (int)promptTokens.size()) > 0) {
        int rc = generate(promptTokens, maxTokens, temperature, environment, out);
        if (rc != ESP_OK) return rc;
        for (TokenID t : out->tokens) all.push_back((int)t);
    } else {
        out->promptTokens = promptTokens;   // nothing to generate: the prompt decoded back (:1427-1437)
    }
    out->text = tokenizer_->decode(all);
    return ESP_OK;
}

int RealModelInferenceEngine::generateTokensForTesting(const MultiModelConfig &config, const std::string &weightDir,
                                                       const std::vector<TokenID> &promptTokens, int maxTokens,
                                                       std::vector<TokenID> *out) {
    std::unique_ptr<RealModelInferenceEngine> e;
    int rc = build(config, weightDir, "", Environment{}, &e);
    if (rc != ESP_OK) return rc;
    GenerationResult r;
    if ((rc = e->generate(promptTokens, maxTokens, 0.0f, Environment{}, &r)) != ESP_OK) return rc;
    *out = r.tokens;
    return ESP_OK;
}

}  // namespace esp
