#include "model_support.h"

#include <cctype>

#include <algorithm>

#include <sys/stat.h>

#include <cstdio>
#include <cstring>
#include <sstream>

#include "json_min.h"

namespace esp {

std::string validateRuntimeConfig(const MultiModelConfig &c) {
    if (c.nLayer <= 0 || c.nHead <= 0 || c.nKVHead <= 0 || c.dModel <= 0 || c.headDim <= 0 || c.hiddenDim <= 0 ||
        c.vocab <= 0 || c.maxSeq <= 0)
        return "model config dimensions must all be > 0";
    if (c.nHead % c.nKVHead != 0) return "nHead must be a multiple of nKVHead";
    return "";
}

std::string joinPath(const std::string &a, const std::string &b) {
    if (a.empty()) return b;
    if (a.back() == '/') return a + b;
    return a + "/" + b;
}

std::string normalizePath(const std::string &path) {
    std::vector<std::string> parts;
    std::stringstream ss(path);
    std::string item;
    const bool absolute = !path.empty() && path[0] == '/';
    while (std::getline(ss, item, '/')) {
        if (item.empty() || item == ".") continue;
        if (item == "..") { if (!parts.empty()) parts.pop_back(); continue; }
        parts.push_back(item);
    }
    std::string out = absolute ? "/" : "";
    for (size_t i = 0; i < parts.size(); i++) out += (i ? "/" : "") + parts[i];
    return out;
}

LayerWeightPaths LayerWeightPaths::forLayer(int layer, const MultiModelConfig &, const std::string &blobDir) {
    const std::string dir = joinPath(joinPath(blobDir, "layers"), std::to_string(layer));
    LayerWeightPaths p;
    p.rmsAtt = joinPath(dir, "rms_att.bin");
    p.qNorm = joinPath(dir, "q_norm.bin");
    p.kNorm = joinPath(dir, "k_norm.bin");
    p.wq = joinPath(dir, "wq.bin");
    p.wk = joinPath(dir, "wk.bin");
    p.wv = joinPath(dir, "wv.bin");
    p.wo = joinPath(dir, "wo.bin");
    p.rmsFfn = joinPath(dir, "rms_ffn.bin");
    p.w1 = joinPath(dir, "w1.bin");
    p.w2 = joinPath(dir, "w2.bin");
    p.w3 = joinPath(dir, "w3.bin");
    return p;
}

bool fileExists(const std::string &path) {
    struct stat st;
    return stat(path.c_str(), &st) == 0 && S_ISREG(st.st_mode);
}
bool directoryExists(const std::string &path) {
    struct stat st;
    return stat(path.c_str(), &st) == 0 && S_ISDIR(st.st_mode);
}
bool readFile(const std::string &path, std::vector<uint8_t> *out) {
    FILE *f = std::fopen(path.c_str(), "rb");
    if (!f) return false;
    std::fseek(f, 0, SEEK_END);
    long n = std::ftell(f);
    std::fseek(f, 0, SEEK_SET);
    out->resize(n > 0 ? (size_t)n : 0);
    size_t got = n > 0 ? std::fread(out->data(), 1, (size_t)n, f) : 0;
    std::fclose(f);
    return got == out->size();
}
bool writeFile(const std::string &path, const void *data, size_t bytes) {
    FILE *f = std::fopen(path.c_str(), "wb");
    if (!f) return false;
    size_t put = bytes ? std::fwrite(data, 1, bytes, f) : 0;
    std::fclose(f);
    return put == bytes;
}
bool makeDirectories(const std::string &path) {
    std::string cur;
    std::stringstream ss(path);
    std::string item;
    if (!path.empty() && path[0] == '/') cur = "/";
    while (std::getline(ss, item, '/')) {
        if (item.empty()) continue;
        cur = joinPath(cur, item);
        if (!directoryExists(cur) && mkdir(cur.c_str(), 0755) != 0 && !directoryExists(cur)) return false;
    }
    return true;
}

uint16_t float_to_half_rne(float v) { return __builtin_bit_cast(uint16_t, (_Float16)v); }
float half_to_float(uint16_t h) { return (float)__builtin_bit_cast(_Float16, h); }

BlobWeightLoaderError BlobWeightLoader::parseHeader(const uint8_t *data, size_t bytes, Header *out) {
    if (bytes < 128) return BlobWeightLoaderError::truncatedHeader;
    auto u32 = [&](size_t off) { return (uint32_t)data[off] | ((uint32_t)data[off + 1] << 8) | ((uint32_t)data[off + 2] << 16) | ((uint32_t)data[off + 3] << 24); };
    Header h;
    h.magic = u32(64);
    h.dataSize = u32(72);
    h.dataOffset = u32(80);
    if (h.magic != 0xDEADBEEFu) return BlobWeightLoaderError::invalidMagic;
    if (h.dataOffset != 128) return BlobWeightLoaderError::invalidDataOffset;
    if (out) *out = h;
    return BlobWeightLoaderError::none;
}

BlobWeightLoaderError BlobWeightLoader::loadFP16(const std::string &path, std::vector<uint16_t> *out) {
    std::vector<uint8_t> raw;
    if (!readFile(path, &raw)) return BlobWeightLoaderError::ioFailure;
    Header h;
    BlobWeightLoaderError e = parseHeader(raw.data(), raw.size(), &h);
    if (e != BlobWeightLoaderError::none) return e;
    if (h.dataSize % 2 != 0) return BlobWeightLoaderError::invalidPayloadSize;
    if (raw.size() < (size_t)h.dataOffset + h.dataSize) return BlobWeightLoaderError::truncatedPayload;
    out->resize(h.dataSize / 2);
    std::memcpy(out->data(), raw.data() + h.dataOffset, h.dataSize);
    return BlobWeightLoaderError::none;
}

BlobWeightLoaderError BlobWeightLoader::load(const std::string &path, std::vector<float> *out) {
    std::vector<uint16_t> h;
    BlobWeightLoaderError e = loadFP16(path, &h);
    if (e != BlobWeightLoaderError::none) return e;
    out->resize(h.size());
    for (size_t i = 0; i < h.size(); i++) (*out)[i] = half_to_float(h[i]);
    return BlobWeightLoaderError::none;
}

static void blob_header(std::vector<uint8_t> &d, size_t payload) {
    d[0] = 1; d[4] = 2;
    d[64] = 0xEF; d[65] = 0xBE; d[66] = 0xAD; d[67] = 0xDE;
    d[68] = 1;
    for (int i = 0; i < 4; i++) d[72 + i] = (uint8_t)((uint32_t)payload >> (8 * i));
    d[80] = 128;
}

std::vector<uint8_t> WeightBlob::build(const float *weights, size_t count) {
    std::vector<uint8_t> d(128 + count * 2, 0);
    blob_header(d, count * 2);
    for (size_t i = 0; i < count; i++) {
        uint16_t h = float_to_half_rne(weights[i]);
        d[128 + 2 * i] = (uint8_t)(h & 0xFF);
        d[128 + 2 * i + 1] = (uint8_t)(h >> 8);
    }
    return d;
}

std::vector<uint8_t> WeightBlob::buildFP16(const uint16_t *weights, size_t count) {
    std::vector<uint8_t> d(128 + count * 2, 0);
    blob_header(d, count * 2);
    std::memcpy(d.data() + 128, weights, count * 2);
    return d;
}

bool resolveLlamaTopLevelWeightPaths(const std::string &weightDir, LlamaTopLevelWeightPaths *out, std::string *error) {
    if (!directoryExists(weightDir)) { if (error) *error = "missing path: " + weightDir; return false; }
    auto required = [&](std::initializer_list<const char *> candidates, const char *label, std::string *dst) {
        for (const char *c : candidates) {
            std::string p = joinPath(weightDir, c);
            // a tensor kept only as a sidecar (exact float32 or packed GGUF blocks) counts as present
            if (fileExists(p) || fileExists(exactFloat32SidecarPath(p)) || fileExists(packedSidecarPath(p, 12)) ||
                fileExists(packedSidecarPath(p, 8)) || fileExists(packedSidecarPath(p, 2))) { *dst = p; return true; }
        }
        if (error) *error = std::string("missing ") + label + " under " + weightDir;
        return false;
    };
    return required({"embeddings/token.bin", "embeddings/token_embeddings.bin"}, "token embedding", &out->tokenEmbedding) &&
           required({"rms_final.bin", "final_norm_gamma.bin", "final_norm.bin"}, "final norm gamma", &out->finalNormGamma) &&
           required({"lm_head.bin", "classifier.bin"}, "lm head", &out->lmHead);
}

std::string exactFloat32SidecarPath(const std::string &p) {
    if (p.size() >= 4 && p.compare(p.size() - 4, 4, ".bin") == 0) return p.substr(0, p.size() - 4) + ".float32.bin";
    return p + ".float32";
}

std::string packedSidecarPath(const std::string &p, int format) {
    const char *tag = format == 8 ? "q8_0" : format == 2 ? "q4_0" : format == 12 ? "q4_k" : "raw";
    const std::string stem = (p.size() >= 4 && p.compare(p.size() - 4, 4, ".bin") == 0) ? p.substr(0, p.size() - 4) : p;
    return stem + "." + tag + ".bin";
}

std::string metadataJSON(const MultiModelConfig &c) {
    std::ostringstream o;
    o.precision(9);
    o << "{\n  \"name\": \"" << json_escape(c.name) << "\",\n  \"nLayer\": " << c.nLayer << ",\n  \"nHead\": " << c.nHead
      << ",\n  \"nKVHead\": " << c.nKVHead << ",\n  \"dModel\": " << c.dModel << ",\n  \"headDim\": " << c.headDim
      << ",\n  \"hiddenDim\": " << c.hiddenDim << ",\n  \"vocab\": " << c.vocab << ",\n  \"maxSeq\": " << c.maxSeq
      << ",\n  \"normEps\": " << c.normEps << ",\n  \"ropeTheta\": " << c.ropeTheta << ",\n  \"architecture\": \""
      << (c.architecture == MultiModelConfig::Architecture::gpt2 ? "gpt2" : "llama") << "\"";
    if (c.hasEosToken) o << ",\n  \"eosToken\": " << c.eosToken;
    o << "\n}\n";
    return o.str();
}

bool loadConfigFromMetadataFile(const std::string &path, MultiModelConfig *out, std::string *error) {
    std::vector<uint8_t> raw;
    if (!readFile(path, &raw)) { if (error) *error = "Failed to read " + path; return false; }
    JsonObject obj;
    std::string perr;
    if (!json_parse_object(std::string(raw.begin(), raw.end()), &obj, &perr)) {
        if (error) *error = "metadata.json is not valid JSON: " + perr;
        return false;
    }
    MultiModelConfig c;
    auto need_int = [&](const char *key, int *dst) {
        auto it = obj.find(key);
        if (it == obj.end() || it->second.kind != JsonValue::Number) { if (error) *error = std::string("metadata.json is missing ") + key; return false; }
        *dst = (int)it->second.number;
        return true;
    };
    if (!need_int("nLayer", &c.nLayer) || !need_int("nHead", &c.nHead) || !need_int("nKVHead", &c.nKVHead) ||
        !need_int("dModel", &c.dModel) || !need_int("headDim", &c.headDim) || !need_int("hiddenDim", &c.hiddenDim) ||
        !need_int("vocab", &c.vocab) || !need_int("maxSeq", &c.maxSeq))
        return false;
    if (obj.count("name") && obj["name"].kind == JsonValue::String) c.name = obj["name"].text;
    if (obj.count("normEps") && obj["normEps"].kind == JsonValue::Number) c.normEps = (float)obj["normEps"].number;
    if (obj.count("ropeTheta") && obj["ropeTheta"].kind == JsonValue::Number) c.ropeTheta = (float)obj["ropeTheta"].number;
    if (obj.count("eosToken") && obj["eosToken"].kind == JsonValue::Number) { c.hasEosToken = true; c.eosToken = (TokenID)obj["eosToken"].number; }
    c.architecture = (obj.count("architecture") && obj["architecture"].text == "gpt2") ? MultiModelConfig::Architecture::gpt2
                                                                                       : MultiModelConfig::Architecture::llama;
    *out = c;
    return true;
}

std::string validateMetadataIfPresent(const MultiModelConfig &config, const std::string &weightDir) {
    const std::string path = joinPath(weightDir, "metadata.json");
    if (!fileExists(path)) return "";
    MultiModelConfig m;
    std::string err;
    if (!loadConfigFromMetadataFile(path, &m, &err)) return err;
    auto mismatch = [](const char *key, int want, int got) {
        return std::string("metadata.json ") + key + "=" + std::to_string(got) + " does not match config " + std::to_string(want);
    };
    if (m.architecture != config.architecture) return "metadata.json architecture does not match config";
    if (m.nLayer != config.nLayer) return mismatch("nLayer", config.nLayer, m.nLayer);
    if (m.nHead != config.nHead) return mismatch("nHead", config.nHead, m.nHead);
    if (m.nKVHead != config.nKVHead) return mismatch("nKVHead", config.nKVHead, m.nKVHead);
    if (m.dModel != config.dModel) return mismatch("dModel", config.dModel, m.dModel);
    if (m.headDim != config.headDim) return mismatch("headDim", config.headDim, m.headDim);
    if (m.hiddenDim != config.hiddenDim) return mismatch("hiddenDim", config.hiddenDim, m.hiddenDim);
    if (m.vocab != config.vocab) return mismatch("vocab", config.vocab, m.vocab);
    if (m.maxSeq != config.maxSeq) return mismatch("maxSeq", config.maxSeq, m.maxSeq);
    return "";
}

// ---- ModelRegistry ----------------------------------------------------------------------------------
namespace {
MultiModelConfig entry(const char *name, int nLayer, int nHead, int nKVHead, int dModel, int headDim, int hiddenDim, int vocab, int maxSeq,
                       MultiModelConfig::Architecture arch, float ropeTheta = 10000.0f, long eos = -1) {
    MultiModelConfig c;
    c.name = name; c.nLayer = nLayer; c.nHead = nHead; c.nKVHead = nKVHead; c.dModel = dModel; c.headDim = headDim;
    c.hiddenDim = hiddenDim; c.vocab = vocab; c.maxSeq = maxSeq; c.normEps = 1e-5f; c.ropeTheta = ropeTheta; c.architecture = arch;
    if (eos >= 0) { c.hasEosToken = true; c.eosToken = (TokenID)eos; }
    return c;
}
}  // namespace

const std::vector<MultiModelConfig> &ModelRegistry::all() {
    using A = MultiModelConfig::Architecture;
    static const std::vector<MultiModelConfig> table = [] {
        std::vector<MultiModelConfig> t = {
            entry("gpt2_124m", 12, 12, 12, 768, 64, 3072, 50257, 1024, A::gpt2),
            entry("stories110m", 12, 12, 12, 768, 64, 2048, 32000, 256, A::llama),
            entry("smolLM_135m", 30, 9, 3, 576, 64, 1536, 49152, 2048, A::llama),
            entry("tinyLlama_1_1b", 22, 32, 4, 2048, 64, 5632, 32000, 2048, A::llama),
            entry("llama3_2_1b", 16, 32, 8, 2048, 64, 8192, 128256, 2048, A::llama, 500000.0f, 128001),
            entry("llama3_2_1b_ctx512", 16, 32, 8, 2048, 64, 8192, 128256, 512, A::llama, 500000.0f, 128001),
            entry("llama3_2_3b", 28, 24, 8, 3072, 128, 8192, 128256, 2048, A::llama, 500000.0f, 128001),
        };
        std::sort(t.begin(), t.end(), [](const MultiModelConfig &a, const MultiModelConfig &b) { return a.name < b.name; });
        return t;
    }();
    return table;
}

const MultiModelConfig *ModelRegistry::config(const std::string &name) {
    for (const MultiModelConfig &c : all()) if (c.name == name) return &c;
    return nullptr;
}

// ---- ClassifierStrategy -----------------------------------------------------------------------------
ClassifierStrategy selectClassifierStrategy(const MultiModelConfig &config, bool hasExactFloat32LMHead) {
    constexpr long kANESRAMElementLimit = 16000000;   // 32 MB of fp16
    size_t a = 0, b = config.name.size();
    while (a < b && std::isspace((unsigned char)config.name[a])) a++;
    while (b > a && std::isspace((unsigned char)config.name[b - 1])) b--;
    std::string name = config.name.substr(a, b - a);
    for (char &ch : name) ch = (char)std::tolower((unsigned char)ch);
    const bool llama = config.architecture == MultiModelConfig::Architecture::llama;
    if (llama && name.find("stories110m") != std::string::npos) return ClassifierStrategy::ane;   // the reference's allowlist entry
    if ((long)config.vocab * (long)config.dModel <= kANESRAMElementLimit) return ClassifierStrategy::ane;
    if (llama && !hasExactFloat32LMHead) return ClassifierStrategy::cpuFP16Tiled;
    return ClassifierStrategy::cpuPartitionedFP32;
}

const char *exactHeadBackendLabel(ClassifierStrategy s) {
    switch (s) {
    case ClassifierStrategy::ane: return "ane_classifier";
    case ClassifierStrategy::cpuPartitionedFP32: return "cpu_partitioned_fp32";
    default: return "cpu_fp16_tiled";
    }
}

}  // namespace esp
