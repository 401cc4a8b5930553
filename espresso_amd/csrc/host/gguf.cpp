#include "gguf.h"

#include <sys/stat.h>
#include <unistd.h>

#include <algorithm>
#include <cctype>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <filesystem>
#include <random>

#include "../context.h"
#include "bundle.h"
#include "json_min.h"

namespace esp {
namespace {

enum : uint32_t { T_U8 = 0, T_I8, T_U16, T_I16, T_U32, T_I32, T_F32, T_BOOL, T_STRING, T_ARRAY, T_U64, T_I64, T_F64 };
enum : uint32_t { GGML_F32 = 0, GGML_F16 = 1, GGML_Q4_0 = 2, GGML_Q8_0 = 8, GGML_Q4_K = 12, GGML_BF16 = 30 };

struct Reader {
    FILE *f = nullptr;
    bool ok = true;
    ~Reader() { if (f) std::fclose(f); }
    template <typename T>
    T get() {
        T v{};
        if (ok && std::fread(&v, sizeof(T), 1, f) != 1) ok = false;
        return v;
    }
    std::string str() {
        uint64_t n = get<uint64_t>();
        if (!ok || n > (1u << 28)) { ok = false; return ""; }
        std::string s((size_t)n, '\0');
        if (n && std::fread(&s[0], 1, (size_t)n, f) != n) ok = false;
        return s;
    }
    void skip(uint64_t n) { if (ok && std::fseek(f, (long)n, SEEK_CUR) != 0) ok = false; }
};

size_t scalar_size(uint32_t t) {
    switch (t) {
    case T_U8: case T_I8: case T_BOOL: return 1;
    case T_U16: case T_I16: return 2;
    case T_U32: case T_I32: case T_F32: return 4;
    case T_U64: case T_I64: case T_F64: return 8;
    default: return 0;
    }
}

bool read_value(Reader &r, uint32_t type, GGUFValue *v) {
    v->type = type;
    switch (type) {
    case T_U8: v->u = r.get<uint8_t>(); break;
    case T_I8: v->u = (uint64_t)(int64_t)r.get<int8_t>(); break;
    case T_U16: v->u = r.get<uint16_t>(); break;
    case T_I16: v->u = (uint64_t)(int64_t)r.get<int16_t>(); break;
    case T_U32: v->u = r.get<uint32_t>(); break;
    case T_I32: v->u = (uint64_t)(int64_t)r.get<int32_t>(); break;
    case T_F32: v->f = r.get<float>(); break;
    case T_BOOL: v->u = r.get<uint8_t>() != 0; break;
    case T_STRING: v->s = r.str(); break;
    case T_U64: v->u = r.get<uint64_t>(); break;
    case T_I64: v->u = (uint64_t)r.get<int64_t>(); break;
    case T_F64: v->f = r.get<double>(); break;
    case T_ARRAY: {
        v->array_type = r.get<uint32_t>();
        v->array_count = r.get<uint64_t>();
        if (v->array_type == T_STRING) { for (uint64_t i = 0; i < v->array_count && r.ok; i++) r.skip(r.get<uint64_t>()); }
        else if (v->array_type == T_ARRAY) r.ok = false;   // nested arrays do not occur in model files
        else { size_t sz = scalar_size(v->array_type); if (!sz) r.ok = false; else r.skip(sz * v->array_count); }
        break;
    }
    default: r.ok = false;
    }
    return r.ok;
}

}  // namespace

size_t GGUFLoader::tensorBytes(uint32_t type, uint64_t elements) {
    switch (type) {
    case GGML_F32: return elements * 4;
    case GGML_F16: case GGML_BF16: return elements * 2;
    case GGML_Q4_0: return elements % 32 ? 0 : elements / 32 * 18;
    case GGML_Q8_0: return elements % 32 ? 0 : elements / 32 * 34;
    case GGML_Q4_K: return elements % 256 ? 0 : elements / 256 * 144;
    default: return 0;
    }
}

bool GGUFLoader::open(const std::string &path, std::string *error) {
    auto bad = [&](const std::string &m) { if (error) *error = m; return false; };
    Reader r;
    r.f = std::fopen(path.c_str(), "rb");
    if (!r.f) return bad("cannot open " + path);
    std::fseek(r.f, 0, SEEK_END);
    file_size_ = (uint64_t)std::ftell(r.f);
    std::fseek(r.f, 0, SEEK_SET);
    if (r.get<uint32_t>() != 0x46554747u) return bad("not a GGUF file (bad magic)");
    version_ = r.get<uint32_t>();
    if (version_ != 2 && version_ != 3) return bad("unsupported GGUF version " + std::to_string(version_));
    const uint64_t n_tensors = r.get<uint64_t>(), n_kv = r.get<uint64_t>();
    if (!r.ok || n_tensors > (1u << 20) || n_kv > (1u << 20)) return bad("truncated or implausible GGUF header");
    meta_.clear();
    tensors_.clear();
    for (uint64_t i = 0; i < n_kv; i++) {
        std::string key = r.str();
        uint32_t type = r.get<uint32_t>();
        GGUFValue v;
        if (!r.ok || !read_value(r, type, &v)) return bad("malformed metadata entry " + std::to_string(i) + " (" + key + ")");
        meta_[key] = v;
    }
    for (uint64_t i = 0; i < n_tensors; i++) {
        GGUFTensorInfo t;
        t.name = r.str();
        uint32_t nd = r.get<uint32_t>();
        if (!r.ok || nd == 0 || nd > 4) return bad("malformed tensor info " + std::to_string(i));
        for (uint32_t d = 0; d < nd; d++) t.dims.push_back(r.get<uint64_t>());
        t.type = r.get<uint32_t>();
        t.offset = r.get<uint64_t>();
        if (!r.ok) return bad("truncated tensor info " + std::to_string(i));
        tensors_.push_back(t);
    }
    int64_t alignment = 32;
    getInt("general.alignment", &alignment);
    if (alignment <= 0) return bad("bad general.alignment");
    const uint64_t pos = (uint64_t)std::ftell(r.f);
    data_start_ = (pos + alignment - 1) / alignment * alignment;
    path_ = path;
    return true;
}

const GGUFTensorInfo *GGUFLoader::find(const std::string &name) const {
    for (const GGUFTensorInfo &t : tensors_) if (t.name == name) return &t;
    return nullptr;
}
bool GGUFLoader::getInt(const std::string &key, int64_t *out) const {
    auto it = meta_.find(key);
    if (it == meta_.end()) return false;
    const uint32_t t = it->second.type;
    if (t == T_F32 || t == T_F64 || t == T_STRING || t == T_ARRAY) return false;
    *out = (int64_t)it->second.u;
    return true;
}
bool GGUFLoader::getFloat(const std::string &key, double *out) const {
    auto it = meta_.find(key);
    if (it == meta_.end()) return false;
    if (it->second.type == T_F32 || it->second.type == T_F64) { *out = it->second.f; return true; }
    int64_t i;
    if (getInt(key, &i)) { *out = (double)i; return true; }
    return false;
}
bool GGUFLoader::getString(const std::string &key, std::string *out) const {
    auto it = meta_.find(key);
    if (it == meta_.end() || it->second.type != T_STRING) return false;
    *out = it->second.s;
    return true;
}

// Element count of a tensor, or 0 when the dimensions are empty, contain a zero or overflow 2^40 elements (a
// malformed or hostile file): every size derived from it stays far inside 64 bits.
static uint64_t checked_elements(const GGUFTensorInfo &t) {
    constexpr uint64_t kMaxElements = (uint64_t)1 << 40;
    if (t.dims.empty()) return 0;
    uint64_t n = 1;
    for (uint64_t d : t.dims) {
        if (d == 0 || d > kMaxElements || n > kMaxElements / d) return 0;
        n *= d;
    }
    return n;
}

bool GGUFLoader::readTensor(const GGUFTensorInfo &t, std::vector<uint8_t> *out, std::string *error) const {
    const uint64_t elements = checked_elements(t);
    if (!elements) { if (error) *error = "tensor " + t.name + " has an empty or oversized shape"; return false; }
    const size_t bytes = tensorBytes(t.type, elements);
    if (!bytes) { if (error) *error = "tensor " + t.name + " has unsupported ggml type " + std::to_string(t.type); return false; }
    // offset <= file_size - data_start - bytes, written so that nothing can wrap
    if (data_start_ > file_size_ || bytes > file_size_ - data_start_ || t.offset > file_size_ - data_start_ - bytes) {
        if (error) *error = "tensor " + t.name + " runs past the end of the file";
        return false;
    }
    FILE *f = std::fopen(path_.c_str(), "rb");
    if (!f) { if (error) *error = "cannot reopen " + path_; return false; }
    bool ok = false;
    try {
        out->resize(bytes);
        ok = fseeko(f, (off_t)(data_start_ + t.offset), SEEK_SET) == 0 && std::fread(out->data(), 1, bytes, f) == bytes;
        if (!ok && error) *error = "short read of tensor " + t.name;
    } catch (const std::bad_alloc &) {
        if (error) *error = "tensor " + t.name + " does not fit in memory";
    }
    std::fclose(f);
    return ok;
}

int GGUFModelLoader::configFromMetadata(const GGUFLoader &g, MultiModelConfig *out) {
    std::string arch;
    if (!g.getString("general.architecture", &arch)) return fail(ESP_ERR_INVALID_ARGUMENT, "GGUF metadata lacks general.architecture");
    std::string lower = arch;
    for (char &ch : lower) ch = (char)std::tolower((unsigned char)ch);
    MultiModelConfig c;
    if (lower == "gpt2") c.architecture = MultiModelConfig::Architecture::gpt2;
    else if (lower == "llama" || lower == "llama2" || lower == "llama3" || lower == "mistral" || lower == "qwen2" || lower == "qwen3")
        c.architecture = MultiModelConfig::Architecture::llama;
    else return fail(ESP_ERR_UNSUPPORTED, "unsupported architecture %s", arch.c_str());
    c.name = arch;
    auto need = [&](const std::string &key, int *dst) {
        int64_t v;
        if (!g.getInt(arch + "." + key, &v)) return fail(ESP_ERR_INVALID_ARGUMENT, "GGUF metadata lacks %s.%s", arch.c_str(), key.c_str());
        *dst = (int)v;
        return ESP_OK;
    };
    int rc;
    if ((rc = need("block_count", &c.nLayer)) != ESP_OK) return rc;
    if ((rc = need("attention.head_count", &c.nHead)) != ESP_OK) return rc;
    if ((rc = need("embedding_length", &c.dModel)) != ESP_OK) return rc;
    if ((rc = need("feed_forward_length", &c.hiddenDim)) != ESP_OK) return rc;
    if ((rc = need("context_length", &c.maxSeq)) != ESP_OK) return rc;
    int64_t v;
    c.nKVHead = g.getInt(arch + ".attention.head_count_kv", &v) ? (int)v : c.nHead;
    c.headDim = g.getInt(arch + ".attention.key_length", &v) ? (int)v : (c.nHead ? c.dModel / c.nHead : 0);
    double f;
    c.normEps = g.getFloat(arch + ".attention.layer_norm_rms_epsilon", &f) ? (float)f : 1e-5f;
    c.ropeTheta = g.getFloat(arch + ".rope.freq_base", &f) ? (float)f : 10000.0f;                    // (:307-308)
    auto tok = g.metadata().find("tokenizer.ggml.tokens");
    if (tok != g.metadata().end() && tok->second.type == T_ARRAY) c.vocab = (int)tok->second.array_count;   // (:317-319)
    else c.vocab = g.getInt(arch + ".vocab_size", &v) ? (int)v : 0;
    if (g.getInt("tokenizer.ggml.eos_token_id", &v)) { c.hasEosToken = true; c.eosToken = (TokenID)v; }
    *out = c;
    return ESP_OK;
}

namespace {

// fp32 values of a tensor stored as F32 / F16 / BF16 / a supported quantised type (decoded on the GPU)
int tensor_to_float(const GGUFTensorInfo &t, const std::vector<uint8_t> &raw, std::vector<float> *out) {
    const size_t n = (size_t)checked_elements(t);
    if (!n || raw.size() != GGUFLoader::tensorBytes(t.type, n)) return fail(ESP_ERR_INVALID_ARGUMENT, "tensor %s: byte count does not match its shape", t.name.c_str());
    try {
        out->resize(n);
    } catch (const std::bad_alloc &) {
        return fail(ESP_ERR_OUT_OF_MEMORY, "tensor %s does not fit in memory", t.name.c_str());
    }
    switch (t.type) {
    case GGML_F32: std::memcpy(out->data(), raw.data(), n * 4); return ESP_OK;
    case GGML_BF16:
        for (size_t i = 0; i < n; i++) {
            uint32_t bits = ((uint32_t)raw[2 * i] | ((uint32_t)raw[2 * i + 1] << 8)) << 16;
            std::memcpy(&(*out)[i], &bits, 4);
        }
        return ESP_OK;
    case GGML_F16: case GGML_Q4_0: case GGML_Q8_0: case GGML_Q4_K:
        return esp_dequantize((int)t.type, raw.data(), n, out->data());
    default: return fail(ESP_ERR_UNSUPPORTED, "tensor %s has unsupported ggml type %u", t.name.c_str(), t.type);
    }
}

int write_blob_from_floats(const std::string &path, const std::vector<float> &v) {
    const std::vector<uint8_t> blob = WeightBlob::build(v.data(), v.size());
    return writeFile(path, blob.data(), blob.size()) ? ESP_OK : fail(ESP_ERR_IO, "cannot write %s", path.c_str());
}

// GGUF stores llama q/k projection rows interleaved per head for pairwise RoPE: stored row (h, j, s)
// holds the half-split row (h, s, j), s in {0,1}, j < head_dim/2.  This restores the half-split order
// that RoPE.applyDecodeStep assumes (Sources/CPUOps/RoPE.swift:56-110).  Rows are whole numbers of
// quantisation blocks, so the reorder is a copy of row bytes.
void undo_qk_interleave(std::vector<uint8_t> &raw, int heads, int head_dim, size_t row_bytes) {
    std::vector<uint8_t> out(raw.size());
    const int half = head_dim / 2;
    for (int h = 0; h < heads; h++)
        for (int s = 0; s < 2; s++)
            for (int j = 0; j < half; j++)
                std::memcpy(&out[(size_t)(h * head_dim + s * half + j) * row_bytes], &raw[(size_t)(h * head_dim + 2 * j + s) * row_bytes], row_bytes);
    raw.swap(out);
}

}  // namespace

int GGUFModelLoader::prepare(const std::string &ggufPath, const std::string &outputDir, const PrepareOptions &options,
                             PreparedModel *out) {
    GGUFLoader g;
    std::string err;
    if (!g.open(ggufPath, &err)) return fail(ESP_ERR_IO, "%s", err.c_str());
    MultiModelConfig c;
    int rc = configFromMetadata(g, &c);
    if (rc != ESP_OK) return rc;
    if (c.architecture != MultiModelConfig::Architecture::llama) return fail(ESP_ERR_UNSUPPORTED, "only llama-family GGUF files are prepared");
    const std::string bad = validateRuntimeConfig(c);
    if (!bad.empty()) return fail(ESP_ERR_INVALID_ARGUMENT, "%s", bad.c_str());
    std::string arch_lower = c.name;
    for (char &ch : arch_lower) ch = (char)std::tolower((unsigned char)ch);
    const bool undo_interleave = options.qkLayout == 1 || (options.qkLayout < 0 && (arch_lower == "llama" || arch_lower == "llama2" ||
                                                                                    arch_lower == "llama3" || arch_lower == "mistral"));
    if (!makeDirectories(joinPath(outputDir, "embeddings"))) return fail(ESP_ERR_IO, "cannot create %s", outputDir.c_str());

    int count = 0;
    const int64_t d_ = c.dModel, ad_ = (int64_t)c.nHead * c.headDim, kd_ = (int64_t)c.nKVHead * c.headDim, hd_ = c.hiddenDim;
    // name in the GGUF file -> path under the weight directory, matrix?, q/k head count for the re-order
    // `rows` x `cols` is the shape the configuration implies (cols = ne[0], the innermost dimension; vectors: rows = 1)
    auto convert = [&](const std::string &gguf_name, const std::string &rel, bool matrix, int qk_heads, bool optional, int64_t rows,
                       int64_t cols) -> int {
        const GGUFTensorInfo *t = g.find(gguf_name);
        if (!t) return optional ? ESP_OK : fail(ESP_ERR_INVALID_ARGUMENT, "GGUF file lacks tensor %s", gguf_name.c_str());
        const bool shape_ok = matrix ? t->dims.size() == 2 && t->dims[0] == (uint64_t)cols && t->dims[1] == (uint64_t)rows
                                     : !t->dims.empty() && t->dims[0] == (uint64_t)cols && checked_elements(*t) == (uint64_t)cols;
        if (!shape_ok || rows <= 0 || cols <= 0)
            return fail(ESP_ERR_INVALID_ARGUMENT, "tensor %s does not have the shape [%lld, %lld] the model configuration implies", gguf_name.c_str(),
                        (long long)rows, (long long)cols);
        std::vector<uint8_t> raw;
        std::string e;
        if (!g.readTensor(*t, &raw, &e)) return fail(ESP_ERR_UNSUPPORTED, "%s", e.c_str());
        const std::string path = joinPath(outputDir, rel);
        if (matrix && qk_heads > 0 && undo_interleave) {
            // rows == qk_heads * headDim was checked against the file above; whole blocks per row
            if (rows != (int64_t)qk_heads * c.headDim || raw.size() % (size_t)rows != 0)
                return fail(ESP_ERR_INVALID_ARGUMENT, "tensor %s: %lld rows are not %d heads of %d", gguf_name.c_str(), (long long)rows, qk_heads, c.headDim);
            undo_qk_interleave(raw, qk_heads, c.headDim, raw.size() / (size_t)rows);
        }
        const bool quantised = t->type == GGML_Q4_0 || t->type == GGML_Q8_0 || t->type == GGML_Q4_K;
        const bool is_embedding = rel == "embeddings/token.bin";
        if (matrix && quantised && !is_embedding) {
            if (!writeFile(packedSidecarPath(path, (int)t->type), raw.data(), raw.size())) return fail(ESP_ERR_IO, "cannot write %s", path.c_str());
            if (!options.emitDequantizedBlobs) { count++; return ESP_OK; }
        }
        if (t->type == GGML_F16) {
            const std::vector<uint8_t> blob = WeightBlob::buildFP16(reinterpret_cast<const uint16_t *>(raw.data()), raw.size() / 2);
            if (!writeFile(path, blob.data(), blob.size())) return fail(ESP_ERR_IO, "cannot write %s", path.c_str());
        } else {
            std::vector<float> values;
            int r = tensor_to_float(*t, raw, &values);
            if (r != ESP_OK) return r;
            if ((r = write_blob_from_floats(path, values)) != ESP_OK) return r;
            const bool wanted = options.exactFloat32SidecarMode == ExactFloat32SidecarMode::selected
                                    ? options.selectedSidecars.count(gguf_name) != 0
                                    : options.exactFloat32SidecarMode != ExactFloat32SidecarMode::none;
            if (options.emitFloat32Sidecars && wanted && (t->type == GGML_F32 || t->type == GGML_BF16) &&
                !writeFile(exactFloat32SidecarPath(path), values.data(), values.size() * 4))
                return fail(ESP_ERR_IO, "cannot write %s", exactFloat32SidecarPath(path).c_str());
        }
        count++;
        return ESP_OK;
    };

    if ((rc = convert("token_embd.weight", "embeddings/token.bin", true, 0, false, c.vocab, d_)) != ESP_OK) return rc;
    if ((rc = convert("output_norm.weight", "rms_final.bin", false, 0, false, 1, d_)) != ESP_OK) return rc;
    if (g.find("output.weight")) {
        if ((rc = convert("output.weight", "lm_head.bin", true, 0, false, c.vocab, d_)) != ESP_OK) return rc;
    } else {
        // tied head: lm_head is the token embedding (materializeTiedLMHeadIfNeeded, :224-263); quantised
        // embeddings keep their packed bytes as the head's packed sidecar
        const GGUFTensorInfo *t = g.find("token_embd.weight");
        std::vector<uint8_t> raw;
        if (!readFile(joinPath(outputDir, "embeddings/token.bin"), &raw) || !writeFile(joinPath(outputDir, "lm_head.bin"), raw.data(), raw.size()))
            return fail(ESP_ERR_IO, "cannot materialise tied lm_head");
        if (t && (t->type == GGML_Q4_0 || t->type == GGML_Q8_0 || t->type == GGML_Q4_K)) {
            std::string e;
            if (!g.readTensor(*t, &raw, &e)) return fail(ESP_ERR_IO, "%s", e.c_str());
            if (!writeFile(packedSidecarPath(joinPath(outputDir, "lm_head.bin"), (int)t->type), raw.data(), raw.size()))
                return fail(ESP_ERR_IO, "cannot write tied lm_head sidecar");
        }
        const std::string emb_sidecar = exactFloat32SidecarPath(joinPath(outputDir, "embeddings/token.bin"));
        if (fileExists(emb_sidecar) && readFile(emb_sidecar, &raw))
            writeFile(exactFloat32SidecarPath(joinPath(outputDir, "lm_head.bin")), raw.data(), raw.size());
    }
    for (int l = 0; l < c.nLayer; l++) {
        const std::string b = "blk." + std::to_string(l) + ".", d = "layers/" + std::to_string(l) + "/";
        if (!makeDirectories(joinPath(outputDir, "layers/" + std::to_string(l)))) return fail(ESP_ERR_IO, "cannot create layer directory");
        if ((rc = convert(b + "attn_norm.weight", d + "rms_att.bin", false, 0, false, 1, d_)) != ESP_OK) return rc;
        if ((rc = convert(b + "attn_q.weight", d + "wq.bin", true, c.nHead, false, ad_, d_)) != ESP_OK) return rc;
        if ((rc = convert(b + "attn_k.weight", d + "wk.bin", true, c.nKVHead, false, kd_, d_)) != ESP_OK) return rc;
        if ((rc = convert(b + "attn_v.weight", d + "wv.bin", true, 0, false, kd_, d_)) != ESP_OK) return rc;
        if ((rc = convert(b + "attn_output.weight", d + "wo.bin", true, 0, false, d_, ad_)) != ESP_OK) return rc;
        if ((rc = convert(b + "ffn_norm.weight", d + "rms_ffn.bin", false, 0, false, 1, d_)) != ESP_OK) return rc;
        if ((rc = convert(b + "ffn_gate.weight", d + "w1.bin", true, 0, false, hd_, d_)) != ESP_OK) return rc;
        if ((rc = convert(b + "ffn_down.weight", d + "w2.bin", true, 0, false, d_, hd_)) != ESP_OK) return rc;
        if ((rc = convert(b + "ffn_up.weight", d + "w3.bin", true, 0, false, hd_, d_)) != ESP_OK) return rc;
        if ((rc = convert(b + "attn_q_norm.weight", d + "q_norm.bin", false, 0, true, 1, c.headDim)) != ESP_OK) return rc;
        if ((rc = convert(b + "attn_k_norm.weight", d + "k_norm.bin", false, 0, true, 1, c.headDim)) != ESP_OK) return rc;
    }
    if (count == 0) return fail(ESP_ERR_INVALID_ARGUMENT, "no tensors converted");
    const std::string meta = metadataJSON(c);
    if (!writeFile(joinPath(outputDir, "metadata.json"), meta.data(), meta.size())) return fail(ESP_ERR_IO, "cannot write metadata.json");
    out->config = c;
    out->weightDir = outputDir;
    out->tensorCount = count;
    return ESP_OK;
}

// ---- prepared-artifact cache ------------------------------------------------------------------------
namespace {

constexpr int kPreparedArtifactCacheVersion = 2;   // 2: the converter options below are part of the key
const char *const kManifestFileName = "prepare-manifest.json";
const char *const kCacheMarkerFileName = ".espresso-gguf-cache-artifact";
// converterCacheEnvironmentKeys (:29-36)
const char *const kConverterEnvironmentKeys[] = {
    "ESPRESSO_FORCE_LLAMA_MATRIX_TRANSPOSE", "ESPRESSO_SKIP_LLAMA_MATRIX_TRANSPOSE", "ESPRESSO_FORCE_QK_INVERSE_INTERLEAVE",
    "ESPRESSO_DIM_MAJOR_TO_HEAD_MAJOR_V_WEIGHT", "ESPRESSO_INVERSE_INTERLEAVE_V_WEIGHT", "ESPRESSO_FORWARD_INTERLEAVE_V_WEIGHT",
};

std::string trimmed(const std::string &v) {
    size_t a = 0, b = v.size();
    while (a < b && std::isspace((unsigned char)v[a])) a++;
    while (b > a && std::isspace((unsigned char)v[b - 1])) b--;
    return v.substr(a, b - a);
}
std::string lowered(std::string v) {
    for (char &c : v) c = (char)std::tolower((unsigned char)c);
    return v;
}
bool isEnabled(const std::string *raw) {   // :607-615
    if (!raw) return false;
    const std::string v = lowered(trimmed(*raw));
    return v == "1" || v == "true" || v == "yes" || v == "on";
}
const std::string *lookup(const std::map<std::string, std::string> &env, const char *key) {
    auto it = env.find(key);
    return it == env.end() ? nullptr : &it->second;
}
const char *sidecarModeName(ExactFloat32SidecarMode m) {   // sidecarModeCacheDescription (:579-593)
    switch (m) {
    case ExactFloat32SidecarMode::none: return "none";
    case ExactFloat32SidecarMode::essential: return "essential";
    case ExactFloat32SidecarMode::selected: return "selected";
    case ExactFloat32SidecarMode::full: return "full";
    default: return "automatic";
    }
}
std::string jsonString(const std::string &v) {
    std::string out = "\"";
    for (char c : v) {
        if (c == '"' || c == '\\') { out += '\\'; out += c; }
        else if ((unsigned char)c < 0x20) { char b[8]; std::snprintf(b, sizeof(b), "\\u%04x", c); out += b; }
        else out += c;
    }
    return out + "\"";
}
std::string standardizedPath(const std::string &path) {
    std::error_code ec;
    const std::filesystem::path abs = std::filesystem::absolute(path, ec);
    return normalizePath(ec ? path : abs.string());
}
bool fileIdentity(const std::string &path, uint64_t *size, double *mtime) {
    struct stat st;
    if (::stat(path.c_str(), &st) != 0) return false;
    *size = (uint64_t)st.st_size;
    *mtime = (double)st.st_mtim.tv_sec + 1e-9 * (double)st.st_mtim.tv_nsec;
    return true;
}
// converterEnvironmentFingerprint (:595-605): the non-empty values of the converter's switches, by key
std::map<std::string, std::string> converterFingerprint(const std::map<std::string, std::string> &env) {
    std::map<std::string, std::string> out;
    for (const char *k : kConverterEnvironmentKeys) {
        const std::string *v = lookup(env, k);
        if (v && !v->empty()) out[k] = *v;
    }
    return out;
}
// The cache payload with its keys in sorted order (cachePayload, :433-443), shared by the key and the manifest.
std::string cachePayloadJSON(const std::string &path, uint64_t size, double mtime, const PrepareOptions &o,
                             const std::map<std::string, std::string> &env, int tensorCount) {
    std::string j = "{\"converterEnvironment\":{";
    bool first = true;
    for (const auto &kv : converterFingerprint(env)) {
        if (!first) j += ",";
        j += jsonString(kv.first) + ":" + jsonString(kv.second);
        first = false;
    }
    char num[64];
    std::snprintf(num, sizeof(num), "%.9f", mtime);
    // the options of this build's converter that change what is written (they are not in the reference's payload)
    j += std::string("},\"emitDequantizedBlobs\":") + (o.emitDequantizedBlobs ? "true" : "false") + ",\"emitFloat32Sidecars\":" +
         (o.emitFloat32Sidecars ? "true" : "false");
    j += ",\"fileSize\":" + std::to_string(size) + ",\"ggufPath\":" + jsonString(path) + ",\"modificationTime\":" + num + ",\"qkLayout\":" + std::to_string(o.qkLayout) +
         ",\"selectedSidecars\":[";
    first = true;
    if (o.exactFloat32SidecarMode == ExactFloat32SidecarMode::selected)
        for (const std::string &n : o.selectedSidecars) {   // std::set: sorted
            if (!first) j += ",";
            j += jsonString(n);
            first = false;
        }
    j += std::string("],\"sidecarMode\":\"") + sidecarModeName(o.exactFloat32SidecarMode) + "\"";
    if (tensorCount >= 0) j += ",\"tensorCount\":" + std::to_string(tensorCount);
    j += ",\"version\":" + std::to_string(kPreparedArtifactCacheVersion) + "}";
    return j;
}
std::string randomSuffix() {
    std::random_device rd;
    char b[40];
    std::snprintf(b, sizeof(b), "%08x%08x%08x", (unsigned)rd(), (unsigned)rd(), (unsigned)rd());
    return b;
}

}  // namespace

PrepareOptions PrepareOptions::environment(const std::map<std::string, std::string> &env) {
    PrepareOptions o;
    if (isEnabled(lookup(env, "ESPRESSO_GGUF_FORCE_FRESH_PREPARE"))) o.artifactCacheEnabled = false;
    else if (const std::string *raw = lookup(env, "ESPRESSO_GGUF_PREPARE_CACHE")) o.artifactCacheEnabled = isEnabled(raw);
    if (const std::string *root = lookup(env, "ESPRESSO_GGUF_PREPARE_CACHE_ROOT")) {
        std::string r = trimmed(*root);
        if (!r.empty() && r[0] == '~') {   // expandingTildeInPath
            const char *home = std::getenv("HOME");
            if (home && (r.size() == 1 || r[1] == '/')) r = std::string(home) + r.substr(1);
        }
        o.cacheRoot = r;
    }
    if (const std::string *names = lookup(env, "ESPRESSO_GGUF_SELECTED_SIDECARS")) {
        size_t at = 0;
        while (at <= names->size()) {
            const size_t comma = names->find(',', at);
            const std::string n = trimmed(names->substr(at, comma == std::string::npos ? std::string::npos : comma - at));
            if (!n.empty()) o.selectedSidecars.insert(n);
            if (comma == std::string::npos) break;
            at = comma + 1;
        }
    }
    const std::string *policy = lookup(env, "ESPRESSO_GGUF_SIDECAR_POLICY");
    const std::string p = policy ? lowered(trimmed(*policy)) : "";
    if (p == "none" || p == "off") o.exactFloat32SidecarMode = ExactFloat32SidecarMode::none;
    else if (p == "essential") o.exactFloat32SidecarMode = ExactFloat32SidecarMode::essential;
    else if (p == "selected") o.exactFloat32SidecarMode = ExactFloat32SidecarMode::selected;
    else if (p == "full") o.exactFloat32SidecarMode = ExactFloat32SidecarMode::full;
    else o.exactFloat32SidecarMode = ExactFloat32SidecarMode::automatic;   // unset, "automatic", "auto" and anything else
    if (o.exactFloat32SidecarMode != ExactFloat32SidecarMode::selected) o.selectedSidecars.clear();
    return o;
}

std::string GGUFModelLoader::defaultPreparedArtifactCacheRoot() {
    const char *xdg = std::getenv("XDG_CACHE_HOME"), *home = std::getenv("HOME");
    std::string base = xdg && xdg[0] ? xdg : (home && home[0] ? joinPath(home, ".cache") : std::filesystem::temp_directory_path().string());
    return joinPath(joinPath(base, "Espresso"), "gguf-prepared");
}

int GGUFModelLoader::artifactCacheKey(const std::string &ggufPath, const PrepareOptions &options,
                                      const std::map<std::string, std::string> &environment, std::string *out) {
    const std::string path = standardizedPath(ggufPath);
    uint64_t size = 0;
    double mtime = 0;
    if (!fileIdentity(path, &size, &mtime)) return fail(ESP_ERR_IO, "cannot stat %s", path.c_str());
    const std::string payload = cachePayloadJSON(path, size, mtime, options, environment, -1);
    *out = sha256_hex(payload.data(), payload.size());
    return ESP_OK;
}

bool GGUFModelLoader::isManagedCachedArtifactDirectory(const std::string &dir) { return fileExists(joinPath(dir, kCacheMarkerFileName)); }

void GGUFModelLoader::cleanup(const std::string &weightDir) {
    if (isManagedCachedArtifactDirectory(weightDir)) return;
    std::error_code ec;
    std::filesystem::remove_all(weightDir, ec);
}

int GGUFModelLoader::prepare(const std::string &ggufPath, const PrepareOptions &options, const std::map<std::string, std::string> &environment,
                             PreparedModel *out) {
    const std::string path = standardizedPath(ggufPath);
    std::error_code ec;
    std::string outputDir;
    if (options.artifactCacheEnabled) {
        std::string key;
        int rc = artifactCacheKey(path, options, environment, &key);
        if (rc != ESP_OK) return rc;
        outputDir = joinPath(options.cacheRoot.empty() ? defaultPreparedArtifactCacheRoot() : options.cacheRoot, key);
        if (directoryExists(outputDir)) {   // loadCachedPreparedModelIfAvailable (:495-533)
            std::vector<uint8_t> raw;
            std::string err;
            JsonNode manifest;
            MultiModelConfig config;
            if (readFile(joinPath(outputDir, kManifestFileName), &raw) && json_parse(std::string(raw.begin(), raw.end()), &manifest, &err) &&
                manifest.kind == JsonNode::Object && manifest.find("tensorCount") && manifest.find("tensorCount")->kind == JsonNode::Number &&
                loadConfigFromMetadataFile(joinPath(outputDir, "metadata.json"), &config, &err)) {
                out->config = config;
                out->weightDir = outputDir;
                out->tensorCount = (int)manifest.find("tensorCount")->number;
                return ESP_OK;
            }
            std::filesystem::remove_all(outputDir, ec);   // an incomplete or unreadable entry is rebuilt
        }
    } else {
        outputDir = joinPath(std::filesystem::temp_directory_path().string(), "espresso_gguf_" + randomSuffix());
    }
    PreparedModel pm;
    // The one converter switch of the reference's environment that this converter has a counterpart for: it forces the
    // Q/K row re-order whatever the architecture says (the value is part of the cache key through converterEnvironment).
    PrepareOptions effective = options;
    if (effective.qkLayout < 0 && isEnabled(lookup(environment, "ESPRESSO_FORCE_QK_INVERSE_INTERLEAVE"))) effective.qkLayout = 1;
    const int rc = prepare(path, outputDir, effective, &pm);
    if (rc != ESP_OK) {
        std::filesystem::remove_all(outputDir, ec);   // shouldCleanupOnFailure (:399-403)
        return rc;
    }
    if (options.artifactCacheEnabled) {   // writePreparedArtifactManifest (:535-566)
        uint64_t size = 0;
        double mtime = 0;
        fileIdentity(path, &size, &mtime);
        const std::string manifest = cachePayloadJSON(path, size, mtime, options, environment, pm.tensorCount) + "\n";
        if (!writeFile(joinPath(outputDir, kManifestFileName), manifest.data(), manifest.size()) ||
            !writeFile(joinPath(outputDir, kCacheMarkerFileName), "", 0)) {
            std::filesystem::remove_all(outputDir, ec);
            return fail(ESP_ERR_IO, "cannot write the cache manifest in %s", outputDir.c_str());
        }
    }
    *out = pm;
    return ESP_OK;
}

}  // namespace esp
