#include "bundle.h"

#include <dirent.h>
#include <sys/stat.h>

#include <algorithm>
#include <climits>
#include <cstdio>
#include <cstring>

#include "json_min.h"

namespace esp {
namespace {

BundleStatus bad(BundleError e, std::string text = {}, long detail = 0, long detail2 = 0) {
    BundleStatus s;
    s.error = e;
    s.text = std::move(text);
    s.detail = detail;
    s.detail2 = detail2;
    return s;
}

bool is_space(char c) { return c == ' ' || c == '\t' || c == '\n' || c == '\r' || c == '\v' || c == '\f'; }
std::string trim(const std::string &s) {
    size_t a = 0, b = s.size();
    while (a < b && is_space(s[a])) a++;
    while (b > a && is_space(s[b - 1])) b--;
    return s.substr(a, b - a);
}
bool is_one_of(const std::string &v, std::initializer_list<const char *> set) {
    for (const char *s : set)
        if (v == s) return true;
    return false;
}
// Int(_:): optional sign, decimal digits, nothing else
bool parse_int_strict(const std::string &s, long *out) {
    size_t i = 0;
    if (i < s.size() && (s[i] == '+' || s[i] == '-')) i++;
    if (i >= s.size()) return false;
    long v = 0;
    for (size_t k = i; k < s.size(); k++) {
        if (s[k] < '0' || s[k] > '9') return false;
        if (v > (LONG_MAX - 9) / 10) return false;
        v = v * 10 + (s[k] - '0');
    }
    *out = s[0] == '-' ? -v : v;
    return true;
}

using Section = std::map<std::string, std::string>;

BundleStatus unquote(const std::string &value, std::string *out) {
    const std::string t = trim(value);
    if (t.empty() || t.front() != '"' || t.back() != '"') return bad(BundleError::UnsupportedValue, value);
    *out = t.size() >= 2 ? t.substr(1, t.size() - 2) : std::string();
    return {};
}
BundleStatus parse_string(const Section &d, const char *key, std::string *out) {
    const auto it = d.find(key);
    if (it == d.end()) return bad(BundleError::EmptyField, key);
    return unquote(it->second, out);
}
BundleStatus parse_string_default(const Section &d, const char *key, const std::string &fallback, std::string *out) {
    if (d.find(key) == d.end()) { *out = fallback; return {}; }
    return parse_string(d, key, out);
}
BundleStatus parse_int(const Section &d, const char *key, long *out) {
    const auto it = d.find(key);
    if (it == d.end() || !parse_int_strict(it->second, out)) return bad(BundleError::UnsupportedValue, key);
    return {};
}
void parse_optional_int(const Section &d, const char *key, bool *has, long *out) {
    const auto it = d.find(key);
    *has = it != d.end() && parse_int_strict(it->second, out);
}
void parse_optional_string(const Section &d, const char *key, bool *has, std::string *out) {
    const auto it = d.find(key);
    *has = it != d.end() && unquote(it->second, out).ok();
}
BundleStatus parse_enum(const Section &d, const char *key, std::initializer_list<const char *> values, std::string *out) {
    BundleStatus st = parse_string(d, key, out);
    if (!st.ok()) return st;
    if (!is_one_of(*out, values)) return bad(BundleError::UnsupportedValue, *out);
    return {};
}
BundleStatus parse_enum_default(const Section &d, const char *key, std::initializer_list<const char *> values, const char *fallback, std::string *out) {
    if (d.find(key) == d.end()) { *out = fallback; return {}; }
    return parse_enum(d, key, values, out);
}
BundleStatus parse_array(const Section &d, const char *key, std::initializer_list<const char *> values, std::vector<std::string> *out) {
    const auto it = d.find(key);
    if (it == d.end()) return bad(BundleError::EmptyField, key);
    const std::string t = trim(it->second);
    if (t.empty() || t.front() != '[' || t.back() != ']') return bad(BundleError::UnsupportedValue, it->second);
    const std::string body = t.size() >= 2 ? t.substr(1, t.size() - 2) : std::string();
    out->clear();
    if (trim(body).empty()) return {};
    size_t i = 0;
    while (i <= body.size()) {
        size_t j = body.find(',', i);
        if (j == std::string::npos) j = body.size();
        if (j > i) {   // split(separator:) drops empty pieces
            std::string item;
            BundleStatus st = unquote(trim(body.substr(i, j - i)), &item);
            if (!st.ok()) return st;
            if (!is_one_of(item, values)) return bad(BundleError::UnsupportedValue, item);
            out->push_back(item);
        }
        i = j + 1;
    }
    return {};
}

BundleStatus non_empty(const std::string &value, const char *field) {
    return trim(value).empty() ? bad(BundleError::EmptyField, field) : BundleStatus{};
}

std::string quoted(const std::string &v) { return "\"" + v + "\""; }

#define ESP_BUNDLE_TRY(expr) do { BundleStatus st__ = (expr); if (!st__.ok()) return st__; } while (0)

// ---- SHA-256 (FIPS 180-4) ----------------------------------------------------------------------------------
const uint32_t kK[64] = {
    0x428a2f98, 0x71374491, 0xb5c0fbcf, 0xe9b5dba5, 0x3956c25b, 0x59f111f1, 0x923f82a4, 0xab1c5ed5, 0xd807aa98, 0x12835b01, 0x243185be,
    0x550c7dc3, 0x72be5d74, 0x80deb1fe, 0x9bdc06a7, 0xc19bf174, 0xe49b69c1, 0xefbe4786, 0x0fc19dc6, 0x240ca1cc, 0x2de92c6f, 0x4a7484aa,
    0x5cb0a9dc, 0x76f988da, 0x983e5152, 0xa831c66d, 0xb00327c8, 0xbf597fc7, 0xc6e00bf3, 0xd5a79147, 0x06ca6351, 0x14292967, 0x27b70a85,
    0x2e1b2138, 0x4d2c6dfc, 0x53380d13, 0x650a7354, 0x766a0abb, 0x81c2c92e, 0x92722c85, 0xa2bfe8a1, 0xa81a664b, 0xc24b8b70, 0xc76c51a3,
    0xd192e819, 0xd6990624, 0xf40e3585, 0x106aa070, 0x19a4c116, 0x1e376c08, 0x2748774c, 0x34b0bcb5, 0x391c0cb3, 0x4ed8aa4a, 0x5b9cca4f,
    0x682e6ff3, 0x748f82ee, 0x78a5636f, 0x84c87814, 0x8cc70208, 0x90befffa, 0xa4506ceb, 0xbef9a3f7, 0xc67178f2};
inline uint32_t rotr(uint32_t x, int n) { return (x >> n) | (x << (32 - n)); }
void sha256_block(uint32_t h[8], const uint8_t *p) {
    uint32_t w[64];
    for (int i = 0; i < 16; i++) w[i] = (uint32_t)p[4 * i] << 24 | (uint32_t)p[4 * i + 1] << 16 | (uint32_t)p[4 * i + 2] << 8 | p[4 * i + 3];
    for (int i = 16; i < 64; i++) {
        const uint32_t s0 = rotr(w[i - 15], 7) ^ rotr(w[i - 15], 18) ^ (w[i - 15] >> 3), s1 = rotr(w[i - 2], 17) ^ rotr(w[i - 2], 19) ^ (w[i - 2] >> 10);
        w[i] = w[i - 16] + s0 + w[i - 7] + s1;
    }
    uint32_t a = h[0], b = h[1], c = h[2], d = h[3], e = h[4], f = h[5], g = h[6], hh = h[7];
    for (int i = 0; i < 64; i++) {
        const uint32_t t1 = hh + (rotr(e, 6) ^ rotr(e, 11) ^ rotr(e, 25)) + ((e & f) ^ (~e & g)) + kK[i] + w[i];
        const uint32_t t2 = (rotr(a, 2) ^ rotr(a, 13) ^ rotr(a, 22)) + ((a & b) ^ (a & c) ^ (b & c));
        hh = g; g = f; f = e; e = d + t1; d = c; c = b; b = a; a = t1 + t2;
    }
    h[0] += a; h[1] += b; h[2] += c; h[3] += d; h[4] += e; h[5] += f; h[6] += g; h[7] += hh;
}

bool is_regular_file(const std::string &path) {
    struct stat st;
    return stat(path.c_str(), &st) == 0 && S_ISREG(st.st_mode);
}

// every regular file below `dir`, as paths relative to `root` with '/' separators
void enumerate_files(const std::string &root, const std::string &relative, std::vector<std::string> *out) {
    const std::string dir = relative.empty() ? root : joinPath(root, relative);
    DIR *d = opendir(dir.c_str());
    if (!d) return;
    while (dirent *e = readdir(d)) {
        const std::string name = e->d_name;
        if (name == "." || name == "..") continue;
        const std::string rel = relative.empty() ? name : relative + "/" + name;
        const std::string full = joinPath(root, rel);
        if (directoryExists(full)) enumerate_files(root, rel, out);
        else if (is_regular_file(full)) out->push_back(rel);
    }
    closedir(d);
}

BundleStatus file_hash(const std::string &path, std::string *out) {
    std::vector<uint8_t> raw;
    if (!readFile(path, &raw)) return bad(BundleError::UnreadableFile, path);
    *out = sha256_hex(raw.data(), raw.size());
    return {};
}

struct Catalog {
    std::string manifestHash;
    std::map<std::string, std::string> fileHashes;
};

BundleStatus compute_catalog(const ESPBundleArchive &a, Catalog *out) {
    ESP_BUNDLE_TRY(file_hash(joinPath(a.bundleDir, ESPBundleLayout::manifestFileName), &out->manifestHash));
    std::vector<std::string> files;
    enumerate_files(a.bundleDir, "", &files);
    const std::string catalog_rel = std::string("signatures/") + ESPBundleLayout::signatureCatalogFileName;
    for (const std::string &rel : files) {
        const size_t slash = rel.rfind('/');
        const std::string last = slash == std::string::npos ? rel : rel.substr(slash + 1);
        if (last == ESPBundleLayout::manifestFileName || rel == catalog_rel) continue;   // ESPBundle.swift:633-637
        ESP_BUNDLE_TRY(file_hash(joinPath(a.bundleDir, rel), &out->fileHashes[rel]));
    }
    return {};
}

BundleStatus validate_reference(const ESPBundleArchive &a, const std::string &reference) {
    if (reference.empty() || reference[0] == '/') return bad(BundleError::InvalidReferencedPath, reference);
    const std::string root = normalizePath(a.bundleDir), resolved = normalizePath(joinPath(root, reference));
    if (resolved != root && resolved.compare(0, root.size() + 1, root + "/") != 0) return bad(BundleError::InvalidReferencedPath, reference);
    if (!fileExists(resolved) || directoryExists(resolved)) return bad(BundleError::MissingReferencedFile, reference);
    return {};
}

}  // namespace

std::string sha256_hex(const void *data, size_t bytes) {
    uint32_t h[8] = {0x6a09e667, 0xbb67ae85, 0x3c6ef372, 0xa54ff53a, 0x510e527f, 0x9b05688c, 0x1f83d9ab, 0x5be0cd19};
    const uint8_t *p = static_cast<const uint8_t *>(data);
    size_t i = 0;
    for (; i + 64 <= bytes; i += 64) sha256_block(h, p + i);
    uint8_t tail[128] = {};
    const size_t rest = bytes - i;
    std::memcpy(tail, p + i, rest);
    tail[rest] = 0x80;
    const size_t total = rest + 9 <= 64 ? 64 : 128;
    const uint64_t bits = (uint64_t)bytes * 8;
    for (int k = 0; k < 8; k++) tail[total - 1 - k] = (uint8_t)(bits >> (8 * k));
    sha256_block(h, tail);
    if (total == 128) sha256_block(h, tail + 64);
    char hex[65];
    for (int k = 0; k < 8; k++) std::snprintf(hex + 8 * k, 9, "%08x", h[k]);
    return std::string(hex, 64);
}

const std::vector<std::string> &ESPBundleLayout::requiredTopLevelEntries() {
    static const std::vector<std::string> v = {"arch", "tokenizer", "weights", "graphs", "states", "adapters", "compiled", "benchmarks", "licenses", "signatures"};
    return v;
}

// ---- manifest ------------------------------------------------------------------------------------------------

BundleStatus ESPManifest::parseTOML(const std::string &text, ESPManifest *out) {
    Section top, compression, optimization, head, draft_section;
    Section *current = &top;
    size_t i = 0;
    while (i <= text.size()) {
        size_t j = i;
        while (j < text.size() && text[j] != '\n' && text[j] != '\r' && text[j] != '\v' && text[j] != '\f') j++;
        const std::string line = trim(text.substr(i, j - i));
        i = j + 1;
        if (line.empty() || line[0] == '#') continue;
        if (line[0] == '[') {
            if (line == "[compression_policy]") current = &compression;
            else if (line == "[optimization]") current = &optimization;
            else if (line == "[output_head]") current = &head;
            else if (line == "[draft]") current = &draft_section;
            else return bad(BundleError::MalformedSection, line);
            continue;
        }
        const size_t eq = line.find('=');
        if (eq == std::string::npos) return bad(BundleError::MalformedLine, line);
        (*current)[trim(line.substr(0, eq))] = trim(line.substr(eq + 1));
    }

    ESPManifest m;
    ESP_BUNDLE_TRY(parse_string(top, "format_version", &m.formatVersion));
    ESP_BUNDLE_TRY(parse_string(top, "model_id", &m.modelID));
    ESP_BUNDLE_TRY(parse_enum(top, "model_family", {"gpt2", "llama", "qwen"}, &m.modelFamily));
    ESP_BUNDLE_TRY(parse_string(top, "architecture_version", &m.architectureVersion));
    ESP_BUNDLE_TRY(parse_string(top, "tokenizer_contract", &m.tokenizerContract));
    ESP_BUNDLE_TRY(parse_array(top, "supported_backends", {"ane-private", "cpu-safe"}, &m.supportedBackends));
    ESP_BUNDLE_TRY(parse_array(top, "supported_profiles", {"prefill_256", "prefill_2048", "decode_1", "decode_2"}, &m.supportedProfiles));
    ESP_BUNDLE_TRY(parse_int(top, "max_context", &m.maxContext));
    bool has_target = false;
    parse_optional_int(top, "context_target_tokens", &has_target, &m.contextTargetTokens);
    if (!has_target) m.contextTargetTokens = m.maxContext;
    ESP_BUNDLE_TRY(parse_string(compression, "name", &m.compressionName));
    ESP_BUNDLE_TRY(parse_int(compression, "weight_bits", &m.weightBits));
    parse_optional_int(compression, "activation_bits", &m.hasActivationBits, &m.activationBits);
    ESP_BUNDLE_TRY(parse_enum_default(top, "model_tier", {"compat", "optimized", "native_fast"}, "compat", &m.modelTier));
    ESP_BUNDLE_TRY(parse_enum_default(top, "behavior_class", {"exact", "near_exact", "approximate"}, "exact", &m.behaviorClass));
    ESP_BUNDLE_TRY(parse_int(top, "adapter_slots", &m.adapterSlots));
    ESP_BUNDLE_TRY(parse_string_default(optimization, "recipe", "legacy", &m.recipe));
    ESP_BUNDLE_TRY(parse_string_default(optimization, "quality_gate", "legacy-compatible", &m.qualityGate));
    parse_optional_string(optimization, "teacher_model", &m.hasTeacherModel, &m.teacherModel);
    parse_optional_string(optimization, "draft_model", &m.hasDraftModel, &m.draftModel);
    parse_optional_string(optimization, "performance_target", &m.hasPerformanceTarget, &m.performanceTarget);
    if (!head.empty()) {
        m.hasOutputHead = true;
        ESPOutputHeadMetadata &h = m.outputHead;
        ESP_BUNDLE_TRY(parse_enum(head, "kind", {"dense", "factored"}, &h.kind));
        ESP_BUNDLE_TRY(parse_enum(head, "behavior_class", {"exact", "near_exact", "approximate"}, &h.behaviorClass));
        parse_optional_int(head, "bottleneck", &h.hasBottleneck, &h.bottleneck);
        parse_optional_int(head, "groups", &h.hasGroups, &h.groups);
        parse_optional_string(head, "projection_ref", &h.hasProjectionRef, &h.projectionRef);
        parse_optional_string(head, "expansion_ref", &h.hasExpansionRef, &h.expansionRef);
    }
    if (!draft_section.empty()) {
        m.hasDraft = true;
        ESPDraftMetadata &d = m.draft;
        ESP_BUNDLE_TRY(parse_enum(draft_section, "kind", {"exact_two_token", "multi_token"}, &d.kind));
        ESP_BUNDLE_TRY(parse_enum(draft_section, "behavior_class", {"exact", "near_exact", "approximate"}, &d.behaviorClass));
        ESP_BUNDLE_TRY(parse_int(draft_section, "horizon", &d.horizon));
        ESP_BUNDLE_TRY(parse_string(draft_section, "verifier", &d.verifier));
        ESP_BUNDLE_TRY(parse_string(draft_section, "rollback", &d.rollback));
        ESP_BUNDLE_TRY(parse_string(draft_section, "artifact_ref", &d.artifactRef));
        ESP_BUNDLE_TRY(parse_string(draft_section, "acceptance_metric", &d.acceptanceMetric));
    }
    ESP_BUNDLE_TRY(parse_string(top, "accuracy_baseline_ref", &m.accuracyBaselineRef));
    ESP_BUNDLE_TRY(parse_string(top, "performance_baseline_ref", &m.performanceBaselineRef));
    ESP_BUNDLE_TRY(parse_string(top, "signature_ref", &m.signatureRef));
    ESP_BUNDLE_TRY(m.validate());
    *out = std::move(m);
    return {};
}

BundleStatus ESPManifest::validate() const {
    ESP_BUNDLE_TRY(non_empty(formatVersion, "format_version"));
    ESP_BUNDLE_TRY(non_empty(modelID, "model_id"));
    ESP_BUNDLE_TRY(non_empty(architectureVersion, "architecture_version"));
    ESP_BUNDLE_TRY(non_empty(tokenizerContract, "tokenizer_contract"));
    ESP_BUNDLE_TRY(non_empty(accuracyBaselineRef, "accuracy_baseline_ref"));
    ESP_BUNDLE_TRY(non_empty(performanceBaselineRef, "performance_baseline_ref"));
    ESP_BUNDLE_TRY(non_empty(signatureRef, "signature_ref"));
    if (supportedBackends.empty()) return bad(BundleError::MissingBackends);
    if (supportedProfiles.empty()) return bad(BundleError::MissingProfiles);
    if (maxContext <= 0) return bad(BundleError::InvalidMaxContext, {}, maxContext);
    if (contextTargetTokens <= 0 || contextTargetTokens > maxContext) return bad(BundleError::InvalidContextTarget, {}, contextTargetTokens);
    if (adapterSlots < 0) return bad(BundleError::InvalidAdapterSlots, {}, adapterSlots);
    if (weightBits <= 0) return bad(BundleError::InvalidWeightBits, {}, weightBits);
    if (hasActivationBits && activationBits <= 0) return bad(BundleError::InvalidActivationBits, {}, activationBits);
    ESP_BUNDLE_TRY(non_empty(recipe, "optimization.recipe"));
    ESP_BUNDLE_TRY(non_empty(qualityGate, "optimization.quality_gate"));
    if (hasOutputHead) {
        const ESPOutputHeadMetadata &h = outputHead;
        if (modelFamily != "llama") return bad(BundleError::InvalidOutputHead, "output-head metadata is supported for llama bundles only");
        if (h.kind == "dense") {
            if (h.hasBottleneck || h.hasGroups || h.hasProjectionRef || h.hasExpansionRef)
                return bad(BundleError::InvalidOutputHead, "dense output head cannot declare factored weights or dimensions");
        } else {
            if (!h.hasBottleneck || h.bottleneck <= 0) return bad(BundleError::InvalidOutputHead, "factored output head requires bottleneck > 0");
            if (!h.hasGroups || h.groups <= 0) return bad(BundleError::InvalidOutputHead, "factored output head requires groups > 0");
            if (!h.hasProjectionRef) return bad(BundleError::EmptyField, "output_head.projection_ref");
            ESP_BUNDLE_TRY(non_empty(h.projectionRef, "output_head.projection_ref"));
            if (!h.hasExpansionRef) return bad(BundleError::EmptyField, "output_head.expansion_ref");
            ESP_BUNDLE_TRY(non_empty(h.expansionRef, "output_head.expansion_ref"));
        }
    }
    if (hasDraft) {
        if (modelFamily != "llama") return bad(BundleError::InvalidDraft, "draft metadata is supported for llama bundles only");
        if (draft.kind != "exact_two_token") return bad(BundleError::InvalidDraft, "only exact_two_token drafts are currently supported");
        if (draft.horizon <= 1) return bad(BundleError::InvalidDraft, "draft horizon must be > 1");
        if (draft.horizon != 2) return bad(BundleError::InvalidDraft, "exact_two_token draft requires horizon == 2");
        ESP_BUNDLE_TRY(non_empty(draft.verifier, "draft.verifier"));
        ESP_BUNDLE_TRY(non_empty(draft.rollback, "draft.rollback"));
        ESP_BUNDLE_TRY(non_empty(draft.acceptanceMetric, "draft.acceptance_metric"));
        ESP_BUNDLE_TRY(non_empty(draft.artifactRef, "draft.artifact_ref"));
    }
    return {};
}

std::string ESPManifest::renderTOML() const {
    std::vector<std::string> lines;
    const auto array = [](const std::vector<std::string> &v) {
        std::string s = "[";
        for (size_t i = 0; i < v.size(); i++) s += (i ? ", " : "") + quoted(v[i]);
        return s + "]";
    };
    lines.push_back("format_version = " + quoted(formatVersion));
    lines.push_back("model_id = " + quoted(modelID));
    lines.push_back("model_family = " + quoted(modelFamily));
    lines.push_back("architecture_version = " + quoted(architectureVersion));
    lines.push_back("tokenizer_contract = " + quoted(tokenizerContract));
    lines.push_back("supported_backends = " + array(supportedBackends));
    lines.push_back("supported_profiles = " + array(supportedProfiles));
    lines.push_back("max_context = " + std::to_string(maxContext));
    lines.push_back("context_target_tokens = " + std::to_string(contextTargetTokens));
    lines.push_back("model_tier = " + quoted(modelTier));
    lines.push_back("behavior_class = " + quoted(behaviorClass));
    lines.push_back("adapter_slots = " + std::to_string(adapterSlots));
    lines.push_back("accuracy_baseline_ref = " + quoted(accuracyBaselineRef));
    lines.push_back("performance_baseline_ref = " + quoted(performanceBaselineRef));
    lines.push_back("signature_ref = " + quoted(signatureRef));
    lines.push_back("[compression_policy]");
    lines.push_back("name = " + quoted(compressionName));
    lines.push_back("weight_bits = " + std::to_string(weightBits));
    if (hasActivationBits) lines.push_back("activation_bits = " + std::to_string(activationBits));
    lines.push_back("[optimization]");
    lines.push_back("recipe = " + quoted(recipe));
    lines.push_back("quality_gate = " + quoted(qualityGate));
    if (hasTeacherModel) lines.push_back("teacher_model = " + quoted(teacherModel));
    if (hasDraftModel) lines.push_back("draft_model = " + quoted(draftModel));
    if (hasPerformanceTarget) lines.push_back("performance_target = " + quoted(performanceTarget));
    if (hasOutputHead) {
        lines.push_back("[output_head]");
        lines.push_back("kind = " + quoted(outputHead.kind));
        lines.push_back("behavior_class = " + quoted(outputHead.behaviorClass));
        if (outputHead.hasBottleneck) lines.push_back("bottleneck = " + std::to_string(outputHead.bottleneck));
        if (outputHead.hasGroups) lines.push_back("groups = " + std::to_string(outputHead.groups));
        if (outputHead.hasProjectionRef) lines.push_back("projection_ref = " + quoted(outputHead.projectionRef));
        if (outputHead.hasExpansionRef) lines.push_back("expansion_ref = " + quoted(outputHead.expansionRef));
    }
    if (hasDraft) {
        lines.push_back("[draft]");
        lines.push_back("kind = " + quoted(draft.kind));
        lines.push_back("behavior_class = " + quoted(draft.behaviorClass));
        lines.push_back("horizon = " + std::to_string(draft.horizon));
        lines.push_back("verifier = " + quoted(draft.verifier));
        lines.push_back("rollback = " + quoted(draft.rollback));
        lines.push_back("artifact_ref = " + quoted(draft.artifactRef));
        lines.push_back("acceptance_metric = " + quoted(draft.acceptanceMetric));
    }
    std::string out;
    for (const std::string &l : lines) out += l + "\n";
    return out;
}

// ---- archive ---------------------------------------------------------------------------------------------------

BundleStatus ESPBundleArchive::open(const std::string &bundleDir, bool verify, ESPBundleArchive *out) {
    const std::string manifest_path = joinPath(bundleDir, ESPBundleLayout::manifestFileName);
    if (!fileExists(manifest_path)) return bad(BundleError::MissingManifest);
    for (const std::string &entry : ESPBundleLayout::requiredTopLevelEntries())
        if (!directoryExists(joinPath(bundleDir, entry))) return bad(BundleError::MissingTopLevelEntry, entry);
    std::vector<uint8_t> raw;
    if (!readFile(manifest_path, &raw)) return bad(BundleError::UnreadableFile, manifest_path);
    ESPBundleArchive a;
    a.bundleDir = bundleDir;
    ESP_BUNDLE_TRY(ESPManifest::parseTOML(std::string(raw.begin(), raw.end()), &a.manifest));
    if (verify) ESP_BUNDLE_TRY(a.verifySignatures());
    if (a.manifest.hasOutputHead && a.manifest.outputHead.kind == "factored") {
        if (a.manifest.outputHead.hasProjectionRef) ESP_BUNDLE_TRY(validate_reference(a, a.manifest.outputHead.projectionRef));
        if (a.manifest.outputHead.hasExpansionRef) ESP_BUNDLE_TRY(validate_reference(a, a.manifest.outputHead.expansionRef));
    }
    if (a.manifest.hasDraft) ESP_BUNDLE_TRY(validate_reference(a, a.manifest.draft.artifactRef));
    *out = std::move(a);
    return {};
}

BundleStatus ESPBundleArchive::verifySignatures() const {
    std::vector<uint8_t> raw;
    if (!readFile(signatureCatalogPath(), &raw)) return bad(BundleError::UnreadableFile, signatureCatalogPath());
    JsonNode root;
    std::string err;
    if (!json_parse(std::string(raw.begin(), raw.end()), &root, &err) || !root.is(JsonNode::Object)) return bad(BundleError::UnreadableFile, signatureCatalogPath());
    const JsonNode *mh = root.find("manifestHash"), *fh = root.find("fileHashes");
    if (!mh || !mh->is(JsonNode::String) || !fh || !fh->is(JsonNode::Object)) return bad(BundleError::UnreadableFile, signatureCatalogPath());
    Catalog computed;
    ESP_BUNDLE_TRY(compute_catalog(*this, &computed));
    if (mh->text != computed.manifestHash) return bad(BundleError::SignatureMismatch, ESPBundleLayout::manifestFileName);
    std::map<std::string, std::string> listed;
    for (const auto &m : fh->members) listed[m.first] = m.second.is(JsonNode::String) ? m.second.text : std::string();
    for (const auto &e : listed) {   // in path order, as the reference reports the first mismatch
        const auto hit = computed.fileHashes.find(e.first);
        if (hit == computed.fileHashes.end() || hit->second != e.second) return bad(BundleError::SignatureMismatch, e.first);
    }
    return {};
}

BundleStatus ESPBundleArchive::writeSignatureCatalog() const {
    Catalog c;
    ESP_BUNDLE_TRY(compute_catalog(*this, &c));
    std::string json = "{\n  \"algorithm\" : \"sha256\",\n  \"fileHashes\" : {";
    bool first = true;
    for (const auto &e : c.fileHashes) {
        json += std::string(first ? "\n" : ",\n") + "    \"" + json_escape(e.first) + "\" : \"" + e.second + "\"";
        first = false;
    }
    json += std::string(first ? "" : "\n  ") + "},\n  \"manifestHash\" : \"" + c.manifestHash + "\"\n}";
    if (!writeFile(signatureCatalogPath(), json.data(), json.size())) return bad(BundleError::UnreadableFile, signatureCatalogPath());
    return {};
}

// ---- selection and the bridge ----------------------------------------------------------------------------------

BundleStatus selectBackend(bool supportsANEPrivate, const ESPManifest &manifest, long requested, ESPRuntimeSelection *out) {
    ESP_BUNDLE_TRY(manifest.validate());
    if (requested >= 0 && requested > manifest.contextTargetTokens)
        return bad(BundleError::RequestedContextExceedsTarget, {}, requested, manifest.contextTargetTokens);
    const auto has = [](const std::vector<std::string> &v, const char *s) { return std::find(v.begin(), v.end(), s) != v.end(); };
    std::string profile;
    if (manifest.contextTargetTokens > 256) {
        if (has(manifest.supportedProfiles, "prefill_2048")) profile = "prefill_2048";
        else if (has(manifest.supportedProfiles, "prefill_256")) profile = "prefill_256";
    } else if (has(manifest.supportedProfiles, "prefill_256")) profile = "prefill_256";
    if (profile.empty()) {
        if (manifest.supportedProfiles.empty()) return bad(BundleError::NoCompatibleProfile);
        profile = manifest.supportedProfiles.front();
    }
    ESPRuntimeSelection s;
    s.profile = profile;
    s.contextTargetTokens = manifest.contextTargetTokens;
    s.hasOutputHead = manifest.hasOutputHead; s.outputHead = manifest.outputHead;
    s.hasDraft = manifest.hasDraft; s.draft = manifest.draft;
    for (const char *backend : {"ane-private", "cpu-safe"}) {
        if (!has(manifest.supportedBackends, backend)) continue;
        if (std::strcmp(backend, "ane-private") == 0) {
            if (!supportsANEPrivate) continue;
            s.backend = backend;
            s.reason = "Private ANE backend is available on this host";
        } else {
            s.backend = backend;
            s.reason = "Fell back to CPU-safe backend";
        }
        *out = std::move(s);
        return {};
    }
    return bad(BundleError::NoCompatibleBackend);
}

Environment environmentOverrides(const ESPRuntimeSelection &sel) {
    Environment env;
    if (sel.hasOutputHead && sel.outputHead.kind == "factored" && sel.outputHead.behaviorClass != "approximate") {
        env["ESPRESSO_BUNDLE_OUTPUT_HEAD_KIND"] = sel.outputHead.kind;
        if (sel.outputHead.hasBottleneck) env["ESPRESSO_BUNDLE_OUTPUT_HEAD_BOTTLENECK"] = std::to_string(sel.outputHead.bottleneck);
        if (sel.outputHead.hasGroups) env["ESPRESSO_BUNDLE_OUTPUT_HEAD_GROUPS"] = std::to_string(sel.outputHead.groups);
        if (sel.outputHead.hasProjectionRef) env["ESPRESSO_BUNDLE_OUTPUT_HEAD_PROJECTION_REF"] = sel.outputHead.projectionRef;
        if (sel.outputHead.hasExpansionRef) env["ESPRESSO_BUNDLE_OUTPUT_HEAD_EXPANSION_REF"] = sel.outputHead.expansionRef;
    }
    if (sel.hasDraft && sel.draft.behaviorClass != "approximate") {
        env["ESPRESSO_BUNDLE_DRAFT_KIND"] = sel.draft.kind;
        env["ESPRESSO_BUNDLE_DRAFT_HORIZON"] = std::to_string(sel.draft.horizon);
        env["ESPRESSO_BUNDLE_DRAFT_VERIFIER"] = sel.draft.verifier;
        env["ESPRESSO_BUNDLE_DRAFT_ROLLBACK"] = sel.draft.rollback;
        env["ESPRESSO_BUNDLE_DRAFT_ARTIFACT_REF"] = sel.draft.artifactRef;
        env["ESPRESSO_BUNDLE_DRAFT_ACCEPTANCE_METRIC"] = sel.draft.acceptanceMetric;
    }
    return env;
}

BundleStatus ESPRuntimeBundle::open(const std::string &bundleDir, bool verify, ESPRuntimeBundle *out) {
    ESPRuntimeBundle b;
    ESP_BUNDLE_TRY(ESPBundleArchive::open(bundleDir, verify, &b.archive));
    std::string err;
    const std::string metadata = joinPath(b.archive.weightsDir(), "metadata.json");
    if (!loadConfigFromMetadataFile(metadata, &b.config, &err)) return bad(BundleError::UnreadableFile, metadata + ": " + err);
    *out = std::move(b);
    return {};
}

int ESPRuntimeBundle::generate(const std::string &prompt, int maxTokens, float temperature, const Environment &environment,
                               GenerationResult *out, ESPRuntimeSelection *selection, BundleStatus *status) const {
    *status = BundleStatus{};
    // countPromptTokens + totalRequestedContextTokens (ESPBundledRuntime.swift:100-109)
    std::unique_ptr<Tokenizer> tokenizer;
    const TokenizerStatus ts = loadTokenizer(config, archive.tokenizerDir(), &tokenizer);
    if (!ts.ok()) return fail(ESP_ERR_INVALID_ARGUMENT, "No tokenizer found in bundle tokenizer directory (error %d %s)", (int)ts.error, ts.text.c_str());
    const long prompt_tokens = (long)tokenizer->encode(prompt).size();
    const long budget = maxTokens > 0 ? maxTokens : 0;
    const long requested = prompt_tokens > LONG_MAX - budget ? LONG_MAX : prompt_tokens + budget;
    const auto disable = environment.find("ESPRESSO_DISABLE_ANE_PRIVATE");
    const bool supports_private = !(disable != environment.end() && disable->second == "1");
    ESPRuntimeSelection sel;
    *status = selectBackend(supports_private, archive.manifest, requested, &sel);
    if (!status->ok()) return fail(ESP_ERR_INVALID_ARGUMENT, "bundle backend selection failed: error %d", (int)status->error);
    Environment env = environment;
    for (const auto &kv : environmentOverrides(sel)) env[kv.first] = kv.second;
    if (sel.backend == "cpu-safe") env["ESPRESSO_USE_CPU_EXACT_DECODE"] = "1";
    if (selection) *selection = sel;
    std::unique_ptr<RealModelInferenceEngine> engine;
    int rc = RealModelInferenceEngine::build(config, archive.weightsDir(), archive.tokenizerDir(), env, &engine);
    if (rc != ESP_OK) return rc;
    return engine->generateText(prompt, maxTokens, temperature, env, out);
}

}  // namespace esp
