// Host-side mirror of the reference's ModelSupport / ANETypes pieces on the decode path, with the
// reference's names: MultiModelConfig, LayerWeightPaths, BlobWeightLoader, WeightBlob, and the
// weight-directory conventions of RealModelInferenceEngine (top-level file candidates, float32
// sidecars, metadata.json).  File references are paths inside the reference checkout.
#pragma once

#include <cstdint>
#include <string>
#include <vector>

namespace esp {

using TokenID = uint32_t;  // Sources/ANETypes (TokenID = UInt32)

// Sources/ModelSupport/MultiModelConfig.swift:3-55
struct MultiModelConfig {
    enum class Architecture { gpt2, llama };
    std::string name;
    int nLayer = 0, nHead = 0, nKVHead = 0, dModel = 0, headDim = 0, hiddenDim = 0, vocab = 0, maxSeq = 0;
    float normEps = 1e-5f;
    float ropeTheta = 10000.0f;
    bool hasEosToken = false;
    TokenID eosToken = 0;
    Architecture architecture = Architecture::llama;
    int attentionDim() const { return nHead * headDim; }
    int kvDim() const { return nKVHead * headDim; }
};

// ModelRegistry (Sources/ModelSupport/ModelRegistry.swift:1-122): the named configurations the reference ships.
struct ModelRegistry {
    static const std::vector<MultiModelConfig> &all();                 // sorted by name
    static const MultiModelConfig *config(const std::string &name);   // nullptr when unknown
};

// ClassifierStrategy (Sources/RealModelInference/ClassifierStrategy.swift:11-69): which output head the reference
// picks for a model.  Every strategy returns the first maximum of the same logits (Sources/Espresso/
// PartitionedArgmax.swift:9), which is what the GPU head computes; the selection is kept for callers that report it.
enum class ClassifierStrategy { ane = 0, cpuPartitionedFP32 = 1, cpuFP16Tiled = 2 };
ClassifierStrategy selectClassifierStrategy(const MultiModelConfig &config, bool hasExactFloat32LMHead);
const char *exactHeadBackendLabel(ClassifierStrategy s);

// validateRuntimeConfig, RealModelInferenceEngine.swift:7615-7634.  Empty string = valid.
std::string validateRuntimeConfig(const MultiModelConfig &c);

// Sources/ModelSupport/LayerWeightPaths.swift:22-84 (llama branch; empty string = nil)
struct LayerWeightPaths {
    std::string rmsAtt, qNorm, kNorm, wq, wk, wv, wo, rmsFfn, w1, w2, w3;
    static LayerWeightPaths forLayer(int layer, const MultiModelConfig &config, const std::string &blobDir);
};

// Sources/ModelSupport/BlobWeightLoader.swift:3-90
enum class BlobWeightLoaderError { none = 0, truncatedHeader, invalidMagic, invalidDataOffset, truncatedPayload, invalidPayloadSize, ioFailure };
struct BlobWeightLoader {
    struct Header { uint32_t magic = 0, dataSize = 0, dataOffset = 0; };
    static BlobWeightLoaderError parseHeader(const uint8_t *data, size_t bytes, Header *out);
    // fp16 payload -> fp32 (exact)
    static BlobWeightLoaderError load(const std::string &path, std::vector<float> *out);
    // the raw fp16 payload, for direct upload
    static BlobWeightLoaderError loadFP16(const std::string &path, std::vector<uint16_t> *out);
};

// Sources/ANETypes/WeightBlob.swift:6-38 — 128-byte header + little-endian fp16 payload (round to nearest even)
struct WeightBlob {
    static std::vector<uint8_t> build(const float *weights, size_t count);
    static std::vector<uint8_t> buildFP16(const uint16_t *weights, size_t count);
};
uint16_t float_to_half_rne(float v);
float half_to_float(uint16_t h);

// RealModelInferenceEngine.swift:2131-2154
struct LlamaTopLevelWeightPaths { std::string tokenEmbedding, finalNormGamma, lmHead; };
bool resolveLlamaTopLevelWeightPaths(const std::string &weightDir, LlamaTopLevelWeightPaths *out, std::string *error);
// RealModelInferenceEngine.swift:7830-7835: "<stem>.float32.bin"
std::string exactFloat32SidecarPath(const std::string &blobPath);
// "<stem>.<q8_0|q4_0|q4_k>.bin": raw GGUF blocks of the same tensor kept next to the blob so that the
// GPU engine uploads the packed bytes instead of dequantised fp16 (this build's addition)
std::string packedSidecarPath(const std::string &blobPath, int format);

// metadata.json (Sources/EspressoGGUF/GGUFModelLoader.swift:203-222; validated at
// RealModelInferenceEngine.swift:7658-7694)
std::string metadataJSON(const MultiModelConfig &c);
bool loadConfigFromMetadataFile(const std::string &path, MultiModelConfig *out, std::string *error);
// Empty string when metadata.json is absent or agrees with `config`.
std::string validateMetadataIfPresent(const MultiModelConfig &config, const std::string &weightDir);

bool fileExists(const std::string &path);
bool directoryExists(const std::string &path);
bool readFile(const std::string &path, std::vector<uint8_t> *out);
bool writeFile(const std::string &path, const void *data, size_t bytes);
bool makeDirectories(const std::string &path);
std::string joinPath(const std::string &a, const std::string &b);
std::string normalizePath(const std::string &path);   // resolves "." and ".." lexically

}  // namespace esp
