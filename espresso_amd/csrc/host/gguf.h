// GGUF container reader and GGUFModelLoader.prepare: the front door that the reference delegates to
// the absent Edgerunner package (GGUFLoader, EspressoModelConfig, WeightConverter; call sites
// Sources/EspressoGGUF/GGUFModelLoader.swift:293-352).  Written from the public GGUF specification
// (versions 2 and 3): header, typed key/value metadata, tensor infos, aligned tensor data.
#pragma once

#include <cstdint>
#include <map>
#include <string>
#include <vector>

#include "model_support.h"

namespace esp {

struct GGUFValue {
    uint32_t type = 0;          // GGUF metadata value type id
    uint64_t u = 0;             // integers and bool
    double f = 0;               // floats
    std::string s;              // strings
    uint32_t array_type = 0;    // arrays: element type and count (elements themselves are skipped)
    uint64_t array_count = 0;
};

struct GGUFTensorInfo {
    std::string name;
    std::vector<uint64_t> dims;  // ne[0] is the innermost (column) dimension
    uint32_t type = 0;           // ggml type id
    uint64_t offset = 0;         // relative to the start of the data section
    uint64_t elements() const { uint64_t n = 1; for (uint64_t d : dims) n *= d; return n; }
};

class GGUFLoader {
  public:
    // Parses header, metadata and tensor infos; returns false with *error set on malformed input.
    bool open(const std::string &path, std::string *error);
    uint32_t version() const { return version_; }
    const std::map<std::string, GGUFValue> &metadata() const { return meta_; }
    const std::vector<GGUFTensorInfo> &tensors() const { return tensors_; }
    const GGUFTensorInfo *find(const std::string &name) const;
    bool getInt(const std::string &key, int64_t *out) const;
    bool getFloat(const std::string &key, double *out) const;
    bool getString(const std::string &key, std::string *out) const;
    // Reads the tensor's bytes (GGUF block layout); false on a short file or an unknown type.
    bool readTensor(const GGUFTensorInfo &t, std::vector<uint8_t> *out, std::string *error) const;
    static size_t tensorBytes(uint32_t type, uint64_t elements);   // 0 = unsupported type

  private:
    std::string path_;
    uint32_t version_ = 0;
    uint64_t data_start_ = 0, file_size_ = 0;
    std::map<std::string, GGUFValue> meta_;
    std::vector<GGUFTensorInfo> tensors_;
};

// GGUFModelLoader.PrepareOptions (Sources/EspressoGGUF/GGUFModelLoader.swift:38-138), reduced to what
// this build acts on.
struct PrepareOptions {
    bool emitDequantizedBlobs = false;   // also write fp16 BLOBFILEs for quantised projections (what the reference's
                                         // own engine reads); the packed sidecars are always written
    bool emitFloat32Sidecars = true;     // exact fp32 sidecars for tensors stored as F32/BF16
    int qkLayout = -1;                   // -1: by architecture; 0: rows as stored; 1: undo the GGUF llama Q/K row interleave
};

struct PreparedModel {     // GGUFModelLoader.PreparedModel (:140-160)
    MultiModelConfig config;
    std::string weightDir;
    int tensorCount = 0;
};

struct GGUFModelLoader {
    // GGUF -> directory of BLOBFILEs / sidecars + metadata.json (GGUFModelLoader.prepare, :273-405).
    static int prepare(const std::string &ggufPath, const std::string &outputDir, const PrepareOptions &options, PreparedModel *out);
    // Metadata -> MultiModelConfig (:297-326)
    static int configFromMetadata(const GGUFLoader &gguf, MultiModelConfig *out);
};

}  // namespace esp
