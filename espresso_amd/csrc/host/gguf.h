// GGUF container reader and GGUFModelLoader.prepare: the front door that the reference delegates to
// the absent Edgerunner package (GGUFLoader, EspressoModelConfig, WeightConverter; call sites
// Sources/EspressoGGUF/GGUFModelLoader.swift:293-352).  Written from the public GGUF specification
// (versions 2 and 3): header, typed key/value metadata, tensor infos, aligned tensor data.
#pragma once

#include <cstdint>
#include <map>
#include <set>
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

// GGUFModelLoader.PrepareOptions (Sources/EspressoGGUF/GGUFModelLoader.swift:38-138).
enum class ExactFloat32SidecarMode { automatic, none, essential, selected, full };

struct PrepareOptions {
    bool emitDequantizedBlobs = false;   // also write fp16 BLOBFILEs for quantised projections (what the reference's
                                         // own engine reads); the packed sidecars are always written
    bool emitFloat32Sidecars = true;     // exact fp32 sidecars for tensors stored as F32/BF16 (subject to the mode below)
    int qkLayout = -1;                   // -1: by architecture; 0: rows as stored; 1: undo the GGUF llama Q/K row interleave
    // Prepared-artifact cache (:38-63): used by the prepare() that chooses the directory itself.
    bool artifactCacheEnabled = true;
    std::string cacheRoot;               // empty: defaultPreparedArtifactCacheRoot()
    // Which tensors get an exact float32 sidecar.  Quantised tensors stay packed in this build, so the mode only
    // matters for tensors stored as F32/BF16: none writes no sidecar, selected only those named (GGUF names), every
    // other mode all of them.
    ExactFloat32SidecarMode exactFloat32SidecarMode = ExactFloat32SidecarMode::automatic;
    std::set<std::string> selectedSidecars;

    // PrepareOptions.environment(_:) (:65-127): ESPRESSO_GGUF_FORCE_FRESH_PREPARE, ESPRESSO_GGUF_PREPARE_CACHE,
    // ESPRESSO_GGUF_PREPARE_CACHE_ROOT, ESPRESSO_GGUF_SIDECAR_POLICY, ESPRESSO_GGUF_SELECTED_SIDECARS.
    static PrepareOptions environment(const std::map<std::string, std::string> &environment);
};

struct PreparedModel {     // GGUFModelLoader.PreparedModel (:140-160)
    MultiModelConfig config;
    std::string weightDir;
    int tensorCount = 0;
};

struct GGUFModelLoader {
    // GGUF -> directory of BLOBFILEs / sidecars + metadata.json into a directory the caller names (the conversion
    // of GGUFModelLoader.prepare, :303-405).
    static int prepare(const std::string &ggufPath, const std::string &outputDir, const PrepareOptions &options, PreparedModel *out);
    // GGUFModelLoader.prepare(ggufURL:options:) (:273-405): returns the cached directory when one matches the file
    // and the options (:495-533); otherwise converts into <cache root>/<key> (cache on: manifest + marker written,
    // :535-566) or into a fresh temporary directory (cache off).
    static int prepare(const std::string &ggufPath, const PrepareOptions &options, const std::map<std::string, std::string> &environment,
                       PreparedModel *out);
    // Metadata -> MultiModelConfig (:297-326)
    static int configFromMetadata(const GGUFLoader &gguf, MultiModelConfig *out);
    // SHA-256 over a sorted-key JSON of cache version, standardised path, file size, modification time, sidecar mode,
    // selected sidecars and the converter environment (:424-447).  The digest is this build's own rendering of that
    // payload: equal inputs give equal keys, any difference in them a different key.
    static int artifactCacheKey(const std::string &ggufPath, const PrepareOptions &options,
                                const std::map<std::string, std::string> &environment, std::string *out);
    static std::string defaultPreparedArtifactCacheRoot();                     // :414-422 ($XDG_CACHE_HOME or ~/.cache here)
    static bool isManagedCachedArtifactDirectory(const std::string &dir);      // :449-453
    static void cleanup(const std::string &weightDir);                         // :408-412: keeps managed cache directories
};

}  // namespace esp
