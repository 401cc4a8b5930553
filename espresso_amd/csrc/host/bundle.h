// The .esp bundle on the reference's side of the decode path: manifest, archive layout, backend selection and
// the bridge that turns a bundle's draft / output-head metadata into the engine's environment.
//   ESPManifest, ESPBundleValidationError, ESPBundleLayout, ESPBundleArchive   Sources/ESPBundle/ESPBundle.swift:4-700
//   ESPRuntimeSelection, ESPRuntimeResolver.selectBackend                      Sources/ESPRuntime/ESPRuntimeContracts.swift:43-138
//   ESPRuntimeBundle.open, ESPRuntimeRunner.resolve / generate, environmentOverrides
//                                                                             Sources/ESPRuntime/ESPBundledRuntime.swift:8-180
// Compilation, conversion, adapters and the command-line tools around bundles are not part of this library.
#pragma once

#include <map>
#include <string>
#include <vector>

#include "engine.h"

namespace esp {

// ESPBundleValidationError (ESPBundle.swift:136-155) and ESPRuntimeSelectionError (ESPRuntimeContracts.swift:71-75)
enum class BundleError : int {
    None = 0,
    EmptyField = 1,              // text = field
    InvalidMaxContext = 2,       // detail = value
    InvalidContextTarget = 3,    // detail = value
    InvalidAdapterSlots = 4,     // detail = value
    MissingBackends = 5,
    MissingProfiles = 6,
    InvalidWeightBits = 7,       // detail = value
    InvalidActivationBits = 8,   // detail = value
    MissingTopLevelEntry = 9,    // text = entry
    MissingManifest = 10,
    MalformedLine = 11,          // text = line
    MalformedSection = 12,       // text = line
    UnsupportedValue = 13,       // text = value or key
    InvalidOutputHead = 14,      // text = message
    InvalidDraft = 15,           // text = message
    InvalidReferencedPath = 16,  // text = reference
    MissingReferencedFile = 17,  // text = reference
    SignatureMismatch = 18,      // text = path
    UnreadableFile = 19,         // text = path
    NoCompatibleBackend = 30,
    NoCompatibleProfile = 31,
    RequestedContextExceedsTarget = 32,   // detail = requested, detail2 = supported
};

struct BundleStatus {
    BundleError error = BundleError::None;
    long detail = 0, detail2 = 0;
    std::string text;
    bool ok() const { return error == BundleError::None; }
};

struct ESPOutputHeadMetadata {
    std::string kind, behaviorClass;            // "dense" | "factored"; "exact" | "near_exact" | "approximate"
    bool hasBottleneck = false, hasGroups = false, hasProjectionRef = false, hasExpansionRef = false;
    long bottleneck = 0, groups = 0;
    std::string projectionRef, expansionRef;
};

struct ESPDraftMetadata {
    std::string kind, behaviorClass;            // "exact_two_token" | "multi_token"
    long horizon = 0;
    std::string verifier, rollback, artifactRef, acceptanceMetric;
};

struct ESPManifest {
    std::string formatVersion, modelID, modelFamily, architectureVersion, tokenizerContract;
    std::vector<std::string> supportedBackends, supportedProfiles;
    long maxContext = 0, contextTargetTokens = 0, adapterSlots = 0;
    std::string compressionName;
    long weightBits = 0, activationBits = 0;
    bool hasActivationBits = false;
    std::string modelTier = "compat", behaviorClass = "exact";
    std::string recipe = "legacy", qualityGate = "legacy-compatible", teacherModel, draftModel, performanceTarget;
    bool hasTeacherModel = false, hasDraftModel = false, hasPerformanceTarget = false;
    bool hasOutputHead = false, hasDraft = false;
    ESPOutputHeadMetadata outputHead;
    ESPDraftMetadata draft;
    std::string accuracyBaselineRef, performanceBaselineRef, signatureRef;

    static BundleStatus parseTOML(const std::string &text, ESPManifest *out);   // ESPBundle.swift:312-394, validated
    BundleStatus validate() const;                                              // :219-266, :402-470
    std::string renderTOML() const;                                             // :268-310
};

struct ESPBundleLayout {
    static constexpr const char *manifestFileName = "manifest.toml";
    static constexpr const char *signatureCatalogFileName = "content-hashes.json";
    static const std::vector<std::string> &requiredTopLevelEntries();
};

struct ESPBundleArchive {
    std::string bundleDir;
    ESPManifest manifest;
    std::string weightsDir() const { return joinPath(bundleDir, "weights"); }
    std::string tokenizerDir() const { return joinPath(bundleDir, "tokenizer"); }
    std::string signatureCatalogPath() const { return joinPath(joinPath(bundleDir, "signatures"), ESPBundleLayout::signatureCatalogFileName); }
    // open(at:verifySignatures:) (:563-590): manifest present, the ten top-level directories, manifest parse, SHA-256
    // catalog check (:600-615), referenced artifacts inside the bundle and present (:641-692)
    static BundleStatus open(const std::string &bundleDir, bool verifySignatures, ESPBundleArchive *out);
    BundleStatus verifySignatures() const;
    // writeSignatureCatalog (:592-598): {"algorithm","fileHashes","manifestHash"}, keys sorted, every regular file
    // except the manifest and the catalog itself
    BundleStatus writeSignatureCatalog() const;
};

struct ESPRuntimeSelection {
    std::string backend, profile, reason;
    long contextTargetTokens = 0;
    bool hasOutputHead = false, hasDraft = false;
    ESPOutputHeadMetadata outputHead;
    ESPDraftMetadata draft;
};

// ESPRuntimeResolver.selectBackend(capabilities:manifest:requestedContextTokens:preferred:) with the default
// preference [ane-private, cpu-safe]; requestedContextTokens < 0 = nil.
BundleStatus selectBackend(bool supportsANEPrivate, const ESPManifest &manifest, long requestedContextTokens, ESPRuntimeSelection *out);
// environmentOverrides(for:) (ESPBundledRuntime.swift:150-179)
Environment environmentOverrides(const ESPRuntimeSelection &selection);

// ESPRuntimeBundle.open(at:) + ESPRuntimeRunner.generate(bundle:prompt:maxTokens:temperature:) (:17-80): config from
// weights/metadata.json, prompt tokens counted with the bundle's tokenizer, backend resolved against
// prompt + maxTokens, the engine built on weights/ and tokenizer/ with the overrides in its environment.
struct ESPRuntimeBundle {
    ESPBundleArchive archive;
    MultiModelConfig config;
    static BundleStatus open(const std::string &bundleDir, bool verifySignatures, ESPRuntimeBundle *out);
    int generate(const std::string &prompt, int maxTokens, float temperature, const Environment &environment, GenerationResult *out,
                 ESPRuntimeSelection *selection, BundleStatus *status) const;
};

std::string sha256_hex(const void *data, size_t bytes);

}  // namespace esp
