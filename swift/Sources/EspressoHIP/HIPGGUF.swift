// UNCOMPILED (no Swift toolchain in the build image).
// GGUFModelLoader.prepare / RunGGUF.main over the C ABI (reference Sources/EspressoGGUF/GGUFModelLoader.swift:267-412,
// RunGGUF.swift:68-113).  Packed GGUF blocks are written beside the BLOBFILEs and uploaded to HBM as they are.
import CEspressoHIP

public struct HIPPreparedModel {
    public let config: ESPModelConfig
    public let weightDir: String
    public let tensorCount: Int
}

public enum HIPGGUFModelLoader {
    public static func prepare(ggufPath: String, outputDir: String) throws(HIPRuntimeError) -> HIPPreparedModel {
        var cfg = ESPModelConfig()
        var count: Int32 = 0
        try hipCheck(esp_gguf_prepare(ggufPath, outputDir, nil, &cfg, &count))
        return HIPPreparedModel(config: cfg, weightDir: outputDir, tensorCount: Int(count))
    }
    public static func cleanup(weightDir: String) { _ = esp_gguf_cleanup(weightDir) }
}

public enum HIPRunGGUF {
    /// prepare -> build -> generate -> cleanup in one call; returns (generated token ids, prompt + generated text).
    public static func main(ggufPath: String, tokenizerDir: String, prompt: String, maxTokens: Int,
                            environment: [String: String] = [:]) throws(HIPRuntimeError) -> (tokens: [UInt32], text: String) {
        var tokens = [UInt32](repeating: 0, count: max(maxTokens, 1))
        var text = [CChar](repeating: 0, count: 1 << 16)
        var textBytes = 0
        var result = ESPGenerationResult()
        var info = ESPRunGGUFInfo()
        let rc: Int32 = withEnvironment(environment) { k, v, n in
            esp_run_gguf(ggufPath, tokenizerDir, prompt, prompt.utf8.count, Int32(maxTokens), k, v, n, &tokens, &text, text.count,
                         &textBytes, &result, &info)
        }
        try hipCheck(rc)
        let bytes = text.prefix(min(textBytes, text.count)).map { UInt8(bitPattern: $0) }
        return (Array(tokens.prefix(Int(result.token_count))), String(decoding: bytes, as: UTF8.self))
    }
}
