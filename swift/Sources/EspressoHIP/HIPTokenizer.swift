// UNCOMPILED (no Swift toolchain in the build image).
// A tokenizer over the C ABI with the members of the reference's Tokenizer protocol (Sources/ModelSupport/Tokenizer.swift):
// loadTokenizer's candidate order (RealModelInferenceEngine.swift:7558-7613) runs inside esp_tokenizer_load_dir.
import CEspressoHIP

public final class HIPTokenizer: @unchecked Sendable {
    private let h: OpaquePointer

    public init(config: ESPModelConfig, tokenizerDir: String) throws(HIPRuntimeError) {
        var c = config
        guard let t = esp_tokenizer_load_dir(&c, tokenizerDir) else { throw HIPRuntimeError(ESP_ERR_IO) }
        h = t
    }
    deinit { esp_tokenizer_free(h) }

    public var vocabSize: Int { Int(esp_tokenizer_vocab_size(h)) }

    public func encode(_ text: String) -> [Int] {
        let n = esp_tokenizer_encode(h, text, text.utf8.count, nil, 0)
        guard n > 0 else { return [] }
        var ids = [Int32](repeating: 0, count: n)
        _ = esp_tokenizer_encode(h, text, text.utf8.count, &ids, ids.count)
        return ids.map(Int.init)
    }

    public func decode(_ tokens: [Int]) -> String {
        let ids = tokens.map(Int32.init)
        let n = esp_tokenizer_decode(h, ids, ids.count, nil, 0)
        guard n > 0 else { return "" }
        var bytes = [CChar](repeating: 0, count: n)
        _ = esp_tokenizer_decode(h, ids, ids.count, &bytes, bytes.count)
        return String(decoding: bytes.map { UInt8(bitPattern: $0) }, as: UTF8.self)
    }
}
