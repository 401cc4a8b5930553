// UNCOMPILED (no Swift toolchain in the build image).
// The llama decoder resident on the GPU, with the method names of the reference's CPUExactLlamaRuntime
// (Sources/RealModelInference/RealModelInferenceEngine.swift:548-850), and the engine-level generate calls.
import CEspressoHIP

public struct HIPRuntimeError: Error, CustomStringConvertible {
    public let code: Int32
    public let description: String
    init(_ code: Int32) { self.code = code; description = String(cString: esp_last_error()) }
}

@inline(__always) func hipCheck(_ rc: Int32) throws(HIPRuntimeError) {
    guard rc == ESP_OK else { throw HIPRuntimeError(rc) }
}

/// C strings for an environment dictionary, alive for the duration of `body` (the reference passes `environment:` dictionaries).
func withEnvironment<R>(_ env: [String: String], _ body: (UnsafePointer<UnsafePointer<CChar>?>?, UnsafePointer<UnsafePointer<CChar>?>?, Int32) throws -> R) rethrows -> R {
    let keys = env.keys.sorted()
    let k = keys.map { strdup($0) }, v = keys.map { strdup(env[$0]!) }
    defer { k.forEach { free($0) }; v.forEach { free($0) } }
    let kp = k.map { UnsafePointer<CChar>($0) }, vp = v.map { UnsafePointer<CChar>($0) }
    return try kp.withUnsafeBufferPointer { kb in try vp.withUnsafeBufferPointer { vb in try body(kb.baseAddress, vb.baseAddress, Int32(keys.count)) } }
}

public func makeModelConfig(name: String, nLayer: Int, nHead: Int, nKVHead: Int, dModel: Int, headDim: Int, hiddenDim: Int,
                            vocab: Int, maxSeq: Int, normEps: Float, ropeTheta: Float, eosToken: Int?) -> ESPModelConfig {
    var c = ESPModelConfig()
    withUnsafeMutableBytes(of: &c.name) { raw in
        let bytes = Array(name.utf8.prefix(raw.count - 1))
        raw.copyBytes(from: bytes)
    }
    c.n_layer = Int32(nLayer); c.n_head = Int32(nHead); c.n_kv_head = Int32(nKVHead); c.d_model = Int32(dModel)
    c.head_dim = Int32(headDim); c.hidden_dim = Int32(hiddenDim); c.vocab = Int32(vocab); c.max_seq = Int32(maxSeq)
    c.norm_eps = normEps; c.rope_theta = ropeTheta; c.eos_token = Int32(eosToken ?? -1); c.architecture = 1
    return c
}

public struct HIPGenerationResult {
    public var tokens: [UInt32]
    public var tokensPerSecond: Double
    public var compileTimeMs: Double
    public var firstTokenLatencyMs: Double
    public var committedExactTokensPerPass: Double?
    public var acceptedFutureTokensPerPass: Double?
    public var exactHeadBackend: String
}

/// RealModelInferenceEngine.build(config:weightDir:tokenizerDir:) + generate (reference :1377, :1405) over the C ABI.
public final class HIPInferenceEngine {
    private let engine: OpaquePointer
    public let runtime: HIPExactLlamaRuntime

    public init(config: ESPModelConfig, weightDir: String, tokenizerDir: String? = nil, environment: [String: String] = [:]) throws(HIPRuntimeError) {
        var cfg = config
        let built: OpaquePointer? = withEnvironment(environment) { k, v, n in
            esp_engine_build(&cfg, weightDir, tokenizerDir, k, v, n)
        }
        guard let built else { throw HIPRuntimeError(ESP_ERR_INVALID_ARGUMENT) }
        engine = built
        runtime = HIPExactLlamaRuntime(borrowed: esp_engine_runtime(built))
    }
    deinit { esp_engine_free(engine) }

    /// Greedy decode, or the exact two-token draft loop when the environment names a draft
    /// (ESPRESSO_BUNDLE_DRAFT_KIND / _HORIZON / _ARTIFACT_REF, reference :5324-5390).
    public func generate(promptTokens: [UInt32], maxTokens: Int, temperature: Float = 0, environment: [String: String] = [:])
        throws(HIPRuntimeError) -> HIPGenerationResult {
        var out = [UInt32](repeating: 0, count: max(maxTokens, 1))
        var r = ESPGenerationResult()
        let rc: Int32 = withEnvironment(environment) { k, v, n in
            esp_engine_generate(engine, promptTokens, Int32(promptTokens.count), Int32(maxTokens), temperature, k, v, n, &out, &r)
        }
        try hipCheck(rc)
        let backend = withUnsafeBytes(of: r.exact_head_backend) { String(cString: $0.bindMemory(to: CChar.self).baseAddress!) }
        return HIPGenerationResult(tokens: Array(out.prefix(Int(r.token_count))), tokensPerSecond: r.tokens_per_second,
                                   compileTimeMs: r.compile_time_ms, firstTokenLatencyMs: r.first_token_latency_ms,
                                   committedExactTokensPerPass: r.has_two_token_stats != 0 ? r.committed_exact_tokens_per_pass : nil,
                                   acceptedFutureTokensPerPass: r.has_two_token_stats != 0 ? r.accepted_future_tokens_per_pass : nil,
                                   exactHeadBackend: backend)
    }
}

public final class HIPExactLlamaRuntime {
    let rt: OpaquePointer
    private let owned: Bool

    init(borrowed: OpaquePointer) { rt = borrowed; owned = false }
    deinit { if owned { esp_llama_free(rt) } }

    public func reset() throws(HIPRuntimeError) { try hipCheck(esp_llama_reset(rt)) }
    public func prefill(_ tokens: [UInt32]) throws(HIPRuntimeError) { try hipCheck(esp_llama_prefill(rt, 0, tokens, Int32(tokens.count))) }
    public func advance(token: UInt32) throws(HIPRuntimeError) { try hipCheck(esp_llama_advance(rt, 0, token)) }
    public func selectGreedyToken() throws(HIPRuntimeError) -> UInt32 {
        var t: UInt32 = 0
        try hipCheck(esp_llama_select_greedy_token(rt, 0, &t))
        return t
    }
    public var visibleTokenCount: Int { Int(esp_llama_visible_token_count(rt, 0)) }
    /// captureCheckpoint() / rollback(to:) of the reference copy every KV cache; here a checkpoint is the visible token count,
    /// because cache rows beyond it are never read.
    public func captureCheckpoint() -> Int { visibleTokenCount }
    public func rollback(to checkpoint: Int) throws(HIPRuntimeError) { try hipCheck(esp_llama_set_visible_token_count(rt, 0, Int32(checkpoint))) }
    public func continueGreedy(steps: Int) throws(HIPRuntimeError) -> [UInt32] {
        var out = [UInt32](repeating: 0, count: steps)
        try hipCheck(esp_llama_continue_greedy(rt, 0, Int32(steps), &out))
        return out
    }
}
