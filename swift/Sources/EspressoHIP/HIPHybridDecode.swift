// UNCOMPILED (no Swift toolchain in the build image).
// The three calls the hybrid decode path makes between its kernel evaluations, on surfaces resident in HBM.  They take the
// place of the Metal submissions in runHybridDecodeTimedFromPreparedInput (reference Sources/Espresso/DecodeForwardPass.swift:
// 1116-1300; kernels MetalAttentionKernel.swift:1756-1886).  All three are synchronous.
import CEspressoHIP

public struct HIPHybridLayerSurfaces {
    public let qOut: HIPSurface, kOut: HIPSurface, vOut: HIPSurface     // decode_qkv outputs 1, 0, 2
    public let kCacheFull: HIPSurface, vCacheFull: HIPSurface           // [kvDim, maxSeq]
    public let projectionContextIn: HIPSurface                         // decode_projection input 0
}

public enum HIPHybridDecode {
    /// One layer's work between decodeQKVOnly.eval() and decodeProjection.eval(): RoPE on lane 0 of q and k, k / v into column
    /// `tokenIndex` of the caches, attention over columns 0 ..< tokenIndex + 1 into the projection's context input.
    public static func attend(_ s: HIPHybridLayerSurfaces, heads: Int, kvHeads: Int, headDim: Int, tokenIndex: Int,
                              ropeTheta: Float, maxSeq: Int, laneSpatial: Int) throws(HIPKernelError) {
        let kvDim = Int32(kvHeads * headDim)
        guard esp_interop_rope_decode(s.qOut.ref, s.kOut.ref, Int32(heads), Int32(kvHeads), Int32(headDim), Int32(tokenIndex),
                                      ropeTheta, Int32(laneSpatial)),
              esp_interop_kv_cache_scatter(s.kOut.ref, s.vOut.ref, s.kCacheFull.ref, s.vCacheFull.ref, kvDim, Int32(tokenIndex),
                                           Int32(maxSeq), Int32(laneSpatial)),
              esp_interop_decode_sdpa(s.qOut.ref, s.kCacheFull.ref, s.vCacheFull.ref, s.projectionContextIn.ref, Int32(heads),
                                      Int32(kvHeads), Int32(headDim), Int32(tokenIndex + 1), 0, Int32(maxSeq), Int32(laneSpatial))
        else { throw .evaluationFailed }
    }

    /// Program text of the three per-layer kernels of HybridDecodeKernelSet (reference Sources/ANERuntime/HybridDecodeKernelSet.swift:30-56),
    /// passed where the reference passes MIL text.  `format`: f16 | q8_0 | q4_0 | q4_k.
    public static func qkvProgram(format: String, dim: Int, qDim: Int, kvDim: Int, laneSpatial: Int, normEps: Float) -> String {
        "program: espresso.hip/1\nkernel: decode_qkv\nformat: \(format)\ndim: \(dim) q_dim: \(qDim) kv_dim: \(kvDim)\nspatial: \(laneSpatial) lanes: 1\nnorm_eps: \(normEps)\n"
    }
    public static func projectionProgram(format: String, dim: Int, qDim: Int, laneSpatial: Int) -> String {
        "program: espresso.hip/1\nkernel: decode_projection\nformat: \(format)\ndim: \(dim) q_dim: \(qDim)\nspatial: \(laneSpatial) lanes: 1\n"
    }
    public static func ffnProgram(format: String, dim: Int, hidden: Int, laneSpatial: Int, normEps: Float) -> String {
        "program: espresso.hip/1\nkernel: decode_ffn\nformat: \(format)\ndim: \(dim) hidden: \(hidden)\nspatial: \(laneSpatial) lanes: 1\nnorm_eps: \(normEps)\n"
    }
}
