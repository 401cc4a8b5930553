// Not compiled in this repository (no Swift toolchain in the build image): the wrapper a maintainer of the reference would add.
//
// Drop-in for Sources/Espresso/MetalExpansionArgmax.swift's FusedExpansionArgmax (lines 966-1088): the factored output head's
// expansion weights live on the GPU, run(projectedSurface:) returns one token per spatial lane and no logits are stored.
import CEspressoHIP

public enum HIPExpansionArgmaxError: Error, Equatable {
    case invalidArguments(String)
    case deviceUnavailable(String)
    case commandExecutionFailed(String)
}

public final class HIPFusedExpansionArgmax {
    private let head: ESPExpansionHeadRef
    public let bottleneck: Int
    public let vocabSize: Int
    public let spatial: Int
    public let groups: Int

    public init(wExpand: UnsafeBufferPointer<Float16>, bottleneck: Int, vocabSize: Int, spatial: Int, groups: Int = 1) throws(HIPExpansionArgmaxError) {
        guard bottleneck > 0, vocabSize > 0, spatial > 0, groups > 0 else { throw .invalidArguments("all dimensions must be > 0") }
        guard vocabSize <= Int(UInt16.max) else { throw .invalidArguments("vocabSize exceeds UInt16 token ids") }
        guard bottleneck % groups == 0, wExpand.count >= vocabSize * (bottleneck / groups) else { throw .invalidArguments("wExpand too small") }
        guard let ref = esp_interop_expansion_head_create(wExpand.baseAddress, Int32(bottleneck), Int32(groups), Int32(vocabSize)) else {
            throw .deviceUnavailable(String(cString: esp_last_error()))
        }
        self.head = ref
        self.bottleneck = bottleneck
        self.vocabSize = vocabSize
        self.spatial = spatial
        self.groups = groups
    }

    deinit { esp_interop_expansion_head_free(head) }

    /// fp32Sums: false follows the NEON routine's fp16 fused multiply-adds (surface_io.c:1521-1700), true the Metal shader's fp32 ones.
    public func run(projectedSurface: HIPSurface, streamCount: Int? = nil, fp32Sums: Bool = false) throws(HIPExpansionArgmaxError) -> [UInt16] {
        let lanes = streamCount ?? spatial
        var indices = [Int32](repeating: 0, count: lanes)
        var values = [Float](repeating: 0, count: lanes)
        guard esp_interop_expansion_head_argmax(head, projectedSurface.ref, 0, Int32(spatial), Int32(lanes), fp32Sums ? 1 : 0, &indices, &values) else {
            throw .commandExecutionFailed(String(cString: esp_last_error()))
        }
        return indices.map { UInt16($0) }
    }
}
