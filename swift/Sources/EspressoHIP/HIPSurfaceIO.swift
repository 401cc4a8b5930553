// UNCOMPILED (no Swift toolchain in the build image).
// SurfaceIO over esp_interop_io_*: same entry points and error cases as the reference's SurfaceIO
// (Sources/ANETypes/SurfaceIO.swift), each body one call into the C function of the same name.
// fp32 on the caller's side, fp16 on the surface; element (c, s) of a [channels, spatial] surface is at c * spatial + s.
import CEspressoHIP

public enum HIPSurfaceIOError: Error, Equatable {      // SurfaceIOError, SurfaceIO.swift:4-7
    case argumentOutOfRange
    case interopCallFailed
}

public enum HIPSurfaceIO {
    public struct FP16ArgmaxResult: Equatable {
        public let index: Int
        public let value: Float
    }
    public struct FP16ReadRegion {
        public let destination: UnsafeMutablePointer<Float>
        public let channelOffset: Int
        public let channels: Int
        public init(destination: UnsafeMutablePointer<Float>, channelOffset: Int, channels: Int) {
            self.destination = destination; self.channelOffset = channelOffset; self.channels = channels
        }
    }
    public struct FP16WriteRegion {
        public let source: UnsafePointer<Float>
        public let channelOffset: Int
        public let channels: Int
        public init(source: UnsafePointer<Float>, channelOffset: Int, channels: Int) {
            self.source = source; self.channelOffset = channelOffset; self.channels = channels
        }
    }
    public struct FP16CopyRegion {
        public let dstChannelOffset: Int
        public let srcChannelOffset: Int
        public let channels: Int
        public init(dstChannelOffset: Int, srcChannelOffset: Int, channels: Int) {
            self.dstChannelOffset = dstChannelOffset; self.srcChannelOffset = srcChannelOffset; self.channels = channels
        }
    }
    public struct FP16SourceCopyRegion {
        public let source: HIPSurface
        public let dstChannelOffset: Int
        public let srcChannelOffset: Int
        public let channels: Int
        public init(source: HIPSurface, dstChannelOffset: Int, srcChannelOffset: Int, channels: Int) {
            self.source = source; self.dstChannelOffset = dstChannelOffset
            self.srcChannelOffset = srcChannelOffset; self.channels = channels
        }
    }

    @inline(__always) private static func i32(_ v: Int) throws(HIPSurfaceIOError) -> Int32 {
        guard let r = Int32(exactly: v), r >= 0 else { throw .argumentOutOfRange }
        return r
    }
    @inline(__always) private static func check(_ ok: Bool) throws(HIPSurfaceIOError) {
        guard ok else { throw .interopCallFailed }
    }

    // The reference's whole-surface write and read trap on misuse (precondition); so do these.
    public static func writeFP16(to surface: HIPSurface, data: UnsafeBufferPointer<Float>, channels: Int, spatial: Int) {
        precondition(channels >= 0 && spatial >= 0 && data.count == channels * spatial)
        precondition(esp_interop_io_write_fp16(surface.ref, data.baseAddress, Int32(channels), Int32(spatial)))
    }
    public static func readFP16(from surface: HIPSurface, into data: UnsafeMutableBufferPointer<Float>,
                                channelOffset: Int, channels: Int, spatial: Int) {
        precondition(channelOffset >= 0 && channels >= 0 && spatial >= 0 && data.count == channels * spatial)
        precondition(esp_interop_io_read_fp16(surface.ref, Int32(channelOffset), data.baseAddress, Int32(channels), Int32(spatial)))
    }
    public static func readFP16Batched(from surface: HIPSurface, spatial: Int, regions: [FP16ReadRegion]) {
        guard !regions.isEmpty else { return }
        var dsts: [UnsafeMutablePointer<Float>?] = regions.map { $0.destination }
        var offs = regions.map { Int32($0.channelOffset) }
        var chans = regions.map { Int32($0.channels) }
        precondition(esp_interop_io_read_fp16_batched(surface.ref, Int32(spatial), &dsts, &offs, &chans, Int32(regions.count)))
    }

    public static func writeFP16At(to surface: HIPSurface, channelOffset: Int, data: UnsafeBufferPointer<Float>,
                                   channels: Int, spatial: Int) throws(HIPSurfaceIOError) {
        guard data.count == channels * spatial else { throw .argumentOutOfRange }
        try check(esp_interop_io_write_fp16_at(surface.ref, try i32(channelOffset), data.baseAddress, try i32(channels), try i32(spatial)))
    }
    public static func writeFP16AtBatched(to surface: HIPSurface, spatial: Int, regions: [FP16WriteRegion]) throws(HIPSurfaceIOError) {
        guard !regions.isEmpty else { return }
        var srcs: [UnsafePointer<Float>?] = regions.map { $0.source }
        var offs = [Int32](), chans = [Int32]()
        for r in regions { offs.append(try i32(r.channelOffset)); chans.append(try i32(r.channels)) }
        try check(esp_interop_io_write_fp16_at_batched(surface.ref, &offs, &srcs, &chans, Int32(regions.count), try i32(spatial)))
    }

    public static func copyFP16(dst: HIPSurface, dstChannelOffset: Int, src: HIPSurface, srcChannelOffset: Int,
                                channels: Int, spatial: Int) throws(HIPSurfaceIOError) {
        try check(esp_interop_io_copy(dst.ref, try i32(dstChannelOffset), src.ref, try i32(srcChannelOffset),
                                      try i32(channels), try i32(spatial)))
    }
    public static func copyFP16Batched(dst: HIPSurface, src: HIPSurface, spatial: Int, regions: [FP16CopyRegion]) throws(HIPSurfaceIOError) {
        guard !regions.isEmpty else { return }
        var d = [Int32](), s = [Int32](), c = [Int32]()
        for r in regions { d.append(try i32(r.dstChannelOffset)); s.append(try i32(r.srcChannelOffset)); c.append(try i32(r.channels)) }
        try check(esp_interop_io_copy_batched(dst.ref, src.ref, &d, &s, &c, Int32(regions.count), try i32(spatial)))
    }
    public static func copyFP16FromMultipleSources(dst: HIPSurface, spatial: Int, regions: [FP16SourceCopyRegion]) throws(HIPSurfaceIOError) {
        guard !regions.isEmpty else { return }
        var srcs: [ESPSurfaceRef?] = regions.map { $0.source.ref }
        var d = [Int32](), s = [Int32](), c = [Int32]()
        for r in regions { d.append(try i32(r.dstChannelOffset)); s.append(try i32(r.srcChannelOffset)); c.append(try i32(r.channels)) }
        try check(esp_interop_io_copy_multi_src(dst.ref, &srcs, &d, &s, &c, Int32(regions.count), try i32(spatial)))
    }

    public static func copyFP16SpatialSlice(dst: HIPSurface, dstChannelOffset: Int, dstSpatialIndex: Int, dstSpatial: Int,
                                            src: HIPSurface, srcChannelOffset: Int, srcSpatialIndex: Int, srcSpatial: Int,
                                            channels: Int) throws(HIPSurfaceIOError) {
        try check(esp_interop_io_copy_fp16_spatial_slice(dst.ref, try i32(dstChannelOffset), try i32(dstSpatialIndex), try i32(dstSpatial),
                                                         src.ref, try i32(srcChannelOffset), try i32(srcSpatialIndex), try i32(srcSpatial),
                                                         try i32(channels)))
    }
    public static func copyTwoFP16SpatialSlices(
        dst0: HIPSurface, dst0ChannelOffset: Int, dst0SpatialIndex: Int, dst0Spatial: Int,
        src0: HIPSurface, src0ChannelOffset: Int, src0SpatialIndex: Int, src0Spatial: Int,
        dst1: HIPSurface, dst1ChannelOffset: Int, dst1SpatialIndex: Int, dst1Spatial: Int,
        src1: HIPSurface, src1ChannelOffset: Int, src1SpatialIndex: Int, src1Spatial: Int,
        channels: Int) throws(HIPSurfaceIOError) {
        try check(esp_interop_io_copy_two_fp16_spatial_slices(
            dst0.ref, try i32(dst0ChannelOffset), try i32(dst0SpatialIndex), try i32(dst0Spatial),
            src0.ref, try i32(src0ChannelOffset), try i32(src0SpatialIndex), try i32(src0Spatial),
            dst1.ref, try i32(dst1ChannelOffset), try i32(dst1SpatialIndex), try i32(dst1Spatial),
            src1.ref, try i32(src1ChannelOffset), try i32(src1SpatialIndex), try i32(src1Spatial), try i32(channels)))
    }

    public static func writeFP16SpatialSlice(to surface: HIPSurface, channelOffset: Int, spatialIndex: Int, spatial: Int,
                                             data: UnsafeBufferPointer<Float>, channels: Int) throws(HIPSurfaceIOError) {
        guard data.count == channels else { throw .argumentOutOfRange }
        try check(esp_interop_io_write_fp16_spatial_slice(surface.ref, try i32(channelOffset), try i32(spatialIndex), try i32(spatial),
                                                          data.baseAddress, try i32(channels)))
    }
    public static func readFP16SpatialSlice(from surface: HIPSurface, channelOffset: Int, spatialIndex: Int, spatial: Int,
                                            into data: UnsafeMutableBufferPointer<Float>, channels: Int) throws(HIPSurfaceIOError) {
        guard data.count == channels else { throw .argumentOutOfRange }
        try check(esp_interop_io_read_fp16_spatial_slice(surface.ref, try i32(channelOffset), try i32(spatialIndex), try i32(spatial),
                                                         data.baseAddress, try i32(channels)))
    }

    /// First maximum of one spatial column (lowest channel wins ties, neon_convert.c:36-101).
    public static func argmaxFP16SpatialSlice(from surface: HIPSurface, channelOffset: Int, spatialIndex: Int, spatial: Int,
                                              channels: Int) throws(HIPSurfaceIOError) -> FP16ArgmaxResult {
        var index: Int32 = 0
        var value: Float = 0
        try check(esp_interop_io_argmax_fp16_spatial_slice(surface.ref, try i32(channelOffset), try i32(spatialIndex), try i32(spatial),
                                                           try i32(channels), &index, &value))
        return FP16ArgmaxResult(index: Int(index), value: value)
    }
    public static func argmaxFP16SpatialSliceWithHint(from surface: HIPSurface, channelOffset: Int, spatialIndex: Int, spatial: Int,
                                                      channels: Int, hint: HIPSurface, hintSpatialIndex: Int, hintSpatial: Int)
        throws(HIPSurfaceIOError) -> FP16ArgmaxResult {
        var index: Int32 = 0
        var value: Float = 0
        try check(esp_interop_io_argmax_fp16_spatial_slice_with_hint(surface.ref, try i32(channelOffset), try i32(spatialIndex), try i32(spatial),
                                                                     try i32(channels), hint.ref, try i32(hintSpatialIndex), try i32(hintSpatial),
                                                                     &index, &value))
        return FP16ArgmaxResult(index: Int(index), value: value)
    }

    public static func writeEmbeddingBatchFP16(to surface: HIPSurface, channelOffset: Int, spatial: Int,
                                               embeddingTable: UnsafeBufferPointer<Float>, vocabSize: Int, dim: Int,
                                               tokenIDs: [UInt16]) throws(HIPSurfaceIOError) {
        guard embeddingTable.count == vocabSize * dim else { throw .argumentOutOfRange }
        var ids = tokenIDs
        try check(esp_interop_io_write_embedding_batch_fp16(surface.ref, try i32(channelOffset), try i32(spatial), embeddingTable.baseAddress,
                                                            try i32(vocabSize), try i32(dim), &ids, try i32(ids.count)))
    }

    private enum BatchArgmax { case locked, parallel(Int), nolock(Int) }
    private static func argmaxBatch(_ kind: BatchArgmax, _ surface: HIPSurface, _ channelOffset: Int, _ spatial: Int, _ channels: Int,
                                    _ streamCount: Int) throws(HIPSurfaceIOError) -> [FP16ArgmaxResult] {
        var idx = [Int32](repeating: 0, count: streamCount)
        var val = [Float](repeating: 0, count: streamCount)
        let (o, s, c, n) = (try i32(channelOffset), try i32(spatial), try i32(channels), try i32(streamCount))
        switch kind {
        case .locked: try check(esp_interop_io_argmax_batch_fp16_spatial(surface.ref, o, s, c, n, &idx, &val))
        case let .parallel(b): try check(esp_interop_io_argmax_batch_fp16_spatial_parallel(surface.ref, o, s, c, n, &idx, &val, try i32(b)))
        case let .nolock(b): try check(esp_interop_io_argmax_batch_fp16_spatial_nolock(surface.ref, o, s, c, n, &idx, &val, try i32(b)))
        }
        return zip(idx, val).map { FP16ArgmaxResult(index: Int($0), value: $1) }
    }
    public static func argmaxBatchFP16Spatial(from surface: HIPSurface, channelOffset: Int, spatial: Int, channels: Int,
                                              streamCount: Int) throws(HIPSurfaceIOError) -> [FP16ArgmaxResult] {
        try argmaxBatch(.locked, surface, channelOffset, spatial, channels, streamCount)
    }
    public static func argmaxBatchFP16SpatialParallel(from surface: HIPSurface, channelOffset: Int, spatial: Int, channels: Int,
                                                      streamCount: Int, nBlocks: Int) throws(HIPSurfaceIOError) -> [FP16ArgmaxResult] {
        try argmaxBatch(.parallel(nBlocks), surface, channelOffset, spatial, channels, streamCount)
    }
    /// The caller holds the read lock (lockRead ... unlockRead).
    public static func argmaxBatchFP16SpatialNolock(from surface: HIPSurface, channelOffset: Int, spatial: Int, channels: Int,
                                                    streamCount: Int, nBlocks: Int) throws(HIPSurfaceIOError) -> [FP16ArgmaxResult] {
        try argmaxBatch(.nolock(nBlocks), surface, channelOffset, spatial, channels, streamCount)
    }

    /// Expansion + arg-max of the factored output head (SurfaceIO.swift:617): logits[v] = sum over the bottleneck
    /// channels of the row's group, fp16 fused multiply-adds, first maximum.
    public static func fusedExpansionArgmax(projection surface: HIPSurface, channelOffset: Int, spatial: Int, bottleneck: Int, groups: Int,
                                            expansionWeightsFP16: UnsafeRawPointer, vocabSize: Int, streamCount: Int, nBlocks: Int)
        throws(HIPSurfaceIOError) -> [FP16ArgmaxResult] {
        var idx = [Int32](repeating: 0, count: streamCount)
        var val = [Float](repeating: 0, count: streamCount)
        try check(esp_interop_fused_expansion_argmax_fp16(surface.ref, try i32(channelOffset), try i32(spatial), try i32(bottleneck), try i32(groups),
                                                          expansionWeightsFP16, try i32(vocabSize), try i32(streamCount), &idx, &val, try i32(nBlocks)))
        return zip(idx, val).map { FP16ArgmaxResult(index: Int($0), value: $1) }
    }

    // lock_read makes the device copy visible to the host; lock_write marks the host copy as the newer one.
    public static func lockWrite(_ surface: HIPSurface) -> Bool { esp_interop_io_lock_write(surface.ref) }
    public static func unlockWrite(_ surface: HIPSurface) -> Bool { esp_interop_io_unlock_write(surface.ref) }
    public static func lockRead(_ surface: HIPSurface) -> Bool { esp_interop_io_lock_read(surface.ref) }
    public static func unlockRead(_ surface: HIPSurface) -> Bool { esp_interop_io_unlock_read(surface.ref) }
    public static func writeFP16Unlocked(to surface: HIPSurface, data: UnsafeBufferPointer<Float>, channels: Int, spatial: Int) {
        precondition(data.count == channels * spatial)
        precondition(esp_interop_io_write_fp16_unlocked(surface.ref, data.baseAddress, Int32(channels), Int32(spatial)))
    }
    public static func readFP16Unlocked(from surface: HIPSurface, into data: UnsafeMutableBufferPointer<Float>,
                                        channelOffset: Int, channels: Int, spatial: Int) {
        precondition(data.count == channels * spatial)
        precondition(esp_interop_io_read_fp16_unlocked(surface.ref, Int32(channelOffset), data.baseAddress, Int32(channels), Int32(spatial)))
    }
}
