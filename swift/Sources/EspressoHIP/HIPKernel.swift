// UNCOMPILED (no Swift toolchain in the build image).
// Kernel handle over esp_interop_*: the shape of ANEKernel (reference Sources/ANERuntime/ANEKernel.swift).
import CEspressoHIP
import Foundation

/// Same cases as the reference's ANEError (Sources/ANERuntime/ANEError.swift:3-19).
public enum HIPKernelError: Error, Sendable, Equatable {
    case invalidArguments(String)
    case compilationFailed
    case evaluationFailed
    case compileBudgetExhausted
    case surfaceAllocationFailed
    case invalidSurfaceIndex(Int)
    case inputSurfaceUnavailable(Int)
    case outputSurfaceUnavailable(Int)
}

/// Reference-counted device surface; stands where IOSurfaceRef stood.  A flat fp16 buffer read as
/// channel-first [channels, spatial], element (c, s) at c * spatial + s.
public final class HIPSurface: @unchecked Sendable {
    let ref: ESPSurfaceRef

    /// Takes ownership of a +1 reference (esp_interop_create_surface, esp_interop_copy_input / _output).
    init(retained: ESPSurfaceRef) { ref = retained }

    public convenience init(bytes: Int) throws(HIPKernelError) {
        guard bytes > 0, let s = esp_interop_create_surface(bytes) else { throw .surfaceAllocationFailed }
        self.init(retained: s)
    }

    public var byteCount: Int { Int(esp_surface_bytes(ref)) }

    deinit { esp_surface_release(ref) }
}

/// One compiled kernel set: program text + weights in, fixed input / output surfaces, synchronous eval.
public struct HIPKernel: ~Copyable {
    private let handle: OpaquePointer

    /// `program` is the "key: value" descriptor documented beside esp_interop_compile (kernel kinds gemv,
    /// rmsnorm_classifier, decode_ffn, decode_qkv, decode_projection).  Weight bytes are copied during the call,
    /// as ane_interop_compile copies its blobs (ANEKernel.swift:221-270): the caller keeps ownership.
    public init(program: String, weights: [(path: String, data: Data)],
                inputSizes: [Int], outputSizes: [Int]) throws(HIPKernelError) {
        guard !inputSizes.isEmpty, !outputSizes.isEmpty else { throw .invalidArguments("no surfaces") }
        let text = Array(program.utf8)
        let cPaths: [UnsafeMutablePointer<CChar>?] = weights.map { strdup($0.path) }
        defer { cPaths.forEach { free($0) } }
        // contiguous copies that stay alive across the call
        let buffers: [UnsafeMutableBufferPointer<UInt8>] = weights.map {
            let b = UnsafeMutableBufferPointer<UInt8>.allocate(capacity: max($0.data.count, 1))
            _ = b.initialize(from: $0.data)
            return b
        }
        defer { buffers.forEach { $0.deallocate() } }
        var paths: [UnsafePointer<CChar>?] = cPaths.map { UnsafePointer($0) }
        var datas: [UnsafePointer<UInt8>?] = buffers.map { UnsafePointer($0.baseAddress) }
        var lens: [Int] = weights.map { $0.data.count }
        var ins = inputSizes, outs = outputSizes
        let created = text.withUnsafeBufferPointer { t in
            esp_interop_compile(t.baseAddress, t.count, &paths, &datas, &lens, Int32(weights.count),
                                Int32(ins.count), &ins, Int32(outs.count), &outs)
        }
        guard let created else {
            switch esp_interop_last_compile_error() {          // same codes as ane_interop.h:18-22
            case ESP_INTEROP_COMPILE_ERROR_INVALID_ARGUMENTS:
                throw .invalidArguments(String(cString: esp_last_error()))
            case ESP_INTEROP_COMPILE_ERROR_DUPLICATE_WEIGHT_PATH:
                throw .invalidArguments("Duplicate weight path detected")
            case ESP_INTEROP_COMPILE_ERROR_SURFACE_ALLOCATION_FAILED:
                throw .surfaceAllocationFailed
            default:
                throw .compilationFailed
            }
        }
        handle = created
    }

    /// Synchronous: outputs are valid on return (ANEKernel.swift:437-444).
    public func eval() throws(HIPKernelError) {
        guard esp_interop_eval(handle) else { throw .evaluationFailed }
    }

    public func inputSurface(at index: Int) throws(HIPKernelError) -> HIPSurface {
        guard index >= 0 else { throw .invalidSurfaceIndex(index) }
        guard let s = esp_interop_copy_input(handle, Int32(index)) else { throw .inputSurfaceUnavailable(index) }
        return HIPSurface(retained: s)
    }

    public func outputSurface(at index: Int) throws(HIPKernelError) -> HIPSurface {
        guard index >= 0 else { throw .invalidSurfaceIndex(index) }
        guard let s = esp_interop_copy_output(handle, Int32(index)) else { throw .outputSurfaceUnavailable(index) }
        return HIPSurface(retained: s)
    }

    /// Zero-copy chaining: input `index` reads `surface` from now on (ane_interop_rebind_input, ane_interop.h:50).
    /// Not to be called while an eval of this handle is running (ANEKernel.swift:611-616).
    public func rebindInput(at index: Int, to surface: HIPSurface) throws(HIPKernelError) {
        guard esp_interop_rebind_input(handle, Int32(index), surface.ref) else {
            throw .invalidArguments("rebindInput(at: \(index))")
        }
    }

    public func lastHWExecutionTimeNS() -> UInt64 { esp_interop_last_hw_execution_time_ns(handle) }
    public var hasPerfStats: Bool { esp_interop_has_perf_stats(handle) }

    deinit { esp_interop_free(handle) }

    // Test hooks of the reference (ane_interop.h:37-41).
    public static var compileCount: Int {
        get { Int(esp_interop_compile_count()) }
        set { esp_interop_set_compile_count(Int32(newValue)) }
    }
    public static var liveHandleCount: Int { Int(esp_interop_live_handle_count()) }
    public static func setForceEvalFailure(_ value: Bool) { esp_interop_set_force_eval_failure(value) }
}
