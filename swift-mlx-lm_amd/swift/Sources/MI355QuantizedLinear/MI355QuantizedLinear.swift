// Swift face of the MI355X quantized-linear library: the value types MetalCompiler's planner and
// executors use for this path, backed by the C ABI instead of generated Metal kernels.
//
//   QuantizationFormat / QuantizationFormatRegistry   MC/STAF/QuantizationFormat.swift:25-153, 1284-1335
//   STAFWeightBufferAccess (packed-weight handle)      MC/STAF/STAFLoader.swift:213-299
//   MetalDispatchStep.metadata / plan entry            MC/Execution/MetalDecodePlan.swift:6-97,
//                                                      MC/Compiler/MetalQuantizationPlan.swift:304-318
//
// Errors keep the reference's convention: plan/compile-time failures throw, programmer errors trap.
import CMI355QLinear
import Foundation

public enum MI355QError: Error, CustomStringConvertible {
    case invalidArgument(String), unsupportedQuantization(String), inconsistentShape(String)
    case deviceSetupFailed(String), outOfMemory(String), kernelNotFound(String), sizeMismatch(String)

    public var description: String { "\(self)" }

    static func check(_ status: mi355q_status) throws {
        guard status != MI355Q_OK else { return }
        let message = String(cString: mi355q_last_error())
        switch status {
        case MI355Q_ERR_UNSUPPORTED_FORMAT: throw MI355QError.unsupportedQuantization(message)
        case MI355Q_ERR_SHAPE: throw MI355QError.inconsistentShape(message)
        case MI355Q_ERR_DEVICE: throw MI355QError.deviceSetupFailed(message)
        case MI355Q_ERR_OUT_OF_MEMORY: throw MI355QError.outOfMemory(message)
        case MI355Q_ERR_KERNEL_NOT_FOUND: throw MI355QError.kernelNotFound(message)
        case MI355Q_ERR_SIZE_MISMATCH: throw MI355QError.sizeMismatch(message)
        default: throw MI355QError.invalidArgument(message)
        }
    }
}

public enum BufferPrecision: UInt32 {
    case float16 = 0, bfloat16 = 1, float32 = 2
    var c: mi355q_dtype { mi355q_dtype(rawValue) }
}

public enum WeightLayout: UInt32 {
    case rowMajorBlocks = 0      // canonical STAF interleaved blocks
    case splitPlanes = 1         // specialized layout of this backend
    case tile16 = 2              // matrix-core decode layout (q4 g64): 1...16 sequences per launch
    var c: mi355q_layout { mi355q_layout(rawValue) }
}

/// Format descriptor with the fields of the reference's `QuantizationFormat` protocol.
public struct QuantizationFormat: Sendable {
    public let schemeIdentifier: UInt8
    public let bits: Int
    public let groupSize: Int
    public let weightsPerBlock: Int
    public let bytesPerBlock: Int
    public let isAligned: Bool
    public let gemvKernelName: String
    public let dequantToBFloatKernelName: String

    init(_ f: mi355q_format) {
        schemeIdentifier = f.scheme_identifier
        bits = Int(f.bits)
        groupSize = Int(f.group_size)
        weightsPerBlock = Int(f.weights_per_block)
        bytesPerBlock = Int(f.bytes_per_block)
        isAligned = f.is_aligned != 0
        gemvKernelName = withUnsafeBytes(of: f.gemv_kernel_name) { String(cString: $0.bindMemory(to: CChar.self).baseAddress!) }
        dequantToBFloatKernelName = withUnsafeBytes(of: f.dequant_to_bfloat_kernel_name) {
            String(cString: $0.bindMemory(to: CChar.self).baseAddress!)
        }
    }
}

public enum QuantizationFormatRegistry {
    /// nil for an unknown pair, as in the reference; callers throw, nothing falls back silently.
    public static func formatForMLXQuantization(bits: Int, groupSize: Int) -> QuantizationFormat? {
        var f = mi355q_format()
        guard mi355q_format_for_mlx_quantization(Int32(bits), Int32(groupSize), &f) == MI355Q_OK else { return nil }
        return QuantizationFormat(f)
    }

    public static func format(for schemeIdentifier: UInt8) -> QuantizationFormat? {
        var f = mi355q_format()
        guard mi355q_format_for_scheme(schemeIdentifier, &f) == MI355Q_OK else { return nil }
        return QuantizationFormat(f)
    }
}

/// One device context = one GPU + the streams the caller creates on it.  Thread-compatible:
/// callers serialise per context, as MetalSubmissionContext does.
public final class MI355Context {
    let handle: OpaquePointer

    public init(deviceIndex: Int = 0) throws {
        var h: OpaquePointer?
        try MI355QError.check(mi355q_context_create(Int32(deviceIndex), &h))
        handle = h!
    }

    deinit { _ = mi355q_context_destroy(handle) }

    public func makeStream() throws -> UnsafeMutableRawPointer {
        var s: UnsafeMutableRawPointer?
        try MI355QError.check(mi355q_stream_create(handle, &s))
        return s!
    }

    public func synchronize(_ stream: UnsafeMutableRawPointer?) throws {
        try MI355QError.check(mi355q_stream_synchronize(handle, stream))
    }
}

/// Packed weight resident in HBM: the analogue of a specialized STAF buffer access.
public final class PackedWeight {
    let handle: OpaquePointer
    public let context: MI355Context

    /// Wraps STAF blocks that already live in device memory (zero copy): `buffer + offset` of the
    /// reference's `STAFWeightBufferAccess`.
    public init(context: MI355Context, format: QuantizationFormat, outputDimension: Int, inputDimension: Int,
                stafBlocks: UnsafeRawPointer, byteCount: Int) throws {
        var h: OpaquePointer?
        try MI355QError.check(mi355q_weight_wrap_staf(context.handle, format.schemeIdentifier, UInt64(outputDimension),
                                                      UInt64(inputDimension), stafBlocks, byteCount, &h))
        handle = h!
        self.context = context
    }

    /// Takes ownership of a handle made by the library (a tensor of an opened container).
    init(context: MI355Context, owning handle: OpaquePointer) {
        self.handle = handle
        self.context = context
    }

    deinit { _ = mi355q_weight_destroy(handle) }

    /// Plan record of the decode step of this projection (kernel name, grid, shape family,
    /// fallback reason): what QuantizationPlanningTests asserts on.
    public func planDecodeStep(sequenceLength: Int = 1, precision: BufferPrecision = .bfloat16) throws -> mi355q_step {
        var step = mi355q_step()
        try MI355QError.check(mi355q_plan_decode_step(handle, UInt32(sequenceLength), precision.c, 0, &step))
        return step
    }
}

/// Encoders of the three dispatch steps of the path.
public extension MI355Context {
    /// Decode projection: buffers 0=input, 1=weight, 2=output; dims come from the weight handle.
    func encodeDecodeProjection(stream: UnsafeMutableRawPointer?, weight: PackedWeight,
                                input: UnsafeRawPointer, output: UnsafeMutableRawPointer,
                                precision: BufferPrecision, sequenceLength: Int = 1) throws {
        try MI355QError.check(mi355q_qgemv(handle, stream, weight.handle, input, precision.c, output, precision.c,
                                           UInt32(sequenceLength), 0, 0, 0))
    }

    /// Prefill projection: sequenceLength is bound at run time, inputRowStride is in elements.
    func encodePrefillProjection(stream: UnsafeMutableRawPointer?, weight: PackedWeight,
                                 input: UnsafeRawPointer, output: UnsafeMutableRawPointer,
                                 precision: BufferPrecision, sequenceLength: Int, inputRowStride: Int) throws {
        try MI355QError.check(mi355q_qgemm(handle, stream, weight.handle, input, precision.c, output, precision.c,
                                           UInt32(sequenceLength), UInt32(inputRowStride), 0, 0))
    }

    /// Output head + greedy argmax in one launch; `logits` may be nil when only the token is needed.
    func encodeOutputHeadArgmax(stream: UnsafeMutableRawPointer?, weight: PackedWeight, hidden: UnsafeRawPointer,
                                precision: BufferPrecision, logits: UnsafeMutablePointer<Float>?,
                                token: UnsafeMutablePointer<Int32>) throws {
        try MI355QError.check(mi355q_lmhead_argmax(handle, stream, weight.handle, hidden, precision.c, logits, token, 0))
    }
}

/// An opened `model.staf` with its payload region resident in HBM: the analogue of `STAFWeightStore`
/// (one buffer, entries by name, file-level metadata).
public final class MI355STAFStore {
    let handle: OpaquePointer
    public let context: MI355Context
    /// Device address of the payload region; tensor `t` lives at `base + t.buffer_offset`.
    public let base: UnsafeMutableRawPointer

    public init(context: MI355Context, url: URL) throws {
        var h: OpaquePointer?
        try MI355QError.check(mi355q_staf_open(url.path, &h))
        var dev: UnsafeMutableRawPointer?
        var bytes: UInt64 = 0
        let status = mi355q_staf_upload(context.handle, h, &dev, &bytes)
        if status != 0 {
            mi355q_staf_close(h)
            try MI355QError.check(status)
        }
        handle = h!
        base = dev!
        self.context = context
    }

    deinit {
        _ = mi355q_buffer_free(context.handle, base)
        mi355q_staf_close(handle)
    }

    /// `entries[name]`
    public func entry(named name: String) -> mi355q_staf_entry? {
        var e = mi355q_staf_entry()
        return mi355q_staf_find(handle, name, &e) == 0 ? e : nil
    }

    /// `resolvedBufferAccess(for:)`: the row-major bytes in place, or this library's specialized copy.
    public func weight(named name: String, layout: WeightLayout = .rowMajorBlocks) throws -> PackedWeight {
        var w: OpaquePointer?
        try MI355QError.check(mi355q_staf_weight(context.handle, handle, base, name, layout.c, &w))
        return PackedWeight(context: context, owning: w!)
    }

    /// `STAFValidator.isValid`
    public static func isValid(stafURL: URL, safetensorsURLs: [URL]) throws -> Bool {
        var valid: Int32 = 0
        var paths = safetensorsURLs.map { strdup($0.path) }
        defer { paths.forEach { free($0) } }
        let status = paths.withUnsafeMutableBufferPointer { buf -> mi355q_status in
            buf.withMemoryRebound(to: UnsafePointer<CChar>?.self) { p in
                mi355q_staf_is_valid(stafURL.path, p.baseAddress, UInt32(p.count), nil, 0, &valid)
            }
        }
        try MI355QError.check(status)
        return valid != 0
    }
}

public extension MI355Context {
    /// Embedding gather (tokenIDs, table, output, embeddingDim, sequenceLength bindings of
    /// `embedding_lookup[_seq]_q{b}_g{g}`); the table may be the tied output head.
    func encodeEmbeddingLookup(stream: UnsafeMutableRawPointer?, table: PackedWeight, tokenIDs: UnsafePointer<Int32>,
                               sequenceLength: Int, output: UnsafeMutableRawPointer, precision: BufferPrecision,
                               embeddingScale: Float? = nil) throws {
        try MI355QError.check(mi355q_embedding_lookup(handle, stream, table.handle, tokenIDs, UInt32(sequenceLength),
                                                      output, precision.c, 0, embeddingScale == nil ? 0 : 1,
                                                      embeddingScale ?? 1))
    }
}
