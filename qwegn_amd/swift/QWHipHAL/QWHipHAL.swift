// QWHipHAL.swift - the Swift-on-Linux side of the drop-in: a HIP HAL that stands where QWHAL's Metal HAL stands
// for the quantized matmul operators, reached through the C module map over libqwhip (CQwhip).
//
// The operator enums keep the reference's names and labels (QWGemm.encodeH16, QWGemmAQ.encode, ...); only the
// encoder type changes: `any MTLComputeCommandEncoder` becomes `QWHipEncoder` (a stream), and `QWHal` wraps a
// `qwhip_device_t`.  Status codes map 1:1 onto the reference's typed errors, thrown before any launch.
//
// This file is not compiled in this repository's environment (no Swift toolchain is installed); the C++ mirror
// in ../../host/qwhost.hpp carries the same surface and is what the tests exercise.
import CQwhip

public enum QWHalError: Error { case deviceUnavailable(String), kernelMissing(String) }
public enum QWGemmError: Error { case f3Blocked(String), badWeights(String), badShape(String), badGeometry(String) }

@inline(__always) func qwCheck(_ st: qwhip_status) throws {
    guard st != QWHIP_OK else { return }
    let msg = String(cString: qwhip_last_error())
    switch st {
    case QWHIP_E_BAD_WEIGHTS, QWHIP_E_NULL, QWHIP_E_BASIS: throw QWGemmError.badWeights(msg)
    case QWHIP_E_BAD_SHAPE: throw QWGemmError.badShape(msg)
    case QWHIP_E_BAD_GEOMETRY: throw QWGemmError.badGeometry(msg)
    case QWHIP_E_BLOCKED: throw QWGemmError.f3Blocked(msg)
    case QWHIP_E_KERNEL_MISSING: throw QWHalError.kernelMissing(msg)
    default: throw QWHalError.deviceUnavailable(msg)
    }
}

public struct QWHipEncoder { public let stream: qwhip_stream_t }

public final class QWHal: @unchecked Sendable {
    let device: qwhip_device_t
    public private(set) var caps = qwhip_caps()
    public init(ordinal: Int32 = 0) throws {
        var d: qwhip_device_t?
        try qwCheck(qwhip_device_create(ordinal, &d))
        device = d!
        qwhip_device_caps(device, &caps)
    }
    deinit { qwhip_device_destroy(device) }
    /// hal.pipeline(name): the kernel-name table of the library; throws kernelMissing like the metallib lookup.
    public func pipeline(_ name: String) throws { try qwCheck(qwhip_kernel_lookup(name, nil)) }
    public func begin() throws -> QWHipEncoder {
        var s: qwhip_stream_t?
        try qwCheck(qwhip_stream_create(device, &s))
        return QWHipEncoder(stream: s!)
    }
    public func end(_ enc: QWHipEncoder) throws {
        try qwCheck(qwhip_stream_sync(enc.stream))
        qwhip_stream_destroy(enc.stream)
    }
}

/// A device region (QWTensorValue's storage on this HAL): base pointer + byte offset, non-owning.
public struct QWHipRegion { public let base: UnsafeMutableRawPointer; public let offset: Int; public let bytes: Int
    var ptr: UnsafeMutableRawPointer { base + offset } }

extension qwhip_weight_view {
    /// From the reference's QWWeightView fields (blocks, n, k, containerKind).
    init(blocks: QWHipRegion, n: Int, k: Int, kind: UInt32, bits: Int, group: Int) {
        self.init(blocks: UnsafeRawPointer(blocks.ptr), bytes: UInt64(blocks.bytes), n: UInt32(n), k: UInt32(k),
                  kind: kind, bits: UInt32(bits), group: UInt32(group))
    }
}

public enum QWGemm {
    /// QWGemm.encodeH16: decode GEMV with direct f16 store (and optional f32 dual store).
    public static func encodeH16(_ enc: QWHipEncoder, hal: QWHal, kernel: String, x: QWHipRegion, wQ4: qwhip_weight_view,
                                 y16: QWHipRegion, y32: QWHipRegion? = nil, rows: Int = 1, xIsRotated: Bool = true) throws {
        try hal.pipeline(kernel)
        var w = wQ4
        try qwCheck(qwhip_gemv(enc.stream, &w, x.ptr, UInt32(QWHIP_F16), UInt32(rows),
                               xIsRotated ? UInt32(QWHIP_X_PREROTATED) : 0, y16.ptr,
                               y32?.ptr.assumingMemoryBound(to: Float.self)))
    }
    /// gemmBatchedH16 (QWEngineDriver): prefill GEMM on the matrix cores.
    public static func gemmBatchedH16(_ enc: QWHipEncoder, hal: QWHal, x: QWHipRegion, w: qwhip_weight_view, y16: QWHipRegion,
                                      rows: Int, workspace: QWHipRegion? = nil) throws {
        try hal.pipeline("qwg_gemm_q4g_h16")
        var wv = w
        try qwCheck(qwhip_gemm(enc.stream, &wv, x.ptr, UInt32(QWHIP_F16), UInt32(rows), 0, y16.ptr, UInt32(QWHIP_F16), 0,
                               UInt32(QWHIP_X_PREROTATED), workspace?.ptr, UInt64(workspace?.bytes ?? 0)))
    }
    /// QWGemm.encodeFwht32
    public static func encodeFwht32(_ enc: QWHipEncoder, hal: QWHal, x: QWHipRegion, count: Int) throws {
        guard count > 0, count % 32 == 0 else { throw QWGemmError.badWeights("fwht32 f16: n must be > 0 and divisible by 32") }
        try hal.pipeline("qwg_fwht32_f16")
        try qwCheck(qwhip_fwht32(enc.stream, x.ptr, UInt32(QWHIP_F16), x.ptr, UInt64(count)))
    }
}
