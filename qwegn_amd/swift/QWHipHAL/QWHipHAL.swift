// QWHipHAL.swift - the Swift-on-Linux side of the drop-in: a HIP HAL that stands where QWHAL's Metal HAL stands
// for the quantized matmul operators, reached through the C module map over libqwhip (CQwhip).
//
// The operator enums keep the reference's names and labels (QWGemm.encodeH16, QWGemmAQ.encode, ...); only the
// encoder type changes: `any MTLComputeCommandEncoder` becomes `QWHipEncoder` (a stream), and `QWHal` wraps a
// `qwhip_device_t`.  Status codes map 1:1 onto the reference's typed errors, thrown before any launch.
//
// This file is not compiled in this repository's environment (no Swift toolchain is installed); the C++ mirror
// in ../../host/qwhost.hpp carries the same surface, door for door, and is what the tests exercise.  Every door
// checks what the reference's door checks and throws the same error case before anything is enqueued.
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
    /// The geometry's gated FFN activation: what QWHal+Constants.swift:60-75 bakes into every pipeline as function constants
    /// 224 (swigluLimit) and 228 / 229 (activationKind .situ(beta:linearBeta:)) is one device-wide setting here.
    public convenience init(geometry: QWModelGeometry, ordinal: Int32 = 0) throws {
        try self.init(ordinal: ordinal)
        if case let .situ(beta, linearBeta) = geometry.descriptor.activationKind {
            try qwCheck(qwhip_device_set_gated_activation(device, UInt32(QWHIP_ACT_BOUNDED), beta, linearBeta))
        } else if let limit = geometry.swigluLimit, limit > 0 {
            try qwCheck(qwhip_device_set_gated_activation(device, UInt32(QWHIP_ACT_SWIGLU_CLAMPED), Float(limit), 0))
        }
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

/// The element types of QWDType that this path uses (Sources/Foundation/QWCore/QWDType.swift).
/// `.q4g` is the weight tag QWGemm.plan takes (HQ4_G32_M5, 20 B per 32 parameters); it is never the type of a tensor value.
public enum QWDType: UInt32 { case f32 = 0, f16 = 1, bf16 = 2, i32 = 3, q4g = 0x100
    var bytes: Int { self == .f32 || self == .i32 ? 4 : 2 } }

/// QWTensorValue on this HAL (Sources/Foundation/QWAlloc/QWArena.swift:49-151): a non-owning device region with an element
/// type and count; the arena that owns it guarantees its lifetime until the stream has drained.
public struct QWTensorValue {
    public let region: QWHipRegion
    public let dtype: QWDType
    public let elementCount: Int
    public init(region: QWHipRegion, dtype: QWDType, elementCount: Int) {
        precondition(elementCount * dtype.bytes <= region.bytes, "tensor value exceeds its region")
        self.region = region; self.dtype = dtype; self.elementCount = elementCount
    }
    /// Zero-copy sub-view (QWArena.swift:62-66): `count` elements of `dtype` (default: this value's) from `byteOffset`.
    public func slice(byteOffset: Int, count: Int, dtype: QWDType? = nil) -> QWTensorValue {
        QWTensorValue(region: QWHipRegion(base: region.base, offset: region.offset + byteOffset, bytes: region.bytes - byteOffset),
                      dtype: dtype ?? self.dtype, elementCount: count)
    }
    var ptr: UnsafeMutableRawPointer { region.ptr }
    var f32: UnsafeMutablePointer<Float> { region.ptr.assumingMemoryBound(to: Float.self) }
    var i32: UnsafeMutablePointer<Int32> { region.ptr.assumingMemoryBound(to: Int32.self) }
}

/// QWWeightView (Sources/Foundation/QWAlloc/QWWeightView.swift:9-152): a validated view of one bank; the initialiser fails
/// (nil) exactly where the reference's does: k % group != 0, n <= 0, an unsupported (bits, group) pair, a short region.
public struct QWWeightView {
    public enum ContainerKind { case incumbentHQ4G32, rotatedHQ(bits: Int, group: Int), nativeAffine(bits: Int, group: Int) }
    public let abi: qwhip_weight_view
    public let kind: ContainerKind
    public var n: Int { Int(abi.n) }
    public var k: Int { Int(abi.k) }
    public var bits: Int { Int(abi.bits) }
    public var groupSize: Int { Int(abi.group) }
    public var isRotated: Bool { if case .nativeAffine = kind { return false } else { return true } }
    public var isIncumbent: Bool { if case .incumbentHQ4G32 = kind { return true } else { return false } }
    public init?(blocks: QWHipRegion, n: Int, k: Int, kind: ContainerKind) {
        let (tag, bits, group): (UInt32, Int, Int)
        switch kind {
        case .incumbentHQ4G32: (tag, bits, group) = (UInt32(QWHIP_KIND_HQ4_G32_M5), 4, 32)
        case .rotatedHQ(let b, let g): (tag, bits, group) = (UInt32(QWHIP_KIND_ROTATED_HQ), b, g)
        case .nativeAffine(let b, let g): (tag, bits, group) = (UInt32(QWHIP_KIND_NATIVE_AFFINE), b, g)
        }
        guard n > 0, k > 0 else { return nil }
        var v = qwhip_weight_view(blocks: blocks, n: n, k: k, kind: tag, bits: bits, group: group)
        guard qwhip_weight_view_validate(&v) == QWHIP_OK else { return nil }
        self.abi = v; self.kind = kind
    }
}

public enum QWEpilogue { case none, siluMulPair }
public enum QWGemmFamily { case f1DecodeGemv, f2LmHeadGemv, f3PrefillGemm, f4AttentionTiles, f5SkinnyGemm }

public struct QWGemmShape: Hashable {
    public let m: Int, n: Int, k: Int
    public init(m: Int, n: Int, k: Int) { self.m = m; self.n = n; self.k = k }
    public func family(vocab: Int? = nil) -> QWGemmFamily {                    // QWGemm.swift:27-33
        if m == 1, let vocab, n == vocab { return .f2LmHeadGemv }
        if m == 1 { return .f1DecodeGemv }
        if m >= 512 { return .f3PrefillGemm }
        if m <= 8 { return .f5SkinnyGemm }
        return .f4AttentionTiles
    }
}

public struct QWGemmPlan {
    /// The reference's backends plus `mfmaGemmF16`, this library's prefill door (planHip only).
    public enum Backend { case handQ4gV4, handQ4gV4H16, handQ4gSiluPair, handQ4gSiluPairH16, handQ4gSkinny, handF16V4, mpsF16,
                          mpsGraphBmmF16, blocked, mfmaGemmF16 }
    public let backend: Backend
    public let kernel: String
    public let threadsPerTG: Int
    public let family: QWGemmFamily
    public let epilogue: QWEpilogue
}

public enum QWGemm {
    /// The reference's dispatch table, row for row (QWGemm.swift:92-133).  `dtype`: .q4g weights are spelled `nil` here
    /// because QWDType on this HAL lists activation types only.
    public static func plan(_ shape: QWGemmShape, quantized: Bool, f16Weights: Bool = false, epi: QWEpilogue,
                            outDtype: QWDType = .f32, vocab: Int? = nil) -> QWGemmPlan {
        let fam = shape.family(vocab: vocab)
        let blocked = QWGemmPlan(backend: .blocked, kernel: "", threadsPerTG: 0, family: fam, epilogue: epi)
        let decode = fam == .f1DecodeGemv || fam == .f2LmHeadGemv
        if quantized && epi == .siluMulPair {
            return outDtype == .f16
                ? QWGemmPlan(backend: .handQ4gSiluPairH16, kernel: "qwg_gemv_q4g_silu_pair_h16", threadsPerTG: 64, family: fam, epilogue: epi)
                : QWGemmPlan(backend: .handQ4gSiluPair, kernel: "qwg_gemv_q4g_silu_pair", threadsPerTG: 64, family: fam, epilogue: epi)
        }
        guard epi == .none else { return blocked }
        if quantized && decode {
            return outDtype == .f16
                ? QWGemmPlan(backend: .handQ4gV4H16, kernel: "qwg_gemv_q4g_v4_h16", threadsPerTG: 32, family: fam, epilogue: epi)
                : QWGemmPlan(backend: .handQ4gV4, kernel: "qwg_gemv_q4g_v4", threadsPerTG: 32, family: fam, epilogue: epi)
        }
        if quantized && fam == .f5SkinnyGemm {
            if (shape.m == 2 || shape.m == 3) && shape.m * shape.k * 2 <= 256 * 1024 {
                return QWGemmPlan(backend: .handQ4gSkinny, kernel: shape.m == 2 ? "qwg_skinny_m2" : "qwg_skinny_m3",
                                  threadsPerTG: 32, family: fam, epilogue: epi)
            }
            return blocked
        }
        if f16Weights && decode {
            return QWGemmPlan(backend: .handF16V4, kernel: "qwg_gemv_f16_v4", threadsPerTG: 32, family: fam, epilogue: epi)
        }
        if quantized && fam == .f3PrefillGemm && shape.k % 32 == 0 {
            return QWGemmPlan(backend: .mpsGraphBmmF16, kernel: "mpsgraph_bmm_f16", threadsPerTG: 0, family: fam, epilogue: epi)
        }
        return blocked
    }

    /// QWGemm.plan with the reference's own labels (QWGemm.swift:92-133): dtype .q4g = quantized weights, .f16 = f16 weights.
    public static func plan(_ shape: QWGemmShape, dtype: QWDType, epi: QWEpilogue, outDtype: QWDType = .f32, vocab: Int? = nil) -> QWGemmPlan {
        plan(shape, quantized: dtype == .q4g, f16Weights: dtype == .f16, epi: epi, outDtype: outDtype, vocab: vocab)
    }

    /// This library's routing: every row count 2...16 streams the bank once (qwhip_gemv), prefill and the remaining F4
    /// shapes run the matrix-core GEMM when K % 64 == 0.
    public static func planHip(_ shape: QWGemmShape, epi: QWEpilogue, outDtype: QWDType = .f32, vocab: Int? = nil) -> QWGemmPlan {
        let base = plan(shape, quantized: true, epi: epi, outDtype: outDtype, vocab: vocab)
        if base.backend != .blocked && base.backend != .mpsGraphBmmF16 { return base }
        let fam = base.family
        if epi == .none && shape.m >= 2 && shape.m <= 16 {
            return QWGemmPlan(backend: .handQ4gSkinny, kernel: shape.m == 3 ? "qwg_skinny_m3" : "qwg_skinny_m2", threadsPerTG: 256, family: fam, epilogue: epi)
        }
        if epi == .none && shape.m > 16 && shape.k % 64 == 0 {
            return QWGemmPlan(backend: .mfmaGemmF16, kernel: "qwg_gemm_q4g_h16", threadsPerTG: 256, family: fam, epilogue: epi)
        }
        return QWGemmPlan(backend: .blocked, kernel: "", threadsPerTG: 0, family: fam, epilogue: epi)
    }

    /// QWGemm.encode (QWGemm.swift:218-283): f32 output; .siluMulPair needs even N and stores f16 activations [rows, N / 2].
    /// xGroupSum is taken and not read (the kernels form the group sums of x themselves); rows defaults to what the plan's kernel
    /// implies (qwg_skinny_m2 / m3 -> 2 / 3, else 1), as the reference derives it.
    public static func encode(_ enc: QWHipEncoder, hal: QWHal, plan: QWGemmPlan, x: QWTensorValue, xGroupSum: QWTensorValue? = nil,
                              wQ4: QWWeightView, y: QWTensorValue, rows rowsArg: Int? = nil, xIsRotated: Bool = true,
                              siluPairPlainOut: Bool = false) throws {
        // siluPairPlainOut: .siluMulPair stores act in the plain basis; the next projection then rotates its input itself
        // (xIsRotated: false there), free at one row, and the gate|up bank is read by the decode GEMV's own kernel.
        let rows = rowsArg ?? (plan.backend == .handQ4gSkinny ? (plan.kernel == "qwg_skinny_m3" ? 3 : 2) : 1)
        switch plan.backend {
        case .blocked:
            if plan.family == .f5SkinnyGemm { throw QWGemmError.badWeights("F5 window: run F1 per row") }
            throw QWGemmError.f3Blocked("no winner raced for this family")
        case .mfmaGemmF16, .mpsGraphBmmF16: throw QWGemmError.f3Blocked("plan resolved to the tensor GEMM - use gemmBatchedH16")
        case .handF16V4, .mpsF16: throw QWGemmError.badWeights("the f16-weight doors have no kernel in this library")
        default: break
        }
        guard x.dtype == .f16 || x.dtype == .bf16, x.elementCount >= rows * wQ4.k else { throw QWGemmError.badWeights("activations must be f16 [rows, k]") }
        try hal.pipeline(plan.kernel)
        var w = wQ4.abi
        let flags: UInt32 = xIsRotated ? UInt32(QWHIP_X_PREROTATED) : 0
        if plan.epilogue == .siluMulPair {
            guard wQ4.n % 2 == 0 else { throw QWGemmError.badWeights("silu_pair needs even N") }
            guard y.dtype == .f16, y.elementCount >= rows * (wQ4.n / 2) else { throw QWGemmError.badWeights("silu_pair output must be f16 [rows, N/2]") }
            try qwCheck(qwhip_gemv_silu_pair(enc.stream, &w, x.ptr, x.dtype.rawValue, UInt32(rows), flags, siluPairPlainOut ? 0 : 1, y.ptr))
            return
        }
        guard y.dtype == .f32, y.elementCount >= rows * wQ4.n else { throw QWGemmError.badWeights("output must be f32 [rows, N]") }
        try qwCheck(qwhip_gemv(enc.stream, &w, x.ptr, x.dtype.rawValue, UInt32(rows), flags, nil, y.f32))
    }

    /// QWGemm.encodeH16 (QWGemm.swift:137-214): decode GEMV with direct f16 store (and optional f32 dual store).
    public static func encodeH16(_ enc: QWHipEncoder, hal: QWHal, plan: QWGemmPlan, x: QWTensorValue, xGroupSum: QWTensorValue? = nil,
                                 wQ4: QWWeightView, y16: QWTensorValue, y32: QWTensorValue? = nil, rows: Int = 1, xIsRotated: Bool = true) throws {
        guard plan.backend == .handQ4gV4H16 || plan.backend == .handQ4gSiluPairH16 || plan.backend == .handQ4gSkinny else {
            throw QWGemmError.badWeights("encodeH16 requires handQ4gV4H16 or handQ4gSiluPairH16")
        }
        guard y16.dtype == .f16 else { throw QWGemmError.badWeights("y16 must have dtype .f16") }
        if plan.epilogue == .siluMulPair { try encode(enc, hal: hal, plan: plan, x: x, wQ4: wQ4, y: y16, rows: rows, xIsRotated: xIsRotated); return }
        guard x.dtype == .f16 || x.dtype == .bf16, x.elementCount >= rows * wQ4.k else { throw QWGemmError.badWeights("activations must be f16 [rows, k]") }
        guard y16.elementCount >= rows * wQ4.n else { throw QWGemmError.badWeights("y16 is short") }
        if let y32, y32.dtype != .f32 || y32.elementCount < rows * wQ4.n { throw QWGemmError.badWeights("y32 must be f32 [rows, N]") }
        try hal.pipeline(plan.kernel)
        var w = wQ4.abi
        try qwCheck(qwhip_gemv(enc.stream, &w, x.ptr, x.dtype.rawValue, UInt32(rows), xIsRotated ? UInt32(QWHIP_X_PREROTATED) : 0, y16.ptr, y32?.f32))
    }

    /// gemmBatchedH16 (Sources/Runtime/QWEngine/Driver/EncodeKernels.swift:119-154): prefill GEMM on the matrix cores;
    /// bf16 rows already in the basis need no workspace (converted while the tile is staged).
    public static func gemmBatchedH16(_ enc: QWHipEncoder, hal: QWHal, x: QWTensorValue, w: QWWeightView, y: QWTensorValue,
                                      rows: Int, xIsRotated: Bool = true, workspace: QWHipRegion? = nil) throws {
        guard w.k % 64 == 0, w.n % 16 == 0 else { throw QWGemmError.badGeometry("tensor GEMM needs K % 64 == 0 and N % 16 == 0") }
        guard x.elementCount >= rows * w.k, y.elementCount >= rows * w.n else { throw QWGemmError.badShape("gemm operands are short") }
        try hal.pipeline("qwg_gemm_q4g_h16")
        var wv = w.abi
        try qwCheck(qwhip_gemm(enc.stream, &wv, x.ptr, x.dtype.rawValue, UInt32(rows), 0, y.ptr, y.dtype.rawValue, 0,
                               xIsRotated ? UInt32(QWHIP_X_PREROTATED) : 0, workspace?.ptr, UInt64(workspace?.bytes ?? 0)))
    }

    /// gemmBatchedH16SwiGLU (EncodeKernels.swift:156-188): dense gate|up GEMM with SwiGLU (+ FWHT-32) fused, act f16 [rows, N / 2].
    public static func gemmBatchedH16SwiGLU(_ enc: QWHipEncoder, hal: QWHal, x: QWTensorValue, w: QWWeightView, act16: QWTensorValue,
                                            rows: Int, rotateAct: Bool = true, workspace: QWHipRegion? = nil) throws {
        guard w.n % 64 == 0, act16.dtype == .f16, act16.elementCount >= rows * (w.n / 2) else { throw QWGemmError.badShape("fused gate_up: act f16 [rows, N/2], N % 64 == 0") }
        try hal.pipeline("qwg_gemm_q4g_h16_swiglu")
        var wv = w.abi
        try qwCheck(qwhip_gemm_swiglu(enc.stream, &wv, x.ptr, x.dtype.rawValue, UInt32(rows), 0, rotateAct ? 1 : 0, act16.ptr, 0,
                                      UInt32(QWHIP_X_PREROTATED), workspace?.ptr, workspace?.bytes ?? 0))
    }

    /// QWGemm.encodeFwht32 (QWGemm.swift:288-300)
    public static func encodeFwht32(_ enc: QWHipEncoder, hal: QWHal, x: QWTensorValue, count countArg: Int? = nil) throws {
        let count = countArg ?? x.elementCount
        guard x.dtype == .f16, count > 0, count % 32 == 0 else { throw QWGemmError.badWeights("fwht32 f16: n must be > 0 and divisible by 32") }
        try hal.pipeline("qwg_fwht32_f16")
        try qwCheck(qwhip_fwht32(enc.stream, x.ptr, UInt32(QWHIP_F16), x.ptr, UInt64(count)))
    }
    /// QWGemm.encodeCast (QWGemm.swift:305-320)
    public static func encodeCast(_ enc: QWHipEncoder, hal: QWHal, x32: QWTensorValue, y16: QWTensorValue, count countArg: Int? = nil) throws {
        let count = countArg ?? x32.elementCount
        guard x32.dtype == .f32, y16.dtype == .f16, count > 0, x32.elementCount >= count, y16.elementCount >= count else { throw QWGemmError.badWeights("cast: f32 -> f16 operands") }
        try hal.pipeline("qwg_cast_f32_to_f16")
        try qwCheck(qwhip_cast_f32_to_f16(enc.stream, x32.f32, y16.ptr, UInt64(count)))
    }
    /// QWGemm.encodeH32F32 (QWGemmF32.swift:46-54)
    public static func encodeH32F32(_ enc: QWHipEncoder, hal: QWHal, x: QWTensorValue, out: QWTensorValue, rows: Int, hidden: Int) throws {
        guard hidden % 32 == 0, x.elementCount >= rows * hidden, out.elementCount >= rows * hidden else { throw QWGemmError.badShape("h32: hidden % 32 == 0") }
        try hal.pipeline("qwg_h32_f32")
        try qwCheck(qwhip_h32_f32(enc.stream, x.f32, out.f32, UInt32(rows), UInt32(hidden)))
    }
    /// QWGemm.encodeHQ4F32V4 / encodeHQ4F32BM (QWGemmF32.swift:178-199, 311-350): fp32 activations, scalar epilogue 0...3.
    public static func encodeHQ4F32V4(_ enc: QWHipEncoder, hal: QWHal, weight: QWWeightView, x: QWTensorValue, y: QWTensorValue,
                                      rows: Int = 1, epi: UInt32 = 0, scale: Float = 1) throws {
        guard x.dtype == .f32, y.dtype == .f32, x.elementCount >= rows * weight.k, y.elementCount >= rows * weight.n else { throw QWGemmError.badWeights("f32 GEMV operands") }
        try hal.pipeline("qwg_gemv_q4g_f32_v4")
        var w = weight.abi
        try qwCheck(qwhip_gemv_f32(enc.stream, &w, x.f32, UInt32(rows), epi, scale, y.f32))
    }
    /// QWGemm.encodeSiluMulF32 / encodeSiluMulSplitF16 / encodeAddF32 (QWGemmF32.swift:83-115)
    /// act16 (optional): the same activations also stored as f16.
    public static func encodeSiluMulF32(_ enc: QWHipEncoder, hal: QWHal, gu: QWTensorValue, act: QWTensorValue, rows: Int, intermediate: Int,
                                        act16: QWTensorValue? = nil) throws {
        guard intermediate % 32 == 0 else { throw QWGemmError.badShape("silu_mul f32: intermediate % 32 == 0") }
        try hal.pipeline("qwg_silu_mul_f32")
        try qwCheck(qwhip_silu_mul_f32(enc.stream, gu.f32, act.f32, UInt32(rows), UInt32(intermediate)))
        if let a16 = act16 { try encodeSiluMulF16(enc, hal: hal, gu: gu, act16: a16, rows: rows, intermediate: intermediate) }
    }
    /// One f16 output instead of the reference's outHi / outLo pair (encodeSiluMulSplitF16): the f32 doors of this library split
    /// their activations inside the GEMM kernel, so no caller needs the halves.
    public static func encodeSiluMulF16(_ enc: QWHipEncoder, hal: QWHal, gu: QWTensorValue, act16: QWTensorValue, rows: Int, intermediate: Int,
                                        rotate: Bool = true) throws {
        try hal.pipeline("qwg_silu_mul_split_f16")
        try qwCheck(qwhip_swiglu_fwht(enc.stream, gu.ptr, gu.dtype.rawValue, act16.ptr, UInt32(rows), UInt32(intermediate), rotate ? 1 : 0))
    }
    public static func encodeAddF32(_ enc: QWHipEncoder, hal: QWHal, a: QWTensorValue, b: QWTensorValue, out: QWTensorValue, count: Int) throws {
        try hal.pipeline("qwg_add_f32")
        try qwCheck(qwhip_add_f32(enc.stream, a.f32, b.f32, out.f32, UInt64(count)))
    }
    /// QWGemm.encodeF32Gemv (QWGemmF32.swift:117-141): dense fp32 weights, epilogue 0 none, 1 silu(y / scale), 2 sigmoid, 3 2 sigmoid(y / scale).
    public static func encodeF32Gemv(_ enc: QWHipEncoder, hal: QWHal, weight: QWTensorValue, x: QWTensorValue, y: QWTensorValue, rows: Int, n: Int,
                                     k: Int, epilogue: UInt32, scale: Float) throws {
        try hal.pipeline(rows >= 4 ? "qwg_f32_gemv_bm" : "qwg_f32_gemv")
        try qwCheck(qwhip_f32_gemv(enc.stream, weight.f32, x.f32, UInt32(rows), UInt32(n), UInt32(k), epilogue, scale, y.f32))
    }
    /// QWGemm.encodeArgmaxFin (QWGemmF32.swift:276-307) over f32 logits: the fold, or the relaxed acceptance of a draft.
    public struct QWVariationalAcceptance { public let draftTokens: QWTensorValue; public let totalRows: Int; public let margin: Float; public let minLogProb: Float }
    public static func encodeArgmaxFin(_ enc: QWHipEncoder, hal: QWHal, logits: QWTensorValue, token: QWTensorValue, vocab: Int, rows: Int = 1,
                                       variational: QWVariationalAcceptance? = nil) throws {
        if let v = variational, v.margin > 0, rows > 1 {
            try hal.pipeline("qwg_head_argmax_fin_variational")
            try qwCheck(qwhip_argmax_f32_variational(enc.stream, logits.f32, UInt32(rows), UInt32(vocab),
                                                     v.draftTokens.ptr.assumingMemoryBound(to: UInt32.self), UInt32(v.totalRows), v.margin, v.minLogProb,
                                                     token.i32))
        } else {
            try hal.pipeline("qwg_head_argmax_fin")
            try qwCheck(qwhip_argmax_f32(enc.stream, logits.f32, UInt32(rows), UInt32(vocab), token.i32))
        }
    }
    /// QWGemm.encodeLatentNormH32F32 (QWGemmF32.swift:57-80): optional RMSNorm (1 + gamma) + H_32 on f32 rows -> f32 and / or f16.
    public static func encodeLatentNormH32F32(_ enc: QWHipEncoder, hal: QWHal, x: QWTensorValue, gamma: QWTensorValue?, out32: QWTensorValue?,
                                              out16: QWTensorValue? = nil, rows: Int, latent: Int, eps: Float = 1e-6, skipOut32: Bool = false) throws {
        let o32 = skipOut32 ? nil : out32
        guard latent > 0, latent % 32 == 0, o32 != nil || out16 != nil else { throw QWGemmError.badShape("latent norm H32: latent % 32 == 0, one output") }
        try hal.pipeline("qwg_latent_norm_h32_f32")
        try qwCheck(qwhip_latent_norm_h32_f32(enc.stream, x.f32, gamma?.ptr, o32?.f32, out16?.ptr, UInt32(rows), UInt32(latent), eps))
    }
    /// QWGemm.encodeMoEBridgeF16ToF32 (QWGemmMoE.swift:337-377): f16 normed hidden -> rotated f32 copy + un-rotated f32 copy.
    public static func encodeMoEBridgeF16ToF32(_ enc: QWHipEncoder, hal: QWHal, x: QWTensorValue, xRot32: QWTensorValue?, xPlain32: QWTensorValue,
                                               rows: Int, hidden: Int, skipRot32: Bool = false) throws {
        guard hidden % 256 == 0 else { throw QWGemmError.badGeometry("moe bridge: hidden must be a multiple of 256") }
        try hal.pipeline("qwg_moe_bridge_f16_to_f32")
        try qwCheck(qwhip_moe_bridge_f16_to_f32(enc.stream, x.ptr, skipRot32 ? nil : xRot32?.f32, xPlain32.f32, UInt32(rows), UInt32(hidden)))
    }
    /// QWGemm.encodeDenseProjF32 (QWGemmF32.swift:413-440): f32 rows in the container's basis -> f32 outputs; 64 rows and more without
    /// an epilogue go through one cast and the f16 GEMM, fewer through the f32 door (its batched matrix-core form from 32 rows on).
    /// naxY16 and maxTileWidth are taken and not used: the GEMM needs no second f16 plane and has no tile-width limit.
    public static func encodeDenseProjF32(_ enc: QWHipEncoder, hal: QWHal, weight: QWWeightView, x: QWTensorValue, y: QWTensorValue,
                                          naxX16: QWTensorValue, naxY16: QWTensorValue, maxTileWidth: Int, rows: Int, epi: UInt32 = 0,
                                          scale: Float = 1, x16Precast: QWTensorValue? = nil, minNaxRows: Int = 64) throws {
        let count = rows * weight.k
        if rows >= max(64, minNaxRows), epi == 0, scale == 1, weight.n % 64 == 0, weight.k % 64 == 0,
           (x16Precast?.elementCount ?? naxX16.elementCount) >= count {
            let x16 = (x16Precast ?? naxX16).slice(byteOffset: 0, count: count, dtype: .f16)
            if x16Precast == nil { try encodeCast(enc, hal: hal, x32: x, y16: x16, count: count) }
            try gemmBatchedH16(enc, hal: hal, x: x16, w: weight, y: y, rows: rows)
        } else {
            try encodeHQ4F32V4(enc, hal: hal, weight: weight, x: x, y: y, rows: rows, epi: epi, scale: scale)
        }
    }

    // ---- MoE doors (QWGemmMoE.swift, QWGemmMoERouter.swift) -------------------------------------------------------
    public static func moeMaxTiles(experts: Int, pairs: Int) -> Int { Int(qwhip_moe_max_tiles(UInt32(experts), UInt32(pairs))) }   // QWGemmMoE.swift:24-26

    /// encodeFnRouterGemm (QWGemmMoERouter.swift:78-113): logits f32 [rows, n] = x . Wr^T, optional shared-expert gate column.
    public static func encodeFnRouterGemm(_ enc: QWHipEncoder, hal: QWHal, weight: QWTensorValue, x: QWTensorValue, y: QWTensorValue,
                                          rows: Int, n: Int, k: Int, shGateWeight: QWTensorValue? = nil, shGateOut: QWTensorValue? = nil) throws {
        precondition(k % 32 == 0, "router GEMM needs K % 32 == 0")
        try hal.pipeline("qwg_router_gemm")
        if let gw = shGateWeight, let go = shGateOut {
            try qwCheck(qwhip_router_gemm_shared_gate(enc.stream, x.ptr, x.dtype.rawValue, weight.ptr, weight.dtype.rawValue, UInt32(rows), UInt32(n),
                                                      UInt32(k), y.f32, gw.f32, go.f32))
        } else {
            try qwCheck(qwhip_router_gemm(enc.stream, x.ptr, x.dtype.rawValue, weight.ptr, weight.dtype.rawValue, UInt32(rows), UInt32(n), UInt32(k), y.f32))
        }
    }
    /// encodeFnMoeRoute (QWGemmMoERouter.swift:10-75): softmax top-k (or the sigmoid / bias / split-feature modes).
    /// guSh / actSh / sharedIntermediate: the shared expert's silu_mul, which the reference folds into this launch, runs after it.
    /// latentLabels / groupIds / numGroups: the groups of each token's routes; the route ids stay plain (the reference packs the
    /// group into their high bits).  routedScale (an addition): constant factor on the weights.
    public static func encodeFnMoeRoute(_ enc: QWHipEncoder, hal: QWHal, logits: QWTensorValue, idx: QWTensorValue, wts: QWTensorValue,
                                        rows: Int, experts: Int, topK: Int, normTopK: Bool, guSh: QWTensorValue? = nil, actSh: QWTensorValue? = nil,
                                        sharedIntermediate: Int = 0, bias: QWTensorValue? = nil, expertBudget: Int = 0,
                                        splitFeature: Bool = false, routedScaleParam: QWTensorValue? = nil, latentLabels: QWTensorValue? = nil,
                                        groupIds: QWTensorValue? = nil, numGroups: Int = 0, routedScale: Float = 1) throws {
        precondition(experts <= 512 && topK <= 16, "route: experts <= 512, K <= 16")
        if let gu = guSh, let act = actSh, sharedIntermediate > 0 {
            try encodeSiluMulF32(enc, hal: hal, gu: gu, act: act, rows: rows, intermediate: sharedIntermediate)
        }

        try hal.pipeline("qwg_moe_route")
        try qwCheck(qwhip_moe_route_ex(enc.stream, logits.f32, UInt32(rows), UInt32(experts), UInt32(topK), normTopK ? 1 : 0, routedScale,
                                       splitFeature ? 1 : 0, bias?.f32, routedScaleParam?.f32, idx.i32, wts.f32))
        if expertBudget > 0 && rows > 1 && rows <= 4 && expertBudget < rows * topK && rows * topK <= 64 {      // QWGemmMoERouter.swift:63-75
            try hal.pipeline("qwg_moe_route_decode")
            try qwCheck(qwhip_moe_route_budget(enc.stream, idx.i32, wts.f32, UInt32(rows), UInt32(topK), UInt32(expertBudget), normTopK ? 1 : 0))
        }
        if let labels = latentLabels, let gids = groupIds, numGroups > 0 {
            try encodeMoELatentGroups(enc, hal: hal, idx: idx, labels: labels, rows: rows, topK: topK, experts: experts, numGroups: numGroups,
                                      groupIds: gids, pairRows: nil)
        }
    }
    /// encodeMoEGroupPairsF32 (QWGemmMoE.swift:68-99): counting sort of the (token, route) pairs by expert + tile list.
    public static func encodeMoEGroupPairsF32(_ enc: QWHipEncoder, hal: QWHal, ids: QWTensorValue, expertOff: QWTensorValue,
                                              sortedPairIdx: QWTensorValue, sortedTok: QWTensorValue, experts: Int, totalPairs: Int, routes: Int,
                                              invPerm: QWTensorValue? = nil, tileE: QWTensorValue? = nil, tileR: QWTensorValue? = nil,
                                              tileCount: QWTensorValue? = nil, compactTail: Bool = true) throws {
        precondition(experts <= 512 && experts % 32 == 0, "group pairs: experts <= 512, multiple of 32")
        try hal.pipeline("qwg_moe_group_pairs_f32")
        try qwCheck(qwhip_moe_group_pairs(enc.stream, ids.i32, UInt32(experts), UInt32(totalPairs), UInt32(routes), expertOff.i32, sortedPairIdx.i32,
                                          sortedTok.i32, invPerm?.i32, tileE?.i32, tileR?.i32, tileCount?.i32, compactTail ? 1 : 0))
    }
    /// encodeMoEGateUpNax / encodeMoENaxSplitF32 (QWGemmMoE.swift:201-296): grouped expert GEMM over the sorted pairs.
    public static func encodeMoEGroupedGemm(_ enc: QWHipEncoder, hal: QWHal, xe: QWTensorValue, bank: QWWeightView, experts: Int,
                                            expertOff: QWTensorValue, tileE: QWTensorValue, tileR: QWTensorValue, tileCount: QWTensorValue,
                                            y: QWTensorValue, pairs: Int, sortedTok: QWTensorValue? = nil) throws {
        let rowsPerExpert = bank.n / experts
        precondition(rowsPerExpert % 64 == 0 && bank.k % 64 == 0, "NAX gate/up needs N and K multiples of 64")
        try hal.pipeline("qwg_moe_nax_gemm")
        var w = bank.abi
        try qwCheck(qwhip_moe_grouped_gemm(enc.stream, &w, UInt32(experts), xe.ptr, xe.dtype.rawValue, 0, sortedTok?.i32, expertOff.i32, tileE.i32,
                                           tileR.i32, tileCount.i32, UInt32(moeMaxTiles(experts: experts, pairs: pairs)), UInt32(pairs), y.ptr,
                                           y.dtype.rawValue, 0))
    }
    /// The gate_up grouped GEMM with SwiGLU (+ FWHT-32) fused (no reference door of its own: encodeMoEGateUpNax followed by encodeSiluMul*).
    public static func encodeMoEGateUpSwiglu(_ enc: QWHipEncoder, hal: QWHal, xe: QWTensorValue, bank: QWWeightView, experts: Int,
                                             sortedTok: QWTensorValue, expertOff: QWTensorValue, tileE: QWTensorValue, tileR: QWTensorValue,
                                             tileCount: QWTensorValue, act16: QWTensorValue, pairs: Int, rotateAct: Bool) throws {
        try hal.pipeline("qwg_moe_nax_gemm")
        var w = bank.abi
        try qwCheck(qwhip_moe_grouped_gemm_swiglu(enc.stream, &w, UInt32(experts), xe.ptr, xe.dtype.rawValue, 0, sortedTok.i32, expertOff.i32, tileE.i32,
                                                  tileR.i32, tileCount.i32, UInt32(moeMaxTiles(experts: experts, pairs: pairs)), UInt32(pairs),
                                                  rotateAct ? 1 : 0, act16.ptr, 0))
    }
    /// encodeMoEDownReduceCombineF32 (QWGemmMoE.swift:299-332)
    /// out (f32 or f16) and out16 are both stored unless skipOut32; unweightedSingle: unit weights; skipShared drops the shared term.
    /// The group sum (ids + numGroups) and scatterPerRoute have doors of their own here: encodeMoECombineGroupsF32, and the
    /// grouped GEMM's gather rows (encodeMoEComposeRows).
    public static func encodeMoEDownReduceCombineF32(_ enc: QWHipEncoder, hal: QWHal, dnAcc: QWTensorValue, invPerm: QWTensorValue?,
                                                     weights: QWTensorValue, shared: QWTensorValue?, gate: QWTensorValue?, out: QWTensorValue,
                                                     hidden: Int, routes: Int, tokens: Int, out16: QWTensorValue? = nil, skipShared: Bool = false,
                                                     unweightedSingle: Bool = false, ids: QWTensorValue? = nil, numGroups: Int = 0,
                                                     scatterPerRoute: Bool = false, skipOut32: Bool = false) throws {
        guard numGroups == 0, !scatterPerRoute else { throw QWGemmError.badShape("combine: group sums and per-route scatter are encodeMoECombineGroupsF32 / encodeMoEComposeRows") }
        guard !skipOut32 || out16 != nil else { throw QWGemmError.badShape("combine: skipOut32 needs out16") }
        try hal.pipeline("qwg_moe_down_reduce_combine_f32")
        for dst in [skipOut32 ? nil : out, out16].compactMap({ $0 }) {
            try qwCheck(qwhip_moe_combine(enc.stream, dnAcc.ptr, dnAcc.dtype.rawValue, invPerm?.i32, unweightedSingle ? nil : weights.f32, UInt32(tokens),
                                          UInt32(routes), UInt32(hidden), skipShared ? nil : shared?.f32, skipShared ? nil : gate?.f32, dst.ptr,
                                          dst.dtype.rawValue))
        }
    }
    /// The same door with invPerm: nil and unweightedSingle (QWGemmMoE.swift:299-332): out = dnAcc + gate * shared, one row per token.
    public static func encodeMoEAddSharedF32(_ enc: QWHipEncoder, hal: QWHal, dnAcc: QWTensorValue, shared: QWTensorValue, gate: QWTensorValue?,
                                             out: QWTensorValue, hidden: Int, tokens: Int) throws {
        try hal.pipeline("qwg_moe_down_reduce_combine_f32")
        try qwCheck(qwhip_moe_combine(enc.stream, dnAcc.ptr, dnAcc.dtype.rawValue, nil, nil, UInt32(tokens), 1, UInt32(hidden), shared.f32, gate?.f32,
                                      out.ptr, out.dtype.rawValue))
    }
    /// encodeMoEGateUpF32R1 with fuseSiluFwht (QWGemmMoE.swift:120-155): routed gate_up with the ids given.
    /// out: f16 [tokens, routes, rowsPerExpert / 2]; the SwiGLU and the rotation always run inside the launch (fuseSiluFwht: false,
    /// the reference's separate gu32 matrix, is refused), and so is a cold bank.
    public static func encodeMoEGateUpF32R1(_ enc: QWHipEncoder, hal: QWHal, x: QWTensorValue, bank: QWWeightView, ids: QWTensorValue,
                                            out: QWTensorValue, rowsPerExpert: Int, routes: Int, tokens: Int, fuseSiluFwht: Bool = false,
                                            coldBank: QWWeightView? = nil, reuseExpertsAcrossTokens: Bool = false, xIsRotated: Bool = true) throws {
        // reuseExpertsAcrossTokens: QWHIP_MOE_REUSE_EXPERTS for 2...4 tokens.  The reference defaults to true; here the launch
        // measured slower with it (rows that share an expert already meet in the L2), so the default is false.  Same bits.
        guard fuseSiluFwht, coldBank == nil, rowsPerExpert > 0, bank.n % rowsPerExpert == 0 else {
            throw QWGemmError.badShape("routed gate_up: fuseSiluFwht only, no cold bank, bank.n a multiple of rowsPerExpert")
        }
        let experts = bank.n / rowsPerExpert
        try hal.pipeline(bank.isIncumbent ? "qwg_moe_gateup_q4g_f32_r1" : "qwg_moe_gateup_aq\(bank.bits)_g\(bank.groupSize)_f32_r1")
        var w = bank.abi
        let flags = (xIsRotated ? UInt32(QWHIP_X_PREROTATED) : 0) | (reuseExpertsAcrossTokens ? UInt32(QWHIP_MOE_REUSE_EXPERTS) : 0)
        try qwCheck(qwhip_moe_gateup_decode(enc.stream, &w, UInt32(experts), x.ptr, x.dtype.rawValue, flags,
                                            ids.i32, UInt32(tokens), UInt32(routes), out.ptr))
    }
    /// encodeMoEGateUpF32R1 with fuseSiluFwht (QWGemmMoE.swift:120-155), routing folded into the launch for an HQ4_G32_M5 bank.
    public static func encodeMoERouteGateUp(_ enc: QWHipEncoder, hal: QWHal, x: QWTensorValue, bank: QWWeightView, experts: Int,
                                            logits: QWTensorValue, idx: QWTensorValue, wts: QWTensorValue, out: QWTensorValue,
                                            routes: Int, tokens: Int, normTopK: Bool, routedScale: Float, xIsRotated: Bool = true,
                                            reuseExpertsAcrossTokens: Bool = false) throws {
        precondition(tokens <= 8, "decode / verify path: at most 8 tokens")
        try hal.pipeline(bank.isIncumbent ? "qwg_moe_gateup_q4g_f32_r1" : "qwg_moe_gateup_aq\(bank.bits)_g\(bank.groupSize)_f32_r1")
        var w = bank.abi
        let flags = (xIsRotated ? UInt32(QWHIP_X_PREROTATED) : 0) | (reuseExpertsAcrossTokens ? UInt32(QWHIP_MOE_REUSE_EXPERTS) : 0)
        try qwCheck(qwhip_moe_route_gateup_decode(enc.stream, &w, UInt32(experts), x.ptr, x.dtype.rawValue, flags,
                                                  logits.f32, UInt32(tokens), UInt32(routes), normTopK ? 1 : 0, routedScale, idx.i32, wts.f32, out.ptr))
    }
    /// encodeMoEDownSharedCombineF32 (QWGemmMoE.swift:157-199)
    /// x: f16 [tokens, routes, k] ([tokens, k] with tokenIndexedX).  routeOutput: one output row per route, no sum and no shared
    /// term.  The group sum (numGroups) is encodeMoEDownGroupsF32, which takes the labels; a cold bank is refused.
    public static func encodeMoEDownSharedCombineF32(_ enc: QWHipEncoder, hal: QWHal, x: QWTensorValue, bank: QWWeightView, rowsPerRoute: Int,
                                                     routes: Int, weights: QWTensorValue, shared: QWTensorValue?, gate: QWTensorValue?,
                                                     out: QWTensorValue, ids: QWTensorValue, tokens: Int, out16: QWTensorValue? = nil,
                                                     coldBank: QWWeightView? = nil, routeOutput: Bool = false, reuseExpertsAcrossTokens: Bool = true,
                                                     skipShared: Bool = false, numGroups: Int = 0, tokenIndexedX: Bool = false) throws {
        guard coldBank == nil, numGroups == 0, rowsPerRoute > 0, bank.n % rowsPerRoute == 0, routeOutput || !tokenIndexedX else {
            throw QWGemmError.badShape("routed down: no cold bank, group sums are encodeMoEDownGroupsF32, bank.n a multiple of rowsPerRoute")
        }
        let experts = bank.n / rowsPerRoute
        if routeOutput {
            try encodeMoERoutedGemv(enc, hal: hal, bank: bank, experts: experts, x16: x, xPerToken: tokenIndexedX, ids: ids, weights: weights,
                                    tokens: tokens, routes: routes, out: out)
            return
        }
        try hal.pipeline(bank.isIncumbent ? "qwg_moe_down_shared_combine_q4g_f32" : "qwg_moe_down_shared_combine_aq\(bank.bits)_g\(bank.groupSize)_f32")
        var w = bank.abi
        for dst in [out, out16].compactMap({ $0 }) {
            try qwCheck(qwhip_moe_down_decode(enc.stream, &w, UInt32(experts), x.ptr, ids.i32, weights.f32, UInt32(tokens), UInt32(routes),
                                              skipShared ? nil : shared?.f32, skipShared ? nil : gate?.f32, dst.ptr, dst.dtype.rawValue))
        }
    }

    // ---- group-latent modes of the same encoders (latentLabels / groupIds / numGroups; the route ids stay plain here) ----
    /// encodeFnMoeRoute(latentLabels:groupIds:numGroups:) (QWGemmMoERouter.swift:10-75): groups of a token's routes, latent row of every route.
    public static func encodeMoELatentGroups(_ enc: QWHipEncoder, hal: QWHal, idx: QWTensorValue, labels: QWTensorValue, rows: Int, topK: Int,
                                             experts: Int, numGroups: Int, groupIds: QWTensorValue, pairRows: QWTensorValue?) throws {
        guard (1...32).contains(numGroups) else { throw QWGemmError.badShape("group-latent moe: 1..32 latent groups") }
        try hal.pipeline("qwg_moe_route")
        try qwCheck(qwhip_moe_latent_groups(enc.stream, idx.i32, labels.i32, UInt32(rows), UInt32(topK), UInt32(experts), UInt32(numGroups),
                                            groupIds.i32, pairRows?.i32))
    }
    /// encodeMoEDownSharedCombineF32(routeOutput: true, tokenIndexedX: true) (QWGemmMoE.swift:157-199): one output row per route.
    public static func encodeMoERoutedGemv(_ enc: QWHipEncoder, hal: QWHal, bank: QWWeightView, experts: Int, x16: QWTensorValue, xPerToken: Bool,
                                           ids: QWTensorValue, weights: QWTensorValue?, tokens: Int, routes: Int, out: QWTensorValue) throws {
        try hal.pipeline(bank.isIncumbent ? "qwg_moe_down_shared_combine_q4g_f32" : "qwg_moe_down_shared_combine_aq\(bank.bits)_g\(bank.groupSize)_f32")
        var w = bank.abi
        try qwCheck(qwhip_moe_routed_gemv(enc.stream, &w, UInt32(experts), x16.ptr, xPerToken ? 1 : 0, ids.i32, weights?.f32, UInt32(tokens),
                                          UInt32(routes), out.ptr, out.dtype.rawValue))
    }
    /// encodeMoEGateUpF32R1 over the latent rows of the routes (row token * numGroups + group of the latent matrix).
    public static func encodeMoEGateUpRowsF32R1(_ enc: QWHipEncoder, hal: QWHal, x: QWTensorValue, bank: QWWeightView, experts: Int, ids: QWTensorValue,
                                                xRows: QWTensorValue, out: QWTensorValue, routes: Int, tokens: Int) throws {
        try hal.pipeline(bank.isIncumbent ? "qwg_moe_gateup_q4g_f32_r1" : "qwg_moe_gateup_aq\(bank.bits)_g\(bank.groupSize)_f32_r1")
        var w = bank.abi
        try qwCheck(qwhip_moe_gateup_decode_rows(enc.stream, &w, UInt32(experts), x.ptr, x.dtype.rawValue, UInt32(QWHIP_X_PREROTATED), ids.i32,
                                                 xRows.i32, UInt32(tokens), UInt32(routes), out.ptr))
    }
    /// encodeMoEDownSharedCombineF32(numGroups:) (QWGemmMoE.swift:157-199): the routed down projection summed by latent group.
    public static func encodeMoEDownGroupsF32(_ enc: QWHipEncoder, hal: QWHal, x: QWTensorValue, bank: QWWeightView, experts: Int, ids: QWTensorValue,
                                              weights: QWTensorValue, labels: QWTensorValue, numGroups: Int, tokens: Int, routes: Int,
                                              out: QWTensorValue) throws {
        try hal.pipeline(bank.isIncumbent ? "qwg_moe_down_shared_combine_q4g_f32" : "qwg_moe_down_shared_combine_aq\(bank.bits)_g\(bank.groupSize)_f32")
        var w = bank.abi
        try qwCheck(qwhip_moe_down_decode_groups(enc.stream, &w, UInt32(experts), x.ptr, ids.i32, weights.f32, labels.i32, UInt32(numGroups),
                                                 UInt32(tokens), UInt32(routes), out.ptr, out.dtype.rawValue))
    }
    /// Gather rows of a grouped GEMM that reads the sorted output of an earlier one (the reference scatters that output back instead).
    public static func encodeMoEComposeRows(_ enc: QWHipEncoder, hal: QWHal, sortedPair: QWTensorValue, pairs: Int, pairRows: QWTensorValue,
                                            rowCount: Int, slotOfRow: QWTensorValue?, rowsOut: QWTensorValue) throws {
        try hal.pipeline("qwg_moe_group_pairs_f32")
        try qwCheck(qwhip_moe_compose_rows(enc.stream, sortedPair.i32, UInt32(pairs), pairRows.i32, UInt32(rowCount), slotOfRow?.i32, rowsOut.i32))
    }
    /// encodeMoEDownReduceCombineF32(numGroups:) (QWGemmMoE.swift:299-332): the sorted down outputs summed by latent group.
    public static func encodeMoECombineGroupsF32(_ enc: QWHipEncoder, hal: QWHal, dnAcc: QWTensorValue, invPerm: QWTensorValue?, weights: QWTensorValue?,
                                                 ids: QWTensorValue, labels: QWTensorValue, tokens: Int, routes: Int, numGroups: Int, width: Int,
                                                 out: QWTensorValue) throws {
        try hal.pipeline("qwg_moe_down_reduce_combine_f32")
        try qwCheck(qwhip_moe_combine_groups(enc.stream, dnAcc.ptr, dnAcc.dtype.rawValue, invPerm?.i32, weights?.f32, ids.i32, labels.i32, UInt32(labels.elementCount), UInt32(tokens),
                                             UInt32(routes), UInt32(numGroups), UInt32(width), out.ptr, out.dtype.rawValue))
    }
}

/// QWGemmAQ (Sources/Operators/QWGEMM/QWGemmAQ.swift): the doors over the bit-stream containers.
public enum QWGemmAQ {
    static func supported(bits: Int, group: Int) -> Bool { qwhip_block_bytes(UInt32(QWHIP_KIND_NATIVE_AFFINE), UInt32(bits), UInt32(group)) != 0 }
    /// The reference's name builders (QWGemmAQ.swift:22-133): nil for an unsupported (bits, group) pair and for every SHVQ
    /// container, which has no kernel in this library.
    static func name(_ head: String, _ bits: Int, _ group: Int, _ tail: String, _ isSHVQ: Bool) -> String? {
        !isSHVQ && supported(bits: bits, group: group) ? "\(head)_aq\(bits)_g\(group)\(tail)" : nil
    }
    public static func kernelName(bits: Int, group: Int, isSHVQ: Bool = false) -> String? { name("qwg_gemv", bits, group, "_v4", isSHVQ) }
    public static func decodeKernelName(bits: Int, group: Int, isSHVQ: Bool = false) -> String? { name("qwg_gemv", bits, group, "_dx_h16_t4", isSHVQ) }
    public static func siluPairKernelName(bits: Int, group: Int, isSHVQ: Bool = false) -> String? { name("qwg_gemv", bits, group, "_silu_pair_dx_h16", isSHVQ) }
    public static func headArgmaxKernelName(bits: Int, group: Int, isSHVQ: Bool = false) -> String? { name("qwg_head_gemv", bits, group, "_argmax", isSHVQ) }
    public static func gemmKernelName(bits: Int, group: Int, isSHVQ: Bool = false) -> String? { name("qwg_gemm", bits, group, "_h16", isSHVQ) }
    public static func swigluGemmKernelName(bits: Int, group: Int, isSHVQ: Bool = false) -> String? { name("qwg_gemm", bits, group, "_h16_swiglu", isSHVQ) }
    public static func f32BMKernelName(bits: Int, group: Int, isSHVQ: Bool = false) -> String? { name("qwg_gemm", bits, group, "_f32_bm", isSHVQ) }
    public static func f32V4KernelName(bits: Int, group: Int, isSHVQ: Bool = false) -> String? { name("qwg_gemv", bits, group, "_f32_v4", isSHVQ) }
    public static func f32V4ArgmaxKernelName(bits: Int, group: Int, isSHVQ: Bool = false) -> String? { name("qwg_gemv", bits, group, "_f32_v4_am", isSHVQ) }
    public static func f32V4Argmax2KernelName(bits: Int, group: Int, isSHVQ: Bool = false) -> String? { name("qwg_gemv", bits, group, "_f32_v4_am2", isSHVQ) }
    public static func naxF32KernelName(bits: Int, group: Int, isSHVQ: Bool = false) -> String? { name("qwg_gemm", bits, group, "_nax_f32", isSHVQ) }
    public static func moeGateUpF32R1KernelName(bits: Int, group: Int, isSHVQ: Bool = false) -> String? { name("qwg_moe_gateup", bits, group, "_f32_r1", isSHVQ) }
    public static func moeDownSharedCombineF32KernelName(bits: Int, group: Int, isSHVQ: Bool = false) -> String? {
        name("qwg_moe_down_shared_combine", bits, group, "_f32", isSHVQ)
    }
    public static func moeNaxGemmKernelName(bits: Int, group: Int, isSHVQ: Bool = false) -> String? { name("qwg_moe_nax_gemm", bits, group, "", isSHVQ) }
    public static func moeNaxSplitF32KernelName(bits: Int, group: Int, isSHVQ: Bool = false) -> String? { name("qwg_moe_nax_split", bits, group, "_f32", isSHVQ) }
    public static func rowBytes(bits: Int, group: Int, k: Int, isSHVQ: Bool = false) -> Int? {                                                            // :135-143
        guard !isSHVQ, supported(bits: bits, group: group), k % group == 0 else { return nil }
        return (k / group) * Int(qwhip_block_bytes(UInt32(QWHIP_KIND_NATIVE_AFFINE), UInt32(bits), UInt32(group)))
    }

    /// QWGemmAQ.encode (QWGemmAQ.swift:192-249): rows 1...16 against one pass over the bank; f32 output.
    /// isSHVQ: the vector-quantised container has no kernel here and is refused.  isRotated (an addition): the bank is a rotated
    /// HQ container, which the reference tells from the weight view's kind before it calls this door.
    public static func encode(_ enc: QWHipEncoder, hal: QWHal, blocks: QWTensorValue, x: QWTensorValue, y: QWTensorValue,
                              n: Int, k: Int, bits: Int, group: Int, rows: Int = 1, isSHVQ: Bool = false, isRotated: Bool = false,
                              xIsRotated: Bool = true) throws {
        guard !isSHVQ else { throw QWGemmError.badWeights("SHVQ containers have no kernel in this library") }
        try encode(enc, hal: hal, blocks: blocks.region, x: x, y: y, n: n, k: k, bits: bits, group: group, rows: rows, isRotated: isRotated,
                   xIsRotated: xIsRotated)
    }
    /// The same door over a raw device region.
    public static func encode(_ enc: QWHipEncoder, hal: QWHal, blocks: QWHipRegion, x: QWTensorValue, y: QWTensorValue,
                              n: Int, k: Int, bits: Int, group: Int, rows: Int = 1, isRotated: Bool = false, xIsRotated: Bool = true) throws {
        guard let name = kernelName(bits: bits, group: group) else { throw QWGemmError.badWeights("no affine-quantised kernel for \(bits)-bit group \(group)") }
        guard k % group == 0, n > 0, rows > 0 else { throw QWGemmError.badWeights("k must be a multiple of \(group) and n positive") }
        guard n < (1 << 24) else { throw QWGemmError.badWeights("bank does not fit the row-count flags") }
        guard let view = QWWeightView(blocks: blocks, n: n, k: k, kind: isRotated ? .rotatedHQ(bits: bits, group: group) : .nativeAffine(bits: bits, group: group)) else {
            throw QWGemmError.badWeights("block bank is short for n rows")
        }
        guard x.elementCount >= rows * k, y.dtype == .f32, y.elementCount >= rows * n else { throw QWGemmError.badWeights("operands are short") }
        try hal.pipeline(name)
        var w = view.abi
        try qwCheck(qwhip_gemv(enc.stream, &w, x.ptr, x.dtype.rawValue, UInt32(rows), xIsRotated ? UInt32(QWHIP_X_PREROTATED) : 0, nil, y.f32))
    }
    /// QWGemmAQ.encodeDecodeT4 (QWGemmAQ.swift:255-304): one f16 row in, f16 out.
    public static func encodeDecodeT4(_ enc: QWHipEncoder, hal: QWHal, blocks: QWTensorValue, x: QWTensorValue, y16: QWTensorValue,
                                      n: Int, k: Int, bits: Int, group: Int, isSHVQ: Bool = false, isRotated: Bool = false,
                                      xIsRotated: Bool = true) throws {
        guard !isSHVQ else { throw QWGemmError.badWeights("SHVQ containers have no kernel in this library") }
        try encodeDecodeT4(enc, hal: hal, blocks: blocks.region, x: x, y16: y16, n: n, k: k, bits: bits, group: group, isRotated: isRotated,
                           xIsRotated: xIsRotated)
    }
    public static func encodeDecodeT4(_ enc: QWHipEncoder, hal: QWHal, blocks: QWHipRegion, x: QWTensorValue, y16: QWTensorValue,
                                      n: Int, k: Int, bits: Int, group: Int, isRotated: Bool = false, xIsRotated: Bool = true) throws {
        guard let name = decodeKernelName(bits: bits, group: group) else { throw QWGemmError.badWeights("no affine-quantised decode kernel for \(bits)-bit group \(group)") }
        guard k % group == 0, n > 0 else { throw QWGemmError.badWeights("k must be a multiple of \(group) and n positive") }
        guard let view = QWWeightView(blocks: blocks, n: n, k: k, kind: isRotated ? .rotatedHQ(bits: bits, group: group) : .nativeAffine(bits: bits, group: group)) else {
            throw QWGemmError.badWeights("block bank is short for n rows")
        }
        guard x.dtype == .f16, x.elementCount >= k, y16.dtype == .f16, y16.elementCount >= n else { throw QWGemmError.badWeights("decode operands must be f16 [k] and f16 [n]") }
        try hal.pipeline(name)
        var w = view.abi
        try qwCheck(qwhip_gemv(enc.stream, &w, x.ptr, UInt32(QWHIP_F16), 1, xIsRotated ? UInt32(QWHIP_X_PREROTATED) : 0, y16.ptr, nil))
    }
    /// QWGemmAQ.encodeHeadArgmax (QWGemmAQ.swift:306-349): logits kept (writeLogits), tokens = greedy argmax, ties to the lower row.
    public static func encodeHeadArgmax(_ enc: QWHipEncoder, hal: QWHal, view: QWWeightView, x: QWTensorValue, logits: QWTensorValue,
                                        tokens: QWTensorValue, rows: Int = 1, xIsRotated: Bool = true) throws {
        guard rows >= 1, rows <= 16 else { throw QWGemmError.badShape("head argmax takes 1...16 rows") }
        guard logits.dtype == .f32, logits.elementCount >= rows * view.n, tokens.dtype == .i32, tokens.elementCount >= rows else {
            throw QWGemmError.badWeights("head argmax: logits f32 [rows, n], tokens i32 [rows]")
        }
        try hal.pipeline("qwg_head_gemv_q4g_argmax")
        var w = view.abi
        try qwCheck(qwhip_head_argmax(enc.stream, &w, x.ptr, x.dtype.rawValue, UInt32(rows), xIsRotated ? UInt32(QWHIP_X_PREROTATED) : 0, logits.f32, tokens.i32))
    }
    /// QWGemmAQ.encodeEmbedAQ (QWGemmAQ.swift:147-187): out f32 [rows, hc, hidden] = the token's row, code * scale + bias.
    public static func encodeEmbedAQ(_ enc: QWHipEncoder, hal: QWHal, blocks: QWTensorValue, token: QWTensorValue, out: QWTensorValue,
                                     hidden: Int, hc: Int, bits: Int, group: Int, rows: Int = 1) throws {
        guard let rb = rowBytes(bits: bits, group: group, k: hidden), rb > 0,            // the table's row count is what its region holds
              let table = QWWeightView(blocks: blocks.region, n: blocks.elementCount * blocks.dtype.bytes / rb, k: hidden,
                                       kind: .nativeAffine(bits: bits, group: group)) else {
            throw QWGemmError.badWeights("no embedding kernel for \(bits)-bit group \(group), or an empty table")
        }
        try encodeEmbedAQ(enc, hal: hal, table: table, token: token, out: out, rows: rows, hc: hc)
    }
    public static func encodeEmbedAQ(_ enc: QWHipEncoder, hal: QWHal, table: QWWeightView, token: QWTensorValue, out: QWTensorValue,
                                     rows: Int, hc: Int = 1) throws {
        guard rows > 0, hc > 0, token.elementCount >= rows, out.dtype == .f32, out.elementCount >= rows * hc * table.k else {
            throw QWGemmError.badWeights("the output must hold rows * hidden * hc f32 values")
        }
        try hal.pipeline("qwg_embed_aq_f32")
        var w = table.abi
        try qwCheck(qwhip_embed_aq_f32(enc.stream, &w, token.i32, UInt32(rows), UInt32(hc), out.f32))
    }
}

/// QWMoEOperator (Sources/Operators/QWGEMM/QWMoEOperator.swift:12-442, +Latent.swift:17-303, +GroupLatent.swift:11-294): the
/// routed-expert block on resident banks.  Types, labels and defaults are the reference's; `Weights.routedScale` and
/// `Scratch.hip` are additions with defaults, `decodeRouterOverride` has no counterpart (the router is always the library's).
/// The encoder is a HIP stream: work on it runs in order, so `concurrentBarriers`, `rotateEncoder` and `profileStage` are taken
/// and have nothing to do.
public enum QWMoEOperator {
    /// QWMoEOperator.Input (QWMoEOperator.swift:12-17)
    public enum Input {
        case f16Normed(QWTensorValue)
        case f32PreRotated(plain: QWTensorValue, rotated: QWTensorValue, prefillPrecast16: QWTensorValue?)
    }
    /// QWMoEOperator.LatentBottleneck (QWMoEOperator.swift:26-41)
    public struct LatentBottleneck {
        public let fc1: QWWeightView           // n = latentDim, k = hidden
        public let normGamma: QWTensorValue?   // f16 [latentDim], plus-one law
        public let normEps: Float
        public let fc2: QWWeightView           // n = hidden, k = latentDim
        public let latentDim: Int
        public init(fc1: QWWeightView, normGamma: QWTensorValue?, normEps: Float = 1e-6, fc2: QWWeightView, latentDim: Int) {
            self.fc1 = fc1; self.normGamma = normGamma; self.normEps = normEps; self.fc2 = fc2; self.latentDim = latentDim
        }
    }
    /// QWMoEOperator.LatentScratch (QWMoEOperator.swift:44-54): f32 [rows, latentDim] twice; bufB16 f16 [rows, latentDim] is
    /// required here (the routed experts read f16 rows at every row count).
    public struct LatentScratch {
        public let bufA32: QWTensorValue, bufB32: QWTensorValue
        public let bufB16: QWTensorValue?
        public init(bufA32: QWTensorValue, bufB32: QWTensorValue, bufB16: QWTensorValue? = nil) {
            self.bufA32 = bufA32; self.bufB32 = bufB32; self.bufB16 = bufB16
        }
    }
    /// QWMoEOperator.Weights (QWMoEOperator.swift:57-128).
    public struct Weights {
        public let router: QWTensorValue                 // [experts (x 2 with splitFeatureRouting), hidden] f32 / f16 / bf16
        public let routerBias: QWTensorValue?, routedScaleParam: QWTensorValue?
        public let splitFeatureRouting: Bool
        public let gateUp: QWWeightView                  // n = experts * 2 * intermediate, k = hidden (latentDim on the latent forms)
        public let down: QWWeightView                    // n = experts * hidden (latentDim), k = intermediate
        public let coldGateUp: QWWeightView?, coldDown: QWWeightView?      // tiered banks: refused when set
        public let sharedGateUp: QWWeightView?, sharedDown: QWWeightView?
        public let sharedGateScalar: QWTensorValue?      // f32 [hidden]
        public let latent: LatentBottleneck?
        public let latentD: QWWeightView?, latentU: QWWeightView?          // n = groups * latentDim, k = hidden; n = groups * hidden, k = latentDim
        public let latentLabels: QWTensorValue?          // i32 [experts]
        public let numLatentGroups: Int, latentDim: Int
        public let hidden: Int, experts: Int, topK: Int, intermediate: Int, sharedIntermediate: Int
        public let normTopK: Bool
        public let reuseExpertsAcrossTokens: Bool        // QWHIP_MOE_REUSE_EXPERTS on the routed gate_up of 2...4 rows (default false here)
        public let moeSpecExpertBudget: Int
        public let routedScale: Float
        public init(router: QWTensorValue, routerBias: QWTensorValue? = nil, routedScaleParam: QWTensorValue? = nil,
                    splitFeatureRouting: Bool = false, gateUp: QWWeightView, down: QWWeightView,
                    coldGateUp: QWWeightView? = nil, coldDown: QWWeightView? = nil,
                    sharedGateUp: QWWeightView? = nil, sharedDown: QWWeightView? = nil, sharedGateScalar: QWTensorValue? = nil,
                    latent: LatentBottleneck? = nil, latentD: QWWeightView? = nil, latentU: QWWeightView? = nil,
                    latentLabels: QWTensorValue? = nil, numLatentGroups: Int = 0, latentDim: Int = 0,
                    hidden: Int, experts: Int, topK: Int, intermediate: Int, sharedIntermediate: Int,
                    normTopK: Bool = true, reuseExpertsAcrossTokens: Bool = false, moeSpecExpertBudget: Int = 0, routedScale: Float = 1) {
            self.router = router; self.routerBias = routerBias; self.routedScaleParam = routedScaleParam
            self.splitFeatureRouting = splitFeatureRouting; self.gateUp = gateUp; self.down = down
            self.coldGateUp = coldGateUp; self.coldDown = coldDown
            self.sharedGateUp = sharedGateUp; self.sharedDown = sharedDown; self.sharedGateScalar = sharedGateScalar
            self.latent = latent; self.latentD = latentD; self.latentU = latentU; self.latentLabels = latentLabels
            self.numLatentGroups = numLatentGroups; self.latentDim = latentDim
            self.hidden = hidden; self.experts = experts; self.topK = topK; self.intermediate = intermediate
            self.sharedIntermediate = sharedIntermediate; self.normTopK = normTopK
            self.reuseExpertsAcrossTokens = reuseExpertsAcrossTokens; self.moeSpecExpertBudget = moeSpecExpertBudget
            self.routedScale = routedScale
        }
        var isGroupLatent: Bool { numLatentGroups > 0 && latentDim > 0 && latentD != nil && latentU != nil && latentLabels != nil }
        var sharedBanks: (QWWeightView, QWWeightView)? {
            if sharedIntermediate > 0, let gu = sharedGateUp, let dn = sharedDown { return (gu, dn) } else { return nil }
        }
    }
    /// What the group-latent prefill needs beyond the reference's scratch: the counting sort of the (token, group) pairs, the
    /// gather rows of the expert GEMM and the up-projection's rows.  Without it that form runs its row counts eight at a time
    /// on the routed GEMVs.
    public struct HipScratch {
        public let gExpOff, gSortedPair, gSortedTok, gInvPerm, gTileE, gTileR, gTileCount: QWTensorValue   // i32, as expOff ... tileCount
        public let rows2: QWTensorValue        // i32 [rows * topK]
        public let upAcc: QWTensorValue        // f32 [rows * groups, hidden]
        public init(gExpOff: QWTensorValue, gSortedPair: QWTensorValue, gSortedTok: QWTensorValue, gInvPerm: QWTensorValue,
                    gTileE: QWTensorValue, gTileR: QWTensorValue, gTileCount: QWTensorValue, rows2: QWTensorValue, upAcc: QWTensorValue) {
            self.gExpOff = gExpOff; self.gSortedPair = gSortedPair; self.gSortedTok = gSortedTok; self.gInvPerm = gInvPerm
            self.gTileE = gTileE; self.gTileR = gTileR; self.gTileCount = gTileCount; self.rows2 = rows2; self.upAcc = upAcc
        }
    }
    /// QWMoEOperator.Scratch (QWMoEOperator.swift:131-192), field for field.  This library's kernels keep their intermediates in
    /// f16 and use the reference's regions for them: the SwiGLU activations [rows * topK, intermediate] live in gu16 (else in
    /// act32), the latent rows of the group form in xLatent16 and zLatent32, the route -> latent-row table in gu32.
    public struct Scratch {
        public let xRot32, xPlain32: QWTensorValue       // f32 [rows, hidden]
        public let logits, idx, wts: QWTensorValue       // f32 [rows, routerCols], i32 [rows, topK], f32 [rows, topK]
        public let gu32, act32: QWTensorValue            // f32 [rows * topK, 2 * intermediate], [rows * topK, intermediate]
        public let guSh32, actSh32: QWTensorValue?
        public let shared, gate: QWTensorValue           // f32 [rows, hidden], f32 [rows]
        public let expOff, sortedPair, sortedTok, invPerm, tileE, tileR, tileCount: QWTensorValue?   // prefill only, i32
        public let gu16, dnHi: QWTensorValue?            // prefill only
        public let dnAcc: QWTensorValue                  // f32 [rows * topK, hidden]
        public let naxX16, naxY16: QWTensorValue?
        public let latent: LatentScratch?
        public let groupIds, onesRoute, xLatent32, xLatent16, zLatent32: QWTensorValue?
        public let maxTileWidth: Int
        public let hip: HipScratch?
        public init(xRot32: QWTensorValue, xPlain32: QWTensorValue, logits: QWTensorValue, idx: QWTensorValue, wts: QWTensorValue,
                    gu32: QWTensorValue, act32: QWTensorValue, guSh32: QWTensorValue?, actSh32: QWTensorValue?,
                    shared: QWTensorValue, gate: QWTensorValue, expOff: QWTensorValue?, sortedPair: QWTensorValue?,
                    sortedTok: QWTensorValue?, invPerm: QWTensorValue?, tileE: QWTensorValue?, tileR: QWTensorValue?,
                    tileCount: QWTensorValue?, gu16: QWTensorValue?, dnHi: QWTensorValue?, dnAcc: QWTensorValue,
                    naxX16: QWTensorValue?, naxY16: QWTensorValue? = nil, latent: LatentScratch? = nil,
                    groupIds: QWTensorValue? = nil, onesRoute: QWTensorValue? = nil, xLatent32: QWTensorValue? = nil,
                    xLatent16: QWTensorValue? = nil, zLatent32: QWTensorValue? = nil, maxTileWidth: Int, hip: HipScratch? = nil) {
            self.xRot32 = xRot32; self.xPlain32 = xPlain32; self.logits = logits; self.idx = idx; self.wts = wts
            self.gu32 = gu32; self.act32 = act32; self.guSh32 = guSh32; self.actSh32 = actSh32; self.shared = shared; self.gate = gate
            self.expOff = expOff; self.sortedPair = sortedPair; self.sortedTok = sortedTok; self.invPerm = invPerm
            self.tileE = tileE; self.tileR = tileR; self.tileCount = tileCount; self.gu16 = gu16; self.dnHi = dnHi; self.dnAcc = dnAcc
            self.naxX16 = naxX16; self.naxY16 = naxY16; self.latent = latent; self.groupIds = groupIds; self.onesRoute = onesRoute
            self.xLatent32 = xLatent32; self.xLatent16 = xLatent16; self.zLatent32 = zLatent32; self.maxTileWidth = maxTileWidth
            self.hip = hip
        }
        /// f16 [pairs, intermediate] inside gu16 (f16 [pairs, 2 * intermediate]) or act32 (f32 [pairs, intermediate]).
        func act16(pairs: Int, intermediate: Int) -> QWTensorValue {
            (gu16 ?? act32).slice(byteOffset: 0, count: pairs * intermediate, dtype: .f16)
        }
        /// The prefill sort's arrays, all present or none.
        var sort: (expOff: QWTensorValue, pair: QWTensorValue, tok: QWTensorValue, inv: QWTensorValue, tileE: QWTensorValue,
                   tileR: QWTensorValue, count: QWTensorValue, dnHi: QWTensorValue)? {
            if let a = expOff, let b = sortedPair, let c = sortedTok, let d = invPerm, let e = tileE, let f = tileR, let g = tileCount,
               let h = dnHi { return (a, b, c, d, e, f, g, h) } else { return nil }
        }
    }

    /// The operator's input in the three forms its stages read: f16 rows in the experts' basis, f32 un-rotated rows for the router,
    /// f32 rows in the basis for the dense shared-expert and latent projections (QWMoEOperator.swift:252-272).
    static func resolve(_ enc: QWHipEncoder, hal: QWHal, scratch s: Scratch, input: Input, rows T: Int, hidden H: Int,
                        needRot32: Bool) throws -> (x16: QWTensorValue, plain: QWTensorValue, rot32: QWTensorValue) {
        switch input {
        case .f16Normed(let x16):
            try QWGemm.encodeMoEBridgeF16ToF32(enc, hal: hal, x: x16, xRot32: s.xRot32, xPlain32: s.xPlain32, rows: T, hidden: H,
                                               skipRot32: !needRot32)
            return (x16, s.xPlain32, s.xRot32)
        case .f32PreRotated(let plain, let rotated, let precast16):
            if let p16 = precast16 { return (p16, plain, rotated) }
            guard let x16 = s.naxX16, x16.elementCount >= T * H else { throw QWGemmError.badShape("moe: f32 input needs scratch.naxX16 f16 [rows, hidden]") }
            try QWGemm.encodeCast(enc, hal: hal, x32: rotated, y16: x16, count: T * H)
            return (x16.slice(byteOffset: 0, count: T * H, dtype: .f16), plain, rotated)
        }
    }
    /// The shared expert on the hidden width (QWMoEOperator.swift:300-340): shared = Wd_sh . silu_mul(Wgu_sh . x).
    /// The f16 rows of the input serve as the gate|up projection's cast; the down projection stages its cast behind them in
    /// naxX16 when the input's f16 rows live there (an f32 input without a precast), as the reference's shAct16 alias does.
    static func encodeShared(_ enc: QWHipEncoder, hal: QWHal, weights w: Weights, scratch s: Scratch,
                             x r: (x16: QWTensorValue, plain: QWTensorValue, rot32: QWTensorValue), rows T: Int) throws -> Bool {
        guard let (shGU, shDown) = w.sharedBanks else { return false }
        guard let guSh = s.guSh32, let actSh = s.actSh32, let nax = s.naxX16 else { throw QWGemmError.badShape("moe: the shared expert needs guSh32, actSh32 and naxX16") }
        let held = r.x16.region.ptr == nax.region.ptr ? T * w.hidden : 0
        let stage = nax.slice(byteOffset: held * 2, count: max(0, nax.elementCount - held))
        try QWGemm.encodeDenseProjF32(enc, hal: hal, weight: shGU, x: r.rot32, y: guSh, naxX16: stage, naxY16: s.naxY16 ?? stage, maxTileWidth: s.maxTileWidth,
                                      rows: T, x16Precast: r.x16)
        try QWGemm.encodeSiluMulF32(enc, hal: hal, gu: guSh, act: actSh, rows: T, intermediate: w.sharedIntermediate)
        try QWGemm.encodeDenseProjF32(enc, hal: hal, weight: shDown, x: actSh, y: s.shared, naxX16: stage, naxY16: s.naxY16 ?? stage, maxTileWidth: s.maxTileWidth,
                                      rows: T)
        return true
    }
    /// out32 / out16 / skipOut32 (QWMoEOperator.swift:200-204): where the last stage stores, and the f16 copy made afterwards.
    static func finish(_ enc: QWHipEncoder, hal: QWHal, out32: QWTensorValue, out16: QWTensorValue?, wrote: QWTensorValue, count: Int) throws {
        if let o16 = out16, wrote.dtype == .f32 { try QWGemm.encodeCast(enc, hal: hal, x32: out32, y16: o16, count: count) }
    }

    /// QWMoEOperator.encodeResident (QWMoEOperator.swift:195-442).  rows > 8 with the sort's scratch present runs the grouped path
    /// (route -> pair sort -> gate_up GEMM with SwiGLU fused -> down GEMM -> combine); otherwise the routed GEMVs, eight rows a launch.
    public static func encodeResident(_ enc: inout QWHipEncoder, hal: QWHal, weights w: Weights, scratch s: Scratch, input: Input,
                                      out32: QWTensorValue, out16: QWTensorValue? = nil, skipOut32: Bool = false, rows T: Int,
                                      supportsGroupedNaxPrefill: Bool = true, concurrentBarriers: Bool = false,
                                      rotateEncoder: ((inout QWHipEncoder) throws -> Void)? = nil,
                                      profileStage: ((String) -> QWHipEncoder?)? = nil) throws {
        guard w.coldGateUp == nil, w.coldDown == nil else { throw QWGemmError.badWeights("moe: tiered (cold) expert banks have no kernel in this library") }
        if let latent = w.latent {
            try encodeResidentLatent(&enc, hal: hal, weights: w, latent: latent, scratch: s, input: input, out32: out32, out16: out16,
                                     skipOut32: skipOut32, rows: T, supportsGroupedNaxPrefill: supportsGroupedNaxPrefill,
                                     concurrentBarriers: concurrentBarriers, rotateEncoder: rotateEncoder, profileStage: profileStage)
            return
        }
        if w.isGroupLatent {
            try encodeResidentGroupLatent(&enc, hal: hal, weights: w, scratch: s, input: input, out32: out32, out16: out16,
                                          skipOut32: skipOut32, rows: T, supportsGroupedNaxPrefill: supportsGroupedNaxPrefill,
                                          concurrentBarriers: concurrentBarriers, rotateEncoder: rotateEncoder, profileStage: profileStage)
            return
        }
        let (H, E, K, I) = (w.hidden, w.experts, w.topK, w.intermediate)
        guard E > 0, E <= 512, K > 0, K <= 16 else { throw QWGemmError.badShape("moe: experts <= 512, routes <= 16") }
        guard w.gateUp.n == E * 2 * I, w.gateUp.k == H, w.down.n == E * H, w.down.k == I else {
            throw QWGemmError.badShape("moe: expert banks do not match (experts, hidden, intermediate)")
        }
        guard !skipOut32 || out16 != nil else { throw QWGemmError.badShape("moe: skipOut32 needs out16") }
        let r = try resolve(enc, hal: hal, scratch: s, input: input, rows: T, hidden: H, needRot32: w.sharedBanks != nil)
        let gateW = w.sharedBanks != nil ? w.sharedGateScalar : nil
        try QWGemm.encodeFnRouterGemm(enc, hal: hal, weight: w.router, x: r.plain, y: s.logits, rows: T, n: w.splitFeatureRouting ? 2 * E : E, k: H,
                                      shGateWeight: gateW, shGateOut: gateW != nil ? s.gate : nil)
        let hasShared = try encodeShared(enc, hal: hal, weights: w, scratch: s, x: r, rows: T)
        let shared = hasShared ? s.shared : nil, gate = gateW != nil ? s.gate : nil
        let dst = skipOut32 ? out16! : out32          // the combine stores either type
        let pairs = T * K
        let act16 = s.act16(pairs: pairs, intermediate: I)
        let plainRoute = w.routerBias == nil && w.routedScaleParam == nil && !w.splitFeatureRouting && w.moeSpecExpertBudget == 0
        if T > 8, supportsGroupedNaxPrefill, let q = s.sort, H % 64 == 0, I % 64 == 0 {
            try QWGemm.encodeFnMoeRoute(enc, hal: hal, logits: s.logits, idx: s.idx, wts: s.wts, rows: T, experts: E, topK: K, normTopK: w.normTopK,
                                        bias: w.routerBias, splitFeature: w.splitFeatureRouting, routedScaleParam: w.routedScaleParam,
                                        routedScale: w.routedScale)
            try QWGemm.encodeMoEGroupPairsF32(enc, hal: hal, ids: s.idx, expertOff: q.expOff, sortedPairIdx: q.pair, sortedTok: q.tok, experts: E,
                                              totalPairs: pairs, routes: K, invPerm: q.inv, tileE: q.tileE, tileR: q.tileR, tileCount: q.count)
            try QWGemm.encodeMoEGateUpSwiglu(enc, hal: hal, xe: r.x16, bank: w.gateUp, experts: E, sortedTok: q.tok, expertOff: q.expOff, tileE: q.tileE,
                                             tileR: q.tileR, tileCount: q.count, act16: act16, pairs: pairs, rotateAct: w.down.isRotated)
            try QWGemm.encodeMoEGroupedGemm(enc, hal: hal, xe: act16, bank: w.down, experts: E, expertOff: q.expOff, tileE: q.tileE, tileR: q.tileR,
                                            tileCount: q.count, y: q.dnHi, pairs: pairs)
            try QWGemm.encodeMoEDownReduceCombineF32(enc, hal: hal, dnAcc: q.dnHi, invPerm: q.inv, weights: s.wts, shared: shared, gate: gate,
                                                     out: dst, hidden: H, routes: K, tokens: T)
        } else {
            if !plainRoute {
                try QWGemm.encodeFnMoeRoute(enc, hal: hal, logits: s.logits, idx: s.idx, wts: s.wts, rows: T, experts: E, topK: K, normTopK: w.normTopK,
                                            bias: w.routerBias, expertBudget: w.moeSpecExpertBudget, splitFeature: w.splitFeatureRouting,
                                            routedScaleParam: w.routedScaleParam, routedScale: w.routedScale)
            }
            var t0 = 0
            while t0 < T {                            // the routed GEMVs take at most eight rows a launch
                let tc = min(8, T - t0)
                let x = r.x16.slice(byteOffset: t0 * H * 2, count: tc * H)
                let idx = s.idx.slice(byteOffset: t0 * K * 4, count: tc * K), wts = s.wts.slice(byteOffset: t0 * K * 4, count: tc * K)
                let act = act16.slice(byteOffset: t0 * K * I * 2, count: tc * K * I)
                if plainRoute {
                    let cols = E
                    try QWGemm.encodeMoERouteGateUp(enc, hal: hal, x: x, bank: w.gateUp, experts: E, logits: s.logits.slice(byteOffset: t0 * cols * 4, count: tc * cols),
                                                    idx: idx, wts: wts, out: act, routes: K, tokens: tc, normTopK: w.normTopK, routedScale: w.routedScale,
                                                    reuseExpertsAcrossTokens: w.reuseExpertsAcrossTokens)
                } else {
                    try QWGemm.encodeMoEGateUpF32R1(enc, hal: hal, x: x, bank: w.gateUp, ids: idx, out: act, rowsPerExpert: 2 * I, routes: K, tokens: tc,
                                                    fuseSiluFwht: true, reuseExpertsAcrossTokens: w.reuseExpertsAcrossTokens)
                }
                try QWGemm.encodeMoEDownSharedCombineF32(enc, hal: hal, x: act, bank: w.down, rowsPerRoute: H, routes: K, weights: wts,
                                                         shared: shared?.slice(byteOffset: t0 * H * 4, count: tc * H),
                                                         gate: gate?.slice(byteOffset: t0 * 4, count: tc),
                                                         out: dst.slice(byteOffset: t0 * H * dst.dtype.bytes, count: tc * H), ids: idx, tokens: tc)
                t0 += tc
            }
        }
        try finish(enc, hal: hal, out32: out32, out16: skipOut32 ? nil : out16, wrote: dst, count: T * H)
    }

    /// QWMoEOperator.encodeResidentLatent (QWMoEOperator+Latent.swift:17-303): fc1 -> route -> rotate -> routed experts in the latent
    /// width -> latent norm -> fc2, the shared expert on the hidden width added under its gate.  out32 is this form's working
    /// buffer and is written also under skipOut32.
    public static func encodeResidentLatent(_ enc: inout QWHipEncoder, hal: QWHal, weights w: Weights, latent: LatentBottleneck, scratch s: Scratch,
                                            input: Input, out32: QWTensorValue, out16: QWTensorValue?, skipOut32: Bool = false, rows T: Int,
                                            supportsGroupedNaxPrefill: Bool, concurrentBarriers: Bool,
                                            rotateEncoder: ((inout QWHipEncoder) throws -> Void)?, profileStage: ((String) -> QWHipEncoder?)?) throws {
        let (H, L, E, K, I) = (w.hidden, latent.latentDim, w.experts, w.topK, w.intermediate)
        guard L > 0, L % 32 == 0, latent.fc1.n == L, latent.fc1.k == H, latent.fc2.n == H, latent.fc2.k == L,
              w.gateUp.n == E * 2 * I, w.gateUp.k == L, w.down.n == E * L, w.down.k == I else {
            throw QWGemmError.badShape("latent moe: banks do not match (hidden, latent, experts, intermediate)")
        }
        guard let ls = s.latent, let bufB16 = ls.bufB16, let nax = s.naxX16 else { throw QWGemmError.badShape("latent moe: scratch.latent (with bufB16) and naxX16 are required") }
        guard !skipOut32 || out16 != nil else { throw QWGemmError.badShape("moe: skipOut32 needs out16") }
        let naxY = s.naxY16 ?? nax
        let r = try resolve(enc, hal: hal, scratch: s, input: input, rows: T, hidden: H, needRot32: true)
        let gateW = w.sharedBanks != nil ? w.sharedGateScalar : nil
        try QWGemm.encodeFnRouterGemm(enc, hal: hal, weight: w.router, x: r.plain, y: s.logits, rows: T, n: w.splitFeatureRouting ? 2 * E : E, k: H,
                                      shGateWeight: gateW, shGateOut: gateW != nil ? s.gate : nil)
        try QWGemm.encodeDenseProjF32(enc, hal: hal, weight: latent.fc1, x: r.rot32, y: ls.bufA32, naxX16: nax, naxY16: naxY, maxTileWidth: s.maxTileWidth, rows: T,
                                      x16Precast: r.x16)
        try QWGemm.encodeFnMoeRoute(enc, hal: hal, logits: s.logits, idx: s.idx, wts: s.wts, rows: T, experts: E, topK: K, normTopK: w.normTopK,
                                    bias: w.routerBias, expertBudget: w.moeSpecExpertBudget, splitFeature: w.splitFeatureRouting,
                                    routedScaleParam: w.routedScaleParam, routedScale: w.routedScale)
        try QWGemm.encodeLatentNormH32F32(enc, hal: hal, x: ls.bufA32, gamma: nil, out32: ls.bufB32, out16: bufB16, rows: T, latent: L, eps: latent.normEps,
                                          skipOut32: true)
        let hasShared = try encodeShared(enc, hal: hal, weights: w, scratch: s, x: r, rows: T)
        let pairs = T * K
        let act16 = s.act16(pairs: pairs, intermediate: I)
        if T > 8, supportsGroupedNaxPrefill, let q = s.sort, L % 64 == 0, I % 64 == 0 {
            try QWGemm.encodeMoEGroupPairsF32(enc, hal: hal, ids: s.idx, expertOff: q.expOff, sortedPairIdx: q.pair, sortedTok: q.tok, experts: E,
                                              totalPairs: pairs, routes: K, invPerm: q.inv, tileE: q.tileE, tileR: q.tileR, tileCount: q.count)
            try QWGemm.encodeMoEGateUpSwiglu(enc, hal: hal, xe: bufB16, bank: w.gateUp, experts: E, sortedTok: q.tok, expertOff: q.expOff, tileE: q.tileE,
                                             tileR: q.tileR, tileCount: q.count, act16: act16, pairs: pairs, rotateAct: w.down.isRotated)
            try QWGemm.encodeMoEGroupedGemm(enc, hal: hal, xe: act16, bank: w.down, experts: E, expertOff: q.expOff, tileE: q.tileE, tileR: q.tileR,
                                            tileCount: q.count, y: q.dnHi, pairs: pairs)
            try QWGemm.encodeMoEDownReduceCombineF32(enc, hal: hal, dnAcc: q.dnHi, invPerm: q.inv, weights: s.wts, shared: nil, gate: nil,
                                                     out: ls.bufA32, hidden: L, routes: K, tokens: T)
        } else {
            var t0 = 0
            while t0 < T {
                let tc = min(8, T - t0)
                let idx = s.idx.slice(byteOffset: t0 * K * 4, count: tc * K), act = act16.slice(byteOffset: t0 * K * I * 2, count: tc * K * I)
                try QWGemm.encodeMoEGateUpF32R1(enc, hal: hal, x: bufB16.slice(byteOffset: t0 * L * 2, count: tc * L), bank: w.gateUp, ids: idx, out: act,
                                                rowsPerExpert: 2 * I, routes: K, tokens: tc, fuseSiluFwht: true,
                                                reuseExpertsAcrossTokens: w.reuseExpertsAcrossTokens)
                try QWGemm.encodeMoEDownSharedCombineF32(enc, hal: hal, x: act, bank: w.down, rowsPerRoute: L, routes: K,
                                                         weights: s.wts.slice(byteOffset: t0 * K * 4, count: tc * K), shared: nil, gate: nil,
                                                         out: ls.bufA32.slice(byteOffset: t0 * L * 4, count: tc * L), ids: idx, tokens: tc)
                t0 += tc
            }
        }
        try QWGemm.encodeLatentNormH32F32(enc, hal: hal, x: ls.bufA32, gamma: latent.normGamma, out32: ls.bufB32, out16: nil, rows: T, latent: L,
                                          eps: latent.normEps)
        try QWGemm.encodeDenseProjF32(enc, hal: hal, weight: latent.fc2, x: ls.bufB32, y: out32, naxX16: nax, naxY16: naxY, maxTileWidth: s.maxTileWidth, rows: T)
        if hasShared {
            try QWGemm.encodeMoEAddSharedF32(enc, hal: hal, dnAcc: out32, shared: s.shared, gate: gateW != nil ? s.gate : nil, out: out32, hidden: H, tokens: T)
        }
        try finish(enc, hal: hal, out32: out32, out16: out16, wrote: out32, count: T * H)
    }

    /// QWMoEOperator.encodeResidentGroupLatent (QWMoEOperator+GroupLatent.swift:11-294): every token's hidden row goes down to the
    /// latent of each group its routes touch (latentD), the routed experts run in the latent width, their outputs are summed by
    /// group and come back up through latentU.
    public static func encodeResidentGroupLatent(_ enc: inout QWHipEncoder, hal: QWHal, weights w: Weights, scratch s: Scratch, input: Input,
                                                 out32: QWTensorValue, out16: QWTensorValue?, skipOut32: Bool = false, rows T: Int,
                                                 supportsGroupedNaxPrefill: Bool, concurrentBarriers: Bool,
                                                 rotateEncoder: ((inout QWHipEncoder) throws -> Void)?, profileStage: ((String) -> QWHipEncoder?)?) throws {
        let (H, L, NG, E, K, I) = (w.hidden, w.latentDim, w.numLatentGroups, w.experts, w.topK, w.intermediate)
        guard let latentD = w.latentD, let latentU = w.latentU, let labels = w.latentLabels else { throw QWGemmError.badWeights("group-latent moe: latentD, latentU and latentLabels") }
        guard (1...32).contains(NG), L > 0, L % 32 == 0, latentD.n == NG * L, latentD.k == H, latentU.n == NG * H, latentU.k == L,
              w.gateUp.n == E * 2 * I, w.gateUp.k == L, w.down.n == E * L, w.down.k == I else {
            throw QWGemmError.badShape("group-latent moe: banks do not match (hidden, groups, latent, experts, intermediate)")
        }
        guard let groupIds = s.groupIds, let onesRoute = s.onesRoute, let xLat = s.xLatent16, let zLat32 = s.zLatent32 else {
            throw QWGemmError.badShape("group-latent moe: scratch groupIds, onesRoute, xLatent16 and zLatent32 are required")
        }
        guard !skipOut32 || out16 != nil else { throw QWGemmError.badShape("moe: skipOut32 needs out16") }
        let (pairs, gpairs) = (T * K, T * NG)
        let zLat = zLat32.slice(byteOffset: 0, count: gpairs * L, dtype: .f16)          // f16 [rows * groups, latentDim]
        let pairRows = s.gu32.slice(byteOffset: 0, count: pairs, dtype: .i32)           // i32 [rows, topK]
        let r = try resolve(enc, hal: hal, scratch: s, input: input, rows: T, hidden: H, needRot32: w.sharedBanks != nil)
        let gateW = w.sharedBanks != nil ? w.sharedGateScalar : nil
        try QWGemm.encodeFnRouterGemm(enc, hal: hal, weight: w.router, x: r.plain, y: s.logits, rows: T, n: w.splitFeatureRouting ? 2 * E : E, k: H,
                                      shGateWeight: gateW, shGateOut: gateW != nil ? s.gate : nil)
        try QWGemm.encodeFnMoeRoute(enc, hal: hal, logits: s.logits, idx: s.idx, wts: s.wts, rows: T, experts: E, topK: K, normTopK: w.normTopK,
                                    bias: w.routerBias, expertBudget: w.moeSpecExpertBudget, splitFeature: w.splitFeatureRouting,
                                    routedScaleParam: w.routedScaleParam, routedScale: w.routedScale)
        try QWGemm.encodeMoELatentGroups(enc, hal: hal, idx: s.idx, labels: labels, rows: T, topK: K, experts: E, numGroups: NG,
                                         groupIds: groupIds, pairRows: pairRows)
        let hasShared = try encodeShared(enc, hal: hal, weights: w, scratch: s, x: r, rows: T)
        let shared = hasShared ? s.shared : nil, gate = gateW != nil ? s.gate : nil
        let dst = skipOut32 ? out16! : out32
        let act16 = s.act16(pairs: pairs, intermediate: I)
        if T > 8, supportsGroupedNaxPrefill, H % 64 == 0, L % 64 == 0, I % 64 == 0, let q = s.sort, let g = s.hip {
            try QWGemm.encodeMoEGroupPairsF32(enc, hal: hal, ids: groupIds, expertOff: g.gExpOff, sortedPairIdx: g.gSortedPair, sortedTok: g.gSortedTok,
                                              experts: NG, totalPairs: gpairs, routes: NG, invPerm: g.gInvPerm, tileE: g.gTileE, tileR: g.gTileR,
                                              tileCount: g.gTileCount)
            try QWGemm.encodeMoEGroupedGemm(enc, hal: hal, xe: r.x16, bank: latentD, experts: NG, expertOff: g.gExpOff, tileE: g.gTileE, tileR: g.gTileR,
                                            tileCount: g.gTileCount, y: xLat, pairs: gpairs, sortedTok: g.gSortedTok)
            try QWGemm.encodeMoEGroupPairsF32(enc, hal: hal, ids: s.idx, expertOff: q.expOff, sortedPairIdx: q.pair, sortedTok: q.tok, experts: E,
                                              totalPairs: pairs, routes: K, invPerm: q.inv, tileE: q.tileE, tileR: q.tileR, tileCount: q.count)
            try QWGemm.encodeMoEComposeRows(enc, hal: hal, sortedPair: q.pair, pairs: pairs, pairRows: pairRows, rowCount: gpairs, slotOfRow: g.gInvPerm,
                                            rowsOut: g.rows2)
            try QWGemm.encodeMoEGateUpSwiglu(enc, hal: hal, xe: xLat, bank: w.gateUp, experts: E, sortedTok: g.rows2, expertOff: q.expOff, tileE: q.tileE,
                                             tileR: q.tileR, tileCount: q.count, act16: act16, pairs: pairs, rotateAct: w.down.isRotated)
            try QWGemm.encodeMoEGroupedGemm(enc, hal: hal, xe: act16, bank: w.down, experts: E, expertOff: q.expOff, tileE: q.tileE, tileR: q.tileR,
                                            tileCount: q.count, y: q.dnHi, pairs: pairs)
            try QWGemm.encodeMoECombineGroupsF32(enc, hal: hal, dnAcc: q.dnHi, invPerm: q.inv, weights: s.wts, ids: s.idx, labels: labels,
                                                 tokens: T, routes: K, numGroups: NG, width: L, out: zLat)
            try QWGemm.encodeMoEGroupedGemm(enc, hal: hal, xe: zLat, bank: latentU, experts: NG, expertOff: g.gExpOff, tileE: g.gTileE, tileR: g.gTileR,
                                            tileCount: g.gTileCount, y: g.upAcc, pairs: gpairs, sortedTok: g.gSortedPair)
            try QWGemm.encodeMoEDownReduceCombineF32(enc, hal: hal, dnAcc: g.upAcc, invPerm: g.gInvPerm, weights: onesRoute, shared: shared, gate: gate,
                                                     out: dst, hidden: H, routes: NG, tokens: T)
        } else {
            var t0 = 0
            while t0 < T {
                let tc = min(8, T - t0)
                let idx = s.idx.slice(byteOffset: t0 * K * 4, count: tc * K), wts = s.wts.slice(byteOffset: t0 * K * 4, count: tc * K)
                let gids = groupIds.slice(byteOffset: t0 * NG * 4, count: tc * NG), ones = onesRoute.slice(byteOffset: t0 * NG * 4, count: tc * NG)
                let act = act16.slice(byteOffset: t0 * K * I * 2, count: tc * K * I)
                // a chunk's latent rows start at row 0 of its own slices: the route -> row table is rebuilt per chunk
                let rowsOfChunk = pairRows.slice(byteOffset: t0 * K * 4, count: tc * K)
                if t0 > 0 {
                    try QWGemm.encodeMoELatentGroups(enc, hal: hal, idx: idx, labels: labels, rows: tc, topK: K, experts: E, numGroups: NG,
                                                     groupIds: gids, pairRows: rowsOfChunk)
                }
                let xl = xLat.slice(byteOffset: t0 * NG * L * 2, count: tc * NG * L), zl = zLat.slice(byteOffset: t0 * NG * L * 2, count: tc * NG * L)
                try QWGemm.encodeMoERoutedGemv(enc, hal: hal, bank: latentD, experts: NG, x16: r.x16.slice(byteOffset: t0 * H * 2, count: tc * H),
                                               xPerToken: true, ids: gids, weights: nil, tokens: tc, routes: NG, out: xl)
                try QWGemm.encodeMoEGateUpRowsF32R1(enc, hal: hal, x: xl, bank: w.gateUp, experts: E, ids: idx, xRows: rowsOfChunk, out: act,
                                                    routes: K, tokens: tc)
                try QWGemm.encodeMoEDownGroupsF32(enc, hal: hal, x: act, bank: w.down, experts: E, ids: idx, weights: wts, labels: labels,
                                                  numGroups: NG, tokens: tc, routes: K, out: zl)
                try QWGemm.encodeMoEDownSharedCombineF32(enc, hal: hal, x: zl, bank: latentU, rowsPerRoute: H, routes: NG, weights: ones,
                                                         shared: shared?.slice(byteOffset: t0 * H * 4, count: tc * H),
                                                         gate: gate?.slice(byteOffset: t0 * 4, count: tc),
                                                         out: dst.slice(byteOffset: t0 * H * dst.dtype.bytes, count: tc * H), ids: gids, tokens: tc)
                t0 += tc
            }
        }
        try finish(enc, hal: hal, out32: out32, out16: skipOut32 ? nil : out16, wrote: dst, count: T * H)
    }
}
