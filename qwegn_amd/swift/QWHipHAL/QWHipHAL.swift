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
public enum QWDType: UInt32 { case f32 = 0, f16 = 1, bf16 = 2, i32 = 3
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
    public static func encode(_ enc: QWHipEncoder, hal: QWHal, plan: QWGemmPlan, x: QWTensorValue, wQ4: QWWeightView,
                              y: QWTensorValue, rows: Int = 1, xIsRotated: Bool = true) throws {
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
            try qwCheck(qwhip_gemv_silu_pair(enc.stream, &w, x.ptr, x.dtype.rawValue, UInt32(rows), flags, 1, y.ptr))
            return
        }
        guard y.dtype == .f32, y.elementCount >= rows * wQ4.n else { throw QWGemmError.badWeights("output must be f32 [rows, N]") }
        try qwCheck(qwhip_gemv(enc.stream, &w, x.ptr, x.dtype.rawValue, UInt32(rows), flags, nil, y.f32))
    }

    /// QWGemm.encodeH16 (QWGemm.swift:137-214): decode GEMV with direct f16 store (and optional f32 dual store).
    public static func encodeH16(_ enc: QWHipEncoder, hal: QWHal, plan: QWGemmPlan, x: QWTensorValue, wQ4: QWWeightView,
                                 y16: QWTensorValue, y32: QWTensorValue? = nil, rows: Int = 1, xIsRotated: Bool = true) throws {
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
    public static func encodeFwht32(_ enc: QWHipEncoder, hal: QWHal, x: QWTensorValue, count: Int) throws {
        guard count > 0, count % 32 == 0 else { throw QWGemmError.badWeights("fwht32 f16: n must be > 0 and divisible by 32") }
        try hal.pipeline("qwg_fwht32_f16")
        try qwCheck(qwhip_fwht32(enc.stream, x.ptr, UInt32(QWHIP_F16), x.ptr, UInt64(count)))
    }
    /// QWGemm.encodeCast (QWGemm.swift:305-320)
    public static func encodeCast(_ enc: QWHipEncoder, hal: QWHal, src32: QWTensorValue, dst16: QWTensorValue, count: Int) throws {
        guard src32.dtype == .f32, dst16.dtype == .f16, src32.elementCount >= count, dst16.elementCount >= count else { throw QWGemmError.badWeights("cast: f32 -> f16 operands") }
        try hal.pipeline("qwg_cast_f32_to_f16")
        try qwCheck(qwhip_cast_f32_to_f16(enc.stream, src32.f32, dst16.ptr, UInt64(count)))
    }
    /// QWGemm.encodeH32F32 (QWGemmF32.swift:46-54)
    public static func encodeH32F32(_ enc: QWHipEncoder, hal: QWHal, x: QWTensorValue, out: QWTensorValue, rows: Int, hidden: Int) throws {
        guard hidden % 32 == 0, x.elementCount >= rows * hidden, out.elementCount >= rows * hidden else { throw QWGemmError.badShape("h32: hidden % 32 == 0") }
        try hal.pipeline("qwg_h32_f32")
        try qwCheck(qwhip_h32_f32(enc.stream, x.f32, out.f32, UInt32(rows), UInt32(hidden)))
    }
    /// QWGemm.encodeHQ4F32V4 / encodeHQ4F32BM (QWGemmF32.swift:178-199, 311-350): fp32 activations, scalar epilogue 0...3.
    public static func encodeHQ4F32V4(_ enc: QWHipEncoder, hal: QWHal, weight: QWWeightView, x: QWTensorValue, y: QWTensorValue,
                                      rows: Int = 1, epilogue: Int = 0, scale: Float = 1) throws {
        guard x.dtype == .f32, y.dtype == .f32, x.elementCount >= rows * weight.k, y.elementCount >= rows * weight.n else { throw QWGemmError.badWeights("f32 GEMV operands") }
        try hal.pipeline("qwg_gemv_q4g_f32_v4")
        var w = weight.abi
        try qwCheck(qwhip_gemv_f32(enc.stream, &w, x.f32, UInt32(rows), UInt32(epilogue), scale, y.f32))
    }
    /// QWGemm.encodeSiluMulF32 / encodeSiluMulSplitF16 / encodeAddF32 (QWGemmF32.swift:83-115)
    public static func encodeSiluMulF32(_ enc: QWHipEncoder, hal: QWHal, gu: QWTensorValue, act: QWTensorValue, rows: Int, inter: Int) throws {
        guard inter % 32 == 0 else { throw QWGemmError.badShape("silu_mul f32: intermediate % 32 == 0") }
        try hal.pipeline("qwg_silu_mul_f32")
        try qwCheck(qwhip_silu_mul_f32(enc.stream, gu.f32, act.f32, UInt32(rows), UInt32(inter)))
    }
    public static func encodeSiluMulSplitF16(_ enc: QWHipEncoder, hal: QWHal, gu: QWTensorValue, act16: QWTensorValue, rows: Int, inter: Int,
                                             rotate: Bool = true) throws {
        try hal.pipeline("qwg_silu_mul_split_f16")
        try qwCheck(qwhip_swiglu_fwht(enc.stream, gu.ptr, gu.dtype.rawValue, act16.ptr, UInt32(rows), UInt32(inter), rotate ? 1 : 0))
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
                                              out16: QWTensorValue?, rows: Int, latent: Int, eps: Float = 1e-6) throws {
        guard latent > 0, latent % 32 == 0, out32 != nil || out16 != nil else { throw QWGemmError.badShape("latent norm H32: latent % 32 == 0, one output") }
        try hal.pipeline("qwg_latent_norm_h32_f32")
        try qwCheck(qwhip_latent_norm_h32_f32(enc.stream, x.f32, gamma?.ptr, out32?.f32, out16?.ptr, UInt32(rows), UInt32(latent), eps))
    }
    /// QWGemm.encodeMoEBridgeF16ToF32 (QWGemmMoE.swift:337-377): f16 normed hidden -> rotated f32 copy + un-rotated f32 copy.
    public static func encodeMoEBridgeF16ToF32(_ enc: QWHipEncoder, hal: QWHal, x: QWTensorValue, xRot32: QWTensorValue?, xPlain32: QWTensorValue,
                                               rows: Int, hidden: Int) throws {
        guard hidden % 256 == 0 else { throw QWGemmError.badGeometry("moe bridge: hidden must be a multiple of 256") }
        try hal.pipeline("qwg_moe_bridge_f16_to_f32")
        try qwCheck(qwhip_moe_bridge_f16_to_f32(enc.stream, x.ptr, xRot32?.f32, xPlain32.f32, UInt32(rows), UInt32(hidden)))
    }
    /// QWGemm.encodeDenseProjF32 (QWGemmF32.swift:413-440): f32 rows in the container's basis -> f32 outputs; 64 rows and more without
    /// an epilogue go through one cast and the f16 GEMM, fewer through the f32 door (its batched matrix-core form from 32 rows on).
    public static func encodeDenseProjF32(_ enc: QWHipEncoder, hal: QWHal, weight: QWWeightView, x: QWTensorValue, y: QWTensorValue,
                                          naxX16: QWTensorValue, rows: Int, epilogue: Int = 0, scale: Float = 1) throws {
        if rows >= 64, epilogue == 0, scale == 1, weight.n % 64 == 0, weight.k % 64 == 0, naxX16.elementCount >= rows * weight.k {
            try encodeCast(enc, hal: hal, src32: x, dst16: naxX16, count: rows * weight.k)
            try gemmBatchedH16(enc, hal: hal, x: naxX16, w: weight, y: y, rows: rows)
        } else {
            try encodeHQ4F32V4(enc, hal: hal, weight: weight, x: x, y: y, rows: rows, epilogue: epilogue, scale: scale)
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
    public static func encodeFnMoeRoute(_ enc: QWHipEncoder, hal: QWHal, logits: QWTensorValue, idx: QWTensorValue, wts: QWTensorValue,
                                        rows: Int, experts: Int, topK: Int, normTopK: Bool, routedScale: Float = 1, bias: QWTensorValue? = nil,
                                        splitFeature: Bool = false, routedScaleParam: QWTensorValue? = nil, expertBudget: Int = 0) throws {
        precondition(experts <= 512 && topK <= 16, "route: experts <= 512, K <= 16")
        try hal.pipeline("qwg_moe_route")
        try qwCheck(qwhip_moe_route_ex(enc.stream, logits.f32, UInt32(rows), UInt32(experts), UInt32(topK), normTopK ? 1 : 0, routedScale,
                                       splitFeature ? 1 : 0, bias?.f32, routedScaleParam?.f32, idx.i32, wts.f32))
        if expertBudget > 0 && rows > 1 && rows <= 4 && expertBudget < rows * topK && rows * topK <= 64 {      // QWGemmMoERouter.swift:63-75
            try hal.pipeline("qwg_moe_route_decode")
            try qwCheck(qwhip_moe_route_budget(enc.stream, idx.i32, wts.f32, UInt32(rows), UInt32(topK), UInt32(expertBudget), normTopK ? 1 : 0))
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
    public static func encodeMoEDownReduceCombineF32(_ enc: QWHipEncoder, hal: QWHal, dnAcc: QWTensorValue, invPerm: QWTensorValue,
                                                     weights: QWTensorValue, shared: QWTensorValue?, gate: QWTensorValue?, out: QWTensorValue,
                                                     hidden: Int, routes: Int, tokens: Int) throws {
        try hal.pipeline("qwg_moe_down_reduce_combine_f32")
        try qwCheck(qwhip_moe_combine(enc.stream, dnAcc.ptr, dnAcc.dtype.rawValue, invPerm.i32, weights.f32, UInt32(tokens), UInt32(routes),
                                      UInt32(hidden), shared?.f32, gate?.f32, out.ptr, out.dtype.rawValue))
    }
    /// The same door with invPerm: nil and unweightedSingle (QWGemmMoE.swift:299-332): out = dnAcc + gate * shared, one row per token.
    public static func encodeMoEAddSharedF32(_ enc: QWHipEncoder, hal: QWHal, dnAcc: QWTensorValue, shared: QWTensorValue, gate: QWTensorValue?,
                                             out: QWTensorValue, hidden: Int, tokens: Int) throws {
        try hal.pipeline("qwg_moe_down_reduce_combine_f32")
        try qwCheck(qwhip_moe_combine(enc.stream, dnAcc.ptr, dnAcc.dtype.rawValue, nil, nil, UInt32(tokens), 1, UInt32(hidden), shared.f32, gate?.f32,
                                      out.ptr, out.dtype.rawValue))
    }
    /// encodeMoEGateUpF32R1 with fuseSiluFwht (QWGemmMoE.swift:120-155): routed gate_up with the ids given.
    public static func encodeMoEGateUpF32R1(_ enc: QWHipEncoder, hal: QWHal, x: QWTensorValue, bank: QWWeightView, experts: Int, ids: QWTensorValue,
                                            out: QWTensorValue, routes: Int, tokens: Int, xIsRotated: Bool = true) throws {
        try hal.pipeline(bank.isIncumbent ? "qwg_moe_gateup_q4g_f32_r1" : "qwg_moe_gateup_aq\(bank.bits)_g\(bank.groupSize)_f32_r1")
        var w = bank.abi
        try qwCheck(qwhip_moe_gateup_decode(enc.stream, &w, UInt32(experts), x.ptr, x.dtype.rawValue, xIsRotated ? UInt32(QWHIP_X_PREROTATED) : 0,
                                            ids.i32, UInt32(tokens), UInt32(routes), out.ptr))
    }
    /// encodeMoEGateUpF32R1 with fuseSiluFwht (QWGemmMoE.swift:120-155), routing folded into the launch for an HQ4_G32_M5 bank.
    public static func encodeMoERouteGateUp(_ enc: QWHipEncoder, hal: QWHal, x: QWTensorValue, bank: QWWeightView, experts: Int,
                                            logits: QWTensorValue, idx: QWTensorValue, wts: QWTensorValue, out: QWTensorValue,
                                            routes: Int, tokens: Int, normTopK: Bool, routedScale: Float, xIsRotated: Bool = true) throws {
        precondition(tokens <= 8, "decode / verify path: at most 8 tokens")
        try hal.pipeline(bank.isIncumbent ? "qwg_moe_gateup_q4g_f32_r1" : "qwg_moe_gateup_aq\(bank.bits)_g\(bank.groupSize)_f32_r1")
        var w = bank.abi
        try qwCheck(qwhip_moe_route_gateup_decode(enc.stream, &w, UInt32(experts), x.ptr, x.dtype.rawValue, xIsRotated ? UInt32(QWHIP_X_PREROTATED) : 0,
                                                  logits.f32, UInt32(tokens), UInt32(routes), normTopK ? 1 : 0, routedScale, idx.i32, wts.f32, out.ptr))
    }
    /// encodeMoEDownSharedCombineF32 (QWGemmMoE.swift:157-199)
    public static func encodeMoEDownSharedCombineF32(_ enc: QWHipEncoder, hal: QWHal, x: QWTensorValue, bank: QWWeightView, experts: Int,
                                                     routes: Int, weights: QWTensorValue, shared: QWTensorValue?, gate: QWTensorValue?,
                                                     out: QWTensorValue, ids: QWTensorValue, tokens: Int) throws {
        try hal.pipeline(bank.isIncumbent ? "qwg_moe_down_shared_combine_q4g_f32" : "qwg_moe_down_shared_combine_aq\(bank.bits)_g\(bank.groupSize)_f32")
        var w = bank.abi
        try qwCheck(qwhip_moe_down_decode(enc.stream, &w, UInt32(experts), x.ptr, ids.i32, weights.f32, UInt32(tokens), UInt32(routes), shared?.f32,
                                          gate?.f32, out.ptr, out.dtype.rawValue))
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
    public static func kernelName(bits: Int, group: Int) -> String? { supported(bits: bits, group: group) ? "qwg_gemv_aq\(bits)_g\(group)_v4" : nil }        // :22-26
    public static func decodeKernelName(bits: Int, group: Int) -> String? { supported(bits: bits, group: group) ? "qwg_gemv_aq\(bits)_g\(group)_dx_h16_t4" : nil }   // :28-36
    public static func rowBytes(bits: Int, group: Int, k: Int) -> Int? {                                                                                  // :135-143
        guard supported(bits: bits, group: group), k % group == 0 else { return nil }
        return (k / group) * Int(qwhip_block_bytes(UInt32(QWHIP_KIND_NATIVE_AFFINE), UInt32(bits), UInt32(group)))
    }

    /// QWGemmAQ.encode (QWGemmAQ.swift:192-249): rows 1...16 against one pass over the bank; f32 output.
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

/// QWMoEOperator.encodeResident (Sources/Operators/QWGEMM/QWMoEOperator.swift:57-442): the routed-expert block on resident banks.
public enum QWMoEOperator {
    public struct Weights {
        public let router: QWTensorValue       // [experts, hidden] f32 / f16 / bf16
        public let gateUp: QWWeightView        // n = experts * 2 * intermediate, k = hidden
        public let down: QWWeightView          // n = experts * hidden, k = intermediate
        public let hidden: Int, experts: Int, topK: Int, intermediate: Int
        public let normTopK: Bool
        public let routedScale: Float
    }
    public struct Scratch {                    // caller-owned (the reference's arena scratch, QWMoEOperator.swift:117-192)
        public let logits: QWTensorValue       // f32 [rows, experts]
        public let idx: QWTensorValue          // i32 [rows, topK]
        public let wts: QWTensorValue          // f32 [rows, topK]
        public let act16: QWTensorValue        // f16 [rows * topK, intermediate]
        public let expOff, sortedPair, sortedTok, invPerm, tileE, tileR, tileCount: QWTensorValue?   // prefill only, i32
        public let dnHi: QWTensorValue?        // f32 or f16 [rows * topK, hidden], prefill only
    }
    /// x: f16 hidden rows in the experts' basis; xPlain: the un-rotated rows the router reads.  rows > 8 runs the grouped path
    /// (route -> pair sort -> gate_up GEMM with SwiGLU fused -> down GEMM -> combine), fewer rows the routed GEMVs.
    public static func encodeResident(_ enc: QWHipEncoder, hal: QWHal, weights w: Weights, scratch s: Scratch, x: QWTensorValue,
                                      xPlain: QWTensorValue, out32: QWTensorValue, rows T: Int, shared: QWTensorValue? = nil,
                                      sharedGate: QWTensorValue? = nil) throws {
        let (H, E, K, I) = (w.hidden, w.experts, w.topK, w.intermediate)
        guard E > 0, E <= 512, K > 0, K <= 16 else { throw QWGemmError.badShape("moe: experts <= 512, routes <= 16") }
        guard w.gateUp.n == E * 2 * I, w.gateUp.k == H, w.down.n == E * H, w.down.k == I else {
            throw QWGemmError.badShape("moe: expert banks do not match (experts, hidden, intermediate)")
        }
        try QWGemm.encodeFnRouterGemm(enc, hal: hal, weight: w.router, x: xPlain, y: s.logits, rows: T, n: E, k: H)
        if T > 8, let expOff = s.expOff, let sortedPair = s.sortedPair, let sortedTok = s.sortedTok, let invPerm = s.invPerm,
           let tileE = s.tileE, let tileR = s.tileR, let tileCount = s.tileCount, let dnHi = s.dnHi, H % 64 == 0, I % 64 == 0, x.dtype == .f16 {
            let pairs = T * K
            try QWGemm.encodeFnMoeRoute(enc, hal: hal, logits: s.logits, idx: s.idx, wts: s.wts, rows: T, experts: E, topK: K, normTopK: w.normTopK,
                                        routedScale: w.routedScale)
            try QWGemm.encodeMoEGroupPairsF32(enc, hal: hal, ids: s.idx, expertOff: expOff, sortedPairIdx: sortedPair, sortedTok: sortedTok, experts: E,
                                              totalPairs: pairs, routes: K, invPerm: invPerm, tileE: tileE, tileR: tileR, tileCount: tileCount)
            try QWGemm.encodeMoEGateUpSwiglu(enc, hal: hal, xe: x, bank: w.gateUp, experts: E, sortedTok: sortedTok, expertOff: expOff, tileE: tileE,
                                             tileR: tileR, tileCount: tileCount, act16: s.act16, pairs: pairs, rotateAct: w.down.isRotated)
            try QWGemm.encodeMoEGroupedGemm(enc, hal: hal, xe: s.act16, bank: w.down, experts: E, expertOff: expOff, tileE: tileE, tileR: tileR,
                                            tileCount: tileCount, y: dnHi, pairs: pairs)
            try QWGemm.encodeMoEDownReduceCombineF32(enc, hal: hal, dnAcc: dnHi, invPerm: invPerm, weights: s.wts, shared: shared, gate: sharedGate,
                                                     out: out32, hidden: H, routes: K, tokens: T)
        } else {
            try QWGemm.encodeMoERouteGateUp(enc, hal: hal, x: x, bank: w.gateUp, experts: E, logits: s.logits, idx: s.idx, wts: s.wts, out: s.act16,
                                            routes: K, tokens: T, normTopK: w.normTopK, routedScale: w.routedScale)
            try QWGemm.encodeMoEDownSharedCombineF32(enc, hal: hal, x: s.act16, bank: w.down, experts: E, routes: K, weights: s.wts, shared: shared,
                                                     gate: sharedGate, out: out32, ids: s.idx, tokens: T)
        }
    }

    // ---- latent-bottleneck sparse MoE (QWMoEOperator+Latent.swift:17-303) ------------------------------------------------
    public struct LatentBottleneck {
        public let fc1: QWWeightView           // n = latentDim, k = hidden
        public let fc2: QWWeightView           // n = hidden, k = latentDim
        public let normGamma: QWTensorValue?   // f16 [latentDim], plus-one law
        public let normEps: Float
        public let latentDim: Int
    }
    public struct LatentWeights {
        public let routed: Weights             // gateUp: k = latentDim; down: n = experts * latentDim
        public let sharedGateUp: QWWeightView?, sharedDown: QWWeightView?
        public let sharedGateScalar: QWTensorValue?      // f32 [hidden]
        public let sharedIntermediate: Int
        public let routerBias: QWTensorValue?, routedScaleParam: QWTensorValue?
        public let splitFeatureRouting: Bool
    }
    public struct LatentScratch {
        public let xRot32, xPlain32: QWTensorValue       // f32 [rows, hidden]
        public let bufA32, bufB32: QWTensorValue         // f32 [rows, latentDim]
        public let bufB16: QWTensorValue                 // f16 [rows, latentDim]
        public let naxX16: QWTensorValue                 // f16 staging of the dense projections
        public let gate: QWTensorValue                   // f32 [rows]
        public let guSh32, actSh32, shared: QWTensorValue
    }
    /// fc1 -> route -> rotate -> routed experts in the latent width -> latent norm -> fc2, the shared expert on the hidden width
    /// added under its gate.  x16: the operator's .f16Normed input.
    public static func encodeResidentLatent(_ enc: QWHipEncoder, hal: QWHal, weights lw: LatentWeights, latent: LatentBottleneck, scratch s: Scratch,
                                            latentScratch ls: LatentScratch, x16: QWTensorValue, out32: QWTensorValue, rows T: Int) throws {
        let w = lw.routed
        let (H, L, E, K, I, ISh) = (w.hidden, latent.latentDim, w.experts, w.topK, w.intermediate, lw.sharedIntermediate)
        guard L > 0, L % 32 == 0, latent.fc1.n == L, latent.fc1.k == H, latent.fc2.n == H, latent.fc2.k == L,
              w.gateUp.n == E * 2 * I, w.gateUp.k == L, w.down.n == E * L, w.down.k == I else {
            throw QWGemmError.badShape("latent moe: banks do not match (hidden, latent, experts, intermediate)")
        }
        let routerCols = lw.splitFeatureRouting ? 2 * E : E
        try QWGemm.encodeMoEBridgeF16ToF32(enc, hal: hal, x: x16, xRot32: ls.xRot32, xPlain32: ls.xPlain32, rows: T, hidden: H)
        let sharedBanks: (QWWeightView, QWWeightView)? = (ISh > 0 && lw.sharedGateUp != nil && lw.sharedDown != nil) ? (lw.sharedGateUp!, lw.sharedDown!) : nil
        let gateW = sharedBanks != nil ? lw.sharedGateScalar : nil
        try QWGemm.encodeFnRouterGemm(enc, hal: hal, weight: w.router, x: ls.xPlain32, y: s.logits, rows: T, n: routerCols, k: H,
                                      shGateWeight: gateW, shGateOut: gateW != nil ? ls.gate : nil)
        try QWGemm.encodeDenseProjF32(enc, hal: hal, weight: latent.fc1, x: ls.xRot32, y: ls.bufA32, naxX16: ls.naxX16, rows: T)
        try QWGemm.encodeFnMoeRoute(enc, hal: hal, logits: s.logits, idx: s.idx, wts: s.wts, rows: T, experts: E, topK: K, normTopK: w.normTopK,
                                    routedScale: w.routedScale, bias: lw.routerBias, splitFeature: lw.splitFeatureRouting,
                                    routedScaleParam: lw.routedScaleParam)
        try QWGemm.encodeLatentNormH32F32(enc, hal: hal, x: ls.bufA32, gamma: nil, out32: nil, out16: ls.bufB16, rows: T, latent: L, eps: latent.normEps)
        if let (shGU, shDown) = sharedBanks {
            try QWGemm.encodeDenseProjF32(enc, hal: hal, weight: shGU, x: ls.xRot32, y: ls.guSh32, naxX16: ls.naxX16, rows: T)
            try QWGemm.encodeSiluMulF32(enc, hal: hal, gu: ls.guSh32, act: ls.actSh32, rows: T, inter: ISh)
            try QWGemm.encodeDenseProjF32(enc, hal: hal, weight: shDown, x: ls.actSh32, y: ls.shared, naxX16: ls.naxX16, rows: T)
        }
        let pairs = T * K
        if T > 8, let expOff = s.expOff, let sortedPair = s.sortedPair, let sortedTok = s.sortedTok, let invPerm = s.invPerm,
           let tileE = s.tileE, let tileR = s.tileR, let tileCount = s.tileCount, let dnHi = s.dnHi, L % 64 == 0, I % 64 == 0 {
            try QWGemm.encodeMoEGroupPairsF32(enc, hal: hal, ids: s.idx, expertOff: expOff, sortedPairIdx: sortedPair, sortedTok: sortedTok, experts: E,
                                              totalPairs: pairs, routes: K, invPerm: invPerm, tileE: tileE, tileR: tileR, tileCount: tileCount)
            try QWGemm.encodeMoEGateUpSwiglu(enc, hal: hal, xe: ls.bufB16, bank: w.gateUp, experts: E, sortedTok: sortedTok, expertOff: expOff, tileE: tileE,
                                             tileR: tileR, tileCount: tileCount, act16: s.act16, pairs: pairs, rotateAct: w.down.isRotated)
            try QWGemm.encodeMoEGroupedGemm(enc, hal: hal, xe: s.act16, bank: w.down, experts: E, expertOff: expOff, tileE: tileE, tileR: tileR,
                                            tileCount: tileCount, y: dnHi, pairs: pairs)
            try QWGemm.encodeMoEDownReduceCombineF32(enc, hal: hal, dnAcc: dnHi, invPerm: invPerm, weights: s.wts, shared: nil, gate: nil,
                                                     out: ls.bufA32, hidden: L, routes: K, tokens: T)
        } else {
            try QWGemm.encodeMoEGateUpF32R1(enc, hal: hal, x: ls.bufB16, bank: w.gateUp, experts: E, ids: s.idx, out: s.act16, routes: K, tokens: T)
            try QWGemm.encodeMoEDownSharedCombineF32(enc, hal: hal, x: s.act16, bank: w.down, experts: E, routes: K, weights: s.wts, shared: nil,
                                                     gate: nil, out: ls.bufA32, ids: s.idx, tokens: T)
        }
        try QWGemm.encodeLatentNormH32F32(enc, hal: hal, x: ls.bufA32, gamma: latent.normGamma, out32: ls.bufB32, out16: nil, rows: T, latent: L,
                                          eps: latent.normEps)
        try QWGemm.encodeDenseProjF32(enc, hal: hal, weight: latent.fc2, x: ls.bufB32, y: out32, naxX16: ls.naxX16, rows: T)
        if sharedBanks != nil {
            try QWGemm.encodeMoEAddSharedF32(enc, hal: hal, dnAcc: out32, shared: ls.shared, gate: gateW != nil ? ls.gate : nil, out: out32, hidden: H,
                                             tokens: T)
        }
    }

    // ---- group-latent sparse MoE (QWMoEOperator+GroupLatent.swift:11-294) ------------------------------------------------
    public struct GroupLatentWeights {
        public let routed: Weights             // gateUp: k = latentDim; down: n = experts * latentDim
        public let latentD: QWWeightView       // n = groups * latentDim, k = hidden
        public let latentU: QWWeightView       // n = groups * hidden, k = latentDim
        public let latentLabels: QWTensorValue // i32 [experts]
        public let numLatentGroups: Int, latentDim: Int
        public let sharedGateUp: QWWeightView?, sharedDown: QWWeightView?
        public let sharedGateScalar: QWTensorValue?
        public let sharedIntermediate: Int
        public let routerBias: QWTensorValue?, routedScaleParam: QWTensorValue?
        public let splitFeatureRouting: Bool
    }
    public struct GroupLatentScratch {
        public let groupIds: QWTensorValue, pairRows: QWTensorValue     // i32 [rows, groups], [rows, topK]
        public let onesRoute: QWTensorValue                             // f32 [rows, groups], all 1
        public let xLatent16, zLatent16: QWTensorValue                  // f16 [rows * groups, latentDim]
        public let naxX16, xe16: QWTensorValue                          // f16 [rows, hidden]
        public let xRot32, xPlain32: QWTensorValue, gate: QWTensorValue
        public let guSh32, actSh32, shared: QWTensorValue
        public let gExpOff, gSortedPair, gSortedTok, gInvPerm, gTileE, gTileR, gTileCount: QWTensorValue?   // prefill: the (token, group) sort
        public let rows2: QWTensorValue?, upAcc: QWTensorValue?         // prefill: i32 [rows * topK], f32 [rows * groups, hidden]
    }
    /// QWMoEOperator.Input (QWMoEOperator.swift:12-17)
    public enum Input {
        case f16Normed(QWTensorValue)
        case f32PreRotated(plain: QWTensorValue, rotated: QWTensorValue, prefillPrecast16: QWTensorValue?)
    }
    public static func encodeResidentGroupLatent(_ enc: QWHipEncoder, hal: QWHal, weights gw: GroupLatentWeights, scratch s: Scratch,
                                                 groupScratch gs: GroupLatentScratch, input: Input, out32: QWTensorValue, rows T: Int) throws {
        let w = gw.routed
        let (H, L, NG, E, K, I, ISh) = (w.hidden, gw.latentDim, gw.numLatentGroups, w.experts, w.topK, w.intermediate, gw.sharedIntermediate)
        guard (1...32).contains(NG), L > 0, L % 32 == 0, gw.latentD.n == NG * L, gw.latentD.k == H, gw.latentU.n == NG * H, gw.latentU.k == L,
              w.gateUp.n == E * 2 * I, w.gateUp.k == L, w.down.n == E * L, w.down.k == I else {
            throw QWGemmError.badShape("group-latent moe: banks do not match (hidden, groups, latent, experts, intermediate)")
        }
        let x16: QWTensorValue, xPlain: QWTensorValue, xRot: QWTensorValue
        switch input {
        case .f16Normed(let x):
            try QWGemm.encodeMoEBridgeF16ToF32(enc, hal: hal, x: x, xRot32: gs.xRot32, xPlain32: gs.xPlain32, rows: T, hidden: H)
            (x16, xPlain, xRot) = (x, gs.xPlain32, gs.xRot32)
        case .f32PreRotated(let plain, let rotated, let precast16):
            if let p16 = precast16 { x16 = p16 } else {
                try QWGemm.encodeCast(enc, hal: hal, src32: rotated, dst16: gs.xe16, count: T * H)
                x16 = gs.xe16
            }
            (xPlain, xRot) = (plain, rotated)
        }
        let sharedBanks: (QWWeightView, QWWeightView)? = (ISh > 0 && gw.sharedGateUp != nil && gw.sharedDown != nil) ? (gw.sharedGateUp!, gw.sharedDown!) : nil
        let gateW = sharedBanks != nil ? gw.sharedGateScalar : nil
        try QWGemm.encodeFnRouterGemm(enc, hal: hal, weight: w.router, x: xPlain, y: s.logits, rows: T, n: gw.splitFeatureRouting ? 2 * E : E, k: H,
                                      shGateWeight: gateW, shGateOut: gateW != nil ? gs.gate : nil)
        try QWGemm.encodeFnMoeRoute(enc, hal: hal, logits: s.logits, idx: s.idx, wts: s.wts, rows: T, experts: E, topK: K, normTopK: w.normTopK,
                                    routedScale: w.routedScale, bias: gw.routerBias, splitFeature: gw.splitFeatureRouting,
                                    routedScaleParam: gw.routedScaleParam)
        try QWGemm.encodeMoELatentGroups(enc, hal: hal, idx: s.idx, labels: gw.latentLabels, rows: T, topK: K, experts: E, numGroups: NG,
                                         groupIds: gs.groupIds, pairRows: gs.pairRows)
        if let (shGU, shDown) = sharedBanks {
            try QWGemm.encodeDenseProjF32(enc, hal: hal, weight: shGU, x: xRot, y: gs.guSh32, naxX16: gs.naxX16, rows: T)
            try QWGemm.encodeSiluMulF32(enc, hal: hal, gu: gs.guSh32, act: gs.actSh32, rows: T, inter: ISh)
            try QWGemm.encodeDenseProjF32(enc, hal: hal, weight: shDown, x: gs.actSh32, y: gs.shared, naxX16: gs.naxX16, rows: T)
        }
        let shared = sharedBanks != nil ? gs.shared : nil, gate = gateW != nil ? gs.gate : nil
        let (pairs, gpairs) = (T * K, T * NG)
        if T > 8, H % 64 == 0, L % 64 == 0, I % 64 == 0, let expOff = s.expOff, let sortedPair = s.sortedPair, let sortedTok = s.sortedTok,
           let invPerm = s.invPerm, let tileE = s.tileE, let tileR = s.tileR, let tileCount = s.tileCount, let dnHi = s.dnHi,
           let gOff = gs.gExpOff, let gPair = gs.gSortedPair, let gTok = gs.gSortedTok, let gInv = gs.gInvPerm, let gTE = gs.gTileE, let gTR = gs.gTileR,
           let gTC = gs.gTileCount, let rows2 = gs.rows2, let upAcc = gs.upAcc {
            try QWGemm.encodeMoEGroupPairsF32(enc, hal: hal, ids: gs.groupIds, expertOff: gOff, sortedPairIdx: gPair, sortedTok: gTok, experts: NG,
                                              totalPairs: gpairs, routes: NG, invPerm: gInv, tileE: gTE, tileR: gTR, tileCount: gTC)
            try QWGemm.encodeMoEGroupedGemm(enc, hal: hal, xe: x16, bank: gw.latentD, experts: NG, expertOff: gOff, tileE: gTE, tileR: gTR, tileCount: gTC,
                                            y: gs.xLatent16, pairs: gpairs, sortedTok: gTok)
            try QWGemm.encodeMoEGroupPairsF32(enc, hal: hal, ids: s.idx, expertOff: expOff, sortedPairIdx: sortedPair, sortedTok: sortedTok, experts: E,
                                              totalPairs: pairs, routes: K, invPerm: invPerm, tileE: tileE, tileR: tileR, tileCount: tileCount)
            try QWGemm.encodeMoEComposeRows(enc, hal: hal, sortedPair: sortedPair, pairs: pairs, pairRows: gs.pairRows, rowCount: gpairs, slotOfRow: gInv,
                                            rowsOut: rows2)
            try QWGemm.encodeMoEGateUpSwiglu(enc, hal: hal, xe: gs.xLatent16, bank: w.gateUp, experts: E, sortedTok: rows2, expertOff: expOff, tileE: tileE,
                                             tileR: tileR, tileCount: tileCount, act16: s.act16, pairs: pairs, rotateAct: w.down.isRotated)
            try QWGemm.encodeMoEGroupedGemm(enc, hal: hal, xe: s.act16, bank: w.down, experts: E, expertOff: expOff, tileE: tileE, tileR: tileR,
                                            tileCount: tileCount, y: dnHi, pairs: pairs)
            try QWGemm.encodeMoECombineGroupsF32(enc, hal: hal, dnAcc: dnHi, invPerm: invPerm, weights: s.wts, ids: s.idx, labels: gw.latentLabels,
                                                 tokens: T, routes: K, numGroups: NG, width: L, out: gs.zLatent16)
            try QWGemm.encodeMoEGroupedGemm(enc, hal: hal, xe: gs.zLatent16, bank: gw.latentU, experts: NG, expertOff: gOff, tileE: gTE, tileR: gTR,
                                            tileCount: gTC, y: upAcc, pairs: gpairs, sortedTok: gPair)
            try QWGemm.encodeMoEDownReduceCombineF32(enc, hal: hal, dnAcc: upAcc, invPerm: gInv, weights: gs.onesRoute, shared: shared, gate: gate,
                                                     out: out32, hidden: H, routes: NG, tokens: T)
        } else {
            try QWGemm.encodeMoERoutedGemv(enc, hal: hal, bank: gw.latentD, experts: NG, x16: x16, xPerToken: true, ids: gs.groupIds, weights: nil,
                                           tokens: T, routes: NG, out: gs.xLatent16)
            try QWGemm.encodeMoEGateUpRowsF32R1(enc, hal: hal, x: gs.xLatent16, bank: w.gateUp, experts: E, ids: s.idx, xRows: gs.pairRows, out: s.act16,
                                                routes: K, tokens: T)
            try QWGemm.encodeMoEDownGroupsF32(enc, hal: hal, x: s.act16, bank: w.down, experts: E, ids: s.idx, weights: s.wts, labels: gw.latentLabels,
                                              numGroups: NG, tokens: T, routes: K, out: gs.zLatent16)
            try QWGemm.encodeMoEDownSharedCombineF32(enc, hal: hal, x: gs.zLatent16, bank: gw.latentU, experts: NG, routes: NG, weights: gs.onesRoute,
                                                     shared: shared, gate: gate, out: out32, ids: gs.groupIds, tokens: T)
        }
    }
}
