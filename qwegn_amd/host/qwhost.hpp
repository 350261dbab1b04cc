// qwhost.hpp - host-side operator layer above the libqwhip C ABI, mirroring the reference's Swift operator API
// for the quantized matmul path name for name: QWHal, QWTensorValue, QWWeightView, QWGemm, QWGemmAQ, QWMoEOperator.
// Argument meaning and error behaviour follow the cited Swift sources: every check runs before the first launch
// and failures surface as the same typed errors (QWGemmError / QWHalError), so a failed encode leaves the stream
// untouched.  Header-only C++17; link against libqwhip.so.
//
// Paths cited below are relative to the reference checkout.
#pragma once
#include <cstdint>
#include <cstring>
#include <limits>
#include <optional>
#include <stdexcept>
#include <string>

#include "../../include/qwhip.h"

namespace qw {

// ---- QWDType (Sources/Foundation/QWCore/QWDType.swift) -----------------------------------------------------------
enum class QWDType { f32, f16, bf16, i32, q4g };
inline size_t dtypeBytes(QWDType d) { return d == QWDType::f32 || d == QWDType::i32 ? 4 : (d == QWDType::q4g ? 1 : 2); }
inline uint32_t abiDType(QWDType d) {
    switch (d) {
        case QWDType::f32: return QWHIP_F32;
        case QWDType::f16: return QWHIP_F16;
        case QWDType::bf16: return QWHIP_BF16;
        default: return QWHIP_I32;
    }
}

// ---- errors (QWGemm.swift:66-80, Sources/Foundation/QWHAL/QWHal.swift:60-77) ---------------------------------------
struct QWGemmError : std::runtime_error {
    enum Kind { f3Blocked, badWeights, badShape, badGeometry } kind;
    QWGemmError(Kind k, const std::string& s) : std::runtime_error(prefix(k) + s), kind(k) {}
    static std::string prefix(Kind k) {
        switch (k) {
            case f3Blocked: return "QWGEMM: F3 prefill path blocked - ";
            case badWeights: return "QWGEMM: weight view invalid - ";
            case badShape: return "QWGEMM: shape invalid - ";
            default: return "QWGEMM: geometry invalid - ";
        }
    }
};
struct QWHalError : std::runtime_error {
    enum Kind { deviceUnavailable, kernelMissing } kind;
    QWHalError(Kind k, const std::string& s) : std::runtime_error(s), kind(k) {}
};

// Maps a C-ABI status onto the Swift error cases; QWHIP_OK passes.
inline void throwIfFailed(qwhip_status st) {
    if (st == QWHIP_OK) return;
    const std::string msg = qwhip_last_error();
    switch (st) {
        case QWHIP_E_BAD_WEIGHTS: case QWHIP_E_NULL: case QWHIP_E_BASIS: throw QWGemmError(QWGemmError::badWeights, msg);
        case QWHIP_E_BAD_SHAPE: throw QWGemmError(QWGemmError::badShape, msg);
        case QWHIP_E_BAD_GEOMETRY: throw QWGemmError(QWGemmError::badGeometry, msg);
        case QWHIP_E_BLOCKED: throw QWGemmError(QWGemmError::f3Blocked, msg);
        case QWHIP_E_KERNEL_MISSING: throw QWHalError(QWHalError::kernelMissing, msg);
        default: throw QWHalError(QWHalError::deviceUnavailable, msg);
    }
}

// ---- QWTensorShape / QWTensorValue (Sources/Foundation/QWAlloc/QWArena.swift:36-151): non-owning typed region ----
struct QWTensorShape {
    size_t elementCount = 0;
    QWDType dtype = QWDType::f16;
};
struct QWTensorValue {
    void* base = nullptr;  // device pointer of the arena region
    size_t offset = 0;     // byte offset of this tensor inside the region
    size_t bytes = 0;      // bytes available from offset on
    QWTensorShape shape;
    void* ptr() const { return (uint8_t*)base + offset; }
    // x.slice(byteOffset:count:dtype:) (QWArena.swift:120-151)
    QWTensorValue slice(size_t byteOffset, size_t count, QWDType dtype) const {
        QWTensorValue t = *this;
        t.offset += byteOffset;
        t.bytes = bytes >= byteOffset ? bytes - byteOffset : 0;
        t.shape = {count, dtype};
        return t;
    }
    static QWTensorValue make(void* base, size_t count, QWDType dtype, size_t offset = 0) {
        return {base, offset, count * dtypeBytes(dtype), {count, dtype}};
    }
};

// ---- QWWeightView (Sources/Foundation/QWAlloc/QWWeightView.swift:9-152) -------------------------------------------
struct QWWeightView {
    struct ContainerKind {
        enum Tag { incumbentHQ4G32, rotatedHQ, nativeAffine } tag = incumbentHQ4G32;
        int bitsV = 4, groupV = 32;
        static ContainerKind incumbent() { return {incumbentHQ4G32, 4, 32}; }
        static ContainerKind rotated(int bits, int group) { return {rotatedHQ, bits, group}; }
        static ContainerKind affine(int bits, int group) { return {nativeAffine, bits, group}; }
        int bits() const { return bitsV; }
        int groupSize() const { return groupV; }
        bool isRotated() const { return tag != nativeAffine; }
        bool isIncumbentContainer() const { return tag == incumbentHQ4G32; }
        uint32_t abiKind() const { return tag == incumbentHQ4G32 ? QWHIP_KIND_HQ4_G32_M5 : (tag == rotatedHQ ? QWHIP_KIND_ROTATED_HQ : QWHIP_KIND_NATIVE_AFFINE); }
        std::string formatName() const {
            if (tag == incumbentHQ4G32) return "HQ4_G32";
            return std::string(tag == rotatedHQ ? "HQ" : "AQ") + std::to_string(bitsV) + "_G" + std::to_string(groupV);
        }
        int groupBytes() const { return (int)qwhip_block_bytes(abiKind(), (uint32_t)bitsV, (uint32_t)groupV); }  // 0 = unsupported
        size_t rowBytes(int k) const { return (size_t)(k / groupV) * (size_t)groupBytes(); }
    };

    QWTensorValue blocks;
    int n = 0, k = 0;
    ContainerKind containerKind;

    int bits() const { return containerKind.bits(); }
    int groupSize() const { return containerKind.groupSize(); }
    bool isRotated() const { return containerKind.isRotated(); }
    size_t rowBytes() const { return containerKind.rowBytes(k); }
    size_t requiredBytes() const { return rowBytes() * (size_t)n; }
    std::string formatName() const { return containerKind.formatName(); }

    // init?(blocks:n:k:containerKind:) - nullopt unless n > 0, k > 0, k % group == 0, the pair is supported and the bytes fit
    static std::optional<QWWeightView> make(const QWTensorValue& blocks, int n, int k, ContainerKind kind) {
        if (n <= 0 || k <= 0 || kind.groupSize() <= 0 || k % kind.groupSize() != 0) return std::nullopt;
        const int gb = kind.groupBytes();
        if (gb == 0) return std::nullopt;
        if (blocks.bytes < (size_t)n * (size_t)(k / kind.groupSize()) * (size_t)gb) return std::nullopt;
        QWWeightView v;
        v.blocks = blocks;
        v.n = n;
        v.k = k;
        v.containerKind = kind;
        return v;
    }
    // init?(blocks:n:k:bits:groupSize:isRotated:) - isRotated has no default: every construction states the basis
    static std::optional<QWWeightView> make(const QWTensorValue& blocks, int n, int k, int bits, int groupSize, bool isRotated,
                                            std::optional<bool> isIncumbentContainer = std::nullopt) {
        const bool incumbent = isIncumbentContainer.value_or(isRotated && bits == 4 && groupSize == 32);
        if (incumbent) {
            if (!(isRotated && bits == 4 && groupSize == 32)) return std::nullopt;
            return make(blocks, n, k, ContainerKind::incumbent());
        }
        return make(blocks, n, k, isRotated ? ContainerKind::rotated(bits, groupSize) : ContainerKind::affine(bits, groupSize));
    }
    std::optional<QWWeightView> subview(const QWTensorValue& b, int n2, int k2) const { return make(b, n2, k2, containerKind); }

    qwhip_weight_view abi() const {
        qwhip_weight_view w;
        w.blocks = blocks.ptr();
        w.bytes = blocks.bytes;
        w.n = (uint32_t)n;
        w.k = (uint32_t)k;
        w.kind = containerKind.abiKind();
        w.bits = (uint32_t)bits();
        w.group = (uint32_t)groupSize();
        return w;
    }
};

// ---- QWHal (Sources/Foundation/QWHAL/QWHal.swift:81-398): device + encoder (= stream) -----------------------------
struct QWHipEncoder {
    qwhip_stream_t stream = nullptr;
};
class QWHal {
public:
    explicit QWHal(int ordinal = 0) {
        qwhip_status st = qwhip_device_create(ordinal, &dev_);
        if (st != QWHIP_OK) throw QWHalError(QWHalError::deviceUnavailable, qwhip_last_error());
        qwhip_device_caps(dev_, &caps);
    }
    ~QWHal() {
        if (dev_) qwhip_device_destroy(dev_);
    }
    QWHal(const QWHal&) = delete;
    QWHal& operator=(const QWHal&) = delete;
    qwhip_caps caps{};
    // hal.pipeline(name): throws QWHalError.kernelMissing(name) (QWHal.swift:291-322); returns the serving launcher's name
    const char* pipeline(const char* name) const {
        const char* launcher = nullptr;
        if (qwhip_kernel_lookup(name, &launcher) != QWHIP_OK) throw QWHalError(QWHalError::kernelMissing, qwhip_last_error());
        return launcher;
    }
    QWHipEncoder begin() {  // hal.begin(): opens an encoder (QWHal.swift:325-350)
        QWHipEncoder e;
        throwIfFailed(qwhip_stream_create(dev_, &e.stream));
        return e;
    }
    void end(QWHipEncoder& e) {  // hal.end(): commit and wait (QWHal.swift:352-378)
        throwIfFailed(qwhip_stream_sync(e.stream));
        qwhip_stream_destroy(e.stream);
        e.stream = nullptr;
    }
    void* alloc(size_t bytes) {
        void* p = nullptr;
        throwIfFailed(qwhip_malloc(dev_, bytes, &p));
        return p;
    }
    void free(void* p) { qwhip_free(dev_, p); }
    qwhip_device_t device() const { return dev_; }
    // The geometry's gated FFN activation, which the reference bakes into its pipelines as function constants 224 / 228 / 229
    // (QWHal+Constants.swift:60-75; QWModelDescriptor.ActivationKind, QWModelDescriptor+Hybrid.swift:182-186)
    struct ActivationKind {
        enum Kind { swiglu, swigluClamped, situ } kind = swiglu;
        float a = 0.0f, b = 0.0f;   // swigluClamped: the limit; situ: beta, linearBeta
        static ActivationKind swiGLU() { return {}; }
        static ActivationKind clamped(float limit) { return {swigluClamped, limit, 0.0f}; }
        static ActivationKind situAndMul(float beta, float linearBeta) { return {situ, beta, linearBeta}; }
    };
    void setActivation(const ActivationKind& k) {
        throwIfFailed(qwhip_device_set_gated_activation(dev_, k.kind == ActivationKind::situ ? QWHIP_ACT_BOUNDED
                                                              : k.kind == ActivationKind::swigluClamped ? QWHIP_ACT_SWIGLU_CLAMPED
                                                                                                        : QWHIP_ACT_SWIGLU,
                                                        k.a, k.b));
    }

private:
    qwhip_device_t dev_ = nullptr;
};

// ---- QWGemm (Sources/Operators/QWGEMM/QWGemm.swift) ---------------------------------------------------------------
enum class QWGemmFamily { f1DecodeGemv, f2LmHeadGemv, f3PrefillGemm, f4AttentionTiles, f5SkinnyGemm };
enum class QWEpilogue { none, siluMulPair };

struct QWGemmShape {
    int m, n, k;
    QWGemmFamily family(std::optional<int> vocab = std::nullopt) const {  // QWGemm.swift:27-33
        if (m == 1 && vocab && n == *vocab) return QWGemmFamily::f2LmHeadGemv;
        if (m == 1) return QWGemmFamily::f1DecodeGemv;
        if (m >= 512) return QWGemmFamily::f3PrefillGemm;
        if (m <= 8) return QWGemmFamily::f5SkinnyGemm;
        return QWGemmFamily::f4AttentionTiles;
    }
};

struct QWGemmPlan {
    // The reference's backends (QWGemm.swift:36-61).  `mfmaGemmF16` is the one addition: the prefill door of this library
    // (planHip only; the reference's own F3 winner is the MPSGraph door `mpsGraphBmmF16`, which has no kernel to encode).
    enum class Backend { handQ4gV4, handQ4gV4H16, handQ4gSiluPair, handQ4gSiluPairH16, handQ4gSkinny, handF16V4, mpsF16,
                         mpsGraphBmmF16, blocked, mfmaGemmF16 };
    Backend backend;
    std::string kernel;  // the reference's kernel name: the key hal.pipeline() resolves
    int threadsPerTG;
    QWGemmFamily family;
    QWEpilogue epilogue;
};

struct QWGemm {
    static constexpr int maxConstantBytes = 256 * 1024;   // QWGemm.swift:90

    // Pure table lookup, row for row the reference's (QWGemm.swift:92-133): same backend, kernel name and threads per
    // threadgroup for every (family, dtype, epilogue, output dtype), `.blocked` wherever the reference blocks.
    static QWGemmPlan plan(const QWGemmShape& shape, QWDType dtype, QWEpilogue epi, QWDType outDtype = QWDType::f32,
                           std::optional<int> vocab = std::nullopt) {
        using B = QWGemmPlan::Backend;
        using F = QWGemmFamily;
        const F fam = shape.family(vocab);
        const QWGemmPlan blocked{B::blocked, "", 0, fam, epi};
        const bool decode = fam == F::f1DecodeGemv || fam == F::f2LmHeadGemv;
        if (dtype == QWDType::q4g && epi == QWEpilogue::siluMulPair)
            return outDtype == QWDType::f16 ? QWGemmPlan{B::handQ4gSiluPairH16, "qwg_gemv_q4g_silu_pair_h16", 64, fam, epi}
                                            : QWGemmPlan{B::handQ4gSiluPair, "qwg_gemv_q4g_silu_pair", 64, fam, epi};
        if (epi != QWEpilogue::none) return blocked;
        if (dtype == QWDType::q4g && decode)
            return outDtype == QWDType::f16 ? QWGemmPlan{B::handQ4gV4H16, "qwg_gemv_q4g_v4_h16", 32, fam, epi}
                                            : QWGemmPlan{B::handQ4gV4, "qwg_gemv_q4g_v4", 32, fam, epi};
        if (dtype == QWDType::q4g && fam == F::f5SkinnyGemm) {
            if ((shape.m == 2 || shape.m == 3) && shape.m * shape.k * 2 <= maxConstantBytes)
                return {B::handQ4gSkinny, shape.m == 2 ? "qwg_skinny_m2" : "qwg_skinny_m3", 32, fam, epi};
            return blocked;
        }
        if (dtype == QWDType::f16 && decode) return {B::handF16V4, "qwg_gemv_f16_v4", 32, fam, epi};
        if (dtype == QWDType::q4g && fam == F::f3PrefillGemm)
            return shape.k % 32 == 0 ? QWGemmPlan{B::mpsGraphBmmF16, "mpsgraph_bmm_f16", 0, fam, epi} : blocked;
        return blocked;
    }

    // This library's routing over the same shapes: where `plan` blocks or names a door that does not exist here, the kernels
    // of libqwhip take the call.  Differences from `plan`: the streaming GEMV takes every row count 2..16 in one pass (the
    // reference's skinny window is M in {2, 3}, its other F5 / F4 shapes are blocked), prefill and the remaining F4 shapes go
    // to the matrix-core GEMM when K % 64 == 0, the f16-weight GEMV and the MPSGraph door have no counterpart, and
    // threadsPerTG is the 256-thread workgroup of the HIP kernels.  encode / encodeH16 accept either plan.
    static QWGemmPlan planHip(const QWGemmShape& shape, QWDType dtype, QWEpilogue epi, QWDType outDtype = QWDType::f32,
                              std::optional<int> vocab = std::nullopt) {
        using B = QWGemmPlan::Backend;
        const QWGemmFamily fam = shape.family(vocab);
        if (dtype != QWDType::q4g) return {B::blocked, "", 0, fam, epi};
        if (epi == QWEpilogue::siluMulPair)
            return outDtype == QWDType::f16 ? QWGemmPlan{B::handQ4gSiluPairH16, "qwg_gemv_q4g_silu_pair_h16", 256, fam, epi}
                                            : QWGemmPlan{B::handQ4gSiluPair, "qwg_gemv_q4g_silu_pair", 256, fam, epi};
        switch (fam) {
            case QWGemmFamily::f1DecodeGemv:
            case QWGemmFamily::f2LmHeadGemv:
                return outDtype == QWDType::f16 ? QWGemmPlan{B::handQ4gV4H16, "qwg_gemv_q4g_v4_h16", 256, fam, epi}
                                                : QWGemmPlan{B::handQ4gV4, "qwg_gemv_q4g_v4", 256, fam, epi};
            case QWGemmFamily::f5SkinnyGemm:
                if (shape.m >= 2) return {B::handQ4gSkinny, shape.m == 3 ? "qwg_skinny_m3" : "qwg_skinny_m2", 256, fam, epi};
                return {B::blocked, "", 0, fam, epi};
            case QWGemmFamily::f3PrefillGemm:
                if (shape.k % 64 == 0) return {B::mfmaGemmF16, "qwg_gemm_q4g_h16", 256, fam, epi};
                return {B::blocked, "", 0, fam, epi};
            default:
                if (shape.m <= 16) return {B::handQ4gSkinny, "qwg_skinny_m2", 256, fam, epi};
                if (shape.k % 64 == 0) return {B::mfmaGemmF16, "qwg_gemm_q4g_h16", 256, fam, epi};
                return {B::blocked, "", 0, fam, epi};
        }
    }

    // Activations given to these doors are in the container's basis (the reference's producers rotate; pass
    // `rotateInKernel` to let the GEMV rotate un-rotated activations in its prologue instead).

    // QWGemm.encode (QWGemm.swift:218-283): f32 output; .siluMulPair needs even N and stores f16 activations.
    static void encode(QWHipEncoder& enc, const QWHal& hal, const QWGemmPlan& plan, const QWTensorValue& x, const QWWeightView& wQ4,
                       const QWTensorValue& y, int rows = 1, bool rotateInKernel = false, bool siluPairPlainOut = false) {
        // siluPairPlainOut: the .siluMulPair epilogue stores act in the plain basis instead of the next projection's; that
        // projection then rotates its input itself (rotateInKernel), which costs nothing at one row, and the gate|up bank is
        // read by the decode GEMV's own kernel (one row, HQ4_G32_M5: 20.7 against 25.6 us on 2 x 17408 x 5120).
        using B = QWGemmPlan::Backend;
        if (plan.backend == B::blocked) {
            if (plan.family == QWGemmFamily::f5SkinnyGemm) throw QWGemmError(QWGemmError::badWeights, "F5 window: run F1 per row");
            throw QWGemmError(QWGemmError::f3Blocked, "no winner raced for this family");
        }
        if (plan.backend == B::mfmaGemmF16 || plan.backend == B::mpsGraphBmmF16)
            throw QWGemmError(QWGemmError::f3Blocked, "plan resolved to the tensor GEMM - use gemmBatchedH16");
        if (plan.backend == B::handF16V4 || plan.backend == B::mpsF16)
            throw QWGemmError(QWGemmError::badWeights, "the f16-weight doors have no kernel in this library");
        if (plan.epilogue == QWEpilogue::siluMulPair && wQ4.n % 2 != 0) throw QWGemmError(QWGemmError::badWeights, "silu_pair needs even N");
        if (x.shape.dtype != QWDType::f16 && x.shape.dtype != QWDType::bf16) throw QWGemmError(QWGemmError::badWeights, "activations must be f16");
        if (x.shape.elementCount < (size_t)rows * (size_t)wQ4.k) throw QWGemmError(QWGemmError::badWeights, "activations are short");
        hal.pipeline(plan.kernel.c_str());
        const qwhip_weight_view w = wQ4.abi();
        const uint32_t flags = rotateInKernel ? 0u : (uint32_t)QWHIP_X_PREROTATED;
        if (plan.epilogue == QWEpilogue::siluMulPair) {
            if (y.shape.dtype != QWDType::f16 || y.shape.elementCount < (size_t)rows * (size_t)(wQ4.n / 2))
                throw QWGemmError(QWGemmError::badWeights, "silu_pair output must be f16 [rows, N/2]");
            throwIfFailed(qwhip_gemv_silu_pair(enc.stream, &w, x.ptr(), abiDType(x.shape.dtype), (uint32_t)rows, flags, siluPairPlainOut ? 0u : 1u, y.ptr()));
            return;
        }
        if (y.shape.dtype != QWDType::f32 || y.shape.elementCount < (size_t)rows * (size_t)wQ4.n)
            throw QWGemmError(QWGemmError::badWeights, "output must be f32 [rows, N]");
        throwIfFailed(qwhip_gemv(enc.stream, &w, x.ptr(), abiDType(x.shape.dtype), (uint32_t)rows, flags, nullptr, (float*)y.ptr()));
    }

    // QWGemm.encodeH16 (QWGemm.swift:137-214): direct f16 store, optional dual f32 store.
    static void encodeH16(QWHipEncoder& enc, const QWHal& hal, const QWGemmPlan& plan, const QWTensorValue& x, const QWWeightView& wQ4,
                          const QWTensorValue& y16, const QWTensorValue* y32 = nullptr, int rows = 1, bool rotateInKernel = false) {
        using B = QWGemmPlan::Backend;
        if (plan.backend != B::handQ4gV4H16 && plan.backend != B::handQ4gSiluPairH16 && plan.backend != B::handQ4gSkinny)
            throw QWGemmError(QWGemmError::badWeights, "encodeH16 requires handQ4gV4H16 or handQ4gSiluPairH16");
        if (y16.shape.dtype != QWDType::f16) throw QWGemmError(QWGemmError::badWeights, "y16 must have dtype .f16");
        if (plan.epilogue == QWEpilogue::siluMulPair) {
            encode(enc, hal, plan, x, wQ4, y16, rows, rotateInKernel);
            return;
        }
        if (x.shape.dtype != QWDType::f16 && x.shape.dtype != QWDType::bf16) throw QWGemmError(QWGemmError::badWeights, "activations must be f16");
        if (x.shape.elementCount < (size_t)rows * (size_t)wQ4.k) throw QWGemmError(QWGemmError::badWeights, "activations are short");
        if (y16.shape.elementCount < (size_t)rows * (size_t)wQ4.n) throw QWGemmError(QWGemmError::badWeights, "y16 is short");
        if (y32 && (y32->shape.dtype != QWDType::f32 || y32->shape.elementCount < (size_t)rows * (size_t)wQ4.n))
            throw QWGemmError(QWGemmError::badWeights, "y32 must be f32 [rows, N]");
        hal.pipeline(plan.kernel.c_str());
        const qwhip_weight_view w = wQ4.abi();
        const uint32_t flags = rotateInKernel ? 0u : (uint32_t)QWHIP_X_PREROTATED;
        throwIfFailed(qwhip_gemv(enc.stream, &w, x.ptr(), abiDType(x.shape.dtype), (uint32_t)rows, flags, y16.ptr(),
                                 y32 ? (float*)y32->ptr() : nullptr));
    }

    // QWGemm.encodeFwht32 (QWGemm.swift:288-300): in-place normalized FWHT-32 over f16 elements.
    static void encodeFwht32(QWHipEncoder& enc, const QWHal& hal, const QWTensorValue& x, std::optional<size_t> count = std::nullopt) {
        const size_t n = count.value_or(x.shape.elementCount);
        if (x.shape.dtype != QWDType::f16 || n == 0 || n % 32 != 0)
            throw QWGemmError(QWGemmError::badWeights, "fwht32 f16: n must be > 0 and divisible by 32");
        hal.pipeline("qwg_fwht32_f16");
        throwIfFailed(qwhip_fwht32(enc.stream, x.ptr(), QWHIP_F16, x.ptr(), n));
    }

    // QWGemm.encodeCast (QWGemm.swift:305-320): the f32 -> f16 seam.
    static void encodeCast(QWHipEncoder& enc, const QWHal& hal, const QWTensorValue& x32, const QWTensorValue& y16,
                           std::optional<size_t> count = std::nullopt) {
        const size_t n = count.value_or(x32.shape.elementCount);
        if (x32.shape.dtype != QWDType::f32 || y16.shape.dtype != QWDType::f16 || n == 0 || x32.shape.elementCount < n ||
            y16.shape.elementCount < n || n % 8 != 0)
            throw QWGemmError(QWGemmError::badWeights, "cast f32->f16: n must fit buffers and divide 8");
        hal.pipeline("qwg_cast_f32_to_f16");
        throwIfFailed(qwhip_cast_f32_to_f16(enc.stream, (const float*)x32.ptr(), y16.ptr(), n));
    }

    // gemmBatchedH16 (Sources/Runtime/QWEngine/Driver/EncodeKernels.swift:119-154) / QWGemm.encodeNaxF32
    // (Sources/Operators/QWGEMM/QWGemmF32.swift:366-402): Y[rows, n] = X[rows, k] . W^T on the matrix cores.
    static void gemmBatchedH16(QWHipEncoder& enc, const QWHal& hal, const QWTensorValue& x, const QWWeightView& w, const QWTensorValue& y,
                               int rows, const QWTensorValue* workspace = nullptr, bool rotateInPrepass = false) {
        if (rows <= 0) throw QWGemmError(QWGemmError::badShape, "rows must be positive");
        if (w.n % 64 != 0 || w.k % 64 != 0) throw QWGemmError(QWGemmError::badGeometry, "tensor GEMM needs N and K multiples of 64");
        if (x.shape.elementCount < (size_t)rows * (size_t)w.k) throw QWGemmError(QWGemmError::badWeights, "activations are short");
        if (y.shape.elementCount < (size_t)rows * (size_t)w.n) throw QWGemmError(QWGemmError::badWeights, "output is short");
        hal.pipeline(w.containerKind.isIncumbentContainer() ? "qwg_gemm_q4g_h16" : ("qwg_gemm_aq" + std::to_string(w.bits()) + "_g" + std::to_string(w.groupSize()) + "_h16").c_str());
        const qwhip_weight_view v = w.abi();
        throwIfFailed(qwhip_gemm(enc.stream, &v, x.ptr(), abiDType(x.shape.dtype), (uint32_t)rows, 0, y.ptr(), abiDType(y.shape.dtype), 0,
                                 rotateInPrepass ? 0u : (uint32_t)QWHIP_X_PREROTATED, workspace ? workspace->ptr() : nullptr,
                                 workspace ? workspace->bytes : 0));
    }

    // gemmBatchedH16SwiGLU (Sources/Runtime/QWEngine/Driver/EncodeKernels.swift:156-190, kernel qwg_gemm_*_h16_swiglu):
    // act16 [rows, inter] = FWHT32(silu(x . Wg^T) * (x . Wu^T)) from a [2 * inter, k] gate|up bank; false when the shape is outside
    // the fused kernel (the caller then runs gemmBatchedH16 + encodeSiluMulSplitF16).
    static bool gemmBatchedH16SwiGLU(QWHipEncoder& enc, const QWHal& hal, const QWTensorValue& x, const QWWeightView& w, const QWTensorValue& act16,
                                     int rows, bool rotate = true, const QWTensorValue* workspace = nullptr, bool rotateInPrepass = false) {
        if (rows <= 0) throw QWGemmError(QWGemmError::badShape, "rows must be positive");
        if (act16.shape.dtype != QWDType::f16 || act16.shape.elementCount < (size_t)rows * (size_t)(w.n / 2) ||
            x.shape.elementCount < (size_t)rows * (size_t)w.k)
            throw QWGemmError(QWGemmError::badWeights, "fused gate_up: x [rows, k], act f16 [rows, n / 2]");
        if (w.n % 64 != 0 || w.k % 64 != 0) return false;
        hal.pipeline(w.containerKind.isIncumbentContainer() ? "qwg_gemm_q4g_h16_swiglu"
                                                            : ("qwg_gemm_aq" + std::to_string(w.bits()) + "_g" + std::to_string(w.groupSize()) + "_h16_swiglu").c_str());
        const qwhip_weight_view v = w.abi();
        throwIfFailed(qwhip_gemm_swiglu(enc.stream, &v, x.ptr(), abiDType(x.shape.dtype), (uint32_t)rows, 0, rotate ? 1u : 0u, act16.ptr(), 0,
                                        rotateInPrepass ? 0u : (uint32_t)QWHIP_X_PREROTATED, workspace ? workspace->ptr() : nullptr,
                                        workspace ? workspace->bytes : 0));
        return true;
    }

    // QWGemm.encodeSiluMulF16 / encodeSiluMulSplitF16 (QWGemmF32.swift:47-115): SwiGLU (+FWHT-32) over gate|up rows.
    static void encodeSiluMulSplitF16(QWHipEncoder& enc, const QWHal& hal, const QWTensorValue& gu, const QWTensorValue& act16, int rows,
                                      int inter, bool rotate = true) {
        if (act16.shape.dtype != QWDType::f16 || act16.shape.elementCount < (size_t)rows * (size_t)inter ||
            gu.shape.elementCount < (size_t)rows * 2 * (size_t)inter)
            throw QWGemmError(QWGemmError::badShape, "silu_mul: buffers do not fit rows x intermediate");
        hal.pipeline("qwg_silu_mul_split_f16");
        throwIfFailed(qwhip_swiglu_fwht(enc.stream, gu.ptr(), abiDType(gu.shape.dtype), act16.ptr(), (uint32_t)rows, (uint32_t)inter, rotate ? 1 : 0));
    }

    // QWGemm.encodeSiluMulF32 (QWGemmF32.swift:83-94): f32 gate|up -> silu(g) * u + H_32, f32 out, or f16 out when act16 is given
    static void encodeSiluMulF32(QWHipEncoder& enc, const QWHal& hal, const QWTensorValue& gu, const QWTensorValue& act, int rows, int inter,
                                 const QWTensorValue* act16 = nullptr) {
        if (inter % 32 != 0) throw QWGemmError(QWGemmError::badShape, "f32 silu-mul needs intermediate % 32 == 0");
        if (gu.shape.dtype != QWDType::f32 || gu.shape.elementCount < (size_t)rows * 2 * (size_t)inter)
            throw QWGemmError(QWGemmError::badShape, "f32 silu-mul: gate|up must be f32 [rows, 2 intermediate]");
        hal.pipeline("qwg_silu_mul_f32");
        if (act16) {
            if (act16->shape.dtype != QWDType::f16 || act16->shape.elementCount < (size_t)rows * (size_t)inter)
                throw QWGemmError(QWGemmError::badShape, "f32 silu-mul: act16 must be f16 [rows, intermediate]");
            throwIfFailed(qwhip_swiglu_fwht(enc.stream, gu.ptr(), QWHIP_F32, act16->ptr(), (uint32_t)rows, (uint32_t)inter, 1));
        } else {
            if (act.shape.dtype != QWDType::f32 || act.shape.elementCount < (size_t)rows * (size_t)inter)
                throw QWGemmError(QWGemmError::badShape, "f32 silu-mul: act must be f32 [rows, intermediate]");
            throwIfFailed(qwhip_silu_mul_f32(enc.stream, (const float*)gu.ptr(), (float*)act.ptr(), (uint32_t)rows, (uint32_t)inter));
        }
    }
    // QWGemm.encodeEmbedBf16F32 (QWGemmF32.swift:352-363): the token's row of a raw bf16 table widened to f32, written hc times
    static void encodeEmbedBf16F32(QWHipEncoder& enc, const QWHal& hal, const QWTensorValue& table, const QWTensorValue& token, const QWTensorValue& out,
                                   int hidden, int hc, int rows = 1) {
        if (hidden <= 0 || hc <= 0 || rows <= 0 || table.shape.dtype != QWDType::bf16 || table.shape.elementCount < (size_t)hidden ||
            token.shape.elementCount < (size_t)rows || out.shape.dtype != QWDType::f32 || out.shape.elementCount < (size_t)rows * (size_t)hidden * (size_t)hc)
            throw QWGemmError(QWGemmError::badShape, "bf16 embedding gather: table bf16 [vocab, hidden], out f32 [rows, hc, hidden]");
        hal.pipeline("qwg_embed_bf16_f32");
        throwIfFailed(qwhip_embed_bf16_f32(enc.stream, table.ptr(), (uint32_t)(table.shape.elementCount / (size_t)hidden), (uint32_t)hidden,
                                           (const int32_t*)token.ptr(), (uint32_t)rows, (uint32_t)hc, (float*)out.ptr()));
    }
    // QWGemm.encodeAddF32 (QWGemmF32.swift:108-115)
    static void encodeAddF32(QWHipEncoder& enc, const QWHal& hal, const QWTensorValue& a, const QWTensorValue& b, const QWTensorValue& out, size_t count) {
        if (a.shape.elementCount < count || b.shape.elementCount < count || out.shape.elementCount < count || a.shape.dtype != QWDType::f32 ||
            b.shape.dtype != QWDType::f32 || out.shape.dtype != QWDType::f32)
            throw QWGemmError(QWGemmError::badShape, "add: f32 buffers of at least count values");
        hal.pipeline("qwg_add_f32");
        throwIfFailed(qwhip_add_f32(enc.stream, (const float*)a.ptr(), (const float*)b.ptr(), (float*)out.ptr(), (uint64_t)count));
    }
    // QWGemm.encodeLatentNormH32F32 (QWGemmF32.swift:57-80): optional RMSNorm (1 + gamma) + H_32 on f32 [rows, latent] -> f32 and/or f16
    static void encodeLatentNormH32F32(QWHipEncoder& enc, const QWHal& hal, const QWTensorValue& x, const QWTensorValue* gamma,
                                       const QWTensorValue& out32, const QWTensorValue* out16, int rows, int latent, float eps = 1e-6f,
                                       bool skipOut32 = false) {
        if (latent <= 0 || latent % 32 != 0) throw QWGemmError(QWGemmError::badShape, "latent norm H32 needs latent % 32 == 0");
        const size_t need = (size_t)rows * (size_t)latent;
        if (x.shape.dtype != QWDType::f32 || x.shape.elementCount < need || (gamma && (gamma->shape.dtype != QWDType::f16 || gamma->shape.elementCount < (size_t)latent)) ||
            (!skipOut32 && (out32.shape.dtype != QWDType::f32 || out32.shape.elementCount < need)) ||
            (out16 && (out16->shape.dtype != QWDType::f16 || out16->shape.elementCount < need)))
            throw QWGemmError(QWGemmError::badShape, "latent norm: buffers do not fit rows x latent");
        hal.pipeline("qwg_latent_norm_h32_f32");
        throwIfFailed(qwhip_latent_norm_h32_f32(enc.stream, (const float*)x.ptr(), gamma ? gamma->ptr() : nullptr, skipOut32 ? nullptr : (float*)out32.ptr(),
                                                out16 ? out16->ptr() : nullptr, (uint32_t)rows, (uint32_t)latent, eps));
    }
    // QWGemm.encodeMoEBridgeF16ToF32 (QWGemmMoE.swift:337-377): f16 normed hidden -> rotated f32 copy + un-rotated f32 copy
    static void encodeMoEBridgeF16ToF32(QWHipEncoder& enc, const QWHal& hal, const QWTensorValue& x, const QWTensorValue& xRot32,
                                        const QWTensorValue& xPlain32, int rows, int hidden, bool skipRot32 = false) {
        if (rows <= 0 || hidden <= 0) throw QWGemmError(QWGemmError::badGeometry, "moe bridge: rows and hidden must be positive");
        if (hidden % 256 != 0) throw QWGemmError(QWGemmError::badGeometry, "moe bridge: hidden must be a multiple of 256");
        const size_t need = (size_t)rows * (size_t)hidden;
        if (x.shape.dtype != QWDType::f16 || xRot32.shape.dtype != QWDType::f32 || xPlain32.shape.dtype != QWDType::f32 ||
            x.shape.elementCount < need || xRot32.shape.elementCount < need || xPlain32.shape.elementCount < need)
            throw QWGemmError(QWGemmError::badShape, "moe bridge: rows x hidden do not fit the buffers");
        hal.pipeline("qwg_moe_bridge_f16_to_f32");
        throwIfFailed(qwhip_moe_bridge_f16_to_f32(enc.stream, x.ptr(), skipRot32 ? nullptr : (float*)xRot32.ptr(), (float*)xPlain32.ptr(),
                                                  (uint32_t)rows, (uint32_t)hidden));
    }

    // QWGemm.encodeHQ4F32V4 / encodeHQ4F32BM (Sources/Operators/QWGEMM/QWGemmF32.swift:178-199,311-350): f32 activations in the
    // container's basis -> f32 outputs; epi 0 none, 1 silu(y/scale), 2 sigmoid, 3 silu(y/scale) + H_32.
    static void encodeHQ4F32V4(QWHipEncoder& enc, const QWHal& hal, const QWWeightView& w, const QWTensorValue& x, const QWTensorValue& y,
                               int rows = 1, uint32_t epi = 0, float scale = 1.0f) {
        if (rows <= 0) throw QWGemmError(QWGemmError::badShape, "rows must be positive");
        if (x.shape.dtype != QWDType::f32 || y.shape.dtype != QWDType::f32 || x.shape.elementCount < (size_t)rows * (size_t)w.k ||
            y.shape.elementCount < (size_t)rows * (size_t)w.n)
            throw QWGemmError(QWGemmError::badWeights, "f32 v4: x f32 [rows, K], y f32 [rows, N]");
        hal.pipeline(w.containerKind.isIncumbentContainer()
                         ? "qwg_gemv_q4g_f32_v4"
                         : ("qwg_gemv_aq" + std::to_string(w.bits()) + "_g" + std::to_string(w.groupSize()) + "_f32_v4").c_str());
        const qwhip_weight_view v = w.abi();
        throwIfFailed(qwhip_gemv_f32(enc.stream, &v, (const float*)x.ptr(), (uint32_t)rows, epi, scale, (float*)y.ptr()));
    }

    // QWGemm.encodeDenseProjF32 (QWGemmF32.swift:413-440): the unified dense projection over `rows` f32 activations in the
    // container's basis.  rows >= minNaxRows with no epilogue: cast to f16 in `naxX16` (rows * k halves, or the caller's
    // `x16Precast`) and run the matrix-core GEMM into the f32 output; otherwise the f32 GEMV family (its batched form for
    // 32 rows and more is the same four-rows-per-pass kernel here).
    static void encodeDenseProjF32(QWHipEncoder& enc, const QWHal& hal, const QWWeightView& w, const QWTensorValue& x, const QWTensorValue& y,
                                   const QWTensorValue& naxX16, int rows, uint32_t epi = 0, float scale = 1.0f,
                                   const QWTensorValue* x16Precast = nullptr, int minNaxRows = 64) {
        const int effectiveMinNax = minNaxRows > 64 ? minNaxRows : 64;
        if (rows >= effectiveMinNax && epi == 0 && scale == 1.0f && w.n % 64 == 0 && w.k % 64 == 0) {
            const size_t count = (size_t)rows * (size_t)w.k;
            if (x16Precast) {
                gemmBatchedH16(enc, hal, x16Precast->slice(0, count, QWDType::f16), w, y, rows);
            } else {
                if (naxX16.shape.elementCount < count) throw QWGemmError(QWGemmError::badWeights, "dense proj: the f16 staging buffer is short");
                const QWTensorValue xHi = naxX16.slice(0, count, QWDType::f16);
                encodeCast(enc, hal, x, xHi, count);
                gemmBatchedH16(enc, hal, xHi, w, y, rows);
            }
        } else {
            encodeHQ4F32V4(enc, hal, w, x, y, rows, epi, scale);
        }
    }

    // QWGemm.encodeH32F32 (QWGemmF32.swift:46-54): out f32 [rows, hidden] = rotate(x) in the normalised Walsh-Hadamard domain.
    static void encodeH32F32(QWHipEncoder& enc, const QWHal& hal, const QWTensorValue& x, const QWTensorValue& out, int rows, int hidden) {
        if (x.shape.dtype != QWDType::f32 || out.shape.dtype != QWDType::f32 || rows <= 0 || hidden <= 0 || hidden % 32 != 0 ||
            x.shape.elementCount < (size_t)rows * (size_t)hidden || out.shape.elementCount < (size_t)rows * (size_t)hidden)
            throw QWGemmError(QWGemmError::badShape, "h32 f32: f32 [rows, hidden], hidden % 32 == 0");
        hal.pipeline("qwg_h32_f32");
        throwIfFailed(qwhip_h32_f32(enc.stream, (const float*)x.ptr(), (float*)out.ptr(), (uint32_t)rows, (uint32_t)hidden));
    }

    // encodeRMSNormFast / encodeRMSNormResidualFast (Sources/Runtime/QWEngine/Driver/EncodeKernels.swift:339-404): y16 = rotate?(
    // rmsnorm(x [+ residual]) * (1 + gamma)); with `residual` the sum is written back to it.
    static void encodeRMSNormFast(QWHipEncoder& enc, const QWHal& hal, const QWTensorValue& x, const QWTensorValue& gamma,
                                  const QWTensorValue& y, int rows, int hidden, float eps, bool rotate = true,
                                  const QWTensorValue* residual = nullptr) {
        if (x.shape.dtype != QWDType::f16 || gamma.shape.dtype != QWDType::f16 || y.shape.dtype != QWDType::f16 ||
            (residual && residual->shape.dtype != QWDType::f16) || rows <= 0 || x.shape.elementCount < (size_t)rows * (size_t)hidden ||
            y.shape.elementCount < (size_t)rows * (size_t)hidden || gamma.shape.elementCount < (size_t)hidden)
            throw QWGemmError(QWGemmError::badShape, "rmsnorm: f16 [rows, hidden] in and out, f16 gamma [hidden]");
        hal.pipeline(residual ? "qwg_rmsnorm_residual" : "qwg_rmsnorm");
        throwIfFailed(qwhip_rmsnorm(enc.stream, x.ptr(), gamma.ptr(), residual ? residual->ptr() : nullptr, (uint32_t)rows, (uint32_t)hidden,
                                    eps, rotate ? 1u : 0u, y.ptr()));
    }

    // ---- MoE encoders (Sources/Operators/QWGEMM/QWGemmMoE.swift, QWGemmMoERouter.swift) ----------------------------
    // encodeF32Gemv (QWGemmF32.swift:117-141): dense fp32 weights [n, k], epilogues 0 none, 1 silu(y / scale), 2 sigmoid, 3 2 sigmoid(y / scale)
    static void encodeF32Gemv(QWHipEncoder& enc, const QWHal& hal, const QWTensorValue& weight, const QWTensorValue& x, const QWTensorValue& y,
                              int rows, int n, int k, uint32_t epilogue, float scale) {
        if (weight.shape.dtype != QWDType::f32 || x.shape.dtype != QWDType::f32 || y.shape.dtype != QWDType::f32 ||
            weight.shape.elementCount < (size_t)n * (size_t)k || x.shape.elementCount < (size_t)rows * (size_t)k ||
            y.shape.elementCount < (size_t)rows * (size_t)n)
            throw QWGemmError(QWGemmError::badShape, "f32 gemv: f32 weight [n, k], x [rows, k], y [rows, n]");
        hal.pipeline(rows >= 4 ? "qwg_f32_gemv_bm" : "qwg_f32_gemv");
        throwIfFailed(qwhip_f32_gemv(enc.stream, (const float*)weight.ptr(), (const float*)x.ptr(), (uint32_t)rows, (uint32_t)n, (uint32_t)k,
                                     epilogue, scale, (float*)y.ptr()));
    }
    // encodeArgmaxFin (QWGemmF32.swift:276-307) over f32 logits [rows, vocab]: the plain fold, or the relaxed acceptance of a draft
    // (QWVariationalAcceptance: logits, draftTokens u32 [totalRows], margin, minLogProb) when margin > 0 and rows > 1
    struct QWVariationalAcceptance {
        QWTensorValue draftTokens;
        int totalRows = 0;
        float margin = 0.0f;
        float minLogProb = -std::numeric_limits<float>::infinity();
    };
    static void encodeArgmaxFin(QWHipEncoder& enc, const QWHal& hal, const QWTensorValue& logits, const QWTensorValue& token, int vocab, int rows = 1,
                                const QWVariationalAcceptance* variational = nullptr) {
        if (logits.shape.dtype != QWDType::f32 || logits.shape.elementCount < (size_t)rows * (size_t)vocab || token.shape.elementCount < (size_t)rows)
            throw QWGemmError(QWGemmError::badShape, "argmax-fin: logits f32 [rows, vocab], token [rows]");
        if (variational && variational->margin > 0 && rows > 1) {
            if (variational->draftTokens.shape.elementCount < (size_t)variational->totalRows)
                throw QWGemmError(QWGemmError::badShape, "argmax-fin: draft tokens are short");
            hal.pipeline("qwg_head_argmax_fin_variational");
            throwIfFailed(qwhip_argmax_f32_variational(enc.stream, (const float*)logits.ptr(), (uint32_t)rows, (uint32_t)vocab,
                                                       (const uint32_t*)variational->draftTokens.ptr(), (uint32_t)variational->totalRows,
                                                       variational->margin, variational->minLogProb, (int32_t*)token.ptr()));
        } else {
            hal.pipeline("qwg_head_argmax_fin");
            throwIfFailed(qwhip_argmax_f32(enc.stream, (const float*)logits.ptr(), (uint32_t)rows, (uint32_t)vocab, (int32_t*)token.ptr()));
        }
    }
    static int moeMaxTiles(int experts, int pairs) { return (int)qwhip_moe_max_tiles((uint32_t)experts, (uint32_t)pairs); }  // QWGemmMoE.swift:24-26

    // encodeFnRouterGemm (QWGemmMoERouter.swift:78-113)
    // shGateWeight f32 [hidden] + shGateOut f32 [rows]: the shared-expert gate sigmoid(x . w) as an extra output column
    static void encodeFnRouterGemm(QWHipEncoder& enc, const QWHal& hal, const QWTensorValue& x, const QWTensorValue& router,
                                   const QWTensorValue& logits, int rows, int experts, int hidden,
                                   const QWTensorValue* shGateWeight = nullptr, const QWTensorValue* shGateOut = nullptr) {
        if (logits.shape.dtype != QWDType::f32 || logits.shape.elementCount < (size_t)rows * (size_t)experts)
            throw QWGemmError(QWGemmError::badShape, "router logits must be f32 [rows, experts]");
        const bool hasShGate = shGateWeight && shGateOut;   // as the reference: one without the other means no gate column
        if (hasShGate && (shGateWeight->shape.dtype != QWDType::f32 || shGateWeight->shape.elementCount < (size_t)hidden ||
                          shGateOut->shape.dtype != QWDType::f32 || shGateOut->shape.elementCount < (size_t)rows))
            throw QWGemmError(QWGemmError::badShape, "shared-expert gate: f32 weight [hidden] and f32 output [rows]");
        hal.pipeline("qwg_router_gemm");
        throwIfFailed(qwhip_router_gemm_shared_gate(enc.stream, x.ptr(), abiDType(x.shape.dtype), router.ptr(), abiDType(router.shape.dtype),
                                                    (uint32_t)rows, (uint32_t)experts, (uint32_t)hidden, (float*)logits.ptr(),
                                                    hasShGate ? (const float*)shGateWeight->ptr() : nullptr,
                                                    hasShGate ? (float*)shGateOut->ptr() : nullptr));
    }
    // encodeFnMoeRoute (QWGemmMoERouter.swift:10-75)
    // bias (f32 [experts]) and / or splitFeature (logits [rows, 2 experts]) switch to sigmoid scoring; routedScaleParam (f32 [experts])
    // replaces the routed scale per selected expert
    static void encodeFnMoeRoute(QWHipEncoder& enc, const QWHal& hal, const QWTensorValue& logits, const QWTensorValue& idx,
                                 const QWTensorValue& wts, int rows, int experts, int topK, bool normTopK, float routedScale = 1.0f,
                                 const QWTensorValue* bias = nullptr, bool splitFeature = false, const QWTensorValue* routedScaleParam = nullptr,
                                 int expertBudget = 0) {
        if (experts > 512 || topK > 16 || topK <= 0) throw QWGemmError(QWGemmError::badShape, "router holds 512 experts and 16 routes");
        if (idx.shape.elementCount < (size_t)rows * (size_t)topK || wts.shape.elementCount < (size_t)rows * (size_t)topK)
            throw QWGemmError(QWGemmError::badShape, "router outputs are short");
        if (logits.shape.elementCount < (size_t)rows * (size_t)experts * (splitFeature ? 2u : 1u) ||
            (bias && (bias->shape.dtype != QWDType::f32 || bias->shape.elementCount < (size_t)experts)) ||
            (routedScaleParam && (routedScaleParam->shape.dtype != QWDType::f32 || routedScaleParam->shape.elementCount < (size_t)experts)))
            throw QWGemmError(QWGemmError::badShape, "router inputs are short");
        hal.pipeline("qwg_moe_route");
        if (!bias && !splitFeature && !routedScaleParam) {
            throwIfFailed(qwhip_moe_route(enc.stream, (const float*)logits.ptr(), (uint32_t)rows, (uint32_t)experts, (uint32_t)topK, normTopK ? 1 : 0,
                                          routedScale, (int32_t*)idx.ptr(), (float*)wts.ptr()));
        } else {
            throwIfFailed(qwhip_moe_route_ex(enc.stream, (const float*)logits.ptr(), (uint32_t)rows, (uint32_t)experts, (uint32_t)topK, normTopK ? 1 : 0,
                                             routedScale, splitFeature ? 1u : 0u, bias ? (const float*)bias->ptr() : nullptr,
                                             routedScaleParam ? (const float*)routedScaleParam->ptr() : nullptr, (int32_t*)idx.ptr(),
                                             (float*)wts.ptr()));
        }
        // the expert budget of a verify window (QWGemmMoERouter.swift:63-75): the door's own condition, silently skipped otherwise
        if (expertBudget > 0 && rows > 1 && rows <= 4 && expertBudget < rows * topK && rows * topK <= 64)
            throwIfFailed(qwhip_moe_route_budget(enc.stream, (int32_t*)idx.ptr(), (float*)wts.ptr(), (uint32_t)rows, (uint32_t)topK,
                                                 (uint32_t)expertBudget, normTopK ? 1 : 0));
    }
    // encodeMoEGroupPairsF32 (QWGemmMoE.swift:68-99)
    static void encodeMoEGroupPairsF32(QWHipEncoder& enc, const QWHal& hal, const QWTensorValue& ids, const QWTensorValue& expertOff,
                                       const QWTensorValue& sortedPairIdx, const QWTensorValue& sortedTok, int experts, int totalPairs,
                                       int routes, const QWTensorValue* invPerm = nullptr, const QWTensorValue* tileE = nullptr,
                                       const QWTensorValue* tileR = nullptr, const QWTensorValue* tileCount = nullptr, bool compactTail = true) {
        if (experts > 512) throw QWGemmError(QWGemmError::badShape, "the expert-sorted pair order holds 512 experts");
        const bool hasTiles = tileE && tileR && tileCount;
        if (hasTiles && (tileE->shape.elementCount < (size_t)moeMaxTiles(experts, totalPairs) ||
                         tileR->shape.elementCount < (size_t)moeMaxTiles(experts, totalPairs)))
            throw QWGemmError(QWGemmError::badShape, "moe group pairs: tile scratch does not fit the tile plan");
        hal.pipeline("qwg_moe_group_pairs_f32");
        throwIfFailed(qwhip_moe_group_pairs(enc.stream, (const int32_t*)ids.ptr(), (uint32_t)experts, (uint32_t)totalPairs, (uint32_t)routes,
                                            (int32_t*)expertOff.ptr(), (int32_t*)sortedPairIdx.ptr(), (int32_t*)sortedTok.ptr(),
                                            invPerm ? (int32_t*)invPerm->ptr() : nullptr, hasTiles ? (int32_t*)tileE->ptr() : nullptr,
                                            hasTiles ? (int32_t*)tileR->ptr() : nullptr, hasTiles ? (int32_t*)tileCount->ptr() : nullptr,
                                            compactTail ? 1 : 0));
    }
    // encodeMoEGateUpNax / encodeMoENaxSplitF32 (QWGemmMoE.swift:201-296): grouped expert GEMM over the sorted pairs
    static void encodeMoEGroupedGemm(QWHipEncoder& enc, const QWHal& hal, const QWWeightView& w, int experts, const QWTensorValue& x,
                                     const QWTensorValue* gather, const QWTensorValue& expertOff, const QWTensorValue& tileE,
                                     const QWTensorValue& tileR, const QWTensorValue& tileCount, int pairs, const QWTensorValue& y) {
        hal.pipeline(gather ? "qwg_moe_nax_gemm" : "qwg_moe_nax_split_f32");
        const qwhip_weight_view v = w.abi();
        throwIfFailed(qwhip_moe_grouped_gemm(enc.stream, &v, (uint32_t)experts, x.ptr(), abiDType(x.shape.dtype), 0,
                                             gather ? (const int32_t*)gather->ptr() : nullptr, (const int32_t*)expertOff.ptr(),
                                             (const int32_t*)tileE.ptr(), (const int32_t*)tileR.ptr(), (const int32_t*)tileCount.ptr(),
                                             (uint32_t)moeMaxTiles(experts, pairs), (uint32_t)pairs, y.ptr(), abiDType(y.shape.dtype), 0));
    }
    // The prefill pair encodeMoEGateUpNax + encodeSiluMul* as one launch: act16 [pairs, inter] = FWHT32(silu(g) * u) of the sorted
    // pairs, bit-identical to the two encoders above (f16 activations; inter % 32 == 0).
    static void encodeMoEGateUpSwiglu(QWHipEncoder& enc, const QWHal& hal, const QWWeightView& w, int experts, const QWTensorValue& x,
                                      const QWTensorValue& gather, const QWTensorValue& expertOff, const QWTensorValue& tileE,
                                      const QWTensorValue& tileR, const QWTensorValue& tileCount, int pairs, const QWTensorValue& act16,
                                      bool rotate = true) {
        if (x.shape.dtype != QWDType::f16 || act16.shape.dtype != QWDType::f16)
            throw QWGemmError(QWGemmError::badShape, "fused gate_up: f16 activations in, f16 act out");
        if (experts <= 0 || w.n % experts != 0 || act16.shape.elementCount < (size_t)pairs * (size_t)(w.n / experts / 2))
            throw QWGemmError(QWGemmError::badShape, "fused gate_up: act does not fit pairs x intermediate");
        hal.pipeline("qwg_moe_nax_gemm");
        hal.pipeline("qwg_silu_mul_f16");
        const qwhip_weight_view v = w.abi();
        throwIfFailed(qwhip_moe_grouped_gemm_swiglu(enc.stream, &v, (uint32_t)experts, x.ptr(), QWHIP_F16, 0, (const int32_t*)gather.ptr(),
                                                    (const int32_t*)expertOff.ptr(), (const int32_t*)tileE.ptr(), (const int32_t*)tileR.ptr(),
                                                    (const int32_t*)tileCount.ptr(), (uint32_t)moeMaxTiles(experts, pairs), (uint32_t)pairs,
                                                    rotate ? 1u : 0u, act16.ptr(), 0));
    }
    // encodeMoEDownReduceCombineF32 (QWGemmMoE.swift:299-332)
    static void encodeMoEDownReduceCombineF32(QWHipEncoder& enc, const QWHal& hal, const QWTensorValue& dn, const QWTensorValue& invPerm,
                                              const QWTensorValue& wts, int rows, int topK, int hidden, const QWTensorValue* shared,
                                              const QWTensorValue* sharedGate, const QWTensorValue& out) {
        hal.pipeline("qwg_moe_down_reduce_combine_f32");
        throwIfFailed(qwhip_moe_combine(enc.stream, dn.ptr(), abiDType(dn.shape.dtype), (const int32_t*)invPerm.ptr(), (const float*)wts.ptr(),
                                        (uint32_t)rows, (uint32_t)topK, (uint32_t)hidden, shared ? (const float*)shared->ptr() : nullptr,
                                        sharedGate ? (const float*)sharedGate->ptr() : nullptr, out.ptr(), abiDType(out.shape.dtype)));
    }
    // the door's invPerm: nil + unweightedSingle form (QWGemmMoE.swift:299-332): out = dn + sharedGate * shared, one row per token
    static void encodeMoEAddSharedF32(QWHipEncoder& enc, const QWHal& hal, const QWTensorValue& dn, int rows, int hidden,
                                      const QWTensorValue& shared, const QWTensorValue* sharedGate, const QWTensorValue& out) {
        const size_t need = (size_t)rows * (size_t)hidden;
        if (dn.shape.elementCount < need || shared.shape.dtype != QWDType::f32 || shared.shape.elementCount < need ||
            out.shape.elementCount < need || (sharedGate && (sharedGate->shape.dtype != QWDType::f32 || sharedGate->shape.elementCount < (size_t)rows)))
            throw QWGemmError(QWGemmError::badShape, "moe shared add: buffers do not fit rows x hidden");
        hal.pipeline("qwg_moe_down_reduce_combine_f32");
        throwIfFailed(qwhip_moe_combine(enc.stream, dn.ptr(), abiDType(dn.shape.dtype), nullptr, nullptr, (uint32_t)rows, 1u, (uint32_t)hidden,
                                        (const float*)shared.ptr(), sharedGate ? (const float*)sharedGate->ptr() : nullptr, out.ptr(),
                                        abiDType(out.shape.dtype)));
    }
    // encodeFnMoeRoute + encodeMoEGateUpF32R1 as one launch (decode / verify): idx / wts are left for the down projection
    static void encodeMoERouteGateUp(QWHipEncoder& enc, const QWHal& hal, const QWWeightView& gateUp, int experts, const QWTensorValue& x,
                                     const QWTensorValue& logits, const QWTensorValue& idx, const QWTensorValue& wts, int rows, int topK,
                                     bool normTopK, float routedScale, const QWTensorValue& act16, bool rotateInKernel = false,
                                     bool reuseExpertsAcrossTokens = false) {
        if (logits.shape.dtype != QWDType::f32 || logits.shape.elementCount < (size_t)rows * (size_t)experts ||
            idx.shape.elementCount < (size_t)rows * (size_t)topK || wts.shape.elementCount < (size_t)rows * (size_t)topK)
            throw QWGemmError(QWGemmError::badShape, "moe route: logits f32 [rows, experts], idx / wts [rows, topK]");
        hal.pipeline("qwg_moe_route");
        hal.pipeline("qwg_moe_gateup_q4g_f32_r1");
        const qwhip_weight_view v = gateUp.abi();
        throwIfFailed(qwhip_moe_route_gateup_decode(enc.stream, &v, (uint32_t)experts, x.ptr(), abiDType(x.shape.dtype),
                                                    (rotateInKernel ? 0u : (uint32_t)QWHIP_X_PREROTATED) |
                                                        (reuseExpertsAcrossTokens ? (uint32_t)QWHIP_MOE_REUSE_EXPERTS : 0u),
                                                    (const float*)logits.ptr(), (uint32_t)rows,
                                                    (uint32_t)topK, normTopK ? 1 : 0, routedScale, (int32_t*)idx.ptr(), (float*)wts.ptr(),
                                                    act16.ptr()));
    }
    // encodeMoEGateUpF32R1 / encodeMoEDownSharedCombineF32 (QWGemmMoE.swift:120-199): decode / verify, rows <= 8
    static void encodeMoEGateUpF32R1(QWHipEncoder& enc, const QWHal& hal, const QWWeightView& gateUp, int experts, const QWTensorValue& x,
                                     const QWTensorValue& idx, int rows, int topK, const QWTensorValue& act16, bool rotateInKernel = false,
                                     bool reuseExpertsAcrossTokens = false) {
        // reuseExpertsAcrossTokens (QWGemmMoE.swift:119-132): default true in the reference, false here (same bits, slower launch)
        hal.pipeline("qwg_moe_gateup_q4g_f32_r1");
        const qwhip_weight_view v = gateUp.abi();
        throwIfFailed(qwhip_moe_gateup_decode(enc.stream, &v, (uint32_t)experts, x.ptr(), abiDType(x.shape.dtype),
                                              (rotateInKernel ? 0u : (uint32_t)QWHIP_X_PREROTATED) |
                                                  (reuseExpertsAcrossTokens ? (uint32_t)QWHIP_MOE_REUSE_EXPERTS : 0u),
                                              (const int32_t*)idx.ptr(), (uint32_t)rows,
                                              (uint32_t)topK, act16.ptr()));
    }
    static void encodeMoEDownSharedCombineF32(QWHipEncoder& enc, const QWHal& hal, const QWWeightView& down, int experts,
                                              const QWTensorValue& act16, const QWTensorValue& idx, const QWTensorValue& wts, int rows, int topK,
                                              const QWTensorValue* shared, const QWTensorValue* sharedGate, const QWTensorValue& out) {
        hal.pipeline("qwg_moe_down_shared_combine_q4g_f32");
        const qwhip_weight_view v = down.abi();
        throwIfFailed(qwhip_moe_down_decode(enc.stream, &v, (uint32_t)experts, act16.ptr(), (const int32_t*)idx.ptr(), (const float*)wts.ptr(),
                                            (uint32_t)rows, (uint32_t)topK, shared ? (const float*)shared->ptr() : nullptr,
                                            sharedGate ? (const float*)sharedGate->ptr() : nullptr, out.ptr(), abiDType(out.shape.dtype)));
    }

    // ---- group-latent doors: the modes of the reference's encoders that carry latentLabels / groupIds / numGroups ----------
    // encodeFnMoeRoute(latentLabels:groupIds:numGroups:) (QWGemmMoERouter.swift:10-75): the groups a token's routes fall into and
    // the latent row of every route
    static void encodeMoELatentGroups(QWHipEncoder& enc, const QWHal& hal, const QWTensorValue& idx, const QWTensorValue& labels, int rows, int topK,
                                      int experts, int numGroups, const QWTensorValue& groupIds, const QWTensorValue* pairRows) {
        if (numGroups <= 0 || numGroups > 32) throw QWGemmError(QWGemmError::badShape, "group-latent moe: 1..32 latent groups");
        if (labels.shape.elementCount < (size_t)experts || groupIds.shape.elementCount < (size_t)rows * (size_t)numGroups ||
            idx.shape.elementCount < (size_t)rows * (size_t)topK || (pairRows && pairRows->shape.elementCount < (size_t)rows * (size_t)topK))
            throw QWGemmError(QWGemmError::badShape, "group-latent moe: labels [experts], groupIds [rows, groups], pairRows [rows, topK]");
        hal.pipeline("qwg_moe_route");
        throwIfFailed(qwhip_moe_latent_groups(enc.stream, (const int32_t*)idx.ptr(), (const int32_t*)labels.ptr(), (uint32_t)rows, (uint32_t)topK,
                                              (uint32_t)experts, (uint32_t)numGroups, (int32_t*)groupIds.ptr(),
                                              pairRows ? (int32_t*)pairRows->ptr() : nullptr));
    }
    // encodeMoEDownSharedCombineF32(routeOutput: true, tokenIndexedX: true) (QWGemmMoE.swift:157-199): one output row per route
    static void encodeMoERoutedGemv(QWHipEncoder& enc, const QWHal& hal, const QWWeightView& bank, int experts, const QWTensorValue& x16,
                                    bool xPerToken, const QWTensorValue& idx, const QWTensorValue* wts, int rows, int routes, const QWTensorValue& out) {
        hal.pipeline("qwg_moe_down_shared_combine_q4g_f32");
        const qwhip_weight_view v = bank.abi();
        throwIfFailed(qwhip_moe_routed_gemv(enc.stream, &v, (uint32_t)experts, x16.ptr(), xPerToken ? 1u : 0u, (const int32_t*)idx.ptr(),
                                            wts ? (const float*)wts->ptr() : nullptr, (uint32_t)rows, (uint32_t)routes, out.ptr(),
                                            abiDType(out.shape.dtype)));
    }
    // encodeMoEGateUpF32R1 over the latent rows of the routes (the reference's packed ids select row token * numGroups + group)
    static void encodeMoEGateUpRowsF32R1(QWHipEncoder& enc, const QWHal& hal, const QWWeightView& gateUp, int experts, const QWTensorValue& x,
                                         const QWTensorValue& idx, const QWTensorValue& xRows, int rows, int topK, const QWTensorValue& act16) {
        hal.pipeline("qwg_moe_gateup_q4g_f32_r1");
        const qwhip_weight_view v = gateUp.abi();
        throwIfFailed(qwhip_moe_gateup_decode_rows(enc.stream, &v, (uint32_t)experts, x.ptr(), abiDType(x.shape.dtype), (uint32_t)QWHIP_X_PREROTATED,
                                                   (const int32_t*)idx.ptr(), (const int32_t*)xRows.ptr(), (uint32_t)rows, (uint32_t)topK, act16.ptr()));
    }
    // encodeMoEDownSharedCombineF32(numGroups:) (QWGemmMoE.swift:157-199): the routed down projection summed by latent group
    static void encodeMoEDownGroupsF32(QWHipEncoder& enc, const QWHal& hal, const QWWeightView& down, int experts, const QWTensorValue& act16,
                                       const QWTensorValue& idx, const QWTensorValue& wts, const QWTensorValue& labels, int numGroups, int rows,
                                       int topK, const QWTensorValue& out) {
        hal.pipeline("qwg_moe_down_shared_combine_q4g_f32");
        const qwhip_weight_view v = down.abi();
        throwIfFailed(qwhip_moe_down_decode_groups(enc.stream, &v, (uint32_t)experts, act16.ptr(), (const int32_t*)idx.ptr(), (const float*)wts.ptr(),
                                                   (const int32_t*)labels.ptr(), (uint32_t)numGroups, (uint32_t)rows, (uint32_t)topK, out.ptr(),
                                                   abiDType(out.shape.dtype)));
    }
    // the gather rows of a grouped GEMM that reads the sorted output of an earlier one (the reference scatters that output back
    // to [token, group] rows instead: encodeMoEDownReduceCombineF32(scatterPerRoute: true))
    static void encodeMoEComposeRows(QWHipEncoder& enc, const QWHal& hal, const QWTensorValue& sortedPair, int pairs, const QWTensorValue& pairRows,
                                     int nRows, const QWTensorValue* slotOfRow, const QWTensorValue& rowsOut) {
        if (sortedPair.shape.elementCount < (size_t)pairs || pairRows.shape.elementCount < (size_t)pairs || rowsOut.shape.elementCount < (size_t)pairs ||
            (slotOfRow && slotOfRow->shape.elementCount < (size_t)nRows))
            throw QWGemmError(QWGemmError::badShape, "moe compose rows: lists are short");
        hal.pipeline("qwg_moe_group_pairs_f32");
        throwIfFailed(qwhip_moe_compose_rows(enc.stream, (const int32_t*)sortedPair.ptr(), (uint32_t)pairs, (const int32_t*)pairRows.ptr(), (uint32_t)nRows,
                                             slotOfRow ? (const int32_t*)slotOfRow->ptr() : nullptr, (int32_t*)rowsOut.ptr()));
    }
    // encodeMoEDownReduceCombineF32(numGroups:) (QWGemmMoE.swift:299-332): the sorted down outputs summed by latent group
    static void encodeMoECombineGroupsF32(QWHipEncoder& enc, const QWHal& hal, const QWTensorValue& dn, const QWTensorValue* invPerm,
                                          const QWTensorValue* wts, const QWTensorValue& idx, const QWTensorValue& labels, int rows, int topK,
                                          int numGroups, int width, const QWTensorValue& out) {
        if (out.shape.elementCount < (size_t)rows * (size_t)numGroups * (size_t)width)
            throw QWGemmError(QWGemmError::badShape, "moe combine by groups: out [rows, groups, width] is short");
        hal.pipeline("qwg_moe_down_reduce_combine_f32");
        throwIfFailed(qwhip_moe_combine_groups(enc.stream, dn.ptr(), abiDType(dn.shape.dtype), invPerm ? (const int32_t*)invPerm->ptr() : nullptr,
                                               wts ? (const float*)wts->ptr() : nullptr, (const int32_t*)idx.ptr(), (const int32_t*)labels.ptr(),
                                               (uint32_t)labels.shape.elementCount, (uint32_t)rows, (uint32_t)topK, (uint32_t)numGroups, (uint32_t)width, out.ptr(),
                                               abiDType(out.shape.dtype)));
    }
};

// ---- QWGemmAQ (Sources/Operators/QWGEMM/QWGemmAQ.swift:192-304): the bit-stream block family ----------------------
struct QWGemmAQ {
    static std::optional<std::string> kernelName(int bits, int group) {
        if (!(bits == 2 || bits == 3 || bits == 4 || bits == 6 || bits == 8)) return std::nullopt;   // QWAQBlock.swift:17-23
        if (!(group == 32 || group == 64 || group == 128 || group == 256)) return std::nullopt;
        return "qwg_gemv_aq" + std::to_string(bits) + "_g" + std::to_string(group) + "_v4";
    }
    // QWGemmAQ.encode: f16 activations [rows, k] -> f32 y [rows, n]; every weight byte read once for up to 16 rows a pass
    static void encode(QWHipEncoder& enc, const QWHal& hal, const QWTensorValue& blocks, const QWTensorValue& x, const QWTensorValue& y,
                       int n, int k, int bits, int group, int rows = 1, bool isRotated = true, bool rotateInKernel = false) {
        const auto name = kernelName(bits, group);
        if (!name) throw QWGemmError(QWGemmError::badWeights, "no affine-quantised kernel for this pair");
        if (k % group != 0 || n <= 0 || rows <= 0) throw QWGemmError(QWGemmError::badWeights, "k must be a multiple of the group and n positive");
        const auto view = QWWeightView::make(blocks, n, k, bits, group, isRotated, false);
        if (!view) throw QWGemmError(QWGemmError::badWeights, "block bank is short for n rows");
        if (x.shape.dtype != QWDType::f16) throw QWGemmError(QWGemmError::badWeights, "activations must be f16");
        if (x.shape.elementCount < (size_t)rows * (size_t)k) throw QWGemmError(QWGemmError::badWeights, "activations are short");
        if (y.shape.dtype != QWDType::f32) throw QWGemmError(QWGemmError::badWeights, "output must be f32");
        if (y.shape.elementCount < (size_t)rows * (size_t)n) throw QWGemmError(QWGemmError::badWeights, "output is short");
        if (n >= (rows > 1 ? (1 << 24) : (1 << 30))) throw QWGemmError(QWGemmError::badWeights, "bank does not fit the row-count flags");
        hal.pipeline(name->c_str());
        const qwhip_weight_view w = view->abi();
        const uint32_t flags = rotateInKernel ? 0u : (uint32_t)QWHIP_X_PREROTATED;
        for (int r0 = 0; r0 < rows; r0 += 16) {  // the reference chunks at 8 rows; one pass here holds 16
            const int chunk = rows - r0 < 16 ? rows - r0 : 16;
            const QWTensorValue xc = x.slice((size_t)r0 * k * 2, (size_t)chunk * k, QWDType::f16);
            const QWTensorValue yc = y.slice((size_t)r0 * n * 4, (size_t)chunk * n, QWDType::f32);
            throwIfFailed(qwhip_gemv(enc.stream, &w, xc.ptr(), QWHIP_F16, (uint32_t)chunk, flags, nullptr, (float*)yc.ptr()));
        }
    }
    // QWGemmAQ.encodeEmbedAQ (QWGemmAQ.swift:147-187): the token's row of a block table decoded to f32, written hc times
    static void encodeEmbedAQ(QWHipEncoder& enc, const QWHal& hal, const QWTensorValue& blocks, const QWTensorValue& token, const QWTensorValue& out,
                              int hidden, int hc, int bits, int group, int rows = 1) {
        if (hidden <= 0 || hc <= 0 || rows <= 0) throw QWGemmError(QWGemmError::badWeights, "the embedding gather needs a positive shape");
        const uint32_t bb = qwhip_block_bytes(QWHIP_KIND_NATIVE_AFFINE, (uint32_t)bits, (uint32_t)group);
        if (bb == 0) throw QWGemmError(QWGemmError::badWeights, "no affine-quantised container for this pair");
        if (hidden % group != 0) throw QWGemmError(QWGemmError::badWeights, "hidden must be a multiple of the group");
        const size_t rowBytes = (size_t)(hidden / group) * bb;
        if (blocks.bytes < rowBytes) throw QWGemmError(QWGemmError::badWeights, "the table is shorter than one row");
        if (token.shape.elementCount < (size_t)rows) throw QWGemmError(QWGemmError::badWeights, "the token tensor is short");
        if (out.shape.dtype != QWDType::f32 || out.shape.elementCount < (size_t)rows * (size_t)hidden * (size_t)hc)
            throw QWGemmError(QWGemmError::badWeights, "the output must hold rows * hidden * hc f32 values");
        hal.pipeline("qwg_embed_aq_f32");
        qwhip_weight_view w = {};
        w.blocks = blocks.ptr();
        w.n = (uint32_t)(blocks.bytes / rowBytes);   // the rows the table holds: a token past them reads the last one
        w.k = (uint32_t)hidden;
        w.kind = QWHIP_KIND_NATIVE_AFFINE;             // the gather decodes in the container's own basis: the tag is not used
        w.bits = (uint32_t)bits;
        w.group = (uint32_t)group;
        w.bytes = (uint64_t)w.n * rowBytes;
        throwIfFailed(qwhip_embed_aq_f32(enc.stream, &w, (const int32_t*)token.ptr(), (uint32_t)rows, (uint32_t)hc, (float*)out.ptr()));
    }
    // QWGemmAQ.encodeDecodeT4: f16 in, f16 out, one row
    static void encodeDecodeT4(QWHipEncoder& enc, const QWHal& hal, const QWTensorValue& blocks, const QWTensorValue& x, const QWTensorValue& y16,
                               int n, int k, int bits, int group, bool isRotated = true, bool rotateInKernel = false) {
        const auto name = kernelName(bits, group);
        if (!name) throw QWGemmError(QWGemmError::badWeights, "no affine-quantised decode kernel for this pair");
        if (k % group != 0 || n <= 0) throw QWGemmError(QWGemmError::badWeights, "k must be a multiple of the group and n positive");
        if (n >= (1 << 24)) throw QWGemmError(QWGemmError::badWeights, "bank does not fit the row-count flags");
        const auto view = QWWeightView::make(blocks, n, k, bits, group, isRotated, false);
        if (!view) throw QWGemmError(QWGemmError::badWeights, "block bank is short for n rows");
        if (x.shape.dtype != QWDType::f16 || x.shape.elementCount < (size_t)k) throw QWGemmError(QWGemmError::badWeights, "activations must be f16 [k]");
        if (y16.shape.dtype != QWDType::f16 || y16.shape.elementCount < (size_t)n) throw QWGemmError(QWGemmError::badWeights, "output must be f16 [n]");
        hal.pipeline(("qwg_gemv_aq" + std::to_string(bits) + "_g" + std::to_string(group) + "_dx_h16_t4").c_str());
        const qwhip_weight_view w = view->abi();
        throwIfFailed(qwhip_gemv(enc.stream, &w, x.ptr(), QWHIP_F16, 1, rotateInKernel ? 0u : (uint32_t)QWHIP_X_PREROTATED, y16.ptr(), nullptr));
    }
    // QWGemmAQ.encodeHeadArgmax (QWGemmAQ.swift:306-349): logits f32 [rows, n] = W . x, tokens i32 [rows] = greedy argmax (ties to
    // the lower row); f16 activations (rotated in the kernel when asked) or f32 activations already in the basis.
    static void encodeHeadArgmax(QWHipEncoder& enc, const QWHal& hal, const QWWeightView& w, const QWTensorValue& x, const QWTensorValue& logits,
                                 const QWTensorValue& tokens, int rows = 1, bool rotateInKernel = false) {
        if (rows <= 0 || rows > 16) throw QWGemmError(QWGemmError::badShape, "head argmax takes 1..16 rows");
        if ((x.shape.dtype != QWDType::f16 && x.shape.dtype != QWDType::f32) || x.shape.elementCount < (size_t)rows * (size_t)w.k)
            throw QWGemmError(QWGemmError::badWeights, "head activations must be f16 or f32 [rows, k]");
        if (logits.shape.dtype != QWDType::f32 || logits.shape.elementCount < (size_t)rows * (size_t)w.n || tokens.shape.dtype != QWDType::i32 ||
            tokens.shape.elementCount < (size_t)rows)
            throw QWGemmError(QWGemmError::badWeights, "head argmax: logits f32 [rows, n], tokens i32 [rows]");
        hal.pipeline(w.containerKind.isIncumbentContainer() ? "qwg_head_gemv_q4g_argmax" : "qwg_gemv_q4g_f32_v4_am");
        const qwhip_weight_view v = w.abi();
        throwIfFailed(qwhip_head_argmax(enc.stream, &v, x.ptr(), abiDType(x.shape.dtype), (uint32_t)rows,
                                        rotateInKernel ? 0u : (uint32_t)QWHIP_X_PREROTATED, (float*)logits.ptr(), (int32_t*)tokens.ptr()));
    }
};

// ---- QWMoEOperator.encodeResident (Sources/Operators/QWGEMM/QWMoEOperator.swift:57-442) ---------------------------
struct QWMoEOperator {
    struct Weights {
        QWTensorValue router;  // [experts, hidden] f32 / f16 / bf16
        QWWeightView gateUp;   // n = experts * 2 * intermediate, k = hidden
        QWWeightView down;     // n = experts * hidden, k = intermediate
        int hidden = 0, experts = 0, topK = 0, intermediate = 0;
        bool normTopK = true;
        float routedScale = 1.0f;
        bool reuseExpertsAcrossTokens = false;   // QWHIP_MOE_REUSE_EXPERTS on the routed gate_up of 2..4 rows
    };
    struct Scratch {  // caller-owned; sizes in elements
        QWTensorValue logits;      // f32 [rows, experts]
        QWTensorValue idx;         // i32 [rows, topK]
        QWTensorValue wts;         // f32 [rows, topK]
        QWTensorValue act16;       // f16 [rows * topK, intermediate]
        // prefill only (rows > 8)
        QWTensorValue expOff, sortedPair, sortedTok, invPerm, tileE, tileR, tileCount;  // i32
        QWTensorValue gu16;        // f16 [rows * topK, 2 * intermediate]; bf16 activations only (f16 rows run the fused gate_up)
        QWTensorValue dnHi;        // f32 or f16 [rows * topK, hidden]
    };
    // x: f16 hidden rows in the experts' basis; xPlain: the un-rotated rows the router reads (may equal x for a standard-basis bank).
    // out = sum_k w_k * expert_k(x) (+ sharedGate * shared when given).  Prefill (rows > 8) runs the grouped path:
    // router -> route -> pair sort -> gate_up GEMM -> SwiGLU+FWHT -> down GEMM -> combine; decode / verify runs the routed GEMVs.
    static void encodeResident(QWHipEncoder& enc, const QWHal& hal, const Weights& w, const Scratch& s, const QWTensorValue& x,
                               const QWTensorValue& xPlain, const QWTensorValue& out, int rows, const QWTensorValue* shared = nullptr,
                               const QWTensorValue* sharedGate = nullptr) {
        const int H = w.hidden, E = w.experts, K = w.topK, I = w.intermediate;
        if (E > 512 || E <= 0 || K <= 0 || K > 16) throw QWGemmError(QWGemmError::badShape, "moe: experts <= 512, routes <= 16");
        if (w.gateUp.n != E * 2 * I || w.gateUp.k != H || w.down.n != E * H || w.down.k != I)
            throw QWGemmError(QWGemmError::badShape, "moe: expert banks do not match (experts, hidden, intermediate)");
        QWGemm::encodeFnRouterGemm(enc, hal, xPlain, w.router, s.logits, rows, E, H);
        const bool fused = x.shape.dtype == QWDType::f16;   // gate_up GEMM + SwiGLU in one launch: gu16 is not needed
        const bool grouped = rows > 8 && s.expOff.base && (fused || s.gu16.base) && s.dnHi.base && H % 64 == 0 && I % 64 == 0;
        if (grouped) {
            const int pairs = rows * K;
            QWGemm::encodeFnMoeRoute(enc, hal, s.logits, s.idx, s.wts, rows, E, K, w.normTopK, w.routedScale);
            QWGemm::encodeMoEGroupPairsF32(enc, hal, s.idx, s.expOff, s.sortedPair, s.sortedTok, E, pairs, K, &s.invPerm, &s.tileE, &s.tileR, &s.tileCount);
            if (fused) {
                QWGemm::encodeMoEGateUpSwiglu(enc, hal, w.gateUp, E, x, s.sortedTok, s.expOff, s.tileE, s.tileR, s.tileCount, pairs, s.act16,
                                              w.down.isRotated());
            } else {
                QWGemm::encodeMoEGroupedGemm(enc, hal, w.gateUp, E, x, &s.sortedTok, s.expOff, s.tileE, s.tileR, s.tileCount, pairs, s.gu16);
                QWGemm::encodeSiluMulSplitF16(enc, hal, s.gu16, s.act16, pairs, I, w.down.isRotated());
            }
            QWGemm::encodeMoEGroupedGemm(enc, hal, w.down, E, s.act16, nullptr, s.expOff, s.tileE, s.tileR, s.tileCount, pairs, s.dnHi);
            QWGemm::encodeMoEDownReduceCombineF32(enc, hal, s.dnHi, s.invPerm, s.wts, rows, K, H, shared, sharedGate, out);
        } else {
            QWGemm::encodeMoERouteGateUp(enc, hal, w.gateUp, E, x, s.logits, s.idx, s.wts, rows, K, w.normTopK, w.routedScale, s.act16, false,
                                         w.reuseExpertsAcrossTokens);
            QWGemm::encodeMoEDownSharedCombineF32(enc, hal, w.down, E, s.act16, s.idx, s.wts, rows, K, shared, sharedGate, out);
        }
    }

    // ---- latent-bottleneck sparse MoE (QWMoEOperator+Latent.swift:17-303): fc1 -> routed experts in the latent width ->
    // latent norm -> fc2, with the shared expert on the full hidden width ---------------------------------------------------
    struct LatentBottleneck {
        QWWeightView fc1;                       // n = latentDim, k = hidden
        QWWeightView fc2;                       // n = hidden, k = latentDim
        std::optional<QWTensorValue> normGamma; // f16 [latentDim], plus-one law; none = rotation only
        float normEps = 1e-6f;
        int latentDim = 0;
    };
    struct LatentWeights {
        Weights routed;                         // gateUp: n = experts * 2 * intermediate, k = latentDim; down: n = experts * latentDim, k = intermediate
        std::optional<QWWeightView> sharedGateUp;   // n = 2 * sharedIntermediate, k = hidden
        std::optional<QWWeightView> sharedDown;     // n = hidden, k = sharedIntermediate
        std::optional<QWTensorValue> sharedGateScalar;   // f32 [hidden]: gate = sigmoid(x . w), a column of the router launch
        int sharedIntermediate = 0;
        std::optional<QWTensorValue> routerBias, routedScaleParam;   // f32 [experts]
        bool splitFeatureRouting = false;
    };
    struct LatentScratch {   // caller-owned
        QWTensorValue xRot32, xPlain32;         // f32 [rows, hidden]
        QWTensorValue bufA32, bufB32;           // f32 [rows, latentDim]
        QWTensorValue bufB16;                   // f16 [rows, latentDim]: what the routed experts read
        QWTensorValue naxX16;                   // f16 staging of the dense projections: rows * max(hidden, latentDim, sharedIntermediate)
        QWTensorValue gate;                     // f32 [rows]
        QWTensorValue guSh32, actSh32, shared;  // f32 [rows, 2 ISh], [rows, ISh], [rows, hidden]
    };
    // x16: f16 normed hidden rows in the rotated basis (the operator's .f16Normed input).  `s.dnHi` holds [rows * topK, latentDim].
    // As in the reference the routed experts read the latent rows as f16 on the grouped path; here the decode path does too.
    static void encodeResidentLatent(QWHipEncoder& enc, const QWHal& hal, const LatentWeights& lw, const LatentBottleneck& latent, const Scratch& s,
                                     const LatentScratch& ls, const QWTensorValue& x16, const QWTensorValue& out32, int rows) {
        const Weights& w = lw.routed;
        const int H = w.hidden, L = latent.latentDim, E = w.experts, K = w.topK, I = w.intermediate, ISh = lw.sharedIntermediate;
        if (E > 512 || E <= 0 || K <= 0 || K > 16) throw QWGemmError(QWGemmError::badShape, "latent moe: experts <= 512, routes <= 16");
        if (L <= 0 || L % 32 != 0 || latent.fc1.n != L || latent.fc1.k != H || latent.fc2.n != H || latent.fc2.k != L)
            throw QWGemmError(QWGemmError::badShape, "latent moe: fc1 is [latent, hidden], fc2 [hidden, latent], latent % 32 == 0");
        if (w.gateUp.n != E * 2 * I || w.gateUp.k != L || w.down.n != E * L || w.down.k != I)
            throw QWGemmError(QWGemmError::badShape, "latent moe: expert banks do not match (experts, latent, intermediate)");
        const bool hasShared = ISh > 0 && lw.sharedGateUp && lw.sharedDown;
        if (hasShared && (lw.sharedGateUp->n != 2 * ISh || lw.sharedGateUp->k != H || lw.sharedDown->n != H || lw.sharedDown->k != ISh))
            throw QWGemmError(QWGemmError::badShape, "latent moe: shared expert banks do not match (hidden, shared intermediate)");
        const int routerCols = lw.splitFeatureRouting ? 2 * E : E;
        QWGemm::encodeMoEBridgeF16ToF32(enc, hal, x16, ls.xRot32, ls.xPlain32, rows, H);
        const bool hasGate = hasShared && lw.sharedGateScalar;
        QWGemm::encodeFnRouterGemm(enc, hal, ls.xPlain32, w.router, s.logits, rows, routerCols, H, hasGate ? &*lw.sharedGateScalar : nullptr,
                           hasGate ? &ls.gate : nullptr);
        QWGemm::encodeDenseProjF32(enc, hal, latent.fc1, ls.xRot32, ls.bufA32, ls.naxX16, rows);
        QWGemm::encodeFnMoeRoute(enc, hal, s.logits, s.idx, s.wts, rows, E, K, w.normTopK, w.routedScale, lw.routerBias ? &*lw.routerBias : nullptr,
                         lw.splitFeatureRouting, lw.routedScaleParam ? &*lw.routedScaleParam : nullptr);
        QWGemm::encodeLatentNormH32F32(enc, hal, ls.bufA32, nullptr, ls.bufB32, &ls.bufB16, rows, L, latent.normEps, true);
        if (hasShared) {
            QWGemm::encodeDenseProjF32(enc, hal, *lw.sharedGateUp, ls.xRot32, ls.guSh32, ls.naxX16, rows);
            QWGemm::encodeSiluMulF32(enc, hal, ls.guSh32, ls.actSh32, rows, ISh);
            QWGemm::encodeDenseProjF32(enc, hal, *lw.sharedDown, ls.actSh32, ls.shared, ls.naxX16, rows);
        }
        const int pairs = rows * K;
        const QWTensorValue xLat16 = ls.bufB16.slice(0, (size_t)rows * (size_t)L, QWDType::f16);
        const bool grouped = rows > 8 && s.expOff.base && s.dnHi.base && L % 64 == 0 && I % 64 == 0;
        if (grouped) {
            QWGemm::encodeMoEGroupPairsF32(enc, hal, s.idx, s.expOff, s.sortedPair, s.sortedTok, E, pairs, K, &s.invPerm, &s.tileE, &s.tileR, &s.tileCount);
            QWGemm::encodeMoEGateUpSwiglu(enc, hal, w.gateUp, E, xLat16, s.sortedTok, s.expOff, s.tileE, s.tileR, s.tileCount, pairs, s.act16,
                                  w.down.isRotated());
            QWGemm::encodeMoEGroupedGemm(enc, hal, w.down, E, s.act16, nullptr, s.expOff, s.tileE, s.tileR, s.tileCount, pairs, s.dnHi);
            QWGemm::encodeMoEDownReduceCombineF32(enc, hal, s.dnHi, s.invPerm, s.wts, rows, K, L, nullptr, nullptr, ls.bufA32);
        } else {
            QWGemm::encodeMoEGateUpF32R1(enc, hal, w.gateUp, E, xLat16, s.idx, rows, K, s.act16);
            QWGemm::encodeMoEDownSharedCombineF32(enc, hal, w.down, E, s.act16, s.idx, s.wts, rows, K, nullptr, nullptr, ls.bufA32);
        }
        QWGemm::encodeLatentNormH32F32(enc, hal, ls.bufA32, latent.normGamma ? &*latent.normGamma : nullptr, ls.bufB32, nullptr, rows, L, latent.normEps);
        QWGemm::encodeDenseProjF32(enc, hal, latent.fc2, ls.bufB32, out32, ls.naxX16, rows);
        if (hasShared) QWGemm::encodeMoEAddSharedF32(enc, hal, out32, rows, H, ls.shared, hasGate ? &ls.gate : nullptr, out32);
    }

    // ---- group-latent sparse MoE (QWMoEOperator+GroupLatent.swift:11-294): latentD[g] -> routed experts in the latent width ->
    // sum by group -> latentU[g], the shared expert on the full hidden width -----------------------------------------------
    struct GroupLatentWeights {
        Weights routed;                         // gateUp: n = experts * 2 * intermediate, k = latentDim; down: n = experts * latentDim, k = intermediate
        QWWeightView latentD;                   // n = numLatentGroups * latentDim, k = hidden (output rotation folded in)
        QWWeightView latentU;                   // n = numLatentGroups * hidden, k = latentDim
        QWTensorValue latentLabels;             // i32 [experts]: the group of every expert
        int numLatentGroups = 0, latentDim = 0;
        std::optional<QWWeightView> sharedGateUp, sharedDown;
        std::optional<QWTensorValue> sharedGateScalar;   // f32 [hidden]
        int sharedIntermediate = 0;
        std::optional<QWTensorValue> routerBias, routedScaleParam;
        bool splitFeatureRouting = false;
    };
    struct GroupLatentScratch {   // caller-owned
        QWTensorValue xRot32, xPlain32;         // f32 [rows, hidden]
        QWTensorValue groupIds;                 // i32 [rows, groups]
        QWTensorValue pairRows;                 // i32 [rows, topK]
        QWTensorValue onesRoute;                // f32 [rows, groups], all 1 (the reference's onesRoute)
        QWTensorValue xLatent16, zLatent16;     // f16 [rows * groups, latentDim]
        QWTensorValue naxX16;                   // f16 staging of the shared expert's projections
        QWTensorValue gate;                     // f32 [rows]
        QWTensorValue guSh32, actSh32, shared;  // f32 [rows, 2 ISh], [rows, ISh], [rows, hidden]
        // prefill only: the sort of the (token, group) pairs, kept beside the experts' sort in Scratch, and its outputs
        QWTensorValue gExpOff, gSortedPair, gSortedTok, gInvPerm, gTileE, gTileR, gTileCount;   // i32
        QWTensorValue rows2;                    // i32 [rows * topK]: gather rows of the experts' gate_up
        QWTensorValue upAcc;                    // f32 [rows * groups, hidden]
        QWTensorValue xe16;                     // f16 [rows, hidden]: the cast of an f32 input without a precast copy
    };
    // The operator's Input (QWMoEOperator.swift:12-17): f16 normed rows in the rotated basis, or f32 rows given both un-rotated
    // and rotated (with an optional f16 copy of the rotated rows).
    struct Input {
        std::optional<QWTensorValue> f16Normed;
        std::optional<QWTensorValue> plain32, rotated32, precast16;
        static Input normed(const QWTensorValue& x16) { Input i; i.f16Normed = x16; return i; }
        static Input preRotated(const QWTensorValue& plain, const QWTensorValue& rotated, const QWTensorValue* precast = nullptr) {
            Input i; i.plain32 = plain; i.rotated32 = rotated; if (precast) i.precast16 = *precast; return i;
        }
    };
    // `s.dnHi` holds [rows * topK, latentDim].  The latents travel as f16 between the stages on both paths (the reference's grouped
    // path does; its decode path keeps them f32).
    static void encodeResidentGroupLatent(QWHipEncoder& enc, const QWHal& hal, const GroupLatentWeights& gw, const Scratch& s,
                                          const GroupLatentScratch& gs, const Input& input, const QWTensorValue& out32, int rows) {
        const Weights& w = gw.routed;
        const int H = w.hidden, L = gw.latentDim, NG = gw.numLatentGroups, E = w.experts, K = w.topK, I = w.intermediate, ISh = gw.sharedIntermediate;
        if (E > 512 || E <= 0 || K <= 0 || K > 16) throw QWGemmError(QWGemmError::badShape, "group-latent moe: experts <= 512, routes <= 16");
        if (NG <= 0 || NG > 32 || L <= 0 || L % 32 != 0 || gw.latentD.n != NG * L || gw.latentD.k != H || gw.latentU.n != NG * H || gw.latentU.k != L)
            throw QWGemmError(QWGemmError::badShape, "group-latent moe: latentD is [groups * latent, hidden], latentU [groups * hidden, latent], 1..32 groups");
        if (w.gateUp.n != E * 2 * I || w.gateUp.k != L || w.down.n != E * L || w.down.k != I)
            throw QWGemmError(QWGemmError::badShape, "group-latent moe: expert banks do not match (experts, latent, intermediate)");
        const bool hasShared = ISh > 0 && gw.sharedGateUp && gw.sharedDown;
        if (hasShared && (gw.sharedGateUp->n != 2 * ISh || gw.sharedGateUp->k != H || gw.sharedDown->n != H || gw.sharedDown->k != ISh))
            throw QWGemmError(QWGemmError::badShape, "group-latent moe: shared expert banks do not match (hidden, shared intermediate)");
        const int routerCols = gw.splitFeatureRouting ? 2 * E : E;
        const bool hasGate = hasShared && gw.sharedGateScalar;
        QWTensorValue x16, xPlain32, xRot32;
        if (input.f16Normed) {
            x16 = *input.f16Normed;
            xPlain32 = gs.xPlain32;
            xRot32 = gs.xRot32;
            QWGemm::encodeMoEBridgeF16ToF32(enc, hal, x16, xRot32, xPlain32, rows, H);
        } else if (input.plain32 && input.rotated32) {
            xPlain32 = *input.plain32;
            xRot32 = *input.rotated32;
            if (input.precast16) {
                x16 = *input.precast16;
            } else {
                if (!gs.xe16.base) throw QWGemmError(QWGemmError::badShape, "group-latent moe: an f32 input without a precast copy needs the xe16 scratch");
                QWGemm::encodeCast(enc, hal, xRot32, gs.xe16, (size_t)rows * (size_t)H);
                x16 = gs.xe16;
            }
        } else {
            throw QWGemmError(QWGemmError::badShape, "group-latent moe: input is f16 normed rows or the f32 (plain, rotated) pair");
        }
        QWGemm::encodeFnRouterGemm(enc, hal, xPlain32, w.router, s.logits, rows, routerCols, H, hasGate ? &*gw.sharedGateScalar : nullptr,
                                   hasGate ? &gs.gate : nullptr);
        QWGemm::encodeFnMoeRoute(enc, hal, s.logits, s.idx, s.wts, rows, E, K, w.normTopK, w.routedScale, gw.routerBias ? &*gw.routerBias : nullptr,
                                 gw.splitFeatureRouting, gw.routedScaleParam ? &*gw.routedScaleParam : nullptr);
        QWGemm::encodeMoELatentGroups(enc, hal, s.idx, gw.latentLabels, rows, K, E, NG, gs.groupIds, &gs.pairRows);
        if (hasShared) {
            QWGemm::encodeDenseProjF32(enc, hal, *gw.sharedGateUp, xRot32, gs.guSh32, gs.naxX16, rows);
            QWGemm::encodeSiluMulF32(enc, hal, gs.guSh32, gs.actSh32, rows, ISh);
            QWGemm::encodeDenseProjF32(enc, hal, *gw.sharedDown, gs.actSh32, gs.shared, gs.naxX16, rows);
        }
        const QWTensorValue* shared = hasShared ? &gs.shared : nullptr;
        const QWTensorValue* gate = hasGate ? &gs.gate : nullptr;
        const int pairs = rows * K, gpairs = rows * NG;
        const bool grouped = rows > 8 && s.expOff.base && s.dnHi.base && gs.gExpOff.base && gs.upAcc.base && H % 64 == 0 && L % 64 == 0 && I % 64 == 0;
        if (grouped) {
            // (token, group) pairs sorted by group: D_g over the sorted rows, kept in sorted order
            QWGemm::encodeMoEGroupPairsF32(enc, hal, gs.groupIds, gs.gExpOff, gs.gSortedPair, gs.gSortedTok, NG, gpairs, NG, &gs.gInvPerm, &gs.gTileE,
                                           &gs.gTileR, &gs.gTileCount);
            QWGemm::encodeMoEGroupedGemm(enc, hal, gw.latentD, NG, x16, &gs.gSortedTok, gs.gExpOff, gs.gTileE, gs.gTileR, gs.gTileCount, gpairs,
                                         gs.xLatent16);
            // the experts' sort; every sorted (token, route) pair reads the sorted latent row of its token and group
            QWGemm::encodeMoEGroupPairsF32(enc, hal, s.idx, s.expOff, s.sortedPair, s.sortedTok, E, pairs, K, &s.invPerm, &s.tileE, &s.tileR, &s.tileCount);
            QWGemm::encodeMoEComposeRows(enc, hal, s.sortedPair, pairs, gs.pairRows, gpairs, &gs.gInvPerm, gs.rows2);
            QWGemm::encodeMoEGateUpSwiglu(enc, hal, w.gateUp, E, gs.xLatent16, gs.rows2, s.expOff, s.tileE, s.tileR, s.tileCount, pairs, s.act16,
                                          w.down.isRotated());
            QWGemm::encodeMoEGroupedGemm(enc, hal, w.down, E, s.act16, nullptr, s.expOff, s.tileE, s.tileR, s.tileCount, pairs, s.dnHi);
            QWGemm::encodeMoECombineGroupsF32(enc, hal, s.dnHi, &s.invPerm, &s.wts, s.idx, gw.latentLabels, rows, K, NG, L, gs.zLatent16);
            // U_g over the groups' sums (rows token * groups + group, gathered in the first sort's order), then the sum over groups
            QWGemm::encodeMoEGroupedGemm(enc, hal, gw.latentU, NG, gs.zLatent16, &gs.gSortedPair, gs.gExpOff, gs.gTileE, gs.gTileR, gs.gTileCount, gpairs,
                                         gs.upAcc);
            QWGemm::encodeMoEDownReduceCombineF32(enc, hal, gs.upAcc, gs.gInvPerm, gs.onesRoute, rows, NG, H, shared, gate, out32);
        } else {
            QWGemm::encodeMoERoutedGemv(enc, hal, gw.latentD, NG, x16, true, gs.groupIds, nullptr, rows, NG, gs.xLatent16);
            QWGemm::encodeMoEGateUpRowsF32R1(enc, hal, w.gateUp, E, gs.xLatent16, s.idx, gs.pairRows, rows, K, s.act16);
            QWGemm::encodeMoEDownGroupsF32(enc, hal, w.down, E, s.act16, s.idx, s.wts, gw.latentLabels, NG, rows, K, gs.zLatent16);
            QWGemm::encodeMoEDownSharedCombineF32(enc, hal, gw.latentU, NG, gs.zLatent16, gs.groupIds, gs.onesRoute, rows, NG, shared, gate, out32);
        }
    }
};

}  // namespace qw
