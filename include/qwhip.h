/* qwhip.h - C ABI of libqwhip: the MI355X (gfx950) HIP HAL and quantized-matmul
 * launchers that stand where the reference's Metal HAL + QWGEMM kernels stand.
 *
 * Every entry point is `extern "C"`, takes plain pointers and sizes, returns a
 * status code (0 = ok), never aborts and never launches partially: all checks
 * run before the first enqueue (the reference throws its typed errors before
 * any bind, Sources/Operators/QWGEMM/QWGemm.swift:66-80).  Device pointers are
 * caller-owned; the library never frees caller memory and allocates nothing
 * inside a launcher.  Launchers enqueue on the given stream and return; order
 * inside a stream replaces the reference's encoder barriers.
 *
 * Paths cited below are relative to the reference checkout.
 */
#ifndef QWHIP_H
#define QWHIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- status codes: map 1:1 onto the Swift error cases ---------------------
 * QWGemmError {badWeights, badShape, badGeometry, f3Blocked}  (QWGemm.swift:66-80)
 * QWHalError.kernelMissing / deviceUnavailable               (Sources/Foundation/QWHAL/QWHal.swift:60-77) */
typedef int32_t qwhip_status;
enum {
    QWHIP_OK = 0,
    QWHIP_E_BAD_WEIGHTS = 1,    /* QWGemmError.badWeights  */
    QWHIP_E_BAD_SHAPE = 2,      /* QWGemmError.badShape    */
    QWHIP_E_BAD_GEOMETRY = 3,   /* QWGemmError.badGeometry */
    QWHIP_E_BLOCKED = 4,        /* QWGemmError.f3Blocked / plan backend .blocked */
    QWHIP_E_KERNEL_MISSING = 5, /* QWHalError.kernelMissing(name) */
    QWHIP_E_DEVICE = 6,         /* QWHalError.deviceUnavailable / any HIP runtime failure */
    QWHIP_E_BASIS = 7,          /* activation basis does not fit the container (QWHal.swift:227-232) */
    QWHIP_E_NULL = 8,           /* a required pointer is NULL */
    QWHIP_E_ALLOC = 9           /* qwhip_malloc failed */
};

/* ---- element types (mirror of QWDType, Sources/Foundation/QWCore/QWDType.swift) */
enum { QWHIP_F32 = 0, QWHIP_F16 = 1, QWHIP_BF16 = 2, QWHIP_I32 = 3 };

/* ---- container kinds (QWWeightView.ContainerKind, Sources/Foundation/QWAlloc/QWWeightView.swift:11-16) */
enum {
    QWHIP_KIND_HQ4_G32_M5 = 0,    /* .incumbentHQ4G32: 20-byte magic-bias blocks, rotated */
    QWHIP_KIND_ROTATED_HQ = 1,    /* .rotatedHQ(bits, group): bit-stream blocks, rotated  */
    QWHIP_KIND_NATIVE_AFFINE = 2  /* .nativeAffine(bits, group): bit-stream blocks, standard basis */
};

/* Non-owning view of one quantized bank [n rows][k/group blocks], row-major
 * (QWWeightView, QWWeightView.swift:86-118).  `bytes` is what the caller's
 * region holds from `blocks` on; a view is valid when n > 0, k > 0,
 * k % group == 0, (bits, group) is a supported pair and
 * bytes >= n * (k/group) * (4 + group*bits/8). */
typedef struct qwhip_weight_view {
    const void* blocks; /* device pointer, >= 4-byte aligned */
    uint64_t bytes;
    uint32_t n;
    uint32_t k;
    uint32_t kind;  /* QWHIP_KIND_* */
    uint32_t bits;  /* 4 for HQ4_G32_M5; {2,3,4,6,8} for blocks */
    uint32_t group; /* 32 for HQ4_G32_M5; {32,64,128,256} for blocks */
} qwhip_weight_view;

typedef struct qwhip_device_s* qwhip_device_t; /* stands for QWHal */
typedef struct qwhip_stream_s* qwhip_stream_t; /* stands for an open command encoder */
typedef struct qwhip_event_s* qwhip_event_t;

typedef struct qwhip_caps {
    char name[64];
    char arch[32];         /* "gfx950" */
    uint32_t compute_units;
    uint32_t wavefront;    /* 64 */
    uint32_t lds_bytes;    /* per workgroup */
    uint32_t l2_bytes;
    uint64_t hbm_bytes;
    uint32_t clock_khz;
    uint32_t has_mfma_f16; /* the reference's caps.isMetal4TensorCapable (QWHal.swift:81-130) */
} qwhip_caps;

/* ---- HAL: device, streams, memory, events --------------------------------- */
/* QWHal.init (QWHal.swift:133-232): opens device `ordinal`, refuses a device that is not gfx950. */
qwhip_status qwhip_device_create(int32_t ordinal, qwhip_device_t* out);
qwhip_status qwhip_device_destroy(qwhip_device_t dev);
/* The gated activation every FFN epilogue of this device applies (qwg_swiglu_mul, Sources/QWMetal/include/qw_weight_basis.metalh:48-66),
 * the counterpart of the reference's pipeline function constants 224 / 228 / 229 that QWHal derives from the model geometry
 * (QWHal+Constants.swift:60-75): kind 0 = SwiGLU silu(g) * u (the default); 1 = SwiGLU with g <= p0 and |u| <= p0 (swigluLimit);
 * 2 = the bounded form p0 tanh(g / p0) sigmoid(g) * p1 tanh(u / p1) (activationKind .situ(beta: p0, linearBeta: p1); p1 <= 0
 * leaves u as it is).  Applies to launches enqueued afterwards on every stream of the device: qwhip_swiglu_fwht,
 * qwhip_silu_mul_f32, qwhip_gemm_swiglu, qwhip_moe_grouped_gemm_swiglu, qwhip_gemv_silu_pair, qwhip_moe_gateup_decode*
 * and qwhip_moe_route_gateup_decode.  Set it once after qwhip_device_create, as the reference builds its pipelines once. */
#define QWHIP_ACT_SWIGLU 0u
#define QWHIP_ACT_SWIGLU_CLAMPED 1u
#define QWHIP_ACT_BOUNDED 2u
qwhip_status qwhip_device_set_gated_activation(qwhip_device_t dev, uint32_t kind, float p0, float p1);
qwhip_status qwhip_device_caps(qwhip_device_t dev, qwhip_caps* out);
/* hal.begin() / hal.end() (QWHal.swift:325-378): a stream is the encoder the launchers take. */
qwhip_status qwhip_stream_create(qwhip_device_t dev, qwhip_stream_t* out);
qwhip_status qwhip_stream_destroy(qwhip_stream_t s);
qwhip_status qwhip_stream_sync(qwhip_stream_t s); /* waitUntilCompleted (QWHal.swift:352-360) */
/* The native hipStream_t behind a stream handle, for callers that time or capture on it. */
void* qwhip_stream_native(qwhip_stream_t s);
/* Arena backing store (QWArena, Sources/Foundation/QWAlloc/QWArena.swift:161-193): 256-byte aligned device memory. */
qwhip_status qwhip_malloc(qwhip_device_t dev, size_t bytes, void** out);
qwhip_status qwhip_free(qwhip_device_t dev, void* p);
qwhip_status qwhip_memcpy_h2d(qwhip_stream_t s, void* dst, const void* src, size_t bytes); /* synchronous */
qwhip_status qwhip_memcpy_d2h(qwhip_stream_t s, void* dst, const void* src, size_t bytes); /* synchronous */
qwhip_status qwhip_memcpy_d2d(qwhip_stream_t s, void* dst, const void* src, size_t bytes); /* async on s */
qwhip_status qwhip_fill_u32(qwhip_stream_t s, void* dst, uint32_t value, size_t count);    /* async fill kernel */
/* Adds the sum of the 32-bit words of a device plane (16-byte aligned, whole 16-byte pieces) into the 256 device words
 * sum[0..255], which the caller clears first (qwhip_fill_u32, 512 words); the checksum is their total mod 2^64.  No
 * counterpart in the reference: it is how a loader checks an uploaded plane against the host copy without reading it
 * back, and - a launch that only reads - the read-bandwidth yardstick bench.py quotes beside the decode GEMV. */
qwhip_status qwhip_plane_checksum(qwhip_stream_t s, const void* plane, size_t bytes, uint64_t* sum);
/* The same word sum over a bank of `rows` rows of `row_bytes` bytes (whole 20-byte pieces, 4-byte aligned, under 4 GiB),
 * read the way the m = 1 HQ4_G32_M5 decode GEMV reads it: its grid, its 20-byte pieces per lane, its window of rows in
 * flight, the arithmetic taken out.  No counterpart in the reference: it is the second yardstick bench.py quotes beside the
 * decode GEMV (what the GEMV's own request pattern costs when nothing is computed). */
qwhip_status qwhip_plane_checksum_rows(qwhip_stream_t s, const void* plane, uint32_t rows, uint32_t row_bytes, uint64_t* sum);
/* GPU timestamps (QWStageCounter, Sources/Foundation/QWHAL/QWStageCounter.swift:1-40). */
qwhip_status qwhip_event_create(qwhip_device_t dev, qwhip_event_t* out);
qwhip_status qwhip_event_destroy(qwhip_event_t e);
qwhip_status qwhip_event_record(qwhip_event_t e, qwhip_stream_t s);
qwhip_status qwhip_event_elapsed_ms(qwhip_event_t start, qwhip_event_t stop, float* ms); /* syncs on stop */
/* hal.pipeline(name) (QWHal.swift:291-322): 0 when `name` (a reference kernel name such as
 * "qwg_gemv_q4g_dx_h16_t4") has a launcher here, else QWHIP_E_KERNEL_MISSING.  `launcher`, when
 * not NULL, receives the name of the qwhip_* entry point that serves it. */
qwhip_status qwhip_kernel_lookup(const char* name, const char** launcher);
/* Text of the last error raised on the calling thread ("" when none). */
const char* qwhip_last_error(void);
const char* qwhip_status_name(qwhip_status st);

/* ---- container helpers ---------------------------------------------------- */
/* QWAQBlock.bytesIfBlockSupported (Sources/Foundation/QWQuant/QWAQBlock.swift:48-86): 0 when unsupported. */
uint32_t qwhip_block_bytes(uint32_t kind, uint32_t bits, uint32_t group);
/* QWWeightView.init? (QWWeightView.swift:107-118): QWHIP_OK or QWHIP_E_BAD_WEIGHTS. */
qwhip_status qwhip_weight_view_validate(const qwhip_weight_view* w);

/* ---- launch flags ---------------------------------------------------------- */
enum {
    /* Activations are already in the container's basis (rotated per 32-group for a rotated
     * container).  Without it the launcher rotates them itself: FWHT-32 in fp32, one f16
     * rounding, fused into the kernel prologue for one row, one pass into the stream's scratch
     * for several (QWWeightView.isRotated contract, QWWeightView.swift:33-38; producer-side
     * rotation Sources/QWMetal/include/qw_dequant.metalh:424-493). */
    QWHIP_X_PREROTATED = 1u << 0,
    /* qwhip_gemv: every activation row gets the bits it would get in a call of its own, whatever m is (one arithmetic for
     * all row counts: the reference's 1- / 2- / 4- / M-row bodies agree bit for bit, qw_dequant_multi_b.metalh:14,486,533) */
    QWHIP_GEMV_ROW_INVARIANT = 1u << 1,
    /* qwhip_moe_gateup_decode*, qwhip_moe_route_gateup_decode on an HQ4_G32_M5 bank: an expert that several of the 2..4 tokens
     * of a verify window (at most 64 routes) route to is read by one workgroup for all of them (encodeMoEGateUpF32R1's
     * reuseExpertsAcrossTokens, QWGemmMoE.swift:119-132).  Without it every (token, route) pair reads its expert's rows itself,
     * and rows that share an expert meet in the L2; the outputs are the same bits either way.  Off by default: on this
     * hardware the launch measured slower with it (the owner of a shared expert runs its tokens one after the other). */
    QWHIP_MOE_REUSE_EXPERTS = 1u << 2
};

/* ---- elementwise seams ------------------------------------------------------ */
/* qwg_fwht32_f16 (Sources/QWMetal/gemm/qwgemm.metal:27-32; QWGemm.encodeFwht32, QWGemm.swift:288-300):
 * normalized FWHT-32 over consecutive 32-groups, src dtype f16/bf16/f32 -> dst f16 (dst may equal src for f16). */
qwhip_status qwhip_fwht32(qwhip_stream_t s, const void* src, uint32_t src_dtype, void* dst_f16, uint64_t n);
/* qwg_rmsnorm / qwg_rmsnorm_residual (Sources/QWMetal/mlp_norm_rope/qwnorm.metal:27-79, 127-189; encodeRMSNormFast /
 * encodeRMSNormResidualFast, Sources/Runtime/QWEngine/Driver/EncodeKernels.swift:339-404): the producer in front of the
 * projections.  y [rows, hidden] f16 = f16(FWHT32(x * rsqrt(mean(x^2) + eps) * (1 + gamma))), fp32 inside, gamma stored raw
 * (plus-one law); with `residual_f16` (in/out, may be NULL) the row normalized is residual <- f16(residual + x), stored
 * back bit-exactly.  hidden % 256 == 0 (the reference driver's contract); `rotate` = 0 leaves the row in the standard basis. */
qwhip_status qwhip_rmsnorm(qwhip_stream_t s, const void* x_f16, const void* gamma_f16, void* residual_f16, uint32_t rows,
                           uint32_t hidden, float eps, uint32_t rotate, void* y_f16);
/* qwg_cast_f32_to_f16 (QWGemm.encodeCast, QWGemm.swift:305-320). */
qwhip_status qwhip_cast_f32_to_f16(qwhip_stream_t s, const float* src, void* dst_f16, uint64_t n);
/* qwg_silu_mul_f16 / qwg_silu_mul_split_f16 (Sources/QWMetal/gemm/qwgemm_batched.metal:58-97;
 * QWGemmF32.swift:47-115): gu [rows, 2*inter] (gate | up) f16 or f32 -> act [rows, inter] f16 =
 * f16(FWHT32(silu(g)*u)); the rotation is skipped when `rotate` is 0 or inter % 32 != 0. */
qwhip_status qwhip_swiglu_fwht(qwhip_stream_t s, const void* gu, uint32_t gu_dtype, void* act_f16,
                               uint32_t rows, uint32_t inter, uint32_t rotate);

/* ---- dequant side output ---------------------------------------------------- */
/* Writes the f16 weights the kernels contract, [n, k] row-major in the container's own basis:
 * RN_f16((1024+q)*scale+bias) for HQ4_G32_M5 (unpack_hq4_word8, qw_dequant.metalh:42-62),
 * RN_f16(code*scale+bias) for blocks (qwg_aq_frag8, Sources/QWMetal/include/qw_gemm_nax.metalh:29-97). */
qwhip_status qwhip_dequant_f16(qwhip_stream_t s, const qwhip_weight_view* w, void* out_f16);

/* ---- decode / verify GEMV: y[m, n] = sum_k W[n, k] * x[m, k] ---------------- */
/* One launcher for the reference's GEMV doors:
 *   QWGemm.encode / encodeH16            (QWGemm.swift:137-283)  -> qwg_gemv_q4g_v4, _v4_h16(_dual), qwg_gemv_q4g_dx_h16_t4
 *   QWGemmAQ.encode / encodeDecodeT4     (QWGemmAQ.swift:192-304) -> qwg_gemv_aq*_v4, qwg_gemv_aq*_dx_h16_t4
 *   qwg_skinny_m2/m3, qwg_gemv_hq4_rows_r_m_t (M = 2..8 verify)
 * x: [m, k] row-major, f16 or bf16; m in 1..16; every weight byte is read once for all m rows.
 * y16 (f16 [m, n]) and/or y32 (f32 [m, n]) receive the result; at least one is required
 * (both = the reference's dual store).  fp32 accumulation.
 * Arithmetic: the kernels chosen for rows already in the container's basis and for m = 1 contract the factorised form
 * of the reference's own GEMVs, scale * sum(code * x) + bias * sum(x) per slice (qwg_aq_slice_dot,
 * Sources/QWMetal/include/qw_dequant_multi.metalh:205-208); the others contract the f16 weights of qwhip_dequant_f16.
 * flags: QWHIP_X_PREROTATED; bits 8..11 pick one kernel for tuning and tests (0 = automatic, 1 = half-wave dot2,
 * 2 = MFMA streamer, 3 = DMA streamer, 4 = column-stationary HQ4 kernel, 5 = column-stationary MFMA kernel,
 * 6 = column-stationary dot2 kernel, 7 = 4x4x4-block MFMA kernel, 8 = transposing MFMA kernel, 9 = split-K MFMA kernel; a
 * kernel that does not take the shape returns QWHIP_E_BAD_GEOMETRY); bits 12..15 its tuning code (bits 12..17 for the
 * column-stationary HQ4 kernel: window form, grid scale, row sets; bits 12..18 for the
 * split-K kernel).  The split-K kernel (automatic for 4-bit banks with k >= 8192 and m >= 6) keeps its partial sums in
 * the stream's scratch: calls on one stream are ordered; calls on different streams do not share it. */
qwhip_status qwhip_gemv(qwhip_stream_t s, const qwhip_weight_view* w, const void* x, uint32_t x_dtype,
                        uint32_t m, uint32_t flags, void* y16, float* y32);

/* gate|up GEMV + SwiGLU (+ FWHT-32 of the result): qwg_gemv_q4g_silu_pair{,_h16,_dx_h16}
 * (qwgemm.metal:204-379; QWGemm.swift:137-283 epilogue .siluMulPair; EncodeKernels.swift:298-326).
 * w holds 2*inter rows: [0, inter) gate, [inter, 2*inter) up.  act16 f16 [m, inter] =
 * f16(FWHT32(silu(g)*u)) with SwiGLU on the fp32 accumulators; `rotate_out` = 0 stores it unrotated.
 * One row is read by the one-row GEMV kernels in a gate|up form (the bank walked as two moving bands); with rotate_out the
 * rotation is a second, small launch over fp32 gated values in the stream's scratch.  Without it the call is 2-3 us shorter
 * (20.7 against 23.5 us on 2 x 17408 x 5120, HQ4_G32_M5): a dense MLP decode step is fastest as this call with rotate_out = 0
 * followed by qwhip_gemv on the down bank without QWHIP_X_PREROTATED, whose fused rotation costs nothing at one row.
 * Two to sixteen rows run qwhip_gemv over the whole bank into an fp32 image in the stream's scratch and qwhip_swiglu_fwht
 * over that (calls on one stream are ordered; calls on different streams do not share the scratch).
 * flags bits 8..11 (tests): 2 = the general kernel, 3 = HQ4_G32_M5 on the MoE decode kernel. */
qwhip_status qwhip_gemv_silu_pair(qwhip_stream_t s, const qwhip_weight_view* w, const void* x, uint32_t x_dtype,
                                  uint32_t m, uint32_t flags, uint32_t rotate_out, void* act16);

/* fp32-activation GEMV with a scalar epilogue: QWGemm.encodeHQ4F32V4 and, for the row counts the reference hands to its
 * batched form, encodeHQ4F32BM (Sources/Operators/QWGEMM/QWGemmF32.swift:178-199,311-350; kernels qwg_gemv_*_f32_v4,
 * qwg_gemm_*_f32_bm, bodies Sources/QWMetal/include/qw_gemm_f32_common.metalh:59-225).
 * x: f32 [m, k] already in the container's basis (the reference rotates it with qwg_h32_f32 first); y: f32 [m, n];
 * every container width (2, 3, 4, 6, 8 bits and HQ4_G32_M5).  All arithmetic in fp32: weights are code * scale + bias
 * without the f16 rounding of qwhip_dequant_f16, as in the reference's f32 dequant (qw_dequant_f32.metalh:1-24).
 * epi: 0 none, 1 silu(y / scale), 2 sigmoid(y), 3 silu(y / scale) followed by the FWHT-32 over each 32 consecutive outputs
 * (a last partial group is padded with zeros).  Up to 31 rows: four activation rows share one pass over the bank, all
 * arithmetic in fp32.  From 32 rows on (where the reference switches to its batched kernels) and k % 64 == 0: the
 * matrix-core form, 64 activation rows per pass over the bank; activations and weights are each split into two f16
 * numbers (22 bits together) and three products are accumulated in fp32 - the same 2e-5 bar.  Every activation row is
 * scaled by a power of two into the f16 range before its split and back at the store (one small launch into the
 * stream's scratch), so any finite fp32 row is taken at every row count. */
qwhip_status qwhip_gemv_f32(qwhip_stream_t s, const qwhip_weight_view* w, const float* x, uint32_t m, uint32_t epi,
                            float scale, float* y);

/* out f32 [rows, hidden] = FWHT-32 of every 32-column group of x, scaled by 1/sqrt(32): QWGemm.encodeH32F32
 * (QWGemmF32.swift:46-54; qwg_h32_f32, Sources/QWMetal/gemm/qwgemm_f32.metal:191-201; butterfly order of
 * qwg_fwht32_lane_f32, Sources/QWMetal/include/qw_weight_basis.metalh:31-38).  out may be x. */
qwhip_status qwhip_h32_f32(qwhip_stream_t s, const float* x, float* out, uint32_t rows, uint32_t hidden);

/* LM head for greedy decoding (QWGemmAQ.encodeHeadArgmax, QWGemmAQ.swift:306-349; qwg_head_gemv_q4g_argmax,
 * qwg_gemv_*_f32_v4_am with the fold of qw_gemm_f32_common.metalh:30-58): logits [m, n] f32 = W . x (as qwhip_gemv), then
 * tokens[m] = argmax with the reference's key rule: floats compared through qw_sortable_f32_u32 (NaN never wins against
 * a number), ties to the lower row.  `logits` is required and kept (the reference's writeLogits); the reference's key
 * scratch is not needed.  x_dtype QWHIP_F32 takes fp32 activations already in the container's basis (the logits are then
 * those of qwhip_gemv_f32 with epilogue 0, and `flags` is unused).  qwhip_argmax_f32 is the fold alone, over any [rows, n]
 * f32 logits.  One row (m = 1, f16 / bf16) over an HQ4_G32_M5 bank folds inside the GEMV's epilogue, as the reference's head
 * kernels do: every workgroup leaves one key in the stream's scratch and the second launch is the one-workgroup fold of those
 * keys (qwg_head_argmax_fin); the token is the same. */
qwhip_status qwhip_head_argmax(qwhip_stream_t s, const qwhip_weight_view* w, const void* x, uint32_t x_dtype, uint32_t m,
                               uint32_t flags, float* logits, int32_t* tokens);
qwhip_status qwhip_argmax_f32(qwhip_stream_t s, const float* logits, uint32_t rows, uint32_t n, int32_t* tokens);
/* QWGemm.encodeArgmaxFin with a QWVariationalAcceptance (QWGemmF32.swift:276-307) -> qwg_head_argmax_fin_variational
 * (Sources/QWMetal/head_sampling/qwhead.metal:271-345), over the logits of a verify window: row r (r + 1 < total_rows) takes
 * draft_tokens[r + 1] instead of its argmax when that token is in the vocabulary, differs from the argmax, its logit is
 * >= max - margin and, for a finite min_log_prob, log softmax(row)[draft] >= min_log_prob (-inf: no probability gate).
 * margin <= 0 or a single row: the plain argmax, as the door decides.  draft_tokens: u32 [total_rows]. */
qwhip_status qwhip_argmax_f32_variational(qwhip_stream_t s, const float* logits, uint32_t rows, uint32_t n, const uint32_t* draft_tokens,
                                          uint32_t total_rows, float margin, float min_log_prob, int32_t* tokens);

/* ---- fp32 seams of the MoE operator chain ------------------------------------ */
/* QWGemm.encodeSiluMulF32 (Sources/Operators/QWGEMM/QWGemmF32.swift:83-94) -> qwg_silu_mul_f32
 * (Sources/QWMetal/gemm/qwgemm_f32.metal:291-317): act f32 [rows, inter] = FWHT32(silu(gate) * up), gu f32 [rows, 2 inter],
 * inter % 32 == 0.  (The door's f16 output is qwhip_swiglu_fwht with an f32 gate|up.) */
qwhip_status qwhip_silu_mul_f32(qwhip_stream_t s, const float* gu, float* act, uint32_t rows, uint32_t inter);
/* QWGemm.encodeMoEBridgeF16ToF32 (Sources/Operators/QWGEMM/QWGemmMoE.swift:337-377) -> qwg_moe_bridge_f16_to_f32
 * (Sources/QWMetal/gemm/qwmoe_bridge_f32.metal:16-78): the f16 normed hidden (rotated basis) -> x_rot32 (widened; NULL =
 * the door's skipRot32) and x_plain32 (un-rotated in fp32 through the f16 hi/lo split).  hidden % 256 == 0. */
qwhip_status qwhip_moe_bridge_f16_to_f32(qwhip_stream_t s, const void* x_f16, float* x_rot32, float* x_plain32, uint32_t rows,
                                         uint32_t hidden);
/* QWGemm.encodeLatentNormH32F32 (QWGemmF32.swift:57-80) -> qwg_latent_norm_h32_f32 (qwgemm_f32.metal:203-288): optional
 * RMSNorm with the plus-one law (gamma f16 [latent], NULL = none) and the 32-point transform on f32 [rows, latent];
 * out32 and / or out16 (NULL = not written; at least one).  latent % 32 == 0. */
qwhip_status qwhip_latent_norm_h32_f32(qwhip_stream_t s, const float* x, const void* gamma_f16, float* out32, void* out16,
                                       uint32_t rows, uint32_t latent, float eps);
/* QWGemm.encodeAddF32 (QWGemmF32.swift:108-115) -> qwg_add_f32: out = a + b over count f32 values. */
qwhip_status qwhip_add_f32(qwhip_stream_t s, const float* a, const float* b, float* out, uint64_t count);

/* Embedding gather over a block table (QWGemmAQ.encodeEmbedAQ, Sources/Operators/QWGEMM/QWGemmAQ.swift:147-187 ->
 * qwg_embed_aq_f32, Sources/QWMetal/gemm/qwgemm_aq_embed.metal:14-52): `table` is the [vocab = n, hidden = k] bank;
 * out f32 [rows, hc, hidden] = the row of tokens[r], value = code * scale + bias in fp32 in the container's own basis,
 * written hc times.  A negative token reads row 0 (as the reference), a token >= n the last row.  Every container
 * (HQ4_G32_M5 too: (q + 1024) * scale + bias).  out 16-byte aligned, rows <= 65535. */
qwhip_status qwhip_embed_aq_f32(qwhip_stream_t s, const qwhip_weight_view* table, const int32_t* tokens, uint32_t rows,
                                uint32_t hc, float* out);

/* The same gather from a raw bf16 table [vocab, hidden] (QWGemm.encodeEmbedBf16F32, Sources/Operators/QWGEMM/QWGemmF32.swift:352-363
 * -> qwg_embed_bf16_f32, Sources/QWMetal/gemm/qwgemm_f32.metal:102-116): out f32 [rows, hc, hidden], exact. */
qwhip_status qwhip_embed_bf16_f32(qwhip_stream_t s, const void* table_bf16, uint32_t vocab, uint32_t hidden, const int32_t* tokens,
                                  uint32_t rows, uint32_t hc, float* out);

/* ---- prefill GEMM: Y[m, n] = X[m, k] . W^T on f16 MFMA, fp32 accumulate ------ */
/* gemmBatchedH16 (Sources/Runtime/QWEngine/Driver/EncodeKernels.swift:119-154) -> qwg_gemm_q4g_h16 /
 * qwg_gemm_aq*_h16; QWGemm.encodeNaxF32 (Sources/Operators/QWGEMM/QWGemmF32.swift:366-402).
 * x: f16 or bf16 [m, ldx]; y: f16, bf16 or f32 [m, ldy]; ldx/ldy in elements (0 = tight; ldx % 8 == 0, ldx < 2^22).
 * Requires k % 64 == 0 and n % 16 == 0 else QWHIP_E_BAD_GEOMETRY (the reference's tensor path
 * requires N, K multiples of 64).  Activations must be in the container's basis
 * (QWHIP_X_PREROTATED) unless `workspace` holds m*k f16 elements for the rotated copy.
 * A problem of few tiles (about m * n <= 128 * 128 * 320) whose workspace also holds fp32 planes of m * n
 * elements (after the activation copy, rounded up to 256 bytes, when there is one) runs its K-steps in 2..8
 * ranges and sums the planes in range order in a second launch, when the K-steps saved outweigh the traffic
 * of the planes; the result depends on the workspace size only through that choice, never on its contents. */
qwhip_status qwhip_gemm(qwhip_stream_t s, const qwhip_weight_view* w, const void* x, uint32_t x_dtype,
                        uint32_t m, uint32_t ldx, void* y, uint32_t y_dtype, uint32_t ldy, uint32_t flags,
                        void* workspace, uint64_t workspace_bytes);

/* qwhip_gemm for callers that cannot allocate device memory or pass a workspace (code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc).  No counterpart in the reference.  Same arguments, checks, kernels and
 * results as qwhip_gemm; the call allocates nothing.  Rows already in the container's basis (QWHIP_X_PREROTATED, or a
 * standard-basis container) are read in place, at any size.  Rows that still have to be rotated are copied, rotated, into
 * a static device array inside the library instead of a caller's workspace: for those m * k * 2 must not exceed
 * qwhip_gemm_noalloc_max_bytes() (8 MiB, held by every GPU the library runs on until the process ends), else
 * QWHIP_E_BAD_SHAPE.  Every call on a GPU shares that GPU's array: calls that overlap in time on one GPU (two streams) race;
 * calls on one stream do not. */
qwhip_status qwhip_gemm_noalloc(qwhip_stream_t s, const qwhip_weight_view* w, const void* x, uint32_t x_dtype,
                                uint32_t m, uint32_t ldx, void* y, uint32_t y_dtype, uint32_t ldy, uint32_t flags);
uint64_t qwhip_gemm_noalloc_max_bytes(void);

/* ---- MoE --------------------------------------------------------------------- */
/* qwg_moe_route (Sources/QWMetal/subsystems/qwrouter.metal:31-169; encodeFnMoeRoute,
 * Sources/Operators/QWGEMM/QWGemmMoERouter.swift:10-75): fp32 softmax over `experts`, top_k rounds of
 * argmax with ties to the lower index, optional renormalisation, x routed_scale.
 * idx i32 [t, top_k] (-1 = none), wts f32 [t, top_k].  experts <= 512, top_k <= 16. */
qwhip_status qwhip_moe_route(qwhip_stream_t s, const float* logits, uint32_t t, uint32_t experts, uint32_t top_k,
                             uint32_t norm_topk, float routed_scale, int32_t* idx, float* wts);

/* The same door with the reference's other routing modes (bias / splitFeature / routedScaleParam of encodeFnMoeRoute,
 * QWGemmMoERouter.swift:10-58; qwrouter.metal:44-46,63-82,146-159): with a selection bias (f32 [experts]) and / or
 * split_feature (logits [t, 2 experts]) the score is sigmoid(l) (+ sigmoid(l')), experts are chosen by score + bias and
 * weighted by the score alone, renormalised by the sum of the selected + 1e-20; scale_param (f32 [experts], may be NULL)
 * replaces routed_scale per selected expert.  bias = NULL, split_feature = 0: the softmax law of qwhip_moe_route. */
qwhip_status qwhip_moe_route_ex(qwhip_stream_t s, const float* logits, uint32_t t, uint32_t experts, uint32_t top_k,
                                uint32_t norm_topk, float routed_scale, uint32_t split_feature, const float* bias,
                                const float* scale_param, int32_t* idx, float* wts);

/* qwg_router_gemm (qwrouter.metal:460-; encodeFnRouterGemm, QWGemmMoERouter.swift:78-113):
 * logits[t, e] = sum_h x[t, h] * Wr[e, h]; x f16/bf16/f32, Wr f32/f16/bf16, fp32 accumulate. */
/* QWGemm.encodeF32Gemv (QWGemmF32.swift:117-141) -> qwg_f32_gemv / qwg_f32_gemv_bm (qwgemm_f32.metal:120-143): dense fp32
 * weights w [n, k], fp32 rows x [rows, k]: y[t, n] = epilogue(w[n] . x[t]); epi 0 none, 1 silu(y / scale), 2 sigmoid(y),
 * 3 2 sigmoid(y / scale).  k up to 16384. */
qwhip_status qwhip_f32_gemv(qwhip_stream_t s, const float* w, const float* x, uint32_t rows, uint32_t n, uint32_t k,
                            uint32_t epi, float scale, float* y);
qwhip_status qwhip_router_gemm(qwhip_stream_t s, const void* x, uint32_t x_dtype, const void* wr, uint32_t w_dtype,
                               uint32_t t, uint32_t experts, uint32_t hidden, float* logits);
/* The same launch with the shared-expert gate column (encodeFnRouterGemm's shGateWeight / shGateOut,
 * QWGemmMoERouter.swift:78-113; qwrouter.metal:467-483,566-574,587-633): sh_gate_out[t] = sigmoid(x[t] . sh_gate_w),
 * sh_gate_w fp32 [hidden].  Both pointers, or neither (then it is qwhip_router_gemm).  hidden <= 16384. */
qwhip_status qwhip_router_gemm_shared_gate(qwhip_stream_t s, const void* x, uint32_t x_dtype, const void* wr, uint32_t w_dtype,
                                           uint32_t t, uint32_t experts, uint32_t hidden, float* logits,
                                           const float* sh_gate_w, float* sh_gate_out);

/* Scratch sizes of the pair sort (MoETilePlan, Sources/Operators/QWGEMM/QWGemmMoE.swift:24-62). */
uint32_t qwhip_moe_max_tiles(uint32_t experts, uint32_t pairs);

/* qwg_moe_group_pairs_f32 (Sources/QWMetal/gemm/qwgemm_moe_group_f32.metal:10-148;
 * encodeMoEGroupPairsF32, QWGemmMoE.swift:68-99): counting sort of the (token, route) pairs by expert
 * id (low 16 bits of ids; negative = skipped), stable in pair order.
 * expert_off i32 [experts+1]; sorted_pair i32 [pairs]; sorted_tok i32 [pairs] (= pair / top_k);
 * inv_perm i32 [pairs] (may be NULL; -1 for skipped pairs); tile_e / tile_r i32 [max_tiles] and
 * tile_count i32 [1] (may be NULL together): 64-row tiles with a compact 16/32/64 tail per expert,
 * tile_r = (code << 24) | row_block_index (Sources/QWMetal/include/qw_moe_tile.metalh:7-34). */
qwhip_status qwhip_moe_group_pairs(qwhip_stream_t s, const int32_t* ids, uint32_t experts, uint32_t pairs,
                                   uint32_t top_k, int32_t* expert_off, int32_t* sorted_pair, int32_t* sorted_tok,
                                   int32_t* inv_perm, int32_t* tile_e, int32_t* tile_r, int32_t* tile_count,
                                   uint32_t compact_tail);

/* Grouped expert GEMM over the sorted pairs: encodeMoEGateUpNax / encodeMoENaxSplitF32
 * (QWGemmMoE.swift:201-296) -> qwg_moe_nax_gemm_body / qwg_moe_nax_split_f32_body
 * (Sources/QWMetal/include/qw_gemm_nax.metalh:436-504).
 * w: ONE view over the expert-major bank, n = experts * rows_per_expert.  Row slot p in
 * [expert_off[e], expert_off[e+1]) uses expert e.  A row of slot p is x[gather[p]] when gather is
 * not NULL (gate_up: gather = sorted_tok) else x[p] (down).  y [pairs, rows_per_expert]. */
qwhip_status qwhip_moe_grouped_gemm(qwhip_stream_t s, const qwhip_weight_view* w, uint32_t experts,
                                    const void* x, uint32_t x_dtype, uint32_t ldx, const int32_t* gather,
                                    const int32_t* expert_off, const int32_t* tile_e, const int32_t* tile_r,
                                    const int32_t* tile_count, uint32_t max_tiles, uint32_t pairs,
                                    void* y, uint32_t y_dtype, uint32_t ldy);

/* Dense gate|up GEMM with the SwiGLU (+ FWHT-32) epilogue fused: the reference's qwg_gemm_q4g_h16_swiglu / qwg_gemm_aq*_h16_swiglu
 * (qmm_t_nax_swiglu_impl, Sources/QWMetal/include/qw_gemm_nax_swiglu.metalh:86-167; door
 * Sources/Runtime/QWEngine/Driver/EncodeKernels.swift:156-190).  w: [2 * inter, k], rows [gate | up]; act f16 [m, inter]
 * = f16(FWHT32(silu(g) * u)) with g, u rounded to f16 first - bit-identical to qwhip_gemm (f16 out) followed by
 * qwhip_swiglu_fwht, without the [m, 2 inter] matrix.  One launch for every container and any m; inter % 32 == 0, act
 * 16-byte aligned with ldact % 8 == 0 (0 = inter); x, flags and workspace as qwhip_gemm (bf16 or un-rotated activations
 * need the workspace: m * k * 2 bytes).  A problem of few tiles and a long K whose workspace also holds, behind the
 * activation copy, an f16 image of the gate|up matrix (m * 2 inter * 2 bytes, rounded up to 256) and fp32 planes of
 * m * 2 inter elements runs as qwhip_gemm does with K ranges and then qwhip_swiglu_fwht from the image, when that is
 * the faster form (packed act rows only; flags bits 8..11 != 0 keep the one launch); as there, the result depends on
 * the workspace size only through that choice. */
qwhip_status qwhip_gemm_swiglu(qwhip_stream_t s, const qwhip_weight_view* w, const void* x, uint32_t x_dtype, uint32_t m,
                               uint32_t ldx, uint32_t rotate_act, void* act_f16, uint32_t ldact, uint32_t flags,
                               void* workspace, size_t workspace_bytes);

/* The gate_up grouped GEMM with the SwiGLU (+ FWHT-32) epilogue fused: act f16 [pairs, inter] in sorted-pair order,
 * inter = rows_per_expert / 2, an expert's rows being [gate | up].  Bit-identical to qwhip_moe_grouped_gemm with f16 output
 * followed by qwhip_swiglu_fwht (both accumulators are rounded to f16 first, SwiGLU and the rotation run in fp32, one f16
 * rounding on store), without writing and re-reading the [pairs, 2 inter] matrix.  The reference fuses the same epilogue
 * into its dense gate_up GEMM (qmm_t_nax_swiglu_impl, Sources/QWMetal/include/qw_gemm_nax_swiglu.metalh:86-167; kernel
 * qwg_gemm_q4g_h16_swiglu) and runs encodeSiluMul* after the grouped one (QWMoEOperator.swift).
 * f16 or bf16 activations; inter % 32 == 0; act 16-byte aligned with ldact % 8 == 0 (0 = inter). */
qwhip_status qwhip_moe_grouped_gemm_swiglu(qwhip_stream_t s, const qwhip_weight_view* w, uint32_t experts,
                                           const void* x, uint32_t x_dtype, uint32_t ldx, const int32_t* gather,
                                           const int32_t* expert_off, const int32_t* tile_e, const int32_t* tile_r,
                                           const int32_t* tile_count, uint32_t max_tiles, uint32_t pairs,
                                           uint32_t rotate_act, void* act_f16, uint32_t ldact);

/* qwg_moe_down_reduce_combine_f32 (Sources/QWMetal/gemm/qwgemm_moe_nax_f16.metal:7-126;
 * encodeMoEDownReduceCombineF32, QWGemmMoE.swift:299-332):
 * out[t, h] = sum_k wts[t, k] * dn[inv_perm[t*top_k + k], h] (+ shared_gate[t] * shared[t, h]).
 * inv_perm = NULL: route k of token t sits in row t*top_k + k (the door's invPerm: nil); wts = NULL: unit weights (its
 * unweightedSingle) - with top_k = 1 that is out = dn + shared_gate * shared, the last step of the latent operator.
 * out may be dn when inv_perm is NULL and top_k = 1. */
qwhip_status qwhip_moe_combine(qwhip_stream_t s, const void* dn, uint32_t dn_dtype, const int32_t* inv_perm,
                               const float* wts, uint32_t t, uint32_t top_k, uint32_t hidden,
                               const float* shared, const float* shared_gate, void* out, uint32_t out_dtype);

/* Decode / verify (t <= 8) routed experts as GEMVs: encodeMoEGateUpF32R1 + encodeMoEDownSharedCombineF32
 * (QWGemmMoE.swift:120-199) -> Sources/QWMetal/include/qw_moe_f32_common.metalh:187-452.
 * gate_up: act16 [t, top_k, inter] = f16(FWHT32(silu(Wg[e].x) * (Wu[e].x))), SwiGLU on fp32 accumulators.
 * down:    out [t, hidden] = sum_k wts[t,k] * Wd[e_k] . act16[t,k]  (+ shared_gate[t]*shared[t]).
 * gate_up flags: QWHIP_X_PREROTATED, QWHIP_MOE_REUSE_EXPERTS; bits 8..11 = 2 keep an HQ4_G32_M5 bank on the general
 * kernel (tests). */
qwhip_status qwhip_moe_gateup_decode(qwhip_stream_t s, const qwhip_weight_view* w_gate_up, uint32_t experts,
                                     const void* x, uint32_t x_dtype, uint32_t flags, const int32_t* idx, uint32_t t,
                                     uint32_t top_k, void* act16);
/* qwhip_moe_route + qwhip_moe_gateup_decode as one launch for the decode step (an HQ4_G32_M5 bank routes inside the gate_up
 * kernel: every workgroup repeats the token's top-k from its router logits with the arithmetic of qwhip_moe_route and
 * leaves idx / wts [t, top_k] for the down projection; other containers run the two launches).  Same results as the two
 * calls; one kernel launch less on a path that is bound by launch latency.  The reference runs encodeFnMoeRoute and
 * encodeMoEGateUpF32R1 back to back (QWMoEOperator.swift); arguments as in those two doors. */
qwhip_status qwhip_moe_route_gateup_decode(qwhip_stream_t s, const qwhip_weight_view* w_gate_up, uint32_t experts,
                                           const void* x, uint32_t x_dtype, uint32_t flags, const float* logits, uint32_t t,
                                           uint32_t top_k, uint32_t norm_topk, float routed_scale, int32_t* idx, float* wts,
                                           void* act16);
qwhip_status qwhip_moe_down_decode(qwhip_stream_t s, const qwhip_weight_view* w_down, uint32_t experts,
                                   const void* act16, const int32_t* idx, const float* wts, uint32_t t,
                                   uint32_t top_k, const float* shared, const float* shared_gate, void* out,
                                   uint32_t out_dtype);

/* encodeFnMoeRoute(expertBudget:) (QWGemmMoERouter.swift:63-75) -> the normTopK & 4 branch of qwg_moe_route_decode
 * (Sources/QWMetal/subsystems/qwrouter.metal:193-268): after qwhip_moe_route* over a verify window of rows = 2..4 (rows * top_k <= 64),
 * at most max(top_k, budget) distinct experts stay.  Row 0 keeps its routes; the other (row, route) pairs are admitted expert by
 * expert in the order of their weights (ties: the lower pair index); the rest get idx -1 and weight 0 (every door skips such a
 * route), and with norm_topk a later row that lost weight is rescaled to its former sum.  budget 0 or >= rows * top_k: no-op.
 * In place on idx / wts [rows, top_k]. */
qwhip_status qwhip_moe_route_budget(qwhip_stream_t s, int32_t* idx, float* wts, uint32_t rows, uint32_t top_k, uint32_t budget,
                                    uint32_t norm_topk);

/* ---- group-latent MoE (QWMoEOperator.encodeResidentGroupLatent, Sources/Operators/QWGEMM/QWMoEOperator+GroupLatent.swift:11-294)
 * Every expert carries the label of one of num_groups (1..32) latent groups.  A token's routes read D_g . x of their
 * expert's group (bank latentD [num_groups * latent, hidden]), run the expert in the latent width, are summed by group
 * with their route weights, and the groups' sums go up through U_g (bank latentU [num_groups * hidden, latent]) and are
 * added.  The reference carries the group in the high bits of its route ids (qwg_moe_route with latentLabels,
 * Sources/QWMetal/subsystems/qwrouter.metal:135-165); here the route ids stay plain and the group rules are these doors. */

/* group_ids [t, num_groups] = g where one of the token's routes has labels[idx] == g, else -1 (qwrouter.metal:163-165);
 * pair_rows [t, top_k] (may be NULL) = t * num_groups + labels[idx[t, k]], the row of route k's latent in a [t, num_groups]
 * matrix, -1 for an absent route.  labels: i32 [experts]. */
qwhip_status qwhip_moe_latent_groups(qwhip_stream_t s, const int32_t* idx, const int32_t* labels, uint32_t t, uint32_t top_k,
                                     uint32_t experts, uint32_t num_groups, int32_t* group_ids, int32_t* pair_rows);
/* The routed projection without the sum over routes (encodeMoEDownSharedCombineF32 with routeOutput and tokenIndexedX,
 * QWGemmMoE.swift:157-199): out [t, top_k, n / experts] = wts[t, r] * W[idx[t, r]] . x_row, zeros where idx < 0.
 * x16: f16 [t, k] when x_per_token != 0 (all routes of a token read its one row), else [t, top_k, k].  wts NULL = 1. */
qwhip_status qwhip_moe_routed_gemv(qwhip_stream_t s, const qwhip_weight_view* w, uint32_t experts, const void* x16,
                                   uint32_t x_per_token, const int32_t* idx, const float* wts, uint32_t t, uint32_t top_k,
                                   void* out, uint32_t out_dtype);
/* qwhip_moe_gateup_decode with the activation row of every (token, route) pair given: pair p reads x row x_rows[p]
 * (the reference's packed ids make its gate_up kernel read row token * numGroups + group of xLatent32). */
qwhip_status qwhip_moe_gateup_decode_rows(qwhip_stream_t s, const qwhip_weight_view* w_gate_up, uint32_t experts,
                                          const void* x, uint32_t x_dtype, uint32_t flags, const int32_t* idx,
                                          const int32_t* x_rows, uint32_t t, uint32_t top_k, void* act16);
/* The routed down projection summed by group (encodeMoEDownSharedCombineF32 with numGroups, QWGemmMoE.swift:157-199):
 * out [t, num_groups, n / experts] = sum over routes r with labels[idx[t, r]] == g of wts[t, r] * Wd[idx[t, r]] . act16[t, r],
 * zeros for a group without routes. */
qwhip_status qwhip_moe_down_decode_groups(qwhip_stream_t s, const qwhip_weight_view* w_down, uint32_t experts,
                                          const void* act16, const int32_t* idx, const float* wts, const int32_t* labels,
                                          uint32_t num_groups, uint32_t t, uint32_t top_k, void* out, uint32_t out_dtype);
/* Prefill: rows_out[p] = slot_of_row[pair_rows[sorted_pair[p]]] for the `pairs` positions of an expert-sorted pair list:
 * the gather rows of a grouped GEMM whose activations are the (sorted) output of an earlier grouped GEMM over n_rows
 * (token, group) rows, slot_of_row being that sort's inv_perm (NULL = the rows are in place). */
qwhip_status qwhip_moe_compose_rows(qwhip_stream_t s, const int32_t* sorted_pair, uint32_t pairs, const int32_t* pair_rows,
                                    uint32_t n_rows, const int32_t* slot_of_row, int32_t* rows_out);
/* qwhip_moe_combine summed by group (encodeMoEDownReduceCombineF32 with numGroups, QWGemmMoE.swift:299-332;
 * qwgemm_moe_nax_f16.metal:51-111): out [t, num_groups, width] = sum over routes k with labels[idx[t, k]] == g of
 * wts[t, k] * dn[inv_perm[t * top_k + k], :], zeros for a group without routes.  inv_perm / wts NULL as in qwhip_moe_combine.
 * labels holds `experts` entries; a route whose id (low 16 bits) is not below `experts` counts as absent, as in
 * qwhip_moe_latent_groups and qwhip_moe_down_decode_groups. */
qwhip_status qwhip_moe_combine_groups(qwhip_stream_t s, const void* dn, uint32_t dn_dtype, const int32_t* inv_perm,
                                      const float* wts, const int32_t* idx, const int32_t* labels, uint32_t experts, uint32_t t,
                                      uint32_t top_k, uint32_t num_groups, uint32_t width, void* out, uint32_t out_dtype);

/* ---- load-time writer (the step before the path) ----------------------------- */
/* qwg_quantize_bf16_to_hq4_g32_m5 (Sources/QWMetal/quant/qw_online_quant.metal:17-55), GPU twin of
 * quant_hq4_blocks (Scripts/quantize/hq4.py:54-123): src [n, k] bf16 or f32 -> 20-byte blocks. */
qwhip_status qwhip_quantize_hq4_g32(qwhip_stream_t s, const void* src, uint32_t src_dtype, uint32_t n, uint32_t k,
                                    uint32_t rotate, void* blocks_out);

/* Bit-stream block writer for the non-M5 containers, the device twin of quant_hq_blocks (Scripts/quantize/hq_blocks.py:436-517; the
 * packer's own GPU path is the quant_hq_simd shader at :260): src [n, k] bf16 or f32 -> [n, k / group] blocks of
 * 4 + group * bits / 8 bytes, byte-identical to the packer.  bits in {2, 3, 4, 6, 8}, group in {32, 64, 128, 256} with
 * k % group == 0 (the packer's gcd rule is the caller's: pass the resolved group); rotate = FWHT-32 over every 32 weights first.
 * mse_clip: 0 plain min / max, 1 the ten-point shrink search (:409-432), 2 the packer's default (the search for 2 and 3 bits).
 * Non-finite weights, which the packer refuses, give unspecified blocks. */
qwhip_status qwhip_quantize_blocks(qwhip_stream_t s, const void* src, uint32_t src_dtype, uint32_t n, uint32_t k,
                                   uint32_t bits, uint32_t group, uint32_t rotate, uint32_t mse_clip, void* blocks_out);

/* Planar HQ8_G32_M5 (quant_hq8_g32_m5 / dequant_hq8_g32_m5_rot, hq_blocks.py:564-615; host reader dequantHQ8Rot,
 * Sources/Foundation/QWQuant/QWPack.swift:326-351): int8 codes [n, k] and f16 scales [n, k / 32] as two planes, symmetric,
 * scale = f16(amax / 127); the dequant writes the rotated-domain fp32 weights code * scale. */
qwhip_status qwhip_quantize_hq8_planar(qwhip_stream_t s, const void* src, uint32_t src_dtype, uint32_t n, uint32_t k,
                                       uint32_t rotate, void* qs_out, void* scales_out_f16);
qwhip_status qwhip_dequant_hq8_planar(qwhip_stream_t s, const void* qs, const void* scales_f16, uint32_t n, uint32_t k,
                                      float* out_f32);

/* qwg_repack_mlx_affine_to_aq_m5 / qwg_repack_mlx_affine_switch_gate_up_to_aq_m5
 * (Sources/QWMetal/quant/qw_online_quant.metal:56-178; QWAQRepack.repackMLXAffine / repackMLXAffineSwitchGateUp,
 * Sources/Foundation/QWLoad/AQRepack.swift:108-250): an MLX affine checkpoint (packed codes u32, scales and biases
 * bf16 or f16, one pair per group) becomes AQ blocks [f16 scale][f16 bias][payload] at the same byte count; the
 * switch variant interleaves gate_proj and up_proj [experts, inter, cols] into one [experts, 2*inter, cols] bank.
 * A header that f16 does not hold exactly (values below 2^-14 excepted) is written as the f16 NaN 0x7e00 and counted
 * in *refused (a device word the caller zeroes first and reads after the stream has drained; the reference door
 * throws headersNotExact when it is not zero). */
qwhip_status qwhip_repack_mlx_affine(qwhip_stream_t s, const void* mlx_w, const void* mlx_scales, const void* mlx_biases,
                                     uint32_t scale_dtype, uint32_t rows, uint32_t cols, uint32_t bits, uint32_t group,
                                     void* dst_blocks, uint32_t* refused);
qwhip_status qwhip_repack_mlx_affine_switch_gate_up(qwhip_stream_t s, const void* gate_w, const void* gate_scales,
                                                    const void* gate_biases, const void* up_w, const void* up_scales,
                                                    const void* up_biases, uint32_t scale_dtype, uint32_t experts,
                                                    uint32_t inter, uint32_t cols, uint32_t bits, uint32_t group,
                                                    void* dst_blocks, uint32_t* refused);

#ifdef __cplusplus
}
#endif
#endif /* QWHIP_H */
