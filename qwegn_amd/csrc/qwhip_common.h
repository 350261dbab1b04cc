// Shared host/device definitions of libqwhip (gfx950 only).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>
#include <utility>

#include "../../include/qwhip.h"

// The gated activation of the FFN epilogues, a device-wide constant like the reference's function constants 224 / 228 / 229
// (QWHal+Constants.swift:60-75): kind 0 SwiGLU, 1 SwiGLU with gate <= p0 and |up| <= p0, 2 the bounded form
// p0 tanh(g / p0) sigmoid(g) * p1 tanh(u / p1) (p1 <= 0: up as it is).
struct qw_act {
    uint32_t kind;
    float p0, p1;
};
struct qwhip_device_s {
    int ordinal;
    hipDeviceProp_t prop;
    qw_act act;
};
// Partial-sum scratch of the split-K verify GEMV: owned by the stream (allocated when the stream is created, never inside a
// launcher), so launches on different streams never share it and launches on one stream use it one after the other.
// The first QWHIP_STREAM_COUNTER_BYTES hold the keys of the head's argmax folds (one per workgroup or row slice), the rest
// holds fp32 partial outputs.
#define QWHIP_STREAM_COUNTER_BYTES (64u << 10)
// The last QWHIP_STREAM_XROT_BYTES hold the rotated copy of several un-rotated activation rows (qwhip_gemv on a rotated
// container: one rotation pass, then the kernels for rows already in the basis).
#define QWHIP_STREAM_XROT_BYTES (1u << 20)
#define QWHIP_STREAM_SCRATCH_BYTES ((8u << 20) + QWHIP_STREAM_COUNTER_BYTES + QWHIP_STREAM_XROT_BYTES)
struct qwhip_stream_s {
    qwhip_device_s* dev;
    hipStream_t stream;
    uint8_t* scratch;
    size_t scratch_bytes;
    // bytes at the top of the partial-sum area that the running call keeps for itself (the gate|up door's fp32 image of a
    // GEMV it launches): the split-K kernel places its partial sums below them.  Zero between calls.
    size_t scratch_reserved = 0;
};
struct qwhip_event_s {
    qwhip_device_s* dev;
    hipEvent_t ev;
};

// ---- host-side error plumbing (hal.hip) ------------------------------------
qwhip_status qwhip_fail(qwhip_status st, const char* fmt, ...);
qwhip_status qwhip_hip_check(hipError_t e, const char* what);
#define QWHIP_TRY_HIP(expr)                                        \
    do {                                                           \
        hipError_t _e = (expr);                                    \
        if (_e != hipSuccess) return qwhip_hip_check(_e, #expr);   \
    } while (0)
#define QWHIP_REQUIRE(p)                                                       \
    do {                                                                       \
        if ((p) == nullptr) return qwhip_fail(QWHIP_E_NULL, "%s is NULL", #p); \
    } while (0)

// elementwise.hip: src (f16 | bf16 | f32) -> f16, no rotation (internal helper of the GEMM pre-pass)
qwhip_status qw_convert_to_f16(qwhip_stream_t s, const void* src, uint32_t src_dtype, void* dst_f16, uint64_t n);

// gemm.hip: resolves this device's address of the static scratch array behind qwhip_gemm_noalloc (device `ordinal` current)
qwhip_status qw_gemm_scratch_init(int ordinal);

static inline uint32_t qwhip_cdiv(uint32_t a, uint32_t b) { return (a + b - 1) / b; }

// Block bytes of a validated view.
static inline uint32_t qwhip_view_block_bytes(const qwhip_weight_view* w) { return 4u + w->group * w->bits / 8u; }
static inline uint64_t qwhip_view_row_bytes(const qwhip_weight_view* w) {
    return (uint64_t)(w->k / w->group) * qwhip_view_block_bytes(w);
}
static inline bool qwhip_view_rotated(const qwhip_weight_view* w) { return w->kind != QWHIP_KIND_NATIVE_AFFINE; }

// ---- device-side types -------------------------------------------------------
typedef _Float16 h1_t;
typedef _Float16 h2_t __attribute__((ext_vector_type(2)));
typedef _Float16 h4_t __attribute__((ext_vector_type(4)));
typedef _Float16 h8_t __attribute__((ext_vector_type(8)));
typedef float f4_t __attribute__((ext_vector_type(4)));
typedef float f16_t __attribute__((ext_vector_type(16)));
typedef uint32_t u4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u2_t __attribute__((ext_vector_type(2)));

// GEMV container families: HQ4_G32_M5 20-byte blocks, 4-bit and 8-bit bit-stream blocks.
enum { QW_FMT_M5 = 0, QW_FMT_B4 = 1, QW_FMT_B8 = 2, QW_FMT_B2 = 3, QW_FMT_B3 = 4, QW_FMT_B6 = 5 };   // B2/B3/B6: 2-, 3- and 6-bit streams

#define QW_INV_SQRT32 0.17677669529663689f /* f32(1/sqrt(32)) = 0x3E3504F3 */

// One HQ4_G32_M5 block: [f16 scale][f16 bias][u32 qs[4]], 4-byte aligned in a bank.
struct __attribute__((packed, aligned(4))) qw_hq4_block {
    uint32_t hdr;
    uint32_t qs[4];
};

__device__ __forceinline__ float qw_bf16_to_f32(uint16_t b) { return __uint_as_float((uint32_t)b << 16); }

// f32 -> bf16 bits, round to nearest even (NaN kept quiet).
__device__ __forceinline__ uint16_t qw_f32_to_bf16(float f) {
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7F800000u) == 0x7F800000u && (u & 0x007FFFFFu)) return (uint16_t)((u >> 16) | 0x40u);
    u += 0x7FFFu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

// Load element i of a typed activation array as fp32.
template <int DT>
__device__ __forceinline__ float qw_load_f32(const void* p, uint64_t i) {
    if constexpr (DT == QWHIP_F16) return (float)((const h1_t*)p)[i];
    else if constexpr (DT == QWHIP_BF16) return qw_bf16_to_f32(((const uint16_t*)p)[i]);
    else return ((const float*)p)[i];
}

// Loads 8 consecutive elements (16-byte aligned for 2-byte types) as fp32.
template <int DT>
__device__ __forceinline__ void qw_load8_f32(const void* p, uint64_t i, float* out) {
    if constexpr (DT == QWHIP_F16) {
        h8_t v = *(const h8_t*)((const h1_t*)p + i);
#pragma unroll
        for (int j = 0; j < 8; ++j) out[j] = (float)v[j];
    } else if constexpr (DT == QWHIP_BF16) {
        u4_t v = *(const u4_t*)((const uint16_t*)p + i);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            out[2 * j] = __uint_as_float(v[j] << 16);
            out[2 * j + 1] = __uint_as_float(v[j] & 0xFFFF0000u);
        }
    } else {
        const f4_t* q = (const f4_t*)((const float*)p + i);
        f4_t a = q[0], b = q[1];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            out[j] = a[j];
            out[4 + j] = b[j];
        }
    }
}

// In-register orthonormal FWHT-32: butterflies h = 1..16 writing (u+v, u-v) to (i, i+h), then one
// multiply by f32(1/sqrt(32)) - the operation order of fwht32_ortho (Scripts/quantize/hq4.py:26-51,
// Sources/Foundation/QWQuant/QWQuant+DequantMath.swift:93-112), so results are bit-identical.
__device__ __forceinline__ void qw_fwht32(float* v) {
#pragma unroll
    for (int h = 1; h < 32; h <<= 1) {
#pragma unroll
        for (int i0 = 0; i0 < 32; i0 += 2 * h) {
#pragma unroll
            for (int j = 0; j < h; ++j) {
                const float a = v[i0 + j], b = v[i0 + j + h];
                v[i0 + j] = a + b;
                v[i0 + j + h] = a - b;
            }
        }
    }
#pragma unroll
    for (int i = 0; i < 32; ++i) v[i] = v[i] * QW_INV_SQRT32;
}

// SwiGLU on fp32: silu(g) * u = g / (1 + exp(-g)) * u  (qwg_swiglu_mul, plain branch,
// Sources/QWMetal/include/qw_weight_basis.metalh:50-63).
__device__ __forceinline__ float qw_swiglu(float g, float u) { return (g / (1.0f + __expf(-g))) * u; }
// The generalized gated activation (qwg_swiglu_mul, all three branches, Sources/QWMetal/include/qw_weight_basis.metalh:48-66);
// `a` is uniform over a launch.
__device__ __forceinline__ float qw_gated(float g, float u, const qw_act a) {
    if (a.kind == 2u) {
        const float gg = a.p0 * tanhf(g / a.p0) * (1.0f / (1.0f + __expf(-g)));
        const float uu = a.p1 > 0.0f ? a.p1 * tanhf(u / a.p1) : u;
        return gg * uu;
    }
    if (a.kind == 1u) {
        g = fminf(g, a.p0);
        u = fminf(fmaxf(u, -a.p0), a.p0);
    }
    return qw_swiglu(g, u);
}

// FWHT-32 over the 32 lanes of a half wavefront (lane j = lane & 31 holds element j), un-normalised, stage order
// h = 1, 2, 4, 8, 16 with v' = (j & h) == 0 ? v + o : o - v, o = the value of lane j ^ h: the arithmetic of the butterfly
// written with lane exchanges through LDS (ds_bpermute), bit for bit, but the partners come by DPP (quad permutes, row
// mirrors: j ^ 4 = half-mirror then quad-reverse, j ^ 8 = mirror then half-mirror) and, across the two 16-lane rows, by
// v_permlane16_swap_b32 - no LDS round trip per stage.  `sg[t]` = (j & (1 << t)) ? -1 : +1.
struct qw_fwht32_signs {
    float sg[5];
    bool odd_row;
};
__device__ __forceinline__ qw_fwht32_signs qw_fwht32_lane_signs(uint32_t lane) {
    qw_fwht32_signs s;
#pragma unroll
    for (int t = 0; t < 5; ++t) s.sg[t] = (lane & (1u << t)) ? -1.0f : 1.0f;
    s.odd_row = (lane & 16u) != 0u;
    return s;
}
#define QW_DPP_F32(v, ctrl) __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), ctrl, 0xF, 0xF, true))
__device__ __forceinline__ float qw_fwht32_lanes(float v, const qw_fwht32_signs& s) {
    v = QW_DPP_F32(v, 0xB1) + s.sg[0] * v;                       // quad_perm [1,0,3,2]: lane ^ 1
    v = QW_DPP_F32(v, 0x4E) + s.sg[1] * v;                       // quad_perm [2,3,0,1]: lane ^ 2
    {
        const float m = QW_DPP_F32(v, 0x141);                    // row_half_mirror: lane ^ 7
        v = QW_DPP_F32(m, 0x1B) + s.sg[2] * v;                   // quad_perm [3,2,1,0]: ^ 3 -> lane ^ 4
    }
    {
        const float m = QW_DPP_F32(v, 0x140);                    // row_mirror: lane ^ 15
        v = QW_DPP_F32(m, 0x141) + s.sg[3] * v;                  // row_half_mirror: ^ 7 -> lane ^ 8
    }
    {
        // (the compiler's builtin for this instruction returns its first result twice: written out)
        float a = v, b = v;
        asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
        // a = rows (0, 0, 2, 2) of v, b = rows (1, 1, 3, 3): the partner row is b for an even row, a for an odd one
        const float o = s.odd_row ? a : b;
        v = o + s.sg[4] * v;
    }
    return v;
}

// A constant pinned in a VGPR (v_and_or_b32 is VOP3: on gfx9 it takes no literal and one scalar operand,
// so one of mask / magic has to live in a vector register to get the single-instruction form).
__device__ __forceinline__ uint32_t qw_vgpr_const(uint32_t c) {
    uint32_t v = c;
    asm volatile("" : "+v"(v));
    return v;
}
__device__ __forceinline__ uint32_t qw_and_or(uint32_t a, uint32_t mask_s, uint32_t magic_v) {
    // plain C on purpose: with the magic in a VGPR the compiler selects v_and_or_b32 itself, and unlike an
    // inline-asm statement the result stays visible to the instruction scheduler as an ordinary VALU op
    return (a & mask_s) | magic_v;
}

// 8 HQ4_G32_M5 weights of one u32 word as four half2 (elements 0..7 in order): the nibble of element
// 8w+j sits at bit 4*(j>>1) + 16*(j&1), so ((word >> 4k) & 0x000F000F) | 0x64006400 viewed as half2 is
// (1024+q[2k], 1024+q[2k+1]); one packed f16 FMA with (scale, bias) gives RN_f16((1024+q)*s + b)
// (unpack_hq4_word8, Sources/QWMetal/include/qw_dequant.metalh:42-62).  `magic` = qw_vgpr_const(0x64006400).
__device__ __forceinline__ void qw_unpack_hq4_word(uint32_t word, h2_t s2, h2_t b2, uint32_t magic, h2_t* w) {
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        const uint32_t m = qw_and_or(word >> (4 * k), 0x000F000Fu, magic);
        w[k] = __builtin_elementwise_fma(__builtin_bit_cast(h2_t, m), s2, b2);
    }
}

__device__ __forceinline__ h2_t qw_splat_lo(uint32_t hdr) { return __builtin_bit_cast(h2_t, (hdr & 0xFFFFu) * 0x10001u); }
__device__ __forceinline__ h2_t qw_splat_hi(uint32_t hdr) { return __builtin_bit_cast(h2_t, (hdr >> 16) * 0x10001u); }

// Sum over the 32 lanes of a half-wavefront (xor butterflies stay inside each aligned 32-lane half).
__device__ __forceinline__ float qw_reduce32(float v) {
#pragma unroll
    for (int off = 16; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}
__device__ __forceinline__ float qw_reduce64(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}

// ------------------------------------------------------------------------------------------------
// FWHT-32 on the matrix cores.  For 16 consecutive 32-groups, rot[g][i] = sum_k H[i][k] x[g][k] is one
// 16x16x32 MFMA per half of the outputs: A = H rows (entries +-1, exact in f16), B = the activations
// (column j = group, lane (j, c) holds x[g_j][8c .. 8c+7] straight from one 16-byte load), fp32
// accumulate; the 1/sqrt(32) is applied in fp32 afterwards and the result is rounded once to f16.
// The products are exact and the sum is an fp32 sum of 32 terms, so the result can differ from the
// butterfly order only in the last fp32 bit before the f16 rounding.  VALU cost per wave and 16
// groups: ~20 instructions instead of ~260 for the in-register butterflies, and the work spreads
// over all four SIMDs of the workgroup.
// ------------------------------------------------------------------------------------------------
__device__ __forceinline__ h8_t qw_hadamard_rows(uint32_t i, uint32_t c) {
    // H[i][8c + e], e = 0..7: sign = parity(i & (8c + e)) = parity(i & 8c) ^ parity(i & e)
    const uint32_t pc = __popc(i & (8u * c)) & 1u;
    u4_t bits;
#pragma unroll
    for (int pr = 0; pr < 4; ++pr) {
        const uint32_t p0 = (pc ^ __popc(i & (uint32_t)(2 * pr))) & 1u;
        const uint32_t p1 = (pc ^ __popc(i & (uint32_t)(2 * pr + 1))) & 1u;
        bits[pr] = (0x3C00u | (p0 << 15)) | ((0x3C00u | (p1 << 15)) << 16);
    }
    return __builtin_bit_cast(h8_t, bits);
}

// 8 activations loaded as 16 raw bytes (f16 or bf16) -> f16
template <int XDT>
__device__ __forceinline__ h8_t qw_x8_from_raw(u4_t raw) {
    if constexpr (XDT == QWHIP_F16) {
        return __builtin_bit_cast(h8_t, raw);
    } else {
        h8_t o;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            o[2 * j] = (h1_t)__uint_as_float(raw[j] << 16);
            o[2 * j + 1] = (h1_t)__uint_as_float(raw[j] & 0xFFFF0000u);
        }
        return o;
    }
}

template <int XDT>
__device__ __forceinline__ h8_t qw_load_x8_f16(const void* x, uint64_t elem) {
    return qw_x8_from_raw<XDT>(*(const u4_t*)((const uint16_t*)x + elem));
}

// Rows i and i + 16 (i = lane & 15) of the 32-point Hadamard matrix, columns 8c .. 8c + 7 (c = lane >> 4), as f16 +-1:
// sign(i, k) = parity(i & k); for i < 16 that is parity(i & 8c) ^ parity(i & e) with only bit 3 of i meeting 8c, and
// row i + 16 flips the sign where k >= 16.
__device__ __forceinline__ void qw_hadamard_pair(uint32_t i, uint32_t c, h8_t& lo, h8_t& hi) {
    const uint32_t b0 = i & 1u, b1 = (i >> 1) & 1u, b2 = (i >> 2) & 1u;
    const uint32_t pc = (c & 1u) & ((i >> 3) & 1u);
    const uint32_t s0 = pc, s1 = pc ^ b0, s2 = pc ^ b1, s3 = s1 ^ b1, s4 = pc ^ b2, s5 = s1 ^ b2, s6 = s2 ^ b2, s7 = s3 ^ b2;
    u4_t w;
    w[0] = 0x3C003C00u | (s0 << 15) | (s1 << 31);
    w[1] = 0x3C003C00u | (s2 << 15) | (s3 << 31);
    w[2] = 0x3C003C00u | (s4 << 15) | (s5 << 31);
    w[3] = 0x3C003C00u | (s6 << 15) | (s7 << 31);
    lo = __builtin_bit_cast(h8_t, w);
    const uint32_t flip = (c >= 2u) ? 0x80008000u : 0u;
    const u4_t v = {w[0] ^ flip, w[1] ^ flip, w[2] ^ flip, w[3] ^ flip};
    hi = __builtin_bit_cast(h8_t, v);
}

// Sum over each aligned 32-lane half; the result is valid in lanes 16..31 (half 0) and 48..63 (half 1).
__device__ __forceinline__ float qw_reduce32_dpp(float v) {
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1, 0xF, 0xF, true));   // quad_perm [1,0,3,2]
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4E, 0xF, 0xF, true));   // quad_perm [2,3,0,1]
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x141, 0xF, 0xF, true));  // row_half_mirror
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x140, 0xF, 0xF, true));  // row_mirror
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x142, 0xA, 0xF, true));  // row_bcast15 into rows 1, 3
    return v;
}

// Rotates (or just converts) the 16 groups of tile `gt` from the operand `xb` this lane loaded and writes
// them to LDS (80-byte pitch per group).
__device__ __forceinline__ void qw_rotate_tile_to_lds(h8_t xb, uint32_t gt, uint32_t nb, uint32_t lane, bool rotate,
                                                      h8_t h_lo, h8_t h_hi, h8_t* xs) {
    const uint32_t j = lane & 15u, c = lane >> 4;
    const uint32_t g = gt * 16u + j;
    h1_t* base = (h1_t*)xs + (uint64_t)g * 40u;
    if (rotate) {
        f4_t d0 = {0.f, 0.f, 0.f, 0.f}, d1 = {0.f, 0.f, 0.f, 0.f};
        d0 = __builtin_amdgcn_mfma_f32_16x16x32_f16(h_lo, xb, d0, 0, 0, 0);
        d1 = __builtin_amdgcn_mfma_f32_16x16x32_f16(h_hi, xb, d1, 0, 0, 0);
        if (g < nb) {
            h4_t o0, o1;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                o0[r] = (h1_t)(d0[r] * QW_INV_SQRT32);
                o1[r] = (h1_t)(d1[r] * QW_INV_SQRT32);
            }
            *(h4_t*)(base + 4u * c) = o0;
            *(h4_t*)(base + 16u + 4u * c) = o1;
        }
    } else if (g < nb) {
        *(h8_t*)(base + 8u * c) = xb;
    }
}


// ---- argument blocks as scalar kernel arguments ---------------------------------------------------------------------
// A kernel that takes its argument block as one struct reads it with scalar loads at the start of every wave: a full memory
// round trip before the first useful load can be issued.  The same members passed as separate, typed kernel arguments are
// preloaded into SGPRs by the command processor (the library is compiled with -amdgpu-kernarg-preload-count; the first 14
// dwords fit, the rest is still loaded) and the wave starts with its pointers in hand: 5.32 -> 5.05 us on the 10 MB decode
// GEMV, 0.1 us on the larger ones, measured side by side.  The arguments keep their types: a pointer rebuilt from two
// 32-bit scalars loses its address space and every access through it becomes a flat instruction (measured: 11.3 -> 12.1 us
// on the 55 MB GEMV).
// QW_ARG_BLOCK(NAME, FIELDS) declares struct NAME from the list FIELDS(X) = X(type, name) ..., a kernel that takes the
// members one by one and runs Body::run(const NAME&), and its launcher.  Body: `static constexpr int kLaunchBound` and
// `static __device__ void run(const NAME&)`.  What the first loads of a wave need comes first in the list.  The kernel takes
// exactly the members: one spare trailing argument cost the 55 MB GEMV 1.6 % (11.27 -> 11.46 us) in the same comparison.
// Kernels that measured no faster this way keep their struct argument (the transposing GEMV).
#define QW_ARG_MEMBER(T, n) T n;
#define QW_ARG_PARAM(T, n) , T n
#define QW_ARG_COPY(T, n) p.n = n;
#define QW_ARG_PASS(T, n) , p.n
#define QW_DROP_FIRST_(first, ...) __VA_ARGS__
#define QW_DROP_FIRST(...) QW_DROP_FIRST_(__VA_ARGS__)
#define QW_ARG_BLOCK(NAME, FIELDS)                                                                                        \
    struct NAME {                                                                                                         \
        FIELDS(QW_ARG_MEMBER)                                                                                             \
    };                                                                                                                    \
    template <typename Body>                                                                                              \
    __global__ __launch_bounds__(Body::kLaunchBound) void qw_typed_kernel_##NAME(QW_DROP_FIRST(FIELDS(QW_ARG_PARAM))) {   \
        NAME p;                                                                                                           \
        FIELDS(QW_ARG_COPY)                                                                                               \
        Body::run(p);                                                                                                     \
    }                                                                                                                     \
    template <typename Body>                                                                                              \
    inline void qw_launch_scalar(dim3 grid, dim3 block, size_t lds, hipStream_t st, const NAME& p) {                      \
        hipLaunchKernelGGL((qw_typed_kernel_##NAME<Body>), grid, block, lds, st FIELDS(QW_ARG_PASS));                     \
    }                                                                                                                     \
    template <typename Body>                                                                                              \
    inline const void* qw_scalar_kernel_ptr(const NAME*) {                                                                \
        return (const void*)qw_typed_kernel_##NAME<Body>;                                                                 \
    }
