// Load-time writer: bf16 / f32 weights -> HQ4_G32_M5 blocks on the device, byte-identical to the
// packer (quant_hq4_blocks, Scripts/quantize/hq4.py:54-123; GPU twin qwg_quantize_bf16_to_hq4_g32_m5,
// Sources/QWMetal/quant/qw_online_quant.metal:17-55).  One lane owns one 32-weight group; every
// operation is a single IEEE fp32 operation in the packer's order (no contraction).
#include "qwhip_common.h"

template <int DT>
__global__ __launch_bounds__(256) void qw_quantize_hq4_kernel(const void* __restrict__ src, uint8_t* __restrict__ out,
                                                               uint64_t groups, uint32_t rotate) {
    const uint64_t g = (uint64_t)blockIdx.x * 256 + threadIdx.x;
    if (g >= groups) return;
    float v[32];
#pragma unroll
    for (int j = 0; j < 4; ++j) qw_load8_f32<DT>(src, g * 32 + 8 * j, v + 8 * j);
    if (rotate) qw_fwht32(v);
    float amax = 0.0f;
#pragma unroll
    for (int i = 0; i < 32; ++i) amax = fmaxf(amax, fabsf(v[i]));
    const h1_t scale16 = (h1_t)fminf(amax / 7.5f, 63.46875f);
    const float s = (float)scale16;
    const h1_t bias16 = (h1_t)(-1032.0f * s);
    const float b = (float)bias16;
    uint32_t q[32];
    if (s > 0.0f) {
#pragma unroll
        for (int i = 0; i < 32; ++i) {
            const float t = floorf((v[i] - b) / s - 1023.5f);
            q[i] = (uint32_t)fminf(fmaxf(t, 0.0f), 15.0f);
        }
    } else {
#pragma unroll
        for (int i = 0; i < 32; ++i) q[i] = 8u;
    }
    qw_hq4_block blk;
    blk.hdr = (uint32_t)__builtin_bit_cast(uint16_t, scale16) | ((uint32_t)__builtin_bit_cast(uint16_t, bias16) << 16);
#pragma unroll
    for (int w = 0; w < 4; ++w) {
        const uint32_t* e = q + 8 * w;
        blk.qs[w] = e[0] | (e[1] << 16) | (e[2] << 4) | (e[3] << 20) | (e[4] << 8) | (e[5] << 24) | (e[6] << 12) | (e[7] << 28);
    }
    *(qw_hq4_block*)(out + g * 20) = blk;
}

extern "C" qwhip_status qwhip_quantize_hq4_g32(qwhip_stream_t s, const void* src, uint32_t src_dtype, uint32_t n, uint32_t k,
                                               uint32_t rotate, void* blocks_out) {
    QWHIP_REQUIRE(s);
    QWHIP_REQUIRE(src);
    QWHIP_REQUIRE(blocks_out);
    if (n == 0 || k == 0 || k % 32 != 0)
        return qwhip_fail(QWHIP_E_BAD_SHAPE, "HQ4_G32_M5 requires a non-empty 2-D tensor with K divisible by 32 (n=%u k=%u)", n, k);
    if (((uintptr_t)src & 15u) || ((uintptr_t)blocks_out & 3u))
        return qwhip_fail(QWHIP_E_BAD_SHAPE, "quantizer needs a 16-byte aligned source and a 4-byte aligned bank");
    const uint64_t groups = (uint64_t)n * (k / 32);
    const dim3 grid((unsigned)((groups + 255) / 256)), block(256);
    if (src_dtype == QWHIP_BF16) hipLaunchKernelGGL(qw_quantize_hq4_kernel<QWHIP_BF16>, grid, block, 0, s->stream, src, (uint8_t*)blocks_out, groups, rotate);
    else if (src_dtype == QWHIP_F32) hipLaunchKernelGGL(qw_quantize_hq4_kernel<QWHIP_F32>, grid, block, 0, s->stream, src, (uint8_t*)blocks_out, groups, rotate);
    else return qwhip_fail(QWHIP_E_BAD_SHAPE, "quantizer source must be bf16 or f32, got dtype %u", src_dtype);
    QWHIP_TRY_HIP(hipGetLastError());
    return QWHIP_OK;
}

// ------------------------------------------------------------------------------------------------
// MLX affine checkpoint -> AQ blocks at the same byte count (qwg_repack_mlx_affine_to_aq_m5 and its switch gate|up
// variant, Sources/QWMetal/quant/qw_online_quant.metal:56-178; doors Sources/Foundation/QWLoad/AQRepack.swift:108-250).
// A block is [f16 scale][f16 bias][payload]: the payload bytes are the checkpoint's, the header is the checkpoint's
// bf16 / f16 scale and bias as f16.  A header that f16 does not hold (overflow, or a value lost in the normal range;
// below 2^-14 the nearest subnormal is accepted) is poisoned with the f16 NaN 0x7e00 and counted in `refused`.
// Threads walk the output dwords (header word or payload word) in order, so both streams are read and written in whole lines.
// ------------------------------------------------------------------------------------------------
__device__ __forceinline__ float qw_read_scale(const uint16_t* p, uint32_t is_f16, uint64_t i) {
    const uint16_t b = p[i];
    return is_f16 ? (float)__builtin_bit_cast(h1_t, b) : qw_bf16_to_f32(b);
}

__device__ __forceinline__ bool qw_f16_header_holds(float raw, h1_t stored) {
    const float back = (float)stored;
    if (back == raw) return true;
    const bool fin = (__float_as_uint(raw) & 0x7F800000u) != 0x7F800000u && (__float_as_uint(back) & 0x7F800000u) != 0x7F800000u;
    return fin && fabsf(raw) < 6.103515625e-5f;
}

// SWITCH: source rows come from two [experts, inter, cols] tensors interleaved per expert as [gate rows | up rows].
// IDX is the type the dword index is divided in: u32 whenever the plane has fewer than 2^32 dwords.  A thread owns four
// consecutive output dwords (one 16-byte store when VEC): one division finds the first dword's block, the others step.
template <bool SWITCH, typename IDX, bool VEC>
__global__ __launch_bounds__(256) void qw_repack_mlx_kernel(const uint32_t* __restrict__ w0, const uint16_t* __restrict__ s0,
                                                            const uint16_t* __restrict__ b0, const uint32_t* __restrict__ w1,
                                                            const uint16_t* __restrict__ s1, const uint16_t* __restrict__ b1,
                                                            uint32_t* __restrict__ dst, uint64_t total, uint32_t groups,
                                                            uint32_t pay_words, uint32_t inter, uint32_t is_f16,
                                                            uint32_t* __restrict__ refused) {
    const uint32_t W = pay_words + 1u;
    const IDX d0 = ((IDX)blockIdx.x * 256u + threadIdx.x) * 4u;
    if ((uint64_t)d0 >= total) return;
    IDX b = d0 / (IDX)W;
    uint32_t j = (uint32_t)(d0 - b * (IDX)W);
    uint32_t out[4];
    uint32_t bad = 0;
#pragma unroll
    for (int t = 0; t < 4; ++t) {
        out[t] = 0u;
        if ((uint64_t)d0 + (uint32_t)t < total) {
            IDX src_group = b;
            const uint32_t* w = w0;
            const uint16_t* sc = s0;
            const uint16_t* bi = b0;
            if constexpr (SWITCH) {
                const IDX out_row = b / (IDX)groups;
                const uint32_t g = (uint32_t)(b - out_row * (IDX)groups);
                const IDX e = out_row / (IDX)(2u * inter);
                const uint32_t local = (uint32_t)(out_row - e * (IDX)(2u * inter));
                const bool up = local >= inter;
                src_group = (e * (IDX)inter + (up ? local - inter : local)) * (IDX)groups + g;
                if (up) {
                    w = w1;
                    sc = s1;
                    bi = b1;
                }
            }
            if (j == 0u) {
                const float rs = qw_read_scale(sc, is_f16, src_group), rb = qw_read_scale(bi, is_f16, src_group);
                const h1_t hs = (h1_t)rs, hb = (h1_t)rb;
                const bool exact = qw_f16_header_holds(rs, hs) && qw_f16_header_holds(rb, hb);
                bad += exact ? 0u : 1u;
                const uint32_t lo = exact ? (uint32_t)__builtin_bit_cast(uint16_t, hs) : 0x7E00u;
                const uint32_t hi = exact ? (uint32_t)__builtin_bit_cast(uint16_t, hb) : 0x7E00u;
                out[t] = lo | (hi << 16);
            } else {
                out[t] = w[(uint64_t)src_group * pay_words + (j - 1u)];
            }
        }
        if (++j == W) {
            j = 0u;
            ++b;
        }
    }
    if (bad) atomicAdd(refused, bad);
    if (VEC && (uint64_t)d0 + 4u <= total) {
        *(u4_t*)(dst + d0) = u4_t{out[0], out[1], out[2], out[3]};
    } else {
#pragma unroll
        for (int t = 0; t < 4; ++t)
            if ((uint64_t)d0 + (uint32_t)t < total) dst[(uint64_t)d0 + (uint32_t)t] = out[t];
    }
}

template <bool SWITCH>
static void qw_repack_launch(hipStream_t st, const void* w0, const void* s0, const void* b0, const void* w1, const void* s1,
                             const void* b1, void* dst, uint64_t total, uint32_t groups, uint32_t pay_words, uint32_t inter,
                             uint32_t is_f16, uint32_t* refused) {
    const dim3 grid((unsigned)((total + 1023u) / 1024u)), block(256);
    const bool vec = ((uintptr_t)dst & 15u) == 0;
    const bool narrow = total + 4u < (1ull << 32);
#define QW_REPACK_GO(IDX, VEC)                                                                                                   \
    hipLaunchKernelGGL((qw_repack_mlx_kernel<SWITCH, IDX, VEC>), grid, block, 0, st, (const uint32_t*)w0, (const uint16_t*)s0,   \
                       (const uint16_t*)b0, (const uint32_t*)w1, (const uint16_t*)s1, (const uint16_t*)b1, (uint32_t*)dst, total, \
                       groups, pay_words, inter, is_f16, refused)
    if (narrow && vec) QW_REPACK_GO(uint32_t, true);
    else if (narrow) QW_REPACK_GO(uint32_t, false);
    else if (vec) QW_REPACK_GO(uint64_t, true);
    else QW_REPACK_GO(uint64_t, false);
#undef QW_REPACK_GO
}

namespace {
qwhip_status repack_checks(qwhip_stream_t s, uint32_t scale_dtype, uint64_t rows, uint32_t cols, uint32_t bits, uint32_t group,
                           const void* dst, const uint32_t* refused) {
    QWHIP_REQUIRE(s);
    QWHIP_REQUIRE(dst);
    QWHIP_REQUIRE(refused);
    if (scale_dtype != QWHIP_BF16 && scale_dtype != QWHIP_F16)
        return qwhip_fail(QWHIP_E_BAD_SHAPE, "MLX scales and biases are bf16 or f16, got dtype %u", scale_dtype);
    if (rows == 0 || cols == 0 || bits == 0 || bits > 8 || group == 0 || cols % group != 0 || (group * bits) % 32 != 0)
        return qwhip_fail(QWHIP_E_BAD_SHAPE, "invalid MLX group layout (rows=%llu cols=%u bits=%u group=%u)",
                          (unsigned long long)rows, cols, bits, group);
    if (((uintptr_t)dst & 3u) != 0) return qwhip_fail(QWHIP_E_BAD_SHAPE, "the AQ plane must be 4-byte aligned");
    return QWHIP_OK;
}
}  // namespace

extern "C" qwhip_status qwhip_repack_mlx_affine(qwhip_stream_t s, const void* mlx_w, const void* mlx_scales, const void* mlx_biases,
                                                uint32_t scale_dtype, uint32_t rows, uint32_t cols, uint32_t bits, uint32_t group,
                                                void* dst_blocks, uint32_t* refused) {
    qwhip_status st = repack_checks(s, scale_dtype, rows, cols, bits, group, dst_blocks, refused);
    if (st != QWHIP_OK) return st;
    QWHIP_REQUIRE(mlx_w);
    QWHIP_REQUIRE(mlx_scales);
    QWHIP_REQUIRE(mlx_biases);
    const uint32_t groups = cols / group, pay_words = group * bits / 32u;
    const uint64_t total = (uint64_t)rows * groups * (pay_words + 1u);
    qw_repack_launch<false>(s->stream, mlx_w, mlx_scales, mlx_biases, nullptr, nullptr, nullptr, dst_blocks, total, groups, pay_words,
                            0u, scale_dtype == QWHIP_F16 ? 1u : 0u, refused);
    QWHIP_TRY_HIP(hipGetLastError());
    return QWHIP_OK;
}

extern "C" qwhip_status qwhip_repack_mlx_affine_switch_gate_up(qwhip_stream_t s, const void* gate_w, const void* gate_scales,
                                                               const void* gate_biases, const void* up_w, const void* up_scales,
                                                               const void* up_biases, uint32_t scale_dtype, uint32_t experts,
                                                               uint32_t inter, uint32_t cols, uint32_t bits, uint32_t group,
                                                               void* dst_blocks, uint32_t* refused) {
    qwhip_status st = repack_checks(s, scale_dtype, (uint64_t)experts * 2u * inter, cols, bits, group, dst_blocks, refused);
    if (st != QWHIP_OK) return st;
    QWHIP_REQUIRE(gate_w);
    QWHIP_REQUIRE(gate_scales);
    QWHIP_REQUIRE(gate_biases);
    QWHIP_REQUIRE(up_w);
    QWHIP_REQUIRE(up_scales);
    QWHIP_REQUIRE(up_biases);
    const uint32_t groups = cols / group, pay_words = group * bits / 32u;
    const uint64_t total = (uint64_t)experts * 2u * inter * groups * (pay_words + 1u);
    qw_repack_launch<true>(s->stream, gate_w, gate_scales, gate_biases, up_w, up_scales, up_biases, dst_blocks, total, groups,
                           pay_words, inter, scale_dtype == QWHIP_F16 ? 1u : 0u, refused);
    QWHIP_TRY_HIP(hipGetLastError());
    return QWHIP_OK;
}
