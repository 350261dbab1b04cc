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
// Bit-stream block writer: bf16 / f32 weights -> [f16 scale][f16 bias][codes, element i at bit i * bits] for bits in
// {2, 3, 4, 6, 8} and groups of 32 .. 256, byte-identical to the packer (quant_hq_blocks, Scripts/quantize/hq_blocks.py:436-517;
// its GPU twin is the quant_hq_simd shader at :260).  A lane owns 32 consecutive weights (one rotation group), the
// group / 32 neighbouring lanes of a quant group share minimum and maximum; every operation is a single IEEE fp32 operation
// in the packer's order:  scale = f16((max - min) / qmax), bias = f16(min), code = clamp(rint((w - bias) / scale), 0, qmax),
// scale == 0 -> code 0.  The 2- and 3-bit widths pick scale and bias by the packer's ten-point shrink search (:409-432):
// the candidate with the smallest mean squared error wins, the first one on ties; the mean is summed in the order of the
// packer's array library (eight running sums over the group's elements in order, 128 elements at a time, combined pairwise),
// which the lanes of a group reproduce by passing the running sums from lane to lane.
// ------------------------------------------------------------------------------------------------
template <int DT, int BITS>
__global__ __launch_bounds__(256) void qw_quantize_blocks_kernel(const void* __restrict__ src, uint8_t* __restrict__ out,
                                                                  uint64_t subgroups, uint32_t lshift, uint32_t rotate, uint32_t mse) {
    const uint64_t sg0 = (uint64_t)blockIdx.x * 256 + threadIdx.x;
    const bool live = sg0 < subgroups;                 // a quant group's lanes are live or idle together
    const uint64_t sg = live ? sg0 : subgroups - 1u;
    const uint32_t L = 1u << lshift, lig = threadIdx.x & (L - 1u);
    float v[32];
#pragma unroll
    for (int j = 0; j < 4; ++j) qw_load8_f32<DT>(src, sg * 32 + 8 * j, v + 8 * j);
    if (rotate) qw_fwht32(v);
    float mn = v[0], mx = v[0];
#pragma unroll
    for (int i = 1; i < 32; ++i) {
        mn = fminf(mn, v[i]);
        mx = fmaxf(mx, v[i]);
    }
    for (uint32_t off = 1; off < L; off <<= 1) {
        mn = fminf(mn, __shfl_xor(mn, (int)off, 64));
        mx = fmaxf(mx, __shfl_xor(mx, (int)off, 64));
    }
    constexpr float qmax = (float)((1 << BITS) - 1);
    h1_t sc16 = (h1_t)((mx - mn) / qmax), bi16 = (h1_t)mn;
    if (mse) {
        const float mid = 0.5f * (mx + mn), half_span = 0.5f * (mx - mn);
        const float shrinks[10] = {1.00f, 0.96f, 0.92f, 0.88f, 0.85f, 0.82f, 0.79f, 0.76f, 0.73f, 0.70f};
        const uint32_t Lh = L < 4u ? L : 4u;           // lanes of one 128-element half
        const uint32_t first = threadIdx.x & ~(L - 1u) & 63u;
        float best = __builtin_inff();
        for (int c = 0; c < 10; ++c) {
            const float c_min = mid - shrinks[c] * half_span, c_max = mid + shrinks[c] * half_span;
            const h1_t s16 = (h1_t)((c_max - c_min) / qmax), b16 = (h1_t)c_min;
            const float s = (float)s16, b = (float)b16;
            const float safe = s > 0.0f ? s : 1.0f;
            float dd[32];
#pragma unroll
            for (int i = 0; i < 32; ++i) {
                float q = fminf(fmaxf(__builtin_rintf((v[i] - b) / safe), 0.0f), qmax);
                q = s > 0.0f ? q : 0.0f;
                const float d = v[i] - (q * s + b);
                dd[i] = d * d;
            }
            float r[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) r[j] = 0.0f;
            for (uint32_t k = 0; k < Lh; ++k) {
                float in[8];
#pragma unroll
                for (int j = 0; j < 8; ++j) in[j] = __shfl_up(r[j], 1, 64);
                if ((lig & (Lh - 1u)) == k) {
#pragma unroll
                    for (int j = 0; j < 8; ++j) {
                        float a = k == 0 ? dd[j] : in[j] + dd[j];
                        a += dd[8 + j];
                        a += dd[16 + j];
                        a += dd[24 + j];
                        r[j] = a;
                    }
                }
            }
            const float res = ((r[0] + r[1]) + (r[2] + r[3])) + ((r[4] + r[5]) + (r[6] + r[7]));
            float sum = __shfl(res, (int)(first + Lh - 1u), 64);
            if (L > 4u) sum = sum + __shfl(res, (int)(first + L - 1u), 64);
            const float err = sum / (float)(32u << lshift);
            if (err < best) {
                best = err;
                sc16 = s16;
                bi16 = b16;
            }
        }
    }
    const float s = (float)sc16, b = (float)bi16;
    const float safe = s > 0.0f ? s : 1.0f;
    uint32_t words[BITS];
#pragma unroll
    for (int w = 0; w < BITS; ++w) words[w] = 0u;
#pragma unroll
    for (int i = 0; i < 32; ++i) {
        float qf = fminf(fmaxf(__builtin_rintf((v[i] - b) / safe), 0.0f), qmax);
        const uint32_t q = s > 0.0f ? (uint32_t)qf : 0u;
        constexpr int dummy = 0;
        (void)dummy;
        const int bit = i * BITS, w = bit >> 5, sh = bit & 31;
        words[w] |= q << sh;
        if (sh + BITS > 32) words[w + 1] |= q >> (32 - sh);
    }
    if (!live) return;
    const uint32_t bb = 4u + (BITS * 4u << lshift);
    uint32_t* dst = (uint32_t*)(out + (sg >> lshift) * bb);
    if (lig == 0u) dst[0] = (uint32_t)__builtin_bit_cast(uint16_t, sc16) | ((uint32_t)__builtin_bit_cast(uint16_t, bi16) << 16);
#pragma unroll
    for (int w = 0; w < BITS; ++w) dst[1 + lig * BITS + w] = words[w];
}

extern "C" qwhip_status qwhip_quantize_blocks(qwhip_stream_t s, const void* src, uint32_t src_dtype, uint32_t n, uint32_t k,
                                              uint32_t bits, uint32_t group, uint32_t rotate, uint32_t mse_clip, void* blocks_out) {
    QWHIP_REQUIRE(s);
    QWHIP_REQUIRE(src);
    QWHIP_REQUIRE(blocks_out);
    if (qwhip_block_bytes(rotate ? QWHIP_KIND_ROTATED_HQ : QWHIP_KIND_NATIVE_AFFINE, bits, group) == 0)
        return qwhip_fail(QWHIP_E_BAD_WEIGHTS, "no block container for %u bits, group %u", bits, group);
    if (n == 0 || k == 0 || k % group != 0)
        return qwhip_fail(QWHIP_E_BAD_SHAPE, "block quantizer requires a non-empty 2-D tensor with K divisible by the group (n=%u k=%u group=%u)", n, k, group);
    if (((uintptr_t)src & 15u) || ((uintptr_t)blocks_out & 3u))
        return qwhip_fail(QWHIP_E_BAD_SHAPE, "quantizer needs a 16-byte aligned source and a 4-byte aligned bank");
    if (mse_clip > 2u) return qwhip_fail(QWHIP_E_BAD_SHAPE, "mse_clip is 0 (off), 1 (on) or 2 (the packer's default: on for 2 and 3 bits)");
    const uint32_t mse = mse_clip == 2u ? (bits <= 3u ? 1u : 0u) : mse_clip;
    const uint64_t subgroups = (uint64_t)n * (k / 32);
    const uint32_t lshift = group == 32 ? 0u : (group == 64 ? 1u : (group == 128 ? 2u : 3u));
    const dim3 grid((unsigned)((subgroups + 255) / 256)), block(256);
#define QW_QB(DT, B) hipLaunchKernelGGL((qw_quantize_blocks_kernel<DT, B>), grid, block, 0, s->stream, src, (uint8_t*)blocks_out, subgroups, lshift, rotate, mse)
#define QW_QB_BITS(DT)                                                                                          \
    switch (bits) {                                                                                             \
        case 2: QW_QB(DT, 2); break; case 3: QW_QB(DT, 3); break; case 4: QW_QB(DT, 4); break;                  \
        case 6: QW_QB(DT, 6); break; default: QW_QB(DT, 8); break;                                              \
    }
    if (src_dtype == QWHIP_BF16) { QW_QB_BITS(QWHIP_BF16) }
    else if (src_dtype == QWHIP_F32) { QW_QB_BITS(QWHIP_F32) }
    else return qwhip_fail(QWHIP_E_BAD_SHAPE, "quantizer source must be bf16 or f32, got dtype %u", src_dtype);
#undef QW_QB_BITS
#undef QW_QB
    QWHIP_TRY_HIP(hipGetLastError());
    return QWHIP_OK;
}

// ------------------------------------------------------------------------------------------------
// Planar HQ8_G32_M5: int8 codes [n, k] + f16 scales [n, k / 32], symmetric, rotated (quant_hq8_g32_m5 /
// dequant_hq8_g32_m5_rot, Scripts/quantize/hq_blocks.py:564-615; host reader dequantHQ8Rot,
// Sources/Foundation/QWQuant/QWPack.swift:326-351):  scale = f16(amax / 127), code = clamp(rint(w_rot / scale), -127, 127),
// scale == 0 -> code 0;  w_rot = code * scale in fp32.  One lane per 32-weight group.
// ------------------------------------------------------------------------------------------------
template <int DT>
__global__ __launch_bounds__(256) void qw_quantize_hq8_planar_kernel(const void* __restrict__ src, int8_t* __restrict__ qs,
                                                                      h1_t* __restrict__ scales, uint64_t groups, uint32_t rotate) {
    const uint64_t g = (uint64_t)blockIdx.x * 256 + threadIdx.x;
    if (g >= groups) return;
    float v[32];
#pragma unroll
    for (int j = 0; j < 4; ++j) qw_load8_f32<DT>(src, g * 32 + 8 * j, v + 8 * j);
    if (rotate) qw_fwht32(v);
    float amax = 0.0f;
#pragma unroll
    for (int i = 0; i < 32; ++i) amax = fmaxf(amax, fabsf(v[i]));
    const h1_t sc16 = (h1_t)(amax / 127.0f);
    const float s = (float)sc16;
    const float safe = s > 0.0f ? s : 1.0f;
    u4_t w[2];
#pragma unroll
    for (int i = 0; i < 32; ++i) {
        const float qf = fminf(fmaxf(__builtin_rintf(v[i] / safe), -127.0f), 127.0f);
        const uint32_t q = s > 0.0f ? ((uint32_t)(int32_t)qf & 0xFFu) : 0u;
        if ((i & 3) == 0) w[i >> 4][(i >> 2) & 3] = q;
        else w[i >> 4][(i >> 2) & 3] |= q << (8 * (i & 3));
    }
    *(u4_t*)(qs + g * 32) = w[0];
    *(u4_t*)(qs + g * 32 + 16) = w[1];
    scales[g] = sc16;
}

__global__ __launch_bounds__(256) void qw_dequant_hq8_planar_kernel(const int8_t* __restrict__ qs, const h1_t* __restrict__ scales,
                                                                     float* __restrict__ out, uint64_t groups) {
    const uint64_t t = (uint64_t)blockIdx.x * 256 + threadIdx.x;   // eight codes per thread
    if (t >= groups * 4u) return;
    const float s = (float)scales[t >> 2];
    const u2_t raw = *(const u2_t*)(qs + t * 8);
    f4_t lo, hi;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        lo[j] = (float)(int8_t)(raw[0] >> (8 * j)) * s;
        hi[j] = (float)(int8_t)(raw[1] >> (8 * j)) * s;
    }
    *(f4_t*)(out + t * 8) = lo;
    *(f4_t*)(out + t * 8 + 4) = hi;
}

extern "C" qwhip_status qwhip_quantize_hq8_planar(qwhip_stream_t s, const void* src, uint32_t src_dtype, uint32_t n, uint32_t k,
                                                  uint32_t rotate, void* qs_out, void* scales_out_f16) {
    QWHIP_REQUIRE(s);
    QWHIP_REQUIRE(src);
    QWHIP_REQUIRE(qs_out);
    QWHIP_REQUIRE(scales_out_f16);
    if (n == 0 || k == 0 || k % 32 != 0)
        return qwhip_fail(QWHIP_E_BAD_SHAPE, "planar HQ8 requires a non-empty 2-D tensor with K divisible by 32 (n=%u k=%u)", n, k);
    if (((uintptr_t)src & 15u) || ((uintptr_t)qs_out & 15u) || ((uintptr_t)scales_out_f16 & 1u))
        return qwhip_fail(QWHIP_E_BAD_SHAPE, "planar HQ8 needs 16-byte aligned source and code planes");
    const uint64_t groups = (uint64_t)n * (k / 32);
    const dim3 grid((unsigned)((groups + 255) / 256)), block(256);
    if (src_dtype == QWHIP_BF16) hipLaunchKernelGGL(qw_quantize_hq8_planar_kernel<QWHIP_BF16>, grid, block, 0, s->stream, src, (int8_t*)qs_out, (h1_t*)scales_out_f16, groups, rotate);
    else if (src_dtype == QWHIP_F32) hipLaunchKernelGGL(qw_quantize_hq8_planar_kernel<QWHIP_F32>, grid, block, 0, s->stream, src, (int8_t*)qs_out, (h1_t*)scales_out_f16, groups, rotate);
    else return qwhip_fail(QWHIP_E_BAD_SHAPE, "quantizer source must be bf16 or f32, got dtype %u", src_dtype);
    QWHIP_TRY_HIP(hipGetLastError());
    return QWHIP_OK;
}

extern "C" qwhip_status qwhip_dequant_hq8_planar(qwhip_stream_t s, const void* qs, const void* scales_f16, uint32_t n, uint32_t k,
                                                 float* out_f32) {
    QWHIP_REQUIRE(s);
    QWHIP_REQUIRE(qs);
    QWHIP_REQUIRE(scales_f16);
    QWHIP_REQUIRE(out_f32);
    if (n == 0 || k == 0 || k % 32 != 0)
        return qwhip_fail(QWHIP_E_BAD_SHAPE, "planar HQ8 requires a non-empty 2-D tensor with K divisible by 32 (n=%u k=%u)", n, k);
    if (((uintptr_t)qs & 7u) || ((uintptr_t)out_f32 & 15u) || ((uintptr_t)scales_f16 & 1u))
        return qwhip_fail(QWHIP_E_BAD_SHAPE, "planar HQ8 dequant needs an 8-byte aligned code plane and a 16-byte aligned output");
    const uint64_t groups = (uint64_t)n * (k / 32);
    const dim3 grid((unsigned)((groups * 4u + 255) / 256)), block(256);
    hipLaunchKernelGGL(qw_dequant_hq8_planar_kernel, grid, block, 0, s->stream, (const int8_t*)qs, (const h1_t*)scales_f16, out_f32, groups);
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
