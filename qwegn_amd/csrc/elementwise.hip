// Elementwise seams of the quantized matmul path: activation rotation, casts, SwiGLU(+FWHT),
// and the dequant-to-f16 side output used to check weights bit-for-bit.
#include "qwhip_common.h"

// ---- FWHT-32 over consecutive 32-groups: src (f16 | bf16 | f32) -> dst f16 ----------------------
// One lane owns one group: 64/128 bytes in, 64 bytes out, all butterflies in registers.
template <int DT>
__global__ __launch_bounds__(256) void qw_fwht32_kernel(const void* __restrict__ src, h1_t* __restrict__ dst,
                                                         uint64_t groups) {
    const uint64_t g = (uint64_t)blockIdx.x * 256 + threadIdx.x;
    if (g >= groups) return;
    float v[32];
#pragma unroll
    for (int j = 0; j < 4; ++j) qw_load8_f32<DT>(src, g * 32 + 8 * j, v + 8 * j);
    qw_fwht32(v);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        h8_t o;
#pragma unroll
        for (int e = 0; e < 8; ++e) o[e] = (h1_t)v[8 * j + e];
        *(h8_t*)(dst + g * 32 + 8 * j) = o;
    }
}

extern "C" qwhip_status qwhip_fwht32(qwhip_stream_t s, const void* src, uint32_t src_dtype, void* dst_f16, uint64_t n) {
    QWHIP_REQUIRE(s);
    if (n == 0) return QWHIP_OK;
    QWHIP_REQUIRE(src);
    QWHIP_REQUIRE(dst_f16);
    if (n % 32 != 0) return qwhip_fail(QWHIP_E_BAD_SHAPE, "fwht32: n=%llu is not a multiple of 32", (unsigned long long)n);
    if (((uintptr_t)src & 15u) || ((uintptr_t)dst_f16 & 15u))
        return qwhip_fail(QWHIP_E_BAD_SHAPE, "fwht32: buffers must be 16-byte aligned");
    const uint64_t groups = n / 32;
    const dim3 grid((unsigned)((groups + 255) / 256)), block(256);
    switch (src_dtype) {
        case QWHIP_F16: hipLaunchKernelGGL(qw_fwht32_kernel<QWHIP_F16>, grid, block, 0, s->stream, src, (h1_t*)dst_f16, groups); break;
        case QWHIP_BF16: hipLaunchKernelGGL(qw_fwht32_kernel<QWHIP_BF16>, grid, block, 0, s->stream, src, (h1_t*)dst_f16, groups); break;
        case QWHIP_F32: hipLaunchKernelGGL(qw_fwht32_kernel<QWHIP_F32>, grid, block, 0, s->stream, src, (h1_t*)dst_f16, groups); break;
        default: return qwhip_fail(QWHIP_E_BAD_SHAPE, "fwht32: unsupported source dtype %u", src_dtype);
    }
    QWHIP_TRY_HIP(hipGetLastError());
    return QWHIP_OK;
}

// ---- any -> f16 convert, 8 elements per lane (n % 8 == 0, 16-byte aligned) ----------------------------------
template <int DT>
__global__ __launch_bounds__(256) void qw_convert_f16_kernel(const void* __restrict__ src, h1_t* __restrict__ dst, uint64_t n8) {
    const uint64_t i = (uint64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n8) return;
    float v[8];
    qw_load8_f32<DT>(src, i * 8, v);
    h8_t o;
#pragma unroll
    for (int e = 0; e < 8; ++e) o[e] = (h1_t)v[e];
    *(h8_t*)(dst + i * 8) = o;
}

qwhip_status qw_convert_to_f16(qwhip_stream_t s, const void* src, uint32_t src_dtype, void* dst_f16, uint64_t n) {
    if (n % 8 != 0) return qwhip_fail(QWHIP_E_BAD_SHAPE, "convert: n=%llu is not a multiple of 8", (unsigned long long)n);
    const uint64_t n8 = n / 8;
    const dim3 grid((unsigned)((n8 + 255) / 256)), block(256);
    switch (src_dtype) {
        case QWHIP_F16: hipLaunchKernelGGL(qw_convert_f16_kernel<QWHIP_F16>, grid, block, 0, s->stream, src, (h1_t*)dst_f16, n8); break;
        case QWHIP_BF16: hipLaunchKernelGGL(qw_convert_f16_kernel<QWHIP_BF16>, grid, block, 0, s->stream, src, (h1_t*)dst_f16, n8); break;
        case QWHIP_F32: hipLaunchKernelGGL(qw_convert_f16_kernel<QWHIP_F32>, grid, block, 0, s->stream, src, (h1_t*)dst_f16, n8); break;
        default: return qwhip_fail(QWHIP_E_BAD_SHAPE, "convert: unsupported source dtype %u", src_dtype);
    }
    QWHIP_TRY_HIP(hipGetLastError());
    return QWHIP_OK;
}

// ---- f32 -> f16 cast ---------------------------------------------------------------------------
__global__ __launch_bounds__(256) void qw_cast_f32_f16_kernel(const float* __restrict__ src, h1_t* __restrict__ dst,
                                                               uint64_t n) {
    uint64_t i = ((uint64_t)blockIdx.x * 256 + threadIdx.x) * 8;
    if (i + 8 <= n && (((uintptr_t)(src + i) & 15u) == 0) && (((uintptr_t)(dst + i) & 15u) == 0)) {
        float v[8];
        qw_load8_f32<QWHIP_F32>(src, i, v);
        h8_t o;
#pragma unroll
        for (int e = 0; e < 8; ++e) o[e] = (h1_t)v[e];
        *(h8_t*)(dst + i) = o;
    } else {
        for (int e = 0; e < 8 && i + e < n; ++e) dst[i + e] = (h1_t)src[i + e];
    }
}

extern "C" qwhip_status qwhip_cast_f32_to_f16(qwhip_stream_t s, const float* src, void* dst_f16, uint64_t n) {
    QWHIP_REQUIRE(s);
    if (n == 0) return QWHIP_OK;
    QWHIP_REQUIRE(src);
    QWHIP_REQUIRE(dst_f16);
    const uint64_t threads = (n + 7) / 8;
    hipLaunchKernelGGL(qw_cast_f32_f16_kernel, dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, s->stream, src,
                       (h1_t*)dst_f16, n);
    QWHIP_TRY_HIP(hipGetLastError());
    return QWHIP_OK;
}

// ---- SwiGLU (+ FWHT-32): gu [rows, 2I] (gate | up) -> act [rows, I] f16 ---------------------------
// SwiGLU runs in fp32 on the values as stored (f16 inputs are the rounded values the fused prefill
// path also sees, Sources/QWMetal/include/qw_gemm_nax_swiglu.metalh:132-152); rotation in fp32, one
// f16 rounding on store.
template <int DT, bool ROT>
__global__ __launch_bounds__(256) void qw_swiglu_fwht_kernel(const void* __restrict__ gu, h1_t* __restrict__ act,
                                                              uint32_t rows, uint32_t inter, const qw_act ga) {
    const uint32_t gpr = inter / 32;  // groups per row
    const uint64_t gid = (uint64_t)blockIdx.x * 256 + threadIdx.x;
    if (gid >= (uint64_t)rows * gpr) return;
    const uint32_t r = (uint32_t)(gid / gpr), g = (uint32_t)(gid % gpr);
    const uint64_t gbase = (uint64_t)r * 2 * inter + 32 * g;
    float v[32];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        float a[8], b[8];
        qw_load8_f32<DT>(gu, gbase + 8 * j, a);
        qw_load8_f32<DT>(gu, gbase + inter + 8 * j, b);
#pragma unroll
        for (int e = 0; e < 8; ++e) v[8 * j + e] = qw_gated(a[e], b[e], ga);
    }
    if (ROT) qw_fwht32(v);
    h1_t* o = act + (uint64_t)r * inter + 32 * g;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        h8_t t;
#pragma unroll
        for (int e = 0; e < 8; ++e) t[e] = (h1_t)v[8 * j + e];
        *(h8_t*)(o + 8 * j) = t;
    }
}

// Ragged tail (inter % 32 != 0): one thread per element, never rotated.
template <int DT>
__global__ __launch_bounds__(256) void qw_swiglu_scalar_kernel(const void* __restrict__ gu, h1_t* __restrict__ act,
                                                                uint32_t rows, uint32_t inter, const qw_act ga) {
    const uint64_t i = (uint64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= (uint64_t)rows * inter) return;
    const uint32_t r = (uint32_t)(i / inter), c = (uint32_t)(i % inter);
    const float g = qw_load_f32<DT>(gu, (uint64_t)r * 2 * inter + c);
    const float u = qw_load_f32<DT>(gu, (uint64_t)r * 2 * inter + inter + c);
    act[i] = (h1_t)qw_gated(g, u, ga);
}

extern "C" qwhip_status qwhip_swiglu_fwht(qwhip_stream_t s, const void* gu, uint32_t gu_dtype, void* act_f16,
                                          uint32_t rows, uint32_t inter, uint32_t rotate) {
    QWHIP_REQUIRE(s);
    if (rows == 0 || inter == 0) return QWHIP_OK;
    QWHIP_REQUIRE(gu);
    QWHIP_REQUIRE(act_f16);
    if (gu_dtype != QWHIP_F16 && gu_dtype != QWHIP_F32)
        return qwhip_fail(QWHIP_E_BAD_SHAPE, "swiglu: gate|up must be f16 or f32, got dtype %u", gu_dtype);
    h1_t* act = (h1_t*)act_f16;
    if (inter % 32 != 0 || ((uintptr_t)gu & 15u) || ((uintptr_t)act_f16 & 15u)) {
        const uint64_t n = (uint64_t)rows * inter;
        const dim3 grid((unsigned)((n + 255) / 256)), block(256);
        if (inter % 32 == 0 && rotate)
            return qwhip_fail(QWHIP_E_BAD_SHAPE, "swiglu: rotated output needs 16-byte aligned buffers");
        if (gu_dtype == QWHIP_F16) hipLaunchKernelGGL(qw_swiglu_scalar_kernel<QWHIP_F16>, grid, block, 0, s->stream, gu, act, rows, inter, s->dev->act);
        else hipLaunchKernelGGL(qw_swiglu_scalar_kernel<QWHIP_F32>, grid, block, 0, s->stream, gu, act, rows, inter, s->dev->act);
    } else {
        const uint64_t groups = (uint64_t)rows * (inter / 32);
        const dim3 grid((unsigned)((groups + 255) / 256)), block(256);
        if (gu_dtype == QWHIP_F16) {
            if (rotate) hipLaunchKernelGGL((qw_swiglu_fwht_kernel<QWHIP_F16, true>), grid, block, 0, s->stream, gu, act, rows, inter, s->dev->act);
            else hipLaunchKernelGGL((qw_swiglu_fwht_kernel<QWHIP_F16, false>), grid, block, 0, s->stream, gu, act, rows, inter, s->dev->act);
        } else {
            if (rotate) hipLaunchKernelGGL((qw_swiglu_fwht_kernel<QWHIP_F32, true>), grid, block, 0, s->stream, gu, act, rows, inter, s->dev->act);
            else hipLaunchKernelGGL((qw_swiglu_fwht_kernel<QWHIP_F32, false>), grid, block, 0, s->stream, gu, act, rows, inter, s->dev->act);
        }
    }
    QWHIP_TRY_HIP(hipGetLastError());
    return QWHIP_OK;
}

// ---- dequant side output: f16 weights [n, k] in the container's own basis ---------------------------
// HQ4_G32_M5: one thread per u32 word (8 weights).
__global__ __launch_bounds__(256) void qw_dequant_hq4_kernel(const uint8_t* __restrict__ bank, h1_t* __restrict__ out,
                                                              uint64_t words) {
    const uint64_t wi = (uint64_t)blockIdx.x * 256 + threadIdx.x;
    if (wi >= words) return;
    const uint64_t blk = wi >> 2;
    const uint32_t j = (uint32_t)(wi & 3);
    const qw_hq4_block* b = (const qw_hq4_block*)(bank + blk * 20);
    const uint32_t hdr = b->hdr;
    h2_t w[4];
    qw_unpack_hq4_word(b->qs[j], qw_splat_lo(hdr), qw_splat_hi(hdr), qw_vgpr_const(0x64006400u), w);
    h8_t o = {w[0][0], w[0][1], w[1][0], w[1][1], w[2][0], w[2][1], w[3][0], w[3][1]};
    *(h8_t*)(out + blk * 32 + 8 * j) = o;
}

// Bit-stream blocks, any (bits, group): one thread per 8 codes (= `bits` payload bytes).
__global__ __launch_bounds__(256) void qw_dequant_blk_kernel(const uint8_t* __restrict__ bank, h1_t* __restrict__ out,
                                                              uint64_t octets, uint32_t bits, uint32_t group) {
    const uint64_t oi = (uint64_t)blockIdx.x * 256 + threadIdx.x;
    if (oi >= octets) return;
    const uint32_t opg = group / 8;  // octets per group
    const uint64_t blk = oi / opg;
    const uint32_t o = (uint32_t)(oi % opg);
    const uint32_t bb = 4 + group * bits / 8;
    const uint8_t* p = bank + blk * bb;
    const h1_t sc = __builtin_bit_cast(h1_t, (uint16_t)(p[0] | (p[1] << 8)));
    const h1_t bi = __builtin_bit_cast(h1_t, (uint16_t)(p[2] | (p[3] << 8)));
    uint64_t stream = 0;
    for (uint32_t b = 0; b < bits; ++b) stream |= (uint64_t)p[4 + o * bits + b] << (8 * b);
    h8_t v;
    const uint32_t mask = (1u << bits) - 1u;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        const h1_t code = (h1_t)(float)((uint32_t)(stream >> (e * bits)) & mask);
        v[e] = __builtin_fmaf16(code, sc, bi);  // RN_f16(code*scale + bias), single rounding
    }
    *(h8_t*)(out + blk * group + 8 * o) = v;
}

extern "C" qwhip_status qwhip_dequant_f16(qwhip_stream_t s, const qwhip_weight_view* w, void* out_f16) {
    QWHIP_REQUIRE(s);
    qwhip_status st = qwhip_weight_view_validate(w);
    if (st != QWHIP_OK) return st;
    QWHIP_REQUIRE(out_f16);
    if ((uintptr_t)out_f16 & 15u) return qwhip_fail(QWHIP_E_BAD_SHAPE, "dequant: output must be 16-byte aligned");
    const uint64_t total = (uint64_t)w->n * w->k;
    const uint64_t threads = total / 8;
    const dim3 grid((unsigned)((threads + 255) / 256)), block(256);
    if (w->kind == QWHIP_KIND_HQ4_G32_M5)
        hipLaunchKernelGGL(qw_dequant_hq4_kernel, grid, block, 0, s->stream, (const uint8_t*)w->blocks, (h1_t*)out_f16, threads);
    else
        hipLaunchKernelGGL(qw_dequant_blk_kernel, grid, block, 0, s->stream, (const uint8_t*)w->blocks, (h1_t*)out_f16, threads,
                           w->bits, w->group);
    QWHIP_TRY_HIP(hipGetLastError());
    return QWHIP_OK;
}

// ---- fp32 seams of the MoE operator chain ----------------------------------------------------------
// One thread per 32-group, the group in registers, the fp32 butterfly of qw_fwht32 (strides 1, 2, 4, 8, 16, then one
// multiply by 1/sqrt(32): the order of fwht32_f32_inplace, Sources/QWMetal/include/qw_dequant.metalh:442-478).

// silu(gate) * up in fp32, then the 32-point transform, fp32 out (qwg_silu_mul_f32, Sources/QWMetal/gemm/qwgemm_f32.metal:291-317;
// door QWGemm.encodeSiluMulF32, Sources/Operators/QWGEMM/QWGemmF32.swift:83-94).  gu fp32 [rows, 2 inter], inter % 32 == 0.
__global__ __launch_bounds__(256) void qw_silu_mul_f32_kernel(const float* __restrict__ gu, float* __restrict__ act, uint32_t rows,
                                                               uint32_t inter, const qw_act ga) {
    const uint64_t gi = (uint64_t)blockIdx.x * 256 + threadIdx.x;
    const uint32_t gpr = inter / 32u;
    if (gi >= (uint64_t)rows * gpr) return;
    const uint32_t r = (uint32_t)(gi / gpr), g = (uint32_t)(gi % gpr);
    const f4_t* gp = (const f4_t*)(gu + (uint64_t)r * 2u * inter + 32u * g);
    const f4_t* up = (const f4_t*)(gu + (uint64_t)r * 2u * inter + inter + 32u * g);
    float v[32];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        const f4_t a = gp[j], b = up[j];
#pragma unroll
        for (int e = 0; e < 4; ++e) v[4 * j + e] = qw_gated(a[e], b[e], ga);
    }
    qw_fwht32(v);
    f4_t* o = (f4_t*)(act + (uint64_t)r * inter + 32u * g);
#pragma unroll
    for (int j = 0; j < 8; ++j) o[j] = f4_t{v[4 * j], v[4 * j + 1], v[4 * j + 2], v[4 * j + 3]};
}

extern "C" qwhip_status qwhip_silu_mul_f32(qwhip_stream_t s, const float* gu, float* act, uint32_t rows, uint32_t inter) {
    QWHIP_REQUIRE(s);
    if (rows == 0) return QWHIP_OK;
    QWHIP_REQUIRE(gu);
    QWHIP_REQUIRE(act);
    if (inter == 0 || inter % 32u != 0) return qwhip_fail(QWHIP_E_BAD_SHAPE, "f32 silu-mul needs intermediate %% 32 == 0, got %u", inter);
    if (((uintptr_t)gu | (uintptr_t)act) & 15u) return qwhip_fail(QWHIP_E_BAD_SHAPE, "f32 silu-mul needs 16-byte aligned buffers");
    const uint64_t groups = (uint64_t)rows * (inter / 32u);
    hipLaunchKernelGGL(qw_silu_mul_f32_kernel, dim3((unsigned)((groups + 255) / 256)), dim3(256), 0, s->stream, gu, act, rows, inter, s->dev->act);
    QWHIP_TRY_HIP(hipGetLastError());
    return QWHIP_OK;
}

// The f32 bridge in front of the MoE chain (qwg_moe_bridge_f16_to_f32, Sources/QWMetal/gemm/qwmoe_bridge_f32.metal:16-78; door
// QWGemm.encodeMoEBridgeF16ToF32, Sources/Operators/QWGEMM/QWGemmMoE.swift:337-377): the f16 normed hidden in the rotated
// basis becomes the rotated fp32 copy (a plain widening; skipped when x_rot32 is null) and the un-rotated fp32 copy the
// router reads - the transform again (it is its own inverse) in fp32, taken through the f16 hi/lo split of the reference's
// helper: plain = f32(hi) + f32(lo), hi = f16(v), lo = f16(v - f32(hi)).
__global__ __launch_bounds__(256) void qw_moe_bridge_kernel(const h1_t* __restrict__ x, float* __restrict__ rot32, float* __restrict__ plain32,
                                                             uint64_t groups) {
    const uint64_t gi = (uint64_t)blockIdx.x * 256 + threadIdx.x;
    if (gi >= groups) return;
    const h8_t* xp = (const h8_t*)(x + 32u * gi);
    float v[32];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const h8_t a = xp[j];
#pragma unroll
        for (int e = 0; e < 8; ++e) v[8 * j + e] = (float)a[e];
    }
    if (rot32) {
        f4_t* o = (f4_t*)(rot32 + 32u * gi);
#pragma unroll
        for (int j = 0; j < 8; ++j) o[j] = f4_t{v[4 * j], v[4 * j + 1], v[4 * j + 2], v[4 * j + 3]};
    }
    qw_fwht32(v);
#pragma unroll
    for (int i = 0; i < 32; ++i) {
        const h1_t hi = (h1_t)v[i];
        const h1_t lo = (h1_t)(v[i] - (float)hi);
        v[i] = (float)hi + (float)lo;
    }
    f4_t* o = (f4_t*)(plain32 + 32u * gi);
#pragma unroll
    for (int j = 0; j < 8; ++j) o[j] = f4_t{v[4 * j], v[4 * j + 1], v[4 * j + 2], v[4 * j + 3]};
}

extern "C" qwhip_status qwhip_moe_bridge_f16_to_f32(qwhip_stream_t s, const void* x_f16, float* x_rot32, float* x_plain32, uint32_t rows,
                                                    uint32_t hidden) {
    QWHIP_REQUIRE(s);
    if (rows == 0 || hidden == 0) return qwhip_fail(QWHIP_E_BAD_GEOMETRY, "moe bridge: rows=%u hidden=%u", rows, hidden);
    if (hidden % 256u != 0) return qwhip_fail(QWHIP_E_BAD_GEOMETRY, "moe bridge: hidden %u must be a multiple of 256", hidden);
    QWHIP_REQUIRE(x_f16);
    QWHIP_REQUIRE(x_plain32);
    if (((uintptr_t)x_f16 | (uintptr_t)x_rot32 | (uintptr_t)x_plain32) & 15u)
        return qwhip_fail(QWHIP_E_BAD_SHAPE, "moe bridge needs 16-byte aligned buffers");
    const uint64_t groups = (uint64_t)rows * (hidden / 32u);
    hipLaunchKernelGGL(qw_moe_bridge_kernel, dim3((unsigned)((groups + 255) / 256)), dim3(256), 0, s->stream, (const h1_t*)x_f16, x_rot32,
                       x_plain32, groups);
    QWHIP_TRY_HIP(hipGetLastError());
    return QWHIP_OK;
}

// Optional RMSNorm (1 + gamma) and the 32-point transform on fp32 [rows, latent], fp32 and / or f16 out
// (qwg_latent_norm_h32_f32, Sources/QWMetal/gemm/qwgemm_f32.metal:203-288; door QWGemm.encodeLatentNormH32F32,
// Sources/Operators/QWGEMM/QWGemmF32.swift:57-80): v = x * rsqrt(mean(x^2) + eps) * (1 + gamma) (gamma f16; no gamma: v = x),
// then the transform; one workgroup per row.
__global__ __launch_bounds__(256) void qw_latent_norm_kernel(const float* __restrict__ x, const h1_t* __restrict__ gamma,
                                                              float* __restrict__ out32, h1_t* __restrict__ out16, uint32_t latent, float eps) {
    __shared__ float wsum[4];
    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    const float* xr = x + (uint64_t)blockIdx.x * latent;
    float rstd = 1.0f;
    if (gamma) {
        float ss = 0.0f;
        for (uint32_t c = tid * 4u; c < latent; c += 1024u) {
            const f4_t a = *(const f4_t*)(xr + c);
            ss = fmaf(a[0], a[0], ss);
            ss = fmaf(a[1], a[1], ss);
            ss = fmaf(a[2], a[2], ss);
            ss = fmaf(a[3], a[3], ss);
        }
        ss = qw_reduce64(ss);
        if (lane == 0) wsum[wave] = ss;
        __syncthreads();
        rstd = rsqrtf(((wsum[0] + wsum[1]) + (wsum[2] + wsum[3])) / (float)latent + eps);
    }
    for (uint32_t g = tid; g < latent / 32u; g += 256u) {
        float v[32];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const f4_t a = *(const f4_t*)(xr + 32u * g + 4 * j);
#pragma unroll
            for (int e = 0; e < 4; ++e) v[4 * j + e] = a[e];
        }
        if (gamma) {
#pragma unroll
            for (int i = 0; i < 32; ++i) v[i] = (v[i] * rstd) * (1.0f + (float)gamma[32u * g + i]);
        }
        qw_fwht32(v);
        const uint64_t at = (uint64_t)blockIdx.x * latent + 32u * g;
        if (out32) {
#pragma unroll
            for (int j = 0; j < 8; ++j) *(f4_t*)(out32 + at + 4 * j) = f4_t{v[4 * j], v[4 * j + 1], v[4 * j + 2], v[4 * j + 3]};
        }
        if (out16) {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                h8_t o;
#pragma unroll
                for (int e = 0; e < 8; ++e) o[e] = (h1_t)v[8 * j + e];
                *(h8_t*)(out16 + at + 8 * j) = o;
            }
        }
    }
}

extern "C" qwhip_status qwhip_latent_norm_h32_f32(qwhip_stream_t s, const float* x, const void* gamma_f16, float* out32, void* out16,
                                                  uint32_t rows, uint32_t latent, float eps) {
    QWHIP_REQUIRE(s);
    if (rows == 0) return QWHIP_OK;
    QWHIP_REQUIRE(x);
    if (!out32 && !out16) return qwhip_fail(QWHIP_E_NULL, "latent norm needs out32 and/or out16");
    if (latent == 0 || latent % 32u != 0) return qwhip_fail(QWHIP_E_BAD_SHAPE, "latent norm H32 needs latent %% 32 == 0, got %u", latent);
    if (((uintptr_t)x | (uintptr_t)out32 | (uintptr_t)out16) & 15u) return qwhip_fail(QWHIP_E_BAD_SHAPE, "latent norm needs 16-byte aligned buffers");
    hipLaunchKernelGGL(qw_latent_norm_kernel, dim3(rows), dim3(256), 0, s->stream, x, (const h1_t*)gamma_f16, out32, (h1_t*)out16, latent, eps);
    QWHIP_TRY_HIP(hipGetLastError());
    return QWHIP_OK;
}

// out = a + b over count fp32 values (qwg_add_f32, qwgemm_f32.metal:319-326; QWGemm.encodeAddF32, QWGemmF32.swift:108-115)
__global__ __launch_bounds__(256) void qw_add_f32_kernel(const float* __restrict__ a, const float* __restrict__ b, float* __restrict__ out,
                                                          uint64_t count) {
    const uint64_t i = (uint64_t)blockIdx.x * 256 + threadIdx.x;
    if (i < count) out[i] = a[i] + b[i];
}

extern "C" qwhip_status qwhip_add_f32(qwhip_stream_t s, const float* a, const float* b, float* out, uint64_t count) {
    QWHIP_REQUIRE(s);
    if (count == 0) return QWHIP_OK;
    QWHIP_REQUIRE(a);
    QWHIP_REQUIRE(b);
    QWHIP_REQUIRE(out);
    if (count > (1ull << 39)) return qwhip_fail(QWHIP_E_BAD_SHAPE, "add: %llu values are more than one launch takes", (unsigned long long)count);
    hipLaunchKernelGGL(qw_add_f32_kernel, dim3((unsigned)((count + 255) / 256)), dim3(256), 0, s->stream, a, b, out, count);
    QWHIP_TRY_HIP(hipGetLastError());
    return QWHIP_OK;
}

// ---- embedding gather over a block table: the token's row decoded to fp32, written hc times ---------
// (qwg_embed_aq_f32, Sources/QWMetal/gemm/qwgemm_aq_embed.metal:14-52; door QWGemmAQ.encodeEmbedAQ,
// Sources/Operators/QWGEMM/QWGemmAQ.swift:147-187).  value = code * scale + bias in fp32 (product rounded, then the sum:
// the law of the container's host twin), in the container's own basis; a negative token reads row 0 as the reference
// does, and a token past the table reads its last row instead of memory outside it.
// One thread per 8 codes of the row (`bits` payload bytes; HQ4_G32_M5: one code word), blockIdx.y = output row.
template <bool M5>
__global__ __launch_bounds__(256) void qw_embed_kernel(const uint8_t* __restrict__ bank, const int32_t* __restrict__ tokens,
                                                        float* __restrict__ out, uint32_t vocab, uint32_t hidden, uint32_t hc,
                                                        uint32_t bits, uint32_t group, uint32_t row_bytes) {
    const uint32_t oi = blockIdx.x * 256u + threadIdx.x;   // octet of the row
    if (oi * 8u >= hidden) return;
    const uint32_t r = blockIdx.y;
    const uint32_t tok = min((uint32_t)max(tokens[r], 0), vocab - 1u);
    const uint8_t* rowp = bank + (uint64_t)tok * row_bytes;
    float v[8];
    if constexpr (M5) {
        const qw_hq4_block* b = (const qw_hq4_block*)(rowp + (oi >> 2) * 20u);
        const h2_t hd = __builtin_bit_cast(h2_t, b->hdr);
        const float sc = (float)hd[0], bi = (float)hd[1];
        const uint32_t q = b->qs[oi & 3u];
#pragma unroll
        for (int e = 0; e < 8; ++e) {   // element e of the word sits at bit 4 (e >> 1) + 16 (e & 1)
            const float code = (float)(((q >> (4 * (e >> 1) + 16 * (e & 1))) & 0xFu) + 1024u);
            v[e] = __fadd_rn(__fmul_rn(code, sc), bi);
        }
    } else {
        const uint32_t opg = group / 8u;
        const uint8_t* p = rowp + (uint64_t)(oi / opg) * (4u + group * bits / 8u);
        const uint32_t o = oi % opg;
        const float sc = (float)__builtin_bit_cast(h1_t, (uint16_t)(p[0] | (p[1] << 8)));
        const float bi = (float)__builtin_bit_cast(h1_t, (uint16_t)(p[2] | (p[3] << 8)));
        uint64_t stream = 0;
        for (uint32_t b = 0; b < bits; ++b) stream |= (uint64_t)p[4 + o * bits + b] << (8 * b);
        const uint32_t mask = (1u << bits) - 1u;
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] = __fadd_rn(__fmul_rn((float)((uint32_t)(stream >> (e * bits)) & mask), sc), bi);
    }
    const f4_t lo = {v[0], v[1], v[2], v[3]}, hi = {v[4], v[5], v[6], v[7]};
    for (uint32_t c = 0; c < hc; ++c) {
        float* dst = out + ((uint64_t)r * hc + c) * hidden + oi * 8u;
        *(f4_t*)dst = lo;
        *(f4_t*)(dst + 4) = hi;
    }
}

extern "C" qwhip_status qwhip_embed_aq_f32(qwhip_stream_t s, const qwhip_weight_view* table, const int32_t* tokens, uint32_t rows,
                                           uint32_t hc, float* out) {
    QWHIP_REQUIRE(s);
    qwhip_status st = qwhip_weight_view_validate(table);
    if (st != QWHIP_OK) return st;
    if (rows == 0) return QWHIP_OK;
    QWHIP_REQUIRE(tokens);
    QWHIP_REQUIRE(out);
    if (hc == 0) return qwhip_fail(QWHIP_E_BAD_WEIGHTS, "the embedding gather needs a positive shape");
    if (rows > 65535u) return qwhip_fail(QWHIP_E_BAD_SHAPE, "the embedding gather takes at most 65535 rows a launch, got %u", rows);
    if ((uintptr_t)out & 15u) return qwhip_fail(QWHIP_E_BAD_SHAPE, "embedding output must be 16-byte aligned");
    const uint32_t hidden = table->k;
    const uint32_t bb = qwhip_block_bytes(table->kind, table->bits, table->group);
    const uint64_t row_bytes = (uint64_t)(hidden / table->group) * bb;
    if (row_bytes >= (1ull << 32)) return qwhip_fail(QWHIP_E_BAD_SHAPE, "embedding rows of %llu bytes are not addressable", (unsigned long long)row_bytes);
    const dim3 grid(qwhip_cdiv(hidden / 8u, 256u), rows), block(256);
    if (table->kind == QWHIP_KIND_HQ4_G32_M5)
        hipLaunchKernelGGL(qw_embed_kernel<true>, grid, block, 0, s->stream, (const uint8_t*)table->blocks, tokens, out, table->n, hidden, hc,
                           table->bits, table->group, (uint32_t)row_bytes);
    else
        hipLaunchKernelGGL(qw_embed_kernel<false>, grid, block, 0, s->stream, (const uint8_t*)table->blocks, tokens, out, table->n, hidden, hc,
                           table->bits, table->group, (uint32_t)row_bytes);
    QWHIP_TRY_HIP(hipGetLastError());
    return QWHIP_OK;
}

// The same gather from a raw bf16 table (qwg_embed_bf16_f32, Sources/QWMetal/gemm/qwgemm_f32.metal:102-116; door
// QWGemm.encodeEmbedBf16F32, Sources/Operators/QWGEMM/QWGemmF32.swift:352-363): a widening, exact.
__global__ __launch_bounds__(256) void qw_embed_bf16_kernel(const uint16_t* __restrict__ table, const int32_t* __restrict__ tokens,
                                                             float* __restrict__ out, uint32_t vocab, uint32_t hidden, uint32_t hc) {
    const uint32_t r = blockIdx.y;
    const uint32_t tok = min((uint32_t)max(tokens[r], 0), vocab - 1u);
    const uint16_t* row = table + (uint64_t)tok * hidden;
    for (uint32_t d = blockIdx.x * 256u + threadIdx.x; d < hidden; d += gridDim.x * 256u) {
        const float v = __uint_as_float((uint32_t)row[d] << 16);
        for (uint32_t c = 0; c < hc; ++c) out[((uint64_t)r * hc + c) * hidden + d] = v;
    }
}

extern "C" qwhip_status qwhip_embed_bf16_f32(qwhip_stream_t s, const void* table_bf16, uint32_t vocab, uint32_t hidden, const int32_t* tokens,
                                             uint32_t rows, uint32_t hc, float* out) {
    QWHIP_REQUIRE(s);
    if (rows == 0) return QWHIP_OK;
    QWHIP_REQUIRE(table_bf16);
    QWHIP_REQUIRE(tokens);
    QWHIP_REQUIRE(out);
    if (vocab == 0 || hidden == 0 || hc == 0) return qwhip_fail(QWHIP_E_BAD_SHAPE, "the embedding gather needs a positive shape");
    if (rows > 65535u) return qwhip_fail(QWHIP_E_BAD_SHAPE, "the embedding gather takes at most 65535 rows a launch, got %u", rows);
    const dim3 grid(min(qwhip_cdiv(hidden, 256u), 4096u), rows), block(256);
    hipLaunchKernelGGL(qw_embed_bf16_kernel, grid, block, 0, s->stream, (const uint16_t*)table_bf16, tokens, out, vocab, hidden, hc);
    QWHIP_TRY_HIP(hipGetLastError());
    return QWHIP_OK;
}

// ------------------------------------------------------------------------------------------------
// RMSNorm with the rotation fused (the producer in front of every projection of a decode layer):
//   y = f16( FWHT32( x * rsqrt(mean(x^2) + eps) * (1 + gamma) ) ),  optionally after  residual <- f16(residual + x)
// (qwg_rmsnorm / qwg_rmsnorm_residual, Sources/QWMetal/mlp_norm_rope/qwnorm.metal:27-79, 127-189; doors
// encodeRMSNormFast / encodeRMSNormResidualFast, Sources/Runtime/QWEngine/Driver/EncodeKernels.swift:339-404).
// Plus-one law: gamma is stored raw and applied as (1 + gamma) in fp32; sum of squares in fp32; the 32-point
// transform in fp32 in the butterfly order of fwht32_f32_inplace (qw_dequant.metalh:442-478: strides 1, 2, 4 inside a
// lane's 8 values, 8 and 16 across 4 lanes, times 1/sqrt(32)); one f16 rounding at the store.
// One workgroup per row; a thread owns 8 consecutive values per 2048-column sweep (16-byte loads, the row stays in
// registers up to 16384 columns); four neighbouring lanes hold one 32-group.
// ------------------------------------------------------------------------------------------------
template <bool RESIDUAL>
__global__ __launch_bounds__(256) void qw_rmsnorm_kernel(const h1_t* __restrict__ x, const h1_t* __restrict__ gamma,
                                                         h1_t* __restrict__ residual, h1_t* __restrict__ y, uint32_t hidden,
                                                         float eps, uint32_t rotate) {
    constexpr int SW = 8;   // sweeps held in registers
    __shared__ float wsum[4];
    const uint32_t tid = threadIdx.x;
    const uint64_t row = (uint64_t)blockIdx.x * hidden;
    h8_t v[SW];
    float acc = 0.f;
#pragma unroll
    for (int k = 0; k < SW; ++k) {
        const uint32_t c = (k * 256u + tid) * 8u;
        if (c < hidden) {
            h8_t xv = *(const h8_t*)(x + row + c);
            if constexpr (RESIDUAL) {
                const h8_t rv = *(const h8_t*)(residual + row + c);
#pragma unroll
                for (int i = 0; i < 8; ++i) xv[i] = (h1_t)((float)xv[i] + (float)rv[i]);
                *(h8_t*)(residual + row + c) = xv;
            }
            v[k] = xv;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const float t = (float)xv[i];
                acc = fmaf(t, t, acc);
            }
        }
    }
    acc = qw_reduce64(acc);
    if ((tid & 63u) == 0u) wsum[tid >> 6] = acc;
    __syncthreads();
    const float total = (wsum[0] + wsum[1]) + (wsum[2] + wsum[3]);
    const float rstd = 1.0f / sqrtf(total / (float)hidden + eps);
#pragma unroll
    for (int k = 0; k < SW; ++k) {
        const uint32_t c = (k * 256u + tid) * 8u;
        if (c >= hidden) continue;   // whole quads of lanes leave together: hidden is a multiple of 32
        const h8_t gv = *(const h8_t*)(gamma + c);
        float f[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) f[i] = (float)v[k][i] * rstd * ((float)gv[i] + 1.0f);
        if (rotate) {
#pragma unroll
            for (int i = 0; i < 8; i += 2) {
                const float a = f[i], b = f[i + 1];
                f[i] = a + b;
                f[i + 1] = a - b;
            }
#pragma unroll
            for (int i = 0; i < 8; i += 4) {
                const float a0 = f[i], a1 = f[i + 1], b0 = f[i + 2], b1 = f[i + 3];
                f[i] = a0 + b0;
                f[i + 1] = a1 + b1;
                f[i + 2] = a0 - b0;
                f[i + 3] = a1 - b1;
            }
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float a = f[i], b = f[i + 4];
                f[i] = a + b;
                f[i + 4] = a - b;
            }
            const bool neg1 = (tid & 1u) != 0u, neg2 = (tid & 2u) != 0u;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const float p = __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, f[i]), 0xB1, 0xF, 0xF, true));
                f[i] = neg1 ? (p - f[i]) : (f[i] + p);
            }
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const float p = __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, f[i]), 0x4E, 0xF, 0xF, true));
                f[i] = (neg2 ? (p - f[i]) : (f[i] + p)) * QW_INV_SQRT32;
            }
        }
        h8_t o;
#pragma unroll
        for (int i = 0; i < 8; ++i) o[i] = (h1_t)f[i];
        *(h8_t*)(y + row + c) = o;
    }
}

extern "C" qwhip_status qwhip_rmsnorm(qwhip_stream_t s, const void* x_f16, const void* gamma_f16, void* residual_f16, uint32_t rows,
                                      uint32_t hidden, float eps, uint32_t rotate, void* y_f16) {
    QWHIP_REQUIRE(s);
    if (rows == 0) return QWHIP_OK;
    QWHIP_REQUIRE(x_f16);
    QWHIP_REQUIRE(gamma_f16);
    QWHIP_REQUIRE(y_f16);
    if (hidden == 0 || hidden % 256u != 0u)
        return qwhip_fail(QWHIP_E_BAD_GEOMETRY, "the norm family needs a hidden that is a multiple of 256, got %u", hidden);
    if (hidden > 16384u) return qwhip_fail(QWHIP_E_BAD_GEOMETRY, "the norm kernel holds rows of at most 16384 columns, got %u", hidden);
    if (((uintptr_t)x_f16 | (uintptr_t)gamma_f16 | (uintptr_t)y_f16 | (uintptr_t)residual_f16) & 15u)
        return qwhip_fail(QWHIP_E_BAD_SHAPE, "the norm kernel needs 16-byte aligned rows");
    if (residual_f16)
        hipLaunchKernelGGL(qw_rmsnorm_kernel<true>, dim3(rows), dim3(256), 0, s->stream, (const h1_t*)x_f16, (const h1_t*)gamma_f16,
                           (h1_t*)residual_f16, (h1_t*)y_f16, hidden, eps, rotate ? 1u : 0u);
    else
        hipLaunchKernelGGL(qw_rmsnorm_kernel<false>, dim3(rows), dim3(256), 0, s->stream, (const h1_t*)x_f16, (const h1_t*)gamma_f16,
                           (h1_t*)nullptr, (h1_t*)y_f16, hidden, eps, rotate ? 1u : 0u);
    QWHIP_TRY_HIP(hipGetLastError());
    return QWHIP_OK;
}

// ------------------------------------------------------------------------------------------------
// Greedy-decoding argmax over logits rows, with the reference's key rule (qw_sortable_f32_u32,
// Sources/QWMetal/include/qw_fastmath_safe.metalh:21-25; fold in qwg_gemv_am_fold4 / qwg_gemv_am_reduce4,
// Sources/QWMetal/include/qw_gemm_f32_common.metalh:30-58): key hi = the float's bits made monotone (NaN -> 0, so it
// never wins against a number), key lo = ~row, larger (hi, lo) wins: ties go to the lower row.
// One workgroup per logits row; 16-byte loads, eight in flight per thread; wave fold by lane exchanges, then LDS across waves.
// ------------------------------------------------------------------------------------------------
__device__ __forceinline__ uint32_t qw_sortable_f32(float x) {
    const uint32_t u = __float_as_uint(x);
    if ((u & 0x7FFFFFFFu) > 0x7F800000u) return 0u;
    return (u & 0x80000000u) ? ~u : (u ^ 0x80000000u);
}

// One workgroup's vector ALU and its loads in flight bound the fold, so the sweep keeps a float maximum and its first row
// per thread (a strict "greater" per element; NaN is never greater) and builds the 64-bit keys only to combine the 1024
// thread results.  That is exact unless the row's maximum is a zero (+0.0 beats -0.0 in the key order, they are equal as
// floats) or no element is greater than -inf (only -inf and NaN): those rows take the key sweep over every element.
// VAR: the relaxed acceptance of a draft (qwg_head_argmax_fin_variational, Sources/QWMetal/head_sampling/qwhead.metal:271-345):
// row r takes draft[r + 1] instead of its argmax when that token's logit is within `margin` of the maximum and, for a finite
// min_log_prob, log softmax(draft) >= min_log_prob (the sum of exponentials runs only for such a candidate).
template <bool VAR>
__global__ __launch_bounds__(1024) void qw_argmax_rows_kernel(const float* __restrict__ logits, uint32_t n, int32_t* __restrict__ tokens,
                                                               const uint32_t* __restrict__ draft, uint32_t total_rows, float margin,
                                                               float min_log_prob) {
    __shared__ unsigned long long best_w[16];
    __shared__ uint32_t slow_path;
    constexpr uint32_t U = 8;   // 16-byte loads in flight per thread
    const uint32_t tid = threadIdx.x;
    const float* row = logits + (uint64_t)blockIdx.x * n;
    const uint32_t n4 = (((uintptr_t)row & 15u) == 0u) ? (n & ~3u) : 0u;
    float mx = -__builtin_inff();
    uint32_t at = 0xFFFFFFFFu;   // no element yet
    for (uint32_t i0 = tid * 4u; i0 < n4; i0 += U * 4096u) {
        f4_t v[U];
#pragma unroll
        for (uint32_t u = 0; u < U; ++u) {
            const uint32_t i = i0 + u * 4096u;
            v[u] = *(const f4_t*)(row + (i < n4 ? i : i0));   // past the end: the batch's first chunk again (never greater)
        }
#pragma unroll
        for (uint32_t u = 0; u < U; ++u) {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const bool gt = v[u][j] > mx;
                mx = gt ? v[u][j] : mx;
                at = gt ? i0 + u * 4096u + j : at;
            }
        }
    }
    for (uint32_t i = n4 + tid; i < n; i += 1024u) {
        const float x = row[i];
        const bool gt = x > mx;
        mx = gt ? x : mx;
        at = gt ? i : at;
    }
    // a thread without an element (or whose elements are all -inf / NaN) offers the key of a NaN at row 0: it loses to any number
    unsigned long long best = at == 0xFFFFFFFFu ? 0xFFFFFFFFull : (((unsigned long long)qw_sortable_f32(mx) << 32) | (uint32_t)~at);
    auto fold = [&]() {
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) {
            const unsigned long long o = __shfl_xor(best, off, 64);
            best = o > best ? o : best;
        }
        if ((tid & 63u) == 0u) best_w[tid >> 6] = best;
        __syncthreads();
        best = best_w[0];
#pragma unroll
        for (int w = 1; w < 16; ++w) best = best_w[w] > best ? best_w[w] : best;
    };
    fold();
    const uint32_t hi = (uint32_t)(best >> 32);
    // maximum +0.0 / -0.0 (keys 0x80000000 / 0x7FFFFFFF), or nothing above -inf (hi 0): decide over every element's key
    if (tid == 0u) slow_path = (hi == 0x80000000u || hi == 0x7FFFFFFFu || hi == 0u) ? 1u : 0u;
    __syncthreads();
    if (slow_path) {
        best = 0ull;
        for (uint32_t i = tid; i < n; i += 1024u) {
            const unsigned long long key = ((unsigned long long)qw_sortable_f32(row[i]) << 32) | (uint32_t)~i;
            best = key > best ? key : best;
        }
        __syncthreads();   // best_w is reused
        fold();
    }
    if constexpr (!VAR) {
        if (tid == 0u) tokens[blockIdx.x] = (int32_t)~(uint32_t)best;
    } else {
        __shared__ uint32_t gate, cand;
        __shared__ float part_w[16];
        const uint32_t out_tok = ~(uint32_t)best, kh = (uint32_t)(best >> 32);
        const float mx_logit = __uint_as_float((kh & 0x80000000u) ? (kh ^ 0x80000000u) : ~kh);
        float draft_logit = 0.0f;
        if (tid == 0u) {
            uint32_t tok = out_tok, g = 0u;
            if (margin > 0.0f && blockIdx.x + 1u < total_rows) {
                const uint32_t d = draft[blockIdx.x + 1u];
                if (d < n && d != out_tok) {
                    draft_logit = row[d];
                    if (draft_logit >= mx_logit - margin) {
                        if (__builtin_isfinite(min_log_prob)) {
                            g = 1u;
                            cand = d;
                        } else {
                            tok = d;
                        }
                    }
                }
            }
            gate = g;
            if (g == 0u) tokens[blockIdx.x] = (int32_t)tok;
        }
        __syncthreads();
        if (gate == 0u) return;   // uniform over the workgroup
        float part = 0.0f;
        for (uint32_t i = tid; i < n; i += 1024u) part += expf(row[i] - mx_logit);
        part = qw_reduce64(part);
        if ((tid & 63u) == 0u) part_w[tid >> 6] = part;
        __syncthreads();
        if (tid == 0u) {
            float total = 0.0f;
#pragma unroll
            for (int w = 0; w < 16; ++w) total += part_w[w];
            const float log_prob = (draft_logit - mx_logit) - logf(total);
            tokens[blockIdx.x] = (int32_t)(log_prob >= min_log_prob ? cand : out_tok);
        }
    }
}

// Few long rows (the head of a decode or verify step): a row is split over `parts` workgroups so that the fold is not the work
// of one compute unit.  Every workgroup folds the keys of its slice and leaves one key in the stream's scratch; a second
// launch of one wavefront per row folds the row's keys into its token.  Same key rule, so the same token as the one-workgroup
// kernel.  (One launch whose last-arriving workgroup folds the keys was measured slower: 6.3 us for one row and 28 us for 16
// rows of 151,936 logits - the release fence in front of the arrival writes the L2 back once per workgroup.)
constexpr uint32_t QW_ARGMAX_SPLIT_ROWS = 16, QW_ARGMAX_SPLIT_PARTS = 64;
__global__ __launch_bounds__(256) void qw_argmax_split_kernel(const float* __restrict__ logits, uint32_t n, uint32_t per,
                                                               unsigned long long* __restrict__ keys) {
    __shared__ unsigned long long best_w[4];
    const uint32_t tid = threadIdx.x, part = blockIdx.x, parts = gridDim.x, r = blockIdx.y;
    const float* row = logits + (uint64_t)r * n;
    const uint32_t lo = min(part * per, n), hi = min(lo + per, n);
    unsigned long long best = 0ull;   // below every element's key (the low word of a key is never 0: rows < 2^30)
    for (uint32_t i = lo + tid; i < hi; i += 256u) {
        const unsigned long long key = ((unsigned long long)qw_sortable_f32(row[i]) << 32) | (uint32_t)~i;
        best = key > best ? key : best;
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        const unsigned long long o = __shfl_xor(best, off, 64);
        best = o > best ? o : best;
    }
    if ((tid & 63u) == 0u) best_w[tid >> 6] = best;
    __syncthreads();
    if (tid == 0u) {
#pragma unroll
        for (int w = 1; w < 4; ++w) best = best_w[w] > best ? best_w[w] : best;
        keys[r * parts + part] = best;
    }
}
__global__ __launch_bounds__(64) void qw_argmax_split_fin_kernel(const unsigned long long* __restrict__ keys, uint32_t parts,
                                                                  int32_t* __restrict__ tokens) {
    unsigned long long best = 0ull;
    for (uint32_t i = threadIdx.x; i < parts; i += 64u) {
        const unsigned long long k = keys[blockIdx.x * parts + i];
        best = k > best ? k : best;
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        const unsigned long long o = __shfl_xor(best, off, 64);
        best = o > best ? o : best;
    }
    if (threadIdx.x == 0u) tokens[blockIdx.x] = (int32_t)~(uint32_t)best;
}

extern "C" qwhip_status qwhip_argmax_f32(qwhip_stream_t s, const float* logits, uint32_t rows, uint32_t n, int32_t* tokens) {
    QWHIP_REQUIRE(s);
    if (rows == 0) return QWHIP_OK;
    QWHIP_REQUIRE(logits);
    QWHIP_REQUIRE(tokens);
    if (n == 0 || n >= (1u << 30)) return qwhip_fail(QWHIP_E_BAD_SHAPE, "argmax over %u logits does not fit the row-count flags", n);
    if (rows <= QW_ARGMAX_SPLIT_ROWS && n >= 32768u && s->scratch && s->scratch_bytes >= QWHIP_STREAM_COUNTER_BYTES) {
        const uint32_t parts = QW_ARGMAX_SPLIT_PARTS, per = (n + parts - 1u) / parts;
        static_assert(QW_ARGMAX_SPLIT_ROWS * QW_ARGMAX_SPLIT_PARTS * 8u <= QWHIP_STREAM_COUNTER_BYTES, "the keys fit the stream's key area");
        unsigned long long* keys = (unsigned long long*)s->scratch;
        hipLaunchKernelGGL(qw_argmax_split_kernel, dim3(parts, rows), dim3(256), 0, s->stream, logits, n, per, keys);
        hipLaunchKernelGGL(qw_argmax_split_fin_kernel, dim3(rows), dim3(64), 0, s->stream, keys, parts, tokens);
        QWHIP_TRY_HIP(hipGetLastError());
        return QWHIP_OK;
    }
    hipLaunchKernelGGL(qw_argmax_rows_kernel<false>, dim3(rows), dim3(1024), 0, s->stream, logits, n, tokens, nullptr, 0u, 0.0f, 0.0f);
    QWHIP_TRY_HIP(hipGetLastError());
    return QWHIP_OK;
}

extern "C" qwhip_status qwhip_argmax_f32_variational(qwhip_stream_t s, const float* logits, uint32_t rows, uint32_t n, const uint32_t* draft_tokens,
                                                     uint32_t total_rows, float margin, float min_log_prob, int32_t* tokens) {
    QWHIP_REQUIRE(s);
    if (rows == 0) return QWHIP_OK;
    QWHIP_REQUIRE(logits);
    QWHIP_REQUIRE(tokens);
    if (n == 0 || n >= (1u << 30)) return qwhip_fail(QWHIP_E_BAD_SHAPE, "argmax over %u logits does not fit the row-count flags", n);
    if (!(margin > 0.0f) || rows < 2u || total_rows < 2u)   // the door's own rule (QWGemmF32.swift:292): plain argmax otherwise
        return qwhip_argmax_f32(s, logits, rows, n, tokens);
    QWHIP_REQUIRE(draft_tokens);
    if (min_log_prob != min_log_prob) return qwhip_fail(QWHIP_E_BAD_SHAPE, "min_log_prob is NaN (-inf switches the probability gate off)");
    hipLaunchKernelGGL(qw_argmax_rows_kernel<true>, dim3(rows), dim3(1024), 0, s->stream, logits, n, tokens, draft_tokens, total_rows, margin,
                       min_log_prob);
    QWHIP_TRY_HIP(hipGetLastError());
    return QWHIP_OK;
}
