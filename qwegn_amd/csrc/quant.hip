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
