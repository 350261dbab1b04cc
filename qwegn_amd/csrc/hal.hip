// HIP HAL of libqwhip: device, streams, memory, events, the kernel-name table and view checks.
// Stands where QWHal stands in the reference (Sources/Foundation/QWHAL/QWHal.swift:81-398).
#include <stdarg.h>
#include <stdio.h>
#include <string.h>

#include <new>

#include "qwhip_common.h"

static thread_local char g_err[512] = "";

qwhip_status qwhip_fail(qwhip_status st, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return st;
}

qwhip_status qwhip_hip_check(hipError_t e, const char* what) {
    if (e == hipSuccess) return QWHIP_OK;
    return qwhip_fail(QWHIP_E_DEVICE, "HIP error %d (%s) at %s", (int)e, hipGetErrorString(e), what);
}

extern "C" const char* qwhip_last_error(void) { return g_err; }

extern "C" const char* qwhip_status_name(qwhip_status st) {
    switch (st) {
        case QWHIP_OK: return "ok";
        case QWHIP_E_BAD_WEIGHTS: return "badWeights";
        case QWHIP_E_BAD_SHAPE: return "badShape";
        case QWHIP_E_BAD_GEOMETRY: return "badGeometry";
        case QWHIP_E_BLOCKED: return "blocked";
        case QWHIP_E_KERNEL_MISSING: return "kernelMissing";
        case QWHIP_E_DEVICE: return "deviceUnavailable";
        case QWHIP_E_BASIS: return "basisMismatch";
        case QWHIP_E_NULL: return "nullPointer";
        case QWHIP_E_ALLOC: return "allocFailed";
        default: return "unknown";
    }
}

extern "C" qwhip_status qwhip_device_create(int32_t ordinal, qwhip_device_t* out) {
    QWHIP_REQUIRE(out);
    *out = nullptr;
    int count = 0;
    if (hipGetDeviceCount(&count) != hipSuccess || count <= 0)
        return qwhip_fail(QWHIP_E_DEVICE, "no HIP device is visible");
    if (ordinal < 0 || ordinal >= count)
        return qwhip_fail(QWHIP_E_DEVICE, "device ordinal %d out of range (%d visible)", ordinal, count);
    qwhip_device_s* d = new (std::nothrow) qwhip_device_s();
    if (!d) return qwhip_fail(QWHIP_E_ALLOC, "out of host memory");
    d->ordinal = ordinal;
    hipError_t e = hipGetDeviceProperties(&d->prop, ordinal);
    if (e != hipSuccess) {
        delete d;
        return qwhip_hip_check(e, "hipGetDeviceProperties");
    }
    // The code objects in this library are gfx950 only: refuse anything else at init, as the
    // reference refuses a metallib whose basis marker does not match (QWHal.swift:227-232).
    if (strncmp(d->prop.gcnArchName, "gfx950", 6) != 0) {
        qwhip_status st = qwhip_fail(QWHIP_E_DEVICE, "device %d is %s; libqwhip holds gfx950 code only", ordinal,
                                     d->prop.gcnArchName);
        delete d;
        return st;
    }
    e = hipSetDevice(ordinal);
    if (e != hipSuccess) {
        delete d;
        return qwhip_hip_check(e, "hipSetDevice");
    }
    // per-device address of the static GEMM scratch (gemm.hip), resolved while this device is current
    const qwhip_status sst = qw_gemm_scratch_init(ordinal);
    if (sst != QWHIP_OK) {
        delete d;
        return sst;
    }
    *out = d;
    return QWHIP_OK;
}

extern "C" qwhip_status qwhip_device_set_gated_activation(qwhip_device_t dev, uint32_t kind, float p0, float p1) {
    QWHIP_REQUIRE(dev);
    if (kind > 2u) return qwhip_fail(QWHIP_E_BAD_SHAPE, "gated activation %u is not one of 0 SwiGLU, 1 clamped SwiGLU, 2 bounded (tanh) form", kind);
    if (kind != 0u && !(p0 > 0.0f)) return qwhip_fail(QWHIP_E_BAD_SHAPE, "gated activation %u needs a positive first parameter", kind);
    dev->act.kind = kind;
    dev->act.p0 = kind ? p0 : 0.0f;
    dev->act.p1 = kind == 2u ? p1 : 0.0f;
    return QWHIP_OK;
}

extern "C" qwhip_status qwhip_device_destroy(qwhip_device_t dev) {
    delete dev;
    return QWHIP_OK;
}

extern "C" qwhip_status qwhip_device_caps(qwhip_device_t dev, qwhip_caps* out) {
    QWHIP_REQUIRE(dev);
    QWHIP_REQUIRE(out);
    memset(out, 0, sizeof(*out));
    snprintf(out->name, sizeof(out->name), "%s", dev->prop.name);
    snprintf(out->arch, sizeof(out->arch), "%s", dev->prop.gcnArchName);
    out->compute_units = (uint32_t)dev->prop.multiProcessorCount;
    out->wavefront = (uint32_t)dev->prop.warpSize;
    out->lds_bytes = (uint32_t)dev->prop.sharedMemPerBlock;
    out->l2_bytes = (uint32_t)dev->prop.l2CacheSize;
    out->hbm_bytes = (uint64_t)dev->prop.totalGlobalMem;
    out->clock_khz = (uint32_t)dev->prop.clockRate;
    out->has_mfma_f16 = 1;
    return QWHIP_OK;
}

extern "C" qwhip_status qwhip_stream_create(qwhip_device_t dev, qwhip_stream_t* out) {
    QWHIP_REQUIRE(dev);
    QWHIP_REQUIRE(out);
    *out = nullptr;
    QWHIP_TRY_HIP(hipSetDevice(dev->ordinal));
    qwhip_stream_s* s = new (std::nothrow) qwhip_stream_s();
    if (!s) return qwhip_fail(QWHIP_E_ALLOC, "out of host memory");
    s->dev = dev;
    hipError_t e = hipStreamCreateWithFlags(&s->stream, hipStreamNonBlocking);
    if (e != hipSuccess) {
        delete s;
        return qwhip_hip_check(e, "hipStreamCreateWithFlags");
    }
    // the stream's split-K scratch: counters zeroed once, here
    e = hipMalloc((void**)&s->scratch, QWHIP_STREAM_SCRATCH_BYTES);
    if (e == hipSuccess) e = hipMemset(s->scratch, 0, QWHIP_STREAM_COUNTER_BYTES);
    if (e != hipSuccess) {
        if (s->scratch) (void)hipFree(s->scratch);
        (void)hipStreamDestroy(s->stream);
        delete s;
        return qwhip_hip_check(e, "stream scratch");
    }
    s->scratch_bytes = QWHIP_STREAM_SCRATCH_BYTES;
    *out = s;
    return QWHIP_OK;
}

extern "C" qwhip_status qwhip_stream_destroy(qwhip_stream_t s) {
    if (!s) return QWHIP_OK;
    hipError_t e = hipStreamDestroy(s->stream);
    if (s->scratch) (void)hipFree(s->scratch);
    delete s;
    return qwhip_hip_check(e, "hipStreamDestroy");
}

extern "C" qwhip_status qwhip_stream_sync(qwhip_stream_t s) {
    QWHIP_REQUIRE(s);
    QWHIP_TRY_HIP(hipStreamSynchronize(s->stream));
    return QWHIP_OK;
}

extern "C" void* qwhip_stream_native(qwhip_stream_t s) { return s ? (void*)s->stream : nullptr; }

extern "C" qwhip_status qwhip_malloc(qwhip_device_t dev, size_t bytes, void** out) {
    QWHIP_REQUIRE(dev);
    QWHIP_REQUIRE(out);
    *out = nullptr;
    if (bytes == 0) bytes = 256;
    QWHIP_TRY_HIP(hipSetDevice(dev->ordinal));
    hipError_t e = hipMalloc(out, bytes);
    if (e != hipSuccess) {
        (void)hipGetLastError();
        return qwhip_fail(QWHIP_E_ALLOC, "hipMalloc(%zu) failed: %s", bytes, hipGetErrorString(e));
    }
    return QWHIP_OK;
}

extern "C" qwhip_status qwhip_free(qwhip_device_t dev, void* p) {
    QWHIP_REQUIRE(dev);
    if (!p) return QWHIP_OK;
    QWHIP_TRY_HIP(hipFree(p));
    return QWHIP_OK;
}

extern "C" qwhip_status qwhip_memcpy_h2d(qwhip_stream_t s, void* dst, const void* src, size_t bytes) {
    QWHIP_REQUIRE(s);
    if (bytes == 0) return QWHIP_OK;
    QWHIP_REQUIRE(dst);
    QWHIP_REQUIRE(src);
    QWHIP_TRY_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, s->stream));
    QWHIP_TRY_HIP(hipStreamSynchronize(s->stream));
    return QWHIP_OK;
}

extern "C" qwhip_status qwhip_memcpy_d2h(qwhip_stream_t s, void* dst, const void* src, size_t bytes) {
    QWHIP_REQUIRE(s);
    if (bytes == 0) return QWHIP_OK;
    QWHIP_REQUIRE(dst);
    QWHIP_REQUIRE(src);
    QWHIP_TRY_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, s->stream));
    QWHIP_TRY_HIP(hipStreamSynchronize(s->stream));
    return QWHIP_OK;
}

extern "C" qwhip_status qwhip_memcpy_d2d(qwhip_stream_t s, void* dst, const void* src, size_t bytes) {
    QWHIP_REQUIRE(s);
    if (bytes == 0) return QWHIP_OK;
    QWHIP_REQUIRE(dst);
    QWHIP_REQUIRE(src);
    QWHIP_TRY_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, s->stream));
    return QWHIP_OK;
}

__global__ void qw_fill_u32_kernel(uint32_t* dst, uint32_t value, size_t count) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; i < count; i += stride) dst[i] = value;
}

extern "C" qwhip_status qwhip_fill_u32(qwhip_stream_t s, void* dst, uint32_t value, size_t count) {
    QWHIP_REQUIRE(s);
    if (count == 0) return QWHIP_OK;
    QWHIP_REQUIRE(dst);
    size_t blocks = (count + 255) / 256;
    if (blocks > 4096) blocks = 4096;
    hipLaunchKernelGGL(qw_fill_u32_kernel, dim3((unsigned)blocks), dim3(256), 0, s->stream, (uint32_t*)dst, value, count);
    QWHIP_TRY_HIP(hipGetLastError());
    return QWHIP_OK;
}

// Sum of the 32-bit words of a plane, added into 256 lanes sum[0..255] whose total is the checksum (integer additions
// commute: the total does not depend on the order the workgroups finish in; 256 words because atomics on one address
// serialize at about 12 ns each).  A grid-wide stride of 16-byte loads at full occupancy (eight workgroups of four waves
// per compute unit: 10.6 us for 55.7 MB out of HBM, against 11.2 .. 12.6 with two to eight loads in flight per thread on
// a quarter of the workgroups) and nothing written but one atomic per workgroup: the launch is also the read-bandwidth
// yardstick of the device.
__global__ __launch_bounds__(256) void qw_plane_checksum_kernel(const u4_t* __restrict__ src, size_t n16, unsigned long long* sum) {
    const size_t stride = (size_t)gridDim.x * 256u;
    size_t i = (size_t)blockIdx.x * 256u + threadIdx.x;
    unsigned long long acc = 0;
    for (; i < n16; i += stride) {
        const u4_t a = src[i];
        acc += (unsigned long long)a[0] + a[1] + a[2] + a[3];
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) acc += __shfl_xor(acc, o, 64);
    __shared__ unsigned long long wsum[4];
    if ((threadIdx.x & 63u) == 0) wsum[threadIdx.x >> 6] = acc;
    __syncthreads();
    if (threadIdx.x == 0) atomicAdd(sum + (blockIdx.x & 255u), wsum[0] + wsum[1] + wsum[2] + wsum[3]);
}

extern "C" qwhip_status qwhip_plane_checksum(qwhip_stream_t s, const void* plane, size_t bytes, uint64_t* sum) {
    QWHIP_REQUIRE(s);
    QWHIP_REQUIRE(sum);
    if (bytes == 0) return QWHIP_OK;
    QWHIP_REQUIRE(plane);
    if ((bytes & 15u) != 0 || ((uintptr_t)plane & 15u) != 0)
        return qwhip_fail(QWHIP_E_BAD_SHAPE, "checksum takes a 16-byte aligned plane of whole 16-byte pieces, got %zu bytes", bytes);
    const size_t n16 = bytes / 16u;
    size_t blocks = (n16 + 1023u) / 1024u;
    if (blocks > 2048u) blocks = 2048u;   // eight workgroups of four waves per compute unit
    hipLaunchKernelGGL(qw_plane_checksum_kernel, dim3((unsigned)blocks), dim3(256), 0, s->stream, (const u4_t*)plane, n16,
                       (unsigned long long*)sum);
    QWHIP_TRY_HIP(hipGetLastError());
    return QWHIP_OK;
}

extern "C" qwhip_status qwhip_event_create(qwhip_device_t dev, qwhip_event_t* out) {
    QWHIP_REQUIRE(dev);
    QWHIP_REQUIRE(out);
    *out = nullptr;
    qwhip_event_s* e = new (std::nothrow) qwhip_event_s();
    if (!e) return qwhip_fail(QWHIP_E_ALLOC, "out of host memory");
    e->dev = dev;
    hipError_t r = hipEventCreate(&e->ev);
    if (r != hipSuccess) {
        delete e;
        return qwhip_hip_check(r, "hipEventCreate");
    }
    *out = e;
    return QWHIP_OK;
}

extern "C" qwhip_status qwhip_event_destroy(qwhip_event_t e) {
    if (!e) return QWHIP_OK;
    hipError_t r = hipEventDestroy(e->ev);
    delete e;
    return qwhip_hip_check(r, "hipEventDestroy");
}

extern "C" qwhip_status qwhip_event_record(qwhip_event_t e, qwhip_stream_t s) {
    QWHIP_REQUIRE(e);
    QWHIP_REQUIRE(s);
    QWHIP_TRY_HIP(hipEventRecord(e->ev, s->stream));
    return QWHIP_OK;
}

extern "C" qwhip_status qwhip_event_elapsed_ms(qwhip_event_t start, qwhip_event_t stop, float* ms) {
    QWHIP_REQUIRE(start);
    QWHIP_REQUIRE(stop);
    QWHIP_REQUIRE(ms);
    QWHIP_TRY_HIP(hipEventSynchronize(stop->ev));
    QWHIP_TRY_HIP(hipEventElapsedTime(ms, start->ev, stop->ev));
    return QWHIP_OK;
}

// ---- kernel-name table ---------------------------------------------------------------------
// Keys are the reference's Metal entry points; values name the launcher that serves them here.
struct qw_kernel_entry {
    const char* name;
    const char* launcher;
};

static const qw_kernel_entry g_kernels[] = {
    {"qwg_fwht32_f16", "qwhip_fwht32"},
    {"qwg_cast_f32_to_f16", "qwhip_cast_f32_to_f16"},
    {"qwg_gemv_q4g_v4", "qwhip_gemv"},
    {"qwg_gemv_q4g_v4_h16", "qwhip_gemv"},
    {"qwg_gemv_q4g_v4_h16_dual", "qwhip_gemv"},
    {"qwg_gemv_q4g_dx_h16_t4", "qwhip_gemv"},
    {"qwg_gemv_q4g_dx_h16_dual_t4", "qwhip_gemv"},
    {"qwg_skinny_m2", "qwhip_gemv"},
    {"qwg_skinny_m3", "qwhip_gemv"},
    {"qwg_gemv_q4g_silu_pair", "qwhip_gemv_silu_pair"},
    {"qwg_gemv_q4g_silu_pair_h16", "qwhip_gemv_silu_pair"},
    {"qwg_gemv_q4g_silu_pair_dx_h16", "qwhip_gemv_silu_pair"},
    {"qwg_gemm_q4g_h16", "qwhip_gemm"},
    {"qwg_gemm_q4g_nax_f32", "qwhip_gemm"},
    {"qwg_gemm_q4g_h16_swiglu", "qwhip_gemm_swiglu"},
    {"qwg_silu_mul_f16", "qwhip_swiglu_fwht"},
    {"qwg_silu_mul_split_f16", "qwhip_swiglu_fwht"},
    {"qwg_moe_route", "qwhip_moe_route"},
    {"qwg_f32_gemv", "qwhip_f32_gemv"},
    {"qwg_f32_gemv_bm", "qwhip_f32_gemv"},
    {"qwg_head_argmax_fin", "qwhip_argmax_f32"},
    {"qwg_head_argmax_fin_variational", "qwhip_argmax_f32_variational"},
    {"qwg_moe_route_decode", "qwhip_moe_route"},
    {"qwg_router_gemm", "qwhip_router_gemm"},
    {"qwg_embed_aq_f32", "qwhip_embed_aq_f32"},
    {"qwg_embed_bf16_f32", "qwhip_embed_bf16_f32"},
    {"qwg_silu_mul_f32", "qwhip_silu_mul_f32"},
    {"qwg_moe_bridge_f16_to_f32", "qwhip_moe_bridge_f16_to_f32"},
    {"qwg_latent_norm_h32_f32", "qwhip_latent_norm_h32_f32"},
    {"qwg_add_f32", "qwhip_add_f32"},
    {"qwg_router_nax", "qwhip_router_gemm"},
    {"qwg_moe_group_pairs_f32", "qwhip_moe_group_pairs"},
    {"qwg_moe_nax_gemm", "qwhip_moe_grouped_gemm"},
    {"qwg_moe_nax_split_f32", "qwhip_moe_grouped_gemm"},
    {"qwg_moe_down_reduce_combine_f32", "qwhip_moe_combine"},
    {"qwg_moe_gateup_q4g_f32_r1", "qwhip_moe_gateup_decode"},
    {"qwg_moe_down_shared_combine_q4g_f32", "qwhip_moe_down_decode"},
    {"qwg_quantize_bf16_to_hq4_g32_m5", "qwhip_quantize_hq4_g32"},
    {"qwg_head_gemv_q4g_argmax", "qwhip_head_argmax"},
    {"qwg_gemv_q4g_f32_v4_am", "qwhip_head_argmax"},
    {"qwg_gemv_q4g_f32_v4_am2", "qwhip_head_argmax"},
    {"qwg_gemv_q4g_f32_v4", "qwhip_gemv_f32"},
    {"qwg_gemm_q4g_f32_bm", "qwhip_gemv_f32"},
    {"qwg_gemm_q4g_f32_bm32", "qwhip_gemv_f32"},
    {"qwg_h32_f32", "qwhip_h32_f32"},
    {"qwg_rmsnorm", "qwhip_rmsnorm"},
    {"qwg_rmsnorm_residual", "qwhip_rmsnorm"},
    {"qwg_rmsnorm_residual_wide", "qwhip_rmsnorm"},
    {"qwg_repack_mlx_affine_to_aq_m5", "qwhip_repack_mlx_affine"},
    {"qwg_repack_mlx_affine_switch_gate_up_to_aq_m5", "qwhip_repack_mlx_affine_switch_gate_up"},
};

static bool qw_parse_aq_name(const char* name, const char** launcher) {
    // qwg_{gemv,gemm,moe_...}_aq<bits>_g<group>_<suffix> for the (bits, group) pairs with kernels here.
    unsigned bits = 0, group = 0;
    char suffix[64] = "";
    const char* lau = nullptr;
    if (sscanf(name, "qwg_gemv_aq%u_g%u_%63s", &bits, &group, suffix) == 3) {
        if (!strcmp(suffix, "v4") || !strcmp(suffix, "dx_h16_t4")) lau = "qwhip_gemv";
        else if (!strcmp(suffix, "f32_v4")) lau = "qwhip_gemv_f32";
        else if (!strcmp(suffix, "f32_v4_am") || !strcmp(suffix, "f32_v4_am2")) lau = "qwhip_head_argmax";
        else if (!strcmp(suffix, "silu_pair_dx_h16")) lau = "qwhip_gemv_silu_pair";
    } else if (sscanf(name, "qwg_gemm_aq%u_g%u_%63s", &bits, &group, suffix) == 3) {
        if (!strcmp(suffix, "h16") || !strcmp(suffix, "nax_f32")) lau = "qwhip_gemm";
        else if (!strcmp(suffix, "f32_bm") || !strcmp(suffix, "f32_bm32")) lau = "qwhip_gemv_f32";
        else if (!strcmp(suffix, "h16_swiglu")) lau = "qwhip_gemm_swiglu";
    } else if (sscanf(name, "qwg_moe_nax_gemm_aq%u_g%u", &bits, &group) == 2 ||
               sscanf(name, "qwg_moe_nax_split_f32_aq%u_g%u", &bits, &group) == 2 ||
               (sscanf(name, "qwg_moe_nax_split_aq%u_g%u_%63s", &bits, &group, suffix) == 3 && !strcmp(suffix, "f32"))) {
        lau = "qwhip_moe_grouped_gemm";
    } else if (sscanf(name, "qwg_head_gemv_aq%u_g%u_%63s", &bits, &group, suffix) == 3 && !strcmp(suffix, "argmax")) {
        lau = "qwhip_head_argmax";
    } else if (sscanf(name, "qwg_moe_gateup_aq%u_g%u_f32_r1", &bits, &group) == 2) {
        lau = "qwhip_moe_gateup_decode";
    } else if (sscanf(name, "qwg_moe_down_shared_combine_aq%u_g%u_f32", &bits, &group) == 2) {
        lau = "qwhip_moe_down_decode";
    }
    if (!lau) return false;
    if (!(bits == 2 || bits == 3 || bits == 4 || bits == 6 || bits == 8)) return false;
    if (!(group == 32 || group == 64 || group == 128 || group == 256)) return false;
    if (launcher) *launcher = lau;
    return true;
}

extern "C" qwhip_status qwhip_kernel_lookup(const char* name, const char** launcher) {
    QWHIP_REQUIRE(name);
    for (const qw_kernel_entry& e : g_kernels) {
        if (!strcmp(e.name, name)) {
            if (launcher) *launcher = e.launcher;
            return QWHIP_OK;
        }
    }
    if (qw_parse_aq_name(name, launcher)) return QWHIP_OK;
    return qwhip_fail(QWHIP_E_KERNEL_MISSING, "kernel missing: %s", name);
}

// ---- container checks ----------------------------------------------------------------------
extern "C" uint32_t qwhip_block_bytes(uint32_t kind, uint32_t bits, uint32_t group) {
    if (kind == QWHIP_KIND_HQ4_G32_M5) return (bits == 4 && group == 32) ? 20u : 0u;
    if (kind != QWHIP_KIND_ROTATED_HQ && kind != QWHIP_KIND_NATIVE_AFFINE) return 0u;
    const bool bits_ok = bits == 2 || bits == 3 || bits == 4 || bits == 6 || bits == 8;
    const bool group_ok = group == 32 || group == 64 || group == 128 || group == 256;
    return (bits_ok && group_ok) ? 4u + group * bits / 8u : 0u;
}

extern "C" qwhip_status qwhip_weight_view_validate(const qwhip_weight_view* w) {
    QWHIP_REQUIRE(w);
    const uint32_t bb = qwhip_block_bytes(w->kind, w->bits, w->group);
    if (bb == 0)
        return qwhip_fail(QWHIP_E_BAD_WEIGHTS, "no container for kind %u, %u-bit group %u", w->kind, w->bits, w->group);
    if (w->n == 0 || w->k == 0 || (w->k % w->group) != 0)
        return qwhip_fail(QWHIP_E_BAD_WEIGHTS, "k must be a multiple of %u and n positive (n=%u k=%u)", w->group, w->n,
                          w->k);
    const uint64_t needed = (uint64_t)w->n * (w->k / w->group) * bb;
    if (w->bytes < needed)
        return qwhip_fail(QWHIP_E_BAD_WEIGHTS, "block bank holds %llu bytes, %llu needed", (unsigned long long)w->bytes,
                          (unsigned long long)needed);
    if (w->blocks == nullptr) return qwhip_fail(QWHIP_E_NULL, "weight view has no blocks");
    if (((uintptr_t)w->blocks & 3u) != 0) return qwhip_fail(QWHIP_E_BAD_WEIGHTS, "block bank must be 4-byte aligned");
    return QWHIP_OK;
}
