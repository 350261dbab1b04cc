// MoE plumbing around the grouped GEMM: router logits, softmax top-k routing, the expert-major pair sort
// with its tile list, and the weighted combine.
#include <algorithm>
#include <atomic>

#include "qwhip_common.h"
#include "qwhip_route.h"

// ------------------------------------------------------------------------------------------------
// Router logits: logits[t, e] = sum_h x[t, h] * Wr[e, h], fp32 accumulate.
// A workgroup owns TT token rows (staged as fp32 in LDS; 8 rows up to hidden = 2048, fewer on wider rows so the tile
// stays within 64 KiB, and no more than the call has) so each router row is read once per TT tokens; blockIdx.y owns a band of `eb` weight rows
// (a multiple of 4, so that few token rows still spread over the chip), a wavefront the band's rows wave, wave+4, ...;
// lanes stride the hidden dimension, so an output's summation order does not depend on the band size.  With a shared-expert gate row (fp32 [hidden]) the workgroup also writes
// sh_out[t] = sigmoid(x[t] . sh_w), the extra output column of the reference's router kernels
// (Sources/QWMetal/subsystems/qwrouter.metal:467-483,566-574,587-633).
// ------------------------------------------------------------------------------------------------
// The scalar epilogues of the dense f32 GEMV door (qwg_f32_gemv, Sources/QWMetal/gemm/qwgemm_f32.metal:120-143):
// 0 none, 1 silu(y / scale), 2 sigmoid(y), 3 2 sigmoid(y / scale).
__device__ __forceinline__ float qw_f32_gemv_epilogue(float y, uint32_t epi, float scale) {
    if (epi == 1u) {
        const float z = y / scale;
        return z / (1.0f + expf(-z));
    }
    if (epi == 2u) return 1.0f / (1.0f + expf(-y));
    if (epi == 3u) return 2.0f / (1.0f + expf(-(y / scale)));
    return y;
}

template <int XDT, int WDT, int TT>
__global__ __launch_bounds__(256) void qw_router_gemm_kernel(const void* __restrict__ x, const void* __restrict__ wr,
                                                              float* __restrict__ logits, uint32_t T, uint32_t E, uint32_t H,
                                                              const float* __restrict__ sh_w, float* __restrict__ sh_out,
                                                              uint32_t epi, float scale, uint32_t eb) {
    extern __shared__ float xs[];  // [TT][H]
    const uint32_t t0 = blockIdx.x * TT;
    const uint32_t nt = min((uint32_t)TT, T - t0);
#pragma unroll
    for (uint32_t r = 0; r < (uint32_t)TT; ++r)
        for (uint32_t h = threadIdx.x; h < H; h += 256) xs[r * H + h] = r < nt ? qw_load_f32<XDT>(x, (uint64_t)(t0 + r) * H + h) : 0.0f;
    __syncthreads();
    const uint32_t wave = threadIdx.x >> 6, lane = threadIdx.x & 63u;
    const uint32_t rows = min(E + (sh_w ? 1u : 0u), (blockIdx.y + 1u) * eb);
    for (uint32_t e = blockIdx.y * eb + wave; e < rows; e += 4) {
        const bool gate_row = e == E;   // wave-uniform
        float acc[TT];
#pragma unroll
        for (int r = 0; r < TT; ++r) acc[r] = 0.0f;
        // eight weight loads in flight per lane, consumed in the order h = lane, lane + 64, ... so the sums do not depend on it
        uint32_t h = lane;
        if (!gate_row) {
            const uint64_t row = (uint64_t)e * H;
            for (; h + 7u * 64u < H; h += 8u * 64u) {
                float w[8];
#pragma unroll
                for (int u = 0; u < 8; ++u) w[u] = qw_load_f32<WDT>(wr, row + h + (uint32_t)u * 64u);
#pragma unroll
                for (int u = 0; u < 8; ++u)
#pragma unroll
                    for (int r = 0; r < TT; ++r) acc[r] = fmaf(w[u], xs[r * H + h + (uint32_t)u * 64u], acc[r]);
            }
        }
        for (; h < H; h += 64) {
            const float w = gate_row ? sh_w[h] : qw_load_f32<WDT>(wr, (uint64_t)e * H + h);
#pragma unroll
            for (int r = 0; r < TT; ++r) acc[r] = fmaf(w, xs[r * H + h], acc[r]);
        }
#pragma unroll
        for (int r = 0; r < TT; ++r) {
            const float v = qw_reduce64(acc[r]);
            if (lane == 0 && (uint32_t)r < nt) {
                if (gate_row) sh_out[t0 + r] = 1.0f / (1.0f + expf(-v));
                else logits[(uint64_t)(t0 + r) * E + e] = qw_f32_gemv_epilogue(v, epi, scale);
            }
        }
    }
}

static qwhip_status qw_router_gemm_impl(qwhip_stream_t s, const void* x, uint32_t x_dtype, const void* wr, uint32_t w_dtype, uint32_t t,
                                        uint32_t experts, uint32_t hidden, float* logits, const float* sh_gate_w, float* sh_gate_out,
                                        uint32_t epi, float scale) {
    QWHIP_REQUIRE(s);
    if (t == 0) return QWHIP_OK;
    QWHIP_REQUIRE(x);
    QWHIP_REQUIRE(wr);
    QWHIP_REQUIRE(logits);
    if ((sh_gate_w != nullptr) != (sh_gate_out != nullptr))
        return qwhip_fail(QWHIP_E_NULL, "router gemm: the shared-expert gate needs both its weight row and its output");
    if (experts == 0 || hidden == 0) return qwhip_fail(QWHIP_E_BAD_SHAPE, "router gemm: empty experts or hidden");
    // token rows per workgroup: the fp32 tile stays within 64 KiB
    uint32_t tt = 8;
    while (tt > 1u && ((size_t)tt * hidden * 4u > 64u * 1024u || tt >= 2u * t)) tt >>= 1;
    const size_t lds = (size_t)tt * hidden * 4u;
    if (lds > 64u * 1024u) return qwhip_fail(QWHIP_E_BAD_SHAPE, "router gemm: hidden %u exceeds the staged row (<= 16384)", hidden);
    // weight rows per workgroup: about 1024 workgroups over the launch, at least one row per wavefront
    const uint32_t gx = qwhip_cdiv(t, tt), rows_total = experts + (sh_gate_w ? 1u : 0u);
    const uint32_t gy_want = std::min(qwhip_cdiv(rows_total, 4u), std::max(1u, 1024u / gx));
    const uint32_t eb = (qwhip_cdiv(rows_total, gy_want) + 3u) & ~3u;
    const dim3 grid(gx, qwhip_cdiv(rows_total, eb)), block(256);
    if (grid.y > 65535u) return qwhip_fail(QWHIP_E_BAD_SHAPE, "router gemm: %u weight rows exceed the launch grid", rows_total);
#define QW_RG(XD, WD, TT) \
    hipLaunchKernelGGL((qw_router_gemm_kernel<XD, WD, TT>), grid, block, lds, s->stream, x, wr, logits, t, experts, hidden, sh_gate_w, sh_gate_out, epi, scale, eb)
#define QW_RG_T(XD, WD)                       \
    switch (tt) {                             \
        case 8: QW_RG(XD, WD, 8); break;      \
        case 4: QW_RG(XD, WD, 4); break;      \
        case 2: QW_RG(XD, WD, 2); break;      \
        default: QW_RG(XD, WD, 1); break;     \
    }
#define QW_RG_W(XD)                                                   \
    switch (w_dtype) {                                                \
        case QWHIP_F32: QW_RG_T(XD, QWHIP_F32) break;                 \
        case QWHIP_F16: QW_RG_T(XD, QWHIP_F16) break;                 \
        case QWHIP_BF16: QW_RG_T(XD, QWHIP_BF16) break;               \
        default: return qwhip_fail(QWHIP_E_BAD_SHAPE, "router gemm: unsupported weight dtype %u", w_dtype); \
    }
    switch (x_dtype) {
        case QWHIP_F32: QW_RG_W(QWHIP_F32) break;
        case QWHIP_F16: QW_RG_W(QWHIP_F16) break;
        case QWHIP_BF16: QW_RG_W(QWHIP_BF16) break;
        default: return qwhip_fail(QWHIP_E_BAD_SHAPE, "router gemm: unsupported activation dtype %u", x_dtype);
    }
#undef QW_RG_W
#undef QW_RG_T
#undef QW_RG
    QWHIP_TRY_HIP(hipGetLastError());
    return QWHIP_OK;
}

extern "C" qwhip_status qwhip_router_gemm_shared_gate(qwhip_stream_t s, const void* x, uint32_t x_dtype, const void* wr, uint32_t w_dtype,
                                                      uint32_t t, uint32_t experts, uint32_t hidden, float* logits,
                                                      const float* sh_gate_w, float* sh_gate_out) {
    return qw_router_gemm_impl(s, x, x_dtype, wr, w_dtype, t, experts, hidden, logits, sh_gate_w, sh_gate_out, 0u, 1.0f);
}

extern "C" qwhip_status qwhip_router_gemm(qwhip_stream_t s, const void* x, uint32_t x_dtype, const void* wr, uint32_t w_dtype,
                                          uint32_t t, uint32_t experts, uint32_t hidden, float* logits) {
    return qw_router_gemm_impl(s, x, x_dtype, wr, w_dtype, t, experts, hidden, logits, nullptr, nullptr, 0u, 1.0f);
}

// Dense fp32-weight GEMV with the scalar epilogues (QWGemm.encodeF32Gemv, Sources/Operators/QWGEMM/QWGemmF32.swift:117-141 ->
// qwg_f32_gemv / qwg_f32_gemv_bm): y[t, n] = epilogue(sum_k W[n, k] x[t, k]) on the router kernel (every weight row read once
// per eight activation rows).
extern "C" qwhip_status qwhip_f32_gemv(qwhip_stream_t s, const float* w, const float* x, uint32_t rows, uint32_t n, uint32_t k,
                                       uint32_t epi, float scale, float* y) {
    if (epi > 3u) return qwhip_fail(QWHIP_E_BAD_SHAPE, "epilogue %u is not one of 0 none, 1 silu(y/scale), 2 sigmoid, 3 2 sigmoid(y/scale)", epi);
    if ((epi == 1u || epi == 3u) && !(scale != 0.0f && scale == scale))
        return qwhip_fail(QWHIP_E_BAD_SHAPE, "epilogue %u divides by its scale, which must be a non-zero number", epi);
    return qw_router_gemm_impl(s, x, QWHIP_F32, w, QWHIP_F32, rows, n, k, y, nullptr, nullptr, epi, scale);
}

// ------------------------------------------------------------------------------------------------
// Routing: one wavefront per token row; lane l holds experts l, l+64, ... (E <= 512 -> <= 8 each).
// fp32 softmax (max-subtracted), top_k rounds of argmax with ties to the lower index, optional
// renormalisation by the sum of the selected, times the routed scale.  Non-finite logits never win.
// ------------------------------------------------------------------------------------------------
template <int JN>   // experts per lane: E <= 64 * JN
__global__ __launch_bounds__(64) void qw_moe_route_kernel(const float* __restrict__ logits, int32_t* __restrict__ idx,
                                                           float* __restrict__ wts, uint32_t E, uint32_t K, uint32_t norm,
                                                           float routed_scale) {
    const uint32_t t = blockIdx.x, lane = threadIdx.x;
    int32_t isel;
    float w;
    qw_route_wave<JN>(logits + (uint64_t)t * E, E, K, norm, routed_scale, lane, isel, w);
    if (lane < K) {
        idx[(uint64_t)t * K + lane] = isel;
        wts[(uint64_t)t * K + lane] = w;
    }
}

extern "C" qwhip_status qwhip_moe_route(qwhip_stream_t s, const float* logits, uint32_t t, uint32_t experts, uint32_t top_k,
                                        uint32_t norm_topk, float routed_scale, int32_t* idx, float* wts) {
    QWHIP_REQUIRE(s);
    if (t == 0) return QWHIP_OK;
    QWHIP_REQUIRE(logits);
    QWHIP_REQUIRE(idx);
    QWHIP_REQUIRE(wts);
    if (experts == 0 || experts > 512) return qwhip_fail(QWHIP_E_BAD_SHAPE, "moe route: experts must be 1..512, got %u", experts);
    if (top_k == 0 || top_k > 16) return qwhip_fail(QWHIP_E_BAD_SHAPE, "moe route: top_k must be 1..16, got %u", top_k);
    const float scale = routed_scale > 0.0f ? routed_scale : 1.0f;
#define QW_ROUTE(J) hipLaunchKernelGGL(qw_moe_route_kernel<J>, dim3(t), dim3(64), 0, s->stream, logits, idx, wts, experts, top_k, \
                                       norm_topk ? 1u : 0u, scale)
    if (experts <= 64) QW_ROUTE(1);
    else if (experts <= 128) QW_ROUTE(2);
    else if (experts <= 256) QW_ROUTE(4);
    else QW_ROUTE(8);
#undef QW_ROUTE
    QWHIP_TRY_HIP(hipGetLastError());
    return QWHIP_OK;
}

// The routing door with the reference's other modes (encodeFnMoeRoute's bias / splitFeature / routedScaleParam,
// Sources/Operators/QWGEMM/QWGemmMoERouter.swift:10-58): sigmoid scoring when a selection bias or split-feature logits
// ([t, 2 experts]) are given, softmax otherwise; a per-expert scale replaces the routed scale when given.
template <int JN>
__global__ __launch_bounds__(64) void qw_moe_route_ex_kernel(const float* __restrict__ logits, int32_t* __restrict__ idx,
                                                              float* __restrict__ wts, uint32_t E, uint32_t K, uint32_t norm,
                                                              float routed_scale, uint32_t split, const float* __restrict__ bias,
                                                              const float* __restrict__ scale_param) {
    const uint32_t t = blockIdx.x, lane = threadIdx.x;
    const float* row = logits + (uint64_t)t * (split ? 2u * E : E);
    int32_t isel;
    float w;
    if (bias || split) qw_route_wave_sigmoid<JN>(row, E, K, norm, split != 0, bias, lane, isel, w);
    else qw_route_wave<JN>(row, E, K, norm, 1.0f, lane, isel, w);
    if (lane < K) {
        const float scale = (scale_param && isel >= 0) ? scale_param[(uint32_t)isel & 0xFFFFu] : routed_scale;
        idx[(uint64_t)t * K + lane] = isel;
        wts[(uint64_t)t * K + lane] = w * scale;
    }
}

extern "C" qwhip_status qwhip_moe_route_ex(qwhip_stream_t s, const float* logits, uint32_t t, uint32_t experts, uint32_t top_k,
                                           uint32_t norm_topk, float routed_scale, uint32_t split_feature, const float* bias,
                                           const float* scale_param, int32_t* idx, float* wts) {
    QWHIP_REQUIRE(s);
    if (t == 0) return QWHIP_OK;
    QWHIP_REQUIRE(logits);
    QWHIP_REQUIRE(idx);
    QWHIP_REQUIRE(wts);
    if (experts == 0 || experts > 512) return qwhip_fail(QWHIP_E_BAD_SHAPE, "moe route: experts must be 1..512, got %u", experts);
    if (top_k == 0 || top_k > 16) return qwhip_fail(QWHIP_E_BAD_SHAPE, "moe route: top_k must be 1..16, got %u", top_k);
    const float scale = routed_scale > 0.0f ? routed_scale : 1.0f;
#define QW_ROUTE(J) hipLaunchKernelGGL(qw_moe_route_ex_kernel<J>, dim3(t), dim3(64), 0, s->stream, logits, idx, wts, experts, top_k, \
                                       norm_topk ? 1u : 0u, scale, split_feature ? 1u : 0u, bias, scale_param)
    if (experts <= 64) QW_ROUTE(1);
    else if (experts <= 128) QW_ROUTE(2);
    else if (experts <= 256) QW_ROUTE(4);
    else QW_ROUTE(8);
#undef QW_ROUTE
    QWHIP_TRY_HIP(hipGetLastError());
    return QWHIP_OK;
}

// ------------------------------------------------------------------------------------------------
// Expert-major pair sort: counting sort by expert id in one 1024-thread workgroup, plus the tile list.
// ------------------------------------------------------------------------------------------------
extern "C" uint32_t qwhip_moe_max_tiles(uint32_t experts, uint32_t pairs) {
    const uint32_t a = experts < pairs ? experts : pairs;
    const uint32_t b = a + (pairs + 63u) / 64u;
    return pairs < b ? pairs : b;
}

__device__ __forceinline__ int qw_moe_tile_block(int c) { return c <= 16 ? 16 : (c <= 32 ? 32 : 64); }
__device__ __forceinline__ int qw_moe_pack_tile_r(int tid_y, int bm) {
    const int code = (bm == 16) ? 1 : ((bm == 32) ? 2 : 3);
    return (code << 24) | (tid_y & 0xFFFFFF);
}

__global__ __launch_bounds__(1024) void qw_moe_group_pairs_kernel(const int32_t* __restrict__ ids, uint32_t experts,
                                                                   uint32_t pairs, uint32_t top_k, int32_t* __restrict__ expert_off,
                                                                   int32_t* __restrict__ sorted_pair, int32_t* __restrict__ sorted_tok,
                                                                   int32_t* __restrict__ inv_perm, int32_t* __restrict__ tile_e,
                                                                   int32_t* __restrict__ tile_r, int32_t* __restrict__ tile_count,
                                                                   uint32_t compact_tail, uint32_t stage_lds) {
    extern __shared__ int32_t lds_sorted[];   // [pairs] when stage_lds
    // Per-wave histograms and cursors: LDS atomics of the 16 waves on one shared set of counters serialize on the few
    // hot addresses (16,384 pairs over 128 experts: 32 us); privately they meet only their own 64 lanes.
    __shared__ int cnt_w[16][512];
    __shared__ int cnt[512];
    __shared__ int off[513];
    __shared__ int tile_off[513];
    const uint32_t tid = threadIdx.x;
    const uint32_t wave = tid >> 6;
    for (uint32_t e = tid; e < 16u * 512u; e += 1024) (&cnt_w[0][0])[e] = 0;
    __syncthreads();
    // ids in batches of 16 per thread: the loads of a batch are issued together (a load per atomic would pay one memory
    // round trip per pair and thread)
    for (uint32_t base = 0; base < pairs; base += 16u * 1024u) {
        int32_t raw[16];
#pragma unroll
        for (int c = 0; c < 16; ++c) {
            const uint32_t i = base + tid + 1024u * c;
            raw[c] = ids[min(i, pairs - 1u)];
            if (i >= pairs) raw[c] = -1;
        }
#pragma unroll
        for (int c = 0; c < 16; ++c) {
            if (raw[c] >= 0) {
                const uint32_t e = (uint32_t)raw[c] & 0xFFFFu;
                if (e < experts) atomicAdd(&cnt_w[wave][e], 1);
            }
        }
    }
    __syncthreads();
    for (uint32_t e = tid; e < experts; e += 1024) {
        int c = 0;
#pragma unroll
        for (int w = 0; w < 16; ++w) c += cnt_w[w][e];
        cnt[e] = c;
    }
    __syncthreads();
    if (tid < 64u) {
        // exclusive scans over <= 512 experts (rows and tiles) by one wave: lane l owns experts 8 l .. 8 l + 7
        int rows8[8], tiles8[8], rsum = 0, tsum = 0;
#pragma unroll
        for (int q = 0; q < 8; ++q) {
            const uint32_t e = 8u * tid + q;
            const int n = e < experts ? cnt[e] : 0;
            int t = 0;
            if (n > 0) {
                if (compact_tail) t = (n >> 6) + ((n & 63) ? 1 : 0);
                else {
                    const int bm = qw_moe_tile_block(n);
                    t = (n + bm - 1) / bm;
                }
            }
            rows8[q] = rsum;
            tiles8[q] = tsum;
            rsum += n;
            tsum += t;
        }
        int rinc = rsum, tinc = tsum;   // inclusive scan over the lanes
#pragma unroll
        for (int d = 1; d < 64; d <<= 1) {
            const int ro = __shfl_up(rinc, d, 64), to = __shfl_up(tinc, d, 64);
            if ((int)tid >= d) {
                rinc += ro;
                tinc += to;
            }
        }
        const int rbase = rinc - rsum, tbase = tinc - tsum;
#pragma unroll
        for (int q = 0; q < 8; ++q) {
            const uint32_t e = 8u * tid + q;
            if (e < experts) {
                off[e] = rbase + rows8[q];
                tile_off[e] = tbase + tiles8[q];
            }
        }
        if (tid == 63u) {
            off[experts] = rinc;
            tile_off[experts] = tinc;
        }
    }
    __syncthreads();
    for (uint32_t e = tid; e <= experts; e += 1024) {
        expert_off[e] = off[e];
        if (e < experts) {   // the waves' slices of the expert's slot range, in wave order: counts become cursors
            int c = off[e];
#pragma unroll
            for (int w = 0; w < 16; ++w) {
                const int n = cnt_w[w][e];
                cnt_w[w][e] = c;
                c += n;
            }
        }
    }
    __syncthreads();
    for (uint32_t base = 0; base < pairs; base += 16u * 1024u) {
        int32_t raw[16];
#pragma unroll
        for (int c = 0; c < 16; ++c) {
            const uint32_t i = base + tid + 1024u * c;
            raw[c] = ids[min(i, pairs - 1u)];
            if (i >= pairs) raw[c] = -2;   // past the list: nothing to place, nothing to mark
        }
#pragma unroll
        for (int c = 0; c < 16; ++c) {
            const uint32_t i = base + tid + 1024u * c;
            if (raw[c] == -2) continue;
            bool placed = false;
            if (raw[c] >= 0) {
                const uint32_t e = (uint32_t)raw[c] & 0xFFFFu;
                if (e < experts) {
                    const int at = atomicAdd(&cnt_w[wave][e], 1);
                    if (stage_lds) {
                        lds_sorted[at] = (int32_t)i;          // written out in slot order below
                    } else {
                        sorted_pair[at] = (int32_t)i;
                        sorted_tok[at] = (int32_t)(i / top_k);
                    }
                    if (inv_perm) inv_perm[i] = at;
                    placed = true;
                }
            }
            if (!placed && inv_perm) inv_perm[i] = -1;
        }
    }
    if (stage_lds) {
        // the sorted list was built in LDS: stores in slot order are whole lines (scattered 4-byte stores from the one
        // CU this kernel runs on cost an address cycle each: 2 x 16,384 of them were most of its time)
        __syncthreads();
        const uint32_t total = (uint32_t)off[experts];
        for (uint32_t j = tid; j < total; j += 1024) {
            const int32_t sp = lds_sorted[j];
            sorted_pair[j] = sp;
            sorted_tok[j] = (int32_t)((uint32_t)sp / top_k);
        }
    }
    if (tile_e) {
        for (uint32_t e = tid; e < experts; e += 1024) {
            const int n = cnt[e];
            int t = tile_off[e];
            if (n <= 0) continue;
            if (compact_tail) {
                const int q = n >> 6, rem = n & 63;
                for (int r = 0; r < q; ++r) {
                    tile_e[t] = (int32_t)e;
                    tile_r[t] = qw_moe_pack_tile_r(r, 64);
                    ++t;
                }
                if (rem > 0) {
                    const int bm = qw_moe_tile_block(rem);
                    tile_e[t] = (int32_t)e;
                    tile_r[t] = qw_moe_pack_tile_r((q * 64) / bm, bm);
                }
            } else {
                const int bm = qw_moe_tile_block(n);
                for (int r = 0; r * bm < n; ++r) {
                    tile_e[t] = (int32_t)e;
                    tile_r[t] = qw_moe_pack_tile_r(r, bm);
                    ++t;
                }
            }
        }
        if (tid == 0) tile_count[0] = tile_off[experts];
    }
}

extern "C" qwhip_status qwhip_moe_group_pairs(qwhip_stream_t s, const int32_t* ids, uint32_t experts, uint32_t pairs,
                                              uint32_t top_k, int32_t* expert_off, int32_t* sorted_pair, int32_t* sorted_tok,
                                              int32_t* inv_perm, int32_t* tile_e, int32_t* tile_r, int32_t* tile_count,
                                              uint32_t compact_tail) {
    QWHIP_REQUIRE(s);
    QWHIP_REQUIRE(ids);
    QWHIP_REQUIRE(expert_off);
    QWHIP_REQUIRE(sorted_pair);
    QWHIP_REQUIRE(sorted_tok);
    if (experts == 0 || experts > 512)
        return qwhip_fail(QWHIP_E_BAD_SHAPE, "the expert-sorted pair order holds 512 experts, got %u", experts);
    if (top_k == 0) return qwhip_fail(QWHIP_E_BAD_SHAPE, "moe group pairs: top_k must be positive");
    const bool tiles = tile_e || tile_r || tile_count;
    if (tiles && !(tile_e && tile_r && tile_count))
        return qwhip_fail(QWHIP_E_BAD_SHAPE, "moe group pairs: tile_e, tile_r and tile_count come together");
    // up to 24,576 pairs the sorted list is staged in LDS (96 KB beside the 38 KB of counters)
    const uint32_t stage = pairs <= 24576u ? 1u : 0u;
    const size_t lds = stage ? (size_t)pairs * 4u : 0u;
    static std::atomic<bool> attr_done{false};
    if (!attr_done.load(std::memory_order_acquire)) {
        QWHIP_TRY_HIP(hipFuncSetAttribute((const void*)qw_moe_group_pairs_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, 96 * 1024));
        attr_done.store(true, std::memory_order_release);
    }
    hipLaunchKernelGGL(qw_moe_group_pairs_kernel, dim3(1), dim3(1024), lds, s->stream, ids, experts, pairs, top_k, expert_off,
                       sorted_pair, sorted_tok, inv_perm, tile_e, tile_r, tile_count, compact_tail ? 1u : 0u, stage);
    QWHIP_TRY_HIP(hipGetLastError());
    return QWHIP_OK;
}

// ------------------------------------------------------------------------------------------------
// Combine: out[t, h] = sum_k wts[t, k] * dn[inv_perm[t*K + k], h] (+ shared_gate[t] * shared[t, h]).
// One thread per 4 consecutive h; fp32 accumulation in rank order.
// ------------------------------------------------------------------------------------------------
template <int DDT, int ODT, int KMAX>   // KMAX: unrolled route slots of the vector path (8 or 16)
__global__ __launch_bounds__(256) void qw_moe_combine_kernel(const void* __restrict__ dn, const int32_t* __restrict__ inv_perm,
                                                              const float* __restrict__ wts, uint32_t T, uint32_t K, uint32_t H,
                                                              const float* __restrict__ shared, const float* __restrict__ shared_gate,
                                                              void* __restrict__ out) {
    const uint32_t t = blockIdx.y;
    const uint32_t h = (blockIdx.x * 256 + threadIdx.x) * 4;
    if (h >= H) return;
    float acc[4] = {0.f, 0.f, 0.f, 0.f};
    if (K <= (uint32_t)KMAX && (H & 3u) == 0u) {
        // every route's slot and weight first, then all the rows' four columns as one load each: the loads of a thread
        // are independent of each other, only the additions keep the rank order
        int32_t slot[KMAX];
        float w[KMAX];
#pragma unroll
        for (uint32_t k = 0; k < (uint32_t)KMAX; ++k) {
            slot[k] = k < K ? (inv_perm ? inv_perm[(uint64_t)t * K + k] : (int32_t)(t * K + k)) : -1;
            w[k] = k < K ? (wts ? wts[(uint64_t)t * K + k] : 1.0f) : 0.0f;
        }
        float v[KMAX][4];
#pragma unroll
        for (uint32_t k = 0; k < (uint32_t)KMAX; ++k) {
            const uint64_t at = (uint64_t)(slot[k] < 0 ? 0 : slot[k]) * H + h;   // an empty route reads row 0 and is not added
            if constexpr (DDT == QWHIP_F32) {
                const f4_t x = *(const f4_t*)((const float*)dn + at);
#pragma unroll
                for (int j = 0; j < 4; ++j) v[k][j] = x[j];
            } else {
                const u2_t x = *(const u2_t*)((const uint16_t*)dn + at);
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const uint16_t b = (uint16_t)(x[j >> 1] >> (16 * (j & 1)));
                    v[k][j] = DDT == QWHIP_F16 ? (float)__builtin_bit_cast(h1_t, b) : qw_bf16_to_f32(b);
                }
            }
        }
#pragma unroll
        for (uint32_t k = 0; k < (uint32_t)KMAX; ++k) {
            if (slot[k] >= 0) {
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[j] = fmaf(w[k], v[k][j], acc[j]);
            }
        }
    } else
    for (uint32_t k = 0; k < K; ++k) {
        const int32_t slot = inv_perm ? inv_perm[(uint64_t)t * K + k] : (int32_t)(t * K + k);
        if (slot < 0) continue;
        const float w = wts ? wts[(uint64_t)t * K + k] : 1.0f;
#pragma unroll
        for (int j = 0; j < 4; ++j)
            if (h + j < H) acc[j] = fmaf(w, qw_load_f32<DDT>(dn, (uint64_t)slot * H + h + j), acc[j]);
    }
    if (shared) {
        const float g = shared_gate ? shared_gate[t] : 1.0f;
#pragma unroll
        for (int j = 0; j < 4; ++j)
            if (h + j < H) acc[j] = fmaf(g, shared[(uint64_t)t * H + h + j], acc[j]);
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        if (h + j < H) {
            const uint64_t o = (uint64_t)t * H + h + j;
            if constexpr (ODT == QWHIP_F32) ((float*)out)[o] = acc[j];
            else if constexpr (ODT == QWHIP_F16) ((h1_t*)out)[o] = (h1_t)acc[j];
            else ((uint16_t*)out)[o] = qw_f32_to_bf16(acc[j]);
        }
    }
}

extern "C" qwhip_status qwhip_moe_combine(qwhip_stream_t s, const void* dn, uint32_t dn_dtype, const int32_t* inv_perm,
                                          const float* wts, uint32_t t, uint32_t top_k, uint32_t hidden, const float* shared,
                                          const float* shared_gate, void* out, uint32_t out_dtype) {
    QWHIP_REQUIRE(s);
    if (t == 0 || hidden == 0) return QWHIP_OK;
    QWHIP_REQUIRE(dn);
    QWHIP_REQUIRE(out);
    if ((uint64_t)t * top_k >= (1ull << 31)) return qwhip_fail(QWHIP_E_BAD_SHAPE, "moe combine: %u x %u route slots", t, top_k);
    const dim3 grid(qwhip_cdiv(hidden, 1024), t), block(256);
#define QW_CB(DD, OD)                                                                                                          \
    do {                                                                                                                       \
        if (top_k <= 8) hipLaunchKernelGGL((qw_moe_combine_kernel<DD, OD, 8>), grid, block, 0, s->stream, dn, inv_perm, wts, t, \
                                           top_k, hidden, shared, shared_gate, out);                                           \
        else hipLaunchKernelGGL((qw_moe_combine_kernel<DD, OD, 16>), grid, block, 0, s->stream, dn, inv_perm, wts, t, top_k,    \
                                hidden, shared, shared_gate, out);                                                             \
    } while (0)
#define QW_CB_O(DD)                                                   \
    switch (out_dtype) {                                              \
        case QWHIP_F32: QW_CB(DD, QWHIP_F32); break;                  \
        case QWHIP_F16: QW_CB(DD, QWHIP_F16); break;                  \
        case QWHIP_BF16: QW_CB(DD, QWHIP_BF16); break;                \
        default: return qwhip_fail(QWHIP_E_BAD_SHAPE, "moe combine: unsupported output dtype %u", out_dtype); \
    }
    switch (dn_dtype) {
        case QWHIP_F32: QW_CB_O(QWHIP_F32) break;
        case QWHIP_F16: QW_CB_O(QWHIP_F16) break;
        case QWHIP_BF16: QW_CB_O(QWHIP_BF16) break;
        default: return qwhip_fail(QWHIP_E_BAD_SHAPE, "moe combine: unsupported input dtype %u", dn_dtype);
    }
#undef QW_CB_O
#undef QW_CB
    QWHIP_TRY_HIP(hipGetLastError());
    return QWHIP_OK;
}

// ------------------------------------------------------------------------------------------------
// Group-latent MoE (QWMoEOperator.encodeResidentGroupLatent, Sources/Operators/QWGEMM/QWMoEOperator+GroupLatent.swift:11-294):
// every expert carries the label of one of num_groups latent groups; a token's routes go through the down-projection D_g of
// their expert's group, the expert in the latent width, and the up-projection U_g of the sum of the group's routes.
// ------------------------------------------------------------------------------------------------

// group_ids[t, g] = g when one of the token's routes falls into group g, else -1 (the rule of qwg_moe_route with
// latentLabels, Sources/QWMetal/subsystems/qwrouter.metal:135-165); pair_rows[t, k] = t * num_groups + label of route k
// (the row of the route's latent among the [t, num_groups] rows), -1 for an absent route.
__global__ __launch_bounds__(256) void qw_moe_latent_groups_kernel(const int32_t* __restrict__ idx, const int32_t* __restrict__ labels,
                                                                    uint32_t T, uint32_t K, uint32_t E, uint32_t NG,
                                                                    int32_t* __restrict__ group_ids, int32_t* __restrict__ pair_rows) {
    const uint32_t t = blockIdx.x * 256u + threadIdx.x;
    if (t >= T) return;
    uint32_t mask = 0;
    for (uint32_t k = 0; k < K; ++k) {
        const int32_t raw = idx[(uint64_t)t * K + k];
        int32_t row = -1;
        if (raw >= 0 && ((uint32_t)raw & 0xFFFFu) < E) {
            const int32_t g = labels[(uint32_t)raw & 0xFFFFu];
            if (g >= 0 && (uint32_t)g < NG) {
                mask |= 1u << g;
                row = (int32_t)(t * NG + (uint32_t)g);
            }
        }
        if (pair_rows) pair_rows[(uint64_t)t * K + k] = row;
    }
    for (uint32_t g = 0; g < NG; ++g) group_ids[(uint64_t)t * NG + g] = (mask >> g) & 1u ? (int32_t)g : -1;
}

extern "C" qwhip_status qwhip_moe_latent_groups(qwhip_stream_t s, const int32_t* idx, const int32_t* labels, uint32_t t, uint32_t top_k,
                                                uint32_t experts, uint32_t num_groups, int32_t* group_ids, int32_t* pair_rows) {
    QWHIP_REQUIRE(s);
    if (t == 0) return QWHIP_OK;
    QWHIP_REQUIRE(idx);
    QWHIP_REQUIRE(labels);
    QWHIP_REQUIRE(group_ids);
    if (num_groups == 0 || num_groups > 32u) return qwhip_fail(QWHIP_E_BAD_SHAPE, "latent groups must be 1..32, got %u", num_groups);
    if (top_k == 0 || experts == 0 || experts > 65535u) return qwhip_fail(QWHIP_E_BAD_SHAPE, "latent groups: top_k %u, experts %u", top_k, experts);
    if ((uint64_t)t * max(top_k, num_groups) >= (1ull << 31)) return qwhip_fail(QWHIP_E_BAD_SHAPE, "latent groups: %u tokens", t);
    hipLaunchKernelGGL(qw_moe_latent_groups_kernel, dim3(qwhip_cdiv(t, 256u)), dim3(256), 0, s->stream, idx, labels, t, top_k, experts,
                       num_groups, group_ids, pair_rows);
    QWHIP_TRY_HIP(hipGetLastError());
    return QWHIP_OK;
}

// rows_out[p] = slot_of_row[pair_rows[sorted_pair[p]]]: the gather row of sorted position p when the routes' activations
// are themselves the output of an earlier grouped GEMM (slot_of_row = that sort's inverse permutation).  Positions whose
// chain breaks (nothing sorted there, absent route, absent group) read row 0 and are never used.
__global__ __launch_bounds__(256) void qw_moe_compose_rows_kernel(const int32_t* __restrict__ sorted_pair, uint32_t n,
                                                                   const int32_t* __restrict__ pair_rows, uint32_t n_rows,
                                                                   const int32_t* __restrict__ slot_of_row, int32_t* __restrict__ rows_out) {
    const uint32_t p = blockIdx.x * 256u + threadIdx.x;
    if (p >= n) return;
    int32_t r = 0;
    const int32_t sp = sorted_pair[p];
    if (sp >= 0 && (uint32_t)sp < n) {
        const int32_t pr = pair_rows[sp];
        if (pr >= 0 && (uint32_t)pr < n_rows) r = slot_of_row ? max(slot_of_row[pr], 0) : pr;
    }
    rows_out[p] = r;
}

extern "C" qwhip_status qwhip_moe_compose_rows(qwhip_stream_t s, const int32_t* sorted_pair, uint32_t pairs, const int32_t* pair_rows,
                                               uint32_t n_rows, const int32_t* slot_of_row, int32_t* rows_out) {
    QWHIP_REQUIRE(s);
    if (pairs == 0) return QWHIP_OK;
    QWHIP_REQUIRE(sorted_pair);
    QWHIP_REQUIRE(pair_rows);
    QWHIP_REQUIRE(rows_out);
    if (pairs >= (1u << 31) || n_rows >= (1u << 31)) return qwhip_fail(QWHIP_E_BAD_SHAPE, "compose rows: %u pairs, %u rows", pairs, n_rows);
    hipLaunchKernelGGL(qw_moe_compose_rows_kernel, dim3(qwhip_cdiv(pairs, 256u)), dim3(256), 0, s->stream, sorted_pair, pairs, pair_rows,
                       n_rows, slot_of_row, rows_out);
    QWHIP_TRY_HIP(hipGetLastError());
    return QWHIP_OK;
}

// out[t * NG + g, :] = sum over the routes k of token t with labels[idx[t, k]] == g of wts[t, k] * dn[inv_perm[t * K + k], :]
// in rank order, zeros for a group without routes (the numGroups mode of qwg_moe_down_reduce_combine_f32,
// Sources/QWMetal/gemm/qwgemm_moe_nax_f16.metal:51-111).  One thread per 4 columns.
template <int DDT, int ODT>
__global__ __launch_bounds__(256) void qw_moe_combine_groups_kernel(const void* __restrict__ dn, const int32_t* __restrict__ inv_perm,
                                                                     const float* __restrict__ wts, const int32_t* __restrict__ idx,
                                                                     const int32_t* __restrict__ labels, uint32_t E, uint32_t K, uint32_t NG,
                                                                     uint32_t W, void* __restrict__ out) {
    const uint32_t row = blockIdx.y, t = row / NG;
    const int32_t g = (int32_t)(row - t * NG);
    const uint32_t c = (blockIdx.x * 256u + threadIdx.x) * 4u;
    if (c >= W) return;
    float acc[4] = {0.f, 0.f, 0.f, 0.f};
    for (uint32_t k = 0; k < K; ++k) {
        const int32_t e = idx[(uint64_t)t * K + k];
        if (e < 0 || ((uint32_t)e & 0xFFFFu) >= E || labels[(uint32_t)e & 0xFFFFu] != g) continue;   // an id past the labels is no route
        const int32_t slot = inv_perm ? inv_perm[(uint64_t)t * K + k] : (int32_t)(t * K + k);
        if (slot < 0) continue;
        const float w = wts ? wts[(uint64_t)t * K + k] : 1.0f;
#pragma unroll
        for (int j = 0; j < 4; ++j)
            if (c + j < W) acc[j] = fmaf(w, qw_load_f32<DDT>(dn, (uint64_t)slot * W + c + j), acc[j]);
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        if (c + j < W) {
            const uint64_t o = (uint64_t)row * W + c + j;
            if constexpr (ODT == QWHIP_F32) ((float*)out)[o] = acc[j];
            else if constexpr (ODT == QWHIP_F16) ((h1_t*)out)[o] = (h1_t)acc[j];
            else ((uint16_t*)out)[o] = qw_f32_to_bf16(acc[j]);
        }
    }
}

extern "C" qwhip_status qwhip_moe_combine_groups(qwhip_stream_t s, const void* dn, uint32_t dn_dtype, const int32_t* inv_perm,
                                                 const float* wts, const int32_t* idx, const int32_t* labels, uint32_t experts, uint32_t t,
                                                 uint32_t top_k, uint32_t num_groups, uint32_t width, void* out, uint32_t out_dtype) {
    QWHIP_REQUIRE(s);
    if (t == 0 || width == 0) return QWHIP_OK;
    QWHIP_REQUIRE(dn);
    QWHIP_REQUIRE(idx);
    QWHIP_REQUIRE(labels);
    QWHIP_REQUIRE(out);
    if (num_groups == 0 || num_groups > 32u) return qwhip_fail(QWHIP_E_BAD_SHAPE, "latent groups must be 1..32, got %u", num_groups);
    if (experts == 0 || experts > 65535u) return qwhip_fail(QWHIP_E_BAD_SHAPE, "moe combine by groups: labels for 1..65535 experts, got %u", experts);
    if ((uint64_t)t * num_groups >= (1ull << 31) || (uint64_t)t * top_k >= (1ull << 31))
        return qwhip_fail(QWHIP_E_BAD_SHAPE, "moe combine by groups: %u tokens", t);
    // grid.y holds 65535 rows: more (token, group) rows go in slabs of whole tokens
    const uint32_t tok_per = 65535u / num_groups;
    for (uint32_t t0 = 0; t0 < t; t0 += tok_per) {
        const uint32_t tt = min(tok_per, t - t0);
        const dim3 grid(qwhip_cdiv(width, 1024), tt * num_groups), block(256);
        const int32_t* ip = inv_perm ? inv_perm + (uint64_t)t0 * top_k : nullptr;
        const float* wp = wts ? wts + (uint64_t)t0 * top_k : nullptr;
        const int32_t* xp = idx + (uint64_t)t0 * top_k;
        const uint64_t orow = (uint64_t)t0 * num_groups * width;
        void* op = (uint8_t*)out + orow * (out_dtype == QWHIP_F32 ? 4u : 2u);
        // identity slots count from the slab's first token: shift the dn base instead
        const void* dp = inv_perm ? dn : (const void*)((const uint8_t*)dn + (uint64_t)t0 * top_k * width * (dn_dtype == QWHIP_F32 ? 4u : 2u));
#define QW_CG(DD, OD) hipLaunchKernelGGL((qw_moe_combine_groups_kernel<DD, OD>), grid, block, 0, s->stream, dp, ip, wp, xp, labels, experts, top_k, num_groups, width, op)
#define QW_CG_O(DD)                                                   \
        switch (out_dtype) {                                          \
            case QWHIP_F32: QW_CG(DD, QWHIP_F32); break;              \
            case QWHIP_F16: QW_CG(DD, QWHIP_F16); break;              \
            case QWHIP_BF16: QW_CG(DD, QWHIP_BF16); break;            \
            default: return qwhip_fail(QWHIP_E_BAD_SHAPE, "moe combine by groups: unsupported output dtype %u", out_dtype); \
        }
        switch (dn_dtype) {
            case QWHIP_F32: QW_CG_O(QWHIP_F32) break;
            case QWHIP_F16: QW_CG_O(QWHIP_F16) break;
            case QWHIP_BF16: QW_CG_O(QWHIP_BF16) break;
            default: return qwhip_fail(QWHIP_E_BAD_SHAPE, "moe combine by groups: unsupported input dtype %u", dn_dtype);
        }
#undef QW_CG_O
#undef QW_CG
        QWHIP_TRY_HIP(hipGetLastError());
    }
    return QWHIP_OK;
}

// ------------------------------------------------------------------------------------------------
// Expert budget over a verify window (the normTopK & 4 branch of qwg_moe_route_decode,
// Sources/QWMetal/subsystems/qwrouter.metal:193-268; door: encodeFnMoeRoute(expertBudget:), QWGemmMoERouter.swift:63-75):
// after the routing of 2..4 rows, at most `budget` distinct experts stay.  Row 0 keeps its routes; the other pairs are
// admitted expert by expert in the order of their weights (ties: the lower pair index) until `budget` distinct experts are in;
// the rest lose their route (idx -1, weight 0), and with `norm` every later row that lost weight is rescaled to its old sum.
// One wavefront, lane p = pair p (rows * top_k <= 64).
// ------------------------------------------------------------------------------------------------
__global__ __launch_bounds__(64) void qw_moe_route_budget_kernel(int32_t* __restrict__ idx, float* __restrict__ wts, uint32_t M, uint32_t K,
                                                                  uint32_t B, uint32_t norm) {
    __shared__ int32_t ids[64];
    __shared__ float ws[64];
    const uint32_t lane = threadIdx.x, total = M * K;
    const int32_t id = lane < total ? idx[lane] : -1;
    const float w = lane < total ? wts[lane] : -1.0f;
    ids[lane] = id;
    ws[lane] = w;
    __syncthreads();
    float orig = 0.0f;   // lane r < M: the row's weight sum before pruning, added in route order
    if (norm && lane < M)
        for (uint32_t k = 0; k < K; ++k) orig += ws[lane * K + k];
    bool keep = lane < K;
    uint32_t unique = 0;
    for (uint32_t s = 0; s < K; ++s) {   // uniform over the wave
        const int32_t e = ids[s];
        if (e < 0) continue;
        bool dup = false;
        for (uint32_t prev = 0; prev < s; ++prev) dup = dup || ids[prev] == e;
        if (!dup) {
            ++unique;
            if (id == e) keep = true;
        }
    }
    while (unique < B) {
        const float cand = (!keep && id >= 0) ? w : -1.0f;
        float best = cand;
#pragma unroll
        for (int d = 32; d >= 1; d >>= 1) best = fmaxf(best, __shfl_xor(best, d, 64));
        if (best < 0.0f) break;
        const unsigned long long hit = __ballot(cand == best);
        const uint32_t win = (uint32_t)__builtin_ctzll(hit);
        if (win >= total) break;
        const int32_t we = ids[win];
        if (id == we) keep = true;
        ++unique;
    }
    const bool pruned = lane < total && !keep;
    if (pruned) {
        idx[lane] = -1;
        wts[lane] = 0.0f;
    }
    __syncthreads();
    ws[lane] = pruned ? 0.0f : w;
    __syncthreads();
    if (norm && lane >= 1u && lane < M) {
        float now = 0.0f;
        for (uint32_t k = 0; k < K; ++k) {
            const float v = ws[lane * K + k];
            if (v > 0.0f) now += v;
        }
        if (now > 0.0f && now < orig * 0.9999f) {
            const float scale = orig / now;
            for (uint32_t k = 0; k < K; ++k) wts[lane * K + k] = ws[lane * K + k] * scale;
        }
    }
}

extern "C" qwhip_status qwhip_moe_route_budget(qwhip_stream_t s, int32_t* idx, float* wts, uint32_t rows, uint32_t top_k, uint32_t budget,
                                               uint32_t norm_topk) {
    QWHIP_REQUIRE(s);
    QWHIP_REQUIRE(idx);
    QWHIP_REQUIRE(wts);
    if (rows < 2u || rows > 4u || top_k == 0 || top_k > 16u || rows * top_k > 64u)
        return qwhip_fail(QWHIP_E_BAD_SHAPE, "expert budget: a window of 2..4 rows of at most 16 routes (rows=%u top_k=%u)", rows, top_k);
    if (budget == 0 || budget >= rows * top_k) return QWHIP_OK;   // nothing to prune
    hipLaunchKernelGGL(qw_moe_route_budget_kernel, dim3(1), dim3(64), 0, s->stream, idx, wts, rows, top_k, max(top_k, budget), norm_topk ? 1u : 0u);
    QWHIP_TRY_HIP(hipGetLastError());
    return QWHIP_OK;
}
