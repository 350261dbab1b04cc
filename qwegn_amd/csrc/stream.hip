// Streaming small-M kernel: y[m, n] = sum_k W[n, k] * x[m, k] for m = 1..16 over any bit-stream / HQ4 container,
// built for the HBM roofline:
//
//   * weights travel global -> LDS on the DMA path (global_load_lds_dwordx4): perfectly coalesced 1 KB wave
//     requests, no VGPRs held while in flight, two stages per wave so the next step streams while this one is
//     contracted.  A step is 16 weight rows x 16 (or 32) 32-column slices of packed blocks, laid out in LDS row by
//     row with an odd pitch in 16-byte slots (unused lanes of the DMA leave the hole), so the per-lane 32-bit
//     reads of 16 rows x 4 slices land on 64 distinct banks;
//   * lane (i, c) = (lane & 15, lane >> 4) owns slice 4*ls + c of row i, dequantizes it to four 8-wide exact-f16
//     MFMA A operands (one header splat per 32 weights), and v_mfma_f32_16x16x32_f16 contracts against the m
//     activation rows (B operand, column j = m);
//   * activations: either the whole rotated [m, k] block lives in LDS (prologue; rotation on the matrix cores), or
//     each step's [m, 512] panel is DMA-staged once per workgroup and shared by its 4 row tiles (m up to 16 without
//     multiplying L2 traffic);
//   * the 4 waves of a workgroup are RW row tiles x KW K-splits (RW*KW = 4); K-splits reduce through LDS.
#include <atomic>

#include "qwhip_common.h"

namespace {

enum { QS_X_FULL = 0, QS_X_STAGED = 1 };

struct qs_params {
    const uint8_t* bank;
    const void* x;
    h1_t* y16;
    float* y32;
    uint32_t N, K, M;
    uint32_t row_bytes;
    uint32_t rotate;
};

template <int BITS, int GROUP>
struct qs_geom {
    static constexpr int BB = 4 + GROUP * BITS / 8;        // block bytes
    static constexpr int SPS = GROUP <= 64 ? 8 : (GROUP == 128 ? 16 : 32);  // 32-column slices per step (>= 4 blocks)
    static constexpr int SPB = GROUP / 32;                 // slices per block
    static constexpr int BPS = SPS / SPB;                  // blocks per row and step
    static constexpr int SB = BPS * BB;                    // bytes per row and step
    static_assert(SB % 16 == 0, "a step must be whole 16-byte pieces");
    static constexpr int PIECES = SB / 16;
    static constexpr int P16 = PIECES | 1;                 // pitch in 16-byte slots, odd
    static constexpr int NI = (16 * P16 + 63) / 64;        // DMA instructions per wave and step
    static constexpr int WSTAGE = NI * 1024;               // bytes per wave and stage
    static constexpr int XCOLS = SPS * 32;
    static constexpr int XP16 = (XCOLS * 2 / 16) | 1;      // staged activation row pitch in slots, odd
};

// natural-order dequant of 8 consecutive columns (chunk j of a slice) into exact f16 weights
template <int BITS, bool M5>
__device__ __forceinline__ h8_t qs_dequant(const uint32_t* q, int j, h2_t s2, h2_t b2, uint32_t magic) {
    h2_t w[4];
    if constexpr (M5) {
        qw_unpack_hq4_word(q[j], s2, b2, magic, w);
    } else if constexpr (BITS == 4) {
        const h2_t neg = {(h1_t)-1024.0f, (h1_t)-1024.0f};
        const uint32_t lo = q[j] & 0x0F0F0F0Fu, hi = (q[j] >> 4) & 0x0F0F0F0Fu;
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const uint32_t sel = 0x0C000C00u | (uint32_t)k | ((uint32_t)(4 + k) << 16);
            const uint32_t m = __builtin_amdgcn_perm(hi, lo, sel) | magic;
            w[k] = __builtin_elementwise_fma(__builtin_bit_cast(h2_t, m) + neg, s2, b2);
        }
    } else {
        const h2_t neg = {(h1_t)-1024.0f, (h1_t)-1024.0f};
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const uint32_t v = q[2 * j + h];
            const uint32_t m0 = __builtin_amdgcn_perm(v, v, 0x0C010C00u) | magic;
            const uint32_t m1 = __builtin_amdgcn_perm(v, v, 0x0C030C02u) | magic;
            w[2 * h] = __builtin_elementwise_fma(__builtin_bit_cast(h2_t, m0) + neg, s2, b2);
            w[2 * h + 1] = __builtin_elementwise_fma(__builtin_bit_cast(h2_t, m1) + neg, s2, b2);
        }
    }
    h8_t a = {w[0][0], w[0][1], w[1][0], w[1][1], w[2][0], w[2][1], w[3][0], w[3][1]};
    return a;
}

// H[i][8c + e], e = 0..7 of the 32-point Hadamard matrix as f16 +-1
__device__ __forceinline__ h8_t qs_hadamard_rows(uint32_t i, uint32_t c) {
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

template <int XDT>
__device__ __forceinline__ h8_t qs_load_x8(const void* x, uint64_t elem) {
    if constexpr (XDT == QWHIP_F16) {
        return *(const h8_t*)((const h1_t*)x + elem);
    } else {
        const u4_t raw = *(const u4_t*)((const uint16_t*)x + elem);
        h8_t o;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            o[2 * j] = (h1_t)__uint_as_float(raw[j] << 16);
            o[2 * j + 1] = (h1_t)__uint_as_float(raw[j] & 0xFFFF0000u);
        }
        return o;
    }
}

// PF = prefetch distance in steps.  Weight stages are wave-private (ring of PF + 1); the staged-activation ring is
// shared by the workgroup and holds PF + 2 stages so that the stage a DMA overwrites was last read two barriers ago.
template <int BITS, int GROUP, bool M5, int KW, int XMODE, int XDT, int PF>
__global__ __launch_bounds__(256) void qw_stream_kernel(const qs_params p) {
    using G = qs_geom<BITS, GROUP>;
    constexpr int RW = 4 / KW;
    constexpr int NQ = BITS == 8 ? 8 : 4;  // payload words per slice
    constexpr int WS = PF + 1;             // weight stages per wave
    constexpr int XS = PF + 2;             // staged-activation stages per workgroup
    constexpr uint32_t XSLOTS = 16u * G::XP16;
    constexpr int XNI = (XSLOTS + 255u) / 256u;          // activation DMA instructions per thread and step
    constexpr uint32_t XSTAGE = XNI * 256u * 16u;
    constexpr int PER = G::NI + (XMODE == QS_X_STAGED ? XNI : 0);  // DMA instructions per wave and step: exact, never skipped
    static_assert(PF * PER <= 63, "vmcnt holds 6 bits");
    extern __shared__ __attribute__((aligned(16))) uint8_t qs_lds[];
    __shared__ f4_t red[4][64];

    const uint32_t tid = threadIdx.x;
    const uint32_t wave = tid >> 6, lane = tid & 63u;
    const uint32_t i = lane & 15u, c = lane >> 4;
    const uint32_t rt = wave / KW, ks = wave % KW;
    const uint32_t N = p.N, K = p.K, M = p.M;
    const uint32_t nsl = K >> 5;
    const uint32_t nsteps = (nsl + G::SPS - 1) / G::SPS;
    const uint32_t n0 = (blockIdx.x * RW + rt) * 16u;

    // LDS carve-up: [4 waves x WS stages of weights][activations]
    uint8_t* wst = qs_lds + wave * WS * G::WSTAGE;
    uint8_t* xls = qs_lds + 4 * WS * G::WSTAGE;
    const uint32_t xfull_pitch = nsl * 80u + 16u;  // QS_X_FULL: bytes per activation row (80-byte pitch per 32-group)

    // ---- per-lane DMA sources of the weight stage: slot = inst*64 + lane -> (row, piece).  Every lane of every
    // instruction loads something (lanes without a piece re-read the start of the bank into a slot nobody reads):
    // no instruction is ever skipped, so the vmcnt arithmetic below is exact.
    uint32_t w_off[G::NI], w_po[G::NI];
    {
        const uint32_t row_lim = N > n0 ? min(16u, N - n0) : 0u;
#pragma unroll
        for (int q = 0; q < G::NI; ++q) {
            const uint32_t slot = q * 64u + lane;
            const uint32_t row = slot / G::P16, piece = slot - row * G::P16;
            const bool ok = row < row_lim && piece < (uint32_t)G::PIECES;
            w_po[q] = ok ? piece * 16u : 0xFFFFFFFFu;
            w_off[q] = ok ? (n0 + row) * p.row_bytes + piece * 16u : 0u;  // row_bytes * N < 2^32 is checked by the launcher
        }
    }
    auto dma_w = [&](uint32_t step, uint32_t stage) {
        const uint32_t soff = step * (uint32_t)G::SB;
#pragma unroll
        for (int q = 0; q < G::NI; ++q) {
            // pieces past the end of the row (ragged last step) fall back to the dummy source; their slices are masked below
            const bool ok = w_po[q] != 0xFFFFFFFFu && soff + w_po[q] + 16u <= p.row_bytes;
            const uint8_t* src = p.bank + (ok ? w_off[q] + soff : 0u);
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)src,
                                             (__attribute__((address_space(3))) void*)(wst + stage * G::WSTAGE + q * 1024), 16, 0, 0);
        }
    };
    // staged activations: [M rows][XCOLS] f16 per step, DMA'd by all 256 threads (row pitch XP16 slots)
    auto dma_x = [&](uint32_t step, uint32_t stage) {
#pragma unroll
        for (int q = 0; q < XNI; ++q) {
            const uint32_t slot = q * 256u + tid;
            const uint32_t m = slot / G::XP16, piece = slot - m * G::XP16;
            const uint32_t col = step * G::XCOLS + piece * 8u;
            const bool ok = m < M && piece < (uint32_t)(G::XCOLS / 8) && col < K;
            const h1_t* src = (const h1_t*)p.x + (ok ? (uint64_t)m * K + col : 0u);
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)src,
                                             (__attribute__((address_space(3))) void*)(xls + stage * XSTAGE + (q * 256u + wave * 64u) * 16u), 16, 0, 0);
        }
    };

    // ---- this wave's steps ----
    const uint32_t per = (nsteps + KW - 1) / KW;
    const uint32_t s0 = min(ks * per, nsteps), s1 = min(s0 + per, nsteps);

    // ---- pipeline fill: steps s0 .. s0 + PF - 1 ----
#pragma unroll
    for (int f = 0; f < PF; ++f) {
        if (s0 + f < s1) {
            dma_w(s0 + f, f % WS);
            if constexpr (XMODE == QS_X_STAGED) dma_x(s0 + f, f % XS);
        }
    }

    if constexpr (XMODE == QS_X_FULL) {
        // whole activation block into LDS, rotated on the matrix cores when asked (16 groups per MFMA pair)
        const h8_t h_lo = qs_hadamard_rows(i, c), h_hi = qs_hadamard_rows(i + 16u, c);
        const uint32_t ngt = (nsl + 15u) >> 4;
        for (uint32_t t = wave; t < M * ngt; t += 4) {
            const uint32_t m = t / ngt, gt = t - m * ngt;
            const uint32_t g = min(gt * 16u + i, nsl - 1);
            const h8_t xb = qs_load_x8<XDT>(p.x, (uint64_t)m * K + (uint64_t)g * 32u + 8u * c);
            h1_t* dst = (h1_t*)(xls + m * xfull_pitch) + (uint64_t)(gt * 16u + i) * 40u;
            if (p.rotate) {
                f4_t d0 = {0.f, 0.f, 0.f, 0.f}, d1 = {0.f, 0.f, 0.f, 0.f};
                d0 = __builtin_amdgcn_mfma_f32_16x16x32_f16(h_lo, xb, d0, 0, 0, 0);
                d1 = __builtin_amdgcn_mfma_f32_16x16x32_f16(h_hi, xb, d1, 0, 0, 0);
                if (gt * 16u + i < nsl) {
                    h4_t o0, o1;
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        o0[r] = (h1_t)(d0[r] * QW_INV_SQRT32);
                        o1[r] = (h1_t)(d1[r] * QW_INV_SQRT32);
                    }
                    *(h4_t*)(dst + 4u * c) = o0;
                    *(h4_t*)(dst + 16u + 4u * c) = o1;
                }
            } else if (gt * 16u + i < nsl) {
                *(h8_t*)(dst + 8u * c) = xb;
            }
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
    }

    const uint32_t magic = qw_vgpr_const(0x64006400u);
    f4_t acc = {0.f, 0.f, 0.f, 0.f};
    const uint32_t wrow = i * (uint32_t)G::P16 * 16u;  // this lane's row inside a weight stage

    for (uint32_t step = s0; step < s1; ++step) {
        const uint32_t rel = step - s0;
        if (step + PF < s1) {
            dma_w(step + PF, (rel + PF) % WS);
            if constexpr (XMODE == QS_X_STAGED) dma_x(step + PF, (rel + PF) % XS);
            asm volatile("s_waitcnt vmcnt(%0)" ::"n"(PF * PER) : "memory");   // everything but the PF newest steps has landed
        } else {
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        }
        if constexpr (XMODE == QS_X_STAGED) __syncthreads();                    // the shared activation stage is complete
        const uint8_t* ws = wst + (rel % WS) * G::WSTAGE + wrow;
        const uint8_t* xs_stage = xls + (rel % XS) * XSTAGE;
#pragma unroll
        for (int ls = 0; ls < G::SPS / 4; ++ls) {
            const uint32_t s = 4u * ls + c;                 // slice inside the step
            const uint32_t gs = step * G::SPS + s;          // slice inside the row
            const bool valid = gs < nsl;
            const uint32_t boff = (s / G::SPB) * (uint32_t)G::BB;
            const uint32_t* wp = (const uint32_t*)(ws + boff);
            uint32_t hdr = wp[0];
            uint32_t q[NQ];
#pragma unroll
            for (int u = 0; u < NQ; ++u) q[u] = wp[1 + (s % G::SPB) * NQ + u];
            if (!valid) {
                hdr = 0;
#pragma unroll
                for (int u = 0; u < NQ; ++u) q[u] = 0;
            }
            h8_t xop[4];
            if (valid && i < M) {
                const h8_t* xp;
                if constexpr (XMODE == QS_X_STAGED) xp = (const h8_t*)(xs_stage + i * (uint32_t)G::XP16 * 16u + s * 64u);
                else xp = (const h8_t*)(xls + i * xfull_pitch + gs * 80u);
#pragma unroll
                for (int j = 0; j < 4; ++j) xop[j] = xp[j];
            } else {
#pragma unroll
                for (int j = 0; j < 4; ++j) xop[j] = h8_t{0, 0, 0, 0, 0, 0, 0, 0};
            }
            const h2_t s2 = qw_splat_lo(hdr), b2 = qw_splat_hi(hdr);
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const h8_t a = qs_dequant<BITS, M5>(q, j, s2, b2, magic);
                acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, xop[j], acc, 0, 0, 0);
            }
        }
    }

    // ---- K-split reduction and store: lane (j = m, c) holds rows n0 + 4c + r ----
    if constexpr (KW > 1) {
        red[wave][lane] = acc;
        __syncthreads();
        if (ks != 0) return;
        acc = red[wave][lane];
#pragma unroll
        for (int k2 = 1; k2 < KW; ++k2) acc += red[wave + k2][lane];
    }
    if (i < M) {
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const uint32_t n = n0 + 4u * c + r;
            if (n < N) {
                if (p.y32) p.y32[(uint64_t)i * N + n] = acc[r];
                if (p.y16) p.y16[(uint64_t)i * N + n] = (h1_t)acc[r];
            }
        }
    }
}

template <int BITS, int GROUP, bool M5>
hipError_t qs_launch_fmt(hipStream_t st, const qs_params& p, int kw, int xmode, uint32_t xdt, int pf, size_t lds) {
    const uint32_t rw = 4u / (uint32_t)kw;
    const dim3 grid(qwhip_cdiv(p.N, 16u * rw)), block(256);
#define QS_GO(KWV, XM, DT, PFV)                                                                                    \
    do {                                                                                                            \
        auto kern = qw_stream_kernel<BITS, GROUP, M5, KWV, XM, DT, PFV>;                                            \
        static std::atomic<bool> attr_done{false};                                                                              \
        if (!attr_done.load(std::memory_order_acquire)) {                                                                                           \
            hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, 156 * 1024); \
            if (e != hipSuccess) return e;                                                                          \
            attr_done.store(true, std::memory_order_release);                                                                                       \
        }                                                                                                           \
        hipLaunchKernelGGL(kern, grid, block, lds, st, p);                                                          \
        return hipGetLastError();                                                                                   \
    } while (0)
#define QS_PF(KWV, XM, DT) do { if (pf >= 3) QS_GO(KWV, XM, DT, 3); else QS_GO(KWV, XM, DT, 1); } while (0)
    if (xmode == QS_X_STAGED) {
        if constexpr (GROUP <= 128) QS_PF(1, QS_X_STAGED, QWHIP_F16);
        else return hipErrorInvalidValue;
    }
    if (xdt == QWHIP_F16) {
        if (kw == 4) QS_PF(4, QS_X_FULL, QWHIP_F16);
        QS_PF(2, QS_X_FULL, QWHIP_F16);
    } else {
        if (kw == 4) QS_PF(4, QS_X_FULL, QWHIP_BF16);
        QS_PF(2, QS_X_FULL, QWHIP_BF16);
    }
#undef QS_PF
#undef QS_GO
}

template <int BITS, int GROUP>
void qs_sizes(size_t* wstage, size_t* xstage, uint32_t* sps) {
    using G = qs_geom<BITS, GROUP>;
    *wstage = (size_t)G::WSTAGE;
    *xstage = (size_t)((16u * G::XP16 + 255u) / 256u) * 256u * 16u;
    *sps = (uint32_t)G::SPS;
}

}  // namespace

// Tries the streaming kernel for a validated GEMV call; returns false when the shape is outside its envelope (the
// caller then falls back to the direct-load kernel).  `kw_override`: 0 = automatic, else 2 / 4.
bool qw_stream_gemv(hipStream_t st, const qwhip_weight_view* w, const void* x, uint32_t x_dtype, uint32_t m, bool rotate,
                    void* y16, float* y32, uint32_t kw_override, hipError_t* err) {
    const uint32_t bb = 4u + w->group * w->bits / 8u;
    const uint64_t row_bytes64 = (uint64_t)(w->k / w->group) * bb;
    const bool m5 = w->kind == QWHIP_KIND_HQ4_G32_M5;
    if (!(w->bits == 4 || w->bits == 8)) return false;
    if (row_bytes64 % 16 != 0) return false;                                        // whole 16-byte pieces per row
    if ((uint64_t)w->n * row_bytes64 >= (1ull << 32)) return false;                 // 32-bit offsets inside the bank
    if (((uintptr_t)w->blocks & 15u) != 0 || ((uintptr_t)x & 15u) != 0) return false;
    const uint32_t nsl = w->k / 32;
    size_t wstage = 0, xstage = 0;
    uint32_t sps = 8;
    switch (w->bits * 1000 + w->group) {
        case 4032: qs_sizes<4, 32>(&wstage, &xstage, &sps); break;
        case 4064: qs_sizes<4, 64>(&wstage, &xstage, &sps); break;
        case 4128: qs_sizes<4, 128>(&wstage, &xstage, &sps); break;
        case 4256: qs_sizes<4, 256>(&wstage, &xstage, &sps); break;
        case 8032: qs_sizes<8, 32>(&wstage, &xstage, &sps); break;
        case 8064: qs_sizes<8, 64>(&wstage, &xstage, &sps); break;
        case 8128: qs_sizes<8, 128>(&wstage, &xstage, &sps); break;
        case 8256: qs_sizes<8, 256>(&wstage, &xstage, &sps); break;
        default: return false;
    }
    const size_t budget = 150 * 1024;
    const size_t xfull = (size_t)m * ((size_t)nsl * 80u + 16u);
    const uint32_t nsteps = (nsl + sps - 1) / sps;
    // activation mode: the whole [m, k] block in LDS when it is small (and whenever it needs rotating or converting),
    // else per-step panels shared by the workgroup's four row tiles
    int xmode = -1, pf = 1, kw = 4;
    size_t lds = 0;
    const bool staged_ok = !rotate && x_dtype == QWHIP_F16 && w->group <= 128;
    const bool full_small = 4 * 2 * wstage + xfull <= 64 * 1024;
    if (full_small && (m <= 2 || !staged_ok)) xmode = QS_X_FULL;
    else if (staged_ok) xmode = QS_X_STAGED;
    else if (4 * 2 * wstage + xfull <= budget) xmode = QS_X_FULL;
    else return false;
    if (xmode == QS_X_FULL) {
        // K-split so that the grid is wide: 16 rows x (K / 4) per wave, or 32 rows x (K / 2)
        kw = nsteps >= 4 ? 4 : 2;
        if (kw_override == 2 || kw_override == 4) kw = (int)kw_override;
        const uint32_t wgs = qwhip_cdiv(w->n, 16u * (4u / (uint32_t)kw));
        const size_t lds3 = 4 * 4 * wstage + xfull;   // PF = 3
        const size_t lds1 = 4 * 2 * wstage + xfull;   // PF = 1
        // deeper prefetch when the grid is too narrow to fill the machine with resident workgroups
        pf = (wgs < 3 * 256 && lds3 <= budget) ? 3 : 1;
        lds = pf == 3 ? lds3 : lds1;
    } else {
        kw = 1;
        const size_t lds3 = 4 * 4 * wstage + 5 * xstage, lds1 = 4 * 2 * wstage + 3 * xstage;
        const uint32_t wgs = qwhip_cdiv(w->n, 64u);
        pf = (wgs < 3 * 256 && lds3 <= budget) ? 3 : 1;
        lds = pf == 3 ? lds3 : lds1;
        if (lds > budget) return false;
    }
    qs_params p;
    p.bank = (const uint8_t*)w->blocks;
    p.x = x;
    p.y16 = (h1_t*)y16;
    p.y32 = y32;
    p.N = w->n;
    p.K = w->k;
    p.M = m;
    p.row_bytes = (uint32_t)row_bytes64;
    p.rotate = rotate ? 1u : 0u;
    hipError_t e;
    switch (w->bits * 1000 + w->group) {
        case 4032: e = m5 ? qs_launch_fmt<4, 32, true>(st, p, kw, xmode, x_dtype, pf, lds) : qs_launch_fmt<4, 32, false>(st, p, kw, xmode, x_dtype, pf, lds); break;
        case 4064: e = qs_launch_fmt<4, 64, false>(st, p, kw, xmode, x_dtype, pf, lds); break;
        case 4128: e = qs_launch_fmt<4, 128, false>(st, p, kw, xmode, x_dtype, pf, lds); break;
        case 4256: e = qs_launch_fmt<4, 256, false>(st, p, kw, xmode, x_dtype, pf, lds); break;
        case 8032: e = qs_launch_fmt<8, 32, false>(st, p, kw, xmode, x_dtype, pf, lds); break;
        case 8064: e = qs_launch_fmt<8, 64, false>(st, p, kw, xmode, x_dtype, pf, lds); break;
        case 8128: e = qs_launch_fmt<8, 128, false>(st, p, kw, xmode, x_dtype, pf, lds); break;
        default: e = qs_launch_fmt<8, 256, false>(st, p, kw, xmode, x_dtype, pf, lds); break;
    }
    *err = e;
    return true;
}
