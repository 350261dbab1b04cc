// Prefill GEMM and MoE grouped GEMM: Y[m, n] = X[m, k] . W_deq[n, k]^T on the f16 matrix cores.
//
// One templated kernel.  A workgroup of WVM x WVN wavefronts owns a BM x BN output tile
// (BM = 32*WM*WVM tokens, BN = 32*WN*WVN weight rows) and walks K in steps of 64:
//   * activations: global (f16 | bf16) -> registers -> f16 LDS tile [BM][64] (144-byte pitch, so the
//     128-bit MFMA operand reads of 16 consecutive rows hit 64 distinct banks);
//   * weights: packed blocks global -> registers -> dequantized to the exact f16 weight
//     (RN_f16((1024+q)*s+b) / RN_f16(code*s+b), one packed f16 FMA) -> f16 LDS tile [BN][64];
//   * v_mfma_f32_32x32x16_f16, A = activations (rows i = tokens), B = weights (columns j = weight rows),
//     fp32 accumulators, f16 / bf16 / f32 store with n contiguous across lanes.
// The next K-step's global loads are issued before the current step's MFMAs, so HBM/L2 latency hides
// behind the matrix cores; LDS is single-buffered (two barriers per step).
//
// Dense launches map workgroups to tiles XCD-aware: the eight XCDs have private L2s and hardware deals
// workgroups round-robin, so workgroup w is re-labelled (w % 8) * per_xcd + w / 8 and consecutive labels
// walk a 4-tile-tall column band: the 32 tiles resident on one XCD share 4 activation panels and 8
// weight panels through its L2.
//
// Grouped launches (MoE) take the tile list of the pair sort: tile t = (expert e, row block) over the
// expert-major slot range [expert_off[e], expert_off[e+1]); slot rows are gathered through `gather`.
#include <mutex>

#include <atomic>

#include "qwhip_common.h"
#include "qw_slice.h"
#include "qw_mfma_2x5.h"

struct qw_gemm_params {
    const uint8_t* bank;
    const void* x;
    void* y;
    uint32_t M, N, K;
    uint32_t ldx, ldy;
    uint32_t gshift, bb;
    uint64_t row_bytes;
    uint32_t tiles_m, tiles_n;
    // grouped
    const int32_t* gather;
    const int32_t* expert_off;
    const int32_t* tile_e;
    const int32_t* tile_r;
    const int32_t* tile_count;
    uint32_t rows_per_expert;
    uint32_t inter, rotate_act;  // fused SwiGLU epilogue: gate rows [0, inter), up rows [inter, 2 inter) of an expert; FWHT-32 on the result
    qw_act act;                  // the device's gated activation (all zero: SwiGLU)
    uint32_t force_gemm2;  // tuning / tests: keep the DMA-fed kernel for the 256 x 320 shape
    uint32_t x_bf16;       // ping-pong kernel: activations are bf16, converted while the tile is staged
};


template <int YDT>
__device__ __forceinline__ void qg_store(void* y, uint64_t idx, float v) {
    if constexpr (YDT == QWHIP_F32) ((float*)y)[idx] = v;
    else if constexpr (YDT == QWHIP_F16) ((h1_t*)y)[idx] = (h1_t)v;
    else ((uint16_t*)y)[idx] = qw_f32_to_bf16(v);
}

template <int WM, int WN, int WVM, int WVN, int FMT, int XDT, int YDT, bool GROUPED>
__global__ __launch_bounds__(WVM* WVN * 64) void qw_gemm_kernel(const qw_gemm_params p) {
    constexpr int NT = WVM * WVN * 64;
    constexpr int BM = 32 * WM * WVM, BN = 32 * WN * WVN, BK = 64;
    constexpr int PITCH = BK + 8;                   // halves: 144 bytes
    constexpr int A_CHUNKS = BM * 8;                // 16-byte chunks per K-step
    constexpr int A_PER = (A_CHUNKS + NT - 1) / NT;
    constexpr int B_ITEMS = BN * 2;                 // (row, 32-column slice) items per K-step
    constexpr int B_PER = (B_ITEMS + NT - 1) / NT;

    extern __shared__ h1_t lds[];
    h1_t* la = lds;
    h1_t* lb = lds + BM * PITCH;

    const uint32_t tid = threadIdx.x;
    const uint32_t wave = tid >> 6, lane = tid & 63u;
    const uint32_t wm = wave / WVN, wn = wave % WVN;

    // ---- tile coordinates -------------------------------------------------------------------------
    uint32_t m0, n0, rows_valid;
    const uint8_t* bank = p.bank;
    if constexpr (GROUPED) {
        const uint32_t t = blockIdx.y;
        if ((int32_t)t >= p.tile_count[0]) return;
        const uint32_t e = (uint32_t)p.tile_e[t];
        const uint32_t packed = (uint32_t)p.tile_r[t];
        const uint32_t code = packed >> 24;
        const uint32_t bm = code == 1u ? 16u : (code == 2u ? 32u : 64u);
        const uint32_t start = (uint32_t)p.expert_off[e] + (packed & 0xFFFFFFu) * bm;
        const uint32_t end = (uint32_t)p.expert_off[e + 1];
        m0 = start;
        rows_valid = min((uint32_t)BM, min(bm, end - start));
        n0 = blockIdx.x * BN;
        bank += (uint64_t)e * p.rows_per_expert * p.row_bytes;
    } else {
        const uint32_t total = p.tiles_m * p.tiles_n;
        const uint32_t per_xcd = (total + 7u) / 8u;
        const uint32_t label = (blockIdx.x & 7u) * per_xcd + (blockIdx.x >> 3);
        if (label >= total) return;
        constexpr uint32_t G = 4;
        const uint32_t band = label / (G * p.tiles_n);
        const uint32_t band_rows = min(G, p.tiles_m - band * G);
        const uint32_t in_band = label - band * G * p.tiles_n;
        const uint32_t tm = band * G + in_band % band_rows;
        const uint32_t tn = in_band / band_rows;
        m0 = tm * BM;
        n0 = tn * BN;
        rows_valid = min((uint32_t)BM, p.M - m0);
    }

    // ---- per-thread copy assignments ---------------------------------------------------------------
    const uint8_t* a_src[A_PER];
    bool a_ok[A_PER];
#pragma unroll
    for (int i = 0; i < A_PER; ++i) {
        const uint32_t c = tid + i * NT;
        const uint32_t row = c >> 3, kc = c & 7u;
        a_ok[i] = (c < (uint32_t)A_CHUNKS) && (row < rows_valid);
        uint64_t src_row = m0 + row;
        if constexpr (GROUPED) {
            if (a_ok[i] && p.gather) src_row = (uint32_t)p.gather[m0 + row];
        }
        a_src[i] = (const uint8_t*)p.x + (a_ok[i] ? (src_row * p.ldx + kc * 8u) * 2u : 0u);
    }
    const uint8_t* b_src[B_PER];
    uint32_t b_sl[B_PER];
#pragma unroll
    for (int i = 0; i < B_PER; ++i) {
        const uint32_t it = tid + i * NT;
        uint32_t n = n0 + (it >> 1);
        if (n >= p.N) n = p.N - 1;
        b_sl[i] = it & 1u;
        b_src[i] = bank + (uint64_t)n * p.row_bytes;
    }

    f16_t acc[WM][WN];
#pragma unroll
    for (int a = 0; a < WM; ++a)
#pragma unroll
        for (int b = 0; b < WN; ++b)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[a][b][r] = 0.0f;

    const uint32_t magic = qw_vgpr_const(0x64006400u);
    const uint32_t nk = p.K / BK;
    u4_t a_reg[A_PER];
    qg_slice<FMT> b_reg[B_PER];

    auto issue_loads = [&](uint32_t kt) {
#pragma unroll
        for (int i = 0; i < A_PER; ++i) {
            if (a_ok[i]) a_reg[i] = *(const u4_t*)(a_src[i] + (uint64_t)kt * (BK * 2));
            else a_reg[i] = u4_t{0, 0, 0, 0};
        }
#pragma unroll
        for (int i = 0; i < B_PER; ++i) {
            if (tid + i * NT < (uint32_t)B_ITEMS) qg_load_slice<FMT>(b_src[i], kt * 2u + b_sl[i], p.gshift, p.bb, b_reg[i]);
        }
    };

    issue_loads(0);
    const uint32_t a_row_l = lane & 31u, k_half = lane >> 5;
    for (uint32_t kt = 0; kt < nk; ++kt) {
        __syncthreads();
        // registers -> LDS
#pragma unroll
        for (int i = 0; i < A_PER; ++i) {
            const uint32_t c = tid + i * NT;
            if (c < (uint32_t)A_CHUNKS) *(h8_t*)(la + (c >> 3) * PITCH + (c & 7u) * 8u) = qg_to_f16x8<XDT>(a_reg[i]);
        }
#pragma unroll
        for (int i = 0; i < B_PER; ++i) {
            const uint32_t it = tid + i * NT;
            if (it < (uint32_t)B_ITEMS) {
                const h2_t s2 = qw_splat_lo(b_reg[i].hdr), b2 = qw_splat_hi(b_reg[i].hdr);
                h1_t* dst = lb + (it >> 1) * PITCH + (it & 1u) * 32u;
#pragma unroll
                for (int j = 0; j < 4; ++j) *(h8_t*)(dst + 8 * j) = qg_dequant_chunk<FMT>(b_reg[i], j, s2, b2, magic);
            }
        }
        __syncthreads();
        if (kt + 1 < nk) issue_loads(kt + 1);
        // MFMA over the 64-wide step: 4 x k16
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) {
            h8_t af[WM], bf[WN];
#pragma unroll
            for (int a = 0; a < WM; ++a)
                af[a] = *(const h8_t*)(la + ((wm * WM + a) * 32 + a_row_l) * PITCH + ks * 16 + k_half * 8);
#pragma unroll
            for (int b = 0; b < WN; ++b)
                bf[b] = *(const h8_t*)(lb + ((wn * WN + b) * 32 + a_row_l) * PITCH + ks * 16 + k_half * 8);
#pragma unroll
            for (int a = 0; a < WM; ++a)
#pragma unroll
                for (int b = 0; b < WN; ++b)
                    acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[a], bf[b], acc[a][b], 0, 0, 0);
        }
    }

    // ---- store: lane holds column j = lane & 31, rows i = 8*(r/4) + 4*(lane >> 5) + (r & 3) -----------
#pragma unroll
    for (int a = 0; a < WM; ++a) {
#pragma unroll
        for (int b = 0; b < WN; ++b) {
            const uint32_t n = n0 + (wn * WN + b) * 32 + (lane & 31u);
            if (n < p.N) {
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const uint32_t row = (wm * WM + a) * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
                    if (row < rows_valid) qg_store<YDT>(p.y, (uint64_t)(m0 + row) * p.ldy + n, acc[a][b][r]);
                }
            }
        }
    }
}

// ------------------------------------------------------------------------------------------------
// Pipelined kernel (f16 activations): the activation tile goes global -> LDS by the DMA path
// (global_load_lds_dwordx4: no VGPRs, no VALU, no ds_write), LDS is double-buffered with an XOR
// swizzle instead of padding (16-byte slot = k-chunk ^ ((row >> 1) & 7): the 16 rows one MFMA operand
// read touches land on 16 distinct slots of a 256-byte bank row), and each K-step needs one barrier:
//   iteration k:  DMA A(k+1) -> stage (k+1)&1 | global loads B(k+2) -> registers
//                 dequant B(k+1) registers -> stage (k+1)&1
//                 MFMAs on stage k&1
//                 wait DMA, barrier
// ------------------------------------------------------------------------------------------------
template <int WM, int WN, int WVM, int WVN, int FMT, int YDT, bool GROUPED>
__global__ __launch_bounds__(WVM* WVN * 64) void qw_gemm2_kernel(const qw_gemm_params p) {
    constexpr int NT = WVM * WVN * 64;
    constexpr int BM = 32 * WM * WVM, BN = 32 * WN * WVN, BK = 64;
    constexpr int A_PER = BM * 8 / NT;  // DMA instructions per thread and K-step
    static_assert((BM * 8) % NT == 0, "activation tile must split evenly over the workgroup");
    constexpr int B_ITEMS = BN * 2;
    constexpr int B_PER = (B_ITEMS + NT - 1) / NT;
    constexpr int B_VMEM = B_PER * (FMT == QG_FMT_B8 ? 3 : 2);  // VMEM loads per thread and K-step for the weights
    constexpr uint32_t A_BYTES = BM * 128, B_BYTES = BN * 128, STAGE = A_BYTES + B_BYTES;

    extern __shared__ __attribute__((aligned(16))) uint8_t lds2[];

    const uint32_t tid = threadIdx.x;
    const uint32_t wave = tid >> 6, lane = tid & 63u;
    const uint32_t wm = wave / WVN, wn = wave % WVN;

    uint32_t m0, n0, rows_valid;
    const uint8_t* bank = p.bank;
    if constexpr (GROUPED) {
        const uint32_t t = blockIdx.y;
        if ((int32_t)t >= p.tile_count[0]) return;
        const uint32_t e = (uint32_t)p.tile_e[t];
        const uint32_t packed = (uint32_t)p.tile_r[t];
        const uint32_t code = packed >> 24;
        const uint32_t bm = code == 1u ? 16u : (code == 2u ? 32u : 64u);
        const uint32_t start = (uint32_t)p.expert_off[e] + (packed & 0xFFFFFFu) * bm;
        const uint32_t end = (uint32_t)p.expert_off[e + 1];
        m0 = start;
        rows_valid = min((uint32_t)BM, min(bm, end - start));
        n0 = blockIdx.x * BN;
        bank += (uint64_t)e * p.rows_per_expert * p.row_bytes;
    } else {
        const uint32_t total = p.tiles_m * p.tiles_n;
        const uint32_t per_xcd = (total + 7u) / 8u;
        const uint32_t label = (blockIdx.x & 7u) * per_xcd + (blockIdx.x >> 3);
        if (label >= total) return;
        constexpr uint32_t G = 4;
        const uint32_t band = label / (G * p.tiles_n);
        const uint32_t band_rows = min(G, p.tiles_m - band * G);
        const uint32_t in_band = label - band * G * p.tiles_n;
        const uint32_t tm = band * G + in_band % band_rows;
        const uint32_t tn = in_band / band_rows;
        m0 = tm * BM;
        n0 = tn * BN;
        rows_valid = min((uint32_t)BM, p.M - m0);
    }

    // ---- DMA sources: chunk c = i*NT + tid -> LDS row c >> 3, slot c & 7 (linear in c, as the DMA writes it) ----
    const uint8_t* a_src[A_PER];
#pragma unroll
    for (int i = 0; i < A_PER; ++i) {
        const uint32_t c = tid + i * NT;
        uint32_t row = c >> 3;
        const uint32_t kc = (c & 7u) ^ ((row >> 1) & 7u);
        if (row >= rows_valid) row = rows_valid - 1;  // tail rows re-read a valid row; their outputs are never stored
        uint64_t src_row = m0 + row;
        if constexpr (GROUPED) {
            if (p.gather) src_row = (uint32_t)p.gather[m0 + row];
        }
        a_src[i] = (const uint8_t*)p.x + (src_row * p.ldx + kc * 8u) * 2u;
    }
    const uint8_t* b_src[B_PER];
    uint32_t b_dst[B_PER];  // LDS byte offset of the row inside the B tile, and the slice's slot base
    uint32_t b_sw[B_PER];
#pragma unroll
    for (int i = 0; i < B_PER; ++i) {
        // every thread owns B_PER items; the surplus ones repeat the last item (same bytes to the same LDS slot), which
        // keeps the K loop free of branches so the dequant can be scheduled into the MFMA shadow
        const uint32_t it = min(tid + i * NT, (uint32_t)B_ITEMS - 1u);
        const uint32_t nl = it >> 1;
        uint32_t n = n0 + nl;
        if (n >= p.N) n = p.N - 1;
        b_src[i] = bank + (uint64_t)n * p.row_bytes;
        b_dst[i] = nl * 128u;
        b_sw[i] = ((nl >> 1) & 7u) | ((it & 1u) << 8);  // swizzle key | slice bit
    }

    f16_t acc[WM][WN];
#pragma unroll
    for (int a = 0; a < WM; ++a)
#pragma unroll
        for (int b = 0; b < WN; ++b)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[a][b][r] = 0.0f;

    const uint32_t magic = qw_vgpr_const(0x64006400u);
    const uint32_t nk = p.K / BK;
    qg_slice<FMT> b_reg[B_PER];

    auto dma_a = [&](uint32_t kt, uint32_t stage) {
#pragma unroll
        for (int i = 0; i < A_PER; ++i) {
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(a_src[i] + (uint64_t)kt * 128u),
                                             (__attribute__((address_space(3))) void*)(lds2 + stage * STAGE + (i * NT + wave * 64) * 16),
                                             16, 0, 0);
        }
    };
    auto load_b = [&](uint32_t kt) {
#pragma unroll
        for (int i = 0; i < B_PER; ++i) qg_load_slice<FMT>(b_src[i], kt * 2u + (b_sw[i] >> 8), p.gshift, p.bb, b_reg[i]);
    };
    auto store_b = [&](uint32_t stage) {
#pragma unroll
        for (int i = 0; i < B_PER; ++i) {
            const h2_t s2 = qw_splat_lo(b_reg[i].hdr), b2 = qw_splat_hi(b_reg[i].hdr);
            uint8_t* row = lds2 + stage * STAGE + A_BYTES + b_dst[i];
            const uint32_t sw = b_sw[i] & 7u, sl4 = (b_sw[i] >> 8) * 4u;
#pragma unroll
            for (int j = 0; j < 4; ++j)
                *(h8_t*)(row + (((sl4 + j) ^ sw) * 16u)) = qg_dequant_chunk<FMT>(b_reg[i], j, s2, b2, magic);
        }
    };

    // ---- prologue: tile 0 in stage 0 ----
    dma_a(0, 0);
    load_b(0);
    store_b(0);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();

    const uint32_t fr_row = lane & 31u, fr_sw = (fr_row >> 1) & 7u, k_half = lane >> 5;
    uint32_t a_off[WM], b_off[WN];
#pragma unroll
    for (int a = 0; a < WM; ++a) a_off[a] = ((wm * WM + a) * 32 + fr_row) * 128u;
#pragma unroll
    for (int b = 0; b < WN; ++b) b_off[b] = A_BYTES + ((wn * WN + b) * 32 + fr_row) * 128u;

    auto mfma_step = [&](const uint8_t* st_base) {
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) {
            const uint32_t slot = ((ks * 2u + k_half) ^ fr_sw) * 16u;
            h8_t af[WM], bf[WN];
#pragma unroll
            for (int a = 0; a < WM; ++a) af[a] = *(const h8_t*)(st_base + a_off[a] + slot);
#pragma unroll
            for (int b = 0; b < WN; ++b) bf[b] = *(const h8_t*)(st_base + b_off[b] + slot);
#pragma unroll
            for (int a = 0; a < WM; ++a)
#pragma unroll
                for (int b = 0; b < WN; ++b)
                    acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[a], bf[b], acc[a][b], 0, 0, 0);
        }
    };

    // steady state, branch-free: the DMA of the next activation tile and the loads of the next weight slices are
    // issued first, the MFMAs of the current tile hide their latency, then the weights are dequantized into the
    // other stage.  No loaded value is carried across the back edge (a loop-carried destination register makes the
    // compiler wait on the load right where it is issued).
    for (uint32_t kt = 0; kt + 1 < nk; ++kt) {
        const uint32_t cur = kt & 1u, nxt = cur ^ 1u;
#ifndef QW_PROBE_SKIP_ADMA
        dma_a(kt + 1, nxt);
#endif
#ifndef QW_PROBE_SKIP_BLOAD
        load_b(kt + 1);
#endif
        __builtin_amdgcn_sched_barrier(0);             // keep the loads at the top: their latency hides behind the MFMAs
        mfma_step(lds2 + cur * STAGE);
        store_b(nxt);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
    }
    mfma_step(lds2 + ((nk - 1) & 1u) * STAGE);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");

#pragma unroll
    for (int a = 0; a < WM; ++a) {
#pragma unroll
        for (int b = 0; b < WN; ++b) {
            const uint32_t n = n0 + (wn * WN + b) * 32 + (lane & 31u);
            if (n < p.N) {
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const uint32_t row = (wm * WM + a) * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
                    if (row < rows_valid) qg_store<YDT>(p.y, (uint64_t)(m0 + row) * p.ldy + n, acc[a][b][r]);
                }
            }
        }
    }
}

// ------------------------------------------------------------------------------------------------
// Ping-pong kernel (f16 activations, 8 waves): the waves of a workgroup form two groups of four, one wave of each group
// per SIMD.  Every K-step both groups read tile k from one LDS stage and write tile k+1 into the other, but in opposite
// order: group 0 multiplies first and fills afterwards, group 1 fills first and multiplies afterwards, so for most of a
// K-step one wave of each SIMD feeds the matrix pipe while the other dequantizes.  One barrier per K-step.  Activations
// and packed weights travel global -> registers one K-step ahead (loads issued before the MFMAs, consumed after them).
// The MFMA phase of the 2 x 5 fragment wave tile is hand-scheduled (qw_mfma_2x5.h).
// ------------------------------------------------------------------------------------------------

#define QG3_BAR_LDS() asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory")
#define QG3_BAR_ALL() asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory")

// SWIGLU (f16 out, two wave columns): the bank is a dense gate|up bank of 2 * inter rows.  A tile's BN weight rows are
// BN / 2 gate rows (wave column 0) and the BN / 2 up rows of the same outputs (wave column 1); the epilogue rounds the
// accumulators to f16 (the values the two-step chain stores) into the waves' LDS slabs, and each pair of waves then reads
// gate and up chunks of the same outputs, applies SwiGLU and the FWHT-32 in fp32 (three stages inside a lane's eight
// columns, two across the four lanes of a 32-column group) and stores act f16 [m, inter]: the reference's fused dense
// gate_up kernel (qwg_gemm_q4g_h16_swiglu: qmm_t_nax_swiglu_impl, Sources/QWMetal/include/qw_gemm_nax_swiglu.metalh:86-167),
// bit-identical to qwhip_gemm with f16 output followed by qwhip_swiglu_fwht.
// XDT = bf16: the activation tile is converted to f16 on its way from the load registers into LDS (12 vector operations
// per 16-byte piece, inside the filling phase), so bf16 activations need no pass of their own and no workspace.
template <int WM, int WN, int WVM, int WVN, int FMT, int YDT, bool SWIGLU = false, int XDT = QWHIP_F16, bool GACT = false>
__global__ __launch_bounds__(WVM* WVN * 64) void qw_gemm3_kernel(const qw_gemm_params p) {
    static_assert(WVM * WVN == 8, "two groups of four waves");
    static_assert(!SWIGLU || (WVN == 2 && YDT == QWHIP_F16), "fused SwiGLU: gate and up wave columns, f16 out");
    constexpr int NT = WVM * WVN * 64;
    constexpr int BM = 32 * WM * WVM, BN = 32 * WN * WVN, BK = 64;
    constexpr int B_ITEMS = BN * 2;
    constexpr int B_PER = (B_ITEMS + NT - 1) / NT;
    constexpr uint32_t A_BYTES = BM * 128, B_BYTES = BN * 128, STAGE = A_BYTES + B_BYTES;

    extern __shared__ __attribute__((aligned(16))) uint8_t lds2[];

    const uint32_t tid = threadIdx.x;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63u;
    const uint32_t wm = wave / WVN, wn = wave % WVN;
    const uint32_t group = wave >> 2;

    uint32_t m0, n0, rows_valid;
    const uint8_t* bank = p.bank;
    const uint32_t total = p.tiles_m * p.tiles_n;
    const uint32_t per_xcd = (total + 7u) / 8u;
    const uint32_t label = (blockIdx.x & 7u) * per_xcd + (blockIdx.x >> 3);
    if (label >= total) return;
    constexpr uint32_t G = 4;
    const uint32_t band = label / (G * p.tiles_n);
    const uint32_t band_rows = min(G, p.tiles_m - band * G);
    const uint32_t in_band = label - band * G * p.tiles_n;
    const uint32_t tm = band * G + in_band % band_rows;
    const uint32_t tn = in_band / band_rows;
    m0 = tm * BM;
    n0 = tn * (SWIGLU ? BN / 2 : BN);    // SWIGLU: n0 counts act columns
    rows_valid = min((uint32_t)BM, p.M - m0);

    // ---- activation tile: chunk c = tid + i * NT -> tile row (tid >> 3) + (NT / 8) * i, 16-byte k-chunk tid & 7.
    // Global -> registers one K-step ahead (coalesced 128-byte rows), registers -> LDS slot (k-chunk ^ ((row >> 1) & 7)).
    // One byte offset per thread and row block; rows past the tile's last one re-read the tile's first row (their
    // outputs are never stored), so any M is taken.
    constexpr int A_LD = BM * 8 / NT;
    static_assert((BM * 8) % NT == 0, "activation tile must split evenly over the workgroup");
    constexpr uint32_t A_BLK = NT / 8;
    const uint32_t a_lds0 = (tid >> 3) * 128u + (((tid & 7u) ^ ((tid >> 4) & 7u)) << 4);   // + i * A_BLK * 128 (swizzle key unchanged)
    const uint64_t a_tile_base = (uint64_t)m0 * p.ldx * 2u;
    uint32_t a_off[A_LD];   // inside the tile: under 4 GiB (the launcher checks 256 * ldx * 2)
#pragma unroll
    for (int i = 0; i < A_LD; ++i) {
        const uint32_t r = (tid >> 3) + (uint32_t)i * A_BLK;
        a_off[i] = (r < rows_valid ? r * p.ldx * 2u : 0u) + (tid & 7u) * 16u;
    }

    // ---- weight tile: item = (tile row, 32-column slice); thread items tid and NT + (tid % (B_ITEMS - NT)) (items past
    // the tile are done redundantly by several threads: identical bytes to the same slot) ----
    static_assert(B_ITEMS >= NT && B_ITEMS <= NT + NT / 2, "the second weight items are covered by group 0 alone");
    uint32_t b_off32[B_PER], b_meta[B_PER];   // byte offset of the row inside the tile's bank rows; LDS row offset | swizzle key << 16 | slice << 20
    const uint8_t* b_tile = bank + (SWIGLU ? 0ull : (uint64_t)n0 * p.row_bytes);
#pragma unroll
    for (int i = 0; i < B_PER; ++i) {
        const uint32_t it = i == 0 ? tid : NT + (B_ITEMS > NT ? tid % (uint32_t)(B_ITEMS > NT ? B_ITEMS - NT : 1) : 0u);
        const uint32_t nl = it >> 1;
        uint32_t n;
        if constexpr (SWIGLU) {
            const uint32_t up = nl >= (uint32_t)(BN / 2) ? 1u : 0u;
            n = up * p.inter + min(n0 + nl - up * (BN / 2), p.inter - 1u);   // whole bank < 4 GiB (checked by the launcher)
        } else {
            n = min(n0 + nl, p.N - 1u) - n0;
        }
        b_off32[i] = n * (uint32_t)p.row_bytes;                     // a tile's rows span < 4 GiB
        b_meta[i] = (nl * 128u) | (((nl >> 1) & 7u) << 16) | ((it & 1u) << 20);
    }
    uint32_t b_voff[B_PER];   // HQ4_G32_M5: row offset + the slice's block inside a K-step
#pragma unroll
    for (int i = 0; i < B_PER; ++i) b_voff[i] = b_off32[i] + (b_meta[i] >> 20) * 20u;
    // bit-stream blocks: lane offsets of the item's header word and of its code words; what the K-step adds is wave-uniform
    // (group 32: two blocks per K-step; larger groups: the K-step's block, and the pair of slices inside it)
    uint32_t b_vh[B_PER], b_vc[B_PER];
    constexpr uint32_t W4 = 4u * (uint32_t)qg_slice_words<FMT>();
#pragma unroll
    for (int i = 0; i < B_PER; ++i) {
        const uint32_t sl = b_meta[i] >> 20;
        b_vh[i] = b_off32[i] + (p.gshift == 0u ? sl * p.bb : 0u);
        b_vc[i] = b_vh[i] + 4u + (p.gshift == 0u ? 0u : sl * W4);
    }

    f16_t acc[WM][WN];
#pragma unroll
    for (int a = 0; a < WM; ++a)
#pragma unroll
        for (int b = 0; b < WN; ++b)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[a][b][r] = 0.0f;

    const uint32_t magic = qw_vgpr_const(0x64006400u);
    // K range: blockIdx.y splits the K-steps (fp32 partial outputs, one [M, ldy] plane per range; gridDim.y = 1 otherwise)
    const uint32_t nk_all = p.K / BK;
    const uint32_t nk_per = (nk_all + gridDim.y - 1u) / gridDim.y;
    const uint32_t kt0 = blockIdx.y * nk_per;
    const uint32_t nk = min(nk_per, nk_all - kt0);

    auto load_a = [&](uint32_t kt, u4_t* a_reg) {
        const uint8_t* xk = (const uint8_t*)p.x + a_tile_base + (uint64_t)(kt0 + kt) * 128u;   // wave-uniform: scalar base + 32-bit lane offset
#pragma unroll
        for (int i = 0; i < A_LD; ++i) {
            asm volatile("" : "+v"(a_off[i]));   // keeps the lane offset a 32-bit register: scalar base + 32-bit offset addressing
            a_reg[i] = *(const u4_t*)(xk + a_off[i]);
        }
    };
    auto store_a = [&](uint32_t stage, const u4_t* a_reg) {
#pragma unroll
        for (int i = 0; i < A_LD; ++i) *(h8_t*)(lds2 + stage * STAGE + a_lds0 + i * (A_BLK * 128u)) = qg_to_f16x8<XDT>(a_reg[i]);
    };
    auto load_b = [&](uint32_t kt, qg_slice<FMT>* b_reg, int nitems) {
#pragma unroll
        for (int i = 0; i < B_PER; ++i) {
            if (i >= nitems) continue;
            if constexpr (FMT == QG_FMT_M5) {   // 20-byte blocks: the K-step moves a wave-uniform base, the lane offset is fixed
                asm volatile("" : "+v"(b_voff[i]));
                qg_load_slice<FMT>(b_tile + (uint64_t)(kt0 + kt) * 40u + b_voff[i], 0u, p.gshift, p.bb, b_reg[i]);
            } else {
                const uint32_t kk = kt0 + kt;
                const uint32_t u_h = p.gshift == 0u ? 2u * kk * p.bb : (kk >> (p.gshift - 1u)) * p.bb;
                const uint32_t u_c = p.gshift == 0u ? u_h : u_h + ((2u * kk) & ((1u << p.gshift) - 1u)) * W4;
                asm volatile("" : "+v"(b_vh[i]), "+v"(b_vc[i]));
                qg_load_slice_at<FMT>(b_tile + u_h + b_vh[i], b_tile + u_c + b_vc[i], b_reg[i]);
            }
        }
    };
    // When the second items number a quarter of the workgroup, each is shared by the two group-0 threads tid and
    // tid + NT / 4: one dequantizes its chunks 0..1, the other 2..3 (half the second pass instead of doing it twice).
    constexpr bool SPLIT2 = (B_ITEMS - NT) * 4 == NT;
    const bool hi_half = (tid & (NT / 4)) != 0;
    auto store_b = [&](uint32_t stage, const qg_slice<FMT>* b_reg, int nitems) {
#pragma unroll
        for (int i = 0; i < B_PER; ++i) {
            if (i >= nitems) break;
            const h2_t s2 = qw_splat_lo(b_reg[i].hdr), b2 = qw_splat_hi(b_reg[i].hdr);
            uint8_t* row = lds2 + stage * STAGE + A_BYTES + (b_meta[i] & 0xFFFFu);
            const uint32_t sw = (b_meta[i] >> 16) & 7u, sl4 = (b_meta[i] >> 20) * 4u;
            if (SPLIT2 && i == 1) {
                // the half of the slice this thread dequantizes (chunks 0..1 or 2..3) moved to the front of a slice of its own
                qg_slice<FMT> half;
                if constexpr (FMT == QG_FMT_B3) {   // 24-bit chunks: the second pair starts in the middle of word 1
                    half.q[0] = hi_half ? __builtin_amdgcn_alignbit(b_reg[i].q[2], b_reg[i].q[1], 16) : b_reg[i].q[0];
                    half.q[1] = hi_half ? b_reg[i].q[2] >> 16 : b_reg[i].q[1];
                    half.q[2] = 0;
                } else {
                    constexpr int HW = qg_slice_words<FMT>() / 2;   // code words of two 8-column chunks
#pragma unroll
                    for (int w = 0; w < HW; ++w) half.q[w] = hi_half ? b_reg[i].q[HW + w] : b_reg[i].q[w];
                }
                const uint32_t j0 = hi_half ? 2u : 0u;
#pragma unroll
                for (int j = 0; j < 2; ++j)
                    *(h8_t*)(row + (((sl4 + j0 + j) ^ sw) * 16u)) = qg_dequant_chunk<FMT>(half, j, s2, b2, magic);
            } else {
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    *(h8_t*)(row + (((sl4 + j) ^ sw) * 16u)) = qg_dequant_chunk<FMT>(b_reg[i], j, s2, b2, magic);
            }
        }
    };

    const uint32_t fr_row = lane & 31u, fr_sw = (fr_row >> 1) & 7u, k_half = lane >> 5;
    // byte address of (row, 16-byte slot) = row * 128 + ((2 ks + k_half) ^ fr_sw) * 16 = (row * 128 | t) ^ (32 ks), t = (k_half ^ fr_sw) * 16
    const uint32_t a_bt = (wm * WM * 32 + fr_row) * 128u + ((k_half ^ fr_sw) << 4);
    const uint32_t b_bt = A_BYTES + (wn * WN * 32 + fr_row) * 128u + ((k_half ^ fr_sw) << 4);

    // MFMAs of one K-step.  Operands of sub-step ks+1 are fetched while sub-step ks runs: the activation fragments are
    // double-buffered, each weight fragment is reloaded right after the two MFMAs that consume it (b-major order), so
    // every LDS read has ten MFMAs of distance to its use.
    auto mfma_step = [&](const uint8_t* st_base) {
        if constexpr (WM == 2 && WN == 5) {
            const uint32_t sb = (uint32_t)(st_base - lds2);
            qg3_mfma_2x5(acc, a_bt + sb + (uint32_t)(uintptr_t)lds2, b_bt + sb + (uint32_t)(uintptr_t)lds2);
            return;
        }
        if constexpr (WM * WN <= 4) {
            // small wave tile: two or four MFMAs per sub-step cannot cover an LDS round trip, so every fragment of the
            // K-step is requested first (48 registers at most) and the MFMAs then run back to back
            h8_t af[4][WM], bf[4][WN];
#pragma unroll
            for (int ks = 0; ks < 4; ++ks) {
#pragma unroll
                for (int a = 0; a < WM; ++a) af[ks][a] = *(const h8_t*)(st_base + (a_bt ^ (32u * ks)) + a * 4096);
#pragma unroll
                for (int b = 0; b < WN; ++b) bf[ks][b] = *(const h8_t*)(st_base + (b_bt ^ (32u * ks)) + b * 4096);
            }
#pragma unroll
            for (int ks = 0; ks < 4; ++ks)
#pragma unroll
                for (int b = 0; b < WN; ++b)
#pragma unroll
                    for (int a = 0; a < WM; ++a)
                        acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[ks][a], bf[ks][b], acc[a][b], 0, 0, 0);
            return;
        }
        h8_t af[2][WM], bf[WN];
        {
            #pragma unroll
            for (int a = 0; a < WM; ++a) af[0][a] = *(const h8_t*)(st_base + a_bt + a * 4096);
#pragma unroll
            for (int b = 0; b < WN; ++b) bf[b] = *(const h8_t*)(st_base + b_bt + b * 4096);
        }
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) {
            const int cur = ks & 1, nxt = cur ^ 1;
            const uint32_t a_nx = a_bt ^ (32u * (ks + 1)), b_nx = b_bt ^ (32u * (ks + 1));
            if (ks < 3) {
#pragma unroll
                for (int a = 0; a < WM; ++a) af[nxt][a] = *(const h8_t*)(st_base + a_nx + a * 4096);
                __builtin_amdgcn_sched_group_barrier(0x100, WM, 0);
            }
#pragma unroll
            for (int b = 0; b < WN; ++b) {
#pragma unroll
                for (int a = 0; a < WM; ++a)
                    acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[cur][a], bf[b], acc[a][b], 0, 0, 0);
                __builtin_amdgcn_sched_group_barrier(0x008, WM, 0);
                if (ks < 3) {
                    bf[b] = *(const h8_t*)(st_base + b_nx + b * 4096);
                    __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
                }
            }
        }
    };

    // ---- prologue: stage 0 ----
    {
        qg_slice<FMT> b_reg[B_PER];
        u4_t a_reg[A_LD];
        load_a(0, a_reg);
        load_b(0, b_reg, B_PER);
        store_a(0, a_reg);
        store_b(0, b_reg, B_PER);
    }
    QG3_BAR_ALL();

    const uint32_t last = nk - 1u;
    // Both groups run  { load tile k+1 (group 0) / k+2 (group 1) into registers; MFMAs of step k; barrier; registers -> LDS
    // stage; barrier }, group 1 half a K-step behind group 0: while one group multiplies, the other fills the next stage.
    // RELOAD (HQ4_G32_M5 banks on the 2 x 5 fragment wave tile): a register is loaded again, for the tile after the one being
    // filled, right after the filling has read it.  The loads then fly for a whole K-step (a load takes ~1800 clocks here;
    // issued ahead of the MFMA phase they held the wave for 400 to 900 clocks while the address unit took them one by
    // one, issued inside it they were ~370 clocks short), spaced by the dequantization between them, and the MFMA phase
    // issues nothing but matrix instructions and LDS reads.  The loads are asm statements with their destinations tied in
    // and out, behind one s_waitcnt vmcnt(0) at the start of the filling: the compiler must not move or copy registers
    // that are in flight across the loop's back edge.
    constexpr bool RELOAD = FMT == QG_FMT_M5 && WM == 2 && WN == 5 && A_LD == 4 && B_PER == 2;
    if constexpr (RELOAD) {
        u4_t a_reg[A_LD], bq[2];
        uint32_t bh[2];
        auto first_loads = [&](uint32_t kt, int nitems) {          // compiler-visible loads ahead of the loop
            qg_slice<FMT> b_reg[B_PER];
            load_a(kt, a_reg);
            load_b(kt, b_reg, nitems);
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                bh[i] = i < nitems ? b_reg[i].hdr : 0u;
#pragma unroll
                for (int w = 0; w < 4; ++w) bq[i][w] = i < nitems ? b_reg[i].q[w] : 0u;
            }
        };
        // fills `stage` from the registers and sends each register off for tile `kn` as soon as it has been read
        auto fill_reload = [&](uint32_t stage, uint32_t kn, int nitems) {
            const uint8_t* xk = (const uint8_t*)p.x + a_tile_base + (uint64_t)(kt0 + kn) * 128u;
            const uint8_t* bk = b_tile + (uint64_t)(kt0 + kn) * 40u;
            asm volatile("s_waitcnt vmcnt(0)" : "+v"(a_reg[0]), "+v"(a_reg[1]), "+v"(a_reg[2]), "+v"(a_reg[3]), "+v"(bh[0]), "+v"(bq[0]), "+v"(bh[1]), "+v"(bq[1]));
#pragma unroll
            for (int i = 0; i < A_LD; ++i) {
                *(h8_t*)(lds2 + stage * STAGE + a_lds0 + i * (A_BLK * 128u)) = qg_to_f16x8<XDT>(a_reg[i]);
                asm volatile("global_load_dwordx4 %0, %1, %2" : "+v"(a_reg[i]) : "v"(a_off[i]), "s"(xk) : "memory");
            }
            qg_slice<FMT> b_reg[B_PER];
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                b_reg[i].hdr = bh[i];
#pragma unroll
                for (int w = 0; w < 4; ++w) b_reg[i].q[w] = bq[i][w];
            }
            store_b(stage, b_reg, nitems);
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                if (i >= nitems) break;
                asm volatile("global_load_dword %0, %2, %3\n\tglobal_load_dwordx4 %1, %2, %3 offset:4"
                             : "+v"(bh[i]), "+v"(bq[i]) : "v"(b_voff[i]), "s"(bk) : "memory");
            }
        };
        if (group == 0) {
            first_loads(min(1u, last), B_PER);
            for (uint32_t kt = 0; kt < nk; ++kt) {
                __builtin_amdgcn_sched_barrier(0);
                __builtin_amdgcn_s_setprio(3);
                mfma_step(lds2 + (kt & 1u) * STAGE);
                __builtin_amdgcn_s_setprio(0);
                __builtin_amdgcn_sched_barrier(0);
                fill_reload((kt + 1u) & 1u, min(kt + 2u, last), B_PER);
                QG3_BAR_LDS();
            }
        } else {
            {
                qg_slice<FMT> b_first[B_PER];
                u4_t a_first[A_LD];
                load_a(min(1u, last), a_first);
                load_b(min(1u, last), b_first, 1);
                store_a(1u, a_first);
                store_b(1u, b_first, 1);
            }
            first_loads(min(2u, last), 1);
            for (uint32_t kt = 0; kt < nk; ++kt) {
                __builtin_amdgcn_sched_barrier(0);
                __builtin_amdgcn_s_setprio(3);
                mfma_step(lds2 + (kt & 1u) * STAGE);
                __builtin_amdgcn_s_setprio(0);
                __builtin_amdgcn_sched_barrier(0);
                QG3_BAR_LDS();
                if (kt + 1u < nk) fill_reload(kt & 1u, min(kt + 3u, last), 1);      // stage (k+2)&1
            }
        }
    } else if (group == 0) {
        for (uint32_t kt = 0; kt < nk; ++kt) {
            qg_slice<FMT> b_reg[B_PER];
            u4_t a_reg[A_LD];
            load_a(min(kt + 1u, last), a_reg);
            load_b(min(kt + 1u, last), b_reg, B_PER);
            __builtin_amdgcn_sched_barrier(0);
            __builtin_amdgcn_s_setprio(3);
            mfma_step(lds2 + (kt & 1u) * STAGE);
            __builtin_amdgcn_s_setprio(0);
            __builtin_amdgcn_sched_barrier(0);
            store_a((kt + 1u) & 1u, a_reg);
            store_b((kt + 1u) & 1u, b_reg, B_PER);
            QG3_BAR_LDS();
        }
    } else {
        {
            qg_slice<FMT> b_reg[B_PER];
            u4_t a_reg[A_LD];
            load_a(min(1u, last), a_reg);
            load_b(min(1u, last), b_reg, 1);
            store_a(1u, a_reg);
            store_b(1u, b_reg, 1);
        }
        for (uint32_t kt = 0; kt < nk; ++kt) {
            qg_slice<FMT> b_reg[B_PER];
            u4_t a_reg[A_LD];
            load_a(min(kt + 2u, last), a_reg);
            load_b(min(kt + 2u, last), b_reg, 1);
            __builtin_amdgcn_sched_barrier(0);
            __builtin_amdgcn_s_setprio(3);
            mfma_step(lds2 + (kt & 1u) * STAGE);
            __builtin_amdgcn_s_setprio(0);
            __builtin_amdgcn_sched_barrier(0);
            QG3_BAR_LDS();
            if (kt + 1u < nk) {
                store_a(kt & 1u, a_reg);         // stage (k+2)&1
                store_b(kt & 1u, b_reg, 1);
            }
        }
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");

    if constexpr (YDT != QWHIP_F32) {
        // 2-byte outputs: each wave transposes its 32-row slabs through a private LDS region (the operand stages are
        // dead by now) and stores 16-byte row chunks; a lane's accumulators are one column of 16 rows, and 2-byte
        // stores from that layout cost one address per element. The host side guarantees 16-byte aligned output rows.
        constexpr uint32_t EP_PITCH = WN * 64 + 16;    // 4 rows apart land 16 banks apart
        constexpr uint32_t EP_CH = WN * 4;             // 16-byte chunks per slab row
        static_assert(8u * 32u * EP_PITCH <= 2u * STAGE, "epilogue slabs must fit the operand stages");
        __syncthreads();
        uint8_t* ep = lds2 + wave * (32u * EP_PITCH);
        const uint32_t w_off = (4u * (lane >> 5)) * EP_PITCH + (lane & 31u) * 2u;
#pragma unroll
        for (int a = 0; a < WM; ++a) {
#pragma unroll
            for (int b = 0; b < WN; ++b) {
#pragma unroll
                for (int r = 0; r < 16; r += 2) {
                    const uint32_t o = w_off + (8u * (r >> 2) + (r & 3)) * EP_PITCH + b * 64u;
                    uint32_t pk;
                    if constexpr (YDT == QWHIP_BF16) {
                        typedef __bf16 bf2_t __attribute__((ext_vector_type(2)));
                        typedef float fl2_t __attribute__((ext_vector_type(2)));
                        const fl2_t v = {acc[a][b][r], acc[a][b][r + 1]};
                        pk = __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf2_t));
                    } else {
                        const h2_t v = {(h1_t)acc[a][b][r], (h1_t)acc[a][b][r + 1]};
                        pk = __builtin_bit_cast(uint32_t, v);
                    }
                    *(uint16_t*)(ep + o) = (uint16_t)pk;
                    *(uint16_t*)(ep + o + EP_PITCH) = (uint16_t)(pk >> 16);
                }
            }
            if constexpr (SWIGLU) {
                __syncthreads();   // the partner wave's slab is complete
                const uint8_t* gs = lds2 + (wm * WVN) * (32u * EP_PITCH);
                const uint8_t* us = gs + 32u * EP_PITCH;
                const uint32_t l4 = lane & 3u;
#pragma unroll
                for (int it = 0; it < (int)(32u * EP_CH / 128u); ++it) {
                    const uint32_t q = (uint32_t)it * 128u + wn * 64u + lane;     // 16-byte chunk of the pair's 32 x (WN * 32) outputs
                    const uint32_t row = q / EP_CH, cc = q - row * EP_CH;
                    const h8_t g8 = *(const h8_t*)(gs + row * EP_PITCH + cc * 16u);
                    const h8_t u8 = *(const h8_t*)(us + row * EP_PITCH + cc * 16u);
                    float v[8];
#pragma unroll
                    for (int e = 0; e < 8; ++e) v[e] = GACT ? qw_gated((float)g8[e], (float)u8[e], p.act) : qw_swiglu((float)g8[e], (float)u8[e]);
                    if (p.rotate_act) {
#pragma unroll
                        for (int h = 1; h < 8; h <<= 1)
#pragma unroll
                            for (int i0 = 0; i0 < 8; i0 += 2 * h)
#pragma unroll
                                for (int jj = 0; jj < h; ++jj) {
                                    const float x0 = v[i0 + jj], x1 = v[i0 + jj + h];
                                    v[i0 + jj] = x0 + x1;
                                    v[i0 + jj + h] = x0 - x1;
                                }
#pragma unroll
                        for (int e = 0; e < 8; ++e) {   // columns 8 apart: the neighbouring lane; 16 apart: two lanes on
                            const float o = __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v[e]), 0xB1, 0xF, 0xF, true));
                            v[e] = (l4 & 1u) == 0u ? v[e] + o : o - v[e];
                        }
#pragma unroll
                        for (int e = 0; e < 8; ++e) {
                            const float o = __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v[e]), 0x4E, 0xF, 0xF, true));
                            v[e] = ((l4 & 2u) == 0u ? v[e] + o : o - v[e]) * QW_INV_SQRT32;
                        }
                    }
                    h8_t o8;
#pragma unroll
                    for (int e = 0; e < 8; ++e) o8[e] = (h1_t)v[e];
                    const uint32_t grow = (wm * WM + a) * 32u + row;
                    const uint32_t n = n0 + cc * 8u;
                    if (grow < rows_valid && n < p.inter)
                        *(h8_t*)((h1_t*)p.y + (uint64_t)(m0 + grow) * p.ldy + n) = o8;
                }
                __syncthreads();   // both waves are done with the slabs before the next row block overwrites them
            } else {
#pragma unroll
                for (int q = 0; q < WN * 2; ++q) {
                    const uint32_t c = q * 64u + lane;
                    const uint32_t row = c / EP_CH, cc = c - row * EP_CH;
                    const u4_t v = *(const u4_t*)(ep + row * EP_PITCH + cc * 16u);
                    const uint32_t grow = (wm * WM + a) * 32u + row;
                    const uint32_t n = n0 + wn * (WN * 32u) + cc * 8u;
                    if (grow < rows_valid && n < p.N)
                        *(u4_t*)((uint16_t*)p.y + (uint64_t)(m0 + grow) * p.ldy + n) = v;
                }
            }
        }
    } else {
#pragma unroll
        for (int a = 0; a < WM; ++a) {
#pragma unroll
            for (int b = 0; b < WN; ++b) {
                const uint32_t n = n0 + (wn * WN + b) * 32 + (lane & 31u);
                if (n < p.N) {
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        const uint32_t row = (wm * WM + a) * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
                        if (row < rows_valid) qg_store<YDT>(p.y, (uint64_t)blockIdx.y * p.M * p.ldy + (uint64_t)(m0 + row) * p.ldy + n, acc[a][b][r]);
                    }
                }
            }
        }
    }
}

// ------------------------------------------------------------------------------------------------
// Grouped kernel with the weights fed straight into the matrix cores' operand registers (f16 activations, 4 waves,
// 64 x 256 tiles of the sorted pair list).  With 64-row tiles the LDS-staged kernels above spend most of their LDS
// bandwidth on weights (written once as f16, read back by both row halves).  Here wave w owns tile columns
// [64 w, 64 w + 64) for all 64 rows (2 x 2 fragments of v_mfma_f32_32x32x16_f16): lane (n = lane & 31, h = lane >> 5)
// loads the 32-column slice 2 kt + h of weight row n of each of its two column fragments - one block per lane and
// fragment, the same loads the staged kernels issue - and dequantizes chunk ks of it (8 columns, exact f16 weights) as
// the second operand of sub-step ks.  The K order inside a K-step is thereby permuted (sub-step ks contracts columns
// 32 h + 8 ks .. + 7); the activation fragments are read from LDS in the same order (16-byte chunk 4 h + ks of the
// row), so only the 64 x 64 activation tile goes through LDS: 8 KB written and 32 KB read per K-step instead of
// 40 KB and 96 KB.  Two LDS stages, one barrier per K-step; blocks and activations travel global -> registers two
// K-steps ahead (a K-step is short here: one step of distance left the waves waiting on memory).
// Grid: one-dimensional and XCD-aware - workgroup L runs on XCD L % 8 (round-robin dispatch), each XCD takes one contiguous
// eighth of the expert-sorted tile list and walks (tile, column tile) column-fastest, so the row tiles of an expert and
// the column tiles of a row tile run side by side under one L2.
// SWIGLU (f16 out): a tile's 256 weight rows are 128 gate rows and the 128 up rows of the same outputs, ordered so that a
// wave's two column fragments are (gate, up) of the same 32 outputs: fragment b, column j of wave w is expert row
// b * inter + 128 * column tile + 32 w + j.  The epilogue rounds both accumulators to f16 (the values the two-step chain
// stores), applies SwiGLU and the FWHT-32 (five lane exchanges) in fp32 and stores act f16 [pair, inter]: the arithmetic of
// qwhip_swiglu_fwht on the f16 gate|up matrix without writing it (the reference's fused form for its dense path:
// qmm_t_nax_swiglu_impl, Sources/QWMetal/include/qw_gemm_nax_swiglu.metalh:86-167).
// ------------------------------------------------------------------------------------------------
template <int FMT, int YDT, bool SWIGLU, bool GACT = false, int XDT = QWHIP_F16>
__global__ __launch_bounds__(256) void qw_gemm4_kernel(const qw_gemm_params p) {
    static_assert(!SWIGLU || YDT == QWHIP_F16, "fused SwiGLU stores f16");
    constexpr uint32_t BM = 64, BN = 256, STAGE = BM * 128u;
    extern __shared__ __attribute__((aligned(16))) uint8_t lds4[];
    const uint32_t tid = threadIdx.x;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63u;

    const uint32_t ncol = p.tiles_n;
    const uint32_t xcd = blockIdx.x & 7u, slot = blockIdx.x >> 3;
    const uint32_t tc = (uint32_t)max(p.tile_count[0], 0);
    const uint32_t per_xcd = (tc + 7u) >> 3;
    const uint32_t ti = slot / ncol, col = slot - ti * ncol;
    const uint32_t t = xcd * per_xcd + ti;
    if (ti >= per_xcd || t >= tc) return;
    const uint32_t e = (uint32_t)p.tile_e[t];
    const uint32_t packed = (uint32_t)p.tile_r[t];
    const uint32_t code = packed >> 24;
    const uint32_t bm = code == 1u ? 16u : (code == 2u ? 32u : 64u);
    const uint32_t m0 = (uint32_t)p.expert_off[e] + (packed & 0xFFFFFFu) * bm;
    const uint32_t rows_valid = min(BM, min(bm, (uint32_t)p.expert_off[e + 1] - m0));
    const uint32_t n0 = col * (SWIGLU ? BN / 2 : BN);
    const uint8_t* bank = p.bank + (uint64_t)e * p.rows_per_expert * p.row_bytes;

    // activation tile: chunk (row = (tid >> 3) + 32 i, 16-byte k-chunk tid & 7) -> LDS slot k-chunk ^ ((row >> 1) & 7)
    uint32_t a_voff[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const uint32_t row = (tid >> 3) + 32u * i;
        const uint32_t r = row < rows_valid ? row : rows_valid - 1u;
        const uint32_t src_row = p.gather ? (uint32_t)p.gather[m0 + r] : m0 + r;
        a_voff[i] = src_row * p.ldx * 2u + (tid & 7u) * 16u;    // activations < 4 GiB (checked by the launcher)
    }
    const uint32_t a_lds0 = (tid >> 3) * 128u + (((tid & 7u) ^ ((tid >> 4) & 7u)) << 4);   // + i * 4096 (swizzle key unchanged)

    // this lane's weight rows (one per column fragment) and K half
    const uint32_t j = lane & 31u, kh = lane >> 5;
    const uint8_t* b_row[2];
#pragma unroll
    for (int b = 0; b < 2; ++b) {
        uint32_t n;
        if constexpr (SWIGLU) n = (b ? p.inter : 0u) + min(n0 + 32u * wave + j, p.inter - 1u);
        else n = min(n0 + 64u * wave + 32u * b + j, p.N - 1u);
        b_row[b] = bank + (uint64_t)n * p.row_bytes;
    }
    // fragment reads: row j (+ 32 a), logical chunk 4 kh + ks -> byte ((4 kh + ks) ^ key) * 16, key = (row >> 1) & 7 (same for a = 0, 1)
    const uint32_t fr_key = (j >> 1) & 7u;
    const uint32_t a_rd = j * 128u;

    f16_t acc[2][2];
#pragma unroll
    for (int a = 0; a < 2; ++a)
#pragma unroll
        for (int b = 0; b < 2; ++b)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[a][b][r] = 0.0f;
    const uint32_t magic = qw_vgpr_const(0x64006400u);
    const uint32_t nk = p.K / 64u;

    auto load_a = [&](uint32_t kt, u4_t* a_reg) {
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            asm volatile("" : "+v"(a_voff[i]));   // scalar base + 32-bit lane offset addressing (see qw_gemm3_kernel)
            a_reg[i] = *(const u4_t*)((const uint8_t*)p.x + (uint64_t)kt * 128u + a_voff[i]);
        }
    };
    auto store_a = [&](uint32_t stage, const u4_t* a_reg) {
#pragma unroll
        for (int i = 0; i < 2; ++i) *(h8_t*)(lds4 + stage * STAGE + a_lds0 + i * 4096u) = qg_to_f16x8<XDT>(a_reg[i]);
    };
    auto load_b = [&](uint32_t kt, qg_slice<FMT>* blk) {
#pragma unroll
        for (int b = 0; b < 2; ++b) qg_load_slice<FMT>(b_row[b], kt * 2u + kh, p.gshift, p.bb, blk[b]);
    };
    auto mfma_step = [&](const uint8_t* st, const qg_slice<FMT>* blk) {
        const h2_t s0 = qw_splat_lo(blk[0].hdr), c0 = qw_splat_hi(blk[0].hdr);
        const h2_t s1 = qw_splat_lo(blk[1].hdr), c1 = qw_splat_hi(blk[1].hdr);
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) {
            const uint32_t off = a_rd + (((4u * kh + (uint32_t)ks) ^ fr_key) << 4);
            const h8_t a0 = *(const h8_t*)(st + off), a1 = *(const h8_t*)(st + off + 4096u);
            const h8_t w0 = qg_dequant_chunk<FMT>(blk[0], ks, s0, c0, magic);
            const h8_t w1 = qg_dequant_chunk<FMT>(blk[1], ks, s1, c1, magic);
            acc[0][0] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a0, w0, acc[0][0], 0, 0, 0);
            acc[1][0] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a1, w0, acc[1][0], 0, 0, 0);
            acc[0][1] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a0, w1, acc[0][1], 0, 0, 0);
            acc[1][1] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a1, w1, acc[1][1], 0, 0, 0);
        }
    };

    // Register pipeline two K-steps deep: at step kt the blocks of kt are contracted, those of kt + 1 are in flight or
    // landed, those of kt + 2 are issued; the activation chunks of kt + 1 (issued a step ago) go to LDS at the end of the
    // step and those of kt + 2 are issued at its start.  Six steps per trip keep every buffer index a constant.
    const uint32_t last = nk - 1u;
    qg_slice<FMT> blk[3][2];
    u4_t a_reg[2][2];
    load_a(0, a_reg[0]);
    load_b(0, blk[0]);
    load_a(min(1u, last), a_reg[1]);
    load_b(min(1u, last), blk[1]);
    store_a(0, a_reg[0]);
    __syncthreads();
    for (uint32_t kt0 = 0; kt0 < nk; kt0 += 6u) {
#pragma unroll
        for (int u = 0; u < 6; ++u) {
            const uint32_t kt = kt0 + (uint32_t)u;
            if (kt >= nk) break;
            load_a(min(kt + 2u, last), a_reg[u & 1]);
            load_b(min(kt + 2u, last), blk[(u + 2) % 3]);
            mfma_step(lds4 + (uint32_t)(u & 1) * STAGE, blk[u % 3]);
            store_a((uint32_t)((u + 1) & 1), a_reg[(u + 1) & 1]);
            __syncthreads();
        }
    }

    // ---- epilogue: per wave, rows 32 a .. + 31 through a private LDS slab, 16-byte row chunks out ----
    if constexpr (SWIGLU) {
        constexpr uint32_t EP_PITCH = 64 + 16;
        __syncthreads();
        uint8_t* ep = lds4 + wave * (32u * EP_PITCH);
        const uint32_t w_off = (4u * kh) * EP_PITCH + j * 2u;
        const qw_fwht32_signs fw_signs = qw_fwht32_lane_signs(j);
#pragma unroll
        for (int a = 0; a < 2; ++a) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const float g = (float)(h1_t)acc[a][0][r], u = (float)(h1_t)acc[a][1][r];
                float v = GACT ? qw_gated(g, u, p.act) : qw_swiglu(g, u);
                if (p.rotate_act) v = qw_fwht32_lanes(v, fw_signs) * QW_INV_SQRT32;
                *(h1_t*)(ep + w_off + (8u * (r >> 2) + (r & 3)) * EP_PITCH) = (h1_t)v;
            }
#pragma unroll
            for (int q = 0; q < 2; ++q) {
                const uint32_t c = q * 64u + lane;
                const uint32_t row = c >> 2, cc = c & 3u;
                const u4_t v = *(const u4_t*)(ep + row * EP_PITCH + cc * 16u);
                const uint32_t grow = 32u * a + row;
                const uint32_t n = n0 + wave * 32u + cc * 8u;
                if (grow < rows_valid && n < p.inter)
                    *(u4_t*)((uint16_t*)p.y + (uint64_t)(m0 + grow) * p.ldy + n) = v;
            }
        }
    } else if constexpr (YDT != QWHIP_F32) {
        constexpr uint32_t EP_PITCH = 2 * 64 + 16;
        __syncthreads();
        uint8_t* ep = lds4 + wave * (32u * EP_PITCH);
        const uint32_t w_off = (4u * kh) * EP_PITCH + j * 2u;
#pragma unroll
        for (int a = 0; a < 2; ++a) {
#pragma unroll
            for (int b = 0; b < 2; ++b) {
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const uint32_t o = w_off + (8u * (r >> 2) + (r & 3)) * EP_PITCH + b * 64u;
                    if constexpr (YDT == QWHIP_BF16) *(uint16_t*)(ep + o) = qw_f32_to_bf16(acc[a][b][r]);
                    else *(h1_t*)(ep + o) = (h1_t)acc[a][b][r];
                }
            }
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const uint32_t c = q * 64u + lane;
                const uint32_t row = c >> 3, cc = c & 7u;
                const u4_t v = *(const u4_t*)(ep + row * EP_PITCH + cc * 16u);
                const uint32_t grow = 32u * a + row;
                const uint32_t n = n0 + wave * 64u + cc * 8u;
                if (grow < rows_valid && n < p.N)
                    *(u4_t*)((uint16_t*)p.y + (uint64_t)(m0 + grow) * p.ldy + n) = v;
            }
        }
    } else {
#pragma unroll
        for (int a = 0; a < 2; ++a) {
#pragma unroll
            for (int b = 0; b < 2; ++b) {
                const uint32_t n = n0 + wave * 64u + 32u * b + j;
                if (n < p.N) {
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        const uint32_t row = 32u * a + 8 * (r >> 2) + 4 * kh + (r & 3);
                        if (row < rows_valid) qg_store<YDT>(p.y, (uint64_t)(m0 + row) * p.ldy + n, acc[a][b][r]);
                    }
                }
            }
        }
    }
}

// ------------------------------------------------------------------------------------------------
// The direct-operand grouped kernel with the bank read the way memory likes it (banks of 20-byte blocks: HQ4_G32_M5 and
// the 4-bit group-32 bit streams; K % 128 == 0, bank 16-byte aligned).  In qw_gemm4_kernel every lane fetches its own 20-byte block: 64 runs of the bank per load instruction, at
// 4-byte alignment - the address unit is what bounds it.  Here the 256 weight rows of a tile are copied raw, 128 columns
// (four blocks = 80 bytes per row) at a time: consecutive threads copy consecutive 16-byte chunks of a row (five per row),
// global -> registers -> LDS, the LDS image being the same bytes in the same order; each lane then reads its block
// (five dwords) from the image for the K-step at hand and dequantizes it into the MFMA operand as before.  Per K-step
// that is 2.5 coalesced load instructions per wave instead of four scattered ones.
// LDS: two activation stages (8 KB each) and one raw stage (256 rows at a pitch of 88 bytes, 22 KB): 38 KB per workgroup,
// four workgroups per CU.  The raw image of K pair kp + 1 is in flight (registers) during K pair kp and replaces the
// stage between two barriers at its end.
// ------------------------------------------------------------------------------------------------
template <int FMT, int YDT, bool SWIGLU, bool GACT = false, int XDT = QWHIP_F16>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(3, 3))) void qw_gemm5_kernel(const qw_gemm_params p) {
    static_assert(!SWIGLU || YDT == QWHIP_F16, "fused SwiGLU stores f16");
    static_assert(FMT == QG_FMT_M5 || FMT == QG_FMT_B4, "20-byte blocks: HQ4_G32_M5 and the 4-bit group-32 bit streams");
    // raw image: row pitch 88 bytes (22 dwords: the 64 lanes of a block read fall on 64 different banks), one stage
    constexpr uint32_t BM = 64, BN = 256, A_STAGE = BM * 128u, RAW_PITCH = 88u, RAW_OFF = 2u * A_STAGE;
    extern __shared__ __attribute__((aligned(16))) uint8_t lds5[];
    const uint32_t tid = threadIdx.x;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63u;

    const uint32_t ncol = p.tiles_n;
    const uint32_t xcd = blockIdx.x & 7u, slot = blockIdx.x >> 3;
    const uint32_t tc = (uint32_t)max(p.tile_count[0], 0);
    const uint32_t per_xcd = (tc + 7u) >> 3;
    const uint32_t ti = slot / ncol, col = slot - ti * ncol;
    const uint32_t t = xcd * per_xcd + ti;
    if (ti >= per_xcd || t >= tc) return;
    const uint32_t e = (uint32_t)p.tile_e[t];
    const uint32_t packed = (uint32_t)p.tile_r[t];
    const uint32_t code = packed >> 24;
    const uint32_t bm = code == 1u ? 16u : (code == 2u ? 32u : 64u);
    const uint32_t m0 = (uint32_t)p.expert_off[e] + (packed & 0xFFFFFFu) * bm;
    const uint32_t rows_valid = min(BM, min(bm, (uint32_t)p.expert_off[e + 1] - m0));
    const uint32_t n0 = col * (SWIGLU ? BN / 2 : BN);
    const uint8_t* bank = p.bank + (uint64_t)e * p.rows_per_expert * p.row_bytes;

    // activation tile: chunk (row = (tid >> 3) + 32 i, 16-byte k-chunk tid & 7) -> LDS slot k-chunk ^ ((row >> 1) & 7)
    uint32_t a_voff[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const uint32_t row = (tid >> 3) + 32u * i;
        const uint32_t r = row < rows_valid ? row : rows_valid - 1u;
        const uint32_t src_row = p.gather ? (uint32_t)p.gather[m0 + r] : m0 + r;
        a_voff[i] = src_row * p.ldx * 2u + (tid & 7u) * 16u;    // activations < 4 GiB (checked by the launcher)
    }
    const uint32_t a_lds0 = (tid >> 3) * 128u + (((tid & 7u) ^ ((tid >> 4) & 7u)) << 4);   // + i * 4096 (swizzle key unchanged)

    // tile row nl (0..255) = 64 wave + 32 fragment + column -> weight row of the expert
    auto bank_row = [&](uint32_t nl) -> uint32_t {
        const uint32_t w = nl >> 6, b = (nl >> 5) & 1u, jj = nl & 31u;
        if constexpr (SWIGLU) return (b ? p.inter : 0u) + min(n0 + 32u * w + jj, p.inter - 1u);
        else return min(n0 + 64u * w + 32u * b + jj, p.N - 1u);
    };
    // raw copy role: 16-byte chunk q = tid + 256 i of the tile's 256 x 80-byte K-pair image
    uint32_t raw_goff[5], raw_loff[5];
#pragma unroll
    for (int i = 0; i < 5; ++i) {
        const uint32_t q = tid + 256u * i, nl = q / 5u, c = q - 5u * nl;
        raw_goff[i] = bank_row(nl) * (uint32_t)p.row_bytes + c * 16u;     // an expert's rows span < 4 GiB
        raw_loff[i] = RAW_OFF + nl * RAW_PITCH + c * 16u;                 // 8-byte aligned
    }
    // contraction role: lane (j, kh) reads block 2 s + kh of tile rows 64 wave + 32 b + j in K-step s of the pair
    const uint32_t j = lane & 31u, kh = lane >> 5;
    const uint32_t rd0 = RAW_OFF + (64u * wave + j) * RAW_PITCH + kh * 20u;   // + 32 rows for the second fragment
    const uint32_t fr_key = (j >> 1) & 7u;
    const uint32_t a_rd = j * 128u;

    f16_t acc[2][2];
#pragma unroll
    for (int a = 0; a < 2; ++a)
#pragma unroll
        for (int b = 0; b < 2; ++b)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[a][b][r] = 0.0f;
    const uint32_t magic = qw_vgpr_const(0x64006400u);
    const uint32_t nk = p.K / 64u, nkp = nk >> 1;

    auto load_a = [&](uint32_t kt, u4_t* a_reg) {
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            asm volatile("" : "+v"(a_voff[i]));   // scalar base + 32-bit lane offset addressing (see qw_gemm3_kernel)
            a_reg[i] = *(const u4_t*)((const uint8_t*)p.x + (uint64_t)kt * 128u + a_voff[i]);
        }
    };
    auto store_a = [&](uint32_t stage, const u4_t* a_reg) {
#pragma unroll
        for (int i = 0; i < 2; ++i) *(h8_t*)(lds5 + stage * A_STAGE + a_lds0 + i * 4096u) = qg_to_f16x8<XDT>(a_reg[i]);
    };
    auto load_raw = [&](uint32_t kp, u4_t* raw) {
#pragma unroll
        for (int i = 0; i < 5; ++i) {
            asm volatile("" : "+v"(raw_goff[i]));
            raw[i] = *(const u4_t*)(bank + (uint64_t)kp * 80u + raw_goff[i]);
        }
    };
    auto store_raw = [&](const u4_t* raw) {
#pragma unroll
        for (int i = 0; i < 5; ++i) {
            *(u2_t*)(lds5 + raw_loff[i]) = u2_t{raw[i][0], raw[i][1]};
            *(u2_t*)(lds5 + raw_loff[i] + 8u) = u2_t{raw[i][2], raw[i][3]};
        }
    };
    auto read_blk = [&](uint32_t s2, qg_slice<FMT>* blk) {
#pragma unroll
        for (int b = 0; b < 2; ++b) {
            const uint32_t* src = (const uint32_t*)(lds5 + rd0 + b * (32u * RAW_PITCH) + s2 * 40u);
            blk[b].hdr = src[0];
#pragma unroll
            for (int w = 0; w < 4; ++w) blk[b].q[w] = src[1 + w];
        }
    };
    auto mfma_step = [&](const uint8_t* st, const qg_slice<FMT>* blk) {
        const h2_t s0 = qw_splat_lo(blk[0].hdr), c0 = qw_splat_hi(blk[0].hdr);
        const h2_t s1 = qw_splat_lo(blk[1].hdr), c1 = qw_splat_hi(blk[1].hdr);
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) {
            const uint32_t off = a_rd + (((4u * kh + (uint32_t)ks) ^ fr_key) << 4);
            const h8_t a0 = *(const h8_t*)(st + off), a1 = *(const h8_t*)(st + off + 4096u);
            const h8_t w0 = qg_dequant_chunk<FMT>(blk[0], ks, s0, c0, magic);
            const h8_t w1 = qg_dequant_chunk<FMT>(blk[1], ks, s1, c1, magic);
            acc[0][0] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a0, w0, acc[0][0], 0, 0, 0);
            acc[1][0] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a1, w0, acc[1][0], 0, 0, 0);
            acc[0][1] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a0, w1, acc[0][1], 0, 0, 0);
            acc[1][1] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a1, w1, acc[1][1], 0, 0, 0);
        }
    };

    const uint32_t last = nk - 1u, lastp = nkp - 1u;
    u4_t raw[5], a_reg[2][2];
    load_raw(0, raw);
    load_a(0, a_reg[0]);
    load_a(min(1u, last), a_reg[1]);
    store_raw(raw);
    load_raw(min(1u, lastp), raw);
    store_a(0, a_reg[0]);
    __syncthreads();
    for (uint32_t kp = 0; kp < nkp; ++kp) {
        const uint32_t kt = 2u * kp;
        qg_slice<FMT> blk[2];
        // K-step 2 kp: activations in stage 0
        load_a(min(kt + 2u, last), a_reg[0]);
        read_blk(0u, blk);
        mfma_step(lds5, blk);
        store_a(1u, a_reg[1]);
        __syncthreads();
        // K-step 2 kp + 1: activations in stage 1
        load_a(min(kt + 3u, last), a_reg[1]);
        read_blk(1u, blk);
        mfma_step(lds5 + A_STAGE, blk);
        store_a(0u, a_reg[0]);
        __syncthreads();          // every wave has read its blocks of this pair: the single raw stage can be replaced
        store_raw(raw);
        load_raw(min(kp + 2u, lastp), raw);
        __syncthreads();
    }

    // ---- epilogue (as qw_gemm4_kernel): per wave, rows 32 a .. + 31 through a private LDS slab, 16-byte row chunks out ----
    if constexpr (SWIGLU) {
        constexpr uint32_t EP_PITCH = 64 + 16;
        uint8_t* ep = lds5 + wave * (32u * EP_PITCH);
        const uint32_t w_off = (4u * kh) * EP_PITCH + j * 2u;
        const qw_fwht32_signs fw_signs = qw_fwht32_lane_signs(j);
#pragma unroll
        for (int a = 0; a < 2; ++a) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const float g = (float)(h1_t)acc[a][0][r], u = (float)(h1_t)acc[a][1][r];
                float v = GACT ? qw_gated(g, u, p.act) : qw_swiglu(g, u);
                if (p.rotate_act) v = qw_fwht32_lanes(v, fw_signs) * QW_INV_SQRT32;
                *(h1_t*)(ep + w_off + (8u * (r >> 2) + (r & 3)) * EP_PITCH) = (h1_t)v;
            }
#pragma unroll
            for (int q = 0; q < 2; ++q) {
                const uint32_t c = q * 64u + lane;
                const uint32_t row = c >> 2, cc = c & 3u;
                const u4_t v = *(const u4_t*)(ep + row * EP_PITCH + cc * 16u);
                const uint32_t grow = 32u * a + row;
                const uint32_t n = n0 + wave * 32u + cc * 8u;
                if (grow < rows_valid && n < p.inter)
                    *(u4_t*)((uint16_t*)p.y + (uint64_t)(m0 + grow) * p.ldy + n) = v;
            }
        }
    } else if constexpr (YDT != QWHIP_F32) {
        constexpr uint32_t EP_PITCH = 2 * 64 + 16;
        uint8_t* ep = lds5 + wave * (32u * EP_PITCH);
        const uint32_t w_off = (4u * kh) * EP_PITCH + j * 2u;
#pragma unroll
        for (int a = 0; a < 2; ++a) {
#pragma unroll
            for (int b = 0; b < 2; ++b) {
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const uint32_t o = w_off + (8u * (r >> 2) + (r & 3)) * EP_PITCH + b * 64u;
                    if constexpr (YDT == QWHIP_BF16) *(uint16_t*)(ep + o) = qw_f32_to_bf16(acc[a][b][r]);
                    else *(h1_t*)(ep + o) = (h1_t)acc[a][b][r];
                }
            }
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const uint32_t c = q * 64u + lane;
                const uint32_t row = c >> 3, cc = c & 7u;
                const u4_t v = *(const u4_t*)(ep + row * EP_PITCH + cc * 16u);
                const uint32_t grow = 32u * a + row;
                const uint32_t n = n0 + wave * 64u + cc * 8u;
                if (grow < rows_valid && n < p.N)
                    *(u4_t*)((uint16_t*)p.y + (uint64_t)(m0 + grow) * p.ldy + n) = v;
            }
        }
    } else {
#pragma unroll
        for (int a = 0; a < 2; ++a) {
#pragma unroll
            for (int b = 0; b < 2; ++b) {
                const uint32_t n = n0 + wave * 64u + 32u * b + j;
                if (n < p.N) {
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        const uint32_t row = 32u * a + 8 * (r >> 2) + 4 * kh + (r & 3);
                        if (row < rows_valid) qg_store<YDT>(p.y, (uint64_t)(m0 + row) * p.ldy + n, acc[a][b][r]);
                    }
                }
            }
        }
    }
}

// ------------------------------------------------------------------------------------------------
// host side
// ------------------------------------------------------------------------------------------------
namespace {

uint32_t log2_u32(uint32_t v) {
    uint32_t r = 0;
    while ((1u << r) < v) ++r;
    return r;
}

template <int WM, int WN, int WVM, int WVN, int FMT, int XDT, int YDT, bool GROUPED>
hipError_t launch_cfg(hipStream_t st, const qw_gemm_params& p, dim3 grid) {
    constexpr int BM = 32 * WM * WVM, BN = 32 * WN * WVN;
    constexpr size_t lds = (size_t)(BM + BN) * 72 * 2;
    auto kern = qw_gemm_kernel<WM, WN, WVM, WVN, FMT, XDT, YDT, GROUPED>;
    static std::atomic<bool> attr_done{false};  // per instantiation
    if (!attr_done.load(std::memory_order_acquire)) {
        hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return e;
        attr_done.store(true, std::memory_order_release);
    }
    hipLaunchKernelGGL(kern, grid, dim3(WVM * WVN * 64), lds, st, p);
    return hipGetLastError();
}

template <int WM, int WN, int WVM, int WVN, int FMT, int YDT, bool GROUPED>
hipError_t launch_cfg2(hipStream_t st, const qw_gemm_params& p, dim3 grid) {
    constexpr int BM = 32 * WM * WVM, BN = 32 * WN * WVN;
    constexpr size_t lds = (size_t)2 * (BM + BN) * 128;
    auto kern = qw_gemm2_kernel<WM, WN, WVM, WVN, FMT, YDT, GROUPED>;
    static std::atomic<bool> attr_done{false};  // per instantiation
    if (!attr_done.load(std::memory_order_acquire)) {
        hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return e;
        attr_done.store(true, std::memory_order_release);
    }
    hipLaunchKernelGGL(kern, grid, dim3(WVM * WVN * 64), lds, st, p);
    return hipGetLastError();
}

template <int WM, int WN, int WVM, int WVN, int FMT, int YDT, bool SWIGLU = false, int XDT = QWHIP_F16, bool GACT = false>
hipError_t launch_cfg3(hipStream_t st, const qw_gemm_params& p, dim3 grid) {
    constexpr int BM = 32 * WM * WVM, BN = 32 * WN * WVN;
    constexpr size_t lds = (size_t)2 * (BM + BN) * 128;
    auto kern = qw_gemm3_kernel<WM, WN, WVM, WVN, FMT, YDT, SWIGLU, XDT, GACT>;
    static std::atomic<bool> attr_done{false};  // per instantiation
    if (!attr_done.load(std::memory_order_acquire)) {
        hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return e;
        attr_done.store(true, std::memory_order_release);
    }
    hipLaunchKernelGGL(kern, grid, dim3(WVM * WVN * 64), lds, st, p);
    return hipGetLastError();
}

// ---- split-K for problems of few tiles: fp32 partial planes, summed in range order ---------------------------------------
template <int YDT>
__global__ __launch_bounds__(256) void qw_splitk_reduce_kernel(const float* __restrict__ part, uint32_t splits, uint32_t M, uint32_t N,
                                                               void* __restrict__ y, uint32_t ldy) {
    const uint32_t n4 = N / 4u;
    const uint64_t i = (uint64_t)blockIdx.x * 256u + threadIdx.x;
    if (i >= (uint64_t)M * n4) return;
    const uint32_t row = (uint32_t)(i / n4), c = (uint32_t)(i - (uint64_t)row * n4) * 4u;
    const uint64_t plane = (uint64_t)M * N;
    typedef float fl4_t __attribute__((ext_vector_type(4)));
    fl4_t acc = *(const fl4_t*)(part + (uint64_t)row * N + c);
    for (uint32_t sidx = 1; sidx < splits; ++sidx) acc += *(const fl4_t*)(part + sidx * plane + (uint64_t)row * N + c);
#pragma unroll
    for (int e = 0; e < 4; ++e) qg_store<YDT>(y, (uint64_t)row * ldy + c + e, acc[e]);
}

template <int FMT, int YDT, bool SWIGLU, bool GACT = false, int XDT = QWHIP_F16>
hipError_t launch_cfg4(hipStream_t st, const qw_gemm_params& p, dim3 grid) {
    // two activation stages, or the four epilogue slabs (32 rows x (128 + 16) bytes each) when they are larger
    constexpr size_t lds = 4u * 32u * 144u;
    static_assert(lds >= 2u * 64u * 128u, "the stages fit the slab allocation");
    hipLaunchKernelGGL((qw_gemm4_kernel<FMT, YDT, SWIGLU, GACT, XDT>), grid, dim3(256), lds, st, p);
    return hipGetLastError();
}

template <int FMT, int YDT, bool SWIGLU, bool GACT = false, int XDT = QWHIP_F16>
hipError_t launch_cfg5(hipStream_t st, const qw_gemm_params& p, dim3 grid) {
    constexpr size_t lds = 2u * 64u * 128u + 256u * 88u;   // two activation stages + one raw K-pair image (38,912 bytes)
    if constexpr (FMT == QG_FMT_M5 || FMT == QG_FMT_B4) {
        hipLaunchKernelGGL((qw_gemm5_kernel<FMT, YDT, SWIGLU, GACT, XDT>), grid, dim3(256), lds, st, p);
        return hipGetLastError();
    } else {
        return hipErrorInvalidValue;   // not reached: gemm5_takes() refuses the 8-bit containers
    }
}
// the raw-copy kernel takes banks of 20-byte blocks (HQ4_G32_M5, 4-bit group 32) whose rows are whole 80-byte K pairs at
// 16-byte aligned addresses
inline bool gemm5_takes(const qw_gemm_params& p, int fmt) {
    return (fmt == QG_FMT_M5 || (fmt == QG_FMT_B4 && p.gshift == 0)) && p.K % 128u == 0 && ((uintptr_t)p.bank & 15u) == 0;
}

// tile shapes of the pipelined kernel
enum { CFG_256x320 = 0, CFG_256x256 = 1, CFG_128x128 = 2, CFG_256x128 = 3, CFG_128x320 = 4, CFG_COUNT = 5 };
static const uint32_t kCfgBM[CFG_COUNT] = {256, 256, 128, 256, 128};
static const uint32_t kCfgBN[CFG_COUNT] = {320, 256, 128, 128, 320};

// the ping-pong kernel takes the 256 x 320 and 128 x 320 tiles at any row count, every container, and 2-byte outputs whose
// rows are 16-byte aligned
inline bool gemm3_takes(const qw_gemm_params& p, int cfg, int fmt, uint32_t ydt) {
    return (cfg == CFG_256x320 || cfg == CFG_128x320) && !p.force_gemm2 &&
           (ydt == QWHIP_F32 || (p.ldy % 8u == 0 && ((uintptr_t)p.y & 15u) == 0));
}

template <int FMT, int YDT>
hipError_t launch_dense2(hipStream_t st, qw_gemm_params& p, int cfg) {
    p.tiles_m = qwhip_cdiv(p.M, kCfgBM[cfg]);
    p.tiles_n = qwhip_cdiv(p.N, kCfgBN[cfg]);
    const uint32_t total = p.tiles_m * p.tiles_n;
    const dim3 grid(((total + 7u) / 8u) * 8u);
    switch (cfg) {
        case CFG_256x320:
            // (the 6- and 8-bit containers spill three to five registers on this tile and still run a sixth faster than on the
            // DMA-fed kernel)
            if (gemm3_takes(p, cfg, FMT, YDT)) {
                if (p.x_bf16) return launch_cfg3<2, 5, 4, 2, FMT, YDT, false, QWHIP_BF16>(st, p, grid);
                return launch_cfg3<2, 5, 4, 2, FMT, YDT>(st, p, grid);
            }
            return launch_cfg2<2, 5, 4, 2, FMT, YDT, false>(st, p, grid);
        case CFG_128x320:
            if (gemm3_takes(p, cfg, FMT, YDT)) {
                if (p.x_bf16) return launch_cfg3<1, 5, 4, 2, FMT, YDT, false, QWHIP_BF16>(st, p, grid);
                return launch_cfg3<1, 5, 4, 2, FMT, YDT>(st, p, grid);
            }
            return launch_cfg2<1, 5, 4, 2, FMT, YDT, false>(st, p, grid);
        case CFG_256x256: return launch_cfg2<2, 4, 4, 2, FMT, YDT, false>(st, p, grid);
        case CFG_256x128: return launch_cfg2<2, 2, 4, 2, FMT, YDT, false>(st, p, grid);
        default: return launch_cfg2<2, 2, 2, 2, FMT, YDT, false>(st, p, grid);
    }
}

template <int FMT>
hipError_t launch_dense2_y(hipStream_t st, qw_gemm_params& p, int cfg, uint32_t ydt) {
    if (ydt == QWHIP_F16) return launch_dense2<FMT, QWHIP_F16>(st, p, cfg);
    if (ydt == QWHIP_BF16) return launch_dense2<FMT, QWHIP_BF16>(st, p, cfg);
    return launch_dense2<FMT, QWHIP_F32>(st, p, cfg);
}

// fallback (bf16 activations converted inside the kernel, no workspace): 128 x 128 tiles only
template <int FMT, int XDT>
hipError_t launch_dense1_y(hipStream_t st, qw_gemm_params& p, uint32_t ydt) {
    p.tiles_m = qwhip_cdiv(p.M, 128u);
    p.tiles_n = qwhip_cdiv(p.N, 128u);
    const uint32_t total = p.tiles_m * p.tiles_n;
    const dim3 grid(((total + 7u) / 8u) * 8u);
    if (ydt == QWHIP_F16) return launch_cfg<2, 2, 2, 2, FMT, XDT, QWHIP_F16, false>(st, p, grid);
    if (ydt == QWHIP_BF16) return launch_cfg<2, 2, 2, 2, FMT, XDT, QWHIP_BF16, false>(st, p, grid);
    return launch_cfg<2, 2, 2, 2, FMT, XDT, QWHIP_F32, false>(st, p, grid);
}

// Rounds of `tiles` over `slots` resident workgroups, the last one priced by how full it is (see choose_cfg).
double priced_rounds(double tiles, double slots) {
    const double full = (double)(uint64_t)((tiles - 1.0) / slots);
    const double f = (tiles - full * slots) / slots;
    return full + (f <= 0.5 ? 0.67 : 0.67 + 0.66 * (f - 0.5));
}

// waste-aware choice among the tile shapes: time ~ rounds of tiles over the CUs x per-tile cost / shape efficiency.
// `pingpong`: the ping-pong kernel is available (2-byte outputs need 16-byte aligned rows) for the 256 x 320 and 128 x 320
// shapes.  `only_pingpong` keeps the choice to those two (bf16 activations with no workspace to convert into: the other
// kernels would fall to the unpipelined one).
int choose_cfg(uint32_t M, uint32_t N, bool eight_bit, bool pingpong, bool only_pingpong) {
    // efficiency of each shape per tile area, on the scale ping-pong 256 x 320 on a 4-bit container = 1 (188 us a round
    // on M = 4096, N = K = 5120).  DMA-fed kernel: 264 us on that tile (0.71), the smaller shapes 0.82 / 0.78 / 0.75 of that;
    // half-height ping-pong tile: 115 us for 256 tiles against 90 us for half a round of the big tile (0.78); 8-bit
    // containers: 206 us a round on the ping-pong 256 x 320 (0.91; 237 - 242 us on the DMA-fed kernel), 132 us on the
    // half-height tile (0.71)
    static const double kEffPp[CFG_COUNT] = {1.00, 0.58, 0.55, 0.53, 0.78};
    static const double kEffPp8[CFG_COUNT] = {0.91, 0.65, 0.62, 0.59, 0.71};
    static const double kEffDma[CFG_COUNT] = {0.71, 0.58, 0.55, 0.53, 0.58};
    const double* eff = !pingpong ? kEffDma : (eight_bit ? kEffPp8 : kEffPp);
    const double resident[CFG_COUNT] = {1, 1, 2, 1, 1};
    // a problem of few tiles is one tile's K loop long whatever the shape, and the small tile's loop is the shortest
    // (N = K = 5120, f16: M = 64 in 65 us on 128 x 128 against 82 us on the half-height ping-pong tile, M = 512 81 against 85;
    // N = K = 2048, M = 2048: 32 against 38).  bf16 rows read in place run the unpipelined kernel on that shape, which holds
    // up to 128 tiles only (M = 256: 88 us against 87)
    if ((uint64_t)qwhip_cdiv(M, 128u) * qwhip_cdiv(N, 128u) <= (only_pingpong ? 128u : 256u)) return CFG_128x128;
    double best = 1e300;
    int best_cfg = only_pingpong ? CFG_128x320 : CFG_128x128;
    for (int c = 0; c < CFG_COUNT; ++c) {
        const bool pp = pingpong && (c == CFG_128x320 || c == CFG_256x320);
        if (only_pingpong && !pp) continue;
        const double tiles = (double)qwhip_cdiv(M, kCfgBM[c]) * qwhip_cdiv(N, kCfgBN[c]);
        const double slots = 256.0 * resident[c];
        // The last round is cheaper than a full one: the clocks are power-bound, so tiles on half the CUs or fewer finish in
        // 0.67 of a full round's time and the cost grows linearly from there (256 x 320 on N = K = 5120: 128 tiles 121 us,
        // 192 tiles 148 us, 256 tiles 180 us; M = 6144, 384 tiles: 301 us = 180 + 121)
        const double cost = priced_rounds(tiles, slots) * resident[c] * kCfgBM[c] * kCfgBN[c] / eff[c];
        if (cost < best) {
            best = cost;
            best_cfg = c;
        }
    }
    return best_cfg;
}

qwhip_status gemm_checks(qwhip_stream_t s, const qwhip_weight_view* w, const void* x, uint32_t x_dtype, void* y,
                         uint32_t y_dtype, int* fmt) {
    QWHIP_REQUIRE(s);
    qwhip_status st = qwhip_weight_view_validate(w);
    if (st != QWHIP_OK) return st;
    QWHIP_REQUIRE(x);
    QWHIP_REQUIRE(y);
    if (x_dtype != QWHIP_F16 && x_dtype != QWHIP_BF16)
        return qwhip_fail(QWHIP_E_BAD_WEIGHTS, "activations must be f16 or bf16, got dtype %u", x_dtype);
    if (y_dtype != QWHIP_F16 && y_dtype != QWHIP_BF16 && y_dtype != QWHIP_F32)
        return qwhip_fail(QWHIP_E_BAD_WEIGHTS, "output must be f16, bf16 or f32, got dtype %u", y_dtype);
    if (w->k % 64 != 0) return qwhip_fail(QWHIP_E_BAD_GEOMETRY, "tensor GEMM needs k %% 64 == 0, got k=%u", w->k);
    if ((uintptr_t)x & 15u) return qwhip_fail(QWHIP_E_BAD_SHAPE, "activations must be 16-byte aligned");
    if (w->kind == QWHIP_KIND_HQ4_G32_M5) *fmt = QG_FMT_M5;
    else if (w->bits == 4) *fmt = QG_FMT_B4;
    else if (w->bits == 8) *fmt = QG_FMT_B8;
    else if (w->bits == 2) *fmt = QG_FMT_B2;
    else if (w->bits == 3) *fmt = QG_FMT_B3;
    else if (w->bits == 6) *fmt = QG_FMT_B6;
    else return qwhip_fail(QWHIP_E_BAD_WEIGHTS, "no tensor GEMM kernel for %u-bit group %u", w->bits, w->group);
    return QWHIP_OK;
}

// runs EXPR with F bound to the container format as a constant
// split-K launch of the half-height ping-pong tile into fp32 planes at `part`, then the sum into y
template <int FMT>
hipError_t launch_splitk(hipStream_t st, const qw_gemm_params& p, uint32_t splits, float* part, void* y, uint32_t y_dtype, uint32_t ldy) {
    {
        qw_gemm_params q = p;
        q.y = part;
        q.ldy = p.N;
        q.tiles_m = qwhip_cdiv(p.M, kCfgBM[CFG_128x320]);
        q.tiles_n = qwhip_cdiv(p.N, kCfgBN[CFG_128x320]);
        const dim3 grid(((q.tiles_m * q.tiles_n + 7u) / 8u) * 8u, splits);
        hipError_t e = p.x_bf16 ? launch_cfg3<1, 5, 4, 2, FMT, QWHIP_F32, false, QWHIP_BF16>(st, q, grid)
                                : launch_cfg3<1, 5, 4, 2, FMT, QWHIP_F32>(st, q, grid);
        if (e != hipSuccess) return e;
        const dim3 rgrid((unsigned)(((uint64_t)p.M * (p.N / 4u) + 255u) / 256u));
        if (y_dtype == QWHIP_F16) hipLaunchKernelGGL(qw_splitk_reduce_kernel<QWHIP_F16>, rgrid, dim3(256), 0, st, part, splits, p.M, p.N, y, ldy);
        else if (y_dtype == QWHIP_BF16) hipLaunchKernelGGL(qw_splitk_reduce_kernel<QWHIP_BF16>, rgrid, dim3(256), 0, st, part, splits, p.M, p.N, y, ldy);
        else hipLaunchKernelGGL(qw_splitk_reduce_kernel<QWHIP_F32>, rgrid, dim3(256), 0, st, part, splits, p.M, p.N, y, ldy);
        return hipGetLastError();
    }
}

// K ranges for a problem of few tiles (0 = one launch): 2..8 ranges of at least 8 K-steps over at most 256 workgroups of
// 128 x 320 tiles, when `workspace_bytes` holds the fp32 planes behind its first `used` bytes and the ranges pay:
// K-steps taken off the tile's loop (0.72 us each) against writing and re-reading the planes (about 5 TB/s together) and
// the second launch (4 us).  N = K = 2048 with a workspace: M = 1536 over 3 ranges took 46 us against 36 us in one launch,
// M = 2048 over 2 ranges 36 against 32; N = K = 5120, M = 1024 over 2: 71 against 84.
uint32_t choose_splits(uint32_t m, uint32_t n, uint32_t k, uint64_t used, uint64_t workspace_bytes) {
    const uint32_t tiles = qwhip_cdiv(m, kCfgBM[CFG_128x320]) * qwhip_cdiv(n, kCfgBN[CFG_128x320]);
    const uint32_t nk = k / 64u;
    const uint64_t plane = (uint64_t)m * n * 4u;
    uint32_t splits = min(min(8u, 256u / tiles), nk / 8u);
    auto pays = [&](uint32_t sp) { return nk * 0.72 * (1.0 - 1.0 / sp) > sp * (double)plane * 2.0 / 5e6 + 4.0; };
    while (splits >= 2u && ((uint64_t)(splits - 1u) * qwhip_cdiv(nk, splits) >= nk || used + splits * plane > workspace_bytes || !pays(splits)))
        --splits;
    return splits < 2u ? 0u : splits;
}

#define QG_FOR_FMT(fmt, e, EXPR)                                                  \
    switch (fmt) {                                                                \
        case QG_FMT_M5: { constexpr int F = QG_FMT_M5; e = (EXPR); } break;       \
        case QG_FMT_B4: { constexpr int F = QG_FMT_B4; e = (EXPR); } break;       \
        case QG_FMT_B8: { constexpr int F = QG_FMT_B8; e = (EXPR); } break;       \
        case QG_FMT_B2: { constexpr int F = QG_FMT_B2; e = (EXPR); } break;       \
        case QG_FMT_B3: { constexpr int F = QG_FMT_B3; e = (EXPR); } break;       \
        case QG_FMT_B6: { constexpr int F = QG_FMT_B6; e = (EXPR); } break;       \
        default: e = hipErrorInvalidValue;                                        \
    }

}  // namespace

// flags bits 8..11: tile shape override for tuning and tests (0 = automatic, 1 + CFG_*; 14 = 256 x 320 on the DMA-fed
// kernel instead of the ping-pong kernel; 15 = the unpipelined kernel).
extern "C" qwhip_status qwhip_gemm(qwhip_stream_t s, const qwhip_weight_view* w, const void* x, uint32_t x_dtype, uint32_t m,
                                   uint32_t ldx, void* y, uint32_t y_dtype, uint32_t ldy, uint32_t flags, void* workspace,
                                   uint64_t workspace_bytes) {
    int fmt = 0;
    qwhip_status st = gemm_checks(s, w, x, x_dtype, y, y_dtype, &fmt);
    if (st != QWHIP_OK) return st;
    if (m == 0) return QWHIP_OK;
    if (w->n % 16 != 0) return qwhip_fail(QWHIP_E_BAD_GEOMETRY, "tensor GEMM needs n %% 16 == 0, got n=%u", w->n);
    if (ldx == 0) ldx = w->k;
    if (ldy == 0) ldy = w->n;
    if (ldx < w->k || ldy < w->n || (ldx % 8) != 0 || ldx >= (1u << 22))   // a tile's 256 activation rows stay under 4 GiB
        return qwhip_fail(QWHIP_E_BAD_SHAPE, "bad leading dimensions ldx=%u ldy=%u for k=%u n=%u", ldx, ldy, w->k, w->n);

    const bool rotate = qwhip_view_rotated(w) && !(flags & QWHIP_X_PREROTATED);
    const uint64_t ws_need = (uint64_t)m * w->k * 2u;
    const bool ws_ok = workspace && workspace_bytes >= ws_need && ldx == w->k && ((uintptr_t)workspace & 15u) == 0;
    const void* xin = x;
    uint32_t xdt = x_dtype;
    const uint32_t ov = (flags >> 8) & 0xFu;
    // 2-byte outputs reach the ping-pong kernel with 16-byte aligned rows only (gemm3_takes)
    const bool pp_ok = y_dtype == QWHIP_F32 || (ldy % 8u == 0 && ((uintptr_t)y & 15u) == 0);
    const bool bf16_in_place = pp_ok && !rotate && x_dtype == QWHIP_BF16 && !ws_ok && !(flags & (1u << 16));
    const int cfg = (ov >= 1 && ov <= CFG_COUNT) ? (int)ov - 1
                                                 : (ov == 14u ? (int)CFG_256x320 : choose_cfg(m, w->n, fmt == QG_FMT_B8, pp_ok, bf16_in_place));
    qw_gemm_params p = {};
    p.M = m;
    p.ldy = ldy;
    p.y = y;
    p.force_gemm2 = ov == 14u ? 1u : 0u;
    // Split-K: a problem of few tiles is one tile's K loop long (80 K-steps of ~1.1 us on K = 5120, whatever M).  When the
    // workspace also holds fp32 partial planes (after the activation copy, if there is one), the K-steps of a tile are dealt
    // over 2..8 workgroups and a second launch sums the planes in range order.
    const bool copy_needed = rotate || (x_dtype == QWHIP_BF16 && (flags & (1u << 16)));   // bf16 rows in the basis are read in place
    const uint64_t sk_used = copy_needed ? ((ws_need + 255u) & ~(uint64_t)255u) : 0u;
    uint32_t splits = 0;
    if (ov == 0u && pp_ok && workspace && ((uintptr_t)workspace & 15u) == 0 && w->n % 4u == 0 && (!copy_needed || ws_ok))
        splits = choose_splits(m, w->n, w->k, sk_used, workspace_bytes);
    // bf16 activations already in the basis: the ping-pong kernel converts them while it stages the tile (no pass of its own,
    // no workspace); flags bit 16 keeps the separate pass, for tests and comparisons
    const bool direct_bf16 = !rotate && x_dtype == QWHIP_BF16 && ov != 15u && !(flags & (1u << 16)) && (splits != 0u || gemm3_takes(p, cfg, fmt, y_dtype));
    if (direct_bf16) {
        p.x_bf16 = 1u;
        xdt = QWHIP_F16;   // dispatch as the f16 kernels do; the kernel itself reads bf16
    } else if (rotate) {
        // rotated f16 copy of the activations in the caller's workspace, then the GEMM reads that
        if (!workspace || workspace_bytes < ws_need)
            return qwhip_fail(QWHIP_E_BASIS,
                              "activations are not in the rotated basis and the workspace holds %llu bytes, %llu needed",
                              (unsigned long long)workspace_bytes, (unsigned long long)ws_need);
        if (!ws_ok) return qwhip_fail(QWHIP_E_BAD_SHAPE, "rotation pre-pass needs tightly packed activations and a 16-byte aligned workspace");
        st = qwhip_fwht32(s, x, x_dtype, workspace, (uint64_t)m * w->k);
        if (st != QWHIP_OK) return st;
        xin = workspace;
        xdt = QWHIP_F16;
    } else if (x_dtype == QWHIP_BF16 && ws_ok) {
        // one bf16 -> f16 pass instead of a conversion in every tile of the GEMM
        st = qw_convert_to_f16(s, x, x_dtype, workspace, (uint64_t)m * w->k);
        if (st != QWHIP_OK) return st;
        xin = workspace;
        xdt = QWHIP_F16;
    }

    p.bank = (const uint8_t*)w->blocks;
    p.x = xin;
    p.N = w->n;
    p.K = w->k;
    p.ldx = ldx;
    p.gshift = log2_u32(w->group / 32);
    p.bb = qwhip_view_block_bytes(w);
    p.row_bytes = qwhip_view_row_bytes(w);
    hipError_t e;
    if (splits != 0u && xdt == QWHIP_F16) {
        float* part = (float*)((uint8_t*)workspace + sk_used);
        QG_FOR_FMT(fmt, e, (launch_splitk<F>(s->stream, p, splits, part, y, y_dtype, ldy)))
        QWHIP_TRY_HIP(e);
        return QWHIP_OK;
    }
    if (xdt != QWHIP_F16 || ov == 15u) {
        if (xdt == QWHIP_F16) {
            QG_FOR_FMT(fmt, e, (launch_dense1_y<F, QWHIP_F16>(s->stream, p, y_dtype)))
        } else {
            QG_FOR_FMT(fmt, e, (launch_dense1_y<F, QWHIP_BF16>(s->stream, p, y_dtype)))
        }
    } else {
        QG_FOR_FMT(fmt, e, (launch_dense2_y<F>(s->stream, p, cfg, y_dtype)))
    }
    QWHIP_TRY_HIP(e);
    return QWHIP_OK;
}

// ---- qwhip_gemm for callers that cannot allocate ------------------------------------------------------------------------
// The f16 copy of the activations (rotated, or converted from bf16) that qwhip_gemm keeps in the caller's workspace lives
// here in a file-scope device array instead.  Each GPU holds its own copy of the array at its own address: the address is
// resolved once per device, with that device current, from qwhip_device_create, and host code only ever uses the resolved
// pointer (the array's name is not a device address on the host side).
#define QW_GEMM_SCRATCH_BYTES (8u << 20)
#define QW_GEMM_SCRATCH_DEVICES 64
static __device__ __align__(256) uint8_t qw_gemm_scratch[QW_GEMM_SCRATCH_BYTES];
static void* qw_gemm_scratch_ptr[QW_GEMM_SCRATCH_DEVICES];   // written under qw_gemm_scratch_mu, read after device creation
static std::mutex qw_gemm_scratch_mu;

// Called by qwhip_device_create with device `ordinal` current.
qwhip_status qw_gemm_scratch_init(int ordinal) {
    if (ordinal < 0 || ordinal >= QW_GEMM_SCRATCH_DEVICES) return QWHIP_OK;   // such a device has no static scratch; the entry point says so
    std::lock_guard<std::mutex> lock(qw_gemm_scratch_mu);
    if (qw_gemm_scratch_ptr[ordinal]) return QWHIP_OK;
    void* ptr = nullptr;
    QWHIP_TRY_HIP(hipGetSymbolAddress(&ptr, HIP_SYMBOL(qw_gemm_scratch)));
    if (!ptr) return qwhip_fail(QWHIP_E_DEVICE, "hipGetSymbolAddress returned no address for the GEMM scratch array");
    qw_gemm_scratch_ptr[ordinal] = ptr;
    return QWHIP_OK;
}

extern "C" uint64_t qwhip_gemm_noalloc_max_bytes(void) { return QW_GEMM_SCRATCH_BYTES; }

extern "C" qwhip_status qwhip_gemm_noalloc(qwhip_stream_t s, const qwhip_weight_view* w, const void* x, uint32_t x_dtype, uint32_t m,
                                           uint32_t ldx, void* y, uint32_t y_dtype, uint32_t ldy, uint32_t flags) {
    QWHIP_REQUIRE(s);
    QWHIP_REQUIRE(w);
    // rows already in the container's basis are read where they lie (bf16 rows are converted while a tile is staged): no
    // copy, so no limit on their size and nothing of the scratch array is touched
    if (!(qwhip_view_rotated(w) && !(flags & QWHIP_X_PREROTATED)))
        return qwhip_gemm(s, w, x, x_dtype, m, ldx, y, y_dtype, ldy, flags, nullptr, 0);
    const uint64_t need = (uint64_t)m * w->k * 2u;
    if (need > QW_GEMM_SCRATCH_BYTES)
        return qwhip_fail(QWHIP_E_BAD_SHAPE, "qwhip_gemm_noalloc: m * k * 2 = %llu bytes exceeds the static scratch of %u bytes; use qwhip_gemm with a workspace",
                          (unsigned long long)need, (unsigned)QW_GEMM_SCRATCH_BYTES);
    const int ord = s->dev->ordinal;
    void* scratch = (ord >= 0 && ord < QW_GEMM_SCRATCH_DEVICES) ? qw_gemm_scratch_ptr[ord] : nullptr;
    if (!scratch) return qwhip_fail(QWHIP_E_DEVICE, "qwhip_gemm_noalloc: device %d has no resolved scratch array", ord);
    // exactly the bytes of the activation copy: the same launches as qwhip_gemm with a workspace of that size (no split-K planes)
    return qwhip_gemm(s, w, x, x_dtype, m, ldx, y, y_dtype, ldy, flags, scratch, need);
}

// Dense gate|up GEMM with the SwiGLU (+ FWHT-32) epilogue fused: act f16 [m, inter], inter = n / 2, the bank's rows being
// [gate | up].  Runs the ping-pong kernel's fused form: every container, any row count, one launch.
extern "C" qwhip_status qwhip_gemm_swiglu(qwhip_stream_t s, const qwhip_weight_view* w, const void* x, uint32_t x_dtype, uint32_t m,
                                          uint32_t ldx, uint32_t rotate_act, void* act_f16, uint32_t ldact, uint32_t flags,
                                          void* workspace, size_t workspace_bytes) {
    int fmt = 0;
    qwhip_status st = gemm_checks(s, w, x, x_dtype, act_f16, QWHIP_F16, &fmt);
    if (st != QWHIP_OK) return st;
    if (m == 0) return QWHIP_OK;
    const uint32_t inter = w->n / 2u;
    if (w->n % 64u != 0) return qwhip_fail(QWHIP_E_BAD_GEOMETRY, "fused gate_up needs an intermediate size %% 32 == 0, got %u rows", w->n);
    if (ldx == 0) ldx = w->k;
    if (ldact == 0) ldact = inter;
    if (ldx < w->k || ldact < inter || (ldx % 8) != 0 || ldx >= (1u << 22) || (ldact % 8) != 0 || ((uintptr_t)act_f16 & 15u) != 0)
        return qwhip_fail(QWHIP_E_BAD_SHAPE, "bad leading dimensions or alignment (ldx=%u ldact=%u, act 16-byte aligned)", ldx, ldact);
    if ((uint64_t)w->n * qwhip_view_row_bytes(w) >= (1ull << 32))
        return qwhip_fail(QWHIP_E_BAD_GEOMETRY, "the fused gate_up GEMM addresses the bank with 32-bit offsets (bank under 4 GiB)");
    const bool rotate = qwhip_view_rotated(w) && !(flags & QWHIP_X_PREROTATED);
    const uint64_t ws_need = (uint64_t)m * w->k * 2u;
    const bool ws_ok = workspace && workspace_bytes >= ws_need && ldx == w->k && ((uintptr_t)workspace & 15u) == 0;
    const void* xin = x;
    if (rotate) {
        if (!ws_ok)
            return qwhip_fail(QWHIP_E_BASIS, "activations are not in the rotated basis: a 16-byte aligned workspace of %llu bytes and packed rows are needed",
                              (unsigned long long)ws_need);
        st = qwhip_fwht32(s, x, x_dtype, workspace, (uint64_t)m * w->k);
        if (st != QWHIP_OK) return st;
        xin = workspace;
    } else if (x_dtype == QWHIP_BF16) {
        if (!ws_ok) return qwhip_fail(QWHIP_E_BAD_GEOMETRY, "bf16 activations need the f16 workspace (%llu bytes, packed rows)", (unsigned long long)ws_need);
        st = qw_convert_to_f16(s, x, x_dtype, workspace, (uint64_t)m * w->k);
        if (st != QWHIP_OK) return st;
        xin = workspace;
    }
    qw_gemm_params p = {};
    p.bank = (const uint8_t*)w->blocks;
    p.x = xin;
    p.y = act_f16;
    p.M = m;
    p.N = w->n;
    p.K = w->k;
    p.ldx = ldx;
    p.ldy = ldact;
    p.gshift = log2_u32(w->group / 32);
    p.bb = qwhip_view_block_bytes(w);
    p.row_bytes = qwhip_view_row_bytes(w);
    p.inter = inter;
    p.rotate_act = rotate_act ? 1u : 0u;
    p.act = s->dev->act;
    // Few tiles and a workspace with room behind the activation copy for an f16 gate|up image and fp32 planes: the K-steps
    // of a tile are dealt over 2..8 workgroups as in qwhip_gemm, the planes are summed into the image and the SwiGLU pass
    // reads that - the two doors called one after the other, from one call.  flags bits 8..11 != 0 keep the one launch.
    {
        const uint64_t x_used = xin == workspace ? ((ws_need + 255u) & ~(uint64_t)255u) : 0u;
        const uint64_t gu_bytes = ((uint64_t)m * w->n * 2u + 255u) & ~(uint64_t)255u;
        uint32_t splits = 0;
        if (((flags >> 8) & 0xFu) == 0u && workspace && ((uintptr_t)workspace & 15u) == 0 && ldact == inter && workspace_bytes >= x_used + gu_bytes)
            splits = choose_splits(m, w->n, w->k, x_used + gu_bytes, workspace_bytes);
        if (splits != 0u) {
            void* gu = (uint8_t*)workspace + x_used;
            float* part = (float*)((uint8_t*)workspace + x_used + gu_bytes);
            hipError_t e;
            QG_FOR_FMT(fmt, e, (launch_splitk<F>(s->stream, p, splits, part, gu, QWHIP_F16, w->n)))
            QWHIP_TRY_HIP(e);
            return qwhip_swiglu_fwht(s, gu, QWHIP_F16, act_f16, m, inter, rotate_act);
        }
    }
    // The half-height tile where it is the cheaper one by the pricing of choose_cfg (0.78 of the big tile's efficiency per
    // area): up to 128 rows, where the big tile is half idle, and where it fills the chip and
    // the big tile does not (I = 17408: 129 .. 256 rows).  Same sums, same results either way.
    p.tiles_n = qwhip_cdiv(inter, 160u);
    const bool half = priced_rounds((double)qwhip_cdiv(m, 128u) * p.tiles_n, 256.0) / 0.78
                      < 2.0 * priced_rounds((double)qwhip_cdiv(m, 256u) * p.tiles_n, 256.0);
    p.tiles_m = qwhip_cdiv(m, half ? 128u : 256u);
    const dim3 grid(((p.tiles_m * p.tiles_n + 7u) / 8u) * 8u);
    hipError_t e;
    // the plain SwiGLU epilogue keeps its own instantiation: the general activation's code costs it 3 % at this size
    const bool ga = p.act.kind != 0u;
    switch (fmt) {
#define QG_SWIGLU3(F) \
    case F: e = half ? (ga ? launch_cfg3<1, 5, 4, 2, F, QWHIP_F16, true, QWHIP_F16, true>(s->stream, p, grid) \
                           : launch_cfg3<1, 5, 4, 2, F, QWHIP_F16, true>(s->stream, p, grid)) \
                     : (ga ? launch_cfg3<2, 5, 4, 2, F, QWHIP_F16, true, QWHIP_F16, true>(s->stream, p, grid) \
                           : launch_cfg3<2, 5, 4, 2, F, QWHIP_F16, true>(s->stream, p, grid)); break;
        QG_SWIGLU3(QG_FMT_M5) QG_SWIGLU3(QG_FMT_B4) QG_SWIGLU3(QG_FMT_B2) QG_SWIGLU3(QG_FMT_B3) QG_SWIGLU3(QG_FMT_B6) QG_SWIGLU3(QG_FMT_B8)
#undef QG_SWIGLU3
        default: e = hipErrorInvalidValue;
    }
    QWHIP_TRY_HIP(e);
    return QWHIP_OK;
}

// ---- grouped (MoE) -----------------------------------------------------------------------------
namespace {
template <int FMT, int XDT>
hipError_t launch_grouped_y(hipStream_t st, const qw_gemm_params& p, dim3 grid, uint32_t ydt) {
    if (ydt == QWHIP_F16) return launch_cfg<2, 2, 1, 4, FMT, XDT, QWHIP_F16, true>(st, p, grid);
    if (ydt == QWHIP_BF16) return launch_cfg<2, 2, 1, 4, FMT, XDT, QWHIP_BF16, true>(st, p, grid);
    return launch_cfg<2, 2, 1, 4, FMT, XDT, QWHIP_F32, true>(st, p, grid);
}
// direct-operand kernels on the 64 x 256 tiles of the list (weights dequantized straight into MFMA operand registers, only
// the activation tile in LDS); bf16 rows become f16 between the load registers and LDS
template <int FMT, int XDT>
hipError_t launch_grouped_direct(hipStream_t st, const qw_gemm_params& p, dim3 grid, uint32_t ydt) {
    qw_gemm_params q = p;
    q.tiles_n = grid.x;
    const dim3 grid1(8u * qwhip_cdiv(grid.y, 8u) * grid.x);   // XCD-aware one-dimensional grid over (tile, column tile)
    if (gemm5_takes(q, FMT)) {
        if (ydt == QWHIP_F16) return launch_cfg5<FMT, QWHIP_F16, false, false, XDT>(st, q, grid1);
        if (ydt == QWHIP_BF16) return launch_cfg5<FMT, QWHIP_BF16, false, false, XDT>(st, q, grid1);
        return launch_cfg5<FMT, QWHIP_F32, false, false, XDT>(st, q, grid1);
    }
    if (ydt == QWHIP_F16) return launch_cfg4<FMT, QWHIP_F16, false, false, XDT>(st, q, grid1);
    if (ydt == QWHIP_BF16) return launch_cfg4<FMT, QWHIP_BF16, false, false, XDT>(st, q, grid1);
    return launch_cfg4<FMT, QWHIP_F32, false, false, XDT>(st, q, grid1);
}
template <int FMT>
hipError_t launch_grouped_xy(hipStream_t st, const qw_gemm_params& p, dim3 grid, uint32_t xdt, uint32_t ydt) {
    if (!p.force_gemm2 && (ydt == QWHIP_F32 || (p.ldy % 8u == 0 && ((uintptr_t)p.y & 15u) == 0))) {
        if (xdt == QWHIP_F16) return launch_grouped_direct<FMT, QWHIP_F16>(st, p, grid, ydt);
        return launch_grouped_direct<FMT, QWHIP_BF16>(st, p, grid, ydt);
    }
    if (xdt == QWHIP_F16) {  // DMA-fed pipelined kernel, 64 x 256 tiles
        if (ydt == QWHIP_F16) return launch_cfg2<2, 2, 1, 4, FMT, QWHIP_F16, true>(st, p, grid);
        if (ydt == QWHIP_BF16) return launch_cfg2<2, 2, 1, 4, FMT, QWHIP_BF16, true>(st, p, grid);
        return launch_cfg2<2, 2, 1, 4, FMT, QWHIP_F32, true>(st, p, grid);
    }
    return launch_grouped_y<FMT, QWHIP_BF16>(st, p, grid, ydt);
}
// fused gate_up: the plain SwiGLU epilogue keeps its own instantiation (GACT = false)
template <int FMT, int XDT>
hipError_t launch_grouped_swiglu(hipStream_t st, const qw_gemm_params& p, dim3 grid, bool ga) {
    if (gemm5_takes(p, FMT)) {
        if (ga) return launch_cfg5<FMT, QWHIP_F16, true, true, XDT>(st, p, grid);
        return launch_cfg5<FMT, QWHIP_F16, true, false, XDT>(st, p, grid);
    }
    if (ga) return launch_cfg4<FMT, QWHIP_F16, true, true, XDT>(st, p, grid);
    return launch_cfg4<FMT, QWHIP_F16, true, false, XDT>(st, p, grid);
}
}  // namespace

extern "C" qwhip_status qwhip_moe_grouped_gemm(qwhip_stream_t s, const qwhip_weight_view* w, uint32_t experts, const void* x,
                                               uint32_t x_dtype, uint32_t ldx, const int32_t* gather,
                                               const int32_t* expert_off, const int32_t* tile_e, const int32_t* tile_r,
                                               const int32_t* tile_count, uint32_t max_tiles, uint32_t pairs, void* y,
                                               uint32_t y_dtype, uint32_t ldy) {
    int fmt = 0;
    qwhip_status st = gemm_checks(s, w, x, x_dtype, y, y_dtype, &fmt);
    if (st != QWHIP_OK) return st;
    QWHIP_REQUIRE(expert_off);
    QWHIP_REQUIRE(tile_e);
    QWHIP_REQUIRE(tile_r);
    QWHIP_REQUIRE(tile_count);
    if (experts == 0 || experts > 512 || w->n % experts != 0)
        return qwhip_fail(QWHIP_E_BAD_SHAPE, "grouped GEMM: %u rows do not split over %u experts (<= 512)", w->n, experts);
    if (pairs == 0 || max_tiles == 0) return QWHIP_OK;
    const uint32_t rows_per_expert = w->n / experts;
    if (rows_per_expert % 16 != 0)
        return qwhip_fail(QWHIP_E_BAD_GEOMETRY, "grouped GEMM needs rows per expert %% 16 == 0, got %u", rows_per_expert);
    if (ldx == 0) ldx = w->k;
    if (ldy == 0) ldy = rows_per_expert;
    if (ldx < w->k || ldy < rows_per_expert || (ldx % 8) != 0)
        return qwhip_fail(QWHIP_E_BAD_SHAPE, "bad leading dimensions ldx=%u ldy=%u", ldx, ldy);
    if ((uint64_t)pairs * ldx * 2u >= (1ull << 32))
        return qwhip_fail(QWHIP_E_BAD_SHAPE, "grouped GEMM addresses its activation rows with 32-bit offsets: %u rows of %u do not fit", pairs, ldx);
    if ((uint64_t)rows_per_expert * qwhip_view_row_bytes(w) >= (1ull << 32))
        return qwhip_fail(QWHIP_E_BAD_GEOMETRY, "grouped GEMM addresses an expert's rows with 32-bit offsets: %u rows do not fit", rows_per_expert);
    qw_gemm_params p = {};
    p.bank = (const uint8_t*)w->blocks;
    p.x = x;
    p.y = y;
    p.M = pairs;
    p.N = rows_per_expert;
    p.K = w->k;
    p.ldx = ldx;
    p.ldy = ldy;
    p.gshift = log2_u32(w->group / 32);
    p.bb = qwhip_view_block_bytes(w);
    p.row_bytes = qwhip_view_row_bytes(w);
    p.gather = gather;
    p.expert_off = expert_off;
    p.tile_e = tile_e;
    p.tile_r = tile_r;
    p.tile_count = tile_count;
    p.rows_per_expert = rows_per_expert;
    const dim3 grid(qwhip_cdiv(rows_per_expert, 256u), max_tiles);
    hipError_t e;
    QG_FOR_FMT(fmt, e, (launch_grouped_xy<F>(s->stream, p, grid, x_dtype, y_dtype)))
    QWHIP_TRY_HIP(e);
    return QWHIP_OK;
}

// Grouped gate|up GEMM with the SwiGLU (+ FWHT-32) epilogue fused: act f16 [pairs, inter] in sorted-pair order, bit-identical
// to qwhip_moe_grouped_gemm (f16 out) followed by qwhip_swiglu_fwht, without the [pairs, 2 inter] matrix in between.
extern "C" qwhip_status qwhip_moe_grouped_gemm_swiglu(qwhip_stream_t s, const qwhip_weight_view* w, uint32_t experts, const void* x,
                                                      uint32_t x_dtype, uint32_t ldx, const int32_t* gather,
                                                      const int32_t* expert_off, const int32_t* tile_e, const int32_t* tile_r,
                                                      const int32_t* tile_count, uint32_t max_tiles, uint32_t pairs,
                                                      uint32_t rotate_act, void* act_f16, uint32_t ldact) {
    int fmt = 0;
    qwhip_status st = gemm_checks(s, w, x, x_dtype, act_f16, QWHIP_F16, &fmt);
    if (st != QWHIP_OK) return st;
    QWHIP_REQUIRE(expert_off);
    QWHIP_REQUIRE(tile_e);
    QWHIP_REQUIRE(tile_r);
    QWHIP_REQUIRE(tile_count);
    if (experts == 0 || experts > 512 || w->n % experts != 0)
        return qwhip_fail(QWHIP_E_BAD_SHAPE, "grouped GEMM: %u rows do not split over %u experts (<= 512)", w->n, experts);
    if (pairs == 0 || max_tiles == 0) return QWHIP_OK;
    const uint32_t rows_per_expert = w->n / experts, inter = rows_per_expert / 2u;
    if (rows_per_expert % 64u != 0)
        return qwhip_fail(QWHIP_E_BAD_GEOMETRY, "fused gate_up needs an intermediate size %% 32 == 0, got %u rows per expert", rows_per_expert);
    if (ldx == 0) ldx = w->k;
    if (ldact == 0) ldact = inter;
    if (ldx < w->k || ldact < inter || (ldx % 8) != 0 || (ldact % 8) != 0 || ((uintptr_t)act_f16 & 15u) != 0)
        return qwhip_fail(QWHIP_E_BAD_SHAPE, "bad leading dimensions or alignment (ldx=%u ldact=%u, act 16-byte aligned)", ldx, ldact);
    if ((uint64_t)pairs * ldx * 2u >= (1ull << 32))
        return qwhip_fail(QWHIP_E_BAD_SHAPE, "grouped GEMM addresses its activation rows with 32-bit offsets: %u rows of %u do not fit", pairs, ldx);
    if ((uint64_t)rows_per_expert * qwhip_view_row_bytes(w) >= (1ull << 32))
        return qwhip_fail(QWHIP_E_BAD_GEOMETRY, "grouped GEMM addresses an expert's rows with 32-bit offsets: %u rows do not fit", rows_per_expert);
    qw_gemm_params p = {};
    p.bank = (const uint8_t*)w->blocks;
    p.x = x;
    p.y = act_f16;
    p.M = pairs;
    p.N = rows_per_expert;
    p.K = w->k;
    p.ldx = ldx;
    p.ldy = ldact;
    p.gshift = log2_u32(w->group / 32);
    p.bb = qwhip_view_block_bytes(w);
    p.row_bytes = qwhip_view_row_bytes(w);
    p.gather = gather;
    p.expert_off = expert_off;
    p.tile_e = tile_e;
    p.tile_r = tile_r;
    p.tile_count = tile_count;
    p.rows_per_expert = rows_per_expert;
    p.inter = inter;
    p.rotate_act = rotate_act ? 1u : 0u;
    p.act = s->dev->act;
    p.tiles_n = qwhip_cdiv(inter, 128u);
    const dim3 grid(8u * qwhip_cdiv(max_tiles, 8u) * p.tiles_n);   // XCD-aware one-dimensional grid over (tile, column tile)
    hipError_t e;
    const bool ga = p.act.kind != 0u;
    if (x_dtype == QWHIP_F16) {
        QG_FOR_FMT(fmt, e, (launch_grouped_swiglu<F, QWHIP_F16>(s->stream, p, grid, ga)))
    } else {
        QG_FOR_FMT(fmt, e, (launch_grouped_swiglu<F, QWHIP_BF16>(s->stream, p, grid, ga)))
    }
    QWHIP_TRY_HIP(e);
    return QWHIP_OK;
}
