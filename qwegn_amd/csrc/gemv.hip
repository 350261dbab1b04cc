// Decode / verify GEMV over quantized banks: y[m, n] = sum_k W[n, k] * x[m, k], m in 1..16.
//
// Two kernel families, both HBM-bound streamers that read every weight byte once:
//
//  * qw_gemv_hq4_dot2_kernel - HQ4_G32_M5, m = 1.  A 32-lane half-wavefront owns R rows; lane l
//    owns blocks l, l+32, ... of each row (640 contiguous bytes per half-wave per step).  The rotated
//    activation lives in LDS (80-byte pitch per 32-group, so 128-bit reads are bank-conflict free) and
//    is reused across the R rows.  Weights are materialised as exact f16 (one packed f16 FMA) and
//    contracted with v_dot2_f32_f16 into fp32.
//
//  * qw_gemv_mfma_kernel - every container, m = 1..16.  A wavefront owns 16*RT rows; lane (i, c) =
//    (lane & 15, lane >> 4) owns 32-column slice 4*it + c of row i of each row tile, dequantizes it to
//    four 8-wide f16 MFMA A operands, and v_mfma_f32_16x16x32_f16 contracts them against the m
//    activation rows held as B operands (column j = m).  The 4 waves of a workgroup split K and reduce
//    through LDS.  VALU does only the dequant; accumulation rides on the matrix cores.
#include <atomic>

#include <type_traits>

#include "qwhip_common.h"

enum { QW_XM_GLOBAL = 0, QW_XM_LDS_ROT = 1 };

// ------------------------------------------------------------------------------------------------
// Rotated-activation staging: group g of row m -> 4 x 16 bytes at LDS offset m*pitch + g*gpitch.
// ------------------------------------------------------------------------------------------------
template <int XDT>
__device__ __forceinline__ void qw_stage_group(const void* x, uint64_t elem0, bool rotate, h8_t* dst) {
    float v[32];
#pragma unroll
    for (int j = 0; j < 4; ++j) qw_load8_f32<XDT>(x, elem0 + 8 * j, v + 8 * j);
    if (rotate) qw_fwht32(v);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        h8_t o;
#pragma unroll
        for (int e = 0; e < 8; ++e) o[e] = (h1_t)v[8 * j + e];
        dst[j] = o;
    }
}

// ------------------------------------------------------------------------------------------------
// Variant A: HQ4_G32_M5, m = 1, dot2.
// Order of issue matters more than instruction count here: the whole kernel is one "breath" of about
// ten microseconds, loads return in order, and nothing can be contracted before the rotated activation
// is in LDS.  So: the activation loads go first, then every weight load of the wave (NB blocks per lane
// per row, all in flight at once), then the rotation (matrix cores), the barrier, and the contraction as
// data arrive.  NB = 0 selects the looped form for rows longer than 8192 columns.
// ------------------------------------------------------------------------------------------------
template <int R, int NB, int XDT>
__global__ __launch_bounds__(256) void qw_gemv_hq4_dot2_kernel(const uint8_t* __restrict__ bank,
                                                                const void* __restrict__ x, h1_t* __restrict__ y16,
                                                                float* __restrict__ y32, uint32_t N, uint32_t K,
                                                                uint32_t rotate) {
    extern __shared__ h8_t xs[];  // 5 h8 per 32-group (4 used): 80-byte pitch
    const uint32_t nb = K >> 5;
    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & 31u;
    const uint32_t wave = tid >> 6, l64 = tid & 63u;
    const uint32_t row0 = (blockIdx.x * 8u + (tid >> 5)) * R;
    const uint32_t ngt = (nb + 15u) >> 4;  // 16-group tiles of the activation

    // 1. activation loads: tiles wave, wave + 4, ... (one 16-byte load per lane and tile)
    constexpr int XT = NB > 0 ? (NB + 1) / 2 : 1;
    h8_t xb[XT];
    if constexpr (NB > 0) {
#pragma unroll
        for (int t = 0; t < XT; ++t) {
            const uint32_t gt = wave + 4u * t;
            const uint32_t g = min(gt * 16u + (l64 & 15u), nb - 1);
            xb[t] = qw_load_x8_f16<XDT>(x, (uint64_t)g * 32u + 8u * (l64 >> 4));
        }
    }
    // 2. weight loads
    const uint8_t* rp[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const uint32_t row = (row0 + r < N) ? row0 + r : N - 1;
        rp[r] = bank + (uint64_t)row * nb * 20u;
    }
    constexpr int NBH = NB > 0 ? NB : 1;
    qw_hq4_block hb[NBH][R];
    if constexpr (NB > 0) {
#pragma unroll
        for (int it = 0; it < NB; ++it) {
            uint32_t g = lane + 32u * it;
            if (g >= nb) g = nb - 1;
#pragma unroll
            for (int r = 0; r < R; ++r) hb[it][r] = *(const qw_hq4_block*)(rp[r] + g * 20u);
        }
    }
    // 3. rotation into LDS
    {
        const h8_t h_lo = qw_hadamard_rows(l64 & 15u, l64 >> 4);
        const h8_t h_hi = qw_hadamard_rows((l64 & 15u) + 16u, l64 >> 4);
        if constexpr (NB > 0) {
#pragma unroll
            for (int t = 0; t < XT; ++t) {
                const uint32_t gt = wave + 4u * t;
                if (gt < ngt) qw_rotate_tile_to_lds(xb[t], gt, nb, l64, rotate != 0, h_lo, h_hi, xs);
            }
        } else {
            for (uint32_t gt = wave; gt < ngt; gt += 4) {
                const uint32_t g = min(gt * 16u + (l64 & 15u), nb - 1);
                const h8_t v = qw_load_x8_f16<XDT>(x, (uint64_t)g * 32u + 8u * (l64 >> 4));
                qw_rotate_tile_to_lds(v, gt, nb, l64, rotate != 0, h_lo, h_hi, xs);
            }
        }
    }
    __syncthreads();
    if (row0 >= N) return;

    const uint32_t magic = qw_vgpr_const(0x64006400u);
    float acc[R];
#pragma unroll
    for (int r = 0; r < R; ++r) acc[r] = 0.0f;

    auto contract = [&](const qw_hq4_block* b, uint32_t g) {
        h8_t xv[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) xv[j] = xs[g * 5 + j];
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const h2_t s2 = qw_splat_lo(b[r].hdr), b2 = qw_splat_hi(b[r].hdr);
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                h2_t w[4];
                qw_unpack_hq4_word(b[r].qs[j], s2, b2, magic, w);
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    const h2_t xp = {xv[j][2 * k], xv[j][2 * k + 1]};
                    acc[r] = __builtin_amdgcn_fdot2(w[k], xp, acc[r], false);
                }
            }
        }
    };
    if constexpr (NB > 0) {
#pragma unroll
        for (int it = 0; it < NB; ++it) {
            const uint32_t g = lane + 32u * it;
            if (g < nb) contract(hb[it], g);
        }
    } else {
        for (uint32_t g = lane; g < nb; g += 32) {
            qw_hq4_block b[R];
#pragma unroll
            for (int r = 0; r < R; ++r) b[r] = *(const qw_hq4_block*)(rp[r] + g * 20u);
            contract(b, g);
        }
    }
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const float v = qw_reduce32(acc[r]);
        if (lane == 0 && row0 + r < N) {
            if (y32) y32[row0 + r] = v;
            if (y16) y16[row0 + r] = (h1_t)v;
        }
    }
}

// ------------------------------------------------------------------------------------------------
// Variant B: MFMA streamer, all containers, m = 1..16.
// ------------------------------------------------------------------------------------------------
// code words of one 32-column slice (= the bit width)
template <int FMT>
__host__ __device__ constexpr int qw_slice_words() {
    return FMT == QW_FMT_B8 ? 8 : FMT == QW_FMT_B2 ? 2 : FMT == QW_FMT_B3 ? 3 : FMT == QW_FMT_B6 ? 6 : 4;
}

template <int FMT>
struct qw_slice {
    uint32_t hdr;
    uint32_t q[qw_slice_words<FMT>()];
};

struct __attribute__((packed, aligned(4))) qw_words4 { uint32_t q[4]; };
struct __attribute__((packed, aligned(4))) qw_words8 { uint32_t q[8]; };
template <int W>
struct __attribute__((packed, aligned(4))) qw_words_n { uint32_t q[W]; };

// Position e of an A operand holds element perm(e) of the 8-column chunk.
template <int FMT>
__device__ __forceinline__ constexpr int qw_perm(int e) {
    if (FMT == QW_FMT_M5 || FMT >= QW_FMT_B2) return e;        // 2-, 3- and 6-bit streams are cut out in natural order
    if (FMT == QW_FMT_B4) return (e >> 1) + 4 * (e & 1);      // 0,4,1,5,2,6,3,7
    return (e & 4) + ((e & 1) << 1) + ((e >> 1) & 1);         // 0,2,1,3,4,6,5,7
}

// Loads slice `s` (32 columns) of the row at `rowp`.  gshift = log2(group / 32).
template <int FMT>
__device__ __forceinline__ void qw_load_slice(const uint8_t* rowp, uint32_t s, uint32_t gshift, uint32_t bb,
                                              qw_slice<FMT>& o) {
    if constexpr (FMT == QW_FMT_M5) {
        const qw_hq4_block b = *(const qw_hq4_block*)(rowp + s * 20u);
        o.hdr = b.hdr;
#pragma unroll
        for (int j = 0; j < 4; ++j) o.q[j] = b.qs[j];
    } else {
        const uint8_t* p = rowp + (uint64_t)(s >> gshift) * bb;
        const uint32_t si = s & ((1u << gshift) - 1u);
        o.hdr = *(const uint32_t*)p;
        if constexpr (FMT == QW_FMT_B4) {
            const qw_words4 w = *(const qw_words4*)(p + 4 + si * 16u);
#pragma unroll
            for (int j = 0; j < 4; ++j) o.q[j] = w.q[j];
        } else if constexpr (FMT == QW_FMT_B8) {
            const qw_words8 w = *(const qw_words8*)(p + 4 + si * 32u);
#pragma unroll
            for (int j = 0; j < 8; ++j) o.q[j] = w.q[j];
        } else {
            // 2-, 3- and 6-bit streams: a slice is `bits` words at a 4-byte aligned offset of the block
            constexpr int W = qw_slice_words<FMT>();
            const uint8_t* src = p + 4 + si * (4u * W);
            if constexpr (W == 6) {
                const qw_words4 w0 = *(const qw_words4*)src;
                const qw_words_n<2> w1 = *(const qw_words_n<2>*)(src + 16);
#pragma unroll
                for (int j = 0; j < 4; ++j) o.q[j] = w0.q[j];
                o.q[4] = w1.q[0];
                o.q[5] = w1.q[1];
            } else {
                const qw_words_n<W> w = *(const qw_words_n<W>*)src;
#pragma unroll
                for (int j = 0; j < W; ++j) o.q[j] = w.q[j];
            }
        }
    }
}

// Dequantizes chunk j (8 columns) of a slice into an MFMA A operand of exact f16 weights:
// RN_f16((1024+q)*s + b) for HQ4_G32_M5, RN_f16(code*s + b) for bit-stream blocks (the magic 1024 is
// stripped exactly before the single f16 FMA, as qwg_aq_frag8 does,
// Sources/QWMetal/include/qw_gemm_nax.metalh:61-71).
template <int FMT>
__device__ __forceinline__ h8_t qw_dequant_chunk(const qw_slice<FMT>& sl, int j, h2_t s2, h2_t b2, uint32_t magic) {
    h2_t w[4];
    if constexpr (FMT == QW_FMT_M5) {
        qw_unpack_hq4_word(sl.q[j], s2, b2, magic, w);
    } else if constexpr (FMT == QW_FMT_B4) {
        const h2_t neg = {(h1_t)-1024.0f, (h1_t)-1024.0f};
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const uint32_t m = qw_and_or(sl.q[j] >> (4 * k), 0x000F000Fu, magic);
            w[k] = __builtin_elementwise_fma(__builtin_bit_cast(h2_t, m) + neg, s2, b2);
        }
    } else if constexpr (FMT >= QW_FMT_B2) {
        // the chunk's 8 codes are the 8 W bits from bit 8 W j of the slice; j is a constant after unrolling, and the word
        // picks are select chains over constant indices so that they never become an indexed (scratch memory) access
        constexpr int W = qw_slice_words<FMT>();
        const h2_t neg = {(h1_t)-1024.0f, (h1_t)-1024.0f};
        const int o = 8 * W * j, wi = o >> 5, sh = o & 31;
        uint32_t lo32 = 0, hi32 = 0;
#pragma unroll
        for (int t = 0; t < W; ++t) {
            lo32 = wi == t ? sl.q[t] : lo32;
            hi32 = wi + 1 == t ? sl.q[t] : hi32;
        }
        const uint64_t win = ((uint64_t)lo32 | ((uint64_t)hi32 << 32)) >> sh;
        constexpr uint32_t mask = (1u << W) - 1u;
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const uint32_t c0 = (uint32_t)(win >> (2 * k * W)) & mask, c1 = (uint32_t)(win >> ((2 * k + 1) * W)) & mask;
            w[k] = __builtin_elementwise_fma(__builtin_bit_cast(h2_t, c0 | (c1 << 16) | magic) + neg, s2, b2);
        }
    } else {
        const h2_t neg = {(h1_t)-1024.0f, (h1_t)-1024.0f};
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const uint32_t q = sl.q[2 * j + h];
            const uint32_t m0 = qw_and_or(q, 0x00FF00FFu, magic);
            const uint32_t m1 = qw_and_or(q >> 8, 0x00FF00FFu, magic);
            w[2 * h] = __builtin_elementwise_fma(__builtin_bit_cast(h2_t, m0) + neg, s2, b2);
            w[2 * h + 1] = __builtin_elementwise_fma(__builtin_bit_cast(h2_t, m1) + neg, s2, b2);
        }
    }
    h8_t a = {w[0][0], w[0][1], w[1][0], w[1][1], w[2][0], w[2][1], w[3][0], w[3][1]};
    return a;
}

template <int FMT>
__device__ __forceinline__ h8_t qw_x_operand(const h8_t* xg, int j) {
    h8_t b;
#pragma unroll
    for (int e = 0; e < 8; ++e) b[e] = xg[j][qw_perm<FMT>(e)];
    return b;
}

// The K loop of one wavefront: rows rp[0..NACC) (one 16-row tile each, this lane's row already folded
// in), K range of this wave (a quarter of the iterations), activations from LDS (XM = LDS_ROT) or
// global memory.  acc[t] += W_t . x over the wave's K range.
template <int FMT, int NACC, int XDT, int XM>
__device__ __forceinline__ void qw_stream_rows(const uint8_t* const* rp, const void* x, const h8_t* xs, uint32_t xpitch8,
                                               uint32_t K, uint32_t M, uint32_t gshift, uint32_t bb, bool rotate,
                                               uint32_t wave, uint32_t i, uint32_t c, uint32_t magic, f4_t* acc, uint32_t nw = 4,
                                               const qw_slice<FMT>* first = nullptr) {
    const uint32_t nsl = K >> 5;
    const uint32_t iters = (nsl + 3) >> 2;
    const uint32_t per = (iters + nw - 1u) / nw;
    const uint32_t it0 = wave * per;
    const uint32_t it1 = min(it0 + per, iters);
    qw_slice<FMT> cur[NACC] = {}, nxt[NACC] = {};
    if (first) {
#pragma unroll
        for (int t = 0; t < NACC; ++t) cur[t] = first[t];
    } else if (it0 < it1) {
        const uint32_t s = min(4u * it0 + c, nsl - 1);
#pragma unroll
        for (int t = 0; t < NACC; ++t) qw_load_slice<FMT>(rp[t], s, gshift, bb, cur[t]);
    }
    for (uint32_t it = it0; it < it1; ++it) {
        const uint32_t s = 4u * it + c;
        const bool valid = s < nsl;
        if (it + 1 < it1) {
            const uint32_t sn = min(s + 4u, nsl - 1);
#pragma unroll
            for (int t = 0; t < NACC; ++t) qw_load_slice<FMT>(rp[t], sn, gshift, bb, nxt[t]);
        }
        h8_t xg[4];
        if (valid && i < M) {
            if constexpr (XM == QW_XM_LDS_ROT) {
#pragma unroll
                for (int j = 0; j < 4; ++j) xg[j] = xs[i * xpitch8 + s * 4 + j];
            } else {
                qw_stage_group<XDT>(x, (uint64_t)i * K + 32u * s, rotate, xg);
            }
        } else {
#pragma unroll
            for (int j = 0; j < 4; ++j) xg[j] = h8_t{0, 0, 0, 0, 0, 0, 0, 0};
        }
        h8_t bop[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) bop[j] = qw_x_operand<FMT>(xg, j);
#pragma unroll
        for (int t = 0; t < NACC; ++t) {
            const h2_t s2 = qw_splat_lo(cur[t].hdr), b2 = qw_splat_hi(cur[t].hdr);
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const h8_t a = qw_dequant_chunk<FMT>(cur[t], j, s2, b2, magic);
                acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, bop[j], acc[t], 0, 0, 0);
            }
        }
#pragma unroll
        for (int t = 0; t < NACC; ++t) cur[t] = nxt[t];
    }
}

// The first iteration's loads of qw_stream_rows, for callers that want them in flight before their own prologue ends
// (the slice index is clamped: a wave with no iterations loads a valid slice it never uses).
template <int FMT, int NACC>
__device__ __forceinline__ void qw_stream_first(const uint8_t* const* rp, uint32_t K, uint32_t gshift, uint32_t bb, uint32_t wave,
                                                uint32_t c, uint32_t nw, qw_slice<FMT>* first) {
    const uint32_t nsl = K >> 5;
    const uint32_t iters = (nsl + 3) >> 2;
    const uint32_t per = (iters + nw - 1u) / nw;
    const uint32_t s = min(4u * wave * per + c, nsl - 1);
#pragma unroll
    for (int t = 0; t < NACC; ++t) qw_load_slice<FMT>(rp[t], s, gshift, bb, first[t]);
}

// idx .. out: the routed (MoE decode) modes; expert_bytes: bytes of one expert's sub-bank.  wpr, sets, nkr: the transposing
// kernel's waves per row set, row sets per workgroup, K ranges.
#define QGV_FIELDS(X)                                                                                                        \
    X(const uint8_t*, bank) X(const void*, x) X(h1_t*, y16) X(float*, y32) X(uint32_t, N) X(uint32_t, K) X(uint32_t, M)          \
    X(uint32_t, gshift) X(uint32_t, bb) X(uint64_t, row_bytes) X(uint32_t, rotate) X(uint32_t, rot_out) X(const int32_t*, idx)   \
    X(const float*, wts) X(uint32_t, top_k) X(uint64_t, expert_bytes) X(const float*, shared) X(const float*, shared_gate)       \
    X(void*, out) X(uint32_t, wpr) X(uint32_t, sets) X(uint32_t, nkr)
QW_ARG_BLOCK(qw_gemv_params, QGV_FIELDS)
// What only the gate|up pair and routed kernels read.  They take the longer argument block; the plain GEMV kernels keep
// the short one (the longer block alone cost the transposing kernel 1.8 % on N = 7168, K = 5120, m = 16 in a same-box
// comparison).  x_rows (gate|up): activation row of every pair (NULL: the pair's token); x_div (down): pairs that share one
// activation row (0 and 1: a row per pair); labels, num_groups > 0 (down): group of every expert; blockIdx.y = token *
// num_groups + group and only the token's routes into that group are summed; act (pair mode): the device's gated activation.
#define QGVX_FIELDS(X) \
    QGV_FIELDS(X) X(const int32_t*, x_rows) X(uint32_t, x_div) X(const int32_t*, labels) X(uint32_t, num_groups) X(qw_act, act)
QW_ARG_BLOCK(qw_gemv_params_x, QGVX_FIELDS)
inline qw_gemv_params qw_gemv_base(const qw_gemv_params_x& a) {
    qw_gemv_params p;
#define QGV_TAKE(T, n) p.n = a.n;
    QGV_FIELDS(QGV_TAKE)
#undef QGV_TAKE
    return p;
}

// PAIR = 1: gate|up pair mode.  The bank holds 2*N rows ([0, N) gate, [N, 2N) up); both are accumulated
// and the epilogue stores act[m, n] = f16(FWHT32(silu(g) * u)) (rotation optional).
// ROUTED = 1 (with PAIR): blockIdx.y is a (token, route) pair; the expert's sub-bank is picked through
// idx[pair], the activation row is the pair's token, the output row is the pair.
template <int FMT, int RT, int XDT, int XM, int PAIR, int ROUTED, int NWV = 4>
struct qw_gemv_mfma_kernel {
typedef typename std::conditional<(PAIR || ROUTED), qw_gemv_params_x, qw_gemv_params>::type params_t;
static constexpr int kLaunchBound = 64 * NWV;
static __device__ __forceinline__ void run(const params_t& p) {
    constexpr uint32_t NTH = 64 * NWV;
    constexpr int NACC = RT * (PAIR ? 2 : 1);
    extern __shared__ h8_t xs[];
    __shared__ f4_t red[NWV][NACC][64];
    const uint32_t tid = threadIdx.x;
    const uint32_t wave = tid >> 6, lane = tid & 63u;
    const uint32_t i = lane & 15u, c = lane >> 4;
    const uint32_t N = p.N, K = p.K, M = p.M;
    const uint32_t nsl = K >> 5;
    const uint32_t xpitch8 = (K >> 3) + 1;  // LDS row pitch in h8 units: K*2 + 16 bytes
    const uint32_t n0 = blockIdx.x * (16u * RT);

    const uint8_t* bank = p.bank;
    const void* x = p.x;
    h1_t* y16 = p.y16;
    // Order of the prologue's memory traffic: the route's expert id first, the activation staging (which does not
    // need it) behind it, then the first weight slices, and only then the barrier that publishes the staged
    // activations: the three round trips overlap instead of queueing.
    int32_t e = 0;
    if constexpr (ROUTED) {
        const uint32_t pair = blockIdx.y;
        e = p.idx[pair];
        y16 += (uint64_t)pair * N;
        const uint32_t xrow = p.x_rows ? (uint32_t)max(p.x_rows[pair], 0) : pair / p.top_k;
        x = (const uint8_t*)x + (uint64_t)xrow * K * 2u;
    }
    if constexpr (XM == QW_XM_LDS_ROT) {
        for (uint32_t idx = tid; idx < M * nsl; idx += NTH) {
            const uint32_t m = idx / nsl, g = idx - m * nsl;
            qw_stage_group<XDT>(x, (uint64_t)m * K + 32u * g, p.rotate != 0, xs + m * xpitch8 + g * 4);
        }
    }
    if constexpr (ROUTED) {
        if (e < 0) {  // no expert: the pair contributes nothing (uniform over the workgroup, before any barrier)
            for (uint32_t n = n0 + tid; n < min(n0 + 16u * RT, N); n += NTH) y16[n] = (h1_t)0.0f;
            return;
        }
        bank += (uint64_t)((uint32_t)e & 0xFFFFu) * p.expert_bytes;
    }

    const uint8_t* rp[NACC];
#pragma unroll
    for (int t = 0; t < RT; ++t) {
        uint32_t row = n0 + 16u * t + i;
        if (row >= N) row = N - 1;
        rp[t] = bank + (uint64_t)row * p.row_bytes;
        if (PAIR) rp[RT + t] = bank + (uint64_t)(row + N) * p.row_bytes;
    }
    qw_slice<FMT> first[NACC];
    qw_stream_first<FMT, NACC>(rp, K, p.gshift, p.bb, wave, c, NWV, first);
    if constexpr (XM == QW_XM_LDS_ROT) __syncthreads();
    f4_t acc[NACC];
#pragma unroll
    for (int t = 0; t < NACC; ++t) acc[t] = f4_t{0.f, 0.f, 0.f, 0.f};
    const uint32_t magic = qw_vgpr_const(0x64006400u);
    qw_stream_rows<FMT, NACC, XDT, XM>(rp, x, xs, xpitch8, K, M, p.gshift, p.bb, p.rotate != 0, wave, i, c, magic, acc, NWV, first);

    // split-K reduction: D[row 4c + r][col i] of every wave -> wave 0
#pragma unroll
    for (int t = 0; t < NACC; ++t) red[wave][t][lane] = acc[t];
    __syncthreads();
    if constexpr (!PAIR) {
        if (wave != 0) return;
#pragma unroll
        for (int t = 0; t < RT; ++t) {
            f4_t v = red[0][t][lane];
#pragma unroll
            for (int w2 = 1; w2 < NWV; ++w2) v += red[w2][t][lane];
            if (i < M) {
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const uint32_t n = n0 + 16u * t + 4u * c + r;
                    if (n < N) {
                        if (p.y32) p.y32[(uint64_t)i * N + n] = v[r];
                        if (y16) y16[(uint64_t)i * N + n] = (h1_t)v[r];
                    }
                }
            }
        }
    } else {
        // SwiGLU on the fp32 sums, then (RT == 2: the workgroup's 32 rows are one 32-group) FWHT-32.
        __shared__ float actbuf[16][16 * RT + 1];
        if (wave == 0) {
#pragma unroll
            for (int t = 0; t < RT; ++t) {
                f4_t g = red[0][t][lane], u = red[0][RT + t][lane];
#pragma unroll
                for (int w2 = 1; w2 < NWV; ++w2) {
                    g += red[w2][t][lane];
                    u += red[w2][RT + t][lane];
                }
#pragma unroll
                for (int r = 0; r < 4; ++r) actbuf[i][16 * t + 4 * c + r] = qw_gated(g[r], u[r], p.act);
            }
        }
        __syncthreads();
        if (tid < M) {
            if constexpr (RT == 2) {
                float v[32];
#pragma unroll
                for (int e = 0; e < 32; ++e) v[e] = actbuf[tid][e];
                if (p.rot_out && n0 + 32u <= N) qw_fwht32(v);
#pragma unroll
                for (int e = 0; e < 32; ++e)
                    if (n0 + e < N) y16[(uint64_t)tid * N + n0 + e] = (h1_t)v[e];
            } else {
                for (int e = 0; e < 16 * RT; ++e)
                    if (n0 + e < N) y16[(uint64_t)tid * N + n0 + e] = (h1_t)actbuf[tid][e];
            }
        }
    }
}
};

// Routed down projection of the decode path: blockIdx.y is a token; the workgroup's 16*RT output rows
// accumulate sum_k wts[t, k] * (W_down[e_k] . act[t, k]) over the token's routes, add the gated shared
// expert, and store.  Activations (SwiGLU output) are already in the rotated basis.
// Wave w takes routes w, w + 8, ... whole (every route is a short row: its loads are all in flight at once and the
// routes of a token stream side by side instead of one after the other); the route partials meet in LDS and are
// summed in wave order.
template <int FMT, int RT, int ODT>
struct qw_moe_down_decode_kernel {
static constexpr int kLaunchBound = 512;
static __device__ __forceinline__ void run(const qw_gemv_params_x& p) {
    __shared__ f4_t red[8][RT][64];
    const uint32_t tid = threadIdx.x;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63u;
    const uint32_t i = lane & 15u, c = lane >> 4;
    const uint32_t N = p.N, K = p.K;
    const uint32_t n0 = blockIdx.x * (16u * RT);
    const uint32_t tok = blockIdx.y;   // the output row
    // group mode: num_groups carries the group count in its low byte and the expert count (the length of labels) above it
    const uint32_t ng = p.num_groups & 0xFFu, n_experts = p.num_groups >> 8;
    const uint32_t src = ng ? tok / ng : tok;
    const int32_t grp = ng ? (int32_t)(tok - src * ng) : 0;
    const uint32_t magic = qw_vgpr_const(0x64006400u);
    f4_t total[RT];
#pragma unroll
    for (int t = 0; t < RT; ++t) total[t] = f4_t{0.f, 0.f, 0.f, 0.f};
    for (uint32_t k = wave; k < p.top_k; k += 8u) {
        const uint32_t pair = src * p.top_k + k;
        const int32_t e = p.idx[pair];
        if (e < 0) continue;
        if (ng && (((uint32_t)e & 0xFFFFu) >= n_experts || p.labels[(uint32_t)e & 0xFFFFu] != grp)) continue;   // an id past the labels is no route
        const float wk = p.wts ? p.wts[pair] : 1.0f;
        const uint8_t* bank = p.bank + (uint64_t)((uint32_t)e & 0xFFFFu) * p.expert_bytes;
        const uint8_t* rp[RT];
#pragma unroll
        for (int t = 0; t < RT; ++t) {
            uint32_t row = n0 + 16u * t + i;
            if (row >= N) row = N - 1;
            rp[t] = bank + (uint64_t)row * p.row_bytes;
        }
        f4_t acc[RT];
#pragma unroll
        for (int t = 0; t < RT; ++t) acc[t] = f4_t{0.f, 0.f, 0.f, 0.f};
        const void* x = (const uint8_t*)p.x + (uint64_t)(p.x_div > 1u ? pair / p.x_div : pair) * K * 2u;
        qw_stream_rows<FMT, RT, QWHIP_F16, QW_XM_GLOBAL>(rp, x, nullptr, 0, K, 1, p.gshift, p.bb, false, 0u, i, c, magic, acc, 1u);
#pragma unroll
        for (int t = 0; t < RT; ++t) total[t] += acc[t] * wk;
    }
#pragma unroll
    for (int t = 0; t < RT; ++t) red[wave][t][lane] = total[t];
    __syncthreads();
    if (wave != 0 || i != 0) return;
#pragma unroll
    for (int t = 0; t < RT; ++t) {
        f4_t v = red[0][t][lane];
#pragma unroll
        for (int w2 = 1; w2 < 8; ++w2) v += red[w2][t][lane];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const uint32_t n = n0 + 16u * t + 4u * c + r;
            if (n < N) {
                float o = v[r];
                const uint64_t at = (uint64_t)tok * N + n;
                if (p.shared) o = fmaf(p.shared_gate ? p.shared_gate[tok] : 1.0f, p.shared[at], o);
                if constexpr (ODT == QWHIP_F32) ((float*)p.out)[at] = o;
                else if constexpr (ODT == QWHIP_F16) ((h1_t*)p.out)[at] = (h1_t)o;
                else ((uint16_t*)p.out)[at] = qw_f32_to_bf16(o);
            }
        }
    }
}
};

// ------------------------------------------------------------------------------------------------
// Variant C: column-stationary MFMA kernel, all containers, m = 1..16, activations already in the container's basis,
// rows of at most 40 K-iterations (k <= 5120).
// One workgroup of 8 waves per compute unit walks the row tiles (16 rows) blockIdx.x, blockIdx.x + gridDim.x, ... so
// the whole grid reads one contiguous band of rows at a time.  Wave w owns K-iterations [w * IPW, (w + 1) * IPW)
// (an iteration = 4 slices of 32 columns; lane (i, c) holds slice 4*it + c of row i) for every row tile, so its
// activation operands - the B operands of v_mfma_f32_16x16x32_f16, column j = activation row - are loaded once and
// stay in registers: no activation traffic in the row loop, whatever m is.  The packed blocks of the next row tile
// are fetched while the current one is dequantized and contracted; the 8 partial 16 x 16 tiles meet in LDS.
// What bounds it today: the MFMA operand layout makes consecutive lanes hold different rows, so every load
// instruction touches 16 rows (about 40 cache lines) and the address unit, not HBM, sets the pace (16 us on
// N = 7168, K = 5120 in 36-byte blocks; the same bytes stream in about 7 us when lanes read consecutive blocks).
// ------------------------------------------------------------------------------------------------
template <int FMT, int XDT, int IPW>
__global__ __launch_bounds__(512) void qw_gemv_colm_kernel(const qw_gemv_params p) {
    __shared__ float red[2][8][64][4];
    const uint32_t tid = threadIdx.x;
    const uint32_t wave = tid >> 6, lane = tid & 63u;
    const uint32_t i = lane & 15u, c = lane >> 4;
    const uint32_t N = p.N, K = p.K, M = p.M;
    const uint32_t nsl = K >> 5;
    const uint32_t tiles = (N + 15u) >> 4;
    const uint32_t magic = qw_vgpr_const(0x64006400u);

    // ---- this wave's activation operands: xop[u][j] = columns 8j..8j+7 of slice 4*(wave*IPW + u) + c of row i.
    // Their loads go out first, the first row tile's loads right behind them (issued before any of the activation
    // data is touched), so the prologue costs one memory round trip, not two.
    h8_t xraw[IPW][4], xop[IPW][4];
    uint32_t sl[IPW];   // slice index per iteration (clamped; invalid slices carry zero operands)
#pragma unroll
    for (int u = 0; u < IPW; ++u) {
        sl[u] = min(4u * (wave * IPW + u) + c, nsl - 1u);
        const uint64_t at = (uint64_t)min(i, M - 1u) * K + 32u * sl[u];   // clamped address: no branches around the loads
#pragma unroll
        for (int j = 0; j < 4; ++j) xraw[u][j] = qw_load_x8_f16<XDT>(p.x, at + 8u * j);
    }
    __builtin_amdgcn_sched_barrier(0);
    auto load_tile = [&](uint32_t t, qw_slice<FMT>* blk) {
        const uint32_t row = min(16u * min(t, tiles - 1u) + i, N - 1u);
        const uint8_t* rowp = p.bank + (uint64_t)row * p.row_bytes;
#pragma unroll
        for (int u = 0; u < IPW; ++u) qw_load_slice<FMT>(rowp, sl[u], p.gshift, p.bb, blk[u]);
    };
    auto compute_tile = [&](uint32_t t, const qw_slice<FMT>* blk, uint32_t buf) {
        f4_t acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int u = 0; u < IPW; ++u) {
            const h2_t s2 = qw_splat_lo(blk[u].hdr), b2 = qw_splat_hi(blk[u].hdr);
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const h8_t a = qw_dequant_chunk<FMT>(blk[u], j, s2, b2, magic);
                acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, xop[u][j], acc, 0, 0, 0);
            }
        }
        // lane (j = activation row, c) holds rows 4c + r of the tile
#pragma unroll
        for (int r = 0; r < 4; ++r) red[buf][wave][lane][r] = acc[r];
        __syncthreads();
        if (tid < 256u && t < tiles) {
            const uint32_t rr = tid & 15u, m = tid >> 4;   // consecutive lanes -> consecutive output rows
            const uint32_t slot = m + 16u * (rr >> 2), comp = rr & 3u;
            float v = 0.f;
#pragma unroll
            for (int w2 = 0; w2 < 8; ++w2) v += red[buf][w2][slot][comp];
            const uint32_t n = 16u * t + rr;
            if (m < M && n < N) {
                if (p.y32) p.y32[(uint64_t)m * N + n] = v;
                if (p.y16) p.y16[(uint64_t)m * N + n] = (h1_t)v;
            }
        }
    };

    // ---- row tiles, two per trip so the register buffers keep static names ----
    const uint32_t G = gridDim.x;
    qw_slice<FMT> bufA[IPW], bufB[IPW];
    uint32_t t = blockIdx.x;
    load_tile(t, bufA);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int u = 0; u < IPW; ++u) {
        const bool ok = 4u * (wave * IPW + u) + c < nsl && i < M;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const h8_t v = qw_x_operand<FMT>(xraw[u], j);
            const u4_t raw = __builtin_bit_cast(u4_t, v);
            const u4_t z = {ok ? raw[0] : 0u, ok ? raw[1] : 0u, ok ? raw[2] : 0u, ok ? raw[3] : 0u};
            xop[u][j] = __builtin_bit_cast(h8_t, z);
        }
    }
    for (; t < tiles; t += 2u * G) {
        load_tile(t + G, bufB);
        compute_tile(t, bufA, 0);
        load_tile(t + 2u * G, bufA);
        compute_tile(t + G, bufB, 1);
    }
}

// ------------------------------------------------------------------------------------------------
// Variant D: transposing MFMA kernel, all containers, m = 1..16, activations already in the container's basis.
// The contraction is variant C's (lane (i, c) dequantizes slice 4u + c of row i to exact f16 weights, four
// v_mfma_f32_16x16x32_f16 per group of four slices against activation operands held in registers), but the bank is
// read the way memory likes it and turned into that layout on chip: a wave owns a chunk of 16 consecutive slices;
// per tile of 16 rows it issues four loads whose lanes (b = lane >> 2, r = lane & 3) read slice b of rows 4q + r
// (four contiguous runs of the bank per instruction instead of sixteen), parks them in a wave-private LDS region
// (row pitch = 16 slices + one 16-byte pad: conflict-free 16-byte reads down a column of rows) and reads each
// lane's (row, slice) back.  The loads of the next tile are in flight while the current one is contracted; no
// workgroup barrier until the end.  Launch shape as the other persistent kernels: grid-stride over row tiles,
// wave wv of a row set owns chunk kr * wpr + wv in K range kr, the 16 x 16 partial tiles accumulate in LDS per
// (tile slot, wave) across K ranges and are summed in wave order at the end.
// ------------------------------------------------------------------------------------------------
template <int FMT, int XDT>
__global__ __launch_bounds__(768) void qw_gemv_colt_kernel(const qw_gemv_params p) {
    constexpr uint32_t PW = FMT == QW_FMT_B8 ? 8 : 4;     // payload dwords per slice
    constexpr uint32_t RS = 16 * PW + 4;                   // row pitch of the payload image, dwords
    constexpr uint32_t HS = 17;                            // row pitch of the header image, dwords
    constexpr uint32_t WAVE_DW = 16 * RS + 16 * HS + 16;   // per-wave region (16-byte multiple)
    extern __shared__ __attribute__((aligned(16))) uint32_t ct_lds[];
    const uint32_t tid = threadIdx.x;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63u;
    const uint32_t nwaves = blockDim.x >> 6;
    const uint32_t wpr = p.wpr, sets = p.sets;
    const uint32_t set = wave / wpr, wv = wave - set * wpr;
    const uint32_t lb = lane >> 2, lr = lane & 3u;      // load role: slice of the chunk, row of the quad
    const uint32_t i = lane & 15u, c = lane >> 4;       // contraction role
    const uint32_t N = p.N, K = p.K, M = p.M;
    const uint32_t nsl = K >> 5;
    const uint32_t magic = qw_vgpr_const(0x64006400u);
    uint32_t* pay = ct_lds + wave * WAVE_DW;
    uint32_t* hdr = pay + 16 * RS;
    f4_t* part = (f4_t*)(ct_lds + nwaves * WAVE_DW);    // [tile slot][wave of the set][lane]

    const uint32_t G = gridDim.x;
    const uint32_t tiles = (N + 15u) >> 4;
    if (blockIdx.x >= tiles) return;
    const uint32_t nt = (tiles - blockIdx.x + G - 1u) / G;   // tile slots of this workgroup
    const uint32_t nmax = (nt + sets - 1u) / sets;            // trip count, uniform over the workgroup
    const uint32_t mine = nt > set ? (nt - set + sets - 1u) / sets : 0u;
    const uint32_t t_first = (mine ? set : 0u) * G + blockIdx.x;
    const uint32_t t_last = t_first + (mine ? mine - 1u : 0u) * G * sets;
    const uint32_t row_bytes = (uint32_t)p.row_bytes;

    for (uint32_t kr = 0; kr < p.nkr; ++kr) {
        const uint32_t chunk = kr * wpr + wv;
        // ---- activation operands of this chunk (issued first), then the first tile's loads ----
        h8_t xraw[4][4], xop[4][4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const uint32_t sx = min(chunk * 16u + 4u * u + c, nsl - 1u);
            const uint64_t at = (uint64_t)min(i, M - 1u) * K + 32u * sx;
#pragma unroll
            for (int j = 0; j < 4; ++j) xraw[u][j] = qw_load_x8_f16<XDT>(p.x, at + 8u * j);
        }
        __builtin_amdgcn_sched_barrier(0);
        const uint32_t gl = min(chunk * 16u + lb, nsl - 1u);   // this lane's slice in the load role
        uint32_t hdr_off, pay_off;
        if constexpr (FMT == QW_FMT_M5) {
            hdr_off = gl * 20u;
            pay_off = hdr_off + 4u;
        } else {
            hdr_off = (gl >> p.gshift) * p.bb;
            pay_off = hdr_off + 4u + (gl & ((1u << p.gshift) - 1u)) * (PW * 4u);
        }
        qw_slice<FMT> ld[4];
        auto issue = [&](uint32_t t) {   // rows 16 t + 4 q + r, clamped into the bank (clamped rows are never stored)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const uint8_t* rp = p.bank + min(16u * t + 4u * q + lr, N - 1u) * row_bytes;
                ld[q].hdr = *(const uint32_t*)(rp + hdr_off);
                if constexpr (FMT == QW_FMT_B8) {
                    const qw_words8 w = *(const qw_words8*)(rp + pay_off);
#pragma unroll
                    for (int k = 0; k < 8; ++k) ld[q].q[k] = w.q[k];
                } else {
                    const qw_words4 w = *(const qw_words4*)(rp + pay_off);
#pragma unroll
                    for (int k = 0; k < 4; ++k) ld[q].q[k] = w.q[k];
                }
            }
        };
        uint32_t t = t_first;
        issue(t);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const bool ok = chunk * 16u + 4u * u + c < nsl && i < M;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const u4_t raw = __builtin_bit_cast(u4_t, qw_x_operand<FMT>(xraw[u], j));
                const u4_t z = {ok ? raw[0] : 0u, ok ? raw[1] : 0u, ok ? raw[2] : 0u, ok ? raw[3] : 0u};
                xop[u][j] = __builtin_bit_cast(h8_t, z);
            }
        }

        uint32_t slot = set;
        for (uint32_t ib = 0; ib < nmax; ++ib) {
            // registers -> LDS image (the previous tile's reads are done: LDS operations of a wave complete in order)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const uint32_t r = 4u * q + lr;
                hdr[r * HS + lb] = ld[q].hdr;
#pragma unroll
                for (uint32_t k = 0; k < PW; k += 4) {
                    const u4_t v = {ld[q].q[k], ld[q].q[k + 1], ld[q].q[k + 2], ld[q].q[k + 3]};
                    *(u4_t*)(pay + r * RS + lb * PW + k) = v;
                }
            }
            t = min(t + G * sets, t_last);
            issue(t);   // next tile (the set's last tile again past the end)
            f4_t acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                qw_slice<FMT> blk;
                blk.hdr = hdr[i * HS + 4u * u + c];
#pragma unroll
                for (uint32_t k = 0; k < PW; k += 4) {
                    const u4_t v = *(const u4_t*)(pay + i * RS + (4u * u + c) * PW + k);
                    blk.q[k] = v[0]; blk.q[k + 1] = v[1]; blk.q[k + 2] = v[2]; blk.q[k + 3] = v[3];
                }
                const h2_t s2 = qw_splat_lo(blk.hdr), b2 = qw_splat_hi(blk.hdr);
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const h8_t a = qw_dequant_chunk<FMT>(blk, j, s2, b2, magic);
                    acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, xop[u][j], acc, 0, 0, 0);
                }
            }
            // lane (j = activation row, c) holds rows 4c + r of the tile
            if (slot < nt) {
                f4_t* dst = part + (size_t)(slot * wpr + wv) * 64u + lane;
                if (kr == 0) *dst = acc;
                else *dst += acc;
            }
            slot += sets;
        }
    }
    __syncthreads();
    // fixed-order sum over the waves of a row set; consecutive threads -> consecutive output rows
    for (uint32_t e = tid; e < nt * 16u * M; e += blockDim.x) {
        const uint32_t rr = e & 15u, sm = e >> 4;
        const uint32_t s = sm / M, m = sm - s * M;
        const uint32_t n = 16u * (s * G + blockIdx.x) + rr;
        if (n >= N) continue;
        const uint32_t src = m + 16u * (rr >> 2), comp = rr & 3u;
        float v = 0.f;
        for (uint32_t w2 = 0; w2 < wpr; ++w2) v += part[(size_t)(s * wpr + w2) * 64u + src][comp];
        if (p.y32) p.y32[(uint64_t)m * N + n] = v;
        if (p.y16) p.y16[(uint64_t)m * N + n] = (h1_t)v;
    }
}

// ------------------------------------------------------------------------------------------------
// host side
// ------------------------------------------------------------------------------------------------
namespace {

typedef qw_gemv_params_x gemv_args;   // the host side fills the long form; plain kernels are handed its base

template <typename K>   // the short argument block for the plain kernel, the long one for the pair / routed forms
void qw_launch_mfma_k(dim3 grid, dim3 block, size_t lds, hipStream_t st, const gemv_args& a) {
    if constexpr (std::is_same<typename K::params_t, qw_gemv_params_x>::value) qw_launch_scalar<K>(grid, block, lds, st, a);
    else qw_launch_scalar<K>(grid, block, lds, st, qw_gemv_base(a));
}

template <int FMT, int RT, int XDT, int XM, int PAIR>
void launch_mfma(hipStream_t st, const gemv_args& a, size_t lds, uint32_t routed_pairs = 0) {
    if constexpr (!PAIR && RT == 1) {
        // Few row tiles, long rows and one or two activation rows: more waves per workgroup split K further, so
        // that the launch keeps enough loads in flight to cover HBM latency (measured on K = 17408, N = 5120:
        // 33.6 -> 26.0 us at m = 1; with more activation rows the extra waves multiply the activation traffic instead).
        if (!routed_pairs && a.M <= 2u) {
            const uint32_t tiles = qwhip_cdiv(a.N, 16u);
            const uint32_t iters = qwhip_cdiv(a.K >> 5, 4u);
            uint32_t nw = 4;
            while (nw < 16u && tiles * nw < 4096u && iters >= 4u * nw) nw *= 2u;
            const dim3 grid(tiles);
            if (nw == 16u) { qw_launch_mfma_k<qw_gemv_mfma_kernel<FMT, RT, XDT, XM, PAIR, 0, 16>>(grid, dim3(1024), lds, st, a); return; }
            if (nw == 8u) { qw_launch_mfma_k<qw_gemv_mfma_kernel<FMT, RT, XDT, XM, PAIR, 0, 8>>(grid, dim3(512), lds, st, a); return; }
        }
    }
    const dim3 block(256);
    if (routed_pairs) {
        if constexpr (PAIR) {
            // one short row set per (route, tile): eight waves split K so that each holds two or more iterations in flight
            const dim3 grid(qwhip_cdiv(a.N, 16u * RT), routed_pairs);
            if (qwhip_cdiv(a.K >> 5, 4u) >= 16u)
                qw_launch_mfma_k<qw_gemv_mfma_kernel<FMT, RT, XDT, XM, PAIR, 1, 8>>(grid, dim3(512), lds, st, a);
            else
                qw_launch_mfma_k<qw_gemv_mfma_kernel<FMT, RT, XDT, XM, PAIR, 1>>(grid, block, lds, st, a);
        }
    } else {
        const dim3 grid(qwhip_cdiv(a.N, 16u * RT));
        qw_launch_mfma_k<qw_gemv_mfma_kernel<FMT, RT, XDT, XM, PAIR, 0>>(grid, block, lds, st, a);
    }
}

template <int FMT, int RT, int XDT, int PAIR>
void launch_mfma_xm(hipStream_t st, const gemv_args& a, int xm, size_t lds, uint32_t routed_pairs = 0) {
    if (xm == QW_XM_LDS_ROT) launch_mfma<FMT, RT, XDT, QW_XM_LDS_ROT, PAIR>(st, a, lds, routed_pairs);
    else launch_mfma<FMT, RT, XDT, QW_XM_GLOBAL, PAIR>(st, a, 0, routed_pairs);
}

template <int FMT, int RT, int PAIR>
void launch_mfma_dt(hipStream_t st, const gemv_args& a, uint32_t xdt, int xm, size_t lds, uint32_t routed_pairs = 0) {
    if (xdt == QWHIP_F16) launch_mfma_xm<FMT, RT, QWHIP_F16, PAIR>(st, a, xm, lds, routed_pairs);
    else launch_mfma_xm<FMT, RT, QWHIP_BF16, PAIR>(st, a, xm, lds, routed_pairs);
}

template <int FMT>
void launch_mfma_rt(hipStream_t st, const gemv_args& a, uint32_t xdt, int xm, size_t lds, int rt) {
    if (rt == 1) launch_mfma_dt<FMT, 1, 0>(st, a, xdt, xm, lds);
    else if (rt == 2) launch_mfma_dt<FMT, 2, 0>(st, a, xdt, xm, lds);
    else launch_mfma_dt<FMT, 4, 0>(st, a, xdt, xm, lds);
}

// Column-stationary kernel (variant C): false when the call is outside its envelope.
template <int FMT>
bool launch_colm(hipStream_t st, const gemv_args& a, uint32_t xdt) {
    const uint32_t iters = qwhip_cdiv(a.K >> 5, 4u);
    if (iters > 40u || a.rotate) return false;
    const uint32_t ipw = qwhip_cdiv(iters, 8u);
    const uint32_t tiles = qwhip_cdiv(a.N, 16u);
    const dim3 grid(min(tiles, 256u)), block(512);
#define QW_COLM(DT, I) hipLaunchKernelGGL((qw_gemv_colm_kernel<FMT, DT, I>), grid, block, 0, st, qw_gemv_base(a))
#define QW_COLM_I(DT)                                                                                  \
    switch (ipw) {                                                                                     \
        case 1: QW_COLM(DT, 1); break; case 2: QW_COLM(DT, 2); break; case 3: QW_COLM(DT, 3); break;   \
        case 4: QW_COLM(DT, 4); break; default: QW_COLM(DT, 5); break;                                 \
    }
    if (xdt == QWHIP_F16) { QW_COLM_I(QWHIP_F16) } else { QW_COLM_I(QWHIP_BF16) }
#undef QW_COLM_I
#undef QW_COLM
    return true;
}

// Transposing kernel (variant D): false when the call is outside its envelope.
template <int FMT, int XDT>
bool launch_colt_1(hipStream_t st, gemv_args a, hipError_t* err) {
    constexpr uint32_t PW = FMT == QW_FMT_B8 ? 8 : 4;
    constexpr uint32_t WAVE_DW = 16 * (16 * PW + 4) + 16 * 17 + 16;
    if ((uint64_t)a.N * a.row_bytes >= (1ull << 32)) return false;   // 32-bit offsets inside the bank
    const uint32_t nsl = a.K >> 5, nch = qwhip_cdiv(nsl, 16u);
    // at most 12 waves per row set (768 threads); longer rows take several K ranges
    a.nkr = qwhip_cdiv(nch, 12u);
    a.wpr = qwhip_cdiv(nch, a.nkr);
    a.sets = max(1u, 12u / a.wpr);
    const uint32_t waves = a.wpr * a.sets;
    const uint32_t tiles = qwhip_cdiv(a.N, 16u);
    uint32_t wgs = min(256u, max(1u, tiles / a.sets));
    size_t lds = 0;
    for (;;) {
        lds = (size_t)waves * WAVE_DW * 4u + (size_t)qwhip_cdiv(tiles, wgs) * a.wpr * 1024u;
        if (lds <= 150u * 1024u || wgs >= tiles) break;
        wgs = min(wgs * 2u, tiles);
    }
    if (lds > 150u * 1024u) return false;
    auto kern = qw_gemv_colt_kernel<FMT, XDT>;
    static std::atomic<size_t> attr_lds{0};   // per instantiation
    if (lds > attr_lds.load(std::memory_order_acquire)) {
        hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, 150 * 1024);
        if (e != hipSuccess) { *err = e; return true; }
        attr_lds.store(150u * 1024u, std::memory_order_release);
    }
    hipLaunchKernelGGL(kern, dim3(wgs), dim3(64u * waves), lds, st, qw_gemv_base(a));
    *err = hipGetLastError();
    return true;
}

template <int FMT>
bool launch_colt(hipStream_t st, const gemv_args& a, uint32_t xdt, hipError_t* err) {
    if (a.rotate) return false;
    return xdt == QWHIP_F16 ? launch_colt_1<FMT, QWHIP_F16>(st, a, err) : launch_colt_1<FMT, QWHIP_BF16>(st, a, err);
}

qwhip_status check_common(qwhip_stream_t s, const qwhip_weight_view* w, const void* x, uint32_t x_dtype, uint32_t m,
                          int* fmt) {
    QWHIP_REQUIRE(s);
    qwhip_status st = qwhip_weight_view_validate(w);
    if (st != QWHIP_OK) return st;
    QWHIP_REQUIRE(x);
    if (x_dtype != QWHIP_F16 && x_dtype != QWHIP_BF16)
        return qwhip_fail(QWHIP_E_BAD_WEIGHTS, "activations must be f16 or bf16, got dtype %u", x_dtype);
    if (m == 0 || m > 16) return qwhip_fail(QWHIP_E_BAD_SHAPE, "gemv handles 1..16 activation rows, got %u", m);
    if (w->n >= (1u << 30)) return qwhip_fail(QWHIP_E_BAD_WEIGHTS, "a bank of %u rows does not fit the row count", w->n);
    if ((uintptr_t)x & 15u) return qwhip_fail(QWHIP_E_BAD_SHAPE, "activations must be 16-byte aligned");
    if (w->kind == QWHIP_KIND_HQ4_G32_M5) *fmt = QW_FMT_M5;
    else if (w->bits == 4) *fmt = QW_FMT_B4;
    else if (w->bits == 8) *fmt = QW_FMT_B8;
    else if (w->bits == 2) *fmt = QW_FMT_B2;
    else if (w->bits == 3) *fmt = QW_FMT_B3;
    else if (w->bits == 6) *fmt = QW_FMT_B6;
    else return qwhip_fail(QWHIP_E_BAD_WEIGHTS, "no gemv kernel for %u-bit group %u", w->bits, w->group);
    return QWHIP_OK;
}

uint32_t log2_u32(uint32_t v) {
    uint32_t r = 0;
    while ((1u << r) < v) ++r;
    return r;
}

}  // namespace

// stream.hip
bool qw_stream_gemv(hipStream_t st, const qwhip_weight_view* w, const void* x, uint32_t x_dtype, uint32_t m, bool rotate,
                    void* y16, float* y32, uint32_t kw_override, hipError_t* err);

// moe_col.hip
bool qw_moe_gateup_col(hipStream_t st, const qwhip_weight_view* w, uint32_t experts, const void* x, uint32_t x_dtype, bool rotate,
                       bool rot_out, const int32_t* idx, uint32_t pairs, uint32_t top_k, void* act16, hipError_t* err,
                       const qw_act act, const float* logits = nullptr, int32_t* idx_out = nullptr, float* wts_out = nullptr, uint32_t norm_topk = 0,
                       float routed_scale = 1.0f, const int32_t* x_rows = nullptr, uint32_t reuse_tokens = 0);
bool qw_moe_down_col(hipStream_t st, const qwhip_weight_view* w, uint32_t experts, const void* act16, const int32_t* idx,
                     const float* wts, uint32_t t, uint32_t top_k, const float* shared, const float* shared_gate, void* out,
                     uint32_t out_dtype, hipError_t* err, uint32_t x_div = 1, const int32_t* labels = nullptr,
                     uint32_t num_groups = 0);

// gemv_quad.hip
bool qw_quad_gemv(hipStream_t st, const qwhip_weight_view* w, int fmt, uint32_t gshift, uint32_t bb, uint64_t row_bytes,
                  const void* x, uint32_t x_dtype, uint32_t m, void* y16, float* y32, uint32_t tune, hipError_t* err);

// gemv_colx.hip
bool qw_colx_gemv(hipStream_t st, const qwhip_weight_view* w, int fmt, uint32_t gshift, uint32_t bb, uint64_t row_bytes,
                  const void* x, uint32_t x_dtype, uint32_t m, bool rotate, void* y16, float* y32, uint32_t tune,
                  hipError_t* err);

// gemv_col.hip
bool qw_col_pair_gemv(hipStream_t st, const qwhip_weight_view* w, const void* x, uint32_t x_dtype, bool rotate, void* act16,
                      float* gated32, const qw_act ga, hipError_t* err);
// gemv_colx.hip
bool qw_colx_pair_gemv(hipStream_t st, const qwhip_weight_view* w, int fmt, uint32_t gshift, uint32_t bb, uint64_t row_bytes,
                       const void* x, uint32_t x_dtype, bool rotate, void* act16, float* gated32, const qw_act ga, hipError_t* err);
extern "C" qwhip_status qwhip_fwht32(qwhip_stream_t s, const void* src, uint32_t src_dtype, void* dst_f16, uint64_t n);
extern "C" qwhip_status qwhip_swiglu_fwht(qwhip_stream_t s, const void* gu, uint32_t gu_dtype, void* act_f16, uint32_t rows, uint32_t inter,
                                          uint32_t rotate);
bool qw_col_gemv(hipStream_t st, const qwhip_weight_view* w, const void* x, uint32_t x_dtype, bool rotate, void* y16,
                 float* y32, uint32_t tune, hipError_t* err, unsigned long long* keys, uint32_t keys_cap, int32_t* token,
                 bool* folded);

// gemv_sk.hip
bool qw_sk_gemv(qwhip_stream_t s, const qwhip_weight_view* w, int fmt, uint32_t gshift, uint32_t bb, uint64_t row_bytes,
                const void* x, uint32_t x_dtype, uint32_t m, void* y16, float* y32, uint32_t tune, hipError_t* err);

// flags bits 8..11: kernel override for tuning and tests (0 = automatic, 1 = dot2, 2 = direct-load mfma, 3 = DMA streamer,
// 4 = column-stationary persistent kernel, 5 = column-stationary MFMA kernel, 6 = column-stationary small-M kernel,
// 7 = 4x4x4-block MFMA kernel, 8 = transposing MFMA kernel, 9 = split-K MFMA kernel);
// bits 12..15: row tiles per wave for the direct-load mfma kernel / K-split of the streamer / tuning code of the
// column-stationary kernel (0 = automatic); bits 12..18: tuning code of the split-K kernel.
// `token` (head door only): where the column-stationary kernel's fused fold leaves the argmax; *folded tells whether it ran
static qwhip_status qw_gemv_impl(qwhip_stream_t s, const qwhip_weight_view* w, const void* x, uint32_t x_dtype, uint32_t m,
                                 uint32_t flags, void* y16, float* y32, int32_t* token, bool* folded) {
    int fmt = 0;
    qwhip_status st = check_common(s, w, x, x_dtype, m, &fmt);
    if (st != QWHIP_OK) return st;
    if (!y16 && !y32) return qwhip_fail(QWHIP_E_NULL, "gemv needs y16 and/or y32");
    const bool rotate = qwhip_view_rotated(w) && !(flags & QWHIP_X_PREROTATED);
    const uint32_t variant = (flags >> 8) & 0xFu;
    uint32_t rt = (flags >> 12) & 0xFu;

    gemv_args a = {};
    a.bank = (const uint8_t*)w->blocks;
    a.x = x;
    a.y16 = (h1_t*)y16;
    a.y32 = y32;
    a.N = w->n;
    a.K = w->k;
    a.M = m;
    a.gshift = log2_u32(w->group / 32);
    a.bb = qwhip_view_block_bytes(w);
    a.row_bytes = qwhip_view_row_bytes(w);
    a.rotate = rotate ? 1u : 0u;
    a.rot_out = 0;

    // Row-count invariance (QWHIP_GEMV_ROW_INVARIANT): every row gets the bits it would get alone, whatever m is - what the
    // reference gets by compiling its 1-, 2-, 4- and M-row bodies without contraction or reassociation
    // (Sources/QWMetal/include/qw_dequant_multi_b.metalh:14,486,533), and what lets serial decode and batched verify agree
    // token for token.  One arithmetic serves every row count: the column-stationary dot2 kernel, whose sums for an
    // activation row do not depend on how many other rows share its registers (four partial sums per slice in a fixed
    // order, a fixed half-wave reduction, the chunks of a row in order), nor on the grid.  Un-rotated rows are rotated by
    // the standalone pass first (m = 1 included), so that every row count contracts the same f16 values.
    if (flags & QWHIP_GEMV_ROW_INVARIANT) {
        if (variant != 0) return qwhip_fail(QWHIP_E_BAD_SHAPE, "the row-invariant mode picks its own kernel (override %u given)", variant);
        const void* xin = x;
        uint32_t xdt = x_dtype;
        if (rotate) {
            const size_t need = (size_t)m * w->k * 2u;
            if (!s->scratch || s->scratch_bytes < QWHIP_STREAM_SCRATCH_BYTES || need > QWHIP_STREAM_XROT_BYTES)
                return qwhip_fail(QWHIP_E_BASIS, "row-invariant gemv: %u un-rotated rows of %u do not fit the stream's rotation scratch; hand them over rotated", m, w->k);
            void* xr = s->scratch + s->scratch_bytes - QWHIP_STREAM_XROT_BYTES;
            st = qwhip_fwht32(s, x, x_dtype, xr, (uint64_t)m * w->k);
            if (st != QWHIP_OK) return st;
            xin = xr;
            xdt = QWHIP_F16;
        }
        // one row over an HQ4_G32_M5 bank: the decode kernel, whose arithmetic the multi-row kernel repeats bit for bit
        if (fmt == QW_FMT_M5 && m == 1) {
            hipError_t e = hipSuccess;
            if (qw_col_gemv(s->stream, w, xin, xdt, false, y16, y32, 0u, &e, nullptr, 0u, nullptr, nullptr)) {
                QWHIP_TRY_HIP(e);
                return QWHIP_OK;
            }
        }
        const uint32_t cpr = (w->k / 32u + 31u) / 32u;
        const uint32_t per = 32u * cpr <= 512u ? 8u : (32u * cpr <= 576u ? 4u : 2u);   // rows the kernel holds at this row length
        for (uint32_t m0 = 0; m0 < m; m0 += per) {
            hipError_t e = hipSuccess;
            const uint32_t mm = min(per, m - m0);
            if (!qw_colx_gemv(s->stream, w, fmt, a.gshift, a.bb, a.row_bytes, (const uint8_t*)xin + (size_t)m0 * w->k * 2u, xdt, mm, false,
                              y16 ? (void*)((h1_t*)y16 + (size_t)m0 * w->n) : nullptr, y32 ? y32 + (size_t)m0 * w->n : nullptr, 0u, &e))
                return qwhip_fail(QWHIP_E_BAD_GEOMETRY, "row-invariant gemv: no column-stationary kernel for n=%u k=%u (rows up to 32768 columns, banks under 4 GiB)", w->n, w->k);
            QWHIP_TRY_HIP(e);
        }
        return QWHIP_OK;
    }
    // Several un-rotated rows on a rotated container: one rotation pass (fp32 butterfly, one f16 rounding: what the fused
    // prologues compute) into the stream's scratch, then the kernels for rows already in the basis, instead of the per-lane
    // rotation of the MFMA streamer.  Kernel overrides keep their own paths.
    const size_t xrot_bytes = (size_t)m * w->k * 2u;
    // two rows whose rotated copy fits the streamers' LDS prologue stay there where that measured level or ahead: the DMA
    // streamer on small banks, the MFMA streamer on 8-bit banks (N = 7168, K = 5120, HQ8: 11.1 against 11.8 us; HQ4_G32_M5,
    // N = 17408, K = 5120: 18.3 against 14.6 us with the pass, so the 4-bit banks take the pass)
    const bool fused_two = fmt < QW_FMT_B2 && m == 2 && ((w->n <= 4096 && w->k <= 8192) || (fmt == QW_FMT_B8 && w->k <= 8192));
    if (variant == 0 && rotate && m > 1 && !fused_two && s->scratch && s->scratch_bytes >= QWHIP_STREAM_SCRATCH_BYTES &&
        xrot_bytes <= QWHIP_STREAM_XROT_BYTES) {
        void* xr = s->scratch + s->scratch_bytes - QWHIP_STREAM_XROT_BYTES;
        st = qwhip_fwht32(s, x, x_dtype, xr, (uint64_t)m * w->k);
        if (st != QWHIP_OK) return st;
        return qw_gemv_impl(s, w, xr, QWHIP_F16, m, flags | QWHIP_X_PREROTATED, y16, y32, token, folded);
    }
    // 2-, 3- and 6-bit streams: the column-stationary dot2 kernel is their one decode kernel (eight rows per launch)
    if (fmt >= QW_FMT_B2) {
        if (rotate && m > 1)
            return qwhip_fail(QWHIP_E_BASIS, "a rotated %u-bit container takes one un-rotated row, or rows already in its basis", w->bits);
        for (uint32_t m0 = 0; m0 < m; m0 += 8u) {
            hipError_t e = hipSuccess;
            const uint32_t mm = min(8u, m - m0);
            if (!qw_colx_gemv(s->stream, w, fmt, a.gshift, a.bb, a.row_bytes, (const uint8_t*)x + (size_t)m0 * w->k * 2u, x_dtype, mm,
                              rotate, y16 ? (void*)((h1_t*)y16 + (size_t)m0 * w->n) : nullptr, y32 ? y32 + (size_t)m0 * w->n : nullptr,
                              rt, &e))
                return qwhip_fail(QWHIP_E_BAD_GEOMETRY, "no %u-bit decode kernel for n=%u k=%u m=%u", w->bits, w->n, w->k, m);
            QWHIP_TRY_HIP(e);
        }
        return QWHIP_OK;
    }
    const size_t lds_dot2 = (size_t)(w->k / 32) * 80u;
    const bool dot2_ok = fmt == QW_FMT_M5 && m == 1 && lds_dot2 <= 60u * 1024u;
    if (variant == 1 && !dot2_ok) return qwhip_fail(QWHIP_E_BAD_GEOMETRY, "dot2 kernel needs HQ4_G32_M5, m = 1, k <= 24576");
    // column-stationary dot2 kernel: one row (rotation fused where needed); it also takes up to eight rows already in the
    // basis (override 6), but its VALU work grows with m (16 dot2 per slice and row).  HQ4_G32_M5 at m = 1 has its own kernel.
    // From two rows on the 4x4x4-block MFMA kernel further below is faster (its cost does not grow with 16 dot2 per row).
    const bool colx_shape = (m == 1 || !rotate) && m <= 8;
    if (variant == 6 || (variant == 0 && colx_shape && !(fmt == QW_FMT_M5 && m == 1) && m == 1)) {
        hipError_t e = hipSuccess;
        if (colx_shape && qw_colx_gemv(s->stream, w, fmt, a.gshift, a.bb, a.row_bytes, x, x_dtype, m, rotate, y16, y32, rt, &e)) {
            QWHIP_TRY_HIP(e);
            return QWHIP_OK;
        }
        if (variant == 6)
            return qwhip_fail(QWHIP_E_BAD_GEOMETRY, "the column-stationary small-M kernel takes m = 1, or m <= 8 rows already in the basis, on rows that fit one workgroup");
    }
    // automatic choice: the DMA streamer where it measured faster than the direct-load kernel (few row tiles, short rows,
    // one or two activation rows), the direct-load kernel otherwise
    const bool stream_auto = !dot2_ok && rotate && m <= 2 && w->n <= 4096 && w->k <= 8192;   // rows already in the basis: kernels below
    if (variant == 3 || (variant == 0 && stream_auto)) {
        hipError_t e = hipSuccess;
        if (qw_stream_gemv(s->stream, w, x, x_dtype, m, rotate, y16, y32, rt, &e)) {
            QWHIP_TRY_HIP(e);
            return QWHIP_OK;
        }
        if (variant == 3) return qwhip_fail(QWHIP_E_BAD_GEOMETRY, "the DMA streamer does not take this shape");
    }
    if (variant == 4 || (variant == 0 && fmt == QW_FMT_M5 && m == 1)) {
        hipError_t e = hipSuccess;
        unsigned long long* keys = token && s->scratch ? (unsigned long long*)s->scratch : nullptr;   // the stream's counter area
        if (fmt == QW_FMT_M5 && m == 1 &&
            qw_col_gemv(s->stream, w, x, x_dtype, rotate, y16, y32, (flags >> 12) & 0xFFFu, &e, keys, QWHIP_STREAM_COUNTER_BYTES / 8u, token, folded)) {
            QWHIP_TRY_HIP(e);
            return QWHIP_OK;
        }
        if (variant == 4) return qwhip_fail(QWHIP_E_BAD_GEOMETRY, "the column-stationary kernel needs HQ4_G32_M5, m = 1, k <= 24576");
    }
    if (variant == 1 || (variant == 0 && dot2_ok)) {
        const uint32_t nbl = qwhip_cdiv(w->k / 32, 32);  // blocks per lane
        const dim3 grid(qwhip_cdiv(w->n, 8u)), block(256);
        const uint32_t nbt = nbl <= 8 ? nbl : 0;
#define QW_DOT2(NBV, DT) hipLaunchKernelGGL((qw_gemv_hq4_dot2_kernel<1, NBV, DT>), grid, block, lds_dot2, s->stream, a.bank, a.x, a.y16, a.y32, a.N, a.K, a.rotate)
#define QW_DOT2_NB(DT)                                                                                                   \
        switch (nbt) {                                                                                                   \
            case 1: QW_DOT2(1, DT); break; case 2: QW_DOT2(2, DT); break; case 3: QW_DOT2(3, DT); break;                 \
            case 4: QW_DOT2(4, DT); break; case 5: QW_DOT2(5, DT); break; case 6: QW_DOT2(6, DT); break;                 \
            case 7: QW_DOT2(7, DT); break; case 8: QW_DOT2(8, DT); break; default: QW_DOT2(0, DT); break;                \
        }
        if (x_dtype == QWHIP_F16) { QW_DOT2_NB(QWHIP_F16) } else { QW_DOT2_NB(QWHIP_BF16) }
#undef QW_DOT2_NB
#undef QW_DOT2
        QWHIP_TRY_HIP(hipGetLastError());
        return QWHIP_OK;
    }

    // split-K matrix-core kernel: activations already in the basis, 2..16 rows.  Its cost is flat in m (two launches, one
    // dequantization per weight whatever m is), so it takes over where rows are long and few and m is large: N = 5120,
    // K = 17408, HQ4_G64 measured 18.7 / 18.7 / 20.7 us at m = 6 / 8 / 16 against 21.2 / 23.2 / 34.9 for the kernels below
    // (16.7 against 18.6 at m = 4); on K = 5120 banks (N = 7168 HQ8, N = 17408 or 5120 HQ4) the kernels below stay ahead.
    // 13..16 rows on an 8-bit stream of short rows take it too, four waves a workgroup, four groups in flight, the image in
    // 128 KiB (tuning code 60): two K ranges and the second launch, 15.7 us on N = 7168, K = 5120 against 16.9 for the
    // transposing kernel and 17.7 for the 4x4x4-block kernel.
    const bool sk_long = !rotate && m >= 6 && w->k >= 8192 && fmt != QW_FMT_B8;
    const bool sk_wide8 = !rotate && m >= 13 && w->k < 8192 && fmt == QW_FMT_B8;
    if (variant == 9 || (variant == 0 && (sk_long || sk_wide8))) {
        hipError_t e = hipSuccess;
        // long rows, more than eight activation rows (1280 bytes of image per slice): a 128 KiB image halves the K ranges
        // (N = 5120, K = 17408: twelve -> six, 20.4 -> 19.3 us at m = 16); up to eight rows have six ranges at 64 KiB
        const uint32_t sk_tune = variant == 9 ? (flags >> 12) & 0x7Fu : (sk_wide8 ? 60u : (m > 8u ? 26u : 0u));
        if (!rotate && qw_sk_gemv(s, w, fmt, a.gshift, a.bb, a.row_bytes, x, x_dtype, m, y16, y32, sk_tune, &e)) {
            QWHIP_TRY_HIP(e);
            return QWHIP_OK;
        }
        if (variant == 9)
            return qwhip_fail(QWHIP_E_BAD_GEOMETRY, "the split-K kernel takes 2..16 rows already in the basis, k %% 128 == 0, partial sums within the stream's scratch");
    }
    // transposing MFMA kernel: activations already in the basis.  Its cost barely grows with m: measured best from 13 rows
    // on (N = 7168, K = 5120, HQ8: 16.0 / 16.9 us at m = 13 / 16 against 16.6 / 17.9 for the 4x4x4-block kernel and 18.6 for
    // the column-stationary MFMA kernel; N = 5120, K = 17408, HQ4_G64: level with the 4x4x4-block kernel, 31.5 / 34.6 us).
    if (variant == 8 || (variant == 0 && !rotate && m >= 13)) {
        hipError_t e = hipSuccess;
        bool done = false;
        if (fmt == QW_FMT_M5) done = launch_colt<QW_FMT_M5>(s->stream, a, x_dtype, &e);
        else if (fmt == QW_FMT_B4) done = launch_colt<QW_FMT_B4>(s->stream, a, x_dtype, &e);
        else done = launch_colt<QW_FMT_B8>(s->stream, a, x_dtype, &e);
        if (done) {
            QWHIP_TRY_HIP(e);
            return QWHIP_OK;
        }
        if (variant == 8) return qwhip_fail(QWHIP_E_BAD_GEOMETRY, "the transposing MFMA kernel needs activations in the basis");
    }
    // 4x4x4-block MFMA kernel: activations already in the basis.  Measured best for 2..12 rows (N = 7168, K = 5120, HQ8:
    // 11.0 / 11.9 / 13.2 us at m = 2 / 4 / 8, 14.4 / 15.7 at m = 9 / 12 against 15.2 / 16.0 for the transposing kernel;
    // N = 5120, K = 17408, HQ4_G64: 23.4 us at m = 8, 25.9 / 27.9 at m = 9 / 12 against 28.1 / 31.1).
    if (variant == 7 || (variant == 0 && !rotate && m >= 2 && m <= 12)) {
        hipError_t e = hipSuccess;
        if (!rotate && qw_quad_gemv(s->stream, w, fmt, a.gshift, a.bb, a.row_bytes, x, x_dtype, m, y16, y32, rt, &e)) {
            QWHIP_TRY_HIP(e);
            return QWHIP_OK;
        }
        if (variant == 7) return qwhip_fail(QWHIP_E_BAD_GEOMETRY, "the 4x4x4-block kernel needs activations in the basis");
    }
    // column-stationary MFMA kernel: activations already in the basis (verify rows, standard-basis containers), k <= 5120
    if (variant == 5 || (variant == 0 && !rotate)) {
        bool done = false;
        if (fmt == QW_FMT_M5) done = launch_colm<QW_FMT_M5>(s->stream, a, x_dtype);
        else if (fmt == QW_FMT_B4) done = launch_colm<QW_FMT_B4>(s->stream, a, x_dtype);
        else done = launch_colm<QW_FMT_B8>(s->stream, a, x_dtype);
        if (done) {
            QWHIP_TRY_HIP(hipGetLastError());
            return QWHIP_OK;
        }
        if (variant == 5) return qwhip_fail(QWHIP_E_BAD_GEOMETRY, "the column-stationary MFMA kernel needs activations in the basis and k <= 5120");
    }
    // mfma streamer.  Rotation in the prologue (LDS) when the rotated rows fit, else per lane.
    const size_t lds_x = (size_t)m * ((size_t)w->k * 2u + 16u);
    const int xm = (rotate && lds_x <= 48u * 1024u) ? QW_XM_LDS_ROT : QW_XM_GLOBAL;
    // two row tiles per wave halve the activation traffic per weight byte: it pays from eight activation rows on
    if (rt != 1 && rt != 2 && rt != 4) rt = (w->n >= 16384 || m >= 8) ? 2u : 1u;
    const size_t lds = xm == QW_XM_LDS_ROT ? lds_x : 0;
    if (fmt == QW_FMT_M5) launch_mfma_rt<QW_FMT_M5>(s->stream, a, x_dtype, xm, lds, (int)rt);
    else if (fmt == QW_FMT_B4) launch_mfma_rt<QW_FMT_B4>(s->stream, a, x_dtype, xm, lds, (int)rt);
    else launch_mfma_rt<QW_FMT_B8>(s->stream, a, x_dtype, xm, lds, (int)rt);
    QWHIP_TRY_HIP(hipGetLastError());
    return QWHIP_OK;
}

extern "C" qwhip_status qwhip_gemv(qwhip_stream_t s, const qwhip_weight_view* w, const void* x, uint32_t x_dtype,
                                   uint32_t m, uint32_t flags, void* y16, float* y32) {
    return qw_gemv_impl(s, w, x, x_dtype, m, flags, y16, y32, nullptr, nullptr);
}

extern "C" qwhip_status qwhip_gemv_silu_pair(qwhip_stream_t s, const qwhip_weight_view* w, const void* x, uint32_t x_dtype,
                                             uint32_t m, uint32_t flags, uint32_t rotate_out, void* act16) {
    int fmt = 0;
    qwhip_status st = check_common(s, w, x, x_dtype, m, &fmt);
    if (st != QWHIP_OK) return st;
    QWHIP_REQUIRE(act16);
    if (w->n % 2 != 0) return qwhip_fail(QWHIP_E_BAD_WEIGHTS, "gate|up bank needs an even row count, got %u", w->n);
    const uint32_t inter = w->n / 2;
    const bool rotate = qwhip_view_rotated(w) && !(flags & QWHIP_X_PREROTATED);
    // One activation row: the one-row GEMV kernels in their gate|up form (gate and up row of a channel in neighbouring row
    // slots of a workgroup, the bank read as two moving bands, the gated activation formed in the epilogue).  With the output
    // rotation the launch leaves gated(g, u) as fp32 in the stream's scratch and the rotation kernel behind it rounds to f16
    // once, as the fused epilogues do.  flags bits 8..11 (tests): 2 = the general kernel, 3 = HQ4_G32_M5 on the MoE decode kernel.
    const bool rot_out = rotate_out && inter % 32 == 0;
    if (m == 1u && ((flags >> 8) & 0xFu) == 0u) {
        float* gated32 = nullptr;
        if (rot_out) {
            if (s->scratch && s->scratch_bytes >= QWHIP_STREAM_COUNTER_BYTES + (size_t)inter * 4u + QWHIP_STREAM_XROT_BYTES)
                gated32 = (float*)(s->scratch + QWHIP_STREAM_COUNTER_BYTES);
        }
        if (!rot_out || gated32) {
            hipError_t e = hipSuccess;
            const bool took = fmt == QW_FMT_M5
                                  ? qw_col_pair_gemv(s->stream, w, x, x_dtype, rotate, act16, gated32, s->dev->act, &e)
                                  : qw_colx_pair_gemv(s->stream, w, fmt, log2_u32(w->group / 32), qwhip_view_block_bytes(w), qwhip_view_row_bytes(w), x,
                                                      x_dtype, rotate, act16, gated32, s->dev->act, &e);
            if (took) {
                QWHIP_TRY_HIP(e);
                return rot_out ? qwhip_fwht32(s, gated32, QWHIP_F32, act16, inter) : QWHIP_OK;
            }
        }
    }
    // Two to sixteen rows: the verify GEMV over the whole gate|up bank into an fp32 image [m, 2 I] at the top of the stream's
    // partial-sum area, then the gated activation (+ rotation) pass over it - every weight is read once whatever m is (the MoE
    // decode kernel reads the bank once per row: 40 / 70 / 125 us at m = 2 / 4 / 8 on 2 x 17408 x 5120).
    if (m >= 2u && m <= 16u && ((flags >> 8) & 0xFu) == 0u && s->scratch && (!rot_out || ((uintptr_t)act16 & 15u) == 0)) {
        const size_t need = (((size_t)m * w->n * 4u) + 255u) & ~(size_t)255u;
        const size_t area = s->scratch_bytes - QWHIP_STREAM_COUNTER_BYTES - QWHIP_STREAM_XROT_BYTES;
        if (need <= area / 2u) {
            float* gu32 = (float*)(s->scratch + QWHIP_STREAM_COUNTER_BYTES + area - need);
            s->scratch_reserved = need;
            st = qw_gemv_impl(s, w, x, x_dtype, m, flags & (QWHIP_X_PREROTATED | QWHIP_GEMV_ROW_INVARIANT), nullptr, gu32, nullptr, nullptr);
            s->scratch_reserved = 0;
            if (st == QWHIP_OK) return qwhip_swiglu_fwht(s, gu32, QWHIP_F32, act16, m, inter, rot_out ? 1u : 0u);
            if (st != QWHIP_E_BAD_GEOMETRY) return st;
        }
    }
    // HQ4_G32_M5 (flags bits 8..11 = 3, or a shape the forms above do not take): the column-stationary gate|up kernel of the MoE
    // decode path, as one dense bank with one "route" per activation row
    if (fmt == QW_FMT_M5 && ((flags >> 8) & 0xFu) != 2u) {
        hipError_t e = hipSuccess;
        if (qw_moe_gateup_col(s->stream, w, 1, x, x_dtype, rotate, rotate_out && inter % 32 == 0, nullptr, m, 1, act16, &e, s->dev->act)) {
            QWHIP_TRY_HIP(e);
            return QWHIP_OK;
        }
    }
    gemv_args a = {};
    a.bank = (const uint8_t*)w->blocks;
    a.x = x;
    a.y16 = (h1_t*)act16;
    a.y32 = nullptr;
    a.N = inter;
    a.K = w->k;
    a.M = m;
    a.gshift = log2_u32(w->group / 32);
    a.bb = qwhip_view_block_bytes(w);
    a.row_bytes = qwhip_view_row_bytes(w);
    a.rotate = rotate ? 1u : 0u;
    a.rot_out = (rotate_out && inter % 32 == 0) ? 1u : 0u;
    a.act = s->dev->act;
    const size_t lds_x = (size_t)m * ((size_t)w->k * 2u + 16u);
    const int xm = (rotate && lds_x <= 48u * 1024u) ? QW_XM_LDS_ROT : QW_XM_GLOBAL;
    const size_t lds = xm == QW_XM_LDS_ROT ? lds_x : 0;
    switch (fmt) {
        case QW_FMT_M5: launch_mfma_dt<QW_FMT_M5, 2, 1>(s->stream, a, x_dtype, xm, lds); break;
        case QW_FMT_B4: launch_mfma_dt<QW_FMT_B4, 2, 1>(s->stream, a, x_dtype, xm, lds); break;
        case QW_FMT_B8: launch_mfma_dt<QW_FMT_B8, 2, 1>(s->stream, a, x_dtype, xm, lds); break;
        case QW_FMT_B2: launch_mfma_dt<QW_FMT_B2, 2, 1>(s->stream, a, x_dtype, xm, lds); break;
        case QW_FMT_B3: launch_mfma_dt<QW_FMT_B3, 2, 1>(s->stream, a, x_dtype, xm, lds); break;
        default: launch_mfma_dt<QW_FMT_B6, 2, 1>(s->stream, a, x_dtype, xm, lds); break;
    }
    QWHIP_TRY_HIP(hipGetLastError());
    return QWHIP_OK;
}

// ---- MoE decode / verify: routing + routed gate|up in one launch -------------------------------------
extern "C" qwhip_status qwhip_moe_route(qwhip_stream_t s, const float* logits, uint32_t t, uint32_t experts, uint32_t top_k,
                                        uint32_t norm_topk, float routed_scale, int32_t* idx, float* wts);
extern "C" qwhip_status qwhip_moe_gateup_decode(qwhip_stream_t s, const qwhip_weight_view* w_gate_up, uint32_t experts,
                                                const void* x, uint32_t x_dtype, uint32_t flags, const int32_t* idx, uint32_t t,
                                                uint32_t top_k, void* act16);
extern "C" qwhip_status qwhip_moe_route_gateup_decode(qwhip_stream_t s, const qwhip_weight_view* w_gate_up, uint32_t experts,
                                                      const void* x, uint32_t x_dtype, uint32_t flags, const float* logits, uint32_t t,
                                                      uint32_t top_k, uint32_t norm_topk, float routed_scale, int32_t* idx, float* wts,
                                                      void* act16) {
    int fmt = 0;
    qwhip_status st = check_common(s, w_gate_up, x, x_dtype, 1, &fmt);
    if (st != QWHIP_OK) return st;
    QWHIP_REQUIRE(logits);
    QWHIP_REQUIRE(idx);
    QWHIP_REQUIRE(wts);
    QWHIP_REQUIRE(act16);
    if (t == 0 || top_k == 0) return QWHIP_OK;
    if (experts == 0 || experts > 512) return qwhip_fail(QWHIP_E_BAD_SHAPE, "moe route: experts must be 1..512, got %u", experts);
    if (top_k > 16) return qwhip_fail(QWHIP_E_BAD_SHAPE, "moe route: top_k must be 1..16, got %u", top_k);
    const float scale = routed_scale > 0.0f ? routed_scale : 1.0f;
    if (fmt == QW_FMT_M5 && w_gate_up->n % (2 * experts) == 0 && (uint64_t)t * top_k <= 65535u) {
        const uint32_t inter = w_gate_up->n / (2 * experts);
        const bool rotate = qwhip_view_rotated(w_gate_up) && !(flags & QWHIP_X_PREROTATED);
        hipError_t e = hipSuccess;
        if (qw_moe_gateup_col(s->stream, w_gate_up, experts, x, x_dtype, rotate, qwhip_view_rotated(w_gate_up) && inter % 32 == 0, nullptr,
                              t * top_k, top_k, act16, &e, s->dev->act, logits, idx, wts, norm_topk ? 1u : 0u, scale, nullptr,
                              (flags & QWHIP_MOE_REUSE_EXPERTS) ? t : 0u)) {
            QWHIP_TRY_HIP(e);
            return QWHIP_OK;
        }
    }
    // other containers and shapes: the two launches
    st = qwhip_moe_route(s, logits, t, experts, top_k, norm_topk, routed_scale, idx, wts);
    if (st != QWHIP_OK) return st;
    return qwhip_moe_gateup_decode(s, w_gate_up, experts, x, x_dtype, flags, idx, t, top_k, act16);
}

// ---- MoE decode / verify (t <= 8): routed experts as GEMVs -----------------------------------------
// x_rows: the activation row of every (token, route) pair; NULL = the pair's token.
static qwhip_status qw_moe_gateup_decode_impl(qwhip_stream_t s, const qwhip_weight_view* w_gate_up, uint32_t experts, const void* x,
                                              uint32_t x_dtype, uint32_t flags, const int32_t* idx, const int32_t* x_rows, uint32_t t,
                                              uint32_t top_k, void* act16) {
    int fmt = 0;
    qwhip_status st = check_common(s, w_gate_up, x, x_dtype, 1, &fmt);
    if (st != QWHIP_OK) return st;
    QWHIP_REQUIRE(idx);
    QWHIP_REQUIRE(act16);
    if (t == 0 || top_k == 0) return QWHIP_OK;
    if (experts == 0 || experts > 512 || w_gate_up->n % (2 * experts) != 0)
        return qwhip_fail(QWHIP_E_BAD_SHAPE, "gate|up bank of %u rows does not split over %u experts", w_gate_up->n, experts);
    if ((uint64_t)t * top_k > 65535u) return qwhip_fail(QWHIP_E_BAD_SHAPE, "decode path holds at most 65535 (token, route) pairs");
    const uint32_t inter = w_gate_up->n / (2 * experts);
    const bool rotate = qwhip_view_rotated(w_gate_up) && !(flags & QWHIP_X_PREROTATED);
    // HQ4_G32_M5 banks take the column-stationary kernel (flags bits 8..11 = 2 keep the general one, for tests)
    if (fmt == QW_FMT_M5 && ((flags >> 8) & 0xFu) != 2u) {
        hipError_t e = hipSuccess;
        if (qw_moe_gateup_col(s->stream, w_gate_up, experts, x, x_dtype, rotate, qwhip_view_rotated(w_gate_up) && inter % 32 == 0,
                              idx, t * top_k, top_k, act16, &e, s->dev->act, nullptr, nullptr, nullptr, 0, 1.0f, x_rows,
                              (flags & QWHIP_MOE_REUSE_EXPERTS) ? t : 0u)) {
            QWHIP_TRY_HIP(e);
            return QWHIP_OK;
        }
    }
    gemv_args a = {};
    a.bank = (const uint8_t*)w_gate_up->blocks;
    a.x = x;
    a.y16 = (h1_t*)act16;
    a.N = inter;
    a.K = w_gate_up->k;
    a.M = 1;
    a.gshift = log2_u32(w_gate_up->group / 32);
    a.bb = qwhip_view_block_bytes(w_gate_up);
    a.row_bytes = qwhip_view_row_bytes(w_gate_up);
    a.rotate = rotate ? 1u : 0u;
    a.rot_out = (qwhip_view_rotated(w_gate_up) && inter % 32 == 0) ? 1u : 0u;
    a.idx = idx;
    a.x_rows = x_rows;
    a.act = s->dev->act;
    a.top_k = top_k;
    a.expert_bytes = (uint64_t)2 * inter * a.row_bytes;
    const size_t lds_x = (size_t)w_gate_up->k * 2u + 16u;
    const int xm = (rotate && lds_x <= 48u * 1024u) ? QW_XM_LDS_ROT : QW_XM_GLOBAL;
    const size_t lds = xm == QW_XM_LDS_ROT ? lds_x : 0;
    const uint32_t pairs = t * top_k;
    switch (fmt) {
        case QW_FMT_M5: launch_mfma_dt<QW_FMT_M5, 2, 1>(s->stream, a, x_dtype, xm, lds, pairs); break;
        case QW_FMT_B4: launch_mfma_dt<QW_FMT_B4, 2, 1>(s->stream, a, x_dtype, xm, lds, pairs); break;
        case QW_FMT_B8: launch_mfma_dt<QW_FMT_B8, 2, 1>(s->stream, a, x_dtype, xm, lds, pairs); break;
        case QW_FMT_B2: launch_mfma_dt<QW_FMT_B2, 2, 1>(s->stream, a, x_dtype, xm, lds, pairs); break;
        case QW_FMT_B3: launch_mfma_dt<QW_FMT_B3, 2, 1>(s->stream, a, x_dtype, xm, lds, pairs); break;
        default: launch_mfma_dt<QW_FMT_B6, 2, 1>(s->stream, a, x_dtype, xm, lds, pairs); break;
    }
    QWHIP_TRY_HIP(hipGetLastError());
    return QWHIP_OK;
}

extern "C" qwhip_status qwhip_moe_gateup_decode(qwhip_stream_t s, const qwhip_weight_view* w_gate_up, uint32_t experts,
                                                const void* x, uint32_t x_dtype, uint32_t flags, const int32_t* idx, uint32_t t,
                                                uint32_t top_k, void* act16) {
    return qw_moe_gateup_decode_impl(s, w_gate_up, experts, x, x_dtype, flags, idx, nullptr, t, top_k, act16);
}

extern "C" qwhip_status qwhip_moe_gateup_decode_rows(qwhip_stream_t s, const qwhip_weight_view* w_gate_up, uint32_t experts,
                                                     const void* x, uint32_t x_dtype, uint32_t flags, const int32_t* idx,
                                                     const int32_t* x_rows, uint32_t t, uint32_t top_k, void* act16) {
    QWHIP_REQUIRE(x_rows);
    return qw_moe_gateup_decode_impl(s, w_gate_up, experts, x, x_dtype, flags, idx, x_rows, t, top_k, act16);
}

// The routed down projection in its three shapes.  rows = output rows (grid.y): tokens, (token, route) pairs with top_k = 1
// and x_div pairs per activation row, or (token, group) pairs with num_groups > 0 (then only the routes whose expert carries
// that group's label are summed).  wts NULL = unit weights.
static qwhip_status qw_moe_down_decode_impl(qwhip_stream_t s, const qwhip_weight_view* w_down, uint32_t experts, const void* act16,
                                            const int32_t* idx, const float* wts, uint32_t t, uint32_t top_k, const float* shared,
                                            const float* shared_gate, void* out, uint32_t out_dtype, uint32_t x_div,
                                            const int32_t* labels, uint32_t num_groups) {
    int fmt = 0;
    qwhip_status st = check_common(s, w_down, act16, QWHIP_F16, 1, &fmt);
    if (st != QWHIP_OK) return st;
    QWHIP_REQUIRE(idx);
    QWHIP_REQUIRE(out);
    if (t == 0 || top_k == 0) return QWHIP_OK;
    if (experts == 0 || experts > 512 || w_down->n % experts != 0)
        return qwhip_fail(QWHIP_E_BAD_SHAPE, "down bank of %u rows does not split over %u experts", w_down->n, experts);
    const uint64_t out_rows = (uint64_t)t * (num_groups ? num_groups : 1u);
    if (out_rows > 65535u) return qwhip_fail(QWHIP_E_BAD_SHAPE, "decode path holds at most 65535 output rows");
    if ((w_down->k * 2u) % 16u != 0) return qwhip_fail(QWHIP_E_BAD_SHAPE, "activation rows must be 16-byte multiples");
    const uint32_t hidden = w_down->n / experts;
    if (fmt == QW_FMT_M5) {
        hipError_t e = hipSuccess;
        if (qw_moe_down_col(s->stream, w_down, experts, act16, idx, wts, t, top_k, shared, shared_gate, out, out_dtype, &e, x_div, labels,
                            num_groups)) {
            QWHIP_TRY_HIP(e);
            return QWHIP_OK;
        }
    }
    gemv_args a = {};
    a.bank = (const uint8_t*)w_down->blocks;
    a.x = act16;
    a.N = hidden;
    a.K = w_down->k;
    a.M = 1;
    a.gshift = log2_u32(w_down->group / 32);
    a.bb = qwhip_view_block_bytes(w_down);
    a.row_bytes = qwhip_view_row_bytes(w_down);
    a.idx = idx;
    a.wts = wts;
    a.top_k = top_k;
    a.expert_bytes = (uint64_t)hidden * a.row_bytes;
    a.shared = shared;
    a.shared_gate = shared_gate;
    a.out = out;
    a.x_div = x_div;
    a.labels = labels;
    a.num_groups = num_groups ? (num_groups | (experts << 8)) : 0u;
    const dim3 grid(qwhip_cdiv(hidden, 16u)), block(512);
    const dim3 g2(grid.x, (uint32_t)out_rows);
#define QW_DD(F, OD) qw_launch_scalar<qw_moe_down_decode_kernel<F, 1, OD>>(g2, block, 0, s->stream, a)
#define QW_DD_O(F)                                                                                          \
    switch (out_dtype) {                                                                                    \
        case QWHIP_F32: QW_DD(F, QWHIP_F32); break;                                                         \
        case QWHIP_F16: QW_DD(F, QWHIP_F16); break;                                                         \
        case QWHIP_BF16: QW_DD(F, QWHIP_BF16); break;                                                       \
        default: return qwhip_fail(QWHIP_E_BAD_SHAPE, "moe down: unsupported output dtype %u", out_dtype);  \
    }
    if (fmt == QW_FMT_M5) { QW_DD_O(QW_FMT_M5) } else if (fmt == QW_FMT_B4) { QW_DD_O(QW_FMT_B4) } else if (fmt == QW_FMT_B8) { QW_DD_O(QW_FMT_B8) }
    else if (fmt == QW_FMT_B2) { QW_DD_O(QW_FMT_B2) } else if (fmt == QW_FMT_B3) { QW_DD_O(QW_FMT_B3) } else { QW_DD_O(QW_FMT_B6) }
#undef QW_DD_O
#undef QW_DD
    QWHIP_TRY_HIP(hipGetLastError());
    return QWHIP_OK;
}

extern "C" qwhip_status qwhip_moe_down_decode(qwhip_stream_t s, const qwhip_weight_view* w_down, uint32_t experts,
                                              const void* act16, const int32_t* idx, const float* wts, uint32_t t, uint32_t top_k,
                                              const float* shared, const float* shared_gate, void* out, uint32_t out_dtype) {
    return qw_moe_down_decode_impl(s, w_down, experts, act16, idx, wts, t, top_k, shared, shared_gate, out, out_dtype, 1u, nullptr, 0u);
}

// out[t, r, :] = wts[t, r] * W[idx[t, r]] . x_row, one output row per route (zeros where idx < 0): the routed projection
// without the sum over routes.
extern "C" qwhip_status qwhip_moe_routed_gemv(qwhip_stream_t s, const qwhip_weight_view* w, uint32_t experts, const void* x16,
                                              uint32_t x_per_token, const int32_t* idx, const float* wts, uint32_t t, uint32_t top_k,
                                              void* out, uint32_t out_dtype) {
    if ((uint64_t)t * top_k > 65535u) return qwhip_fail(QWHIP_E_BAD_SHAPE, "decode path holds at most 65535 (token, route) pairs");
    return qw_moe_down_decode_impl(s, w, experts, x16, idx, wts, t * top_k, 1u, nullptr, nullptr, out, out_dtype,
                                   x_per_token ? top_k : 1u, nullptr, 0u);
}

// out[t, g, :] = sum over the routes r of token t with labels[idx[t, r]] == g of wts[t, r] * W_down[idx[t, r]] . act16[t, r, :]
// (zeros for a group none of the token's routes falls into).
extern "C" qwhip_status qwhip_moe_down_decode_groups(qwhip_stream_t s, const qwhip_weight_view* w_down, uint32_t experts,
                                                     const void* act16, const int32_t* idx, const float* wts, const int32_t* labels,
                                                     uint32_t num_groups, uint32_t t, uint32_t top_k, void* out, uint32_t out_dtype) {
    QWHIP_REQUIRE(labels);
    if (num_groups == 0 || num_groups > 32u) return qwhip_fail(QWHIP_E_BAD_SHAPE, "latent groups must be 1..32, got %u", num_groups);
    return qw_moe_down_decode_impl(s, w_down, experts, act16, idx, wts, t, top_k, nullptr, nullptr, out, out_dtype, 1u, labels, num_groups);
}

// gemv_f32.hip
uint32_t qw_f32_gemv_rows(const qwhip_weight_view* w, uint64_t row_bytes);
void qw_f32_gemv(hipStream_t st, const qwhip_weight_view* w, int fmt, uint32_t gshift, uint32_t bb, uint64_t row_bytes,
                 const float* x, uint32_t m, uint32_t epi, float scale, float* y);
void qw_h32_f32_launch(hipStream_t st, const float* x, float* out, uint32_t rows, uint32_t hidden);
// gemm_f32.hip
bool qw_f32_gemm(hipStream_t st, const qwhip_weight_view* w, int fmt, uint32_t gshift, uint32_t bb, uint64_t row_bytes,
                 const float* x, uint32_t m, uint32_t epi, float scale, float* y, float* row_down);

// fp32 activations in the container's basis -> fp32 outputs with the scalar epilogues of the reference's f32 family
// (QWGemm.encodeHQ4F32V4 / encodeHQ4F32BM, Sources/Operators/QWGEMM/QWGemmF32.swift:178-199,311-350): the rows go through
// the column-stationary fp32 kernel four (long rows: two, one) at a time, as the reference's v4 door walks them; from 32
// rows on (where the reference switches to its batched kernels) the matrix-core form of gemm_f32.hip reads the bank once
// per 64 rows.
extern "C" qwhip_status qwhip_gemv_f32(qwhip_stream_t s, const qwhip_weight_view* w, const float* x, uint32_t m, uint32_t epi,
                                       float scale, float* y) {
    QWHIP_REQUIRE(s);
    qwhip_status st = qwhip_weight_view_validate(w);
    if (st != QWHIP_OK) return st;
    QWHIP_REQUIRE(x);
    QWHIP_REQUIRE(y);
    int fmt = 0;
    st = check_common(s, w, x, QWHIP_F16, 1, &fmt);   // format lookup, alignment and row-count limits
    if (st != QWHIP_OK) return st;
    if (m == 0 || m > 65535u) return qwhip_fail(QWHIP_E_BAD_SHAPE, "the f32 gemv takes 1..65535 activation rows, got %u", m);
    if (epi > 3u) return qwhip_fail(QWHIP_E_BAD_SHAPE, "epilogue %u is not one of 0 none, 1 silu(y/scale), 2 sigmoid, 3 silu(y/scale) + H32", epi);
    if ((epi == 1u || epi == 3u) && !(scale != 0.0f && scale == scale))
        return qwhip_fail(QWHIP_E_BAD_SHAPE, "epilogue %u divides by its scale, which must be a non-zero number", epi);
    const uint64_t row_bytes = qwhip_view_row_bytes(w);
    const uint32_t per = qw_f32_gemv_rows(w, row_bytes);
    if (per == 0) return qwhip_fail(QWHIP_E_BAD_GEOMETRY, "no f32 gemv kernel for n=%u k=%u (rows up to 32768 columns, banks under 1 GiB)", w->n, w->k);
    const uint32_t gshift = log2_u32(w->group / 32), bb = qwhip_view_block_bytes(w);
    // the batched form keeps one scaling factor per activation row (at most 65535 floats) at the head of the stream's
    // partial-sum scratch: launches on a stream are ordered, and nothing else of this call uses the scratch
    float* row_down = s->scratch ? (float*)(s->scratch + QWHIP_STREAM_COUNTER_BYTES) : nullptr;
    const bool batched = m >= 32u && qw_f32_gemm(s->stream, w, fmt, gshift, bb, row_bytes, x, m, epi, scale, y, row_down);
    if (batched) QWHIP_TRY_HIP(hipGetLastError());
    for (uint32_t m0 = 0; !batched && m0 < m; m0 += per) {
        const uint32_t mm = min(per, m - m0);
        qw_f32_gemv(s->stream, w, fmt, gshift, bb, row_bytes, x + (size_t)m0 * w->k, mm, epi, scale, y + (size_t)m0 * w->n);
        QWHIP_TRY_HIP(hipGetLastError());
    }
    if (epi == 3u) {
        qw_h32_f32_launch(s->stream, y, y, m, w->n);
        QWHIP_TRY_HIP(hipGetLastError());
    }
    return QWHIP_OK;
}

// out f32 [rows, hidden] = FWHT-32 of x in the normalised Walsh-Hadamard domain (QWGemm.encodeH32F32,
// Sources/Operators/QWGEMM/QWGemmF32.swift:46-54; qwg_h32_f32, Sources/QWMetal/gemm/qwgemm_f32.metal:191-201); in place allowed.
extern "C" qwhip_status qwhip_h32_f32(qwhip_stream_t s, const float* x, float* out, uint32_t rows, uint32_t hidden) {
    QWHIP_REQUIRE(s);
    QWHIP_REQUIRE(x);
    QWHIP_REQUIRE(out);
    if (rows == 0 || rows > 65535u || hidden == 0 || hidden % 32u != 0)
        return qwhip_fail(QWHIP_E_BAD_SHAPE, "the rotation needs 1..65535 rows of a multiple of 32 columns (rows=%u hidden=%u)", rows, hidden);
    qw_h32_f32_launch(s->stream, x, out, rows, hidden);
    QWHIP_TRY_HIP(hipGetLastError());
    return QWHIP_OK;
}

// LM head for greedy decoding: logits = W . x over the vocabulary rows, then the argmax of each activation row with the
// reference's key rule (QWGemmAQ.encodeHeadArgmax, Sources/Operators/QWGEMM/QWGemmAQ.swift:306-349; qwg_head_gemv_*_argmax,
// qwg_gemv_*_f32_v4_am).  Two launches on the stream: the GEMV of qwhip_gemv into `logits` (which the caller keeps, as
// with the reference's writeLogits), and one workgroup per row folding it.  One un-rotated or rotated row over an
// HQ4_G32_M5 bank folds inside the GEMV's epilogue, as the reference's head kernels do (a key per workgroup in the stream's
// scratch), and the second launch is the one-workgroup fold of those keys (the reference's qwg_head_argmax_fin).
extern "C" qwhip_status qwhip_argmax_f32(qwhip_stream_t s, const float* logits, uint32_t rows, uint32_t n, int32_t* tokens);
extern "C" qwhip_status qwhip_head_argmax(qwhip_stream_t s, const qwhip_weight_view* w, const void* x, uint32_t x_dtype, uint32_t m,
                                          uint32_t flags, float* logits, int32_t* tokens) {
    QWHIP_REQUIRE(logits);
    QWHIP_REQUIRE(tokens);
    bool folded = false;
    qwhip_status st = x_dtype == QWHIP_F32 ? qwhip_gemv_f32(s, w, (const float*)x, m, 0u, 1.0f, logits)
                                           : qw_gemv_impl(s, w, x, x_dtype, m, flags, nullptr, logits, m == 1u ? tokens : nullptr, &folded);
    if (st != QWHIP_OK) return st;
    if (folded) return QWHIP_OK;
    return qwhip_argmax_f32(s, logits, m, w->n, tokens);
}
