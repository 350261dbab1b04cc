// Small-M GEMV over any 4- or 8-bit container, column-stationary persistent form: m = 1..8 activation rows already in
// the container's basis, or one row with the FWHT-32 fused in front.
//
// Same launch shape as the m = 1 HQ4 kernel of gemv_col.hip: a fixed population of workgroups walks the bank once
// (row slot s of workgroup w is bank row s * gridDim.x + w, so the grid reads one contiguous band of rows at a time);
// a 32-lane half-wavefront (set, chunk) owns slice columns 32 * chunk .. + 31 (a slice = 32 columns) of the rows
// set, set + sets, ...  Consecutive lanes read consecutive slices of a row: every load instruction covers a
// contiguous run of the bank.  A lane keeps its 32 activations of each of the MR activation rows in registers
// (16 f16 pairs per row), so the row loop has no activation traffic and its cost per weight byte grows only by
// 16 v_dot2_f32_f16 per extra activation row.
//
// Arithmetic.  The packed codes are used directly as f16 operands: a 4-bit code masked in place at bits 0..3 / 16..19
// of a word reads as the f16 subnormal q * 2^-24 (at bits 4..7 / 20..23 as 16 q * 2^-24), an 8-bit code at bits
// 0..7 / 16..23 likewise (v_dot2_f32_f16 honours f16 subnormals; products are exact, accumulation is fp32).  The affine
// part is applied once per slice:  sum_i w_i x_i = s * sum_i q_i x_i + b * S,  S = sum_i x_i  (HQ4_G32_M5:
// s * (sum_i q_i x_i + 1024 S) + b * S) - the factorisation of the reference's bit-stream GEMVs
// (qwg_aq_slice_dot, Sources/QWMetal/include/qw_dequant_multi.metalh:205-208).
// Element order inside a word fixes which activations pair up: HQ4_G32_M5 keeps element 8w + j at bit
// 4 (j >> 1) + 16 (j & 1) (unpack_hq4_word8, qw_dequant.metalh:42-62), the bit-stream containers element i at bit
// i * bits, so a masked 4-bit word holds elements (k, k + 4), a masked 8-bit word elements (k, k + 2) and a masked 2-bit
// word elements (k, k + 8) (sixteen codes a word; the four mask positions of a byte read as q, 4 q, 16 q and 64 q times
// 2^-24 and get one accumulator each).  A 3-bit stream has no two codes 16 bits apart, but any 32-bit window of it holds a
// code start within bits 0..2 of each half: six windows of the slice's 96 bits (one funnel shift each), placed so that the
// low half's codes start at bit 1 and the high half's at bit 0, give 15 pairs under three masks (fields at bits 1/0, 4/3,
// 7/6: the values read as 2 q, q; 16 q, 8 q; 128 q, 64 q times 2^-24); the low activation of each pair is halved once in
// the prologue so that both halves of a pair share a scale, and each mask gets its own accumulator.  Codes 30 and 31
// are cut out the plain way.  A 6-bit stream works the same way with one pair a window: the window at bit 6 e holds code e
// at bits 0..5 and code e + 3 at bits 18..23 (four times its value: the high activation of the pair is quartered in the
// prologue), fifteen windows for the pairs (e, e + 3) and codes 30, 31 cut out the plain way, one scale class.
#include "qwhip_common.h"

namespace {

#define QCX_FIELDS(X)                                                                                                       \
    X(const uint8_t*, bank) X(const void*, x) X(h1_t*, y16) X(float*, y32) X(uint32_t, N) X(uint32_t, K) X(uint32_t, M)         \
    X(uint32_t, nsl) X(uint32_t, cpr) X(uint32_t, sets) X(uint32_t, gshift) X(uint32_t, bb) X(uint32_t, row_bytes)
QW_ARG_BLOCK(qcx_params, QCX_FIELDS)
// The gate|up form (dense MLP decode, one activation row): the bank holds I gate rows and then the I up rows of the same
// channels, N = 2 I; row slots 2 c and 2 c + 1 of a workgroup are the gate and the up row of its channel c (row sets of even
// index walk the gate half of the bank, odd ones the up half), and the epilogue stores gated(g, u) on the fp32 sums:
// f16 into y16 [I], or fp32 into y32 [I] for a rotation pass behind the launch.
#define QCX_PAIR_FIELDS(X) QCX_FIELDS(X) X(qw_act, ga)
QW_ARG_BLOCK(qcx_params_pair, QCX_PAIR_FIELDS)
__device__ __forceinline__ const qcx_params& qcx_base(const qcx_params& p) { return p; }
__device__ __forceinline__ qcx_params qcx_base(const qcx_params_pair& f) {
    qcx_params p;
#define QCX_TAKE(T, n) p.n = f.n;
    QCX_FIELDS(QCX_TAKE)
#undef QCX_TAKE
    return p;
}

// payload dwords of one 32-column slice: bits * 32 / 32 (HQ4_G32_M5 and 4-bit streams: 4)
template <int FMT>
struct qcx_fmt {
    static constexpr int BITS = FMT == QW_FMT_B8 ? 8 : (FMT == QW_FMT_B2 ? 2 : (FMT == QW_FMT_B3 ? 3 : (FMT == QW_FMT_B6 ? 6 : 4)));
    static constexpr int PW = BITS;
};

struct __attribute__((packed, aligned(4))) qcx_words4 { uint32_t q[4]; };
struct __attribute__((packed, aligned(4))) qcx_words8 { uint32_t q[8]; };

template <int FMT>
struct qcx_slice {
    uint32_t hdr;
    uint32_t q[qcx_fmt<FMT>::PW];
};

// The 16 operand pairs of one activation row for this lane's slice, in the order the masked code words come out.
// 3-bit streams: operand i pairs the elements (QCX_B3_LO[i], QCX_B3_HI[i]); operands 0..6 sit under the first mask
// (6 = codes 30, 31, cut out the plain way), 7..12 under the second, 13..15 under the third
__device__ constexpr int QCX_B3_LO[16] = {0, 3, 10, 13, 20, 23, 30, 1, 4, 11, 14, 21, 24, 2, 12, 22};
__device__ constexpr int QCX_B3_HI[16] = {5, 8, 15, 18, 25, 28, 31, 6, 9, 16, 19, 26, 29, 7, 17, 27};

template <int FMT>
__device__ __forceinline__ float qcx_operands(const h8_t* v, h2_t* xo) {
    const h2_t one = {(h1_t)1.0f, (h1_t)1.0f};
    float s0 = 0.f, s1 = 0.f;
    if constexpr (FMT == QW_FMT_B6) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const h2_t nat = {v[j][2 * k], v[j][2 * k + 1]};
                if (k & 1) s1 = __builtin_amdgcn_fdot2(nat, one, s1, false);
                else s0 = __builtin_amdgcn_fdot2(nat, one, s0, false);
            }
        }
#pragma unroll
        for (int i = 0; i < 15; ++i) {   // operand i: elements (e, e + 3), e = 6 (i / 3) + i % 3
            const int lo = 6 * (i / 3) + i % 3, hi = lo + 3;
            xo[i] = h2_t{v[lo >> 3][lo & 7], v[hi >> 3][hi & 7] * (h1_t)0.25f};
        }
        xo[15] = h2_t{v[3][6], v[3][7]};
        return s0 + s1;
    }
    if constexpr (FMT == QW_FMT_B3) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const h2_t nat = {v[j][2 * k], v[j][2 * k + 1]};
                if (k & 1) s1 = __builtin_amdgcn_fdot2(nat, one, s1, false);
                else s0 = __builtin_amdgcn_fdot2(nat, one, s0, false);
            }
        }
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const int lo = QCX_B3_LO[i], hi = QCX_B3_HI[i];
            const h1_t xl = v[lo >> 3][lo & 7], xh = v[hi >> 3][hi & 7];
            xo[i] = h2_t{i == 6 ? xl : xl * (h1_t)0.5f, xh};   // the windows' low fields read twice their code
        }
        return s0 + s1;
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            h2_t pr;
            if constexpr (FMT == QW_FMT_M5) pr = h2_t{v[j][2 * k], v[j][2 * k + 1]};
            else if constexpr (FMT == QW_FMT_B4) pr = h2_t{v[j][k], v[j][k + 4]};
            else if constexpr (FMT == QW_FMT_B2) pr = h2_t{v[2 * (j >> 1)][4 * (j & 1) + k], v[2 * (j >> 1) + 1][4 * (j & 1) + k]};
            else pr = h2_t{v[j][4 * (k >> 1) + (k & 1)], v[j][4 * (k >> 1) + (k & 1) + 2]};
            if (k & 1) s1 = __builtin_amdgcn_fdot2(pr, one, s1, false);
            else s0 = __builtin_amdgcn_fdot2(pr, one, s0, false);
            xo[4 * j + k] = pr;
        }
    }
    return s0 + s1;
}

// MR activation rows, D slices in flight per lane.  blockDim.x = 32 * cpr * sets;
// dynamic LDS = rows-per-workgroup * cpr * MR * 4 bytes (+ nsl * 80 bytes in front with ROT).
// ROT (MR = 1 only): the activation row arrives un-rotated; the FWHT-32 of its groups runs on the matrix cores into
// an LDS image (16 groups per wave and tile), and each lane then reads its own column from there.
template <int FMT, int XDT, int MR, int D, int LB, bool ROT, typename P = qcx_params>
struct qw_gemv_colx_kernel {
static constexpr int kLaunchBound = LB;
static __device__ __forceinline__ void run(const P& pp) {
    constexpr bool PAIR = !std::is_same<P, qcx_params>::value;
    const qcx_params& p = qcx_base(pp);
    static_assert(!ROT || MR == 1, "fused rotation is built for one activation row");
    static_assert(!PAIR || MR == 1, "the gate|up form is built for one activation row");
    extern __shared__ h8_t qcx_lds[];
    h8_t* xs = qcx_lds;                                                     // ROT: 80 bytes per 32-group (64 used)
    float* qcx_part = (float*)(qcx_lds + (ROT ? (size_t)p.nsl * 5 : 0));    // [row slot][chunk][MR]
    const uint32_t cpr = p.cpr, N = p.N, sets = p.sets;
    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & 31u, hw = tid >> 5;
    const uint32_t set = hw / cpr, chunk = hw - set * cpr;
    const uint32_t g0 = chunk * 32u + lane;
    const bool gvalid = g0 < p.nsl;
    const uint32_t g = gvalid ? g0 : p.nsl - 1u;
    const uint32_t G = gridDim.x;
    uint32_t nrows, nmax, step, mine, first_row;
    if constexpr (PAIR) {
        // channel c of this workgroup is bank channel c G + blockIdx.x; set j walks the channels j / 2, + sets / 2, ... of half
        // j & 1 (sets is even), so row slot trip * sets + j is (channel, half) = (slot / 2, slot & 1)
        const uint32_t h2 = sets >> 1, I = N >> 1;
        if (blockIdx.x >= I) return;
        const uint32_t nch = (I - blockIdx.x + G - 1u) / G;
        const uint32_t sub = set >> 1, half = set & 1u;
        nrows = 2u * nch;
        nmax = (nch + h2 - 1u) / h2;
        step = G * h2 * p.row_bytes;
        mine = nch > sub ? (nch - sub + h2 - 1u) / h2 : 0u;
        first_row = half * I + (mine ? sub : 0u) * G + blockIdx.x;
    } else {
        if (blockIdx.x >= N) return;
        nrows = (N - blockIdx.x + G - 1u) / G;               // row slots of this workgroup
        nmax = (nrows + sets - 1u) / sets;                   // trip count, uniform over the workgroup
        step = G * sets * p.row_bytes;                       // bytes between consecutive rows of one set
        mine = nrows > set ? (nrows - set + sets - 1u) / sets : 0u;
        first_row = (mine ? set : 0u) * G + blockIdx.x;
    }
    uint32_t hdr_off, pay_off;
    if constexpr (FMT == QW_FMT_M5) {
        hdr_off = g * 20u;
        pay_off = hdr_off + 4u;
    } else {
        hdr_off = (g >> p.gshift) * p.bb;
        pay_off = hdr_off + 4u + (g & ((1u << p.gshift) - 1u)) * (4u * qcx_fmt<FMT>::PW);
    }
    uint32_t off = first_row * p.row_bytes;
    const uint32_t off_max = off + (mine ? mine - 1u : 0u) * step;   // loads past the set's last row re-read it

    // 1. activation loads first (they return in order, ahead of the weight prefetch); rows past M re-read row M - 1
    u4_t xraw[MR][4];   // 8 two-byte activations per register quad, converted one activation row at a time below
    constexpr int XT = 5;                                  // rotation tiles per wave: covers 2 * cpr tiles over cpr / 2 waves
    h8_t xv[ROT ? XT : 1];
    const uint32_t wave = tid >> 6, l64 = tid & 63u, nwf = blockDim.x >> 6;   // full waves only take rotation tiles
    if constexpr (ROT) {
#pragma unroll
        for (int t = 0; t < XT; ++t) {
            const uint32_t gg = min((wave + nwf * t) * 16u + (l64 & 15u), p.nsl - 1u);
            xv[t] = qw_load_x8_f16<XDT>(p.x, (uint64_t)gg * 32u + 8u * (l64 >> 4));
        }
    } else {
#pragma unroll
        for (int m = 0; m < MR; ++m) {
            const uint64_t at = (uint64_t)min((uint32_t)m, p.M - 1u) * p.K + (uint64_t)g * 32u;
#pragma unroll
            for (int j = 0; j < 4; ++j) xraw[m][j] = *(const u4_t*)((const uint16_t*)p.x + at + 8u * j);
        }
    }
    __builtin_amdgcn_sched_barrier(0);
    // 2. first weight rows
    qcx_slice<FMT> buf[D];
    auto issue = [&](int slot) {
        // one 32-bit sum per address (the bank is under 4 GiB): scalar base + 32-bit lane offset addressing
        const uint32_t o_hdr = (uint32_t)off + hdr_off, o_pay = (uint32_t)off + pay_off;
        buf[slot].hdr = *(const uint32_t*)(p.bank + o_hdr);
        if constexpr (FMT == QW_FMT_B2 || FMT == QW_FMT_B3 || FMT == QW_FMT_B6) {
#pragma unroll
            for (int j = 0; j < qcx_fmt<FMT>::PW; ++j) buf[slot].q[j] = *(const uint32_t*)(p.bank + o_pay + 4 * j);
        } else if constexpr (FMT == QW_FMT_B8) {
            const qcx_words8 w = *(const qcx_words8*)(p.bank + o_pay);
#pragma unroll
            for (int j = 0; j < 8; ++j) buf[slot].q[j] = w.q[j];
        } else {
            const qcx_words4 w = *(const qcx_words4*)(p.bank + o_pay);
#pragma unroll
            for (int j = 0; j < 4; ++j) buf[slot].q[j] = w.q[j];
        }
        off = min(off + step, off_max);
    };
#pragma unroll
    for (int j = 0; j < D; ++j) issue(j);
    __builtin_amdgcn_sched_barrier(0);
    // 3. this lane's operands
    if constexpr (ROT) {
        if (wave < nwf) {
            h8_t h_lo, h_hi;
            qw_hadamard_pair(l64 & 15u, l64 >> 4, h_lo, h_hi);
#pragma unroll
            for (int t = 0; t < XT; ++t) qw_rotate_tile_to_lds(xv[t], wave + nwf * t, p.nsl, l64, true, h_lo, h_hi, xs);
        }
        __syncthreads();
    }
    h2_t xo[MR][16];
    float S[MR];
#pragma unroll
    for (int m = 0; m < MR; ++m) {
        h8_t xr[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            if constexpr (ROT) {
                xr[j] = xs[g * 5u + j];
            } else if constexpr (XDT == QWHIP_F16) {
                xr[j] = __builtin_bit_cast(h8_t, xraw[m][j]);
            } else {
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    xr[j][2 * e] = (h1_t)__uint_as_float(xraw[m][j][e] << 16);
                    xr[j][2 * e + 1] = (h1_t)__uint_as_float(xraw[m][j][e] & 0xFFFF0000u);
                }
            }
        }
        S[m] = qcx_operands<FMT>(xr, xo[m]);
        __builtin_amdgcn_sched_barrier(0);   // keeps the conversion of row m + 1 from overlapping row m's registers
    }

    uint32_t rslot = set;   // row slot being consumed
    for (uint32_t ib = 0; ib < nmax; ib += D) {
#pragma unroll
        for (int j = 0; j < D; ++j) {
            if (ib + j >= nmax) break;
            const qcx_slice<FMT> b = buf[j];
            issue(j);
            uint32_t ow[16];   // masked code words, operand order
            if constexpr (FMT == QW_FMT_B6) {
                // window i at bit 6 e of the 192-bit slice, e = 6 (i / 3) + i % 3: code e at bits 0..5, code e + 3 at bits 18..23
                constexpr uint32_t M = 0x00FC003Fu;
#pragma unroll
                for (int i = 0; i < 15; ++i) {
                    const int bit = 6 * (6 * (i / 3) + i % 3), wd = bit >> 5, sh = bit & 31;
                    const uint32_t win = sh == 0 ? b.q[wd] : __builtin_amdgcn_alignbit(b.q[wd + 1], b.q[wd], sh);
                    ow[i] = win & M;
                }
                ow[15] = ((b.q[5] >> 20) & 0x3Fu) | ((b.q[5] >> 10) & 0x003F0000u);   // codes 30 and 31
            } else if constexpr (FMT == QW_FMT_B3) {
                // windows of the 96-bit slice at bits -1, 8, 29, 38, 59, 68: low-half codes start at window bit 1, high-half
                // codes at bit 16 (elements: QCX_B3_LO / QCX_B3_HI)
                const uint32_t w0 = b.q[0], w1 = b.q[1], w2 = b.q[2];
                const uint32_t wa = w0 << 1;
                const uint32_t wb = __builtin_amdgcn_alignbit(w1, w0, 8);
                const uint32_t wc = __builtin_amdgcn_alignbit(w1, w0, 29);
                const uint32_t wd = __builtin_amdgcn_alignbit(w2, w1, 6);
                const uint32_t we = __builtin_amdgcn_alignbit(w2, w1, 27);
                const uint32_t wf = w2 >> 4;
                constexpr uint32_t M0 = 0x0007000Eu, M1 = 0x00380070u, M2 = 0x01C00380u;
                ow[0] = wa & M0;
                ow[1] = wb & M0;
                ow[2] = wc & M0;
                ow[3] = wd & M0;
                ow[4] = we & M0;
                ow[5] = wf & M0;
                ow[6] = ((w2 >> 26) & 7u) | ((w2 >> 13) & 0x00070000u);   // codes 30 and 31
                ow[7] = wa & M1;
                ow[8] = wb & M1;
                ow[9] = wc & M1;
                ow[10] = wd & M1;
                ow[11] = we & M1;
                ow[12] = wf & M1;
                ow[13] = wa & M2;
                ow[14] = wc & M2;
                ow[15] = we & M2;
            } else if constexpr (FMT == QW_FMT_B2) {
                // operand 8 w + j: elements (16 w + j, 16 w + j + 8), masked in place at bits 2 (j & 3) of the bytes 0 / 2 of the
                // word (j < 4) or of the word shifted down a byte (j >= 4)
#pragma unroll
                for (int w = 0; w < 2; ++w) {
                    const uint32_t q = b.q[w], q8 = q >> 8;
                    ow[8 * w + 0] = q & 0x00030003u;
                    ow[8 * w + 1] = q & 0x000C000Cu;
                    ow[8 * w + 2] = q & 0x00300030u;
                    ow[8 * w + 3] = q & 0x00C000C0u;
                    ow[8 * w + 4] = q8 & 0x00030003u;
                    ow[8 * w + 5] = q8 & 0x000C000Cu;
                    ow[8 * w + 6] = q8 & 0x00300030u;
                    ow[8 * w + 7] = q8 & 0x00C000C0u;
                }
            } else if constexpr (FMT == QW_FMT_B8) {
#pragma unroll
                for (int w = 0; w < 8; ++w) {
                    ow[2 * w] = b.q[w] & 0x00FF00FFu;
                    ow[2 * w + 1] = (b.q[w] >> 8) & 0x00FF00FFu;
                }
            } else {
#pragma unroll
                for (int w = 0; w < 4; ++w) {
                    const uint32_t q = b.q[w], q8 = q >> 8;
                    ow[4 * w + 0] = q & 0x000F000Fu;
                    ow[4 * w + 1] = q & 0x00F000F0u;
                    ow[4 * w + 2] = q8 & 0x000F000Fu;
                    ow[4 * w + 3] = q8 & 0x00F000F0u;
                }
            }
            const h2_t hd = __builtin_bit_cast(h2_t, b.hdr);
            const float sc = (float)hd[0], bi = (float)hd[1];
#pragma unroll
            for (int m = 0; m < MR; ++m) {
                float a0 = 0.f, a1 = 0.f, a2 = 0.f, a3 = 0.f;
                if constexpr (FMT == QW_FMT_M5) {
                    // The arithmetic of the m = 1 kernel of gemv_col.hip (qw_gemv_colw_kernel), operation for operation: two
                    // sums in word order (codes at bits 0..3 / 4..7), s q + ((1024 s + b) S 2^-24) at 2^-24 of full scale,
                    // the factor back after the chunk sum - so that a row gets the same bits from either kernel.
#pragma unroll
                    for (int i = 0; i < 16; i += 2) {
                        a0 = __builtin_amdgcn_fdot2(__builtin_bit_cast(h2_t, ow[i + 0]), xo[m][i + 0], a0, false);
                        a1 = __builtin_amdgcn_fdot2(__builtin_bit_cast(h2_t, ow[i + 1]), xo[m][i + 1], a1, false);
                    }
                    const float mt = __builtin_fmaf(sc, 1024.0f, bi) * (S[m] * 5.9604644775390625e-08f);
                    float v = __builtin_fmaf(sc, __builtin_fmaf(a1, 0.0625f, a0), mt);
                    v = gvalid ? v : 0.0f;
                    v = qw_reduce32_dpp(v);
                    if (lane == 31u && rslot < nrows) qcx_part[(rslot * cpr + chunk) * MR + m] = v;
                    continue;
                }
                if constexpr (FMT == QW_FMT_B3) {
                    // a0, a1: the first mask's seven operands; a2: the second mask's six; a3: the third mask's three
#pragma unroll
                    for (int i = 0; i < 7; ++i) {
                        if (i & 1) a1 = __builtin_amdgcn_fdot2(__builtin_bit_cast(h2_t, ow[i]), xo[m][i], a1, false);
                        else a0 = __builtin_amdgcn_fdot2(__builtin_bit_cast(h2_t, ow[i]), xo[m][i], a0, false);
                    }
#pragma unroll
                    for (int i = 7; i < 13; ++i) a2 = __builtin_amdgcn_fdot2(__builtin_bit_cast(h2_t, ow[i]), xo[m][i], a2, false);
#pragma unroll
                    for (int i = 13; i < 16; ++i) a3 = __builtin_amdgcn_fdot2(__builtin_bit_cast(h2_t, ow[i]), xo[m][i], a3, false);
                } else {
#pragma unroll
                    for (int i = 0; i < 16; i += 4) {
                        a0 = __builtin_amdgcn_fdot2(__builtin_bit_cast(h2_t, ow[i + 0]), xo[m][i + 0], a0, false);
                        a1 = __builtin_amdgcn_fdot2(__builtin_bit_cast(h2_t, ow[i + 1]), xo[m][i + 1], a1, false);
                        a2 = __builtin_amdgcn_fdot2(__builtin_bit_cast(h2_t, ow[i + 2]), xo[m][i + 2], a2, false);
                        a3 = __builtin_amdgcn_fdot2(__builtin_bit_cast(h2_t, ow[i + 3]), xo[m][i + 3], a3, false);
                    }
                }
                float q;
                if constexpr (FMT == QW_FMT_B3) {
                    q = __builtin_fmaf(a2, 2097152.0f, (a0 + a1) * 16777216.0f);   // fields at bits 4 / 3 of the halves: 8 q
                    q = __builtin_fmaf(a3, 262144.0f, q);                          // bits 7 / 6: 64 q
                } else if constexpr (FMT == QW_FMT_B8 || FMT == QW_FMT_B6) {
                    q = ((a0 + a1) + (a2 + a3)) * 16777216.0f;
                } else if constexpr (FMT == QW_FMT_B2) {
                    q = __builtin_fmaf(a1, 4194304.0f, a0 * 16777216.0f);     // codes at bits 0..1 and 2..3 of a byte
                    q = __builtin_fmaf(a2, 1048576.0f, q);                    // bits 4..5
                    q = __builtin_fmaf(a3, 262144.0f, q);                     // bits 6..7
                } else {
                    q = __builtin_fmaf(a0 + a2, 16777216.0f, FMT == QW_FMT_M5 ? 1024.0f * S[m] : 0.0f);   // codes at bits 0..3
                    q = __builtin_fmaf(a1 + a3, 1048576.0f, q);                                           // codes at bits 4..7
                }
                float v = __builtin_fmaf(sc, q, bi * S[m]);
                v = gvalid ? v : 0.0f;
                v = qw_reduce32_dpp(v);
                if (lane == 31u && rslot < nrows) qcx_part[(rslot * cpr + chunk) * MR + m] = v;
            }
            rslot += sets;
        }
    }
    __syncthreads();
    if constexpr (PAIR) {
        for (uint32_t c = tid; 2u * c < nrows; c += blockDim.x) {
            float gsum = 0.f, usum = 0.f;
            for (uint32_t k = 0; k < cpr; ++k) {
                gsum += qcx_part[(2u * c) * cpr + k];
                usum += qcx_part[(2u * c + 1u) * cpr + k];
            }
            if constexpr (FMT == QW_FMT_M5) {
                gsum *= 16777216.0f;
                usum *= 16777216.0f;
            }
            const float a = qw_gated(gsum, usum, pp.ga);
            if (p.y32) p.y32[c * G + blockIdx.x] = a;
            else p.y16[c * G + blockIdx.x] = (h1_t)a;
        }
        return;
    }
    // 4. fixed-order sum of the chunk partials of each (row, activation row)
    for (uint32_t t = tid; t < nrows * p.M; t += blockDim.x) {
        const uint32_t m = t / nrows, s = t - m * nrows;
        float v = 0.f;
        for (uint32_t c = 0; c < cpr; ++c) v += qcx_part[(s * cpr + c) * MR + m];
        if constexpr (FMT == QW_FMT_M5) v *= 16777216.0f;
        const uint64_t at = (uint64_t)m * N + s * G + blockIdx.x;
        if (p.y32) p.y32[at] = v;
        if (p.y16) p.y16[at] = (h1_t)v;
    }
}
};

template <int FMT, int XDT, int MR, int D, int LB, bool ROT = false>
void qcx_launch1(hipStream_t st, const qcx_params& p, uint32_t wgs, uint32_t threads, size_t lds) {
    qw_launch_scalar<qw_gemv_colx_kernel<FMT, XDT, MR, D, LB, ROT>>(dim3(wgs), dim3(threads), lds, st, p);
}

template <int FMT, int XDT>
void qcx_launch_m(hipStream_t st, const qcx_params& p, uint32_t mr, bool rotate, uint32_t wgs, uint32_t threads, size_t lds) {
    if (rotate) qcx_launch1<FMT, XDT, 1, 2, 1024, true>(st, p, wgs, threads, lds);
    else if (mr == 1) qcx_launch1<FMT, XDT, 1, 2, 1024>(st, p, wgs, threads, lds);
    else if (mr == 2) qcx_launch1<FMT, XDT, 2, 2, 1024>(st, p, wgs, threads, lds);
    else if (mr == 4) qcx_launch1<FMT, XDT, 4, 3, 576>(st, p, wgs, threads, lds);
    else qcx_launch1<FMT, XDT, 8, 3, 512>(st, p, wgs, threads, lds);
}

}  // namespace

// Gate|up form of the column-stationary kernel for one activation row over a validated gate|up bank of n = 2 I rows (any
// container the kernel takes): gated(Wg . x, Wu . x) on the fp32 sums, as f16 into act16 [I] or as fp32 into gated32 [I] (for a
// rotation pass behind the launch).  false when the shape is outside the envelope.
bool qw_colx_pair_gemv(hipStream_t st, const qwhip_weight_view* w, int fmt, uint32_t gshift, uint32_t bb, uint64_t row_bytes,
                       const void* x, uint32_t x_dtype, bool rotate, void* act16, float* gated32, const qw_act ga, hipError_t* err) {
    if (w->n & 1u) return false;
    const uint32_t inter = w->n / 2u;
    const uint32_t nsl = w->k / 32u, cpr = (nsl + 31u) / 32u;
    if (64u * cpr > 1024u || inter < 64u) return false;               // two row sets at least
    if ((uint64_t)w->n * row_bytes >= (1ull << 32)) return false;     // 32-bit offsets inside the bank
    if (((uintptr_t)x & 15u) != 0) return false;
    uint32_t sets = min(8u, max(2u, 512u / (32u * cpr))) & ~1u;       // even, at most eight waves a workgroup where two sets allow
    const uint32_t h2 = sets / 2u;
    const uint32_t threads = 32u * cpr * sets;
    const uint32_t waves = (threads + 63u) / 64u;
    uint32_t wgs = 256u * max(1u, (16u + waves / 2u) / waves);
    wgs = min(wgs, max(1u, inter / h2));
    const uint32_t ch_per_wg = qwhip_cdiv(inter, wgs);
    if (rotate && (threads >> 6) * 5u * 16u < nsl) return false;      // rotation tiles: five per full wave
    const size_t lds = (size_t)2u * ch_per_wg * cpr * 4u + (rotate ? (size_t)nsl * 80u : 0u);
    if (lds > 60u * 1024u) return false;
    qcx_params_pair p;
    p.bank = (const uint8_t*)w->blocks;
    p.x = x;
    p.y16 = (h1_t*)act16;
    p.y32 = gated32;
    p.N = w->n;
    p.K = w->k;
    p.M = 1;
    p.nsl = nsl;
    p.cpr = cpr;
    p.sets = sets;
    p.gshift = gshift;
    p.bb = bb;
    p.row_bytes = (uint32_t)row_bytes;
    p.ga = ga;
#define QCX_PAIR(F, DT)                                                                                                         \
    do {                                                                                                                        \
        if (rotate) qw_launch_scalar<qw_gemv_colx_kernel<F, DT, 1, 2, 1024, true, qcx_params_pair>>(dim3(wgs), dim3(threads), lds, st, p);   \
        else qw_launch_scalar<qw_gemv_colx_kernel<F, DT, 1, 2, 1024, false, qcx_params_pair>>(dim3(wgs), dim3(threads), lds, st, p);         \
    } while (0)
#define QCX_PAIR_F(DT)                                                  \
    switch (fmt) {                                                      \
        case QW_FMT_M5: QCX_PAIR(QW_FMT_M5, DT); break;                 \
        case QW_FMT_B4: QCX_PAIR(QW_FMT_B4, DT); break;                 \
        case QW_FMT_B8: QCX_PAIR(QW_FMT_B8, DT); break;                 \
        case QW_FMT_B2: QCX_PAIR(QW_FMT_B2, DT); break;                 \
        case QW_FMT_B3: QCX_PAIR(QW_FMT_B3, DT); break;                 \
        default: QCX_PAIR(QW_FMT_B6, DT); break;                        \
    }
    if (x_dtype == QWHIP_F16) { QCX_PAIR_F(QWHIP_F16) } else { QCX_PAIR_F(QWHIP_BF16) }
#undef QCX_PAIR_F
#undef QCX_PAIR
    *err = hipGetLastError();
    return true;
}

// Tries the column-stationary small-M kernel for a validated call; false when the shape is outside its envelope:
// up to eight activation rows already in the container's basis, or one row to rotate (`rotate`).
// fmt: QW_FMT_M5 / QW_FMT_B4 / QW_FMT_B8, and the 2-, 3- and 6-bit streams QW_FMT_B2 / B3 / B6.  `tune`: 0 = automatic; bits 0..1 scale the grid (1 -> half, 2 -> double).
bool qw_colx_gemv(hipStream_t st, const qwhip_weight_view* w, int fmt, uint32_t gshift, uint32_t bb, uint64_t row_bytes,
                  const void* x, uint32_t x_dtype, uint32_t m, bool rotate, void* y16, float* y32, uint32_t tune,
                  hipError_t* err) {
    if (m == 0 || m > 8 || (rotate && m != 1)) return false;
    const uint32_t mr = m <= 1 ? 1u : (m <= 2 ? 2u : (m <= 4 ? 4u : 8u));
    const uint32_t nsl = w->k / 32u, cpr = (nsl + 31u) / 32u;
    // threads per workgroup follow the register budget: 128 VGPRs up to two activation rows, 170 for four, 256 for eight
    const uint32_t lb = mr <= 2 ? 1024u : (mr == 4 ? 576u : 512u);
    const uint32_t waves_cu = mr <= 2 ? 16u : (mr == 4 ? 12u : 8u);
    if (32u * cpr > lb) return false;
    if ((uint64_t)w->n * row_bytes >= (1ull << 32)) return false;   // 32-bit offsets inside the bank
    if (((uintptr_t)x & 15u) != 0) return false;
    uint32_t sets = lb / (32u * cpr);
    sets = min(sets, 8u);
    // One or two activation rows: at most eight waves behind a workgroup's two barriers (fifteen-wave workgroups measured
    // 3 % slower on 7168 x 5120 at 8 bits), and where sixteen waves per compute unit would leave a half-wave fewer than three
    // rows, eight waves with twice the rows each (a wave's start-up - activations, operands - is paid half as often:
    // 4096 x 4096 at 4 bits 5.04 -> 4.74 us).
    if (mr <= 2u) sets = min(sets, max(1u, 512u / (32u * cpr)));
    if ((tune >> 2) & 3u) sets = min(sets, ((tune >> 2) & 3u) + 1u);   // tuning: at most 2 / 3 / 4 row sets per workgroup
    const uint32_t threads = 32u * cpr * sets;
    const uint32_t waves = (threads + 63u) / 64u;
    const uint32_t target = (mr <= 2u && (uint64_t)w->n * cpr < 3u * 256u * 32u) ? 8u : waves_cu;
    uint32_t wgs = 256u * max(1u, (target + waves / 2u) / waves);
    if ((tune & 3u) == 1u) wgs /= 2u;
    if ((tune & 3u) == 2u) wgs *= 2u;
    wgs = min(wgs, max(1u, w->n / sets));
    const uint32_t rows_per_wg = qwhip_cdiv(w->n, wgs);
    if (rotate && (threads >> 6) * 5u * 16u < nsl) return false;   // rotation tiles: five per full wave
    const size_t lds = (size_t)rows_per_wg * cpr * mr * 4u + (rotate ? (size_t)nsl * 80u : 0u);
    if (lds > 60u * 1024u) return false;
    qcx_params p;
    p.bank = (const uint8_t*)w->blocks;
    p.x = x;
    p.y16 = (h1_t*)y16;
    p.y32 = y32;
    p.N = w->n;
    p.K = w->k;
    p.M = m;
    p.nsl = nsl;
    p.cpr = cpr;
    p.sets = sets;
    p.gshift = gshift;
    p.bb = bb;
    p.row_bytes = (uint32_t)row_bytes;
    if (x_dtype == QWHIP_F16) {
        if (fmt == QW_FMT_M5) qcx_launch_m<QW_FMT_M5, QWHIP_F16>(st, p, mr, rotate, wgs, threads, lds);
        else if (fmt == QW_FMT_B4) qcx_launch_m<QW_FMT_B4, QWHIP_F16>(st, p, mr, rotate, wgs, threads, lds);
        else if (fmt == QW_FMT_B8) qcx_launch_m<QW_FMT_B8, QWHIP_F16>(st, p, mr, rotate, wgs, threads, lds);
        else if (fmt == QW_FMT_B2) qcx_launch_m<QW_FMT_B2, QWHIP_F16>(st, p, mr, rotate, wgs, threads, lds);
        else if (fmt == QW_FMT_B3) qcx_launch_m<QW_FMT_B3, QWHIP_F16>(st, p, mr, rotate, wgs, threads, lds);
        else qcx_launch_m<QW_FMT_B6, QWHIP_F16>(st, p, mr, rotate, wgs, threads, lds);
    } else {
        if (fmt == QW_FMT_M5) qcx_launch_m<QW_FMT_M5, QWHIP_BF16>(st, p, mr, rotate, wgs, threads, lds);
        else if (fmt == QW_FMT_B4) qcx_launch_m<QW_FMT_B4, QWHIP_BF16>(st, p, mr, rotate, wgs, threads, lds);
        else if (fmt == QW_FMT_B8) qcx_launch_m<QW_FMT_B8, QWHIP_BF16>(st, p, mr, rotate, wgs, threads, lds);
        else if (fmt == QW_FMT_B2) qcx_launch_m<QW_FMT_B2, QWHIP_BF16>(st, p, mr, rotate, wgs, threads, lds);
        else if (fmt == QW_FMT_B3) qcx_launch_m<QW_FMT_B3, QWHIP_BF16>(st, p, mr, rotate, wgs, threads, lds);
        else qcx_launch_m<QW_FMT_B6, QWHIP_BF16>(st, p, mr, rotate, wgs, threads, lds);
    }
    *err = hipGetLastError();
    return true;
}
