// Small-M GEMV (m = 1..16) over any 4- or 8-bit container, activations already in the container's basis:
// coalesced block loads feeding the 16-block matrix instruction v_mfma_f32_4x4x4_16B_f16.
//
// That instruction multiplies 16 independent 4x4x4 blocks; block b lives in lanes 4b .. 4b + 3:
//     D[b][i][j] = sum_k A[lane 4b + i][k] * B[lane 4b + j][k],  lane 4b + j holds D[b][0..3][j]
// (layout and exactness with f16 subnormal operands checked on the device).  Here block b is one 32-column slice of
// the bank, i is one of 4 consecutive bank rows and j one of 4 activation rows: lane (b, i) loads slice b of row i
// (16 consecutive slices x 4 rows per wave and load: four contiguous runs of the bank per instruction), lane (b, j)
// keeps the 32 activations of row 4 mg + j for slice b in registers, and 8 matrix instructions per group of four
// activation rows contract the slice.  Because the blocks are independent each slice meets its own activations: no
// transposition, no LDS on the way in, and the VALU cost no longer grows with m (16 v_dot2 per slice and row in the
// dot2 form against 2 matrix instructions here).
//
// Arithmetic is the factorised form of the reference's bit-stream GEMVs (qwg_aq_slice_dot,
// Sources/QWMetal/include/qw_dequant_multi.metalh:205-208): the masked code words are the A operands as they are
// (f16 subnormals q * 2^-24, 16 q * 2^-24 for the nibbles at bits 4..7 / 20..23), products exact, fp32 accumulation,
// and  s * sum(q x) + b * sum(x)  per slice and row afterwards (HQ4_G32_M5: s * (sum(q x) + 1024 sum(x)) + b * sum(x),
// unpack_hq4_word8, qw_dequant.metalh:42-62).  The header of row i reaches the lanes of its block by quad broadcast.
//
// Launch shape: persistent, grid-stride over row quads (quad slot s of workgroup w is quad s * gridDim.x + w, so the
// grid reads one contiguous band of the bank at a time).  Wave wv of a row set owns slice chunk kr * wpr + wv
// (16 slices) in K range kr; long rows take several K ranges, the activations of one range in registers at a time
// (the next range's fetched meanwhile, the weight prefetch running on across the boundary), partial sums
// accumulating in LDS per (quad slot, wave, 16-lane row) and summed in a fixed order at the end.
#include <atomic>

#include "qwhip_common.h"

namespace {

#define QQ_FIELDS(X)                                                                                                        \
    X(const uint8_t*, bank) X(const void*, x) X(h1_t*, y16) X(float*, y32) X(uint32_t, N) X(uint32_t, K) X(uint32_t, M)         \
    X(uint32_t, nsl) X(uint32_t, wpr) X(uint32_t, sets) X(uint32_t, nkr) X(uint32_t, gshift) X(uint32_t, bb) X(uint32_t, row_bytes)
QW_ARG_BLOCK(qq_params, QQ_FIELDS)

struct __attribute__((packed, aligned(4))) qq_words4 { uint32_t q[4]; };
struct __attribute__((packed, aligned(4))) qq_words8 { uint32_t q[8]; };

template <int FMT>
struct qq_slice {
    uint32_t hdr;
    uint32_t q[FMT == QW_FMT_B8 ? 8 : 4];
};

#define QQ_DPP(v, ctrl) __builtin_amdgcn_update_dpp(0, (int)(v), ctrl, 0xF, 0xF, true)
#define QQ_DPP_F32(v, ctrl) __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), ctrl, 0xF, 0xF, true))

// MG groups of four activation rows, D row quads in flight per lane.  blockDim.x = 64 * wpr * sets;
// dynamic LDS = quad-slots-per-workgroup * (4 wpr) * (4 MG) * 16 bytes.
template <int FMT, int XDT, int MG, int D, int LB>
struct qw_gemv_quad_kernel {
static constexpr int kLaunchBound = LB;
static __device__ __forceinline__ void run(const qq_params& p) {
    extern __shared__ f4_t qq_part[];   // [quad slot][wave of the set * 4 + 16-lane row][activation row] -> 4 bank rows
    const uint32_t N = p.N, wpr = p.wpr, sets = p.sets;
    const uint32_t tid = threadIdx.x;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6), l64 = tid & 63u;
    const uint32_t b = l64 >> 2, j = l64 & 3u;
    const uint32_t set = wave / wpr, wv = wave - set * wpr;
    const uint32_t G = gridDim.x;
    const uint32_t NQ = (N + 3u) >> 2;
    if (blockIdx.x >= NQ) return;
    const uint32_t nq = (NQ - blockIdx.x + G - 1u) / G;    // quad slots of this workgroup
    const uint32_t nmax = (nq + sets - 1u) / sets;          // trip count, uniform over the workgroup
    const uint32_t mine = nq > set ? (nq - set + sets - 1u) / sets : 0u;
    const uint32_t W16 = wpr * 4u;
    const uint32_t step = G * sets * 4u * p.row_bytes;      // bytes between consecutive quads of one set

    // this lane's bank row inside a quad is j (the A role); rows past the bank re-read its last row (never stored)
    const uint32_t q_first = (mine ? set : 0u) * G + blockIdx.x;
    const uint32_t off_first = min(4u * q_first + j, N - 1u) * p.row_bytes;
    const uint32_t last_quad = q_first + (mine ? mine - 1u : 0u) * G * sets;
    const uint32_t off_max = min(4u * last_quad + j, N - 1u) * p.row_bytes;   // loads past the set's last quad re-read it
    // slice of this lane in K range kr (clamped into the row) and its byte offsets inside a bank row
    auto slice_of = [&](uint32_t kr, uint32_t& hdr_off, uint32_t& pay_off) {
        const uint32_t g = min((kr * wpr + wv) * 16u + b, p.nsl - 1u);
        if constexpr (FMT == QW_FMT_M5) {
            hdr_off = g * 20u;
            pay_off = hdr_off + 4u;
        } else {
            hdr_off = (g >> p.gshift) * p.bb;
            pay_off = hdr_off + 4u + (g & ((1u << p.gshift) - 1u)) * (FMT == QW_FMT_B8 ? 32u : 16u);
        }
        return g;
    };
    // The weight prefetch runs ahead of the consumer across K ranges: after the last quad of a range it goes on with
    // the first quad of the next one, so a range boundary costs no memory round trip.
    uint32_t i_kr = 0, i_left = nmax, i_off = off_first, i_hdr, i_pay;
    slice_of(0, i_hdr, i_pay);
    qq_slice<FMT> buf[D];
    auto issue = [&](int slot) {
        // one 32-bit sum per address (the bank is under 4 GiB): scalar base + 32-bit lane offset addressing
        const uint32_t o_hdr = i_off + i_hdr, o_pay = i_off + i_pay;
        buf[slot].hdr = *(const uint32_t*)(p.bank + o_hdr);
        if constexpr (FMT == QW_FMT_B8) {
            const qq_words8 w = *(const qq_words8*)(p.bank + o_pay);
#pragma unroll
            for (int c = 0; c < 8; ++c) buf[slot].q[c] = w.q[c];
        } else {
            const qq_words4 w = *(const qq_words4*)(p.bank + o_pay);
#pragma unroll
            for (int c = 0; c < 4; ++c) buf[slot].q[c] = w.q[c];
        }
        i_off = min(i_off + step, off_max);
        if (--i_left == 0u && i_kr + 1u < p.nkr) {   // uniform over the workgroup
            ++i_kr;
            slice_of(i_kr, i_hdr, i_pay);
            i_off = off_first;
            i_left = nmax;
        }   // past the last range i_off stays on the last quad: its slices again (still in the caches, never consumed), where
            // the range's first quads, read long ago, would come from HBM a second time
    };
    // Activations of a K range: with up to eight activation rows the next range's are fetched while this one is
    // contracted (they share the registers of the raw loads); with more rows they are loaded at the range's start.
    constexpr bool XPF = MG <= 2;
    u4_t xraw[MG][4];
    auto load_x = [&](uint32_t kr) {
        uint32_t ho, po;
        const uint32_t g = slice_of(kr, ho, po);
#pragma unroll
        for (int mg = 0; mg < MG; ++mg) {
            const uint64_t at = (uint64_t)min(4u * mg + j, p.M - 1u) * p.K + (uint64_t)g * 32u;
#pragma unroll
            for (int c = 0; c < 4; ++c) xraw[mg][c] = *(const u4_t*)((const uint16_t*)p.x + at + 8u * c);
        }
    };
    // 1. activation loads of the first K range first, then the first row quads
    if (XPF) load_x(0);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int d = 0; d < D; ++d) issue(d);
    __builtin_amdgcn_sched_barrier(0);

    for (uint32_t kr = 0; kr < p.nkr; ++kr) {
        const bool gvalid = (kr * wpr + wv) * 16u + b < p.nsl;
        if (!XPF) load_x(kr);
        // 2. B operands: pairs in the order the masked code words come out, zero for slices past the row's end
        h4_t xb[MG][8];
        float S[MG];
#pragma unroll
        for (int mg = 0; mg < MG; ++mg) {
            h8_t xr[4];
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                if constexpr (XDT == QWHIP_F16) {
                    xr[c] = __builtin_bit_cast(h8_t, xraw[mg][c]);
                } else {
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        xr[c][2 * e] = (h1_t)__uint_as_float(xraw[mg][c][e] << 16);
                        xr[c][2 * e + 1] = (h1_t)__uint_as_float(xraw[mg][c][e] & 0xFFFF0000u);
                    }
                }
                if (!gvalid) xr[c] = h8_t{0, 0, 0, 0, 0, 0, 0, 0};
            }
            const h2_t one = {(h1_t)1.0f, (h1_t)1.0f};
            float s0 = 0.f, s1 = 0.f;
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                // operand pair k of word group c, as in the dot2 form: M5 (2k, 2k+1), 4-bit stream (k, k+4),
                // 8-bit stream word 2c + (k >> 1): (k & 1, (k & 1) + 2)
                h2_t pr[4];
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    if constexpr (FMT == QW_FMT_M5) pr[k] = h2_t{xr[c][2 * k], xr[c][2 * k + 1]};
                    else if constexpr (FMT == QW_FMT_B4) pr[k] = h2_t{xr[c][k], xr[c][k + 4]};
                    else pr[k] = h2_t{xr[c][4 * (k >> 1) + (k & 1)], xr[c][4 * (k >> 1) + (k & 1) + 2]};
                    if (k & 1) s1 = __builtin_amdgcn_fdot2(pr[k], one, s1, false);
                    else s0 = __builtin_amdgcn_fdot2(pr[k], one, s0, false);
                }
                if constexpr (FMT == QW_FMT_B8) {   // one scale: consecutive pairs share an instruction
                    xb[mg][2 * c] = h4_t{pr[0][0], pr[0][1], pr[1][0], pr[1][1]};
                    xb[mg][2 * c + 1] = h4_t{pr[2][0], pr[2][1], pr[3][0], pr[3][1]};
                } else {                            // low-nibble pairs (0, 2) and high-nibble pairs (1, 3) apart
                    xb[mg][2 * c] = h4_t{pr[0][0], pr[0][1], pr[2][0], pr[2][1]};
                    xb[mg][2 * c + 1] = h4_t{pr[1][0], pr[1][1], pr[3][0], pr[3][1]};
                }
            }
            S[mg] = s0 + s1;
            __builtin_amdgcn_sched_barrier(0);
        }

        if (XPF && kr + 1u < p.nkr) load_x(kr + 1u);
        uint32_t qslot = set;   // quad slot being consumed
        for (uint32_t ib = 0; ib < nmax; ib += D) {
#pragma unroll
            for (int d = 0; d < D; ++d) {
                if (ib + d >= nmax) break;
                const qq_slice<FMT> blk = buf[d];
                issue(d);
                // A operands: masked code words, paired like the B operands
                h4_t aw[8];
                if constexpr (FMT == QW_FMT_B8) {
#pragma unroll
                    for (int w = 0; w < 8; ++w) {
                        // bytes (0, 2) and (1, 3) of the word as two pairs of f16 subnormals: one mask, one byte permute
                        const uint32_t lo = blk.q[w] & 0x00FF00FFu, hi = __builtin_amdgcn_perm(blk.q[w], blk.q[w], 0x0C030C01u);
                        const u2_t pk = {lo, hi};
                        aw[w] = __builtin_bit_cast(h4_t, pk);
                    }
                } else {
#pragma unroll
                    for (int w = 0; w < 4; ++w) {
                        const uint32_t q = blk.q[w], q8 = q >> 8;
                        const u2_t lo = {q & 0x000F000Fu, q8 & 0x000F000Fu};
                        const u2_t hi = {q & 0x00F000F0u, q8 & 0x00F000F0u};
                        aw[2 * w] = __builtin_bit_cast(h4_t, lo);
                        aw[2 * w + 1] = __builtin_bit_cast(h4_t, hi);
                    }
                }
                // the four headers of this block's rows
                float sc[4], bi[4];
                const uint32_t hq[4] = {(uint32_t)QQ_DPP(blk.hdr, 0x00), (uint32_t)QQ_DPP(blk.hdr, 0x55),
                                        (uint32_t)QQ_DPP(blk.hdr, 0xAA), (uint32_t)QQ_DPP(blk.hdr, 0xFF)};   // quad_perm [i,i,i,i]
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const h2_t hd = __builtin_bit_cast(h2_t, hq[i]);
                    sc[i] = (float)hd[0];
                    bi[i] = (float)hd[1];
                    if constexpr (FMT == QW_FMT_B8) sc[i] *= 16777216.0f;   // the codes are f16 subnormals code * 2^-24: exact, once per header
                }
#pragma unroll
                for (int mg = 0; mg < MG; ++mg) {
                    f4_t a0 = {0.f, 0.f, 0.f, 0.f}, a1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int t = 0; t < 8; t += 2) {
                        a0 = __builtin_amdgcn_mfma_f32_4x4x4f16(aw[t], xb[mg][t], a0, 0, 0, 0);
                        a1 = __builtin_amdgcn_mfma_f32_4x4x4f16(aw[t + 1], xb[mg][t + 1], a1, 0, 0, 0);
                    }
                    f4_t v;
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        float q;
                        if constexpr (FMT == QW_FMT_B8) {
                            q = a0[i] + a1[i];
                        } else {
                            q = __builtin_fmaf(a0[i], 16777216.0f, FMT == QW_FMT_M5 ? 1024.0f * S[mg] : 0.0f);
                            q = __builtin_fmaf(a1[i], 1048576.0f, q);
                        }
                        float r = __builtin_fmaf(sc[i], q, bi[i] * S[mg]);
                        r += QQ_DPP_F32(r, 0x114);   // row_shr:4
                        r += QQ_DPP_F32(r, 0x118);   // row_shr:8: lanes 12..15 of each 16-lane row hold its four blocks
                        v[i] = r;
                    }
                    if ((l64 & 12u) == 12u && qslot < nq) {
                        f4_t* dst = qq_part + ((size_t)(qslot * W16 + wv * 4u + (l64 >> 4)) * (4u * MG) + 4u * mg + j);
                        if (kr == 0) *dst = v;
                        else *dst += v;
                    }
                }
                qslot += sets;
            }
        }
        // the next range's first quads are already in flight, in the slots after the last one consumed: turn the
        // window so that they sit in slots 0, 1, ... again
        if (kr + 1u < p.nkr) {
            for (uint32_t k = nmax % D; k > 0u; --k) {
                const qq_slice<FMT> first = buf[0];
#pragma unroll
                for (int d = 0; d + 1 < D; ++d) buf[d] = buf[d + 1];
                buf[D - 1] = first;
            }
        }
    }
    __syncthreads();
    // fixed-order sum of the partials of each (quad slot, activation row, bank row)
    for (uint32_t t = tid; t < nq * p.M * 4u; t += blockDim.x) {
        const uint32_t i = t & 3u, sm = t >> 2;
        const uint32_t s = sm / p.M, m = sm - s * p.M;
        const uint32_t row = 4u * (s * G + blockIdx.x) + i;
        if (row >= N) continue;
        float v = 0.f;
        for (uint32_t w = 0; w < W16; ++w) v += qq_part[(size_t)(s * W16 + w) * (4u * MG) + m][i];
        const uint64_t at = (uint64_t)m * N + row;
        if (p.y32) p.y32[at] = v;
        if (p.y16) p.y16[at] = (h1_t)v;
    }
}
};

template <int FMT, int XDT, int MG>
void qq_launch1(hipStream_t st, const qq_params& p, uint32_t wgs, uint32_t threads, size_t lds) {
    constexpr int D = FMT == QW_FMT_B8 ? 2 : 3;
    using kern = qw_gemv_quad_kernel<FMT, XDT, MG, D, 768>;
    static std::atomic<bool> attr_done{false};   // per instantiation
    if (!attr_done.load(std::memory_order_acquire)) {
        (void)hipFuncSetAttribute(qw_scalar_kernel_ptr<kern>((const qq_params*)nullptr), hipFuncAttributeMaxDynamicSharedMemorySize, 96 * 1024);
        attr_done.store(true, std::memory_order_release);
    }
    qw_launch_scalar<kern>(dim3(wgs), dim3(threads), lds, st, p);
}

template <int FMT, int XDT>
void qq_launch_m(hipStream_t st, const qq_params& p, uint32_t mg, uint32_t wgs, uint32_t threads, size_t lds) {
    if (mg == 1) qq_launch1<FMT, XDT, 1>(st, p, wgs, threads, lds);
    else if (mg == 2) qq_launch1<FMT, XDT, 2>(st, p, wgs, threads, lds);
    else if (mg == 3) qq_launch1<FMT, XDT, 3>(st, p, wgs, threads, lds);
    else qq_launch1<FMT, XDT, 4>(st, p, wgs, threads, lds);
}

}  // namespace

// Tries the 4x4x4-block kernel for a validated call whose activations are already in the container's basis; false when
// the shape is outside its envelope.  fmt: QW_FMT_M5 / QW_FMT_B4 / QW_FMT_B8.
// `tune`: 0 = automatic; bits 0..1 scale the grid (1 -> half, 2 -> double).
bool qw_quad_gemv(hipStream_t st, const qwhip_weight_view* w, int fmt, uint32_t gshift, uint32_t bb, uint64_t row_bytes,
                  const void* x, uint32_t x_dtype, uint32_t m, void* y16, float* y32, uint32_t tune, hipError_t* err) {
    if (m == 0 || m > 16) return false;
    if ((uint64_t)w->n * row_bytes >= (1ull << 32)) return false;   // 32-bit offsets inside the bank
    if (((uintptr_t)x & 15u) != 0) return false;
    const uint32_t mg = (m + 3u) / 4u;
    const uint32_t nsl = w->k / 32u, nch = (nsl + 15u) / 16u;
    // at most 12 waves per row set (768 threads); longer rows take several K ranges
    const uint32_t nkr = (nch + 11u) / 12u;
    const uint32_t wpr = (nch + nkr - 1u) / nkr;
    const uint32_t sets = max(1u, 12u / wpr);
    const uint32_t threads = 64u * wpr * sets;
    const uint32_t nquads = (w->n + 3u) / 4u;
    uint32_t wgs = 256u * max(1u, 12u / (wpr * sets));
    if ((tune & 3u) == 1u) wgs /= 2u;
    if ((tune & 3u) == 2u) wgs *= 2u;
    wgs = max(1u, min(wgs, nquads / sets));
    size_t lds = 0;
    for (;;) {
        lds = (size_t)qwhip_cdiv(nquads, wgs) * (wpr * 4u) * (4u * mg) * 16u;
        if (lds <= 96u * 1024u || wgs >= nquads) break;   // more workgroups re-read the activations: one per CU while it fits
        wgs = min(wgs * 2u, nquads);
    }
    if (lds > 96u * 1024u) return false;
    qq_params p;
    p.bank = (const uint8_t*)w->blocks;
    p.x = x;
    p.y16 = (h1_t*)y16;
    p.y32 = y32;
    p.N = w->n;
    p.K = w->k;
    p.M = m;
    p.nsl = nsl;
    p.wpr = wpr;
    p.sets = sets;
    p.nkr = nkr;
    p.gshift = gshift;
    p.bb = bb;
    p.row_bytes = (uint32_t)row_bytes;
    if (x_dtype == QWHIP_F16) {
        if (fmt == QW_FMT_M5) qq_launch_m<QW_FMT_M5, QWHIP_F16>(st, p, mg, wgs, threads, lds);
        else if (fmt == QW_FMT_B4) qq_launch_m<QW_FMT_B4, QWHIP_F16>(st, p, mg, wgs, threads, lds);
        else qq_launch_m<QW_FMT_B8, QWHIP_F16>(st, p, mg, wgs, threads, lds);
    } else {
        if (fmt == QW_FMT_M5) qq_launch_m<QW_FMT_M5, QWHIP_BF16>(st, p, mg, wgs, threads, lds);
        else if (fmt == QW_FMT_B4) qq_launch_m<QW_FMT_B4, QWHIP_BF16>(st, p, mg, wgs, threads, lds);
        else qq_launch_m<QW_FMT_B8, QWHIP_BF16>(st, p, mg, wgs, threads, lds);
    }
    *err = hipGetLastError();
    return true;
}
