// GEMV over any container with fp32 activations and fp32 outputs, with the scalar epilogues of the reference's f32 family
// (qwg_gemv_*_f32_v4 / qwg_gemm_*_f32_bm, Sources/QWMetal/include/qw_gemm_f32_common.metalh:15-19,152-225;
// doors QWGemm.encodeHQ4F32V4 / encodeHQ4F32BM, Sources/Operators/QWGEMM/QWGemmF32.swift:178-199,311-350).
//
// Launch shape: the column-stationary persistent form of gemv_colx.hip - a fixed population of workgroups walks the bank
// once (row slot s of workgroup w is bank row s * gridDim.x + w); a 32-lane half-wavefront (set, chunk) owns slice
// columns 32 * chunk .. + 31 (a slice = 32 columns) of the rows set, set + sets, ...; a lane keeps its 32 fp32
// activations of each of the MR activation rows in registers.
//
// Arithmetic: all in fp32.  The reference dequantises one weight as fma(float(code [+ 1024]), scale, bias) in fp32 and
// feeds an fp32 FMA chain (qwg_unpack_hq4_word8_f32 / qwg_dot_hq4_block_f32_reg, qw_dequant_f32.metalh:10-58); here the
// affine part is applied once per slice, sum_i w_i x_i = scale * sum_i code_i x_i + bias * sum_i x_i (HQ4_G32_M5: bias stands
// for fma(1024, scale, bias), rounded once), codes converted to fp32 exactly.  Both differ from the exact sum only by
// fp32 rounding.
#include "qwhip_common.h"

namespace {

#define QF_FIELDS(X)                                                                                                        \
    X(const uint8_t*, bank) X(const float*, x) X(float*, y) X(uint32_t, N) X(uint32_t, K) X(uint32_t, M) X(uint32_t, nsl)       \
    X(uint32_t, cpr) X(uint32_t, sets) X(uint32_t, gshift) X(uint32_t, bb) X(uint32_t, row_bytes) X(uint32_t, epi) X(float, scale)
QW_ARG_BLOCK(qf_params, QF_FIELDS)

template <int FMT>
struct qf_fmt {
    static constexpr int BITS = FMT == QW_FMT_B8 ? 8 : (FMT == QW_FMT_B2 ? 2 : (FMT == QW_FMT_B3 ? 3 : (FMT == QW_FMT_B6 ? 6 : 4)));
    static constexpr int PW = BITS;   // payload dwords of one 32-column slice
};

// Code of element e (0..31) of a slice, cut out at compile-time positions.  HQ4_G32_M5 keeps element 8w + j at bit
// 4 (j >> 1) + 16 (j & 1) of word w (unpack_hq4_word8, qw_dequant.metalh:42-62); the bit streams element e at bit e * bits.
template <int FMT>
__device__ __forceinline__ uint32_t qf_code(const uint32_t* q, int e) {
    constexpr int BITS = qf_fmt<FMT>::BITS;
    if constexpr (FMT == QW_FMT_M5) {
        const int w = e >> 3, j = e & 7;
        return (q[w] >> (4 * (j >> 1) + 16 * (j & 1))) & 15u;
    } else {
        const int off = e * BITS, wd = off >> 5, sh = off & 31;
        uint32_t c = q[wd] >> sh;
        if (sh + BITS > 32) c |= q[wd + 1] << (32 - sh);
        return c & ((1u << BITS) - 1u);
    }
}

// Byte B of a word as a float, one instruction.
template <int B>
__device__ __forceinline__ float qf_ubyte(uint32_t v) {
    float r;
    if constexpr (B == 0) asm("v_cvt_f32_ubyte0 %0, %1" : "=v"(r) : "v"(v));
    else if constexpr (B == 1) asm("v_cvt_f32_ubyte1 %0, %1" : "=v"(r) : "v"(v));
    else if constexpr (B == 2) asm("v_cvt_f32_ubyte2 %0, %1" : "=v"(r) : "v"(v));
    else asm("v_cvt_f32_ubyte3 %0, %1" : "=v"(r) : "v"(v));
    return r;
}

__device__ __forceinline__ float qf_epilogue(float v, uint32_t epi, float scale) {
    if (epi == 1u || epi == 3u) {
        const float z = v / scale;
        return z / (1.0f + expf(-z));
    }
    if (epi == 2u) return 1.0f / (1.0f + expf(-v));
    return v;
}

// MR activation rows, three (MR = 4: four) slices in flight per lane.  blockDim.x = 32 * cpr * sets;
// dynamic LDS = rows-per-workgroup * cpr * MR * 4 bytes.
template <int FMT, int MR, int LB>
struct qw_gemv_f32_kernel {
static constexpr int kLaunchBound = LB;
static __device__ __forceinline__ void run(const qf_params& p) {
    constexpr int D = MR == 4 ? 4 : 3, PW = qf_fmt<FMT>::PW;
    extern __shared__ float qf_part[];   // [row slot][chunk][MR]
    const uint32_t cpr = p.cpr, N = p.N, sets = p.sets;
    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & 31u, hw = tid >> 5;
    const uint32_t set = hw / cpr, chunk = hw - set * cpr;
    const uint32_t g0 = chunk * 32u + lane;
    const bool gvalid = g0 < p.nsl;
    const uint32_t g = gvalid ? g0 : p.nsl - 1u;
    const uint32_t G = gridDim.x;
    if (blockIdx.x >= N) return;
    const uint32_t nrows = (N - blockIdx.x + G - 1u) / G;   // row slots of this workgroup
    const uint32_t nmax = (nrows + sets - 1u) / sets;       // trip count, uniform over the workgroup
    const uint32_t step = G * sets * p.row_bytes;
    const uint32_t mine = nrows > set ? (nrows - set + sets - 1u) / sets : 0u;
    uint32_t hdr_off, pay_off;
    if constexpr (FMT == QW_FMT_M5) {
        hdr_off = g * 20u;
        pay_off = hdr_off + 4u;
    } else {
        hdr_off = (g >> p.gshift) * p.bb;
        pay_off = hdr_off + 4u + (g & ((1u << p.gshift) - 1u)) * (4u * PW);
    }
    uint32_t off = ((mine ? set : 0u) * G + blockIdx.x) * p.row_bytes;
    const uint32_t off_max = off + (mine ? mine - 1u : 0u) * step;   // loads past the set's last row re-read it

    // activations first; rows past M re-read row M - 1
    f4_t xv[MR][8];
#pragma unroll
    for (int m = 0; m < MR; ++m) {
        const float* xp = p.x + (uint64_t)min((uint32_t)m, p.M - 1u) * p.K + (uint64_t)g * 32u;
#pragma unroll
        for (int j = 0; j < 8; ++j) xv[m][j] = *(const f4_t*)(xp + 4 * j);
    }
    __builtin_amdgcn_sched_barrier(0);
    uint32_t hdr[D], q[D][PW];
    auto issue = [&](int slot) {
        const uint8_t* rp = p.bank + off;
        hdr[slot] = *(const uint32_t*)(rp + hdr_off);
#pragma unroll
        for (int j = 0; j < PW; ++j) q[slot][j] = *(const uint32_t*)(rp + pay_off + 4 * j);
        off = min(off + step, off_max);
    };
#pragma unroll
    for (int j = 0; j < D; ++j) issue(j);
    __builtin_amdgcn_sched_barrier(0);
    float S[MR];
#pragma unroll
    for (int m = 0; m < MR; ++m) {
        f4_t t = (xv[m][0] + xv[m][1]) + (xv[m][2] + xv[m][3]);
        t += (xv[m][4] + xv[m][5]) + (xv[m][6] + xv[m][7]);
        S[m] = (t[0] + t[1]) + (t[2] + t[3]);
    }

    uint32_t rslot = set;
    for (uint32_t ib = 0; ib < nmax; ib += D) {
#pragma unroll
        for (int j = 0; j < D; ++j) {
            if (ib + j >= nmax) break;
            uint32_t qq[PW];
#pragma unroll
            for (int t = 0; t < PW; ++t) qq[t] = q[j][t];
            const h2_t hd = __builtin_bit_cast(h2_t, hdr[j]);
            issue(j);
            const float sc = (float)hd[0];
            // HQ4_G32_M5: weight = (1024 + code) * scale + bias = code * scale + (1024 * scale + bias); the bracket is formed with
            // one rounding, so the large terms cancel before they meet the activations
            const float bi = FMT == QW_FMT_M5 ? __builtin_fmaf(1024.0f, sc, (float)hd[1]) : (float)hd[1];
            float acc[MR][4];
#pragma unroll
            for (int m = 0; m < MR; ++m) acc[m][0] = acc[m][1] = acc[m][2] = acc[m][3] = 0.f;
            auto contract = [&](float c, int e) {
#pragma unroll
                for (int m = 0; m < MR; ++m) acc[m][e & 3] = __builtin_fmaf(c, xv[m][e >> 2][e & 3], acc[m][e & 3]);
            };
            if constexpr (FMT == QW_FMT_M5 || FMT == QW_FMT_B4 || FMT == QW_FMT_B8) {
                // byte-aligned codes: one mask per four codes, then the byte-to-float conversions
#pragma unroll
                for (int w = 0; w < PW; ++w) {
                    if constexpr (FMT == QW_FMT_B8) {
                        contract(qf_ubyte<0>(qq[w]), 4 * w + 0);
                        contract(qf_ubyte<1>(qq[w]), 4 * w + 1);
                        contract(qf_ubyte<2>(qq[w]), 4 * w + 2);
                        contract(qf_ubyte<3>(qq[w]), 4 * w + 3);
                    } else {
                        // HQ4_G32_M5: the nibble at bit 4 t + 16 u is element 2 t + u of the word; streams: nibble i is element i
                        constexpr bool M5 = FMT == QW_FMT_M5;
                        const uint32_t lo = qq[w] & 0x0F0F0F0Fu, hi = (qq[w] >> 4) & 0x0F0F0F0Fu;
                        contract(qf_ubyte<0>(lo), 8 * w + 0);
                        contract(qf_ubyte<1>(lo), 8 * w + (M5 ? 4 : 2));
                        contract(qf_ubyte<2>(lo), 8 * w + (M5 ? 1 : 4));
                        contract(qf_ubyte<3>(lo), 8 * w + (M5 ? 5 : 6));
                        contract(qf_ubyte<0>(hi), 8 * w + (M5 ? 2 : 1));
                        contract(qf_ubyte<1>(hi), 8 * w + (M5 ? 6 : 3));
                        contract(qf_ubyte<2>(hi), 8 * w + (M5 ? 3 : 5));
                        contract(qf_ubyte<3>(hi), 8 * w + (M5 ? 7 : 7));
                    }
                }
            } else {
#pragma unroll
                for (int e = 0; e < 32; ++e) contract((float)qf_code<FMT>(qq, e), e);
            }
#pragma unroll
            for (int m = 0; m < MR; ++m) {
                const float qs = (acc[m][0] + acc[m][1]) + (acc[m][2] + acc[m][3]);
                float v = __builtin_fmaf(sc, qs, bi * S[m]);
                v = gvalid ? v : 0.0f;
                v = qw_reduce32_dpp(v);
                if (lane == 31u && rslot < nrows) qf_part[(rslot * cpr + chunk) * MR + m] = v;
            }
            rslot += sets;
        }
    }
    __syncthreads();
    // fixed-order sum of the chunk partials of each (row, activation row), then the scalar epilogue
    for (uint32_t t = tid; t < nrows * p.M; t += blockDim.x) {
        const uint32_t m = t / nrows, s = t - m * nrows;
        float v = 0.f;
        for (uint32_t c = 0; c < cpr; ++c) v += qf_part[(s * cpr + c) * MR + m];
        p.y[(uint64_t)m * N + s * G + blockIdx.x] = qf_epilogue(v, p.epi, p.scale);
    }
}
};

// In-place capable FWHT-32 over consecutive groups of 32 outputs of each row, butterfly order and scaling of
// qwg_fwht32_lane_f32 (Sources/QWMetal/include/qw_weight_basis.metalh:31-38); a last partial group is padded with zeros
// (the v4 kernel's epilogue 3 reads rows past N as 0, qw_gemm_f32_common.metalh:171-196).
__global__ __launch_bounds__(256) void qw_h32_f32_kernel(const float* x, float* out, uint32_t hidden, uint32_t padded) {
    const uint32_t col = blockIdx.x * 256u + threadIdx.x;
    if (col >= padded) return;   // padded is a multiple of 32: whole 32-lane groups leave together
    const uint64_t at = (uint64_t)blockIdx.y * hidden + col;
    float v = col < hidden ? x[at] : 0.0f;
    v = qw_fwht32_lanes(v, qw_fwht32_lane_signs(threadIdx.x & 31u));   // the same stages and sums, partners by DPP
    if (col < hidden) out[at] = v * 0.17677669529663689f;
}

template <int FMT>
void qf_launch(hipStream_t st, const qf_params& p, uint32_t mr, uint32_t wgs, uint32_t threads, size_t lds) {
    if (mr == 1) qw_launch_scalar<qw_gemv_f32_kernel<FMT, 1, 1024>>(dim3(wgs), dim3(threads), lds, st, p);
    else if (mr == 2) qw_launch_scalar<qw_gemv_f32_kernel<FMT, 2, 768>>(dim3(wgs), dim3(threads), lds, st, p);
    else qw_launch_scalar<qw_gemv_f32_kernel<FMT, 4, 512>>(dim3(wgs), dim3(threads), lds, st, p);
}

}  // namespace

void qw_h32_f32_launch(hipStream_t st, const float* x, float* out, uint32_t rows, uint32_t hidden) {
    const uint32_t padded = (hidden + 31u) & ~31u;
    hipLaunchKernelGGL(qw_h32_f32_kernel, dim3((padded + 255u) / 256u, rows), dim3(256), 0, st, x, out, hidden, padded);
}

// Largest number of activation rows (4, 2, 1 or 0 = none) the kernel takes per launch on this bank.
uint32_t qw_f32_gemv_rows(const qwhip_weight_view* w, uint64_t row_bytes) {
    if ((uint64_t)w->n * row_bytes >= (1ull << 30)) return 0;   // 32-bit offsets inside the bank, one row step past its end included
    const uint32_t cpr = (w->k / 32u + 31u) / 32u;
    if (32u * cpr <= 512u) return 4;
    if (32u * cpr <= 768u) return 2;
    return 32u * cpr <= 1024u ? 1u : 0u;
}

// One launch over m <= qw_f32_gemv_rows() activation rows already in the container's basis; epilogue 3's rotation is the
// caller's second launch.
void qw_f32_gemv(hipStream_t st, const qwhip_weight_view* w, int fmt, uint32_t gshift, uint32_t bb, uint64_t row_bytes,
                 const float* x, uint32_t m, uint32_t epi, float scale, float* y) {
    const uint32_t mr = m <= 1 ? 1u : (m <= 2 ? 2u : 4u);
    const uint32_t nsl = w->k / 32u, cpr = (nsl + 31u) / 32u;
    const uint32_t lb = mr == 1 ? 1024u : (mr == 2 ? 768u : 512u);
    const uint32_t waves_cu = lb / 64u;
    const uint32_t sets = min(lb / (32u * cpr), 8u);
    const uint32_t threads = 32u * cpr * sets;
    const uint32_t waves = (threads + 63u) / 64u;
    uint32_t wgs = min(256u * max(1u, waves_cu / waves), max(1u, w->n / sets));
    // the partial sums of a workgroup's rows stay in LDS: more, smaller workgroups when the bank has very many rows
    while ((size_t)qwhip_cdiv(w->n, wgs) * cpr * mr * 4u > 60u * 1024u) wgs *= 2u;
    const size_t lds = (size_t)qwhip_cdiv(w->n, wgs) * cpr * mr * 4u;
    qf_params p;
    p.bank = (const uint8_t*)w->blocks;
    p.x = x;
    p.y = y;
    p.N = w->n;
    p.K = w->k;
    p.M = m;
    p.nsl = nsl;
    p.cpr = cpr;
    p.sets = sets;
    p.gshift = gshift;
    p.bb = bb;
    p.row_bytes = (uint32_t)row_bytes;
    p.epi = epi;
    p.scale = scale;
    if (fmt == QW_FMT_M5) qf_launch<QW_FMT_M5>(st, p, mr, wgs, threads, lds);
    else if (fmt == QW_FMT_B4) qf_launch<QW_FMT_B4>(st, p, mr, wgs, threads, lds);
    else if (fmt == QW_FMT_B8) qf_launch<QW_FMT_B8>(st, p, mr, wgs, threads, lds);
    else if (fmt == QW_FMT_B2) qf_launch<QW_FMT_B2>(st, p, mr, wgs, threads, lds);
    else if (fmt == QW_FMT_B3) qf_launch<QW_FMT_B3>(st, p, mr, wgs, threads, lds);
    else qf_launch<QW_FMT_B6>(st, p, mr, wgs, threads, lds);
}
