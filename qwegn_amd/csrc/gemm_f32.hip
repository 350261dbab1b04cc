// Batched GEMM over any container with fp32 activations and fp32 outputs, on the f16 matrix cores: the form the
// reference gives 32 activation rows and more (qwg_gemm_*_f32_bm / _bm32, body qwg_gemm_f32_bm_body,
// Sources/QWMetal/include/qw_gemm_f32_common.metalh:59-142; door QWGemm.encodeHQ4F32BM,
// Sources/Operators/QWGEMM/QWGemmF32.swift:311-350).  Every 64 activation rows read the bank once.
//
// Arithmetic.  The reference multiplies fp32 activations with fp32 weights fma(float(code [+ 1024]), scale, bias)
// (qw_dequant_f32.metalh:10-24) on fp32 simdgroup matrices.  Here both operands are split into two f16 numbers,
//   v = hi + lo / 2048,  hi = RN_f16(v),  lo = RN_f16((v - hi) * 2048)     (|v - hi - lo / 2048| <= 2^-22 |v|),
// and three f16 matrix products are accumulated in fp32: x_hi w_hi into one accumulator, x_hi w_lo + x_lo w_hi into a
// second one that joins the first scaled by 1 / 2048 at the store; the dropped product x_lo w_lo is below 2^-22 of the
// largest term.  The scaling by 2048 keeps the low parts out of the f16 subnormal range.
// Any fp32 activation row is taken: a first launch finds the largest magnitude of every row and leaves the power of two
// that brings it into [2^13, 2^14) (the top of the f16 range, so that elements 2^27 times smaller than the largest still
// split into normal f16 numbers); the rows are multiplied by it on their way into the split - exactly - and the sums by
// its reciprocal at the store.  Without it a row with |x| > 65504 became inf - inf = NaN and rows below 2^-14 lost their
// low parts; the reference's batched f32 kernels (qwg_gemm_*_f32_bm) take any fp32.
//
// Launch: a workgroup of four waves owns 64 activation rows x 64 weight rows and walks K in steps of 64: activations
// global f32 -> registers -> two f16 LDS tiles, packed slices global -> registers -> two f16 LDS tiles (half a slice per
// thread), v_mfma_f32_32x32x16_f16 over the four tiles; the next step's loads are issued before the products.
#include <type_traits>

#include "qwhip_common.h"

namespace {

struct qgf_params {
    const uint8_t* bank;
    const float* x;
    float* y;
    uint32_t M, N, K, gshift, bb, epi;
    uint64_t row_bytes;
    float scale;
    const float* row_down;   // [M] powers of two: row r is contracted as x[r] * row_down[r]
};

// row_down[r] = 2^-e with 2^e <= max |x[r]| * 2^-13 < 2^(e + 1); 1 for a row of zeros.  e is kept inside the exponents
// whose powers of two and their reciprocals are normal floats (a row whose largest magnitude is below 2^-113 is scaled
// by 2^126 only); a row that holds inf or NaN gets a finite factor and stays non-finite.
__global__ __launch_bounds__(256) void qw_row_scale_kernel(const float* __restrict__ x, uint32_t M, uint32_t K, float* __restrict__ row_down) {
    const uint32_t row = blockIdx.x * 4u + (threadIdx.x >> 6), lane = threadIdx.x & 63u;
    if (row >= M) return;
    const uint32_t* xr = (const uint32_t*)(x + (uint64_t)row * K);
    uint32_t mx = 0u;
    for (uint32_t c = lane * 4u; c + 3u < K; c += 256u) {
        const u4_t v = *(const u4_t*)(xr + c);
        mx = max(max(mx, v[0] & 0x7FFFFFFFu), max(max(v[1] & 0x7FFFFFFFu, v[2] & 0x7FFFFFFFu), v[3] & 0x7FFFFFFFu));
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) mx = max(mx, (uint32_t)__shfl_xor((int)mx, o, 64));
    if (lane == 0u) {
        int e = (int)(mx >> 23) - 127 - 13;
        e = mx == 0u ? 0 : min(max(e, -126), 126);
        row_down[row] = __uint_as_float((uint32_t)(127 - e) << 23);
    }
}


template <int FMT>
struct qgf_fmt {
    static constexpr int BITS = FMT == QW_FMT_B8 ? 8 : (FMT == QW_FMT_B2 ? 2 : (FMT == QW_FMT_B3 ? 3 : (FMT == QW_FMT_B6 ? 6 : 4)));
    static constexpr int PW = BITS;   // payload dwords of one 32-column slice
};

// Code of element e (0..31) of a slice, cut out at compile-time positions.  HQ4_G32_M5 keeps element 8w + j at bit
// 4 (j >> 1) + 16 (j & 1) of word w (unpack_hq4_word8, Sources/QWMetal/include/qw_dequant.metalh:42-62); the bit streams
// element e at bit e * bits.
template <int FMT>
__device__ __forceinline__ uint32_t qgf_code(const uint32_t* q, int e) {
    constexpr int BITS = qgf_fmt<FMT>::BITS;
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

__device__ __forceinline__ float qgf_epilogue(float v, uint32_t epi, float scale) {
    if (epi == 1u || epi == 3u) {
        const float z = v / scale;
        return z / (1.0f + expf(-z));
    }
    if (epi == 2u) return 1.0f / (1.0f + expf(-v));
    return v;
}

__device__ __forceinline__ void qgf_split(float v, h1_t& hi, h1_t& lo) {
    hi = (h1_t)v;
    lo = (h1_t)((v - (float)hi) * 2048.0f);
}

template <int FMT>
__global__ __launch_bounds__(256) void qw_gemm_f32x_kernel(const qgf_params p) {
    constexpr int PW = qgf_fmt<FMT>::PW;
    constexpr uint32_t BM = 64, BN = 64, PITCH = 72;            // halves: 144 bytes per tile row
    constexpr uint32_t TILE = BM * PITCH;                         // halves per LDS tile
    __shared__ __attribute__((aligned(16))) h1_t lds[4 * TILE];   // x hi | x lo | w hi | w lo
    h1_t *xa = lds, *xl = lds + TILE, *wa = lds + 2 * TILE, *wl = lds + 3 * TILE;
    const uint32_t tid = threadIdx.x, lane = tid & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t wm = wave >> 1, wn = wave & 1u;
    const uint32_t m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;

    // activation role: four 16-byte pieces per thread (row = c >> 4, piece = c & 15 of the row's 64 columns)
    const float* a_src[4];
    bool a_ok[4];
    float a_down[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const uint32_t c = tid + 256u * i, row = c >> 4;
        a_ok[i] = m0 + row < p.M;
        a_src[i] = p.x + (uint64_t)(a_ok[i] ? m0 + row : 0u) * p.K + (c & 15u) * 4u;
        a_down[i] = p.row_down[a_ok[i] ? m0 + row : 0u];
    }
    // weight role: half `half` (16 columns) of slice `sl` of tile row `wr`
    const uint32_t item = tid & 127u, wr = item >> 1, sl = item & 1u;
    const uint32_t half = wave >> 1;   // uniform over a wave
    const uint8_t* wrow = p.bank + (uint64_t)min(n0 + wr, p.N - 1u) * p.row_bytes;

    f4_t a_reg[4];
    uint32_t hdr, q[PW];
    auto issue = [&](uint32_t kt) {
#pragma unroll
        for (int i = 0; i < 4; ++i) a_reg[i] = a_ok[i] ? *(const f4_t*)(a_src[i] + (uint64_t)kt * 64u) : f4_t{0.f, 0.f, 0.f, 0.f};
        const uint32_t s = kt * 2u + sl;
        const uint8_t* hp;
        const uint8_t* wp;
        if constexpr (FMT == QW_FMT_M5) {
            hp = wrow + s * 20u;
            wp = hp + 4;
        } else {
            hp = wrow + (uint64_t)(s >> p.gshift) * p.bb;
            wp = hp + 4 + (s & ((1u << p.gshift) - 1u)) * (4u * PW);
        }
        hdr = *(const uint32_t*)hp;
#pragma unroll
        for (int j = 0; j < PW; ++j) q[j] = *(const uint32_t*)(wp + 4 * j);
    };
    // 16 weights of the slice from element E0 on, split and parked
    auto park_weights = [&](auto e0_c) {
        constexpr int E0 = decltype(e0_c)::value;
        const h2_t hd = __builtin_bit_cast(h2_t, hdr);
        const float sc = (float)hd[0];
        const float bi = FMT == QW_FMT_M5 ? __builtin_fmaf(1024.0f, sc, (float)hd[1]) : (float)hd[1];
        h8_t hi[2], lo[2];
#pragma unroll
        for (int e = 0; e < 16; ++e) {
            const float w = __builtin_fmaf((float)qgf_code<FMT>(q, E0 + e), sc, bi);
            h1_t h, l;
            qgf_split(w, h, l);
            hi[e >> 3][e & 7] = h;
            lo[e >> 3][e & 7] = l;
        }
        h1_t* dh = wa + wr * PITCH + sl * 32u + E0;
        h1_t* dl = wl + wr * PITCH + sl * 32u + E0;
        *(h8_t*)dh = hi[0];
        *(h8_t*)(dh + 8) = hi[1];
        *(h8_t*)dl = lo[0];
        *(h8_t*)(dl + 8) = lo[1];
    };

    f16_t acc = {}, acc_lo = {};
    const uint32_t nk = p.K / 64u;
    const uint32_t frow = lane & 31u, k_half = lane >> 5;
    issue(0);
    for (uint32_t kt = 0; kt < nk; ++kt) {
        __syncthreads();
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const uint32_t c = tid + 256u * i;
            h4_t hi, lo;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                h1_t h, l;
                qgf_split(a_reg[i][e] * a_down[i], h, l);
                hi[e] = h;
                lo[e] = l;
            }
            *(h4_t*)(xa + (c >> 4) * PITCH + (c & 15u) * 4u) = hi;
            *(h4_t*)(xl + (c >> 4) * PITCH + (c & 15u) * 4u) = lo;
        }
        if (half == 0u) park_weights(std::integral_constant<int, 0>{});
        else park_weights(std::integral_constant<int, 16>{});
        __syncthreads();
        if (kt + 1u < nk) issue(kt + 1u);
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) {
            const uint32_t ao = (wm * 32u + frow) * PITCH + ks * 16u + k_half * 8u;
            const uint32_t bo = (wn * 32u + frow) * PITCH + ks * 16u + k_half * 8u;
            const h8_t ah = *(const h8_t*)(xa + ao), al = *(const h8_t*)(xl + ao);
            const h8_t bh = *(const h8_t*)(wa + bo), bl = *(const h8_t*)(wl + bo);
            acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(ah, bh, acc, 0, 0, 0);
            acc_lo = __builtin_amdgcn_mfma_f32_32x32x16_f16(ah, bl, acc_lo, 0, 0, 0);
            acc_lo = __builtin_amdgcn_mfma_f32_32x32x16_f16(al, bh, acc_lo, 0, 0, 0);
        }
    }
    // lane holds weight row (output column) n = lane & 31, activation rows 8 (r / 4) + 4 (lane >> 5) + (r & 3)
    const uint32_t n = n0 + wn * 32u + frow;
    if (n < p.N) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const uint32_t row = m0 + wm * 32u + 8u * (r >> 2) + 4u * k_half + (r & 3);
            if (row < p.M) {
                const float up = 1.0f / p.row_down[row];     // a power of two: exact
                p.y[(uint64_t)row * p.N + n] = qgf_epilogue(__builtin_fmaf(acc_lo[r], 1.0f / 2048.0f, acc[r]) * up, p.epi, p.scale);
            }
        }
    }
}

}  // namespace

// Runs the batched form for a validated call; false when the shape is outside it (K not a multiple of 64).
// `row_down`: device scratch for m floats (the rows' scaling factors, written by the first of the two launches).
// Epilogue 3's rotation over the outputs is the caller's second launch, as for the GEMV form.
bool qw_f32_gemm(hipStream_t st, const qwhip_weight_view* w, int fmt, uint32_t gshift, uint32_t bb, uint64_t row_bytes,
                 const float* x, uint32_t m, uint32_t epi, float scale, float* y, float* row_down) {
    if (w->k % 64u != 0 || ((uintptr_t)x & 15u) != 0 || !row_down) return false;
    hipLaunchKernelGGL(qw_row_scale_kernel, dim3(qwhip_cdiv(m, 4u)), dim3(256), 0, st, x, m, w->k, row_down);
    qgf_params p;
    p.row_down = row_down;
    p.bank = (const uint8_t*)w->blocks;
    p.x = x;
    p.y = y;
    p.M = m;
    p.N = w->n;
    p.K = w->k;
    p.gshift = gshift;
    p.bb = bb;
    p.epi = epi;
    p.row_bytes = row_bytes;
    p.scale = scale;
    const dim3 grid(qwhip_cdiv(w->n, 64u), qwhip_cdiv(m, 64u));
    switch (fmt) {
#define QGF_GO(F) case F: hipLaunchKernelGGL(qw_gemm_f32x_kernel<F>, grid, dim3(256), 0, st, p); break;
        QGF_GO(QW_FMT_M5) QGF_GO(QW_FMT_B4) QGF_GO(QW_FMT_B8) QGF_GO(QW_FMT_B2) QGF_GO(QW_FMT_B3) QGF_GO(QW_FMT_B6)
#undef QGF_GO
        default: return false;
    }
    return true;
}
