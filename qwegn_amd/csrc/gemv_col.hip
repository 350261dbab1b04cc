// Decode GEMV (m = 1) over an HQ4_G32_M5 bank, column-stationary persistent form.
//
// The launch is a fixed population of workgroups that together walk the bank once, top to bottom: row slot s of
// workgroup w is bank row s * gridDim.x + w, so at any moment the whole grid is fetching one contiguous band of rows
// (what the HBM channels like) and every workgroup has the same number of rows to within one.
//
// Inside a workgroup a 32-lane half-wavefront (set, chunk) owns block columns 32*chunk .. 32*chunk + 31 of the rows
// set, set + SETS, ... of the workgroup.  A lane therefore multiplies the same 32 activations for the whole kernel and
// keeps them in registers (16 packed pairs); the main loop has no LDS reads, only a rolling window of D block loads
// per lane, the nibble unpack, 16 v_dot2_f32_f16 and a half-wave reduction per row.
//
// Arithmetic.  A block dequantizes as w = (1024 + q) * s + b (unpack_hq4_word8, Sources/QWMetal/include/
// qw_dequant.metalh:42-62).  The kernel never forms w: the masked nibble pairs are used directly as f16 operands -
// bits 0..3 / 16..19 of a word read as two f16 subnormals q * 2^-24, bits 4..7 / 20..23 as 16 q * 2^-24
// (v_dot2_f32_f16 honours f16 subnormals; products are exact, accumulation is fp32) - and the affine part is applied once
// per block:  sum_i w_i x_i = s * sum_i q_i x_i + (1024 s + b) * S,  S = sum_i x_i,
// the same factorisation the reference's bit-stream GEMVs use (qwg_aq_slice_dot, qw_dequant_multi.metalh:205-208).
// The activations are the f16-rounded rotated values the reference's producers would have stored.
#include <type_traits>

#include "qwhip_common.h"

namespace {

#define QC_FIELDS(X) X(const uint8_t*, bank) X(const void*, x) X(h1_t*, y16) X(float*, y32) X(uint32_t, N) X(uint32_t, nb) X(uint32_t, cpr) X(uint32_t, rotate)
QW_ARG_BLOCK(qc_params, QC_FIELDS)
// The head's form of the kernel takes one more argument: keys [gridDim.x], the workgroup's argmax key (monotone float bits
// << 32 | ~row) over its rows.  It is a second instantiation with its own argument block: the decode kernel's argument
// block and code stay as they are without it (with the extra member and epilogue in the one kernel the N = 17408, K = 5120
// launch took 11.6 us instead of 11.3 in a same-box comparison).
#define QC_FOLD_FIELDS(X) QC_FIELDS(X) X(unsigned long long*, keys)
QW_ARG_BLOCK(qc_params_fold, QC_FOLD_FIELDS)
// The gate|up form of the kernel (dense MLP decode without the output rotation): the bank holds I gate rows and then the I up
// rows of the same channels; row slots 2 c and 2 c + 1 of a workgroup are the gate and the up row of its channel c, so that
// the gated activation is formed in the epilogue and act f16 [I] is what gets stored (y16).  N = 2 I.
#define QC_PAIR_FIELDS(X) QC_FIELDS(X) X(qw_act, ga)
QW_ARG_BLOCK(qc_params_pair, QC_PAIR_FIELDS)
__device__ __forceinline__ const qc_params& qc_base(const qc_params& p) { return p; }
__device__ __forceinline__ qc_params qc_base(const qc_params_pair& f) {
    qc_params p;
#define QC_TAKE(T, n) p.n = f.n;
    QC_FIELDS(QC_TAKE)
#undef QC_TAKE
    return p;
}
__device__ __forceinline__ qc_params qc_base(const qc_params_fold& f) {
    qc_params p;
#define QC_TAKE(T, n) p.n = f.n;
    QC_FIELDS(QC_TAKE)
#undef QC_TAKE
    return p;
}

// A float's bits made monotone as an unsigned number; NaN -> 0, so it never wins (qw_sortable_f32_u32,
// Sources/QWMetal/include/qw_fastmath_safe.metalh:21-25).
__device__ __forceinline__ uint32_t qc_sortable_f32(float x) {
    const uint32_t u = __float_as_uint(x);
    if ((u & 0x7FFFFFFFu) > 0x7F800000u) return 0u;
    return (u & 0x80000000u) ? ~u : (u ^ 0x80000000u);
}

// SETS row sets per workgroup, D blocks in flight per lane, D0 of them issued before the activation prologue.
// blockDim.x = 32 * cpr * SETS; dynamic LDS = nb * 80 + rows-per-workgroup * cpr * 4 bytes.
template <int XDT, int SETS, int D, int D0, typename P = qc_params>
struct qw_gemv_col_kernel {
static constexpr int kLaunchBound = 1024;
static __device__ __forceinline__ void run(const P& pp) {
    constexpr bool FOLD = std::is_same<P, qc_params_fold>::value;
    constexpr bool PAIR = std::is_same<P, qc_params_pair>::value;
    static_assert(!PAIR || SETS % 2 == 0, "gate and up rows sit in row sets of opposite parity");
    const qc_params& p = qc_base(pp);
    // 16-group activation tiles per full wave: ceil(2 cpr / full waves).  One row set with an odd cpr ends in a half
    // wave, which takes no tile (its upper lanes do not exist): cpr = 13 leaves 6 full waves for 26 tiles.
    constexpr int XT = SETS == 1 ? 5 : (SETS == 2 ? 2 : 1);
    extern __shared__ h8_t qc_lds[];
    const uint32_t nb = p.nb, cpr = p.cpr, N = p.N;
    h8_t* xs = qc_lds;                                 // 80 bytes per 32-group (64 used)
    float* part = (float*)(qc_lds + (size_t)nb * 5);   // [row slot][chunk] partial sums
    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & 31u, hw = tid >> 5;
    const uint32_t wave = tid >> 6, l64 = tid & 63u;
    const uint32_t nw = blockDim.x >> 6;               // full waves
    const bool tiler = wave < nw;
    const uint32_t set = hw / cpr, chunk = hw - set * cpr;
    const uint32_t g0 = chunk * 32u + lane;
    const bool gvalid = g0 < nb;
    const uint32_t g = gvalid ? g0 : nb - 1u;
    const uint32_t G = gridDim.x;
    const uint32_t row_bytes = nb * 20u;
    uint32_t nrows, nmax, step, mine, off;
    if constexpr (PAIR) {
        // channel c of this workgroup is bank channel c G + blockIdx.x; set j walks the channels c = j / 2, + SETS / 2, ... of
        // half j & 1 (0: gate rows, 1: up rows, I rows further on), so slot trip * SETS + j is (channel, half) = (slot / 2, slot & 1)
        constexpr uint32_t H2 = SETS / 2;
        const uint32_t I = N >> 1;
        if (blockIdx.x >= I) return;
        const uint32_t nch = (I - blockIdx.x + G - 1u) / G;      // channels of this workgroup
        const uint32_t sub = set >> 1, half = set & 1u;
        nrows = 2u * nch;
        nmax = (nch + H2 - 1u) / H2;
        step = G * H2 * row_bytes;
        mine = nch > sub ? (nch - sub + H2 - 1u) / H2 : 0u;
        off = (half * I + (mine ? sub : 0u) * G + blockIdx.x) * row_bytes + g * 20u;
    } else {
        if (blockIdx.x >= N) return;
        nrows = (N - blockIdx.x + G - 1u) / G;               // row slots of this workgroup
        nmax = (nrows + SETS - 1u) / SETS;                   // trip count, uniform over the workgroup
        step = G * SETS * row_bytes;                         // bytes between consecutive rows of one set
        mine = nrows > set ? (nrows - set + SETS - 1u) / SETS : 0u;
        off = ((mine ? set : 0u) * G + blockIdx.x) * row_bytes + g * 20u;
    }
    const uint32_t off_max = off + (mine ? mine - 1u : 0u) * step;   // loads past the set's last row re-read it

    // 1. activation loads go first: loads return in order, and the rotation must not queue behind the weight prefetch
    h8_t xv[XT];
#pragma unroll
    for (int t = 0; t < XT; ++t) {
        const uint32_t gt = wave + nw * t;
        const uint32_t gg = min(gt * 16u + (l64 & 15u), nb - 1u);
        xv[t] = qw_load_x8_f16<XDT>(p.x, (uint64_t)gg * 32u + 8u * (l64 >> 4));
    }
    __builtin_amdgcn_sched_barrier(0);
    // 2. first weight rows
    qw_hq4_block buf[D];
    auto issue = [&](int slot) {
        buf[slot] = *(const qw_hq4_block*)(p.bank + off);
        off = min(off + step, off_max);
    };
#pragma unroll
    for (int j = 0; j < D0; ++j) issue(j);
    __builtin_amdgcn_sched_barrier(0);
    // 3. rotation on the matrix cores into the shared image
    {
        h8_t h_lo, h_hi;
        qw_hadamard_pair(l64 & 15u, l64 >> 4, h_lo, h_hi);
        if (tiler) {
#pragma unroll
            for (int t = 0; t < XT; ++t) qw_rotate_tile_to_lds(xv[t], wave + nw * t, nb, l64, p.rotate != 0, h_lo, h_hi, xs);
        }
    }
    __syncthreads();
    // 4. this lane's column: 16 operand pairs and the group sum S
    h2_t xo[16];
    float S;
    {
        const h8_t* src = xs + g * 5;
        const h2_t one = {(h1_t)1.0f, (h1_t)1.0f};
        float s0 = 0.f, s1 = 0.f;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const h8_t v = src[j];
#pragma unroll
            for (int e2 = 0; e2 < 4; ++e2) {
                const h2_t pr = {v[2 * e2], v[2 * e2 + 1]};
                if (e2 & 1) s1 = __builtin_amdgcn_fdot2(pr, one, s1, false);
                else s0 = __builtin_amdgcn_fdot2(pr, one, s0, false);
                xo[4 * j + e2] = pr;
            }
        }
        S = s0 + s1;
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int j = D0; j < D; ++j) issue(j);
    __builtin_amdgcn_sched_barrier(0);

    uint32_t rslot = set;   // row slot being consumed
    for (uint32_t ib = 0; ib < nmax; ib += D) {
#pragma unroll
        for (int j = 0; j < D; ++j) {
            if (ib + j >= nmax) break;
            const qw_hq4_block b = buf[j];
            float lo0 = 0.f, lo1 = 0.f, hi0 = 0.f, hi1 = 0.f;
#pragma unroll
            for (int w4 = 0; w4 < 4; ++w4) {
                const uint32_t w = b.qs[w4], w8 = w >> 8;
                const uint32_t m0 = w & 0x000F000Fu, m1 = w & 0x00F000F0u, m2 = w8 & 0x000F000Fu, m3 = w8 & 0x00F000F0u;
                lo0 = __builtin_amdgcn_fdot2(__builtin_bit_cast(h2_t, m0), xo[4 * w4 + 0], lo0, false);
                hi0 = __builtin_amdgcn_fdot2(__builtin_bit_cast(h2_t, m1), xo[4 * w4 + 1], hi0, false);
                lo1 = __builtin_amdgcn_fdot2(__builtin_bit_cast(h2_t, m2), xo[4 * w4 + 2], lo1, false);
                hi1 = __builtin_amdgcn_fdot2(__builtin_bit_cast(h2_t, m3), xo[4 * w4 + 3], hi1, false);
            }
            issue(j);
            const h2_t hd = __builtin_bit_cast(h2_t, b.hdr);
            // s * sum(q x) + (1024 s + b) * S: the header sum is exact in fp32 (two f16 values a factor 1024 / 1032 apart),
            // so the large terms 1024 s S and b S never meet as rounded fp32 numbers
            const float sc = (float)hd[0];
            const float q = __builtin_fmaf(hi0 + hi1, 0.0625f, lo0 + lo1);
            float v = __builtin_fmaf(sc * 16777216.0f, q, __builtin_fmaf(sc, 1024.0f, (float)hd[1]) * S);
            v = gvalid ? v : 0.0f;
            v = qw_reduce32_dpp(v);
            if (lane == 31u && rslot < nrows) part[rslot * cpr + chunk] = v;
            rslot += SETS;
        }
    }
    __syncthreads();
    // 5. fixed-order sum of the chunk partials of each row; with `keys` also the greedy-decoding fold of the reference's
    // head kernels (qwg_gemv_am_fold4 / qwg_gemv_am_reduce4, Sources/QWMetal/include/qw_gemm_f32_common.metalh:30-58):
    // larger (monotone bits, ~row) wins, so ties go to the lower row
    if constexpr (PAIR) {
        for (uint32_t c = tid; 2u * c < nrows; c += blockDim.x) {
            float gsum = 0.f, usum = 0.f;
            for (uint32_t k = 0; k < cpr; ++k) {
                gsum += part[(2u * c) * cpr + k];
                usum += part[(2u * c + 1u) * cpr + k];
            }
            const float a = qw_gated(gsum, usum, pp.ga);
            if (p.y32) p.y32[c * G + blockIdx.x] = a;         // fp32 for a rotation pass behind the launch
            else p.y16[c * G + blockIdx.x] = (h1_t)a;
        }
        return;
    }
    unsigned long long best = 0ull;
    for (uint32_t s = tid; s < nrows; s += blockDim.x) {
        float v = 0.f;
        for (uint32_t c = 0; c < cpr; ++c) v += part[s * cpr + c];
        const uint32_t row = s * G + blockIdx.x;
        if (p.y32) p.y32[row] = v;
        if (p.y16) p.y16[row] = (h1_t)v;
        if constexpr (FOLD) {
            const unsigned long long key = ((unsigned long long)qc_sortable_f32(v) << 32) | (uint32_t)~row;
            best = key > best ? key : best;
        }
    }
    if constexpr (FOLD) {
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) {
            const unsigned long long other = __shfl_xor(best, o, 64);
            best = other > best ? other : best;
        }
        __syncthreads();                                   // the partial sums are read: their LDS is free
        unsigned long long* wbest = (unsigned long long*)part;
        if ((tid & 63u) == 0u) wbest[tid >> 6] = best;
        __syncthreads();
        if (tid == 0u) {
            const uint32_t nwaves = (blockDim.x + 63u) >> 6;
            for (uint32_t wv = 1; wv < nwaves; ++wv) best = wbest[wv] > best ? wbest[wv] : best;
            pp.keys[blockIdx.x] = best;
        }
    }
}
};

// The same kernel with the block loads issued and awaited by hand, and with less vector work per row.
// A compiled rolling window drains once per trip: the register allocator reuses a load's destination as a temporary,
// copies the value out at the loop's ends, and every copy waits for its load, so a wave has at most D rows in flight right
// after a trip's start and none at its end.  Here the loads are `asm volatile` statements whose destination registers are
// tied in and out ("+v": the same registers all the way round the loop), and each row is consumed behind an
// s_waitcnt vmcnt(2 (D - 1)): exactly the two loads of the oldest row have to have landed, the D - 1 younger rows stay in
// flight.  The activation loads are issued by hand as well: the compiler does not know of the block loads behind them and
// would wait for everything (vmcnt(0)) before the rotation.
// Rows are consumed in groups of D, slot j of a group after slot j - 1.  The first group is padded at its head with `pad`
// dummies (row 0 fetched once more, its arithmetic skipped by a scalar branch) so that the last group is whole and every
// slot index is a constant - a slot picked at run time makes the compiler copy registers whose loads are still in flight.
// Vector work per row (the SIMDs are nearly as busy as the memory system: a workgroup's waves do not spread evenly over the
// four SIMDs of a compute unit, and the fullest SIMD sets the pace): the row's address is a scalar base that moves by one
// row stride per issue plus a lane offset that never changes; the first product of each sum does not accumulate (no
// register to clear); the sums run at 2^-24 of their value so that the scale is used as the f16 it is loaded as
// (v' = s q + ((1024 s + b) S 2^-24): the same roundings as fma(s 2^24, q, (1024 s + b) S), a power of two apart) and the
// factor comes back once per row in the epilogue; lanes past the row's last block multiply zeros instead of being
// masked; the partial sums of all rows, the one a short set does not have included, go to LDS unconditionally.
template <int XDT, int SETS, int D, int D0 = D>
struct qw_gemv_colw_kernel {
static constexpr int kLaunchBound = 1024;
template <int N>
static __device__ __forceinline__ void wait_row(uint32_t& hdr, u4_t& q) {
    asm volatile("s_waitcnt vmcnt(%2)" : "+v"(hdr), "+v"(q) : "n"(N));
}
template <int U, typename F>
static __device__ __forceinline__ void static_for(F&& f) {
    if constexpr (U < D) {
        f(std::integral_constant<int, U>{});
        static_for<U + 1>(f);
    }
}
static __device__ __forceinline__ float dot2_first(uint32_t a, h2_t b) {
    float d;
    asm("v_dot2_f32_f16 %0, %1, %2, 0" : "=v"(d) : "v"(a), "v"(b));
    return d;
}
static __device__ __forceinline__ void run(const qc_params& p) {
    constexpr int XT = SETS == 1 ? 5 : (SETS == 2 ? 2 : 1);
    extern __shared__ h8_t qc_lds[];
    const uint32_t nb = p.nb, cpr = p.cpr, N = p.N;
    h8_t* xs = qc_lds;
    float* part = (float*)(qc_lds + (size_t)nb * 5);
    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & 31u, hw = tid >> 5;
    const uint32_t wave = tid >> 6, l64 = tid & 63u;
    const uint32_t threads = 32u * cpr * SETS;   // blockDim.x, without the load from the dispatch packet ahead of the first loads
    const uint32_t nw = threads >> 6;
    const bool tiler = wave < nw;
    const uint32_t set = hw / cpr, chunk = hw - set * cpr;
    const uint32_t g0 = chunk * 32u + lane;
    const bool gvalid = g0 < nb;
    const uint32_t g = gvalid ? g0 : nb - 1u;
    const uint32_t G = gridDim.x;
    if (blockIdx.x >= N) return;
    const uint32_t nrows = (N - blockIdx.x + G - 1u) / G;
    const uint32_t nmax = (nrows + SETS - 1u) / SETS;        // rows of the fullest set: the trip count, workgroup-uniform
    const uint32_t ngroups = (nmax + D - 1u) / D;
    const uint32_t pad = ngroups * D - nmax;                 // dummies at the head of the first group, 0 .. D - 1
    const uint32_t row_bytes = nb * 20u;
    const uint32_t step = G * SETS * row_bytes;              // bytes between consecutive rows of one set
    const uint32_t mine = nrows > set ? (nrows - set + SETS - 1u) / SETS : 0u;
    // lane offset inside a row band (added, unsigned, to the band's scalar base: it can never step back a band); a set
    // without rows walks set 0's, and a set one row short reads set 0's last row where it has none (set 0 is never short)
    const uint32_t voff0 = blockIdx.x * row_bytes + g * 20u;
    const uint32_t voff = mine ? set * G * row_bytes + voff0 : voff0;
    const uint32_t voff_last = mine < nmax ? voff0 : voff;

    // 1. activation loads, by hand
    u4_t xraw[XT];
#pragma unroll
    for (int t = 0; t < XT; ++t) {
        const uint32_t gt = wave + nw * t;
        const uint32_t gg = min(gt * 16u + (l64 & 15u), nb - 1u);
        const uint32_t xoff = (gg * 32u + 8u * (l64 >> 4)) * 2u;
        asm volatile("global_load_dwordx4 %0, %1, %2" : "=&v"(xraw[t]) : "v"(xoff), "s"(p.x) : "memory");
    }
    // 2. the first D rows
    uint32_t hdr[D];
    u4_t qv[D];
#pragma unroll
    for (int j = 0; j < D; ++j) {
        hdr[j] = 0u;
        qv[j] = u4_t{0u, 0u, 0u, 0u};
    }
    const uint8_t* rowp = p.bank;                 // scalar: the band of the row the next issue fetches
    int32_t krow = -(int32_t)pad;                 // its index; the dummies (< 0) fetch row 0
    const int32_t klast = (int32_t)nmax - 1;
    auto issue = [&](int slot) {
        // the set's last row always lands in slot D - 1
        const uint32_t vo = (slot == D - 1 && krow == klast) ? voff_last : voff;
        asm volatile("global_load_dword %0, %2, %3\n\tglobal_load_dwordx4 %1, %2, %3 offset:4"
                     : "+v"(hdr[slot]), "+v"(qv[slot]) : "v"(vo), "s"(rowp) : "memory");
        rowp += krow >= 0 ? step : 0u;
        ++krow;
    };
    // D0 of the window's D rows go out ahead of the activation prologue, the rest behind it: every load queued here
    // delays the activation loads of the waves that start later on the same compute unit
#pragma unroll
    for (int j = 0; j < D0; ++j) issue(j);
    // 3. rotation on the matrix cores into the shared image: the XT activation loads have landed, the 2 D0 block loads fly on
#pragma unroll
    for (int t = 0; t < XT; ++t) asm volatile("s_waitcnt vmcnt(%1)" : "+v"(xraw[t]) : "n"(2 * D0));
    {
        h8_t h_lo, h_hi;
        qw_hadamard_pair(l64 & 15u, l64 >> 4, h_lo, h_hi);
        if (tiler) {
#pragma unroll
            for (int t = 0; t < XT; ++t)
                qw_rotate_tile_to_lds(qw_x8_from_raw<XDT>(xraw[t]), wave + nw * t, nb, l64, p.rotate != 0, h_lo, h_hi, xs);
        }
    }
    __syncthreads();
    // 4. this lane's column: 16 operand pairs and the group sum S (zeros past the row's last block)
    h2_t xo[16];
    float Sp;
    {
        const h8_t* src = xs + g * 5;
        const h2_t one = {(h1_t)1.0f, (h1_t)1.0f};
        const h2_t zero = {(h1_t)0.0f, (h1_t)0.0f};
        float s0 = 0.f, s1 = 0.f;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const h8_t v = src[j];
#pragma unroll
            for (int e2 = 0; e2 < 4; ++e2) {
                const h2_t pr = {v[2 * e2], v[2 * e2 + 1]};
                if (e2 & 1) s1 = __builtin_amdgcn_fdot2(pr, one, s1, false);
                else s0 = __builtin_amdgcn_fdot2(pr, one, s0, false);
                xo[4 * j + e2] = gvalid ? pr : zero;
            }
        }
        Sp = gvalid ? (s0 + s1) * 5.9604644775390625e-08f : 0.0f;     // S 2^-24
    }

    // partial sums: row slot r of the workgroup at part[r cpr + chunk]
    uint32_t part_at = (uint32_t)(uintptr_t)part + ((set * cpr + chunk) << 2);
    const uint32_t part_step = (SETS * cpr) << 2;
    auto consume = [&](int slot) {
        const uint32_t w0 = qv[slot][0], w1 = qv[slot][1], w2 = qv[slot][2], w3 = qv[slot][3];
        float lo = dot2_first(w0 & 0x000F000Fu, xo[0]);
        float hi = dot2_first(w0 & 0x00F000F0u, xo[1]);
        lo = __builtin_amdgcn_fdot2(__builtin_bit_cast(h2_t, (w0 >> 8) & 0x000F000Fu), xo[2], lo, false);
        hi = __builtin_amdgcn_fdot2(__builtin_bit_cast(h2_t, (w0 >> 8) & 0x00F000F0u), xo[3], hi, false);
#define QCW_WORD(W, B)                                                                                        \
        lo = __builtin_amdgcn_fdot2(__builtin_bit_cast(h2_t, W & 0x000F000Fu), xo[B + 0], lo, false);         \
        hi = __builtin_amdgcn_fdot2(__builtin_bit_cast(h2_t, W & 0x00F000F0u), xo[B + 1], hi, false);         \
        lo = __builtin_amdgcn_fdot2(__builtin_bit_cast(h2_t, (W >> 8) & 0x000F000Fu), xo[B + 2], lo, false);  \
        hi = __builtin_amdgcn_fdot2(__builtin_bit_cast(h2_t, (W >> 8) & 0x00F000F0u), xo[B + 3], hi, false);
        QCW_WORD(w1, 4)
        QCW_WORD(w2, 8)
        QCW_WORD(w3, 12)
#undef QCW_WORD
        const h2_t hd = __builtin_bit_cast(h2_t, hdr[slot]);
        const float sc = (float)hd[0];
        const float m = __builtin_fmaf(sc, 1024.0f, (float)hd[1]) * Sp;   // the header sum is exact in fp32
        const float q = __builtin_fmaf(hi, 0.0625f, lo);
        float v = __builtin_fmaf(sc, q, m);
        v = qw_reduce32_dpp(v);
        if (lane == 31u) *(__attribute__((address_space(3))) float*)(uintptr_t)part_at = v;
        part_at += part_step;
    };
#pragma unroll
    for (int j = D0; j < D; ++j) issue(j);
    int32_t kcons = -(int32_t)pad;                // scalar: the row being consumed; a dummy's arithmetic is skipped
    for (uint32_t grp = 0; grp + 1u < ngroups; ++grp) {
#pragma unroll
        for (int j = 0; j < D; ++j) {
            wait_row<2 * (D - 1)>(hdr[j], qv[j]);
            if (kcons >= 0) consume(j);
            ++kcons;
            issue(j);
        }
    }
    static_for<0>([&](auto uc) {
        constexpr int u = decltype(uc)::value;
        wait_row<2 * (D - 1 - u)>(hdr[u], qv[u]);
        if (kcons >= 0) consume(u);
        ++kcons;
    });
    __syncthreads();
    // 5. fixed-order sum of the chunk partials of each row, back at full scale
    for (uint32_t s = tid; s < nrows; s += threads) {
        float v = 0.f;
        for (uint32_t c = 0; c < cpr; ++c) v += part[s * cpr + c];
        v *= 16777216.0f;
        const uint32_t row = s * G + blockIdx.x;
        if (p.y32) p.y32[row] = v;
        if (p.y16) p.y16[row] = (h1_t)v;
    }
}
};

// The hand-issued window with the arithmetic taken out: every lane adds up the 32-bit words of the 20-byte pieces it
// fetches (the rows, the grid, the pieces and the window of qw_gemv_colw_kernel<.., 3, 3>) and a workgroup adds its total into
// sum[blockIdx.x & 255].  What this launch takes over a bank is what the decode GEMV's own request pattern costs.
#define QCS_FIELDS(X) X(const uint8_t*, bank) X(unsigned long long*, sum) X(uint32_t, N) X(uint32_t, nb) X(uint32_t, cpr)
QW_ARG_BLOCK(qcs_params, QCS_FIELDS)
template <int SETS>
struct qw_rows_checksum_kernel {
static constexpr int kLaunchBound = 1024;
static constexpr int D = 3;
static __device__ __forceinline__ void run(const qcs_params& p) {
    __shared__ unsigned long long wsum[16];
    const uint32_t nb = p.nb, cpr = p.cpr, N = p.N;
    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & 31u, hw = tid >> 5;
    const uint32_t set = hw / cpr, chunk = hw - set * cpr;
    const uint32_t g0 = chunk * 32u + lane;
    const bool gvalid = g0 < nb;
    const uint32_t g = gvalid ? g0 : nb - 1u;
    const uint32_t G = gridDim.x;
    if (blockIdx.x >= N) return;
    const uint32_t nrows = (N - blockIdx.x + G - 1u) / G;
    const uint32_t nmax = (nrows + SETS - 1u) / SETS;
    const uint32_t ngroups = (nmax + D - 1u) / D;
    const uint32_t pad = ngroups * D - nmax;
    const uint32_t row_bytes = nb * 20u;
    const uint32_t step = G * SETS * row_bytes;
    const uint32_t mine = nrows > set ? (nrows - set + SETS - 1u) / SETS : 0u;
    const uint32_t voff0 = blockIdx.x * row_bytes + g * 20u;
    const uint32_t voff = mine ? set * G * row_bytes + voff0 : voff0;
    const uint32_t voff_last = mine < nmax ? voff0 : voff;
    uint32_t hdr[D];
    u4_t qv[D];
#pragma unroll
    for (int j = 0; j < D; ++j) {
        hdr[j] = 0u;
        qv[j] = u4_t{0u, 0u, 0u, 0u};
    }
    const uint8_t* rowp = p.bank;
    int32_t krow = -(int32_t)pad;
    const int32_t klast = (int32_t)nmax - 1;
    auto issue = [&](int slot) {
        const uint32_t vo = (slot == D - 1 && krow == klast) ? voff_last : voff;
        asm volatile("global_load_dword %0, %2, %3\n\tglobal_load_dwordx4 %1, %2, %3 offset:4"
                     : "+v"(hdr[slot]), "+v"(qv[slot]) : "v"(vo), "s"(rowp) : "memory");
        rowp += krow >= 0 ? step : 0u;
        ++krow;
    };
#pragma unroll
    for (int j = 0; j < D; ++j) issue(j);
    unsigned long long acc = 0ull;
    int32_t kcons = -(int32_t)pad;
    auto consume = [&](int slot) {      // a row of this lane's own set only (a short set's last fetch is set 0's row)
        if (kcons >= 0 && gvalid && (uint32_t)kcons < mine)
            acc += (unsigned long long)hdr[slot] + qv[slot][0] + qv[slot][1] + qv[slot][2] + qv[slot][3];
        ++kcons;
    };
    for (uint32_t grp = 0; grp + 1u < ngroups; ++grp) {
#pragma unroll
        for (int j = 0; j < D; ++j) {
            asm volatile("s_waitcnt vmcnt(%2)" : "+v"(hdr[j]), "+v"(qv[j]) : "n"(2 * (D - 1)));
            consume(j);
            issue(j);
        }
    }
    asm volatile("s_waitcnt vmcnt(4)" : "+v"(hdr[0]), "+v"(qv[0]));
    consume(0);
    asm volatile("s_waitcnt vmcnt(2)" : "+v"(hdr[1]), "+v"(qv[1]));
    consume(1);
    asm volatile("s_waitcnt vmcnt(0)" : "+v"(hdr[2]), "+v"(qv[2]));
    consume(2);
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) acc += __shfl_xor(acc, o, 64);
    if ((tid & 63u) == 0u) wsum[tid >> 6] = acc;
    __syncthreads();
    if (tid == 0u) {
        unsigned long long total = 0ull;
        for (uint32_t wv = 0; wv < ((32u * cpr * SETS + 63u) >> 6); ++wv) total += wsum[wv];
        atomicAdd(p.sum + (blockIdx.x & 255u), total);
    }
}
};

// Folds the workgroups' keys into the token: one workgroup.
__global__ __launch_bounds__(256) void qw_col_keys_fin_kernel(const unsigned long long* __restrict__ keys, uint32_t count, int32_t* token) {
    __shared__ unsigned long long wbest[4];
    unsigned long long best = 0ull;
    for (uint32_t i = threadIdx.x; i < count; i += 256u) best = keys[i] > best ? keys[i] : best;
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        const unsigned long long other = __shfl_xor(best, o, 64);
        best = other > best ? other : best;
    }
    if ((threadIdx.x & 63u) == 0u) wbest[threadIdx.x >> 6] = best;
    __syncthreads();
    if (threadIdx.x == 0u) {
        for (int wv = 1; wv < 4; ++wv) best = wbest[wv] > best ? wbest[wv] : best;
        *token = (int32_t)~(uint32_t)best;
    }
}

// kind: 0 = the hand-issued window (three rows, two of them ahead of the prologue), 1 = the compiled window (the head's
// fold rides in its epilogue), 2..5 = other hand-issued windows for tuning
template <int XDT, int SETS>
hipError_t qc_launch(hipStream_t st, const qc_params& p, uint32_t wgs, uint32_t threads, size_t lds, uint32_t kind, unsigned long long* keys) {
    if (keys) {
        qc_params_fold pf;
#define QC_TAKE(T, n) pf.n = p.n;
        QC_FIELDS(QC_TAKE)
#undef QC_TAKE
        pf.keys = keys;
        qw_launch_scalar<qw_gemv_col_kernel<XDT, SETS, 2, 2, qc_params_fold>>(dim3(wgs), dim3(threads), lds, st, pf);
        return hipGetLastError();
    }
    switch (kind) {
        case 1: qw_launch_scalar<qw_gemv_col_kernel<XDT, SETS, 2, 2>>(dim3(wgs), dim3(threads), lds, st, p); break;
        case 2: qw_launch_scalar<qw_gemv_colw_kernel<XDT, SETS, 2, 2>>(dim3(wgs), dim3(threads), lds, st, p); break;
        case 3: qw_launch_scalar<qw_gemv_colw_kernel<XDT, SETS, 3, 3>>(dim3(wgs), dim3(threads), lds, st, p); break;
        case 4: qw_launch_scalar<qw_gemv_colw_kernel<XDT, SETS, 4, 2>>(dim3(wgs), dim3(threads), lds, st, p); break;
        case 5: qw_launch_scalar<qw_gemv_colw_kernel<XDT, SETS, 6, 3>>(dim3(wgs), dim3(threads), lds, st, p); break;
        default: qw_launch_scalar<qw_gemv_colw_kernel<XDT, SETS, 3, 2>>(dim3(wgs), dim3(threads), lds, st, p); break;
    }
    return hipGetLastError();
}

}  // namespace

// Tries the column-stationary kernel for a validated m = 1 HQ4_G32_M5 call; false when the shape is outside its envelope.
// `tune` (tests and tuning): bits 0..2 pick the kernel (0 = automatic: the hand-issued window of three rows, two of them
// ahead of the prologue; 1 = the compiled window; 2..5 = hand-issued windows of (2, 2), (3, 3), (4, 2), (6, 3) rows), bits
// 3..4 scale the grid (1 -> half, 2 -> double, 3 -> one and a half), bit 5 asks for four row sets per workgroup.
// `keys` (NULL, or room for `keys_cap` entries) + `token`: the head's greedy-decoding fold rides in the epilogue (compiled
// window) and a second, one-workgroup launch writes *token; a grid larger than keys_cap drops the fold (*folded = false) and
// the caller folds the logits.
bool qw_col_gemv(hipStream_t st, const qwhip_weight_view* w, const void* x, uint32_t x_dtype, bool rotate, void* y16,
                 float* y32, uint32_t tune, hipError_t* err, unsigned long long* keys, uint32_t keys_cap, int32_t* token,
                 bool* folded) {
    if (w->kind != QWHIP_KIND_HQ4_G32_M5) return false;
    const uint32_t nb = w->k / 32u, cpr = (nb + 31u) / 32u;
    if (cpr > 32u) return false;
    if ((uint64_t)w->n * nb * 20u >= (1ull << 32)) return false;   // 32-bit offsets inside the bank
    if (((uintptr_t)x & 15u) != 0) return false;
    uint32_t sets = cpr <= 3u ? 4u : (cpr <= 12u ? 2u : 1u);
    if ((tune & 0x20u) && cpr <= 8u) sets = 4u;
    const uint32_t threads = 32u * cpr * sets;
    const uint32_t waves = (threads + 63u) / 64u;
    const uint32_t kind = keys ? 1u : (tune & 7u);
    static const uint32_t kWindow[6] = {3u, 0u, 2u, 3u, 4u, 6u};
    const uint32_t wdepth = kWindow[kind <= 5u ? kind : 0u];       // 0: the compiled window
    // Waves per compute unit, measured on N = 17408, K = 5120.  Compiled window: 10 (11.2-11.3 us; 11.5 with 20, 13.5+ with
    // 5).  Hand-issued window: 20 (10.8-10.9 us on 1024 workgroups; 11.4 on 512 with the same window, 11.1 on 768; deeper
    // windows 11.1-11.9, a window of two 11.3).  At least four rows per set, at most 128 row slots per workgroup.
    uint32_t wgs = (256u * (wdepth ? 20u : 10u) + waves / 2u) / waves;
    // whole multiples of the 256 compute units: a grid that leaves some of them a workgroup more than the others was up to
    // 19 % slower (5120 x 17408: 569 workgroups 13.6 us, 512 workgroups 11.2 us; K = 6144 .. 18432 5-10 %)
    if (!(tune & 0x40u)) wgs = max(256u, (wgs + 128u) / 256u * 256u);   // tune bit 6 (tests): the unrounded grid
    if ((tune >> 3 & 3u) == 1u) wgs /= 2u;
    if ((tune >> 3 & 3u) == 2u) wgs *= 2u;
    if ((tune >> 3 & 3u) == 3u) wgs += wgs / 2u;
    wgs = min(wgs, max(1u, w->n / (sets * 4u)));
    wgs = max(wgs, qwhip_cdiv(w->n, 128u));
    if (!(tune & 0x40u) && wgs > 256u && wgs % 256u != 0u && (wgs + 255u) / 256u * 256u <= max(1u, w->n / (sets * 4u)))
        wgs = (wgs + 255u) / 256u * 256u;                          // the row-slot limit raised the grid: up to the next whole multiple
    const uint32_t rows_per_wg = qwhip_cdiv(w->n, wgs);
    // partial sums: one float per (row slot, chunk); the hand-issued window rounds the trip count up to whole groups and
    // stores every row slot of every group
    const size_t part_rows = wdepth ? (size_t)qwhip_cdiv(qwhip_cdiv(rows_per_wg, sets), wdepth) * wdepth * sets : rows_per_wg;
    const size_t lds = (size_t)nb * 80u + part_rows * cpr * 4u;
    if (lds > 60u * 1024u) return false;
    qc_params p;
    p.bank = (const uint8_t*)w->blocks;
    p.x = x;
    p.y16 = (h1_t*)y16;
    p.y32 = y32;
    p.N = w->n;
    p.nb = nb;
    p.cpr = cpr;
    p.rotate = rotate ? 1u : 0u;
    const bool fold = keys && token && wgs <= keys_cap && (size_t)rows_per_wg * cpr * 4u >= 8u * waves;
    unsigned long long* fold_keys = fold ? keys : nullptr;
    if (folded) *folded = fold;
    hipError_t e;
    if (x_dtype == QWHIP_F16) {
        e = sets == 4 ? qc_launch<QWHIP_F16, 4>(st, p, wgs, threads, lds, kind, fold_keys)
          : sets == 2 ? qc_launch<QWHIP_F16, 2>(st, p, wgs, threads, lds, kind, fold_keys)
                      : qc_launch<QWHIP_F16, 1>(st, p, wgs, threads, lds, kind, fold_keys);
    } else {
        e = sets == 4 ? qc_launch<QWHIP_BF16, 4>(st, p, wgs, threads, lds, kind, fold_keys)
          : sets == 2 ? qc_launch<QWHIP_BF16, 2>(st, p, wgs, threads, lds, kind, fold_keys)
                      : qc_launch<QWHIP_BF16, 1>(st, p, wgs, threads, lds, kind, fold_keys);
    }
    if (e == hipSuccess && fold) {
        hipLaunchKernelGGL(qw_col_keys_fin_kernel, dim3(1), dim3(256), 0, st, keys, wgs, token);
        e = hipGetLastError();
    }
    *err = e;
    return true;
}

// Gate|up form of the column-stationary kernel for one activation row over a validated HQ4_G32_M5 gate|up bank (n = 2 I rows):
// act f16 [I] = gated(Wg . x, Wu . x) on the fp32 sums, no output rotation (or the same as fp32 into gated32 [I]).  The workgroups walk the gate half and the up half
// of the bank as two bands, like the decode GEMV walks its one.  false when the shape is outside the envelope (rows longer
// than 12288 columns take one row set per workgroup, which cannot hold a gate and an up row side by side).
bool qw_col_pair_gemv(hipStream_t st, const qwhip_weight_view* w, const void* x, uint32_t x_dtype, bool rotate, void* act16,
                      float* gated32, const qw_act ga, hipError_t* err) {
    if (w->kind != QWHIP_KIND_HQ4_G32_M5 || (w->n & 1u)) return false;
    const uint32_t nb = w->k / 32u, cpr = (nb + 31u) / 32u, inter = w->n / 2u;
    if (cpr > 12u || inter < 64u) return false;
    if ((uint64_t)w->n * nb * 20u >= (1ull << 32)) return false;   // 32-bit offsets inside the bank
    if (((uintptr_t)x & 15u) != 0) return false;
    const uint32_t sets = cpr <= 3u ? 4u : 2u, h2 = sets / 2u;
    const uint32_t threads = 32u * cpr * sets;
    const uint32_t waves = (threads + 63u) / 64u;
    uint32_t wgs = (256u * 10u + waves / 2u) / waves;              // ten waves per compute unit, as the compiled window of the GEMV
    wgs = max(256u, (wgs + 128u) / 256u * 256u);                   // whole multiples of the compute units
    wgs = min(wgs, max(1u, inter / (h2 * 4u)));                    // at least four channels per set
    wgs = max(wgs, qwhip_cdiv(inter, 64u));                        // at most 128 row slots per workgroup
    const uint32_t ch_per_wg = qwhip_cdiv(inter, wgs);
    const size_t lds = (size_t)nb * 80u + (size_t)2u * ch_per_wg * cpr * 4u;
    if (lds > 60u * 1024u) return false;
    qc_params_pair p;
    p.bank = (const uint8_t*)w->blocks;
    p.x = x;
    p.y16 = (h1_t*)act16;
    p.y32 = gated32;                                               // not NULL: gated(g, u) as fp32 [I] instead of act16
    p.N = w->n;
    p.nb = nb;
    p.cpr = cpr;
    p.rotate = rotate ? 1u : 0u;
    p.ga = ga;
    if (x_dtype == QWHIP_F16) {
        if (sets == 4u) qw_launch_scalar<qw_gemv_col_kernel<QWHIP_F16, 4, 2, 2, qc_params_pair>>(dim3(wgs), dim3(threads), lds, st, p);
        else qw_launch_scalar<qw_gemv_col_kernel<QWHIP_F16, 2, 2, 2, qc_params_pair>>(dim3(wgs), dim3(threads), lds, st, p);
    } else {
        if (sets == 4u) qw_launch_scalar<qw_gemv_col_kernel<QWHIP_BF16, 4, 2, 2, qc_params_pair>>(dim3(wgs), dim3(threads), lds, st, p);
        else qw_launch_scalar<qw_gemv_col_kernel<QWHIP_BF16, 2, 2, 2, qc_params_pair>>(dim3(wgs), dim3(threads), lds, st, p);
    }
    *err = hipGetLastError();
    return true;
}

// The word sum of a bank of `rows` rows of `row_bytes` bytes (whole 20-byte pieces), read with the decode GEMV's own launch:
// see qw_rows_checksum_kernel.  Same 256 caller-cleared sums as qwhip_plane_checksum.
extern "C" qwhip_status qwhip_plane_checksum_rows(qwhip_stream_t s, const void* plane, uint32_t rows, uint32_t row_bytes, uint64_t* sum) {
    QWHIP_REQUIRE(s);
    QWHIP_REQUIRE(sum);
    if (rows == 0 || row_bytes == 0) return QWHIP_OK;
    QWHIP_REQUIRE(plane);
    const uint32_t nb = row_bytes / 20u, cpr = (nb + 31u) / 32u;
    if (row_bytes % 20u != 0 || ((uintptr_t)plane & 3u) != 0 || cpr > 32u || (uint64_t)rows * row_bytes >= (1ull << 32))
        return qwhip_fail(QWHIP_E_BAD_SHAPE, "row checksum takes rows of whole 20-byte pieces, at most 1024 of them, under 4 GiB in all; got %u rows of %u bytes", rows, row_bytes);
    const uint32_t sets = cpr <= 3u ? 4u : (cpr <= 12u ? 2u : 1u);
    const uint32_t threads = 32u * cpr * sets, waves = (threads + 63u) / 64u;
    uint32_t wgs = (256u * 20u + waves / 2u) / waves;      // the decode GEMV's grid
    wgs = min(wgs, max(1u, rows / (sets * 4u)));
    wgs = max(wgs, qwhip_cdiv(rows, 128u));
    qcs_params p;
    p.bank = (const uint8_t*)plane;
    p.sum = (unsigned long long*)sum;
    p.N = rows;
    p.nb = nb;
    p.cpr = cpr;
    if (sets == 4) qw_launch_scalar<qw_rows_checksum_kernel<4>>(dim3(wgs), dim3(threads), 0, s->stream, p);
    else if (sets == 2) qw_launch_scalar<qw_rows_checksum_kernel<2>>(dim3(wgs), dim3(threads), 0, s->stream, p);
    else qw_launch_scalar<qw_rows_checksum_kernel<1>>(dim3(wgs), dim3(threads), 0, s->stream, p);
    QWHIP_TRY_HIP(hipGetLastError());
    return QWHIP_OK;
}
