// Verify GEMV (m = 2..16 activation rows already in the container's basis) on the matrix cores, split along K.
//
// A wavefront owns a tile of 16 bank rows for one K range and contracts it with v_mfma_f32_16x16x32_f16: operand A is
// 16 bank rows x 32 columns of exact f16 weights (RN_f16((1024 + q) s + b) / RN_f16(code s + b): the weights of
// qwhip_dequant_f16), operand B the same 32 columns of up to 16 activation rows, the fp32 accumulator the 16 x 16 tile of
// outputs.  Which 32 columns one instruction contracts is free as long as both operands agree, and that freedom removes
// every transposition: lane (row r, quarter c) owns the whole 32-column slice 4 g + c of its bank row (consecutive
// quarters own consecutive slices: 64..144 contiguous bytes per row and request), dequantizes its four 8-column chunks
// with its own header, and instruction j of group g contracts chunk j of the four slices 4 g .. 4 g + 3 - lane (n, c) of
// operand B reads chunk j of slice 4 g + c of activation row n from the workgroup's LDS image.  The cost of a slice is the
// dequantization (about 12 vector operations per 8 weights) whatever the number of activation rows.
//
// The slices go from the bank to per-wave landing slots in LDS (global_load_lds), D groups ahead of their use, and the
// waits are explicit: loads that land in registers and are carried around the loop get copied by the register allocator
// at the loop head, each copy waits for its load, and the window of loads in flight empties once per trip.
//
// K is split over workgroups because the activation image has to fit LDS (80 bytes per activation row and slice: the
// pitch that spreads a 16-lane operand read over all banks): workgroup (band, kr) stages the activations of K range kr
// once and its waves walk row tiles band * waves + wave, + bands * waves, ...  With one K range a tile's outputs are
// stored directly.  With several, every (tile, range) wave writes its 16 x 16 fp32 partial to the stream's scratch and a
// second, small launch adds the partials in range order and stores the outputs (stream order makes the partials visible;
// an in-kernel hand-over through device-scope fences measured five to twenty times slower than the whole GEMV).
// Measured (N = 5120, K = 17408, 4-bit): 18.7 .. 20.7 us for m = 2 .. 16, of which 3.8 us staging and first requests,
// 12.5 us the loop (4.4 TB/s), about 3 us the second launch.
#include <atomic>
#include <type_traits>

#include "qwhip_common.h"
#include "qw_slice.h"

namespace {

// part: [K range][activation row][padded bank row]
#define QSK_FIELDS(X)                                                                                                       \
    X(const uint8_t*, bank) X(const void*, x) X(float*, part) X(uint32_t, N) X(uint32_t, K) X(uint32_t, M) X(uint32_t, nsl)     \
    X(uint32_t, ks) X(uint32_t, nkr) X(uint32_t, bands) X(uint32_t, gshift) X(h1_t*, y16) X(float*, y32) X(uint32_t, bb)        \
    X(uint32_t, ntiles) X(uint64_t, row_bytes)
QW_ARG_BLOCK(qsk_params, QSK_FIELDS)

template <int N, int I = 0, class F>
__device__ __forceinline__ void qw_static_for(F&& f) {
    if constexpr (I < N) {
        f(std::integral_constant<int, I>{});
        qw_static_for<N, I + 1>(f);
    }
}

typedef __attribute__((address_space(3))) uint8_t* qsk_lds_ptr;
typedef const __attribute__((address_space(1))) void* qsk_gptr;

// Bytes of one wave's landing slot: 64 headers, then the 64 lanes' code words in pieces of 16 bytes.
template <int FMT>
__host__ __device__ constexpr uint32_t qsk_slot_bytes() { return 256u + 256u * (uint32_t)qg_slice_words<FMT>(); }

// One group of a lane: its slice (header + code words) out of landing slot SLOT of its wave, and the four 8-column pieces
// of its activation operand.  The slices travel from the bank into LDS without passing registers (global_load_lds), so no
// register is reserved for a load in flight and nothing the compiler does with registers around the loop can wait for
// one; the wait for the slot (NEWER = slots requested after it), the reads and the wait for the reads are one statement.
template <int FMT, int SLOT, int NEWER>
__device__ __forceinline__ void qsk_take(uint32_t land4, uint32_t land16, uint32_t xa, qg_slice<FMT>& sl, u4_t (&b)[4]) {
    constexpr int SB = (int)qsk_slot_bytes<FMT>(), LOADS = FMT == QG_FMT_B8 ? 3 : 2;
    u4_t w0, w1;
    if constexpr (FMT == QG_FMT_B8) {
        asm volatile(
            "s_waitcnt vmcnt(%[n])\n\t"
            "ds_read_b32 %[h], %[a4] offset:%[oh]\n\t"
            "ds_read_b128 %[w0], %[a16] offset:%[ow]\n\t"
            "ds_read_b128 %[w1], %[a16] offset:%[ow1]\n\t"
            "ds_read_b128 %[b0], %[xa]\n\t"
            "ds_read_b128 %[b1], %[xa] offset:16\n\t"
            "ds_read_b128 %[b2], %[xa] offset:32\n\t"
            "ds_read_b128 %[b3], %[xa] offset:48\n\t"
            "s_waitcnt lgkmcnt(0)"
            : [h] "=&v"(sl.hdr), [w0] "=&v"(w0), [w1] "=&v"(w1), [b0] "=&v"(b[0]), [b1] "=&v"(b[1]), [b2] "=&v"(b[2]), [b3] "=&v"(b[3])
            : [a4] "v"(land4), [a16] "v"(land16), [xa] "v"(xa), [n] "n"(NEWER * LOADS), [oh] "n"(SLOT * SB), [ow] "n"(SLOT * SB + 256),
              [ow1] "n"(SLOT * SB + 256 + 1024)
            : "memory");
#pragma unroll
        for (int j = 0; j < 4; ++j) sl.q[j] = w0[j], sl.q[4 + j] = w1[j];
    } else {
        asm volatile(
            "s_waitcnt vmcnt(%[n])\n\t"
            "ds_read_b32 %[h], %[a4] offset:%[oh]\n\t"
            "ds_read_b128 %[w0], %[a16] offset:%[ow]\n\t"
            "ds_read_b128 %[b0], %[xa]\n\t"
            "ds_read_b128 %[b1], %[xa] offset:16\n\t"
            "ds_read_b128 %[b2], %[xa] offset:32\n\t"
            "ds_read_b128 %[b3], %[xa] offset:48\n\t"
            "s_waitcnt lgkmcnt(0)"
            : [h] "=&v"(sl.hdr), [w0] "=&v"(w0), [b0] "=&v"(b[0]), [b1] "=&v"(b[1]), [b2] "=&v"(b[2]), [b3] "=&v"(b[3])
            : [a4] "v"(land4), [a16] "v"(land16), [xa] "v"(xa), [n] "n"(NEWER * LOADS), [oh] "n"(SLOT * SB), [ow] "n"(SLOT * SB + 256)
            : "memory");
#pragma unroll
        for (int j = 0; j < 4; ++j) sl.q[j] = w0[j];
    }
}

// MP * 8 activation rows in the LDS image, D slice groups in flight per lane.  blockDim.x = 64 * waves; dynamic LDS =
// waves * D landing slots (first: their addresses stay below 64 KiB), then the image of ks slices at MP * 640 bytes each.
template <int FMT, int XDT, int MP, int D>
struct qw_gemv_sk_kernel {
static constexpr int kLaunchBound = 512;
static __device__ __forceinline__ void run(const qsk_params& p) {
    extern __shared__ __attribute__((aligned(16))) uint8_t qsk_lds[];
    constexpr uint32_t ACTS = 8u * MP, SLB = ACTS * 80u, SB = qsk_slot_bytes<FMT>();
    const uint32_t tid = threadIdx.x, lane = tid & 63u, W = blockDim.x >> 6;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t kr = blockIdx.x % p.nkr, band = blockIdx.x / p.nkr;
    const uint32_t s0 = kr * p.ks;                      // first slice of this K range
    const uint32_t ks = min(p.ks, p.nsl - s0);          // its slices: a multiple of 4
    const uint32_t ng = ks >> 2;                        // groups of four slices
    const uint32_t nw = (p.ks >> 2) / D;                // windows of D groups a wave walks per tile (p.ks is whole windows)
    const uint32_t r16 = lane & 15u, c = lane >> 4;
    const uint32_t tstep = p.bands * W;
    const uint32_t magic = qw_vgpr_const(0x64006400u);
    const qsk_lds_ptr lds0 = (qsk_lds_ptr)qsk_lds;
    const qsk_lds_ptr land = lds0 + wave * (D * SB);    // this wave's landing slots
    uint8_t* const ximg = qsk_lds + W * (D * SB);
    const uint32_t land4 = (uint32_t)(uintptr_t)land + lane * 4u, land16 = (uint32_t)(uintptr_t)land + lane * 16u;

    // the slice this lane requests for group g of tile t: slice s0 + 4 g + c of bank row 16 t + r16 (rows past the bank
    // re-read its last row, groups past a short last range its last group: their products are never stored / meet zero
    // activations)
    uint32_t t = band * W + wave;
    const uint32_t ntw = t < p.ntiles ? (p.ntiles - t + tstep - 1u) / tstep : 0u;   // tiles of this wave
    const uint8_t* rowp = p.bank;
    uint32_t gi = 0;
    auto start_tile = [&](uint32_t tt) {
        const uint32_t row = min(min(tt, p.ntiles - 1u) * 16u + r16, p.N - 1u);
        rowp = p.bank + (uint64_t)row * p.row_bytes;
        gi = 0;
    };
    auto request = [&](int slot) {
        const uint32_t sidx = s0 + 4u * min(gi, ng - 1u) + c;
        const qsk_lds_ptr dst = land + slot * (int)SB;
        const uint8_t *hp, *wp;
        if constexpr (FMT == QG_FMT_M5) {
            hp = rowp + sidx * 20u;
            wp = hp + 4;
        } else {
            hp = rowp + (uint64_t)(sidx >> p.gshift) * p.bb;
            wp = hp + 4 + (sidx & ((1u << p.gshift) - 1u)) * (4u * qg_slice_words<FMT>());
        }
        __builtin_amdgcn_global_load_lds((qsk_gptr)hp, dst, 4, 0, 0);
        __builtin_amdgcn_global_load_lds((qsk_gptr)wp, dst + 256, 16, 0, 0);
        if constexpr (FMT == QG_FMT_B8) __builtin_amdgcn_global_load_lds((qsk_gptr)(wp + 16), dst + 256 + 1024, 16, 0, 0);
        ++gi;
    };
    if (ntw) {
        start_tile(t);
#pragma unroll
        for (int d = 0; d < D; ++d) request(d);
    }

    // the activations of this K range: a thread takes 16-byte piece idx of eight activation rows at a time (eight requests
    // out before the first is parked: one memory round trip per eight pieces); rows past m and slices past a short last
    // range are zero
    {
        const uint32_t per_act = 4u * p.ks;
        const uint16_t* xs = (const uint16_t*)p.x + (uint64_t)s0 * 32u;
        for (uint32_t idx = tid; idx < per_act; idx += blockDim.x) {
            const bool live = (idx >> 2) < ks;
            uint8_t* dst = ximg + (idx >> 2) * SLB + (idx & 3u) * 16u;
#pragma unroll
            for (int m0 = 0; m0 < (int)ACTS; m0 += 8) {
                u4_t raw[8];
#pragma unroll
                for (int u = 0; u < 8; ++u) {
                    raw[u] = u4_t{0u, 0u, 0u, 0u};
                    if (live && (uint32_t)(m0 + u) < p.M) raw[u] = *(const u4_t*)(xs + (uint64_t)(m0 + u) * p.K + idx * 8u);
                }
#pragma unroll
                for (int u = 0; u < 8; ++u) *(h8_t*)(dst + (m0 + u) * 80) = qg_to_f16x8<XDT>(raw[u]);
            }
        }
    }
    __syncthreads();

    const uint32_t xrd = (uint32_t)(uintptr_t)(qsk_lds_ptr)ximg + c * SLB + (r16 & (ACTS - 1u)) * 80u;   // + 4 g * SLB + 16 j
    const uint32_t n16 = p.ntiles * 16u;
    f4_t acc0, acc1;
    // one group: take slot SLOT, request its next occupant (REFILL), contract
    auto group = [&](auto slot_c, auto newer_c, auto refill_c, uint32_t g) {
        constexpr int SLOT = decltype(slot_c)::value, NEWER = decltype(newer_c)::value;
        qg_slice<FMT> sl;
        u4_t b[4];
        qsk_take<FMT, SLOT, NEWER>(land4, land16, xrd + g * (4u * SLB), sl, b);
        if constexpr (decltype(refill_c)::value) request(SLOT);
        const h2_t s2 = qw_splat_lo(sl.hdr), b2 = qw_splat_hi(sl.hdr);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const h8_t a = qg_dequant_chunk<FMT>(sl, j, s2, b2, magic);
            if (j & 1) acc1 = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, __builtin_bit_cast(h8_t, b[j]), acc1, 0, 0, 0);
            else acc0 = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, __builtin_bit_cast(h8_t, b[j]), acc0, 0, 0, 0);
        }
    };
    for (uint32_t ti = 0; ti < ntw; ++ti, t += tstep) {
        acc0 = f4_t{0.f, 0.f, 0.f, 0.f};
        acc1 = acc0;
        const bool last_tile = ti + 1u == ntw;
        const uint32_t nfull = last_tile ? nw - 1u : nw;
        // windows whose slots are all refilled (the tile's last window from the next tile): D - 1 newer requests behind each
        for (uint32_t w = 0; w < nfull; ++w) {
            if (w + 1u == nw) start_tile(t + tstep);
            qw_static_for<D>([&](auto d) { group(d, std::integral_constant<int, D - 1>{}, std::true_type{}, w * D + decltype(d)::value); });
        }
        // the wave's last window: nothing follows, slot d has the D - 1 - d later slots behind it
        if (last_tile)
            qw_static_for<D>([&](auto d) {
                group(d, std::integral_constant<int, D - 1 - decltype(d)::value>{}, std::false_type{}, (nw - 1u) * D + decltype(d)::value);
            });
        const f4_t acc = acc0 + acc1;
        // the accumulator holds outputs (bank row 16 t + 4 c + e, activation row r16), e = 0..3
        const uint32_t rbase = t * 16u + 4u * c;
        if (p.nkr == 1u) {
            if (r16 < p.M) {
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    if (rbase + e < p.N) {
                        if (p.y32) p.y32[(uint64_t)r16 * p.N + rbase + e] = acc[e];
                        if (p.y16) p.y16[(uint64_t)r16 * p.N + rbase + e] = (h1_t)acc[e];
                    }
                }
            }
            continue;
        }
        if (r16 < p.M) *(f4_t*)(p.part + ((uint64_t)(kr * p.M + r16) * n16 + rbase)) = acc;
    }
}
};

// Second launch of a split call: y[m][row] = sum over the K ranges of the partials, in range order.
__global__ __launch_bounds__(256) void qw_gemv_sk_reduce_kernel(const float* __restrict__ part, h1_t* y16, float* y32, uint32_t N,
                                                                uint32_t M, uint32_t n16, uint32_t nkr) {
    const uint32_t q4 = blockIdx.x * 256u + threadIdx.x;   // four consecutive bank rows of one activation row
    const uint32_t per_m = n16 >> 2;
    if (q4 >= M * per_m) return;
    const uint32_t m = q4 / per_m, row = (q4 - m * per_m) * 4u;
    f4_t sum = {0.f, 0.f, 0.f, 0.f};
    for (uint32_t q0 = 0; q0 < nkr; q0 += 8u) {   // eight partials requested at a time, added in range order
        f4_t v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const uint32_t q = min(q0 + u, nkr - 1u);
            v[u] = *(const f4_t*)(part + ((uint64_t)(q * M + m) * n16 + row));
        }
#pragma unroll
        for (int u = 0; u < 8; ++u)
            if (q0 + u < nkr) sum += v[u];
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        if (row + e < N) {
            if (y32) y32[(uint64_t)m * N + row + e] = sum[e];
            if (y16) y16[(uint64_t)m * N + row + e] = (h1_t)sum[e];
        }
    }
}

template <int FMT, int XDT, int MP>
hipError_t qsk_launch(hipStream_t st, const qsk_params& p, uint32_t wgs, uint32_t threads, size_t lds, uint32_t depth) {
    // one attribute per instantiation: the image may take most of the 160 KiB of a compute unit
#define QSK_GO(DD)                                                                                                  \
    {                                                                                                               \
        using kern = qw_gemv_sk_kernel<FMT, XDT, MP, DD>;                                                           \
        static std::atomic<bool> attr_done{false};                                                                  \
        if (!attr_done.load(std::memory_order_acquire)) {                                                           \
            hipError_t e = hipFuncSetAttribute(qw_scalar_kernel_ptr<kern>((const qsk_params*)nullptr), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024); \
            if (e != hipSuccess) return e;                                                                          \
            attr_done.store(true, std::memory_order_release);                                                       \
        }                                                                                                           \
        qw_launch_scalar<kern>(dim3(wgs), dim3(threads), lds, st, p);                                               \
    }
    if (depth == 3) QSK_GO(3) else if (depth == 4) QSK_GO(4) else if (depth == 6) QSK_GO(6) else QSK_GO(2)
#undef QSK_GO
    return hipGetLastError();
}

}  // namespace

// Tries the split-K matrix-core kernel for a validated call with m = 2..16 rows already in the container's basis; false when
// the shape is outside its envelope (rows that are not whole groups of four slices, partial sums that do not fit the stream's
// scratch).  fmt: QW_FMT_M5 / QW_FMT_B4 / QW_FMT_B8 (the same codes as the GEMM's).
// `tune`: bits 0..2 groups in flight (0 = 2), bits 3..4 LDS budget (0 = 64 KiB, 1 = 32, 2 = 96, 3 = 128), bits 5..6 waves per
// workgroup (0 = 8, 1 = 4, 2 = 2).
bool qw_sk_gemv(qwhip_stream_t s, const qwhip_weight_view* w, int fmt, uint32_t gshift, uint32_t bb, uint64_t row_bytes,
                const void* x, uint32_t x_dtype, uint32_t m, void* y16, float* y32, uint32_t tune, hipError_t* err) {
    if (m < 2u || m > 16u) return false;
    if (fmt != QW_FMT_M5 && fmt != QW_FMT_B4 && fmt != QW_FMT_B8) return false;
    const uint32_t nsl = w->k / 32u;
    if (nsl % 4u != 0 || ((uintptr_t)x & 15u) != 0) return false;
    const uint32_t mp = m <= 8u ? 1u : 2u;
    const uint32_t budget_sel = (tune >> 3) & 3u;
    const uint32_t budget = (budget_sel == 1u ? 32u : budget_sel == 2u ? 96u : budget_sel == 3u ? 128u : 64u) * 1024u;
    const uint32_t slb = mp * 640u;
    const uint32_t ks_max = (budget / slb) & ~3u;
    if (ks_max < 4u) return false;
    uint32_t depth = tune & 7u;
    if (depth != 3u && depth != 4u && depth != 6u) depth = 2u;
    const uint32_t win = 4u * depth;                        // slices per window of groups in flight
    if (ks_max < win) return false;
    uint32_t nkr = qwhip_cdiv(nsl, ks_max / win * win);
    const uint32_t ks = qwhip_cdiv(qwhip_cdiv(nsl, nkr), win) * win;   // whole windows; the last range may be short
    nkr = qwhip_cdiv(nsl, ks);
    const uint32_t wsel = (tune >> 5) & 3u;
    const uint32_t waves = wsel == 1u ? 4u : (wsel == 2u ? 2u : 8u);
    const uint32_t ntiles = qwhip_cdiv(w->n, 16u);
    const uint32_t slot_bytes = fmt == QW_FMT_B8 ? qsk_slot_bytes<QG_FMT_B8>() : qsk_slot_bytes<QG_FMT_M5>();
    const size_t landing = (size_t)waves * depth * slot_bytes;   // below 64 KiB: at most 8 * 6 * 2304 bytes would not be
    if (landing > 60u * 1024u) return false;
    const size_t lds = landing + (size_t)ks * slb;
    if (lds > 160u * 1024u) return false;
    const uint32_t per_cu = max(1u, min(min(8u, 32u / waves), (uint32_t)((160u * 1024u) / (lds + 512u))));
    uint32_t bands = max(1u, 256u * per_cu / nkr);
    bands = min(bands, qwhip_cdiv(ntiles, waves));
    // partial sums live in the stream's scratch
    const uint64_t part_bytes = nkr > 1u ? (uint64_t)nkr * m * ntiles * 16u * 4u : 0u;
    if (nkr > 1u && (!s->scratch || part_bytes + s->scratch_reserved > s->scratch_bytes - QWHIP_STREAM_COUNTER_BYTES - QWHIP_STREAM_XROT_BYTES))
        return false;
    qsk_params p;
    p.bank = (const uint8_t*)w->blocks;
    p.x = x;
    p.y16 = (h1_t*)y16;
    p.y32 = y32;
    p.part = (float*)(s->scratch ? s->scratch + QWHIP_STREAM_COUNTER_BYTES : nullptr);
    p.N = w->n;
    p.K = w->k;
    p.M = m;
    p.nsl = nsl;
    p.ks = ks;
    p.nkr = nkr;
    p.bands = bands;
    p.gshift = gshift;
    p.bb = bb;
    p.ntiles = ntiles;
    p.row_bytes = row_bytes;
    const uint32_t wgs = bands * nkr, threads = 64u * waves;
    hipError_t e;
#define QSK_FMT(F)                                                                                              \
    e = x_dtype == QWHIP_F16 ? (mp == 1u ? qsk_launch<F, QWHIP_F16, 1>(s->stream, p, wgs, threads, lds, depth)  \
                                         : qsk_launch<F, QWHIP_F16, 2>(s->stream, p, wgs, threads, lds, depth)) \
                             : (mp == 1u ? qsk_launch<F, QWHIP_BF16, 1>(s->stream, p, wgs, threads, lds, depth) \
                                         : qsk_launch<F, QWHIP_BF16, 2>(s->stream, p, wgs, threads, lds, depth));
    if (fmt == QW_FMT_M5) { QSK_FMT(QG_FMT_M5) }
    else if (fmt == QW_FMT_B4) { QSK_FMT(QG_FMT_B4) }
    else { QSK_FMT(QG_FMT_B8) }
#undef QSK_FMT
    if (e == hipSuccess && nkr > 1u) {
        const uint32_t quads = m * ntiles * 4u;
        hipLaunchKernelGGL(qw_gemv_sk_reduce_kernel, dim3(qwhip_cdiv(quads, 256u)), dim3(256), 0, s->stream, p.part, p.y16, p.y32, p.N, m,
                           ntiles * 16u, nkr);
        e = hipGetLastError();
    }
    *err = e;
    return true;
}
