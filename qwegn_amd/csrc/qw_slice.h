// Slices of a quantized bank as the matrix-core kernels consume them: loading the packed words of one 32-column slice of a
// row, and dequantizing 8 consecutive columns of it to the exact f16 weights (RN_f16((1024 + q) * s + b) for HQ4_G32_M5,
// unpack_hq4_word8, Sources/QWMetal/include/qw_dequant.metalh:42-62; RN_f16(code * s + b) for the bit-stream blocks,
// qwg_aq_frag8, Sources/QWMetal/include/qw_gemm_nax.metalh:29-97).  Shared by the prefill / grouped GEMM kernels and the
// split-K verify kernel.
#pragma once
#include "qwhip_common.h"

enum { QG_FMT_M5 = 0, QG_FMT_B4 = 1, QG_FMT_B8 = 2, QG_FMT_B2 = 3, QG_FMT_B3 = 4, QG_FMT_B6 = 5 };

// code words of one 32-column slice: 32 * bits / 32
template <int FMT>
__host__ __device__ constexpr int qg_slice_words() {
    return FMT == QG_FMT_B8 ? 8 : FMT == QG_FMT_B2 ? 2 : FMT == QG_FMT_B3 ? 3 : FMT == QG_FMT_B6 ? 6 : 4;
}

struct __attribute__((packed, aligned(4))) qg_words4 { uint32_t q[4]; };
struct __attribute__((packed, aligned(4))) qg_words8 { uint32_t q[8]; };
template <int W>
struct __attribute__((packed, aligned(4))) qg_words_n { uint32_t q[W]; };

template <int FMT>
struct qg_slice {
    uint32_t hdr;
    uint32_t q[qg_slice_words<FMT>()];
};

template <int FMT>
__device__ __forceinline__ void qg_load_slice(const uint8_t* rowp, uint32_t s, uint32_t gshift, uint32_t bb, qg_slice<FMT>& o) {
    if constexpr (FMT == QG_FMT_M5) {
        const qw_hq4_block b = *(const qw_hq4_block*)(rowp + s * 20u);
        o.hdr = b.hdr;
#pragma unroll
        for (int j = 0; j < 4; ++j) o.q[j] = b.qs[j];
    } else {
        const uint8_t* p = rowp + (uint64_t)(s >> gshift) * bb;
        const uint32_t si = s & ((1u << gshift) - 1u);
        o.hdr = *(const uint32_t*)p;
        if constexpr (FMT == QG_FMT_B4) {
            const qg_words4 w = *(const qg_words4*)(p + 4 + si * 16u);
#pragma unroll
            for (int j = 0; j < 4; ++j) o.q[j] = w.q[j];
        } else if constexpr (FMT == QG_FMT_B8) {
            const qg_words8 w = *(const qg_words8*)(p + 4 + si * 32u);
#pragma unroll
            for (int j = 0; j < 8; ++j) o.q[j] = w.q[j];
        } else {
            // 2-, 3- and 6-bit streams: a slice is `bits` words, at a 4-byte aligned offset of the block
            constexpr int W = qg_slice_words<FMT>();
            const uint8_t* src = p + 4 + si * (4u * W);
            if constexpr (W == 6) {   // 24 bytes as 16 + 8: one aggregate of six words is left in scratch memory by the compiler
                const qg_words4 w0 = *(const qg_words4*)src;
                const qg_words_n<2> w1 = *(const qg_words_n<2>*)(src + 16);
#pragma unroll
                for (int j = 0; j < 4; ++j) o.q[j] = w0.q[j];
                o.q[4] = w1.q[0];
                o.q[5] = w1.q[1];
            } else {
                const qg_words_n<W> w = *(const qg_words_n<W>*)src;
#pragma unroll
                for (int j = 0; j < W; ++j) o.q[j] = w.q[j];
            }
        }
    }
}

// The same slice of a bit-stream block from its two addresses: the block's header word and the slice's code words
// (callers that keep a wave-uniform base and a fixed 32-bit lane offset for each).
template <int FMT>
__device__ __forceinline__ void qg_load_slice_at(const uint8_t* hdr_p, const uint8_t* src, qg_slice<FMT>& o) {
    static_assert(FMT != QG_FMT_M5, "bit-stream blocks");
    o.hdr = *(const uint32_t*)hdr_p;
    if constexpr (FMT == QG_FMT_B4) {
        const qg_words4 w = *(const qg_words4*)src;
#pragma unroll
        for (int j = 0; j < 4; ++j) o.q[j] = w.q[j];
    } else if constexpr (FMT == QG_FMT_B8) {
        const qg_words8 w = *(const qg_words8*)src;
#pragma unroll
        for (int j = 0; j < 8; ++j) o.q[j] = w.q[j];
    } else {
        constexpr int W = qg_slice_words<FMT>();
        if constexpr (W == 6) {
            const qg_words4 w0 = *(const qg_words4*)src;
            const qg_words_n<2> w1 = *(const qg_words_n<2>*)(src + 16);
#pragma unroll
            for (int j = 0; j < 4; ++j) o.q[j] = w0.q[j];
            o.q[4] = w1.q[0];
            o.q[5] = w1.q[1];
        } else {
            const qg_words_n<W> w = *(const qg_words_n<W>*)src;
#pragma unroll
            for (int j = 0; j < W; ++j) o.q[j] = w.q[j];
        }
    }
}

// 8 consecutive columns (chunk j of the slice) in natural order, as exact f16 weights.
template <int FMT>
__device__ __forceinline__ h8_t qg_dequant_chunk(const qg_slice<FMT>& sl, int j, h2_t s2, h2_t b2, uint32_t magic) {
    h2_t w[4];
    if constexpr (FMT == QG_FMT_M5) {
        qw_unpack_hq4_word(sl.q[j], s2, b2, magic, w);
    } else if constexpr (FMT == QG_FMT_B4) {
        // bit stream: element e of the word at bit 4e.  lo = even elements, hi = odd elements, one byte each.
        const h2_t neg = {(h1_t)-1024.0f, (h1_t)-1024.0f};
        const uint32_t lo = sl.q[j] & 0x0F0F0F0Fu;         // e0 e2 e4 e6
        const uint32_t hi = (sl.q[j] >> 4) & 0x0F0F0F0Fu;  // e1 e3 e5 e7
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            // bytes: [lo.b_k, 0, hi.b_k, 0]
            const uint32_t sel = 0x0C000C00u | (uint32_t)k | ((uint32_t)(4 + k) << 16);
            const uint32_t m = __builtin_amdgcn_perm(hi, lo, sel) | 0x64006400u;
            w[k] = __builtin_elementwise_fma(__builtin_bit_cast(h2_t, m) + neg, s2, b2);
        }
    } else if constexpr (FMT == QG_FMT_B2 || FMT == QG_FMT_B3 || FMT == QG_FMT_B6) {
        // bit stream of W-bit codes: the chunk's 8 codes are the 8 W bits from bit 8 W j of the slice.  j is a constant
        // after unrolling at every call site, so the word picks and shifts fold.
        constexpr int W = qg_slice_words<FMT>();
        const h2_t neg = {(h1_t)-1024.0f, (h1_t)-1024.0f};
        const int o = 8 * W * j, wi = o >> 5, sh = o & 31;
        // word picks as select chains over constant indices: they fold to one register for a constant j and never turn
        // into an indexed (scratch memory) access
        uint32_t lo32 = 0, hi32 = 0;
#pragma unroll
        for (int t = 0; t < W; ++t) {
            lo32 = wi == t ? sl.q[t] : lo32;
            hi32 = wi + 1 == t ? sl.q[t] : hi32;
        }
        const uint64_t lo = lo32, hi = hi32;
        const uint64_t win = (lo | (hi << 32)) >> sh;
        constexpr uint32_t mask = (1u << W) - 1u;
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const uint32_t c0 = (uint32_t)(win >> (2 * k * W)) & mask, c1 = (uint32_t)(win >> ((2 * k + 1) * W)) & mask;
            const uint32_t m = c0 | (c1 << 16) | 0x64006400u;
            w[k] = __builtin_elementwise_fma(__builtin_bit_cast(h2_t, m) + neg, s2, b2);
        }
    } else {
        const h2_t neg = {(h1_t)-1024.0f, (h1_t)-1024.0f};
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const uint32_t q = sl.q[2 * j + h];  // e0 e1 e2 e3 (bytes)
            const uint32_t m0 = __builtin_amdgcn_perm(q, q, 0x0C010C00u) | 0x64006400u;
            const uint32_t m1 = __builtin_amdgcn_perm(q, q, 0x0C030C02u) | 0x64006400u;
            w[2 * h] = __builtin_elementwise_fma(__builtin_bit_cast(h2_t, m0) + neg, s2, b2);
            w[2 * h + 1] = __builtin_elementwise_fma(__builtin_bit_cast(h2_t, m1) + neg, s2, b2);
        }
    }
    h8_t a = {w[0][0], w[0][1], w[1][0], w[1][1], w[2][0], w[2][1], w[3][0], w[3][1]};
    return a;
}

template <int XDT>
__device__ __forceinline__ h8_t qg_to_f16x8(u4_t raw) {
    if constexpr (XDT == QWHIP_F16) {
        return __builtin_bit_cast(h8_t, raw);
    } else {
        // a bf16 pair widens with one shift and one mask; v_cvt_pk_f16_f32 rounds both to f16 (to nearest even, exact for
        // every bf16 value f16 holds as a normal number)
        typedef float fl2_t __attribute__((ext_vector_type(2)));
        u4_t o;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const fl2_t v = {__uint_as_float(raw[j] << 16), __uint_as_float(raw[j] & 0xFFFF0000u)};
            o[j] = __builtin_bit_cast(uint32_t, __builtin_convertvector(v, h2_t));
        }
        return __builtin_bit_cast(h8_t, o);
    }
}

