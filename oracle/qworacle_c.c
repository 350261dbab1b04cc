/* CPU oracle, C restatement (TEST INFRASTRUCTURE ONLY - never linked into libqwhip).
 *
 * Scalar C twins of the numpy oracle for the pieces the CPU baseline times and the tests cross-check:
 *   qwo_fwht32            - Scripts/quantize/hq4.py:26-51, Sources/Foundation/QWQuant/QWQuant+DequantMath.swift:93-112
 *   qwo_quant_hq4         - Scripts/quantize/hq4.py:54-123
 *   qwo_dequant_hq4_rot   - Scripts/quantize/hq4.py:131-154 (f16_round form), QWQuant+DequantMath.swift:75-91
 *   qwo_dequant_blocks_rot- Scripts/quantize/hq_blocks.py:520-541, Sources/Foundation/QWQuant/QWAQBlock.swift:91-135
 *   qwo_oracle_gemv       - Scripts/oracle/gen_s1_q4_fixtures.py:28-31: dequantize the bank to fp32 (f16-rounded
 *                           weights), then one fp32 matrix-vector product
 * Pinned by tests/test_oracle_c.py against the numpy oracle, which is itself pinned on the reference's
 * golden fixtures (tests/test_oracle_golden.py).  All arithmetic is IEEE fp32, one operation at a time
 * (compiled with -ffp-contract=off). */
#include <math.h>
#include <stdint.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

/* threads the parallel loops below run on (reported beside the CPU baseline) */
int qwo_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

/* IEEE binary16 <-> binary32, round to nearest even, subnormals kept (gcc 11 on x86 has no _Float16). */
static inline float h2f(uint16_t h) {
    const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1Fu, man = h & 0x3FFu, bits;
    if (exp == 0) {
        if (man == 0) bits = sign;
        else {
            int e = -1;
            do { man <<= 1; ++e; } while (!(man & 0x400u));
            bits = sign | ((uint32_t)(127 - 15 - e) << 23) | ((man & 0x3FFu) << 13);
        }
    } else if (exp == 31) bits = sign | 0x7F800000u | (man << 13);
    else bits = sign | ((exp + 112u) << 23) | (man << 13);
    float f;
    memcpy(&f, &bits, 4);
    return f;
}
static inline uint16_t f2h(float f) {
    uint32_t x;
    memcpy(&x, &f, 4);
    const uint16_t sign = (uint16_t)((x >> 16) & 0x8000u);
    x &= 0x7FFFFFFFu;
    if (x >= 0x7F800000u) return (uint16_t)(sign | 0x7C00u | (x > 0x7F800000u ? 0x200u : 0u));
    if (x >= 0x477FF000u) return (uint16_t)(sign | 0x7C00u);            /* rounds to >= 65520 -> inf */
    if (x >= 0x38800000u) {                                              /* normal half */
        const uint32_t r = x - 0x38000000u;                             /* rebias exponent by -112 */
        const uint32_t rounded = r + 0xFFFu + ((r >> 13) & 1u);
        return (uint16_t)(sign | (rounded >> 13));
    }
    if (x < 0x33000000u) return sign;                                    /* < 2^-25 -> 0 (2^-25 itself ties to even 0) */
    {                                                                    /* subnormal half */
        const uint32_t e = x >> 23;
        const uint32_t m = (x & 0x7FFFFFu) | 0x800000u;
        const uint32_t shift = 126u - e;                                 /* 14..24 */
        const uint32_t halfbit = 1u << (shift - 1);
        uint32_t q = m >> shift;
        const uint32_t rem = m & ((1u << shift) - 1u);
        if (rem > halfbit || (rem == halfbit && (q & 1u))) ++q;
        return (uint16_t)(sign | q);
    }
}

void qwo_fwht32(float* p) {
    for (int h = 1; h < 32; h <<= 1)
        for (int i0 = 0; i0 < 32; i0 += 2 * h)
            for (int j = 0; j < h; ++j) {
                const float u = p[i0 + j], v = p[i0 + j + h];
                p[i0 + j] = u + v;
                p[i0 + j + h] = u - v;
            }
    const float s = 0.17677669529663689f;
    for (int i = 0; i < 32; ++i) p[i] = p[i] * s;
}

/* w [n, k] f32 -> blocks [n, k/32, 20] */
void qwo_quant_hq4(const float* w, int64_t n, int64_t k, int rotate, uint8_t* out) {
    const int64_t groups = n * (k / 32);
#pragma omp parallel for
    for (int64_t g = 0; g < groups; ++g) {
        float v[32];
        memcpy(v, w + g * 32, sizeof(v));
        if (rotate) qwo_fwht32(v);
        float amax = 0.0f;
        for (int i = 0; i < 32; ++i) amax = fmaxf(amax, fabsf(v[i]));
        const uint16_t s16 = f2h(fminf(amax / 7.5f, 63.46875f));
        const float s = h2f(s16);
        const uint16_t b16 = f2h(-1032.0f * s);
        const float b = h2f(b16);
        uint32_t q[32];
        for (int i = 0; i < 32; ++i) {
            if (s > 0.0f) {
                float t = floorf((v[i] - b) / s - 1023.5f);
                t = t < 0.0f ? 0.0f : (t > 15.0f ? 15.0f : t);
                q[i] = (uint32_t)t;
            } else q[i] = 8u;
        }
        uint8_t* o = out + g * 20;
        memcpy(o, &s16, 2);
        memcpy(o + 2, &b16, 2);
        for (int wd = 0; wd < 4; ++wd) {
            const uint32_t* e = q + 8 * wd;
            const uint32_t word = e[0] | (e[1] << 16) | (e[2] << 4) | (e[3] << 20) | (e[4] << 8) | (e[5] << 24) | (e[6] << 12) | (e[7] << 28);
            memcpy(o + 4 + 4 * wd, &word, 4);
        }
    }
}

/* blocks [n, k/32, 20] -> rotated-domain fp32 weights [n, k]; f16_round != 0 rounds each weight through f16 */
void qwo_dequant_hq4_rot(const uint8_t* blocks, int64_t n, int64_t k, int f16_round, float* out) {
    const int64_t groups = n * (k / 32);
    static const int sh[8] = {0, 16, 4, 20, 8, 24, 12, 28};
#pragma omp parallel for
    for (int64_t g = 0; g < groups; ++g) {
        const uint8_t* p = blocks + g * 20;
        uint16_t s16, b16;
        memcpy(&s16, p, 2);
        memcpy(&b16, p + 2, 2);
        const float s = h2f(s16), b = h2f(b16);
        for (int wd = 0; wd < 4; ++wd) {
            uint32_t word;
            memcpy(&word, p + 4 + 4 * wd, 4);
            for (int e = 0; e < 8; ++e) {
                const float q = (float)((word >> sh[e]) & 0xFu);
                float wv = (q + 1024.0f) * s;
                wv = wv + b;
                if (f16_round) wv = h2f(f2h(wv));
                out[g * 32 + 8 * wd + e] = wv;
            }
        }
    }
}

/* bit-stream blocks [n, k/group, 4 + group*bits/8] -> block-domain fp32 weights [n, k] */
void qwo_dequant_blocks_rot(const uint8_t* blocks, int64_t n, int64_t k, int bits, int group, int f16_round, float* out) {
    const int64_t nb = n * (k / group);
    const int bb = 4 + group * bits / 8;
#pragma omp parallel for
    for (int64_t g = 0; g < nb; ++g) {
        const uint8_t* p = blocks + g * bb;
        uint16_t s16, b16;
        memcpy(&s16, p, 2);
        memcpy(&b16, p + 2, 2);
        const float s = h2f(s16), b = h2f(b16);
        const uint8_t* pay = p + 4;
        for (int i = 0; i < group; ++i) {
            const int bit = i * bits, byte = bit >> 3, off = bit & 7;
            uint32_t v = (uint32_t)pay[byte] >> off;
            if (8 - off < bits) v |= (uint32_t)pay[byte + 1] << (8 - off);
            v &= (1u << bits) - 1u;
            float wv = (float)v * s;
            wv = wv + b;
            if (f16_round) wv = h2f(f2h(wv));
            out[g * group + i] = wv;
        }
    }
}

/* y[n] = sum_k wq[n, k] * x[k] in fp32, rows in parallel, serial accumulation inside a row */
void qwo_sgemv(const float* wq, const float* x, int64_t n, int64_t k, float* y) {
#pragma omp parallel for
    for (int64_t r = 0; r < n; ++r) {
        float acc = 0.0f;
        const float* w = wq + r * k;
        for (int64_t c = 0; c < k; ++c) acc += w[c] * x[c];
        y[r] = acc;
    }
}

/* The reference's CPU oracle form for HQ4_G32_M5: dequant the whole bank (scratch [n, k] fp32), then sgemv. */
void qwo_oracle_gemv_hq4(const uint8_t* blocks, const uint16_t* x_rot_f16, int64_t n, int64_t k, float* scratch, float* xf,
                         float* y) {
    qwo_dequant_hq4_rot(blocks, n, k, 1, scratch);
    for (int64_t c = 0; c < k; ++c) xf[c] = h2f(x_rot_f16[c]);
    qwo_sgemv(scratch, xf, n, k, y);
}

/* Same form for a bit-stream container (scratch [n, k] fp32, xf [k] fp32). */
void qwo_oracle_gemv_blocks(const uint8_t* blocks, const uint16_t* x_f16, int64_t n, int64_t k, int bits, int group,
                            float* scratch, float* xf, float* y) {
    qwo_dequant_blocks_rot(blocks, n, k, bits, group, 1, scratch);
    for (int64_t c = 0; c < k; ++c) xf[c] = h2f(x_f16[c]);
    qwo_sgemv(scratch, xf, n, k, y);
}
