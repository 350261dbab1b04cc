// Top-k routing of one token row by one wavefront (all 64 lanes active): lane l holds experts l, l + 64, ... (E <= 64 JN).
// fp32 softmax (max-subtracted), top_k rounds of argmax with ties to the lower index, optional renormalisation by the sum
// of the selected, times the routed scale; non-finite logits never win.  On return lane r < K holds rank r's expert
// (-1: none) and weight.
#pragma once
#include "qwhip_common.h"

__device__ __forceinline__ bool qw_finite(float v) { return (__float_as_uint(v) & 0x7F800000u) != 0x7F800000u; }

// Wave-wide maximum / sum, uniform result: four DPP steps inside each row of 16 lanes, then four lane reads.
#define QW_DPP_F32(v, ctrl) __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), ctrl, 0xF, 0xF, true))
#define QW_LANE_F32(v, l) __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), l))
__device__ __forceinline__ float qw_wave_max(float v) {
    v = fmaxf(v, QW_DPP_F32(v, 0xB1));
    v = fmaxf(v, QW_DPP_F32(v, 0x4E));
    v = fmaxf(v, QW_DPP_F32(v, 0x141));
    v = fmaxf(v, QW_DPP_F32(v, 0x140));
    return fmaxf(fmaxf(QW_LANE_F32(v, 0), QW_LANE_F32(v, 16)), fmaxf(QW_LANE_F32(v, 32), QW_LANE_F32(v, 48)));
}
__device__ __forceinline__ float qw_wave_sum(float v) {
    v += QW_DPP_F32(v, 0xB1);
    v += QW_DPP_F32(v, 0x4E);
    v += QW_DPP_F32(v, 0x141);
    v += QW_DPP_F32(v, 0x140);
    return (QW_LANE_F32(v, 0) + QW_LANE_F32(v, 16)) + (QW_LANE_F32(v, 32) + QW_LANE_F32(v, 48));
}

template <int JN>   // experts per lane: E <= 64 * JN
__device__ __forceinline__ void qw_route_wave(const float* __restrict__ row, uint32_t E, uint32_t K, uint32_t norm, float routed_scale,
                                              uint32_t lane, int32_t& isel_out, float& w_out) {
    float p[JN];
    bool ok[JN];
    float mx = -3.4e38f;
    bool any_finite = false;
#pragma unroll
    for (uint32_t j = 0; j < JN; ++j) {
        const uint32_t id = lane + 64u * j;
        float v = 0.0f;
        ok[j] = false;
        if (id < E) {
            v = row[id];
            ok[j] = qw_finite(v);
            if (ok[j]) {
                mx = any_finite ? fmaxf(mx, v) : v;
                any_finite = true;
            }
        }
        p[j] = v;
    }
    mx = qw_wave_max(mx);
    float total = 0.0f;
#pragma unroll
    for (uint32_t j = 0; j < JN; ++j) {
        p[j] = ok[j] ? expf(p[j] - mx) : 0.0f;
        total += p[j];
    }
    total = qw_wave_sum(total);
#pragma unroll
    for (uint32_t j = 0; j < JN; ++j) {
        ok[j] = ok[j] && total > 0.0f;
        p[j] = ok[j] ? p[j] / total : -1e30f;
    }
    // Selection rounds on the scalar unit: the wave maximum comes from four DPP steps inside each row of 16 lanes and
    // four lane reads, the owner of the maximum from ballots in ascending expert order (ties go to the lower id).
    // Cross-lane permutes through LDS would put two dependent ~100-clock round trips on every one of the 6 x top_k steps.
    float cand[JN];
#pragma unroll
    for (uint32_t j = 0; j < JN; ++j) cand[j] = ok[j] ? p[j] : -1.0f;   // probabilities are >= 0
    float wsel = 0.0f;  // lane r keeps the weight of rank r (K <= 16 < 64)
    int32_t isel = -1;
    for (uint32_t r = 0; r < K; ++r) {
        float lm = cand[0];
#pragma unroll
        for (uint32_t j = 1; j < JN; ++j) lm = fmaxf(lm, cand[j]);
        const float wm = qw_wave_max(lm);
        uint32_t bi = 0xFFFFFFFFu;
        if (wm >= 0.0f) {
#pragma unroll
            for (uint32_t j = 0; j < JN; ++j) {
                const unsigned long long m = __ballot(cand[j] == wm);
                if (bi == 0xFFFFFFFFu && m != 0ull) bi = 64u * j + (uint32_t)__builtin_ctzll(m);
            }
        }
        if (bi != 0xFFFFFFFFu && (bi & 63u) == lane) {
#pragma unroll
            for (uint32_t j = 0; j < JN; ++j)
                if (j == (bi >> 6)) cand[j] = -1.0f;
        }
        if (lane == r) {
            wsel = bi != 0xFFFFFFFFu ? wm : 0.0f;
            isel = bi != 0xFFFFFFFFu ? (int32_t)bi : -1;
        }
    }
    // sum of the selected in rank order (lane 0 .. K-1), as the reference's serial loop
    float acc = 0.0f;
#pragma unroll
    for (uint32_t r = 0; r < 16; ++r)
        if (r < K) acc += __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, wsel), r));
    float w = wsel;
    if (norm) w = acc > 0.0f ? w / acc : 0.0f;
    isel_out = isel;
    w_out = w * routed_scale;
}

// Sigmoid scoring of the same routine (the reference's selection-bias and split-feature modes,
// Sources/QWMetal/subsystems/qwrouter.metal:63-82,113-159): score = sigmoid(l) (+ sigmoid(l') of the row's second half with
// split features), experts are selected by score + bias (ties to the lower index), the weight of a selected expert is its
// score without the bias, renormalised by the sum of the selected + 1e-20.  The caller applies the routed scale.
template <int JN>
__device__ __forceinline__ void qw_route_wave_sigmoid(const float* __restrict__ row, uint32_t E, uint32_t K, uint32_t norm, bool split,
                                                      const float* __restrict__ bias, uint32_t lane, int32_t& isel_out, float& w_out) {
    constexpr float NONE = -3.4e38f;
    float ex[JN], cand[JN];
#pragma unroll
    for (uint32_t j = 0; j < JN; ++j) {
        const uint32_t id = lane + 64u * j;
        ex[j] = 0.0f;
        cand[j] = NONE;
        if (id < E) {
            const float l0 = row[id];
            float sc = 1.0f / (1.0f + expf(-l0));
            bool okv = qw_finite(l0);
            if (split) {
                const float l1 = row[E + id];
                sc += 1.0f / (1.0f + expf(-l1));
                okv = okv && qw_finite(l1);
            }
            const float score = bias ? sc + bias[id] : sc;
            okv = okv && qw_finite(sc) && qw_finite(score);
            ex[j] = sc;
            if (okv) cand[j] = score;
        }
    }
    float wsel = 0.0f;
    int32_t isel = -1;
    for (uint32_t r = 0; r < K; ++r) {
        float lm = cand[0];
#pragma unroll
        for (uint32_t j = 1; j < JN; ++j) lm = fmaxf(lm, cand[j]);
        const float wm = qw_wave_max(lm);
        uint32_t bi = 0xFFFFFFFFu;
        if (wm > NONE) {
#pragma unroll
            for (uint32_t j = 0; j < JN; ++j) {
                const unsigned long long m = __ballot(cand[j] == wm);
                if (bi == 0xFFFFFFFFu && m != 0ull) bi = 64u * j + (uint32_t)__builtin_ctzll(m);
            }
        }
        bi = __builtin_amdgcn_readfirstlane(bi);
        float own = 0.0f;
        if (bi != 0xFFFFFFFFu && (bi & 63u) == lane) {
#pragma unroll
            for (uint32_t j = 0; j < JN; ++j)
                if (j == (bi >> 6)) {
                    own = ex[j];
                    cand[j] = NONE;
                }
        }
        const float pw = bi != 0xFFFFFFFFu ? QW_LANE_F32(own, bi & 63u) : 0.0f;
        if (lane == r) {
            wsel = pw;
            isel = bi != 0xFFFFFFFFu ? (int32_t)bi : -1;
        }
    }
    float acc = 0.0f;
#pragma unroll
    for (uint32_t r = 0; r < 16; ++r)
        if (r < K) acc += __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, wsel), r));
    float w = wsel;
    if (norm) {
        acc += 1e-20f;
        w = acc > 0.0f ? w / acc : 0.0f;
    }
    isel_out = isel;
    w_out = w;
}
