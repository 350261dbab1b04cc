// MoE decode (a handful of tokens) over HQ4_G32_M5 expert banks, column-stationary form.
//
// Both routed projections of the decode path (encodeMoEGateUpF32R1 / encodeMoEDownSharedCombineF32,
// Sources/Operators/QWGEMM/QWGemmMoE.swift:120-199) read a few short rows from each routed expert: the launch is
// latency bound, so what matters is that every byte is requested at once, by loads whose lanes read consecutive
// blocks.  A lane owns one block column for the whole kernel, keeps its 32 activations in registers as 16 f16 pairs
// and contracts the masked nibble pairs directly as f16 subnormal operands of v_dot2_f32_f16:
//     sum_i w_i x_i = s * (sum_i q_i x_i + 1024 S) + b * S,   S = sum_i x_i      (w = (1024 + q) s + b,
// unpack_hq4_word8, Sources/QWMetal/include/qw_dequant.metalh:42-62).  A half-wavefront covers 32 block columns of a
// row and reduces with DPP; the per-chunk partial sums meet in LDS and are added in chunk order.
#include "qwhip_common.h"
#include "qwhip_route.h"

namespace {

// 16 operand pairs and their sum from the 32 activations v[0..3] of one block column.
__device__ __forceinline__ float qmc_operands(const h8_t* v, h2_t* xo) {
    const h2_t one = {(h1_t)1.0f, (h1_t)1.0f};
    float s0 = 0.f, s1 = 0.f;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
#pragma unroll
        for (int e2 = 0; e2 < 4; ++e2) {
            const h2_t pr = {v[j][2 * e2], v[j][2 * e2 + 1]};
            if (e2 & 1) s1 = __builtin_amdgcn_fdot2(pr, one, s1, false);
            else s0 = __builtin_amdgcn_fdot2(pr, one, s0, false);
            xo[4 * j + e2] = pr;
        }
    }
    return s0 + s1;
}

// One block against the lane's operands: s * (sum q x + 1024 S) + b * S.
__device__ __forceinline__ float qmc_block_dot(const qw_hq4_block& b, const h2_t* xo, float S, float c1) {
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
    const h2_t hd = __builtin_bit_cast(h2_t, b.hdr);
    float q = __builtin_fmaf(lo0 + lo1, 16777216.0f, c1);   // the low nibbles read as q * 2^-24, the high ones as 16 q * 2^-24
    q = __builtin_fmaf(hi0 + hi1, 1048576.0f, q);
    return __builtin_fmaf((float)hd[0], q, (float)hd[1] * S);
}

// ------------------------------------------------------------------------------------------------
// gate|up: grid (ceil(I / 32), pairs).  A workgroup owns 32 gate rows and the 32 matching up rows of the pair's expert
// (row slot s: up = s >> 5, n = n0 + (s & 31)); set j of SETS takes slots j * R .. j * R + R - 1, R = 64 / SETS.
// Epilogue: act[pair, n] = f16(FWHT32(silu(g) * u)) over the 32 outputs of the workgroup (rotation optional).
// blockDim.x = 32 * cpr * SETS; dynamic LDS = nb * 80 + 64 * cpr * 4 bytes.
// ------------------------------------------------------------------------------------------------
// logits, idx_out, wts_out, experts, norm, routed_scale (JN > 0): the routing is done here.  The first wave of every workgroup
// routes the pair's token from its router logits (the arithmetic of qw_moe_route_kernel, so the same experts and weights) and
// the workgroup takes rank pair % top_k; the workgroups of the first row block leave the pair's expert and weight in idx_out /
// wts_out for the down projection.  x_rows: activation row of every pair (NULL: the pair's token).  ga: the device's gated
// activation (all zero: SwiGLU).
#define QMC_GU_FIELDS(X)                                                                                                     \
    X(const uint8_t*, bank) X(const void*, x) X(h1_t*, act) X(const int32_t*, idx) X(const float*, logits) X(uint32_t, top_k)    \
    X(uint32_t, nb) X(uint32_t, cpr) X(uint32_t, I) X(uint32_t, rotate) X(uint32_t, rot_out) X(uint64_t, expert_bytes)           \
    X(const int32_t*, x_rows) X(uint32_t, experts) X(int32_t*, idx_out) X(float*, wts_out) X(uint32_t, norm)                     \
    X(float, routed_scale) X(qw_act, ga)
QW_ARG_BLOCK(qmc_gu_params, QMC_GU_FIELDS)

// MT > 1 (a verify window of 2 .. MT tokens, at most 64 pairs): an expert that several tokens route to is read once
// (reuseExpertsAcrossTokens of encodeMoEGateUpF32R1, Sources/Operators/QWGEMM/QWGemmMoE.swift:119-132; the leader / follower scan of
// Sources/QWMetal/include/qw_moe_f32_common.metalh:213-232).  A pair is primary when it is its token's first route to its
// expert; a primary pair whose expert an earlier token also routes to leaves (that token's workgroup computes it); the
// first token's primary pair gathers the primary pairs of the later tokens and runs every row block against all of their
// activation rows.  A token's second route to one expert runs alone.  Every pair's outputs come from the same operations
// in the same order as in a launch of its own.  Dynamic LDS = MT * (nb * 80 + 64 * cpr * 4) bytes, blockDim.x <= 512.
template <int XDT, int SETS, int JN = 0, int MT = 1>
struct qw_moe_gateup_col_kernel {
static constexpr int kLaunchBound = MT > 1 ? 512 : 1024;
static __device__ __forceinline__ void run(const qmc_gu_params& p) {
    constexpr int R = 64 / SETS;
    constexpr int D = R < 8 ? R : 8;             // rows in flight per lane
    constexpr int XT = SETS == 2 ? 2 : 1;        // 16-group activation tiles per wave: ceil(2 cpr / (cpr * SETS / 2))
    extern __shared__ h8_t qmc_lds[];
    const uint32_t nb = p.nb, cpr = p.cpr, I = p.I;
    h8_t* xs = qmc_lds;                                       // [MT][nb] groups of 80 bytes
    float* part = (float*)(qmc_lds + (size_t)MT * nb * 5);   // [MT][64 row slots][cpr]
    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & 31u, hw = tid >> 5;
    const uint32_t wave = tid >> 6, l64 = tid & 63u;
    const uint32_t nw = blockDim.x >> 6;
    const uint32_t set = hw / cpr, chunk = hw - set * cpr;
    const uint32_t g0 = chunk * 32u + lane;
    const bool gvalid = g0 < nb;
    const uint32_t g = gvalid ? g0 : nb - 1u;
    const uint32_t pair = blockIdx.y, n0 = blockIdx.x * 32u;
    const uint32_t row_bytes = nb * 20u;

    // memory order: the route's expert id, the token's activations, the first weight rows; the rotation runs under them
    int32_t e = 0;                               // no route list: one dense gate|up bank
    if constexpr (JN == 0 && MT == 1) e = p.idx ? p.idx[pair] : 0;
    const uint32_t token = pair / p.top_k;
    uint32_t xrow = token;
    if constexpr (MT == 1) xrow = (JN == 0 && p.x_rows) ? (uint32_t)max(p.x_rows[pair], 0) : token;
    h8_t xv[MT][XT];
    if constexpr (MT == 1) {
        const uint8_t* x = (const uint8_t*)p.x + (uint64_t)xrow * nb * 64u;
#pragma unroll
        for (int t = 0; t < XT; ++t) {
            const uint32_t gg = min((wave + nw * t) * 16u + (l64 & 15u), nb - 1u);
            xv[0][t] = qw_load_x8_f16<XDT>(x, (uint64_t)gg * 32u + 8u * (l64 >> 4));
        }
    }
    __builtin_amdgcn_sched_barrier(0);
    uint32_t mcount = 1u;
    uint32_t slot[MT];
#pragma unroll
    for (int m = 0; m < MT; ++m) slot[m] = pair;
    if constexpr (MT > 1) {
        // the window's route table: lane l holds pair l's expert (and activation row)
        __shared__ int32_t tab_e[64];
        __shared__ float tab_w[64];
        const uint32_t pairs = gridDim.y, K = p.top_k, ntok = pairs / K;   // pairs <= 64, 2 <= ntok <= MT
        int32_t my_e = -1;
        if constexpr (JN > 0) {
            if (wave < ntok) {   // one wave per token routes it
                int32_t isel;
                float wsel;
                qw_route_wave<JN>(p.logits + (uint64_t)wave * p.experts, p.experts, K, p.norm, p.routed_scale, l64, isel, wsel);
                if (l64 < K) {
                    tab_e[wave * K + l64] = isel;
                    tab_w[wave * K + l64] = wsel;
                }
            }
            __syncthreads();
            if (l64 < pairs) my_e = tab_e[l64];
            if (blockIdx.x == 0 && tid == 0) {
                p.idx_out[pair] = tab_e[pair];
                p.wts_out[pair] = tab_w[pair];
            }
        } else {
            if (l64 < pairs) my_e = p.idx[l64];
        }
        uint32_t my_row = l64 / K;
        if constexpr (JN == 0) {
            if (p.x_rows && l64 < pairs) my_row = (uint32_t)max(p.x_rows[l64], 0);
        }
        e = __builtin_amdgcn_readlane(my_e, pair);
        if (e >= 0) {
            const unsigned long long match = __ballot(my_e == e);   // lanes past the table hold -1
            const uint32_t kmask = (1u << K) - 1u, rank = pair - token * K;
            const uint32_t own = (uint32_t)(match >> (token * K)) & kmask;
            if ((uint32_t)__builtin_ctz(own) == rank) {             // primary: the token's first route to this expert
                for (uint32_t t2 = 0; t2 < token; ++t2)
                    if (((uint32_t)(match >> (t2 * K)) & kmask) != 0u) return;   // an earlier token's workgroup computes this pair
                for (uint32_t t2 = token + 1u; t2 < ntok; ++t2) {
                    const uint32_t mt = (uint32_t)(match >> (t2 * K)) & kmask;
                    if (mt != 0u && mcount < (uint32_t)MT) {
                        const uint32_t sl = t2 * K + (uint32_t)__builtin_ctz(mt);
#pragma unroll
                        for (int m = 1; m < MT; ++m)
                            if ((uint32_t)m == mcount) slot[m] = sl;
                        ++mcount;
                    }
                }
            }
        }
        // every slot's activation row is loaded (a spare slot repeats the pair's own row) so that no load sits under a branch
#pragma unroll
        for (int m = 0; m < MT; ++m) {
            const uint32_t xr = (uint32_t)__builtin_amdgcn_readlane((int)my_row, slot[m]);
            const uint8_t* x = (const uint8_t*)p.x + (uint64_t)xr * nb * 64u;
#pragma unroll
            for (int t = 0; t < XT; ++t) {
                const uint32_t gg = min((wave + nw * t) * 16u + (l64 & 15u), nb - 1u);
                xv[m][t] = qw_load_x8_f16<XDT>(x, (uint64_t)gg * 32u + 8u * (l64 >> 4));
            }
        }
    }
    if constexpr (JN > 0 && MT == 1) {
        __shared__ int32_t e_route;
        if (wave == 0) {   // one wave routes (the others would only compete for the same SIMDs), the workgroup reads its result
            int32_t isel;
            float wsel;
            qw_route_wave<JN>(p.logits + (uint64_t)token * p.experts, p.experts, p.top_k, p.norm, p.routed_scale, l64, isel, wsel);
            const uint32_t rank = pair - token * p.top_k;
            if (l64 == rank) {
                e_route = isel;
                if (blockIdx.x == 0) {
                    p.idx_out[pair] = isel;
                    p.wts_out[pair] = wsel;
                }
            }
        }
        __syncthreads();
        e = e_route;
    }
    h1_t* act = p.act + (uint64_t)pair * I;
    if (e < 0) {   // no expert: the pair contributes nothing (uniform over the workgroup)
        if (tid < 32u && n0 + tid < I) act[n0 + tid] = (h1_t)0.0f;
        return;
    }
    const uint8_t* bank = p.bank + (uint64_t)((uint32_t)e & 0xFFFFu) * p.expert_bytes;
    auto row_off = [&](uint32_t r) {   // r-th row of this set
        const uint32_t s = set * R + min(r, (uint32_t)R - 1u);
        const uint32_t n = min(n0 + (s & 31u), I - 1u);
        return ((s >> 5) * I + n) * row_bytes + g * 20u;
    };
    qw_hq4_block buf[D];
#pragma unroll
    for (int j = 0; j < D; ++j) buf[j] = *(const qw_hq4_block*)(bank + row_off(j));
    __builtin_amdgcn_sched_barrier(0);
    {
        h8_t h_lo, h_hi;
        qw_hadamard_pair(l64 & 15u, l64 >> 4, h_lo, h_hi);
#pragma unroll
        for (int m = 0; m < MT; ++m)
#pragma unroll
            for (int t = 0; t < XT; ++t)
                qw_rotate_tile_to_lds(xv[m][t], wave + nw * t, nb, l64, p.rotate != 0, h_lo, h_hi, xs + (size_t)m * nb * 5);
    }
    __syncthreads();
    // The lane's blocks stay in registers while the slots pass over them: slot 0 consumes each block as it lands, the
    // further slots of a shared expert take their operands from LDS one after the other.
    h2_t xo[16];
    const float S = qmc_operands(xs + g * 5, xo);
    const float c1 = 1024.0f * S;
#pragma unroll
    for (int r0 = 0; r0 < R; r0 += D) {
        qw_hq4_block blk[D];
#pragma unroll
        for (int j = 0; j < D; ++j) {
            blk[j] = buf[j];
            if (r0 + D + j < R) buf[j] = *(const qw_hq4_block*)(bank + row_off(r0 + D + j));
            float v = qmc_block_dot(blk[j], xo, S, c1);
            v = gvalid ? v : 0.0f;
            v = qw_reduce32_dpp(v);
            if (lane == 31u) part[(set * R + r0 + j) * cpr + chunk] = v;
        }
        if constexpr (MT > 1) {
            for (uint32_t m = 1; m < mcount; ++m) {
                h2_t xm[16];
                const float Sm = qmc_operands(xs + ((size_t)m * nb + g) * 5, xm);
                const float cm = 1024.0f * Sm;
#pragma unroll
                for (int j = 0; j < D; ++j) {
                    // the nibble masks are formed again for every slot: hoisted out of this loop they would occupy
                    // 16 registers per block for the whole kernel
                    qw_hq4_block b = blk[j];
                    asm volatile("" : "+v"(b.qs[0]), "+v"(b.qs[1]), "+v"(b.qs[2]), "+v"(b.qs[3]));
                    float v = qmc_block_dot(b, xm, Sm, cm);
                    v = gvalid ? v : 0.0f;
                    v = qw_reduce32_dpp(v);
                    if (lane == 31u) part[(m * 64u + set * R + r0 + j) * cpr + chunk] = v;
                }
            }
        }
    }
    __syncthreads();
    if (wave < mcount) {
        // a whole wave runs a slot's transform (its upper half repeats the lower half's outputs: the cross-row exchange
        // wants every row of the wave live); the lower half stores
        const uint32_t o32 = l64 & 31u;
        const float* pm = part + (size_t)wave * 64u * cpr;
        float gsum = 0.f, usum = 0.f;
        for (uint32_t c = 0; c < cpr; ++c) {
            gsum += pm[o32 * cpr + c];
            usum += pm[(32u + o32) * cpr + c];
        }
        float a = qw_gated(gsum, usum, p.ga);
        // the butterfly order of the serial transform (pairs h apart: lower = a + b, upper = a - b), across lanes by DPP
        if (p.rot_out && n0 + 32u <= I) a = qw_fwht32_lanes(a, qw_fwht32_lane_signs(o32)) * QW_INV_SQRT32;
        uint32_t sl = slot[0];
#pragma unroll
        for (int m = 1; m < MT; ++m)
            if ((uint32_t)m == wave) sl = slot[m];
        if (l64 < 32u && n0 + l64 < I) p.act[(uint64_t)sl * I + n0 + l64] = (h1_t)a;
    }
}
};

// ------------------------------------------------------------------------------------------------
// down + combine: grid (ceil(H / (SETS * D)), tokens).  The token's routes are laid side by side as one virtual row of
// top_k * nbI blocks: virtual block v belongs to route k = v / nbI, block b = v % nbI of that expert's row, so a lane's
// column fixes its expert, its 32 activations (act[token, k, 32 b ..]) and its route weight.
//   out[token, n] = sum_k wts[k] * (W_down[e_k][n, :] . act[k, :]) (+ shared_gate * shared[n])
// blockDim.x = 32 * cprv * SETS, cprv = ceil(top_k * nbI / 32); set j takes rows n0 + j * D .. + D - 1.
// ------------------------------------------------------------------------------------------------
// labels, num_groups > 0: blockIdx.y = token * num_groups + group, and only the token's routes whose expert carries that
// group's label are summed.  x_div: pairs that share one activation row (1: a row per pair).
#define QMC_DN_FIELDS(X)                                                                                                     \
    X(const uint8_t*, bank) X(const h1_t*, act) X(const int32_t*, idx) X(const float*, wts) X(void*, out) X(uint32_t, top_k)     \
    X(uint32_t, nbI) X(uint32_t, nbv) X(uint32_t, cprv) X(uint32_t, H) X(uint32_t, sets) X(uint64_t, expert_bytes)               \
    X(const float*, shared) X(const float*, shared_gate) X(const int32_t*, labels) X(uint32_t, num_groups) X(uint32_t, x_div)
QW_ARG_BLOCK(qmc_dn_params, QMC_DN_FIELDS)

template <int ODT, int D, bool GRP = false>   // GRP: one output row per (token, latent group)
struct qw_moe_down_col_kernel {
static constexpr int kLaunchBound = 1024;
static __device__ __forceinline__ void run(const qmc_dn_params& p) {
    __shared__ float part[1024];   // [sets * D rows][cprv]
    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & 31u, hw = tid >> 5;
    const uint32_t cprv = p.cprv, H = p.H;
    const uint32_t set = hw / cprv, chunk = hw - set * cprv;
    const uint32_t tok = blockIdx.y, n0 = blockIdx.x * (p.sets * D);   // tok: the output row
    // group mode: num_groups carries the group count in its low byte and the expert count (the length of labels) above it
    const uint32_t ng = p.num_groups & 0xFFu, n_experts = p.num_groups >> 8;
    const uint32_t src = GRP ? tok / ng : tok;
    const int32_t grp = GRP ? (int32_t)(tok - src * ng) : 0;
    const uint32_t v0 = chunk * 32u + lane;
    const bool vvalid = v0 < p.nbv;
    const uint32_t v = vvalid ? v0 : 0u;
    const uint32_t k = v / p.nbI, b = v - k * p.nbI;
    const uint32_t pair = src * p.top_k + k;
    const int32_t e = p.idx[pair];
    const float wk = p.wts ? p.wts[pair] : 1.0f;
    bool valid = vvalid && e >= 0;
    if constexpr (GRP) {
        valid = valid && ((uint32_t)e & 0xFFFFu) < n_experts;       // an id past the labels is no route
        valid = valid && p.labels[valid ? ((uint32_t)e & 0xFFFFu) : 0u] == grp;
    }
    const uint32_t row_bytes = p.nbI * 20u;
    // activations do not wait for the expert id; the weight rows follow as soon as it is known
    h8_t xr[4];
    const h8_t* xsrc = (const h8_t*)(p.act + ((uint64_t)(p.x_div > 1u ? pair / p.x_div : pair) * p.nbI + b) * 32u);
#pragma unroll
    for (int j = 0; j < 4; ++j) xr[j] = xsrc[j];
    const uint8_t* base = p.bank + (uint64_t)(valid ? ((uint32_t)e & 0xFFFFu) : 0u) * p.expert_bytes + b * 20u;
    qw_hq4_block buf[D];
#pragma unroll
    for (int j = 0; j < D; ++j) {
        const uint32_t n = min(n0 + set * D + j, H - 1u);
        if constexpr (GRP) {   // lanes of other groups' routes read nothing
            buf[j] = qw_hq4_block{};
            if (valid) buf[j] = *(const qw_hq4_block*)(base + (uint64_t)n * row_bytes);
        } else {
            buf[j] = *(const qw_hq4_block*)(base + (uint64_t)n * row_bytes);
        }
    }
    h2_t xo[16];
    const float S = qmc_operands(xr, xo);
    const float c1 = 1024.0f * S;
#pragma unroll
    for (int j = 0; j < D; ++j) {
        float r = qmc_block_dot(buf[j], xo, S, c1) * wk;
        r = valid ? r : 0.0f;
        r = qw_reduce32_dpp(r);
        if (lane == 31u) part[(set * D + j) * cprv + chunk] = r;
    }
    __syncthreads();
    if (tid < p.sets * D) {
        const uint32_t n = n0 + tid;
        if (n < H) {
            float o = 0.f;
            for (uint32_t c = 0; c < cprv; ++c) o += part[tid * cprv + c];
            const uint64_t at = (uint64_t)tok * H + n;
            if (p.shared) o = fmaf(p.shared_gate ? p.shared_gate[tok] : 1.0f, p.shared[at], o);
            if constexpr (ODT == QWHIP_F32) ((float*)p.out)[at] = o;
            else if constexpr (ODT == QWHIP_F16) ((h1_t*)p.out)[at] = (h1_t)o;
            else ((uint16_t*)p.out)[at] = qw_f32_to_bf16(o);
        }
    }
}
};

}  // namespace

// Routed gate|up projection with the SwiGLU (+ rotation) epilogue for a validated HQ4_G32_M5 bank; false when the shape
// is outside the kernel's envelope (the caller then takes the general kernel).
bool qw_moe_gateup_col(hipStream_t st, const qwhip_weight_view* w, uint32_t experts, const void* x, uint32_t x_dtype, bool rotate,
                       bool rot_out, const int32_t* idx, uint32_t pairs, uint32_t top_k, void* act16, hipError_t* err,
                       const qw_act act, const float* logits, int32_t* idx_out, float* wts_out, uint32_t norm_topk, float routed_scale,
                       const int32_t* x_rows, uint32_t reuse_tokens) {
    if (w->kind != QWHIP_KIND_HQ4_G32_M5) return false;
    const uint32_t inter = w->n / (2u * experts);
    const uint32_t nb = w->k / 32u, cpr = (nb + 31u) / 32u;
    if (cpr > 16u || pairs > 65535u) return false;
    if ((uint64_t)2u * inter * nb * 20u >= (1ull << 32)) return false;   // 32-bit offsets inside an expert's sub-bank
    // experts shared by the 2..4 tokens of a verify window are read once when the window's route table fits one wavefront
    // and four activation rows fit the workgroup's LDS; the workgroup is then at most 512 threads wide
    constexpr uint32_t kReuseRows = 4;
    const bool reuse = reuse_tokens >= 2u && reuse_tokens <= kReuseRows && (idx || logits) && top_k >= 1u && top_k <= 16u &&
                       pairs == reuse_tokens * top_k && pairs <= 64u && cpr <= 8u &&
                       kReuseRows * ((size_t)nb * 80u + (size_t)64u * cpr * 4u) <= 60u * 1024u;
    const uint32_t sets = reuse ? (cpr <= 2u ? 8u : (cpr <= 4u ? 4u : 2u)) : (cpr <= 4u ? 8u : (cpr <= 8u ? 4u : 2u));
    const size_t lds = (reuse ? kReuseRows : 1u) * ((size_t)nb * 80u + (size_t)64u * cpr * 4u);
    if (lds > 60u * 1024u) return false;
    qmc_gu_params p;
    p.bank = (const uint8_t*)w->blocks;
    p.x = x;
    p.act = (h1_t*)act16;
    p.idx = idx;
    p.x_rows = x_rows;
    p.ga = act;
    p.I = inter;
    p.nb = nb;
    p.cpr = cpr;
    p.top_k = top_k;
    p.rotate = rotate ? 1u : 0u;
    p.rot_out = rot_out ? 1u : 0u;
    p.expert_bytes = (uint64_t)2u * inter * nb * 20u;
    p.logits = logits;
    p.idx_out = idx_out;
    p.wts_out = wts_out;
    p.experts = experts;
    p.norm = norm_topk;
    p.routed_scale = routed_scale;
    const dim3 grid(qwhip_cdiv(inter, 32u), pairs), block(32u * cpr * sets);
#define QMC_GU(DT, S, J, M) qw_launch_scalar<qw_moe_gateup_col_kernel<DT, S, J, M>>(grid, block, lds, st, p)
#define QMC_GU_M(DT, J, M)                                                                                              \
    do {                                                                                                                \
        if (sets == 8u) QMC_GU(DT, 8, J, M); else if (sets == 4u) QMC_GU(DT, 4, J, M); else QMC_GU(DT, 2, J, M);        \
    } while (0)
#define QMC_GU_S(DT, J)                                                            \
    do {                                                                           \
        if (reuse) QMC_GU_M(DT, J, (int)kReuseRows); else QMC_GU_M(DT, J, 1);      \
    } while (0)
    if (!logits) {
        if (x_dtype == QWHIP_F16) QMC_GU_S(QWHIP_F16, 0); else QMC_GU_S(QWHIP_BF16, 0);
    } else if (experts <= 128u) {   // routing in the kernel: two experts per lane cover the usual 64 / 128, eight cover up to 512
        if (x_dtype == QWHIP_F16) QMC_GU_S(QWHIP_F16, 2); else QMC_GU_S(QWHIP_BF16, 2);
    } else {
        if (x_dtype == QWHIP_F16) QMC_GU_S(QWHIP_F16, 8); else QMC_GU_S(QWHIP_BF16, 8);
    }
#undef QMC_GU_S
#undef QMC_GU_M
#undef QMC_GU
    *err = hipGetLastError();
    return true;
}

// Routed down projection + weighted combine (+ gated shared expert) for a validated HQ4_G32_M5 bank; false when the
// shape is outside the kernel's envelope.
bool qw_moe_down_col(hipStream_t st, const qwhip_weight_view* w, uint32_t experts, const void* act16, const int32_t* idx,
                     const float* wts, uint32_t t, uint32_t top_k, const float* shared, const float* shared_gate, void* out,
                     uint32_t out_dtype, hipError_t* err, uint32_t x_div, const int32_t* labels, uint32_t num_groups) {
    if (w->kind != QWHIP_KIND_HQ4_G32_M5) return false;
    const uint32_t hidden = w->n / experts;
    const uint32_t nbI = w->k / 32u;
    const uint32_t nbv = top_k * nbI, cprv = (nbv + 31u) / 32u;
    const uint32_t out_rows = t * (num_groups ? num_groups : 1u);
    if (cprv > 32u || out_rows > 65535u) return false;
    if (((uintptr_t)act16 & 15u) != 0) return false;
    uint32_t sets = 1;
    while (sets < 8u && 32u * cprv * sets * 2u <= 1024u) sets *= 2u;
    constexpr int D = 2;
    qmc_dn_params p;
    p.bank = (const uint8_t*)w->blocks;
    p.act = (const h1_t*)act16;
    p.idx = idx;
    p.wts = wts;
    p.shared = shared;
    p.shared_gate = shared_gate;
    p.out = out;
    p.H = hidden;
    p.nbI = nbI;
    p.nbv = nbv;
    p.cprv = cprv;
    p.top_k = top_k;
    p.sets = sets;
    p.expert_bytes = (uint64_t)hidden * nbI * 20u;
    p.x_div = x_div;
    p.labels = labels;
    p.num_groups = num_groups ? (num_groups | (experts << 8)) : 0u;
    const dim3 grid(qwhip_cdiv(hidden, sets * D), out_rows), block(32u * cprv * sets);
#define QMC_DN(OD)                                                                                            \
    do {                                                                                                      \
        if (num_groups) qw_launch_scalar<qw_moe_down_col_kernel<OD, D, true>>(grid, block, 0, st, p);         \
        else qw_launch_scalar<qw_moe_down_col_kernel<OD, D, false>>(grid, block, 0, st, p);                   \
    } while (0)
    if (out_dtype == QWHIP_F32) QMC_DN(QWHIP_F32);
    else if (out_dtype == QWHIP_F16) QMC_DN(QWHIP_F16);
    else if (out_dtype == QWHIP_BF16) QMC_DN(QWHIP_BF16);
    else return false;
#undef QMC_DN
    *err = hipGetLastError();
    return true;
}
