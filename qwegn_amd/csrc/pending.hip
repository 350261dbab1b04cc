// Entry points whose kernels are not in the library yet: they refuse with QWHIP_E_BLOCKED, as the
// reference's plan table refuses a family without a winner (QWGemm.swift:119-131).
#include "qwhip_common.h"

#define QW_PENDING(name) return qwhip_fail(QWHIP_E_BLOCKED, name ": no kernel in this build")

extern "C" qwhip_status qwhip_moe_route(qwhip_stream_t, const float*, uint32_t, uint32_t, uint32_t, uint32_t, float, int32_t*,
                                        float*) { QW_PENDING("qwhip_moe_route"); }
extern "C" qwhip_status qwhip_router_gemm(qwhip_stream_t, const void*, uint32_t, const void*, uint32_t, uint32_t, uint32_t,
                                          uint32_t, float*) { QW_PENDING("qwhip_router_gemm"); }
extern "C" uint32_t qwhip_moe_max_tiles(uint32_t experts, uint32_t pairs) {
    const uint32_t a = experts < pairs ? experts : pairs;
    const uint32_t b = a + (pairs + 63u) / 64u;
    return pairs < b ? pairs : b;
}
extern "C" qwhip_status qwhip_moe_group_pairs(qwhip_stream_t, const int32_t*, uint32_t, uint32_t, uint32_t, int32_t*, int32_t*,
                                              int32_t*, int32_t*, int32_t*, int32_t*, int32_t*, uint32_t) { QW_PENDING("qwhip_moe_group_pairs"); }
extern "C" qwhip_status qwhip_moe_combine(qwhip_stream_t, const void*, uint32_t, const int32_t*, const float*, uint32_t, uint32_t,
                                          uint32_t, const float*, const float*, void*, uint32_t) { QW_PENDING("qwhip_moe_combine"); }
extern "C" qwhip_status qwhip_moe_gateup_decode(qwhip_stream_t, const qwhip_weight_view*, uint32_t, const void*, uint32_t, uint32_t,
                                                const int32_t*, uint32_t, uint32_t, void*) { QW_PENDING("qwhip_moe_gateup_decode"); }
extern "C" qwhip_status qwhip_moe_down_decode(qwhip_stream_t, const qwhip_weight_view*, uint32_t, const void*, const int32_t*,
                                              const float*, uint32_t, uint32_t, const float*, const float*, void*, uint32_t) { QW_PENDING("qwhip_moe_down_decode"); }
extern "C" qwhip_status qwhip_quantize_hq4_g32(qwhip_stream_t, const void*, uint32_t, uint32_t, uint32_t, uint32_t, void*) { QW_PENDING("qwhip_quantize_hq4_g32"); }
