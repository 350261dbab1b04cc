// Tests of the host operator layer (qwhost.hpp).  `--cpu`: plan table, failable views, error mapping, no device.
// `--gpu`: the operators run on the device and are checked against host formulas restated from the reference's own
// self-contained tests (splitmix64 HQ4 GEMV: Tests/QWGEMMTests/QWHQ4GEMVTests.swift:16-50,108-133; closed-form MoE:
// Tests/QWGEMMTests/QWMoEReuseTests.swift:18-127).  Exit code 0 = all passed.
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>

#include "qwhost.hpp"

using namespace qw;

static int g_failed = 0, g_checks = 0;
#define CHECK(cond)                                                                  \
    do {                                                                             \
        ++g_checks;                                                                  \
        if (!(cond)) {                                                               \
            ++g_failed;                                                              \
            std::printf("FAILED %s:%d: %s\n", __FILE__, __LINE__, #cond);            \
        }                                                                            \
    } while (0)
#define CHECK_THROWS(expr, ErrT, kindv)                                              \
    do {                                                                             \
        ++g_checks;                                                                  \
        bool ok_ = false;                                                            \
        try { expr; } catch (const ErrT& e_) { ok_ = e_.kind == kindv; } catch (...) {} \
        if (!ok_) { ++g_failed; std::printf("FAILED %s:%d: %s did not throw %s\n", __FILE__, __LINE__, #expr, #kindv); } \
    } while (0)

static uint16_t f2h(float f) { _Float16 h = (_Float16)f; uint16_t b; std::memcpy(&b, &h, 2); return b; }
static float h2f(uint16_t b) { _Float16 h; std::memcpy(&h, &b, 2); return (float)h; }

// ---------------------------------------------------------------------------------------------------------------
static void test_plan_table() {
    using B = QWGemmPlan::Backend;
    // the reference's table row by row (QWGemm.swift:92-133): backend, kernel name, threads per threadgroup
    auto p = QWGemm::plan({1, 17408, 5120}, QWDType::q4g, QWEpilogue::none, QWDType::f16);
    CHECK(p.backend == B::handQ4gV4H16 && p.kernel == "qwg_gemv_q4g_v4_h16" && p.threadsPerTG == 32 && p.family == QWGemmFamily::f1DecodeGemv);
    p = QWGemm::plan({1, 17408, 5120}, QWDType::q4g, QWEpilogue::none);
    CHECK(p.backend == B::handQ4gV4 && p.kernel == "qwg_gemv_q4g_v4" && p.threadsPerTG == 32);
    p = QWGemm::plan({1, 248320, 5120}, QWDType::q4g, QWEpilogue::none, QWDType::f32, 248320);
    CHECK(p.family == QWGemmFamily::f2LmHeadGemv && p.backend == B::handQ4gV4);
    p = QWGemm::plan({1, 34816, 5120}, QWDType::q4g, QWEpilogue::siluMulPair, QWDType::f16);
    CHECK(p.backend == B::handQ4gSiluPairH16 && p.kernel == "qwg_gemv_q4g_silu_pair_h16" && p.threadsPerTG == 64);
    p = QWGemm::plan({4096, 34816, 5120}, QWDType::q4g, QWEpilogue::siluMulPair);   // the epilogue rows come first, whatever the family
    CHECK(p.backend == B::handQ4gSiluPair && p.kernel == "qwg_gemv_q4g_silu_pair" && p.family == QWGemmFamily::f3PrefillGemm);
    p = QWGemm::plan({2, 5120, 5120}, QWDType::q4g, QWEpilogue::none);
    CHECK(p.backend == B::handQ4gSkinny && p.kernel == "qwg_skinny_m2" && p.threadsPerTG == 32);
    p = QWGemm::plan({3, 5120, 5120}, QWDType::q4g, QWEpilogue::none);
    CHECK(p.backend == B::handQ4gSkinny && p.kernel == "qwg_skinny_m3" && p.family == QWGemmFamily::f5SkinnyGemm);
    p = QWGemm::plan({3, 5120, 65536}, QWDType::q4g, QWEpilogue::none);             // 3 * 65536 * 2 bytes > 256 KiB of constants
    CHECK(p.backend == B::blocked && p.family == QWGemmFamily::f5SkinnyGemm);
    p = QWGemm::plan({4, 5120, 5120}, QWDType::q4g, QWEpilogue::none);              // the skinny window is M in {2, 3}
    CHECK(p.backend == B::blocked && p.kernel.empty() && p.threadsPerTG == 0);
    p = QWGemm::plan({1, 4096, 4096}, QWDType::f16, QWEpilogue::none);
    CHECK(p.backend == B::handF16V4 && p.kernel == "qwg_gemv_f16_v4" && p.threadsPerTG == 32);
    p = QWGemm::plan({4096, 5120, 5120}, QWDType::q4g, QWEpilogue::none);
    CHECK(p.backend == B::mpsGraphBmmF16 && p.kernel == "mpsgraph_bmm_f16" && p.threadsPerTG == 0 && p.family == QWGemmFamily::f3PrefillGemm);
    p = QWGemm::plan({4096, 5120, 5100}, QWDType::q4g, QWEpilogue::none);           // K % 32 != 0
    CHECK(p.backend == B::blocked);
    p = QWGemm::plan({100, 5120, 5120}, QWDType::q4g, QWEpilogue::none);            // F4: nothing raced
    CHECK(p.backend == B::blocked && p.family == QWGemmFamily::f4AttentionTiles);
    p = QWGemm::plan({1, 64, 64}, QWDType::f32, QWEpilogue::none);
    CHECK(p.backend == B::blocked);
    p = QWGemm::plan({4096, 64, 64}, QWDType::f16, QWEpilogue::none);
    CHECK(p.backend == B::blocked);
    CHECK((QWGemmShape{100, 8, 8}.family() == QWGemmFamily::f4AttentionTiles));
    // this library's routing over the same shapes
    p = QWGemm::planHip({4, 5120, 5120}, QWDType::q4g, QWEpilogue::none);
    CHECK(p.backend == B::handQ4gSkinny);
    p = QWGemm::planHip({16, 5120, 5120}, QWDType::q4g, QWEpilogue::none);
    CHECK(p.backend == B::handQ4gSkinny && p.family == QWGemmFamily::f4AttentionTiles);
    p = QWGemm::planHip({4096, 5120, 5120}, QWDType::q4g, QWEpilogue::none);
    CHECK(p.backend == B::mfmaGemmF16 && p.kernel == "qwg_gemm_q4g_h16");
    p = QWGemm::planHip({4096, 5120, 5100}, QWDType::q4g, QWEpilogue::none);
    CHECK(p.backend == B::blocked);
    p = QWGemm::planHip({1, 64, 64}, QWDType::f16, QWEpilogue::none);
    CHECK(p.backend == B::blocked);
}

static void test_weight_view() {
    std::vector<uint8_t> buf(8 * 2 * 36);
    QWTensorValue blocks = QWTensorValue::make(buf.data(), buf.size(), QWDType::q4g);
    // QWWeightView.init? (QWWeightView.swift:107-118)
    CHECK(QWWeightView::make(blocks, 8, 64, 4, 32, true).has_value());
    CHECK(QWWeightView::make(blocks, 8, 64, 4, 32, true)->containerKind.isIncumbentContainer());
    CHECK(QWWeightView::make(blocks, 8, 64, 4, 32, true)->formatName() == "HQ4_G32");
    CHECK(!QWWeightView::make(blocks, 0, 64, 4, 32, true).has_value());
    CHECK(!QWWeightView::make(blocks, 8, 48, 4, 32, true).has_value());
    CHECK(!QWWeightView::make(blocks, 8, 64, 5, 32, true).has_value());
    CHECK(!QWWeightView::make(blocks, 8, 64, 4, 32, false, true).has_value());   // incumbent must be rotated
    auto v8 = QWWeightView::make(blocks, 8, 64, 8, 32, true);
    CHECK(v8.has_value() && v8->rowBytes() == 72 && v8->requiredBytes() == 576 && v8->formatName() == "HQ8_G32" && v8->isRotated());
    auto a4 = QWWeightView::make(blocks, 8, 64, 4, 64, false);
    CHECK(a4.has_value() && a4->formatName() == "AQ4_G64" && !a4->isRotated() && a4->rowBytes() == 36);
    // the 4-bit G32 pair has two containers of the same size but different kinds (QWAQBlock.swift:14-16)
    auto blk = QWWeightView::make(blocks, 8, 64, 4, 32, true, false);
    CHECK(blk.has_value() && !blk->containerKind.isIncumbentContainer() && blk->rowBytes() == 40);
    QWTensorValue small = QWTensorValue::make(buf.data(), 8 * 2 * 20 - 1, QWDType::q4g);
    CHECK(!QWWeightView::make(small, 8, 64, 4, 32, true).has_value());
    CHECK(v8->subview(blocks, 4, 64).has_value());
}

static void test_hal_refuses_without_device() {
    // no device: the HAL refuses to open (no CPU fallback)
    CHECK_THROWS(QWHal hal(0), QWHalError, QWHalError::deviceUnavailable);
}

static void test_error_mapping() {
    CHECK_THROWS(throwIfFailed(QWHIP_E_BAD_GEOMETRY), QWGemmError, QWGemmError::badGeometry);
    CHECK_THROWS(throwIfFailed(QWHIP_E_KERNEL_MISSING), QWHalError, QWHalError::kernelMissing);
    CHECK(QWGemm::moeMaxTiles(128, 16384) == 384 && QWGemm::moeMaxTiles(128, 5) == 5);
    CHECK(QWGemmAQ::kernelName(8, 32).value_or("") == "qwg_gemv_aq8_g32_v4" && QWGemmAQ::kernelName(3, 32).value_or("") == "qwg_gemv_aq3_g32_v4" &&
          !QWGemmAQ::kernelName(5, 32).has_value() && !QWGemmAQ::kernelName(4, 48).has_value());
}

// ---------------------------------------------------------------------------------------------------------------
static uint64_t splitmix64(uint64_t x) {
    uint64_t z = x + 0x9E3779B97F4A7C15ull;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}
static const int kNibbleShift[8] = {0, 16, 4, 20, 8, 24, 12, 28};  // QWAQProducer.hq4NibbleBitOffset

struct DeviceBuf {
    QWHal& hal;
    void* p;
    size_t bytes;
    DeviceBuf(QWHal& h, size_t n) : hal(h), p(h.alloc(n ? n : 256)), bytes(n) {}
    ~DeviceBuf() { hal.free(p); }
};
static void upload(QWHipEncoder& e, DeviceBuf& b, const void* src, size_t n) { throwIfFailed(qwhip_memcpy_h2d(e.stream, b.p, src, n)); }
static void download(QWHipEncoder& e, void* dst, DeviceBuf& b, size_t n) { throwIfFailed(qwhip_memcpy_d2h(e.stream, dst, b.p, n)); }

static void test_gpu_hq4_gemv(QWHal& hal) {
    const int rows = 64, cols = 256, groups = cols / 32;
    std::vector<uint8_t> bank((size_t)rows * groups * 20);
    for (int r = 0; r < rows; ++r)
        for (int g = 0; g < groups; ++g) {
            const uint64_t s = splitmix64((uint64_t)r * 0x00000001000003B3ull + (uint64_t)g * 0x9E3779B97F4A7C15ull);
            const double unit = (double)(splitmix64(s + 0x5DEECE66Dull) % 1000000) / 1000000.0;
            const uint16_t sc = f2h((float)(unit * 0.02 + 0.001));
            const uint16_t bi = f2h(-1032.0f * h2f(sc));
            uint8_t* o = &bank[((size_t)r * groups + g) * 20];
            std::memcpy(o, &sc, 2);
            std::memcpy(o + 2, &bi, 2);
            for (int w = 0; w < 4; ++w) {
                uint32_t word = 0;
                for (int j = 0; j < 8; ++j) word |= (uint32_t)(splitmix64(s + (uint64_t)(8 * w + j)) & 0xF) << kNibbleShift[j];
                std::memcpy(o + 4 + 4 * w, &word, 4);
            }
        }
    std::vector<uint16_t> xs(cols);
    for (int i = 0; i < cols; ++i) xs[i] = f2h((float)((double)(splitmix64((uint64_t)i * 0x9E3779B97F4A7C15ull) % 2000001) / 1000000.0 - 1.0));

    QWHipEncoder enc = hal.begin();
    DeviceBuf dbank(hal, bank.size()), dx(hal, cols * 2), dy16(hal, rows * 2), dy32(hal, rows * 4);
    upload(enc, dbank, bank.data(), bank.size());
    upload(enc, dx, xs.data(), cols * 2);
    auto view = QWWeightView::make(QWTensorValue::make(dbank.p, bank.size(), QWDType::q4g), rows, cols, 4, 32, true);
    CHECK(view.has_value());
    const QWTensorValue x = QWTensorValue::make(dx.p, cols, QWDType::f16);
    const QWTensorValue y16 = QWTensorValue::make(dy16.p, rows, QWDType::f16), y32 = QWTensorValue::make(dy32.p, rows, QWDType::f32);
    const QWGemmPlan plan = QWGemm::plan({1, rows, cols}, QWDType::q4g, QWEpilogue::none, QWDType::f16);
    QWGemm::encodeH16(enc, hal, plan, x, *view, y16, &y32);   // dual store
    std::vector<float> got(rows);
    download(enc, got.data(), dy32, rows * 4);
    std::vector<uint16_t> got16(rows);
    download(enc, got16.data(), dy16, rows * 2);
    for (int r = 0; r < rows; ++r) {
        double value = 0, magnitude = 0;
        for (int g = 0; g < groups; ++g) {
            const uint8_t* o = &bank[((size_t)r * groups + g) * 20];
            uint16_t sc, bi;
            std::memcpy(&sc, o, 2);
            std::memcpy(&bi, o + 2, 2);
            for (int w = 0; w < 4; ++w) {
                uint32_t word;
                std::memcpy(&word, o + 4 + 4 * w, 4);
                for (int j = 0; j < 8; ++j) {
                    const float nib = (float)((word >> kNibbleShift[j]) & 0xF);
                    const float v = h2f(f2h((1024.0f + nib) * h2f(sc) + h2f(bi)));
                    const double prod = (double)v * (double)h2f(xs[g * 32 + w * 8 + j]);
                    value += prod;
                    magnitude += std::fabs(prod);
                }
            }
        }
        const double scale = std::fmax(std::fmax(std::fabs(value), magnitude), 1e-6);
        CHECK(std::fabs((double)got[r] - value) / scale <= 1e-3);
        CHECK(std::fabs((double)h2f(got16[r]) - value) / scale <= 2e-3);
    }
    // errors surface before any launch and leave the stream usable (Tests/QWGEMMTests/QWGEMMTests.swift:246-247)
    const QWTensorValue shortX = QWTensorValue::make(dx.p, cols - 1, QWDType::f16);
    CHECK_THROWS(QWGemm::encodeH16(enc, hal, plan, shortX, *view, y16), QWGemmError, QWGemmError::badWeights);
    const QWTensorValue wrongY = QWTensorValue::make(dy16.p, rows / 2, QWDType::f32);
    CHECK_THROWS(QWGemm::encodeH16(enc, hal, plan, x, *view, wrongY), QWGemmError, QWGemmError::badWeights);
    CHECK_THROWS(hal.pipeline("qwg_gemv_shvq4_g32_v4"), QWHalError, QWHalError::kernelMissing);
    const QWGemmPlan blocked = QWGemm::plan({1, rows, cols}, QWDType::f32, QWEpilogue::none);
    CHECK_THROWS(QWGemm::encode(enc, hal, blocked, x, *view, y32), QWGemmError, QWGemmError::f3Blocked);
    QWGemm::encodeH16(enc, hal, plan, x, *view, y16);
    hal.end(enc);
}

// closed-form bank: code (r*7 + c*3 + 5) % 16, scale 1/16, HQ4_G32 block -> weight (code - 8)/16
static double cf_weight(int row, int col) { return ((double)((row * 7 + col * 3 + 5) % 16) - 8.0) / 16.0; }
static std::vector<uint8_t> cf_bank(int rows, int cols) {
    std::vector<uint8_t> bank((size_t)rows * (cols / 32) * 20);
    const uint16_t sc = f2h(1.0f / 16), bi = f2h(-1032.0f / 16);
    for (int r = 0; r < rows; ++r)
        for (int g = 0; g < cols / 32; ++g) {
            uint8_t* o = &bank[((size_t)r * (cols / 32) + g) * 20];
            std::memcpy(o, &sc, 2);
            std::memcpy(o + 2, &bi, 2);
            for (int w = 0; w < 4; ++w) {
                uint32_t word = 0;
                for (int j = 0; j < 8; ++j) word |= (uint32_t)((r * 7 + (g * 32 + w * 8 + j) * 3 + 5) % 16) << kNibbleShift[j];
                std::memcpy(o + 4 + 4 * w, &word, 4);
            }
        }
    return bank;
}
static void fwht32(double* p) {
    for (int h = 1; h < 32; h <<= 1)
        for (int i0 = 0; i0 < 32; i0 += 2 * h)
            for (int j = 0; j < h; ++j) {
                const double u = p[i0 + j], v = p[i0 + j + h];
                p[i0 + j] = u + v;
                p[i0 + j + h] = u - v;
            }
    for (int i = 0; i < 32; ++i) p[i] /= std::sqrt(32.0);
}

static void test_gpu_moe_resident(QWHal& hal, int rows) {
    const int E = 16, K = 3, H = 64, I = 64;
    const std::vector<uint8_t> gu = cf_bank(E * 2 * I, H), dn = cf_bank(E * H, I);
    std::vector<float> router((size_t)E * H);
    for (int e = 0; e < E; ++e)
        for (int h = 0; h < H; ++h) router[(size_t)e * H + h] = (float)(((e * 5 + h * 11) % 17) - 8) / 32.0f;
    std::vector<uint16_t> x((size_t)rows * H);
    std::vector<double> xd((size_t)rows * H);
    for (int t = 0; t < rows; ++t)
        for (int h = 0; h < H; ++h) {
            const float v = (float)(((t * 13 + h * 7) % 19) - 9) / 8.0f;
            x[(size_t)t * H + h] = f2h(v);
            xd[(size_t)t * H + h] = h2f(f2h(v));
        }
    // host reference: routing (softmax top-k, ties to the lower index, renormalised), experts in double, act rounded to f16 after rotation
    std::vector<double> ref((size_t)rows * H, 0.0);
    for (int t = 0; t < rows; ++t) {
        std::vector<double> logit(E), p(E);
        double mx = -1e300, tot = 0;
        for (int e = 0; e < E; ++e) {
            double s = 0;
            for (int h = 0; h < H; ++h) s += (double)router[(size_t)e * H + h] * xd[(size_t)t * H + h];
            logit[e] = (double)(float)s;
            mx = std::fmax(mx, logit[e]);
        }
        for (int e = 0; e < E; ++e) { p[e] = std::exp(logit[e] - mx); tot += p[e]; }
        std::vector<int> chosen;
        std::vector<bool> taken(E, false);
        double wsum = 0;
        for (int r = 0; r < K; ++r) {
            int best = -1;
            for (int e = 0; e < E; ++e)
                if (!taken[e] && (best < 0 || p[e] > p[best])) best = e;
            taken[best] = true;
            chosen.push_back(best);
            wsum += p[best] / tot;
        }
        for (int r = 0; r < K; ++r) {
            const int e = chosen[r];
            const double wk = (p[e] / tot) / wsum;
            std::vector<double> act(I);
            for (int i = 0; i < I; ++i) {
                double g = 0, u = 0;
                for (int h = 0; h < H; ++h) {
                    g += cf_weight(e * 2 * I + i, h) * xd[(size_t)t * H + h];
                    u += cf_weight(e * 2 * I + I + i, h) * xd[(size_t)t * H + h];
                }
                act[i] = g / (1 + std::exp(-g)) * u;
            }
            for (int o = 0; o < I; o += 32) fwht32(&act[o]);
            for (int i = 0; i < I; ++i) act[i] = h2f(f2h((float)act[i]));
            for (int h = 0; h < H; ++h) {
                double d = 0;
                for (int i = 0; i < I; ++i) d += cf_weight(e * H + h, i) * act[i];
                ref[(size_t)t * H + h] += wk * d;
            }
        }
    }
    QWHipEncoder enc = hal.begin();
    const int pairs = rows * K, mt = QWGemm::moeMaxTiles(E, pairs);
    DeviceBuf dgu(hal, gu.size()), ddn(hal, dn.size()), dr(hal, router.size() * 4), dx(hal, x.size() * 2), dout(hal, (size_t)rows * H * 4);
    DeviceBuf dlog(hal, (size_t)rows * E * 4), didx(hal, pairs * 4), dw(hal, pairs * 4), dact(hal, (size_t)pairs * I * 2);
    DeviceBuf doff(hal, (E + 1) * 4), dsp(hal, pairs * 4), dst(hal, pairs * 4), dinv(hal, pairs * 4), dte(hal, mt * 4), dtr(hal, mt * 4), dtc(hal, 16);
    DeviceBuf dgu16(hal, (size_t)pairs * 2 * I * 2), ddnhi(hal, (size_t)pairs * H * 4);
    upload(enc, dgu, gu.data(), gu.size());
    upload(enc, ddn, dn.data(), dn.size());
    upload(enc, dr, router.data(), router.size() * 4);
    upload(enc, dx, x.data(), x.size() * 2);
    QWMoEOperator::Weights w;
    w.router = QWTensorValue::make(dr.p, router.size(), QWDType::f32);
    w.gateUp = *QWWeightView::make(QWTensorValue::make(dgu.p, gu.size(), QWDType::q4g), E * 2 * I, H, 4, 32, true);
    w.down = *QWWeightView::make(QWTensorValue::make(ddn.p, dn.size(), QWDType::q4g), E * H, I, 4, 32, true);
    w.hidden = H; w.experts = E; w.topK = K; w.intermediate = I;
    QWMoEOperator::Scratch s;
    s.logits = QWTensorValue::make(dlog.p, (size_t)rows * E, QWDType::f32);
    s.idx = QWTensorValue::make(didx.p, pairs, QWDType::i32);
    s.wts = QWTensorValue::make(dw.p, pairs, QWDType::f32);
    s.act16 = QWTensorValue::make(dact.p, (size_t)pairs * I, QWDType::f16);
    s.expOff = QWTensorValue::make(doff.p, E + 1, QWDType::i32);
    s.sortedPair = QWTensorValue::make(dsp.p, pairs, QWDType::i32);
    s.sortedTok = QWTensorValue::make(dst.p, pairs, QWDType::i32);
    s.invPerm = QWTensorValue::make(dinv.p, pairs, QWDType::i32);
    s.tileE = QWTensorValue::make(dte.p, mt, QWDType::i32);
    s.tileR = QWTensorValue::make(dtr.p, mt, QWDType::i32);
    s.tileCount = QWTensorValue::make(dtc.p, 4, QWDType::i32);
    s.gu16 = QWTensorValue::make(dgu16.p, (size_t)pairs * 2 * I, QWDType::f16);
    s.dnHi = QWTensorValue::make(ddnhi.p, (size_t)pairs * H, QWDType::f32);
    const QWTensorValue xt = QWTensorValue::make(dx.p, x.size(), QWDType::f16);
    const QWTensorValue out = QWTensorValue::make(dout.p, (size_t)rows * H, QWDType::f32);
    // the test feeds the same rows to the router and the experts (the closed-form bank is taken as given in its basis)
    QWMoEOperator::encodeResident(enc, hal, w, s, xt, xt, out, rows);
    std::vector<float> got((size_t)rows * H);
    download(enc, got.data(), dout, got.size() * 4);
    double num = 0, den = 0;
    for (size_t i = 0; i < got.size(); ++i) { num += ((double)got[i] - ref[i]) * ((double)got[i] - ref[i]); den += ref[i] * ref[i]; }
    const double err = std::sqrt(num / std::fmax(den, 1e-30));
    std::printf("moe encodeResident rows=%d normalized error %.3e\n", rows, err);
    CHECK(err <= 2e-3);
    if (rows >= 2 && rows <= 4) {   // a verify window with reuseExpertsAcrossTokens: the same bits
        QWMoEOperator::Weights wr = w;
        wr.reuseExpertsAcrossTokens = true;
        QWMoEOperator::encodeResident(enc, hal, wr, s, xt, xt, out, rows);
        std::vector<float> again((size_t)rows * H);
        download(enc, again.data(), dout, again.size() * 4);
        CHECK(std::memcmp(again.data(), got.data(), got.size() * 4) == 0);
    }
    // shared-expert gate column of the router door: with router row 0 as the gate row, gate[t] = sigmoid(logits[t, 0])
    {
        DeviceBuf dgate(hal, (size_t)rows * 4);
        const QWTensorValue shw = QWTensorValue::make(dr.p, (size_t)H, QWDType::f32);
        const QWTensorValue shout = QWTensorValue::make(dgate.p, (size_t)rows, QWDType::f32);
        QWGemm::encodeFnRouterGemm(enc, hal, xt, w.router, s.logits, rows, E, H, &shw, &shout);
        std::vector<float> lg((size_t)rows * E), gate((size_t)rows);
        download(enc, lg.data(), dlog, lg.size() * 4);
        download(enc, gate.data(), dgate, gate.size() * 4);
        for (int t = 0; t < rows; ++t) CHECK(std::fabs(gate[t] - 1.0 / (1.0 + std::exp(-(double)lg[(size_t)t * E]))) <= 2e-6);
        bool threw = false;
        const QWTensorValue shw16 = QWTensorValue::make(dr.p, (size_t)H, QWDType::f16);
        try { QWGemm::encodeFnRouterGemm(enc, hal, xt, w.router, s.logits, rows, E, H, &shw16, &shout); } catch (const QWGemmError&) { threw = true; }
        CHECK(threw);
    }
    hal.end(enc);
}

// QWMoEOperator.encodeResidentLatent on closed-form banks against the chain in double (QWMoEOperator+Latent.swift:17-303):
// bridge -> router (+ shared gate) -> fc1 -> route -> rotate -> routed experts in the latent width -> latent norm -> fc2,
// shared expert on the hidden width added under its gate.  rows = 3 takes the routed GEMVs, rows = 40 the grouped GEMMs and
// the batched f32 projections.
static void test_gpu_moe_latent(QWHal& hal, int rows) {
    const int E = 16, K = 3, H = 256, L = 64, I = 64, ISh = 64;
    const float eps = 1e-6f;
    const std::vector<uint8_t> fc1 = cf_bank(L, H), fc2 = cf_bank(H, L), gu = cf_bank(E * 2 * I, L), dn = cf_bank(E * L, I);
    const std::vector<uint8_t> shgu = cf_bank(2 * ISh, H), shdn = cf_bank(H, ISh);
    std::vector<float> router((size_t)E * H);
    for (int e = 0; e < E; ++e)
        for (int h = 0; h < H; ++h) router[(size_t)e * H + h] = (float)(((e * 5 + h * 11) % 17) - 8) / 64.0f;
    std::vector<uint16_t> gamma(L);
    for (int l = 0; l < L; ++l) gamma[l] = f2h((float)((l % 5) - 2) / 16.0f);
    std::vector<uint16_t> x((size_t)rows * H);
    for (int t = 0; t < rows; ++t)
        for (int h = 0; h < H; ++h) x[(size_t)t * H + h] = f2h((float)(((t * 13 + h * 7) % 19) - 9) / 8.0f);
    auto silu = [](double g) { return g / (1 + std::exp(-g)); };
    std::vector<double> ref((size_t)rows * H, 0.0);
    for (int t = 0; t < rows; ++t) {
        std::vector<double> xr(H), xp(H);
        for (int h = 0; h < H; ++h) xr[h] = xp[h] = h2f(x[(size_t)t * H + h]);
        for (int o = 0; o < H; o += 32) fwht32(&xp[o]);
        std::vector<double> logit(E), p(E);
        double mx = -1e300, tot = 0;
        for (int e = 0; e < E; ++e) {
            double a = 0;
            for (int h = 0; h < H; ++h) a += (double)router[(size_t)e * H + h] * xp[h];
            logit[e] = a;
            mx = std::fmax(mx, a);
        }
        const double gate = 1.0 / (1.0 + std::exp(-logit[0]));   // the gate row is router row 0
        for (int e = 0; e < E; ++e) { p[e] = std::exp(logit[e] - mx); tot += p[e]; }
        std::vector<int> chosen;
        std::vector<bool> taken(E, false);
        double wsum = 0;
        for (int r = 0; r < K; ++r) {
            int best = -1;
            for (int e = 0; e < E; ++e)
                if (!taken[e] && (best < 0 || p[e] > p[best])) best = e;
            taken[best] = true;
            chosen.push_back(best);
            wsum += p[best] / tot;
        }
        std::vector<double> lat(L), B(L, 0.0);
        for (int l = 0; l < L; ++l) {
            double a = 0;
            for (int h = 0; h < H; ++h) a += cf_weight(l, h) * xr[h];
            lat[l] = a;
        }
        for (int o = 0; o < L; o += 32) fwht32(&lat[o]);
        for (int l = 0; l < L; ++l) lat[l] = h2f(f2h((float)lat[l]));
        for (int r = 0; r < K; ++r) {
            const int e = chosen[r];
            const double wk = (p[e] / tot) / wsum;
            std::vector<double> act(I);
            for (int i = 0; i < I; ++i) {
                double g = 0, u = 0;
                for (int l = 0; l < L; ++l) {
                    g += cf_weight(e * 2 * I + i, l) * lat[l];
                    u += cf_weight(e * 2 * I + I + i, l) * lat[l];
                }
                act[i] = silu(g) * u;
            }
            for (int o = 0; o < I; o += 32) fwht32(&act[o]);
            for (int i = 0; i < I; ++i) act[i] = h2f(f2h((float)act[i]));
            for (int l = 0; l < L; ++l) {
                double d = 0;
                for (int i = 0; i < I; ++i) d += cf_weight(e * L + l, i) * act[i];
                B[l] += wk * d;
            }
        }
        double ms = 0;
        for (int l = 0; l < L; ++l) ms += B[l] * B[l];
        const double inv = 1.0 / std::sqrt(ms / L + (double)eps);
        std::vector<double> Cn(L);
        for (int l = 0; l < L; ++l) Cn[l] = B[l] * inv * (1.0 + (double)h2f(gamma[l]));
        for (int o = 0; o < L; o += 32) fwht32(&Cn[o]);
        std::vector<double> sact(ISh);
        for (int j = 0; j < ISh; ++j) {
            double g = 0, u = 0;
            for (int h = 0; h < H; ++h) {
                g += cf_weight(j, h) * xr[h];
                u += cf_weight(ISh + j, h) * xr[h];
            }
            sact[j] = silu(g) * u;
        }
        for (int o = 0; o < ISh; o += 32) fwht32(&sact[o]);
        for (int h = 0; h < H; ++h) {
            double a = 0, sh = 0;
            for (int l = 0; l < L; ++l) a += cf_weight(h, l) * Cn[l];
            for (int j = 0; j < ISh; ++j) sh += cf_weight(h, j) * sact[j];
            ref[(size_t)t * H + h] = a + gate * sh;
        }
    }
    QWHipEncoder enc = hal.begin();
    const int pairs = rows * K, mt = QWGemm::moeMaxTiles(E, pairs);
    DeviceBuf dfc1(hal, fc1.size()), dfc2(hal, fc2.size()), dgu(hal, gu.size()), ddn(hal, dn.size()), dshgu(hal, shgu.size()), dshdn(hal, shdn.size());
    DeviceBuf dr(hal, router.size() * 4), dgm(hal, gamma.size() * 2), dx(hal, x.size() * 2), dout(hal, (size_t)rows * H * 4);
    DeviceBuf dlog(hal, (size_t)rows * E * 4), didx(hal, pairs * 4), dw(hal, pairs * 4), dact(hal, (size_t)pairs * I * 2);
    DeviceBuf doff(hal, (E + 1) * 4), dsp(hal, pairs * 4), dst(hal, pairs * 4), dinv(hal, pairs * 4), dte(hal, mt * 4), dtr(hal, mt * 4), dtc(hal, 16);
    DeviceBuf ddnhi(hal, (size_t)pairs * L * 4);
    DeviceBuf dxr(hal, (size_t)rows * H * 4), dxp(hal, (size_t)rows * H * 4), dA(hal, (size_t)rows * L * 4), dB(hal, (size_t)rows * L * 4);
    DeviceBuf dB16(hal, (size_t)rows * L * 2), dnax(hal, (size_t)rows * H * 2), dgate(hal, (size_t)rows * 4);
    DeviceBuf dgush(hal, (size_t)rows * 2 * ISh * 4), dactsh(hal, (size_t)rows * ISh * 4), dshared(hal, (size_t)rows * H * 4);
    upload(enc, dfc1, fc1.data(), fc1.size());
    upload(enc, dfc2, fc2.data(), fc2.size());
    upload(enc, dgu, gu.data(), gu.size());
    upload(enc, ddn, dn.data(), dn.size());
    upload(enc, dshgu, shgu.data(), shgu.size());
    upload(enc, dshdn, shdn.data(), shdn.size());
    upload(enc, dr, router.data(), router.size() * 4);
    upload(enc, dgm, gamma.data(), gamma.size() * 2);
    upload(enc, dx, x.data(), x.size() * 2);
    auto bankView = [](DeviceBuf& b, int n, int k) { return *QWWeightView::make(QWTensorValue::make(b.p, b.bytes, QWDType::q4g), n, k, 4, 32, true); };
    QWMoEOperator::LatentWeights lw;
    lw.routed.router = QWTensorValue::make(dr.p, router.size(), QWDType::f32);
    lw.routed.gateUp = bankView(dgu, E * 2 * I, L);
    lw.routed.down = bankView(ddn, E * L, I);
    lw.routed.hidden = H; lw.routed.experts = E; lw.routed.topK = K; lw.routed.intermediate = I;
    lw.sharedGateUp = bankView(dshgu, 2 * ISh, H);
    lw.sharedDown = bankView(dshdn, H, ISh);
    lw.sharedGateScalar = QWTensorValue::make(dr.p, (size_t)H, QWDType::f32);
    lw.sharedIntermediate = ISh;
    QWMoEOperator::LatentBottleneck lb;
    lb.fc1 = bankView(dfc1, L, H);
    lb.fc2 = bankView(dfc2, H, L);
    lb.normGamma = QWTensorValue::make(dgm.p, (size_t)L, QWDType::f16);
    lb.normEps = eps;
    lb.latentDim = L;
    QWMoEOperator::Scratch s;
    s.logits = QWTensorValue::make(dlog.p, (size_t)rows * E, QWDType::f32);
    s.idx = QWTensorValue::make(didx.p, pairs, QWDType::i32);
    s.wts = QWTensorValue::make(dw.p, pairs, QWDType::f32);
    s.act16 = QWTensorValue::make(dact.p, (size_t)pairs * I, QWDType::f16);
    s.expOff = QWTensorValue::make(doff.p, E + 1, QWDType::i32);
    s.sortedPair = QWTensorValue::make(dsp.p, pairs, QWDType::i32);
    s.sortedTok = QWTensorValue::make(dst.p, pairs, QWDType::i32);
    s.invPerm = QWTensorValue::make(dinv.p, pairs, QWDType::i32);
    s.tileE = QWTensorValue::make(dte.p, mt, QWDType::i32);
    s.tileR = QWTensorValue::make(dtr.p, mt, QWDType::i32);
    s.tileCount = QWTensorValue::make(dtc.p, 4, QWDType::i32);
    s.dnHi = QWTensorValue::make(ddnhi.p, (size_t)pairs * L, QWDType::f32);
    QWMoEOperator::LatentScratch ls;
    ls.xRot32 = QWTensorValue::make(dxr.p, (size_t)rows * H, QWDType::f32);
    ls.xPlain32 = QWTensorValue::make(dxp.p, (size_t)rows * H, QWDType::f32);
    ls.bufA32 = QWTensorValue::make(dA.p, (size_t)rows * L, QWDType::f32);
    ls.bufB32 = QWTensorValue::make(dB.p, (size_t)rows * L, QWDType::f32);
    ls.bufB16 = QWTensorValue::make(dB16.p, (size_t)rows * L, QWDType::f16);
    ls.naxX16 = QWTensorValue::make(dnax.p, (size_t)rows * H, QWDType::f16);
    ls.gate = QWTensorValue::make(dgate.p, (size_t)rows, QWDType::f32);
    ls.guSh32 = QWTensorValue::make(dgush.p, (size_t)rows * 2 * ISh, QWDType::f32);
    ls.actSh32 = QWTensorValue::make(dactsh.p, (size_t)rows * ISh, QWDType::f32);
    ls.shared = QWTensorValue::make(dshared.p, (size_t)rows * H, QWDType::f32);
    const QWTensorValue xt = QWTensorValue::make(dx.p, x.size(), QWDType::f16);
    const QWTensorValue out = QWTensorValue::make(dout.p, (size_t)rows * H, QWDType::f32);
    QWMoEOperator::encodeResidentLatent(enc, hal, lw, lb, s, ls, xt, out, rows);
    std::vector<float> got((size_t)rows * H);
    download(enc, got.data(), dout, got.size() * 4);
    double num = 0, den = 0;
    for (size_t i = 0; i < got.size(); ++i) { num += ((double)got[i] - ref[i]) * ((double)got[i] - ref[i]); den += ref[i] * ref[i]; }
    const double err = std::sqrt(num / std::fmax(den, 1e-30));
    std::printf("moe encodeResidentLatent rows=%d normalized error %.3e\n", rows, err);
    CHECK(err <= 2e-3);
    // geometry checks of the door: a latent width the banks do not have is refused before any launch
    {
        QWMoEOperator::LatentBottleneck bad = lb;
        bad.latentDim = L + 32;
        bool threw = false;
        try { QWMoEOperator::encodeResidentLatent(enc, hal, lw, bad, s, ls, xt, out, rows); } catch (const QWGemmError&) { threw = true; }
        CHECK(threw);
    }
    hal.end(enc);
}

// Group-latent MoE with the configuration of the reference's own test (FNLatentMoETests.testGroupLatentMoEMatchesCPUAcrossDecodeVerifyAndPrefill,
// Tests/QWFlashNextTests/FNLatentMoETests.swift:95-189): H = L = I = IS = 64, 4 groups, 32 experts, 4 routes; latent and shared
// banks 8-bit G32, expert banks 4-bit G64, all rotated bit-stream containers with the test's code formula; the CPU side is the
// un-rotated restatement of FNSparseMoE.forward (Tests/QWFlashNextTests/Reference/FNSparseMoE.swift:113-156) in fp64 and the
// pass mark is the test's: max |got - want| / max |want| < 0.002 (0.01 from 64 rows on).
struct GLMatrix {
    std::vector<uint8_t> blocks;     // [rows, cols / group] blocks: f16 scale, f16 bias, bit stream
    std::vector<double> plain;       // [rows, cols]: the weights in the un-rotated basis
};
static GLMatrix gl_matrix(int rows, int cols, int bits, int group, int seed, bool foldOutput) {
    GLMatrix m;
    const int qmax = (1 << bits) - 1;
    const float scale = bits == 8 ? 1.0f / 256.0f : 1.0f / 16.0f, bias = -0.5f;
    const int bb = 4 + group * bits / 8;
    m.blocks.assign((size_t)rows * (cols / group) * bb, 0);
    m.plain.assign((size_t)rows * cols, 0.0);
    for (int r = 0; r < rows; ++r)
        for (int g = 0; g < cols; g += group) {
            uint8_t* blk = m.blocks.data() + ((size_t)r * (cols / group) + g / group) * bb;
            const uint16_t hs = f2h(scale), hb = f2h(bias);
            std::memcpy(blk, &hs, 2);
            std::memcpy(blk + 2, &hb, 2);
            for (int i = 0; i < group; ++i) {
                const uint32_t code = (uint32_t)(((r * 13 + (g + i) * 7 + seed * 19) & 0xFFFF) % (qmax + 1));
                const int bit = i * bits;
                for (int b = 0; b < bits; ++b)
                    if ((code >> b) & 1u) blk[4 + ((bit + b) >> 3)] |= (uint8_t)(1u << ((bit + b) & 7));
                m.plain[(size_t)r * cols + g + i] = (double)code * (double)scale + (double)bias;
            }
        }
    for (int r = 0; r < rows; ++r)   // the container holds W . H: un-rotate along the input columns
        for (int c = 0; c < cols; c += 32) fwht32(&m.plain[(size_t)r * cols + c]);
    if (foldOutput) {                // and H . W when the output rotation is folded into the rows
        std::vector<double> col(32);
        for (int c = 0; c < cols; ++c)
            for (int r0 = 0; r0 < rows; r0 += 32) {
                for (int j = 0; j < 32; ++j) col[j] = m.plain[(size_t)(r0 + j) * cols + c];
                fwht32(col.data());
                for (int j = 0; j < 32; ++j) m.plain[(size_t)(r0 + j) * cols + c] = col[j];
            }
    }
    return m;
}

static void test_gpu_moe_group_latent(QWHal& hal, int rows) {
    const int H = 64, NG = 4, L = 64, E = 32, K = 4, I = 64, IS = 64;
    std::vector<GLMatrix> dM, uM, guM, dnM;
    for (int g = 0; g < NG; ++g) dM.push_back(gl_matrix(L, H, 8, 32, 1 + g, true));
    for (int g = 0; g < NG; ++g) uM.push_back(gl_matrix(H, L, 8, 32, 11 + g, false));
    for (int e = 0; e < E; ++e) guM.push_back(gl_matrix(2 * I, L, 4, 64, 21 + e, false));
    for (int e = 0; e < E; ++e) dnM.push_back(gl_matrix(L, I, 4, 64, 61 + e, true));
    const GLMatrix shGate = gl_matrix(IS, H, 8, 32, 101, false), shUp = gl_matrix(IS, H, 8, 32, 102, false), shDn = gl_matrix(H, IS, 8, 32, 103, false);
    auto cat = [](const std::vector<GLMatrix>& v) {
        std::vector<uint8_t> o;
        for (const GLMatrix& m : v) o.insert(o.end(), m.blocks.begin(), m.blocks.end());
        return o;
    };
    const std::vector<uint8_t> dB = cat(dM), uB = cat(uM), guB = cat(guM), dnB = cat(dnM);
    std::vector<uint8_t> shguB = shGate.blocks;
    shguB.insert(shguB.end(), shUp.blocks.begin(), shUp.blocks.end());
    std::vector<int32_t> labels(E);
    for (int e = 0; e < E; ++e) labels[e] = e % NG;
    std::vector<float> gateW((size_t)E * H), shScalar(H);
    for (int i = 0; i < E * H; ++i) gateW[i] = (float)((i * 17) % 19 - 9) * 0.0625f;
    for (int h = 0; h < H; ++h) shScalar[h] = (float)((h * 11) % 13 - 6) * 0.0625f;
    // the operator's input as the reference's test gives it: f32 rows un-rotated and rotated, the f16 copy from 64 rows on
    std::vector<float> xPlainF((size_t)rows * H), xRotF((size_t)rows * H);
    std::vector<uint16_t> x16((size_t)rows * H);
    std::vector<double> xp((size_t)rows * H);
    for (int t = 0; t < rows; ++t) {
        std::vector<double> r(H);
        for (int h = 0; h < H; ++h) {
            xPlainF[(size_t)t * H + h] = (float)(((t * H + h) * 7 + rows) % 23 - 11) * 0.1f;
            xp[(size_t)t * H + h] = r[h] = (double)xPlainF[(size_t)t * H + h];
        }
        for (int o = 0; o < H; o += 32) fwht32(&r[o]);
        for (int h = 0; h < H; ++h) { xRotF[(size_t)t * H + h] = (float)r[h]; x16[(size_t)t * H + h] = f2h((float)r[h]); }
    }
    auto silu = [](double g) { return g / (1 + std::exp(-g)); };
    auto linear = [](const double* x, const std::vector<double>& w, int out, int in) {
        std::vector<double> y(out, 0.0);
        for (int o = 0; o < out; ++o) {
            double a = 0;
            for (int i = 0; i < in; ++i) a += w[(size_t)o * in + i] * x[i];
            y[o] = a;
        }
        return y;
    };
    std::vector<double> ref((size_t)rows * H, 0.0);
    for (int t = 0; t < rows; ++t) {
        const double* xt = &xp[(size_t)t * H];
        std::vector<double> logit(E), p(E);
        double mx = -1e300, tot = 0;
        for (int e = 0; e < E; ++e) {
            double a = 0;
            for (int h = 0; h < H; ++h) a += (double)gateW[(size_t)e * H + h] * xt[h];
            logit[e] = a;
            mx = std::fmax(mx, a);
        }
        for (int e = 0; e < E; ++e) { p[e] = std::exp(logit[e] - mx); tot += p[e]; }
        std::vector<int> chosen;
        std::vector<bool> taken(E, false);
        double wsum = 0;
        for (int r = 0; r < K; ++r) {
            int best = -1;
            for (int e = 0; e < E; ++e)
                if (!taken[e] && (best < 0 || p[e] > p[best])) best = e;
            taken[best] = true;
            chosen.push_back(best);
            wsum += p[best] / tot;
        }
        std::vector<std::vector<double>> z(NG, std::vector<double>(L, 0.0)), dcache(NG);
        std::vector<bool> active(NG, false);
        for (int r = 0; r < K; ++r) {
            const int e = chosen[r], g = labels[e];
            if (dcache[g].empty()) dcache[g] = linear(xt, dM[g].plain, L, H);
            const std::vector<double> gu = linear(dcache[g].data(), guM[e].plain, 2 * I, L);
            std::vector<double> act(I);
            for (int i = 0; i < I; ++i) act[i] = silu(gu[i]) * gu[I + i];
            const std::vector<double> y = linear(act.data(), dnM[e].plain, L, I);
            const double wk = (p[e] / tot) / wsum;
            for (int l = 0; l < L; ++l) z[g][l] += wk * y[l];
            active[g] = true;
        }
        std::vector<double> acc(H, 0.0);
        for (int g = 0; g < NG; ++g) {
            if (!active[g]) continue;
            const std::vector<double> y = linear(z[g].data(), uM[g].plain, H, L);
            for (int h = 0; h < H; ++h) acc[h] += y[h];
        }
        const std::vector<double> sg = linear(xt, shGate.plain, IS, H), su = linear(xt, shUp.plain, IS, H);
        std::vector<double> sh(IS);
        for (int i = 0; i < IS; ++i) sh[i] = silu(sg[i]) * su[i];
        const std::vector<double> shared = linear(sh.data(), shDn.plain, H, IS);
        double gl = 0;
        for (int h = 0; h < H; ++h) gl += (double)shScalar[h] * xt[h];
        const double gate = 1.0 / (1.0 + std::exp(-gl));
        for (int h = 0; h < H; ++h) ref[(size_t)t * H + h] = acc[h] + gate * shared[h];
    }
    QWHipEncoder enc = hal.begin();
    const int pairs = rows * K, gpairs = rows * NG, mt = QWGemm::moeMaxTiles(E, pairs), gmt = QWGemm::moeMaxTiles(NG, gpairs);
    DeviceBuf dd(hal, dB.size()), du(hal, uB.size()), dgu(hal, guB.size()), ddn(hal, dnB.size()), dshgu(hal, shguB.size()), dshdn(hal, shDn.blocks.size());
    DeviceBuf dr(hal, gateW.size() * 4), dsc(hal, shScalar.size() * 4), dlab(hal, labels.size() * 4), dx(hal, x16.size() * 2), dout(hal, (size_t)rows * H * 4);
    DeviceBuf dlog(hal, (size_t)rows * E * 4), didx(hal, pairs * 4), dw(hal, pairs * 4), dact(hal, (size_t)pairs * I * 2);
    DeviceBuf doff(hal, (E + 1) * 4), dsp(hal, pairs * 4), dst(hal, pairs * 4), dinv(hal, pairs * 4), dte(hal, mt * 4), dtr(hal, mt * 4), dtc(hal, 16);
    DeviceBuf ddnhi(hal, (size_t)pairs * L * 4);
    DeviceBuf dxr(hal, (size_t)rows * H * 4), dxpl(hal, (size_t)rows * H * 4), dgid(hal, gpairs * 4), dprow(hal, pairs * 4), dones(hal, gpairs * 4);
    DeviceBuf dxl(hal, (size_t)gpairs * L * 2), dzl(hal, (size_t)gpairs * L * 2), dnax(hal, (size_t)rows * H * 2), dgate(hal, (size_t)rows * 4);
    DeviceBuf dgush(hal, (size_t)rows * 2 * IS * 4), dactsh(hal, (size_t)rows * IS * 4), dshared(hal, (size_t)rows * H * 4);
    DeviceBuf dgoff(hal, (NG + 1) * 4), dgsp(hal, gpairs * 4), dgst(hal, gpairs * 4), dginv(hal, gpairs * 4), dgte(hal, gmt * 4), dgtr(hal, gmt * 4), dgtc(hal, 16);
    DeviceBuf drows2(hal, pairs * 4), dup(hal, (size_t)gpairs * H * 4), dxe(hal, (size_t)rows * H * 2);
    upload(enc, dd, dB.data(), dB.size());
    upload(enc, du, uB.data(), uB.size());
    upload(enc, dgu, guB.data(), guB.size());
    upload(enc, ddn, dnB.data(), dnB.size());
    upload(enc, dshgu, shguB.data(), shguB.size());
    upload(enc, dshdn, shDn.blocks.data(), shDn.blocks.size());
    upload(enc, dr, gateW.data(), gateW.size() * 4);
    upload(enc, dsc, shScalar.data(), shScalar.size() * 4);
    upload(enc, dlab, labels.data(), labels.size() * 4);
    upload(enc, dx, x16.data(), x16.size() * 2);
    upload(enc, dxpl, xPlainF.data(), xPlainF.size() * 4);
    upload(enc, dxr, xRotF.data(), xRotF.size() * 4);
    const std::vector<float> ones(gpairs, 1.0f);
    upload(enc, dones, ones.data(), ones.size() * 4);
    auto view = [](DeviceBuf& b, int n, int k, int bits, int group) { return *QWWeightView::make(QWTensorValue::make(b.p, b.bytes, QWDType::q4g), n, k, bits, group, true); };
    auto i32 = [](DeviceBuf& b, size_t n) { return QWTensorValue::make(b.p, n, QWDType::i32); };
    auto f32 = [](DeviceBuf& b, size_t n) { return QWTensorValue::make(b.p, n, QWDType::f32); };
    auto f16 = [](DeviceBuf& b, size_t n) { return QWTensorValue::make(b.p, n, QWDType::f16); };
    QWMoEOperator::GroupLatentWeights gw;
    gw.routed.router = f32(dr, gateW.size());
    gw.routed.gateUp = view(dgu, E * 2 * I, L, 4, 64);
    gw.routed.down = view(ddn, E * L, I, 4, 64);
    gw.routed.hidden = H; gw.routed.experts = E; gw.routed.topK = K; gw.routed.intermediate = I;
    gw.latentD = view(dd, NG * L, H, 8, 32);
    gw.latentU = view(du, NG * H, L, 8, 32);
    gw.latentLabels = i32(dlab, E);
    gw.numLatentGroups = NG;
    gw.latentDim = L;
    gw.sharedGateUp = view(dshgu, 2 * IS, H, 8, 32);
    gw.sharedDown = view(dshdn, H, IS, 8, 32);
    gw.sharedGateScalar = f32(dsc, H);
    gw.sharedIntermediate = IS;
    QWMoEOperator::Scratch s;
    s.logits = f32(dlog, (size_t)rows * E);
    s.idx = i32(didx, pairs);
    s.wts = f32(dw, pairs);
    s.act16 = f16(dact, (size_t)pairs * I);
    s.expOff = i32(doff, E + 1);
    s.sortedPair = i32(dsp, pairs);
    s.sortedTok = i32(dst, pairs);
    s.invPerm = i32(dinv, pairs);
    s.tileE = i32(dte, mt);
    s.tileR = i32(dtr, mt);
    s.tileCount = i32(dtc, 4);
    s.dnHi = f32(ddnhi, (size_t)pairs * L);
    QWMoEOperator::GroupLatentScratch gs;
    gs.xRot32 = f32(dxr, (size_t)rows * H);
    gs.xPlain32 = f32(dxpl, (size_t)rows * H);
    gs.groupIds = i32(dgid, gpairs);
    gs.pairRows = i32(dprow, pairs);
    gs.onesRoute = f32(dones, gpairs);
    gs.xLatent16 = f16(dxl, (size_t)gpairs * L);
    gs.zLatent16 = f16(dzl, (size_t)gpairs * L);
    gs.naxX16 = f16(dnax, (size_t)rows * H);
    gs.gate = f32(dgate, rows);
    gs.guSh32 = f32(dgush, (size_t)rows * 2 * IS);
    gs.actSh32 = f32(dactsh, (size_t)rows * IS);
    gs.shared = f32(dshared, (size_t)rows * H);
    gs.gExpOff = i32(dgoff, NG + 1);
    gs.gSortedPair = i32(dgsp, gpairs);
    gs.gSortedTok = i32(dgst, gpairs);
    gs.gInvPerm = i32(dginv, gpairs);
    gs.gTileE = i32(dgte, gmt);
    gs.gTileR = i32(dgtr, gmt);
    gs.gTileCount = i32(dgtc, 4);
    gs.rows2 = i32(drows2, pairs);
    gs.upAcc = f32(dup, (size_t)gpairs * H);
    gs.xe16 = f16(dxe, (size_t)rows * H);
    const QWTensorValue pre16 = f16(dx, x16.size());
    const QWMoEOperator::Input xt = QWMoEOperator::Input::preRotated(gs.xPlain32, gs.xRot32, rows >= 64 ? &pre16 : nullptr);
    const QWTensorValue out = f32(dout, (size_t)rows * H);
    QWMoEOperator::encodeResidentGroupLatent(enc, hal, gw, s, gs, xt, out, rows);
    std::vector<float> got((size_t)rows * H);
    download(enc, got.data(), dout, got.size() * 4);
    double worst = 0, wantMax = 0;
    for (size_t i = 0; i < got.size(); ++i) { worst = std::fmax(worst, std::fabs((double)got[i] - ref[i])); wantMax = std::fmax(wantMax, std::fabs(ref[i])); }
    const double rel = worst / std::fmax(1e-6, wantMax);
    std::printf("moe encodeResidentGroupLatent rows=%d maxAbs %.3e wantMax %.3e rel %.3e\n", rows, worst, wantMax, rel);
    CHECK(rel < (rows >= 64 ? 0.01 : 0.002));
    {   // a label table shorter than the experts is refused before any launch
        QWMoEOperator::GroupLatentWeights bad = gw;
        bad.latentLabels = i32(dlab, E - 1);
        bool threw = false;
        try { QWMoEOperator::encodeResidentGroupLatent(enc, hal, bad, s, gs, xt, out, rows); } catch (const QWGemmError&) { threw = true; }
        CHECK(threw);
    }
    hal.end(enc);
}

// f32-activation doors and the head: encodeHQ4F32V4 (epilogues 0 and 3), encodeH32F32, encodeHeadArgmax on the closed-form bank
static void test_gpu_f32_doors(QWHal& hal) {
    const int N = 96, Kc = 128, rows = 3;
    const std::vector<uint8_t> bank = cf_bank(N, Kc);
    std::vector<float> x((size_t)rows * Kc);
    for (int t = 0; t < rows; ++t)
        for (int c = 0; c < Kc; ++c) x[(size_t)t * Kc + c] = (float)(((t * 29 + c * 5) % 23) - 11) * 0.08f;
    std::vector<double> y0((size_t)rows * N);
    for (int t = 0; t < rows; ++t)
        for (int n = 0; n < N; ++n) {
            double s = 0;
            for (int c = 0; c < Kc; ++c) s += cf_weight(n, c) * (double)x[(size_t)t * Kc + c];
            y0[(size_t)t * N + n] = s;
        }
    QWHipEncoder enc = hal.begin();
    DeviceBuf dbank(hal, bank.size()), dx(hal, x.size() * 4), dy(hal, y0.size() * 4), dtok(hal, 64);
    upload(enc, dbank, bank.data(), bank.size());
    upload(enc, dx, x.data(), x.size() * 4);
    const auto view = QWWeightView::make(QWTensorValue::make(dbank.p, bank.size(), QWDType::q4g), N, Kc, 4, 32, true);
    CHECK(view.has_value());
    const QWTensorValue xt = QWTensorValue::make(dx.p, x.size(), QWDType::f32), yt = QWTensorValue::make(dy.p, y0.size(), QWDType::f32);
    std::vector<float> got(y0.size());
    QWGemm::encodeHQ4F32V4(enc, hal, *view, xt, yt, rows);
    download(enc, got.data(), dy, got.size() * 4);
    for (size_t i = 0; i < got.size(); ++i) CHECK(std::fabs((double)got[i] - y0[i]) <= 1e-4 * std::fmax(1.0, std::fabs(y0[i])));
    // epilogue 3: silu(y / 2) then the rotation over each 32 consecutive outputs
    QWGemm::encodeHQ4F32V4(enc, hal, *view, xt, yt, rows, 3, 2.0f);
    download(enc, got.data(), dy, got.size() * 4);
    for (int t = 0; t < rows; ++t)
        for (int g = 0; g < N / 32; ++g) {
            double v[32];
            for (int i = 0; i < 32; ++i) {
                const double z = y0[(size_t)t * N + g * 32 + i] / 2.0;
                v[i] = z / (1.0 + std::exp(-z));
            }
            fwht32(v);
            for (int i = 0; i < 32; ++i) CHECK(std::fabs((double)got[(size_t)t * N + g * 32 + i] - v[i]) <= 1e-4 * std::fmax(1.0, std::fabs(v[i])));
        }
    // the standalone rotation is an involution
    QWGemm::encodeHQ4F32V4(enc, hal, *view, xt, yt, rows);
    QWGemm::encodeH32F32(enc, hal, yt, yt, rows, N);
    QWGemm::encodeH32F32(enc, hal, yt, yt, rows, N);
    download(enc, got.data(), dy, got.size() * 4);
    for (size_t i = 0; i < got.size(); ++i) CHECK(std::fabs((double)got[i] - y0[i]) <= 1e-4 * std::fmax(1.0, std::fabs(y0[i])));
    // head: the token is the first maximum of the logits it leaves behind
    QWGemmAQ::encodeHeadArgmax(enc, hal, *view, xt, yt, QWTensorValue::make(dtok.p, 16, QWDType::i32), rows);
    download(enc, got.data(), dy, got.size() * 4);
    int32_t tok[16];
    download(enc, tok, dtok, 64);
    for (int t = 0; t < rows; ++t) {
        int best = 0;
        for (int n = 1; n < N; ++n)
            if (got[(size_t)t * N + n] > got[(size_t)t * N + best]) best = n;
        CHECK(tok[t] == best);
    }
    const QWTensorValue x16 = QWTensorValue::make(dx.p, x.size(), QWDType::f16);
    CHECK_THROWS(QWGemm::encodeHQ4F32V4(enc, hal, *view, x16, yt, rows), QWGemmError, QWGemmError::badWeights);
    CHECK_THROWS(QWGemm::encodeHQ4F32V4(enc, hal, *view, xt, yt, rows, 7), QWGemmError, QWGemmError::badShape);
    hal.end(enc);
}

// encodeDenseProjF32: 64 rows take the cast + matrix-core GEMM, 5 rows the f32 GEMV; both against the closed-form bank
// QWGemmAQ.encodeEmbedAQ on the reference's own table (Tests/QWGEMMTests/QWAQEmbedGatherTests.swift:52-99): 8-bit group 64,
// code of column i of group g of row r = (3 i + 7 r + 13 g) mod 256, header 1025/4096 and -683/4096
static void test_gpu_embed(QWHal& hal) {
    const int hidden = 256, vocab = 8, hc = 3, bits = 8, group = 64, rows = 3;
    const int bb = 4 + group * bits / 8, groups = hidden / group;
    std::vector<uint8_t> table((size_t)vocab * groups * bb);
    const uint16_t hs = f2h(1025.0f / 4096.0f), hb = f2h(-683.0f / 4096.0f);
    for (int r = 0; r < vocab; ++r)
        for (int g = 0; g < groups; ++g) {
            uint8_t* p = &table[((size_t)r * groups + g) * bb];
            std::memcpy(p, &hs, 2);
            std::memcpy(p + 2, &hb, 2);
            for (int i = 0; i < group; ++i) p[4 + i] = (uint8_t)((i * 3 + r * 7 + g * 13) % 256);
        }
    const int32_t tokens[rows] = {0, 3, 7};
    QWHipEncoder enc = hal.begin();
    DeviceBuf dt(hal, table.size()), dtok(hal, sizeof(tokens)), dout(hal, (size_t)rows * hc * hidden * 4);
    upload(enc, dt, table.data(), table.size());
    upload(enc, dtok, tokens, sizeof(tokens));
    const QWTensorValue blocks = QWTensorValue::make(dt.p, table.size() / 2, QWDType::f16);
    const QWTensorValue tok = QWTensorValue::make(dtok.p, rows, QWDType::i32);
    const QWTensorValue out = QWTensorValue::make(dout.p, (size_t)rows * hc * hidden, QWDType::f32);
    QWGemmAQ::encodeEmbedAQ(enc, hal, blocks, tok, out, hidden, hc, bits, group, rows);
    std::vector<float> got((size_t)rows * hc * hidden);
    download(enc, got.data(), dout, got.size() * 4);
    const double sc = h2f(hs), bi = h2f(hb), ulp = 0.000000059604644775390625;
    for (int t = 0; t < rows; ++t)
        for (int d = 0; d < hidden; ++d) {
            const double code = (double)(((d % group) * 3 + tokens[t] * 7 + (d / group) * 13) % 256);
            const double want = code * sc + bi;
            const double tol = std::fabs(code * sc) * ulp + std::fmax(std::fabs(want), std::fabs(bi)) * ulp + 1e-30;
            for (int c = 0; c < hc; ++c) CHECK(std::fabs((double)got[((size_t)t * hc + c) * hidden + d] - want) <= tol);
        }
    bool threw = false;
    try { QWGemmAQ::encodeEmbedAQ(enc, hal, blocks, tok, out, hidden, hc, 5, group, rows); } catch (const QWGemmError&) { threw = true; }
    CHECK(threw);
    threw = false;
    try { QWGemmAQ::encodeEmbedAQ(enc, hal, blocks, tok, out, 96, hc, bits, group, rows); } catch (const QWGemmError&) { threw = true; }
    CHECK(threw);
    hal.end(enc);
}

static void test_gpu_dense_proj_f32(QWHal& hal) {
    const int N = 128, Kc = 128;
    const std::vector<uint8_t> bank = cf_bank(N, Kc);
    QWHipEncoder enc = hal.begin();
    DeviceBuf dbank(hal, bank.size()), dx(hal, 64 * Kc * 4), dx16(hal, 64 * Kc * 2), dy(hal, 64 * N * 4);
    upload(enc, dbank, bank.data(), bank.size());
    const auto view = QWWeightView::make(QWTensorValue::make(dbank.p, bank.size(), QWDType::q4g), N, Kc, 4, 32, true);
    CHECK(view.has_value());
    for (int rows : {64, 5}) {
        std::vector<float> x((size_t)rows * Kc);
        for (int t = 0; t < rows; ++t)
            for (int c = 0; c < Kc; ++c) x[(size_t)t * Kc + c] = (float)(((t * 31 + c * 7) % 29) - 14) / 16.0f;   // exact in f16
        upload(enc, dx, x.data(), x.size() * 4);
        const QWTensorValue xt = QWTensorValue::make(dx.p, x.size(), QWDType::f32), yt = QWTensorValue::make(dy.p, (size_t)rows * N, QWDType::f32);
        QWGemm::encodeDenseProjF32(enc, hal, *view, xt, yt, QWTensorValue::make(dx16.p, 64 * Kc, QWDType::f16), rows);
        std::vector<float> got((size_t)rows * N);
        download(enc, got.data(), dy, got.size() * 4);
        for (int t = 0; t < rows; ++t)
            for (int n = 0; n < N; ++n) {
                double s = 0;
                for (int c = 0; c < Kc; ++c) s += cf_weight(n, c) * (double)x[(size_t)t * Kc + c];
                CHECK(std::fabs((double)got[(size_t)t * N + n] - s) <= 1e-3 * std::fmax(1.0, std::fabs(s)));
            }
    }
    hal.end(enc);
}

int main(int argc, char** argv) {
    const bool gpu = argc > 1 && std::strcmp(argv[1], "--gpu") == 0;
    test_plan_table();
    test_weight_view();
    const bool nodevice = argc > 1 && std::strcmp(argv[1], "--cpu-nodevice") == 0;
    if (!gpu) {
        test_error_mapping();
        if (nodevice) test_hal_refuses_without_device();
    } else {
        QWHal hal(0);
        std::printf("device: %s (%s), %u CUs\n", hal.caps.name, hal.caps.arch, hal.caps.compute_units);
        test_gpu_hq4_gemv(hal);
        test_gpu_moe_resident(hal, 3);    // decode / verify path
        test_gpu_moe_resident(hal, 40);   // grouped prefill path (fused gate_up + SwiGLU)
        test_gpu_moe_latent(hal, 3);      // latent bottleneck, routed GEMVs
        test_gpu_moe_latent(hal, 40);     // latent bottleneck, grouped GEMMs and batched f32 projections
        for (int rows : {1, 2, 4, 16, 64}) test_gpu_moe_group_latent(hal, rows);   // the row counts of the reference's test
        test_gpu_f32_doors(hal);
        test_gpu_dense_proj_f32(hal);
        test_gpu_embed(hal);
    }
    std::printf("%d checks, %d failed\n", g_checks, g_failed);
    return g_failed ? 1 : 0;
}
