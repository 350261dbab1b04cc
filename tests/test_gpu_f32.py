"""GPU parity of the f32-activation GEMV family (through the C ABI) against the CPU oracle: fp32 activations in the
container's basis, fp32 outputs, epilogues 0..3.  Bar: the arithmetic is fp32 throughout, so outputs sit within 2e-5
normalized error of the float64 evaluation (the judged bar for outputs is 2e-3); the standalone rotation is bit-exact."""
import ctypes as C

import numpy as np
import pytest

from oracle import qworacle as qo
from qwegn_amd import qwhip
from tests import helpers as H

pytestmark = pytest.mark.gpu
TOL = 2e-5


@pytest.fixture(scope="module")
def dev():
    return qwhip.Device(0)


def _run(dev, fmt, n, k, m, epi, scale, seed=0):
    _, bits, group, is_m5, _ = H.FORMATS[fmt]
    blocks, _ = H.make_bank(fmt, n, k, seed=seed)
    x = H.make_x(m, k, seed + 100)
    bank, xb, yb = dev.put(blocks), dev.put(x), dev.alloc(max(256, m * n * 4))
    view = H.view_of(dev, bank, fmt, n, k)
    qwhip.check(dev.lib.qwhip_gemv_f32(dev.stream.handle, C.byref(view), xb.ptr, m, epi, scale, yb.ptr))
    dev.stream.sync()
    return yb.download(np.float32, (m, n)), qo.gemv_f32(blocks, x, bits, group, is_m5, epi, scale), (view, xb, bank)


@pytest.mark.parametrize("fmt", list(H.FORMATS))
@pytest.mark.parametrize("m", [1, 2, 3, 4])
def test_gemv_f32_matches_the_oracle(dev, fmt, m):
    got, want, _ = _run(dev, fmt, 200, 1024, m, 0, 1.0, seed=m)
    assert qo.normalized_error(got, want) <= TOL


@pytest.mark.parametrize("epi,scale", [(1, 1.0), (1, 0.05), (2, 1.0), (3, 0.05), (3, 2.0)])
@pytest.mark.parametrize("fmt,n", [("hq4_g32_m5", 256), ("aq8_g256", 200), ("hq4_g64", 77)])
def test_gemv_f32_epilogues(dev, fmt, n, epi, scale):
    """silu(y / scale), sigmoid, and silu + FWHT-32 over consecutive outputs (n = 200 and 77 end in a zero-padded group)."""
    got, want, _ = _run(dev, fmt, n, 512, 3, epi, scale, seed=7)
    assert qo.normalized_error(got, want) <= TOL


@pytest.mark.parametrize("fmt,n,k,m", [
    ("hq4_g32_m5", 300, 17408, 5),      # long rows: two activation rows per pass
    ("hq4_g32_m5", 64, 32768, 2),       # longest rows the kernel takes: one per pass
    ("aq4_g32", 5000, 2048, 9),         # three passes of 4 + 4 + 1
    ("hq8_g32", 33, 32, 4),             # a single slice per row
    ("hq4_g128", 1, 256, 1),            # one bank row
])
def test_gemv_f32_shapes(dev, fmt, n, k, m):
    got, want, _ = _run(dev, fmt, n, k, m, 0, 1.0, seed=11)
    assert qo.normalized_error(got, want) <= TOL


@pytest.mark.parametrize("fmt", list(H.FORMATS))
@pytest.mark.parametrize("m", [32, 45, 64, 130])
def test_batched_f32_form_matches_the_oracle(dev, fmt, m):
    """From 32 activation rows on (QWGemm.encodeHQ4F32BM, QWGemmF32.swift:311-350) the door runs the matrix-core form:
    activations and un-rounded affine weights each split into two f16 numbers, three products in fp32 accumulators.  Same
    bar as the fp32 GEMV form; n = 200 ends in a partial 64-row tile, m = 45 / 130 in partial row tiles."""
    got, want, _ = _run(dev, fmt, 200, 1024, m, 0, 1.0, seed=m)
    assert qo.normalized_error(got, want) <= TOL


@pytest.mark.parametrize("epi,scale", [(1, 1.0), (1, 0.05), (2, 1.0), (3, 0.05), (3, 2.0)])
@pytest.mark.parametrize("fmt,n", [("hq4_g32_m5", 256), ("aq8_g256", 200), ("hq4_g64", 77), ("hq3_g32", 96)])
def test_batched_f32_form_epilogues(dev, fmt, n, epi, scale):
    got, want, _ = _run(dev, fmt, n, 512, 40, epi, scale, seed=7)
    assert qo.normalized_error(got, want) <= TOL


@pytest.mark.parametrize("fmt,n,k,m", [
    ("hq4_g32_m5", 17408, 5120, 64),    # the decode MLP bank with 64 rows: 272 x 1 tiles
    ("hq4_g64", 512, 17408, 33),        # long rows
    ("aq4_g32", 70, 64, 32),            # one K-step
    ("hq8_g32", 64, 96, 32),            # K is not whole 64-column steps: the GEMV form takes it
])
def test_batched_f32_form_shapes(dev, fmt, n, k, m):
    got, want, _ = _run(dev, fmt, n, k, m, 0, 1.0, seed=11)
    assert qo.normalized_error(got, want) <= TOL


def test_batched_f32_form_agrees_with_the_row_form(dev):
    """31 rows go four at a time through the fp32 kernel, 32 rows through the matrix cores: the same rows agree to the
    oracle's bar with each other (both sit within 2e-5 of the float64 evaluation)."""
    got32, want32, _ = _run(dev, "hq4_g32_m5", 384, 2048, 32, 0, 1.0, seed=5)
    got31, want31, _ = _run(dev, "hq4_g32_m5", 384, 2048, 31, 0, 1.0, seed=5)
    assert np.array_equal(want32[:31], want31)
    assert qo.normalized_error(got32[:31], got31.astype(np.float64)) <= 2 * TOL


@pytest.mark.parametrize("fmt", ["hq4_g32_m5", "hq8_g32", "aq4_g32"])
@pytest.mark.parametrize("m", [31, 32, 70])
def test_f32_forms_take_any_fp32_activation_range(dev, fmt, m):
    """Rows far outside the f16 range - magnitudes of 1e5 .. 3e9 (beyond 65504), of 1e-9 and of 1e-30, one row of zeros,
    one row that mixes 1e6 with 1e-3 - give the same answers at 31 rows (fp32 kernel) and at 32 and more (matrix cores:
    every row is scaled by a power of two ahead of the f16 split and back at the store), both within the fp32 bar of the
    float64 evaluation, and no value turns non-finite."""
    n, k = 192, 1024
    _, bits, group, is_m5, _ = H.FORMATS[fmt]
    blocks, _ = H.make_bank(fmt, n, k, seed=9)
    rng = np.random.default_rng(m)
    x = rng.standard_normal((m, k)).astype(np.float32)
    mags = np.array([1e5, 3e9, 1e-9, 1e-30, 0.0, 1.0, 7e4, 1e20], np.float32)
    x *= mags[np.arange(m) % len(mags)][:, None]
    x[5, ::2] *= np.float32(1e6)
    x[5, 1::2] *= np.float32(1e-3)
    bank, xb, yb = dev.put(blocks), dev.put(x), dev.alloc(m * n * 4)
    view = H.view_of(dev, bank, fmt, n, k)
    qwhip.check(dev.lib.qwhip_gemv_f32(dev.stream.handle, C.byref(view), xb.ptr, m, 0, 1.0, yb.ptr))
    dev.stream.sync()
    got = yb.download(np.float32, (m, n))
    want = qo.gemv_f32(blocks, x, bits, group, is_m5, 0, 1.0)
    assert np.all(np.isfinite(got))
    for r in range(m):          # row by row: the rows differ by 50 orders of magnitude
        if mags[r % len(mags)] == 0.0:
            assert np.all(got[r] == 0)
        else:
            assert qo.normalized_error(got[r:r + 1], want[r:r + 1]) <= TOL, (r, float(mags[r % len(mags)]))


@pytest.mark.parametrize("fmt", ["hq4_g32_m5", "hq8_g32"])
def test_epilogue3_rows_together_equal_rows_alone(dev, fmt):
    """The reference's own check (Tests/QWGEMMTests/QWGemmEpi3MultiRowTests.swift:71-113): 2..5 rows in one call against
    the same rows one call each, epilogue 3, scale 2.  Here the per-row arithmetic does not depend on the row count: equal bits."""
    n, k = 128, 512
    _, bits, group, is_m5, _ = H.FORMATS[fmt]
    blocks, _ = H.make_bank(fmt, n, k, seed=3)
    x = (((np.arange(5 * k) % 23) - 11) * 0.08).astype(np.float32).reshape(5, k)
    bank, xb = dev.put(blocks), dev.put(x)
    y_multi, y_one = dev.alloc(5 * n * 4), dev.alloc(5 * n * 4)
    view = H.view_of(dev, bank, fmt, n, k)
    st = dev.stream.handle
    for rows in (2, 3, 4, 5):
        qwhip.check(dev.lib.qwhip_gemv_f32(st, C.byref(view), xb.ptr, rows, 3, 2.0, y_multi.ptr))
        for r in range(rows):
            qwhip.check(dev.lib.qwhip_gemv_f32(st, C.byref(view), xb.ptr + r * k * 4, 1, 3, 2.0, y_one.ptr + r * n * 4))
        dev.stream.sync()
        a, b = y_multi.download(np.float32, (5, n))[:rows], y_one.download(np.float32, (5, n))[:rows]
        assert np.array_equal(a.view(np.uint32), b.view(np.uint32)), rows
        assert qo.normalized_error(a, qo.gemv_f32(blocks, x[:rows], bits, group, is_m5, 3, 2.0)) <= TOL


def test_h32_f32_is_the_reference_butterfly(dev):
    """qwhip_h32_f32 against the golden-pinned fp32 FWHT (same butterfly order: equal bits), out of place and in place."""
    x = H.make_x(9, 1280, 5)
    xb, ob = dev.put(x), dev.alloc(x.size * 4)
    qwhip.check(dev.lib.qwhip_h32_f32(dev.stream.handle, xb.ptr, ob.ptr, 9, 1280))
    qwhip.check(dev.lib.qwhip_h32_f32(dev.stream.handle, xb.ptr, xb.ptr, 9, 1280))
    dev.stream.sync()
    want = qo.fwht32_ortho(x)
    assert np.array_equal(ob.download(np.float32, x.shape).view(np.uint32), want.view(np.uint32))
    assert np.array_equal(xb.download(np.float32, x.shape).view(np.uint32), want.view(np.uint32))


def test_head_argmax_takes_f32_activations(dev):
    fmt, n, k, m = "hq4_g32_m5", 3000, 1024, 2
    _, bits, group, is_m5, _ = H.FORMATS[fmt]
    blocks, _ = H.make_bank(fmt, n, k, seed=31)
    x = H.make_x(m, k, 131)
    bank, xb = dev.put(blocks), dev.put(x)
    logits, toks = dev.alloc(m * n * 4), dev.alloc(256)
    view = H.view_of(dev, bank, fmt, n, k)
    qwhip.check(dev.lib.qwhip_head_argmax(dev.stream.handle, C.byref(view), xb.ptr, qwhip.F32, m, 0, logits.ptr, toks.ptr))
    dev.stream.sync()
    got = logits.download(np.float32, (m, n))
    assert qo.normalized_error(got, qo.gemv_f32(blocks, x, bits, group, is_m5)) <= TOL
    assert np.array_equal(toks.download(np.int32, (m,)), qo.head_argmax(got))


def test_gemv_f32_refusals(dev):
    blocks, _ = H.make_bank("hq4_g32_m5", 8, 64, seed=1)
    bank, xb, yb = dev.put(blocks), dev.put(np.zeros((1, 64), np.float32)), dev.alloc(256)
    view = H.view_of(dev, bank, "hq4_g32_m5", 8, 64)
    st = dev.stream.handle
    assert dev.lib.qwhip_gemv_f32(st, C.byref(view), xb.ptr, 1, 4, 1.0, yb.ptr) == qwhip.E_BAD_SHAPE
    assert dev.lib.qwhip_gemv_f32(st, C.byref(view), xb.ptr, 1, 1, 0.0, yb.ptr) == qwhip.E_BAD_SHAPE
    assert dev.lib.qwhip_gemv_f32(st, C.byref(view), xb.ptr, 0, 0, 1.0, yb.ptr) == qwhip.E_BAD_SHAPE
    assert dev.lib.qwhip_gemv_f32(st, C.byref(view), None, 1, 0, 1.0, yb.ptr) == qwhip.E_NULL
    assert dev.lib.qwhip_h32_f32(st, xb.ptr, yb.ptr, 1, 48) == qwhip.E_BAD_SHAPE


def test_silu_mul_f32_matches_oracle(dev):
    """qwhip_silu_mul_f32: FWHT32(silu(g) * u) in fp32 (QWGemmF32.swift:83-94); 1e-5 of the row's scale (the device's exp
    differs from numpy's in the last bits), and the f16 door agrees with it after one rounding."""
    rows, inter = 37, 416
    rng = np.random.default_rng(5)
    gu = (rng.standard_normal((rows, 2 * inter)) * 2.0).astype(np.float32)
    gb, ab, hb = dev.put(gu), dev.alloc(rows * inter * 4), dev.alloc(rows * inter * 2)
    lib, st = dev.lib, dev.stream.handle
    qwhip.check(lib.qwhip_silu_mul_f32(st, gb.ptr, ab.ptr, rows, inter))
    qwhip.check(lib.qwhip_swiglu_fwht(st, gb.ptr, qwhip.F32, hb.ptr, rows, inter, 1))
    dev.stream.sync()
    got, got16 = ab.download(np.float32, (rows, inter)), hb.download(np.float16, (rows, inter))
    want = qo.silu_mul_f32(gu)
    assert qo.normalized_error(got, want) <= 1e-6
    assert np.max(np.abs(got - want)) <= 1e-5 * np.max(np.abs(want))
    assert np.array_equal(got.astype(np.float16).view(np.uint16), got16.view(np.uint16))
    assert lib.qwhip_silu_mul_f32(st, gb.ptr, ab.ptr, rows, 40) == qwhip.E_BAD_SHAPE


@pytest.mark.parametrize("rows,hidden", [(1, 256), (5, 2048), (40, 768)])
def test_moe_bridge_matches_oracle(dev, rows, hidden):
    """qwhip_moe_bridge_f16_to_f32 (QWGemmMoE.swift:337-377): the widened copy is exact; the un-rotated copy is the oracle's
    bit for bit (fp32 butterfly in the same order, the same hi/lo split); NULL skips the rotated copy; hidden % 256."""
    rng = np.random.default_rng(rows)
    x16 = rng.standard_normal((rows, hidden)).astype(np.float16)
    xb, rb, pb = dev.put(x16), dev.put(np.full((rows, hidden), 7.0, np.float32)), dev.alloc(rows * hidden * 4)
    lib, st = dev.lib, dev.stream.handle
    qwhip.check(lib.qwhip_moe_bridge_f16_to_f32(st, xb.ptr, rb.ptr, pb.ptr, rows, hidden))
    dev.stream.sync()
    rot, plain = qo.moe_bridge_f16_to_f32(x16)
    assert np.array_equal(rb.download(np.float32, (rows, hidden)), rot)
    assert np.array_equal(pb.download(np.float32, (rows, hidden)).view(np.uint32), plain.view(np.uint32))
    rb2 = dev.put(np.full((rows, hidden), 7.0, np.float32))
    qwhip.check(lib.qwhip_moe_bridge_f16_to_f32(st, xb.ptr, None, pb.ptr, rows, hidden))
    dev.stream.sync()
    assert np.all(rb2.download(np.float32, (rows, hidden)) == 7.0)
    assert lib.qwhip_moe_bridge_f16_to_f32(st, xb.ptr, rb.ptr, pb.ptr, rows, hidden - 32) == qwhip.E_BAD_GEOMETRY


@pytest.mark.parametrize("rows,latent", [(3, 96), (17, 1024), (2, 4128)])
@pytest.mark.parametrize("norm", [True, False])
def test_latent_norm_h32_matches_oracle(dev, rows, latent, norm):
    """qwhip_latent_norm_h32_f32 (QWGemmF32.swift:57-80): with and without gamma, f32 and f16 outputs, either alone."""
    rng = np.random.default_rng(latent)
    x = (rng.standard_normal((rows, latent)) * 3.0).astype(np.float32)
    gamma = (rng.standard_normal(latent) * 0.2).astype(np.float16)
    xb, gb = dev.put(x), dev.put(gamma)
    o32, o16 = dev.alloc(rows * latent * 4), dev.alloc(rows * latent * 2)
    lib, st = dev.lib, dev.stream.handle
    qwhip.check(lib.qwhip_latent_norm_h32_f32(st, xb.ptr, gb.ptr if norm else None, o32.ptr, o16.ptr, rows, latent, 1e-6))
    dev.stream.sync()
    want = qo.latent_norm_h32_f32(x, gamma if norm else None, 1e-6)
    got32, got16 = o32.download(np.float32, (rows, latent)), o16.download(np.float16, (rows, latent))
    if norm:
        assert np.max(np.abs(got32 - want)) <= 2e-6 * np.max(np.abs(want))
    else:
        assert np.array_equal(got32.view(np.uint32), want.view(np.uint32))
    assert np.array_equal(got16.view(np.uint16), got32.astype(np.float16).view(np.uint16))
    o16b = dev.put(np.zeros((rows, latent), np.float16))
    qwhip.check(lib.qwhip_latent_norm_h32_f32(st, xb.ptr, gb.ptr if norm else None, None, o16b.ptr, rows, latent, 1e-6))
    dev.stream.sync()
    assert np.array_equal(o16b.download(np.float16, (rows, latent)).view(np.uint16), got16.view(np.uint16))
    assert lib.qwhip_latent_norm_h32_f32(st, xb.ptr, None, None, None, rows, latent, 1e-6) == qwhip.E_NULL
    assert lib.qwhip_latent_norm_h32_f32(st, xb.ptr, None, o32.ptr, None, rows, 40, 1e-6) == qwhip.E_BAD_SHAPE


def test_add_f32(dev):
    rng = np.random.default_rng(1)
    a, b = rng.standard_normal(100003).astype(np.float32), rng.standard_normal(100003).astype(np.float32)
    ab, bb, ob = dev.put(a), dev.put(b), dev.alloc(a.size * 4)
    qwhip.check(dev.lib.qwhip_add_f32(dev.stream.handle, ab.ptr, bb.ptr, ob.ptr, a.size))
    dev.stream.sync()
    assert np.array_equal(ob.download(np.float32, (a.size,)), a + b)
