"""GPU parity of the prefill GEMM (f16 MFMA, fp32 accumulate) against the fp64 oracle, through the C ABI.
Bar: normalized error <= 2e-3 (bf16 / f16 stores); fp32 stores are held to 2e-5."""
import ctypes as C

import numpy as np
import pytest

from oracle import qworacle as qo
from qwegn_amd import qwhip
from tests import helpers as H

pytestmark = pytest.mark.gpu
TOL = 2e-3


@pytest.fixture(scope="module")
def dev():
    return qwhip.Device(0)


def run_gemm(dev, fmt, m, n, k, *, xdtype="bf16", ydtype="bf16", prerot=True, cfg=0, seed=0, workspace=True, workspace_bytes=None):
    blocks, w16 = H.make_bank(fmt, n, k, seed=seed)
    x32 = H.make_x(m, k, seed + 7)
    rotate = H.FORMATS[fmt][4]
    if xdtype == "bf16":
        x_val, x_host, xcode = qo.round_bf16(x32), qo.f32_to_bf16_bits(x32), qwhip.BF16
    else:
        x_host, xcode = x32.astype(np.float16), qwhip.F16
        x_val = x_host.astype(np.float32)
    if prerot or not rotate:
        # activations arrive in the container's basis; the kernel converts them to f16
        x_basis = x_val.astype(np.float16)
        flags = qwhip.X_PREROTATED
    else:
        x_basis = qo.fwht32_ortho(x_val).astype(np.float16)
        flags = 0
    flags |= (cfg << 8)
    ysize = {"bf16": 2, "f16": 2, "f32": 4}[ydtype]
    ycode = {"bf16": qwhip.BF16, "f16": qwhip.F16, "f32": qwhip.F32}[ydtype]
    bank, xb, yb = dev.put(blocks), dev.put(x_host), dev.alloc(m * n * ysize)
    ws = dev.alloc(workspace_bytes if workspace_bytes else m * k * 2) if workspace else None
    view = H.view_of(dev, bank, fmt, n, k)
    st = dev.lib.qwhip_gemm(dev.stream.handle, C.byref(view), xb.ptr, xcode, m, 0, yb.ptr, ycode, 0, flags,
                            ws.ptr if ws else None, ws.nbytes if ws else 0)
    out = None
    if st == qwhip.OK:
        dev.stream.sync()
        if ydtype == "bf16":
            out = qo.bf16_bits_to_f32(yb.download(np.uint16, (m, n)))
        elif ydtype == "f16":
            out = yb.download(np.float16, (m, n)).astype(np.float32)
        else:
            out = yb.download(np.float32, (m, n))
    for b in (bank, xb, yb, ws):
        if b is not None:
            b.free()
    ref = qo.matmul_ref_f64(x_basis, w16)
    return st, out, ref


@pytest.mark.parametrize("cfg", [1, 2, 3, 4, 5, 14, 15])
def test_gemm_hq4_tile_shapes_f32_out(dev, cfg):
    st, out, ref = run_gemm(dev, "hq4_g32_m5", 512, 640, 1024, ydtype="f32", cfg=cfg)
    assert st == qwhip.OK
    assert qo.normalized_error(out, ref) <= 2e-5


@pytest.mark.parametrize("m,n,k", [(1, 16, 64), (37, 48, 128), (300, 336, 192), (257, 1040, 320)])
def test_gemm_ragged_shapes(dev, m, n, k):
    st, out, ref = run_gemm(dev, "hq4_g32_m5", m, n, k, ydtype="f32")
    assert st == qwhip.OK
    assert qo.normalized_error(out, ref) <= 2e-5


@pytest.mark.parametrize("fmt", ["aq4_g32", "hq4_g64", "hq8_g32", "hq4_g128", "aq8_g256", "aq2_g64", "hq3_g32", "hq6_g32", "aq6_g128"])
@pytest.mark.parametrize("xdtype,ydtype", [("f16", "f16"), ("bf16", "bf16")])
def test_gemm_block_formats(dev, fmt, xdtype, ydtype):
    st, out, ref = run_gemm(dev, fmt, 192, 256, 768, xdtype=xdtype, ydtype=ydtype, seed=3)
    assert st == qwhip.OK
    assert qo.normalized_error(out, ref) <= TOL


@pytest.mark.parametrize("fmt", ["aq2_g64", "hq3_g32", "hq6_g32", "aq6_g128"])
@pytest.mark.parametrize("cfg,xdtype,workspace", [(15, "f16", True), (0, "bf16", False), (1, "f16", True), (2, "f16", True), (3, "f16", True)])
def test_gemm_narrow_and_six_bit_streams_on_every_kernel(dev, fmt, cfg, xdtype, workspace):
    """2-, 3- and 6-bit streams (codes cut out of the slice's words, also across word boundaries) on the unpipelined kernel
    (f16, and bf16 converted in the tile) and on the DMA-fed kernel's tile shapes, fp32 out, ragged in both directions."""
    st, out, ref = run_gemm(dev, fmt, 300, 336, 384, xdtype=xdtype, ydtype="f32", cfg=cfg, seed=11, workspace=workspace)
    assert st == qwhip.OK
    assert qo.normalized_error(out, ref) <= 2e-5


@pytest.mark.parametrize("fmt", ["hq4_g32_m5", "aq4_g32", "hq8_g32", "hq4_g64", "aq2_g64", "hq3_g32", "hq6_g32"])
@pytest.mark.parametrize("cfg", [1, 5])
def test_gemm_pingpong_kernel_ragged_tiles(dev, fmt, cfg):
    """The 8-wave ping-pong kernel (256 x 320 and 128 x 320 tiles; the 8-bit containers run the DMA-fed kernel at these
    shapes) on a shape whose last tile row holds one 64-row block and whose last tile column is ragged, for every weight
    format family."""
    st, out, ref = run_gemm(dev, fmt, 320, 400, 640, xdtype="f16", ydtype="f32", cfg=cfg, seed=5)
    assert st == qwhip.OK
    assert qo.normalized_error(out, ref) <= 2e-5
    st, out, ref = run_gemm(dev, fmt, 64, 320, 64, xdtype="bf16", ydtype="bf16", cfg=cfg, seed=6)   # a single K-step
    assert st == qwhip.OK
    assert qo.normalized_error(out, ref) <= TOL


@pytest.mark.parametrize("fmt", ["hq4_g32_m5", "aq4_g32", "hq4_g64", "aq2_g64", "hq3_g32", "hq6_g32"])
@pytest.mark.parametrize("m", [1, 37, 100, 257, 333, 575])
@pytest.mark.parametrize("cfg", [1, 5])
def test_gemm_pingpong_kernel_ragged_rows(dev, fmt, m, cfg):
    """Row counts that are not whole 64-row blocks on the ping-pong kernel (256 x 320 and 128 x 320 tiles): threads whose row
    lies past the last one re-read the tile's first row and store nothing (last tile rows of 1 to 77 rows; one tile of
    fewer than 64)."""
    st, out, ref = run_gemm(dev, fmt, m, 400, 320, xdtype="f16", ydtype="f32", cfg=cfg, seed=7)
    assert st == qwhip.OK
    assert qo.normalized_error(out, ref) <= 2e-5
    st, out, ref = run_gemm(dev, fmt, m, 336, 192, xdtype="bf16", ydtype="bf16", cfg=cfg, seed=8)
    assert st == qwhip.OK
    assert qo.normalized_error(out, ref) <= TOL


def test_gemm_half_height_tile_at_2048_rows(dev):
    """M = 2048 on the benchmark bank: the automatic choice is the ping-pong kernel's 128 x 320 tile (256 tiles)."""
    st, out, ref = run_gemm(dev, "hq4_g32_m5", 2048, 5120, 5120, xdtype="bf16", ydtype="bf16")
    assert st == qwhip.OK
    assert qo.normalized_error(out, ref) <= TOL


def test_gemm_ragged_rows_at_the_prefill_shape(dev):
    """M = 4001 on the benchmark bank (automatic dispatch, bf16 in / bf16 out): the last tile row holds 161 rows."""
    st, out, ref = run_gemm(dev, "hq4_g32_m5", 4001, 5120, 5120, xdtype="bf16", ydtype="bf16")
    assert st == qwhip.OK
    assert qo.normalized_error(out, ref) <= TOL


@pytest.mark.parametrize("fmt", ["hq4_g32_m5", "hq4_g64", "aq2_g64", "hq3_g32", "hq6_g32", "hq8_g32"])
@pytest.mark.parametrize("m,n,k", [(64, 640, 1024), (200, 400, 2048), (37, 336, 1536), (512, 1280, 5120)])
def test_gemm_split_k_with_a_workspace_for_partial_planes(dev, fmt, m, n, k):
    """Few tiles and a workspace that holds fp32 partial planes: the K-steps of a tile are dealt over several workgroups and a
    second launch sums the planes (2 to 8 ranges here, with a short last range at k = 1536: 24 K-steps over 3 ranges of 8,
    and at k = 2048 behind the rotated copy of un-rotated rows).  Same bar as the one-launch form."""
    big = 64 << 20
    st, out, ref = run_gemm(dev, fmt, m, n, k, xdtype="f16", ydtype="f32", seed=9, workspace_bytes=big)
    assert st == qwhip.OK
    assert qo.normalized_error(out, ref) <= 2e-5
    st, out1, _ = run_gemm(dev, fmt, m, n, k, xdtype="f16", ydtype="f32", seed=9, workspace=False)
    assert qo.normalized_error(out, out1) <= 2e-6          # the ranges only change the order of the fp32 sums
    st, out, ref = run_gemm(dev, fmt, m, n, k, xdtype="bf16", ydtype="bf16", seed=10, workspace_bytes=big)
    assert st == qwhip.OK
    assert qo.normalized_error(out, ref) <= TOL
    st, out, ref = run_gemm(dev, fmt, m, n, k, xdtype="f16", ydtype="f16", prerot=False, seed=11, workspace_bytes=big)
    assert st == qwhip.OK
    assert qo.normalized_error(out, ref) <= TOL


@pytest.mark.parametrize("fmt", ["hq4_g32_m5", "hq4_g64", "hq8_g32"])
@pytest.mark.parametrize("m,ws_mb", [(333, 0), (333, 64), (2100, 0)])
def test_gemm_strided_rows_on_every_ping_pong_form(dev, fmt, m, ws_mb):
    """Activation rows ldx > k apart and output rows ldy > n apart (both in elements) through the one-launch forms (256 x 320
    and 128 x 320 tiles, ragged row counts) and the split-K form: padding columns of the output stay untouched."""
    n, k, ldx, ldy = 656, 1024, 1024 + 64, 656 + 8
    blocks, w16 = H.make_bank(fmt, n, k, seed=13)
    x32 = H.make_x(m, k, 17)
    xp = np.zeros((m, ldx), np.float16)
    xp[:, :k] = x32.astype(np.float16)
    xp[:, k:] = np.float16(777.0)                      # never read
    bank, xb = dev.put(blocks), dev.put(xp)
    yb = dev.put(np.full((m, ldy), 0x7FC0, np.uint16))  # bf16 NaN pattern in the padding
    ws = dev.alloc(ws_mb << 20) if ws_mb else None
    view = H.view_of(dev, bank, fmt, n, k)
    st = dev.lib.qwhip_gemm(dev.stream.handle, C.byref(view), xb.ptr, qwhip.F16, m, ldx, yb.ptr, qwhip.BF16, ldy, qwhip.X_PREROTATED,
                            ws.ptr if ws else None, ws.nbytes if ws else 0)
    assert st == qwhip.OK
    dev.stream.sync()
    raw = yb.download(np.uint16, (m, ldy))
    for b in (bank, xb, yb, ws):
        if b is not None:
            b.free()
    assert np.all(raw[:, n:] == 0x7FC0)
    ref = qo.matmul_ref_f64(xp[:, :k], w16)
    assert qo.normalized_error(qo.bf16_bits_to_f32(raw[:, :n]), ref) <= TOL


def test_gemm_rotation_prepass_with_workspace(dev):
    st, out, ref = run_gemm(dev, "hq4_g32_m5", 130, 256, 512, prerot=False, ydtype="f32")
    assert st == qwhip.OK
    assert qo.normalized_error(out, ref) <= 2e-5
    st, _, _ = run_gemm(dev, "hq4_g32_m5", 130, 256, 512, prerot=False, workspace=False)
    assert st == qwhip.E_BASIS


def test_gemm_geometry_errors(dev):
    st, _, _ = run_gemm(dev, "hq4_g32_m5", 8, 24, 64)      # n % 16 != 0
    assert st == qwhip.E_BAD_GEOMETRY
    st, _, _ = run_gemm(dev, "hq4_g32_m5", 8, 32, 96)      # k % 64 != 0
    assert st == qwhip.E_BAD_GEOMETRY


def test_gemm_matches_per_row_gemv(dev):
    """Kernel-vs-kernel: batched GEMM against the per-row GEMV, max |diff| in f16 < 0.05
    (Tests/QWGEMMTests/QWBatchedGemmTests.swift:130-139)."""
    fmt, m, n, k = "hq4_g32_m5", 16, 512, 1024
    blocks, _ = H.make_bank(fmt, n, k, seed=9)
    x16 = H.make_x(m, k, 10).astype(np.float16)
    bank, xb = dev.put(blocks), dev.put(x16)
    yg, yv = dev.alloc(m * n * 2), dev.alloc(m * n * 2)
    view = H.view_of(dev, bank, fmt, n, k)
    lib, st = dev.lib, dev.stream.handle
    qwhip.check(lib.qwhip_gemm(st, C.byref(view), xb.ptr, qwhip.F16, m, 0, yg.ptr, qwhip.F16, 0, qwhip.X_PREROTATED, None, 0))
    qwhip.check(lib.qwhip_gemv(st, C.byref(view), xb.ptr, qwhip.F16, m, qwhip.X_PREROTATED, yv.ptr, None))
    a = yg.download(np.float16, (m, n)).astype(np.float32)
    b = yv.download(np.float16, (m, n)).astype(np.float32)
    assert np.max(np.abs(a - b)) < 0.05


def test_gemm_full_size_prefill_config(dev):
    """HQ4_G32 prefill GEMM at its benchmark shape: M = 4096, K = 5120, N = 5120, bf16 in / bf16 out."""
    st, out, ref = run_gemm(dev, "hq4_g32_m5", 4096, 5120, 5120, xdtype="bf16", ydtype="bf16")
    assert st == qwhip.OK
    assert qo.normalized_error(out, ref) <= TOL


@pytest.mark.parametrize("fmt,xdtype,prerot", [("hq4_g32_m5", "f16", True), ("hq4_g32_m5", "bf16", True), ("hq4_g64", "f16", False),
                                               ("hq3_g32", "f16", True), ("aq2_g64", "f16", True),
                                               ("aq4_g32", "f16", True)])
@pytest.mark.parametrize("m,inter,k,rot", [(64, 160, 128, 1), (256, 352, 256, 1), (320, 1024, 192, 0), (576, 96, 64, 1), (37, 160, 128, 1),
                                           (333, 352, 256, 0)])
def test_gemm_swiglu_equals_gemm_then_swiglu(dev, fmt, xdtype, prerot, m, inter, k, rot):
    """qwhip_gemm_swiglu == qwhip_gemm (f16 out) + qwhip_swiglu_fwht, bit for bit (column tiles of 160 outputs with a partial
    last one, several row tiles, bf16 and un-rotated activations through the workspace), and within the bar of the oracle."""
    n = 2 * inter
    blocks, w16 = H.make_bank(fmt, n, k, seed=5)
    x32 = H.make_x(m, k, 12)
    rotate = H.FORMATS[fmt][4]
    if xdtype == "bf16":
        x_val, x_host, xcode = qo.round_bf16(x32), qo.f32_to_bf16_bits(x32), qwhip.BF16
    else:
        x_host, xcode = x32.astype(np.float16), qwhip.F16
        x_val = x_host.astype(np.float32)
    flags = qwhip.X_PREROTATED if (prerot or not rotate) else 0
    x_basis = x_val.astype(np.float16) if flags else qo.fwht32_ortho(x_val).astype(np.float16)
    bank, xb = dev.put(blocks), dev.put(x_host)
    gu, act2, act1 = dev.alloc(m * n * 2), dev.put(np.zeros((m, inter), np.float16)), dev.put(np.zeros((m, inter), np.float16))
    ws = dev.alloc(m * k * 2)
    view = H.view_of(dev, bank, fmt, n, k)
    lib, st = dev.lib, dev.stream.handle
    qwhip.check(lib.qwhip_gemm(st, C.byref(view), xb.ptr, xcode, m, 0, gu.ptr, qwhip.F16, 0, flags, ws.ptr, ws.nbytes))
    qwhip.check(lib.qwhip_swiglu_fwht(st, gu.ptr, qwhip.F16, act2.ptr, m, inter, rot))
    qwhip.check(lib.qwhip_gemm_swiglu(st, C.byref(view), xb.ptr, xcode, m, 0, rot, act1.ptr, 0, flags, ws.ptr, ws.nbytes))
    dev.stream.sync()
    one, two = act1.download(np.float16, (m, inter)), act2.download(np.float16, (m, inter))
    assert np.array_equal(one.view(np.uint16), two.view(np.uint16))
    g = qo.matmul_ref_f64(x_basis, w16).astype(np.float16).astype(np.float32)
    want = qo.swiglu_fwht_f16(g[:, :inter], g[:, inter:], rotate=bool(rot)).astype(np.float32)
    assert qo.normalized_error(one.astype(np.float32), want) <= TOL


@pytest.mark.parametrize("fmt,m", [("hq8_g32", 128), ("hq3_g32", 64), ("hq6_g32", 128), ("aq6_g128", 75), ("hq4_g32_m5", 37), ("aq2_g64", 200)])
@pytest.mark.parametrize("xdtype,prerot", [("f16", True), ("bf16", False)])
def test_gemm_swiglu_every_container_and_row_count_in_one_launch(dev, fmt, m, xdtype, prerot):
    """The 6- and 8-bit containers and ragged row counts on the fused door (once two launches through the workspace): the same
    bits as the two doors called one after the other, whatever workspace beyond the activation copy is handed over (K = 384 is
    too short for K ranges, which a roomy workspace would otherwise bring)."""
    inter, k = 224, 384
    n = 2 * inter
    rotate = H.FORMATS[fmt][4]
    blocks, _ = H.make_bank(fmt, n, k, seed=4)
    x32 = H.make_x(m, k, 13)
    if xdtype == "bf16":
        x_host, xcode = qo.f32_to_bf16_bits(x32), qwhip.BF16
    else:
        x_host, xcode = x32.astype(np.float16), qwhip.F16
    flags = qwhip.X_PREROTATED if (prerot or not rotate) else 0
    bank, xb = dev.put(blocks), dev.put(x_host)
    gu, act2, act1 = dev.alloc(m * n * 2), dev.put(np.zeros((m, inter), np.float16)), dev.put(np.zeros((m, inter), np.float16))
    ws1, ws2 = dev.alloc(m * k * 2), dev.alloc(m * n * 2 + m * k * 2)
    view = H.view_of(dev, bank, fmt, n, k)
    lib, st = dev.lib, dev.stream.handle
    qwhip.check(lib.qwhip_gemm(st, C.byref(view), xb.ptr, xcode, m, 0, gu.ptr, qwhip.F16, 0, flags, ws1.ptr, ws1.nbytes))
    qwhip.check(lib.qwhip_swiglu_fwht(st, gu.ptr, qwhip.F16, act2.ptr, m, inter, 1))
    qwhip.check(lib.qwhip_gemm_swiglu(st, C.byref(view), xb.ptr, xcode, m, 0, 1, act1.ptr, 0, flags, ws2.ptr, ws2.nbytes))
    dev.stream.sync()
    one, two = act1.download(np.float16, (m, inter)), act2.download(np.float16, (m, inter))
    assert np.array_equal(one.view(np.uint16), two.view(np.uint16))
    assert np.any(one != 0)
    # a workspace that holds only the activation copy is enough: the door is one launch for every container and row count
    assert lib.qwhip_gemm_swiglu(st, C.byref(view), xb.ptr, xcode, m, 0, 1, act1.ptr, 0, flags, ws1.ptr, ws1.nbytes) == qwhip.OK
    dev.stream.sync()


@pytest.mark.parametrize("fmt", ["hq4_g32_m5", "hq4_g64", "hq8_g32", "hq3_g32"])
@pytest.mark.parametrize("m,inter,k,xdtype,prerot", [(64, 320, 2048, "f16", True), (100, 480, 1536, "bf16", True), (37, 160, 1024, "f16", False),
                                                     (128, 800, 5120, "bf16", False)])
def test_gemm_swiglu_split_k_with_a_roomy_workspace(dev, fmt, m, inter, k, xdtype, prerot):
    """Few tiles, a long K and a workspace with room for an f16 gate|up image and fp32 planes behind the activation copy: the
    fused door deals the K-steps over several workgroups, sums the planes and runs the SwiGLU pass - the same bits as qwhip_gemm
    (which splits the same way when neither workspace binds) followed by qwhip_swiglu_fwht, within the bar of the oracle, and
    within rounding of its own one-launch form (flags bits 8..11 set keep that)."""
    n = 2 * inter
    blocks, w16 = H.make_bank(fmt, n, k, seed=6)
    x32 = H.make_x(m, k, 14)
    rotate = H.FORMATS[fmt][4]
    if xdtype == "bf16":
        x_val, x_host, xcode = qo.round_bf16(x32), qo.f32_to_bf16_bits(x32), qwhip.BF16
    else:
        x_host, xcode = x32.astype(np.float16), qwhip.F16
        x_val = x_host.astype(np.float32)
    flags = qwhip.X_PREROTATED if (prerot or not rotate) else 0
    x_basis = x_val.astype(np.float16) if flags else qo.fwht32_ortho(x_val).astype(np.float16)
    bank, xb = dev.put(blocks), dev.put(x_host)
    gu = dev.alloc(m * n * 2)
    acts = [dev.put(np.zeros((m, inter), np.float16)) for _ in range(3)]
    ws = dev.alloc(64 << 20)
    view = H.view_of(dev, bank, fmt, n, k)
    lib, st = dev.lib, dev.stream.handle
    # bf16 rows go through the separate conversion pass in both doors (flags bit 16 asks qwhip_gemm for it), so both split alike
    qwhip.check(lib.qwhip_gemm(st, C.byref(view), xb.ptr, xcode, m, 0, gu.ptr, qwhip.F16, 0, flags | (1 << 16), ws.ptr, ws.nbytes))
    qwhip.check(lib.qwhip_swiglu_fwht(st, gu.ptr, qwhip.F16, acts[0].ptr, m, inter, 1))
    qwhip.check(lib.qwhip_gemm_swiglu(st, C.byref(view), xb.ptr, xcode, m, 0, 1, acts[1].ptr, 0, flags, ws.ptr, ws.nbytes))
    qwhip.check(lib.qwhip_gemm_swiglu(st, C.byref(view), xb.ptr, xcode, m, 0, 1, acts[2].ptr, 0, flags | (1 << 8), ws.ptr, ws.nbytes))
    dev.stream.sync()
    two, split, one = (a.download(np.float16, (m, inter)) for a in acts)
    for b in (bank, xb, gu, ws, *acts):
        b.free()
    assert np.array_equal(split.view(np.uint16), two.view(np.uint16))
    g = qo.matmul_ref_f64(x_basis, w16).astype(np.float16).astype(np.float32)
    want = qo.swiglu_fwht_f16(g[:, :inter], g[:, inter:], rotate=True).astype(np.float32)
    assert qo.normalized_error(split.astype(np.float32), want) <= TOL
    assert qo.normalized_error(one.astype(np.float32), want) <= TOL
    assert qo.normalized_error(split.astype(np.float32), one.astype(np.float32)) <= TOL


def test_gemm_swiglu_refusals(dev):
    blocks, _ = H.make_bank("hq8_g32", 128, 64, seed=1)
    bank, xb, act = dev.put(blocks), dev.put(np.zeros((64, 64), np.float16)), dev.alloc(64 * 64 * 2)
    v8 = H.view_of(dev, bank, "hq8_g32", 128, 64)
    lib, st = dev.lib, dev.stream.handle
    assert lib.qwhip_gemm_swiglu(st, C.byref(v8), xb.ptr, qwhip.F16, 64, 0, 1, act.ptr, 0, qwhip.X_PREROTATED, None, 0) == qwhip.OK   # every container
    blocks4, _ = H.make_bank("hq4_g32_m5", 128, 64, seed=1)
    bank4 = dev.put(blocks4)
    v4 = H.view_of(dev, bank4, "hq4_g32_m5", 128, 64)
    assert lib.qwhip_gemm_swiglu(st, C.byref(v4), xb.ptr, qwhip.F16, 37, 0, 1, act.ptr, 0, qwhip.X_PREROTATED, None, 0) == qwhip.OK   # any row count
    assert lib.qwhip_gemm_swiglu(st, C.byref(v4), xb.ptr, qwhip.F16, 64, 0, 1, act.ptr, 0, 0, None, 0) == qwhip.E_BASIS   # rotation needs the workspace
    assert lib.qwhip_gemm_swiglu(st, C.byref(v4), xb.ptr, qwhip.BF16, 64, 0, 1, act.ptr, 0, qwhip.X_PREROTATED, None, 0) == qwhip.E_BAD_GEOMETRY
