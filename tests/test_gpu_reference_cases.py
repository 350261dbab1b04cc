"""The reference's own self-contained GPU test cases for this path, restated through the C ABI: the data
generators (integer hashes, closed-form codes) and the host formulas come from the cited XCTest files; the
expected values are computed here in numpy / float64.  Nothing is read from the reference at run time."""
import ctypes as C

import numpy as np
import pytest

from oracle import qworacle as qo
from qwegn_amd import qwhip

pytestmark = pytest.mark.gpu
M64 = (1 << 64) - 1


@pytest.fixture(scope="module")
def dev():
    return qwhip.Device(0)


def splitmix64(x: int) -> int:
    z = (x + 0x9E3779B97F4A7C15) & M64
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & M64
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & M64
    return z ^ (z >> 31)


def test_hq4_decode_gemv_matches_the_host_formula(dev):
    """Tests/QWGEMMTests/QWHQ4GEMVTests.swift:16-50,108-133: splitmix64 codes and scales, bias = f16(-1032*scale),
    host value sum f16((1024+nib)*sc+bi)*x; |got - ref| / max(|ref|, sum|w*x|) <= 1e-3."""
    rows, cols = 64, 256
    groups = cols // 32

    def seed(r, g):
        return splitmix64(((r * 0x00000001000003B3) + g * 0x9E3779B97F4A7C15) & M64)

    blocks = np.zeros((rows, groups, 20), dtype=np.uint8)
    for r in range(rows):
        for g in range(groups):
            s = seed(r, g)
            codes = np.array([splitmix64((s + i) & M64) & 0xF for i in range(32)])
            unit = (splitmix64((s + 0x5DEECE66D) & M64) % 1_000_000) / 1_000_000.0
            sc = np.float16(unit * 0.02 + 0.001)
            bi = np.float16(np.float32(-1032.0) * np.float32(sc))
            blocks[r, g, 0:2] = np.array([sc]).view(np.uint8)
            blocks[r, g, 2:4] = np.array([bi]).view(np.uint8)
            blocks[r, g, 4:] = qo.hq4_interleave(codes[None, :]).view(np.uint8).reshape(16)
    xs = np.array([np.float16((splitmix64((i * 0x9E3779B97F4A7C15) & M64) % 2_000_001) / 1_000_000.0 - 1.0) for i in range(cols)],
                  dtype=np.float16)
    bank, xb, yb = dev.put(blocks), dev.put(xs), dev.alloc(rows * 4)
    view = dev.view(bank, rows, cols, qwhip.KIND_HQ4_G32_M5)
    for variant in (1, 2):
        qwhip.check(dev.lib.qwhip_gemv(dev.stream.handle, C.byref(view), xb.ptr, qwhip.F16, 1, qwhip.X_PREROTATED | (variant << 8),
                                       None, yb.ptr))
        got = yb.download(np.float32, (rows,)).astype(np.float64)
        w = qo.weights_f16_exact(blocks, 4, 32, True).astype(np.float64)
        prod = w * xs.astype(np.float64)[None, :]
        value, magnitude = prod.sum(1), np.abs(prod).sum(1)
        err = np.abs(got - value) / np.maximum(np.maximum(np.abs(value), magnitude), 1e-6)
        assert np.all(err <= 1e-3)


def _closed_form_bank(rows, cols, fmt):
    """Tests/QWGEMMTests/QWMoEReuseTests.swift:18-44: code (r*7 + c*3 + 5) % 16, weight (code - 8)/16."""
    r = np.arange(rows)[:, None]
    c = np.arange(cols)[None, :]
    codes = (r * 7 + c * 3 + 5) % 16
    if fmt == "incumbent":                     # HQ4_G32 block, scale 1/16 -> bias f16(-1032/16) = -64.5
        blocks = np.zeros((rows, cols // 32, 20), dtype=np.uint8)
        blocks[..., 0:2] = np.array([1.0 / 16], dtype=np.float16).view(np.uint8)
        blocks[..., 2:4] = np.array([-1032.0 / 16], dtype=np.float16).view(np.uint8)
        blocks[..., 4:] = qo.hq4_interleave(codes.reshape(rows, cols // 32, 32)).view(np.uint8).reshape(rows, cols // 32, 16)
    else:                                      # AQ4_G64, scale 1/16, bias -0.5, standard basis
        blocks = np.zeros((rows, cols // 64, 36), dtype=np.uint8)
        blocks[..., 0:2] = np.array([1.0 / 16], dtype=np.float16).view(np.uint8)
        blocks[..., 2:4] = np.array([-0.5], dtype=np.float16).view(np.uint8)
        blocks[..., 4:] = qo.pack_bitstream(codes.reshape(rows, cols // 64, 64), 4)
    return blocks, (codes.astype(np.float64) - 8.0) / 16.0


@pytest.mark.parametrize("fmt", ["incumbent", "aq4_g64"])
@pytest.mark.parametrize("tokens", [1, 2, 5])
def test_moe_expert_reuse_and_independent_rows_match_cpu(dev, fmt, tokens):
    """Tests/QWGEMMTests/QWMoEReuseTests.swift:46-186: 15 experts, 3 routes, hidden = intermediate = 64, id patterns
    with repeats and an empty route; routed gate_up + SwiGLU (+FWHT in the rotated basis) + down + weighted combine
    with a gated shared row, against a float64 evaluation."""
    experts, routes, hidden, inter = 15, 3, 64, 64
    patterns = [[0, 1, 2, 1, 3, 2, 0, 3, -1, 3, 1, 0, 4, 5, 6], list(range(15))]
    gate_blocks, gate_w = _closed_form_bank(experts * 2 * inter, hidden, fmt)
    down_blocks, down_w = _closed_form_bank(experts * hidden, inter, fmt)
    rotated = fmt == "incumbent"
    kind, bits, group = (qwhip.KIND_HQ4_G32_M5, 4, 32) if rotated else (qwhip.KIND_NATIVE_AFFINE, 4, 64)
    rng = np.random.default_rng(tokens)
    xs = (rng.integers(-8, 9, size=(tokens, hidden)) / 8.0).astype(np.float16)      # in the container's basis
    ws = (rng.integers(1, 9, size=(tokens * routes,)) / 8.0).astype(np.float32)
    shared = (rng.integers(-4, 5, size=(tokens, hidden)) / 4.0).astype(np.float32)
    gates = (rng.integers(0, 5, size=(tokens,)) / 4.0).astype(np.float32)
    gub, dnb = dev.put(gate_blocks), dev.put(down_blocks)
    vgu = dev.view(gub, experts * 2 * inter, hidden, kind, bits, group)
    vdn = dev.view(dnb, experts * hidden, inter, kind, bits, group)
    for pattern in patterns:
        ids = np.array(pattern[: tokens * routes], dtype=np.int32)
        gw = gate_w.reshape(experts, 2 * inter, hidden)
        dw = down_w.reshape(experts, hidden, inter)
        idx2 = ids.reshape(tokens, routes)
        ref = qo.moe_forward_f64(xs, idx2, ws.reshape(tokens, routes), gw, dw, act_f16=True, rotate_act=rotated)
        ref += gates[:, None].astype(np.float64) * shared
        xb, ib, wb, sb, gb = dev.put(xs), dev.put(ids), dev.put(ws), dev.put(shared), dev.put(gates)
        act, out = dev.alloc(ids.size * inter * 2), dev.alloc(tokens * hidden * 4)
        lib, st = dev.lib, dev.stream.handle
        qwhip.check(lib.qwhip_moe_gateup_decode(st, C.byref(vgu), experts, xb.ptr, qwhip.F16, qwhip.X_PREROTATED, ib.ptr, tokens,
                                                routes, act.ptr))
        qwhip.check(lib.qwhip_moe_down_decode(st, C.byref(vdn), experts, act.ptr, ib.ptr, wb.ptr, tokens, routes, sb.ptr, gb.ptr,
                                              out.ptr, qwhip.F32))
        got = out.download(np.float32, (tokens, hidden))
        assert qo.normalized_error(got, ref) <= 2e-3


def test_small_tiles_match_the_64_row_tiles_bit_for_bit(dev):
    """Compact 16/32-row tail tiles against uncompacted tile lists: the grouped GEMM result does not depend on the
    tile list (Tests/QWGEMMTests/QWMoETailCompactTests.swift:185-188, bit-identical)."""
    from tests import helpers as H
    experts, hidden, rows_per, k = 8, 256, 128, 2
    t = 37
    blocks, _ = H.make_bank("hq4_g32_m5", experts * rows_per, hidden, seed=2)
    rng = np.random.default_rng(3)
    x16 = rng.standard_normal((t, hidden)).astype(np.float16)
    ids = np.stack([rng.choice(experts, size=k, replace=False) for _ in range(t)]).astype(np.int32)
    pairs = t * k
    lib, st = dev.lib, dev.stream.handle
    bank, xb, ib = dev.put(blocks), dev.put(x16), dev.put(ids)
    view = H.view_of(dev, bank, "hq4_g32_m5", experts * rows_per, hidden)
    mt = lib.qwhip_moe_max_tiles(experts, pairs)
    outs = []
    for compact in (1, 0):
        off, sp, stok, inv = dev.alloc((experts + 1) * 4), dev.alloc(pairs * 4), dev.alloc(pairs * 4), dev.alloc(pairs * 4)
        te, tr, tc = dev.alloc(mt * 4 + 64), dev.alloc(mt * 4 + 64), dev.alloc(16)
        y = dev.alloc(pairs * rows_per * 4)
        qwhip.check(lib.qwhip_moe_group_pairs(st, ib.ptr, experts, pairs, k, off.ptr, sp.ptr, stok.ptr, inv.ptr, te.ptr, tr.ptr, tc.ptr, compact))
        # uncompacted lists can hold more tiles than the compact bound; size the launch by what was written
        dev.stream.sync()
        ntiles = int(tc.download(np.int32, (1,))[0])
        qwhip.check(lib.qwhip_moe_grouped_gemm(st, C.byref(view), experts, xb.ptr, qwhip.F16, 0, stok.ptr, off.ptr, te.ptr, tr.ptr, tc.ptr,
                                               max(ntiles, 1), pairs, y.ptr, qwhip.F32, 0))
        got = y.download(np.float32, (pairs, rows_per))
        order = inv.download(np.int32, (pairs,))
        outs.append(got[order])                    # back to pair order: slot order inside an expert is arbitrary
    assert np.array_equal(outs[0].view(np.uint32), outs[1].view(np.uint32))
