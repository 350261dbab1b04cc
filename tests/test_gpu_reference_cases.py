"""The reference's own self-contained GPU test cases for this path, restated through the C ABI: the data
generators (integer hashes, closed-form codes) and the host formulas come from the cited XCTest files; the
expected values are computed here in numpy / float64.  Nothing is read from the reference at run time."""
import ctypes as C

import numpy as np
import pytest

from oracle import qworacle as qo
from qwegn_amd import qwhip
from tests import helpers as H

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


def _mlx_checkpoint(rng, rows, cols, bits, group, f16):
    """A synthetic MLX affine tensor: packed codes, and one (scale, bias) pair per group in bf16 or f16."""
    groups, payload = cols // group, group * bits // 8
    w = rng.integers(0, 256, size=(rows, groups * payload), dtype=np.uint8)
    sc = (rng.uniform(1e-3, 0.05, size=rows * groups)).astype(np.float32)
    bi = (-sc * rng.uniform(2, 9, size=rows * groups)).astype(np.float32)
    if f16:
        return w, sc.astype(np.float16).view(np.uint16), bi.astype(np.float16).view(np.uint16)
    return w, qo.f32_to_bf16_bits(sc), qo.f32_to_bf16_bits(bi)


@pytest.mark.parametrize("bits,group", [(4, 32), (4, 64), (8, 32), (8, 128), (3, 32), (2, 64)])
@pytest.mark.parametrize("f16", [False, True])
def test_mlx_repack_writes_the_oracles_bytes(dev, bits, group, f16):
    """qwhip_repack_mlx_affine vs the oracle's restatement of qwg_repack_mlx_affine_to_aq_m5, byte for byte, with
    headers f16 cannot hold (too large, NaN, infinite, below 2^-14) in the mix: poisoned and counted, or accepted."""
    rng = np.random.default_rng(bits * 100 + group + f16)
    rows, cols = 37, 4 * group
    w, s16, b16 = _mlx_checkpoint(rng, rows, cols, bits, group, f16)
    if not f16:
        s16[3], b16[7], s16[11], b16[20] = 0x7F00, 0x7FC0, 0x7F80, 0x0080     # 1.7e38, NaN, +inf, 1.2e-38 (bf16)
    else:
        s16[3], b16[7] = 0x7E00, 0x0001                                         # NaN, smallest subnormal (f16)
    want, refused = qo.repack_mlx_affine(w, s16, b16, rows, cols, bits, group, scale_is_f16=f16)
    wb, sb, bb_ = dev.put(w), dev.put(s16), dev.put(b16)
    out = dev.alloc(want.nbytes)
    cnt = dev.put(np.zeros(1, np.uint32))
    qwhip.check(dev.lib.qwhip_repack_mlx_affine(dev.stream.handle, wb.ptr, sb.ptr, bb_.ptr, qwhip.F16 if f16 else qwhip.BF16,
                                                rows, cols, bits, group, out.ptr, cnt.ptr))
    dev.stream.sync()
    assert np.array_equal(out.download(np.uint8, want.shape), want)
    assert int(cnt.download(np.uint32, (1,))[0]) == refused and refused >= 1


def test_mlx_repack_switch_gate_up_interleaves_experts(dev):
    """qwhip_repack_mlx_affine_switch_gate_up: [experts, inter, cols] gate and up tensors -> one [experts, 2*inter, cols]
    bank, byte for byte; the bank then multiplies like any other AQ4_G64 bank."""
    rng = np.random.default_rng(77)
    experts, inter, cols, bits, group = 3, 40, 256, 4, 64
    gw, gs, gb = _mlx_checkpoint(rng, experts * inter, cols, bits, group, False)
    uw, us, ub = _mlx_checkpoint(rng, experts * inter, cols, bits, group, False)
    want, refused = qo.repack_mlx_affine_switch_gate_up(gw, gs, gb, uw, us, ub, experts, inter, cols, bits, group, False)
    bufs = [dev.put(a) for a in (gw, gs, gb, uw, us, ub)]
    out, cnt = dev.alloc(want.nbytes), dev.put(np.zeros(1, np.uint32))
    qwhip.check(dev.lib.qwhip_repack_mlx_affine_switch_gate_up(dev.stream.handle, *[b.ptr for b in bufs], qwhip.BF16, experts, inter,
                                                               cols, bits, group, out.ptr, cnt.ptr))
    dev.stream.sync()
    assert refused == 0 and int(cnt.download(np.uint32, (1,))[0]) == 0
    assert np.array_equal(out.download(np.uint8, want.shape), want)
    n = experts * 2 * inter
    x16 = rng.standard_normal((1, cols)).astype(np.float16)
    xb, y32 = dev.put(x16), dev.alloc(n * 4)
    view = dev.view(out, n, cols, qwhip.KIND_NATIVE_AFFINE, bits, group)
    qwhip.check(dev.lib.qwhip_gemv(dev.stream.handle, C.byref(view), xb.ptr, qwhip.F16, 1, 0, None, y32.ptr))
    dev.stream.sync()
    ref = qo.matmul_ref_f64(x16, qo.weights_f16_exact(want, bits, group, False))
    assert qo.normalized_error(y32.download(np.float32, (1, n)), ref) <= 2e-3


def test_mlx_repack_rejects_bad_layouts_before_launch(dev):
    z = dev.put(np.zeros(64, np.uint8))
    st = dev.stream.handle
    assert dev.lib.qwhip_repack_mlx_affine(st, z.ptr, z.ptr, z.ptr, qwhip.F32, 1, 64, 4, 32, z.ptr, z.ptr) == qwhip.E_BAD_SHAPE
    assert dev.lib.qwhip_repack_mlx_affine(st, z.ptr, z.ptr, z.ptr, qwhip.BF16, 1, 48, 4, 32, z.ptr, z.ptr) == qwhip.E_BAD_SHAPE
    assert dev.lib.qwhip_repack_mlx_affine(st, z.ptr, z.ptr, z.ptr, qwhip.BF16, 1, 64, 4, 32, z.ptr, None) == qwhip.E_NULL


def test_pack_plane_mover_feeds_the_kernels(dev, golden_dir, tmp_path):
    """selfpack.qwp through the plane mover: the device bank dequantizes to the f16 weights of the pack's own blocks
    (bit-exact), and multiplies like them.  A synthetic expert stack becomes one [E * N, K] bank."""
    from qwegn_amd import pack as qp
    from tests.test_pack import write_pack

    p = qp.Pack(golden_dir / "selfpack.qwp")
    buf, view = p.upload(dev, "w_test", chunk_bytes=50_000)        # several chunks
    n, k = view.n, view.k
    blocks = np.asarray(p.plane("w_test")[1]).reshape(n, k // 32, 20)
    w16 = qo.weights_f16_exact(blocks, 4, 32, True)
    out = dev.alloc(n * k * 2)
    qwhip.check(dev.lib.qwhip_dequant_f16(dev.stream.handle, C.byref(view), out.ptr))
    dev.stream.sync()
    assert np.array_equal(out.download(np.float16, (n, k)).view(np.uint16), w16.view(np.uint16))
    x16 = np.random.default_rng(4).standard_normal((1, k)).astype(np.float16)
    xb, y32 = dev.put(x16), dev.alloc(n * 4)
    qwhip.check(dev.lib.qwhip_gemv(dev.stream.handle, C.byref(view), xb.ptr, qwhip.F16, 1, 0, None, y32.ptr))
    dev.stream.sync()
    ref = qo.matmul_ref_f64(qo.rotate_activation_f16(x16), w16)
    assert qo.normalized_error(y32.download(np.float32, (1, n)), ref) <= 2e-3
    raw_buf, raw_view = p.upload(dev, "norm_test")
    assert raw_view is None and np.array_equal(raw_buf.download(np.uint8, (512,)), np.asarray(p.plane("norm_test")[1]))

    rng = np.random.default_rng(1)
    experts, rows, kk = 4, 16, 256
    w = (rng.standard_normal((experts * rows, kk)) * 0.02).astype(np.float32)
    hq4 = qo.quant_hq4_blocks(w)
    write_pack(tmp_path / "e.qwp", {"mlp.experts.down": ({"shape": [experts, rows, kk], "experts": experts,
                                                           "e_hq4": rows * (kk // 32) * 20}, hq4.tobytes(), "hq4_off")})
    ebuf, eview = qp.Pack(tmp_path / "e.qwp").upload(dev, "mlp.experts.down")
    assert (eview.n, eview.k, eview.kind) == (experts * rows, kk, qwhip.KIND_HQ4_G32_M5)
    eout = dev.alloc(experts * rows * kk * 2)
    qwhip.check(dev.lib.qwhip_dequant_f16(dev.stream.handle, C.byref(eview), eout.ptr))
    dev.stream.sync()
    assert np.array_equal(eout.download(np.float16, (experts * rows, kk)).view(np.uint16),
                          qo.weights_f16_exact(hq4, 4, 32, True).view(np.uint16))


@pytest.mark.parametrize("rows,hidden", [(1, 5120), (7, 2048), (33, 256), (4, 16384)])
@pytest.mark.parametrize("residual", [False, True])
@pytest.mark.parametrize("rotate", [1, 0])
def test_rmsnorm_with_rotation_matches_oracle(dev, rows, hidden, residual, rotate):
    """qwhip_rmsnorm vs the oracle's restatement of qwg_rmsnorm / qwg_rmsnorm_residual: max |diff| <= 1e-3 on the f16
    output (the reference's own bar, Tests/QWNormTests/QWNormTests.swift:8-10), at most one f16 ulp (or 2e-6 absolute)
    anywhere (the kernel's fp32 sum of squares runs in another order), and the residual update bit-exact."""
    rng = np.random.default_rng(rows * 7 + hidden)
    x16 = (rng.standard_normal((rows, hidden)) * 1.5).astype(np.float16)
    gam = (rng.standard_normal(hidden) * 0.1).astype(np.float16)
    res = (rng.standard_normal((rows, hidden)) * 2.0).astype(np.float16) if residual else None
    eps = 1e-6
    want, want_res = qo.rmsnorm_rot_f16(x16, gam, eps, rotate=bool(rotate), residual16=res)
    xb, gb, yb = dev.put(x16), dev.put(gam), dev.alloc(rows * hidden * 2)
    rb = dev.put(res) if residual else None
    qwhip.check(dev.lib.qwhip_rmsnorm(dev.stream.handle, xb.ptr, gb.ptr, rb.ptr if residual else None, rows, hidden, eps, rotate, yb.ptr))
    dev.stream.sync()
    got = yb.download(np.float16, (rows, hidden))
    assert np.max(np.abs(got.astype(np.float32) - want.astype(np.float32))) <= 1e-3 * max(1.0, float(np.max(np.abs(want))))
    ulp = np.abs(got.view(np.int16).astype(np.int32) - want.view(np.int16).astype(np.int32))
    diff = np.abs(got.astype(np.float32) - want.astype(np.float32))
    assert np.all((ulp <= 1) | (diff <= 2e-6))     # coefficients that cancel to ~1e-5 carry the fp32 error of their terms
    assert np.mean(ulp == 0) >= 0.98
    if residual:
        assert np.array_equal(rb.download(np.float16, (rows, hidden)).view(np.uint16), want_res.view(np.uint16))


def test_rmsnorm_refuses_the_geometries_the_reference_driver_refuses(dev):
    z = dev.put(np.zeros(4096, np.float16))
    st = dev.stream.handle
    assert dev.lib.qwhip_rmsnorm(st, z.ptr, z.ptr, None, 1, 1000, 1e-6, 1, z.ptr) == qwhip.E_BAD_GEOMETRY     # hidden % 256
    assert dev.lib.qwhip_rmsnorm(st, z.ptr, None, None, 1, 1024, 1e-6, 1, z.ptr) == qwhip.E_NULL
    assert dev.lib.qwhip_rmsnorm(st, z.ptr, z.ptr, None, 0, 1024, 1e-6, 1, z.ptr) == qwhip.OK                 # no rows: nothing to do


def test_argmax_fold_key_rule(dev):
    """qwhip_argmax_f32 against the oracle's fold: ties to the lower row, NaN never wins, -0 < +0, infinities, rows whose
    length is not a multiple of four and rows that start unaligned."""
    rng = np.random.default_rng(8)
    for rows, n in [(3, 151936), (5, 1001), (2, 7), (16, 4096), (16, 40001), (17, 33000), (1, 32768)]:   # up to 16 long rows: split over 64 workgroups each
        logits = rng.standard_normal((rows, n)).astype(np.float32)
        logits[0, [n // 3, n // 2]] = 11.0
        if rows > 1:
            logits[1, n - 1] = np.nan
        if rows > 2:
            logits[2, :] = np.nan
        lb, tb = dev.put(logits), dev.alloc(max(256, rows * 4))
        qwhip.check(dev.lib.qwhip_argmax_f32(dev.stream.handle, lb.ptr, rows, n, tb.ptr))
        dev.stream.sync()
        assert np.array_equal(tb.download(np.int32, (rows,)), qo.head_argmax(logits)), (rows, n)


@pytest.mark.parametrize("fmt,m", [("hq4_g32_m5", 1), ("hq4_g32_m5", 3), ("aq4_g32", 2), ("hq8_g32", 1)])
def test_head_argmax_picks_the_oracles_token(dev, fmt, m):
    """qwhip_head_argmax: logits within the judged bar of the fp64 reference, and the token is the fold of the device's own
    logits (and the oracle's whenever its two best logits are further apart than the error bar)."""
    from tests import helpers as H
    n, k = 3000, 1024
    blocks, w16 = H.make_bank(fmt, n, k, seed=31)
    x16 = H.make_x(m, k, 131).astype(np.float16)
    bank, xb = dev.put(blocks), dev.put(x16)
    logits, toks = dev.alloc(m * n * 4), dev.alloc(256)
    view = H.view_of(dev, bank, fmt, n, k)
    qwhip.check(dev.lib.qwhip_head_argmax(dev.stream.handle, C.byref(view), xb.ptr, qwhip.F16, m, 0, logits.ptr, toks.ptr))
    dev.stream.sync()
    got = logits.download(np.float32, (m, n))
    ref = qo.matmul_ref_f64(H.x_in_basis(x16, fmt), w16)
    assert qo.normalized_error(got, ref) <= 2e-3
    tok = toks.download(np.int32, (m,))
    assert np.array_equal(tok, qo.head_argmax(got))
    top2 = np.sort(ref, axis=1)[:, -2:]
    clear = (top2[:, 1] - top2[:, 0]) > 1e-2 * np.abs(top2[:, 1])
    assert np.array_equal(tok[clear], np.argmax(ref, axis=1)[clear])


@pytest.mark.parametrize("n,k,prerot", [(50021, 1024, False), (151936, 512, True), (4100, 5120, False)])
def test_head_argmax_fold_inside_the_gemv_epilogue(dev, n, k, prerot):
    """One row over an HQ4_G32_M5 bank: the fold rides in the GEMV's epilogue (a key per workgroup, then a one-workgroup
    fold).  The token equals the fold of the logits the same call wrote, and the tie rule holds through it: the winning
    bank row is copied to a higher and (where there is room) a lower row - equal logits, the lowest of them wins."""
    from tests import helpers as H
    fmt = "hq4_g32_m5"
    blocks, _ = H.make_bank(fmt, n, k, seed=n % 97)
    x16 = H.make_x(1, k, 17).astype(np.float16)
    xin = H.x_in_basis(x16, fmt) if prerot else x16
    flags = qwhip.X_PREROTATED if prerot else 0
    lib, st = dev.lib, dev.stream.handle
    bank, xb = dev.put(blocks), dev.put(xin)
    logits, tok = dev.alloc(n * 4), dev.alloc(256)
    view = H.view_of(dev, bank, fmt, n, k)
    qwhip.check(lib.qwhip_head_argmax(st, C.byref(view), xb.ptr, qwhip.F16, 1, flags, logits.ptr, tok.ptr))
    dev.stream.sync()
    got = logits.download(np.float32, (1, n))
    first = int(tok.download(np.int32, (1,))[0])
    assert first == int(qo.head_argmax(got)[0])
    # duplicate the winner
    rows = blocks.reshape(n, -1).copy()
    lower = first - 3 if first >= 3 else None
    rows[min(first + 5, n - 1)] = rows[first]
    if lower is not None:
        rows[lower] = rows[first]
    bank2 = dev.put(rows)
    view2 = H.view_of(dev, bank2, fmt, n, k)
    qwhip.check(lib.qwhip_head_argmax(st, C.byref(view2), xb.ptr, qwhip.F16, 1, flags, logits.ptr, tok.ptr))
    dev.stream.sync()
    got2 = logits.download(np.float32, (1, n))
    want = lower if lower is not None else first
    assert got2[0, want] == got2[0, first] == got[0, first]
    assert int(tok.download(np.int32, (1,))[0]) == want == int(qo.head_argmax(got2)[0])
    # the standalone fold over the same logits agrees
    qwhip.check(lib.qwhip_argmax_f32(st, logits.ptr, 1, n, tok.ptr))
    dev.stream.sync()
    assert int(tok.download(np.int32, (1,))[0]) == want
    for b in (bank, bank2, xb, logits, tok):
        b.free()


def test_argmax_rows_whose_maximum_is_a_zero_or_nothing_above_minus_infinity(dev):
    """The rows the fast sweep cannot decide by float compares alone: maximum +-0.0 (the key order puts +0.0 above -0.0, rows in
    either order, also split over threads), only -inf and NaN, and a long row (several chunks per thread) with a late tie."""
    n = 70000
    rng = np.random.default_rng(3)
    base = -np.abs(rng.standard_normal((6, n)).astype(np.float32)) - 1.0
    base[0, [5, 40000]] = [-0.0, 0.0]            # +0.0 wins although it comes later
    base[1, [7, 4103]] = [0.0, -0.0]             # the same thread sees both: the earlier +0.0 wins
    base[2, :] = -np.inf
    base[2, 100] = np.nan                        # nothing above -inf: the first -inf
    base[3, :] = np.nan
    base[3, 65000] = -np.inf                     # a single number among NaNs
    base[4, [69999, 33333]] = 7.5                # late tie: the lower row
    base[5, [12, 13]] = [-0.0, -0.0]             # only negative zeros at the top
    lb, tb = dev.put(base), dev.alloc(256)
    qwhip.check(dev.lib.qwhip_argmax_f32(dev.stream.handle, lb.ptr, 6, n, tb.ptr))
    dev.stream.sync()
    got = tb.download(np.int32, (6,))
    assert list(got) == [40000, 7, 0, 65000, 33333, 12]
    assert np.array_equal(got, qo.head_argmax(base))


def _embed_table(bits, group, vocab, hidden):
    """The table of the reference's gather test (Tests/QWGEMMTests/QWAQEmbedGatherTests.swift:52-66): code of column i of
    group g of row r = (3 i + 7 r + 13 g) mod 2^bits, header 1025/4096, -683/4096 (f16-exact, not powers of two)."""
    i = np.arange(group)[None, None, :]
    r = np.arange(vocab)[:, None, None]
    g = np.arange(hidden // group)[None, :, None]
    codes = ((3 * i + 7 * r + 13 * g) % (1 << bits)).astype(np.uint8)
    hdr = np.array([1025.0 / 4096.0, -683.0 / 4096.0], np.float16).view(np.uint8)
    blocks = np.empty((vocab, hidden // group, 4 + group * bits // 8), np.uint8)
    blocks[..., :4] = hdr
    blocks[..., 4:] = qo.pack_bitstream(codes, bits)
    return blocks, codes.reshape(vocab, hidden)


@pytest.mark.parametrize("bits", [2, 3, 4, 6, 8])
@pytest.mark.parametrize("group", [32, 64, 128, 256])
def test_embed_gather_every_pair(dev, bits, group):
    """The reference's own gather cases (QWAQEmbedGatherTests.swift:101-168): hidden 256, vocab 8, tokens 0, 3, 7 written
    three times, and one copy of row 2; checked against code * scale + bias in f64 within the reference's tolerance
    (product ulp + result ulp) and bit for bit against the oracle; a negative token reads row 0, one past the table its last row."""
    hidden, vocab = 256, 8
    blocks, codes = _embed_table(bits, group, vocab, hidden)
    kind = qwhip.KIND_NATIVE_AFFINE
    bank = dev.put(blocks)
    view = dev.view(bank, vocab, hidden, kind, bits, group)
    sc, bi = float(np.float16(1025.0 / 4096.0)), float(np.float16(-683.0 / 4096.0))
    for tokens, hc in (([0, 3, 7], 3), ([2], 1), ([-5, 8, 1], 2)):
        tb, ob = dev.put(np.array(tokens, np.int32)), dev.alloc(len(tokens) * hc * hidden * 4)
        qwhip.check(dev.lib.qwhip_embed_aq_f32(dev.stream.handle, C.byref(view), tb.ptr, len(tokens), hc, ob.ptr))
        dev.stream.sync()
        got = ob.download(np.float32, (len(tokens), hc, hidden))
        rows = np.clip(np.array(tokens), 0, vocab - 1)
        code = codes[rows].astype(np.float64)
        want = code * sc + bi
        ulp = 2.0 ** -24
        tol = np.abs(code * sc) * ulp + np.maximum(np.abs(want), abs(bi)) * ulp + 1e-30
        assert np.all(np.abs(got.astype(np.float64) - want[:, None, :]) <= tol[:, None, :])
        oracle = qo.embed_aq_f32(blocks, rows, hc, bits, group)
        assert np.array_equal(got.view(np.uint32), oracle.view(np.uint32))
        tb.free(); ob.free()
    bank.free()


def test_embed_gather_hq4_m5_and_errors(dev):
    """HQ4_G32_M5 tables decode with (q + 1024) * scale + bias, bit for bit the oracle's fp32 dequant; shape errors."""
    from tests import helpers as H
    vocab, hidden = 40, 512
    blocks, _ = H.make_bank("hq4_g32_m5", vocab, hidden, seed=31)
    bank = dev.put(blocks)
    view = H.view_of(dev, bank, "hq4_g32_m5", vocab, hidden)
    tokens = np.array([39, 0, 17, 17], np.int32)
    tb, ob = dev.put(tokens), dev.alloc(4 * 2 * hidden * 4)
    lib, st = dev.lib, dev.stream.handle
    qwhip.check(lib.qwhip_embed_aq_f32(st, C.byref(view), tb.ptr, 4, 2, ob.ptr))
    dev.stream.sync()
    got = ob.download(np.float32, (4, 2, hidden))
    want = qo.embed_aq_f32(blocks, tokens, 2, 4, 32, True)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    assert lib.qwhip_embed_aq_f32(st, C.byref(view), tb.ptr, 4, 0, ob.ptr) == qwhip.E_BAD_WEIGHTS
    assert lib.qwhip_embed_aq_f32(st, C.byref(view), None, 4, 1, ob.ptr) == qwhip.E_NULL
    assert lib.qwhip_embed_aq_f32(st, C.byref(view), tb.ptr, 0, 1, None) == qwhip.OK


def test_embed_gather_bf16_table(dev):
    """Raw bf16 table -> f32, hc copies, exact (QWGemmF32.swift:352-363); negative and out-of-table tokens are clamped."""
    vocab, hidden, hc = 50, 1000, 2
    rng = np.random.default_rng(6)
    table = qo.f32_to_bf16_bits(rng.standard_normal((vocab, hidden)).astype(np.float32))
    tokens = np.array([49, 0, 7, -1, 50], np.int32)
    tb, kb, ob = dev.put(table), dev.put(tokens), dev.alloc(tokens.size * hc * hidden * 4)
    qwhip.check(dev.lib.qwhip_embed_bf16_f32(dev.stream.handle, tb.ptr, vocab, hidden, kb.ptr, tokens.size, hc, ob.ptr))
    dev.stream.sync()
    got = ob.download(np.float32, (tokens.size, hc, hidden))
    want = qo.bf16_bits_to_f32(table)[np.clip(tokens, 0, vocab - 1)]
    assert np.array_equal(got[:, 0], want) and np.array_equal(got[:, 1], want)
    assert dev.lib.qwhip_embed_bf16_f32(dev.stream.handle, tb.ptr, vocab, hidden, kb.ptr, 1, 0, ob.ptr) == qwhip.E_BAD_SHAPE


# ---- load-time writers for the non-M5 containers -----------------------------------------------------------------------
BLOCK_CASES = [
    # name in hq_blocks_golden.npz, bits, group, rotate
    ("aq4_g32_std", 4, 32, False), ("hq4_g32_blk", 4, 32, True), ("hq4_g64", 4, 64, True), ("hq8_g32", 8, 32, True),
    ("hq8_g64", 8, 64, True), ("hq6_g32", 6, 32, True), ("hq4_g128", 4, 128, True), ("hq8_g256", 8, 256, True),
    ("hq2_g64", 2, 64, True), ("hq3_g32", 3, 32, True),
]


@pytest.mark.parametrize("name,bits,group,rotate", BLOCK_CASES)
def test_device_block_quantizer_writes_the_packers_bytes(dev, golden_dir, name, bits, group, rotate):
    """qwhip_quantize_blocks against the block bytes the reference's quant_hq_blocks wrote for the same input
    (tests/golden/hq_blocks_golden.npz: an outlier, a constant group, tiny values, ties; the 2- and 3-bit cases run the
    shrink search), f32 source."""
    gold = np.load(golden_dir / "hq_blocks_golden.npz")
    w = gold["w"]
    want = gold[f"{name}__blocks"]
    n, k = w.shape
    src, out = dev.put(w), dev.alloc(want.nbytes)
    qwhip.check(dev.lib.qwhip_quantize_blocks(dev.stream.handle, src.ptr, qwhip.F32, n, k, bits, group, int(rotate), 2, out.ptr))
    got = out.download(np.uint8, want.shape)
    assert np.array_equal(got, want)
    for b in (src, out):
        b.free()


@pytest.mark.parametrize("fmt", ["aq4_g32", "hq4_g64", "hq8_g32", "hq8_g64", "hq4_g128", "aq8_g256", "hq6_g32", "aq6_g128", "aq2_g64", "hq3_g32"])
@pytest.mark.parametrize("src_dtype", ["f32", "bf16"])
def test_device_block_quantizer_matches_the_oracle_on_seeded_weights(dev, fmt, src_dtype):
    """Every container of the tests on N(0, 0.02) weights: device bytes == the oracle's bytes; bf16 sources are widened
    exactly.  k = 1536 gives ragged group counts per wave for the wide groups; a bank written on the device dequantizes to the
    oracle's f16 weights bit for bit."""
    kind, bits, group, is_m5, rotate = H.FORMATS[fmt]
    n, k = 40, 1536
    w = H.make_weights(n, k, seed=17)
    if src_dtype == "bf16":
        bits16 = qo.f32_to_bf16_bits(w)
        w = qo.bf16_bits_to_f32(bits16)
        src, code = dev.put(bits16), qwhip.BF16
    else:
        src, code = dev.put(w), qwhip.F32
    want, eff = qo.quant_hq_blocks(w, bits=bits, group=group, is_m5=False, rotate=rotate)
    out = dev.alloc(want.nbytes)
    qwhip.check(dev.lib.qwhip_quantize_blocks(dev.stream.handle, src.ptr, code, n, k, bits, group, int(rotate), 2, out.ptr))
    assert np.array_equal(out.download(np.uint8, want.shape), want)
    deq = dev.alloc(n * k * 2)
    view = dev.view(out, n, k, kind, bits, group)
    qwhip.check(dev.lib.qwhip_dequant_f16(dev.stream.handle, C.byref(view), deq.ptr))
    assert np.array_equal(deq.download(np.float16, (n, k)).view(np.uint16), qo.weights_f16_exact(want, bits, group, False).view(np.uint16))
    for b in (src, out, deq):
        b.free()


def test_block_quantizer_rejects_bad_calls(dev):
    src, out = dev.put(np.zeros((4, 96), np.float32)), dev.alloc(4096)
    lib, st = dev.lib, dev.stream.handle
    assert lib.qwhip_quantize_blocks(st, src.ptr, qwhip.F32, 4, 96, 5, 32, 1, 2, out.ptr) == qwhip.E_BAD_WEIGHTS     # no 5-bit container
    assert lib.qwhip_quantize_blocks(st, src.ptr, qwhip.F32, 4, 96, 4, 64, 1, 2, out.ptr) == qwhip.E_BAD_SHAPE       # 96 % 64
    assert lib.qwhip_quantize_blocks(st, src.ptr, qwhip.F16, 4, 96, 4, 32, 1, 2, out.ptr) == qwhip.E_BAD_SHAPE       # f16 source
    assert lib.qwhip_quantize_blocks(st, src.ptr, qwhip.F32, 4, 96, 4, 32, 1, 3, out.ptr) == qwhip.E_BAD_SHAPE       # mse_clip
    assert lib.qwhip_quantize_blocks(st, src.ptr, qwhip.F32, 4, 96, 4, 32, 1, 2, out.ptr) == qwhip.OK
    dev.stream.sync()


def test_planar_hq8_device_writer_and_reader(dev, golden_dir):
    """qwhip_quantize_hq8_planar writes the reference's planes for the golden input (hq_blocks_golden.npz); the reference's
    planar pack goes reader -> device planes -> qwhip_dequant_hq8_planar and lands within 1e-6 of selfpack_hq8.qwp.dq8rot.f32.bin
    (the bar of Tests/QWQuantTests/QWHQ8PackTests.swift:30-44), bit-identical to the oracle's dequant."""
    from qwegn_amd import pack as qpack
    gold = np.load(golden_dir / "hq_blocks_golden.npz")
    w = gold["w"]
    n, k = w.shape
    src, qs, sc = dev.put(w), dev.alloc(n * k), dev.alloc(n * (k // 32) * 2)
    qwhip.check(dev.lib.qwhip_quantize_hq8_planar(dev.stream.handle, src.ptr, qwhip.F32, n, k, 1, qs.ptr, sc.ptr))
    assert np.array_equal(qs.download(np.int8, (n, k)), gold["hq8_planar__qs"])
    assert np.array_equal(sc.download(np.uint16, (n, k // 32)), gold["hq8_planar__scales"])
    pk = qpack.Pack(golden_dir / "selfpack_hq8.qwp")
    name = next(nm for nm, e in pk.tensors.items() if e.hq8_quantized)
    dq, ds, pn, pkk = pk.upload_hq8(dev, name)
    out = dev.alloc(pn * pkk * 4)
    qwhip.check(dev.lib.qwhip_dequant_hq8_planar(dev.stream.handle, dq.ptr, ds.ptr, pn, pkk, out.ptr))
    got = out.download(np.float32, (pn, pkk))
    want = np.frombuffer((golden_dir / "selfpack_hq8.qwp.dq8rot.f32.bin").read_bytes(), dtype=np.float32).reshape(pn, pkk)
    assert np.max(np.abs(got - want)) <= 1e-6
    host_q, host_s = pk.hq8_planes(name)
    assert np.array_equal(got.view(np.uint32), qo.dequant_hq8_planar_rot(np.asarray(host_q), np.asarray(host_s)).view(np.uint32))


def test_pack_writer_quantizes_on_the_device_and_round_trips(dev, tmp_path):
    """PackWriter.add_weights: fp32 weights -> device quantizer -> pack file -> reader -> device bank: the bank's bytes are the
    oracle's for an HQ4_G32_M5 expert stack and an HQ8_G64 projection (group resolved by gcd as the packer does: 64 stays 64)."""
    from qwegn_amd import pack as qpack
    experts, rows, k = 2, 16, 512
    w3 = H.make_weights(experts * rows, k, seed=41).reshape(experts, rows, k)
    w2 = H.make_weights(24, k, seed=42)
    with qpack.PackWriter(tmp_path / "dev.qwp", {"source": "device-writer"}) as wr:
        wr.add_weights(dev, "mlp.experts.down", w3)
        wr.add_weights(dev, "o_proj", w2, bits=8, group=64, is_m5=False)
    pk = qpack.Pack(tmp_path / "dev.qwp")
    assert np.array_equal(np.asarray(pk.plane("mlp.experts.down")[1]), qo.quant_hq4_blocks(w3.reshape(-1, k)).ravel().view(np.uint8))
    want, _ = qo.quant_hq_blocks(w2, bits=8, group=64, is_m5=False, rotate=True)
    buf, view = pk.upload(dev, "o_proj")
    assert (view.n, view.k, view.bits, view.group) == (24, k, 8, 64)
    assert np.array_equal(buf.download(np.uint8, (want.nbytes,)), want.ravel().view(np.uint8))



@pytest.mark.parametrize("rows,row_bytes", [(17408, 3200), (300, 3200), (7, 640), (513, 10880), (45, 5120), (2050, 1940), (1, 20)])
def test_row_checksum_is_the_hosts_word_sum(dev, rows, row_bytes):
    """qwhip_plane_checksum_rows (the decode GEMV's launch with the arithmetic taken out) adds every 32-bit word of the
    bank exactly once: ragged row slots, short sets, fewer rows than a window, a partly filled last chunk of lanes, a
    workgroup that ends in a half wave; refusals for rows that are not whole 20-byte pieces."""
    rng = np.random.default_rng(rows)
    host = rng.integers(0, 1 << 32, size=rows * row_bytes // 4, dtype=np.uint32)
    lib, st = dev.lib, dev.stream.handle
    plane, out = dev.put(host), dev.alloc(256 * 8)
    qwhip.check(lib.qwhip_fill_u32(st, out.ptr, 0, 512))
    qwhip.check(lib.qwhip_plane_checksum_rows(st, plane.ptr, rows, row_bytes, out.ptr))
    dev.stream.sync()
    assert int(out.download(np.uint64, (256,)).sum()) == int(host.astype(np.uint64).sum())
    assert lib.qwhip_plane_checksum_rows(st, plane.ptr, rows, row_bytes + 4, out.ptr) == qwhip.E_BAD_SHAPE
    assert lib.qwhip_plane_checksum_rows(st, plane.ptr, 0, row_bytes, out.ptr) == qwhip.OK


@pytest.mark.parametrize("nbytes", [16, 4096 + 16, 3 * 1024 * 1024 + 48, 55705600])
def test_plane_checksum_is_the_hosts_word_sum(dev, nbytes):
    """The sum of a plane's 32-bit words, exact in 64 bits whatever order the workgroups finish in; it adds into the 256
    words the caller cleared (two calls double their total); unaligned planes and ragged sizes are refused before any launch."""
    rng = np.random.default_rng(nbytes)
    host = rng.integers(0, 1 << 32, size=nbytes // 4, dtype=np.uint64).astype(np.uint32)
    plane, out = dev.put(host), dev.alloc(256 * 8)
    lib, st = dev.lib, dev.stream.handle
    qwhip.check(lib.qwhip_fill_u32(st, out.ptr, 0, 512))
    qwhip.check(lib.qwhip_plane_checksum(st, plane.ptr, nbytes, out.ptr))
    dev.stream.sync()
    want = int(host.astype(np.uint64).sum())
    assert int(out.download(np.uint64, (256,)).sum()) == want
    qwhip.check(lib.qwhip_plane_checksum(st, plane.ptr, nbytes, out.ptr))
    dev.stream.sync()
    assert int(out.download(np.uint64, (256,)).sum()) == 2 * want
    assert lib.qwhip_plane_checksum(st, plane.ptr, nbytes - 4, out.ptr) == qwhip.E_BAD_SHAPE
    if nbytes > 16:
        assert lib.qwhip_plane_checksum(st, plane.ptr + 4, nbytes - 16, out.ptr) == qwhip.E_BAD_SHAPE
    assert lib.qwhip_plane_checksum(st, plane.ptr, 0, out.ptr) == qwhip.OK
    plane.free()
    out.free()


@pytest.mark.parametrize("rows,vocab", [(4, 1000), (3, 151936), (2, 37)])
def test_argmax_variational_acceptance(dev, rows, vocab):
    """Relaxed acceptance of a draft over a verify window against the oracle: plain argmax without a margin, the margin rule, the
    log-probability gate on both sides of its threshold, out-of-vocabulary and last-row drafts."""
    import math
    rng = np.random.default_rng(rows + vocab)
    lg = rng.standard_normal((rows, vocab)).astype(np.float32)
    top = qo.head_argmax(lg)
    draft = rng.integers(0, vocab, rows + 1).astype(np.uint32)
    second = np.argsort(-lg[0], kind="stable")[1]
    draft[1] = second                                      # a near miss for row 0
    if rows > 2:
        draft[3] = vocab + 5                               # not a token
    lb, db, tb = dev.put(lg), dev.put(draft), dev.alloc(rows * 4)
    lib, st = dev.lib, dev.stream.handle

    def run(total, margin, min_lp):
        qwhip.check(lib.qwhip_argmax_f32_variational(st, lb.ptr, rows, vocab, db.ptr, total, margin, min_lp, tb.ptr))
        dev.stream.sync()
        return tb.download(np.int32, (rows,))

    assert np.array_equal(run(rows + 1, 0.0, -math.inf), top)
    gap = float(lg[0, top[0]] - lg[0, second])
    for margin in (gap * 0.5, gap * 1.5, 100.0):
        want = qo.head_argmax_variational(lg, draft, margin)
        assert np.array_equal(run(rows + 1, margin, -math.inf), want)
    assert run(rows + 1, gap * 1.5, -math.inf)[0] == second and run(rows + 1, gap * 0.5, -math.inf)[0] == top[0]
    want_short = qo.head_argmax_variational(lg, draft[:rows], 100.0)
    assert np.array_equal(run(rows, 100.0, -math.inf), want_short) and want_short[rows - 1] == top[rows - 1]
    mx = lg[0].astype(np.float64).max()
    lp = float(lg[0, second] - mx - np.log(np.exp(lg[0].astype(np.float64) - mx).sum()))
    assert run(rows + 1, gap * 1.5, lp - 0.01)[0] == second
    assert run(rows + 1, gap * 1.5, lp + 0.01)[0] == top[0]
    for min_lp in (lp - 0.01, lp + 0.01, -3.0):
        assert np.array_equal(run(rows + 1, 100.0, min_lp), qo.head_argmax_variational(lg, draft, 100.0, min_lp))
    assert lib.qwhip_argmax_f32_variational(st, lb.ptr, rows, vocab, db.ptr, rows + 1, 1.0, math.nan, tb.ptr) == qwhip.E_BAD_SHAPE


@pytest.mark.parametrize("rows,n,k", [(1, 40, 256), (5, 33, 100), (20, 8, 4096), (1, 4099, 512), (3000, 7, 64), (9, 1030, 96)])
@pytest.mark.parametrize("epi,scale", [(0, 1.0), (1, 2.0), (2, 1.0), (3, 0.5)])
def test_dense_f32_gemv_with_epilogues(dev, rows, n, k, epi, scale):
    rng = np.random.default_rng(n + k)
    w = (rng.standard_normal((n, k)) / np.sqrt(k)).astype(np.float32)
    x = rng.standard_normal((rows, k)).astype(np.float32)
    wb, xb, yb = dev.put(w), dev.put(x), dev.alloc(rows * n * 4)
    qwhip.check(dev.lib.qwhip_f32_gemv(dev.stream.handle, wb.ptr, xb.ptr, rows, n, k, epi, scale, yb.ptr))
    dev.stream.sync()
    got = yb.download(np.float32, (rows, n))
    assert qo.normalized_error(got, qo.f32_gemv(w, x, epi, scale)) <= 2e-6
    assert dev.lib.qwhip_f32_gemv(dev.stream.handle, wb.ptr, xb.ptr, rows, n, k, 4, 1.0, yb.ptr) == qwhip.E_BAD_SHAPE
    assert dev.lib.qwhip_f32_gemv(dev.stream.handle, wb.ptr, xb.ptr, rows, n, k, 1, 0.0, yb.ptr) == qwhip.E_BAD_SHAPE
