"""GPU parity of the MoE pieces (router, routing, pair sort + tile list, grouped GEMM, combine, decode
GEMVs) and of the whole routed block against the CPU oracle, through the C ABI."""
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


def _route(dev, logits, k, norm=True, scale=1.0):
    t, e = logits.shape
    lb, ib, wb = dev.put(logits.astype(np.float32)), dev.alloc(t * k * 4), dev.alloc(t * k * 4)
    qwhip.check(dev.lib.qwhip_moe_route(dev.stream.handle, lb.ptr, t, e, k, 1 if norm else 0, scale, ib.ptr, wb.ptr))
    return ib.download(np.int32, (t, k)), wb.download(np.float32, (t, k))


@pytest.mark.parametrize("t,e,k", [(64, 128, 8), (5, 8, 2), (33, 512, 16), (7, 100, 3)])
def test_moe_route_matches_oracle(dev, t, e, k):
    rng = np.random.default_rng(e + k)
    logits = rng.standard_normal((t, e)).astype(np.float32)
    idx, wts = _route(dev, logits, k, norm=True, scale=2.5)
    ridx, rwts = qo.moe_route(logits, k, norm_topk=True, routed_scale=2.5)
    assert np.array_equal(idx, ridx)
    np.testing.assert_allclose(wts, rwts, rtol=2e-6, atol=1e-9)
    idx2, wts2 = _route(dev, logits, k, norm=False)
    ridx2, rwts2 = qo.moe_route(logits, k, norm_topk=False)
    assert np.array_equal(idx2, ridx2)
    np.testing.assert_allclose(wts2, rwts2, rtol=2e-6, atol=1e-9)


def test_moe_route_ties_and_non_finite(dev):
    logits = np.zeros((3, 64), dtype=np.float32)          # all tied: lowest indices win, in order
    logits[1, 10] = np.inf                                 # non-finite never wins
    logits[1, 11] = np.nan
    logits[2, :] = -np.inf                                 # nothing to select
    logits[2, 5] = 1.0
    idx, wts = _route(dev, logits, 4)
    assert idx[0].tolist() == [0, 1, 2, 3]
    assert 10 not in idx[1] and 11 not in idx[1] and idx[1].tolist() == [0, 1, 2, 3]
    assert idx[2].tolist() == [5, -1, -1, -1]
    assert wts[2].tolist() == [1.0, 0.0, 0.0, 0.0]
    np.testing.assert_allclose(wts[0], 0.25, rtol=1e-6)


@pytest.mark.parametrize("xdt", ["f32", "bf16", "f16"])
def test_router_gemm(dev, xdt):
    t, e, h = 19, 128, 2048
    rng = np.random.default_rng(1)
    x = rng.standard_normal((t, h)).astype(np.float32)
    wr = (rng.standard_normal((e, h)) * 0.05).astype(np.float32)
    if xdt == "f32":
        xh, code, xv = x, qwhip.F32, x
    elif xdt == "bf16":
        xh, code, xv = qo.f32_to_bf16_bits(x), qwhip.BF16, qo.round_bf16(x)
    else:
        xh, code = x.astype(np.float16), qwhip.F16
        xv = xh.astype(np.float32)
    xb, wb, lb = dev.put(xh), dev.put(wr), dev.alloc(t * e * 4)
    qwhip.check(dev.lib.qwhip_router_gemm(dev.stream.handle, xb.ptr, code, wb.ptr, qwhip.F32, t, e, h, lb.ptr))
    got = lb.download(np.float32, (t, e))
    ref = xv.astype(np.float64) @ wr.astype(np.float64).T
    assert qo.normalized_error(got, ref) <= 1e-5


@pytest.mark.parametrize("t,e,h,wdt", [(19, 128, 2048, "f32"), (5, 64, 4096, "bf16"), (33, 40, 5120, "f32"), (3, 8, 16384, "f16")])
def test_router_gemm_shared_gate_and_wide_rows(dev, t, e, h, wdt):
    """The shared-expert gate column sigmoid(x . w) beside the logits, on hidden sizes that take 8, 4, 2 and 1 token rows
    per workgroup; the logits are those of the plain door bit for bit."""
    rng = np.random.default_rng(4)
    x = rng.standard_normal((t, h)).astype(np.float32)
    wr = (rng.standard_normal((e, h)) * 0.05).astype(np.float32)
    shw = (rng.standard_normal(h) * 0.03).astype(np.float32)
    if wdt == "f32":
        wh, wcode, wv = wr, qwhip.F32, wr
    elif wdt == "bf16":
        wh, wcode, wv = qo.f32_to_bf16_bits(wr), qwhip.BF16, qo.round_bf16(wr)
    else:
        wh, wcode = wr.astype(np.float16), qwhip.F16
        wv = wh.astype(np.float32)
    xb, wb, sb = dev.put(x), dev.put(wh), dev.put(shw)
    l1, l2, go = dev.alloc(t * e * 4), dev.alloc(t * e * 4), dev.alloc(t * 4)
    lib, st = dev.lib, dev.stream.handle
    qwhip.check(lib.qwhip_router_gemm_shared_gate(st, xb.ptr, qwhip.F32, wb.ptr, wcode, t, e, h, l1.ptr, sb.ptr, go.ptr))
    qwhip.check(lib.qwhip_router_gemm(st, xb.ptr, qwhip.F32, wb.ptr, wcode, t, e, h, l2.ptr))
    dev.stream.sync()
    got, plain, gate = l1.download(np.float32, (t, e)), l2.download(np.float32, (t, e)), go.download(np.float32, (t,))
    assert np.array_equal(got.view(np.uint32), plain.view(np.uint32))
    assert qo.normalized_error(got, x.astype(np.float64) @ wv.astype(np.float64).T) <= 1e-5
    np.testing.assert_allclose(gate, qo.router_shared_gate_f64(x, shw), rtol=0, atol=2e-6)
    assert lib.qwhip_router_gemm_shared_gate(st, xb.ptr, qwhip.F32, wb.ptr, wcode, t, e, h, l1.ptr, sb.ptr, None) == qwhip.E_NULL
    assert lib.qwhip_router_gemm(st, xb.ptr, qwhip.F32, wb.ptr, wcode, t, e, 16388, l1.ptr) == qwhip.E_BAD_SHAPE


@pytest.mark.parametrize("t,e,k", [(33, 128, 8), (5, 40, 4), (9, 512, 16), (7, 100, 3)])
@pytest.mark.parametrize("mode", ["bias", "split", "bias+split", "softmax+scale"])
@pytest.mark.parametrize("norm", [0, 1])
def test_route_modes_match_oracle(dev, t, e, k, mode, norm):
    """qwhip_moe_route_ex: sigmoid scoring with a selection bias and / or split-feature logits, and the per-expert scale;
    the choice is the oracle's exactly (ties and non-finite logits included), the weights within 2e-6."""
    rng = np.random.default_rng(t * 7 + e)
    split = "split" in mode
    lg = rng.standard_normal((t, 2 * e if split else e)).astype(np.float32)
    lg[0, 1] = lg[0, 0]                                        # a tie
    lg[t - 1, 2] = np.nan
    lg[t - 1, 3] = -np.inf
    bias = (rng.standard_normal(e) * 0.5).astype(np.float32) if "bias" in mode else None
    scale = (rng.random(e) + 0.5).astype(np.float32) if "scale" in mode else None
    lb, ib, wb = dev.put(lg), dev.alloc(t * k * 4), dev.alloc(t * k * 4)
    bb = dev.put(bias) if bias is not None else None
    sb = dev.put(scale) if scale is not None else None
    qwhip.check(dev.lib.qwhip_moe_route_ex(dev.stream.handle, lb.ptr, t, e, k, norm, 1.5, 1 if split else 0, bb.ptr if bb else None,
                                           sb.ptr if sb else None, ib.ptr, wb.ptr))
    dev.stream.sync()
    idx, wts = ib.download(np.int32, (t, k)), wb.download(np.float32, (t, k))
    ridx, rwts = qo.moe_route_ex(lg, k, bool(norm), 1.5, bias=bias, split_feature=split, scale_param=scale)
    assert np.array_equal(idx, ridx)
    np.testing.assert_allclose(wts, rwts, rtol=2e-6, atol=1e-9)


def _group(dev, ids, experts, top_k, compact=True):
    pairs = ids.size
    mt = max(1, dev.lib.qwhip_moe_max_tiles(experts, pairs))
    b = dict(ids=dev.put(ids.astype(np.int32)), off=dev.alloc((experts + 1) * 4), sp=dev.alloc(pairs * 4), stok=dev.alloc(pairs * 4),
             inv=dev.alloc(pairs * 4), te=dev.alloc(mt * 4), tr=dev.alloc(mt * 4), tc=dev.alloc(16))
    qwhip.check(dev.lib.qwhip_moe_group_pairs(dev.stream.handle, b["ids"].ptr, experts, pairs, top_k, b["off"].ptr, b["sp"].ptr,
                                              b["stok"].ptr, b["inv"].ptr, b["te"].ptr, b["tr"].ptr, b["tc"].ptr, 1 if compact else 0))
    dev.stream.sync()
    out = dict(off=b["off"].download(np.int32, (experts + 1,)), sp=b["sp"].download(np.int32, (pairs,)),
               stok=b["stok"].download(np.int32, (pairs,)), inv=b["inv"].download(np.int32, (pairs,)),
               tc=int(b["tc"].download(np.int32, (1,))[0]))
    out["te"] = b["te"].download(np.int32, (mt,))[: out["tc"]]
    out["tr"] = b["tr"].download(np.int32, (mt,))[: out["tc"]]
    out["bufs"], out["max_tiles"] = b, mt
    return out


@pytest.mark.parametrize("t,e,k,compact", [(300, 128, 8, True), (300, 128, 8, False), (3, 16, 2, True), (2048, 128, 8, True), (50, 512, 16, True)])
def test_moe_group_pairs_invariants_and_tiles(dev, t, e, k, compact):
    """Sort invariants (Tests/QWFlashNextMetalTests/MoE/FNMetalMoEGroupTests.swift:80-92) and the tile list
    against the closed forms of QWGemmMoE.swift:24-62 / qw_moe_tile.metalh."""
    rng = np.random.default_rng(t + e)
    ids = np.stack([rng.choice(e, size=k, replace=False) for _ in range(t)]).astype(np.int32)
    ids[rng.random(ids.shape) < 0.02] = -1                     # a few empty routes
    g = _group(dev, ids, e, k, compact)
    ref = qo.moe_group_pairs(ids, e, k, compact_tail=compact)
    valid = int((ids >= 0).sum())
    assert g["off"][0] == 0 and g["off"][e] == valid and np.all(np.diff(g["off"]) >= 0)
    assert np.array_equal(g["off"], ref["expertOff"])
    sp = g["sp"][:valid]
    assert np.array_equal(np.sort(sp), np.flatnonzero(ids.ravel() >= 0))           # each valid pair exactly once
    assert np.array_equal(g["stok"][:valid], sp // k)
    assert np.array_equal(g["inv"][sp], np.arange(valid))                           # invPerm o sortedPairIdx = id
    assert np.all(g["inv"][ids.ravel() < 0] == -1)
    flat = ids.ravel()
    for ex in range(e):                                                             # slots of expert ex hold its pairs
        assert np.all(flat[sp[g["off"][ex]:g["off"][ex + 1]]] == ex)
    assert g["tc"] == ref["tileCount"] <= g["max_tiles"]
    assert np.array_equal(g["te"], ref["tileE"]) and np.array_equal(g["tr"], ref["tileR"])


def _moe_banks(experts, hidden, inter, seed, fmt="hq4_g32_m5"):
    gu_blocks, gu16 = H.make_bank(fmt, experts * 2 * inter, hidden, seed)
    dn_blocks, dn16 = H.make_bank(fmt, experts * hidden, inter, seed + 1)
    return gu_blocks, gu16.reshape(experts, 2 * inter, hidden), dn_blocks, dn16.reshape(experts, hidden, inter)


def _hidden_rows(rng, t, hidden, xdt):
    """Hidden rows in the experts' basis as the device takes them (f16 values, or bf16 bit patterns), their dtype code, and
    the values they hold."""
    x32 = rng.standard_normal((t, hidden)).astype(np.float32)
    if xdt == "f16":
        xh = qo.rotate_activation_f16(x32)
        return xh, qwhip.F16, xh.astype(np.float32)
    bits = qo.f32_to_bf16_bits(qo.fwht32_ortho(x32))
    return bits, qwhip.BF16, qo.bf16_bits_to_f32(bits)


@pytest.mark.parametrize("xdt", ["f16", "bf16"])
@pytest.mark.parametrize("t,experts,hidden,inter,k", [(40, 8, 256, 128, 2), (130, 16, 512, 192, 4)])
def test_moe_prefill_chain_matches_oracle(dev, t, experts, hidden, inter, k, xdt):
    """route -> pair sort -> grouped gate_up GEMM -> SwiGLU+FWHT -> grouped down GEMM -> combine; f16 and bf16 hidden rows."""
    fmt = "hq4_g32_m5"
    gu_blocks, gu16, dn_blocks, dn16 = _moe_banks(experts, hidden, inter, seed=11)
    rng = np.random.default_rng(5)
    x16, xcode, xval = _hidden_rows(rng, t, hidden, xdt)                                     # rotated hidden rows
    logits = rng.standard_normal((t, experts)).astype(np.float32)
    idx, wts = _route(dev, logits, k)
    g = _group(dev, idx, experts, k)
    pairs = t * k
    lib, st, b = dev.lib, dev.stream.handle, g["bufs"]
    gub, dnb, xb = dev.put(gu_blocks), dev.put(dn_blocks), dev.put(x16)
    gu_out, act, dn_out, out = dev.alloc(pairs * 2 * inter * 2), dev.alloc(pairs * inter * 2), dev.alloc(pairs * hidden * 4), dev.alloc(t * hidden * 4)
    wb = dev.put(wts)
    vgu = H.view_of(dev, gub, fmt, experts * 2 * inter, hidden)
    vdn = H.view_of(dev, dnb, fmt, experts * hidden, inter)
    qwhip.check(lib.qwhip_moe_grouped_gemm(st, C.byref(vgu), experts, xb.ptr, xcode, 0, b["stok"].ptr, b["off"].ptr, b["te"].ptr,
                                           b["tr"].ptr, b["tc"].ptr, g["max_tiles"], pairs, gu_out.ptr, qwhip.F16, 0))
    qwhip.check(lib.qwhip_swiglu_fwht(st, gu_out.ptr, qwhip.F16, act.ptr, pairs, inter, 1))
    qwhip.check(lib.qwhip_moe_grouped_gemm(st, C.byref(vdn), experts, act.ptr, qwhip.F16, 0, None, b["off"].ptr, b["te"].ptr,
                                           b["tr"].ptr, b["tc"].ptr, g["max_tiles"], pairs, dn_out.ptr, qwhip.F32, 0))
    qwhip.check(lib.qwhip_moe_combine(st, dn_out.ptr, qwhip.F32, b["inv"].ptr, wb.ptr, t, k, hidden, None, None, out.ptr, qwhip.F32))
    dev.stream.sync()
    got = out.download(np.float32, (t, hidden))
    ref = qo.moe_forward_f64(xval, idx, wts, gu16, dn16, act_f16=True, rotate_act=True)
    assert qo.normalized_error(got, ref) <= TOL
    assert np.allclose(qo.moe_forward_grouped_f64(xval, idx, wts, gu16, dn16, act_f16=True, rotate_act=True), ref, rtol=1e-3, atol=1e-5)


@pytest.mark.parametrize("fmt", ["hq4_g32_m5", "hq4_g32", "hq4_g64", "hq8_g32", "aq2_g64", "hq3_g32", "hq6_g32"])
@pytest.mark.parametrize("t,experts,hidden,inter,k,rot", [(40, 8, 256, 128, 2, 1), (130, 16, 512, 192, 4, 1), (300, 4, 128, 64, 2, 0),
                                                          (64, 8, 192, 448, 3, 1)])
@pytest.mark.parametrize("xdt", ["f16", "bf16"])
def test_fused_gate_up_swiglu_equals_the_two_step_chain(dev, fmt, t, experts, hidden, inter, k, rot, xdt):
    """qwhip_moe_grouped_gemm_swiglu == qwhip_moe_grouped_gemm (f16 out) + qwhip_swiglu_fwht, bit for bit, on the rows of the
    sorted list (intermediate sizes with a partial 128-column tile included), and the chain built on it meets the oracle;
    f16 and bf16 hidden rows on every container."""
    gu_blocks, gu16, dn_blocks, dn16 = _moe_banks(experts, hidden, inter, seed=13, fmt=fmt)
    rng = np.random.default_rng(9)
    x16, xcode, xval = _hidden_rows(rng, t, hidden, xdt)
    logits = rng.standard_normal((t, experts)).astype(np.float32)
    idx, wts = _route(dev, logits, k)
    g = _group(dev, idx, experts, k)
    pairs = t * k
    lib, st, b = dev.lib, dev.stream.handle, g["bufs"]
    gub, xb = dev.put(gu_blocks), dev.put(x16)
    gu_out = dev.alloc(pairs * 2 * inter * 2)
    act2, act1 = dev.put(np.zeros((pairs, inter), np.float16)), dev.put(np.zeros((pairs, inter), np.float16))
    vgu = H.view_of(dev, gub, fmt, experts * 2 * inter, hidden)
    qwhip.check(lib.qwhip_moe_grouped_gemm(st, C.byref(vgu), experts, xb.ptr, xcode, 0, b["stok"].ptr, b["off"].ptr, b["te"].ptr,
                                           b["tr"].ptr, b["tc"].ptr, g["max_tiles"], pairs, gu_out.ptr, qwhip.F16, 0))
    qwhip.check(lib.qwhip_swiglu_fwht(st, gu_out.ptr, qwhip.F16, act2.ptr, pairs, inter, rot))
    qwhip.check(lib.qwhip_moe_grouped_gemm_swiglu(st, C.byref(vgu), experts, xb.ptr, xcode, 0, b["stok"].ptr, b["off"].ptr,
                                                  b["te"].ptr, b["tr"].ptr, b["tc"].ptr, g["max_tiles"], pairs, rot, act1.ptr, 0))
    dev.stream.sync()
    valid = int(g["off"][experts])
    two, one = act2.download(np.float16, (pairs, inter))[:valid], act1.download(np.float16, (pairs, inter))[:valid]
    assert np.array_equal(one.view(np.uint16), two.view(np.uint16))
    # against the oracle: act of sorted slot p = swiglu(x[tok] . gate_e, x[tok] . up_e), rotated
    e_of = np.repeat(np.arange(experts), np.diff(g["off"]))
    xs = xval[g["stok"][:valid]].astype(np.float64)
    gu = np.einsum("pk,pnk->pn", xs, gu16[e_of].astype(np.float64)).astype(np.float16).astype(np.float32)
    want = qo.swiglu_fwht_f16(gu[:, :inter], gu[:, inter:], rotate=bool(rot)).astype(np.float32)
    assert qo.normalized_error(one.astype(np.float32), want) <= TOL


def test_fused_gate_up_swiglu_refusals(dev):
    blocks, _ = H.make_bank("hq4_g32_m5", 4 * 2 * 48, 64, 1)
    bank, xb, act = dev.put(blocks), dev.put(np.zeros((4, 64), np.float16)), dev.alloc(4096)
    z = dev.put(np.zeros(64, np.int32))
    lib, st = dev.lib, dev.stream.handle
    v = H.view_of(dev, bank, "hq4_g32_m5", 4 * 2 * 48, 64)
    args = (z.ptr, z.ptr, z.ptr, z.ptr, 4, 4, 1, act.ptr, 0)
    assert lib.qwhip_moe_grouped_gemm_swiglu(st, C.byref(v), 4, xb.ptr, qwhip.F16, 0, None, *args) == qwhip.E_BAD_GEOMETRY   # inter = 48
    v2 = H.view_of(dev, bank, "hq4_g32_m5", 4 * 2 * 48, 64)
    assert lib.qwhip_moe_grouped_gemm_swiglu(st, C.byref(v2), 3, xb.ptr, qwhip.F32, 0, None, *args) == qwhip.E_BAD_WEIGHTS   # f32 activations
    assert lib.qwhip_moe_grouped_gemm_swiglu(st, C.byref(v2), 5, xb.ptr, qwhip.BF16, 0, None, *args) == qwhip.E_BAD_SHAPE    # 384 rows over 5 experts


def test_grouped_gemm_refuses_expert_of_4gib(dev):
    """One expert whose rows span 4 GiB or more is refused by both doors before any launch: the kernels address the rows
    of an expert with 32-bit offsets. The bank is device memory that nothing reads."""
    k, rows = 16384, 419456                      # 419456 rows x 10240 bytes = 4.0002 GiB
    bank = dev.alloc(rows * (k // 32) * 20)
    xb, out, z = dev.put(np.zeros((4, k), np.float16)), dev.alloc(4096), dev.put(np.zeros(64, np.int32))
    lib, st = dev.lib, dev.stream.handle
    v = H.view_of(dev, bank, "hq4_g32_m5", rows, k)
    tiles = (z.ptr, z.ptr, z.ptr, z.ptr, 4, 4)
    assert lib.qwhip_moe_grouped_gemm(st, C.byref(v), 1, xb.ptr, qwhip.F16, 0, None, *tiles, out.ptr, qwhip.F16, 0) == qwhip.E_BAD_GEOMETRY
    assert lib.qwhip_moe_grouped_gemm_swiglu(st, C.byref(v), 1, xb.ptr, qwhip.F16, 0, None, *tiles, 1, out.ptr, 0) == qwhip.E_BAD_GEOMETRY


# (format, gate_up kernel override): HQ4_G32_M5 runs the column-stationary kernels, override 2 keeps its gate_up on the
# general kernel; the bit-stream container runs the general kernels for both projections.
@pytest.mark.parametrize("fmt,gu_flags", [("hq4_g32_m5", 0), ("hq4_g32_m5", 2 << 8), ("hq4_g32", 0), ("hq3_g32", 0), ("hq6_g32", 0)])
@pytest.mark.parametrize("experts,hidden,inter,k", [(16, 512, 192, 4), (8, 1280, 96, 3), (4, 2048, 768, 4)])
@pytest.mark.parametrize("t", [1, 3, 8])
@pytest.mark.parametrize("xdt", ["f16", "bf16"])
def test_moe_decode_chain_matches_oracle(dev, t, xdt, experts, hidden, inter, k, fmt, gu_flags):
    """Decode / verify path: routed gate_up GEMV (+SwiGLU+FWHT) and routed down GEMV with weighted combine,
    un-rotated activations in, fused rotation; shapes with partial 32-block chunks and ragged row tiles."""
    gu_blocks, gu16, dn_blocks, dn16 = _moe_banks(experts, hidden, inter, seed=21, fmt=fmt)
    rng = np.random.default_rng(6)
    x32 = rng.standard_normal((t, hidden)).astype(np.float32)
    if xdt == "f16":
        xh, code, xv = x32.astype(np.float16), qwhip.F16, x32.astype(np.float16).astype(np.float32)
    else:
        xh, code, xv = qo.f32_to_bf16_bits(x32), qwhip.BF16, qo.round_bf16(x32)
    logits = rng.standard_normal((t, experts)).astype(np.float32)
    idx, wts = _route(dev, logits, k)
    idx[0, k - 1] = -1                                         # an empty route is skipped
    shared = rng.standard_normal((t, hidden)).astype(np.float32)
    gate = rng.random(t).astype(np.float32)
    lib, st = dev.lib, dev.stream.handle
    gub, dnb, xb, ib, wb = dev.put(gu_blocks), dev.put(dn_blocks), dev.put(xh), dev.put(idx), dev.put(wts)
    sb, gb = dev.put(shared), dev.put(gate)
    act, out = dev.alloc(t * k * inter * 2), dev.alloc(t * hidden * 4)
    vgu = H.view_of(dev, gub, fmt, experts * 2 * inter, hidden)
    vdn = H.view_of(dev, dnb, fmt, experts * hidden, inter)
    qwhip.check(lib.qwhip_moe_gateup_decode(st, C.byref(vgu), experts, xb.ptr, code, gu_flags, ib.ptr, t, k, act.ptr))
    qwhip.check(lib.qwhip_moe_down_decode(st, C.byref(vdn), experts, act.ptr, ib.ptr, wb.ptr, t, k, sb.ptr, gb.ptr, out.ptr, qwhip.F32))
    dev.stream.sync()
    got = out.download(np.float32, (t, hidden))
    x_rot = qo.fwht32_ortho(xv).astype(np.float16)
    ref = qo.moe_forward_f64(x_rot, idx, wts, gu16, dn16, act_f16=True, rotate_act=True) + gate[:, None].astype(np.float64) * shared
    assert qo.normalized_error(got, ref) <= TOL
    a = act.download(np.float16, (t, k, inter))
    assert np.all(a[0, k - 1] == 0)


@pytest.mark.parametrize("xdt", ["f16", "bf16"])
@pytest.mark.parametrize("hidden,inter", [(256, 96), (2048, 160), (3072, 64), (5120, 40)])
@pytest.mark.parametrize("t,k,experts", [(2, 8, 12), (3, 4, 6), (4, 8, 40), (4, 16, 20), (4, 8, 8)])
def test_gateup_decode_reads_a_shared_expert_once_with_the_same_bits(dev, t, k, experts, hidden, inter, xdt):
    """A verify window of 2..4 tokens whose rows share experts: QWHIP_MOE_REUSE_EXPERTS reads a shared expert once for all
    of its tokens (encodeMoEGateUpF32R1's reuseExpertsAcrossTokens, QWGemmMoE.swift:119-132; QWMoEReuseTests.swift:46-186 compares
    the two modes) and must leave the bits of the launch that keeps every (token, route) pair to itself.  Few experts force
    sharing (with 8 experts and top-8 every token routes to all of them); the list also holds a repeated expert inside one
    token, an absent route, and the route door is run on the same window."""
    fmt = "hq4_g32_m5"
    gu_blocks, _ = H.make_bank(fmt, experts * 2 * inter, hidden, 77)
    rng = np.random.default_rng(1000 * t + k + hidden)
    x32 = rng.standard_normal((t, hidden)).astype(np.float32)
    xh, code = (x32.astype(np.float16), qwhip.F16) if xdt == "f16" else (qo.f32_to_bf16_bits(x32), qwhip.BF16)
    logits = rng.standard_normal((t, experts)).astype(np.float32)
    ref_idx, _ = qo.moe_route(logits, min(k, experts), True, 1.0)
    idx = np.full((t, k), -1, np.int32)
    idx[:, :ref_idx.shape[1]] = ref_idx
    if k > ref_idx.shape[1]:
        idx[:, ref_idx.shape[1]:] = rng.integers(0, experts, (t, k - ref_idx.shape[1]))   # repeats inside a token
    idx[t - 1, 1] = idx[t - 1, 0]                              # a token's second route to one expert
    idx[0, k - 1] = -1                                         # an absent route
    shared_pairs = sum(int(np.isin(idx[r][idx[r] >= 0], idx[:r][idx[:r] >= 0]).sum()) for r in range(1, t))
    assert shared_pairs > 0
    lib, st = dev.lib, dev.stream.handle
    gub, xb, ib = dev.put(gu_blocks), dev.put(xh), dev.put(idx)
    v = H.view_of(dev, gub, fmt, experts * 2 * inter, hidden)
    a1, a2 = dev.put(np.full((t, k, inter), 3, np.float16)), dev.put(np.full((t, k, inter), 5, np.float16))
    qwhip.check(lib.qwhip_moe_gateup_decode(st, C.byref(v), experts, xb.ptr, code, qwhip.MOE_REUSE_EXPERTS, ib.ptr, t, k, a1.ptr))
    qwhip.check(lib.qwhip_moe_gateup_decode(st, C.byref(v), experts, xb.ptr, code, 0, ib.ptr, t, k, a2.ptr))
    dev.stream.sync()
    one, two = a1.download(np.uint16, (t, k, inter)), a2.download(np.uint16, (t, k, inter))
    assert np.array_equal(one, two)
    assert np.all(one[idx < 0] == 0) and np.any(one != 0)
    if k <= experts:   # the same window through the door that routes inside the launch
        i1, w1, i2, w2 = (dev.alloc(t * k * 4 + 256) for _ in range(4))
        lb = dev.put(logits)
        qwhip.check(lib.qwhip_moe_route_gateup_decode(st, C.byref(v), experts, xb.ptr, code, qwhip.MOE_REUSE_EXPERTS, lb.ptr, t, k, 1, 1.0, i1.ptr, w1.ptr, a1.ptr))
        qwhip.check(lib.qwhip_moe_route_gateup_decode(st, C.byref(v), experts, xb.ptr, code, 0, lb.ptr, t, k, 1, 1.0,
                                                      i2.ptr, w2.ptr, a2.ptr))
        dev.stream.sync()
        assert np.array_equal(i1.download(np.int32, (t, k)), ref_idx) and np.array_equal(i2.download(np.int32, (t, k)), ref_idx)
        assert np.array_equal(w1.download(np.uint32, (t, k)), w2.download(np.uint32, (t, k)))
        assert np.array_equal(a1.download(np.uint16, (t, k, inter)), a2.download(np.uint16, (t, k, inter)))


@pytest.mark.parametrize("fmt", ["hq4_g32_m5", "hq4_g64"])
@pytest.mark.parametrize("t", [1, 3])
def test_decode_chain_replays_from_a_hip_graph(dev, fmt, t):
    """The decode doors only enqueue kernels, so a caller bound by launch latency can capture the chain (routing + gate_up,
    down + combine) as a HIP graph.  The graph is replayed several times with eager launches and synchronisations of the
    same doors in between (on other buffers and other inputs), and every replay must leave the eager chain's bits."""
    experts, hidden, inter, k = 16, 512, 192, 4
    gu_blocks, _, dn_blocks, _ = _moe_banks(experts, hidden, inter, seed=31, fmt=fmt)
    rng = np.random.default_rng(12)
    lib, st = dev.lib, dev.stream.handle
    gub, dnb = dev.put(gu_blocks), dev.put(dn_blocks)
    vgu = H.view_of(dev, gub, fmt, experts * 2 * inter, hidden)
    vdn = H.view_of(dev, dnb, fmt, experts * hidden, inter)

    def buffers():
        return dict(x=dev.alloc(t * hidden * 2), lg=dev.alloc(t * experts * 4), idx=dev.alloc(t * k * 4 + 256), wts=dev.alloc(t * k * 4 + 256),
                    act=dev.alloc(t * k * inter * 2), out=dev.alloc(t * hidden * 4))

    def chain(b):
        qwhip.check(lib.qwhip_moe_route_gateup_decode(st, C.byref(vgu), experts, b["x"].ptr, qwhip.F16, 0, b["lg"].ptr, t, k, 1, 1.0,
                                                      b["idx"].ptr, b["wts"].ptr, b["act"].ptr))
        qwhip.check(lib.qwhip_moe_down_decode(st, C.byref(vdn), experts, b["act"].ptr, b["idx"].ptr, b["wts"].ptr, t, k, None, None,
                                              b["out"].ptr, qwhip.F32))

    def fill(b):
        b["x"].upload(rng.standard_normal((t, hidden)).astype(np.float16))
        b["lg"].upload(rng.standard_normal((t, experts)).astype(np.float32))

    g, e = buffers(), buffers()          # the graph's buffers and the eager chain's
    fill(g)
    chain(g)                             # the kernels are loaded before the capture
    dev.stream.sync()
    graph = qwhip.Graph(dev.stream, lambda: chain(g))
    for replay in range(4):
        fill(g)                                            # new inputs in the captured buffers
        e["x"].upload(g["x"].download(np.float16, (t, hidden)))
        e["lg"].upload(g["lg"].download(np.float32, (t, experts)))
        g["out"].upload(np.full((t, hidden), 7.0, np.float32))
        graph.launch()
        chain(e)                                           # the same doors, eagerly, behind the replay on the stream
        dev.stream.sync()
        assert np.array_equal(g["out"].download(np.uint32, (t, hidden)), e["out"].download(np.uint32, (t, hidden))), replay
        assert np.array_equal(g["idx"].download(np.int32, (t, k)), e["idx"].download(np.int32, (t, k))), replay
    graph.destroy()


@pytest.mark.parametrize("fmt", ["hq4_g32_m5", "hq4_g32"])
@pytest.mark.parametrize("t,experts,hidden,inter,k", [(1, 128, 512, 96, 8), (3, 16, 1280, 192, 4), (8, 200, 256, 64, 3)])
def test_fused_route_gateup_decode_equals_the_two_launches(dev, fmt, t, experts, hidden, inter, k):
    """qwhip_moe_route_gateup_decode leaves the ids, weights and activations of qwhip_moe_route + qwhip_moe_gateup_decode, bit
    for bit (the HQ4_G32_M5 bank routes inside the gate_up kernel, the bit-stream bank runs the two launches)."""
    gu_blocks, _, _, _ = _moe_banks(experts, hidden, inter, seed=23, fmt=fmt)
    rng = np.random.default_rng(8)
    xh = rng.standard_normal((t, hidden)).astype(np.float16)
    logits = rng.standard_normal((t, experts)).astype(np.float32)
    logits[0, 3] = np.inf                                      # a non-finite logit never wins
    logits[t - 1, 5] = logits[t - 1, 9]                        # a tie goes to the lower id
    lib, st = dev.lib, dev.stream.handle
    gub, xb, lb = dev.put(gu_blocks), dev.put(xh), dev.put(logits)
    vgu = H.view_of(dev, gub, fmt, experts * 2 * inter, hidden)
    i2, w2, a2 = dev.alloc(t * k * 4 + 256), dev.alloc(t * k * 4 + 256), dev.alloc(t * k * inter * 2)
    i1, w1, a1 = dev.alloc(t * k * 4 + 256), dev.alloc(t * k * 4 + 256), dev.alloc(t * k * inter * 2)
    qwhip.check(lib.qwhip_moe_route(st, lb.ptr, t, experts, k, 1, 2.5, i2.ptr, w2.ptr))
    qwhip.check(lib.qwhip_moe_gateup_decode(st, C.byref(vgu), experts, xb.ptr, qwhip.F16, 0, i2.ptr, t, k, a2.ptr))
    qwhip.check(lib.qwhip_moe_route_gateup_decode(st, C.byref(vgu), experts, xb.ptr, qwhip.F16, 0, lb.ptr, t, k, 1, 2.5, i1.ptr, w1.ptr, a1.ptr))
    dev.stream.sync()
    assert np.array_equal(i1.download(np.int32, (t, k)), i2.download(np.int32, (t, k)))
    assert np.array_equal(w1.download(np.uint32, (t, k)), w2.download(np.uint32, (t, k)))
    assert np.array_equal(a1.download(np.uint16, (t, k, inter)), a2.download(np.uint16, (t, k, inter)))
    ref_idx, ref_w = qo.moe_route(logits, k, True, 2.5)
    assert np.array_equal(i1.download(np.int32, (t, k)), ref_idx)


def test_online_quantizer_writes_the_packers_bytes(dev):
    """Device HQ4_G32_M5 quantizer vs the oracle's restatement of the packer, byte-identical
    (Tests/QWFlashNextMetalTests/QUANT/FNMetalOnlineQuantTests.swift:243), bf16 and f32 sources, rotate on/off."""
    w = H.make_weights(96, 1024, seed=4)
    w[3, :32] = 0.0
    w[5, 7] = 3.0
    for src_kind in ("f32", "bf16"):
        if src_kind == "bf16":
            host, code, val = qo.f32_to_bf16_bits(w), qwhip.BF16, qo.round_bf16(w)
        else:
            host, code, val = w, qwhip.F32, w
        for rotate in (1, 0):
            sb, ob = dev.put(host), dev.alloc(96 * 32 * 20)
            qwhip.check(dev.lib.qwhip_quantize_hq4_g32(dev.stream.handle, sb.ptr, code, 96, 1024, rotate, ob.ptr))
            got = ob.download(np.uint8, (96, 32, 20))
            assert np.array_equal(got, qo.quant_hq4_blocks(val, rotate=bool(rotate)))


def test_swiglu_fwht_matches_oracle(dev):
    rng = np.random.default_rng(2)
    rows, inter = 9, 160
    gu = (rng.standard_normal((rows, 2 * inter)) * 2).astype(np.float16)
    gb, ab = dev.put(gu), dev.alloc(rows * inter * 2)
    for rotate in (1, 0):
        qwhip.check(dev.lib.qwhip_swiglu_fwht(dev.stream.handle, gb.ptr, qwhip.F16, ab.ptr, rows, inter, rotate))
        got = ab.download(np.float16, (rows, inter)).astype(np.float32)
        want = qo.swiglu_fwht_f16(gu[:, :inter].astype(np.float32), gu[:, inter:].astype(np.float32), rotate=bool(rotate)).astype(np.float32)
        assert np.max(np.abs(got - want)) <= 2e-3 * max(1.0, float(np.max(np.abs(want))))


@pytest.mark.parametrize("t", [1, 2048])
def test_moe_full_size_operator(t):
    """C4 at its real shape (128 experts, top-8, hidden 2048, intermediate 768, bf16 hidden rows): device-quantized banks
    byte-checked against the oracle on expert 0, routing identical, EVERY token against the fp64 oracle (prefill: the
    oracle's expert-ordered form, which makes the 155 GFLOP of fp64 products a matter of seconds)."""
    import argparse

    import bench
    out = bench.run_moe(argparse.Namespace(steps=2, warmup=1, no_cpu=True), t, "full-size parity")
    assert out["normalized_error"] <= TOL and out["tokens_checked"] == t and out["config"]["activations"] == "bf16"
    assert out["worst_token_error"] <= TOL


def test_moe_full_size_operator_f16_rows():
    """The same prefill batch on f16 hidden rows (the reference's own activation type), every token."""
    import argparse

    import bench
    out = bench.run_moe(argparse.Namespace(steps=2, warmup=1, no_cpu=True, moe_f16=True), 2048, "full-size parity, f16 rows")
    assert out["normalized_error"] <= TOL and out["tokens_checked"] == 2048 and out["config"]["activations"] == "f16"


@pytest.mark.parametrize("hidden", [256, 1000])
@pytest.mark.parametrize("dtype", ["f32", "f16"])
def test_combine_identity_slots_and_unit_weights(dev, hidden, dtype):
    """The door's invPerm: nil and unweightedSingle forms (encodeMoEDownReduceCombineF32, QWGemmMoE.swift:299-332): without
    a permutation route k of token t is row t * top_k + k, without weights every route counts once; with one route that is
    out = dn + gate * shared (the last step of the latent operator), in place when the types agree."""
    rng = np.random.default_rng(hidden)
    t, k = 5, 3
    dn = rng.standard_normal((t * k, hidden)).astype(np.float32)
    dn_h = dn.astype(np.float16) if dtype == "f16" else dn
    wts = rng.random((t, k)).astype(np.float32)
    shared = rng.standard_normal((t, hidden)).astype(np.float32)
    gate = rng.random(t).astype(np.float32)
    lib, st = dev.lib, dev.stream.handle
    code = qwhip.F16 if dtype == "f16" else qwhip.F32
    d_dn, d_w, d_sh, d_g, d_out = dev.put(dn_h), dev.put(wts), dev.put(shared), dev.put(gate), dev.alloc(t * hidden * 4)
    base = dn_h.astype(np.float64).reshape(t, k, hidden)
    # identity slots with weights
    qwhip.check(lib.qwhip_moe_combine(st, d_dn.ptr, code, None, d_w.ptr, t, k, hidden, None, None, d_out.ptr, qwhip.F32))
    dev.stream.sync()
    want = (base * wts[:, :, None].astype(np.float64)).sum(1)
    assert np.max(np.abs(d_out.download(np.float32, (t, hidden)) - want)) <= 1e-5 * np.abs(want).max()
    # unit weights with the gated shared rows
    qwhip.check(lib.qwhip_moe_combine(st, d_dn.ptr, code, None, None, t, k, hidden, d_sh.ptr, d_g.ptr, d_out.ptr, qwhip.F32))
    dev.stream.sync()
    want = base.sum(1) + gate[:, None].astype(np.float64) * shared
    assert np.max(np.abs(d_out.download(np.float32, (t, hidden)) - want)) <= 1e-5 * np.abs(want).max()
    if dtype == "f32":   # one route, in place: dn += gate * shared
        rows = dev.put(dn[:t])
        qwhip.check(lib.qwhip_moe_combine(st, rows.ptr, qwhip.F32, None, None, t, 1, hidden, d_sh.ptr, d_g.ptr, rows.ptr, qwhip.F32))
        dev.stream.sync()
        want = dn[:t].astype(np.float64) + gate[:, None].astype(np.float64) * shared
        assert np.max(np.abs(rows.download(np.float32, (t, hidden)) - want)) <= 1e-6 * np.abs(want).max()
        rows.free()
    for b in (d_dn, d_w, d_sh, d_g, d_out):
        b.free()


# ---- group-latent MoE: the doors and the whole block -------------------------------------------------------------------
def _latent_routes(rng, t, e, k, ng, hole=True):
    idx = np.stack([rng.permutation(e)[:k] for _ in range(t)]).astype(np.int32)
    if hole and t * k > 1:
        idx[0, k - 1] = -1
    wts = (rng.random((t, k)) + 0.1).astype(np.float32)
    labels = rng.integers(0, ng, e).astype(np.int32)
    return idx, wts, labels


@pytest.mark.parametrize("t,e,k,ng", [(1, 32, 4, 4), (7, 100, 8, 8), (300, 128, 8, 32), (5, 16, 2, 1)])
def test_latent_groups_and_compose_rows(dev, t, e, k, ng):
    """group ids / latent rows of the routes against the oracle's rule, and the composed gather rows of a second sort."""
    rng = np.random.default_rng(t + ng)
    idx, _, labels = _latent_routes(rng, t, e, k, ng)
    lib, st = dev.lib, dev.stream.handle
    ib, lb, gb, rb = dev.put(idx), dev.put(labels), dev.alloc(t * ng * 4), dev.alloc(t * k * 4)
    qwhip.check(lib.qwhip_moe_latent_groups(st, ib.ptr, lb.ptr, t, k, e, ng, gb.ptr, rb.ptr))
    dev.stream.sync()
    gids, rows = qo.moe_latent_groups(idx, labels, ng)
    assert np.array_equal(gb.download(np.int32, (t, ng)), gids)
    assert np.array_equal(rb.download(np.int32, (t, k)), rows)
    pairs = t * k
    sp = rng.permutation(pairs).astype(np.int32)
    slot = rng.permutation(t * ng).astype(np.int32)
    slot[gids.ravel() < 0] = -1                                 # rows of absent groups have no slot
    ob, spb, slb = dev.alloc(pairs * 4), dev.put(sp), dev.put(slot)
    qwhip.check(lib.qwhip_moe_compose_rows(st, spb.ptr, pairs, rb.ptr, t * ng, slb.ptr, ob.ptr))
    dev.stream.sync()
    pr = rows.ravel()[sp]
    want = np.where(pr >= 0, np.maximum(slot[np.maximum(pr, 0)], 0), 0)
    assert np.array_equal(ob.download(np.int32, (pairs,)), want)
    assert lib.qwhip_moe_latent_groups(st, ib.ptr, lb.ptr, t, k, e, 33, gb.ptr, rb.ptr) == qwhip.E_BAD_SHAPE


@pytest.mark.parametrize("fmt", ["hq4_g32_m5", "hq8_g32", "hq4_g64"])
@pytest.mark.parametrize("t,ng,lat,hidden", [(1, 4, 64, 256), (3, 8, 96, 512), (8, 4, 40, 1280)])
def test_routed_gemv_keeps_one_row_per_route(dev, fmt, t, ng, lat, hidden):
    """out[t, r] = wts * W[idx[t, r]] . x: every route its own output row, one activation row per token or per route, unit
    weights when none are given, zeros for an absent route."""
    blocks, w16 = H.make_bank(fmt, ng * lat, hidden, 41)
    w = w16.reshape(ng, lat, hidden).astype(np.float64)
    rng = np.random.default_rng(3)
    ids = np.tile(np.arange(ng, dtype=np.int32), (t, 1))
    ids[rng.random((t, ng)) < 0.3] = -1
    wts = (rng.random((t, ng)) + 0.2).astype(np.float32)
    x_tok = rng.standard_normal((t, hidden)).astype(np.float16)
    x_rt = rng.standard_normal((t, ng, hidden)).astype(np.float16)
    lib, st = dev.lib, dev.stream.handle
    bank, ib, wb = dev.put(blocks), dev.put(ids), dev.put(wts)
    v = H.view_of(dev, bank, fmt, ng * lat, hidden)
    for per_token, x, wbuf, odt in ((1, x_tok, None, qwhip.F16), (0, x_rt, wb, qwhip.F32)):
        out, xb = dev.put(np.full((t, ng, lat), 7, np.float32)), dev.put(x)
        qwhip.check(lib.qwhip_moe_routed_gemv(st, C.byref(v), ng, xb.ptr, per_token, ib.ptr, wbuf.ptr if wbuf else None, t, ng,
                                              out.ptr, odt))
        dev.stream.sync()
        if odt == qwhip.F16:
            got = out.download(np.float16, (2 * t * ng * lat,))[: t * ng * lat]
        else:
            got = out.download(np.float32, (t * ng * lat,))
        got = got.reshape(t, ng, lat).astype(np.float64)
        ref = np.zeros((t, ng, lat))
        for r in range(t):
            for g in range(ng):
                if ids[r, g] >= 0:
                    xv = (x[r] if per_token else x[r, g]).astype(np.float64)
                    ref[r, g] = (wts[r, g] if wbuf else 1.0) * (w[ids[r, g]] @ xv)
        assert qo.normalized_error(got, ref) <= TOL
        assert np.all(got[ids < 0] == 0)


@pytest.mark.parametrize("fmt,gu_flags", [("hq4_g32_m5", 0), ("hq4_g32_m5", 2 << 8), ("hq4_g64", 0)])
@pytest.mark.parametrize("t,e,k,ng,lat,inter", [(1, 16, 4, 4, 64, 64), (4, 32, 4, 4, 256, 96), (8, 8, 3, 2, 1792, 64)])
def test_gateup_decode_rows_reads_the_given_rows(dev, fmt, gu_flags, t, e, k, ng, lat, inter):
    """qwhip_moe_gateup_decode_rows == qwhip_moe_gateup_decode over the gathered rows, bit for bit."""
    gu_blocks, _ = H.make_bank(fmt, e * 2 * inter, lat, 43)
    rng = np.random.default_rng(t)
    idx, _, labels = _latent_routes(rng, t, e, k, ng)
    _, rows = qo.moe_latent_groups(idx, labels, ng)
    xl = rng.standard_normal((t * ng, lat)).astype(np.float16)
    lib, st = dev.lib, dev.stream.handle
    bank, ib = dev.put(gu_blocks), dev.put(idx)
    v = H.view_of(dev, bank, fmt, e * 2 * inter, lat)
    a1, a2 = dev.put(np.full((t * k, inter), 3, np.float16)), dev.put(np.full((t * k, inter), 5, np.float16))
    flags = qwhip.X_PREROTATED | gu_flags
    xlb, rwb, gab = dev.put(xl), dev.put(rows), dev.put(xl[np.maximum(rows.ravel(), 0)])
    qwhip.check(lib.qwhip_moe_gateup_decode_rows(st, C.byref(v), e, xlb.ptr, qwhip.F16, flags, ib.ptr, rwb.ptr, t, k, a1.ptr))
    qwhip.check(lib.qwhip_moe_gateup_decode(st, C.byref(v), e, gab.ptr, qwhip.F16, flags, ib.ptr, t * k, 1, a2.ptr))
    dev.stream.sync()
    one, two = a1.download(np.float16, (t * k, inter)), a2.download(np.float16, (t * k, inter))
    assert np.array_equal(one.view(np.uint16), two.view(np.uint16))
    assert np.any(one != 0) and np.all(one[idx.ravel() < 0] == 0)
    if 2 <= t <= 4:   # a shared expert read once: every pair still reads its own latent row
        a3 = dev.put(np.full((t * k, inter), 7, np.float16))
        qwhip.check(lib.qwhip_moe_gateup_decode_rows(st, C.byref(v), e, xlb.ptr, qwhip.F16, flags | qwhip.MOE_REUSE_EXPERTS, ib.ptr, rwb.ptr, t, k,
                                                     a3.ptr))
        dev.stream.sync()
        assert np.array_equal(a3.download(np.uint16, (t * k, inter)), two.view(np.uint16))


@pytest.mark.parametrize("fmt", ["hq4_g32_m5", "hq4_g64", "hq8_g32"])
@pytest.mark.parametrize("t,e,k,ng,lat,inter", [(1, 16, 4, 4, 64, 64), (4, 32, 8, 8, 160, 128), (8, 8, 3, 2, 1792, 64)])
def test_down_decode_groups_sums_the_routes_of_each_group(dev, fmt, t, e, k, ng, lat, inter):
    dn_blocks, dn16 = H.make_bank(fmt, e * lat, inter, 47)
    w = dn16.reshape(e, lat, inter).astype(np.float64)
    rng = np.random.default_rng(ng + t)
    idx, wts, labels = _latent_routes(rng, t, e, k, ng)
    act = rng.standard_normal((t, k, inter)).astype(np.float16)
    lib, st = dev.lib, dev.stream.handle
    bank = dev.put(dn_blocks)
    v = H.view_of(dev, bank, fmt, e * lat, inter)
    out = dev.put(np.full((t, ng, lat), 9, np.float32))
    ab, ib, wb, lb = dev.put(act), dev.put(idx), dev.put(wts), dev.put(labels)
    qwhip.check(lib.qwhip_moe_down_decode_groups(st, C.byref(v), e, ab.ptr, ib.ptr, wb.ptr, lb.ptr, ng, t, k, out.ptr, qwhip.F32))
    dev.stream.sync()
    got = out.download(np.float32, (t, ng, lat)).astype(np.float64)
    ref = np.zeros((t, ng, lat))
    for r in range(t):
        for j in range(k):
            if idx[r, j] >= 0:
                ref[r, labels[idx[r, j]]] += wts[r, j] * (w[idx[r, j]] @ act[r, j].astype(np.float64))
    assert qo.normalized_error(got, ref) <= TOL
    gids, _ = qo.moe_latent_groups(idx, labels, ng)
    assert np.all(got[gids < 0] == 0)


@pytest.mark.parametrize("t,k,ng,width,ddt,odt,perm", [(5, 4, 4, 64, "f32", "f16", True), (300, 8, 8, 1792, "f16", "f32", True),
                                                       (3, 3, 2, 100, "f32", "f32", False)])
def test_combine_groups(dev, t, k, ng, width, ddt, odt, perm):
    rng = np.random.default_rng(width)
    e = 4 * ng
    idx, wts, labels = _latent_routes(rng, t, e, k, ng)
    pairs = t * k
    dn = rng.standard_normal((pairs, width)).astype(np.float32)
    dnh = dn.astype(np.float16) if ddt == "f16" else dn
    inv = rng.permutation(pairs).astype(np.int32) if perm else None
    if perm:
        inv[idx.ravel() < 0] = -1
    lib, st = dev.lib, dev.stream.handle
    out = dev.alloc(t * ng * width * 4)
    db, pb, wb, ib, lb = dev.put(dnh), (dev.put(inv) if perm else None), dev.put(wts), dev.put(idx), dev.put(labels)
    qwhip.check(lib.qwhip_moe_combine_groups(st, db.ptr, qwhip.F16 if ddt == "f16" else qwhip.F32, pb.ptr if perm else None,
                                             wb.ptr, ib.ptr, lb.ptr, e, t, k, ng, width, out.ptr, qwhip.F16 if odt == "f16" else qwhip.F32))
    dev.stream.sync()
    got = out.download(np.float16 if odt == "f16" else np.float32, (t, ng, width)).astype(np.float64)
    ref = np.zeros((t, ng, width))
    for r in range(t):
        for j in range(k):
            if idx[r, j] < 0:
                continue
            slot = int(inv[r * k + j]) if perm else r * k + j
            ref[r, labels[idx[r, j]]] += float(wts[r, j]) * dnh[slot].astype(np.float64)
    assert qo.normalized_error(got, ref) <= (2e-3 if odt == "f16" else 1e-6)
    # a route whose id is not below the expert count has no label: it counts as absent (nothing past the labels is read)
    idx2 = idx.copy()
    idx2[0, 0] = e + 5
    idx2[t - 1, k - 1] = (7 << 16) | e
    ib2 = dev.put(idx2)
    qwhip.check(lib.qwhip_moe_combine_groups(st, db.ptr, qwhip.F16 if ddt == "f16" else qwhip.F32, pb.ptr if perm else None,
                                             wb.ptr, ib2.ptr, lb.ptr, e, t, k, ng, width, out.ptr, qwhip.F16 if odt == "f16" else qwhip.F32))
    dev.stream.sync()
    got2 = out.download(np.float16 if odt == "f16" else np.float32, (t, ng, width)).astype(np.float64)
    for (r, j) in ((0, 0), (t - 1, k - 1)):
        if idx[r, j] >= 0:
            slot = int(inv[r * k + j]) if perm else r * k + j
            ref[r, labels[idx[r, j]]] -= float(wts[r, j]) * dnh[slot].astype(np.float64)
    assert qo.normalized_error(got2, ref) <= (2e-3 if odt == "f16" else 1e-5)


def _group_latent_block(dev, fmts, t, e, k, ng, hidden, lat, inter, x16, idx, wts, labels, banks):
    """The block from the doors: decode (t <= 8) through the routed GEMVs, prefill through two pair sorts and the grouped GEMMs."""
    lib, st = dev.lib, dev.stream.handle
    f_lat, f_exp = fmts
    bd, bu, bgu, bdn = dev.put(banks["d"]), dev.put(banks["u"]), dev.put(banks["gu"]), dev.put(banks["dn"])
    vd = H.view_of(dev, bd, f_lat, ng * lat, hidden)
    vu = H.view_of(dev, bu, f_lat, ng * hidden, lat)
    vgu = H.view_of(dev, bgu, f_exp, e * 2 * inter, lat)
    vdn = H.view_of(dev, bdn, f_exp, e * lat, inter)
    ones = dev.put(np.ones((t, ng), np.float32))
    xb, ib, wb, lb = dev.put(x16), dev.put(idx), dev.put(wts), dev.put(labels)
    gids, rows = dev.alloc(t * ng * 4), dev.alloc(t * k * 4)
    out = dev.alloc(t * hidden * 4)
    pairs = t * k
    qwhip.check(lib.qwhip_moe_latent_groups(st, ib.ptr, lb.ptr, t, k, e, ng, gids.ptr, rows.ptr))
    act = dev.alloc(pairs * inter * 2)
    z16 = dev.alloc(t * ng * lat * 2)
    if t <= 8:
        xl = dev.alloc(t * ng * lat * 2)
        qwhip.check(lib.qwhip_moe_routed_gemv(st, C.byref(vd), ng, xb.ptr, 1, gids.ptr, None, t, ng, xl.ptr, qwhip.F16))
        qwhip.check(lib.qwhip_moe_gateup_decode_rows(st, C.byref(vgu), e, xl.ptr, qwhip.F16, qwhip.X_PREROTATED, ib.ptr, rows.ptr, t, k, act.ptr))
        qwhip.check(lib.qwhip_moe_down_decode_groups(st, C.byref(vdn), e, act.ptr, ib.ptr, wb.ptr, lb.ptr, ng, t, k, z16.ptr, qwhip.F16))
        qwhip.check(lib.qwhip_moe_down_decode(st, C.byref(vu), ng, z16.ptr, gids.ptr, ones.ptr, t, ng, None, None, out.ptr, qwhip.F32))
    else:
        dev.stream.sync()
        g1 = _group(dev, gids.download(np.int32, (t, ng)), ng, ng)
        b1 = g1["bufs"]
        n1 = t * ng
        xl = dev.alloc(n1 * lat * 2)
        qwhip.check(lib.qwhip_moe_grouped_gemm(st, C.byref(vd), ng, xb.ptr, qwhip.F16, 0, b1["stok"].ptr, b1["off"].ptr, b1["te"].ptr, b1["tr"].ptr,
                                               b1["tc"].ptr, g1["max_tiles"], n1, xl.ptr, qwhip.F16, 0))
        g2 = _group(dev, idx, e, k)
        b2 = g2["bufs"]
        rows2 = dev.alloc(pairs * 4)
        qwhip.check(lib.qwhip_moe_compose_rows(st, b2["sp"].ptr, pairs, rows.ptr, n1, b1["inv"].ptr, rows2.ptr))
        qwhip.check(lib.qwhip_moe_grouped_gemm_swiglu(st, C.byref(vgu), e, xl.ptr, qwhip.F16, 0, rows2.ptr, b2["off"].ptr, b2["te"].ptr, b2["tr"].ptr,
                                                      b2["tc"].ptr, g2["max_tiles"], pairs, 1, act.ptr, 0))
        dn = dev.alloc(pairs * lat * 4)
        qwhip.check(lib.qwhip_moe_grouped_gemm(st, C.byref(vdn), e, act.ptr, qwhip.F16, 0, None, b2["off"].ptr, b2["te"].ptr, b2["tr"].ptr,
                                               b2["tc"].ptr, g2["max_tiles"], pairs, dn.ptr, qwhip.F32, 0))
        qwhip.check(lib.qwhip_moe_combine_groups(st, dn.ptr, qwhip.F32, b2["inv"].ptr, wb.ptr, ib.ptr, lb.ptr, e, t, k, ng, lat, z16.ptr, qwhip.F16))
        yu = dev.alloc(n1 * hidden * 4)
        qwhip.check(lib.qwhip_moe_grouped_gemm(st, C.byref(vu), ng, z16.ptr, qwhip.F16, 0, b1["sp"].ptr, b1["off"].ptr, b1["te"].ptr, b1["tr"].ptr,
                                               b1["tc"].ptr, g1["max_tiles"], n1, yu.ptr, qwhip.F32, 0))
        qwhip.check(lib.qwhip_moe_combine(st, yu.ptr, qwhip.F32, b1["inv"].ptr, None, t, ng, hidden, None, None, out.ptr, qwhip.F32))
    dev.stream.sync()
    return out.download(np.float32, (t, hidden))


@pytest.mark.parametrize("fmts", [("hq8_g32", "hq4_g64"), ("hq4_g32_m5", "hq4_g32_m5")])
@pytest.mark.parametrize("t,e,k,ng,hidden,lat,inter", [(1, 32, 4, 4, 64, 64, 64), (4, 32, 4, 4, 256, 128, 64), (8, 64, 8, 8, 512, 192, 128),
                                                       (16, 32, 4, 4, 64, 64, 64), (64, 32, 4, 4, 256, 128, 64), (130, 64, 8, 8, 512, 192, 128)])
def test_group_latent_block_matches_oracle(dev, fmts, t, e, k, ng, hidden, lat, inter):
    """latentD -> routed experts in the latent width -> sum by group -> latentU, decode and prefill forms, against
    moe_group_latent_forward_f64 (the sizes of FNLatentMoETests among them: H = L = I = 64, 32 experts, 4 groups, 4 routes)."""
    f_lat, f_exp = fmts
    banks, w = {}, {}
    banks["d"], w["d"] = H.make_bank(f_lat, ng * lat, hidden, 51)
    banks["u"], w["u"] = H.make_bank(f_lat, ng * hidden, lat, 52)
    banks["gu"], w["gu"] = H.make_bank(f_exp, e * 2 * inter, lat, 53)
    banks["dn"], w["dn"] = H.make_bank(f_exp, e * lat, inter, 54)
    rng = np.random.default_rng(t * 7 + ng)
    x16 = qo.rotate_activation_f16(rng.standard_normal((t, hidden)).astype(np.float32))
    logits = rng.standard_normal((t, e)).astype(np.float32)
    idx, wts = _route(dev, logits, k)
    labels = (np.arange(e) % ng).astype(np.int32)
    if t >= 4:
        labels[idx[1]] = labels[idx[1, 0]]                    # one token with all its routes in one group
    got = _group_latent_block(dev, fmts, t, e, k, ng, hidden, lat, inter, x16, idx, wts, labels, banks)
    ref = qo.moe_group_latent_forward_f64(x16, idx, wts, labels, w["d"].reshape(ng, lat, hidden), w["gu"].reshape(e, 2 * inter, lat),
                                          w["dn"].reshape(e, lat, inter), w["u"].reshape(ng, hidden, lat))
    assert qo.normalized_error(got, ref) <= TOL


@pytest.mark.parametrize("m,k,e,budget,norm", [(2, 8, 32, 10, 1), (4, 16, 64, 20, 1), (3, 4, 8, 6, 0), (4, 8, 128, 9, 1), (2, 4, 16, 2, 1), (4, 16, 512, 40, 1)])
def test_route_budget_matches_oracle(dev, m, k, e, budget, norm):
    """The expert budget of a verify window: ids identical to the oracle, weights to 1e-6; duplicates across rows, ties and a
    route already empty included; no-op and refused shapes."""
    rng = np.random.default_rng(m * 100 + k)
    lg = rng.standard_normal((m, e)).astype(np.float32)
    lg[1] = lg[0] + rng.standard_normal(e).astype(np.float32) * 0.05          # row 1 shares most experts with row 0
    idx, wts = _route(dev, lg, k)
    if m > 2:
        idx[2, k - 1], wts[2, k - 1] = -1, 0.0
        wts[2, 0] = wts[m - 1, 1]                                              # a tie between two candidates
    ib, wb = dev.put(idx), dev.put(wts)
    lib, st = dev.lib, dev.stream.handle
    qwhip.check(lib.qwhip_moe_route_budget(st, ib.ptr, wb.ptr, m, k, budget, norm))
    dev.stream.sync()
    gi, gw = ib.download(np.int32, (m, k)), wb.download(np.float32, (m, k))
    ri, rw = qo.moe_route_budget(idx, wts, budget, bool(norm))
    assert np.array_equal(gi, ri)
    np.testing.assert_allclose(gw, rw, rtol=1e-6, atol=0)
    assert np.array_equal(gi[0], idx[0]) and len({int(v) for v in gi.ravel() if v >= 0}) <= max(k, budget)
    qwhip.check(lib.qwhip_moe_route_budget(st, ib.ptr, wb.ptr, m, k, m * k, norm))   # nothing to prune
    dev.stream.sync()
    assert np.array_equal(ib.download(np.int32, (m, k)), gi)
    assert lib.qwhip_moe_route_budget(st, ib.ptr, wb.ptr, 5, 4, 3, 1) == qwhip.E_BAD_SHAPE
    assert lib.qwhip_moe_route_budget(st, ib.ptr, wb.ptr, 1, 4, 3, 1) == qwhip.E_BAD_SHAPE
