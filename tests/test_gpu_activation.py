"""The device's gated FFN activation (qwhip_device_set_gated_activation): SwiGLU, clamped SwiGLU and the bounded tanh form on
every door that carries the epilogue, against the oracle's gated_act; the fused doors stay bit-identical to their two-step
forms under every activation."""
import contextlib
import ctypes as C

import numpy as np
import pytest

from oracle import qworacle as qo
from qwegn_amd import qwhip
from tests import helpers as H

pytestmark = pytest.mark.gpu
TOL = 2e-3
ACTS = [(1, 0.5, 0.0), (2, 1.0, 0.75), (2, 4.0, 25.0), (2, 0.8, 0.0)]     # (kind, p0, p1); sized so that the bounds bite


@pytest.fixture(scope="module")
def dev():
    return qwhip.Device(0)


@contextlib.contextmanager
def activation(dev, kind, p0, p1):
    qwhip.check(dev.lib.qwhip_device_set_gated_activation(dev.handle, kind, p0, p1))
    try:
        yield
    finally:
        dev.stream.sync()
        qwhip.check(dev.lib.qwhip_device_set_gated_activation(dev.handle, 0, 0.0, 0.0))


def _act_ref(g, u, act, rotate, f16_out=True):
    v = qo.gated_act(g, u, *act).astype(np.float32)
    if rotate:
        v = qo.fwht32_ortho(v)
    return v.astype(np.float16).astype(np.float32) if f16_out else v


@pytest.mark.parametrize("act", ACTS)
def test_elementwise_doors(dev, act):
    """qwhip_swiglu_fwht (f16 and f32 inputs, rotated, plain and the ragged scalar form) and qwhip_silu_mul_f32."""
    rng = np.random.default_rng(3)
    rows, inter = 5, 96
    gu = (rng.standard_normal((rows, 2 * inter)) * 2).astype(np.float32)
    lib, st = dev.lib, dev.stream.handle
    with activation(dev, *act):
        for dt, code in ((np.float16, qwhip.F16), (np.float32, qwhip.F32)):
            src = gu.astype(dt)
            sb = dev.put(src)
            for rot in (1, 0):
                out = dev.alloc(rows * inter * 2)
                qwhip.check(lib.qwhip_swiglu_fwht(st, sb.ptr, code, out.ptr, rows, inter, rot))
                dev.stream.sync()
                got = out.download(np.float16, (rows, inter)).astype(np.float32)
                s32 = src.astype(np.float32)
                assert qo.normalized_error(got, _act_ref(s32[:, :inter], s32[:, inter:], act, bool(rot))) <= 1e-3
        rag = (rng.standard_normal((3, 2 * 40)) * 2).astype(np.float32)
        rb, ro = dev.put(rag), dev.alloc(3 * 40 * 2)
        qwhip.check(lib.qwhip_swiglu_fwht(st, rb.ptr, qwhip.F32, ro.ptr, 3, 40, 0))
        gb, ab = dev.put(gu), dev.alloc(rows * inter * 4)
        qwhip.check(lib.qwhip_silu_mul_f32(st, gb.ptr, ab.ptr, rows, inter))
        dev.stream.sync()
        assert qo.normalized_error(ro.download(np.float16, (3, 40)).astype(np.float32), _act_ref(rag[:, :40], rag[:, 40:], act, False)) <= 1e-3
        assert qo.normalized_error(ab.download(np.float32, (rows, inter)), _act_ref(gu[:, :inter], gu[:, inter:], act, True, f16_out=False)) <= 2e-6
    # back on SwiGLU afterwards
    gb, out = dev.put(gu.astype(np.float16)), dev.alloc(rows * inter * 2)
    qwhip.check(lib.qwhip_swiglu_fwht(st, gb.ptr, qwhip.F16, out.ptr, rows, inter, 1))
    dev.stream.sync()
    s32 = gu.astype(np.float16).astype(np.float32)
    assert qo.normalized_error(out.download(np.float16, (rows, inter)).astype(np.float32), _act_ref(s32[:, :inter], s32[:, inter:], (0, 0, 0), True)) <= 1e-3


@pytest.mark.parametrize("act", ACTS)
@pytest.mark.parametrize("fmt,m,inter,k", [("hq4_g32_m5", 256, 352, 256), ("hq4_g64", 64, 160, 128), ("hq8_g32", 128, 96, 256)])
def test_dense_gate_up_gemm(dev, act, fmt, m, inter, k):
    """qwhip_gemm_swiglu == qwhip_gemm (f16 out) + qwhip_swiglu_fwht bit for bit, and both meet the oracle."""
    n = 2 * inter
    blocks, w16 = H.make_bank(fmt, n, k, seed=5)
    x16 = (H.make_x(m, k, 12) * 2).astype(np.float16)
    bank, xb = dev.put(blocks), dev.put(x16)
    gu, act2, act1 = dev.alloc(m * n * 2), dev.put(np.zeros((m, inter), np.float16)), dev.put(np.zeros((m, inter), np.float16))
    ws = dev.alloc(max(m * k * 2, m * n * 2) + 256)
    view = H.view_of(dev, bank, fmt, n, k)
    lib, st = dev.lib, dev.stream.handle
    with activation(dev, *act):
        qwhip.check(lib.qwhip_gemm(st, C.byref(view), xb.ptr, qwhip.F16, m, 0, gu.ptr, qwhip.F16, 0, qwhip.X_PREROTATED, ws.ptr, ws.nbytes))
        qwhip.check(lib.qwhip_swiglu_fwht(st, gu.ptr, qwhip.F16, act2.ptr, m, inter, 1))
        qwhip.check(lib.qwhip_gemm_swiglu(st, C.byref(view), xb.ptr, qwhip.F16, m, 0, 1, act1.ptr, 0, qwhip.X_PREROTATED, ws.ptr, ws.nbytes))
        dev.stream.sync()
    one, two = act1.download(np.float16, (m, inter)), act2.download(np.float16, (m, inter))
    assert np.array_equal(one.view(np.uint16), two.view(np.uint16))
    g = qo.matmul_ref_f64(x16, w16).astype(np.float16).astype(np.float32)
    assert qo.normalized_error(one.astype(np.float32), _act_ref(g[:, :inter], g[:, inter:], act, True)) <= TOL


@pytest.mark.parametrize("act", ACTS)
@pytest.mark.parametrize("fmt,gu_flags", [("hq4_g32_m5", 0), ("hq4_g32_m5", 2 << 8), ("hq4_g64", 0)])
def test_decode_gate_up_doors(dev, act, fmt, gu_flags):
    """qwhip_gemv_silu_pair and qwhip_moe_gateup_decode / qwhip_moe_route_gateup_decode (column-stationary and general kernels)."""
    inter, k, e, top_k, t = 96, 512, 8, 2, 3
    blocks, w16 = H.make_bank(fmt, e * 2 * inter, k, seed=12)
    w = w16.reshape(e, 2 * inter, k)
    rng = np.random.default_rng(5)
    x16 = (rng.standard_normal((t, k)) * 2).astype(np.float16)
    logits = rng.standard_normal((t, e)).astype(np.float32)
    bank, xb, lb = dev.put(blocks), dev.put(x16), dev.put(logits)
    lib, st = dev.lib, dev.stream.handle
    vall = H.view_of(dev, bank, fmt, e * 2 * inter, k)
    vone = H.view_of(dev, bank, fmt, 2 * inter, k)
    a_pair, a_dec, a_fused = dev.alloc(t * inter * 2), dev.alloc(t * top_k * inter * 2), dev.alloc(t * top_k * inter * 2)
    ib, wb, ib2, wb2 = dev.alloc(t * top_k * 4), dev.alloc(t * top_k * 4), dev.alloc(t * top_k * 4), dev.alloc(t * top_k * 4)
    fl = qwhip.X_PREROTATED | gu_flags
    with activation(dev, *act):
        qwhip.check(lib.qwhip_gemv_silu_pair(st, C.byref(vone), xb.ptr, qwhip.F16, t, fl, 1, a_pair.ptr))
        qwhip.check(lib.qwhip_moe_route(st, lb.ptr, t, e, top_k, 1, 1.0, ib.ptr, wb.ptr))
        qwhip.check(lib.qwhip_moe_gateup_decode(st, C.byref(vall), e, xb.ptr, qwhip.F16, fl, ib.ptr, t, top_k, a_dec.ptr))
        qwhip.check(lib.qwhip_moe_route_gateup_decode(st, C.byref(vall), e, xb.ptr, qwhip.F16, qwhip.X_PREROTATED, lb.ptr, t, top_k, 1, 1.0,
                                                      ib2.ptr, wb2.ptr, a_fused.ptr))
        dev.stream.sync()
    idx = ib.download(np.int32, (t, top_k))
    gu0 = qo.matmul_ref_f64(x16, w[0])
    assert qo.normalized_error(a_pair.download(np.float16, (t, inter)).astype(np.float32),
                               _act_ref(gu0[:, :inter].astype(np.float32), gu0[:, inter:].astype(np.float32), act, True)) <= TOL
    want = np.zeros((t, top_k, inter), np.float32)
    for r in range(t):
        for j in range(top_k):
            gu = (w[idx[r, j]].astype(np.float64) @ x16[r].astype(np.float64)).astype(np.float32)
            want[r, j] = _act_ref(gu[None, :inter], gu[None, inter:], act, True)[0]
    assert qo.normalized_error(a_dec.download(np.float16, (t, top_k, inter)).astype(np.float32), want) <= TOL
    assert qo.normalized_error(a_fused.download(np.float16, (t, top_k, inter)).astype(np.float32), want) <= TOL


@pytest.mark.parametrize("act", ACTS[:2])
@pytest.mark.parametrize("fmt", ["hq4_g32_m5", "hq4_g64"])
def test_grouped_gate_up_gemm(dev, act, fmt):
    """qwhip_moe_grouped_gemm_swiglu == grouped GEMM (f16 out) + qwhip_swiglu_fwht bit for bit under the activation."""
    t, e, k_routes, hidden, inter = 70, 8, 2, 256, 128
    blocks, _ = H.make_bank(fmt, e * 2 * inter, hidden, 13)
    rng = np.random.default_rng(9)
    x16 = (rng.standard_normal((t, hidden)) * 2).astype(np.float16)
    ids = np.stack([rng.permutation(e)[:k_routes] for _ in range(t)]).astype(np.int32)
    pairs = t * k_routes
    lib, st = dev.lib, dev.stream.handle
    mt = max(1, lib.qwhip_moe_max_tiles(e, pairs))
    idb, off, sp, stok, inv = dev.put(ids), dev.alloc((e + 1) * 4), dev.alloc(pairs * 4), dev.alloc(pairs * 4), dev.alloc(pairs * 4)
    te, tr, tc = dev.alloc(mt * 4), dev.alloc(mt * 4), dev.alloc(16)
    qwhip.check(lib.qwhip_moe_group_pairs(st, idb.ptr, e, pairs, k_routes, off.ptr, sp.ptr, stok.ptr, inv.ptr, te.ptr, tr.ptr, tc.ptr, 1))
    bank, xb = dev.put(blocks), dev.put(x16)
    v = H.view_of(dev, bank, fmt, e * 2 * inter, hidden)
    gu = dev.alloc(pairs * 2 * inter * 2)
    a2, a1 = dev.put(np.zeros((pairs, inter), np.float16)), dev.put(np.zeros((pairs, inter), np.float16))
    with activation(dev, *act):
        qwhip.check(lib.qwhip_moe_grouped_gemm(st, C.byref(v), e, xb.ptr, qwhip.F16, 0, stok.ptr, off.ptr, te.ptr, tr.ptr, tc.ptr, mt, pairs,
                                               gu.ptr, qwhip.F16, 0))
        qwhip.check(lib.qwhip_swiglu_fwht(st, gu.ptr, qwhip.F16, a2.ptr, pairs, inter, 1))
        qwhip.check(lib.qwhip_moe_grouped_gemm_swiglu(st, C.byref(v), e, xb.ptr, qwhip.F16, 0, stok.ptr, off.ptr, te.ptr, tr.ptr, tc.ptr, mt,
                                                      pairs, 1, a1.ptr, 0))
        dev.stream.sync()
    one, two = a1.download(np.float16, (pairs, inter)), a2.download(np.float16, (pairs, inter))
    assert np.array_equal(one.view(np.uint16), two.view(np.uint16)) and np.any(one != 0)


def test_setter_refusals(dev):
    lib = dev.lib
    assert lib.qwhip_device_set_gated_activation(dev.handle, 3, 1.0, 1.0) == qwhip.E_BAD_SHAPE
    assert lib.qwhip_device_set_gated_activation(dev.handle, 1, 0.0, 0.0) == qwhip.E_BAD_SHAPE
    assert lib.qwhip_device_set_gated_activation(dev.handle, 2, -1.0, 1.0) == qwhip.E_BAD_SHAPE
    assert lib.qwhip_device_set_gated_activation(None, 0, 0.0, 0.0) == qwhip.E_NULL
    qwhip.check(lib.qwhip_device_set_gated_activation(dev.handle, 0, 0.0, 0.0))
