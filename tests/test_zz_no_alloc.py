"""qwhip_gemm_noalloc (the prefill GEMM for callers that cannot allocate or pass a workspace) against qwhip_gemm with a
caller workspace: same bits, on two calls in a row, the second with a smaller input, so that what the first call left in
the library's static scratch array cannot leak into the second.  Both calls also stay inside the judged bar against the
fp64 oracle."""
import ctypes as C

import numpy as np
import pytest

from oracle import qworacle as qo
from qwegn_amd import qwhip
from tests import helpers as H

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def dev():
    return qwhip.Device(0)


def _both(dev, view, x_host, xcode, m, n, k, flags, with_ws=True):
    """(noalloc output, qwhip_gemm output) as raw bf16 bits; qwhip_gemm with a workspace of the activation copy, or with none."""
    xb = dev.put(x_host)
    y_a, y_b, ws = dev.alloc(m * n * 2), dev.alloc(m * n * 2), dev.alloc(m * k * 2)
    st = dev.stream.handle
    qwhip.check(dev.lib.qwhip_fill_u32(st, y_a.ptr, 0xFFFFFFFF, m * n // 2))
    qwhip.check(dev.lib.qwhip_fill_u32(st, y_b.ptr, 0xFFFFFFFF, m * n // 2))
    qwhip.check(dev.lib.qwhip_gemm_noalloc(st, C.byref(view), xb.ptr, xcode, m, 0, y_a.ptr, qwhip.BF16, 0, flags))
    qwhip.check(dev.lib.qwhip_gemm(st, C.byref(view), xb.ptr, xcode, m, 0, y_b.ptr, qwhip.BF16, 0, flags, ws.ptr if with_ws else None,
                                   ws.nbytes if with_ws else 0))
    dev.stream.sync()
    a, b = y_a.download(np.uint16, (m, n)), y_b.download(np.uint16, (m, n))
    for buf in (xb, y_a, y_b, ws):
        buf.free()
    return a, b


@pytest.mark.parametrize("fmt,xdtype,prerot", [("hq4_g32_m5", "bf16", False), ("hq4_g32_m5", "bf16", True), ("hq8_g32", "f16", False)])
def test_gemm_noalloc_matches_gemm_with_workspace_twice(dev, fmt, xdtype, prerot):
    n, k = 640, 1024
    blocks, w16 = H.make_bank(fmt, n, k, seed=21)
    bank = dev.put(blocks)
    view = H.view_of(dev, bank, fmt, n, k)
    for m, seed in ((320, 31), (64, 32)):          # the second call is smaller than the first
        x32 = H.make_x(m, k, seed)
        if xdtype == "bf16":
            x_val, x_host, xcode = qo.round_bf16(x32), qo.f32_to_bf16_bits(x32), qwhip.BF16
        else:
            x_host, xcode = x32.astype(np.float16), qwhip.F16
            x_val = x_host.astype(np.float32)
        x_basis = (x_val if prerot else qo.fwht32_ortho(x_val)).astype(np.float16)
        # rows to rotate go through the static scratch (= qwhip_gemm with a workspace of that size); rows in the basis are
        # read in place (= qwhip_gemm without a workspace)
        got, want = _both(dev, view, x_host, xcode, m, n, k, qwhip.X_PREROTATED if prerot else 0, with_ws=not prerot)
        assert np.array_equal(got, want), f"m={m}: static-scratch GEMM differs from the workspace GEMM"
        assert qo.normalized_error(qo.bf16_bits_to_f32(got), qo.matmul_ref_f64(x_basis, w16)) <= 2e-3
    bank.free()


@pytest.mark.parametrize("xdtype", ["bf16", "f16"])
def test_gemm_noalloc_reads_rows_in_the_basis_in_place_at_any_size(dev, xdtype):
    """Rows already in the container's basis need no copy: a call whose activations exceed the static scratch (8.65 MB of rows)
    is taken, and gives the bits of qwhip_gemm reading the rows in place (no workspace); against qwhip_gemm with a workspace -
    which may pick another tile shape, i.e. another order inside a K-step - it agrees to rounding."""
    n, k, m = 320, 2048, 2112
    assert m * k * 2 > dev.lib.qwhip_gemm_noalloc_max_bytes()
    blocks, w16 = H.make_bank("hq4_g32_m5", n, k, seed=5)
    bank = dev.put(blocks)
    view = H.view_of(dev, bank, "hq4_g32_m5", n, k)
    x32 = H.make_x(m, k, 41)
    if xdtype == "bf16":
        x_val, x_host, xcode = qo.round_bf16(x32), qo.f32_to_bf16_bits(x32), qwhip.BF16
    else:
        x_host, xcode = x32.astype(np.float16), qwhip.F16
        x_val = x_host.astype(np.float32)
    got, want = _both(dev, view, x_host, xcode, m, n, k, qwhip.X_PREROTATED, with_ws=False)
    assert np.array_equal(got, want)
    _, want_ws = _both(dev, view, x_host, xcode, m, n, k, qwhip.X_PREROTATED, with_ws=True)
    assert qo.normalized_error(qo.bf16_bits_to_f32(got), qo.bf16_bits_to_f32(want_ws).astype(np.float64)) <= 2e-3
    assert qo.normalized_error(qo.bf16_bits_to_f32(got), qo.matmul_ref_f64(x_val.astype(np.float16), w16)) <= 2e-3
    bank.free()


def test_gemm_noalloc_rejects_sizes_beyond_its_scratch(dev):
    cap = dev.lib.qwhip_gemm_noalloc_max_bytes()
    assert cap == 8 << 20
    n, k = 64, 4096
    blocks, _ = H.make_bank("hq4_g32_m5", n, k, seed=1)
    bank = dev.put(blocks)
    view = H.view_of(dev, bank, "hq4_g32_m5", n, k)
    m = cap // (2 * k) + 64                        # one 64-row block past the limit
    xb, yb = dev.put(np.zeros((m, k), np.float16)), dev.alloc(m * n * 2)
    st = dev.stream.handle
    assert dev.lib.qwhip_gemm_noalloc(st, C.byref(view), xb.ptr, qwhip.F16, m, 0, yb.ptr, qwhip.F16, 0, 0) == qwhip.E_BAD_SHAPE
    assert b"exceeds the static scratch" in dev.lib.qwhip_last_error()
    m_ok = cap // (2 * k)                          # exactly the limit is taken
    assert dev.lib.qwhip_gemm_noalloc(st, C.byref(view), xb.ptr, qwhip.F16, m_ok, 0, yb.ptr, qwhip.F16, 0, 0) == qwhip.OK
    dev.stream.sync()
    for buf in (bank, xb, yb):
        buf.free()
