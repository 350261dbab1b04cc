"""The oracle's C restatement (oracle/qworacle_c.c) against the numpy oracle, which the golden fixtures pin."""
import ctypes as C
import pathlib

import numpy as np
import pytest

from oracle import build_oracle
from oracle import qworacle as qo


@pytest.fixture(scope="module")
def clib():
    if not build_oracle.LIB.exists():
        build_oracle.build()
    return C.CDLL(str(build_oracle.LIB))


def _p(a):
    return a.ctypes.data_as(C.c_void_p)


def _wide_range_weights(n, k, seed):
    rng = np.random.default_rng(seed)
    w = rng.standard_normal((n, k)).astype(np.float32)
    w *= np.float32(10.0) ** rng.uniform(-9, 3, size=(n, 1)).astype(np.float32)   # exercises f16 subnormal scales and the clamp
    w[1, :32] = 0.0
    w[2, 5] = 1e4
    return w


@pytest.mark.parametrize("rotate", [1, 0])
def test_c_quantizer_bytes_equal_numpy(clib, rotate):
    w = _wide_range_weights(64, 512, 3)
    out = np.empty((64, 16, 20), dtype=np.uint8)
    clib.qwo_quant_hq4(_p(w), C.c_int64(64), C.c_int64(512), rotate, _p(out))
    assert np.array_equal(out, qo.quant_hq4_blocks(w, rotate=bool(rotate)))


def test_c_dequant_equals_numpy(clib):
    w = _wide_range_weights(32, 256, 4)
    blocks = qo.quant_hq4_blocks(w)
    for f16_round in (0, 1):
        out = np.empty((32, 256), dtype=np.float32)
        clib.qwo_dequant_hq4_rot(_p(blocks), C.c_int64(32), C.c_int64(256), f16_round, _p(out))
        assert np.array_equal(out.view(np.uint32), qo.dequant_hq4_rot(blocks, bool(f16_round)).view(np.uint32))
    for bits, group in [(4, 32), (4, 64), (8, 32), (6, 128), (3, 32), (2, 256)]:
        blk, _ = qo.quant_hq_blocks(w, bits=bits, group=group, rotate=True)
        for f16_round in (0, 1):
            out = np.empty((32, 256), dtype=np.float32)
            clib.qwo_dequant_blocks_rot(_p(blk), C.c_int64(32), C.c_int64(256), bits, group, f16_round, _p(out))
            want = qo.dequant_hq_blocks_rot(blk, bits, group, False, bool(f16_round))
            assert np.array_equal(out.view(np.uint32), want.view(np.uint32)), (bits, group, f16_round)


def test_c_fwht_equals_numpy(clib):
    x = np.random.default_rng(0).standard_normal((8, 32)).astype(np.float32)
    y = x.copy()
    for r in range(8):
        clib.qwo_fwht32(_p(y[r]))
    assert np.array_equal(y.view(np.uint32), qo.fwht32_ortho(x).view(np.uint32))


def test_c_oracle_gemv_matches_numpy_form(clib):
    n, k = 256, 1024
    w = (np.random.default_rng(1).standard_normal((n, k)) * 0.02).astype(np.float32)
    blocks = qo.quant_hq4_blocks(w)
    x16 = qo.rotate_activation_f16(np.random.default_rng(2).standard_normal(k).astype(np.float32))
    scratch, xf, y = np.empty((n, k), np.float32), np.empty(k, np.float32), np.empty(n, np.float32)
    clib.qwo_oracle_gemv_hq4(_p(blocks), _p(x16.view(np.uint16)), C.c_int64(n), C.c_int64(k), _p(scratch), _p(xf), _p(y))
    want = qo.cpu_oracle_gemv(blocks, x16)
    np.testing.assert_allclose(y, want, rtol=2e-4, atol=2e-5)
    ref = qo.matmul_ref_f64(x16[None, :], qo.weights_f16_exact(blocks, 4, 32, True))[0]
    assert qo.normalized_error(y, ref) < 1e-5


@pytest.mark.parametrize("bits,group,rotate", [(4, 32, False), (8, 32, True), (4, 64, True)])
def test_c_oracle_gemv_blocks_matches_f64(clib, bits, group, rotate):
    n, k = 128, 512
    w = (np.random.default_rng(3).standard_normal((n, k)) * 0.02).astype(np.float32)
    blocks, _ = qo.quant_hq_blocks(w, bits=bits, group=group, rotate=rotate)
    x16 = np.random.default_rng(4).standard_normal(k).astype(np.float16)
    scratch, xf, y = np.empty((n, k), np.float32), np.empty(k, np.float32), np.empty(n, np.float32)
    clib.qwo_oracle_gemv_blocks(_p(blocks), _p(x16.view(np.uint16)), C.c_int64(n), C.c_int64(k), bits, group, _p(scratch), _p(xf), _p(y))
    ref = qo.matmul_ref_f64(x16[None, :], qo.weights_f16_exact(blocks, bits, group, False))[0]
    assert qo.normalized_error(y, ref) < 1e-5
    assert clib.qwo_threads() >= 1
