"""Pins the oracle on what the mathematics fixes, independent of the golden vectors: closed forms,
invariants, brute force on tiny inputs and scalar restatements of the reference's host readers.  Each
check is chosen so a plausible mistake (wrong nibble order, wrong rounding mode, a dropped term, a
transposed butterfly) fails it."""
from fractions import Fraction

import numpy as np
import pytest

from oracle import qworacle as qo


def test_fwht_is_the_dense_hadamard_and_self_inverse():
    # Sylvester H32 built by Kronecker products; natural (Hadamard) order is what the (i, i+h) butterflies give
    h = np.array([[1.0]])
    for _ in range(5):
        h = np.block([[h, h], [h, -h]])
    x = np.random.default_rng(0).standard_normal((5, 64)).astype(np.float32)
    want = (x.reshape(-1, 32).astype(np.float64) @ h.T / np.sqrt(32.0)).reshape(x.shape)
    got = qo.fwht32_ortho(x)
    assert np.max(np.abs(got - want)) < 1e-5
    assert np.max(np.abs(qo.fwht32_ortho(got) - x)) < 1e-5
    # unit vectors: column i of H/sqrt(32), exactly +-f32(1/sqrt(32))
    e = np.eye(32, dtype=np.float32)
    col = qo.fwht32_ortho(e)
    assert np.all(np.abs(col) == qo.INV_SQRT32)
    assert np.array_equal(np.sign(col), np.sign(h))
    assert qo.INV_SQRT32.view(np.uint32) == 0x3E3504F3


def _rn_f16(frac: Fraction) -> np.float16:
    """Exact round-to-nearest-even of a rational to binary16 (brute force over the two neighbours)."""
    f = float(frac)                       # doubles hold these values exactly (checked by the caller)
    assert Fraction(f) == frac
    lo = np.float16(f)
    # np.float16(double) is correctly rounded; confirm against the neighbours with exact arithmetic
    cands = [lo, np.nextafter(lo, np.float16(np.inf)), np.nextafter(lo, np.float16(-np.inf))]
    cands = [c for c in cands if np.isfinite(c)]
    best = min(cands, key=lambda c: (abs(Fraction(float(c)) - frac), int(c.view(np.uint16)) & 1))
    return best


def test_f16_weight_closed_form_brute_force():
    """RN_f16((1024+q)*s + b) and RN_f16(code*s + b) against exact rational arithmetic."""
    rng = np.random.default_rng(1)
    scales = np.concatenate([rng.uniform(1e-4, 0.2, 40), [6e-8, 3.0e-5, 63.46875]]).astype(np.float16)
    for s16 in scales:
        b16 = np.float16(np.float32(-1032.0) * np.float32(s16))
        blocks = np.zeros((1, 1, 20), dtype=np.uint8)
        blocks[0, 0, 0:2] = np.array([s16]).view(np.uint8)
        blocks[0, 0, 2:4] = np.array([b16]).view(np.uint8)
        q = np.arange(32) % 16
        blocks[0, 0, 4:] = qo.hq4_interleave(q[None, :]).view(np.uint8).reshape(16)
        w16 = qo.weights_f16_exact(blocks, 4, 32, True)[0]
        for i in range(16):
            exact = (1024 + int(q[i])) * Fraction(float(s16)) + Fraction(float(b16))
            assert w16[i] == _rn_f16(exact), (s16, i)
        # block family: code*s + b with an unrelated bias
        bias = np.float16(-7.5 * float(s16))
        blk = np.zeros((1, 1, 36), dtype=np.uint8)
        blk[0, 0, 0:2] = np.array([s16]).view(np.uint8)
        blk[0, 0, 2:4] = np.array([bias]).view(np.uint8)
        codes = (np.arange(32) * 37 + 11) % 256
        blk[0, 0, 4:] = codes
        w8 = qo.weights_f16_exact(blk, 8, 32, False)[0]
        for i in range(32):
            exact = int(codes[i]) * Fraction(float(s16)) + Fraction(float(bias))
            assert w8[i] == _rn_f16(exact), (s16, i)


def test_affine_weights_are_the_exact_values_behind_the_f16_weights():
    """weights_affine_f64 is the un-rounded (q+1024)*s + b / code*s + b: exact rational arithmetic on a few blocks,
    and rounding it to f16 reproduces weights_f16_exact on seeded banks of every container family."""
    s16, b16 = np.float16(0.0123), np.float16(-0.071)
    blk = np.zeros((1, 1, 36), dtype=np.uint8)
    blk[0, 0, 0:2] = np.array([s16]).view(np.uint8)
    blk[0, 0, 2:4] = np.array([b16]).view(np.uint8)
    codes = (np.arange(32) * 29 + 3) % 256
    blk[0, 0, 4:] = codes
    w = qo.weights_affine_f64(blk, 8, 32, False)[0]
    for i in range(32):
        assert Fraction(float(w[i])) == int(codes[i]) * Fraction(float(s16)) + Fraction(float(b16))
    rng = np.random.default_rng(3)
    wsrc = (rng.standard_normal((8, 256)) * 0.02).astype(np.float32)
    for bits, group, is_m5 in [(4, 32, True), (4, 32, False), (4, 64, False), (8, 32, False), (8, 128, False)]:
        blocks, _ = qo.quant_hq_blocks(wsrc, bits=bits, group=group, is_m5=is_m5, rotate=True)
        exact = qo.weights_affine_f64(blocks, bits, group, is_m5)
        assert np.array_equal(exact.astype(np.float16), qo.weights_f16_exact(blocks, bits, group, is_m5))


def test_hq4_nibble_order_matches_the_scalar_reader():
    """Element 8w+j sits at bit 4*(j>>1) + 16*(j&1) of word w (QWAQProducer.swift:85-87; reader shifts
    0,16,4,20,8,24,12,28 in QWQuant+DequantMath.swift:82-89)."""
    q = np.arange(32) % 16
    words = qo.hq4_interleave(q[None, :])[0]
    for w in range(4):
        for j in range(8):
            shift = 4 * (j >> 1) + 16 * (j & 1)
            assert (int(words[w]) >> shift) & 0xF == q[8 * w + j]
    blocks = np.zeros((1, 1, 20), dtype=np.uint8)
    blocks[0, 0, 4:] = words.view(np.uint8)
    assert np.array_equal(qo.hq4_codes(blocks)[0, 0], q)


def test_hq4_quantizer_invariants():
    rng = np.random.default_rng(2)
    w = (rng.standard_normal((16, 256)) * 0.02).astype(np.float32)
    w[0, :32] = 0.0                                       # scale 0 -> code 8 everywhere, bias -0
    blocks = qo.quant_hq4_blocks(w, rotate=False)
    s = np.ascontiguousarray(blocks[..., 0:2]).view(np.float16)[..., 0]
    b = np.ascontiguousarray(blocks[..., 2:4]).view(np.float16)[..., 0]
    assert np.array_equal(b, (np.float32(-1032.0) * s.astype(np.float32)).astype(np.float16))     # bias law
    codes = qo.hq4_codes(blocks)
    assert np.all(codes[0, 0] == 8) and s[0, 0] == 0
    v = w.reshape(16, 8, 32)
    deq = qo.dequant_hq4_rot(blocks).reshape(16, 8, 32)
    sf = s.astype(np.float32)[..., None]
    inner = (codes > 0) & (codes < 15)
    assert np.all(np.abs(deq - v)[inner] <= (0.5 * sf * 1.01 + 1e-9).repeat(32, -1)[inner])          # brackets v within scale/2
    for g in range(8):                                                                           # code monotone in v
        order = np.argsort(v[3, g], kind="stable")
        assert np.all(np.diff(codes[3, g][order].astype(int)) >= 0)
    amax = np.abs(v).max(-1)
    assert np.array_equal(s, np.minimum(amax / np.float32(7.5), np.float32(63.46875)).astype(np.float16))
    # the scale clamp
    big = np.full((1, 32), 1000.0, dtype=np.float32)
    sb = np.ascontiguousarray(qo.quant_hq4_blocks(big, rotate=False)[..., 0:2]).view(np.float16)
    assert float(sb[0, 0, 0]) == 63.46875


def _read_bits_scalar(payload: bytes, bits: int, index: int) -> int:
    """Scalar restatement of QWAQBlock.readBits (QWAQBlock.swift:115-126)."""
    bit = index * bits
    byte, off = bit >> 3, bit & 7
    v = payload[byte] >> off
    taken = 8 - off
    if taken < bits:
        v |= payload[byte + 1] << taken
    return v & ((1 << bits) - 1)


@pytest.mark.parametrize("bits", [2, 3, 4, 6, 8])
@pytest.mark.parametrize("group", [32, 64, 128, 256])
def test_bitstream_layout_and_size_law(bits, group):
    assert qo.hq_block_bytes(bits, group) == 4 + group * bits // 8
    rng = np.random.default_rng(bits * 1000 + group)
    q = rng.integers(0, 1 << bits, size=(3, group))
    payload = qo.pack_bitstream(q, bits)
    assert payload.shape == (3, group * bits // 8)
    for r in range(3):
        raw = payload[r].tobytes()
        assert [_read_bits_scalar(raw, bits, i) for i in range(group)] == q[r].tolist()
    assert np.array_equal(qo.unpack_bitstream(payload, bits, group), q)


def test_block_quantizer_invariants():
    rng = np.random.default_rng(3)
    w = (rng.standard_normal((8, 256)) * 0.02).astype(np.float32)
    w[1, 64:128] = 0.5                                          # constant group: scale 0, codes 0, bias = value
    for bits, group in [(4, 32), (4, 64), (8, 32)]:
        blocks, eff = qo.quant_hq_blocks(w, bits=bits, group=group, rotate=False)
        assert eff == group and blocks.shape == (8, 256 // group, 4 + group * bits // 8)
        s, b = qo.hq_block_header(blocks)
        v = w.reshape(8, 256 // group, group)
        assert np.array_equal(b, v.min(-1).astype(np.float16).astype(np.float32))
        qmax = (1 << bits) - 1
        assert np.array_equal(s, ((v.max(-1) - v.min(-1)) / np.float32(qmax)).astype(np.float16).astype(np.float32))
        codes = qo.hq_block_codes(blocks, bits, group)
        const = (v.max(-1) == v.min(-1))
        assert np.all(codes[const] == 0)
        deq = qo.dequant_hq_blocks_rot(blocks, bits, group).reshape(v.shape)
        inner = (codes > 0) & (codes < qmax)
        tol = 0.5 * s[..., None] * 1.01 + 1e-9
        assert np.all(np.abs(deq - v)[inner] <= np.broadcast_to(tol, v.shape)[inner])
    # round-half-even, not half-up: (w - b)/s = 0.5 and 1.5 and 2.5 -> 0, 2, 2
    g = np.zeros((1, 32), dtype=np.float32)
    g[0, :4] = [0.0, 0.5, 1.5, 2.5]
    g[0, 31] = 15.0                                            # min 0, max 15 -> scale 1, bias 0 (4-bit)
    blk, _ = qo.quant_hq_blocks(g, bits=4, group=32, rotate=False)
    assert qo.hq_block_codes(blk, 4, 32)[0, 0, :4].tolist() == [0, 0, 2, 2]
    with pytest.raises(ValueError):
        qo.resolve_group_size(48, 32)
    assert qo.resolve_group_size(96, 64) == 32                  # gcd clamp (hq_blocks.py:106-114)


def test_rotation_preserves_products():
    """(x H)(W H)^T = x W^T: the whole point of rotating both sides."""
    rng = np.random.default_rng(4)
    w = rng.standard_normal((6, 128)).astype(np.float32)
    x = rng.standard_normal((2, 128)).astype(np.float32)
    a = x.astype(np.float64) @ w.astype(np.float64).T
    b = qo.fwht32_ortho(x).astype(np.float64) @ qo.fwht32_ortho(w).astype(np.float64).T
    assert np.max(np.abs(a - b)) < 1e-4


def test_route_is_textbook_softmax_topk():
    rng = np.random.default_rng(5)
    logits = rng.standard_normal((20, 24)).astype(np.float32)
    idx, wts = qo.moe_route(logits, 4, norm_topk=True)
    p = np.exp(logits.astype(np.float64) - logits.max(1, keepdims=True))
    p /= p.sum(1, keepdims=True)
    want_idx = np.argsort(-p, axis=1, kind="stable")[:, :4]
    assert np.array_equal(idx, want_idx)
    sel = np.take_along_axis(p, want_idx, 1)
    np.testing.assert_allclose(wts, sel / sel.sum(1, keepdims=True), rtol=1e-5)
    np.testing.assert_allclose(wts.sum(1), 1.0, rtol=1e-6)
    idx2, w2 = qo.moe_route(np.zeros((1, 8), np.float32), 3, norm_topk=False)
    assert idx2[0].tolist() == [0, 1, 2] and np.allclose(w2, 1 / 8)


def test_group_pairs_brute_force_and_tile_closed_forms():
    rng = np.random.default_rng(6)
    for t, e, k in [(1, 4, 2), (9, 8, 3), (200, 16, 4), (70, 4, 1)]:
        ids = np.stack([rng.choice(e, size=k, replace=False) for _ in range(t)]).astype(np.int32)
        ids[rng.random(ids.shape) < 0.1] = -1
        for compact in (True, False):
            g = qo.moe_group_pairs(ids, e, k, compact_tail=compact)
            flat = ids.ravel()
            valid = np.flatnonzero(flat >= 0)
            assert g["expertOff"][0] == 0 and g["expertOff"][e] == valid.size
            assert sorted(g["sortedPairIdx"].tolist()) == valid.tolist()
            assert np.array_equal(g["invPerm"][g["sortedPairIdx"]], np.arange(valid.size))
            assert np.array_equal(g["sortedTok"], g["sortedPairIdx"] // k)
            covered = np.zeros(valid.size, dtype=int)
            for te, tr in zip(g["tileE"], g["tileR"]):
                code, rb = tr >> 24, tr & 0xFFFFFF
                bm = {1: 16, 2: 32, 3: 64}[code]
                lo = g["expertOff"][te] + rb * bm
                hi = min(lo + bm, g["expertOff"][te + 1])
                assert lo < hi
                covered[lo:hi] += 1
            assert np.all(covered == 1)                         # tiles partition the slots exactly
            assert g["tileCount"] <= qo.moe_max_tiles(e, ids.size) or ids.size == 0
    # closed forms (qw_moe_tile.metalh:7-16, QWGemmMoE.swift:24-26)
    assert [qo.moe_tile_block(c) for c in (1, 16, 17, 32, 33, 64, 1000)] == [16, 16, 32, 32, 64, 64, 64]
    assert qo.moe_pack_tile_r(5, 16) == (1 << 24) | 5 and qo.moe_pack_tile_r(2, 64) == (3 << 24) | 2
    assert qo.moe_max_tiles(128, 16384) == 128 + 256 and qo.moe_max_tiles(128, 3) == 3
    # 70 rows of one expert with compact tail: one 64-row tile + one 16-row tail at row 64 = block index 4
    g = qo.moe_group_pairs(np.zeros(70, np.int32), 4, 1, compact_tail=True)
    assert g["tileR"].tolist() == [qo.moe_pack_tile_r(0, 64), qo.moe_pack_tile_r(4, 16)]


def test_swiglu_closed_form():
    g = np.array([0.0, 1.0, -2.0, 30.0, -30.0], dtype=np.float32)
    u = np.array([3.0, 2.0, 0.5, 1.0, 1.0], dtype=np.float32)
    want = g.astype(np.float64) / (1 + np.exp(-g.astype(np.float64))) * u
    np.testing.assert_allclose(qo.swiglu(g, u), want, rtol=1e-6, atol=1e-12)
    assert qo.swiglu_fwht_f16(np.ones((1, 48), np.float32), np.ones((1, 48), np.float32)).shape == (1, 48)  # I % 32 != 0: not rotated


def test_rmsnorm_closed_forms():
    """The norm restatement against what the mathematics fixes: a constant row (one non-zero coefficient per 32-group,
    c * rstd * (1 + g) * sqrt(32)), the plus-one law at gamma = 0 on a unit-RMS row (y = FWHT32(x)), Parseval between the
    rotated and the standard-basis output, and the exact residual update."""
    h, eps = 512, 1e-6
    c, g = np.float16(0.75), np.float16(0.125)
    y, _ = qo.rmsnorm_rot_f16(np.full((2, h), c, np.float16), np.full(h, g, np.float16), eps)
    want0 = float(c) / np.sqrt(float(c) ** 2 + eps) * (1.0 + float(g)) * np.sqrt(32.0)
    yv = y.astype(np.float64).reshape(2, h // 32, 32)
    assert np.allclose(yv[..., 0], want0, rtol=1e-3) and np.all(yv[..., 1:] == 0.0)
    rng = np.random.default_rng(0)
    x = rng.standard_normal((3, h)).astype(np.float32)
    x16 = (x / np.sqrt((x ** 2).mean(axis=1, keepdims=True))).astype(np.float16)          # unit RMS up to f16 rounding
    y, _ = qo.rmsnorm_rot_f16(x16, np.zeros(h, np.float16), 0.0)
    rms = np.sqrt((x16.astype(np.float64) ** 2).mean(axis=1, keepdims=True))
    assert np.max(np.abs(y.astype(np.float64) - qo.fwht32_ortho((x16.astype(np.float64) / rms).astype(np.float32)))) <= 2e-3
    gam = (rng.standard_normal(h) * 0.1).astype(np.float16)
    yr, _ = qo.rmsnorm_rot_f16(x16, gam, eps, rotate=True)
    yp, _ = qo.rmsnorm_rot_f16(x16, gam, eps, rotate=False)
    assert np.allclose((yr.astype(np.float64) ** 2).sum(axis=1), (yp.astype(np.float64) ** 2).sum(axis=1), rtol=2e-3)
    # transpose check: the rotated output is the transform of the plain one (up to the one f16 rounding each)
    assert np.max(np.abs(qo.fwht32_ortho(yp.astype(np.float32)) - yr.astype(np.float32))) <= 4e-3
    res = rng.standard_normal((3, h)).astype(np.float16)
    y2, res_out = qo.rmsnorm_rot_f16(x16, gam, eps, residual16=res)
    assert np.array_equal(res_out, (x16.astype(np.float32) + res.astype(np.float32)).astype(np.float16))
    y3, _ = qo.rmsnorm_rot_f16(res_out, gam, eps)
    assert np.array_equal(y2.view(np.uint16), y3.view(np.uint16))


def test_head_argmax_key_rule():
    """The sortable key is monotone on every finite float and the infinities, NaN maps to 0; the fold is numpy's first
    maximum whenever no NaN is the only candidate."""
    rng = np.random.default_rng(2)
    v = np.concatenate([rng.standard_normal(4000).astype(np.float32) * 1e3, np.array([-0.0, 0.0, np.inf, -np.inf, 1e-45, -1e-45], np.float32)])
    order = np.argsort(v, kind="stable")
    k = qo.sortable_f32_u32(v)[order].astype(np.int64)
    assert np.all(np.diff(k) >= 0) and qo.sortable_f32_u32(np.array([-0.0], np.float32))[0] < qo.sortable_f32_u32(np.array([0.0], np.float32))[0]
    assert qo.sortable_f32_u32(np.array([np.nan], np.float32))[0] == 0
    logits = rng.standard_normal((5, 1000)).astype(np.float32)
    assert np.array_equal(qo.head_argmax(logits), np.argmax(logits, axis=1))
    logits[0, [7, 300]] = 9.0                  # tie: the lower row
    logits[1, 5] = np.nan                      # NaN never wins
    logits[2, :] = np.nan                      # nothing but NaN: row 0
    logits[3, 999] = np.inf
    assert list(qo.head_argmax(logits)[:4]) == [7, int(np.nanargmax(logits[1])), 0, 999]


def test_f32_gemv_family_closed_forms():
    """The f32-activation GEMV restatement, pinned without retyping it: one-hot activations read single weights back (codes
    and headers are pinned on the golden blocks), the epilogues obey sigmoid(v) + sigmoid(-v) = 1 and silu(z) - silu(-z) = z,
    and epilogue 3's rotation is the golden-pinned fp32 FWHT (an involution; an impulse gives a +-1/sqrt(32) row)."""
    rng = np.random.default_rng(5)
    for bits, group, is_m5 in ((4, 32, True), (4, 64, False), (8, 32, False), (3, 32, False)):
        w = rng.standard_normal((40, 128)).astype(np.float32) * 0.02
        blocks, _ = qo.quant_hq_blocks(w, bits=bits, group=group, is_m5=is_m5, rotate=False)
        s, b = qo.hq_block_header(blocks) if not is_m5 else (
            np.ascontiguousarray(blocks[..., 0:2]).view(np.float16)[..., 0], np.ascontiguousarray(blocks[..., 2:4]).view(np.float16)[..., 0])
        codes = (qo.hq4_codes(blocks).reshape(40, 128).astype(np.int64) + 1024) if is_m5 else qo.hq_block_codes(blocks, bits, group).reshape(40, 128)
        for col in (0, 37, 127):
            x = np.zeros((1, 128), np.float32)
            x[0, col] = 1.0
            want = codes[:, col].astype(np.float64) * s[:, col // group].astype(np.float64) + b[:, col // group].astype(np.float64)
            assert np.array_equal(qo.gemv_f32(blocks, x, bits, group, is_m5)[0], want)
        x = rng.standard_normal((3, 128)).astype(np.float32)
        y = qo.gemv_f32(blocks, x, bits, group, is_m5)
        assert np.allclose(qo.gemv_f32(blocks, x, bits, group, is_m5, 2) + qo.gemv_f32(blocks, -x, bits, group, is_m5, 2), 1.0, atol=1e-15)
        assert np.allclose(qo.gemv_f32(blocks, x, bits, group, is_m5, 1, 0.25) - qo.gemv_f32(blocks, -x, bits, group, is_m5, 1, 0.25), y / 0.25, atol=1e-12)
        y3 = qo.gemv_f32(blocks, x, bits, group, is_m5, 3, 2.0)           # 40 outputs: one whole group and a padded one
        y1 = qo.gemv_f32(blocks, x, bits, group, is_m5, 1, 2.0)
        padded = np.zeros((3, 64))
        padded[:, :40] = y1
        assert np.allclose(y3, qo.fwht32_ortho(padded.astype(np.float32))[:, :40], atol=1e-6)
        assert np.allclose(qo.h32_groups_f64(qo.h32_groups_f64(padded)), padded, atol=1e-14)
    e = np.zeros((1, 32))
    e[0, 5] = 1.0
    row = qo.h32_groups_f64(e)[0] * np.sqrt(32.0)
    assert np.allclose(np.abs(row), 1.0) and row[0] == 1.0 and row[5] == np.float64((-1) ** bin(5).count("1"))
    assert qo.v4_epilogue_f64(np.array([0.0]), 2, 1.0)[0] == 0.5 and qo.v4_epilogue_f64(np.array([0.0]), 1, 3.0)[0] == 0.0


def test_router_shared_gate_closed_forms():
    """sigmoid(x . w): zero weights give exactly 1/2, negating the weight row gives the complement, a one-hot weight row
    reads sigmoid of one activation (against math.exp), and large dots saturate to 0 / 1 without overflow warnings."""
    import math
    rng = np.random.default_rng(3)
    x = rng.standard_normal((7, 96)).astype(np.float32)
    w = rng.standard_normal(96).astype(np.float32)
    assert np.array_equal(qo.router_shared_gate_f64(x, np.zeros(96, np.float32)), np.full(7, 0.5))
    g, gn = qo.router_shared_gate_f64(x, w), qo.router_shared_gate_f64(x, -w)
    np.testing.assert_allclose(g + gn, 1.0, rtol=0, atol=1e-15)
    onehot = np.zeros(96, np.float32)
    onehot[11] = 2.0
    want = [1.0 / (1.0 + math.exp(-2.0 * float(v))) for v in x[:, 11]]
    np.testing.assert_allclose(qo.router_shared_gate_f64(x, onehot), want, rtol=1e-15)
    with np.errstate(over="ignore"):
        big = qo.router_shared_gate_f64(np.array([[1e4], [-1e4]], np.float32), np.array([1.0], np.float32))
    assert big[0] == 1.0 and big[1] == 0.0


def test_embed_gather_reads_the_token_row():
    """The gather against the reference's own recipe (Tests/QWGEMMTests/QWAQEmbedGatherTests.swift:52-99): known codes and a
    header that is f16-exact but no power of two; the f64 law within product ulp + result ulp, hc copies equal, negative
    tokens read row 0, and the M5 container reads (q + 1024) * scale + bias of its own element order."""
    for bits, group in ((2, 64), (3, 32), (6, 128), (8, 256), (4, 32)):
        hidden, vocab = 256, 8
        i = np.arange(group)[None, None, :]
        r = np.arange(vocab)[:, None, None]
        g = np.arange(hidden // group)[None, :, None]
        codes = ((3 * i + 7 * r + 13 * g) % (1 << bits)).astype(np.uint8)
        blocks = np.empty((vocab, hidden // group, 4 + group * bits // 8), np.uint8)
        blocks[..., :4] = np.array([1025.0 / 4096.0, -683.0 / 4096.0], np.float16).view(np.uint8)
        blocks[..., 4:] = qo.pack_bitstream(codes, bits)
        out = qo.embed_aq_f32(blocks, [0, 3, 7, -2], 3, bits, group)
        assert out.shape == (4, 3, hidden) and out.dtype == np.float32
        code = codes.reshape(vocab, hidden)[[0, 3, 7, 0]].astype(np.float64)
        want = code * (1025.0 / 4096.0) + (-683.0 / 4096.0)
        tol = np.abs(code * 1025.0 / 4096.0) * 2.0 ** -24 + np.maximum(np.abs(want), 683.0 / 4096.0) * 2.0 ** -24
        assert np.all(np.abs(out[:, 0].astype(np.float64) - want) <= tol)
        assert np.array_equal(out[:, 0], out[:, 1]) and np.array_equal(out[:, 0], out[:, 2])
    w = (np.random.default_rng(2).standard_normal((6, 64)) * 0.02).astype(np.float32)
    m5, _ = qo.quant_hq_blocks(w, bits=4, group=32, is_m5=True, rotate=True)
    got = qo.embed_aq_f32(m5, [5, 1], 1, 4, 32, True)[:, 0]
    assert np.array_equal(got, qo.dequant_hq4_rot(m5)[[5, 1]])


def test_f32_seams_closed_forms():
    """silu_mul_f32: a constant gate|up row gives sqrt(32) * silu(g) * u in column 0 of every group and zeros elsewhere;
    bridge: the un-rotated copy of a rotated one-hot-in-standard-basis row is that one-hot (involution), the rotated copy
    is the input widened, and the split keeps ~21 bits; latent norm: constant row with gamma 0 -> sqrt(32) * sign in column
    0, gamma = 1 doubles it (plus-one law), no gamma = the bare transform, Parseval for the normalized row."""
    import math
    g, u = 0.75, -1.5
    gu = np.concatenate([np.full((2, 64), g, np.float32), np.full((2, 64), u, np.float32)], axis=1)
    out = qo.silu_mul_f32(gu)
    want0 = math.sqrt(32.0) * (g / (1.0 + math.exp(-g))) * u
    np.testing.assert_allclose(out[:, ::32], want0, rtol=2e-6)
    mask = np.ones(64, bool)
    mask[::32] = False
    assert np.all(np.abs(out[:, mask]) <= 1e-6)
    e = np.zeros((1, 256), np.float32)
    e[0, 37] = 1.0
    x16 = qo.fwht32_ortho(e).astype(np.float16)          # +-1/sqrt(32): f16-exact up to its rounding
    rot, plain = qo.moe_bridge_f16_to_f32(x16)
    assert np.array_equal(rot, x16.astype(np.float32))
    np.testing.assert_allclose(plain, e, atol=2e-3 * 0.18)
    rng = np.random.default_rng(8)
    y16 = rng.standard_normal((3, 256)).astype(np.float16)
    rot, plain = qo.moe_bridge_f16_to_f32(y16)
    np.testing.assert_allclose(plain, qo.fwht32_ortho(y16.astype(np.float32)), rtol=0, atol=4 * 2.0 ** -21)   # hi/lo keeps 21+ bits
    c = np.full((2, 96), -3.0, np.float32)
    n0 = qo.latent_norm_h32_f32(c, np.zeros(96, np.float16), eps=0.0)
    np.testing.assert_allclose(n0[:, ::32], -math.sqrt(32.0), rtol=1e-6)
    n1 = qo.latent_norm_h32_f32(c, np.ones(96, np.float16), eps=0.0)
    np.testing.assert_allclose(n1, 2.0 * n0, rtol=1e-6, atol=1e-6)
    r = rng.standard_normal((4, 128)).astype(np.float32)
    assert np.array_equal(qo.latent_norm_h32_f32(r), qo.fwht32_ortho(r))
    nr = qo.latent_norm_h32_f32(r, np.zeros(128, np.float16), eps=0.0)
    np.testing.assert_allclose((nr.astype(np.float64) ** 2).mean(axis=1), 1.0, rtol=1e-5)


def test_route_modes_closed_forms():
    """Sigmoid routing: without a bias the choice is the top-k of the logits (sigmoid is monotone) and normalised weights sum
    to one; a large bias forces an expert in while its weight stays its own small score; split features add two sigmoids;
    ties go to the lower index; a per-expert scale multiplies the normalised weight; no bias and no split = the softmax door."""
    import math
    rng = np.random.default_rng(12)
    lg = rng.standard_normal((6, 40)).astype(np.float32)
    idx, w = qo.moe_route_ex(lg, 4, True, 1.0, bias=np.zeros(40, np.float32))
    for r in range(6):
        assert sorted(idx[r].tolist()) == sorted(np.argsort(-lg[r], kind="stable")[:4].tolist())
        assert abs(float(w[r].sum()) - 1.0) < 1e-6
        assert np.all(np.diff(lg[r, idx[r]]) <= 0)                       # rank order = descending score
    bias = np.zeros(40, np.float32)
    bias[17] = 5.0
    lg2 = lg.copy()
    lg2[:, 17] = -6.0
    idx2, w2 = qo.moe_route_ex(lg2, 4, False, 1.0, bias=bias)
    assert np.all(idx2[:, 0] == 17)
    np.testing.assert_allclose(w2[:, 0], 1.0 / (1.0 + math.exp(6.0)), rtol=1e-6)      # the score, not score + bias
    sp = np.concatenate([lg, np.zeros_like(lg)], axis=1)                              # second half: sigmoid(0) = 1/2 everywhere
    idx3, w3 = qo.moe_route_ex(sp, 4, False, 1.0, split_feature=True)
    idx1, w1 = qo.moe_route_ex(lg, 4, False, 1.0, bias=np.zeros(40, np.float32))
    assert np.array_equal(idx3, idx1)
    np.testing.assert_allclose(w3, w1 + 0.5, rtol=1e-6)
    tie = np.zeros((1, 8), np.float32)
    idx4, _ = qo.moe_route_ex(tie, 3, True, 1.0, bias=np.zeros(8, np.float32))
    assert idx4[0].tolist() == [0, 1, 2]
    scale = np.arange(40, dtype=np.float32) + 1.0
    idx5, w5 = qo.moe_route_ex(lg, 4, True, 7.0, bias=np.zeros(40, np.float32), scale_param=scale)
    np.testing.assert_allclose(w5, w * scale[idx5], rtol=1e-6)
    a, b = qo.moe_route_ex(lg, 4, True, 2.5), qo.moe_route(lg, 4, True, 2.5)
    assert np.array_equal(a[0], b[0]) and np.allclose(a[1], b[1], rtol=1e-6)
    nan = lg.copy()
    nan[0, 3] = np.nan
    nan[0, 5] = np.inf
    idx6, _ = qo.moe_route_ex(nan, 40, False, 1.0, bias=np.zeros(40, np.float32))
    assert 3 not in idx6[0].tolist() and 5 not in idx6[0].tolist() and (idx6[0] == -1).sum() == 2


def test_grouped_moe_forward_equals_the_per_token_form():
    """moe_forward_grouped_f64 (work ordered by expert, matrix products) against moe_forward_f64 (the golden-pinned per-token
    loop): empty routes, ids with flag bits above bit 15, an expert nobody routes to, f16 hand-over with and without the
    rotation.  Without the f16 rounding of the activation the two agree to fp64 summation order; with it, a value that sits
    on an f16 rounding boundary may round the other way, hence the looser bar there."""
    rng = np.random.default_rng(77)
    t, e, k, h, inter = 37, 9, 3, 64, 96
    x = rng.standard_normal((t, h)).astype(np.float16)
    gu = (rng.standard_normal((e, 2 * inter, h)) * 0.2).astype(np.float16)
    dn = (rng.standard_normal((e, h, inter)) * 0.2).astype(np.float16)
    idx = np.stack([rng.permutation(e - 1)[:k] for _ in range(t)]).astype(np.int32)     # expert e - 1 is never routed
    idx[2, 1] = -1
    idx[5] = -1
    idx[7, 0] |= 3 << 16
    wts = rng.random((t, k)).astype(np.float32)
    a = qo.moe_forward_grouped_f64(x, idx, wts, gu, dn, act_f16=False, rotate_act=False)
    b = qo.moe_forward_f64(x, idx, wts, gu, dn, act_f16=False, rotate_act=False)
    np.testing.assert_allclose(a, b, rtol=1e-12, atol=1e-12)
    assert np.all(a[5] == 0)
    for rot in (False, True):
        a = qo.moe_forward_grouped_f64(x, idx, wts, gu, dn, act_f16=True, rotate_act=rot)
        b = qo.moe_forward_f64(x, idx, wts, gu, dn, act_f16=True, rotate_act=rot)
        assert qo.normalized_error(a, b) <= 1e-6
    none = qo.moe_forward_grouped_f64(x[:2], np.full((2, k), -1, np.int32), wts[:2], gu, dn, True, True)
    assert none.shape == (2, h) and np.all(none == 0)


def test_group_latent_block_identities():
    """moe_group_latent_forward_f64: (1) one group with identity D and U is the plain routed block; (2) without the f16
    hand-over roundings the grouped sum equals the per-route expansion sum_k w_k U_g(k) down_k(swiglu(gu_k(D_g(k) x)))
    (U_g is linear, so summing before or after it agrees); (3) swapping the labels of two experts that are not routed
    changes nothing, relabelling a routed one does; moe_latent_groups marks exactly the labels of the routes."""
    rng = np.random.default_rng(31)
    t, e, k, h, lat, inter, ng = 5, 12, 3, 64, 32, 64, 4
    x = rng.standard_normal((t, h))
    gu = rng.standard_normal((e, 2 * inter, lat)) * 0.2
    dn = rng.standard_normal((e, lat, inter)) * 0.2
    d = rng.standard_normal((ng, lat, h)) * 0.2
    u = rng.standard_normal((ng, h, lat)) * 0.2
    idx = np.stack([rng.permutation(e)[:k] for _ in range(t)]).astype(np.int32)
    idx[1, 2] = -1
    wts = rng.random((t, k)).astype(np.float32)
    labels = (np.arange(e) % ng).astype(np.int32)
    # (1)
    eye_d, eye_u = np.eye(lat)[None], np.eye(lat)[None]
    xl = rng.standard_normal((t, lat)).astype(np.float16)
    one = qo.moe_group_latent_forward_f64(xl, idx, wts, np.zeros(e, np.int32), eye_d, gu, dn, eye_u, latent_f16=False)
    np.testing.assert_allclose(one, qo.moe_forward_f64(xl, idx, wts, gu, dn, act_f16=True, rotate_act=True), rtol=1e-12, atol=1e-12)
    # (2)
    got = qo.moe_group_latent_forward_f64(x, idx, wts, labels, d, gu, dn, u, act_f16=False, rotate_act=False, latent_f16=False)
    want = np.zeros((t, h))
    for r in range(t):
        for j in range(k):
            ex = int(idx[r, j])
            if ex < 0:
                continue
            g = int(labels[ex])
            a = gu[ex] @ (d[g] @ x[r])
            act = a[:inter] / (1.0 + np.exp(-a[:inter])) * a[inter:]
            want[r] += float(wts[r, j]) * (u[g] @ (dn[ex] @ act))
    np.testing.assert_allclose(got, want, rtol=1e-10, atol=1e-10)
    # (3)
    unused = sorted(set(range(e)) - set(int(v) for v in idx.ravel() if v >= 0))
    if len(unused) >= 2 and labels[unused[0]] != labels[unused[1]]:
        l2 = labels.copy()
        l2[unused[0]], l2[unused[1]] = labels[unused[1]], labels[unused[0]]
        assert np.array_equal(qo.moe_group_latent_forward_f64(x, idx, wts, l2, d, gu, dn, u), qo.moe_group_latent_forward_f64(x, idx, wts, labels, d, gu, dn, u))
    l3 = labels.copy()
    l3[idx[0, 0]] = (labels[idx[0, 0]] + 1) % ng
    assert not np.allclose(qo.moe_group_latent_forward_f64(x, idx, wts, l3, d, gu, dn, u)[0], qo.moe_group_latent_forward_f64(x, idx, wts, labels, d, gu, dn, u)[0])
    gids, rows = qo.moe_latent_groups(idx, labels, ng)
    for r in range(t):
        have = {int(labels[v]) for v in idx[r] if v >= 0}
        assert {int(g) for g in gids[r] if g >= 0} == have and all(gids[r, g] in (-1, g) for g in range(ng))
        for j in range(k):
            assert rows[r, j] == (-1 if idx[r, j] < 0 else r * ng + labels[idx[r, j]])


def test_gated_activation_limits():
    """gated_act: kind 0 is swiglu; a clamp beyond every input changes nothing, a gate above the limit acts as the limit and up
    saturates at +-limit; the bounded form tends to SwiGLU for large parameters (x - beta tanh(x / beta) ~ x^3 / (3 beta^2)),
    is bounded by beta * linear_beta, keeps the sign structure, and equals its textbook value at a hand-computed point."""
    import math
    rng = np.random.default_rng(17)
    g, u = rng.standard_normal(500) * 3, rng.standard_normal(500) * 3
    base = qo.swiglu(g, u).astype(np.float64)
    np.testing.assert_allclose(qo.gated_act(g, u), base, rtol=1e-6, atol=1e-7)
    np.testing.assert_allclose(qo.gated_act(g, u, 1, 100.0), qo.gated_act(g, u), rtol=0, atol=0)
    lim = 1.5
    got = qo.gated_act(np.array([0.5, 9.0, 9.0, -4.0]), np.array([7.0, -7.0, 0.25, 0.5]), 1, lim)
    silu = lambda v: v / (1.0 + math.exp(-v))
    np.testing.assert_allclose(got, [silu(0.5) * lim, silu(lim) * -lim, silu(lim) * 0.25, silu(-4.0) * 0.5], rtol=1e-12)
    far = qo.gated_act(g, u, 2, 1e4, 1e4)
    np.testing.assert_allclose(far, qo.gated_act(g, u), rtol=1e-6, atol=1e-9)
    b, lb = 4.0, 25.0
    big = qo.gated_act(np.array([50.0, -50.0, 50.0]), np.array([1e3, 1e3, -1e3]), 2, b, lb)
    np.testing.assert_allclose(big, [b * lb, 0.0, -b * lb], rtol=1e-9, atol=1e-12)
    assert np.all(np.abs(qo.gated_act(g * 10, u * 10, 2, b, lb)) <= b * lb)
    one = qo.gated_act(np.array([2.0]), np.array([-3.0]), 2, b, lb)[0]
    want = (b * math.tanh(2.0 / b) / (1.0 + math.exp(-2.0))) * (lb * math.tanh(-3.0 / lb))
    assert abs(one - want) <= 1e-14 and abs(want - (-4.8611)) < 1e-3      # 4 tanh(.5) = 1.8485, sigmoid(2) = .8808, 25 tanh(-.12) = -2.9857: 1.8485 * .8808 * -2.9857
    np.testing.assert_allclose(qo.gated_act(g, u, 2, b, 0.0), b * np.tanh(g / b) / (1 + np.exp(-g)) * u, rtol=1e-12)


def test_route_budget_rules():
    """moe_route_budget: a hand-worked window, the invariants the reference's test asserts (row 0 never pruned, at most `budget`
    distinct experts, pruned routes weigh nothing: Tests/QWGEMMTests/QWErnie55MoETests.swift:332-343), renormalised rows keep their
    sum, and the no-op cases."""
    idx = np.array([[5, 2], [7, 2], [9, 4]], np.int32)
    wts = np.array([[0.6, 0.4], [0.7, 0.3], [0.55, 0.45]], np.float32)
    # row 0 holds {5, 2}; budget 3 admits the heaviest other pair: (1, 0) -> expert 7; experts 9 and 4 go
    i3, w3 = qo.moe_route_budget(idx, wts, 3, norm_topk=False)
    assert i3.tolist() == [[5, 2], [7, 2], [-1, -1]] and w3.tolist() == [[np.float32(0.6), np.float32(0.4)], [np.float32(0.7), np.float32(0.3)], [0.0, 0.0]]
    # budget 4: 7 (0.7) then 9 (0.55); expert 4 is pruned and row 2 is rescaled to its old sum 1.0
    i4, w4 = qo.moe_route_budget(idx, wts, 4, norm_topk=True)
    assert i4.tolist() == [[5, 2], [7, 2], [9, -1]]
    np.testing.assert_allclose(w4[2], [1.0, 0.0], rtol=1e-6)
    np.testing.assert_allclose(w4[:2], wts[:2], rtol=0)
    # a budget below top_k still keeps row 0 whole
    i1, _ = qo.moe_route_budget(idx, wts, 1, norm_topk=False)
    assert i1.tolist() == [[5, 2], [-1, 2], [-1, -1]]
    rng = np.random.default_rng(2)
    for m, k, e, b in [(2, 8, 32, 10), (4, 16, 64, 20), (3, 4, 8, 6), (4, 8, 128, 9)]:
        lg = rng.standard_normal((m, e)).astype(np.float32)
        ids, w = qo.moe_route(lg, k, True)
        bi, bw = qo.moe_route_budget(ids, w, b, norm_topk=True)
        assert np.array_equal(bi[0], ids[0]) and np.array_equal(bw[0], w[0])
        assert len({int(v) for v in bi.ravel() if v >= 0}) <= max(k, b)
        assert np.all(bw[bi < 0] == 0) and np.all((bi == ids) | (bi == -1))
        for r in range(1, m):
            if np.any(bi[r] >= 0):
                assert abs(float(bw[r].sum()) - float(w[r].sum())) <= 2e-6
    same_i, same_w = qo.moe_route_budget(idx, wts, 6)
    assert np.array_equal(same_i, idx) and np.array_equal(same_w, wts)


def test_variational_acceptance_and_f32_gemv_closed_forms():
    """head_argmax_variational: no margin = the plain argmax; a margin wider than the spread and no probability gate accepts every
    valid draft that is not the argmax; the last row and out-of-vocabulary drafts keep the argmax; the probability gate on a
    two-spike row follows log softmax = -log(1 + e^(a - b) + (v - 2) e^(low - b)).  f32_gemv: identity weights expose the
    epilogues (silu(x / s), sigmoid, 2 sigmoid(x / s) = 1 + tanh(x / 2s))."""
    import math
    rng = np.random.default_rng(4)
    lg = rng.standard_normal((5, 50)).astype(np.float32)
    draft = np.array([3, 7, 49, 50, 11, 2], np.int64)
    assert np.array_equal(qo.head_argmax_variational(lg, draft, 0.0), qo.head_argmax(lg))
    wide = qo.head_argmax_variational(lg, draft, 100.0)
    plain = qo.head_argmax(lg)
    assert wide[0] == 7 and wide[1] == 49 and wide[2] == plain[2] and wide[3] == 11 and wide[4] == 2
    short = qo.head_argmax_variational(lg, draft[:5], 100.0)
    assert short[4] == plain[4]
    a, b, low, v = 5.0, 4.0, -20.0, 50
    row = np.full((2, v), low, np.float32)
    row[:, 9], row[:, 17] = a, b
    lp = -math.log(1.0 + math.exp(a - b) + (v - 2) * math.exp(low - b))
    d2 = np.array([0, 17, 17], np.int64)
    assert qo.head_argmax_variational(row, d2, 2.0, lp - 1e-3)[0] == 17
    assert qo.head_argmax_variational(row, d2, 2.0, lp + 1e-3)[0] == 9
    assert qo.head_argmax_variational(row, d2, 0.5)[0] == 9           # outside the margin
    x = rng.standard_normal((3, 6))
    eye = np.eye(6)
    np.testing.assert_allclose(qo.f32_gemv(eye, x), x)
    np.testing.assert_allclose(qo.f32_gemv(eye, x, 1, 2.0), (x / 2) / (1 + np.exp(-x / 2)), rtol=1e-12)
    np.testing.assert_allclose(qo.f32_gemv(eye, x, 2), 1 / (1 + np.exp(-x)), rtol=1e-12)
    np.testing.assert_allclose(qo.f32_gemv(eye, x, 3, 2.0), 1 + np.tanh(x / 4), rtol=1e-12)
    w = rng.standard_normal((4, 6))
    np.testing.assert_allclose(qo.f32_gemv(w, x), np.einsum("tk,nk->tn", x, w), rtol=1e-12)
