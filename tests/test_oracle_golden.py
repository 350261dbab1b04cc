"""Pins the CPU oracle against every golden vector the reference's own tests hold for
the path (copied as data into tests/golden/) and against the vectors written by
tests/golden/gen_hq_blocks_golden.py from the reference's block quantizer."""
import json
import struct

import numpy as np
import pytest

from oracle import qworacle as qo


def _qwp(path):
    raw = path.read_bytes()
    assert raw[:4] == b"QWP1"
    # JSON trailer at EOF (Scripts/quantize/pack.py:115-316)
    start = raw.rfind(b'{"provenance"')
    return raw, json.loads(raw[start:].decode())


def test_hq4_quantizer_matches_reference_bytes(golden_dir):
    """aq_quantizer_golden.json: bf16 4x64 input and the 8 exact 20-byte blocks
    (Scripts/quantize/test_aq_golden.py:39-44)."""
    doc = json.loads((golden_dir / "aq_quantizer_golden.json").read_text())
    bf16 = np.frombuffer(bytes.fromhex(doc["bf16"]), dtype="<u2").reshape(doc["rows"], doc["cols"])
    want = np.frombuffer(bytes.fromhex(doc["blocks"]), dtype=np.uint8).reshape(doc["rows"], doc["cols"] // 32, 20)
    got = qo.quant_hq4_blocks(qo.bf16_bits_to_f32(bf16))
    assert np.array_equal(got, want)


def test_hq4_dequant_fwht_bit_identical_to_numpy_golden(golden_dir):
    """selfpack.qwp + selfpack.qwp.dq4.npy: 262,144 standard-domain fp32 answers, bit-identical
    (Tests/QWQuantTests/QWQuantTests.swift:69-85)."""
    raw, trailer = _qwp(golden_dir / "selfpack.qwp")
    ent = trailer["tensors"]["w_test"]
    n, k = ent["shape"]
    off = ent["hq4_off"]
    blocks = np.frombuffer(raw, dtype=np.uint8, count=n * (k // 32) * 20, offset=off).reshape(n, k // 32, 20)
    want = np.load(golden_dir / "selfpack.qwp.dq4.npy")
    got = qo.dequant_hq4(blocks)
    assert got.dtype == np.float32 and got.shape == want.shape
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_planar_hq8_dequant_matches_golden(golden_dir):
    """selfpack_hq8.qwp (+ .dq8rot.f32.bin), abs <= 1e-6 (Tests/QWQuantTests/QWHQ8PackTests.swift:30-44)."""
    raw, trailer = _qwp(golden_dir / "selfpack_hq8.qwp")
    ent = trailer["tensors"]["w_test8"]
    n, k = ent["shape"]
    qs = np.frombuffer(raw, dtype=np.int8, count=n * k, offset=ent["hq8_off"]).reshape(n, k)
    sc = np.frombuffer(raw, dtype=np.float16, count=n * (k // 32), offset=ent["hq8_s_off"]).reshape(n, k // 32)
    want = np.frombuffer((golden_dir / "selfpack_hq8.qwp.dq8rot.f32.bin").read_bytes(), dtype=np.float32).reshape(n, k)
    got = qo.dequant_hq8_planar_rot(qs, sc)
    assert np.max(np.abs(got - want)) <= 1e-6


def test_aq_block_unpack_matches_mlx_witness(golden_dir):
    """aq_repack_golden.json: 4-bit G64 MLX codes and dequantized values; the AQ bit stream for
    4 bits is byte b = elements 2b, 2b+1 (Scripts/oracle/gen_aq_fixtures.py:61-102)."""
    doc = json.loads((golden_dir / "aq_repack_golden.json").read_text())
    rows, cols, group, bits = doc["rows"], doc["cols"], doc["group"], doc["bits"]
    packed = np.frombuffer(bytes.fromhex(doc["packed"]), dtype=np.uint8).reshape(rows, cols // group, group * bits // 8)
    codes = np.frombuffer(bytes.fromhex(doc["codes"]), dtype=np.uint8).reshape(rows, cols // group, group)
    scales = np.frombuffer(bytes.fromhex(doc["scales"]), dtype=np.float32).reshape(rows, cols // group)
    biases = np.frombuffer(bytes.fromhex(doc["biases"]), dtype=np.float32).reshape(rows, cols // group)
    values = np.frombuffer(bytes.fromhex(doc["values"]), dtype=np.float32).reshape(rows, cols)
    assert np.array_equal(qo.unpack_bitstream(packed, bits, group), codes)
    assert np.array_equal(qo.pack_bitstream(codes, bits), packed)
    # build AQ blocks from the MLX header and decode them with the oracle
    blocks = np.empty((rows, cols // group, qo.hq_block_bytes(bits, group)), dtype=np.uint8)
    blocks[..., 0:2] = scales.astype(np.float16).view(np.uint8).reshape(rows, -1, 2)
    blocks[..., 2:4] = biases.astype(np.float16).view(np.uint8).reshape(rows, -1, 2)
    blocks[..., 4:] = packed
    got = qo.dequant_hq_blocks_rot(blocks, bits, group)
    # MLX scales/biases here are f16-representable? compare with the header actually stored
    s16 = scales.astype(np.float16).astype(np.float32)
    b16 = biases.astype(np.float16).astype(np.float32)
    want = (codes.astype(np.float32) * s16[..., None] + b16[..., None]).reshape(rows, cols)
    assert np.array_equal(got, want)
    if np.array_equal(s16, scales) and np.array_equal(b16, biases):
        assert np.max(np.abs(got - values)) < 1e-5


def test_mlx_repack_keeps_the_witness_codes_and_values(golden_dir):
    """aq_repack_golden.json through the repacker: the payload of every block is the MLX packed bytes, the header the
    f16 of the (bf16-rounded) MLX scale and bias, and the dequantized block is the witness's value wherever the header
    is exact in bf16 and f16 alike."""
    doc = json.loads((golden_dir / "aq_repack_golden.json").read_text())
    rows, cols, group, bits = doc["rows"], doc["cols"], doc["group"], doc["bits"]
    packed = np.frombuffer(bytes.fromhex(doc["packed"]), dtype=np.uint8).reshape(rows, cols * bits // 8)
    scales = np.frombuffer(bytes.fromhex(doc["scales"]), dtype=np.float32)
    biases = np.frombuffer(bytes.fromhex(doc["biases"]), dtype=np.float32)
    values = np.frombuffer(bytes.fromhex(doc["values"]), dtype=np.float32).reshape(rows, cols)
    s16, b16 = qo.f32_to_bf16_bits(scales), qo.f32_to_bf16_bits(biases)
    blocks, refused = qo.repack_mlx_affine(packed, s16, b16, rows, cols, bits, group, scale_is_f16=False)
    assert refused == 0 and blocks.shape == (rows, cols // group, qo.hq_block_bytes(bits, group))
    assert np.array_equal(blocks[..., 4:].reshape(rows, -1), packed)
    hs, hb = qo.hq_block_header(blocks)
    assert np.array_equal(hs.ravel(), qo.bf16_bits_to_f32(s16).astype(np.float16).astype(np.float32))
    got = qo.dequant_hq_blocks_rot(blocks, bits, group)
    exact = (qo.bf16_bits_to_f32(s16) == scales) & (qo.bf16_bits_to_f32(b16) == biases)
    cols_ok = np.repeat(exact.reshape(rows, -1), group, axis=1)
    if cols_ok.any():
        assert np.max(np.abs(got[cols_ok] - values[cols_ok])) < 1e-5


def test_f16_header_rule_on_every_bf16_value():
    """The exactness rule against first principles on all 65,536 bf16 patterns: a finite bf16 value is held by f16 iff it
    is 0, or 2^-14 <= |v| <= 65504 (8 significant bits always fit f16's 11); smaller magnitudes are accepted by the
    rule anyway, larger ones overflow and are refused; infinities convert back to themselves; NaN never does."""
    bits = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    v = qo.bf16_bits_to_f32(bits)
    with np.errstate(over="ignore", invalid="ignore"):
        holds = qo.f16_header_holds(v, v.astype(np.float16))
    with np.errstate(invalid="ignore"):
        a = np.abs(v.astype(np.float64))
    want = np.where(np.isnan(v), False, np.where(np.isinf(v), True, a <= 65504.0 + 16.0 - 1e-9))
    # |v| in (65504, 65520) would round down to 65504 and be refused by the round trip; bf16 has no value there
    assert not np.any((a > 65504.0) & (a < 65536.0))
    assert np.array_equal(holds, want)
    blocks, refused = qo.repack_mlx_affine(np.zeros((1, 16), np.uint8), np.array([0x7F00], np.uint16), np.array([0x3F80], np.uint16),
                                           1, 32, 4, 32, scale_is_f16=False)       # scale 1.7e38: refused, both halves poisoned
    assert refused == 1 and bytes(blocks[0, 0, :4]) == b"\x00\x7e\x00\x7e"


CASES = [
    ("aq4_g32_std", 4, 32, False, False),
    ("hq4_g32_blk", 4, 32, False, True),
    ("hq4_g64", 4, 64, False, True),
    ("hq8_g32", 8, 32, False, True),
    ("hq8_g64", 8, 64, False, True),
    ("hq6_g32", 6, 32, False, True),
    ("hq4_g128", 4, 128, False, True),
    ("hq8_g256", 8, 256, False, True),
    ("hq2_g64", 2, 64, False, True),
    ("hq3_g32", 3, 32, False, True),
    ("hq4_g32_m5", 4, 32, True, True),
]


@pytest.fixture(scope="module")
def blk_golden(golden_dir):
    return np.load(golden_dir / "hq_blocks_golden.npz")


@pytest.mark.parametrize("name,bits,group,is_m5,rotate", CASES)
def test_block_quantizer_bytes_match_reference(blk_golden, name, bits, group, is_m5, rotate):
    w = blk_golden["w"]
    got, eff = qo.quant_hq_blocks(w, bits=bits, group=group, is_m5=is_m5, rotate=rotate)
    assert eff == group
    assert np.array_equal(got, blk_golden[f"{name}__blocks"])


@pytest.mark.parametrize("name,bits,group,is_m5,rotate", CASES)
def test_block_dequant_matches_reference(blk_golden, name, bits, group, is_m5, rotate):
    blocks = blk_golden[f"{name}__blocks"]
    got = qo.dequant_hq_blocks_rot(blocks, bits, group, is_m5)
    assert np.array_equal(got.view(np.uint32), blk_golden[f"{name}__deq_rot"].view(np.uint32))
    got16 = qo.dequant_hq_blocks_rot(blocks, bits, group, is_m5, f16_round=True)
    assert np.array_equal(got16.view(np.uint32), blk_golden[f"{name}__deq_rot_f16"].view(np.uint32))
    # the single-rounding f16 weight the kernels materialise equals the reference's f16_round form here
    w16 = qo.weights_f16_exact(blocks, bits, group, is_m5)
    assert np.array_equal(w16.astype(np.float32), got16)


def test_planar_hq8_quantizer_and_fwht_match_reference(blk_golden):
    qs, sc = qo.quant_hq8_planar(blk_golden["w"])
    assert np.array_equal(qs, blk_golden["hq8_planar__qs"])
    assert np.array_equal(sc.view(np.uint16), blk_golden["hq8_planar__scales"])
    got = qo.fwht32_ortho(blk_golden["fwht__in"])
    assert np.array_equal(got.view(np.uint32), blk_golden["fwht__out"].view(np.uint32))


def test_sparse_moe_golden(golden_dir):
    """fn_goldens.json key sparse_moe (hidden 16, 8 experts, top-2, I = 12): routing + routed
    experts + shared expert, torch-generated (Tests/QWFlashNextTests/fixtures/fn_goldens.json)."""
    doc = json.loads((golden_dir / "fn_sparse_moe_golden.json").read_text())["sparse_moe"]

    def arr(d):
        return np.array(d["data"], dtype=np.float32).reshape(d["shape"])

    w = {k: arr(v) for k, v in doc["weights"].items()}
    x = arr(doc["input"])
    want = arr(doc["output"])
    h, e, k, i = doc["hidden"], doc["experts"], doc["top_k"], doc["expert_intermediate"]
    xt = x.reshape(-1, h)
    logits = (xt.astype(np.float32) @ w["gate.weight"].T).astype(np.float32)
    idx, wts = qo.moe_route(logits, k, norm_topk=doc["norm_topk_prob"])
    routed = qo.moe_forward_f64(xt, idx, wts, w["experts.gate_up_proj"], w["experts.down_proj"],
                                act_f16=False, rotate_act=False)
    # shared expert scaled by a sigmoid gate (FNSparseMoE.forward)
    g = xt @ w["shared_expert.gate_proj.weight"].T
    u = xt @ w["shared_expert.up_proj.weight"].T
    sh = (g / (1 + np.exp(-g)) * u) @ w["shared_expert.down_proj.weight"].T
    gate = 1.0 / (1.0 + np.exp(-(xt @ w["shared_expert_gate.weight"].T)))
    got = routed + gate * sh
    assert np.max(np.abs(got - want.reshape(-1, h))) < 2e-5
