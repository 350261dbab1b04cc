"""CPU oracle for the quantized matrix-multiply path (TEST INFRASTRUCTURE ONLY).

This module restates, in numpy, the reference's algorithms for the QWGEMM path:
the HQ4_G32_M5 and HQ/AQ block quantizers, their dequantizers, the 32-point
orthonormal Walsh-Hadamard rotation, the oracle matmul forms, SwiGLU, the MoE
router (softmax and sigmoid / bias / split-feature modes, the shared-expert gate), the
expert-major pair sort with its tile list, the whole routed MoE block, and the seams
either side of the path (RMSNorm + rotation, LM-head argmax, the f32 GEMV family, the
embedding gather, the f32 bridge / SwiGLU / latent norm of the MoE chain, the MLX
repacker).  Only tests, the smoke check and the benchmark's CPU-baseline leg may
import it; the product path (libqwhip) never does.

Every function cites the reference file:line it follows (paths relative to the
reference checkout).  How each function is pinned is listed next to it:

  golden  = byte/bit-exact against a fixture under tests/golden/
  math    = closed forms / invariants / brute force in tests/test_oracle_*.py

Nothing in this file is "parity unpinned" except `quant_hq_blocks` for bits in
{2, 3} when the MSE-clip search meets a near-tie between two shrink candidates
(the reference's torch `mean` summation order is not restated); the golden
vectors for those two widths are still checked and pass.
"""
from __future__ import annotations

import math

import numpy as np

GROUP = 32
HQ4_BLOCK_BYTES = 20
# f32(1/sqrt(32)) = 0x3E3504F3  (Scripts/quantize/hq4.py:18)
INV_SQRT32 = np.float32(1.0 / math.sqrt(32.0))
BIAS_LAW = np.float32(-1032.0)       # hq4.py:21
SCALE_DIVISOR = np.float32(7.5)      # hq4.py:22
MAX_SCALE = np.float32(63.46875)     # hq4.py:23

VALID_BITS = (2, 3, 4, 6, 8)         # hq_blocks.py:18
VALID_GROUPS = (32, 64, 128, 256)    # hq_blocks.py:19


# --------------------------------------------------------------------------- #
# small numeric helpers
# --------------------------------------------------------------------------- #
def f32_to_bf16_bits(values: np.ndarray) -> np.ndarray:
    """f32 -> bf16 bit patterns, round-to-nearest-even (Scripts/oracle/gen_aq_fixtures.py:32-36)."""
    bits = np.ascontiguousarray(values, dtype=np.float32).view(np.uint32)
    rounding = ((bits >> 16) & 1) + np.uint32(0x7FFF)
    return (((bits + rounding) & np.uint32(0xFFFF0000)) >> 16).astype(np.uint16)


def bf16_bits_to_f32(bits: np.ndarray) -> np.ndarray:
    return (np.asarray(bits).astype(np.uint32) << 16).view(np.float32)


def round_bf16(values: np.ndarray) -> np.ndarray:
    return bf16_bits_to_f32(f32_to_bf16_bits(values))


# --------------------------------------------------------------------------- #
# FWHT-32  (pinned: golden selfpack.qwp.dq4.npy, hq_blocks_golden fwht; math: H*H = I, vs dense Hadamard)
# --------------------------------------------------------------------------- #
def fwht32_ortho(x: np.ndarray) -> np.ndarray:
    """Orthonormal 32-point Walsh-Hadamard transform over the last axis' 32-groups.

    fp32 butterflies h = 1, 2, 4, 8, 16 writing (u+v, u-v) to (i, i+h), then ONE
    multiply by f32(1/sqrt(32)).  Follows Scripts/quantize/hq4.py:26-51 and
    Sources/Foundation/QWQuant/QWQuant+DequantMath.swift:93-112.
    """
    orig = x.shape
    assert orig[-1] % 32 == 0
    y = np.array(x, dtype=np.float32, copy=True).reshape(-1, 32)
    h = 1
    while h < 32:
        y = y.reshape(-1, 32 // (2 * h), 2, h)
        u = y[:, :, 0, :].copy()
        v = y[:, :, 1, :].copy()
        y[:, :, 0, :] = u + v
        y[:, :, 1, :] = u - v
        y = y.reshape(-1, 32)
        h *= 2
    return (y * INV_SQRT32).astype(np.float32).reshape(orig)


# --------------------------------------------------------------------------- #
# HQ4_G32_M5  (pinned: golden aq_quantizer_golden.json, hq_blocks_golden hq4_g32_m5, selfpack.qwp)
# --------------------------------------------------------------------------- #
def hq4_interleave(q: np.ndarray) -> np.ndarray:
    """codes [..., 32] (int) -> u32 words [..., 4] in the HQ4_G32_M5 nibble order.

    word = q0 | q1<<16 | q2<<4 | q3<<20 | q4<<8 | q5<<24 | q6<<12 | q7<<28
    (Scripts/quantize/hq4.py:112-118, Sources/Foundation/QWQuant/QWAQProducer.swift:85-87).
    """
    q8 = q.astype(np.uint32).reshape(*q.shape[:-1], 4, 8)
    return ((q8[..., 0] << 0) | (q8[..., 1] << 16) | (q8[..., 2] << 4) | (q8[..., 3] << 20)
            | (q8[..., 4] << 8) | (q8[..., 5] << 24) | (q8[..., 6] << 12) | (q8[..., 7] << 28)).astype(np.uint32)


def hq4_codes(blocks: np.ndarray) -> np.ndarray:
    """blocks [..., 20] u8 -> codes [..., 32] u8 (inverse of hq4_interleave; hq4.py:138-149)."""
    qs = np.ascontiguousarray(blocks[..., 4:20]).view(np.uint32)
    q = np.empty(blocks.shape[:-1] + (32,), dtype=np.uint8)
    for j in range(4):
        raw = qs[..., j]
        for e, sh in enumerate((0, 16, 4, 20, 8, 24, 12, 28)):
            q[..., 8 * j + e] = (raw >> sh) & 0xF
    return q


def quant_hq4_blocks(w: np.ndarray, rotate: bool = True) -> np.ndarray:
    """[N, K] f32 -> HQ4_G32_M5 blocks [N, K/32, 20] u8.  Follows hq4.py:54-123.

    scale = f16(min(amax/7.5, 63.46875)); bias = f16(-1032*f32(scale));
    q = clamp(floor((v - bias)/scale - 1023.5), 0, 15); scale == 0 -> code 8.
    All arithmetic is IEEE fp32, one operation at a time.
    """
    w = np.ascontiguousarray(w, dtype=np.float32)
    if w.ndim != 2 or w.shape[0] <= 0 or w.shape[1] <= 0 or w.shape[1] % GROUP:
        raise ValueError("HQ4_G32_M5 requires a non-empty 2-D tensor with K divisible by 32")
    if not np.isfinite(w).all():
        raise ValueError("HQ4_G32_M5 source weights must be finite")
    n, k = w.shape
    g = k // GROUP
    v = fwht32_ortho(w) if rotate else w
    v = v.reshape(n, g, GROUP)
    amax = np.abs(v).max(axis=-1)
    scale16 = np.minimum(amax / SCALE_DIVISOR, MAX_SCALE).astype(np.float16)
    s = scale16.astype(np.float32)
    bias16 = (BIAS_LAW * s).astype(np.float16)
    b = bias16.astype(np.float32)
    safe = np.where(s > 0, s, np.float32(1.0))[..., None]
    qf = np.floor((v - b[..., None]) / safe - np.float32(1023.5))
    q = np.where(s[..., None] > 0, np.clip(qf, 0, 15), np.float32(8.0)).astype(np.int32)
    blocks = np.empty((n, g, HQ4_BLOCK_BYTES), dtype=np.uint8)
    blocks[..., 0:2] = scale16.view(np.uint8).reshape(n, g, 2)
    blocks[..., 2:4] = bias16.view(np.uint8).reshape(n, g, 2)
    blocks[..., 4:20] = hq4_interleave(q).view(np.uint8).reshape(n, g, 16)
    return blocks


def dequant_hq4_rot(blocks: np.ndarray, f16_round: bool = False) -> np.ndarray:
    """HQ4 blocks [N, G, 20] -> rotated-domain weights [N, 32 G] f32.

    w = (q + 1024) * scale + bias, fp32 multiply then fp32 add (hq4.py:131-154,
    QWQuant+DequantMath.swift:75-91).  With f16_round the result is rounded once
    more to f16 (the form the GPU kernels contract; the intermediate fp32 value is
    exact, so this equals RN_f16 of the exact real value).
    """
    n, g, bb = blocks.shape
    assert bb == HQ4_BLOCK_BYTES
    scale = np.ascontiguousarray(blocks[..., 0:2]).view(np.float16).astype(np.float32)
    bias = np.ascontiguousarray(blocks[..., 2:4]).view(np.float16).astype(np.float32)
    q = hq4_codes(blocks).astype(np.float32)
    w = (q + np.float32(1024.0)) * scale + bias
    if f16_round:
        w = w.astype(np.float16).astype(np.float32)
    return w.reshape(n, g * GROUP)


def dequant_hq4(blocks: np.ndarray) -> np.ndarray:
    """Standard-domain dequant: rotate the decoded groups back (hq4.py:157-158)."""
    return fwht32_ortho(dequant_hq4_rot(blocks, f16_round=False))


# --------------------------------------------------------------------------- #
# HQ/AQ block family  (pinned: golden hq_blocks_golden.npz, aq_repack_golden.json; math: size law, bit stream)
# --------------------------------------------------------------------------- #
def resolve_group_size(k: int, requested: int) -> int:
    """hq_blocks.py:106-114."""
    if k <= 0 or k % 32:
        raise ValueError(f"Inner dimension K={k} must be a positive multiple of 32")
    if requested not in VALID_GROUPS:
        raise ValueError(f"Unsupported group size {requested}")
    eff = math.gcd(k, requested)
    if eff not in VALID_GROUPS:
        raise ValueError(f"Resolved group size {eff} not supported")
    return eff


def hq_block_bytes(bits: int, group: int) -> int:
    """4-byte header + group*bits/8 payload (hq_blocks.py:118-121, QWAQBlock.swift:36-46)."""
    if bits not in VALID_BITS or group not in VALID_GROUPS:
        raise ValueError(f"Unsupported (bits={bits}, group={group})")
    return group * bits // 8 + 4


def pack_bitstream(q: np.ndarray, bits: int) -> np.ndarray:
    """codes [..., G] -> continuous little-endian bit stream [..., G*bits/8] u8;
    element i occupies bits [i*bits, (i+1)*bits)  (hq_blocks.py:125-163, QWAQBlock.swift:115-167)."""
    q = np.asarray(q).astype(np.uint64) & ((1 << bits) - 1)
    g = q.shape[-1]
    nbytes = g * bits // 8
    # work in chunks of 8 elements = `bits` bytes
    q8 = q.reshape(*q.shape[:-1], g // 8, 8)
    word = np.zeros(q8.shape[:-1], dtype=np.uint64)
    for j in range(8):
        word |= q8[..., j] << np.uint64(j * bits)
    out = np.empty(q8.shape[:-1] + (bits,), dtype=np.uint8)
    for b in range(bits):
        out[..., b] = ((word >> np.uint64(8 * b)) & np.uint64(0xFF)).astype(np.uint8)
    return out.reshape(*q.shape[:-1], nbytes)


def unpack_bitstream(payload: np.ndarray, bits: int, group: int) -> np.ndarray:
    """Inverse of pack_bitstream -> codes [..., group] u8 (hq_blocks.py:167-195, QWAQBlock.readBits)."""
    p = np.asarray(payload, dtype=np.uint8)
    p8 = p.reshape(*p.shape[:-1], group // 8, bits).astype(np.uint64)
    word = np.zeros(p8.shape[:-1], dtype=np.uint64)
    for b in range(bits):
        word |= p8[..., b] << np.uint64(8 * b)
    out = np.empty(p8.shape[:-1] + (8,), dtype=np.uint8)
    mask = np.uint64((1 << bits) - 1)
    for j in range(8):
        out[..., j] = ((word >> np.uint64(j * bits)) & mask).astype(np.uint8)
    return out.reshape(*p.shape[:-1], group)


def _mse_optimal_scale_bias(wf, w_min, w_max, qmax):
    """10-point shrink search for 2/3-bit groups (hq_blocks.py:409-432)."""
    half = np.float32(0.5)
    mid = half * (w_max + w_min)
    half_span = half * (w_max - w_min)
    best_scale = ((w_max - w_min) / qmax).astype(np.float16)
    best_bias = w_min.astype(np.float16)
    best_err = np.full(w_min.shape, np.inf, dtype=np.float32)
    for shrink in (1.00, 0.96, 0.92, 0.88, 0.85, 0.82, 0.79, 0.76, 0.73, 0.70):
        sh = np.float32(shrink)
        c_min = mid - sh * half_span
        c_max = mid + sh * half_span
        sc16 = ((c_max - c_min) / qmax).astype(np.float16)
        bi16 = c_min.astype(np.float16)
        sc32 = sc16.astype(np.float32)[..., None]
        bi32 = bi16.astype(np.float32)[..., None]
        safe = np.where(sc32 > 0, sc32, np.float32(1.0))
        q = np.clip(np.rint((wf - bi32) / safe), 0, qmax)
        q = np.where(sc32 > 0, q, np.float32(0.0))
        recon = q * sc32 + bi32
        d = wf - recon
        err = (d * d).mean(axis=-1, dtype=np.float32)
        better = err < best_err
        best_err = np.where(better, err, best_err)
        best_scale = np.where(better, sc16, best_scale)
        best_bias = np.where(better, bi16, best_bias)
    return best_scale, best_bias


def quant_hq_blocks(w: np.ndarray, bits: int = 4, group: int = 32, is_m5: bool = False,
                    rotate: bool = True, mse_clip: bool | None = None):
    """[N, K] f32 -> ([N, K/G, 4 + G*bits/8] u8, effective group).  Follows hq_blocks.py:436-517.

    Optional FWHT over 32-element groups (always 32, whatever G), per group
    scale = f16((max-min)/qmax), bias = f16(min), q = clamp(rint((w-bias)/scale), 0, qmax),
    scale == 0 -> code 0.  (4, 32, is_m5) delegates to the HQ4_G32_M5 writer.
    """
    w = np.ascontiguousarray(w, dtype=np.float32)
    if w.ndim != 2:
        raise ValueError("quant_hq_blocks expects a 2-D tensor")
    n, k = w.shape
    eff = resolve_group_size(k, group)
    if bits == 4 and eff == 32 and is_m5:
        return quant_hq4_blocks(w, rotate=rotate), 32
    if bits not in VALID_BITS:
        raise ValueError(f"Unsupported bits={bits}")
    if not np.isfinite(w).all():
        raise ValueError("quant_hq_blocks rejects non-finite weights")
    use_mse = (bits in (2, 3)) if mse_clip is None else bool(mse_clip)
    nb = k // eff
    qmax = np.float32((1 << bits) - 1)
    wf = (fwht32_ortho(w) if rotate else w).reshape(n, nb, eff)
    w_min = wf.min(axis=-1)
    w_max = wf.max(axis=-1)
    if use_mse:
        scale16, bias16 = _mse_optimal_scale_bias(wf, w_min, w_max, qmax)
    else:
        scale16 = ((w_max - w_min) / qmax).astype(np.float16)
        bias16 = w_min.astype(np.float16)
    s = scale16.astype(np.float32)[..., None]
    b = bias16.astype(np.float32)[..., None]
    safe = np.where(s > 0, s, np.float32(1.0))
    q = np.clip(np.rint((wf - b) / safe), 0, qmax).astype(np.uint8)
    q = np.where(s > 0, q, np.uint8(0))
    out = np.empty((n, nb, hq_block_bytes(bits, eff)), dtype=np.uint8)
    out[..., 0:2] = scale16.view(np.uint8).reshape(n, nb, 2)
    out[..., 2:4] = bias16.view(np.uint8).reshape(n, nb, 2)
    out[..., 4:] = pack_bitstream(q, bits)
    return out, eff


def hq_block_codes(blocks: np.ndarray, bits: int, group: int) -> np.ndarray:
    return unpack_bitstream(blocks[..., 4:], bits, group)


def hq_block_header(blocks: np.ndarray):
    """(scale f32 [N, nb], bias f32 [N, nb]) from the little-endian f16 header (QWAQBlock.swift:107-111)."""
    s = np.ascontiguousarray(blocks[..., 0:2]).view(np.float16)[..., 0].astype(np.float32)
    b = np.ascontiguousarray(blocks[..., 2:4]).view(np.float16)[..., 0].astype(np.float32)
    return s, b


def dequant_hq_blocks_rot(blocks: np.ndarray, bits: int = 4, group: int = 32, is_m5: bool = False,
                          f16_round: bool = False) -> np.ndarray:
    """Blocks -> block-domain weights [N, K] f32: w = code*scale + bias in fp32
    (hq_blocks.py:520-541; host twin QWAQBlock.swift:91-104)."""
    if bits == 4 and group == 32 and is_m5:
        return dequant_hq4_rot(blocks, f16_round=f16_round)
    n, nb, bb = blocks.shape
    if bb != hq_block_bytes(bits, group):
        raise ValueError("block size does not match (bits, group)")
    s, b = hq_block_header(blocks)
    q = hq_block_codes(blocks, bits, group).astype(np.float32)
    w = q * s[..., None] + b[..., None]
    if f16_round:
        w = w.astype(np.float16).astype(np.float32)
    return w.reshape(n, nb * group)


def embed_aq_f32(blocks: np.ndarray, tokens, hc: int = 1, bits: int = 4, group: int = 32, is_m5: bool = False) -> np.ndarray:
    """Embedding gather over a block table [vocab, K/group, block bytes] -> f32 [rows, hc, hidden]: the token's row decoded
    with the container's own law (code*scale + bias in fp32, block domain), written hc times; a negative token reads row 0
    (Sources/QWMetal/gemm/qwgemm_aq_embed.metal:14-52; QWGemmAQ.swift:147-187)."""
    tok = np.maximum(np.asarray(tokens, dtype=np.int64), 0)
    rows = dequant_hq_blocks_rot(np.asarray(blocks)[tok], bits, group, is_m5)
    return np.repeat(rows[:, None, :], hc, axis=1).astype(np.float32)


def dequant_hq_blocks(blocks, bits=4, group=32, is_m5=False, f16_round=False) -> np.ndarray:
    """Standard-domain dequant of a ROTATED bank (hq_blocks.py:545-561)."""
    return fwht32_ortho(dequant_hq_blocks_rot(blocks, bits, group, is_m5, f16_round))


def weights_f16_exact(blocks: np.ndarray, bits: int, group: int, is_m5: bool) -> np.ndarray:
    """The f16 weight every GPU kernel must materialise: RN_f16 of the EXACT real value
    (q+1024)*s + b  (M5; one half2 FMA, Sources/QWMetal/include/qw_dequant.metalh:42-62) or
    code*s + b  (blocks; `Float16(code*scale+bias)` in double,
    Tests/QWGEMMTests/QWAQBatchedGemmTests.swift:88-92).  Evaluated in float64, where the
    product and the sum are exact, then rounded once."""
    if is_m5:
        n, g, _ = blocks.shape
        s = np.ascontiguousarray(blocks[..., 0:2]).view(np.float16).astype(np.float64)
        b = np.ascontiguousarray(blocks[..., 2:4]).view(np.float16).astype(np.float64)
        q = hq4_codes(blocks).astype(np.float64)
        return ((q + 1024.0) * s + b).astype(np.float16).reshape(n, g * GROUP)
    n, nb, _ = blocks.shape
    s, b = hq_block_header(blocks)
    q = hq_block_codes(blocks, bits, group).astype(np.float64)
    return (q * s.astype(np.float64)[..., None] + b.astype(np.float64)[..., None]).astype(np.float16).reshape(n, nb * group)


def f16_header_holds(raw: np.ndarray, stored: np.ndarray) -> np.ndarray:
    """qwg_f16_header_holds (Sources/QWMetal/quant/qw_online_quant.metal:62-69): `stored = half(raw)` holds `raw` when it
    converts back to it, or when both are finite and |raw| < 2^-14 (the subnormal range of f16, where the nearest
    2^-24 step is accepted)."""
    raw = np.asarray(raw, dtype=np.float32)
    back = np.asarray(stored, dtype=np.float16).astype(np.float32)
    with np.errstate(invalid="ignore"):
        same = back == raw
        small = np.isfinite(raw) & np.isfinite(back) & (np.abs(raw) < np.float32(6.103515625e-5))
    return same | small


def _mlx_header_f32(bits16: np.ndarray, is_f16: bool) -> np.ndarray:
    b = np.ascontiguousarray(bits16, dtype=np.uint16)
    return b.view(np.float16).astype(np.float32) if is_f16 else bf16_bits_to_f32(b)


def repack_mlx_affine(mlx_w: np.ndarray, scales16: np.ndarray, biases16: np.ndarray, rows: int, cols: int, bits: int,
                      group: int, scale_is_f16: bool):
    """qwg_repack_mlx_affine_to_aq_m5 (qw_online_quant.metal:71-122): MLX packed codes [rows, cols*bits/8] bytes and one
    bf16/f16 (scale, bias) pair per group -> AQ blocks [rows, cols/group, 4 + group*bits/8] at the same byte count.
    Payload bytes are copied; a header f16 does not hold is the f16 NaN 0x7e00 in both halves and is counted.
    Returns (blocks u8, refused count)."""
    groups, payload = cols // group, group * bits // 8
    w = np.ascontiguousarray(mlx_w).view(np.uint8).reshape(rows, groups, payload)
    with np.errstate(over="ignore"):
        rs = _mlx_header_f32(scales16, scale_is_f16).reshape(rows, groups)
        rb = _mlx_header_f32(biases16, scale_is_f16).reshape(rows, groups)
        hs, hb = rs.astype(np.float16), rb.astype(np.float16)
    exact = f16_header_holds(rs, hs) & f16_header_holds(rb, hb)
    blocks = np.empty((rows, groups, 4 + payload), dtype=np.uint8)
    poison = np.uint16(0x7E00)
    blocks[..., 0:2] = np.where(exact, hs.view(np.uint16), poison).astype(np.uint16)[..., None].view(np.uint8)
    blocks[..., 2:4] = np.where(exact, hb.view(np.uint16), poison).astype(np.uint16)[..., None].view(np.uint8)
    blocks[..., 4:] = w
    return blocks, int((~exact).sum())


def repack_mlx_affine_switch_gate_up(gate_w, gate_s, gate_b, up_w, up_s, up_b, experts: int, inter: int, cols: int, bits: int,
                                     group: int, scale_is_f16: bool):
    """qwg_repack_mlx_affine_switch_gate_up_to_aq_m5 (qw_online_quant.metal:124-178): gate_proj and up_proj
    [experts, inter, cols] interleaved per expert into one [experts, 2*inter, cols] AQ bank (gate rows, then up rows)."""
    g, rg = repack_mlx_affine(gate_w, gate_s, gate_b, experts * inter, cols, bits, group, scale_is_f16)
    u, ru = repack_mlx_affine(up_w, up_s, up_b, experts * inter, cols, bits, group, scale_is_f16)
    nb, bb = g.shape[1], g.shape[2]
    out = np.concatenate([g.reshape(experts, inter, nb, bb), u.reshape(experts, inter, nb, bb)], axis=1)
    return out.reshape(experts * 2 * inter, nb, bb), rg + ru


def weights_affine_f64(blocks: np.ndarray, bits: int, group: int, is_m5: bool) -> np.ndarray:
    """The un-rounded real weights (q+1024)*s + b (M5) / code*s + b (blocks) in float64: what the reference's
    factorised GEMVs contract, scale * sum(code * x) + bias * sum(x) per slice (qwg_aq_slice_dot,
    Sources/QWMetal/include/qw_dequant_multi.metalh:205-208).  Differs from `weights_f16_exact` only by the f16
    rounding of each weight; pinned through it (same codes, same headers)."""
    if is_m5:
        n, g, _ = blocks.shape
        s = np.ascontiguousarray(blocks[..., 0:2]).view(np.float16).astype(np.float64)
        b = np.ascontiguousarray(blocks[..., 2:4]).view(np.float16).astype(np.float64)
        q = hq4_codes(blocks).astype(np.float64)
        return ((q + 1024.0) * s + b).reshape(n, g * GROUP)
    n, nb, _ = blocks.shape
    s, b = hq_block_header(blocks)
    q = hq_block_codes(blocks, bits, group).astype(np.float64)
    return (q * s.astype(np.float64)[..., None] + b.astype(np.float64)[..., None]).reshape(n, nb * group)


# --------------------------------------------------------------------------- #
# planar HQ8_G32_M5  (pinned: golden selfpack_hq8.qwp + .dq8rot.f32.bin, hq_blocks_golden hq8_planar)
# --------------------------------------------------------------------------- #
def quant_hq8_planar(w: np.ndarray):
    """[N, K] -> (int8 [N, K], f16 scales [N, K/32]); symmetric, rotated (hq_blocks.py:564-607)."""
    w = np.ascontiguousarray(w, dtype=np.float32)
    n, k = w.shape
    g = k // GROUP
    v = fwht32_ortho(w).reshape(n, g, GROUP)
    amax = np.abs(v).max(axis=-1)
    scale16 = (amax / np.float32(127.0)).astype(np.float16)
    s = scale16.astype(np.float32)[..., None]
    safe = np.where(s > 0, s, np.float32(1.0))
    q = np.where(s > 0, np.clip(np.rint(v / safe), -127.0, 127.0), np.float32(0.0))
    return q.reshape(n, k).astype(np.int8), scale16


def dequant_hq8_planar_rot(qs: np.ndarray, scales: np.ndarray) -> np.ndarray:
    """hq_blocks.py:610-615; Sources/Foundation/QWQuant/QWPack.swift:326-351."""
    n, k = qs.shape
    sc = np.asarray(scales, dtype=np.float16).astype(np.float32)
    return (qs.astype(np.float32).reshape(n, k // GROUP, GROUP) * sc[:, :, None]).reshape(n, k)


# --------------------------------------------------------------------------- #
# matmul forms
# --------------------------------------------------------------------------- #
def matmul_ref_f64(x: np.ndarray, w_f16: np.ndarray) -> np.ndarray:
    """The judged reference: fp64 evaluation of x[M,K] . W_deq[N,K]^T with the f16 weights."""
    return np.asarray(x, dtype=np.float64) @ np.asarray(w_f16, dtype=np.float64).T


def cpu_oracle_gemv(blocks: np.ndarray, x_rot_f16: np.ndarray, bits=4, group=32, is_m5=True) -> np.ndarray:
    """The reference's CPU oracle form: dequantize the whole bank to fp32 (f16-rounded
    weights), then one fp32 product (Scripts/oracle/gen_s1_q4_fixtures.py:28-31,
    gen_mlp_fixtures.py:74-91)."""
    wq = dequant_hq_blocks_rot(blocks, bits, group, is_m5, f16_round=True)
    xf = np.asarray(x_rot_f16, dtype=np.float16).astype(np.float32)
    return (xf @ wq.T).astype(np.float32) if xf.ndim == 2 else (wq @ xf).astype(np.float32)


def normalized_error(y, y_ref) -> float:
    y = np.asarray(y, dtype=np.float64).ravel()
    r = np.asarray(y_ref, dtype=np.float64).ravel()
    d = np.linalg.norm(r)
    return float(np.linalg.norm(y - r) / d) if d > 0 else float(np.linalg.norm(y))


def rotate_activation_f16(x: np.ndarray) -> np.ndarray:
    """x (f16 / bf16-as-f32 / f32) -> FWHT-32 in fp32 -> one f16 rounding: the rotated f16
    activation the reference's producers hand to the GEMV
    (Sources/QWMetal/include/qw_dequant.metalh:424-493)."""
    return fwht32_ortho(np.asarray(x).astype(np.float32)).astype(np.float16)


def rmsnorm_rot_f16(x16: np.ndarray, gamma16: np.ndarray, eps: float, rotate: bool = True, residual16: np.ndarray | None = None):
    """qwg_rmsnorm / qwg_rmsnorm_residual (Sources/QWMetal/mlp_norm_rope/qwnorm.metal:27-79, 127-189):
    y = f16(fwht32(x * rsqrt(mean(x^2) + eps) * (1 + gamma))), gamma stored raw (plus-one law), fp32 products in the
    kernel's order ((x * rstd) * (gamma + 1)), fp32 transform in the butterfly order of fwht32_f32_inplace
    (qw_dequant.metalh:442-478, the order of `fwht32_ortho`), one f16 rounding at the end.  With `residual16` the row
    normalized is f16(f32(residual) + f32(x)), which is also returned (the kernel stores it back).
    The mean of squares is evaluated in float64 and rounded to fp32 (the kernel's fp32 summation order is not part of
    the contract).  Returns (y f16, residual_out f16 or None)."""
    x = np.asarray(x16, dtype=np.float16)
    res_out = None
    if residual16 is not None:
        x = (x.astype(np.float32) + np.asarray(residual16, dtype=np.float16).astype(np.float32)).astype(np.float16)
        res_out = x
    xf = x.astype(np.float32)
    ms = (xf.astype(np.float64) ** 2).mean(axis=-1, keepdims=True)
    rstd = (1.0 / np.sqrt(ms + np.float64(np.float32(eps)))).astype(np.float32)
    f = (xf * rstd) * (np.asarray(gamma16, dtype=np.float16).astype(np.float32) + np.float32(1.0))
    if rotate:
        f = fwht32_ortho(f)
    return f.astype(np.float16), res_out


def sortable_f32_u32(x: np.ndarray) -> np.ndarray:
    """qw_sortable_f32_u32 (Sources/QWMetal/include/qw_fastmath_safe.metalh:21-25): float bits made monotone as
    unsigned integers, NaN -> 0."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    key = np.where(u & np.uint32(0x80000000), ~u, u ^ np.uint32(0x80000000))
    return np.where((u & np.uint32(0x7FFFFFFF)) > np.uint32(0x7F800000), np.uint32(0), key).astype(np.uint32)


def head_argmax(logits: np.ndarray) -> np.ndarray:
    """The fold of the head's argmax epilogue (qwg_gemv_am_fold4 / qwg_gemv_am_reduce4,
    Sources/QWMetal/include/qw_gemm_f32_common.metalh:30-58): per row the largest (sortable(v), ~row) pair wins, so ties
    go to the lower row and NaN never beats a number."""
    keys = sortable_f32_u32(np.atleast_2d(logits)).astype(np.uint64) << np.uint64(32)
    rows = np.arange(keys.shape[-1], dtype=np.uint64)
    keys = keys | ((~rows) & np.uint64(0xFFFFFFFF))
    return (~(keys.max(axis=-1) & np.uint64(0xFFFFFFFF)) & np.uint64(0xFFFFFFFF)).astype(np.int32)


def v4_epilogue_f64(y: np.ndarray, epi: int, scale: float) -> np.ndarray:
    """The scalar epilogue of the f32 GEMV/GEMM family in float64: 0 none, 1 and 3 silu(y / scale), 2 sigmoid(y)
    (qwg_apply_v4_epi_f32, Sources/QWMetal/include/qw_gemm_f32_common.metalh:15-19; the batched body :131-132)."""
    y = np.asarray(y, dtype=np.float64)
    if epi in (1, 3):
        z = y / float(scale)
        return z / (1.0 + np.exp(-z))
    if epi == 2:
        return 1.0 / (1.0 + np.exp(-y))
    return y


def h32_groups_f64(y: np.ndarray) -> np.ndarray:
    """Normalised 32-point Walsh-Hadamard transform of every 32 consecutive outputs of each row in float64; a last partial
    group is padded with zeros, as epilogue 3 of the v4 kernel reads rows past N
    (Sources/QWMetal/include/qw_gemm_f32_common.metalh:171-196; qwg_fwht32_lane_f32, qw_weight_basis.metalh:31-38)."""
    y = np.atleast_2d(np.asarray(y, dtype=np.float64))
    rows, n = y.shape
    padded = np.zeros((rows, (n + 31) // 32 * 32))
    padded[:, :n] = y
    i = np.arange(32)
    signs = np.array([[1.0 - 2.0 * (bin(a & b).count("1") & 1) for b in i] for a in i])   # Sylvester order
    out = padded.reshape(rows, -1, 32) @ signs.T / np.sqrt(32.0)
    return out.reshape(rows, -1)[:, :n]


def gemv_f32(blocks: np.ndarray, x_f32: np.ndarray, bits: int, group: int, is_m5: bool, epi: int = 0, scale: float = 1.0) -> np.ndarray:
    """f32-activation GEMV with epilogue (QWGemm.encodeHQ4F32V4 / encodeHQ4F32BM, Sources/Operators/QWGEMM/QWGemmF32.swift:
    178-199,311-350) in float64: y = epilogue(x . W^T) over the un-rounded affine weights code * scale + bias
    (qwg_unpack_hq4_word8_f32, Sources/QWMetal/include/qw_dequant_f32.metalh:10-24), epilogue 3 adding the FWHT-32 over
    consecutive outputs.  x is already in the container's basis."""
    w = weights_affine_f64(blocks, bits, group, is_m5)
    y = v4_epilogue_f64(np.atleast_2d(np.asarray(x_f32, dtype=np.float64)) @ w.T, epi, scale)
    return h32_groups_f64(y) if epi == 3 else y


def swiglu(gate: np.ndarray, up: np.ndarray) -> np.ndarray:
    """silu(g)*u = g/(1+exp(-g))*u in fp32 (Sources/QWMetal/include/qw_weight_basis.metalh:50-63,
    plain SwiGLU branch; Scripts/oracle/gen_mlp_fixtures.py:79)."""
    g = np.asarray(gate, dtype=np.float32)
    u = np.asarray(up, dtype=np.float32)
    with np.errstate(over="ignore"):
        return (g / (np.float32(1.0) + np.exp(-g))) * u


def swiglu_fwht_f16(gate, up, rotate: bool = True) -> np.ndarray:
    """SwiGLU in fp32 then FWHT-32 in fp32 then one f16 rounding; the rotation is skipped
    when I % 32 != 0 (Sources/QWMetal/include/qw_gemm_nax_swiglu.metalh:78-80)."""
    a = swiglu(gate, up)
    if rotate and a.shape[-1] % 32 == 0:
        a = fwht32_ortho(a)
    return a.astype(np.float16)


def silu_mul_f32(gu: np.ndarray) -> np.ndarray:
    """f32 gate|up [rows, 2 I] -> FWHT32(silu(g) * u) in fp32 [rows, I]
    (qwg_silu_mul_f32, Sources/QWMetal/gemm/qwgemm_f32.metal:291-317; I % 32 == 0)."""
    gu = np.asarray(gu, dtype=np.float32)
    inter = gu.shape[-1] // 2
    return fwht32_ortho(swiglu(gu[..., :inter], gu[..., inter:]))


def moe_bridge_f16_to_f32(x16: np.ndarray):
    """The f32 bridge in front of the MoE chain (Sources/QWMetal/gemm/qwmoe_bridge_f32.metal:16-78): the f16 hidden in the
    rotated basis -> (rotated f32 copy = a widening, un-rotated f32 copy = the transform again in fp32, taken through the
    f16 hi/lo split: f32(hi) + f32(lo), hi = f16(v), lo = f16(v - f32(hi)))."""
    rot = np.asarray(x16, dtype=np.float16).astype(np.float32)
    v = fwht32_ortho(rot)
    hi = v.astype(np.float16)
    lo = (v - hi.astype(np.float32)).astype(np.float16)
    return rot, hi.astype(np.float32) + lo.astype(np.float32)


def latent_norm_h32_f32(x: np.ndarray, gamma16=None, eps: float = 1e-6) -> np.ndarray:
    """Optional RMSNorm with the plus-one law, then FWHT-32, on f32 [rows, L] -> f32
    (qwg_latent_norm_h32_f32, Sources/QWMetal/gemm/qwgemm_f32.metal:203-288): v = (x * rstd) * (1 + gamma),
    rstd = rsqrt(mean(x^2) + eps); the mean of squares in float64 rounded to fp32 (the kernel's summation order is not
    part of the contract).  No gamma: the transform alone."""
    x = np.asarray(x, dtype=np.float32)
    if gamma16 is None:
        return fwht32_ortho(x)
    ms = (x.astype(np.float64) ** 2).mean(axis=-1, keepdims=True)
    rstd = (1.0 / np.sqrt(ms + np.float64(np.float32(eps)))).astype(np.float32)
    g1 = np.float32(1.0) + np.asarray(gamma16, dtype=np.float16).astype(np.float32)
    return fwht32_ortho((x * rstd) * g1)


# --------------------------------------------------------------------------- #
# MoE router  (pinned: golden fn_sparse_moe_golden.json end to end; math: textbook softmax/top-k, tie rule)
# --------------------------------------------------------------------------- #
def router_shared_gate_f64(x: np.ndarray, sh_gate_w: np.ndarray) -> np.ndarray:
    """Shared-expert gate of the router launch: sigmoid(x[t] . w), one scalar per token row
    (Sources/QWMetal/subsystems/qwrouter.metal:566-574,633; QWGemmMoERouter.swift:69-113 shGateWeight / shGateOut)."""
    v = np.asarray(x, dtype=np.float64) @ np.asarray(sh_gate_w, dtype=np.float64).reshape(-1)
    return 1.0 / (1.0 + np.exp(-v))


def moe_route(logits: np.ndarray, top_k: int, norm_topk: bool = True, routed_scale: float = 1.0):
    """f32 softmax (max-subtracted) -> K rounds of argmax, ties to the LOWER index ->
    weights renormalised by the sum of the selected -> x routed scale.
    Returns (idx i32 [T, K], wts f32 [T, K]).  Non-finite logits are never selected; a row
    with fewer than K candidates writes idx -1 / weight 0.
    Sources/QWMetal/subsystems/qwrouter.metal:31-169;
    Tests/QWFlashNextTests/Reference/FNSparseMoE.swift:88-104."""
    lg = np.asarray(logits, dtype=np.float32)
    t, e = lg.shape
    idx = np.full((t, top_k), -1, dtype=np.int32)
    wts = np.zeros((t, top_k), dtype=np.float32)
    for r in range(t):
        row = lg[r]
        fin = np.isfinite(row)
        if not fin.any():
            continue
        mx = row[fin].max()
        ex = np.where(fin, np.exp(np.where(fin, row - mx, np.float32(0))).astype(np.float32), np.float32(0))
        total = np.float32(0)
        for v in ex:                      # sequential fp32 sum, as FNSparseMoE.route
            total = np.float32(total + v)
        if not total > 0:
            continue
        p = (ex / total).astype(np.float32)
        cand = [i for i in range(e) if fin[i]]
        order = sorted(cand, key=lambda i: (-float(p[i]), i))[:top_k]
        sel = np.array([p[i] for i in order], dtype=np.float32)
        if norm_topk:
            acc = np.float32(0)
            for v in sel:
                acc = np.float32(acc + v)
            sel = (sel / acc).astype(np.float32) if acc > 0 else np.zeros_like(sel)
        sel = (sel * np.float32(routed_scale)).astype(np.float32)
        idx[r, :len(order)] = order
        wts[r, :len(order)] = sel
    return idx, wts


def moe_route_ex(logits: np.ndarray, top_k: int, norm_topk: bool = True, routed_scale: float = 1.0, bias=None,
                 split_feature: bool = False, scale_param=None):
    """The router's other modes (Sources/QWMetal/subsystems/qwrouter.metal:44-46,63-82,113-159): with a selection bias and / or
    split-feature logits [T, 2E] the score is sigmoid(l) (+ sigmoid(l')) in fp32, experts are chosen by score + bias (K rounds
    of argmax, ties to the lower index; non-finite logits or scores never win) and weighted by the score alone, renormalised
    by the fp32 sum of the selected (rank order) + 1e-20; a per-expert scale replaces the routed scale.  Without bias and
    split features it is moe_route (softmax) with the per-expert scale."""
    lg = np.asarray(logits, dtype=np.float32)
    if bias is None and not split_feature:
        idx, wts = moe_route(lg, top_k, norm_topk, 1.0)
    else:
        t = lg.shape[0]
        e = lg.shape[1] // 2 if split_feature else lg.shape[1]
        idx = np.full((t, top_k), -1, dtype=np.int32)
        wts = np.zeros((t, top_k), dtype=np.float32)
        one = np.float32(1.0)
        with np.errstate(over="ignore", invalid="ignore"):
            for r in range(t):
                l0 = lg[r, :e]
                sc = one / (one + np.exp(-l0).astype(np.float32))
                ok = np.isfinite(l0)
                if split_feature:
                    l1 = lg[r, e:2 * e]
                    sc = (sc + one / (one + np.exp(-l1).astype(np.float32))).astype(np.float32)
                    ok &= np.isfinite(l1)
                score = (sc + np.asarray(bias, dtype=np.float32)).astype(np.float32) if bias is not None else sc
                ok &= np.isfinite(sc) & np.isfinite(score)
                order = sorted([i for i in range(e) if ok[i]], key=lambda i: (-float(score[i]), i))[:top_k]
                sel = np.array([sc[i] for i in order], dtype=np.float32)
                if norm_topk:
                    acc = np.float32(0)
                    for v in sel:
                        acc = np.float32(acc + v)
                    acc = np.float32(acc + np.float32(1e-20))
                    sel = (sel / acc).astype(np.float32) if acc > 0 else np.zeros_like(sel)
                idx[r, :len(order)] = order
                wts[r, :len(order)] = sel
    if scale_param is not None:
        sp = np.asarray(scale_param, dtype=np.float32)
        scale = np.where(idx >= 0, sp[np.maximum(idx, 0)], np.float32(1.0)).astype(np.float32)
    else:
        scale = np.float32(routed_scale if routed_scale > 0 else 1.0)
    return idx, (wts * scale).astype(np.float32)


# --------------------------------------------------------------------------- #
# expert-major pair sort and tile list  (pinned: math - permutation invariants, closed-form tile counts)
# --------------------------------------------------------------------------- #
def moe_max_tiles(experts: int, pairs: int) -> int:
    """Sources/Operators/QWGEMM/QWGemmMoE.swift:24-26."""
    return min(pairs, min(experts, pairs) + (pairs + 63) // 64)


def moe_tile_block(c: int) -> int:
    """Sources/QWMetal/include/qw_moe_tile.metalh:7-10."""
    return 16 if c <= 16 else (32 if c <= 32 else 64)


def moe_pack_tile_r(tid_y: int, bm: int) -> int:
    """qw_moe_tile.metalh:13-16."""
    code = 1 if bm == 16 else (2 if bm == 32 else 3)
    return (code << 24) | (tid_y & 0xFFFFFF)


def moe_group_pairs(ids: np.ndarray, experts: int, top_k: int, compact_tail: bool = True):
    """Counting sort of (token, route) pairs by expert id, stable in pair order.

    Returns dict(expertOff i32[E+1], sortedPairIdx, sortedTok, invPerm, tileE, tileR, tileCount).
    Pairs whose id is negative or >= experts are skipped (their invPerm stays -1).  The
    reference's slot order inside an expert is arbitrary (atomic cursor); stable order is
    one valid instance.  Sources/QWMetal/gemm/qwgemm_moe_group_f32.metal:10-148."""
    flat = np.asarray(ids, dtype=np.int32).ravel()
    p = flat.size
    e_of = np.where(flat >= 0, flat & 0xFFFF, -1)
    valid = (e_of >= 0) & (e_of < experts)
    counts = np.bincount(e_of[valid], minlength=experts).astype(np.int32)
    off = np.zeros(experts + 1, dtype=np.int32)
    off[1:] = np.cumsum(counts)
    order = np.argsort(np.where(valid, e_of, experts), kind="stable")[: int(valid.sum())].astype(np.int32)
    sorted_tok = (order // top_k).astype(np.int32)
    inv = np.full(p, -1, dtype=np.int32)
    inv[order] = np.arange(order.size, dtype=np.int32)
    tile_e, tile_r = [], []
    for e in range(experts):
        c = int(counts[e])
        if c <= 0:
            continue
        if compact_tail:
            q, rem = c >> 6, c & 63
            for r in range(q):
                tile_e.append(e)
                tile_r.append(moe_pack_tile_r(r, 64))
            if rem > 0:
                bm = moe_tile_block(rem)
                tile_e.append(e)
                tile_r.append(moe_pack_tile_r((q * 64) // bm, bm))
        else:
            bm = moe_tile_block(c)
            r = 0
            while r * bm < c:
                tile_e.append(e)
                tile_r.append(moe_pack_tile_r(r, bm))
                r += 1
    return dict(expertOff=off, sortedPairIdx=order, sortedTok=sorted_tok, invPerm=inv,
                tileE=np.array(tile_e, dtype=np.int32), tileR=np.array(tile_r, dtype=np.int32),
                tileCount=len(tile_e))


# --------------------------------------------------------------------------- #
# routed MoE block  (pinned: golden fn_sparse_moe_golden.json with fp32 weights; math for the quantized form)
# --------------------------------------------------------------------------- #
def moe_forward_f64(x, idx, wts, gate_up_w, down_w, act_f16: bool, rotate_act: bool):
    """out[t] = sum_k wts[t,k] * W_down[e_k] . act_k,  act_k = SwiGLU(W_gu[e_k] . x[t]).

    gate_up_w [E, 2I, H], down_w [E, H, I] are the (already dequantized) weights in the
    basis the activations are given in; rows [0, I) = gate, [I, 2I) = up
    (Tests/QWFlashNextTests/Reference/FNSparseMoE.swift:7-8,106-160;
    Tests/QWGEMMTests/QWMoEReuseTests.swift:89-127).  With act_f16 the SwiGLU result is
    rounded to f16 (optionally FWHT-rotated first) before the down projection, as the
    kernels store it.  All products in fp64."""
    x = np.asarray(x, dtype=np.float64)
    t, h = x.shape
    e, two_i, _ = gate_up_w.shape
    i = two_i // 2
    out = np.zeros((t, down_w.shape[1]), dtype=np.float64)
    for r in range(t):
        for k in range(idx.shape[1]):
            ex = int(idx[r, k])
            if ex < 0:
                continue
            ex &= 0xFFFF
            gu = gate_up_w[ex].astype(np.float64) @ x[r]
            g, u = gu[:i], gu[i:]
            act = g / (1.0 + np.exp(-g)) * u
            if act_f16:
                a32 = act.astype(np.float32)
                if rotate_act and i % 32 == 0:
                    a32 = fwht32_ortho(a32)
                act = a32.astype(np.float16).astype(np.float64)
            out[r] += float(wts[r, k]) * (down_w[ex].astype(np.float64) @ act)
    return out


def moe_forward_grouped_f64(x, idx, wts, gate_up_w, down_w, act_f16: bool, rotate_act: bool):
    """moe_forward_f64 with the work ordered by expert instead of by token: the rows routed to expert e are gathered,
    contracted with that expert's gate|up and down weights as two fp64 matrix products, and scattered back weighted.
    Same sums per (token, route) as moe_forward_f64 up to fp64 summation order (pinned against it in
    tests/test_oracle_math.py); it exists so that a whole prefill batch (thousands of tokens, every expert) can be
    checked in seconds.  gate_up_w / down_w: anything indexable by expert that returns [2I, H] / [H, I] weights
    (Tests/QWFlashNextTests/Reference/FNSparseMoE.swift:106-160 is the per-token form)."""
    x = np.asarray(x, dtype=np.float64)
    idx = np.asarray(idx)
    t = x.shape[0]
    ids = np.where(idx < 0, -1, idx & 0xFFFF)
    out = None
    for ex in np.unique(ids[ids >= 0]):
        rows, slots = np.nonzero(ids == ex)
        gu_w = np.asarray(gate_up_w[int(ex)], dtype=np.float64)
        dn_w = np.asarray(down_w[int(ex)], dtype=np.float64)
        i = gu_w.shape[0] // 2
        gu = x[rows] @ gu_w.T
        g, u = gu[:, :i], gu[:, i:]
        act = g / (1.0 + np.exp(-g)) * u
        if act_f16:
            a32 = act.astype(np.float32)
            if rotate_act and i % 32 == 0:
                a32 = fwht32_ortho(a32)
            act = a32.astype(np.float16).astype(np.float64)
        part = (act @ dn_w.T) * np.asarray(wts, dtype=np.float64)[rows, slots][:, None]
        if out is None:
            out = np.zeros((t, dn_w.shape[0]), dtype=np.float64)
        np.add.at(out, rows, part)
    if out is None:
        out = np.zeros((t, np.asarray(down_w[0]).shape[0]), dtype=np.float64)
    return out


# --------------------------------------------------------------------------- #
# group-latent routed MoE block  (no golden in the reference: pinned by the identities of tests/test_oracle_math.py -
# one identity group reduces it to moe_forward_f64, and the per-route expansion by linearity of U_g)
# --------------------------------------------------------------------------- #
def moe_latent_groups(idx: np.ndarray, labels: np.ndarray, num_groups: int):
    """group_ids [t, NG] = g where a route of the token carries label g, else -1; pair_rows [t, k] = t * NG + label of
    the route, -1 for an absent route (activeMask / groupIds, Sources/QWMetal/subsystems/qwrouter.metal:135-165)."""
    idx = np.asarray(idx)
    t, k = idx.shape
    gids = np.full((t, num_groups), -1, dtype=np.int32)
    rows = np.full((t, k), -1, dtype=np.int32)
    for r in range(t):
        for j in range(k):
            e = int(idx[r, j])
            if e < 0:
                continue
            g = int(labels[e & 0xFFFF])
            if 0 <= g < num_groups:
                gids[r, g] = g
                rows[r, j] = r * num_groups + g
    return gids, rows


def moe_group_latent_forward_f64(x, idx, wts, labels, latent_d_w, gate_up_w, down_w, latent_u_w, act_f16: bool = True,
                                 rotate_act: bool = True, latent_f16: bool = True):
    """out[t] = sum over active groups g of U_g . z_g,  z_g = sum over the token's routes k with labels[e_k] == g of
    wts[t, k] * W_down[e_k] . SwiGLU(W_gu[e_k] . (D_g . x[t]))
    (FNSparseMoE.forward, Tests/QWFlashNextTests/Reference/FNSparseMoE.swift:113-139).

    latent_d_w [NG, L, H], gate_up_w [E, 2I, L], down_w [E, L, I], latent_u_w [NG, H, L]: dequantized weights in the
    basis the kernels contract them in.  latent_f16 rounds D_g . x and z_g to f16, as the kernels hand them on; act_f16 /
    rotate_act as in moe_forward_f64.  All products in fp64."""
    x = np.asarray(x, dtype=np.float64)
    t = x.shape[0]
    ng, lat, _ = latent_d_w.shape
    i = gate_up_w.shape[1] // 2
    out = np.zeros((t, latent_u_w.shape[1]), dtype=np.float64)
    r16 = (lambda v: v.astype(np.float32).astype(np.float16).astype(np.float64)) if latent_f16 else (lambda v: v)
    for r in range(t):
        z = np.zeros((ng, lat), dtype=np.float64)
        xin = {}
        for k in range(idx.shape[1]):
            e = int(idx[r, k])
            if e < 0:
                continue
            e &= 0xFFFF
            g = int(labels[e])
            if g not in xin:
                xin[g] = r16(latent_d_w[g].astype(np.float64) @ x[r])
            gu = gate_up_w[e].astype(np.float64) @ xin[g]
            gt, up = gu[:i], gu[i:]
            act = gt / (1.0 + np.exp(-gt)) * up
            if act_f16:
                a32 = act.astype(np.float32)
                if rotate_act and i % 32 == 0:
                    a32 = fwht32_ortho(a32)
                act = a32.astype(np.float16).astype(np.float64)
            z[g] += float(wts[r, k]) * (down_w[e].astype(np.float64) @ act)
        for g in xin:
            out[r] += latent_u_w[g].astype(np.float64) @ r16(z[g])
    return out


# --------------------------------------------------------------------------- #
# generalized gated FFN activation  (pinned by limits: tests/test_oracle_math.py)
# --------------------------------------------------------------------------- #
def gated_act(gate, up, kind: int = 0, p0: float = 0.0, p1: float = 0.0) -> np.ndarray:
    """qwg_swiglu_mul (Sources/QWMetal/include/qw_weight_basis.metalh:48-66) in fp64: kind 0 silu(g) * u; kind 1 the same
    with g <= p0 and |u| <= p0 (QW_FC_SWIGLU_LIMIT); kind 2 p0 tanh(g / p0) sigmoid(g) * p1 tanh(u / p1), u as it is when
    p1 <= 0 (QW_FC_SITU_BETA / QW_FC_SITU_LIN_BETA; the reference's own restatement: situRef,
    Tests/QWGEMMTests/QWErnie55MoETests.swift:120-125)."""
    g = np.asarray(gate, dtype=np.float64)
    u = np.asarray(up, dtype=np.float64)
    if kind == 2:
        gg = p0 * np.tanh(g / p0) / (1.0 + np.exp(-g))
        uu = p1 * np.tanh(u / p1) if p1 > 0 else u
        return gg * uu
    if kind == 1:
        g = np.minimum(g, p0)
        u = np.clip(u, -p0, p0)
    return g / (1.0 + np.exp(-g)) * u


def moe_route_budget(idx: np.ndarray, wts: np.ndarray, budget: int, norm_topk: bool = True):
    """Expert budget over a verify window of 2..4 routed rows (the `normTopK & 4` branch of qwg_moe_route_decode,
    Sources/QWMetal/subsystems/qwrouter.metal:193-268): row 0 keeps its routes, the other pairs are admitted expert by expert
    in the order of their weights (ties to the lower pair index) until max(top_k, budget) distinct experts are in, the rest
    get idx -1 and weight 0; with norm_topk a later row that lost weight is rescaled to its former sum (fp32)."""
    idx = np.array(idx, dtype=np.int32)
    wts = np.array(wts, dtype=np.float32)
    m, k = idx.shape
    total = m * k
    if budget <= 0 or budget >= total:
        return idx, wts
    b = max(k, budget)
    ids, w = idx.ravel().copy(), wts.ravel().copy()
    orig = [np.float32(0)] * m
    for r in range(m):
        s = np.float32(0)
        for j in range(k):
            s = np.float32(s + w[r * k + j])
        orig[r] = s
    keep = [p < k for p in range(total)]
    unique = 0
    for s in range(k):
        e = int(ids[s])
        if e < 0 or any(int(ids[p]) == e for p in range(s)):
            continue
        unique += 1
        for p in range(total):
            if int(ids[p]) == e:
                keep[p] = True
    while unique < b:
        cand = [float(w[p]) if (not keep[p] and ids[p] >= 0) else -1.0 for p in range(total)]
        best = max(cand)
        if best < 0:
            break
        win = cand.index(best)
        for p in range(total):
            if ids[p] == ids[win]:
                keep[p] = True
        unique += 1
    out_i, out_w = ids.copy(), w.copy()
    for p in range(total):
        if not keep[p]:
            out_i[p], out_w[p] = -1, np.float32(0)
    if norm_topk:
        for r in range(1, m):
            now = np.float32(0)
            for j in range(k):
                if out_w[r * k + j] > 0:
                    now = np.float32(now + out_w[r * k + j])
            if now > 0 and now < np.float32(orig[r] * np.float32(0.9999)):
                scale = np.float32(orig[r] / now)
                for j in range(k):
                    out_w[r * k + j] = np.float32(out_w[r * k + j] * scale)
    return out_i.reshape(m, k), out_w.reshape(m, k)


# --------------------------------------------------------------------------- #
# consumers of the head and the dense fp32 GEMV  (pinned by closed forms: tests/test_oracle_math.py)
# --------------------------------------------------------------------------- #
def head_argmax_variational(logits: np.ndarray, draft_tokens, margin: float, min_log_prob: float = -np.inf) -> np.ndarray:
    """Relaxed acceptance of a draft over a verify window (qwg_head_argmax_fin_variational,
    Sources/QWMetal/head_sampling/qwhead.metal:271-345): row r takes draft_tokens[r + 1] instead of its argmax when the draft is in
    the vocabulary, is not the argmax, logit(draft) >= max - margin and - for a finite min_log_prob - its log-probability
    (logit - max - log sum exp(logits - max)) reaches min_log_prob."""
    lg = np.asarray(logits, dtype=np.float32)
    rows, vocab = lg.shape
    out = head_argmax(lg).astype(np.int64)
    draft = np.asarray(draft_tokens, dtype=np.int64)
    if not margin > 0:
        return out
    for r in range(rows):
        if r + 1 >= len(draft):
            continue
        d = int(draft[r + 1])
        if not (0 <= d < vocab) or d == out[r]:
            continue
        mx = np.float64(lg[r, out[r]])
        dl = np.float64(lg[r, d])
        if not dl >= mx - np.float64(np.float32(margin)):
            continue
        if np.isfinite(min_log_prob):
            finite = lg[r][np.isfinite(lg[r]) | (lg[r] == -np.inf)].astype(np.float64)
            lp = (dl - mx) - np.log(np.sum(np.exp(finite - mx)))
            if lp >= min_log_prob:
                out[r] = d
        else:
            out[r] = d
    return out


def f32_gemv(w: np.ndarray, x: np.ndarray, epi: int = 0, scale: float = 1.0) -> np.ndarray:
    """Dense fp32-weight GEMV with its scalar epilogues in fp64 (qwg_f32_gemv, Sources/QWMetal/gemm/qwgemm_f32.metal:120-143):
    0 none, 1 silu(y / scale), 2 sigmoid(y), 3 2 sigmoid(y / scale)."""
    y = np.asarray(x, dtype=np.float64) @ np.asarray(w, dtype=np.float64).T
    if epi == 1:
        z = y / scale
        return z / (1.0 + np.exp(-z))
    if epi == 2:
        return 1.0 / (1.0 + np.exp(-y))
    if epi == 3:
        return 2.0 / (1.0 + np.exp(-(y / scale)))
    return y
