"""Seeded synthetic inputs shared by the GPU parity tests, the smoke check and the benchmark."""
from __future__ import annotations

import numpy as np

from oracle import qworacle as qo
from qwegn_amd import qwhip

FORMATS = {
    # name: (kind, bits, group, is_m5, rotate)
    "hq4_g32_m5": (qwhip.KIND_HQ4_G32_M5, 4, 32, True, True),
    "aq4_g32": (qwhip.KIND_NATIVE_AFFINE, 4, 32, False, False),
    "hq4_g32": (qwhip.KIND_ROTATED_HQ, 4, 32, False, True),
    "hq4_g64": (qwhip.KIND_ROTATED_HQ, 4, 64, False, True),
    "hq4_g128": (qwhip.KIND_ROTATED_HQ, 4, 128, False, True),
    "hq8_g32": (qwhip.KIND_ROTATED_HQ, 8, 32, False, True),
    "hq8_g64": (qwhip.KIND_ROTATED_HQ, 8, 64, False, True),
    "aq8_g256": (qwhip.KIND_NATIVE_AFFINE, 8, 256, False, False),
    # 2-, 3- and 6-bit streams
    "aq2_g64": (qwhip.KIND_NATIVE_AFFINE, 2, 64, False, False),
    "hq3_g32": (qwhip.KIND_ROTATED_HQ, 3, 32, False, True),
    "hq6_g32": (qwhip.KIND_ROTATED_HQ, 6, 32, False, True),
    "aq6_g128": (qwhip.KIND_NATIVE_AFFINE, 6, 128, False, False),
}


def make_weights(n: int, k: int, seed: int, std: float = 0.02) -> np.ndarray:
    rng = np.random.default_rng(seed)
    return (rng.standard_normal((n, k), dtype=np.float32) * np.float32(std)).astype(np.float32)


def make_bank(fmt: str, n: int, k: int, seed: int):
    """Quantizes seeded N(0, 0.02) weights with the oracle's restatement of the reference quantizer.
    Returns (blocks u8 [n, k/g, bb], w_f16 [n, k] exact f16 weights in the container's basis)."""
    kind, bits, group, is_m5, rotate = FORMATS[fmt]
    w = make_weights(n, k, seed)
    blocks, eff = qo.quant_hq_blocks(w, bits=bits, group=group, is_m5=is_m5, rotate=rotate)
    assert eff == group
    return blocks, qo.weights_f16_exact(blocks, bits, group, is_m5)


def make_x(m: int, k: int, seed: int, outliers: bool = False) -> np.ndarray:
    """f32 N(0,1) activations; with `outliers`, 0.1 % of the entries are scaled by 20."""
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((m, k), dtype=np.float32)
    if outliers:
        mask = rng.random((m, k)) < 0.001
        x = np.where(mask, x * np.float32(20.0), x).astype(np.float32)
    return x


def x_in_basis(x16: np.ndarray, fmt: str) -> np.ndarray:
    """The f16 activations the kernel contracts: rotated per 32-group for a rotated container."""
    rotate = FORMATS[fmt][4]
    return qo.rotate_activation_f16(x16) if rotate else np.asarray(x16, dtype=np.float16)


def view_of(dev, buf, fmt: str, n: int, k: int):
    kind, bits, group, _, _ = FORMATS[fmt]
    return dev.view(buf, n, k, kind, bits, group)
