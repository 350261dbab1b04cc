#!/usr/bin/env python3
"""Writes tests/golden/hq_blocks_golden.npz: seeded inputs and the exact block
bytes the reference's block quantizer (`Scripts/quantize/hq_blocks.py:436-517`,
`quant_hq_blocks`) produces for them, for every (bits, group, rotate) case the
matmul path consumes.  No committed byte-level golden exists in the reference for
the non-M5 block pairs, so these vectors are made by importing the reference's
quantizer once, in the build container only; the reference source itself is not
copied.  Run:  python3 tests/golden/gen_hq_blocks_golden.py /root/reference
"""
import pathlib
import sys

import numpy as np


def main(ref_root: str) -> None:
    sys.path.insert(0, str(pathlib.Path(ref_root) / "Scripts" / "quantize"))
    import hq_blocks  # the reference quantizer (imported, never copied)

    rng = np.random.default_rng(20261125)
    out = {}
    cases = [
        # name, bits, group, is_m5, rotate
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
    n, k = 12, 512
    w = (rng.standard_normal((n, k)) * 0.02).astype(np.float32)
    # a few hard rows: an outlier, a constant group (scale 0), tiny values, ties
    w[1, 5] = 0.9
    w[2, 64:128] = 0.0125
    w[3] *= 1e-6
    w[4, :32] = np.arange(32, dtype=np.float32) / 64.0
    w[5, :64] = 0.0
    out["w"] = w
    for name, bits, group, is_m5, rotate in cases:
        blocks, eff = hq_blocks.quant_hq_blocks(w, bits=bits, group=group, is_m5=is_m5, rotate=rotate)
        assert eff == group
        out[f"{name}__blocks"] = np.ascontiguousarray(blocks)
        out[f"{name}__deq_rot"] = hq_blocks.dequant_hq_blocks_rot(blocks, bits=bits, group=group, is_m5=is_m5)
        out[f"{name}__deq_rot_f16"] = hq_blocks.dequant_hq_blocks_rot(
            blocks, bits=bits, group=group, is_m5=is_m5, f16_round=True)
    qs, sc = hq_blocks.quant_hq8_g32_m5(w)
    out["hq8_planar__qs"] = qs
    out["hq8_planar__scales"] = sc.view(np.uint16)
    out["fwht__in"] = w[:2]
    out["fwht__out"] = hq_blocks._fwht32_torch(__import__("torch").from_numpy(w[:2].copy())).numpy()
    path = pathlib.Path(__file__).resolve().parent / "hq_blocks_golden.npz"
    np.savez_compressed(path, **out)
    print("wrote", path, path.stat().st_size, "bytes")


if __name__ == "__main__":
    main(sys.argv[1] if len(sys.argv) > 1 else "/root/reference")
