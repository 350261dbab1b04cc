"""The Swift shim's doors carry the reference's argument labels.

tests/golden/swift_door_labels.json holds the labels of every static function of QWGemm, QWGemmAQ and QWMoEOperator in the
reference (Sources/Operators/QWGEMM/*.swift; written by tests/golden/swift_door_labels.py).  A call site of the reference
compiles against the shim when a shim overload of the same name has the reference's labels in the reference's order
(defaulted extras may sit between or behind them).  The doors for which that does not hold are listed here with the
reason; the integration notes carry the same list.
"""
import importlib.util
import json
from pathlib import Path

ROOT = Path(__file__).resolve().parent.parent
SHIM = ROOT / "qwegn_amd" / "swift" / "QWHipHAL" / "QWHipHAL.swift"

# reference doors the shim does not carry
ABSENT = {
    "QWGemm.blockArgmaxSlots": "key scratch of the two-stage argmax; the head's fold needs none here",
    "QWGemm.configureDenseNax": "sampling state of the Metal tensor path",
    "QWGemm.dispatchTileChunks": "indirect dispatch helper of the Metal grouped GEMM",
    "QWGemm.encodeEmbedBf16F32": "bf16 embedding table: served by the C ABI and the C++ host layer only",
    "QWGemm.encodeHQ4F32BM": "folded into encodeHQ4F32V4 (the library picks the batched form from 32 rows on)",
    "QWGemm.encodeHQ4F32V4Argmax": "QWGemmAQ.encodeHeadArgmax with f32 rows",
    "QWGemm.encodeMoEGateUpNax": "encodeMoEGroupedGemm / encodeMoEGateUpSwiglu (the tile plan is not a parameter here)",
    "QWGemm.encodeMoENaxSplitF32": "encodeMoEGroupedGemm on f16 rows (no hi / lo planes)",
    "QWGemm.encodeMoESpanIds": "tiered expert residency (cold banks) is outside this library",
    "QWGemm.encodeNaxF32": "gemmBatchedH16 with an f32 output",
    "QWGemm.encodeSiluMulSplitF16": "hi / lo halves are never needed; encodeSiluMulF16 stores one f16 matrix",
    "QWGemm.moeSliceCount": "tile slicing of the Metal grouped GEMM",
    "QWGemm.naxRowChunk": "row chunking of the Metal tensor GEMM",
    "QWGemmAQ.gdnInProjDecodeKernelName": "GDN in-projection kernels are outside the path",
    "QWGemmAQ.gdnInProjPrefillKernelName": "GDN in-projection kernels are outside the path",
    "QWGemmAQ.hcDownInjectF32KernelName": "hyper-connection kernels are outside the path",
    "QWGemmAQ.hcNormDownInjectF32KernelName": "hyper-connection kernels are outside the path",
    "QWGemmAQ.hcUpMixH32F32KernelName": "hyper-connection kernels are outside the path",
    "QWMoEOperator.canUseNaxDenseProj": "routing rule of the Metal tensor path; encodeDenseProjF32 decides by itself",
    "QWMoEOperator.groupedNaxMinRows": "row threshold of the Metal grouped path; the grouped path starts above 8 rows here",
}
# doors the shim carries under the same name with other labels
DELTAS = {
    "QWGemm.encodeArgmaxFin": "keysHi / keysLo / slots -> logits / vocab: the fold reads the f32 logits, there is no key scratch",
    "QWGemmAQ.encodeHeadArgmax": "y / keysHi / keysLo / writeLogits -> logits / tokens / rows: logits are always kept, tokens "
                                 "are written by the same launch",
    "QWGemm.encodeMoEGroupPairsF32": "tilePlan / directSlotTok -> compactTail: the tile shape is the library's own",
    "QWGemm.encodeMoEGateUpF32R1": "tileFilter dropped (no cold-bank tiles)",
    "QWGemm.encodeMoEDownSharedCombineF32": "tileFilter dropped (no cold-bank tiles)",
}


def _load():
    spec = importlib.util.spec_from_file_location("swift_door_labels", ROOT / "tests" / "golden" / "swift_door_labels.py")
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    ref = json.loads((ROOT / "tests" / "golden" / "swift_door_labels.json").read_text())
    return ref, mod.swift_doors(SHIM.read_text())


def _in_order(want, have):
    it = iter(have)
    return all(label in it for label in want)


def test_every_reference_door_is_carried_or_listed():
    ref, shim = _load()
    assert len(ref) >= 60
    for name in ref:
        assert (name in shim) != (name in ABSENT), name
    assert set(ABSENT) <= set(ref) and set(DELTAS) <= set(ref)


def test_carried_doors_take_the_reference_labels_in_order():
    ref, shim = _load()
    checked = 0
    for name, overloads in ref.items():
        if name in ABSENT:
            continue
        for labels in overloads:
            fits = any(_in_order(labels, mine) for mine in shim[name])
            assert fits != (name in DELTAS), (name, labels, shim[name])
            checked += 1
    assert checked >= 40


def test_the_three_operator_doors_match_label_for_label():
    """QWGemm.encodeH16, QWGemmAQ.encode and QWMoEOperator.encodeResident: the reference's labels are a prefix-preserving
    subsequence, and what the shim adds comes after the last of them or is one of the rotation switches."""
    ref, shim = _load()
    for name, extras in (("QWGemm.encodeH16", {"rows", "xIsRotated"}), ("QWGemm.encode", {"rows", "xIsRotated", "siluPairPlainOut"}),
                         ("QWGemmAQ.encode", {"isRotated", "xIsRotated"}), ("QWMoEOperator.encodeResident", set()),
                         ("QWMoEOperator.encodeResidentLatent", set()), ("QWMoEOperator.encodeResidentGroupLatent", set())):
        want = ref[name][0]
        best = [mine for mine in shim[name] if _in_order(want, mine)]
        assert best, name
        assert any(set(mine) - set(want) <= extras for mine in best), (name, best)
