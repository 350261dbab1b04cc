"""QWP1 pack reader: the two packs the reference's own tests hold, synthetic packs in the writer's layout
(Scripts/quantize/pack.py:115-316: magic, u64 LE trailer length, 256-byte aligned raw planes, 16 KiB aligned quant
planes, JSON trailer at EOF), and the reader's error cases.  No GPU."""
import json

import numpy as np
import pytest

from oracle import qworacle as qo
from qwegn_amd import pack as qp


def write_pack(path, tensors: dict, provenance=None):
    """tensors: name -> (entry dict without offsets, plane bytes, offset key).  Returns the entries written."""
    body = bytearray(b"QWP1" + b"\0" * 8)
    entries = {}
    for name, (entry, plane, key) in tensors.items():
        align = 256 if key == "raw_off" else 16384
        body += b"\0" * ((-len(body)) % align)
        entries[name] = dict(entry, **{key: len(body)})
        body += bytes(plane)
    trailer = json.dumps({"provenance": provenance or {"source": "test"}, "tensors": entries}).encode()
    body[4:12] = len(trailer).to_bytes(8, "little")
    path.write_bytes(bytes(body) + trailer)
    return entries


def test_reads_the_reference_packs(golden_dir):
    p = qp.Pack(golden_dir / "selfpack.qwp")
    assert set(p.tensors) == {"norm_test", "w_test"} and p.provenance["source"] == "selfpack"
    e = p.entry("w_test")
    assert e.shape == (256, 1024) and e.quantized and e.is_incumbent_hq4 and e.hq_block_bytes == 20
    layout, plane = p.plane("w_test")
    assert layout == qp.PlaneLayout.HQ4 and plane.nbytes == 256 * 32 * 20 and e.hq4_off == 16384
    blocks = np.asarray(plane).reshape(256, 32, 20)
    want = np.load(golden_dir / "selfpack.qwp.dq4.npy")
    assert np.array_equal(qo.dequant_hq4(blocks).view(np.uint32), want.view(np.uint32))     # the plane is the golden's
    layout, raw = p.plane("norm_test")
    assert layout == qp.PlaneLayout.RAW and raw.nbytes == 512 and p.entry("norm_test").raw_off == 256
    assert p.weight_geometry("w_test") == (256, 1024, qp.qwhip.KIND_HQ4_G32_M5, 4, 32)
    # planar HQ8 entries have no verbatim plane layout (PlaneLayout.resolve returns nil for them)
    p8 = qp.Pack(golden_dir / "selfpack_hq8.qwp")
    e8 = p8.entry("w_test8")
    assert e8.hq8_quantized and not e8.quantized and qp.PlaneLayout.resolve(e8) is None
    # the planar reader hands out the two planes; their host dequant is the reference's stored answer (<= 1e-6)
    name8 = next(nm for nm, e in p8.tensors.items() if e.hq8_quantized)
    qs, sc = p8.hq8_planes(name8)
    assert qs.dtype == np.int8 and sc.dtype == np.float16 and qs.shape == tuple(e8.shape) and sc.shape == (e8.shape[0], e8.shape[1] // 32)
    want = np.frombuffer((golden_dir / "selfpack_hq8.qwp.dq8rot.f32.bin").read_bytes(), dtype=np.float32).reshape(qs.shape)
    assert np.max(np.abs(qo.dequant_hq8_planar_rot(np.asarray(qs), np.asarray(sc)) - want)) <= 1e-6
    with pytest.raises(qp.QWQuantError) as err:
        p8.plane("w_test8")
    assert err.value.case == "badPlane"


def test_expert_stacks_and_block_families(tmp_path):
    rng = np.random.default_rng(0)
    experts, n, k = 3, 8, 128
    w = (rng.standard_normal((experts * n, k)) * 0.02).astype(np.float32)
    hq4 = qo.quant_hq4_blocks(w)
    blk, _ = qo.quant_hq_blocks(w[:n], bits=8, group=64, is_m5=False, rotate=True)
    ents = write_pack(tmp_path / "t.qwp", {
        "experts.gate_up": ({"shape": [experts, n, k], "experts": experts, "e_hq4": n * (k // 32) * 20}, hq4.tobytes(), "hq4_off"),
        "proj": ({"shape": [n, k], "hq": {"bits": 8, "group": 64}}, blk.tobytes(), "hq4_off"),
        "bias": ({"shape": [k], "kind": "f32"}, np.arange(k, dtype=np.float32).tobytes(), "raw_off"),
    })
    assert ents["experts.gate_up"]["hq4_off"] % 16384 == 0 and ents["bias"]["raw_off"] % 256 == 0
    p = qp.Pack(tmp_path / "t.qwp")
    layout, plane = p.plane("experts.gate_up")
    assert plane.nbytes == experts * n * 4 * 20 and np.array_equal(np.asarray(plane), hq4.ravel().view(np.uint8))
    assert p.weight_geometry("experts.gate_up") == (experts * n, k, qp.qwhip.KIND_HQ4_G32_M5, 4, 32)
    assert p.weight_geometry("proj") == (n, k, qp.qwhip.KIND_ROTATED_HQ, 8, 64)
    assert p.plane("proj")[1].nbytes == n * 2 * 68 and p.plane("bias")[1].nbytes == 4 * k
    assert qp.PlaneLayout.byte_count("hq4", qp.QWQTensorEntry((4, 96), hq4_off=0, hq=qp.QWHQFormat(4, 64))) is None   # 96 % 64
    assert qp.PlaneLayout.byte_count("hq4", qp.QWQTensorEntry((4, 64), hq4_off=0, hq=qp.QWHQFormat(5, 64))) is None   # 5 bits
    assert qp.PlaneLayout.byte_count("hq4", qp.QWQTensorEntry((4, 64), hq4_off=0, hq=qp.QWHQFormat(4, 32, "shvq1"))) is None


def test_reader_error_cases(tmp_path):
    def case(data):
        f = tmp_path / "bad.qwp"
        f.write_bytes(data)
        with pytest.raises(qp.QWQuantError) as err:
            qp.Pack(f)
        return err.value.case

    with pytest.raises(qp.QWQuantError) as err:
        qp.Pack(tmp_path / "missing.qwp")
    assert err.value.case == "modelFileMissing"
    assert case(b"QWP1" + b"\0" * 8) == "truncated"                                   # nothing after the header
    assert case(b"QWPX" + (2).to_bytes(8, "little") + b"{}") == "badMagic"
    assert case(b"QWP1" + (999).to_bytes(8, "little") + b"{}") == "truncated"          # trailer longer than the file
    assert case(b"QWP1" + (2).to_bytes(8, "little") + b"{}") == "badHeader"            # no provenance / tensors
    write_pack(tmp_path / "short.qwp", {"w": ({"shape": [4, 64]}, b"\0" * 10, "hq4_off")})   # plane shorter than its shape
    p = qp.Pack(tmp_path / "short.qwp")
    with pytest.raises(qp.QWQuantError) as err:
        p.plane("w")
    assert err.value.case == "badPlane"
    with pytest.raises(qp.QWQuantError) as err:
        p.entry("nope")
    assert err.value.case == "unknownTensor"


def test_writer_reproduces_the_reference_packs_byte_for_byte(golden_dir, tmp_path):
    """PackWriter given the reference packs' own planes and provenance writes the same files: header, plane offsets and padding,
    the trailer's text (Scripts/quantize/pack.py:115-316 wrote tests/golden/selfpack.qwp and selfpack_hq8.qwp)."""
    src = qp.Pack(golden_dir / "selfpack.qwp")
    with qp.PackWriter(tmp_path / "again.qwp", src.provenance) as wr:
        wr.add_raw("norm_test", np.asarray(src.plane("norm_test")[1]).view(np.uint16))
        wr.add_blocks("w_test", src.entry("w_test").shape, np.asarray(src.plane("w_test")[1]))
    assert (tmp_path / "again.qwp").read_bytes() == (golden_dir / "selfpack.qwp").read_bytes()
    src8 = qp.Pack(golden_dir / "selfpack_hq8.qwp")
    qs, sc = src8.hq8_planes("w_test8")
    with qp.PackWriter(tmp_path / "again8.qwp", src8.provenance) as wr:
        wr.add_hq8_planar("w_test8", np.asarray(qs), np.asarray(sc))
    assert (tmp_path / "again8.qwp").read_bytes() == (golden_dir / "selfpack_hq8.qwp").read_bytes()


def test_writer_round_trips_block_families_and_expert_stacks(tmp_path):
    rng = np.random.default_rng(3)
    experts, n, k = 2, 6, 256
    w = (rng.standard_normal((experts * n, k)) * 0.02).astype(np.float32)
    stack = qo.quant_hq4_blocks(w)
    blk, _ = qo.quant_hq_blocks(w[:n], bits=6, group=128, is_m5=False, rotate=True)
    with qp.PackWriter(tmp_path / "w.qwp", {"source": "writer-test"}) as wr:
        e1 = wr.add_blocks("m.experts.gate_up", (experts, n, k), stack)
        e2 = wr.add_blocks("proj", (n, k), blk, bits=6, group=128, is_m5=False)
        e3 = wr.add_raw("gamma", np.arange(k, dtype=np.float32), kind="f32")
        with pytest.raises(qp.QWQuantError):
            wr.add_raw("gamma", np.zeros(4, np.float32), kind="f32")          # duplicate name
        with pytest.raises(qp.QWQuantError):
            wr.add_blocks("odd", (experts, 5, k), stack[: experts * 5])        # odd rows per expert
        with pytest.raises(qp.QWQuantError):
            wr.add_blocks("short", (n, k), blk[:-1], bits=6, group=128, is_m5=False)
    assert e1["hq4_off"] % 16384 == 0 and e2["hq4_off"] % 16384 == 0 and e3["raw_off"] % 256 == 0
    assert e1["experts"] == experts and e1["e_hq4"] == n * (k // 32) * 20 and "hq" not in e1 and e2["hq"] == {"bits": 6, "group": 128}
    p = qp.Pack(tmp_path / "w.qwp")
    assert np.array_equal(np.asarray(p.plane("m.experts.gate_up")[1]), stack.ravel().view(np.uint8))
    assert p.weight_geometry("m.experts.gate_up") == (experts * n, k, qp.qwhip.KIND_HQ4_G32_M5, 4, 32)
    assert p.weight_geometry("proj") == (n, k, qp.qwhip.KIND_ROTATED_HQ, 6, 128)
    assert np.array_equal(np.asarray(p.plane("proj")[1]), blk.ravel().view(np.uint8))
    assert np.array_equal(np.asarray(p.plane("gamma")[1]).view(np.float32), np.arange(k, dtype=np.float32))


def test_pack_writer_leaves_no_file_when_its_body_fails(tmp_path):
    """A with-body that raises must not leave something that reads as a complete pack of the tensors added so far: no
    trailer is written and the partial file is removed; a clean exit still writes the pack."""
    path = tmp_path / "partial.qwp"
    with pytest.raises(RuntimeError):
        with qp.PackWriter(path, {"source": "writer-test"}) as wr:
            wr.add_raw("gamma", np.arange(64, dtype=np.float32), kind="f32")
            raise RuntimeError("quantization failed midway")
    assert not path.exists()
    with qp.PackWriter(path, {"source": "writer-test"}) as wr:
        wr.add_raw("gamma", np.arange(64, dtype=np.float32), kind="f32")
    assert np.array_equal(np.asarray(qp.Pack(path).plane("gamma")[1]).view(np.float32), np.arange(64, dtype=np.float32))
