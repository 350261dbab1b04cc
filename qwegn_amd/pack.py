"""QWP1 pack reader and plane mover: the on-disk step in front of the quantized matmul path.

Mirrors, name for name, the parts of the reference that find a tensor's bytes in a pack and move them into a
device bank:
  * `Pack`            <- `QWQuant.Pack`      (Sources/Foundation/QWQuant/QWPack.swift:37-139): file = "QWP1", u64 LE header
                         length, planes, JSON trailer at EOF `{provenance, tensors{name: entry}}`;
  * `QWQTensorEntry`  <- `QWQTensorEntry`    (Sources/Foundation/QWQuant/QWQuantTypes.swift:69-149);
  * `PlaneLayout`     <- `PlaneLayout`       (Sources/Foundation/QWLoad/PlaneLayout.swift:6-67): the single authority for the
                         byte count and offset of a verbatim plane (raw bf16/f32, or HQ blocks incl. 3-D expert stacks).
The writer is `pack_file` (Scripts/quantize/pack.py:115-316).  The reference's model-identity checks (geometry
digests against a model descriptor) belong to its control plane and are not restated here.
"""
from __future__ import annotations

import dataclasses
import json
import os
import pathlib

import numpy as np

from . import qwhip

MAGIC = b"QWP1"
GROUP = 32          # QWHQ4Layout.group
BLOCK_BYTES = 20    # QWHQ4Layout.blockBytes


class QWQuantError(Exception):
    """`QWQuantError` cases of the reader: modelFileMissing, truncated, badMagic, badHeader, unknownTensor, badPlane."""

    def __init__(self, case: str, detail: str = ""):
        super().__init__(f"{case}: {detail}" if detail else case)
        self.case = case


def aq_block_supported(bits: int, group: int) -> bool:
    """QWAQBlock.isBlockSupported (Sources/Foundation/QWQuant/QWAQBlock.swift:17-36)."""
    return bits in (2, 3, 4, 6, 8) and group in (32, 64, 128, 256) and (group * bits) % 8 == 0


def aq_block_bytes(bits: int, group: int) -> int:
    return 4 + group * bits // 8


@dataclasses.dataclass(frozen=True)
class QWHQFormat:
    bits: int
    group: int
    vq: str | None = None


@dataclasses.dataclass(frozen=True)
class QWQTensorEntry:
    shape: tuple[int, ...]
    hq4_off: int | None = None
    q8_off: int | None = None
    q8_s_off: int | None = None
    hq8_off: int | None = None
    hq8_s_off: int | None = None
    raw_off: int | None = None
    kind: str | None = None
    experts: int | None = None
    e_hq4: int | None = None
    hq: QWHQFormat | None = None

    @staticmethod
    def decode(obj: dict) -> "QWQTensorEntry":
        if not isinstance(obj, dict) or not isinstance(obj.get("shape"), list):
            raise QWQuantError("badHeader", "a tensor entry needs a shape")
        hq = obj.get("hq")
        fmt = QWHQFormat(int(hq["bits"]), int(hq["group"]), hq.get("vq")) if isinstance(hq, dict) else None
        opt = lambda k: None if obj.get(k) is None else int(obj[k])  # noqa: E731
        return QWQTensorEntry(tuple(int(d) for d in obj["shape"]), opt("hq4_off"), opt("q8_off"), opt("q8_s_off"), opt("hq8_off"),
                              opt("hq8_s_off"), opt("raw_off"), obj.get("kind"), opt("experts"), opt("e_hq4"), fmt)

    @property
    def hq_bits(self) -> int:
        return self.hq.bits if self.hq else 4

    @property
    def hq_group(self) -> int:
        return self.hq.group if self.hq else GROUP

    @property
    def is_incumbent_hq4(self) -> bool:
        return self.hq is None

    @property
    def is_shvq(self) -> bool:
        return self.hq is not None and self.hq.vq == "shvq1"

    @property
    def hq_block_bytes(self) -> int:
        return aq_block_bytes(self.hq.bits, self.hq.group) if self.hq else BLOCK_BYTES

    @property
    def raw_elem_bytes(self) -> int:
        return 4 if self.kind == "f32" else 2

    @property
    def quantized(self) -> bool:
        return self.raw_off is None and self.hq4_off is not None

    @property
    def hq8_quantized(self) -> bool:
        return self.raw_off is None and self.hq8_off is not None and self.hq4_off is None


class PlaneLayout:
    """`raw` or `hq4` (every HQ block plane rides the hq4_off key); sizes and offsets for the mover come from here only."""

    RAW, HQ4 = "raw", "hq4"

    @staticmethod
    def resolve(e: QWQTensorEntry) -> str | None:
        if e.raw_off is not None:
            return PlaneLayout.RAW
        if e.hq4_off is not None:
            return PlaneLayout.HQ4
        return None

    @staticmethod
    def offset(layout: str, e: QWQTensorEntry) -> int | None:
        return e.raw_off if layout == PlaneLayout.RAW else e.hq4_off

    @staticmethod
    def byte_count(layout: str, e: QWQTensorEntry) -> int | None:
        if not e.shape or any(d < 0 for d in e.shape):
            return None
        if layout == PlaneLayout.RAW:
            return int(np.prod(e.shape, dtype=np.int64)) * e.raw_elem_bytes
        if e.experts is not None and e.e_hq4 is not None and len(e.shape) == 3:
            return None if e.experts < 0 or e.e_hq4 < 0 else e.experts * e.e_hq4
        if len(e.shape) < 2:
            return None
        n, k = e.shape[0], int(np.prod(e.shape[1:], dtype=np.int64))
        grp = e.hq_group
        if grp <= 0 or k % grp != 0:
            return None
        if not e.is_incumbent_hq4 and (e.is_shvq or not aq_block_supported(e.hq_bits, grp)):
            return None     # SHVQ containers are outside this build
        return n * (k // grp) * e.hq_block_bytes


class Pack:
    """Memory-mapped QWP1 pack: header check, JSON trailer, per-tensor planes, and the mover into device banks."""

    def __init__(self, path):
        self.path = pathlib.Path(path)
        if not self.path.is_file():
            raise QWQuantError("modelFileMissing", str(self.path))
        count = self.path.stat().st_size
        if count <= 12:
            raise QWQuantError("truncated")
        self.raw = np.memmap(self.path, dtype=np.uint8, mode="r")
        if bytes(self.raw[:4]) != MAGIC:
            raise QWQuantError("badMagic")
        hdr_len = int.from_bytes(bytes(self.raw[4:12]), "little")
        if hdr_len > count - 12:
            raise QWQuantError("truncated")
        try:
            header = json.loads(bytes(self.raw[count - hdr_len:]).decode("utf-8"))
            self.provenance = dict(header["provenance"])
            self.tensors = {name: QWQTensorEntry.decode(obj) for name, obj in header["tensors"].items()}
        except QWQuantError:
            raise
        except Exception as exc:   # malformed JSON, missing keys
            raise QWQuantError("badHeader", str(exc)) from exc
        self.data_end = count - hdr_len

    def entry(self, name: str) -> QWQTensorEntry:
        if name not in self.tensors:
            raise QWQuantError("unknownTensor", name)
        return self.tensors[name]

    def plane(self, name: str) -> tuple[str, np.ndarray]:
        """(layout, the plane's bytes as a view of the mapping); refuses planes that leave the data region."""
        e = self.entry(name)
        layout = PlaneLayout.resolve(e)
        if layout is None:
            raise QWQuantError("badPlane", f"{name} has no verbatim plane")
        off, nbytes = PlaneLayout.offset(layout, e), PlaneLayout.byte_count(layout, e)
        if nbytes is None or off is None or off < 12 or off + nbytes > self.data_end:
            raise QWQuantError("badPlane", f"{name}: offset {off} size {nbytes} outside the pack's data")
        return layout, self.raw[off:off + nbytes]

    def hq8_planes(self, name: str) -> tuple[np.ndarray, np.ndarray]:
        """Planar HQ8_G32_M5 entry: (int8 codes [n, k], f16 scales [n, k / 32]) as views of the mapping
        (QWQuant.Pack.dequantHQ8Rot reads the same two planes, Sources/Foundation/QWQuant/QWPack.swift:326-351)."""
        e = self.entry(name)
        if not e.hq8_quantized or e.hq8_s_off is None or len(e.shape) != 2 or e.shape[1] % GROUP != 0:
            raise QWQuantError("badPlane", f"{name} is not a 2-D planar HQ8 tensor")
        n, k = e.shape
        q_bytes, s_bytes = n * k, n * (k // GROUP) * 2
        for off, size in ((e.hq8_off, q_bytes), (e.hq8_s_off, s_bytes)):
            if off < 12 or off + size > self.data_end:
                raise QWQuantError("badPlane", f"{name}: offset {off} size {size} outside the pack's data")
        qs = self.raw[e.hq8_off:e.hq8_off + q_bytes].view(np.int8).reshape(n, k)
        scales = self.raw[e.hq8_s_off:e.hq8_s_off + s_bytes].view(np.float16).reshape(n, k // GROUP)
        return qs, scales

    def upload_hq8(self, dev: "qwhip.Device", name: str):
        """Moves a planar HQ8 entry into two device buffers: (codes, scales, n, k); qwhip_dequant_hq8_planar reads them."""
        qs, scales = self.hq8_planes(name)
        return dev.put(np.ascontiguousarray(qs)), dev.put(np.ascontiguousarray(scales)), qs.shape[0], qs.shape[1]

    def weight_geometry(self, name: str) -> tuple[int, int, int, int, int]:
        """(rows, k, kind, bits, group) of a quantized entry as the weight view wants it: an expert stack
        [E, N, K] is one bank of E * N rows (expert e at row e * N)."""
        e = self.entry(name)
        if not e.quantized or len(e.shape) not in (2, 3):
            raise QWQuantError("badPlane", f"{name} is not a 2-D or expert-stacked quantized tensor")
        rows = e.shape[0] if len(e.shape) == 2 else e.shape[0] * e.shape[1]
        k = e.shape[-1]
        if e.is_incumbent_hq4:
            return rows, k, qwhip.KIND_HQ4_G32_M5, 4, GROUP
        if e.is_shvq:
            raise QWQuantError("badPlane", f"{name}: SHVQ containers are outside this build")
        return rows, k, qwhip.KIND_ROTATED_HQ, e.hq_bits, e.hq_group

    def upload(self, dev: "qwhip.Device", name: str, chunk_bytes: int = 64 << 20):
        """Plane mover: streams the plane into a fresh device buffer in chunks (the mapping is never read whole) and
        returns (buffer, weight view) for quantized planes, (buffer, None) for raw ones."""
        layout, plane = self.plane(name)
        e = self.entry(name)
        view_args = None
        if layout == PlaneLayout.HQ4:
            rows, k, kind, bits, group = self.weight_geometry(name)
            per_row = (k // group) * e.hq_block_bytes
            if len(e.shape) == 3 and e.e_hq4 != e.shape[1] * per_row:
                raise QWQuantError("badPlane", f"{name}: expert stride {e.e_hq4} is not {e.shape[1]} rows of {per_row} bytes")
            if rows * per_row != plane.nbytes:
                raise QWQuantError("badPlane", f"{name}: {plane.nbytes} bytes for {rows} rows of {per_row}")
            view_args = (rows, k, kind, bits, group)
        buf = dev.alloc(max(int(plane.nbytes), 256))
        for start in range(0, plane.nbytes, chunk_bytes):
            part = np.ascontiguousarray(plane[start:start + chunk_bytes])
            qwhip.check(dev.lib.qwhip_memcpy_h2d(dev.stream.handle, buf.ptr + start, part.ctypes.data, part.nbytes))
            dev.stream.sync()   # the staging array dies at the end of the iteration
        if view_args is None:
            return buf, None
        return buf, dev.view(buf, *view_args, nbytes=int(plane.nbytes))


class PackWriter:
    """Writes a QWP1 pack in the layout the reference's packer gives it (pack_file, Scripts/quantize/pack.py:115-316): magic,
    the trailer's byte count at offset 4, planes, JSON trailer {"provenance", "tensors"} at the end of the file.  Raw and planar
    planes start and end on 256-byte boundaries, block planes on 16 KiB boundaries; entries keep the order they were added in
    and carry exactly the keys the reader's schema knows (shape, kind, raw_off | hq4_off | hq8_off + hq8_s_off, experts, e_hq4, hq).
    Planes are bytes the caller already holds: quantized with the device writers (`add_weights`) or copied from elsewhere."""

    RAW_ALIGN, BLOCK_ALIGN = 256, 16384

    def __init__(self, path, provenance: dict):
        self.path = pathlib.Path(path)
        self.provenance = dict(provenance)
        self.index: dict[str, dict] = {}
        self._f = open(self.path, "wb")
        self._f.write(MAGIC + b"\0" * 8)
        self._pad(self.RAW_ALIGN)

    def _pad(self, alignment: int) -> int:
        off = self._f.tell()
        fill = (-off) % alignment
        self._f.write(b"\0" * fill)
        return off + fill

    def _claim(self, name: str) -> None:
        if self._f is None:
            raise QWQuantError("badPlane", "the pack is closed")
        if name in self.index:
            raise QWQuantError("badPlane", f"duplicate tensor: {name}")

    def add_raw(self, name: str, values: np.ndarray, kind: str = "bf16") -> dict:
        """A verbatim plane: bf16 bits (u16) or f32 values."""
        self._claim(name)
        arr = np.ascontiguousarray(values)
        if kind == "bf16" and arr.dtype != np.uint16:
            raise QWQuantError("badPlane", f"{name}: bf16 planes are handed over as their 16-bit patterns")
        if kind == "f32":
            arr = arr.astype("<f4", copy=False)
        elif kind != "bf16":
            raise QWQuantError("badPlane", f"{name}: raw kind {kind}")
        entry = {"shape": list(arr.shape), "kind": kind, "raw_off": self._pad(self.RAW_ALIGN)}
        self._f.write(arr.tobytes())
        self._pad(self.RAW_ALIGN)
        self.index[name] = entry
        return entry

    def add_blocks(self, name: str, shape, blocks: np.ndarray, bits: int = 4, group: int = GROUP, is_m5: bool = True) -> dict:
        """A block plane for a [N, K] tensor or an expert stack [E, N, K] (stored as one bank of E * N rows, e_hq4 bytes per
        expert; N even as the packer demands).  `blocks`: the bank's bytes in row order."""
        self._claim(name)
        shape = [int(d) for d in shape]
        if len(shape) not in (2, 3) or shape[-1] % group != 0 or (len(shape) == 3 and shape[1] % 2 != 0):
            raise QWQuantError("badPlane", f"{name}: shape {shape} does not fit group {group}")
        m5 = is_m5 and bits == 4 and group == GROUP
        bb = BLOCK_BYTES if m5 else aq_block_bytes(bits, group)
        if not m5 and not aq_block_supported(bits, group):
            raise QWQuantError("badPlane", f"{name}: no container for {bits} bits, group {group}")
        rows = shape[0] if len(shape) == 2 else shape[0] * shape[1]
        data = np.ascontiguousarray(blocks).view(np.uint8).ravel()
        if data.nbytes != rows * (shape[-1] // group) * bb:
            raise QWQuantError("badPlane", f"{name}: {data.nbytes} bytes for {rows} rows of {(shape[-1] // group) * bb}")
        entry = {"shape": shape}
        if len(shape) == 3:
            entry["experts"] = shape[0]
            entry["e_hq4"] = shape[1] * (shape[2] // group) * bb
        entry["hq4_off"] = self._pad(self.BLOCK_ALIGN)
        if not m5:
            entry["hq"] = {"bits": int(bits), "group": int(group)}
        self._f.write(data.tobytes())
        self._pad(self.BLOCK_ALIGN)
        self.index[name] = entry
        return entry

    def add_hq8_planar(self, name: str, qs: np.ndarray, scales: np.ndarray) -> dict:
        """Planar HQ8_G32_M5: int8 codes [N, K], then f16 scales [N, K / 32], each plane on its own 256-byte boundary."""
        self._claim(name)
        qs = np.ascontiguousarray(qs, dtype=np.int8)
        scales = np.ascontiguousarray(scales, dtype=np.float16)
        if qs.ndim != 2 or qs.shape[1] % GROUP != 0 or scales.shape != (qs.shape[0], qs.shape[1] // GROUP):
            raise QWQuantError("badPlane", f"{name}: planar HQ8 wants 2-D codes and one scale per 32 columns")
        entry = {"shape": list(qs.shape), "hq8_off": self._pad(self.RAW_ALIGN)}
        self._f.write(qs.tobytes())
        entry["hq8_s_off"] = self._pad(self.RAW_ALIGN)
        self._f.write(scales.tobytes())
        self._pad(self.RAW_ALIGN)
        self.index[name] = entry
        return entry

    def add_weights(self, dev: "qwhip.Device", name: str, w: np.ndarray, bits: int = 4, group: int = GROUP, is_m5: bool = True,
                    rotate: bool = True) -> dict:
        """Quantizes fp32 weights [N, K] or [E, N, K] on the device (qwhip_quantize_hq4_g32 / qwhip_quantize_blocks, the group
        resolved as the packer does: gcd(K, requested)) and adds the bank."""
        import math
        w = np.ascontiguousarray(w, dtype=np.float32)
        k = w.shape[-1]
        rows = int(np.prod(w.shape[:-1], dtype=np.int64))
        eff = math.gcd(k, group)
        m5 = is_m5 and bits == 4 and eff == GROUP
        bb = BLOCK_BYTES if m5 else aq_block_bytes(bits, eff)
        src, out = dev.put(w), dev.alloc(max(rows * (k // eff) * bb, 256))
        if m5:
            qwhip.check(dev.lib.qwhip_quantize_hq4_g32(dev.stream.handle, src.ptr, qwhip.F32, rows, k, int(rotate), out.ptr))
        else:
            qwhip.check(dev.lib.qwhip_quantize_blocks(dev.stream.handle, src.ptr, qwhip.F32, rows, k, bits, eff, int(rotate), 2, out.ptr))
        blocks = out.download(np.uint8, (rows * (k // eff) * bb,))
        src.free()
        out.free()
        return self.add_blocks(name, w.shape, blocks, bits, eff, is_m5)

    def close(self) -> pathlib.Path:
        trailer = json.dumps({"provenance": self.provenance, "tensors": self.index}).encode()
        self._f.write(trailer)
        self._f.seek(4)
        self._f.write(len(trailer).to_bytes(8, "little"))
        self._f.close()
        self._f = None
        return self.path

    def __enter__(self):
        return self

    def __exit__(self, exc_type, exc, tb):
        if self._f is not None:
            if exc_type is None:
                self.close()
            else:
                # the body failed: no trailer, and the partial file goes (it must not pass for a whole pack of the
                # tensors added so far)
                self._f.close()
                self._f = None
                try:
                    os.unlink(self.path)
                except OSError:
                    pass
        return False
