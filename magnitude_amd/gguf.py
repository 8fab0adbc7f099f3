"""GGUF tensor reader: locates the quantized tensor payloads of a model file and hands them to
`qproj_upload` verbatim (the bytes a ggml buffer's `set_tensor` would receive).

The reference only inspects GGUF *headers* (inference/crates/icn-models/src/gguf.rs:76-238: magic,
versions 2 and 3, the metadata value types at :395-452, tensor infos, `general.alignment` with
default 32 at :138, the same size bounds); the payload is read by llama.cpp.  This module follows
the same header rules and bounds, then goes one step further: tensor data starts at the header end
rounded up to the alignment, each tensor at its recorded offset, `nelements / block * type_size`
bytes long.  `write` produces files of the same layout for tests and synthetic models.
"""
from __future__ import annotations

import mmap
import os
import struct
from dataclasses import dataclass
from typing import Dict, List, Optional, Tuple

import numpy as np

MAGIC = b"GGUF"
MAX_METADATA_ENTRIES = 1_000_000
MAX_TENSORS = 10_000_000
MAX_STRING_BYTES = 16 * 1024 * 1024
MAX_DIMS = 8

# ggml type id -> (elements per block, bytes per block)
TYPE_LAYOUT = {
    0: (1, 4), 1: (1, 2), 2: (32, 18), 3: (32, 20), 6: (32, 22), 7: (32, 24), 8: (32, 34), 9: (32, 36),
    10: (256, 84), 11: (256, 110), 12: (256, 144), 13: (256, 176), 14: (256, 210), 15: (256, 292),
    24: (1, 1), 25: (1, 2), 26: (1, 4), 27: (1, 8), 28: (1, 8), 30: (1, 2),
}
TYPE_NAMES = {0: "F32", 1: "F16", 2: "Q4_0", 3: "Q4_1", 6: "Q5_0", 7: "Q5_1", 8: "Q8_0", 9: "Q8_1", 10: "Q2_K",
              11: "Q3_K", 12: "Q4_K", 13: "Q5_K", 14: "Q6_K", 15: "Q8_K", 24: "I8", 25: "I16", 26: "I32",
              27: "I64", 28: "F64", 30: "BF16"}
PROJECTION_TYPES = (8, 12, 14)   # what the projection library takes


class GgufError(ValueError):
    pass


def tensor_storage_bytes(ggml_type: int, shape) -> int:
    """nelements / block * type_size; the first dimension must hold whole blocks"""
    if ggml_type not in TYPE_LAYOUT or not shape:
        raise GgufError("tensor storage shape or type is invalid")
    block, size = TYPE_LAYOUT[ggml_type]
    if shape[0] % block:
        raise GgufError("tensor storage shape or type is invalid")
    n = 1
    for d in shape:
        n *= int(d)
    return n // block * size


@dataclass
class TensorInfo:
    name: str
    shape: Tuple[int, ...]     # ggml order: shape[0] is the contiguous (K) dimension
    ggml_type: int
    offset: int                # from the start of the data section
    nbytes: int


class _Reader:
    def __init__(self, buf, length):
        self.buf, self.pos, self.length = buf, 0, length

    def take(self, n):
        if n < 0 or self.pos + n > self.length:
            raise GgufError("header extends beyond end of file")
        b = self.buf[self.pos:self.pos + n]
        self.pos += n
        return b

    def num(self, fmt):
        return struct.unpack("<" + fmt, self.take(struct.calcsize(fmt)))[0]

    def string(self):
        n = self.num("Q")
        if n > MAX_STRING_BYTES:
            raise GgufError("metadata string exceeds inspection bound")
        return bytes(self.take(n)).decode("utf-8")

    _SCALAR = {0: "B", 1: "b", 2: "H", 3: "h", 4: "I", 5: "i", 6: "f", 7: "?", 10: "Q", 11: "q", 12: "d"}

    def value(self, vtype):
        if vtype in self._SCALAR:
            return self.num(self._SCALAR[vtype])
        if vtype == 8:
            return self.string()
        if vtype == 9:
            etype, count = self.num("I"), self.num("Q")
            if count > MAX_METADATA_ENTRIES:
                raise GgufError("metadata array exceeds inspection bound")
            return [self.value(etype) for _ in range(count)]
        raise GgufError("unknown metadata value type")


class GgufFile:
    """Header of a GGUF file plus zero-copy views of its tensor payloads."""

    def __init__(self, path: str):
        self.path = path
        self._fh = open(path, "rb")
        size = os.fstat(self._fh.fileno()).st_size
        if size < 24:
            self._fh.close()
            raise GgufError("header extends beyond end of file")
        self._mm = mmap.mmap(self._fh.fileno(), 0, access=mmap.ACCESS_READ)
        try:
            self._parse(size)
        except Exception:
            self.close()
            raise

    def _parse(self, size):
        r = _Reader(self._mm, size)
        if bytes(r.take(4)) != MAGIC:
            raise GgufError("invalid GGUF magic")
        self.version = r.num("I")
        if self.version not in (2, 3):
            raise GgufError(f"unsupported GGUF version {self.version}")
        n_tensors, n_meta = r.num("Q"), r.num("Q")
        if n_tensors > MAX_TENSORS:
            raise GgufError("tensor count exceeds inspection bound")
        if n_meta > MAX_METADATA_ENTRIES:
            raise GgufError("metadata count exceeds inspection bound")
        self.metadata: Dict[str, object] = {}
        for _ in range(n_meta):
            key = r.string()
            self.metadata[key] = r.value(r.num("I"))
        self.tensors: Dict[str, TensorInfo] = {}
        for _ in range(n_tensors):
            name = r.string()
            nd = r.num("I")
            if nd == 0 or nd > MAX_DIMS:
                raise GgufError("tensor dimension count is invalid")
            shape = tuple(r.num("Q") for _ in range(nd))
            gtype = r.num("I")
            nbytes = tensor_storage_bytes(gtype, shape)
            self.tensors[name] = TensorInfo(name, shape, gtype, r.num("Q"), nbytes)
        align = self.metadata.get("general.alignment", 32)
        if not isinstance(align, int) or align <= 0 or align & (align - 1):
            raise GgufError("GGUF alignment is invalid")
        self.alignment = align
        self.data_offset = (r.pos + align - 1) & ~(align - 1)
        if self.data_offset > size:
            raise GgufError("GGUF header extends beyond end of file")
        for t in self.tensors.values():
            if t.offset % align or self.data_offset + t.offset + t.nbytes > size:
                raise GgufError(f"tensor {t.name!r} lies outside the file or off its alignment")

    def close(self):
        if getattr(self, "_mm", None) is not None:
            self._mm.close()
            self._mm = None
        self._fh.close()

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    def tensor_bytes(self, name: str) -> np.ndarray:
        """the tensor's GGUF bytes as a read-only uint8 view of the mapped file"""
        t = self.tensors[name]
        return np.frombuffer(self._mm, dtype=np.uint8, count=t.nbytes, offset=self.data_offset + t.offset)

    def projection_tensors(self) -> List[TensorInfo]:
        """the tensors the projection library takes: Q8_0 / Q4_K / Q6_K matrices [K, N] or expert stacks [K, N, E]"""
        return [t for t in self.tensors.values() if t.ggml_type in PROJECTION_TYPES and len(t.shape) in (2, 3)]

    def upload(self, ctx, name: str):
        """uploads one matrix (or expert stack) through qproj_upload; returns the Weight"""
        t = self.tensors[name]
        if t.ggml_type not in PROJECTION_TYPES or len(t.shape) not in (2, 3):
            raise GgufError(f"tensor {name!r} ({TYPE_NAMES.get(t.ggml_type, t.ggml_type)}, {t.shape}) is not a "
                            f"Q8_0/Q4_K/Q6_K projection matrix")
        k, n = t.shape[0], t.shape[1]
        e = t.shape[2] if len(t.shape) == 3 else 1
        return ctx.upload(t.ggml_type, k, n, self.tensor_bytes(name), n_expert=e)

    def upload_all(self, ctx, names=None) -> dict:
        names = names if names is not None else [t.name for t in self.projection_tensors()]
        return {n: self.upload(ctx, n) for n in names}


def _pack_string(s: str) -> bytes:
    b = s.encode("utf-8")
    return struct.pack("<Q", len(b)) + b


def _pack_value(v) -> bytes:
    if isinstance(v, bool):
        return struct.pack("<I?", 7, v)
    if isinstance(v, int):
        return struct.pack("<Iq", 11, v) if v < 0 else (struct.pack("<II", 4, v) if v < 2 ** 32 else struct.pack("<IQ", 10, v))
    if isinstance(v, float):
        return struct.pack("<If", 6, v)
    if isinstance(v, str):
        return struct.pack("<I", 8) + _pack_string(v)
    if isinstance(v, (list, tuple)):
        if all(isinstance(x, str) for x in v):
            return struct.pack("<IIQ", 9, 8, len(v)) + b"".join(_pack_string(x) for x in v)
        if all(isinstance(x, int) and not isinstance(x, bool) for x in v):
            return struct.pack("<IIQ", 9, 5, len(v)) + b"".join(struct.pack("<i", x) for x in v)
        if all(isinstance(x, float) for x in v):
            return struct.pack("<IIQ", 9, 6, len(v)) + b"".join(struct.pack("<f", x) for x in v)
    raise GgufError(f"cannot encode metadata value {v!r}")


def write(path: str, tensors, metadata: Optional[dict] = None, version: int = 3, alignment: int = 32) -> None:
    """tensors: iterable of (name, shape in ggml order, ggml_type, bytes-like payload)"""
    tensors = list(tensors)
    meta = dict(metadata or {})
    if alignment != 32:
        meta["general.alignment"] = alignment
    head = MAGIC + struct.pack("<IQQ", version, len(tensors), len(meta))
    for k, v in meta.items():
        head += _pack_string(k) + _pack_value(v)
    offsets, off = [], 0
    for name, shape, gtype, data in tensors:
        nbytes = tensor_storage_bytes(gtype, shape)
        if len(memoryview(data).cast("B")) != nbytes:
            raise GgufError(f"tensor {name!r}: payload size does not match its shape and type")
        offsets.append(off)
        off = (off + nbytes + alignment - 1) & ~(alignment - 1)
    for (name, shape, gtype, _), o in zip(tensors, offsets):
        head += _pack_string(name) + struct.pack("<I", len(shape)) + b"".join(struct.pack("<Q", d) for d in shape)
        head += struct.pack("<IQ", gtype, o)
    pad = (-len(head)) % alignment
    with open(path, "wb") as f:
        f.write(head + b"\0" * pad)
        for (_, shape, gtype, data), o in zip(tensors, offsets):
            b = bytes(memoryview(data).cast("B"))
            f.write(b + b"\0" * ((-len(b)) % alignment))
