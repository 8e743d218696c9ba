"""TEST INFRASTRUCTURE ONLY -- a plain-Python reader and writer of the GGUF container, used to check the
library's reader (`fh_gguf_*`) and to write small synthetic model files for the parity tests.  Nothing in the
product imports it.

Written from the published container layout (ggml `docs/gguf.md`, the document the reference names at
fusor-ml/gguf/src/lib.rs:1) and the reference's reader / writer, fusor-ml/gguf/src/lib.rs:559-613 / :615-668:

    magic "GGUF" | version u32 | tensor count | key/value count            (counts: u32 in v1, u64 in v2/v3)
    key/value:   string key | value type u32 | value
    string:      length (u32 in v1, u64 after) | bytes            (trailing NUL bytes dropped on read, :330-332)
    array:       element type u32 | count | elements
    tensor info: string name | n_dims u32 | dims (innermost first; reversed on read, :583) | ggml type u32 |
                 offset u64 (relative to the payload start)
    payload:     starts at the next multiple of `general.alignment` (default 32, :597-606)

Pinned by: the reference's own `test_round_trip_empty` (:2509-2536: an empty version-3 file is 24 bytes and its
payload offset reads back as 32) and `test_gguf_version_round_trip` (:144-155), both repeated in
tests/test_gguf_reader.py, and a byte string assembled by hand from the layout above in the same file.
"""
from __future__ import annotations

import struct
from typing import Dict, List, Tuple

import numpy as np

U8, I8, U16, I16, U32, I32, F32, BOOL, STRING, ARRAY, U64, I64, F64 = range(13)
_FMT = {U8: "<B", I8: "<b", U16: "<H", I16: "<h", U32: "<I", I32: "<i", F32: "<f", BOOL: "<B", U64: "<Q", I64: "<q",
        F64: "<d"}
# elements per block, bytes per block (fusor-ml/gguf/src/lib.rs:98-121)
BLOCK = {0: (1, 4), 1: (1, 2), 2: (32, 18), 6: (32, 22), 8: (32, 34), 12: (256, 144), 13: (256, 176), 14: (256, 210)}
KNOWN_TYPES = {0, 1, 2, 3, 6, 7, 8, 9, 10, 11, 12, 13, 14, 15}


class GgufError(Exception):
    pass


class Typed:
    """A metadata value with an explicit wire type (plain Python values are typed by `_infer`)."""

    def __init__(self, vtype: int, value, elem_type: int = None):
        self.vtype, self.value, self.elem_type = vtype, value, elem_type


class _Reader:
    def __init__(self, data: bytes):
        self.d, self.p, self.v = data, 0, 3

    def take(self, n: int) -> bytes:
        if self.p + n > len(self.d):
            raise GgufError("io error: unexpected end of file")
        b = self.d[self.p:self.p + n]
        self.p += n
        return b

    def num(self, t: int):
        f = _FMT[t]
        return struct.unpack(f, self.take(struct.calcsize(f)))[0]

    def length(self) -> int:
        return self.num(U32) if self.v == 1 else self.num(U64)

    def string(self) -> bytes:
        return self.take(self.length()).rstrip(b"\0")

    def value(self, t: int):
        if t > F64:
            raise GgufError(f"invalid value type {t}")
        if t == BOOL:
            b = self.num(U8)
            if b > 1:
                raise GgufError("invalid bool value")
            return bool(b)
        if t == STRING:
            return self.string()
        if t == ARRAY:
            et = self.num(U32)
            if et > F64:
                raise GgufError(f"invalid value type {et}")
            n = self.length()
            return [self.value(et) for _ in range(n)]
        return self.num(t)


class GgufRef:
    """version, metadata {key bytes: (type, value)}, tensors {name bytes: (ggml type, shape tuple, offset)},
    alignment, data_offset."""

    def __init__(self, data: bytes):
        r = _Reader(data)
        magic = r.take(4)
        if magic not in (b"GGUF", b"FUGG"):
            raise GgufError("invalid magic bytes")
        self.version = r.num(U32)
        if self.version not in (1, 2, 3):
            raise GgufError(f"unsupported version {self.version}")
        r.v = self.version
        nt, nkv = r.length(), r.length()
        self.metadata: Dict[bytes, Tuple[int, object]] = {}
        for _ in range(nkv):
            key = r.string()
            t = r.num(U32)
            self.metadata[key] = (t, r.value(t))
        self.tensors: Dict[bytes, Tuple[int, Tuple[int, ...], int]] = {}
        for _ in range(nt):
            name = r.string()
            nd = r.num(U32)
            dims = [r.length() & 0xFFFFFFFF for _ in range(nd)]
            ty = r.num(U32)
            if ty not in KNOWN_TYPES:
                raise GgufError(f"unsupported dtype {ty}")
            off = r.num(U64)
            self.tensors[name] = (ty, tuple(reversed(dims)), off)
        self.alignment = 32
        a = self.metadata.get(b"general.alignment")
        if a is not None and a[0] in (U8, U16, U32, I8, I16, I32) and a[1] >= 0:
            self.alignment = a[1]
        self.data_offset = -(-r.p // self.alignment) * self.alignment
        self.data = data

    def get_value(self, key: bytes):
        """Suffix lookup of fusor-ml/gguf/src/lib.rs:301-311."""
        if key.startswith(b"."):
            hits = [k for k in self.metadata if k.endswith(key)]
            if not hits:
                return None
            return self.metadata[min(hits, key=len)]
        return self.metadata.get(key)

    def tensor_bytes(self, name: bytes) -> np.ndarray:
        ty, shape, off = self.tensors[name]
        elems = int(np.prod(shape, dtype=np.uint64)) & 0xFFFFFFFF
        be, bb = BLOCK[ty]
        if elems % be:
            raise GgufError(f"tensor size ({elems}) is not a multiple of the block size ({be})")
        n = elems // be * bb
        s = self.data_offset + off
        if s + n > len(self.data):
            raise GgufError("io error: unexpected end of file")
        return np.frombuffer(self.data, np.uint8, n, s)


def _infer(v) -> Typed:
    if isinstance(v, Typed):
        return v
    if isinstance(v, bool):
        return Typed(BOOL, v)
    if isinstance(v, int):
        return Typed(U32 if 0 <= v < 2 ** 32 else I64, v)
    if isinstance(v, float):
        return Typed(F32, v)
    if isinstance(v, (str, bytes)):
        return Typed(STRING, v)
    if isinstance(v, (list, tuple)):
        return Typed(ARRAY, list(v))
    raise TypeError(type(v))


def _put_len(out: List[bytes], n: int, version: int) -> None:
    out.append(struct.pack("<I" if version == 1 else "<Q", n))


def _put_value(out: List[bytes], tv: Typed, version: int) -> None:
    t, v = tv.vtype, tv.value
    if t == STRING:
        b = v.encode() if isinstance(v, str) else v
        _put_len(out, len(b), version)
        out.append(b)
    elif t == ARRAY:
        elems = [_infer(e) for e in v]
        et = tv.elem_type if tv.elem_type is not None else elems[0].vtype
        out.append(struct.pack("<I", et))
        _put_len(out, len(elems), version)
        for e in elems:
            _put_value(out, Typed(et, e.value, e.elem_type), version)
    else:
        out.append(struct.pack(_FMT[t], v))


def write_gguf(metadata: dict, tensors: List[Tuple[str, int, Tuple[int, ...], np.ndarray]], version: int = 3,
               alignment: int = None, magic: bytes = b"GGUF") -> bytes:
    """metadata: {key: value or Typed}; tensors: (name, ggml type, row-major shape, raw bytes).  Payloads are
    laid out in order, each starting at a multiple of the alignment (`general.alignment` is added to the metadata
    when `alignment` is given)."""
    md = dict(metadata)
    if alignment is not None:
        md["general.alignment"] = Typed(U32, alignment)
    a = alignment or 32
    out: List[bytes] = [magic, struct.pack("<I", version)]
    _put_len(out, len(tensors), version)
    _put_len(out, len(md), version)
    for k, v in md.items():
        kb = k.encode() if isinstance(k, str) else k
        _put_len(out, len(kb), version)
        out.append(kb)
        tv = _infer(v)
        out.append(struct.pack("<I", tv.vtype))
        _put_value(out, tv, version)
    off = 0
    offsets = []
    for name, ty, shape, raw in tensors:
        nb = name.encode() if isinstance(name, str) else name
        _put_len(out, len(nb), version)
        out.append(nb)
        out.append(struct.pack("<I", len(shape)))
        for d in reversed(shape):
            _put_len(out, int(d), version)
        out.append(struct.pack("<IQ", ty, off))
        offsets.append(off)
        off += -(-np.asarray(raw).nbytes // a) * a
    head = b"".join(out)
    start = -(-len(head) // a) * a
    if not tensors:
        return head  # as the reference's writer: nothing is padded behind an empty tensor directory
    body = bytearray(start + off)
    body[:len(head)] = head
    for (name, ty, shape, raw), o in zip(tensors, offsets):
        b = np.ascontiguousarray(raw).view(np.uint8).reshape(-1).tobytes()
        body[start + o:start + o + len(b)] = b
    return bytes(body)
