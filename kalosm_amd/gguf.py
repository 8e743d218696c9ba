"""Host-side handle of a GGUF file: `GgufMetadata` (fusor-ml/gguf/src/lib.rs:288-319, read at :559-613) and the
`VarBuilder` lookups (fusor-ml/fusor/src/varbuilder.rs:79-160), bound to the fh_gguf_* entry points of
libfusor_hip.so.  Parsing happens in the library; nothing here needs a device except `VarBuilder.get`."""
from __future__ import annotations

import ctypes as C
from typing import Dict, List, Optional, Tuple, Union

import numpy as np

from . import _lib
from ._lib import FusorHipError, GgufTensor, check

U8, I8, U16, I16, U32, I32, F32, BOOL, STRING, ARRAY, U64, I64, F64 = range(13)
_NP = {U8: "<u1", I8: "<i1", U16: "<u2", I16: "<i2", U32: "<u4", I32: "<i4", F32: "<f4", BOOL: "u1", U64: "<u8",
       I64: "<i8", F64: "<f8"}


class GgufTensorMetadata:
    """GgufTensorMetadata (gguf/src/lib.rs:254-259): `ty`, `shape` (row-major), `offset`."""

    def __init__(self, ty: int, shape: Tuple[int, ...], offset: int):
        self.ty, self.shape, self.offset = ty, shape, offset

    def __repr__(self):
        return f"GgufTensorMetadata(ty={self.ty}, shape={self.shape}, offset={self.offset})"


class GgufMetadata:
    """Open with `GgufMetadata.read(path)` or `GgufMetadata.read_bytes(buffer)`."""

    def __init__(self, handle, keep=None):
        self._lib = _lib.load()
        self._h, self._keep = handle, keep
        v, nt, nk, al, off = C.c_uint32(), C.c_uint64(), C.c_uint64(), C.c_uint64(), C.c_uint64()
        check(self._lib.fh_gguf_info(handle, C.byref(v), C.byref(nt), C.byref(nk), C.byref(al), C.byref(off)))
        self.version, self.alignment, self.tensor_data_offset = v.value, al.value, off.value
        self._n_tensors, self._n_meta = nt.value, nk.value
        self._infos: Optional[Dict[str, GgufTensorMetadata]] = None
        self._index: Dict[str, int] = {}

    @staticmethod
    def read(path: str) -> "GgufMetadata":
        h = C.c_void_p()
        check(_lib.load().fh_gguf_open(str(path).encode(), C.byref(h)))
        return GgufMetadata(h)

    @staticmethod
    def read_bytes(data: Union[bytes, bytearray, np.ndarray]) -> "GgufMetadata":
        a = np.frombuffer(data, np.uint8) if not isinstance(data, np.ndarray) else np.ascontiguousarray(data).view(np.uint8)
        h = C.c_void_p()
        check(_lib.load().fh_gguf_open_memory(a.ctypes.data_as(C.c_void_p), a.size, C.byref(h)))
        return GgufMetadata(h, keep=(a, data))

    def close(self) -> None:
        if self._h:
            self._lib.fh_gguf_close(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    # ---- metadata ---------------------------------------------------------------------------
    def keys(self) -> List[str]:
        out = []
        k, t = C.c_char_p(), C.c_uint32()
        for i in range(self._n_meta):
            check(self._lib.fh_gguf_meta_key(self._h, i, C.byref(k), C.byref(t)))
            out.append(k.value.decode(errors="replace"))
        return out

    def get_value(self, key: str):
        """GgufMetadata::get_value (:301-311): None when the key is absent; a key starting with '.' matches the
        shortest stored key ending with it.  Strings come back as `str`, arrays as lists (numpy for numbers)."""
        kb = key.encode()
        full, t = C.c_char_p(), C.c_uint32()
        st = self._lib.fh_gguf_meta_find(self._h, kb, C.byref(full), C.byref(t))
        if st == _lib.FH_ERR_NOT_FOUND:
            return None
        check(st)
        t = t.value
        if t in (U8, U16, U32, U64, I8, I16, I32, I64):
            v = C.c_int64()
            check(self._lib.fh_gguf_meta_int(self._h, kb, C.byref(v)))
            return v.value & 0xFFFFFFFFFFFFFFFF if t == U64 else v.value
        if t in (F32, F64):
            v = C.c_double()
            check(self._lib.fh_gguf_meta_float(self._h, kb, C.byref(v)))
            return v.value
        if t == BOOL:
            v = C.c_int32()
            check(self._lib.fh_gguf_meta_bool(self._h, kb, C.byref(v)))
            return bool(v.value)
        if t == STRING:
            p, n = C.c_void_p(), C.c_uint64()
            check(self._lib.fh_gguf_meta_string(self._h, kb, C.byref(p), C.byref(n)))
            return C.string_at(p, n.value).decode(errors="replace")
        et, n, packed = C.c_uint32(), C.c_uint64(), C.c_void_p()
        check(self._lib.fh_gguf_meta_array(self._h, kb, C.byref(et), C.byref(n), C.byref(packed)))
        if et.value in _NP:
            dt = np.dtype(_NP[et.value])
            a = np.frombuffer(C.string_at(packed, n.value * dt.itemsize), dt) if n.value else np.empty(0, dt)
            return a.astype(bool) if et.value == BOOL else a
        if et.value == STRING:
            out = []
            p, ln = C.c_void_p(), C.c_uint64()
            for i in range(n.value):
                check(self._lib.fh_gguf_meta_array_string(self._h, kb, i, C.byref(p), C.byref(ln)))
                out.append(C.string_at(p, ln.value).decode(errors="replace"))
            return out
        raise FusorHipError(_lib.FH_ERR_UNSUPPORTED, f"'{key}': arrays of arrays are parsed but not converted here")

    def architecture(self) -> Optional[str]:
        """GgufMetadata::architecture (:313-318)."""
        return self.get_value("general.architecture")

    # ---- tensors ----------------------------------------------------------------------------
    @property
    def tensor_infos(self) -> Dict[str, GgufTensorMetadata]:
        if self._infos is None:
            infos = {}
            t = GgufTensor()
            for i in range(self._n_tensors):
                check(self._lib.fh_gguf_tensor_info(self._h, i, C.byref(t)))
                name = t.name.decode(errors="replace")
                infos[name] = GgufTensorMetadata(t.ggml_type, tuple(t.shape[:t.rank]), t.offset)
                self._index[name] = i
            self._infos = infos
        return self._infos

    def read_tensor_bytes(self, name: str) -> np.ndarray:
        """GgufTensorMetadata::read_tensor_bytes (:262-273): a copy of the raw block stream."""
        idx = C.c_uint64()
        check(self._lib.fh_gguf_tensor_find(self._h, name.encode(), C.byref(idx)))
        p, n = C.c_void_p(), C.c_size_t()
        check(self._lib.fh_gguf_tensor_data(self._h, idx.value, C.byref(p), C.byref(n)))
        return np.frombuffer(C.string_at(p, n.value), np.uint8)


class VarBuilder:
    """fusor::VarBuilder over one file (varbuilder.rs:26-160): `pp` prefixes, `get`, `contains_key`."""

    def __init__(self, metadata: GgufMetadata, path: Tuple[str, ...] = ()):
        self.metadata_, self.path = metadata, tuple(path)

    @staticmethod
    def from_gguf(path: str) -> "VarBuilder":
        return VarBuilder(GgufMetadata.read(path))

    def pp(self, s) -> "VarBuilder":
        return VarBuilder(self.metadata_, self.path + (str(s),))

    def _full(self, name: str) -> str:
        return ".".join(self.path + (name,))

    def contains_key(self, key: str) -> bool:
        return self._full(key) in self.metadata_.tensor_infos

    def list_all_keys(self) -> List[str]:
        return list(self.metadata_.tensor_infos)

    def get(self, key: str, device):
        from .fusor import QMatrix
        h = C.c_void_p()
        check(device._lib.fh_qmatrix_from_gguf_tensor(device._h, self.metadata_._h, self._full(key).encode(), C.byref(h)))
        return QMatrix(device, h)

    def metadata(self) -> GgufMetadata:
        return self.metadata_

    def get_metadata(self, key: str):
        return self.metadata_.get_value(key)

    def architecture(self) -> Optional[str]:
        return self.metadata_.architecture()
