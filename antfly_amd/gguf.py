"""GGUF container, mirroring gguf/format.zig (parse), gguf/tensor_types.zig (byteLen) and
gguf/tensor_catalog.zig (Catalog) of the reference over the library's C ABI.  The
parser and the file mapping live in the shared library; this module only names things."""
from __future__ import annotations

import ctypes as C
from dataclasses import dataclass
from typing import List, Optional

import numpy as np

from . import _lib
from ._lib import check

MAGIC = b"GGUF"
DEFAULT_ALIGNMENT = 32

# format.MetadataValueType
U8, I8, U16, I16, U32, I32, F32, BOOL, STRING, ARRAY, U64, I64, F64 = range(13)


def _text(raw: bytes) -> str:
    """Names and strings are byte strings in the file (format.zig keeps them as []const u8);
    bytes that are not UTF-8 survive a round trip through str as surrogate escapes."""
    return raw.decode("utf-8", "surrogateescape")


def _raw(text: str) -> bytes:
    return text.encode("utf-8", "surrogateescape")


@dataclass
class Header:
    version: int
    tensor_count: int
    metadata_count: int


@dataclass
class TensorInfo:
    name: str
    dimensions: List[int]     # as stored: fastest-varying first
    tensor_type: int          # raw GGUF id
    type_name: str
    is_quantized: bool
    offset: int
    data_offset: int
    byte_len: Optional[int]   # None when the type's size rule is unknown

    @property
    def shape(self) -> List[int]:
        """normalizedShapeFromDims (models/tensor_store.zig:654-658): [out, in] for a matrix."""
        return list(reversed(self.dimensions))


@dataclass
class MetadataEntry:
    key: str
    value_type: int
    value: object             # scalar or str; for arrays the element count
    element_type: Optional[int] = None


def byteLen(tensor_type: int, dimensions, bitnet_dialect: bool = False) -> Optional[int]:
    """tensor_types.byteLen; bitnet_dialect reads id 39 as TL2."""
    dims = (C.c_uint64 * max(len(dimensions), 1))(*dimensions)
    n = _lib.lib().afhip_gguf_tensor_byte_len(tensor_type, int(bitnet_dialect), dims, len(dimensions))
    return int(n) if n else None


class File:
    """format.File plus the bytes it describes.  `parse(bytes)` borrows the buffer, `open(path)` maps the file."""

    def __init__(self, handle, keepalive=None):
        self._h = handle
        self._keepalive = keepalive
        s = _lib.GgufSummary()
        check(_lib.lib().afhip_gguf_get_summary(self._h, C.byref(s)))
        self.header = Header(int(s.version), int(s.tensor_count), int(s.metadata_count))
        self.alignment = int(s.alignment)
        self.data_region_offset = int(s.data_region_offset)
        self.file_len = int(s.file_len)

    @classmethod
    def parse(cls, data) -> "File":
        arr = np.frombuffer(data, dtype=np.uint8)
        h = C.c_void_p()
        check(_lib.lib().afhip_gguf_parse(arr.ctypes.data if arr.size else None, arr.size, C.byref(h)))
        return cls(h.value, keepalive=(data, arr))

    @classmethod
    def open(cls, path: str) -> "File":
        h = C.c_void_p()
        check(_lib.lib().afhip_gguf_open(str(path).encode(), C.byref(h)))
        return cls(h.value)

    @property
    def handle(self):
        return self._h

    def close(self) -> None:
        if self._h:
            _lib.lib().afhip_gguf_close(self._h)
            self._h = None

    deinit = close

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    @staticmethod
    def _tensor(info: _lib.GgufTensorInfo) -> TensorInfo:
        return TensorInfo(
            name=_text(C.string_at(info.name, info.name_len)),
            dimensions=[int(info.dimensions[i]) for i in range(min(info.n_dimensions, _lib.GGUF_MAX_DIMS))],
            tensor_type=int(info.tensor_type), type_name=info.type_name.decode(),
            is_quantized=bool(info.is_quantized), offset=int(info.offset), data_offset=int(info.data_offset),
            byte_len=int(info.byte_len) or None)

    @property
    def tensors(self) -> List[TensorInfo]:
        out = []
        for i in range(self.header.tensor_count):
            info = _lib.GgufTensorInfo()
            check(_lib.lib().afhip_gguf_tensor_at(self._h, i, C.byref(info)))
            out.append(self._tensor(info))
        return out

    @staticmethod
    def _entry(m: _lib.GgufMetadata) -> MetadataEntry:
        t = int(m.value_type)
        if t == STRING:
            value = _text(C.string_at(m.str, m.str_len))
        elif t == ARRAY:
            return MetadataEntry(_text(C.string_at(m.key, m.key_len)), t, int(m.count), int(m.element_type))
        elif t in (F32, F64):
            value = float(m.f64)
        elif t == BOOL:
            value = bool(m.u64)
        elif t in (I8, I16, I32, I64):
            value = int(m.i64)
        else:
            value = int(m.u64)
        return MetadataEntry(_text(C.string_at(m.key, m.key_len)), t, value)

    @property
    def metadata(self) -> List[MetadataEntry]:
        out = []
        for i in range(self.header.metadata_count):
            m = _lib.GgufMetadata()
            check(_lib.lib().afhip_gguf_metadata_at(self._h, i, C.byref(m)))
            out.append(self._entry(m))
        return out

    def findMetadata(self, key: str) -> Optional[MetadataEntry]:
        m = _lib.GgufMetadata()
        rc = _lib.lib().afhip_gguf_find_metadata(self._h, _raw(key), C.byref(m))
        if rc == _lib.ERR_TENSOR_NOT_FOUND:
            return None
        check(rc)
        return self._entry(m)

    def tensorData(self, name: str) -> np.ndarray:
        """The tensor's raw bytes, copied out of the image (ErrTensorNotFound / UnexpectedEndOfFile as the C ABI)."""
        info = _lib.GgufTensorInfo()
        check(_lib.lib().afhip_gguf_find_tensor(self._h, _raw(name), C.byref(info)))
        ptr, n = C.c_void_p(), C.c_size_t()
        check(_lib.lib().afhip_gguf_tensor_data(self._h, C.byref(info), C.byref(ptr), C.byref(n)))
        return np.frombuffer(C.string_at(ptr.value, n.value), dtype=np.uint8)


class Catalog:
    """gguf/tensor_catalog.zig."""

    def __init__(self, file: File):
        self.file = file

    def count(self) -> int:
        return self.file.header.tensor_count

    def find(self, name: str) -> Optional[TensorInfo]:
        info = _lib.GgufTensorInfo()
        rc = _lib.lib().afhip_gguf_find_tensor(self.file.handle, _raw(name), C.byref(info))
        if rc == _lib.ERR_TENSOR_NOT_FOUND:
            return None
        check(rc)
        return File._tensor(info)
