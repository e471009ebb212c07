"""Builds GGUF images for the tests, field by field as the reference's own tests do
(gguf/format.zig:310-400: magic, version, counts, metadata entries, tensor infos,
padding to the alignment, tensor data)."""
import struct

import numpy as np

from antfly_amd import gguf


def le(fmt, v):
    return struct.pack("<" + fmt, v)


def string(s) -> bytes:
    b = s if isinstance(s, bytes) else s.encode()
    return le("Q", len(b)) + b


_SCALAR = {gguf.U8: "B", gguf.I8: "b", gguf.U16: "H", gguf.I16: "h", gguf.U32: "I", gguf.I32: "i", gguf.F32: "f",
           gguf.BOOL: "B", gguf.U64: "Q", gguf.I64: "q", gguf.F64: "d"}


def value(vtype, v) -> bytes:
    if vtype == gguf.STRING:
        return string(v)
    if vtype == gguf.ARRAY:
        elem_type, items = v
        return le("I", elem_type) + le("Q", len(items)) + b"".join(value(elem_type, x) for x in items)
    return le(_SCALAR[vtype], v)


def build(metadata, tensors, alignment=None, version=3) -> bytes:
    """metadata: [(key, value_type, value)]; tensors: [(name, dims (fastest first), raw_type, bytes)].
    Tensor data is laid out in order, each tensor padded to the alignment."""
    align = alignment if alignment is not None else gguf.DEFAULT_ALIGNMENT
    out = bytearray(gguf.MAGIC + le("I", version) + le("Q", len(tensors)) + le("Q", len(metadata)))
    for key, vtype, v in metadata:
        out += string(key) + le("I", vtype) + value(vtype, v)
    offset, offsets = 0, []
    for _, _, _, data in tensors:
        offsets.append(offset)
        offset += len(data)
        offset += (-offset) % max(align, 1)
    for (name, dims, raw_type, _), off in zip(tensors, offsets):
        out += string(name) + le("I", len(dims)) + b"".join(le("Q", d) for d in dims) + le("I", raw_type) + le("Q", off)
    out += b"\0" * ((-len(out)) % max(align, 1))
    for _, _, _, data in tensors:
        out += bytes(np.asarray(data, dtype=np.uint8).tobytes()) if not isinstance(data, (bytes, bytearray)) else data
        out += b"\0" * ((-len(out)) % max(align, 1))
    return bytes(out)
