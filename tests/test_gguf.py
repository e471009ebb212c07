"""The GGUF container through the C ABI (host code, no GPU): the reference's own parser
tests (gguf/format.zig:310-365, gguf/tensor_catalog.zig:35-57, gguf/tensor_types.zig:315-342)
re-stated on the same bytes, plus the error paths."""
import numpy as np
import pytest

from antfly_amd import _lib, gguf
from tests import gguf_util as W


def reference_minimal_file() -> bytes:
    # format.zig:310-336, byte for byte
    data = bytearray(b"GGUF" + W.le("I", 3) + W.le("Q", 1) + W.le("Q", 2))
    data += W.string("general.architecture") + W.le("I", gguf.STRING) + W.string("llama")
    data += W.string("general.alignment") + W.le("I", gguf.U32) + W.le("I", 64)
    data += W.string("tok_embeddings.weight") + W.le("I", 2) + W.le("Q", 8) + W.le("Q", 4) + W.le("I", 1) + W.le("Q", 0)
    while len(data) % 64:
        data.append(0)
    data += bytes(64)
    return bytes(data)


def test_parse_minimal_gguf_file_like_the_reference():
    with gguf.File.parse(reference_minimal_file()) as f:
        assert f.header.version == 3 and f.header.tensor_count == 1 and f.header.metadata_count == 2
        assert f.alignment == 64
        assert len(f.metadata) == 2
        t = f.tensors[0]
        assert t.name == "tok_embeddings.weight"
        assert f.data_region_offset == 192 and t.data_offset == 192
        assert t.dimensions == [8, 4] and t.shape == [4, 8] and t.type_name == "F16" and not t.is_quantized
        assert t.byte_len == 64
        assert f.findMetadata("general.architecture").value == "llama"
        assert f.findMetadata("general.alignment").value == 64
        assert f.findMetadata("missing") is None
        assert len(f.tensorData("tok_embeddings.weight")) == 64


def single_tensor_file(architecture: str, raw_type: int) -> bytes:
    # format.zig:367-390
    data = bytearray(b"GGUF" + W.le("I", 3) + W.le("Q", 1) + W.le("Q", 1))
    data += W.string("general.architecture") + W.le("I", gguf.STRING) + W.string(architecture)
    data += W.string("test.weight") + W.le("I", 2) + W.le("Q", 256) + W.le("Q", 4) + W.le("I", raw_type) + W.le("Q", 0)
    while len(data) % gguf.DEFAULT_ALIGNMENT:
        data.append(0)
    data += bytes(128)
    return bytes(data)


def test_tensor_type_39_by_architecture_dialect():
    with gguf.File.parse(single_tensor_file("llama", 39)) as f:
        assert f.tensors[0].type_name == "MXFP4" and f.alignment == 32
    with gguf.File.parse(single_tensor_file("bitnet-b1.58", 39)) as f:
        assert f.tensors[0].type_name == "TL2" and f.tensors[0].tensor_type == 39


def test_catalog_finds_tensor_by_name():
    img = W.build([], [("test.weight", [4, 8], 1, bytes(64))])
    with gguf.File.parse(img) as f:
        cat = gguf.Catalog(f)
        assert cat.count() == 1
        assert cat.find("test.weight") is not None and cat.find("test.weight").data_offset == f.data_region_offset
        assert cat.find("missing") is None


def test_byte_len_table():
    # the reference's own expectations, gguf/tensor_types.zig:315-342 ("tensor byte length for dense and k-quants")
    ref = [(0, [4], 16), (1, [4], 8), (24, [4], 4), (25, [4], 8), (26, [4], 16), (27, [4], 32), (28, [4], 32),
           (41, [128], 18), (36, [256], 96), (37, [256], 256), (38, [256], 96), (13, [256], 176), (20, [32], 18),
           (23, [256], 136), (16, [256], 66), (17, [256], 74), (18, [256], 98), (19, [256], 50), (21, [256], 110),
           (22, [256], 82), (29, [256], 56), (34, [256], 54), (35, [256], 66), (39, [32], 17), (40, [64], 36)]
    for raw, dims, want in ref:
        assert gguf.byteLen(raw, dims) == want, raw
    assert gguf.byteLen(39, [6912, 4], bitnet_dialect=True) == 5856      # TL2
    assert gguf.byteLen(39, [128, 4], bitnet_dialect=True) is None
    # the shapes of this library's own path
    assert gguf.byteLen(2, [4096, 14336]) == 33030144       # Q4_0 FFN matrix
    assert gguf.byteLen(8, [4096, 4096]) == 17825792        # Q8_0
    assert gguf.byteLen(12, [256, 10]) == 1440              # Q4_K: 144 bytes per 256 values
    assert gguf.byteLen(8, [33]) == 68                      # a partial block still takes a whole one
    assert gguf.byteLen(4, [32]) is None and gguf.byteLen(9999, [32]) is None   # ids the table does not hold
    assert gguf.byteLen(0, [2 ** 40, 2 ** 40]) is None      # overflow


def test_metadata_value_types_and_arrays():
    md = [("a.u8", gguf.U8, 200), ("a.i8", gguf.I8, -5), ("a.u16", gguf.U16, 60000), ("a.i16", gguf.I16, -30000),
          ("a.u32", gguf.U32, 4000000000), ("a.i32", gguf.I32, -7), ("a.f32", gguf.F32, 0.5), ("a.bool", gguf.BOOL, 1),
          ("a.str", gguf.STRING, "héllo"), ("a.u64", gguf.U64, 2 ** 63 + 1), ("a.i64", gguf.I64, -2 ** 62),
          ("a.f64", gguf.F64, 1e300), ("a.arr", gguf.ARRAY, (gguf.STRING, ["x", "yy", "zzz"])),
          ("a.nums", gguf.ARRAY, (gguf.I32, [1, 2, 3, 4]))]
    with gguf.File.parse(W.build(md, [])) as f:
        got = {e.key: e for e in f.metadata}
        for key, vtype, v in md:
            if vtype == gguf.ARRAY:
                assert got[key].value == len(v[1]) and got[key].element_type == v[0]
            else:
                assert got[key].value_type == vtype and got[key].value == v, key
        assert f.alignment == gguf.DEFAULT_ALIGNMENT and f.header.tensor_count == 0


def test_parser_errors():
    good = reference_minimal_file()
    with pytest.raises(_lib.InvalidGgufMagic):
        gguf.File.parse(b"GGML" + good[4:])
    for cut in (0, 3, 10, 23, 40, 100, 150):  # inside the magic, the header, a key, a value, a tensor info
        with pytest.raises(_lib.UnexpectedEndOfFile):
            gguf.File.parse(good[:cut])
    with pytest.raises(_lib.UnsupportedMetadataType):
        gguf.File.parse(b"GGUF" + W.le("I", 3) + W.le("Q", 0) + W.le("Q", 1) + W.string("k") + W.le("I", 13) + bytes(8))
    nested = b"GGUF" + W.le("I", 3) + W.le("Q", 0) + W.le("Q", 1) + W.string("k") + W.le("I", gguf.ARRAY) + \
        W.le("I", gguf.ARRAY) + W.le("Q", 0)
    with pytest.raises(_lib.UnsupportedNestedMetadataArray):
        gguf.File.parse(nested)
    # counts that no file of this size can hold
    with pytest.raises(_lib.UnexpectedEndOfFile):
        gguf.File.parse(b"GGUF" + W.le("I", 3) + W.le("Q", 2 ** 60) + W.le("Q", 0))
    # a tensor whose bytes run past the end of the image
    img = W.build([], [("w", [64, 2], 8, bytes(136))])
    with gguf.File.parse(img[:-40]) as f:
        with pytest.raises(_lib.UnexpectedEndOfFile):
            f.tensorData("w")
        with pytest.raises(_lib.TensorNotFound):
            f.tensorData("nope")
    # a tensor offset that wraps 64 bits when the data region's start is added would land back inside the image
    with gguf.File.parse(img) as f:
        region = f.data_region_offset
    at = img.index(W.le("I", 8) + W.le("Q", 0)) + 4       # the offset field of "w" (type 8, offset 0)
    for offset in (2 ** 64 - region, 2 ** 64 - region + 32, 2 ** 64 - 1):
        with pytest.raises(_lib.UnexpectedEndOfFile):
            gguf.File.parse(img[:at] + W.le("Q", offset) + img[at + 8:])


def test_truncated_and_corrupted_images_fail_cleanly():
    """Every prefix of a valid image and seeded byte corruptions of its header region either
    parse (and then every tensor / metadata accessor works or reports an error) or raise one
    of the library's errors; nothing reads outside the image."""
    rng = np.random.default_rng(7)
    img = W.build([("general.architecture", gguf.STRING, "llama"), ("n", gguf.U32, 7),
                   ("toks", gguf.ARRAY, (gguf.STRING, ["a", "bc", "def"]))],
                  [("a.weight", [64, 4], 2, bytes(4 * 2 * 18)), ("b.weight", [64, 4], 8, bytes(4 * 2 * 34)),
                   ("n.weight", [64], 0, bytes(256))])
    with gguf.File.parse(img) as whole:
        header = whole.data_region_offset

    def walk(image):
        try:
            with gguf.File.parse(image) as f:
                for t in f.tensors:
                    try:
                        data = f.tensorData(t.name)
                        assert len(data) == t.byte_len
                    except _lib.HipError:
                        pass
                assert len(f.metadata) == f.header.metadata_count
            return True
        except _lib.HipError:
            return False

    assert walk(img)
    results = [walk(img[:cut]) for cut in range(header)]  # a cut anywhere is an error or a parse, never a crash
    infos_end = results.index(True) if True in results else header
    assert infos_end > header - gguf.DEFAULT_ALIGNMENT  # only cuts inside the alignment padding still parse
    assert all(results[infos_end:])
    parsed = 0
    for _ in range(3000):
        b = bytearray(img)
        for _ in range(int(rng.integers(1, 4))):
            pos = int(rng.integers(0, header))
            kind = int(rng.integers(0, 3))
            if kind == 0:
                b[pos] = int(rng.integers(0, 256))
            elif kind == 1:
                b[pos] ^= 1 << int(rng.integers(0, 8))
            else:
                b[pos:pos + 8] = [0, 2 ** 64 - 1, 2 ** 63, 2 ** 32 - 1, 2 ** 31][int(rng.integers(0, 5))].to_bytes(8, "little")[:len(b) - pos]
        parsed += walk(bytes(b))
    assert 0 < parsed < 3000


def test_open_maps_a_file(tmp_path):
    blocks = np.arange(2 * 2 * 34, dtype=np.uint8)
    img = W.build([("general.architecture", gguf.STRING, "llama")],
                  [("blk.0.attn_q.weight", [64, 2], 8, blocks.tobytes()), ("tail", [3], 0, np.float32([1, 2, 3]).tobytes())])
    path = tmp_path / "tiny.gguf"
    path.write_bytes(img)
    with gguf.File.open(str(path)) as f:
        assert f.file_len == len(img) and [t.name for t in f.tensors] == ["blk.0.attn_q.weight", "tail"]
        q = f.tensors[0]
        assert q.shape == [2, 64] and q.type_name == "Q8_0" and q.is_quantized and q.byte_len == 136
        assert np.array_equal(f.tensorData("blk.0.attn_q.weight"), blocks)
        assert f.tensors[1].data_offset % 32 == 0
        assert np.array_equal(f.tensorData("tail").view(np.float32), np.float32([1, 2, 3]))
    with pytest.raises(_lib.FileNotAccessible):
        gguf.File.open(str(tmp_path / "missing.gguf"))
    empty = tmp_path / "empty.gguf"
    empty.write_bytes(b"")
    with pytest.raises(_lib.UnexpectedEndOfFile):
        gguf.File.open(str(empty))
