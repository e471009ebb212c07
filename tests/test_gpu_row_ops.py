"""GPU parity for the row operators on quantized tensors (get_rows = embedding lookup,
cpy_q_to_f32, cpy_f32_to_q, set_rows), through the C ABI, against the CPU oracle's
dequantizers and weight quantizers.  Everything here is bit-exact: one f32 multiply
per value on the way out, integer codes and an f16 scale on the way in."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")

from antfly_amd import _lib, kernels, synth  # noqa: E402
from antfly_amd.hip_compute import HipCompute  # noqa: E402
from oracle import oracle as O  # noqa: E402
from tests import gpu_util as G  # noqa: E402

Q4, Q8, F32 = _lib.TYPE_Q4_0, _lib.TYPE_Q8_0, _lib.TYPE_F32
RAW, PREP = _lib.LAYOUT_RAW, _lib.LAYOUT_PREPARED


def bits(a):
    return np.ascontiguousarray(a, np.float32).view(np.uint32)


def weights_with_odd_scales(fmt, seed, rows, dim):
    """Synthetic blocks whose fp16 scales also cover subnormals, zero and the largest finite half."""
    w = synth.weights(fmt, seed, rows, dim).copy()
    blocks = w.reshape(-1, O.BLOCK_BYTES[fmt])
    odd = np.array([0x0001, 0x03FF, 0x0400, 0x0000, 0x8000, 0x7BFF, 0xFBFF, 0x3C00], dtype=np.uint16)
    n = min(len(odd), blocks.shape[0])
    blocks[:n, 0:2] = odd[:n].view(np.uint8).reshape(n, 2)
    return w


@pytest.mark.parametrize("fmt", [Q8, Q4])
@pytest.mark.parametrize("layout", [RAW, PREP])
@pytest.mark.parametrize("rows,dim", [(3, 64), (7, 4096), (33, 288)])
def test_dequantize_whole_tensor_bit_exact(fmt, layout, rows, dim):
    print(f"case: cpy_q_to_f32 fmt={fmt} layout={layout} rows={rows} dim={dim}", flush=True)
    w = weights_with_odd_scales(fmt, 3, rows, dim)
    wd = G.prepare(fmt, w, rows, dim) if layout == PREP else G.to_dev(w)
    out = torch.full((rows, dim), float("nan"), dtype=torch.float32, device=G.DEV)
    kernels.launchDequantizeF32(G.stream(), fmt, layout, G.buf(out), G.buf(wd), rows, dim)
    torch.cuda.synchronize()
    want = O.dequantize(fmt, w).reshape(rows, dim)
    assert np.array_equal(bits(out.cpu().numpy()), bits(want))


@pytest.mark.parametrize("fmt", [Q8, Q4])
@pytest.mark.parametrize("layout", [RAW, PREP])
def test_embedding_lookup_bit_exact(fmt, layout):
    vocab, dim = 500, 1024
    print(f"case: get_rows fmt={fmt} layout={layout}", flush=True)
    w = weights_with_odd_scales(fmt, 4, vocab, dim)
    wd = G.prepare(fmt, w, vocab, dim) if layout == PREP else G.to_dev(w)
    ids = np.array([499, 0, 7, 7, 123, 0, 498, 1, 250], dtype=np.int64)
    idd = G.to_dev(ids)
    out = torch.full((len(ids), dim), float("nan"), dtype=torch.float32, device=G.DEV)
    kernels.launchEmbeddingLookupF32(G.stream(), fmt, layout, G.buf(out), G.buf(wd), G.buf(idd), len(ids), dim, vocab)
    torch.cuda.synchronize()
    table = O.dequantize(fmt, w).reshape(vocab, dim)
    assert np.array_equal(bits(out.cpu().numpy()), bits(table[ids]))


def test_embedding_lookup_dense_table_and_checks():
    vocab, dim = 40, 100  # a dense table needs no multiple of 32
    table = synth.activations(5, vocab, dim)
    td = G.to_dev(table)
    ids = np.array([39, 3, 3, 0], dtype=np.int64)
    idd = G.to_dev(ids)
    out = torch.empty((4, dim), dtype=torch.float32, device=G.DEV)
    kernels.launchEmbeddingLookupF32(G.stream(), F32, RAW, G.buf(out), G.buf(td), G.buf(idd), 4, dim, vocab)
    torch.cuda.synchronize()
    assert np.array_equal(out.cpu().numpy(), table[ids])
    w = G.to_dev(synth.weights(Q8, 1, 4, 64))
    o = torch.empty((2, 64), dtype=torch.float32, device=G.DEV)
    with pytest.raises(_lib.InvalidHipState):  # a quantized row is whole blocks
        kernels.launchEmbeddingLookupF32(G.stream(), Q8, RAW, G.buf(o), G.buf(w), G.buf(idd), 2, 48, 4)
    with pytest.raises(_lib.InvalidHipState):  # short id buffer
        kernels.launchEmbeddingLookupF32(G.stream(), Q8, RAW, G.buf(o), G.buf(w), G.buf(idd[:1]), 2, 64, 4)
    with pytest.raises(_lib.UnsupportedTensorType):
        kernels.launchEmbeddingLookupF32(G.stream(), 14, RAW, G.buf(o), G.buf(w), G.buf(idd), 2, 64, 4)


def rows_for_quantizer(seed, rows, dim):
    """Values that exercise the quantizers: normal data, a zero block, exact ties, huge and tiny blocks."""
    x = synth.activations(seed, rows, dim)
    b = x.reshape(-1, 32)
    b[1] = 0.0
    b[2] = 0.0
    b[2, :8] = [127.0, 0.5, -0.5, 1.5, -1.5, 126.5, -2.5, 63.5]     # Q8_0: scale 1, ties away from zero
    b[3] = 0.0
    b[3, :8] = [8.0, 0.5, -0.5, 1.5, -1.5, 7.5, -7.5, -8.0]         # Q4_0: scale 1
    b[4] *= np.float32(3.0e4)                                         # scale near the top of fp16
    b[5] *= np.float32(1.0e-6)                                        # subnormal fp16 scale
    b[6] *= np.float32(1.0e-9)                                        # scale rounds to zero in fp16
    b[7, :] = np.float32(-2.5)                                        # every value the (negative) maximum
    return x


@pytest.mark.parametrize("fmt", [Q8, Q4])
@pytest.mark.parametrize("rows,dim", [(1, 32), (4, 256), (9, 4096), (5, 1024), (7, 3072), (1, 2048)])  # (the last three: a ragged last group of 1024-value runs)
def test_quantize_rows_matches_weight_quantizers(fmt, rows, dim):
    print(f"case: cpy_f32_to_q fmt={fmt} rows={rows} dim={dim}", flush=True)
    x = rows_for_quantizer(6, rows, dim) if rows * dim >= 256 else synth.activations(6, rows, dim)
    xd = G.to_dev(x)
    nbytes = rows * dim // 32 * O.BLOCK_BYTES[fmt]
    out = torch.full((nbytes + 2,), 0xEE, dtype=torch.uint8, device=G.DEV)
    kernels.launchQuantizeRows(G.stream(), fmt, G.buf(out[:nbytes]), G.buf(xd), rows, dim)
    torch.cuda.synchronize()
    got = out.cpu().numpy()
    assert got[nbytes] == 0xEE and got[nbytes + 1] == 0xEE
    want = O.quantize_weights(fmt, x)
    assert np.array_equal(got[:nbytes], want)


@pytest.mark.parametrize("fmt", [Q8, Q4])
def test_set_rows_scatters_whole_rows(fmt):
    dst_rows, dim = 10, 128
    x = synth.activations(8, 3, dim)
    ids = np.array([9, 0, 4], dtype=np.int64)
    row_bytes = dim // 32 * O.BLOCK_BYTES[fmt]
    out = torch.full((dst_rows * row_bytes,), 0xEE, dtype=torch.uint8, device=G.DEV)
    xd, idd = G.to_dev(x), G.to_dev(ids)  # both stay alive until the kernel has run
    kernels.launchQuantizeRows(G.stream(), fmt, G.buf(out), G.buf(xd), 3, dim, G.buf(idd), dst_rows)
    torch.cuda.synchronize()
    got = out.cpu().numpy().reshape(dst_rows, row_bytes)
    want = O.quantize_weights(fmt, x).reshape(3, row_bytes)
    for t, r in enumerate(ids):
        assert np.array_equal(got[r], want[t])
    untouched = [r for r in range(dst_rows) if r not in ids]
    assert (got[untouched] == 0xEE).all()


@pytest.mark.parametrize("fmt", [Q8, Q4])
def test_set_rows_on_whole_runs_aligned_and_not(fmt):
    """Rows of whole 1024-value runs take the kernel that stores 16 bytes at a time: scattered rows, row ids outside the
    destination, and a destination that is not 16-byte aligned (which falls back to the piecewise kernel) give the same bytes."""
    dst_rows, dim = 7, 2048
    x = rows_for_quantizer(18, 5, dim)
    ids = np.array([6, -1, 2, dst_rows, 0], dtype=np.int64)
    row_bytes = dim // 32 * O.BLOCK_BYTES[fmt]
    want = O.quantize_weights(fmt, x).reshape(5, row_bytes)
    xd, idd = G.to_dev(x), G.to_dev(ids)
    for shift in (0, 2):
        print(f"case: set_rows on runs fmt={fmt} destination offset {shift}", flush=True)
        canvas = torch.full((16 + (dst_rows + 2) * row_bytes,), 0xC3, dtype=torch.uint8, device=G.DEV)
        dst = canvas[shift + row_bytes : shift + (dst_rows + 1) * row_bytes]
        kernels.launchQuantizeRows(G.stream(), fmt, G.buf(dst), G.buf(xd), 5, dim, row_ids_i64=G.buf(idd), dst_rows=dst_rows)
        torch.cuda.synchronize()
        got = canvas.cpu().numpy()[shift : shift + (dst_rows + 2) * row_bytes].reshape(dst_rows + 2, row_bytes)
        assert np.array_equal(got[1 + 6], want[0]) and np.array_equal(got[1 + 2], want[2]) and np.array_equal(got[1 + 0], want[4])
        assert (got[[0, 2, 4, 5, 6, dst_rows + 1]] == 0xC3).all()  # canaries and the rows nobody addressed


def test_quantize_then_dequantize_full_size_properties():
    """A whole FFN matrix (14336 x 4096 values): Q8_0 codes survive dequantize -> quantize unchanged
    (max |q| = 127 makes the recomputed scale the stored one), and the matmul on the device-quantized
    weights equals the matmul on the oracle-quantized ones."""
    rows, dim = 14336, 4096
    x = synth.activations(12, 512, dim)
    x = np.tile(x, (rows // 512, 1)) * np.linspace(0.5, 2.0, rows, dtype=np.float32)[:, None]
    xd = G.to_dev(x)
    nbytes = rows * dim // 32 * 34
    q = torch.empty(nbytes, dtype=torch.uint8, device=G.DEV)
    kernels.launchQuantizeRows(G.stream(), Q8, G.buf(q), G.buf(xd), rows, dim)
    back = torch.empty((rows, dim), dtype=torch.float32, device=G.DEV)
    kernels.launchDequantizeF32(G.stream(), Q8, RAW, G.buf(back), G.buf(q), rows, dim)
    q2 = torch.empty_like(q)
    kernels.launchQuantizeRows(G.stream(), Q8, G.buf(q2), G.buf(back), rows, dim)
    torch.cuda.synchronize()
    assert torch.equal(q, q2)
    sample = slice(0, 64 * dim // 32 * 34)
    assert np.array_equal(q.cpu().numpy()[sample], O.quantize_weights(Q8, x[:64]))
    err = (back - xd).abs().amax(dim=1) / xd.abs().amax(dim=1)
    assert float(err.max()) <= 0.5 / 127 + 1e-3  # half a step of the block's scale, plus the f16 rounding of the scale


def test_backend_embedding_lookup(kats):
    vocab, dim = 300, 512
    with HipCompute() as cb:
        for fmt in (Q8, Q4):
            print(f"case: backend embeddingLookup fmt={fmt}", flush=True)
            w = synth.weights(fmt, 17, vocab, dim)
            for keep_raw in (False, True):
                name = f"token_embd.{fmt}.{keep_raw}"
                cb.insertWeightFromLoaded(name, fmt, w, [vocab, dim], keep_raw_layout=keep_raw)
                wt = cb.getWeight(name)
                ids = [5, 299, 0, 5]
                out = cb.embeddingLookup(wt, ids, 4, dim)
                assert out.shape == [4, dim] and out.dtype == _lib.DTYPE_F32
                table = O.dequantize(fmt, w).reshape(vocab, dim)
                assert np.array_equal(bits(cb.toFloat32(out).reshape(4, dim)), bits(table[ids]))
                cb.freeTensor(out)
                with pytest.raises(_lib.InvalidTokenId):
                    cb.embeddingLookup(wt, [0, vocab], 2, dim)
                with pytest.raises(_lib.InvalidTokenId):
                    cb.embeddingLookup(wt, [-1], 1, dim)
                with pytest.raises(_lib.InvalidShape):
                    cb.embeddingLookup(wt, [1, 2], 3, dim)
                with pytest.raises(_lib.InvalidShape):
                    cb.embeddingLookup(wt, [1], 1, 500)
        dense = synth.activations(18, 20, 48)
        cb.insertWeightFromTensor("pos_embd", dense, [20, 48])
        out = cb.embeddingLookup(cb.getWeight("pos_embd"), [19, 0], 2, 48)
        assert np.array_equal(cb.toFloat32(out).reshape(2, 48), dense[[19, 0]])


@pytest.mark.parametrize("fmt", [Q8, Q4])
def test_row_ids_outside_the_tensor_touch_nothing(fmt):
    """get_rows: an id outside [0, vocab) comes out as a row of zeros; set_rows: a row id outside
    [0, dst_rows) is skipped.  Neither reads nor writes outside the tensors (the kernels check:
    the launcher has no way to)."""
    vocab, dim = 12, 256
    w = synth.weights(fmt, 61, vocab, dim)
    ids = np.array([3, -1, vocab, 11, 1 << 40], dtype=np.int64)
    for layout in (RAW, PREP):
        wd = G.prepare(fmt, w, vocab, dim) if layout == PREP else G.to_dev(w)
        out = torch.full((ids.size, dim), float("nan"), dtype=torch.float32, device=G.DEV)
        ids_d = G.to_dev(ids)
        kernels.launchEmbeddingLookupF32(G.stream(), fmt, layout, G.buf(out), G.buf(wd), G.buf(ids_d), ids.size, dim, vocab)
        torch.cuda.synchronize()
        got = out.cpu().numpy()
        dense = O.dequantize(fmt, w).reshape(vocab, dim)
        assert np.array_equal(got[0], dense[3]) and np.array_equal(got[3], dense[11])
        assert not got[[1, 2, 4]].any()
    # set_rows into a 6-row destination guarded by canaries on both sides
    dst_rows, bb = 6, (18 if fmt == Q4 else 34)
    row_bytes = dim // 32 * bb
    x = synth.activations(62, 4, dim)
    canvas = torch.full(((dst_rows + 2) * row_bytes,), 0xAB, dtype=torch.uint8, device=G.DEV)
    dst = canvas[row_bytes : (dst_rows + 1) * row_bytes]
    rid = np.array([5, -2, dst_rows, 0], dtype=np.int64)
    x_d, rid_d = G.to_dev(x), G.to_dev(rid)  # (kept alive until the launch has run)
    kernels.launchQuantizeRows(G.stream(), fmt, G.buf(dst), G.buf(x_d), 4, dim, row_ids_i64=G.buf(rid_d), dst_rows=dst_rows)
    torch.cuda.synchronize()
    got = canvas.cpu().numpy().reshape(dst_rows + 2, row_bytes)
    want = O.quantize_weights(fmt, x).reshape(4, row_bytes)
    assert np.array_equal(got[1 + 5], want[0]) and np.array_equal(got[1 + 0], want[3])
    untouched = [0, 2, 3, 4, 5, dst_rows + 1]  # canaries and the rows nobody addressed
    assert (got[untouched] == 0xAB).all()


@pytest.mark.parametrize("nbytes", [16, 4096 + 16, 1 << 20, (1 << 20) + 7])
def test_stream_copy_copies_whole_16_byte_units(nbytes):
    """The diagnostic copy kernel (the calibrator of the write counter): dst = src over the
    whole 16-byte units of src.len, nothing past them, and a too-short dst is refused."""
    print(f"case: stream_copy nbytes={nbytes}", flush=True)
    rng = np.random.default_rng(nbytes)
    src = G.to_dev(rng.integers(0, 256, nbytes + 16, dtype=np.uint8))
    dst = torch.full((nbytes + 64,), 0xAB, dtype=torch.uint8, device="cuda")
    kernels.launchStreamCopy(G.stream(), _lib.Buffer(src.data_ptr(), nbytes), G.buf(dst))
    torch.cuda.synchronize()
    n = nbytes // 16 * 16
    assert torch.equal(dst[:n], src[:n])
    assert bool((dst[n:] == 0xAB).all())
    with pytest.raises(_lib.HipError):
        kernels.launchStreamCopy(G.stream(), _lib.Buffer(src.data_ptr(), nbytes), _lib.Buffer(dst.data_ptr(), n - 16))
