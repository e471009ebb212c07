"""GPU parity for GGUF Q4_K (144-byte super-blocks), through the C ABI, against the CPU
oracle.  The engine computes this format in f32 on the dequantized weights and its own
outputs depend on its vector width, so the matmul is held to a tolerance: max-relative
error <= 1e-3 stated, <= 2e-5 in practice (against the oracle's f32 sum and its f64 sum).
Dequantization (get_rows, cpy_q_to_f32) is bit-exact."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")

from antfly_amd import _lib, kernels, synth  # noqa: E402
from antfly_amd.hip_compute import HipCompute  # noqa: E402
from oracle import oracle as O  # noqa: E402
from tests import gpu_util as G  # noqa: E402

Q4K = _lib.TYPE_Q4_K
RAW, PREP = _lib.LAYOUT_RAW, _lib.LAYOUT_PREPARED
TOL, TIGHT = 1e-3, 2e-5


def device_weight(layout, w, out_dim, in_dim):
    return G.prepare(Q4K, w, out_dim, in_dim) if layout == PREP else G.to_dev(w)


def q4k_block(d_bits, dmin_bits, scales12, qs128):
    return np.concatenate([np.array([d_bits, dmin_bits], np.uint16).view(np.uint8), np.asarray(scales12, np.uint8),
                           np.asarray(qs128, np.uint8)])


def test_reference_vectors(kats):
    k = kats["q4_k"]
    u = k["uniform_block"]
    scales = [u["scales_first4"]] * 4 + [0] * 4 + [u["scales_last4"]] * 4
    m = k["direct_matmul"]
    print("case: q4_k direct matmul kat", flush=True)
    w = np.concatenate([q4k_block(15360, 0, scales, [f] * 128) for f in m["row_qs_fill"]])
    x = np.full((1, m["in_dim"]), m["input_fill"], np.float32)
    for layout in (RAW, PREP):
        y = G.linear(Q4K, layout, x, device_weight(layout, w, m["out_dim"], m["in_dim"]), 1, m["in_dim"], m["out_dim"])
        assert np.abs(y[0] - np.array(m["expected"])).max() <= m["tolerance_abs"]
    h = k["header_packing"]
    print("case: q4_k header packing kat", flush=True)
    raw = np.array(h["header"] + h["qs_32"] * 4, np.uint8)
    want = np.array([h["scs"][sub] * (i % 16) - h["mins"][sub] for sub in range(8) for i in range(32)], np.float32)
    for layout in (RAW, PREP):
        out = torch.empty(256, dtype=torch.float32, device=G.DEV)
        wd = device_weight(layout, raw, 1, 256)
        kernels.launchDequantizeF32(G.stream(), Q4K, layout, G.buf(out), G.buf(wd), 1, 256)
        torch.cuda.synchronize()
        assert np.array_equal(out.cpu().numpy(), want)


@pytest.mark.parametrize("out_dim,in_dim", [(1, 256), (32, 512), (45, 1024), (100, 4096)])
def test_tile_major_repack_is_a_pure_permutation(out_dim, in_dim):
    print(f"case: q4_k tile-major repack out={out_dim} in={in_dim}", flush=True)
    w = synth.weights(Q4K, 3, out_dim, in_dim)
    want = G.numpy_prepare_q4k(w, out_dim, in_dim)
    assert kernels.preparedWeightBytes(Q4K, out_dim, in_dim) == want.size == (out_dim + 31) // 32 * (in_dim // 256) * 4608
    got = G.prepare(Q4K, w, out_dim, in_dim).cpu().numpy()
    assert np.array_equal(got, want)
    if out_dim % 32 == 0:
        assert np.array_equal(np.sort(got), np.sort(w))  # same bytes, other places


@pytest.mark.parametrize("layout", [RAW, PREP])
@pytest.mark.parametrize("rows,dim", [(1, 256), (5, 1024), (3, 4096), (40, 512)])
def test_dequantize_and_get_rows_bit_exact(rows, dim, layout):
    print(f"case: q4_k cpy_q_to_f32 / get_rows rows={rows} dim={dim} layout={layout}", flush=True)
    vocab = rows + 7
    w = synth.weights(Q4K, 2, vocab, dim).copy()
    w[0:4] = np.array([0x0001, 0x7BFF], np.uint16).view(np.uint8)  # subnormal d, largest finite dmin
    wd = device_weight(layout, w, vocab, dim)
    table = O.dequantize_q4_k(w).reshape(vocab, dim)
    out = torch.empty((vocab, dim), dtype=torch.float32, device=G.DEV)
    kernels.launchDequantizeF32(G.stream(), Q4K, layout, G.buf(out), G.buf(wd), vocab, dim)
    torch.cuda.synchronize()
    assert np.array_equal(out.cpu().numpy().view(np.uint32), table.view(np.uint32))
    ids = np.array([vocab - 1, 0, 3, 3][:rows + 1], dtype=np.int64)
    idd = G.to_dev(ids)
    emb = torch.empty((len(ids), dim), dtype=torch.float32, device=G.DEV)
    kernels.launchEmbeddingLookupF32(G.stream(), Q4K, layout, G.buf(emb), G.buf(wd), G.buf(idd), len(ids), dim, vocab)
    torch.cuda.synchronize()
    assert np.array_equal(emb.cpu().numpy().view(np.uint32), table[ids].view(np.uint32))


def values_for_q4k_quantizer(seed, rows, dim):
    """Normal data of mixed magnitudes, a zero sub-block, a zero super-block, one-signed sub-blocks, exact ties."""
    rng = np.random.default_rng(seed)
    x = (rng.standard_normal((rows * dim // 32, 32)) * np.exp2(rng.integers(-10, 10, (rows * dim // 32, 1)))).astype(np.float32)
    x[1] = 0.0
    x[3] = np.abs(x[3])
    x[4] = -np.abs(x[4])
    x[5] = np.round(x[5] * 4) / 4
    x[6, :] = np.float32(-2.5)
    if x.shape[0] >= 24:
        x[8:16] = 0.0
        x[16:24] = np.abs(x[16:24])  # no minimum in the whole super-block: dmin = 1, m = 0
    return x.reshape(rows, dim)


@pytest.mark.parametrize("rows,dim", [(1, 256), (3, 1024), (9, 4096), (130, 512)])
def test_quantize_rows_matches_weight_quantizer(rows, dim, kats):
    print(f"case: q4_k cpy_f32_to_q rows={rows} dim={dim}", flush=True)
    x = values_for_q4k_quantizer(31, rows, dim)
    if dim == 256:  # the block whose bytes the reference's own test fixes (gguf/quant_codec.zig:2925-2955)
        h = kats["q4_k"]["header_packing"]
        x = np.array([h["scs"][sub] * (i % 16) - h["mins"][sub] for sub in range(8) for i in range(32)], np.float32).reshape(1, 256)
    xd = G.to_dev(x)
    nbytes = rows * dim // 256 * 144
    out = torch.full((nbytes + 16,), 0xEE, dtype=torch.uint8, device=G.DEV)
    kernels.launchQuantizeRows(G.stream(), Q4K, G.buf(out[:nbytes]), G.buf(xd), rows, dim)
    torch.cuda.synchronize()
    got = out.cpu().numpy()
    assert (got[nbytes:] == 0xEE).all()
    assert np.array_equal(got[:nbytes], O.quantize_q4_k(x))
    if dim == 256:
        assert got[:nbytes].tolist() == h["header"] + h["qs_32"] * 4
    # and back: the dequantized bytes are the oracle's dequantization of the same bytes
    back = torch.empty((rows, dim), dtype=torch.float32, device=G.DEV)
    kernels.launchDequantizeF32(G.stream(), Q4K, RAW, G.buf(back), G.buf(out[:nbytes]), rows, dim)
    torch.cuda.synchronize()
    assert np.array_equal(back.cpu().numpy().view(np.uint32), O.dequantize_q4_k(got[:nbytes]).reshape(rows, dim).view(np.uint32))


def test_set_rows_scatters_and_skips_rows_outside():
    dst_rows, dim = 6, 512
    row_bytes = dim // 256 * 144
    x = values_for_q4k_quantizer(32, 4, dim)
    canvas = torch.full(((dst_rows + 2) * row_bytes,), 0xAB, dtype=torch.uint8, device=G.DEV)
    dst = canvas[row_bytes:(dst_rows + 1) * row_bytes]
    rid = np.array([5, -2, dst_rows, 0], dtype=np.int64)
    x_d, rid_d = G.to_dev(x), G.to_dev(rid)  # (kept alive until the launch has run)
    kernels.launchQuantizeRows(G.stream(), Q4K, G.buf(dst), G.buf(x_d), 4, dim, row_ids_i64=G.buf(rid_d), dst_rows=dst_rows)
    torch.cuda.synchronize()
    got = canvas.cpu().numpy().reshape(dst_rows + 2, row_bytes)
    want = O.quantize_q4_k(x).reshape(4, row_bytes)
    assert np.array_equal(got[1 + 5], want[0]) and np.array_equal(got[1 + 0], want[3])
    assert (got[[0, 2, 3, 4, 5, dst_rows + 1]] == 0xAB).all()
    with pytest.raises(_lib.InvalidHipState):  # a row is whole super-blocks
        kernels.launchQuantizeRows(G.stream(), Q4K, G.buf(dst), G.buf(x_d), 4, 288)
    with pytest.raises(_lib.InvalidHipState):  # destination too short
        kernels.launchQuantizeRows(G.stream(), Q4K, G.buf(dst[:row_bytes]), G.buf(x_d), 4, dim)


def test_quantize_full_size_round_trip_properties():
    """A whole FFN matrix (14336 x 4096): every value comes back within half a nibble step of its sub-block plus
    the 6-bit rounding of the sub-block's scale and minimum; the first rows equal the oracle's bytes."""
    rows, dim = 14336, 4096
    x = synth.activations(12, 512, dim)
    x = np.tile(x, (rows // 512, 1)) * np.linspace(0.5, 2.0, rows, dtype=np.float32)[:, None]
    xd = G.to_dev(x)
    q = torch.empty(rows * dim // 256 * 144, dtype=torch.uint8, device=G.DEV)
    kernels.launchQuantizeRows(G.stream(), Q4K, G.buf(q), G.buf(xd), rows, dim)
    back = torch.empty((rows, dim), dtype=torch.float32, device=G.DEV)
    kernels.launchDequantizeF32(G.stream(), Q4K, RAW, G.buf(back), G.buf(q), rows, dim)
    torch.cuda.synchronize()
    assert np.array_equal(q[:16 * dim // 256 * 144].cpu().numpy(), O.quantize_q4_k(x[:16]))
    sub = xd.view(rows, dim // 256, 8, 32)
    mins = (-sub.amin(dim=3)).clamp_min(0)
    span = sub.amax(dim=3) + mins
    bound = span.amax(dim=2) / 30 + 15 * (span.amax(dim=2) / 15 / 63) * 0.51 + mins.amax(dim=2) / 63 * 0.51
    err = (back - xd).abs().view(rows, dim // 256, 256).amax(dim=2)
    assert bool((err <= bound * 1.05).all())  # 5 %: the fp16 rounding of d and dmin


SHAPES = [(1, 256, 1), (1, 256, 7), (2, 512, 33), (1, 4096, 64), (2, 4096, 130), (3, 1024, 40), (5, 4096, 96),
          (1, 14336, 48), (2, 14336, 20), (9, 2048, 24), (1, 16384, 8), (3, 16384, 12), (4, 14336, 8)]


TILED_SHAPES = SHAPES + [(1, 1024, 300), (6, 4096, 70), (7, 1024, 257), (8, 2048, 96), (9, 1024, 64), (17, 512, 40),
                        (2, 4096, 1000), (4, 4096, 96), (3, 8192, 200), (4, 1024, 8192), (3, 4096, 8200),
                        (1, 4096, 14336), (2, 14336, 4096), (1, 4096, 32064),  # these three: full FFN and vocabulary-sized matrices
                        # few column tiles on a long K: two workgroups a tile, half of K each (a last share with idle wavefronts)
                        (1, 11008, 100), (2, 8192, 2048), (5, 11008, 260), (8, 4096, 4096)]


@pytest.mark.parametrize("layout,rows,in_dim,out_dim", [(RAW, *s) for s in SHAPES] + [(PREP, *s) for s in TILED_SHAPES])
def test_linear_matches_oracle(layout, rows, in_dim, out_dim):
    print(f"case: q4_k linear layout={layout} rows={rows} in={in_dim} out={out_dim}", flush=True)
    w = synth.weights(Q4K, 11, out_dim, in_dim)
    x = synth.activations(12, rows, in_dim)
    y = G.linear(Q4K, layout, x, device_weight(layout, w, out_dim, in_dim), rows, in_dim, out_dim)
    ref64 = O.linear_q4_k(x, w, rows, in_dim, out_dim, f64=True)
    ref32 = O.linear_q4_k(x, w, rows, in_dim, out_dim)
    err64, err32 = G.max_rel_err(y, ref64), G.max_rel_err(y, ref32.astype(np.float64))
    assert err64 <= TOL and err64 <= TIGHT, err64
    assert err32 <= TOL and err32 <= TIGHT, err32


def test_decode_rows_on_extreme_activations():
    """Up to four rows run on fixed-point activations (a power-of-two scale per super-block of 256 values): zero
    super-blocks, outliers 10^6 times their neighbours, magnitudes near the ends of the f32 range; a row that
    holds an infinity comes out non-finite and leaves the other rows alone."""
    in_dim, out_dim = 2048, 96
    w = synth.weights(Q4K, 91, out_dim, in_dim)
    wd = device_weight(PREP, w, out_dim, in_dim)
    rng = np.random.default_rng(92)
    base = synth.activations(93, 4, in_dim)
    cases = {
        "zero super-blocks": base * np.repeat(np.array([0, 1, 1, 0, 1, 0, 1, 1], np.float32), 256)[None, :],
        "outliers": base * np.where(rng.random((4, in_dim)) < 0.004, 1.0e6, 1.0).astype(np.float32),
        "huge": base * np.float32(1.0e30),
        "tiny": base * np.float32(1.0e-32),
        "mixed scales per super-block": base * np.repeat(np.exp2(rng.integers(-40, 40, 8)).astype(np.float32), 256)[None, :],
    }
    for name, x in cases.items():
        print(f"case: q4_k decode extremes: {name}", flush=True)
        for rows in (1, 2, 3, 4):
            y = G.linear(Q4K, PREP, x[:rows].copy(), wd, rows, in_dim, out_dim)
            ref = O.linear_q4_k(x[:rows].copy(), w, rows, in_dim, out_dim, f64=True)
            err = G.max_rel_err(y, ref)
            assert err <= TIGHT, (name, rows, err)
    x = base.copy()
    x[0, 700] = np.inf
    for rows in (2, 4):
        y = G.linear(Q4K, PREP, x[:rows].copy(), wd, rows, in_dim, out_dim)
        assert not np.isfinite(y[0]).any()
        assert np.isfinite(y[1:]).all()
        assert G.max_rel_err(y[1:], O.linear_q4_k(x[1:rows].copy(), w, rows - 1, in_dim, out_dim, f64=True)) <= TIGHT


@pytest.mark.parametrize("rows,in_dim,out_dim", [(3, 4096, 200), (5, 1024, 96), (8, 4096, 14336), (6, 14336, 100), (7, 16384, 40)])
def test_three_to_eight_rows_with_and_without_scratch(rows, in_dim, out_dim):
    """With the caller's scratch X becomes digit planes once and the int8 kernel runs on them; without it the bf16
    kernel (or several launches of the two-row kernel) serves the rows.  Both are held to the oracle."""
    print(f"case: q4_k rows with / without scratch rows={rows} in={in_dim} out={out_dim}", flush=True)
    w = synth.weights(Q4K, 95, out_dim, in_dim)
    x = synth.activations(96, rows, in_dim)
    x[rows - 1, :256] = 0.0
    wd = device_weight(PREP, w, out_dim, in_dim)
    ref = O.linear_q4_k(x, w, rows, in_dim, out_dim, f64=True)
    xd = G.to_dev(x)
    need = kernels.workspaceBytes(Q4K, rows, in_dim, out_dim)
    assert need >= in_dim // 256 * (8192 + 32 + 256)
    scratch = torch.empty(need, dtype=torch.uint8, device=G.DEV)
    for ws in (G.buf(scratch), kernels.NO_BUFFER):
        y = torch.full((rows, out_dim), float("nan"), dtype=torch.float32, device=G.DEV)
        kernels.launchLinearF32(G.stream(), Q4K, PREP, G.buf(y), G.buf(xd), G.buf(wd), rows, in_dim, out_dim, ws)
        torch.cuda.synchronize()
        err = G.max_rel_err(y.cpu().numpy(), ref)
        assert err <= TIGHT, (ws is kernels.NO_BUFFER, err)


def test_digit_plane_rows_pair_and_bias():
    """Three to eight rows: a pair call makes the digit planes once and runs both matrices on them; each half equals
    the single op bit for bit, and a bias is added to that value in f32."""
    rows, in_dim, out_dim = 5, 1024, 640
    wa, wb = synth.weights(Q4K, 97, out_dim, in_dim), synth.weights(Q4K, 98, out_dim, in_dim)
    x = synth.activations(99, rows, in_dim)
    da, db = device_weight(PREP, wa, out_dim, in_dim), device_weight(PREP, wb, out_dim, in_dim)
    ya, yb = G.linear_pair(Q4K, PREP, x, da, db, rows, in_dim, out_dim)
    assert np.array_equal(ya, G.linear(Q4K, PREP, x, da, rows, in_dim, out_dim))
    assert np.array_equal(yb, G.linear(Q4K, PREP, x, db, rows, in_dim, out_dim))
    assert G.max_rel_err(yb, O.linear_q4_k(x, wb, rows, in_dim, out_dim, f64=True)) <= TIGHT
    bias = synth.activations(100, 1, out_dim).reshape(-1)
    assert np.array_equal(G.linear_bias(Q4K, PREP, x, da, bias, rows, in_dim, out_dim), ya + bias[None, :])


@pytest.mark.parametrize("rows,in_dim,out_dim", [(1, 8192, 640), (2, 14336, 300), (5, 4096, 640), (8, 11008, 1000)])
def test_two_k_shares_pair_and_bias(rows, in_dim, out_dim):
    """Few column tiles on a long K: the plain op gives each tile to two workgroups with half of K each.  Each half of a
    pair still equals the single op bit for bit (the rule counts one matrix); a call with a bias keeps one workgroup a
    tile and sums in another order: the plain value plus the bias within the op's bound."""
    print(f"case: q4_k two K shares rows={rows} in={in_dim} out={out_dim}", flush=True)
    wa, wb = synth.weights(Q4K, 197, out_dim, in_dim), synth.weights(Q4K, 198, out_dim, in_dim)
    x = synth.activations(199, rows, in_dim)
    da, db = device_weight(PREP, wa, out_dim, in_dim), device_weight(PREP, wb, out_dim, in_dim)
    ya, yb = G.linear_pair(Q4K, PREP, x, da, db, rows, in_dim, out_dim)
    assert np.array_equal(ya, G.linear(Q4K, PREP, x, da, rows, in_dim, out_dim))
    assert np.array_equal(yb, G.linear(Q4K, PREP, x, db, rows, in_dim, out_dim))
    ref = O.linear_q4_k(x, wa, rows, in_dim, out_dim, f64=True)
    assert G.max_rel_err(ya, ref) <= TIGHT
    bias = synth.activations(200, 1, out_dim).reshape(-1)
    yb_ = G.linear_bias(Q4K, PREP, x, da, bias, rows, in_dim, out_dim)
    assert G.max_rel_err(yb_ - bias[None, :], ref) <= TIGHT
    assert G.max_rel_err(yb_, (ya + bias[None, :]).astype(np.float64)) <= TIGHT


Q8K_SHAPES = [(1, 2048, 512), (1, 3072, 2048), (2, 3072, 600), (4, 512, 1000), (9, 768, 513), (64, 1536, 512), (77, 2048, 520)]


@pytest.mark.parametrize("layout", [RAW, PREP])
@pytest.mark.parametrize("rows,in_dim,out_dim", Q8K_SHAPES)
def test_q8k_activation_route_on_the_gated_shapes(layout, rows, in_dim, out_dim):
    """The CPU engine's gated short-K shapes (native_compute.zig:3468-3479): activations quantized
    to Q8_K, integer sub-block dots.  Against the oracle's restatement of that route; the f32 route
    is a different number there (about 1e-3 .. 1e-2 away), so this also shows which route ran."""
    print(f"case: q4_k q8k route layout={layout} rows={rows} in={in_dim} out={out_dim}", flush=True)
    assert O.uses_q4k_q8k_activation(rows, in_dim, out_dim)
    assert _lib.lib().afhip_uses_q8k_activation_quant(Q4K, rows, in_dim, out_dim) == 1
    w = synth.weights(Q4K, 71, out_dim, in_dim)
    x = synth.activations(72, rows, in_dim)
    wd = device_weight(layout, w, out_dim, in_dim)
    y = G.linear(Q4K, layout, x, wd, rows, in_dim, out_dim)
    ref = O.linear_q4_k_q8k(x, w, rows, in_dim, out_dim)
    err = G.max_rel_err(y, ref.astype(np.float64))
    assert err <= TOL and err <= TIGHT, err
    f32_route = O.linear_q4_k(x, w, rows, in_dim, out_dim, f64=True)
    assert G.max_rel_err(y, f32_route) > 10 * TIGHT
    # The launcher needs the scratch on these shapes -- except where the quantizer runs inside the matmul launch
    # (one, two or four rows of a repacked tensor), which reads none: there a call without scratch is the same call.
    yd = torch.full((rows, out_dim), float("nan"), dtype=torch.float32, device=G.DEV)
    if layout == PREP and rows in (1, 2, 4):
        kernels.launchLinearF32(G.stream(), Q4K, layout, G.buf(yd), G.buf(G.to_dev(x)), G.buf(wd), rows, in_dim, out_dim,
                                kernels.NO_BUFFER)
        torch.cuda.synchronize()
        assert np.array_equal(yd.cpu().numpy().view(np.uint32), y.view(np.uint32))
    else:
        with pytest.raises(_lib.InvalidHipState):
            kernels.launchLinearF32(G.stream(), Q4K, layout, G.buf(yd), G.buf(G.to_dev(x)), G.buf(wd), rows, in_dim, out_dim,
                                    kernels.NO_BUFFER)
    # AFHIP_DISPATCH_AUTO_F32_ACTIVATIONS keeps the same shape on f32 activations (the engine's CUDA backend): the
    # f32 route's number, with or without scratch
    yf = G.linear(Q4K, layout, x, wd, rows, in_dim, out_dim, dispatch=_lib.DISPATCH_AUTO_F32_ACTIVATIONS)
    assert G.max_rel_err(yf, f32_route) <= TIGHT
    assert G.max_rel_err(yf, O.linear_q4_k(x, w, rows, in_dim, out_dim).astype(np.float64)) <= TIGHT


@pytest.mark.parametrize("in_dim,out_dim", [(512, 520), (2048, 8192), (3072, 1000)])
def test_q8k_route_decode_rows_equal_the_rows_of_a_larger_call(in_dim, out_dim):
    """With one, two or four rows the quantizer runs inside the matmul launch; nine rows take the separate quantizer.  A row's
    result does not depend on which: rows 0 .. r-1 of the nine-row product are the r-row product, bit for bit."""
    print(f"case: q4_k q8k fused quantizer in={in_dim} out={out_dim}", flush=True)
    w = synth.weights(Q4K, 79, out_dim, in_dim)
    x = synth.activations(80, 9, in_dim)
    x[1, :256] = 0.0  # a zero block: scale 1
    wd = device_weight(PREP, w, out_dim, in_dim)
    y9 = G.linear(Q4K, PREP, x, wd, 9, in_dim, out_dim)
    for rows in (1, 2, 4):
        assert O.uses_q4k_q8k_activation(rows, in_dim, out_dim)
        y = G.linear(Q4K, PREP, x[:rows].copy(), wd, rows, in_dim, out_dim)
        assert np.array_equal(y.view(np.uint32), y9[:rows].view(np.uint32)), rows


def test_q8k_gate_neighbours_stay_on_the_f32_route():
    for rows, in_dim, out_dim in [(3, 2048, 512), (1, 1024, 512), (1, 2048, 511), (5, 3072, 640), (16, 512, 512)]:
        assert not O.uses_q4k_q8k_activation(rows, in_dim, out_dim)
        assert _lib.lib().afhip_uses_q8k_activation_quant(Q4K, rows, in_dim, out_dim) == 0
        w = synth.weights(Q4K, 73, out_dim, in_dim)
        x = synth.activations(74, rows, in_dim)
        y = G.linear(Q4K, PREP, x, device_weight(PREP, w, out_dim, in_dim), rows, in_dim, out_dim)
        assert G.max_rel_err(y, O.linear_q4_k(x, w, rows, in_dim, out_dim, f64=True)) <= TIGHT
    assert _lib.lib().afhip_uses_q8k_activation_quant(_lib.TYPE_Q4_0, 1, 2048, 512) == 0


def test_q8k_route_pair_and_bias():
    rows, in_dim, out_dim = 2, 2048, 640
    wa, wb = synth.weights(Q4K, 75, out_dim, in_dim), synth.weights(Q4K, 76, out_dim, in_dim)
    x = synth.activations(77, rows, in_dim)
    da, db = device_weight(PREP, wa, out_dim, in_dim), device_weight(PREP, wb, out_dim, in_dim)
    ya, yb = G.linear_pair(Q4K, PREP, x, da, db, rows, in_dim, out_dim)
    assert np.array_equal(ya, G.linear(Q4K, PREP, x, da, rows, in_dim, out_dim))
    assert np.array_equal(yb, G.linear(Q4K, PREP, x, db, rows, in_dim, out_dim))
    bias = synth.activations(78, 1, out_dim).reshape(-1)
    yb2 = G.linear_bias(Q4K, PREP, x, da, bias, rows, in_dim, out_dim)
    assert np.array_equal(yb2, ya + bias[None, :])


PREFILL_SHAPES = [(7, 4096, 64), (10, 1024, 300), (11, 512, 33), (40, 2048, 256), (41, 1024, 257), (100, 512, 1000),
                  (128, 4096, 512), (3, 14336, 40), (45, 14336, 96), (300, 256, 64), (8, 512, 40), (9, 512, 40), (12, 512, 40), (13, 4096, 300), (7, 4096, 300), (3, 14336, 64), (5, 14336, 200), (33, 1024, 64), (64, 1024, 96), (20, 2560, 700), (50, 14336, 64),
                  (81, 768, 500)]


@pytest.mark.parametrize("rows,in_dim,out_dim", PREFILL_SHAPES)
def test_prefill_gemm_matches_oracle(rows, in_dim, out_dim):
    """More rows than one GEMV launch holds: the split kernel + MFMA GEMM (with the caller's scratch), and
    the same rows served by the GEMV a launch at a time (no scratch) -- both against the oracle."""
    print(f"case: q4_k prefill rows={rows} in={in_dim} out={out_dim}", flush=True)
    w = synth.weights(Q4K, 61, out_dim, in_dim)
    x = synth.activations(62, rows, in_dim)
    wd = device_weight(PREP, w, out_dim, in_dim)
    ref64 = O.linear_q4_k(x, w, rows, in_dim, out_dim, f64=True)
    y = G.linear(Q4K, PREP, x, wd, rows, in_dim, out_dim)  # G.linear lends afhip_linear_workspace_bytes of scratch
    err = G.max_rel_err(y, ref64)
    assert err <= TOL and err <= TIGHT, err
    xd = G.to_dev(x)
    y2 = torch.full((rows, out_dim), float("nan"), dtype=torch.float32, device=G.DEV)
    kernels.launchLinearF32(G.stream(), Q4K, PREP, G.buf(y2), G.buf(xd), G.buf(wd), rows, in_dim, out_dim, kernels.NO_BUFFER)
    torch.cuda.synchronize()
    err2 = G.max_rel_err(y2.cpu().numpy(), ref64)
    assert err2 <= TIGHT, err2


def test_prefill_full_size_with_epilogue():
    rows, in_dim, out_dim = 512, 4096, 14336
    print("case: q4_k prefill full size", flush=True)
    w = synth.weights(Q4K, 63, out_dim, in_dim)
    x = synth.activations(64, rows, in_dim)
    wd = device_weight(PREP, w, out_dim, in_dim)
    y = G.linear(Q4K, PREP, x, wd, rows, in_dim, out_dim)
    sample = np.r_[0:3, 37:43, 255, 509:512]
    ref = O.linear_q4_k(x[sample], w, len(sample), in_dim, out_dim, f64=True)
    assert G.max_rel_err(y[sample], ref) <= TIGHT
    # linearity in X: rows scaled by powers of two scale exactly
    y4 = G.linear(Q4K, PREP, x * 4.0, wd, rows, in_dim, out_dim)
    assert np.array_equal(y4, y * 4.0)
    b = synth.activations(65, 1, out_dim)[0]
    yb = G.linear_bias(Q4K, PREP, x, wd, b, rows, in_dim, out_dim)
    assert np.array_equal(yb, y + b[None, :])


def test_linear_argument_checks():
    w = G.to_dev(synth.weights(Q4K, 1, 4, 256))
    x = G.to_dev(synth.activations(2, 1, 256))
    y = torch.empty((1, 4), dtype=torch.float32, device=G.DEV)
    ws = kernels.NO_BUFFER
    with pytest.raises(_lib.InvalidHipState):  # K must be whole super-blocks
        kernels.launchLinearF32(G.stream(), Q4K, RAW, G.buf(y), G.buf(x), G.buf(w), 1, 128, 4, ws)
    with pytest.raises(_lib.InvalidHipState):  # short weight buffer
        kernels.launchLinearF32(G.stream(), Q4K, RAW, G.buf(y), G.buf(x), G.buf(w), 1, 256, 5, ws)
    d = torch.empty(4, dtype=torch.int32, device=G.DEV)
    with pytest.raises(_lib.HipError):  # no integer route, so no block dots
        kernels.launchBlockDots(G.stream(), Q4K, RAW, G.buf(d), G.buf(x), G.buf(w), 1, 256, 4, ws)
    assert kernels.workspaceBytes(Q4K, 2, 4096, 4096) == 0  # one or two decode rows need no scratch
    # three to eight rows: room for X as digit planes (8 KB a super-block + scales and sums); optional, see below
    assert kernels.workspaceBytes(Q4K, 4, 4096, 4096) == 16 * 8192 + 16 * 32 + 16 * 256
    assert kernels.workspaceBytes(Q4K, 2048, 4096, 14336) == 2048 * 4096 * 6 + 2048 * 128 * 8  # the split of X for the prefill GEMM
    assert kernels.workspaceBytes(Q4K, 64, 4096, 4096) > 64 * 4096 * 6 + 64 * 128 * 8  # ... plus partial sums when K is shared out
    big_w = torch.zeros(4 * 128 * 144, dtype=torch.uint8, device=G.DEV)
    big_x = torch.zeros(32768, dtype=torch.float32, device=G.DEV)
    with pytest.raises(_lib.HipOpUnsupported):  # K beyond what one workgroup's slices cover
        kernels.launchLinearF32(G.stream(), Q4K, RAW, G.buf(y), G.buf(big_x), G.buf(big_w), 1, 32768, 4, ws)


@pytest.mark.parametrize("layout", [RAW, PREP])
def test_full_size_ffn_matrix_and_pair(layout):
    """Llama-3-8B FFN shapes in Q4_K (33 MB per matrix, as Q4_0): decode rows, a pair, scaling property."""
    RAW = layout  # the body below runs on the layout under test
    in_dim, out_dim = 4096, 14336
    wa, wb = synth.weights(Q4K, 21, out_dim, in_dim), synth.weights(Q4K, 22, out_dim, in_dim)
    da, db = device_weight(layout, wa, out_dim, in_dim), device_weight(layout, wb, out_dim, in_dim)
    for rows in (1, 2, 4) if layout == _lib.LAYOUT_RAW else (1, 2, 4, 8):
        print(f"case: q4_k full size layout={layout} rows={rows}", flush=True)
        x = synth.activations(30 + rows, rows, in_dim)
        y = G.linear(Q4K, RAW, x, da, rows, in_dim, out_dim)
        ref = O.linear_q4_k(x, wa, rows, in_dim, out_dim, f64=True)
        err = G.max_rel_err(y, ref)
        assert err <= TOL and err <= TIGHT, err
        ya, yb = G.linear_pair(Q4K, RAW, x, da, db, rows, in_dim, out_dim)
        assert np.array_equal(ya, y)
        assert np.array_equal(yb, G.linear(Q4K, RAW, x, db, rows, in_dim, out_dim))
        # every product scales exactly with a power of two
        assert np.array_equal(G.linear(Q4K, RAW, x * 4.0, da, rows, in_dim, out_dim), y * 4.0)
    # down projection: K = 14336
    wd_ = synth.weights(Q4K, 23, 4096, 14336)
    x = synth.activations(40, 1, 14336)
    y = G.linear(Q4K, RAW, x, device_weight(layout, wd_, 4096, 14336), 1, 14336, 4096)
    assert G.max_rel_err(y, O.linear_q4_k(x, wd_, 1, 14336, 4096, f64=True)) <= TIGHT


def test_backend_ops_on_q4_k():
    in_dim, out_dim, rows = 512, 1000, 3
    w = synth.weights(Q4K, 51, out_dim, in_dim)
    x = synth.activations(52, rows, in_dim)
    with HipCompute() as cb:
        print("case: backend q4_k ops", flush=True)
        cb.insertWeightFromLoaded("raw.weight", Q4K, w, [out_dim, in_dim], keep_raw_layout=True)
        assert cb.getWeight("raw.weight").layout == _lib.LAYOUT_RAW
        cb.insertWeightFromLoaded("output.weight", Q4K, w, [out_dim, in_dim])
        wt = cb.getWeight("output.weight")
        assert wt.quant_type == Q4K and wt.layout == _lib.LAYOUT_PREPARED and wt.shape == [out_dim, in_dim]
        assert wt.byte_len == (out_dim + 31) // 32 * (in_dim // 256) * 4608
        xt = cb.fromFloat32(x, [rows, in_dim])
        y = cb.toFloat32(cb.linearNoBias(xt, wt, rows, in_dim, out_dim)).reshape(rows, out_dim)
        ref = O.linear_q4_k(x, w, rows, in_dim, out_dim, f64=True)
        assert G.max_rel_err(y, ref) <= TIGHT
        stats = cb.debugStats()
        assert stats["launches_small_batch"] == 1 and stats["launches_activation_quant"] == 0 and stats["launches_prepare"] == 1
        # the fused lm_head is one matmul on the last row alone: at this K (512) and width that is one of
        # the shapes on which the engine quantizes the activations to Q8_K
        token = cb.linearNoBiasArgmaxLastRow(xt, wt, rows, in_dim, out_dim)
        assert O.uses_q4k_q8k_activation(1, in_dim, out_dim) and not O.uses_q4k_q8k_activation(rows, in_dim, out_dim)
        last = cb.toFloat32(cb.linearNoBias(cb.fromFloat32(x[-1:].copy(), [1, in_dim]), wt, 1, in_dim, out_dim)).reshape(out_dim)
        assert cb.debugStats()["launches_activation_quant"] == 2
        assert token == int(np.argmax(last))
        ref_last = O.linear_q4_k_q8k(x[-1:], w, 1, in_dim, out_dim)[0]
        assert G.max_rel_err(last[None, :], ref_last[None, :].astype(np.float64)) <= TIGHT
        assert token == O.argmax(ref_last) or ref_last.max() - ref_last[token] <= TIGHT * np.abs(ref_last).max()
        # the same gated shape on the tensor kept in the GGUF layout (the backend lends the Q8_K scratch there too)
        raw_last = cb.toFloat32(cb.linearNoBias(cb.fromFloat32(x[-1:].copy(), [1, in_dim]), cb.getWeight("raw.weight"), 1, in_dim, out_dim))
        assert G.max_rel_err(raw_last.reshape(1, out_dim), ref_last[None, :].astype(np.float64)) <= TIGHT
        emb = cb.toFloat32(cb.embeddingLookup(wt, [999, 0], 2, in_dim)).reshape(2, in_dim)
        assert np.array_equal(emb.view(np.uint32), O.dequantize_q4_k(w).reshape(out_dim, in_dim)[[999, 0]].view(np.uint32))
        with pytest.raises(_lib.InvalidHipState):
            cb.linearNoBias(cb.fromFloat32(x[:, :128].copy(), [rows, 128]), wt, rows, 128, out_dim * 4)  # K not whole super-blocks
