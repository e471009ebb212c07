"""GPU parity: the HIP path, called through the C ABI, against the CPU oracle on
the same seeded inputs.  Bar: bit-exact for everything integer (quantized
activations, block sums, int32 block dots, repacked bytes, fp16 decode) and
max-relative error <= 1e-3 on the f32 outputs (the tolerance the benchmark
definition states); the f32 checks also hold a much tighter engineering bound."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")

from antfly_amd import _lib, kernels, synth  # noqa: E402
from oracle import oracle as O  # noqa: E402
from tests import gpu_util as G  # noqa: E402

Q4, Q8 = _lib.TYPE_Q4_0, _lib.TYPE_Q8_0
RAW, PREP = _lib.LAYOUT_RAW, _lib.LAYOUT_PREPARED
TOL = 1e-3          # stated tolerance on scaled outputs (max-relative, fp32 accumulate)
TIGHT = 2e-5        # what f32 accumulation in a different order actually needs


def smoke_row(fmt, scale, value):
    hb = np.array([scale], dtype=np.float16).view(np.uint8)
    if fmt == Q8:
        return np.concatenate([hb, np.full(32, value, dtype=np.int8).view(np.uint8)])
    nib = (value + 8) & 0xF
    return np.concatenate([hb, np.full(16, nib | (nib << 4), dtype=np.uint8)])


def test_library_smokes():
    print("case: afhip_smoke_q8_0 / afhip_smoke_q4_0", flush=True)
    kernels.smokeQ8_0()
    kernels.smokeQ4_0()


@pytest.mark.parametrize("fmt", [Q8, Q4])
@pytest.mark.parametrize("layout", [RAW, PREP])
def test_reference_gpu_smoke_kat(kats, fmt, layout):
    k = kats["gpu_smoke"]
    print(f"case: gpu_smoke fmt={fmt} layout={layout}", flush=True)
    x = np.stack([np.arange(1, 33), -np.arange(1, 33)]).astype(np.float32)
    w = np.concatenate([smoke_row(fmt, r["scale"], r["value"]) for r in k["weight_rows"]])
    wd = G.prepare(fmt, w, 3, 32) if layout == PREP else G.to_dev(w)
    y = G.linear(fmt, layout, x, wd, 2, 32, 3)
    assert np.abs(y.reshape(-1) - np.array(k["expected"])).max() <= k["tolerance_abs"]


def test_q4_0_nibble_order_kat(kats):
    k = kats["q4_0_nibble_order"]
    blk = np.full(18, k["fill_byte"], dtype=np.uint8)
    blk[0:2] = np.array([k["scale_bits"]], dtype=np.uint16).view(np.uint8)
    blk[2], blk[3] = k["qs0"], k["qs1"]
    x = np.zeros((1, 32), dtype=np.float32)
    x[0, k["input_ones_at"]] = 1.0
    for layout in (RAW, PREP):
        wd = G.prepare(Q4, blk, 1, 32) if layout == PREP else G.to_dev(blk)
        y = G.linear(Q4, layout, x, wd, 1, 32, 1)
        assert abs(y[0, 0] - k["expected"]) <= k["tolerance_abs"]


def test_fp16_decode_all_bit_patterns_on_device():
    bits = np.arange(65536, dtype=np.uint16)
    src = G.to_dev(bits.view(np.int16))
    dst = torch.empty(65536, dtype=torch.float32, device=G.DEV)
    kernels.launchDecodeFp16(G.stream(), G.buf(dst), G.buf(src), 65536)
    torch.cuda.synchronize()
    got = dst.cpu().numpy()
    want = bits.view(np.float16).astype(np.float32)
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got[~nan].view(np.uint32), want[~nan].view(np.uint32))


@pytest.mark.parametrize("rows,in_dim", [(1, 32), (3, 256), (5, 14336), (8, 4096), (64, 4096)])
def test_activation_quantizer_bit_exact(rows, in_dim):
    print(f"case: quantize_activations rows={rows} in_dim={in_dim}", flush=True)
    x = synth.activations(100 + rows, rows, in_dim)
    x[0, :32] = 0.0                       # zero block -> scale 1, q 0
    if in_dim >= 64:
        x[rows - 1, 32:64] = [127.0, 0.5, -0.5, 1.5, -1.5, 126.5, -2.5] + [0.25] * 25  # ties
        x[rows - 1, -32:] *= 1e-30        # tiny magnitudes
    if in_dim >= 4096:
        # every half-integer and its two float neighbours, both signs: block max 127 makes
        # the scale and its reciprocal exactly 1, so these hit the rounding rule directly
        k = np.arange(0, 127, dtype=np.float32) + np.float32(0.5)
        edge = np.concatenate([k, np.nextafter(k, np.float32(0)), np.nextafter(k, np.float32(200)),
                               [0.49999997, 0.25, 126.99999, 127.0]]).astype(np.float32)
        edge = np.concatenate([edge, -edge])
        nblk = (edge.size + 30) // 31
        pad = np.zeros(nblk * 31, np.float32)
        pad[: edge.size] = edge
        blocks = np.concatenate([np.full((nblk, 1), 127.0, np.float32), pad.reshape(nblk, 31)], axis=1)
        x[0, 64 : 64 + blocks.size] = blocks.reshape(-1)
    qw, sw, sumw = O.quantize_activation_rows(x, rows, in_dim)
    xd = G.to_dev(x)
    q = torch.empty(rows * in_dim, dtype=torch.int8, device=G.DEV)
    s = torch.empty(rows * in_dim // 32, dtype=torch.float32, device=G.DEV)
    sums = torch.empty(rows * in_dim // 32, dtype=torch.int32, device=G.DEV)
    kernels.launchQuantizeActivations(G.stream(), G.buf(xd), rows, in_dim, G.buf(q), G.buf(s), G.buf(sums))
    torch.cuda.synchronize()
    assert np.array_equal(q.cpu().numpy().reshape(rows, in_dim), qw)
    assert np.array_equal(s.cpu().numpy().view(np.uint32).reshape(rows, -1), sw.view(np.uint32))
    assert np.array_equal(sums.cpu().numpy().reshape(rows, -1), sumw)


@pytest.mark.parametrize("fmt", [Q8, Q4])
@pytest.mark.parametrize("out_dim,in_dim", [(37, 160), (8, 4096), (5, 8224), (130, 32)])
def test_prepare_weight_is_a_pure_repack(fmt, out_dim, in_dim):
    w = synth.weights(fmt, 7, out_dim, in_dim)
    got = G.prepare(fmt, w, out_dim, in_dim).cpu().numpy()
    want = G.numpy_prepare(fmt, w, out_dim, in_dim)
    assert got.size == want.size == kernels.preparedWeightBytes(fmt, out_dim, in_dim)
    assert np.array_equal(got, want)


SHAPES_A = [  # (rows, in_dim, out_dim): all take the activation-quantized route
    (1, 4096, 512), (2, 96, 515), (3, 2048, 640), (4, 4096, 1024), (5, 1120, 513),
    (6, 256, 600), (7, 160, 777), (8, 4096, 512), (9, 256, 512), (17, 512, 530),
    (33, 96, 513), (64, 1056, 640), (130, 256, 1030), (257, 512, 512),
    (16, 14336, 512), (70, 8224, 520),  # long K on the MFMA kernel: many ring stages, a one-block last stage
    (8, 14336, 516), (7, 9216, 512),    # small batch with a long K: one launch with more than 128 KB of LDS
    # the decode kernel with the quantized activations awaited through a counter (several rows, or one long row, and
    # wavefronts that do not quantize): quantizers with a ragged last block set, every row count, one long row in
    # two and four K slices, a wide matrix (full-size workgroups)
    (2, 4096, 4100), (3, 4096, 2052), (4, 4096, 6144), (2, 1120, 3000), (4, 992, 8200), (1, 6144, 1030), (1, 14336, 2050),
    (2, 2080, 14336),
    # ... and the long-K kernel (K > 4096, two to seven rows, sixteen-wavefront workgroups): full and ragged last slice,
    # ragged columns, the most rows the counter form takes
    (2, 8192, 2048), (4, 9216, 4100), (3, 14336, 4096), (7, 8192, 4096), (5, 4128, 2100),
    (2, 14336, 2048), (2, 12288, 4100),  # (two rows take that kernel from K = 12288 on; below, the decode kernel with K slices)
    (2, 11008, 1030), (2, 6144, 4100),
    # (three and four rows on whole 256-value runs of K take the eight-row MFMA kernel where that measured faster; the
    # long-K kernel keeps a K that is not such a multiple, and three rows of Q4_0 on a long K and few columns)
    (4, 8224, 1030), (3, 6144, 2050), (4, 14336, 1030), (2, 14336, 4100), (3, 11008, 4096),
    # the single-shot MFMA kernel (5..64 rows): every count of live result registers, two row tiles, a K
    # that ends inside a wavefront's run of blocks, a second K share of one block, ragged columns
    (24, 4096, 544), (25, 2048, 512), (32, 4128, 513), (48, 320, 520), (12, 3072, 1000),
    (70, 512, 8200), (128, 1056, 8192), (97, 256, 8224),  # three and four row tiles (Q4_0 on a wide matrix)
    (100, 512, 4700), (66, 1024, 6150),  # ... and on a matrix whose tiled-GEMM grid would take a second round
    # the eight-row MFMA kernel (5..8 rows on a grid of at least a workgroup per compute unit): one live
    # wavefront and a ragged last tile; 64-column tiles, ragged; K shares with a short last share; a
    # wavefront with half its blocks
    (8, 512, 8200), (5, 4096, 12290), (7, 9216, 4112), (6, 256, 16416),
    # ... on 16-column tiles (4096 to 4608 columns and one K share): full, ragged last tile, one live wavefront
    (5, 4096, 4096), (8, 1024, 4600), (6, 256, 4100),
    # ... with the column count of a workgroup picked to spread the matrix evenly over the compute units: 56 of a
    # workgroup's 64 columns live (14336), 48 and 40 (three column groups; ragged last tile), 24 (two groups, 6144)
    (8, 512, 14336), (6, 1024, 11008), (5, 256, 10000), (7, 2048, 6144), (8, 256, 9000),
    (5, 8192, 7168),  # ... 56 columns with two K shares (Q4_0)
    # three and four rows on more columns than one round of the decode kernel's workgroups: Q4_0 takes the eight-row kernel
    (4, 256, 16448), (3, 256, 33000), (4, 4096, 28672), (4, 4096, 33000),  # (four rows of 4096 values: from two rounds on)
    (3, 2048, 14400), (4, 2048, 11040),  # ... and Q8_0 on wide matrices with K of 2048 to 4096
    # nine to 32 rows on 64-column tiles: every count of live result registers, ragged columns, one live
    # wavefront with half its blocks, K shares with a short last share
    (9, 512, 12290), (16, 4096, 12288), (17, 256, 12300), (24, 1024, 12352), (32, 512, 12290), (29, 9216, 12288),
    (33, 1024, 12352), (48, 512, 12290), (64, 4096, 12288),  # ... and two row tiles
    # ... on fewer columns, where the K shares fill the grid: four shares and the reduce launch, two shares adding to
    # the result themselves with a ragged last tile (Q4_0), two shares of Q8_0
    (16, 14336, 4096), (12, 8192, 8190), (20, 4096, 8192), (17, 512, 10250),
]


@pytest.mark.parametrize("fmt", [Q8, Q4])
@pytest.mark.parametrize("layout", [RAW, PREP])
@pytest.mark.parametrize("rows,in_dim,out_dim", SHAPES_A)
def test_block_dots_bit_exact_and_outputs_within_tolerance(fmt, layout, rows, in_dim, out_dim):
    print(f"case: route A fmt={fmt} layout={layout} rows={rows} in={in_dim} out={out_dim}", flush=True)
    assert O.uses_activation_quant(rows, in_dim, out_dim)
    x = synth.activations(rows * 1000 + in_dim, rows, in_dim)
    x[0, :32] = 0.0
    w = synth.weights(fmt, out_dim, out_dim, in_dim)
    wd = G.prepare(fmt, w, out_dim, in_dim) if layout == PREP else G.to_dev(w)
    dots = G.block_dots(fmt, layout, x, wd, rows, in_dim, out_dim)
    assert np.array_equal(dots, O.block_dots(fmt, x, w, rows, in_dim, out_dim))
    y = G.linear(fmt, layout, x, wd, rows, in_dim, out_dim)
    y64 = O.linear_act_f64(fmt, x, w, rows, in_dim, out_dim)
    for workers in (1, 8):  # every thread plan of the reference
        ref = O.linear_no_bias(fmt, x, w, rows, in_dim, out_dim, workers=workers)
        err = G.max_rel_err(y, ref.astype(np.float64))
        assert err <= TOL and err <= TIGHT, err
    assert G.max_rel_err(y, y64) <= TIGHT


SHAPES_B = [(1, 32, 3), (2, 64, 600), (3, 96, 11), (4, 4096, 100), (1, 64, 4096), (12, 128, 40)]


@pytest.mark.parametrize("fmt", [Q8, Q4])
@pytest.mark.parametrize("layout", [RAW, PREP])
@pytest.mark.parametrize("rows,in_dim,out_dim", SHAPES_B)
def test_f32_route_matches_oracle(fmt, layout, rows, in_dim, out_dim):
    print(f"case: route B fmt={fmt} layout={layout} rows={rows} in={in_dim} out={out_dim}", flush=True)
    assert not O.uses_activation_quant(rows, in_dim, out_dim)
    x = synth.activations(rows + in_dim, rows, in_dim)
    w = synth.weights(fmt, 3 * out_dim, out_dim, in_dim)
    wd = G.prepare(fmt, w, out_dim, in_dim) if layout == PREP else G.to_dev(w)
    y = G.linear(fmt, layout, x, wd, rows, in_dim, out_dim)
    ref = O.linear_no_bias(fmt, x, w, rows, in_dim, out_dim)
    dense = O.dequantize(fmt, w).reshape(out_dim, in_dim).astype(np.float64)
    y64 = x.astype(np.float64) @ dense.T
    assert G.max_rel_err(y, ref.astype(np.float64)) <= TIGHT
    assert G.max_rel_err(y, y64) <= TIGHT


@pytest.mark.parametrize("fmt", [Q8, Q4])
@pytest.mark.parametrize("rows", [6, 12])  # 12 rows forced onto the GEMV kernels: activations quantized by their own kernel
def test_forced_dispatch_kinds_agree(fmt, rows):
    """A plan may force any kernel family; all of them compute the same op."""
    in_dim, out_dim = 512, 640
    x = synth.activations(77, rows, in_dim)
    w = synth.weights(fmt, 78, out_dim, in_dim)
    wd = G.prepare(fmt, w, out_dim, in_dim)
    want = O.block_dots(fmt, x, w, rows, in_dim, out_dim)
    base = G.linear(fmt, PREP, x, wd, rows, in_dim, out_dim)
    for dispatch in (0, 1, 2, 3):
        assert np.array_equal(G.block_dots(fmt, PREP, x, wd, rows, in_dim, out_dim, dispatch), want)
        y = G.linear(fmt, PREP, x, wd, rows, in_dim, out_dim, dispatch)
        assert G.max_rel_err(y, base.astype(np.float64)) <= TIGHT


# ---- two matmuls that share X (linearNoBiasPair, ops/ops.zig:909) ----------------

PAIR_SHAPES = [  # rows, in_dim, out_dim: fused GEMV, small-batch GEMV with K slices, ragged columns, MFMA GEMM, f32 route
    (1, 4096, 1024), (2, 512, 514), (4, 2048, 640), (5, 8224, 513), (8, 4096, 512), (12, 256, 530), (40, 512, 640),
    (3, 64, 100), (20, 2048, 300),  # the last: MFMA GEMM with K shared out over workgroups, both matrices through one scratch
    (6, 512, 8200), (7, 9216, 4112),  # the eight-row MFMA kernel, one launch over both matrices; with K shares
    (20, 512, 12290),                 # the 32-row MFMA kernel on 64-column tiles, both matrices
    (4, 512, 8200), (3, 256, 16500),  # four and three rows whose two matrices together exceed one (two) rounds of the decode kernel
    (12, 9216, 520),                  # the eight-row kernel on two groups of eight rows (Q8_0; Q4_0 on a long K), both matrices
]


@pytest.mark.parametrize("fmt", [Q8, Q4])
@pytest.mark.parametrize("layout", [RAW, PREP])
@pytest.mark.parametrize("rows,in_dim,out_dim", PAIR_SHAPES)
def test_pair_equals_two_single_ops(fmt, layout, rows, in_dim, out_dim):
    """Each half of a pair is bit-identical to the single op on that matrix where both take the same kernel (and so
    equal to the oracle within the single op's bound), within that bound of it otherwise; the op is the engine's
    two-call fallback fused."""
    print(f"case: pair fmt={fmt} layout={layout} rows={rows} in={in_dim} out={out_dim}", flush=True)
    x = synth.activations(510 + rows, rows, in_dim)
    wa = synth.weights(fmt, 511, out_dim, in_dim)
    wb = synth.weights(fmt, 512, out_dim, in_dim)
    da = G.prepare(fmt, wa, out_dim, in_dim) if layout == PREP else G.to_dev(wa)
    db = G.prepare(fmt, wb, out_dim, in_dim) if layout == PREP else G.to_dev(wb)
    ya, yb = G.linear_pair(fmt, layout, x, da, db, rows, in_dim, out_dim)
    sa, sb = G.linear(fmt, layout, x, da, rows, in_dim, out_dim), G.linear(fmt, layout, x, db, rows, in_dim, out_dim)
    # Three and four rows of Q4_0: the pair's two matrices together may exceed one (two) rounds of the decode kernel's
    # workgroups (64 columns a compute unit, 256 units) where one matrix does not; the pair then runs on the eight-row
    # MFMA kernel and a single op on the decode kernel -- the same block dots, another f32 summation order.
    one_round = 256 * 64 * (1 if rows == 4 and rows * in_dim < 16384 else 2)
    routes_differ = (fmt == Q4 and layout == PREP and rows in (3, 4) and in_dim <= 4096 and in_dim % 256 == 0 and
                     out_dim <= one_round < 2 * out_dim)
    if routes_differ:
        assert G.max_rel_err(ya, sa.astype(np.float64)) <= TIGHT and G.max_rel_err(yb, sb.astype(np.float64)) <= TIGHT
    else:
        assert np.array_equal(ya, sa)
        assert np.array_equal(yb, sb)
    ref_b = O.linear_no_bias(fmt, x, wb, rows, in_dim, out_dim, workers=8)
    assert G.max_rel_err(yb, ref_b.astype(np.float64)) <= TIGHT


# ---- the benchmark configurations at full size ---------------------------------

FULL = [
    ("C1", Q8, [1], 4096, 4096),
    ("C4", Q8, [128, 512, 2048], 4096, 4096),
    ("C4-q4", Q4, [128], 4096, 4096),
    ("C2", Q4, [1, 2, 4, 8], 4096, 14336),
    ("C3", Q4, [1, 5], 14336, 4096),
    ("C5-qkv", Q4, [1, 5], 4096, 6144),   # the decode-step sweep: attention projections at one and five rows
    ("C5-o", Q4, [1, 5], 4096, 4096),
]
# element-wise relative error over outputs above 1e-3 of their row maximum (information; the gate
# is the row-normalised figure): collected here and printed by the last full-size case
ELEMENTWISE = {}


@pytest.mark.parametrize("name,fmt,row_list,in_dim,out_dim", FULL)
def test_full_size_decode_configs(name, fmt, row_list, in_dim, out_dim):
    w = synth.weights(fmt, 1234, out_dim, in_dim)
    wd = G.prepare(fmt, w, out_dim, in_dim)
    prepared = O.Prepared(fmt, w, out_dim, in_dim)
    for rows in row_list:
        print(f"case: {name} fmt={fmt} rows={rows} in={in_dim} out={out_dim}", flush=True)
        x = synth.activations(4321 + rows, rows, in_dim)
        y = G.linear(fmt, PREP, x, wd, rows, in_dim, out_dim)
        ref = prepared.linear(x, rows, workers=8)
        err = G.max_rel_err(y, ref.astype(np.float64))
        assert err <= TOL and err <= TIGHT, err
        ELEMENTWISE[(name, rows)] = G.elementwise_rel_err(y, ref.astype(np.float64))
        print(f"  row-normalised max-rel {err:.2e}, element-wise (|want| > 1e-3 row max) {ELEMENTWISE[(name, rows)]:.2e}", flush=True)
        assert ELEMENTWISE[(name, rows)] <= 100 * TOL  # cancellation near zero amplifies by at most 1/floor
        # block dots on a slice of output columns and rows (the full tensor is rows x out x in/32 ints)
        sub, rsub = 64, min(rows, 40)
        wsub = w[: sub * (in_dim // 32) * O.BLOCK_BYTES[fmt]]
        wsub_d = G.prepare(fmt, wsub, sub, in_dim)
        dots = G.block_dots(fmt, PREP, x[:rsub], wsub_d, rsub, in_dim, sub,
                            dispatch=-1 if rows <= 8 else 3)  # rows >= 9: the MFMA kernel
        assert np.array_equal(dots, O.block_dots(fmt, x[:rsub], wsub, rsub, in_dim, sub))
        # linearity in X is NOT a property of this op (activations are re-quantized);
        # scaling X by a power of two is: scales double, int8 values stay.
        y2 = G.linear(fmt, PREP, x * 2.0, wd, rows, in_dim, out_dim)
        assert np.array_equal(y2, y * 2.0)
    prepared.close()


@pytest.mark.parametrize("rows", [1, 5])
def test_full_size_gate_up_pair(rows):
    """The decode step's gate + up projections as the one pair call the engine makes
    (architectures/gpt.zig:5398-5440): each half bit-identical to the single op on that
    matrix, one half against the oracle."""
    in_dim, out_dim = 4096, 14336
    print(f"case: C5 pair rows={rows} in={in_dim} out={out_dim}", flush=True)
    x = synth.activations(8800 + rows, rows, in_dim)
    wa = synth.weights(Q4, 8801, out_dim, in_dim)
    wb = synth.weights(Q4, 8802, out_dim, in_dim)
    da, db = G.prepare(Q4, wa, out_dim, in_dim), G.prepare(Q4, wb, out_dim, in_dim)
    ya, yb = G.linear_pair(Q4, PREP, x, da, db, rows, in_dim, out_dim)
    assert np.array_equal(ya, G.linear(Q4, PREP, x, da, rows, in_dim, out_dim))
    assert np.array_equal(yb, G.linear(Q4, PREP, x, db, rows, in_dim, out_dim))
    prepared = O.Prepared(Q4, wb, out_dim, in_dim)
    ref = prepared.linear(x, rows, workers=8)
    prepared.close()
    err = G.max_rel_err(yb, ref.astype(np.float64))
    assert err <= TOL and err <= TIGHT, err


@pytest.mark.parametrize("fmt_name,fmt", [("q4_0", Q4), ("q8_0", Q8)])
@pytest.mark.parametrize("case,rows,in_dim,out_dim", [("k256_n64", 5, 256, 64), ("k96_n512", 5, 96, 512)])
def test_committed_tiny_vectors(fmt_name, fmt, case, rows, in_dim, out_dim):
    """The HIP path against tests/golden/tiny_vectors.npz (no oracle call): quantized activations,
    scales, sums and int32 block dots bit-exact, outputs within tolerance."""
    import os

    g = np.load(os.path.join(os.path.dirname(__file__), "golden", "tiny_vectors.npz"), allow_pickle=False)
    key = f"{fmt_name}_{case}_"
    x, w = g[key + "x"], g[key + "w_raw"]
    print(f"case: tiny vectors {key}", flush=True)
    xd = G.to_dev(x)
    q = torch.empty(rows * in_dim, dtype=torch.int8, device=G.DEV)
    s = torch.empty(rows * in_dim // 32, dtype=torch.float32, device=G.DEV)
    sums = torch.empty(rows * in_dim // 32, dtype=torch.int32, device=G.DEV)
    kernels.launchQuantizeActivations(G.stream(), G.buf(xd), rows, in_dim, G.buf(q), G.buf(s), G.buf(sums))
    torch.cuda.synchronize()
    assert np.array_equal(q.cpu().numpy().reshape(rows, in_dim), g[key + "qx"])
    assert np.array_equal(s.cpu().numpy().view(np.uint32).reshape(rows, -1), g[key + "sx"].view(np.uint32))
    assert np.array_equal(sums.cpu().numpy().reshape(rows, -1), g[key + "sumx"])
    for layout in (RAW, PREP):
        wd = G.prepare(fmt, w, out_dim, in_dim) if layout == PREP else G.to_dev(w)
        assert np.array_equal(G.block_dots(fmt, layout, x, wd, rows, in_dim, out_dim), g[key + "block_dots"])
        y = G.linear(fmt, layout, x, wd, rows, in_dim, out_dim)
        assert G.max_rel_err(y, g[key + "y_op"].astype(np.float64)) <= TIGHT


@pytest.mark.parametrize("fmt,rows,in_dim,out_dim,pair", [(Q4, 29, 9216, 12288, False), (Q8, 20, 2048, 12290, True),
                                                          (Q4, 20, 512, 12290, True), (Q4, 12, 8192, 12352, True), (Q4, 40, 8192, 12288, True)])
def test_thirty_two_row_kernel_with_k_shares_and_pairs(fmt, rows, in_dim, out_dim, pair):
    """On this chip the 32-row kernel's grid bound (one workgroup per compute unit) keeps launches with
    K shares or two matrices on the older kernel; with the bound lifted they take the 32-row kernel and
    must give what the older kernel gives to f32 summation order, and the oracle's result within its bound."""
    print(f"case: 32-row kernel, bound lifted fmt={fmt} rows={rows} in={in_dim} out={out_dim} pair={pair}", flush=True)
    x = synth.activations(5100 + rows, rows, in_dim)
    wa = synth.weights(fmt, 5101, out_dim, in_dim)
    da = G.prepare(fmt, wa, out_dim, in_dim)
    db = G.prepare(fmt, synth.weights(fmt, 5102, out_dim, in_dim), out_dim, in_dim) if pair else None

    def run():
        if pair:
            return G.linear_pair(fmt, PREP, x, da, db, rows, in_dim, out_dim)
        return (G.linear(fmt, PREP, x, da, rows, in_dim, out_dim),)

    older = run()
    _lib.lib().afhip_tune_batch32_max_workgroups(1000000)
    try:
        got = run()
    finally:
        _lib.lib().afhip_tune_batch32_max_workgroups(-1)
    ref = O.linear_no_bias(fmt, x, wa, rows, in_dim, out_dim, workers=8)
    err = G.max_rel_err(got[0], ref.astype(np.float64))
    assert err <= TOL and err <= TIGHT, err
    for a, b in zip(got, older):
        assert G.max_rel_err(a, b.astype(np.float64)) <= TIGHT
    if pair:  # each half of the pair equals the single op on that matrix, bit for bit
        _lib.lib().afhip_tune_batch32_max_workgroups(1000000)
        try:
            assert np.array_equal(got[0], G.linear(fmt, PREP, x, da, rows, in_dim, out_dim))
            assert np.array_equal(got[1], G.linear(fmt, PREP, x, db, rows, in_dim, out_dim))
        finally:
            _lib.lib().afhip_tune_batch32_max_workgroups(-1)

