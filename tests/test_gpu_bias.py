"""GPU parity for the biased linears (`linear`, `linearPair`, `linearTriple`; ops/ops.zig:1728,
:915, :921).  The engine's CPU op on a quantized weight is the no-bias product followed by
addLinearBiasRows (ops/native_compute.zig:5065-5077, :5197-5203); here the kernel that writes
Y adds the bias, so every element must be *exactly* the no-bias launch's value plus its bias,
and within the f32 bound of the oracle."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")

from antfly_amd import _lib, kernels, synth  # noqa: E402
from antfly_amd.hip_compute import HipCompute  # noqa: E402
from oracle import oracle as O  # noqa: E402
from tests import gpu_util as G  # noqa: E402

Q4, Q8, Q4K = _lib.TYPE_Q4_0, _lib.TYPE_Q8_0, _lib.TYPE_Q4_K
RAW, PREP = _lib.LAYOUT_RAW, _lib.LAYOUT_PREPARED
TIGHT = 2e-5

# rows, in_dim, out_dim: fused GEMV (one slice / K slices), multi-row fused, pre-quantized rows
# kernel, both MFMA tiles, ragged columns, the f32 route
SHAPES = [(1, 4096, 1024), (1, 512, 514), (2, 2048, 640), (4, 1024, 600), (5, 8224, 513), (8, 4096, 512),
          (12, 256, 530), (40, 512, 640), (300, 512, 1024), (3, 64, 100),
          (20, 2048, 300), (33, 8224, 200),  # MFMA GEMM with K shared out over workgroups: the reduce kernel adds the bias
          (7, 512, 8200), (5, 9216, 4112),  # the eight-row MFMA kernel; with K shares (the reduce kernel adds the bias)
          (18, 512, 12290),
          (12, 4096, 520), (40, 3072, 300),
          (12, 9216, 300)]  # Q4_0 too as two groups of eight rows (long K): two K shares, the reduce kernel adds the bias  # one K share that the plain op runs as two shares of four wavefronts each: the same bits  # the 32-row MFMA kernel on 64-column tiles


def bias_vector(seed, out_dim):
    return (synth.activations(seed, 1, out_dim)[0] * 3.0).astype(np.float32)


def reference_bias_vectors():
    """The inputs of the reference's own test of a biased Q8_0 pair (ops/native_compute.zig:39163-39223):
    3 x 32 activations (idx % 7) - 3, two 2 x 32 matrices with scale 1.0 and small integer
    weights, biases {0.25, -0.5} and {-0.75, 0.125}.  Everything is a small integer, so the
    expected outputs are exact in any summation order."""
    rows, in_dim, out_dim = 3, 32, 2
    x = np.array([(i % 7) - 3 for i in range(rows * in_dim)], np.float32).reshape(rows, in_dim)
    qa = np.array([(i % 5) - 2 for i in range(32)], np.int8)
    qb = np.array([(i % 3) + 1 for i in range(32)], np.int8)
    scale = np.array([0x00, 0x3C], np.uint8)
    wa = np.concatenate([np.concatenate([scale, qa.view(np.uint8)])] * out_dim)
    wb = np.concatenate([np.concatenate([scale, qb.view(np.uint8)])] * out_dim)
    ba, bb = np.array([0.25, -0.5], np.float32), np.array([-0.75, 0.125], np.float32)
    ya = (x.astype(np.int64) @ np.tile(qa.astype(np.int64), (out_dim, 1)).T).astype(np.float32) + ba
    yb = (x.astype(np.int64) @ np.tile(qb.astype(np.int64), (out_dim, 1)).T).astype(np.float32) + bb
    return rows, in_dim, out_dim, x, wa, wb, ba, bb, ya, yb


def test_reference_biased_pair_vectors():
    rows, in_dim, out_dim, x, wa, wb, ba, bb, ya, yb = reference_bias_vectors()
    print("case: biased Q8_0 pair, reference test inputs", flush=True)
    assert np.array_equal(O.linear(Q8, x, wa, ba, rows, in_dim, out_dim), ya)  # the checker itself
    assert np.array_equal(O.linear(Q8, x, wb, bb, rows, in_dim, out_dim), yb)
    for layout in (RAW, PREP):
        da = G.prepare(Q8, wa, out_dim, in_dim) if layout == PREP else G.to_dev(wa)
        db = G.prepare(Q8, wb, out_dim, in_dim) if layout == PREP else G.to_dev(wb)
        ga, gb = G.linear_pair_bias(Q8, layout, x, da, ba, db, bb, rows, in_dim, out_dim)
        assert np.array_equal(ga, ya) and np.array_equal(gb, yb)
        assert np.array_equal(G.linear_bias(Q8, layout, x, da, ba, rows, in_dim, out_dim), ya)


@pytest.mark.parametrize("fmt", [Q8, Q4])
@pytest.mark.parametrize("layout", [RAW, PREP])
@pytest.mark.parametrize("rows,in_dim,out_dim", SHAPES)
def test_bias_is_added_to_the_no_bias_result(fmt, layout, rows, in_dim, out_dim):
    print(f"case: linear+bias fmt={fmt} layout={layout} rows={rows} in={in_dim} out={out_dim}", flush=True)
    x = synth.activations(610 + rows, rows, in_dim)
    wa, wb = synth.weights(fmt, 611, out_dim, in_dim), synth.weights(fmt, 612, out_dim, in_dim)
    ba, bb = bias_vector(613, out_dim), bias_vector(614, out_dim)
    da = G.prepare(fmt, wa, out_dim, in_dim) if layout == PREP else G.to_dev(wa)
    db = G.prepare(fmt, wb, out_dim, in_dim) if layout == PREP else G.to_dev(wb)
    plain = G.linear(fmt, layout, x, da, rows, in_dim, out_dim)
    y = G.linear_bias(fmt, layout, x, da, ba, rows, in_dim, out_dim)
    assert np.array_equal(y, plain + ba[None, :])  # one f32 add per element, nothing else changes
    ref = O.linear(fmt, x, wa, ba, rows, in_dim, out_dim, workers=8)
    assert G.max_rel_err(y, ref.astype(np.float64)) <= TIGHT
    # the pair: each half is the single biased op on that matrix
    ya, yb = G.linear_pair_bias(fmt, layout, x, da, ba, db, bb, rows, in_dim, out_dim)
    assert np.array_equal(ya, y)
    assert np.array_equal(yb, G.linear_bias(fmt, layout, x, db, bb, rows, in_dim, out_dim))


@pytest.mark.parametrize("rows", [1, 2, 3, 4, 7])
def test_q4_k_bias(rows):
    in_dim, out_dim = 1024, 514
    print(f"case: Q4_K linear+bias rows={rows}", flush=True)
    x = synth.activations(620 + rows, rows, in_dim)
    w = synth.weights(Q4K, 621, out_dim, in_dim)
    b = bias_vector(622, out_dim)
    wd = G.to_dev(w)
    plain = G.linear(Q4K, RAW, x, wd, rows, in_dim, out_dim)
    y = G.linear_bias(Q4K, RAW, x, wd, b, rows, in_dim, out_dim)
    assert np.array_equal(y, plain + b[None, :])
    ref = O.add_linear_bias_rows(O.linear_q4_k(x, w, rows, in_dim, out_dim), b, rows, out_dim)
    assert G.max_rel_err(y, ref.astype(np.float64)) <= TIGHT


def linear_epilogue(fmt, layout, x, w_dev, rows, in_dim, out_dim, bias=None, residual=None, activation=0, dispatch=-1):
    xd = G.to_dev(x.astype(np.float32))
    keep = [xd]
    bb = rb = kernels.NO_BUFFER
    if bias is not None:
        keep.append(G.to_dev(bias.astype(np.float32)))
        bb = G.buf(keep[-1])
    if residual is not None:
        keep.append(G.to_dev(residual.astype(np.float32)))
        rb = G.buf(keep[-1])
    y = torch.full((rows, out_dim), float("nan"), dtype=torch.float32, device=G.DEV)
    ws = torch.empty(max(kernels.workspaceBytes(fmt, rows, in_dim, out_dim), 16), dtype=torch.uint8, device=G.DEV)
    kernels.launchLinearEpilogueF32(G.stream(), fmt, layout, G.buf(y), G.buf(xd), G.buf(w_dev), rows, in_dim, out_dim, bb, rb,
                                    activation, G.buf(ws), dispatch)
    torch.cuda.synchronize()
    return y.cpu().numpy()


EPILOGUE_SHAPES = [(1, 4096, 1024), (1, 8224, 513), (3, 1024, 600), (6, 2048, 640), (40, 512, 640), (300, 512, 1024), (20, 2048, 300),
                   (3, 64, 100), (6, 512, 8200)]


@pytest.mark.parametrize("fmt", [Q8, Q4, Q4K])
@pytest.mark.parametrize("rows,in_dim,out_dim", EPILOGUE_SHAPES)
def test_fused_epilogues(fmt, rows, in_dim, out_dim):
    """linearRelu / linearQuickGelu / linearGelu / linearAdd (ops/ops.zig:2164-2230): the stored value is
    act(product + bias) + residual.  relu and the residual add are exact functions of the bias op's
    value; the two gelus are checked against the oracle's formulas applied to that value."""
    if fmt == Q4K and in_dim % 256 != 0:
        pytest.skip("Q4_K rows are whole 256-value super-blocks")
    layout = RAW if fmt == Q4K else PREP
    print(f"case: fused epilogues fmt={fmt} rows={rows} in={in_dim} out={out_dim}", flush=True)
    x = synth.activations(650 + rows, rows, in_dim) * 4.0
    w = synth.weights(fmt, 651, out_dim, in_dim)
    b = bias_vector(652, out_dim)
    res = synth.activations(653, rows, out_dim)
    wd = G.to_dev(w) if fmt == Q4K else G.prepare(fmt, w, out_dim, in_dim)
    biased = G.linear_bias(fmt, layout, x, wd, b, rows, in_dim, out_dim)
    plain = G.linear(fmt, layout, x, wd, rows, in_dim, out_dim)
    assert np.array_equal(linear_epilogue(fmt, layout, x, wd, rows, in_dim, out_dim), plain)  # nothing set: the plain op
    assert (biased < 0).any() and (biased > 0).any()
    relu = linear_epilogue(fmt, layout, x, wd, rows, in_dim, out_dim, bias=b, activation=_lib.ACTIVATION_RELU)
    assert np.array_equal(relu, np.maximum(biased, 0))
    add = linear_epilogue(fmt, layout, x, wd, rows, in_dim, out_dim, bias=b, residual=res)
    assert np.array_equal(add, biased + res)
    assert np.array_equal(linear_epilogue(fmt, layout, x, wd, rows, in_dim, out_dim, residual=res), plain + res)
    for act, kind in ((_lib.ACTIVATION_QUICK_GELU, O.QUICK_GELU), (_lib.ACTIVATION_GELU, O.GELU)):
        got = linear_epilogue(fmt, layout, x, wd, rows, in_dim, out_dim, bias=b, activation=act)
        want = O.apply_activation(kind, biased)
        assert np.allclose(got, want, rtol=3e-6, atol=1e-6 * np.abs(biased).max()), (act, np.abs(got - want).max())
    both = linear_epilogue(fmt, layout, x, wd, rows, in_dim, out_dim, bias=b, residual=res, activation=_lib.ACTIVATION_RELU)
    assert np.array_equal(both, np.maximum(biased, 0) + res)
    # end to end against the engine's CPU definition
    if fmt != Q4K:
        ref = O.apply_activation(O.RELU, O.linear(fmt, x, w, b, rows, in_dim, out_dim, workers=8))
        assert G.max_rel_err(relu, ref.astype(np.float64)) <= TIGHT


def test_bias_argument_errors():
    rows, in_dim, out_dim = 2, 512, 512
    x = G.to_dev(synth.activations(1, rows, in_dim))
    w = G.to_dev(synth.weights(Q8, 2, out_dim, in_dim))
    y = torch.zeros(rows, out_dim, device=G.DEV)
    ws = torch.empty(kernels.workspaceBytes(Q8, rows, in_dim, out_dim), dtype=torch.uint8, device=G.DEV)
    short = torch.zeros(out_dim - 1, device=G.DEV)
    with pytest.raises(_lib.InvalidHipState):
        kernels.launchLinearBiasF32(G.stream(), Q8, RAW, G.buf(y), G.buf(x), G.buf(w), G.buf(short), rows, in_dim, out_dim,
                                    G.buf(ws))
    with pytest.raises(_lib.InvalidHipState):
        kernels.launchLinearBiasF32(G.stream(), Q8, RAW, G.buf(y), G.buf(x), G.buf(w), kernels.NO_BUFFER, rows, in_dim,
                                    out_dim, G.buf(ws))
    # a residual shorter than Y, an activation that does not exist, activation on a pair
    res = torch.zeros(rows * out_dim - 1, device=G.DEV)
    bias = torch.zeros(out_dim, device=G.DEV)
    with pytest.raises(_lib.InvalidHipState):
        kernels.launchLinearEpilogueF32(G.stream(), Q8, RAW, G.buf(y), G.buf(x), G.buf(w), rows, in_dim, out_dim, G.buf(bias),
                                        G.buf(res), 0, G.buf(ws))
    with pytest.raises(_lib.HipError):
        kernels.launchLinearEpilogueF32(G.stream(), Q8, RAW, G.buf(y), G.buf(x), G.buf(w), rows, in_dim, out_dim, G.buf(bias),
                                        kernels.NO_BUFFER, 7, G.buf(ws))
    torch.cuda.synchronize()


@pytest.mark.parametrize("fmt", [Q8, Q4, Q4K])
def test_backend_fused_linear_ops(fmt):
    """ComputeBackend linearRelu / linearQuickGelu / linearGelu / linearAdd: a fused op equals the
    composition of the backend's own `linear` with the activation / the add."""
    rows, in_dim, out_dim = 3, 1024, 768
    print(f"case: backend fused linear ops fmt={fmt}", flush=True)
    cb = HipCompute()
    try:
        x = synth.activations(660, rows, in_dim) * 4.0
        w = synth.weights(fmt, 661, out_dim, in_dim)
        b, res = bias_vector(662, out_dim), synth.activations(663, rows, out_dim)
        cb.insertWeightFromLoaded("blk.0.ffn_up.weight", fmt, w, [out_dim, in_dim])
        wt = cb.getWeight("blk.0.ffn_up.weight")
        xt, bt, rt = cb.fromFloat32(x, [rows, in_dim]), cb.fromFloat32(b, [out_dim]), cb.fromFloat32(res, [rows, out_dim])
        lin = cb.linear(xt, wt, bt, rows, in_dim, out_dim)
        base = cb.toFloat32(lin).reshape(rows, out_dim)

        def values(t):
            assert t is not None and t.shape == [rows, out_dim]
            out = cb.toFloat32(t).reshape(rows, out_dim)
            cb.freeTensor(t)
            return out

        assert np.array_equal(values(cb.linearRelu(xt, wt, bt, rows, in_dim, out_dim)), np.maximum(base, 0))
        assert np.array_equal(values(cb.linearAdd(xt, wt, bt, rt, rows, in_dim, out_dim)), base + res)
        scale = 1e-6 * np.abs(base).max()
        assert np.allclose(values(cb.linearQuickGelu(xt, wt, bt, rows, in_dim, out_dim)),
                           O.apply_activation(O.QUICK_GELU, base), rtol=3e-6, atol=scale)
        assert np.allclose(values(cb.linearGelu(xt, wt, bt, rows, in_dim, out_dim)), O.apply_activation(O.GELU, base),
                           rtol=3e-6, atol=scale)
        # a dense f32 weight has no fused path here: the optional op answers None
        cb.insertWeightFromTensor("dense.weight", np.zeros((4, in_dim), np.float32), [4, in_dim])
        dense = cb.getWeight("dense.weight")
        b4 = cb.fromFloat32(np.zeros(4, np.float32), [4])
        assert cb.linearRelu(xt, dense, b4, rows, in_dim, 4) is None
        with pytest.raises(_lib.InvalidShape):
            cb.linearAdd(xt, wt, bt, bt, rows, in_dim, out_dim)  # residual of the wrong size
        for t in (lin, xt, bt, rt, b4):
            cb.freeTensor(t)
    finally:
        cb.deinit()


@pytest.mark.parametrize("fmt", [Q8, Q4])
def test_backend_linear_pair_triple(fmt):
    """ComputeBackend linearPair / linearTriple match the separate biased linears exactly
    (the reference's own tests of the wrappers, ops/native_compute.zig:39225-39326)."""
    rows, in_dim, out_dim = 3, 1024, 768
    print(f"case: backend linear / linearPair / linearTriple fmt={fmt}", flush=True)
    cb = HipCompute()
    try:
        x = synth.activations(630, rows, in_dim)
        xt = cb.fromFloat32(x, [rows, in_dim])
        ws, bs, wts, bts, singles = [], [], [], [], []
        for i, name in enumerate(("attn_q", "attn_k", "attn_v")):
            ws.append(synth.weights(fmt, 631 + i, out_dim, in_dim))
            bs.append(bias_vector(641 + i, out_dim))
            cb.insertWeightFromLoaded(f"blk.0.{name}.weight", fmt, ws[i], [out_dim, in_dim])
            wts.append(cb.getWeight(f"blk.0.{name}.weight"))
            bts.append(cb.fromFloat32(bs[i], [out_dim]))
            t = cb.linear(xt, wts[i], bts[i], rows, in_dim, out_dim)
            assert t.shape == [rows, out_dim]
            singles.append(cb.toFloat32(t).reshape(rows, out_dim))
            cb.freeTensor(t)
            ref = O.linear(fmt, x, ws[i], bs[i], rows, in_dim, out_dim, workers=8)
            assert G.max_rel_err(singles[i], ref.astype(np.float64)) <= TIGHT
        pair = cb.linearPair(xt, wts[0], bts[0], wts[1], bts[1], rows, in_dim, out_dim)
        triple = cb.linearTriple(xt, wts[0], bts[0], wts[1], bts[1], wts[2], bts[2], rows, in_dim, out_dim)
        for i, t in enumerate(pair):
            assert np.array_equal(cb.toFloat32(t).reshape(rows, out_dim), singles[i])
        for i, t in enumerate(triple):
            assert np.array_equal(cb.toFloat32(t).reshape(rows, out_dim), singles[i])
        for t in (*pair, *triple):
            cb.freeTensor(t)
        # error contract (cuda_compute.zig:551-554): bias must be f32 with out_dim elements
        bad = cb.fromFloat32(np.zeros(out_dim + 1, np.float32), [out_dim + 1])
        with pytest.raises(_lib.InvalidShape):
            cb.linear(xt, wts[0], bad, rows, in_dim, out_dim)
        with pytest.raises(_lib.InvalidShape):
            cb.linearTriple(xt, wts[0], bts[0], wts[1], bts[1], wts[2], bad, rows, in_dim, out_dim)
        with pytest.raises(_lib.UnsupportedTensorType):
            cb.linear(xt, wts[0], wts[1], rows, in_dim, out_dim)  # a quantized tensor is no bias
        for t in (bad, xt, *bts):
            cb.freeTensor(t)
    finally:
        cb.deinit()
