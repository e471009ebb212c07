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
          (12, 256, 530), (40, 512, 640), (300, 512, 1024), (3, 64, 100)]


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
    torch.cuda.synchronize()


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
