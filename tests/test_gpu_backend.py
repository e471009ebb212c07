"""The backend object (HipCompute) through the C ABI: same op contract, ownership
and error behaviour as the reference's CUDA backend (ops/cuda/cuda_compute.zig)
and the native planned op (ops/native_compute.zig:42750-42831)."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

pytest.importorskip("torch")

from antfly_amd import _lib, quant_matmul as qm, synth  # noqa: E402
from antfly_amd.hip_compute import HipCompute  # noqa: E402
from oracle import oracle as O  # noqa: E402
from tests import gpu_util as G  # noqa: E402

Q4, Q8 = _lib.TYPE_Q4_0, _lib.TYPE_Q8_0


@pytest.fixture()
def cb():
    c = HipCompute()
    yield c
    c.deinit()


def test_backend_identity(cb):
    assert cb.backendKind() == "hip"
    assert "gfx950" in cb.deviceName()
    assert cb.stream != 0


@pytest.mark.parametrize("fmt", [Q8, Q4])
@pytest.mark.parametrize("keep_raw", [False, True])
def test_linear_no_bias_matches_cpu_engine(cb, fmt, keep_raw):
    rows, in_dim, out_dim = 5, 1024, 768
    print(f"case: backend linearNoBias fmt={fmt} keep_raw={keep_raw}", flush=True)
    w = synth.weights(fmt, 5, out_dim, in_dim)
    x = synth.activations(6, rows, in_dim)
    cb.insertWeightFromLoaded("blk.0.ffn_up.weight", fmt, w, [out_dim, in_dim], keep_raw_layout=keep_raw)
    wt = cb.getWeight("blk.0.ffn_up.weight")
    assert wt.dtype == _lib.DTYPE_U8 and wt.quant_type == fmt and wt.elem_count == out_dim * in_dim
    assert wt.shape == [out_dim, in_dim] and wt.byte_len >= w.size
    assert wt.layout == (_lib.LAYOUT_RAW if keep_raw else _lib.LAYOUT_PREPARED)
    xt = cb.fromFloat32(x, [rows, in_dim])
    yt = cb.linearNoBias(xt, wt, rows, in_dim, out_dim)
    assert yt.shape == [rows, out_dim] and yt.dtype == _lib.DTYPE_F32 and yt.quant_type is None
    y = cb.toFloat32(yt).reshape(rows, out_dim)
    ref = O.linear_no_bias(fmt, x, w, rows, in_dim, out_dim, workers=8)
    assert G.max_rel_err(y, ref.astype(np.float64)) <= 2e-5
    # weights are borrowed: freeing the handle is a no-op and the weight stays usable
    cb.freeTensor(wt)
    yt2 = cb.linearNoBias(xt, cb.getWeight("blk.0.ffn_up.weight"), rows, in_dim, out_dim)
    assert np.array_equal(cb.toFloat32(yt2).reshape(rows, out_dim), y)
    stats = cb.debugStats()
    assert stats["launches_small_batch"] == 2 and stats["resident_weight_bytes"] >= w.size
    assert stats["launches_prepare"] == (0 if keep_raw else 1)
    # five rows: a separate kernel quantizes the activations, once per op
    assert stats["launches_activation_quant"] == 2
    # two rows on repacked weights: the GEMV quantizes them in its own prologue; the
    # generic kernels (raw GGUF layout) always read activations quantized beforehand
    x2t = cb.fromFloat32(x[:2], [2, in_dim])
    y2 = cb.toFloat32(cb.linearNoBias(x2t, wt, 2, in_dim, out_dim)).reshape(2, out_dim)
    ref2 = O.linear_no_bias(fmt, x[:2], w, 2, in_dim, out_dim, workers=8)
    assert G.max_rel_err(y2, ref2.astype(np.float64)) <= 2e-5
    assert cb.debugStats()["launches_activation_quant"] == (3 if keep_raw else 2)
    for t in (yt, yt2, xt):
        cb.freeTensor(t)
    assert cb.debugStats()["pooled_buffers"] >= 2


@pytest.mark.parametrize("rows", [1, 5, 24])
def test_linear_no_bias_pair(cb, rows):
    """linearNoBiasPair (ops/ops.zig:909): (X @ Wa^T, X @ Wb^T), both equal to the single op."""
    in_dim, out_dim = 1024, 768
    print(f"case: backend linearNoBiasPair rows={rows}", flush=True)
    x = synth.activations(16, rows, in_dim)
    wa, wb = synth.weights(Q4, 17, out_dim, in_dim), synth.weights(Q4, 18, out_dim, in_dim)
    cb.insertWeightFromLoaded("gate", Q4, wa, [out_dim, in_dim])
    cb.insertWeightFromLoaded("up", Q4, wb, [out_dim, in_dim])
    cb.insertWeightFromLoaded("up_raw", Q4, wb, [out_dim, in_dim], keep_raw_layout=True)
    xt = cb.fromFloat32(x, [rows, in_dim])
    first, second = cb.linearNoBiasPair(xt, cb.getWeight("gate"), cb.getWeight("up"), rows, in_dim, out_dim)
    assert first.shape == [rows, out_dim] and second.shape == [rows, out_dim]
    ya, yb = cb.toFloat32(first), cb.toFloat32(second)
    assert np.array_equal(ya, cb.toFloat32(cb.linearNoBias(xt, cb.getWeight("gate"), rows, in_dim, out_dim)))
    assert np.array_equal(yb, cb.toFloat32(cb.linearNoBias(xt, cb.getWeight("up"), rows, in_dim, out_dim)))
    ref = O.linear_no_bias(Q4, x, wb, rows, in_dim, out_dim, workers=8)
    assert G.max_rel_err(yb.reshape(rows, out_dim), ref.astype(np.float64)) <= 2e-5
    # different layouts: served as two independent ops, same results
    f2, s2 = cb.linearNoBiasPair(xt, cb.getWeight("gate"), cb.getWeight("up_raw"), rows, in_dim, out_dim)
    assert np.array_equal(cb.toFloat32(f2), ya)
    assert G.max_rel_err(cb.toFloat32(s2).reshape(rows, out_dim), ref.astype(np.float64)) <= 2e-5
    with pytest.raises(_lib.InvalidShape):
        cb.linearNoBiasPair(xt, cb.getWeight("gate"), cb.getWeight("up"), rows, in_dim, out_dim + 1)


def test_freed_buffers_are_reused(cb):
    x = synth.activations(1, 4, 256)
    a = cb.fromFloat32(x, [4, 256])
    ptr = a.device_ptr
    cb.freeTensor(a)
    allocs = cb.debugStats()["device_allocs"]
    b = cb.fromFloat32(x, [4, 256])
    assert b.device_ptr == ptr and cb.debugStats()["device_allocs"] == allocs
    cb.freeTensor(b)


def test_op_errors(cb):
    in_dim, out_dim = 256, 512
    w = synth.weights(Q8, 1, out_dim, in_dim)
    cb.insertWeightFromLoaded("w", Q8, w, [out_dim, in_dim])
    cb.insertWeightFromLoaded("w_q6k", 14, np.zeros(210 * 2, np.uint8), [2, 256])  # resident, but no kernel here
    cb.insertWeightFromTensor("w_dense", np.zeros((out_dim, in_dim), np.float32), [out_dim, in_dim])
    x = cb.fromFloat32(synth.activations(2, 2, in_dim), [2, in_dim])
    with pytest.raises(_lib.WeightNotFound):
        cb.getWeight("missing")
    with pytest.raises(_lib.InvalidShape):
        cb.linearNoBias(x, cb.getWeight("w"), 3, in_dim, out_dim)        # input count mismatch
    with pytest.raises(_lib.InvalidShape):
        cb.linearNoBias(x, cb.getWeight("w"), 2, in_dim, out_dim + 1)    # weight count mismatch
    with pytest.raises(_lib.UnsupportedTensorType):
        cb.linearNoBias(cb.getWeight("w"), cb.getWeight("w"), 2, in_dim, out_dim)  # quantized input
    with pytest.raises(_lib.UnsupportedTensorType):
        cb.linearNoBias(cb.fromFloat32(np.zeros(2 * 256, np.float32), [2, 256]), cb.getWeight("w_q6k"), 2, 256, 2)
    with pytest.raises(_lib.HipOpUnsupported):
        cb.linearNoBias(x, cb.getWeight("w_dense"), 2, in_dim, out_dim)
    with pytest.raises(_lib.InvalidShape):
        cb.fromFloat32(np.zeros(8, np.float32), [3, 3])
    with pytest.raises(_lib.InvalidShape):
        cb.fromFloat32(np.zeros(8, np.float32), [-1, 8])
    with pytest.raises(_lib.UnsupportedTensorType):
        cb.toFloat32(cb.getWeight("w"))
    # in_dim not a multiple of 32: the launcher rejects it (kernels.zig:1231)
    cb.insertWeightFromLoaded("w_bad", Q8, np.zeros(34 * 4, np.uint8), [4, 33], keep_raw_layout=True)
    xb = cb.fromFloat32(np.zeros(33, np.float32), [1, 33])
    with pytest.raises(_lib.InvalidHipState):
        cb.linearNoBias(xb, cb.getWeight("w_bad"), 1, 33, 4)
    # zero rows: a valid empty result
    empty = cb.fromFloat32(np.zeros(0, np.float32), [0, in_dim])
    out = cb.linearNoBias(empty, cb.getWeight("w"), 0, in_dim, out_dim)
    assert out.shape == [0, out_dim] and cb.toFloat32(out).size == 0


def test_planned_op_follows_reference_test(cb, kats):
    k = kats["planned_op"]
    rows, in_dim, out_dim = k["rows"], k["in_dim"], k["out_dim"]

    def fill(n, seed, scale):  # fillNativeQuantDispatchValues, native_compute.zig:42444-42449
        idx = np.arange(n)
        return ((((idx * 17 + seed * 31 + 7) % 67) - 33) * scale).astype(np.float32)

    x = fill(rows * in_dim, rows, 0.015)
    w = O.quantize_weights(Q8, fill(out_dim * in_dim, in_dim, 0.0125))
    cb.insertWeightFromLoaded("planned_q8_0.weight", Q8, w, [out_dim, in_dim])
    wt = cb.getWeight("planned_q8_0.weight")
    xt = cb.fromFloat32(x, [rows, in_dim])
    good = qm.OperatorPlan(qm.OperatorPlanKind.quant_matmul, qm.plan(qm.Shape(rows, in_dim, out_dim, qm.Format.q8_0)))
    out = cb.linearNoBiasWithPlan(xt, wt, rows, in_dim, out_dim, good)
    y = cb.toFloat32(out)
    assert y.size == rows * out_dim and np.isfinite(y).all()
    ref = O.linear_no_bias(Q8, x.reshape(rows, in_dim), w, rows, in_dim, out_dim)
    assert G.max_rel_err(y.reshape(rows, out_dim), ref.astype(np.float64)) <= 2e-5
    eager = cb.toFloat32(cb.linearNoBiasWithPlan(xt, wt, rows, in_dim, out_dim, None))
    assert np.array_equal(eager, y)

    bad_rows = qm.OperatorPlan(qm.OperatorPlanKind.quant_matmul, qm.plan(qm.Shape(rows + 1, in_dim, out_dim, qm.Format.q8_0)))
    bad_fmt = qm.OperatorPlan(qm.OperatorPlanKind.quant_matmul, qm.plan(qm.Shape(rows, in_dim, out_dim, qm.Format.q4_0)))
    fallback = qm.plan(qm.Shape(rows, in_dim, out_dim, qm.Format.q8_0))
    fallback.operator = qm.Operator.fallback
    row_plan = qm.OperatorPlan(qm.OperatorPlanKind.quant_row, None)
    for bad in (bad_rows, bad_fmt, qm.OperatorPlan(qm.OperatorPlanKind.quant_matmul, fallback), row_plan):
        with pytest.raises(_lib.InvalidPartitionPlan):
            cb.linearNoBiasWithPlan(xt, wt, rows, in_dim, out_dim, bad)


def test_torch_memory_can_be_wrapped(cb):
    import torch

    rows, in_dim, out_dim = 2, 512, 512
    w = synth.weights(Q4, 3, out_dim, in_dim)
    x = synth.activations(4, rows, in_dim)
    cb.insertWeightFromLoaded("w", Q4, w, [out_dim, in_dim])
    xd = torch.from_numpy(x).to("cuda:0")
    torch.cuda.synchronize()
    xt = cb.wrapDeviceFloat32(xd.data_ptr(), [rows, in_dim])
    y = cb.toFloat32(cb.linearNoBias(xt, cb.getWeight("w"), rows, in_dim, out_dim)).reshape(rows, out_dim)
    ref = O.linear_no_bias(Q4, x, w, rows, in_dim, out_dim)
    assert G.max_rel_err(y, ref.astype(np.float64)) <= 2e-5
    cb.freeTensor(xt)  # does not free torch's memory
    assert torch.equal(xd.cpu(), torch.from_numpy(x))


@pytest.mark.parametrize("fmt", [Q8, Q4])
def test_lm_head_ops(cb, fmt, kats):
    """argmaxLastRow, linearNoBiasArgmaxLastRow(+Tensor) and linearNoBiasGrouped on the backend object."""
    rows, in_dim, out_dim = 3, 512, 2048
    print(f"case: backend lm_head ops fmt={fmt}", flush=True)
    lr = kats["argmax"]["last_row"]
    t = cb.fromFloat32(np.array(lr["data"], np.float32), [lr["rows"], lr["dim"]])
    assert cb.argmaxLastRow(t, lr["rows"], lr["dim"]) == lr["expect"]
    with pytest.raises(_lib.InvalidShape):
        cb.argmaxLastRow(t, 0, 3)
    with pytest.raises(_lib.InvalidShape):
        cb.argmaxLastRow(t, 2, 4)
    cb.freeTensor(t)

    w = synth.weights(fmt, 21, out_dim, in_dim)
    x = synth.activations(22, rows, in_dim)
    cb.insertWeightFromLoaded("lm_head.weight", fmt, w, [out_dim, in_dim])
    wt = cb.getWeight("lm_head.weight")
    xt = cb.fromFloat32(x, [rows, in_dim])
    logits = cb.linearNoBias(xt, wt, rows, in_dim, out_dim)
    want = cb.argmaxLastRow(logits, rows, out_dim)
    assert want == int(np.argmax(cb.toFloat32(logits).reshape(rows, out_dim)[-1]))
    before = cb.debugStats()["launches_mmv"]
    assert cb.linearNoBiasArgmaxLastRow(xt, wt, rows, in_dim, out_dim) == want
    assert cb.debugStats()["launches_mmv"] == before + 1  # one GEMV over the last row, whatever `rows` is
    tt = cb.linearNoBiasArgmaxLastRowTensor(xt, wt, rows, in_dim, out_dim)
    assert tt.shape == [1] and tt.dtype == _lib.DTYPE_F32
    assert cb.toFloat32(tt).tolist() == [float(want)]
    cb.freeTensor(tt)
    ref = O.linear_no_bias(fmt, x, w, rows, in_dim, out_dim, workers=8)
    ref_token = O.argmax_last_row(ref, rows, out_dim)
    assert want == ref_token or ref[-1, ref_token] - ref[-1, want] <= 2e-5 * np.abs(ref[-1]).max()
    with pytest.raises(_lib.InvalidShape):
        cb.linearNoBiasArgmaxLastRow(xt, wt, rows, in_dim, out_dim + 1)

    # grouped: the weight is the concatenation of the projections, one linear serves them
    y = cb.toFloat32(logits)
    g = cb.linearNoBiasGrouped(xt, wt, rows, in_dim, out_dim, [1024, 512, 512], 3)
    assert g.shape == [rows, out_dim] and np.array_equal(cb.toFloat32(g), y)
    cb.freeTensor(g)
    for dims, n in (([1024, 512], 2), ([1024, 0, 1024], 3), ([2048], 0)):
        with pytest.raises(_lib.InvalidShape):
            cb.linearNoBiasGrouped(xt, wt, rows, in_dim, out_dim, dims, n)
    for t in (logits, xt):
        cb.freeTensor(t)



def test_gguf_file_to_device_weights(cb, tmp_path):
    """A GGUF file on disk -> mapped -> resident weights -> the same results as weights inserted from memory."""
    from antfly_amd import gguf
    from tests import gguf_util as W

    in_dim, out_dim, rows = 512, 768, 3
    w4 = synth.weights(Q4, 31, out_dim, in_dim)
    w8 = synth.weights(Q8, 32, out_dim, in_dim)
    norm = synth.activations(33, 1, in_dim)[0]
    img = W.build([("general.architecture", gguf.STRING, "llama"), ("llama.block_count", gguf.U32, 1)],
                  [("blk.0.ffn_gate.weight", [in_dim, out_dim], Q4, w4.tobytes()),
                   ("blk.0.ffn_up.weight", [in_dim, out_dim], Q8, w8.tobytes()),
                   ("blk.0.ffn_norm.weight", [in_dim], 0, norm.tobytes()),
                   ("blk.0.attn_q.weight", [256, 2], 14, bytes(420))])  # Q6_K: not a format this backend computes on
    path = tmp_path / "model.gguf"
    path.write_bytes(img)
    x = synth.activations(34, rows, in_dim)
    with gguf.File.open(str(path)) as f:
        print("case: backend loadGguf", flush=True)
        assert cb.loadGguf(f) == (3, 1)
        with pytest.raises(_lib.UnsupportedTensorType):
            cb.insertWeightFromGguf(f, "blk.0.attn_q.weight")
        with pytest.raises(_lib.TensorNotFound):
            cb.insertWeightFromGguf(f, "blk.9.missing")
        cb.insertWeightFromGguf(f, "blk.0.ffn_up.weight", key="raw_up", keep_raw_layout=True)
    # the file is closed and unmapped: the weights live on the device
    xt = cb.fromFloat32(x, [rows, in_dim])
    for name, fmt, w in (("blk.0.ffn_gate.weight", Q4, w4), ("blk.0.ffn_up.weight", Q8, w8), ("raw_up", Q8, w8)):
        wt = cb.getWeight(name)
        assert wt.quant_type == fmt and wt.shape == [out_dim, in_dim]
        cb.insertWeightFromLoaded("direct", fmt, w, [out_dim, in_dim], keep_raw_layout=(name == "raw_up"))
        y = cb.toFloat32(cb.linearNoBias(xt, wt, rows, in_dim, out_dim))
        y_direct = cb.toFloat32(cb.linearNoBias(xt, cb.getWeight("direct"), rows, in_dim, out_dim))
        assert np.array_equal(y, y_direct)
        ref = O.linear_no_bias(fmt, x, w, rows, in_dim, out_dim, workers=8)
        assert G.max_rel_err(y.reshape(rows, out_dim), ref.astype(np.float64)) <= 2e-5
    nt = cb.getWeight("blk.0.ffn_norm.weight")
    assert nt.dtype == _lib.DTYPE_F32 and nt.shape == [in_dim]
    assert np.array_equal(cb.toFloat32(nt), norm)


def test_phase_timing_is_opt_in(cb):
    """afhip_compute_set_phase_timing: device time of the stand-alone activation quantizer and of
    the compute kernels per linear op (the engine's timing snapshot, ops/ops.zig:649-713)."""
    in_dim, out_dim = 1024, 768
    w = synth.weights(_lib.TYPE_Q8_0, 70, out_dim, in_dim)
    cb.insertWeightFromLoaded("timed.weight", _lib.TYPE_Q8_0, w, [out_dim, in_dim])
    wt = cb.getWeight("timed.weight")
    x = synth.activations(71, 24, in_dim)
    xt = cb.fromFloat32(x, [24, in_dim])
    cb.freeTensor(cb.linearNoBias(xt, wt, 24, in_dim, out_dim))
    s0 = cb.debugStats()
    assert s0["timed_ops"] == 0 and s0["activation_quant_ns"] == 0 and s0["compute_ns"] == 0
    cb.setPhaseTiming(True)
    y = cb.toFloat32(cb.linearNoBias(xt, wt, 24, in_dim, out_dim)).reshape(24, out_dim)  # quantizer + MFMA GEMM
    s1 = cb.debugStats()
    assert s1["timed_ops"] == 1 and s1["activation_quant_ns"] > 0 and s1["compute_ns"] > 0
    x1 = cb.fromFloat32(x[:1], [1, in_dim])
    cb.freeTensor(cb.linearNoBias(x1, wt, 1, in_dim, out_dim))  # one row: quantized in the kernel's prologue
    s2 = cb.debugStats()
    assert s2["timed_ops"] == 2 and s2["compute_ns"] > s1["compute_ns"]
    cb.setPhaseTiming(False)
    cb.freeTensor(cb.linearNoBias(xt, wt, 24, in_dim, out_dim))
    assert cb.debugStats()["timed_ops"] == 2
    ref = O.linear_no_bias(_lib.TYPE_Q8_0, x, w, 24, in_dim, out_dim, workers=8)
    assert G.max_rel_err(y, ref.astype(np.float64)) <= 2e-5


def test_q4k_route_switch_of_the_backend(cb):
    """Q4_K on one of the CPU engine's gated shapes (one row, K = 2048): by default the backend follows that engine
    onto Q8_K activations; afhip_compute_set_q4k_f32_activations keeps f32 activations, which is what the engine's
    CUDA backend computes (ops/cuda/cuda_compute.zig:708).  The two numbers differ by the activation quantization."""
    in_dim, out_dim = 2048, 1024
    w = synth.weights(_lib.TYPE_Q4_K, 90, out_dim, in_dim)
    cb.insertWeightFromLoaded("switch.weight", _lib.TYPE_Q4_K, w, [out_dim, in_dim])
    wt = cb.getWeight("switch.weight")
    x = synth.activations(91, 1, in_dim)
    xt = cb.fromFloat32(x, [1, in_dim])
    assert O.uses_q4k_q8k_activation(1, in_dim, out_dim)
    q8k = O.linear_q4_k_q8k(x, w, 1, in_dim, out_dim).astype(np.float64)
    f32 = O.linear_q4_k(x, w, 1, in_dim, out_dim, f64=True)
    y = cb.toFloat32(cb.linearNoBias(xt, wt, 1, in_dim, out_dim)).reshape(1, out_dim)
    assert G.max_rel_err(y, q8k) <= 2e-5 and G.max_rel_err(y, f32) > 2e-4
    cb.setQ4KF32Activations(True)
    y = cb.toFloat32(cb.linearNoBias(xt, wt, 1, in_dim, out_dim)).reshape(1, out_dim)
    assert G.max_rel_err(y, f32) <= 2e-5 and G.max_rel_err(y, q8k) > 2e-4
    cb.setQ4KF32Activations(False)
    y = cb.toFloat32(cb.linearNoBias(xt, wt, 1, in_dim, out_dim)).reshape(1, out_dim)
    assert G.max_rel_err(y, q8k) <= 2e-5
