"""GPU parity for the greedy lm_head ops: argmax over the last row and
argmax(X[last] @ W^T) without the logits matrix, through the C ABI, against the
CPU oracle.  Token ids are integers: they must be equal, except where two logits
are closer than the f32 accumulation tolerance (then either is the reference's
answer under some thread plan, and the test says which case it hit)."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")

from antfly_amd import _lib, kernels, synth  # noqa: E402
from oracle import oracle as O  # noqa: E402
from tests import gpu_util as G  # noqa: E402

Q4, Q8 = _lib.TYPE_Q4_0, _lib.TYPE_Q8_0
RAW, PREP = _lib.LAYOUT_RAW, _lib.LAYOUT_PREPARED
TIGHT = 2e-5


def device_argmax(data: np.ndarray, rows: int, dim: int):
    """Both forms of the launcher: one workgroup (no workspace) and many workgroups + key pick."""
    x = G.to_dev(np.asarray(data, np.float32).reshape(rows, dim))
    got = []
    for with_workspace in (False, True):
        tok = torch.full((2,), -1, dtype=torch.int32, device=G.DEV)
        tok_f = torch.full((2,), -1.0, dtype=torch.float32, device=G.DEV)
        ws = kernels.NO_BUFFER
        if with_workspace:
            scratch = torch.full((kernels.argmaxWorkspaceBytes(dim) + 8,), 0xFF, dtype=torch.uint8, device=G.DEV)
            ws = G.buf(scratch)
        kernels.launchArgmaxLastRowF32(G.stream(), G.buf(tok[:1]), G.buf(tok_f[:1]), G.buf(x), rows, dim, ws)
        torch.cuda.synchronize()
        t, tf = tok.cpu().numpy(), tok_f.cpu().numpy()
        assert t[1] == -1 and tf[1] == -1.0  # one word each, nothing past it
        assert float(t[0]) == tf[0]
        got.append(int(t[0]))
    assert got[0] == got[1]
    return got[0]


def test_argmax_reference_vectors(kats):
    for case in kats["argmax"]["cases"]:
        print(f"case: argmax kat {case['data']}", flush=True)
        assert device_argmax(case["data"], 1, len(case["data"])) == case["expect"]
    lr = kats["argmax"]["last_row"]
    assert device_argmax(lr["data"], lr["rows"], lr["dim"]) == lr["expect"]


@pytest.mark.parametrize("dim", [1, 63, 64, 65, 1000, 1024, 1025, 16384, 16385, 24577, 32000, 128256])
def test_argmax_matches_oracle(dim):
    rng = np.random.default_rng(dim)
    print(f"case: argmax dim={dim}", flush=True)
    rows = 3
    # few distinct values: many equal maxima, the first one must win
    ties = rng.integers(-4, 5, size=(rows, dim)).astype(np.float32)
    assert device_argmax(ties, rows, dim) == O.argmax_last_row(ties, rows, dim)
    smooth = rng.standard_normal((rows, dim)).astype(np.float32)
    assert device_argmax(smooth, rows, dim) == O.argmax_last_row(smooth, rows, dim)
    # the maximum in the last position, and all-negative rows
    smooth[-1, -1] = 100.0
    assert device_argmax(smooth, rows, dim) == dim - 1
    # equal maxima in different workgroups' chunks: the lowest index
    smooth[-1, 0] = smooth[-1, dim // 2] = 100.0
    assert device_argmax(smooth, rows, dim) == 0
    neg = -np.abs(smooth) - 1.0
    assert device_argmax(neg, rows, dim) == O.argmax_last_row(neg, rows, dim)


def test_argmax_special_values():
    cases = [
        [-1.0, -0.0, 0.0],
        [0.0, -0.0, 0.0],
        [-np.inf, -np.inf],
        [1.0, np.inf, np.nan, np.inf],
        [np.nan, -2.0, np.nan, -1.0],
        [np.nan, np.nan],
        [-3.4e38, -1e-45, -2e-45],
    ]
    for c in cases:
        print(f"case: argmax special {c}", flush=True)
        assert device_argmax(c, 1, len(c)) == O.argmax(c)


def test_argmax_rejects_empty_shapes():
    x = torch.zeros(8, dtype=torch.float32, device=G.DEV)
    tok = torch.zeros(1, dtype=torch.int32, device=G.DEV)
    for rows, dim in ((0, 4), (2, 0)):
        with pytest.raises(_lib.InvalidShape):
            kernels.launchArgmaxLastRowF32(G.stream(), G.buf(tok), kernels.NO_BUFFER, G.buf(x), rows, dim)
    with pytest.raises(_lib.InvalidShape):  # the tensor is shorter than rows * dim
        kernels.launchArgmaxLastRowF32(G.stream(), G.buf(tok), kernels.NO_BUFFER, G.buf(x), 3, 4)


def linear_argmax(fmt, layout, x, w_dev, rows, in_dim, out_dim) -> int:
    xd = G.to_dev(x.astype(np.float32))
    ws = torch.empty(kernels.linearArgmaxWorkspaceBytes(fmt, in_dim, out_dim), dtype=torch.uint8, device=G.DEV)
    tok = torch.full((1,), -1, dtype=torch.int32, device=G.DEV)
    tok_f = torch.full((1,), -1.0, dtype=torch.float32, device=G.DEV)
    kernels.launchLinearArgmaxLastRowF32(G.stream(), fmt, layout, G.buf(tok), G.buf(tok_f), G.buf(xd), G.buf(w_dev), rows,
                                         in_dim, out_dim, G.buf(ws))
    torch.cuda.synchronize()
    assert float(tok.item()) == tok_f.item()
    return int(tok.item())


LM_SHAPES = [(1, 256, 1000), (5, 1024, 777), (3, 4096, 32000), (2, 14336, 1030),
             (1, 64, 300)]  # the last one takes the f32 route


@pytest.mark.parametrize("fmt", [Q8, Q4])
@pytest.mark.parametrize("layout", [RAW, PREP])
@pytest.mark.parametrize("rows,in_dim,out_dim", LM_SHAPES)
def test_linear_argmax_last_row(fmt, layout, rows, in_dim, out_dim):
    print(f"case: linear argmax fmt={fmt} layout={layout} rows={rows} in={in_dim} out={out_dim}", flush=True)
    w = synth.weights(fmt, 77, out_dim, in_dim)
    x = synth.activations(78, rows, in_dim)
    wd = G.prepare(fmt, w, out_dim, in_dim) if layout == PREP else G.to_dev(w)
    token = linear_argmax(fmt, layout, x, wd, rows, in_dim, out_dim)
    # the same kernels' logits for the last row give the same token
    logits = G.linear(fmt, layout, x[-1:], wd, 1, in_dim, out_dim)
    assert token == int(np.argmax(logits[0]))
    # the reference: logits of all rows, argmax of the last one
    ref = O.linear_no_bias(fmt, x, w, rows, in_dim, out_dim, workers=8)
    want = O.argmax_last_row(ref, rows, out_dim)
    if token != want:  # a near tie inside the accumulation tolerance
        last = ref[-1].astype(np.float64)
        assert last[want] - last[token] <= TIGHT * np.abs(last).max(), (token, want)
        print(f"  near tie: device {token}, oracle {want}", flush=True)


def test_linear_argmax_planted_winner_full_vocabulary():
    """Llama-3 lm_head shape (128256 x 4096, Q4_0): a planted row must win wherever it sits."""
    in_dim, out_dim, fmt = 4096, 128256, Q4
    w = synth.weights(fmt, 9, out_dim, in_dim).copy()
    x = synth.activations(10, 2, in_dim)
    blocks = w.reshape(out_dim, in_dim // 32, 18)
    for planted in (0, 70001, out_dim - 1):
        print(f"case: lm_head planted={planted}", flush=True)
        wp = blocks.copy()
        # weights that follow the sign of the last row of X with the largest scale in the matrix
        sign = (x[-1].reshape(-1, 32) > 0)
        nib = np.where(sign, 15, 0).astype(np.uint8)
        wp[planted, :, 2:] = nib[:, :16] | (nib[:, 16:] << 4)
        wp[planted, :, 0:2] = np.array([1.0], dtype=np.float16).view(np.uint8)
        wd = G.prepare(fmt, wp.reshape(-1), out_dim, in_dim)
        assert linear_argmax(fmt, PREP, x, wd, 2, in_dim, out_dim) == planted
        del wd
