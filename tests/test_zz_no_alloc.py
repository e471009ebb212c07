"""The entry point that allocates nothing (afhip_launch_linear_f32_static): same results, bit
for bit, as afhip_launch_linear_f32 with a caller-provided workspace -- on two calls in a row,
the second with a smaller input (the library's scratch array keeps the first call's contents)."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")

from antfly_amd import _lib, kernels, synth  # noqa: E402
from oracle import oracle as O  # noqa: E402
from tests import gpu_util as G  # noqa: E402

Q4, Q8 = _lib.TYPE_Q4_0, _lib.TYPE_Q8_0
PREP = _lib.LAYOUT_PREPARED


def static_linear(fmt, x, w_dev, rows, in_dim, out_dim):
    """One eager call, then the same call recorded into a HIP graph and replayed: a library that
    allocated device memory inside the call could not be captured (hipMalloc is refused while a
    stream is capturing)."""
    xd = G.to_dev(x.astype(np.float32))
    y = torch.full((rows, out_dim), float("nan"), dtype=torch.float32, device=G.DEV)
    kernels.launchLinearF32Static(G.stream(), fmt, PREP, G.buf(y), G.buf(xd), G.buf(w_dev), rows, in_dim, out_dim)
    torch.cuda.synchronize()
    eager = y.cpu().numpy()
    y.fill_(float("nan"))
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        kernels.launchLinearF32Static(torch.cuda.current_stream().cuda_stream, fmt, PREP, G.buf(y), G.buf(xd), G.buf(w_dev), rows,
                                      in_dim, out_dim)
    graph.replay()
    torch.cuda.synchronize()
    assert np.array_equal(y.cpu().numpy(), eager)
    return eager


@pytest.mark.parametrize("fmt", [Q4, Q8])
def test_static_scratch_entry_matches_workspace_entry(fmt):
    kernels.staticScratchInit()
    # first call: MFMA GEMM with K shared out over workgroups (quantized X and partial sums in
    # the scratch); second, smaller: eight rows through the small-batch kernels (quantized X only)
    cases = [(96, 4096, 1024), (8, 1024, 640), (1, 4096, 512)]
    for rows, in_dim, out_dim in cases:
        print(f"case: static scratch fmt={fmt} rows={rows} in={in_dim} out={out_dim}", flush=True)
        assert 0 < kernels.workspaceBytes(fmt, rows, in_dim, out_dim) or rows == 1
        x = synth.activations(7000 + rows, rows, in_dim)
        w = synth.weights(fmt, 7001 + rows, out_dim, in_dim)
        wd = G.prepare(fmt, w, out_dim, in_dim)
        got = static_linear(fmt, x, wd, rows, in_dim, out_dim)
        want = G.linear(fmt, PREP, x, wd, rows, in_dim, out_dim)
        assert np.array_equal(got, want)
        ref = O.linear_no_bias(fmt, x, w, rows, in_dim, out_dim, workers=8)
        assert G.max_rel_err(got, ref.astype(np.float64)) <= 2e-5


def test_static_scratch_entry_refuses_what_does_not_fit():
    rows, in_dim, out_dim = 4096, 14336, 512  # 56 MiB of quantized activations
    assert kernels.workspaceBytes(Q4, rows, in_dim, out_dim) > kernels.STATIC_SCRATCH_BYTES
    one = torch.zeros(16, dtype=torch.uint8, device=G.DEV)
    with pytest.raises(_lib.HipOpUnsupported):
        kernels.launchLinearF32Static(G.stream(), Q4, PREP, G.buf(one), G.buf(one), G.buf(one), rows, in_dim, out_dim)
