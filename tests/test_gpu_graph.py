"""The launchers under HIP graph capture: a decode-like sequence of calls recorded once and
replayed several times, with eager work and synchronizations of the same program between the
replays, must give on every replay exactly the bytes the eager calls gave.  (Every kernel here
is deterministic -- K slices and K shares are summed in a fixed order -- so the comparison is
bit for bit.)  Shapes cover every kernel family: fused GEMV, quantizer + rows kernel,
quantizer + MFMA GEMM, the Q4_K decode kernel, the Q4_K prefill GEMM with K shared out over
workgroups (partial sums + ordered reduce), the lm_head argmax and a row operator."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")

from antfly_amd import _lib, kernels, synth  # noqa: E402
from tests import gpu_util as G  # noqa: E402

Q4, Q8, Q4K = _lib.TYPE_Q4_0, _lib.TYPE_Q8_0, _lib.TYPE_Q4_K
PREP = _lib.LAYOUT_PREPARED

# (format, rows, in_dim, out_dim)
CALLS = [
    (Q4, 1, 1024, 1536),    # fused GEMV
    (Q8, 2, 1024, 640),     # fused GEMV, two rows
    (Q4, 6, 1024, 1536),    # quantizer + rows kernel
    (Q8, 40, 1024, 640),    # quantizer + MFMA GEMM
    (Q4K, 1, 1024, 200),    # Q4_K int8 decode kernel (ragged last tile)
    (Q4K, 5, 1024, 200),    # Q4_K digit-plane kernel + int8 kernel on the planes, several rows
    (Q4K, 20, 4096, 300),   # Q4_K prefill GEMM, K shared out over workgroups
    (Q4K, 70, 1024, 200),   # Q4_K prefill GEMM, three row groups
    (Q4, 7, 512, 8200),     # compact-fragment quantizer + eight-row MFMA kernel
]


def test_graph_replays_equal_eager():
    st = G.stream()
    ops = []
    for i, (fmt, rows, k, n) in enumerate(CALLS):
        w = G.prepare(fmt, synth.weights(fmt, 900 + i, n, k), n, k)
        x = G.to_dev(synth.activations(950 + i, rows, k))
        y = torch.zeros((rows, n), dtype=torch.float32, device=G.DEV)
        ws = torch.empty(max(kernels.workspaceBytes(fmt, rows, k, n), 16), dtype=torch.uint8, device=G.DEV)
        ops.append((fmt, rows, k, n, w, x, y, ws))
    # greedy head on the last row of the 6-row activations, and a dequantize of one weight
    head_fmt, head_rows, head_k, head_n = Q4, 6, 1024, 1536
    head_w, head_x = ops[2][4], ops[2][5]
    token = torch.zeros(1, dtype=torch.int32, device=G.DEV)
    head_ws = torch.empty(max(kernels.linearArgmaxWorkspaceBytes(head_fmt, head_k, head_n), 16),
                          dtype=torch.uint8, device=G.DEV)
    deq = torch.zeros((640, 1024), dtype=torch.float32, device=G.DEV)

    def run_all(s):
        for fmt, rows, k, n, w, x, y, ws in ops:
            kernels.launchLinearF32(s, fmt, PREP, G.buf(y), G.buf(x), G.buf(w), rows, k, n, G.buf(ws), -1)
        kernels.launchLinearArgmaxLastRowF32(s, head_fmt, PREP, G.buf(token), kernels.NO_BUFFER, G.buf(head_x), G.buf(head_w),
                                             head_rows, head_k, head_n, G.buf(head_ws))
        kernels.launchDequantizeF32(s, Q8, PREP, G.buf(deq), G.buf(ops[1][4]), 640, 1024)

    def snapshot():
        torch.cuda.synchronize()
        return [o[6].cpu().numpy().copy() for o in ops] + [token.cpu().numpy().copy(), deq.cpu().numpy().copy()]

    def clear():
        for o in ops:
            o[6].fill_(float("nan"))
        token.fill_(-1)
        deq.fill_(float("nan"))

    print("case: eager pass (also the first call of every shape class, outside any capture)", flush=True)
    run_all(st)
    want = snapshot()
    assert all(np.isfinite(a).all() for a in want[:-2])

    print("case: capture", flush=True)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        run_all(torch.cuda.current_stream().cuda_stream)

    for replay in range(4):
        print(f"case: replay {replay}", flush=True)
        clear()
        # the program's own eager work between replays: a different call through the same scratch
        fmt, rows, k, n, w, x, y, ws = ops[3]
        kernels.launchLinearF32(st, fmt, PREP, G.buf(y), G.buf(x), G.buf(w), rows, k, n, G.buf(ws), -1)
        torch.cuda.synchronize()
        clear()
        graph.replay()
        got = snapshot()
        for idx, (a, b) in enumerate(zip(got, want)):
            assert a.tobytes() == b.tobytes(), f"replay {replay}: output {idx} differs from the eager result"
