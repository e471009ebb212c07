#!/usr/bin/env python3
"""Benchmark of the MI355X quantized matmul (Q4_0 / Q8_0 `linearNoBias`).

One "step" = the Q4_0 decode GEMV at the Llama-3-8B FFN-up shape (x f32 [1 x 4096],
W [14336 x 4096] in 18-byte blocks), the configuration the headline metric is quoted on,
once on each of `--copies` (16) distinct copies of the weight: 16 launches, 528 MB --
more than the 256 MB Infinity Cache holds, so every launch streams its 33 MB from HBM.

Prints ONE JSON line: metric/value/unit as the benchmark definition names them,
`roofline` for the dominant kernel (algorithmic bytes / HIP-event time against
8 TB/s), `cpu_baseline` (the CPU restatement of the engine's own route, timed on
this host), plus `extra` with the other configurations (small-batch GEMV, K-long
GEMV, Q8_0 GEMV, prefill GEMM).
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_BPS = 8.0e12           # MI355X HBM3E
INT8_MFMA_PEAK_OPS = 5.0e15     # MI355X dense int8 MFMA
BF16_MFMA_PEAK_FLOPS = 2.5e15   # MI355X dense bf16 MFMA
Q4, Q8, Q4K = 2, 8, 12
BLOCK_BYTES = {Q4: 18, Q8: 34}


TRAFFIC_FILE = os.path.join("profiles", "gemv_q4_0_m1_and_gemm_q8_0_m512_counters.md")


def measured_traffic(key="traffic_bytes_per_launch_gemv_q4_0_m1"):
    """HBM bytes per launch of a kernel from the committed counter summary (rocprofv3 --pmc
    FETCH_SIZE / WRITE_SIZE runs of `bench.py --counter-probe`, each scaled by a kernel of
    known traffic in the same run), or None when that file or line is not there.  The figure
    is not measured by this run: `traffic_source` in the output names the file."""
    try:
        with open(os.path.join(ROOT, TRAFFIC_FILE)) as f:
            for line in f:
                if line.startswith(key + ":"):
                    return int(float(line.split(":", 1)[1]))
    except OSError:
        pass
    return None


# Sources a kernel's traffic figure depends on: the counter summary records their hash
# (`kernel_source_sha256_<kernel>: ...`), and a line whose hash no longer matches is reported as stale.
TRAFFIC_SOURCES = {
    "gemv_q4_0_m1": ("gemv_kernels.hip", "gemv_common.h", "device_common.h"),
    "gemm_q8_0_m512": ("gemm_kernels.hip", "device_common.h"),
}


def kernel_source_hash(kernel):
    import hashlib
    h = hashlib.sha256()
    for name in TRAFFIC_SOURCES[kernel]:
        with open(os.path.join(ROOT, "antfly_amd", "csrc", name), "rb") as f:
            h.update(f.read())
    return h.hexdigest()[:16]


def traffic_is_stale(kernel):
    """True when the committed counter summary was made from other kernel sources than the ones in the tree
    (or does not say which)."""
    recorded = None
    try:
        with open(os.path.join(ROOT, TRAFFIC_FILE)) as f:
            for line in f:
                if line.startswith(f"kernel_source_sha256_{kernel}:"):
                    recorded = line.split(":", 1)[1].strip()
    except OSError:
        pass
    try:
        return recorded != kernel_source_hash(kernel)
    except OSError:
        return True


def gemv_bytes(fmt, rows, in_dim, out_dim):
    """Algorithmic bytes of one call: weights once + f32 activations + f32 outputs."""
    return out_dim * (in_dim // 32) * BLOCK_BYTES[fmt] + 4 * rows * in_dim + 4 * rows * out_dim


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=2000)
    ap.add_argument("--warmup", type=int, default=100)
    ap.add_argument("--copies", type=int, default=16, help="distinct weight copies to rotate over")
    ap.add_argument("--no-extra", action="store_true", help="headline configuration only")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--eager", action="store_true", help="launch every step from the host instead of replaying a HIP graph")
    ap.add_argument("--cpu-seconds", type=float, default=10.0)
    ap.add_argument("--repeats", type=int, default=5,
                    help="the timed region (exactly --steps steps) is run this many times; the median run is reported")
    ap.add_argument("--counter-probe", action="store_true",
                    help="for hardware-counter runs: 40 eager launches each of the headline GEMV, of the plain "
                         "read kernel and of the plain copy kernel over the same number of bytes, of the Q8_0 M=512 GEMM, of the 16-row batch kernel and of the Q4_K kernels "
                         "(M=1 and M=512), then exit")
    ap.add_argument("--only", choices=["gemm_q8_m512", "gemm_q8_m128", "gemm_q8_m2048", "row_ops"], default=None,
                    help="launch only this configuration 200 times (for a kernel trace of one shape) and exit")
    ap.add_argument("--shapes", default=None,
                    help="comma-separated fmt:rows:in_dim:out_dim (fmt q4 / q8 / q4k; q4p / q8p: pair calls): time only these calls, print one line each, exit")
    ap.add_argument("--probe", choices=["gemv", "rates", "gemm", "read", "timeline", "timeline8"], default=None,
                    help="timeline8: the same for the eight-row MFMA kernel (afhip_launch_rows8_timeline; --probe-rows 5 or 8): when a wavefront's weight stages are there, when its K loop ends; timeline: the Q4_0 decode kernel's wavefronts read the 100 MHz clock at their phases (afhip_launch_gemv_timeline; --probe-rows 1, 2 or 4): when the quantized activations are ready, when a wavefront's block dots are done; read: a kernel that only reads the headline matrix's 33 MB, swept over workgroup size, loads in flight per lane and load hint (afhip_launch_stream_read_shaped); gemm: the Q8_0 M=512 prefill kernel's own clock readings (afhip_launch_gemm_stamps): cycles in the K loop, waiting for loads and at barriers, and the clock the chip held; rates: instruction issue rates of a SIMD (afhip_launch_rate_probe), print a table, exit; gemv: time the one-row Q4_0 decode kernel with parts left out (afhip_launch_gemv_probe) next to "
                         "a kernel that only reads the same bytes, print a table, exit")
    ap.add_argument("--probe-shape", default="4096:14336",
                    help="--probe timeline: K:N of the matrix, K at most 4096 (one row: 16384; default: the headline's 4096:14336)")
    ap.add_argument("--probe-rows", type=int, choices=[1, 2, 4, 5, 8], default=1,
                    help="--probe gemv: rows of X (the decode kernel's instantiation for that many rows)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)", file=sys.stderr)
        return 2

    import torch

    from antfly_amd import _lib, kernels, synth
    from antfly_amd._lib import Buffer

    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        return 2
    dev = "cuda:0"
    torch.cuda.set_device(0)
    stream = torch.cuda.current_stream().cuda_stream

    def buf(t):
        return Buffer(t.data_ptr(), t.numel() * t.element_size())

    def prepared_copies(fmt, out_dim, in_dim, copies, seed):
        raw = torch.from_numpy(synth.weights(fmt, seed, out_dim, in_dim)).to(dev)
        out = []
        for _ in range(copies):
            p = torch.empty(kernels.preparedWeightBytes(fmt, out_dim, in_dim), dtype=torch.uint8, device=dev)
            kernels.launchPrepareWeight(stream, fmt, buf(p), buf(raw), out_dim, in_dim)
            out.append(p)
        torch.cuda.synchronize()
        return out

    def time_config(fmt, rows, in_dim, out_dim, steps, warmup, copies, seed, repeats=1, pair=False):
        """Returns (wall seconds, event seconds) for `steps` back-to-back calls: the median of
        `repeats` runs of the same timed region.  pair: every call is one pair call (two matrices of
        this shape that share X, as gate and up do)."""
        ws = prepared_copies(fmt, out_dim, in_dim, copies, seed)
        x = torch.from_numpy(synth.activations(seed + 1, rows, in_dim)).to(dev)
        y = torch.empty((rows, out_dim), dtype=torch.float32, device=dev)
        y2 = torch.empty((rows, out_dim), dtype=torch.float32, device=dev) if pair else None
        wsb = kernels.workspaceBytes(fmt, rows, in_dim, out_dim)
        scratch = torch.empty(max(wsb, 16), dtype=torch.uint8, device=dev)
        bx, by, bs = buf(x), buf(y), buf(scratch)
        bws = [buf(w) for w in ws]
        launch = _lib.lib().afhip_launch_linear_f32
        launch_pair = _lib.lib().afhip_launch_linear_pair_f32

        def step(i, st):
            if pair:
                rc = launch_pair(st, fmt, _lib.LAYOUT_PREPARED, by, buf(y2), bx, bws[(2 * i) % copies], bws[(2 * i + 1) % copies],
                                 rows, in_dim, out_dim, bs, -1)
            else:
                rc = launch(st, fmt, _lib.LAYOUT_PREPARED, by, bx, bws[i % copies], rows, in_dim, out_dim, bs, -1)
            if rc != 0:
                raise RuntimeError(f"launch failed: {rc}")

        for i in range(warmup):
            step(i, stream)
        torch.cuda.synchronize()
        # Launch-bound loop: record `chunk` consecutive calls into one HIP graph and
        # replay it, so the host's launch rate is not what gets measured.
        chunk = 1
        if not args.eager:
            chunk = max(d for d in range(1, min(steps, 256) + 1) if steps % d == 0)
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                cs = torch.cuda.current_stream().cuda_stream
                for i in range(chunk):
                    step(i, cs)
            graph.replay()
            torch.cuda.synchronize()
        walls, events = [], []
        for _ in range(max(1, repeats)):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            e0.record()
            if args.eager:
                for i in range(steps):
                    step(i, stream)
            else:
                for _ in range(steps // chunk):
                    graph.replay()
            e1.record()
            torch.cuda.synchronize()
            walls.append(time.perf_counter() - t0)
            events.append(e0.elapsed_time(e1) * 1e-3)
        mid = sorted(range(len(events)), key=lambda i: events[i])[len(events) // 2]  # the median run, by device time
        return walls[mid], events[mid]

    def time_lm_head(out_dim=128256, in_dim=4096, steps=40, copies=2):
        """argmax(x @ W^T) over a Llama-3 vocabulary, Q4_0: GEMV into scratch + argmax kernel per call."""
        ws = prepared_copies(Q4, out_dim, in_dim, copies, 31)
        x = torch.from_numpy(synth.activations(32, 1, in_dim)).to(dev)
        scratch = torch.empty(kernels.linearArgmaxWorkspaceBytes(Q4, in_dim, out_dim), dtype=torch.uint8, device=dev)
        token = torch.zeros(2, dtype=torch.int32, device=dev)
        bx, bs, bt = buf(x), buf(scratch), buf(token[:1])
        bws = [buf(w) for w in ws]

        def step(i, st):
            kernels.launchLinearArgmaxLastRowF32(st, Q4, _lib.LAYOUT_PREPARED, bt, kernels.NO_BUFFER, bx, bws[i % copies],
                                                 1, in_dim, out_dim, bs)

        for i in range(4):
            step(i, stream)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            cs = torch.cuda.current_stream().cuda_stream
            for i in range(steps):
                step(i, cs)
        graph.replay()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        graph.replay()
        e1.record()
        torch.cuda.synchronize()
        sec = e0.elapsed_time(e1) * 1e-3 / steps
        b = gemv_bytes(Q4, 1, in_dim, out_dim)
        return {"what": "greedy lm_head: Q4_0 GEMV over a 128256-token vocabulary into scratch, then the argmax kernel",
                "us_per_call": round(sec * 1e6, 3), "GBps": round(b / sec / 1e9, 1),
                "frac_hbm_peak": round(b / sec / HBM_PEAK_BPS, 4)}

    def time_row_ops(rows=14336, dim=4096, steps=20):
        """cpy_q_to_f32 / cpy_f32_to_q over one FFN matrix and an embedding lookup: HBM-bound copies."""
        def timed(fn):
            for _ in range(3):
                fn(stream)
            torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                cs = torch.cuda.current_stream().cuda_stream
                for _ in range(steps):
                    fn(cs)
            graph.replay()
            torch.cuda.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            graph.replay()
            e1.record()
            torch.cuda.synchronize()
            return e0.elapsed_time(e1) * 1e-3 / steps

        out = {}
        f32_bytes = rows * dim * 4
        dense = torch.empty((rows, dim), dtype=torch.float32, device=dev)
        for name, fmt, bb, bv in (("q4_0", Q4, 18, 32), ("q8_0", Q8, 34, 32), ("q4_k", Q4K, 144, 256)):
            w = prepared_copies(fmt, rows, dim, 1, 41)[0]
            q_bytes = rows * dim // bv * bb
            sec = timed(lambda st: kernels.launchDequantizeF32(st, fmt, _lib.LAYOUT_PREPARED, buf(dense), buf(w), rows, dim))
            out[f"cpy_{name}_to_f32"] = {"us_per_call": round(sec * 1e6, 2),
                                        "GBps": round((q_bytes + f32_bytes) / sec / 1e9, 1),
                                        "frac_hbm_peak": round((q_bytes + f32_bytes) / sec / HBM_PEAK_BPS, 4)}
            raw = torch.empty(q_bytes, dtype=torch.uint8, device=dev)
            sec = timed(lambda st: kernels.launchQuantizeRows(st, fmt, buf(raw), buf(dense), rows, dim))
            out[f"cpy_f32_to_{name}"] = {"us_per_call": round(sec * 1e6, 2),
                                        "GBps": round((q_bytes + f32_bytes) / sec / 1e9, 1),
                                        "frac_hbm_peak": round((q_bytes + f32_bytes) / sec / HBM_PEAK_BPS, 4)}
            tokens = 512
            ids = torch.randint(0, rows, (tokens,), dtype=torch.int64, device=dev)
            emb = torch.empty((tokens, dim), dtype=torch.float32, device=dev)
            sec = timed(lambda st: kernels.launchEmbeddingLookupF32(st, fmt, _lib.LAYOUT_PREPARED, buf(emb), buf(w), buf(ids),
                                                                   tokens, dim, rows))
            moved = tokens * dim // bv * bb + tokens * dim * 4
            out[f"get_rows_{name}_512_tokens"] = {"us_per_call": round(sec * 1e6, 2), "GBps": round(moved / sec / 1e9, 1)}
        out["what"] = (f"row operators on a {rows} x {dim} tensor: dequantize all of it, quantize all of it "
                       "(bytes = quantized + f32 side), embedding lookup of 512 rows")
        return out

    def decode_sweep(layers=32, token_steps=20):
        """Matmuls of one Llama-3-8B-shaped decode step (Q4_0, 32 layers of QKV, O, gate, up,
        down), every layer with its own weight memory, as one HIP graph per token."""
        shapes = [("qkv", 6144, 4096), ("o", 4096, 4096), ("gate", 14336, 4096), ("up", 14336, 4096),
                  ("down", 4096, 14336)]
        launch = _lib.lib().afhip_launch_linear_f32
        launch_pair = _lib.lib().afhip_launch_linear_pair_f32  # gate + up share X: the engine's linearNoBiasPair
        # one layer of synthetic weights, repacked into `layers` separate device buffers
        per_layer = []
        for li, (_, n, k) in enumerate(shapes):
            per_layer.append(prepared_copies(Q4, n, k, layers, 500 + li))
        weight_bytes = layers * sum(n * (k // 32) * 18 for _, n, k in shapes)
        out = {"what": "32 layers x (QKV 6144x4096, O 4096x4096, gate and up 14336x4096, down 4096x14336), Q4_0, "
                       "one set of random weights repacked into 32 distinct device copies; matmuls only, gate and up as "
                       "one pair call (shared X)",
               "weight_bytes_per_token": weight_bytes}
        for m in (1, 2, 4, 5):
            xs = {k: torch.from_numpy(synth.activations(900 + k, m, k)).to(dev) for k in (4096, 14336)}
            ys = {n: torch.empty((m, n), dtype=torch.float32, device=dev) for n in (6144, 4096, 14336)}
            y_up = torch.empty((m, 14336), dtype=torch.float32, device=dev)
            wsb = max(kernels.workspaceBytes(Q4, m, k, n) for _, n, k in shapes)
            scratch = torch.empty(max(wsb, 16), dtype=torch.uint8, device=dev)

            def token(st):
                for layer in range(layers):
                    for li, (name, n, k) in enumerate(shapes):
                        if name == "up":
                            continue  # computed with "gate"
                        if name == "gate":
                            rc = launch_pair(st, Q4, _lib.LAYOUT_PREPARED, buf(ys[n]), buf(y_up), buf(xs[k]),
                                             buf(per_layer[li][layer]), buf(per_layer[li + 1][layer]), m, k, n,
                                             buf(scratch), -1)
                        else:
                            rc = launch(st, Q4, _lib.LAYOUT_PREPARED, buf(ys[n]), buf(xs[k]), buf(per_layer[li][layer]), m,
                                        k, n, buf(scratch), -1)
                        if rc != 0:
                            raise RuntimeError(f"launch failed: {rc}")

            token(stream)
            torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                token(torch.cuda.current_stream().cuda_stream)
            graph.replay()
            torch.cuda.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(token_steps):
                graph.replay()
            e1.record()
            torch.cuda.synchronize()
            t = e0.elapsed_time(e1) * 1e-3 / token_steps
            out[f"m{m}"] = {"us_per_step": round(t * 1e6, 1), "steps_per_s": round(1.0 / t, 1),
                            "tokens_per_s": round(m / t, 1), "weight_GBps": round(weight_bytes / t / 1e9, 1),
                            "frac_hbm_peak": round(weight_bytes / t / HBM_PEAK_BPS, 4)}
        return out

    def time_quantizer(rows, in_dim, steps=200):
        """The stand-alone activation quantizer (the first kernel of a prefill call), per launch."""
        x = torch.from_numpy(synth.activations(5, rows, in_dim)).to(dev)
        q = torch.empty(rows * in_dim, dtype=torch.int8, device=dev)
        sc = torch.empty(rows * in_dim // 32, dtype=torch.float32, device=dev)
        sm = torch.empty(rows * in_dim // 32, dtype=torch.int32, device=dev)
        call = lambda st: kernels.launchQuantizeActivations(st, buf(x), rows, in_dim, buf(q), buf(sc), buf(sm))
        for _ in range(5):
            call(stream)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            cs = torch.cuda.current_stream().cuda_stream
            for _ in range(steps):
                call(cs)
        graph.replay()
        torch.cuda.synchronize()
        times = []
        for _ in range(5):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            graph.replay()
            e1.record()
            torch.cuda.synchronize()
            times.append(e0.elapsed_time(e1) * 1e-3 / steps)
        return sorted(times)[2]

    def gemm_roofline(m=512, k=4096, n=4096, steps=200):
        """Second half of the metric: the Q8_0 prefill GEMM (activation quantizer + int8-MFMA kernel)."""
        w_s, e_s = time_config(Q8, m, k, n, steps, 20, 4, 7, repeats=args.repeats)
        t_op = e_s / steps
        t_quant = time_quantizer(m, k)
        t_kernel = max(t_op - t_quant, 1e-9)
        ops = 2.0 * m * k * n
        return {"bound": "int8_mfma", "achieved": round(ops / t_op / 1e12, 2), "peak": INT8_MFMA_PEAK_OPS / 1e12,
                "unit": "TOP/s", "frac": round(ops / t_op / INT8_MFMA_PEAK_OPS, 4),
                "kernel": "quantize_activations_kernel + gemm_i8_kernel<Q8_0> (64 x 128 tiles)",
                "workload": f"Q8_0 prefill GEMM, x f32 [{m}x{k}] quantized on the GPU, W [{n}x{k}] 34-byte blocks",
                "ops_per_launch": ops, "us_per_op": round(t_op * 1e6, 3), "us_quantizer": round(t_quant * 1e6, 3),
                "us_kernel_by_subtraction": round(t_kernel * 1e6, 3),
                "frac_kernel_by_subtraction": round(ops / t_kernel / INT8_MFMA_PEAK_OPS, 4),
                "traffic": measured_traffic("traffic_bytes_per_launch_gemm_q8_0_m512"), "traffic_source": TRAFFIC_FILE,
                "traffic_stale": traffic_is_stale("gemm_q8_0_m512"),
                "note": "achieved and frac are the whole op (activation quantizer + GEMM kernel, HIP events in this run); "
                        "us_kernel_by_subtraction = op time minus the quantizer launched alone, a side figure; "
                        "every (row, column, block) term also costs one convert and one f32 multiply-add on the vector ALU"}

    if args.shapes:
        for spec in args.shapes.split(","):
            f, r, k, n = spec.split(":")
            pair = f.endswith("p")  # q4p / q8p: pair calls (two matrices, one X)
            fmt = {"q4": Q4, "q8": Q8, "q4k": Q4K}[f[:-1] if pair else f]
            r, k, n = int(r), int(k), int(n)
            wbytes = n * (k // 32) * BLOCK_BYTES[fmt] if fmt != Q4K else n * (k // 256) * 144
            copies = max(2, min(16, (600 << 20) // wbytes))
            w_s, e_s = time_config(fmt, r, k, n, 400, 20, copies, 99, repeats=3, pair=pair)
            if pair:
                wbytes *= 2
            b = wbytes + 4 * r * (k + n * (2 if pair else 1))
            print(json.dumps({"shape": spec, "us_per_call": round(e_s / 400 * 1e6, 3), "GBps": round(b * 400 / e_s / 1e9, 1),
                              "frac_hbm_peak": round(b * 400 / e_s / HBM_PEAK_BPS, 4)}), flush=True)
        return 0

    if args.only == "row_ops":
        print(json.dumps({"only": "row_ops", "row_ops_14336x4096": time_row_ops()}))
        return 0
    if args.only:
        m = int(args.only.rsplit("m", 1)[1])
        w_s, e_s = time_config(Q8, m, 4096, 4096, 200, 20, 4, 7, repeats=1)
        print(json.dumps({"only": args.only, "us_per_op": round(e_s / 200 * 1e6, 3),
                          "TOPS": round(2.0 * m * 4096 * 4096 * 200 / e_s / 1e12, 2)}))
        return 0

    if args.probe == "rates":
        lib = _lib.lib()
        sink = torch.zeros(65536 + (2 << 18) + 2048, dtype=torch.int32, device=dev)
        iterations = 2000
        # (pattern, name, instructions the "per instruction" column divides by, wavefronts per SIMD to run)
        patterns = [
            (0, "32 v_fma_f32", 32, (1, 2, 4)),
            (1, "32 v_cvt_f32_i32", 32, (1, 2, 4)),
            (2, "32 v_sub_f32", 32, (1, 2, 4)),
            (3, "16 x (v_cvt_f32_i32 -> v_fma_f32 that consumes it)", 32, (1, 2, 4)),
            (21, "32 v_dot8_i32_i4, 32 accumulators", 32, (1, 2, 4)),
            (22, "32 v_dot8_i32_i4, 8 chains of 4 (the decode kernel's block dot)", 32, (1, 2, 4)),
            (23, "32 v_dot4_i32_i8, 32 accumulators", 32, (1, 2, 4)),
            (4, "4 v_mfma_i32_32x32x32_i8", 4, (1, 2, 4)),
            (5, "2 v_mfma_f32_32x32x1_2b_f32", 2, (1, 2, 4)),
            (6, "4 x (int8 MFMA + 8 v_fma_f32), one wavefront", 4, (1, 2, 4)),
            (7, "4 x (int8 MFMA + 8 cvt + 8 fma), one wavefront", 4, (1, 2, 4)),
            (8, "4 x (int8 MFMA + 16 cvt + 16 fma), one wavefront", 4, (1, 2, 4)),
            (9, "GEMM recipe, 4 tile-blocks: 4 int8 MFMA + 2 f32 rank-1 MFMA + 64 cvt + 64 fma, two register sets", 4, (1, 2)),
            (10, "the same with v_sub_f32 for the conversion", 4, (1, 2)),
            (13, "4 tile-blocks: 4 int8 MFMA + 4 f32 rank-1 MFMA + 64 fma (bias term on the matrix pipe)", 4, (1, 2)),
            (11, "wavefronts 0-3: 4 int8 MFMA; wavefronts 4+: 32 v_fma_f32", 1, (2, 4)),
            (12, "wavefronts 0-3: 4 int8 MFMA; wavefronts 4+: 32 v_cvt_f32_i32", 1, (2,)),
            (15, "4 tile-blocks on one register set: 2 x (2 int8 MFMA + 1 f32 rank-1 MFMA, wait, 32 cvt + 32 fma)", 4, (1, 2, 4)),
            (14, "8 ds_read_b128 (1 KiB each per wavefront, lane l at byte 16 l), waited for together", 8, (1, 2, 4)),
            (16, "8 ds_read_b128 of MFMA fragments from XOR-swizzled 128-byte rows", 8, (1, 2, 4)),
            (17, "8 global_load_lds_dwordx4 (1 KiB each per wavefront, from L2), waited for together", 8, (1, 2, 4)),
            (18, "8 global_load_lds_dword (256 B each per wavefront)", 8, (1, 2, 4)),
            (19, "8 global_load_lds_ushort (128 B each per wavefront)", 8, (1, 2, 4)),
            (20, "8 global_load_dwordx4 to registers, wait, 8 ds_write_b128", 8, (1, 2, 4)),
        ]

        def run(pattern, waves):
            n = int(lib.afhip_rate_probe_wavefronts(waves))
            stamps = torch.zeros((n, 4), dtype=torch.int32, device=dev)
            for _ in range(2):  # the first launch warms the clocks up
                rc = lib.afhip_launch_rate_probe(stream, pattern, waves, iterations, buf(sink), buf(stamps))
                if rc != 0:
                    raise RuntimeError(f"rate probe failed: {rc}")
                torch.cuda.synchronize()
            return stamps.cpu().numpy().view(np.uint32).astype(np.int64)

        def placement(st):
            hw, xcc = st[:, 2], st[:, 3] & 0xF
            # HW_ID (gfx9 layout): simd [5:4], cu [11:8], sh [12], se [15:13]
            key = (xcc << 12) | (((hw >> 13) & 7) << 8) | (((hw >> 12) & 1) << 7) | (((hw >> 8) & 0xF) << 2) | ((hw >> 4) & 3)
            return key

        print(f"{iterations} rounds per wavefront; cycles = s_memtime differences read by the wavefronts, clock = cycles / (s_memrealtime ticks / 100 MHz)")
        print("| pattern (one round) | wavefronts per SIMD | cycles per round and wavefront (median; min-max) | SIMD cycles per instruction (from the SIMD's last wavefront to finish) | clock GHz | SIMDs hosting exactly that many wavefronts |")
        print("|---|---|---|---|---|---|")
        out = {}
        for pattern, name, per_round, wave_counts in patterns:
            for waves in wave_counts:
                st = run(pattern, waves)
                key = placement(st)
                simds, counts = np.unique(key, return_counts=True)
                exact = int((counts == waves).sum())
                ghz = float(np.median(st[:, 0] / (st[:, 1] / 100e6))) / 1e9
                if pattern in (11, 12):
                    # two roles: report each
                    wave_in_group = np.arange(st.shape[0]) % (4 * waves)
                    for role, sel in (("MFMA wavefronts", wave_in_group < 4), ("vector wavefronts", wave_in_group >= 4)):
                        cyc = st[sel, 0] / iterations
                        print(f"| {name} -- {role} | {waves} | {np.median(cyc):.1f}; {cyc.min():.1f}-{cyc.max():.1f} | | {ghz:.3f} | {exact} of {len(simds)} |")
                        out[f"{name} -- {role} @{waves}"] = round(float(np.median(cyc)), 2)
                    continue
                cyc = st[:, 0] / iterations
                med = float(np.median(cyc))
                # Throughput of a SIMD: its wavefronts start together and the oldest is served first, so the
                # work of all of them is done when the last one finishes.
                order = np.argsort(key, kind="stable")
                last = np.maximum.reduceat(cyc[order], np.flatnonzero(np.r_[True, np.diff(key[order]) != 0]))
                busy = float(np.median(last))
                print(f"| {name} | {waves} | {med:.1f}; {cyc.min():.1f}-{cyc.max():.1f} | {busy / waves / per_round:.2f} | {ghz:.3f} | {exact} of {len(simds)} |")
                out[f"{name} @{waves}"] = round(med, 2)
                out[f"{name} @{waves} simd_cycles_per_instruction"] = round(busy / waves / per_round, 2)
        print(json.dumps({"probe": "rates", "cycles_per_round": out}))
        return 0

    if args.probe == "read":
        copies, per_graph, replays = args.copies, 100, 10
        w_bytes = 14336 * (4096 // 32) * 18
        srcs = [torch.randint(0, 255, (w_bytes,), dtype=torch.uint8, device=dev) for _ in range(copies)]
        sink = torch.zeros(4, dtype=torch.int32, device=dev)
        lib = _lib.lib()

        def timed(call):
            for i in range(10):
                call(i, stream)
            torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                cs = torch.cuda.current_stream().cuda_stream
                for i in range(per_graph):
                    call(i, cs)
            graph.replay()
            torch.cuda.synchronize()
            out = []
            for _ in range(5):
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record()
                for _ in range(replays):
                    graph.replay()
                e1.record()
                torch.cuda.synchronize()
                out.append(e0.elapsed_time(e1) * 1e3 / (per_graph * replays))
            return sorted(out)[2]

        print(f"read of {w_bytes} bytes per launch, {copies} buffers in turn (more than the 256 MB last-level cache), graph replays")
        print("| threads per workgroup | 16-byte loads in flight per lane | workgroups | hint | us per launch | GB/s | % of 8 TB/s |")
        print("|---|---|---|---|---|---|---|")
        t = timed(lambda i, st: lib.afhip_launch_stream_read(st, Buffer(srcs[i % copies].data_ptr(), w_bytes), buf(sink)))
        print(f"| 256 | 1 (afhip_launch_stream_read) | {(w_bytes // 16 + 255) // 256} | non-temporal | {t:.3f} | {w_bytes / t / 1e3:.0f} | {w_bytes / t / 1e3 / 80:.1f} |")
        best = {}
        for threads in (256, 512, 1024):
            for loads in (1, 2, 4, 8, 16):
                for hint in (1, 0):
                    def call(i, st, threads=threads, loads=loads, hint=hint):
                        rc = lib.afhip_launch_stream_read_shaped(st, Buffer(srcs[i % copies].data_ptr(), w_bytes), buf(sink), threads, loads, hint)
                        if rc != 0:
                            raise RuntimeError(f"read probe failed: {rc}")
                    t = timed(call)
                    groups = (w_bytes // 16 + threads * loads - 1) // (threads * loads)
                    print(f"| {threads} | {loads} | {groups} | {'non-temporal' if hint else 'plain'} | {t:.3f} | {w_bytes / t / 1e3:.0f} | {w_bytes / t / 1e3 / 80:.1f} |", flush=True)
                    best[(threads, loads, hint)] = t
        k = min(best, key=best.get)
        print(json.dumps({"probe": "read", "best_us": round(best[k], 3), "best_shape": {"threads": k[0], "loads_per_lane": k[1], "nontemporal": k[2]}}))
        return 0

    if args.probe == "gemm":
        lib = _lib.lib()
        m, k, n = 512, 4096, 4096
        ws = prepared_copies(Q8, n, k, 4, 7)
        x = torch.from_numpy(synth.activations(8, m, k)).to(dev)
        q = torch.empty(m * k, dtype=torch.int8, device=dev)
        sc = torch.empty(m * k // 32, dtype=torch.float32, device=dev)
        sm = torch.empty(m * k // 32, dtype=torch.int32, device=dev)
        y = torch.zeros((m, n), dtype=torch.float32, device=dev)
        kernels.launchQuantizeActivations(stream, buf(x), m, k, buf(q), buf(sc), buf(sm))
        launches = 300  # back to back, so that the clocks are those of a sustained run; the last launch is read
        for i in range(launches):
            rc = lib.afhip_launch_gemm_stamps(stream, buf(y), buf(q), buf(sc), buf(ws[i % 4]), m, k, n)
            if rc != 0:
                raise RuntimeError(f"gemm stamps failed: {rc}")
        torch.cuda.synchronize()
        groups = ((n + 127) // 128 + 7) // 8 * ((m + 63) // 64) * 8
        st = y.cpu().numpy().reshape(-1).view(np.int32)[: groups * 16 * 8].reshape(groups, 16, 8).astype(np.int64)
        ghz = float(np.median(st[:, :, 1] / (st[:, :, 4] / 100e6))) / 1e9
        print(f"Q8_0 prefill kernel, M={m}, K={k}, N={n}: {groups} workgroups x 16 wavefronts, launch {launches} of {launches} back to back")
        print(f"clock held in the K loop: {ghz:.3f} GHz (loop cycles / 100 MHz reference ticks, median over wavefronts)")
        print("| per wavefront, shader-clock cycles | median | min | max |")
        print("|---|---|---|---|")
        for name, col in (("before the K loop", 0), ("K loop", 1), ("... of which waiting for its own loads", 2),
                          ("... of which waiting at the workgroup barrier", 3), ("after the K loop", 5)):
            v = st[:, :, col]
            print(f"| {name} | {int(np.median(v))} | {v.min()} | {v.max()} |")
        print("| wavefront of the workgroup (launch order = age on its SIMD) | K loop | waiting at barriers |")
        print("|---|---|---|")
        for wv in range(16):
            print(f"| {wv} | {int(np.median(st[:, wv, 1]))} | {int(np.median(st[:, wv, 3]))} |")
        tile_blocks = (m // 32) * (n // 32) * (k // 32) / (groups * 4)  # per SIMD
        print(f"tile-blocks (32 x 32 outputs x one 32-value block) per SIMD: {tile_blocks:.0f}; loop cycles per tile-block and SIMD: "
              f"{float(np.median(st[:, :, 1])) / tile_blocks:.0f}")
        print(json.dumps({"probe": "gemm", "clock_ghz": round(ghz, 3), "loop_cycles_median": int(np.median(st[:, :, 1])),
                          "barrier_cycles_median": int(np.median(st[:, :, 3])), "load_wait_cycles_median": int(np.median(st[:, :, 2]))}))
        return 0

    if args.probe == "timeline":
        import ctypes
        lib = _lib.lib()
        in_dim, out_dim = (int(v) for v in args.probe_shape.split(":"))
        copies, prows = args.copies, args.probe_rows
        ws = prepared_copies(Q4, out_dim, in_dim, copies, 2024)
        x = torch.from_numpy(synth.activations(2025, prows, in_dim)).to(dev)
        stamps = torch.zeros(1 << 18, dtype=torch.int32, device=dev)
        groups, waves = ctypes.c_size_t(0), ctypes.c_size_t(0)
        for i in range(64):  # back to back, weights rotating; the last launch's readings are the ones looked at
            rc = lib.afhip_launch_gemv_timeline(stream, prows, buf(stamps), buf(x), buf(ws[i % copies]), in_dim, out_dim,
                                                ctypes.byref(groups), ctypes.byref(waves))
            if rc != 0:
                raise RuntimeError(f"timeline probe failed: {rc}")
        torch.cuda.synchronize()
        g, w = groups.value, waves.value
        st = stamps.cpu().numpy().view(np.uint32)[: g * w * 8].reshape(g, w, 8).astype(np.int64)
        t0 = st[:, :, 0].min()
        ns = (st - t0) * 10
        ns[st == 0] = -1  # a reading that wavefront does not take
        print(f"Q4_0 decode kernel, {prows} row(s), K={in_dim}, N={out_dim}: {g} workgroups x {w} wavefronts; ns after the launch's first wavefront began, median over workgroups")
        print("| wavefront | begins | activations ready | block dots done | reduction done | (quantizer) past the barrier behind its requests for X | X arrived | blocks quantized |")
        print("|---|---|---|---|---|---|---|---|")
        for wv in range(w):
            cells = []
            for k in (0, 1, 2, 3, 4, 5, 6):
                col = ns[:, wv, k]
                cells.append("" if (col < 0).all() else str(int(np.median(col[col >= 0]))))
            print(f"| {wv} | " + " | ".join(cells) + " |")
        first = ns[:, :, 0].min(axis=1)
        print(f"workgroups begin {int(first.min())} .. {int(first.max())} ns (median {int(np.median(first))}); the last wavefront of the launch ends at {int(ns[:, :, 3].max())} ns")
        print(json.dumps({"probe": "timeline", "rows": prows, "workgroups": g, "wavefronts": w, "activations_ready_ns_median": int(np.median(ns[:, :, 1])),
                          "launch_ends_ns": int(ns[:, :, 3].max())}))
        return 0

    if args.probe == "timeline8":
        import ctypes
        lib = _lib.lib()
        in_dim, out_dim, copies = 4096, 14336, args.copies
        prows = args.probe_rows if args.probe_rows >= 5 else 8
        ws = prepared_copies(Q4, out_dim, in_dim, copies, 2024)
        x = torch.from_numpy(synth.activations(2025, prows, in_dim)).to(dev)
        stamps = torch.zeros(1 << 18, dtype=torch.int32, device=dev)
        work = torch.empty(kernels.workspaceBytes(Q4, 8, in_dim, out_dim), dtype=torch.uint8, device=dev)
        groups, cols = ctypes.c_size_t(0), ctypes.c_size_t(0)
        takes = []  # five runs of 64 launches back to back, weights rotating; each run's last launch is read
        for take in range(5):
            for i in range(64):
                rc = lib.afhip_launch_rows8_timeline(stream, prows, buf(stamps), buf(x), buf(ws[i % copies]), in_dim, out_dim, buf(work),
                                                     ctypes.byref(groups), ctypes.byref(cols))
                if rc != 0:
                    raise RuntimeError(f"timeline8 probe failed: {rc}")
            torch.cuda.synchronize()
            g, w = groups.value, 8
            st = stamps.cpu().numpy().view(np.uint32)[: g * w * 8].reshape(g, w, 8).astype(np.int64)
            takes.append((st - st[:, :, 0].min()) * 10)
        ns = np.median(np.stack(takes), axis=0)  # per reading, the median of the five runs
        print(f"Q4_0 eight-row MFMA kernel, {prows} rows, K={in_dim}, N={out_dim}: {g} workgroups of {cols.value} columns x {w} wavefronts; "
              "ns after the launch's first wavefront began, median over workgroups (each reading: median of five runs)")
        print("| wavefront | begins | stage 0 there | stage 1 | stage 2 | stage 3 | last stage | K loop done | workgroup reduced |")
        print("|---|---|---|---|---|---|---|---|---|")
        for wv in range(w):
            print(f"| {wv} | " + " | ".join(str(int(np.median(ns[:, wv, k]))) for k in range(8)) + " |")
        first = ns[:, :, 0].min(axis=1)
        print(f"workgroups begin {int(first.min())} .. {int(first.max())} ns (median {int(np.median(first))}); the last wavefront of the launch ends at {int(ns[:, :, 7].max())} ns")
        print("| per workgroup, ns | median | min | max |")
        print("|---|---|---|---|")
        for name, v in (("entry to the first stage there (slowest wavefront)", (ns[:, :, 1] - ns[:, :, 0]).max(axis=1)),
                        ("first stage there to the last stage there", (ns[:, :, 5] - ns[:, :, 1]).max(axis=1)),
                        ("last stage there to K loop done", (ns[:, :, 6] - ns[:, :, 5]).max(axis=1)),
                        ("K loop done to reduced", (ns[:, :, 7] - ns[:, :, 6]).min(axis=1)),
                        ("whole workgroup", ns[:, :, 7].max(axis=1) - first)):
            print(f"| {name} | {int(np.median(v))} | {int(v.min())} | {int(v.max())} |")
        print(json.dumps({"probe": "timeline8", "rows": prows, "workgroups": g, "columns_per_workgroup": cols.value,
                          "first_stage_there_ns_median": int(np.median(ns[:, :, 1])), "launch_ends_ns": int(ns[:, :, 7].max())}))
        return 0

    if args.probe == "gemv":
        in_dim, out_dim, copies, per_graph, replays = 4096, 14336, args.copies, 100, 10
        ws = prepared_copies(Q4, out_dim, in_dim, copies, 2024)
        prows = args.probe_rows
        x = torch.from_numpy(synth.activations(2025, prows, in_dim)).to(dev)
        y = torch.empty((prows, out_dim), dtype=torch.float32, device=dev)
        sink = torch.zeros(4, dtype=torch.int32, device=dev)
        w_bytes = out_dim * (in_dim // 32) * 18
        lib = _lib.lib()

        def timed(call):
            for i in range(10):
                call(i, stream)
            torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                cs = torch.cuda.current_stream().cuda_stream
                for i in range(per_graph):
                    call(i, cs)
            graph.replay()
            torch.cuda.synchronize()
            out = []
            for _ in range(7):
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record()
                for _ in range(replays):
                    graph.replay()
                e1.record()
                torch.cuda.synchronize()
                out.append(e0.elapsed_time(e1) * 1e3 / (per_graph * replays))
            return sorted(out)[3]

        rows_out = []
        t = timed(lambda i, st: lib.afhip_launch_stream_read(st, Buffer(ws[i % copies].data_ptr(), w_bytes), buf(sink)))
        rows_out.append(("read only: the same 33,030,144 bytes, 16 B per lane, nothing else", t))
        names = {0: "the decode kernel as launched by afhip_launch_linear_f32", 1: "without the block dots",
                 2: "without the store of Y", 3: "without dots and store", 4: "without the activation prologue",
                 5: "without prologue and dots", 6: "without prologue and store", 7: "loads and the wavefront reduction only"}
        for probe in range(8):
            def call(i, st, probe=probe):
                rc = lib.afhip_launch_gemv_probe_rows(st, probe, prows, buf(y), buf(x), buf(ws[i % copies]), in_dim, out_dim)
                if rc != 0:
                    raise RuntimeError(f"probe failed: {rc}")
            rows_out.append((f"probe {probe}: {names[probe]}", timed(call)))
        nbytes = gemv_bytes(Q4, prows, in_dim, out_dim)
        print(f"rows of X: {prows}")
        print("| variant | us per launch | GB/s | % of 8 TB/s |")
        print("|---|---|---|---|")
        for name, us in rows_out:
            print(f"| {name} | {us:.3f} | {nbytes / us / 1e3:.0f} | {nbytes / us / 1e3 / 80:.1f} |")
        print(json.dumps({"probe": "gemv", "rows": prows, "us_per_launch": {n: round(u, 3) for n, u in rows_out}}))
        return 0

    if args.counter_probe:
        n_launch, copies = 40, 8
        launch = _lib.lib().afhip_launch_linear_f32
        ws = prepared_copies(Q4, 14336, 4096, copies, 2024)
        x = torch.from_numpy(synth.activations(2025, 1, 4096)).to(dev)
        y = torch.empty((1, 14336), dtype=torch.float32, device=dev)
        scratch = torch.empty(max(kernels.workspaceBytes(Q4, 1, 4096, 14336), 16), dtype=torch.uint8, device=dev)
        for i in range(n_launch):
            launch(stream, Q4, _lib.LAYOUT_PREPARED, buf(y), buf(x), buf(ws[i % copies]), 1, 4096, 14336, buf(scratch), -1)
        torch.cuda.synchronize()
        w_bytes = 14336 * 128 * 18
        srcs = [torch.full((w_bytes,), 1, dtype=torch.uint8, device=dev) for _ in range(copies)]
        sink = torch.zeros(4, dtype=torch.int32, device=dev)
        for i in range(n_launch):
            _lib.lib().afhip_launch_stream_read(stream, buf(srcs[i % copies]), buf(sink))
        torch.cuda.synchronize()
        for i in range(n_launch):  # the plain copy: the same bytes read once and written once
            _lib.lib().afhip_launch_stream_copy(stream, buf(srcs[i % copies]), buf(srcs[(i + copies // 2) % copies]))
        torch.cuda.synchronize()
        wg = prepared_copies(Q8, 4096, 4096, 2, 7)
        xg = torch.from_numpy(synth.activations(8, 512, 4096)).to(dev)
        yg = torch.empty((512, 4096), dtype=torch.float32, device=dev)
        sg = torch.empty(kernels.workspaceBytes(Q8, 512, 4096, 4096), dtype=torch.uint8, device=dev)
        for i in range(n_launch):
            launch(stream, Q8, _lib.LAYOUT_PREPARED, buf(yg), buf(xg), buf(wg[i % 2]), 512, 4096, 4096, buf(sg), -1)
        torch.cuda.synchronize()
        # batched decode, 16 rows on the FFN matrix: fragment quantizer + single-shot MFMA kernel
        xb = torch.from_numpy(synth.activations(9, 16, 4096)).to(dev)
        yb = torch.empty((16, 14336), dtype=torch.float32, device=dev)
        sb = torch.empty(kernels.workspaceBytes(Q4, 16, 4096, 14336), dtype=torch.uint8, device=dev)
        for i in range(n_launch):
            launch(stream, Q4, _lib.LAYOUT_PREPARED, buf(yb), buf(xb), buf(ws[i % copies]), 16, 4096, 14336, buf(sb), -1)
        torch.cuda.synchronize()
        # speculative verify, 8 rows on the FFN matrix: compact-fragment quantizer + eight-row MFMA kernel
        x8 = torch.from_numpy(synth.activations(10, 8, 4096)).to(dev)
        y8 = torch.empty((8, 14336), dtype=torch.float32, device=dev)
        s8 = torch.empty(kernels.workspaceBytes(Q4, 8, 4096, 14336), dtype=torch.uint8, device=dev)
        for i in range(n_launch):
            launch(stream, Q4, _lib.LAYOUT_PREPARED, buf(y8), buf(x8), buf(ws[i % copies]), 8, 4096, 14336, buf(s8), -1)
        torch.cuda.synchronize()
        # Q4_K on the same matrix: the decode kernel (one row) and the prefill GEMM (512 rows)
        wk = prepared_copies(Q4K, 14336, 4096, copies, 31)
        for m in (1, 512):
            xk = torch.from_numpy(synth.activations(32 + m, m, 4096)).to(dev)
            yk = torch.empty((m, 14336), dtype=torch.float32, device=dev)
            sk = torch.empty(max(kernels.workspaceBytes(Q4K, m, 4096, 14336), 16), dtype=torch.uint8, device=dev)
            for i in range(n_launch):
                launch(stream, Q4K, _lib.LAYOUT_PREPARED, buf(yk), buf(xk), buf(wk[i % copies]), m, 4096, 14336, buf(sk), -1)
            torch.cuda.synchronize()
        print(json.dumps({"counter_probe": {"launches_each": n_launch, "gemv_bytes": gemv_bytes(Q4, 1, 4096, 14336),
                                            "stream_read_bytes": w_bytes,
                                            "stream_copy_bytes": w_bytes,
                                            "kernel_source_sha256": {k: kernel_source_hash(k) for k in TRAFFIC_SOURCES}}}))
        return 0

    # ---- headline: Q4_0 decode GEMV, M=1, K=4096, N=14336 --------------------------
    rows, in_dim, out_dim = 1, 4096, 14336
    launches = args.steps * args.copies  # a step visits every weight copy once
    wall, ev = time_config(Q4, rows, in_dim, out_dim, launches, args.warmup * args.copies, args.copies, 2024,
                           repeats=args.repeats)
    nbytes = gemv_bytes(Q4, rows, in_dim, out_dim)
    value = nbytes * launches / wall / 1e9
    achieved = nbytes * launches / ev / 1e9
    result = {
        "metric": "Q4 GEMV HBM GB/s (% of 8TB/s) K=4096,N=14336; Q8 GEMM M=512 TOPS",
        "value": round(value, 2),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "repeats": args.repeats,
        "ms_per_step": round(wall / args.steps * 1e3, 6),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "int8 dot / f32 accumulate",
        "data": "synthetic (seeded SplitMix64: x~N(0,1), Q4_0 nibbles uniform, fp16 scales |N(0,0.02)|/7)",
        "config": {"workload": "Q4_0 decode GEMV, x f32 [1x4096], W [14336x4096] 18-byte blocks (Llama-3-8B FFN-up)",
                   "rows": rows, "in_dim": in_dim, "out_dim": out_dim, "weight_copies": args.copies,
                   "launches_per_step": args.copies, "bytes_per_launch": nbytes, "bytes_per_step": nbytes * args.copies,
                   "step": "one GEMV launch on each of the weight copies (every launch reads its weights from HBM, not from "
                           "the 256 MB Infinity Cache)"},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 2), "peak": HBM_PEAK_BPS / 1e9, "unit": "GB/s",
                     "frac": round(achieved * 1e9 / HBM_PEAK_BPS, 4), "traffic": measured_traffic(),
                     "traffic_stale": traffic_is_stale("gemv_q4_0_m1"),
                     "traffic_source": TRAFFIC_FILE + " (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE of `bench.py --counter-probe`; not measured by this run)",
                     "kernel": "gemv_fused_kernel<Q4_0, rows=1>", "us_per_launch": round(ev / launches * 1e6, 3)},
    }

    result["roofline_gemm"] = gemm_roofline()

    # ---- other configurations ---------------------------------------------------------
    if not args.no_extra:
        extra = {}

        def time_stream_read(nbytes_read, steps, copies):
            """A kernel that only reads `nbytes_read` bytes, launched like the GEMV above."""
            srcs = [torch.full((nbytes_read,), 1, dtype=torch.uint8, device=dev) for _ in range(copies)]
            sink = torch.zeros(4, dtype=torch.int32, device=dev)
            read = _lib.lib().afhip_launch_stream_read
            bufs = [buf(t) for t in srcs]
            for i in range(20):
                read(stream, bufs[i % copies], buf(sink))
            torch.cuda.synchronize()
            chunk = max(d for d in range(1, min(steps, 256) + 1) if steps % d == 0)
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                cs = torch.cuda.current_stream().cuda_stream
                for i in range(chunk):
                    read(cs, bufs[i % copies], buf(sink))
            graph.replay()
            torch.cuda.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(steps // chunk):
                graph.replay()
            e1.record()
            torch.cuda.synchronize()
            return e0.elapsed_time(e1) * 1e-3 / steps

        w_bytes = out_dim * (in_dim // 32) * 18
        t_small = time_stream_read(w_bytes, max(64, args.steps // 4), args.copies)
        t_large = time_stream_read(8 * w_bytes, 64, 4)
        extra["stream_read_only"] = {
            "what": "kernel that only reads N bytes (16 B per lane, all loads at once), same launch pattern",
            "33MB_us": round(t_small * 1e6, 3), "33MB_GBps": round(w_bytes / t_small / 1e9, 1),
            "264MB_us": round(t_large * 1e6, 3), "264MB_GBps": round(8 * w_bytes / t_large / 1e9, 1),
        }
        small_steps = max(50, args.steps // 4)
        for name, fmt, r, k, n in [
            ("q8_gemv_m1_k4096_n4096", Q8, 1, 4096, 4096),
            ("q8_gemv_m1_k4096_n14336", Q8, 1, 4096, 14336),
            ("q4_gemv_m2_k4096_n14336", Q4, 2, 4096, 14336),
            ("q4_gemv_m3_k4096_n14336", Q4, 3, 4096, 14336),
            ("q4_gemv_m4_k4096_n14336", Q4, 4, 4096, 14336),
            ("q8_gemv_m2_k4096_n14336", Q8, 2, 4096, 14336),
            ("q8_gemv_m4_k4096_n14336", Q8, 4, 4096, 14336),
            ("q4_gemv_m2_k14336_n4096", Q4, 2, 14336, 4096),    # long K, few rows: K shared out over workgroups + reduce kernel
            ("q4_gemv_m4_k14336_n4096", Q4, 4, 14336, 4096),
            ("q4_batch_m8_k4096_n14336", Q4, 8, 4096, 14336),   # speculative verify: compact-fragment quantizer + eight-row MFMA kernel
            ("q4_gemv_m1_k14336_n4096", Q4, 1, 14336, 4096),
            ("q4_batch_m5_k14336_n4096", Q4, 5, 14336, 4096),
            ("q8_batch_m8_k4096_n14336", Q8, 8, 4096, 14336),
            ("q4_batch_m16_k4096_n14336", Q4, 16, 4096, 14336),  # batched decode: fragment quantizer + single-shot MFMA kernel
            ("q4_batch_m32_k4096_n14336", Q4, 32, 4096, 14336),
            ("q4_batch_m64_k4096_n14336", Q4, 64, 4096, 14336),
            ("q4_batch_m16_k14336_n4096", Q4, 16, 14336, 4096),  # K longer than one share: partial sums + reduce kernel
            ("q4_batch_m16_k4096_n4096", Q4, 16, 4096, 4096),
            ("q4_batch_m5_k4096_n4096", Q4, 5, 4096, 4096),
        ]:
            copies = args.copies if fmt == Q4 or n > 4096 else 2 * args.copies
            w_s, e_s = time_config(fmt, r, k, n, small_steps, 20, copies, 99)
            b = gemv_bytes(fmt, r, k, n)
            extra[name] = {"us_per_call": round(e_s / small_steps * 1e6, 3),
                           "GBps": round(b * small_steps / e_s / 1e9, 1),
                           "frac_hbm_peak": round(b * small_steps / e_s / HBM_PEAK_BPS, 4)}
        for name, r, k, n in [("q4k_gemv_m1_k4096_n14336", 1, 4096, 14336), ("q4k_gemv_m2_k4096_n14336", 2, 4096, 14336),
                              ("q4k_gemv_m5_k4096_n14336", 5, 4096, 14336), ("q4k_gemv_m8_k4096_n14336", 8, 4096, 14336),
                              ("q4k_gemv_m1_k14336_n4096", 1, 14336, 4096), ("q4k_gemv_m5_k14336_n4096", 5, 14336, 4096)]:
            w_s, e_s = time_config(Q4K, r, k, n, small_steps, 20, args.copies, 77)
            b = n * (k // 256) * 144 + 4 * r * (k + n)
            extra[name] = {"what": "Q4_K (144-byte super-blocks, tile-major device layout), f32-accurate: fixed-point activations on int8 MFMA "
                                   "(3+ rows: digit planes made once by their own launch, included)",
                           "us_per_call": round(e_s / small_steps * 1e6, 3),
                           "GBps": round(b * small_steps / e_s / 1e9, 1),
                           "frac_hbm_peak": round(b * small_steps / e_s / HBM_PEAK_BPS, 4)}
        for m in (32, 128, 512):
            w_s, e_s = time_config(Q4K, m, 4096, 14336, 40, 5, 2, 78)
            flops = 2.0 * m * 4096 * 14336
            # the kernel issues three bf16 MFMA products per f32 product (X as hi + mid + lo parts), so the
            # matrix-core work is 3 x 2MNK flop, priced against the dense bf16 peak
            extra[f"q4k_gemm_m{m}_k4096_n14336"] = {
                "what": "Q4_K prefill: X split once into three bf16 parts, bf16-MFMA GEMM, f32-accurate; per call incl. the split",
                "us_per_call": round(e_s / 40 * 1e6, 1),
                "TFLOPs_f32_equivalent": round(flops * 40 / e_s / 1e12, 1),
                "bf16_mfma_TFLOPs_issued": round(3 * flops * 40 / e_s / 1e12, 1),
                "frac_bf16_mfma_peak": round(3 * flops * 40 / e_s / BF16_MFMA_PEAK_FLOPS, 4)}
        for m in (128, 512, 2048):
            gsteps = 200
            w_s, e_s = time_config(Q8, m, 4096, 4096, gsteps, 20, 4, 7)
            ops = 2.0 * m * 4096 * 4096
            extra[f"q8_gemm_m{m}_k4096_n4096"] = {"what": "activation quantizer + int8-MFMA GEMM kernel, per call",
                                                 "us_per_call": round(e_s / gsteps * 1e6, 3),
                                                 "TOPS": round(ops * gsteps / e_s / 1e12, 3),
                                                 "frac_int8_mfma_peak": round(ops * gsteps / e_s / INT8_MFMA_PEAK_OPS, 5)}
        extra["q4_lm_head_argmax_k4096_n128256"] = time_lm_head()
        extra["row_ops_14336x4096"] = time_row_ops()
        extra["llama3_8b_decode_matmuls"] = decode_sweep()
        result["extra"] = extra

    # ---- CPU baseline: the engine's CPU route restated in C, on this host --------------
    if not args.no_cpu:
        from oracle import oracle as O

        w = synth.weights(Q4, 2024, out_dim, in_dim)
        x = synth.activations(2025, rows, in_dim)
        prepared = O.Prepared(Q4, w, out_dim, in_dim)
        workers = min(8, os.cpu_count() or 1)  # the reference pool caps at 8 workers
        y = np.zeros((rows, out_dim), dtype=np.float32)
        for _ in range(3):
            prepared.linear(x, rows, workers=workers, y=y)
        calls, t0 = 0, time.perf_counter()
        while True:
            prepared.linear(x, rows, workers=workers, y=y)
            calls += 1
            dt = time.perf_counter() - t0
            if (dt >= args.cpu_seconds and calls >= 20) or dt >= 3 * args.cpu_seconds:
                break
        prepared.close()
        # the GEMM half on the same cores: row-split over min(8, rows) workers as the engine plans it
        # (ops/native_compute.zig:9756-9776), a bounded number of calls
        gm, gk, gn = 512, 4096, 4096
        gw = synth.weights(Q8, 7, gn, gk)
        gx = synth.activations(8, gm, gk)
        gprep = O.Prepared(Q8, gw, gn, gk)
        gy = np.zeros((gm, gn), dtype=np.float32)
        gprep.linear(gx, gm, workers=workers, y=gy)
        gcalls, g0 = 0, time.perf_counter()
        while True:
            gprep.linear(gx, gm, workers=workers, y=gy)
            gcalls += 1
            gdt = time.perf_counter() - g0
            if (gdt >= args.cpu_seconds and gcalls >= 3) or gdt >= 3 * args.cpu_seconds:
                break
        gprep.close()
        result["cpu_baseline_gemm"] = {
            "value": round(2.0 * gm * gk * gn * gcalls / gdt / 1e12, 4), "unit": "TOP/s", "cores": workers, "kind": "port",
            "sample": f"{gcalls} calls of the same Q8_0 [{gm}x{gk}]x[{gn}x{gk}] prefill matmul (activation quantizer + int8 block "
                      f"dots + f32 scaled accumulate) in {gdt:.1f} s ({gdt / gcalls * 1e3:.1f} ms/call), rows split over {workers} threads",
            "host_cpus": os.cpu_count(),
        }
        result["cpu_baseline"] = {
            "value": round(nbytes * calls / dt / 1e9, 3), "unit": "GB/s", "cores": workers, "kind": "port",
            "sample": f"{calls} calls of the same Q4_0 [1x4096]x[14336x4096] GEMV in {dt:.1f} s "
                      f"({dt / calls * 1e6:.0f} us/call), column-split over {workers} threads as the engine does",
            "host_cpus": os.cpu_count(),
        }
    print(json.dumps(result))
    return 0


if __name__ == "__main__":
    sys.exit(main())
