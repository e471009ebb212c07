#!/usr/bin/env python3
"""Benchmark of the MI355X quantized matmul (Q4_0 / Q8_0 `linearNoBias`).

One "step" = one Q4_0 decode GEMV at the Llama-3-8B FFN-up shape
(x f32 [1 x 4096], W [14336 x 4096] in 18-byte blocks), the configuration the
headline metric is quoted on.  Weights rotate over more distinct copies than the
256 MB Infinity Cache holds, so every step streams its 33 MB from HBM.

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
Q4, Q8, Q4K = 2, 8, 12
BLOCK_BYTES = {Q4: 18, Q8: 34}


def measured_traffic():
    """HBM bytes per launch of the headline kernel from the committed counter summary
    (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of `bench.py --counter-probe`, each scaled
    by a kernel of known traffic in the same run), or None when that file is not there."""
    path = os.path.join(ROOT, "profiles", "gemv_q4_0_m1_and_gemm_q8_0_m512_counters.md")
    try:
        with open(path) as f:
            for line in f:
                if line.startswith("traffic_bytes_per_launch_gemv_q4_0_m1:"):
                    return int(float(line.split(":", 1)[1]))
    except OSError:
        pass
    return None


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
    ap.add_argument("--counter-probe", action="store_true",
                    help="for hardware-counter runs: 40 eager launches each of the headline GEMV, of the plain "
                         "read kernel over the same number of bytes, of the Q8_0 M=512 GEMM and of the Q4_K kernels "
                         "(M=1 and M=512), then exit")
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

    def time_config(fmt, rows, in_dim, out_dim, steps, warmup, copies, seed):
        """Returns (wall seconds, event seconds) for `steps` back-to-back calls."""
        ws = prepared_copies(fmt, out_dim, in_dim, copies, seed)
        x = torch.from_numpy(synth.activations(seed + 1, rows, in_dim)).to(dev)
        y = torch.empty((rows, out_dim), dtype=torch.float32, device=dev)
        wsb = kernels.workspaceBytes(fmt, rows, in_dim, out_dim)
        scratch = torch.empty(max(wsb, 16), dtype=torch.uint8, device=dev)
        bx, by, bs = buf(x), buf(y), buf(scratch)
        bws = [buf(w) for w in ws]
        launch = _lib.lib().afhip_launch_linear_f32

        def step(i, st):
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
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
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
        wall = time.perf_counter() - t0
        return wall, e0.elapsed_time(e1) * 1e-3

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
        for name, fmt, bb in (("q4_0", Q4, 18), ("q8_0", Q8, 34)):
            w = prepared_copies(fmt, rows, dim, 1, 41)[0]
            q_bytes = rows * dim // 32 * bb
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
            moved = tokens * dim // 32 * bb + tokens * dim * 4
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
        for m in (1, 5):
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
        wg = prepared_copies(Q8, 4096, 4096, 2, 7)
        xg = torch.from_numpy(synth.activations(8, 512, 4096)).to(dev)
        yg = torch.empty((512, 4096), dtype=torch.float32, device=dev)
        sg = torch.empty(kernels.workspaceBytes(Q8, 512, 4096, 4096), dtype=torch.uint8, device=dev)
        for i in range(n_launch):
            launch(stream, Q8, _lib.LAYOUT_PREPARED, buf(yg), buf(xg), buf(wg[i % 2]), 512, 4096, 4096, buf(sg), -1)
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
                                            "stream_read_bytes": w_bytes}}))
        return 0

    # ---- headline: Q4_0 decode GEMV, M=1, K=4096, N=14336 --------------------------
    rows, in_dim, out_dim = 1, 4096, 14336
    wall, ev = time_config(Q4, rows, in_dim, out_dim, args.steps, args.warmup, args.copies, 2024)
    nbytes = gemv_bytes(Q4, rows, in_dim, out_dim)
    value = nbytes * args.steps / wall / 1e9
    achieved = nbytes * args.steps / ev / 1e9
    result = {
        "metric": "Q4 GEMV HBM GB/s (% of 8TB/s) K=4096,N=14336; Q8 GEMM M=512 TOPS",
        "value": round(value, 2),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(wall / args.steps * 1e3, 6),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "int8 dot / f32 accumulate",
        "data": "synthetic (seeded SplitMix64: x~N(0,1), Q4_0 nibbles uniform, fp16 scales |N(0,0.02)|/7)",
        "config": {"workload": "Q4_0 decode GEMV, x f32 [1x4096], W [14336x4096] 18-byte blocks (Llama-3-8B FFN-up)",
                   "rows": rows, "in_dim": in_dim, "out_dim": out_dim, "weight_copies": args.copies,
                   "bytes_per_step": nbytes},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 2), "peak": HBM_PEAK_BPS / 1e9, "unit": "GB/s",
                     "frac": round(achieved * 1e9 / HBM_PEAK_BPS, 4), "traffic": measured_traffic(),
                     "kernel": "gemv_fused_kernel<Q4_0, rows=1>", "us_per_launch": round(ev / args.steps * 1e6, 3)},
    }

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
            ("q4_gemv_m4_k4096_n14336", Q4, 4, 4096, 14336),
            ("q4_gemv_m8_k4096_n14336", Q4, 8, 4096, 14336),
            ("q4_gemv_m1_k14336_n4096", Q4, 1, 14336, 4096),
            ("q4_gemv_m5_k14336_n4096", Q4, 5, 14336, 4096),
            ("q4_batch_m16_k4096_n14336", Q4, 16, 4096, 14336),  # batched decode: quantizer + MFMA GEMM, 32-row tiles
            ("q4_batch_m64_k4096_n14336", Q4, 64, 4096, 14336),
            ("q4_batch_m16_k14336_n4096", Q4, 16, 14336, 4096),  # few column tiles: K shared out over workgroups
        ]:
            copies = args.copies if fmt == Q4 or n > 4096 else 2 * args.copies
            w_s, e_s = time_config(fmt, r, k, n, small_steps, 20, copies, 99)
            b = gemv_bytes(fmt, r, k, n)
            extra[name] = {"us_per_call": round(e_s / small_steps * 1e6, 3),
                           "GBps": round(b * small_steps / e_s / 1e9, 1),
                           "frac_hbm_peak": round(b * small_steps / e_s / HBM_PEAK_BPS, 4)}
        for name, r, k, n in [("q4k_gemv_m1_k4096_n14336", 1, 4096, 14336), ("q4k_gemv_m2_k4096_n14336", 2, 4096, 14336),
                              ("q4k_gemv_m5_k4096_n14336", 5, 4096, 14336), ("q4k_gemv_m1_k14336_n4096", 1, 14336, 4096)]:
            w_s, e_s = time_config(Q4K, r, k, n, small_steps, 20, args.copies, 77)
            b = n * (k // 256) * 144 + 4 * r * (k + n)
            extra[name] = {"what": "Q4_K (144-byte super-blocks, tile-major device layout), f32-accurate on bf16 MFMA",
                           "us_per_call": round(e_s / small_steps * 1e6, 3),
                           "GBps": round(b * small_steps / e_s / 1e9, 1),
                           "frac_hbm_peak": round(b * small_steps / e_s / HBM_PEAK_BPS, 4)}
        for m in (32, 128, 512):
            w_s, e_s = time_config(Q4K, m, 4096, 14336, 40, 5, 2, 78)
            flops = 2.0 * m * 4096 * 14336
            extra[f"q4k_gemm_m{m}_k4096_n14336"] = {
                "what": "Q4_K prefill: X split once into three bf16 parts, bf16-MFMA GEMM, f32-accurate; per call incl. the split",
                "us_per_call": round(e_s / 40 * 1e6, 1),
                "TFLOPs_f32_equivalent": round(flops * 40 / e_s / 1e12, 1),
                "frac_f32_mfma_peak": round(flops * 40 / e_s / 157.3e12, 3)}
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
