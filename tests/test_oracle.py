"""Pins the CPU oracle against the reference's known-answer vectors and against
what the mathematics fixes (closed forms, brute force, invariants).  No GPU."""
import os

import numpy as np
import pytest

from antfly_amd import synth
from oracle import oracle as O

Q4, Q8 = O.FMT_Q4_0, O.FMT_Q8_0
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def smoke_row(fmt, scale, value):
    """Same bytes as the reference's smoke-row writers (ops/cuda/kernels.zig:2516-2531)."""
    hb = np.array([scale], dtype=np.float16).view(np.uint8)
    if fmt == Q8:
        return np.concatenate([hb, np.full(32, value, dtype=np.int8).view(np.uint8)])
    nib = (value + 8) & 0xF
    return np.concatenate([hb, np.full(16, nib | (nib << 4), dtype=np.uint8)])


# ---------------------------------------------------------------- geometry / fp16

def test_block_sizes(kats):
    assert O.lib().afo_block_bytes(Q4) == kats["block_sizes"]["q4_0"]["bytes"] == 18
    assert O.lib().afo_block_bytes(Q8) == kats["block_sizes"]["q8_0"]["bytes"] == 34
    assert O.lib().afo_block_bytes(12) == 0
    assert O.lib().afo_byte_len(Q4, 4096 * 14336) == 33030144
    assert O.lib().afo_byte_len(Q8, 4096 * 4096) == 17825792
    assert O.lib().afo_byte_len(Q8, 33) == 0


def test_fp16_reference_constants(kats):
    for bits, want in kats["fp16_constants"]["cases"]:
        assert O.fp16_to_f32(bits) == want


def test_fp16_decode_all_bit_patterns():
    bits = np.arange(65536, dtype=np.uint16)
    want = bits.view(np.float16).astype(np.float32)
    got = np.array([O.fp16_to_f32(int(b)) for b in bits], dtype=np.float32)
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got[~nan].view(np.uint32), want[~nan].view(np.uint32))


def test_fp16_encode_matches_ieee_rne():
    rng = np.random.default_rng(7)
    vals = np.concatenate([
        rng.standard_normal(20000).astype(np.float32) * 10.0 ** rng.integers(-9, 5, 20000),
        np.arange(65536, dtype=np.uint16).view(np.float16).astype(np.float32),  # exact halves
        np.array([0.0, -0.0, 65504.0, 65519.9, 65520.0, 1e9, 5.96e-8, 2.98e-8, 2.99e-8, 6.1e-5], np.float32),
    ])
    vals = vals[np.isfinite(vals)]
    # midpoints between adjacent halves exercise ties-to-even
    h = np.arange(0, 0x7BFF, 37, dtype=np.uint16)
    mid = (h.view(np.float16).astype(np.float64) + (h + 1).astype(np.uint16).view(np.float16).astype(np.float64)) / 2
    vals = np.concatenate([vals, mid.astype(np.float32)])
    with np.errstate(over="ignore"):
        want = vals.astype(np.float16).view(np.uint16)
    got = np.array([O.f32_to_fp16(float(v)) for v in vals], dtype=np.uint16)
    assert np.array_equal(got, want)


# ---------------------------------------------------------------- block codecs

def test_smoke_row_writer_layout(kats):
    k = kats["smoke_row_writer"]
    r8 = smoke_row(Q8, k["scale"], k["value"])
    assert list(r8[:2]) == k["q8_0_bytes_head"] and set(r8[2:]) == {k["q8_0_fill"]} and r8.size == 34
    r4 = smoke_row(Q4, k["scale"], k["value"])
    assert list(r4[:2]) == k["q4_0_bytes_head"] and set(r4[2:]) == {k["q4_0_fill"]} and r4.size == 18


def test_q4_0_nibble_order_and_offset(kats):
    k = kats["q4_0_nibble_order"]
    blk = np.full(18, k["fill_byte"], dtype=np.uint8)
    blk[0:2] = np.array([k["scale_bits"]], dtype=np.uint16).view(np.uint8)
    blk[2], blk[3] = k["qs0"], k["qs1"]
    deq = O.dequantize(Q4, blk)
    for idx, want in k["dequant"].items():
        assert deq[int(idx)] == want
    x = np.zeros((1, 32), dtype=np.float32)
    x[0, k["input_ones_at"]] = 1.0
    y = O.linear_f32(Q4, x, blk, 1, 32, 1)
    assert abs(y[0, 0] - k["expected"]) <= k["tolerance_abs"]
    v, s = O.block_values_i8(Q4, blk)
    assert s == 1.0 and v[0] == -8 and v[1] == -6 and v[16] == -7 and v[17] == -5 and v[5] == 0


@pytest.mark.parametrize("name,fmt", [("q8_0_direct", Q8), ("q4_0_direct", Q4)])
def test_direct_matmul_kats(kats, name, fmt):
    k = kats[name]
    rows = []
    for r in k["rows"]:
        hb = np.array([r["scale_bits"]], dtype=np.uint16).view(np.uint8)
        if fmt == Q8:
            rows.append(np.concatenate([hb, np.full(32, r["q"], np.int8).view(np.uint8)]))
        else:
            rows.append(np.concatenate([hb, np.full(16, r["fill_byte"], np.uint8)]))
    w = np.concatenate(rows)
    x = np.full((1, 32), k["input_fill"], dtype=np.float32)
    y = O.linear_f32(fmt, x, w, 1, 32, k["out_dim"])
    assert np.allclose(y[0], k["expected"], atol=k["tolerance_abs"], rtol=0)
    # the engine op takes the same (f32) route at this shape
    assert not O.uses_activation_quant(1, 32, k["out_dim"])
    assert np.array_equal(O.linear_no_bias(fmt, x, w, 1, 32, k["out_dim"]), y)


@pytest.mark.parametrize("fmt", [Q8, Q4])
def test_gpu_smoke_kat_on_oracle(kats, fmt):
    k = kats["gpu_smoke"]
    x = np.stack([np.arange(1, 33), -np.arange(1, 33)]).astype(np.float32)
    w = np.concatenate([smoke_row(fmt, r["scale"], r["value"]) for r in k["weight_rows"]])
    y = O.linear_no_bias(fmt, x, w, k["rows"], k["in_dim"], k["out_dim"])
    assert np.allclose(y.reshape(-1), k["expected"], atol=k["tolerance_abs"], rtol=0)


def test_weight_quantizers_closed_form(kats):
    rng = np.random.default_rng(3)
    for _ in range(50):
        x = (rng.standard_normal(32) * rng.uniform(1e-3, 30)).astype(np.float32)
        # Q8_0: scale = max|x|/127 stored as fp16, q = round-half-away(x * (1/scale)) clamped
        raw = O.quantize_weights(Q8, x)
        scale32 = np.float32(np.abs(x).max()) / np.float32(127.0)
        assert raw[:2].view(np.float16)[0] == np.float16(scale32)
        inv = np.float32(1.0) / scale32
        t = x * inv
        want = np.clip(np.sign(t) * np.floor(np.abs(t) + np.float32(0.5)), -127, 127).astype(np.int8)
        assert np.array_equal(raw[2:].view(np.int8), want)
        assert np.abs(want).max() == 127
        # Q4_0: scale = max|x|/8 >= 0, q = clamp(round(x/scale) + 8, 0, 15), lo | hi<<4
        raw4 = O.quantize_weights(Q4, x)
        s4 = np.float32(np.abs(x).max()) / np.float32(8.0)
        assert raw4[:2].view(np.float16)[0] == np.float16(s4)
        t4 = x * (np.float32(1.0) / s4)
        q4 = np.clip(np.sign(t4) * np.floor(np.abs(t4) + np.float32(0.5)) + 8, 0, 15).astype(np.uint8)
        assert np.array_equal(raw4[2:], q4[:16] | (q4[16:] << 4))
        deq = O.dequantize(Q4, raw4)
        assert np.abs(deq - x).max() <= kats["quantizer_roundtrip"]["q4_0_tolerance"] * float(s4)
    z = np.zeros(32, np.float32)
    r8, r4 = O.quantize_weights(Q8, z), O.quantize_weights(Q4, z)
    assert r8[:2].view(np.float16)[0] == 1.0 and not r8[2:].any()
    assert r4[:2].view(np.float16)[0] == 1.0 and set(r4[2:]) == {0x88}
    unit = np.concatenate([np.array([0x3C00], np.uint16).view(np.uint8), np.ones(32, np.uint8)])
    assert np.array_equal(O.dequantize(Q8, unit), np.ones(32, np.float32))


# ---------------------------------------------------------------- activation quantizer

def test_activation_quantizer_invariants_and_rounding():
    x = synth.activations(11, 3, 256)
    x[1, 32:64] = 0.0  # zero block
    q, s, sums = O.quantize_activation_rows(x, 3, 256)
    blocks = x.reshape(3, 8, 32)
    max_abs = np.abs(blocks).max(axis=2)
    want_s = np.where(max_abs == 0, np.float32(1.0), max_abs / np.float32(127.0)).astype(np.float32)
    assert np.array_equal(s, want_s)
    assert np.abs(q).max() <= 127
    qb = q.reshape(3, 8, 32)
    assert np.all(np.abs(qb).max(axis=2)[max_abs > 0] == 127)
    assert not qb[1, 1].any() and s[1, 1] == 1.0
    assert np.array_equal(sums, qb.astype(np.int32).sum(axis=2))
    inv = np.where(max_abs == 0, np.float32(0.0), np.float32(1.0) / want_s).astype(np.float32)
    t = blocks * inv[:, :, None]
    want_q = np.clip(np.sign(t) * np.floor(np.abs(t) + np.float32(0.5)), -127, 127).astype(np.int8)
    assert np.array_equal(qb, want_q)
    # ties round away from zero: max = 127 makes scale = 1 and inv = 1 exactly
    blk = np.zeros((1, 32), np.float32)
    blk[0, :7] = [127.0, 0.5, -0.5, 1.5, -1.5, 126.5, -2.5]
    q2, s2, _ = O.quantize_activation_rows(blk, 1, 32)
    assert s2[0, 0] == 1.0
    assert list(q2[0, :7]) == [127, 1, -1, 2, -2, 127, -3]


def test_i8_dot_reference_pattern_and_brute_force(kats):
    i = np.arange(32)
    x = ((i % 17) - 8).astype(np.int8)
    w = (((5 * i + 3) % 19) - 9).astype(np.int8)
    assert O.dot_i8_block(x, w) == int((x.astype(np.int64) * w.astype(np.int64)).sum())
    rng = np.random.default_rng(5)
    for _ in range(200):
        a = rng.integers(-128, 128, 32).astype(np.int8)
        b = rng.integers(-128, 128, 32).astype(np.int8)
        assert O.dot_i8_block(a, b) == int((a.astype(np.int64) * b.astype(np.int64)).sum())
    full = np.full(32, -127, np.int8)
    assert O.dot_i8_block(full, full) == 516128  # largest |dot| the quantizers can produce


# ---------------------------------------------------------------- matmuls

def _numpy_route_a(fmt, x, w_raw, rows, in_dim, out_dim):
    """float64 closed form: sum_b sx*sw*dot_b with the quantizers restated in numpy."""
    kb = in_dim // 32
    bb = O.BLOCK_BYTES[fmt]
    wb = np.asarray(w_raw, np.uint8).reshape(out_dim, kb, bb)
    sw = wb[:, :, :2].copy().view(np.float16).astype(np.float64).reshape(out_dim, kb)
    if fmt == Q8:
        qw = wb[:, :, 2:].view(np.int8).astype(np.int64)
    else:
        qs = wb[:, :, 2:]
        qw = np.concatenate([(qs & 0xF).astype(np.int64) - 8, (qs >> 4).astype(np.int64) - 8], axis=2)
    blocks = x.reshape(rows, kb, 32)
    max_abs = np.abs(blocks).max(axis=2)
    sx = np.where(max_abs == 0, np.float32(1), max_abs / np.float32(127)).astype(np.float32)
    inv = np.where(max_abs == 0, np.float32(0), np.float32(1) / sx).astype(np.float32)
    t = blocks * inv[:, :, None]
    qx = np.clip(np.sign(t) * np.floor(np.abs(t) + np.float32(0.5)), -127, 127).astype(np.int64)
    dots = np.einsum("rbk,obk->rob", qx, qw)
    y = np.einsum("rob,rb,ob->ro", dots.astype(np.float64), sx.astype(np.float64), sw)
    return dots, y


@pytest.mark.parametrize("fmt", [Q8, Q4])
@pytest.mark.parametrize("rows", [1, 2, 3, 5])
def test_route_a_matches_independent_numpy_closed_form(fmt, rows):
    in_dim, out_dim = 160, 37
    x = synth.activations(21 + rows, rows, in_dim)
    w = synth.weights(fmt, 99, out_dim, in_dim)
    dots_np, y_np = _numpy_route_a(fmt, x, w, rows, in_dim, out_dim)
    assert np.array_equal(O.block_dots(fmt, x, w, rows, in_dim, out_dim), dots_np)
    y64 = O.linear_act_f64(fmt, x, w, rows, in_dim, out_dim)
    assert np.allclose(y64, y_np, rtol=1e-12, atol=0)
    qx, sx, sums = O.quantize_activation_rows(x, rows, in_dim)
    y = O.linear_act_range(fmt, qx, sx, sums, w, rows, in_dim, out_dim, 0, out_dim)
    scale = np.abs(y_np).max()
    assert np.abs(y - y_np).max() <= 2e-6 * scale
    # every association / column range the reference can take agrees to f32 rounding
    for assoc in (O.ASSOC_PAIR, O.ASSOC_SINGLE):
        ya = O.linear_act_assoc(fmt, assoc, x, w, rows, in_dim, out_dim)
        assert np.abs(ya - y_np).max() <= 2e-6 * scale
    yr = np.zeros_like(y)
    for o0, o1 in [(0, 5), (5, 18), (18, 37)]:
        O.linear_act_range(fmt, qx, sx, sums, w, rows, in_dim, out_dim, o0, o1, y=yr)
    assert np.abs(yr - y).max() <= 1e-6 * scale
    if fmt == Q8:
        assert np.array_equal(yr, y)  # Q8_0 has one association on every path


@pytest.mark.parametrize("fmt", [Q8, Q4])
def test_route_b_equals_dequantize_then_matmul(fmt, kats):
    k = kats["q4_0_multirow_vs_dense"]
    rows, in_dim, out_dim = k["rows"], k["in_dim"], k["out_dim"]
    bb = O.BLOCK_BYTES[fmt]
    n = out_dim * (in_dim // 32) * bb
    w = ((37 * np.arange(n) + 11) & 0xFF).astype(np.uint8)
    w.reshape(-1, bb)[:, 0] = 0x00
    w.reshape(-1, bb)[:, 1] = 0x3C
    x = (synth.uniform01(0x5EED1234, 0, rows * in_dim) * 2 - 1).astype(np.float32).reshape(rows, in_dim)
    dense = O.dequantize(fmt, w).reshape(out_dim, in_dim).astype(np.float64)
    want = x.astype(np.float64) @ dense.T
    got = O.linear_f32(fmt, x, w, rows, in_dim, out_dim)
    assert np.abs(got - want).max() <= k["tolerance_abs"]


def test_activation_quant_route_stays_close_to_f32_route(kats):
    k = kats["act_quant_vs_f32"]
    rows, in_dim, out_dim = k["rows"], k["in_dim"], k["out_dim"]
    x = (((np.arange(rows * in_dim) % 17) - 8) / np.float32(9.0)).astype(np.float32).reshape(rows, in_dim)
    dense = (((np.arange(out_dim * in_dim) % 23) - 11) / np.float32(32.0)).astype(np.float32)
    w = O.quantize_weights(Q8, dense)
    exact = O.linear_f32(Q8, x, w, rows, in_dim, out_dim)
    qx, sx, sums = O.quantize_activation_rows(x, rows, in_dim)
    quant = O.linear_act_range(Q8, qx, sx, sums, w, rows, in_dim, out_dim, 0, out_dim)
    assert np.abs(quant - exact).max() <= k["tolerance_abs"]
    assert np.abs(quant - exact).max() > 0  # they are different computations


@pytest.mark.parametrize("fmt", [Q8, Q4])
def test_engine_op_route_gate_and_thread_plans(fmt):
    # below the gate: f32 route
    x = synth.activations(1, 2, 64)
    w = synth.weights(fmt, 2, 600, 64)
    assert not O.uses_activation_quant(2, 64, 600)
    assert np.array_equal(O.linear_no_bias(fmt, x, w, 2, 64, 600), O.linear_f32(fmt, x, w, 2, 64, 600))
    # at the gate: activation-quantized route, any thread plan within f32 rounding
    rows, in_dim, out_dim = 5, 96, 640
    x = synth.activations(4, rows, in_dim)
    w = synth.weights(fmt, 5, out_dim, in_dim)
    assert O.uses_activation_quant(rows, in_dim, out_dim)
    y1 = O.linear_no_bias(fmt, x, w, rows, in_dim, out_dim, workers=1)
    y8 = O.linear_no_bias(fmt, x, w, rows, in_dim, out_dim, workers=8)
    y64 = O.linear_act_f64(fmt, x, w, rows, in_dim, out_dim)
    scale = np.abs(y64).max()
    assert np.abs(y1 - y64).max() <= 2e-6 * scale and np.abs(y8 - y64).max() <= 2e-6 * scale
    if fmt == Q8:
        assert np.array_equal(y1, y8)
    for r in (1, 2):
        ya = O.linear_no_bias(fmt, x[:r], w, r, in_dim, out_dim, workers=1)
        yb = O.linear_no_bias(fmt, x[:r], w, r, in_dim, out_dim, workers=8)
        assert np.abs(ya - yb).max() <= 1e-6 * scale
    # errors
    with pytest.raises(ValueError):
        O.linear_no_bias(fmt, x, w, 1, 33, 4)
    with pytest.raises(ValueError):
        O.linear_no_bias(12, x, w, 1, 32, 4)


def test_thread_plan_matches_reference_policy():
    assert O.thread_plan(1, 4096, 14336) == (8, True)     # decode: 8 column chunks
    assert O.thread_plan(2, 4096, 14336) == (8, True)
    assert O.thread_plan(4, 4096, 14336) == (4, False)    # rows > 2: row split, min(8, rows)
    assert O.thread_plan(5, 14336, 4096) == (5, False)
    assert O.thread_plan(512, 4096, 4096) == (8, False)
    assert O.thread_plan(1, 4096, 300) == (1, False)      # out < 512 and one row: serial
    assert O.thread_plan(1, 4096, 576) == (8, True)       # 576/64 = 9 -> capped at 8
    assert O.thread_plan(1, 4096, 512, max_workers=8, cpu_count=4) == (4, True)
    assert O.thread_plan(1, 32, 100) == (1, False)        # below the 16384 work-unit floor


@pytest.mark.parametrize("fmt", [Q8, Q4])
def test_timing_path_matches_faithful_path(fmt):
    rows, in_dim, out_dim = 5, 256, 515
    x = synth.activations(8, rows, in_dim)
    w = synth.weights(fmt, 9, out_dim, in_dim)
    p = O.Prepared(fmt, w, out_dim, in_dim)
    want = O.linear_act_assoc(fmt, O.ASSOC_PAIR, x, w, rows, in_dim, out_dim)
    for workers in (1, 8):
        assert np.array_equal(p.linear(x, rows, workers=workers), want)
    assert np.array_equal(p.linear(x[:1], 1, workers=8), want[:1])
    p.close()


# ---------------------------------------------------------------- Q4_K

def q4k_block(d_bits, dmin_bits, scales12, qs128):
    return np.concatenate([np.array([d_bits, dmin_bits], np.uint16).view(np.uint8), np.asarray(scales12, np.uint8),
                           np.asarray(qs128, np.uint8)])


def test_q4_k_reference_vectors(kats):
    k = kats["q4_k"]
    u = k["uniform_block"]
    scales = [u["scales_first4"]] * 4 + [0] * 4 + [u["scales_last4"]] * 4
    blk = q4k_block(u["d_bits"], 0, scales, [u["qs_fill"]] * 128)
    assert np.abs(O.dequantize_q4_k(blk) - u["expect_all"]).max() <= u["tolerance_abs"]
    m = k["direct_matmul"]
    w = np.concatenate([q4k_block(15360, 0, scales, [f] * 128) for f in m["row_qs_fill"]])
    x = np.full((1, m["in_dim"]), m["input_fill"], np.float32)
    y = O.linear_q4_k(x, w, 1, m["in_dim"], m["out_dim"])
    assert np.abs(y[0] - np.array(m["expected"])).max() <= m["tolerance_abs"]
    # the reference's quantizer test fixes the bytes of a block whose values are scs*q - mins with d = dmin = 1:
    # decoding those bytes must give the values back exactly (a wrong bit in the 6-bit unpack fails here)
    h = k["header_packing"]
    scs, mins = O.q4k_unpack_scale_mins(h["header"][4:16])
    assert scs.tolist() == h["scs"] and mins.tolist() == h["mins"]
    raw = np.array(h["header"] + h["qs_32"] * 4, np.uint8)
    want = np.array([h["scs"][sub] * (i % 16) - h["mins"][sub] for sub in range(8) for i in range(32)], np.float32)
    assert np.array_equal(O.dequantize_q4_k(raw), want)


def numpy_dequantize_q4_k(raw):
    """Independent restatement: published ggml Q4_K layout, vectorised."""
    b = np.asarray(raw, np.uint8).reshape(-1, 144)
    d = b[:, 0:2].copy().view(np.float16).astype(np.float32)[:, 0]
    dmin = b[:, 2:4].copy().view(np.float16).astype(np.float32)[:, 0]
    s = b[:, 4:16].astype(np.uint8)
    sc = np.empty((b.shape[0], 8), np.uint8)
    mn = np.empty((b.shape[0], 8), np.uint8)
    sc[:, :4], mn[:, :4] = s[:, 0:4] & 63, s[:, 4:8] & 63
    sc[:, 4:] = (s[:, 8:12] & 0x0F) | ((s[:, 0:4] >> 6) << 4)
    mn[:, 4:] = (s[:, 8:12] >> 4) | ((s[:, 4:8] >> 6) << 4)
    qs = b[:, 16:].reshape(-1, 4, 32)
    q = np.stack([qs & 0x0F, qs >> 4], axis=2).reshape(-1, 8, 32).astype(np.float32)   # sub-blocks 2c, 2c+1
    dsc = (d[:, None] * sc.astype(np.float32)).astype(np.float32)
    dmn = (dmin[:, None] * mn.astype(np.float32)).astype(np.float32)
    return ((dsc[:, :, None] * q).astype(np.float32) - dmn[:, :, None]).astype(np.float32).reshape(-1)


def test_q4_k_against_independent_numpy_form():
    w = synth.weights(synth.Q4_K, 3, 6, 512)
    w[0:4] = np.array([0x0001, 0x7BFF], np.uint16).view(np.uint8)  # subnormal d, largest finite dmin
    deq = O.dequantize_q4_k(w)
    assert np.array_equal(deq.view(np.uint32), numpy_dequantize_q4_k(w).view(np.uint32))
    x = synth.activations(4, 5, 512)
    wf = np.nan_to_num(deq.reshape(6, 512).astype(np.float64), posinf=0, neginf=0)
    w2 = synth.weights(synth.Q4_K, 5, 6, 512)
    wf2 = O.dequantize_q4_k(w2).reshape(6, 512).astype(np.float64)
    y64 = O.linear_q4_k(x, w2, 5, 512, 6, f64=True)
    assert np.abs(y64 - x.astype(np.float64) @ wf2.T).max() <= 1e-12 * np.abs(y64).max() + 1e-15
    y = O.linear_q4_k(x, w2, 5, 512, 6)
    assert np.abs(y - y64).max() <= 2e-6 * np.abs(y64).max()
    with pytest.raises(ValueError):
        O.linear_q4_k(np.zeros((1, 128), np.float32), np.zeros(0, np.uint8), 1, 128, 0)
    del wf


def numpy_pack_q4_k(d, dmin, sc, mn, q):
    """Independent packer of the published ggml Q4_K layout: sc, mn [n, 8] (6 bits), q [n, 8, 32] nibbles."""
    n = sc.shape[0]
    b = np.zeros((n, 144), np.uint8)
    b[:, 0:2] = np.asarray(d, np.float16).reshape(n, 1).view(np.uint8)
    b[:, 2:4] = np.asarray(dmin, np.float16).reshape(n, 1).view(np.uint8)
    b[:, 4:8] = (sc[:, :4] & 63) | ((sc[:, 4:] >> 4) << 6)
    b[:, 8:12] = (mn[:, :4] & 63) | ((mn[:, 4:] >> 4) << 6)
    b[:, 12:16] = (sc[:, 4:] & 15) | ((mn[:, 4:] & 15) << 4)
    qq = q.reshape(n, 4, 2, 32)
    b[:, 16:] = (qq[:, :, 0, :] | (qq[:, :, 1, :] << 4)).reshape(n, 128)
    return b.reshape(-1)


def round_half_away_f32(v):
    v64 = np.asarray(v, np.float32).astype(np.float64)  # exact; + 0.5 is exact in f64 too
    return np.sign(v64) * np.floor(np.abs(v64) + 0.5)


def numpy_quantize_q4_k(x):
    """Vectorised f32 restatement of the quantizer from its description (quant_codec.zig:1183-1238)."""
    f = np.float32
    v = np.asarray(x, f).reshape(-1, 8, 32)
    lo, hi = v.min(axis=2), v.max(axis=2)
    mm = np.maximum(-lo, f(0))
    rng = (hi + mm).astype(f)
    scale = np.where(rng == 0, f(1), (rng / f(15)).astype(f)).astype(f)
    max_scale, max_min = scale.max(axis=1), mm.max(axis=1)
    d = np.where(max_scale == 0, f(1), (max_scale / f(63)).astype(f)).astype(f)
    dmin = np.where(max_min == 0, f(1), (max_min / f(63)).astype(f)).astype(f)
    sc = np.clip(round_half_away_f32((scale / d[:, None]).astype(f)), 0, 63).astype(np.uint8)
    mn = np.clip(round_half_away_f32((mm / dmin[:, None]).astype(f)), 0, 63).astype(np.uint8)
    mn[max_min == 0] = 0
    inv = np.where(scale == 0, f(0), (f(1) / scale).astype(f)).astype(f)
    t = ((v + mm[:, :, None]).astype(f) * inv[:, :, None]).astype(f)
    q = np.clip(round_half_away_f32(t), 0, 15).astype(np.uint8)
    return numpy_pack_q4_k(d, dmin, sc, mn, q)


def test_q4_k_quantizer_reference_vectors(kats):
    k = kats["q4_k"]
    h = k["header_packing"]
    x = np.array([h["scs"][sub] * (i % 16) - h["mins"][sub] for sub in range(8) for i in range(32)], np.float32)
    assert O.quantize_q4_k(x).tolist() == h["header"] + h["qs_32"] * 4
    r = k["quantizer_round_trip"]
    ramp = (r["start"] + r["step"] * np.arange(r["count"])).astype(np.float32)
    assert np.abs(O.dequantize_q4_k(O.quantize_q4_k(ramp)) - ramp).max() <= r["tolerance_abs"]


def test_q4_k_quantizer_by_construction_and_against_numpy_form():
    rng = np.random.default_rng(41)
    # values on a grid the format represents exactly: x = 2^e * (sc * q - m) with one sub-block at sc = 63, one
    # at m = 63 (so d = dmin = 2^e), every sub-block spanning q = 0 .. 15 -> the bytes are known in advance
    n = 24
    sc = rng.integers(1, 64, (n, 8)).astype(np.uint8)
    mn = rng.integers(0, 64, (n, 8)).astype(np.uint8)
    sc[np.arange(n), rng.integers(0, 8, n)] = 63
    mn[np.arange(n), rng.integers(0, 8, n)] = 63
    q = rng.integers(0, 16, (n, 8, 32)).astype(np.uint8)
    q[:, :, 3], q[:, :, 17] = 0, 15
    e = np.exp2(rng.integers(-9, 6, n)).astype(np.float32)
    x = (e[:, None, None] * (sc[:, :, None].astype(np.float32) * q - mn[:, :, None].astype(np.float32))).astype(np.float32)
    want = numpy_pack_q4_k(e, e, sc, mn, q)
    got = O.quantize_q4_k(x)
    assert np.array_equal(got, want)
    assert np.array_equal(O.dequantize_q4_k(got), x.reshape(-1))
    # an all-zero super-block: every sub-block scale is 1, d = 1/63 -> sc = 63; no minimum -> dmin = 1, m = 0
    z = O.quantize_q4_k(np.zeros(256, np.float32))
    assert np.array_equal(z, numpy_pack_q4_k([np.float32(1) / np.float32(63)], [1.0], np.full((1, 8), 63, np.uint8),
                                             np.zeros((1, 8), np.uint8), np.zeros((1, 8, 32), np.uint8)))
    # all-positive values: no offset, nibble = round(15 x / max); all-negative: offset -min, the largest value is
    # not at nibble 15
    pos = np.tile(np.linspace(1.0, 3.0, 32, dtype=np.float32), 8)
    bp = O.quantize_q4_k(pos)
    assert bp[2:4].tolist() == [0x00, 0x3C] and not bp[8:12].any() and (bp[12:16] >> 4).tolist() == [0] * 4
    assert (bp[16:48] & 15).tolist() == [int(np.floor(15.0 * v / 3.0 + 0.5)) for v in pos[:32].astype(np.float64)]
    neg = -pos
    bn = O.quantize_q4_k(neg)
    assert (bn[16:48] & 15).tolist() == [int(np.floor((float(v) + 3.0) / (np.float32(2.0) / np.float32(15.0)) + 0.5)) for v in neg[:32]]
    # random data, random magnitudes per sub-block, ties included: byte-identical to the vectorised restatement
    xr = (rng.standard_normal((64, 8, 32)) * np.exp2(rng.integers(-12, 12, (64, 8, 1)))).astype(np.float32)
    xr[5, 2] = 0.0
    xr[6] = np.abs(xr[6])
    xr[7, :, :] = np.round(xr[7] * 2) / 2
    assert np.array_equal(O.quantize_q4_k(xr), numpy_quantize_q4_k(xr))
    # and close to the input: nibble rounding (scale / 2) plus the 6-bit rounding of scale and minimum
    deq = O.dequantize_q4_k(O.quantize_q4_k(xr)).reshape(64, 8, 32)
    span = (xr.max(axis=2) + np.maximum(-xr.min(axis=2), 0)).max(axis=1)
    mins = np.maximum(-xr.min(axis=2), 0).max(axis=1)
    bound = span / 30 + 15 * (span / 15 / 63) * 0.51 + mins / 63 * 0.51
    assert (np.abs(deq - xr).max(axis=(1, 2)) <= bound * 1.01 + 1e-30).all()


# ---------------------------------------------------------------- Q4_K with Q8_K activations

def test_q8k_route_gate_is_the_reference_list():
    """shouldUseQ4Q5KQ8KActivationShape, native_compute.zig:3468-3479, case by case."""
    yes_rows = [1, 2, 4, 9, 50, 64, 77, 154, 197, 231, 257, 308, 514]
    for blocks in (2, 3, 6, 8, 12):
        for rows in yes_rows:
            assert O.uses_q4k_q8k_activation(rows, blocks * 256, 512), (rows, blocks)
        for rows in (0, 3, 5, 8, 16, 32, 63, 65, 100, 385, 462, 513, 1024):
            assert not O.uses_q4k_q8k_activation(rows, blocks * 256, 4096), (rows, blocks)
        assert not O.uses_q4k_q8k_activation(1, blocks * 256, 511)
    for blocks in (1, 4, 5, 7, 9, 10, 11, 13, 16, 56):
        assert not O.uses_q4k_q8k_activation(1, blocks * 256, 4096), blocks
    assert not O.uses_q4k_q8k_activation(1, 2048 + 32, 4096)


def test_q8_k_quantizer_invariants_and_closed_forms():
    """quantizeQ8_KBlock: the reference's own checks (block sums = sums of the stored bytes,
    quant_codec.zig:3342-3360; ramp round trip within 1.5, :3329-3340) and the quantized values
    themselves from exact rational arithmetic wherever the exact quotient is not within 1e-4 of a tie."""
    from fractions import Fraction
    i = np.arange(256)
    cases = [((i % 31 - 15) * 0.25).astype(np.float32), (-48.0 + 0.375 * i).astype(np.float32),
             synth.activations(5, 1, 256).reshape(-1), np.zeros(256, np.float32),
             np.where(i % 2 == 0, 3.0, -3.0).astype(np.float32)]
    for x in cases:
        q, d, bs = O.quantize_q8_k(x)
        assert np.array_equal(bs, q.astype(np.int32).reshape(16, 16).sum(axis=1).astype(np.int16))
        m = float(np.abs(x).max())
        if m == 0.0:
            assert d[0] == 1.0 and not q.any()
            continue
        assert d[0] == np.float32(m) / np.float32(127.0)
        assert np.abs(q.astype(np.float64) * float(d[0]) - x).max() <= 1.5
        assert np.abs(q).max() == 127 and np.abs(q.astype(np.int32)).max() <= 127
        checked = 0
        for v, got in zip(x.tolist(), q.tolist()):
            t = Fraction(v) * 127 / Fraction(m)
            frac = abs(t) - int(abs(t))
            if abs(frac - Fraction(1, 2)) < Fraction(1, 10000):
                continue
            want = int(abs(t) + Fraction(1, 2)) * (1 if t >= 0 else -1)
            assert got == want, (v, got, want)
            checked += 1
        assert checked > 200
    q, d, bs = O.quantize_q8_k(np.concatenate([cases[0], cases[2]]))  # blocks are independent
    assert np.array_equal(q[:256], O.quantize_q8_k(cases[0])[0]) and np.array_equal(q[256:], O.quantize_q8_k(cases[2])[0])


def test_q4_k_q8k_route_against_brute_force_and_the_dequantized_dot():
    """The route's sum restated independently: integer sub-block dots by numpy on the unpacked
    nibbles, combined in float64 -- and the property the reference tests its Q8_K routes with
    (native_compute.zig:42279-42346): the result is the f32-route product of the DEQUANTIZED
    activations q * d.  A dropped min term, a swapped nibble order or a wrong sub-block index fails both."""
    rows, in_dim, out_dim = 4, 768, 9
    kb = in_dim // 256
    x = synth.activations(21, rows, in_dim)
    x[1, 256:512] = 0.0  # an all-zero activation block
    w = synth.weights(synth.Q4_K, 22, out_dim, in_dim)
    y = O.linear_q4_k_q8k(x, w, rows, in_dim, out_dim)
    q, d, bs = O.quantize_q8_k(x)
    q = q.reshape(rows, kb, 8, 32).astype(np.int64)
    d = d.reshape(rows, kb).astype(np.float64)
    b = w.reshape(out_dim, kb, 144)
    dw = b[:, :, 0:2].copy().view(np.float16).astype(np.float64)[..., 0]
    dmin = b[:, :, 2:4].copy().view(np.float16).astype(np.float64)[..., 0]
    want = np.zeros((rows, out_dim))
    for o in range(out_dim):
        for k in range(kb):
            scs, mins = O.q4k_unpack_scale_mins(b[o, k, 4:16])
            qs = b[o, k, 16:].reshape(4, 32)
            nib = np.stack([qs & 15, qs >> 4], axis=1).reshape(8, 32).astype(np.int64)
            for r in range(rows):
                dots = (q[r, k] * nib).sum(axis=1)
                sums = q[r, k].sum(axis=1)
                want[r, o] += d[r, k] * float(((dw[o, k] * scs) * dots - (dmin[o, k] * mins) * sums).sum())
    scale = np.abs(want).max(axis=1, keepdims=True)
    assert (np.abs(y - want) / scale).max() <= 2e-6
    xq = (q.reshape(rows, kb, 256) * d[:, :, None]).reshape(rows, in_dim).astype(np.float32)
    via_dequant = O.linear_q4_k(xq, w, rows, in_dim, out_dim, f64=True)
    assert (np.abs(y - via_dequant) / scale).max() <= 2e-6
    # and it stays close to the f32 route on the unquantized activations (the reference's own
    # bound is 1e-2 of the value or 5e-2, native_compute.zig:42392-42437)
    f32_route = O.linear_q4_k(x, w, rows, in_dim, out_dim, f64=True)
    assert (np.abs(y - f32_route) / scale).max() <= 2e-2
    assert (np.abs(y - f32_route) / scale).max() > 1e-5  # it IS another route
    with pytest.raises(ValueError):
        O.linear_q4_k_q8k(np.zeros((1, 128), np.float32), np.zeros(0, np.uint8), 1, 128, 0)


# ---------------------------------------------------------------- greedy token pick

def test_argmax_reference_vectors_and_properties(kats):
    for case in kats["argmax"]["cases"]:
        assert O.argmax(case["data"]) == case["expect"]
    lr = kats["argmax"]["last_row"]
    assert O.argmax_last_row(lr["data"], lr["rows"], lr["dim"]) == lr["expect"]
    with pytest.raises(ValueError):
        O.argmax_last_row([], 0, 3)
    # against numpy (first index of the maximum) on random rows with many ties
    rng = np.random.default_rng(5)
    for n in (1, 7, 64, 1000):
        v = rng.integers(-3, 4, size=n).astype(np.float32)
        assert O.argmax(v) == int(np.argmax(v))
    # equal values: the first one; -0 equals +0; infinities order; NaNs never win
    assert O.argmax([1.0, 5.0, 5.0, 2.0]) == 1
    assert O.argmax([-1.0, -0.0, 0.0]) == 1
    assert O.argmax([-np.inf, -np.inf]) == 0
    assert O.argmax([1.0, np.inf, np.nan, np.inf]) == 1
    assert O.argmax([np.nan, -2.0, np.nan, -1.0]) == 3
    assert O.argmax([np.nan, np.nan]) == 0


def test_biased_linear_is_the_no_bias_op_plus_bias_rows():
    """The reference's own biased Q8_0 test inputs (ops/native_compute.zig:39163-39223): small
    integers and scale 1.0, so the expected values are exact; and the general definition
    (:5065-5077, :5197-5203) against numpy broadcasting."""
    rows, in_dim, out_dim = 3, 32, 2
    x = np.array([(i % 7) - 3 for i in range(rows * in_dim)], np.float32).reshape(rows, in_dim)
    q = np.array([(i % 5) - 2 for i in range(32)], np.int8)
    w = np.concatenate([np.concatenate([np.array([0x00, 0x3C], np.uint8), q.view(np.uint8)])] * out_dim)
    bias = np.array([0.25, -0.5], np.float32)
    want = (x.astype(np.int64) @ np.tile(q.astype(np.int64), (out_dim, 1)).T).astype(np.float32) + bias
    assert np.array_equal(O.linear(Q8, x, w, bias, rows, in_dim, out_dim), want)
    assert want[0, 0] != want[0, 1] and want[0, 0] - bias[0] == want[0, 1] - bias[1]  # same weights, different bias

    rows, in_dim, out_dim = 5, 512, 700
    x = synth.activations(71, rows, in_dim)
    bias = synth.activations(72, 1, out_dim)[0]
    for fmt in (Q4, Q8):
        w = synth.weights(fmt, 73, out_dim, in_dim)
        plain = O.linear_no_bias(fmt, x, w, rows, in_dim, out_dim)
        assert np.array_equal(O.linear(fmt, x, w, bias, rows, in_dim, out_dim), plain + bias[None, :])


def test_activations_against_float64_closed_forms():
    """relu / quick_gelu / tanh-form gelu (backends/activations.zig:43-127) against the formulas in
    float64, plus the values the mathematics fixes: f(0) = 0, f(x) -> x for large x, -> 0 for
    very negative x, gelu(x) - gelu(-x) = x, quick_gelu(x) - quick_gelu(-x) = x."""
    x = np.concatenate([np.linspace(-12, 12, 4801), [0.0, 1e-6, -1e-6, 30.0, -30.0, 88.0, -88.0]]).astype(np.float32)
    x64 = x.astype(np.float64)
    assert np.array_equal(O.apply_activation(O.RELU, x), np.maximum(x, 0))
    qg = O.apply_activation(O.QUICK_GELU, x)
    assert np.allclose(qg, x64 / (1 + np.exp(-1.702 * x64)), rtol=2e-6, atol=1e-30)
    g = O.apply_activation(O.GELU, x)
    assert np.allclose(g, 0.5 * x64 * (1 + np.tanh(0.7978845608028654 * (x64 + 0.044715 * x64 ** 3))), rtol=2e-6, atol=1e-7)
    for kind in (O.RELU, O.QUICK_GELU, O.GELU):
        y = O.apply_activation(kind, np.float32([0.0, 30.0, -30.0]))
        assert y[0] == 0 and y[1] == 30.0 and abs(y[2]) < 1e-20
    for got in (qg, g):  # f(x) - f(-x) = x: pairs of the symmetric grid
        sym = got[:4801]
        assert np.allclose(sym - sym[::-1], x[:4801], rtol=1e-5, atol=1e-6)
    assert np.array_equal(O.apply_activation(0, x), x)


def test_synth_is_chunk_invariant_and_in_range():
    a = synth.splitmix64(42, 0, 1000)
    b = np.concatenate([synth.splitmix64(42, 0, 333), synth.splitmix64(42, 333, 667)])
    assert np.array_equal(a, b)
    w8 = synth.weights(Q8, 1, 8, 64).reshape(-1, 34)
    q = w8[:, 2:].view(np.int8)
    assert q.min() >= -127 and q.max() <= 127
    s = w8[:, :2].copy().view(np.float16).astype(np.float32)
    assert (s >= 0).all() and s.max() < 0.02 * 6 / 127
    w4 = synth.weights(Q4, 1, 8, 64)
    assert w4.size == synth.weight_bytes(Q4, 8, 64) == 8 * 2 * 18
    x = synth.activations(3, 64, 512)
    assert abs(float(x.mean())) < 0.02 and abs(float(x.std()) - 1.0) < 0.02


def test_oracle_reproduces_committed_tiny_vectors():
    """tests/golden/tiny_vectors.npz (written by tests/golden/make_tiny_vectors.py) holds the
    oracle's intermediates for two tiny shapes per format; the oracle as built now must give the
    same bits, and the fixture must be self-consistent with what the mathematics fixes."""
    import importlib.util

    spec = importlib.util.spec_from_file_location("make_tiny_vectors", os.path.join(ROOT, "tests", "golden", "make_tiny_vectors.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    want = np.load(os.path.join(ROOT, "tests", "golden", "tiny_vectors.npz"), allow_pickle=False)
    got = mod.build()
    assert sorted(want.files) == sorted(got)
    for name in want.files:
        assert np.array_equal(want[name], got[name]), name
    # independent of the oracle: the block dots are the integer sums of products of the stored
    # quantized activations and the weights as numpy unpacks them
    for fmt_name, fmt in mod.FORMATS:
        for case, rows, in_dim, out_dim in mod.CASES:
            key = f"{fmt_name}_{case}_"
            raw = want[key + "w_raw"].reshape(out_dim, in_dim // 32, -1)
            if fmt == Q8:
                wq = raw[:, :, 2:].view(np.int8).astype(np.int64)
            else:
                b = raw[:, :, 2:].astype(np.int64)
                wq = np.concatenate([(b & 15) - 8, (b >> 4) - 8], axis=2)
            qx = want[key + "qx"].reshape(rows, in_dim // 32, 32).astype(np.int64)
            dots = np.einsum("rbi,obi->rob", qx, wq)
            assert np.array_equal(dots, want[key + "block_dots"].astype(np.int64)), key
            d = raw[:, :, :2].copy().view(np.float16).astype(np.float64)[:, :, 0]
            y64 = np.einsum("rb,ob,rob->ro", want[key + "sx"].astype(np.float64), d, dots.astype(np.float64))
            for assoc in ("y_pair_assoc", "y_single_assoc"):
                assert np.abs(want[key + assoc] - y64).max() <= 2e-6 * np.abs(y64).max(), (key, assoc)
            gate = bool(want[key + "uses_activation_quant"][0])
            assert gate == (out_dim >= 512 and in_dim // 32 >= 3)
            assert np.array_equal(want[key + "y_op"], want[key + ("y_single_assoc" if gate else "y_f32_route")]) or gate
