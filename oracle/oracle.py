"""ctypes front end of the CPU oracle (libqmatmul_oracle.so).

TEST INFRASTRUCTURE ONLY: imported by tests/, __graft_entry__.smoke() and the
cpu_baseline leg of bench.py.  The product package never imports this module.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libqmatmul_oracle.so")

FMT_Q4_0 = 2
FMT_Q8_0 = 8
FMT_Q4_K = 12
BLOCK_BYTES = {FMT_Q4_0: 18, FMT_Q8_0: 34, FMT_Q4_K: 144}
BLOCK_VALUES = {FMT_Q4_0: 32, FMT_Q8_0: 32, FMT_Q4_K: 256}
ASSOC_PAIR = 0
ASSOC_SINGLE = 1


def build() -> str:
    subprocess.check_call(["make", "-s", "-C", HERE, "-B"])
    return LIB_PATH


_lib = None


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            build()
        L = C.CDLL(LIB_PATH)
        sz, vp, i32, u16, f32 = C.c_size_t, C.c_void_p, C.c_int, C.c_uint16, C.c_float
        L.afo_block_bytes.restype = sz
        L.afo_block_bytes.argtypes = [i32]
        L.afo_byte_len.restype = sz
        L.afo_byte_len.argtypes = [i32, sz]
        L.afo_fp16_to_f32.restype = f32
        L.afo_fp16_to_f32.argtypes = [u16]
        L.afo_f32_to_fp16.restype = u16
        L.afo_f32_to_fp16.argtypes = [f32]
        L.afo_quantize_q8_0_block.argtypes = [vp, vp]
        L.afo_quantize_q4_0_block.argtypes = [vp, vp]
        L.afo_dequantize.argtypes = [i32, vp, sz, vp]
        L.afo_block_values_i8.argtypes = [i32, vp, vp, vp]
        L.afo_quantize_activation_rows.argtypes = [vp, sz, sz, vp, vp, vp]
        L.afo_dot_i8_block.restype = C.c_int32
        L.afo_dot_i8_block.argtypes = [vp, vp]
        L.afo_block_dots.argtypes = [i32, vp, vp, sz, sz, sz, vp]
        L.afo_uses_activation_quant.argtypes = [sz, sz, sz]
        L.afo_linear_act_range.argtypes = [i32, vp, vp, vp, vp, vp, sz, sz, sz, sz, sz]
        L.afo_linear_act_assoc.argtypes = [i32, i32, vp, vp, vp, vp, sz, sz, sz]
        L.afo_linear_f32.argtypes = [i32, vp, vp, vp, sz, sz, sz]
        L.afo_linear_no_bias.argtypes = [i32, vp, vp, vp, sz, sz, sz, i32]
        L.afo_q4k_unpack_scale_mins.argtypes = [vp, vp, vp]
        L.afo_dequantize_q4_k.argtypes = [vp, sz, vp]
        L.afo_quantize_q4_k_block.argtypes = [vp, vp]
        L.afo_quantize_q4_k_block.restype = None
        L.afo_linear_q4_k.argtypes = [vp, vp, vp, sz, sz, sz]
        L.afo_linear_q4_k_f64.argtypes = [vp, vp, vp, sz, sz, sz]
        L.afo_uses_q4k_q8k_activation.argtypes = [sz, sz, sz]
        L.afo_quantize_q8_k.argtypes = [vp, sz, vp, vp, vp]
        L.afo_quantize_q8_k.restype = None
        L.afo_linear_q4_k_q8k.argtypes = [vp, vp, vp, sz, sz, sz]
        L.afo_argmax.restype = sz
        L.afo_argmax.argtypes = [vp, sz]
        L.afo_argmax_last_row.restype = C.c_long
        L.afo_argmax_last_row.argtypes = [vp, sz, sz]
        L.afo_add_linear_bias_rows.restype = None
        L.afo_add_linear_bias_rows.argtypes = [vp, vp, sz, sz]
        L.afo_apply_activation.restype = None
        L.afo_apply_activation.argtypes = [i32, vp, sz]
        L.afo_linear_act_f64.argtypes = [i32, vp, vp, vp, sz, sz, sz]
        L.afo_thread_plan.argtypes = [sz, sz, sz, i32, i32, vp]
        L.afo_prepare.restype = vp
        L.afo_prepare.argtypes = [i32, vp, sz, sz]
        L.afo_prepared_free.argtypes = [vp]
        L.afo_linear_prepared.argtypes = [vp, vp, vp, sz, i32]
        _lib = L
    return _lib


def _p(a: np.ndarray) -> int:
    return a.ctypes.data


def _f32(a) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=np.float32)


def _u8(a) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=np.uint8)


def fp16_to_f32(bits: int) -> float:
    return float(lib().afo_fp16_to_f32(bits))


def f32_to_fp16(value: float) -> int:
    return int(lib().afo_f32_to_fp16(np.float32(value)))


def quantize_weights(fmt: int, w: np.ndarray) -> np.ndarray:
    """f32 [.., K] -> raw GGUF block bytes (reference weight quantizers)."""
    w = _f32(w).reshape(-1, 32)
    out = np.zeros((w.shape[0], BLOCK_BYTES[fmt]), dtype=np.uint8)
    fn = lib().afo_quantize_q8_0_block if fmt == FMT_Q8_0 else lib().afo_quantize_q4_0_block
    for i in range(w.shape[0]):
        fn(_p(w[i]), _p(out[i]))
    return out.reshape(-1)


def dequantize(fmt: int, raw: np.ndarray) -> np.ndarray:
    raw = _u8(raw)
    nb = raw.size // BLOCK_BYTES[fmt]
    out = np.empty(nb * 32, dtype=np.float32)
    rc = lib().afo_dequantize(fmt, _p(raw), nb, _p(out))
    assert rc == 0
    return out


def block_values_i8(fmt: int, raw_block: np.ndarray):
    raw_block = _u8(raw_block)
    v = np.empty(32, dtype=np.int8)
    s = np.empty(1, dtype=np.float32)
    lib().afo_block_values_i8(fmt, _p(raw_block), _p(v), _p(s))
    return v, float(s[0])


def quantize_activation_rows(x: np.ndarray, rows: int, in_dim: int):
    x = _f32(x)
    kb = in_dim // 32
    q = np.empty(rows * in_dim, dtype=np.int8)
    s = np.empty(rows * kb, dtype=np.float32)
    sums = np.empty(rows * kb, dtype=np.int32)
    lib().afo_quantize_activation_rows(_p(x), rows, in_dim, _p(q), _p(s), _p(sums))
    return q.reshape(rows, in_dim), s.reshape(rows, kb), sums.reshape(rows, kb)


def dot_i8_block(a: np.ndarray, b: np.ndarray) -> int:
    a = np.ascontiguousarray(a, dtype=np.int8)
    b = np.ascontiguousarray(b, dtype=np.int8)
    return int(lib().afo_dot_i8_block(_p(a), _p(b)))


def block_dots(fmt, x, w_raw, rows, in_dim, out_dim) -> np.ndarray:
    x, w_raw = _f32(x), _u8(w_raw)
    out = np.empty((rows, out_dim, in_dim // 32), dtype=np.int32)
    rc = lib().afo_block_dots(fmt, _p(x), _p(w_raw), rows, in_dim, out_dim, _p(out))
    if rc != 0:
        raise ValueError(f"afo_block_dots rc={rc}")
    return out


def uses_activation_quant(rows, in_dim, out_dim) -> bool:
    return bool(lib().afo_uses_activation_quant(rows, in_dim, out_dim))


def linear_act_range(fmt, qx, sx, sums, w_raw, rows, in_dim, out_dim, o0, o1, y=None):
    qx = np.ascontiguousarray(qx, dtype=np.int8)
    sx = _f32(sx)
    sums = np.ascontiguousarray(sums, dtype=np.int32)
    w_raw = _u8(w_raw)
    if y is None:
        y = np.zeros((rows, out_dim), dtype=np.float32)
    rc = lib().afo_linear_act_range(fmt, _p(qx), _p(sx), _p(sums), _p(w_raw), _p(y), rows,
                                    in_dim, out_dim, o0, o1)
    if rc != 0:
        raise ValueError(f"afo_linear_act_range rc={rc}")
    return y


def linear_act_assoc(fmt, assoc, x, w_raw, rows, in_dim, out_dim) -> np.ndarray:
    qx, sx, _ = quantize_activation_rows(x, rows, in_dim)
    w_raw = _u8(w_raw)
    y = np.zeros((rows, out_dim), dtype=np.float32)
    rc = lib().afo_linear_act_assoc(fmt, assoc, _p(qx), _p(sx), _p(w_raw), _p(y), rows, in_dim,
                                    out_dim)
    if rc != 0:
        raise ValueError(f"afo_linear_act_assoc rc={rc}")
    return y


def linear_f32(fmt, x, w_raw, rows, in_dim, out_dim) -> np.ndarray:
    x, w_raw = _f32(x), _u8(w_raw)
    y = np.zeros((rows, out_dim), dtype=np.float32)
    rc = lib().afo_linear_f32(fmt, _p(x), _p(w_raw), _p(y), rows, in_dim, out_dim)
    if rc != 0:
        raise ValueError(f"afo_linear_f32 rc={rc}")
    return y


def linear_no_bias(fmt, x, w_raw, rows, in_dim, out_dim, workers=1) -> np.ndarray:
    """The reference engine's CPU op (route chosen by the reference gate)."""
    x, w_raw = _f32(x), _u8(w_raw)
    y = np.zeros((rows, out_dim), dtype=np.float32)
    rc = lib().afo_linear_no_bias(fmt, _p(x), _p(w_raw), _p(y), rows, in_dim, out_dim, workers)
    if rc != 0:
        raise ValueError(f"afo_linear_no_bias rc={rc}")
    return y


def add_linear_bias_rows(y, bias, rows, out_dim) -> np.ndarray:
    """y[r][o] + bias[o] in f32 (a new array)."""
    out = np.array(_f32(y), dtype=np.float32).reshape(rows, out_dim).copy()
    bias = _f32(bias)
    assert bias.size == out_dim
    lib().afo_add_linear_bias_rows(_p(out), _p(bias), rows, out_dim)
    return out


def linear(fmt, x, w_raw, bias, rows, in_dim, out_dim, workers=1) -> np.ndarray:
    """The engine's biased `linear` on a quantized weight: the no-bias op, then the bias rows."""
    return add_linear_bias_rows(linear_no_bias(fmt, x, w_raw, rows, in_dim, out_dim, workers), bias, rows, out_dim)


RELU, QUICK_GELU, GELU = 1, 2, 3


def apply_activation(kind: int, y) -> np.ndarray:
    """relu / quick_gelu / tanh-form gelu of every element (a new array)."""
    out = np.array(_f32(y), dtype=np.float32).copy()
    lib().afo_apply_activation(kind, _p(out), out.size)
    return out


def linear_act_f64(fmt, x, w_raw, rows, in_dim, out_dim) -> np.ndarray:
    x, w_raw = _f32(x), _u8(w_raw)
    y = np.zeros((rows, out_dim), dtype=np.float64)
    rc = lib().afo_linear_act_f64(fmt, _p(x), _p(w_raw), _p(y), rows, in_dim, out_dim)
    if rc != 0:
        raise ValueError(f"afo_linear_act_f64 rc={rc}")
    return y


def q4k_unpack_scale_mins(scales12):
    sc = _u8(scales12)
    assert sc.size == 12
    scs, mins = np.zeros(8, np.uint8), np.zeros(8, np.uint8)
    lib().afo_q4k_unpack_scale_mins(_p(sc), _p(scs), _p(mins))
    return scs, mins


def dequantize_q4_k(raw) -> np.ndarray:
    r = _u8(raw)
    assert r.size % 144 == 0
    out = np.zeros(r.size // 144 * 256, np.float32)
    lib().afo_dequantize_q4_k(_p(r), r.size // 144, _p(out))
    return out


def quantize_q4_k(w) -> np.ndarray:
    """f32 [.., 256 n] -> raw Q4_K super-blocks (the reference's weight quantizer)."""
    w = _f32(w).reshape(-1, 256)
    out = np.zeros((w.shape[0], 144), dtype=np.uint8)
    for i in range(w.shape[0]):
        lib().afo_quantize_q4_k_block(_p(w[i]), _p(out[i]))
    return out.reshape(-1)


def uses_q4k_q8k_activation(rows, in_dim, out_dim) -> bool:
    return bool(lib().afo_uses_q4k_q8k_activation(rows, in_dim, out_dim))


def quantize_q8_k(x):
    """(q int8 [n], d f32 [n / 256], bsums int16 [n / 16]) of a flat f32 array of whole 256-blocks."""
    xx = _f32(x)
    assert xx.size % 256 == 0
    nb = xx.size // 256
    q, d, bs = np.zeros(nb * 256, np.int8), np.zeros(nb, np.float32), np.zeros(nb * 16, np.int16)
    lib().afo_quantize_q8_k(_p(xx), nb, _p(q), _p(d), _p(bs))
    return q, d, bs


def linear_q4_k_q8k(x, w_raw, rows, in_dim, out_dim) -> np.ndarray:
    xx, w = _f32(x), _u8(w_raw)
    assert xx.size == rows * in_dim and w.size == out_dim * (in_dim // 256) * 144
    y = np.zeros((rows, out_dim), np.float32)
    if lib().afo_linear_q4_k_q8k(_p(xx), _p(w), _p(y), rows, in_dim, out_dim) != 0:
        raise ValueError("InvalidQuantizedLinearShape")
    return y


def linear_q4_k(x, w_raw, rows, in_dim, out_dim, f64=False) -> np.ndarray:
    xx, w = _f32(x), _u8(w_raw)
    assert xx.size == rows * in_dim and w.size == out_dim * (in_dim // 256) * 144
    y = np.zeros((rows, out_dim), np.float64 if f64 else np.float32)
    rc = (lib().afo_linear_q4_k_f64 if f64 else lib().afo_linear_q4_k)(_p(xx), _p(w), _p(y), rows, in_dim, out_dim)
    if rc != 0:
        raise ValueError("InvalidQuantizedLinearShape")
    return y


def argmax(data) -> int:
    d = _f32(data).reshape(-1)
    return int(lib().afo_argmax(_p(d), d.size))


def argmax_last_row(data, rows: int, dim: int) -> int:
    """Token id of the last row; ValueError for an empty shape (error.InvalidTensorShape)."""
    d = _f32(data).reshape(-1)
    assert d.size == rows * dim
    r = lib().afo_argmax_last_row(_p(d), rows, dim)
    if r < 0:
        raise ValueError("InvalidTensorShape")
    return int(r)


def thread_plan(rows, in_dim, out_dim, max_workers=8, cpu_count=8):
    cs = C.c_int(0)
    n = lib().afo_thread_plan(rows, in_dim, out_dim, max_workers, cpu_count, C.addressof(cs))
    return int(n), bool(cs.value)


class Prepared:
    """Unpacked weights for the timed CPU baseline."""

    def __init__(self, fmt, w_raw, out_dim, in_dim):
        w_raw = _u8(w_raw)
        self.out_dim, self.in_dim = out_dim, in_dim
        self.h = lib().afo_prepare(fmt, _p(w_raw), out_dim, in_dim)
        if not self.h:
            raise ValueError("afo_prepare failed")

    def linear(self, x, rows, workers=1, y=None) -> np.ndarray:
        x = _f32(x)
        if y is None:
            y = np.zeros((rows, self.out_dim), dtype=np.float32)
        rc = lib().afo_linear_prepared(self.h, _p(x), _p(y), rows, workers)
        assert rc == 0
        return y

    def close(self):
        if self.h:
            lib().afo_prepared_free(self.h)
            self.h = None

    def __del__(self):
        self.close()
