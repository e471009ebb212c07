"""`HipCompute`: the backend object behind the engine's ComputeBackend op
interface, mirroring ops/cuda/cuda_compute.zig of the reference (method names
and error behaviour follow the vtable entries on the quantized-linear path:
linearNoBias ops/ops.zig:890, linearNoBiasPlanned :895, fromFloat32, toFloat32,
getWeight, freeTensor).  All work happens behind the C ABI."""
from __future__ import annotations

import ctypes as C

import numpy as np

from . import _lib, quant_matmul
from ._lib import check


class HipTensor:
    """Opaque tensor handle (CT).  Borrowed handles (weights) are not freed."""

    def __init__(self, handle: int, borrowed: bool = False):
        self.handle = handle
        self.borrowed = borrowed

    @property
    def dtype(self) -> int:
        return _lib.lib().afhip_tensor_dtype(self.handle)

    @property
    def quant_type(self):
        q = _lib.lib().afhip_tensor_quant_type(self.handle)
        return None if q < 0 else q

    @property
    def layout(self) -> int:
        return _lib.lib().afhip_tensor_layout(self.handle)

    @property
    def elem_count(self) -> int:
        return _lib.lib().afhip_tensor_elem_count(self.handle)

    @property
    def shape(self):
        n = _lib.lib().afhip_tensor_rank(self.handle)
        out = (C.c_int64 * max(n, 1))()
        check(_lib.lib().afhip_tensor_shape(self.handle, out, n))
        return [int(out[i]) for i in range(n)]

    @property
    def device_ptr(self) -> int:
        return _lib.lib().afhip_tensor_device_ptr(self.handle)

    @property
    def byte_len(self) -> int:
        return _lib.lib().afhip_tensor_byte_len(self.handle)


class HipCompute:
    def __init__(self):
        h = C.c_void_p()
        check(_lib.lib().afhip_compute_create(C.byref(h)))
        self._h = h

    # -- lifecycle -----------------------------------------------------
    def deinit(self) -> None:
        if self._h:
            _lib.lib().afhip_compute_destroy(self._h)
            self._h = None

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.deinit()

    def __del__(self):
        try:
            self.deinit()
        except Exception:
            pass

    def backendKind(self) -> str:
        return "hip" if _lib.lib().afhip_compute_backend_kind(self._h) == 1 else "unknown"

    @property
    def stream(self) -> int:
        return _lib.lib().afhip_compute_stream(self._h) or 0

    def synchronize(self) -> None:
        check(_lib.lib().afhip_compute_synchronize(self._h))

    def deviceName(self) -> str:
        buf = C.create_string_buffer(256)
        check(_lib.lib().afhip_compute_device_name(self._h, buf, 256))
        return buf.value.decode()

    # -- weights ---------------------------------------------------------
    def insertWeightFromLoaded(self, key: str, tensor_type: int, raw_bytes, shape, keep_raw_layout: bool = False) -> None:
        raw = np.ascontiguousarray(raw_bytes, dtype=np.uint8)
        shp = (C.c_int64 * max(len(shape), 1))(*shape)
        check(_lib.lib().afhip_compute_insert_weight_from_loaded(self._h, key.encode(), tensor_type, raw.ctypes.data,
                                                                 raw.size, shp, len(shape), int(keep_raw_layout)))

    def insertWeightFromTensor(self, key: str, data, shape) -> None:
        arr = np.ascontiguousarray(data, dtype=np.float32)
        shp = (C.c_int64 * max(len(shape), 1))(*shape)
        check(_lib.lib().afhip_compute_insert_weight_f32(self._h, key.encode(), arr.ctypes.data, shp, len(shape)))

    def insertWeightFromGguf(self, file, tensor_name: str, key: str = None, keep_raw_layout: bool = False) -> None:
        """One tensor of an open gguf.File becomes a resident weight (models/tensor_store.zig:370-392)."""
        check(_lib.lib().afhip_compute_insert_weight_from_gguf(self._h, file.handle, tensor_name.encode(),
                                                               key.encode() if key is not None else None,
                                                               int(keep_raw_layout)))

    def loadGguf(self, file, keep_raw_layout: bool = False):
        """Every F32 / Q4_0 / Q8_0 tensor of the file, under its own name; returns (loaded, skipped)."""
        loaded, skipped = C.c_size_t(), C.c_size_t()
        check(_lib.lib().afhip_compute_load_gguf(self._h, file.handle, int(keep_raw_layout), C.byref(loaded),
                                                 C.byref(skipped)))
        return int(loaded.value), int(skipped.value)

    def getWeight(self, name: str) -> HipTensor:
        h = C.c_void_p()
        check(_lib.lib().afhip_compute_get_weight(self._h, name.encode(), C.byref(h)))
        return HipTensor(h.value, borrowed=True)

    # -- tensors ---------------------------------------------------------
    def fromFloat32(self, data, shape=None) -> HipTensor:
        arr = np.ascontiguousarray(data, dtype=np.float32)
        if shape is None:
            shape = [arr.size]
        shp = (C.c_int32 * max(len(shape), 1))(*shape)
        h = C.c_void_p()
        check(_lib.lib().afhip_compute_from_float32(self._h, arr.ctypes.data, arr.size, shp, len(shape), C.byref(h)))
        return HipTensor(h.value)

    def wrapDeviceFloat32(self, device_ptr: int, shape) -> HipTensor:
        shp = (C.c_int64 * max(len(shape), 1))(*shape)
        h = C.c_void_p()
        check(_lib.lib().afhip_compute_wrap_device_f32(self._h, device_ptr, shp, len(shape), C.byref(h)))
        return HipTensor(h.value)

    def toFloat32(self, tensor: HipTensor) -> np.ndarray:
        out = np.empty(tensor.elem_count, dtype=np.float32)
        check(_lib.lib().afhip_compute_to_float32(self._h, tensor.handle, out.ctypes.data, out.size))
        return out

    def evalTensor(self, tensor: HipTensor) -> None:
        check(_lib.lib().afhip_compute_eval_tensor(self._h, tensor.handle))

    def freeTensor(self, tensor: HipTensor) -> None:
        if tensor is not None and tensor.handle:
            _lib.lib().afhip_compute_free_tensor(self._h, tensor.handle)
            if not tensor.borrowed:
                tensor.handle = None

    free = freeTensor

    def embeddingLookup(self, weight: HipTensor, ids, total: int, dim: int) -> HipTensor:
        """ops/ops.zig:824, :1673: weight[ids[i]] for each i as f32 [total, dim] (f32, Q4_0 or Q8_0 table)."""
        arr = np.ascontiguousarray(ids, dtype=np.int64)
        h = C.c_void_p()
        check(_lib.lib().afhip_compute_embedding_lookup(self._h, weight.handle,
                                                        arr.ctypes.data_as(C.POINTER(C.c_int64)), arr.size, total, dim,
                                                        C.byref(h)))
        return HipTensor(h.value)

    # -- the op ------------------------------------------------------------
    def linearNoBias(self, input: HipTensor, weight: HipTensor, rows: int, in_dim: int, out_dim: int) -> HipTensor:
        h = C.c_void_p()
        check(_lib.lib().afhip_compute_linear_no_bias(self._h, input.handle, weight.handle, rows, in_dim, out_dim,
                                                      C.byref(h)))
        return HipTensor(h.value)

    def linearNoBiasPair(self, input: HipTensor, weight_a: HipTensor, weight_b: HipTensor, rows: int, in_dim: int,
                         out_dim: int):
        """ops/ops.zig:909, :1828-1849: (first, second) = (X @ Wa^T, X @ Wb^T)."""
        ha, hb = C.c_void_p(), C.c_void_p()
        check(_lib.lib().afhip_compute_linear_no_bias_pair(self._h, input.handle, weight_a.handle, weight_b.handle, rows,
                                                           in_dim, out_dim, C.byref(ha), C.byref(hb)))
        return HipTensor(ha.value), HipTensor(hb.value)

    def linear(self, input: HipTensor, weight: HipTensor, bias: HipTensor, rows: int, in_dim: int,
               out_dim: int) -> HipTensor:
        """ops/ops.zig:1728: Y = X @ W^T + bias, bias an f32 tensor of out_dim elements."""
        h = C.c_void_p()
        check(_lib.lib().afhip_compute_linear(self._h, input.handle, weight.handle, bias.handle, rows, in_dim, out_dim,
                                              C.byref(h)))
        return HipTensor(h.value)

    def _linear_activation(self, activation, input, weight, bias, rows, in_dim, out_dim):
        h = C.c_void_p()
        rc = _lib.lib().afhip_compute_linear_activation(self._h, input.handle, weight.handle, bias.handle, activation, rows,
                                                        in_dim, out_dim, C.byref(h))
        if rc == _lib.ERR_OP_UNSUPPORTED:
            return None  # the engine's optional fast path: the caller composes linear + activation
        check(rc)
        return HipTensor(h.value)

    def linearRelu(self, input: HipTensor, weight: HipTensor, bias: HipTensor, rows: int, in_dim: int, out_dim: int):
        """ops/ops.zig:2177: relu(X @ W^T + bias), or None when this weight has no fused path."""
        return self._linear_activation(_lib.ACTIVATION_RELU, input, weight, bias, rows, in_dim, out_dim)

    def linearQuickGelu(self, input: HipTensor, weight: HipTensor, bias: HipTensor, rows: int, in_dim: int, out_dim: int):
        """ops/ops.zig:2164: y / (1 + exp(-1.702 y)) of y = X @ W^T + bias, or None."""
        return self._linear_activation(_lib.ACTIVATION_QUICK_GELU, input, weight, bias, rows, in_dim, out_dim)

    def linearGelu(self, input: HipTensor, weight: HipTensor, bias: HipTensor, rows: int, in_dim: int, out_dim: int):
        """ops/ops.zig:2205: tanh-form gelu of X @ W^T + bias, or None."""
        return self._linear_activation(_lib.ACTIVATION_GELU, input, weight, bias, rows, in_dim, out_dim)

    def linearAdd(self, input: HipTensor, weight: HipTensor, bias: HipTensor, residual: HipTensor, rows: int, in_dim: int,
                  out_dim: int):
        """ops/ops.zig:2218: X @ W^T + bias + residual, or None when this weight has no fused path."""
        h = C.c_void_p()
        rc = _lib.lib().afhip_compute_linear_add(self._h, input.handle, weight.handle, bias.handle, residual.handle, rows,
                                                 in_dim, out_dim, C.byref(h))
        if rc == _lib.ERR_OP_UNSUPPORTED:
            return None
        check(rc)
        return HipTensor(h.value)

    def linearPair(self, input: HipTensor, weight_a: HipTensor, bias_a: HipTensor, weight_b: HipTensor,
                   bias_b: HipTensor, rows: int, in_dim: int, out_dim: int):
        """ops/ops.zig:915, :1846-1885: (first, second) = (X @ Wa^T + ba, X @ Wb^T + bb)."""
        ha, hb = C.c_void_p(), C.c_void_p()
        check(_lib.lib().afhip_compute_linear_pair(self._h, input.handle, weight_a.handle, bias_a.handle, weight_b.handle,
                                                   bias_b.handle, rows, in_dim, out_dim, C.byref(ha), C.byref(hb)))
        return HipTensor(ha.value), HipTensor(hb.value)

    def linearTriple(self, input: HipTensor, weight_a: HipTensor, bias_a: HipTensor, weight_b: HipTensor,
                     bias_b: HipTensor, weight_c: HipTensor, bias_c: HipTensor, rows: int, in_dim: int, out_dim: int):
        """ops/ops.zig:921, :1887-1910: the three biased Q/K/V projections of one input."""
        ha, hb, hc = C.c_void_p(), C.c_void_p(), C.c_void_p()
        check(_lib.lib().afhip_compute_linear_triple(self._h, input.handle, weight_a.handle, bias_a.handle,
                                                     weight_b.handle, bias_b.handle, weight_c.handle, bias_c.handle, rows,
                                                     in_dim, out_dim, C.byref(ha), C.byref(hb), C.byref(hc)))
        return HipTensor(ha.value), HipTensor(hb.value), HipTensor(hc.value)

    def linearNoBiasGrouped(self, input: HipTensor, weight: HipTensor, rows: int, in_dim: int, out_dim: int,
                            projection_out_dims, num_projections: int) -> HipTensor:
        """ops/ops.zig:901, :1786-1800: `weight` is the concatenation of the projections along the output axis."""
        dims = (C.c_uint32 * max(len(projection_out_dims), 1))(*projection_out_dims)
        if num_projections > len(projection_out_dims):
            raise _lib.InvalidShape(_lib.ERR_INVALID_SHAPE)
        h = C.c_void_p()
        check(_lib.lib().afhip_compute_linear_no_bias_grouped(self._h, input.handle, weight.handle, rows, in_dim,
                                                              out_dim, dims, num_projections, C.byref(h)))
        return HipTensor(h.value)

    def argmaxLastRow(self, tensor: HipTensor, rows: int, dim: int) -> int:
        """ops/ops.zig:1282, :2551: token id from the last row of a [rows, dim] tensor."""
        token = C.c_uint32()
        check(_lib.lib().afhip_compute_argmax_last_row(self._h, tensor.handle, rows, dim, C.byref(token)))
        return int(token.value)

    def linearNoBiasArgmaxLastRow(self, input: HipTensor, weight: HipTensor, rows: int, in_dim: int, out_dim: int) -> int:
        """ops/ops.zig:1292, :2565: argmax(input @ weight^T) for the last input row."""
        token = C.c_uint32()
        check(_lib.lib().afhip_compute_linear_no_bias_argmax_last_row(self._h, input.handle, weight.handle, rows, in_dim,
                                                                      out_dim, C.byref(token)))
        return int(token.value)

    def linearNoBiasArgmaxLastRowTensor(self, input: HipTensor, weight: HipTensor, rows: int, in_dim: int,
                                        out_dim: int) -> HipTensor:
        """ops/ops.zig:1297, :2572: the token id as an f32 [1] backend tensor."""
        h = C.c_void_p()
        check(_lib.lib().afhip_compute_linear_no_bias_argmax_last_row_tensor(self._h, input.handle, weight.handle, rows,
                                                                             in_dim, out_dim, C.byref(h)))
        return HipTensor(h.value)

    def linearNoBiasPlanned(self, input: HipTensor, weight: HipTensor, rows: int, in_dim: int, out_dim: int,
                            operator_plan: "quant_matmul.OperatorPlan") -> HipTensor:
        req = _lib.PlannedRequest(input.handle, weight.handle, rows, in_dim, out_dim, operator_plan.to_c())
        h = C.c_void_p()
        check(_lib.lib().afhip_compute_linear_no_bias_planned(self._h, C.byref(req), C.byref(h)))
        return HipTensor(h.value)

    def linearNoBiasWithPlan(self, input, weight, rows, in_dim, out_dim, op_plan=None) -> HipTensor:
        """ops/ops.zig:1762-1784: planned op when a plan is given, eager op otherwise."""
        if op_plan is not None:
            return self.linearNoBiasPlanned(input, weight, rows, in_dim, out_dim, op_plan)
        return self.linearNoBias(input, weight, rows, in_dim, out_dim)

    # -- counters ------------------------------------------------------------
    def setPhaseTiming(self, enabled: bool) -> None:
        """Opt-in device time per phase (activation quantizer / compute) in debugStats(); every
        linear op then waits for its own events, so this is for debugging runs only."""
        check(_lib.lib().afhip_compute_set_phase_timing(self._h, 1 if enabled else 0))

    def setQ4KF32Activations(self, enabled: bool) -> None:
        """Q4_K linear ops with f32 activations on every shape (the engine's CUDA backend,
        ops/cuda/cuda_compute.zig:708) instead of following the CPU engine onto its Q8_K route."""
        check(_lib.lib().afhip_compute_set_q4k_f32_activations(self._h, 1 if enabled else 0))

    def debugStats(self) -> dict:
        s = _lib.DebugStats()
        check(_lib.lib().afhip_compute_debug_stats(self._h, C.byref(s)))
        return {name: int(getattr(s, name)) for name, _ in s._fields_}
