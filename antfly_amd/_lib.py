"""Loads libantfly_hip_qmatmul.so and declares its C ABI (include/antfly_hip_qmatmul.h).

There is no fallback: if the library is missing, import fails loudly.
"""
from __future__ import annotations

import ctypes as C
import os

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(PKG_DIR, "lib", "libantfly_hip_qmatmul.so")

# enum afhip_error
OK = 0
ERR_INVALID_STATE = -1
ERR_UNSUPPORTED_TENSOR_TYPE = -2
ERR_INVALID_SHAPE = -3
ERR_WEIGHT_NOT_FOUND = -4
ERR_OP_UNSUPPORTED = -5
ERR_INVALID_PARTITION_PLAN = -6
ERR_UNAVAILABLE = -7
ERR_NO_DEVICES = -8
ERR_OUT_OF_MEMORY = -9
ERR_INVALID_ARGUMENT = -10
ERR_SMOKE_MISMATCH = -11
ERR_INVALID_TOKEN_ID = -12
ERR_GGUF_INVALID_MAGIC = -13
ERR_GGUF_UNEXPECTED_EOF = -14
ERR_GGUF_UNSUPPORTED_METADATA = -15
ERR_GGUF_NESTED_ARRAY = -16
ERR_TENSOR_NOT_FOUND = -17
ERR_IO = -18

TYPE_F32, TYPE_Q4_0, TYPE_Q8_0, TYPE_Q4_K = 0, 2, 8, 12
ACTIVATION_NONE, ACTIVATION_RELU, ACTIVATION_QUICK_GELU, ACTIVATION_GELU = 0, 1, 2, 3
LAYOUT_RAW, LAYOUT_PREPARED = 0, 1
# a launcher's `dispatch` besides a kind (0 .. 3): choose by rows; ... and keep Q4_K on f32 activations everywhere
DISPATCH_AUTO, DISPATCH_AUTO_F32_ACTIVATIONS = -1, -2
DTYPE_F32, DTYPE_U8 = 0, 1


class Buffer(C.Structure):
    """afhip_buffer: a device allocation (ptr, len)."""

    _fields_ = [("ptr", C.c_uint64), ("len", C.c_size_t)]


class QuantPlan(C.Structure):
    _fields_ = [
        ("dispatch", C.c_uint8),
        ("primitive", C.c_uint8),
        ("op", C.c_uint8),
        ("row_bucket", C.c_uint8),
        ("format", C.c_uint16),
        ("rows", C.c_size_t),
        ("in_dim", C.c_size_t),
        ("out_dim", C.c_size_t),
    ]


class OperatorPlan(C.Structure):
    _fields_ = [("kind", C.c_int), ("quant_matmul", QuantPlan)]


class PlannedRequest(C.Structure):
    _fields_ = [
        ("input", C.c_void_p),
        ("weight", C.c_void_p),
        ("rows", C.c_size_t),
        ("in_dim", C.c_size_t),
        ("out_dim", C.c_size_t),
        ("operator_plan", OperatorPlan),
    ]


class DebugStats(C.Structure):
    _fields_ = [(n, C.c_uint64) for n in (
        "h2d_bytes", "d2h_bytes", "resident_weight_bytes", "pooled_buffers", "device_allocs",
        "launches_mmv", "launches_small_batch", "launches_mm", "launches_f32_route",
        "launches_activation_quant", "launches_prepare", "scratch_bytes",
        "activation_quant_ns", "compute_ns", "timed_ops")]


GGUF_MAX_DIMS = 8


class GgufSummary(C.Structure):
    _fields_ = [("version", C.c_uint32), ("tensor_count", C.c_uint64), ("metadata_count", C.c_uint64),
                ("alignment", C.c_uint64), ("data_region_offset", C.c_uint64), ("file_len", C.c_uint64)]


class GgufTensorInfo(C.Structure):
    _fields_ = [("name", C.c_void_p), ("name_len", C.c_size_t), ("n_dimensions", C.c_uint32),
                ("dimensions", C.c_uint64 * GGUF_MAX_DIMS), ("tensor_type", C.c_uint32), ("type_name", C.c_char_p),
                ("is_quantized", C.c_int), ("offset", C.c_uint64), ("data_offset", C.c_uint64),
                ("byte_len", C.c_uint64)]


class GgufMetadata(C.Structure):
    _fields_ = [("key", C.c_void_p), ("key_len", C.c_size_t), ("value_type", C.c_uint32),
                ("element_type", C.c_uint32), ("count", C.c_uint64), ("u64", C.c_uint64), ("i64", C.c_int64),
                ("f64", C.c_double), ("str", C.c_void_p), ("str_len", C.c_size_t)]


# name -> (restype, argtypes); the loader test checks every one is exported.
_sz, _vp, _i, _st = C.c_size_t, C.c_void_p, C.c_int, C.c_int
SIGNATURES = {
    "afhip_status_string": (C.c_char_p, [_st]),
    "afhip_quant_matmul_select": (_i, [_sz, _sz, _sz, _i]),
    "afhip_quant_matmul_plan": (None, [_sz, _sz, _sz, _i, C.POINTER(QuantPlan)]),
    "afhip_quant_row_bucket": (_i, [_sz]),
    "afhip_quant_format_from_tensor_type": (_i, [_i]),
    "afhip_uses_activation_quant": (_i, [_sz, _sz, _sz]),
    "afhip_uses_q8k_activation_quant": (_i, [_i, _sz, _sz, _sz]),
    "afhip_linear_workspace_bytes": (_sz, [_i, _sz, _sz, _sz]),
    "afhip_launch_linear_f32": (_st, [_vp, _i, _i, Buffer, Buffer, Buffer, _sz, _sz, _sz, Buffer, _i]),
    "afhip_launch_gemv_probe": (_st, [_vp, _i, Buffer, Buffer, Buffer, _sz, _sz]),
    "afhip_launch_gemv_probe_rows": (_st, [_vp, _i, _sz, Buffer, Buffer, Buffer, _sz, _sz]),
    "afhip_launch_gemv_timeline": (_st, [_vp, _sz, Buffer, Buffer, Buffer, _sz, _sz, C.POINTER(_sz), C.POINTER(_sz)]),
    "afhip_launch_rows8_timeline": (_st, [_vp, _sz, Buffer, Buffer, Buffer, _sz, _sz, Buffer, C.POINTER(_sz), C.POINTER(_sz)]),
    "afhip_static_scratch_init": (_st, []),
    "afhip_launch_linear_f32_static": (_st, [_vp, _i, _i, Buffer, Buffer, Buffer, _sz, _sz, _sz, _i]),
    "afhip_launch_linear_pair_f32": (_st, [_vp, _i, _i, Buffer, Buffer, Buffer, Buffer, Buffer, _sz, _sz, _sz, Buffer, _i]),
    "afhip_launch_linear_bias_f32": (_st, [_vp, _i, _i, Buffer, Buffer, Buffer, Buffer, _sz, _sz, _sz, Buffer, _i]),
    "afhip_launch_linear_epilogue_f32": (_st, [_vp, _i, _i, Buffer, Buffer, Buffer, Buffer, Buffer, _i, _sz, _sz, _sz, Buffer, _i]),
    "afhip_launch_linear_pair_bias_f32": (_st, [_vp, _i, _i, Buffer, Buffer, Buffer, Buffer, Buffer, Buffer, Buffer, _sz, _sz, _sz, Buffer, _i]),
    "afhip_launch_linear_q8_0_f32": (_st, [_vp, Buffer, Buffer, Buffer, _sz, _sz, _sz, Buffer]),
    "afhip_launch_linear_q4_0_f32": (_st, [_vp, Buffer, Buffer, Buffer, _sz, _sz, _sz, Buffer]),
    "afhip_weight_layout_bytes": (_sz, [_i, _i, _sz, _sz]),
    "afhip_prepared_weight_bytes": (_sz, [_i, _sz, _sz]),
    "afhip_launch_prepare_weight": (_st, [_vp, _i, Buffer, Buffer, _sz, _sz]),
    "afhip_launch_quantize_activations": (_st, [_vp, Buffer, _sz, _sz, Buffer, Buffer, Buffer]),
    "afhip_launch_block_dots": (_st, [_vp, _i, _i, Buffer, Buffer, Buffer, _sz, _sz, _sz, Buffer, _i]),
    "afhip_argmax_workspace_bytes": (_sz, [_sz]),
    "afhip_launch_argmax_last_row_f32": (_st, [_vp, Buffer, Buffer, Buffer, _sz, _sz, Buffer]),
    "afhip_linear_argmax_workspace_bytes": (_sz, [_i, _sz, _sz]),
    "afhip_launch_linear_argmax_last_row_f32": (_st, [_vp, _i, _i, Buffer, Buffer, Buffer, Buffer, _sz, _sz, _sz, Buffer]),
    "afhip_launch_embedding_lookup_f32": (_st, [_vp, _i, _i, Buffer, Buffer, Buffer, _sz, _sz, _sz]),
    "afhip_launch_dequantize_f32": (_st, [_vp, _i, _i, Buffer, Buffer, _sz, _sz]),
    "afhip_launch_quantize_rows": (_st, [_vp, _i, Buffer, Buffer, Buffer, _sz, _sz, _sz]),
    "afhip_launch_decode_fp16": (_st, [_vp, Buffer, Buffer, _sz]),
    "afhip_launch_stream_read": (_st, [_vp, Buffer, Buffer]),
    "afhip_launch_stream_copy": (_st, [_vp, Buffer, Buffer]),
    "afhip_launch_stream_read_shaped": (_st, [_vp, Buffer, Buffer, _i, _i, _i]),
    "afhip_tune_batch32_max_workgroups": (_st, [C.c_long]),
    "afhip_launch_gemm_stamps": (_st, [_vp, Buffer, Buffer, Buffer, Buffer, _sz, _sz, _sz]),
    "afhip_launch_rate_probe": (_st, [_vp, _i, _i, _i, Buffer, Buffer]),
    "afhip_rate_probe_wavefronts": (_sz, [_i]),
    "afhip_compute_create": (_st, [C.POINTER(_vp)]),
    "afhip_compute_destroy": (None, [_vp]),
    "afhip_compute_backend_kind": (_i, [_vp]),
    "afhip_compute_stream": (_vp, [_vp]),
    "afhip_compute_synchronize": (_st, [_vp]),
    "afhip_compute_device_name": (_st, [_vp, C.c_char_p, _sz]),
    "afhip_compute_insert_weight_from_loaded": (_st, [_vp, C.c_char_p, _i, _vp, _sz, C.POINTER(C.c_int64), _sz, _i]),
    "afhip_compute_insert_weight_f32": (_st, [_vp, C.c_char_p, _vp, C.POINTER(C.c_int64), _sz]),
    "afhip_compute_get_weight": (_st, [_vp, C.c_char_p, C.POINTER(_vp)]),
    "afhip_compute_from_float32": (_st, [_vp, _vp, _sz, C.POINTER(C.c_int32), _sz, C.POINTER(_vp)]),
    "afhip_compute_to_float32": (_st, [_vp, _vp, _vp, _sz]),
    "afhip_compute_wrap_device_f32": (_st, [_vp, C.c_uint64, C.POINTER(C.c_int64), _sz, C.POINTER(_vp)]),
    "afhip_compute_free_tensor": (None, [_vp, _vp]),
    "afhip_compute_eval_tensor": (_st, [_vp, _vp]),
    "afhip_tensor_dtype": (_i, [_vp]),
    "afhip_tensor_quant_type": (_i, [_vp]),
    "afhip_tensor_layout": (_i, [_vp]),
    "afhip_tensor_elem_count": (_sz, [_vp]),
    "afhip_tensor_rank": (_sz, [_vp]),
    "afhip_tensor_shape": (_st, [_vp, C.POINTER(C.c_int64), _sz]),
    "afhip_tensor_device_ptr": (C.c_uint64, [_vp]),
    "afhip_tensor_byte_len": (_sz, [_vp]),
    "afhip_compute_embedding_lookup": (_st, [_vp, _vp, C.POINTER(C.c_int64), _sz, _sz, _sz, C.POINTER(_vp)]),
    "afhip_compute_linear_no_bias": (_st, [_vp, _vp, _vp, _sz, _sz, _sz, C.POINTER(_vp)]),
    "afhip_compute_linear_no_bias_pair": (_st, [_vp, _vp, _vp, _vp, _sz, _sz, _sz, C.POINTER(_vp), C.POINTER(_vp)]),
    "afhip_compute_linear": (_st, [_vp, _vp, _vp, _vp, _sz, _sz, _sz, C.POINTER(_vp)]),
    "afhip_compute_linear_activation": (_st, [_vp, _vp, _vp, _vp, _i, _sz, _sz, _sz, C.POINTER(_vp)]),
    "afhip_compute_linear_add": (_st, [_vp, _vp, _vp, _vp, _vp, _sz, _sz, _sz, C.POINTER(_vp)]),
    "afhip_compute_linear_pair": (_st, [_vp, _vp, _vp, _vp, _vp, _vp, _sz, _sz, _sz, C.POINTER(_vp), C.POINTER(_vp)]),
    "afhip_compute_linear_triple": (_st, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _sz, _sz, _sz, C.POINTER(_vp), C.POINTER(_vp), C.POINTER(_vp)]),
    "afhip_compute_linear_no_bias_grouped": (_st, [_vp, _vp, _vp, _sz, _sz, _sz, C.POINTER(C.c_uint32), _sz, C.POINTER(_vp)]),
    "afhip_compute_argmax_last_row": (_st, [_vp, _vp, _sz, _sz, C.POINTER(C.c_uint32)]),
    "afhip_compute_linear_no_bias_argmax_last_row": (_st, [_vp, _vp, _vp, _sz, _sz, _sz, C.POINTER(C.c_uint32)]),
    "afhip_compute_linear_no_bias_argmax_last_row_tensor": (_st, [_vp, _vp, _vp, _sz, _sz, _sz, C.POINTER(_vp)]),
    "afhip_compute_linear_no_bias_planned": (_st, [_vp, C.POINTER(PlannedRequest), C.POINTER(_vp)]),
    "afhip_gguf_parse": (_st, [_vp, _sz, C.POINTER(_vp)]),
    "afhip_gguf_open": (_st, [C.c_char_p, C.POINTER(_vp)]),
    "afhip_gguf_close": (None, [_vp]),
    "afhip_gguf_get_summary": (_st, [_vp, C.POINTER(GgufSummary)]),
    "afhip_gguf_tensor_at": (_st, [_vp, _sz, C.POINTER(GgufTensorInfo)]),
    "afhip_gguf_find_tensor": (_st, [_vp, C.c_char_p, C.POINTER(GgufTensorInfo)]),
    "afhip_gguf_tensor_data": (_st, [_vp, C.POINTER(GgufTensorInfo), C.POINTER(_vp), C.POINTER(_sz)]),
    "afhip_gguf_tensor_byte_len": (C.c_uint64, [C.c_uint32, _i, C.POINTER(C.c_uint64), _sz]),
    "afhip_gguf_metadata_at": (_st, [_vp, _sz, C.POINTER(GgufMetadata)]),
    "afhip_gguf_find_metadata": (_st, [_vp, C.c_char_p, C.POINTER(GgufMetadata)]),
    "afhip_compute_insert_weight_from_gguf": (_st, [_vp, _vp, C.c_char_p, C.c_char_p, _i]),
    "afhip_compute_load_gguf": (_st, [_vp, _vp, _i, C.POINTER(_sz), C.POINTER(_sz)]),
    "afhip_compute_debug_stats": (_st, [_vp, C.POINTER(DebugStats)]),
    "afhip_compute_set_phase_timing": (_st, [_vp, _i]),
    "afhip_compute_set_q4k_f32_activations": (_st, [_vp, _i]),
    "afhip_smoke_q8_0": (_st, []),
    "afhip_smoke_q4_0": (_st, []),
}

_lib = None


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                f"{LIB_PATH} is missing: build it with `make -C antfly_amd/csrc` "
                "(or __graft_entry__.build()); there is no CPU fallback")
        L = C.CDLL(LIB_PATH)
        for name, (restype, argtypes) in SIGNATURES.items():
            fn = getattr(L, name)  # AttributeError if the library does not export it
            fn.restype = restype
            fn.argtypes = argtypes
        _lib = L
    return _lib


class HipError(Exception):
    """An error union member of the backend (negative) or a hipError_t (positive)."""

    def __init__(self, status: int):
        self.status = status
        try:
            self.name = lib().afhip_status_string(status).decode()
        except Exception:  # pragma: no cover
            self.name = str(status)
        super().__init__(f"error.{self.name} ({status})")


class InvalidHipState(HipError):
    pass


class UnsupportedTensorType(HipError):
    pass


class InvalidShape(HipError):
    pass


class WeightNotFound(HipError):
    pass


class HipOpUnsupported(HipError):
    pass


class InvalidPartitionPlan(HipError):
    pass


class HipUnavailable(HipError):
    pass


class NoHipDevices(HipError):
    pass


class HipSmokeMismatch(HipError):
    pass


class InvalidTokenId(HipError):
    pass


class InvalidGgufMagic(HipError):
    pass


class UnexpectedEndOfFile(HipError):
    pass


class UnsupportedMetadataType(HipError):
    pass


class UnsupportedNestedMetadataArray(HipError):
    pass


class TensorNotFound(HipError):
    pass


class FileNotAccessible(HipError):
    pass


_ERRORS = {
    ERR_INVALID_STATE: InvalidHipState,
    ERR_UNSUPPORTED_TENSOR_TYPE: UnsupportedTensorType,
    ERR_INVALID_SHAPE: InvalidShape,
    ERR_WEIGHT_NOT_FOUND: WeightNotFound,
    ERR_OP_UNSUPPORTED: HipOpUnsupported,
    ERR_INVALID_PARTITION_PLAN: InvalidPartitionPlan,
    ERR_UNAVAILABLE: HipUnavailable,
    ERR_NO_DEVICES: NoHipDevices,
    ERR_SMOKE_MISMATCH: HipSmokeMismatch,
    ERR_INVALID_TOKEN_ID: InvalidTokenId,
    ERR_GGUF_INVALID_MAGIC: InvalidGgufMagic,
    ERR_GGUF_UNEXPECTED_EOF: UnexpectedEndOfFile,
    ERR_GGUF_UNSUPPORTED_METADATA: UnsupportedMetadataType,
    ERR_GGUF_NESTED_ARRAY: UnsupportedNestedMetadataArray,
    ERR_TENSOR_NOT_FOUND: TensorNotFound,
    ERR_IO: FileNotAccessible,
}


def check(status: int) -> None:
    if status != OK:
        raise _ERRORS.get(status, HipError)(status)
