"""Stream-ordered kernel launchers on raw device pointers, mirroring the
launcher half of ops/cuda/kernels.zig (launchLinearQ8_0F32 :1221-1254,
launchLinearQ4_0F32 :1256-1289) of the reference."""
from __future__ import annotations

from . import _lib
from ._lib import Buffer, check

NO_BUFFER = Buffer(0, 0)


def workspaceBytes(tensor_type: int, rows: int, in_dim: int, out_dim: int) -> int:
    return _lib.lib().afhip_linear_workspace_bytes(tensor_type, rows, in_dim, out_dim)


def launchLinearF32(stream, tensor_type, layout, dst: Buffer, input: Buffer, weight: Buffer, rows, in_dim, out_dim,
                    workspace: Buffer = NO_BUFFER, dispatch: int = -1) -> None:
    check(_lib.lib().afhip_launch_linear_f32(stream, tensor_type, layout, dst, input, weight, rows, in_dim, out_dim,
                                             workspace, dispatch))


STATIC_SCRATCH_BYTES = 16 << 20


def staticScratchInit() -> None:
    check(_lib.lib().afhip_static_scratch_init())


def launchLinearF32Static(stream, tensor_type, layout, dst: Buffer, input: Buffer, weight: Buffer, rows, in_dim, out_dim,
                          dispatch: int = -1) -> None:
    """launchLinearF32 without a workspace argument and without any allocation: the scratch is
    a device array inside the library (one per GPU, shared by all calls on it)."""
    check(_lib.lib().afhip_launch_linear_f32_static(stream, tensor_type, layout, dst, input, weight, rows, in_dim,
                                                    out_dim, dispatch))


def launchLinearPairF32(stream, tensor_type, layout, dst_a: Buffer, dst_b: Buffer, input: Buffer, weight_a: Buffer,
                        weight_b: Buffer, rows, in_dim, out_dim, workspace: Buffer = NO_BUFFER,
                        dispatch: int = -1) -> None:
    """Two matmuls of one shape that share X (gate + up): X is quantized once."""
    check(_lib.lib().afhip_launch_linear_pair_f32(stream, tensor_type, layout, dst_a, dst_b, input, weight_a, weight_b,
                                                  rows, in_dim, out_dim, workspace, dispatch))


def launchLinearBiasF32(stream, tensor_type, layout, dst: Buffer, input: Buffer, weight: Buffer, bias: Buffer, rows, in_dim,
                        out_dim, workspace: Buffer = NO_BUFFER, dispatch: int = -1) -> None:
    """Y = X @ W^T + bias (f32 [out_dim]), the bias added by the kernel that writes Y."""
    check(_lib.lib().afhip_launch_linear_bias_f32(stream, tensor_type, layout, dst, input, weight, bias, rows, in_dim,
                                                  out_dim, workspace, dispatch))


def launchLinearEpilogueF32(stream, tensor_type, layout, dst: Buffer, input: Buffer, weight: Buffer, rows, in_dim, out_dim,
                            bias: Buffer = NO_BUFFER, residual: Buffer = NO_BUFFER, activation: int = 0,
                            workspace: Buffer = NO_BUFFER, dispatch: int = -1) -> None:
    """Y = act(X @ W^T + bias) + residual, all by the kernel that writes Y (bias, residual optional)."""
    check(_lib.lib().afhip_launch_linear_epilogue_f32(stream, tensor_type, layout, dst, input, weight, bias, residual,
                                                      activation, rows, in_dim, out_dim, workspace, dispatch))


def launchLinearPairBiasF32(stream, tensor_type, layout, dst_a: Buffer, dst_b: Buffer, input: Buffer, weight_a: Buffer,
                            bias_a: Buffer, weight_b: Buffer, bias_b: Buffer, rows, in_dim, out_dim,
                            workspace: Buffer = NO_BUFFER, dispatch: int = -1) -> None:
    """Two biased matmuls of one shape that share X."""
    check(_lib.lib().afhip_launch_linear_pair_bias_f32(stream, tensor_type, layout, dst_a, dst_b, input, weight_a, bias_a,
                                                       weight_b, bias_b, rows, in_dim, out_dim, workspace, dispatch))


def launchLinearQ8_0F32(stream, dst: Buffer, input: Buffer, weight_raw: Buffer, rows, in_dim, out_dim,
                        workspace: Buffer = NO_BUFFER) -> None:
    check(_lib.lib().afhip_launch_linear_q8_0_f32(stream, dst, input, weight_raw, rows, in_dim, out_dim, workspace))


def launchLinearQ4_0F32(stream, dst: Buffer, input: Buffer, weight_raw: Buffer, rows, in_dim, out_dim,
                        workspace: Buffer = NO_BUFFER) -> None:
    check(_lib.lib().afhip_launch_linear_q4_0_f32(stream, dst, input, weight_raw, rows, in_dim, out_dim, workspace))


def weightLayoutBytes(tensor_type, layout, out_dim, in_dim) -> int:
    """Size of a [out_dim, in_dim] weight in a device layout (raw or prepared)."""
    return int(_lib.lib().afhip_weight_layout_bytes(tensor_type, layout, out_dim, in_dim))


def preparedWeightBytes(tensor_type, out_dim, in_dim) -> int:
    """Size of the PREPARED layout (Q4_K pads out_dim to whole 32-column tiles)."""
    return int(_lib.lib().afhip_prepared_weight_bytes(tensor_type, out_dim, in_dim))


def launchPrepareWeight(stream, tensor_type, dst_prepared: Buffer, src_raw: Buffer, out_dim, in_dim) -> None:
    check(_lib.lib().afhip_launch_prepare_weight(stream, tensor_type, dst_prepared, src_raw, out_dim, in_dim))


def launchQuantizeActivations(stream, input: Buffer, rows, in_dim, q: Buffer, scales: Buffer,
                              sums: Buffer = NO_BUFFER) -> None:
    check(_lib.lib().afhip_launch_quantize_activations(stream, input, rows, in_dim, q, scales, sums))


def launchBlockDots(stream, tensor_type, layout, dots: Buffer, input: Buffer, weight: Buffer, rows, in_dim, out_dim,
                    workspace: Buffer = NO_BUFFER, dispatch: int = -1) -> None:
    check(_lib.lib().afhip_launch_block_dots(stream, tensor_type, layout, dots, input, weight, rows, in_dim, out_dim,
                                             workspace, dispatch))


def argmaxWorkspaceBytes(dim: int) -> int:
    return _lib.lib().afhip_argmax_workspace_bytes(dim)


def launchArgmaxLastRowF32(stream, token_u32: Buffer, token_f32: Buffer, input: Buffer, rows, dim,
                           workspace: Buffer = NO_BUFFER) -> None:
    """Token id of the last row of f32 [rows, dim]: as u32 and / or as f32 (either buffer may be NO_BUFFER).
    With a workspace of argmaxWorkspaceBytes(dim) a long row is scanned by many workgroups."""
    check(_lib.lib().afhip_launch_argmax_last_row_f32(stream, token_u32, token_f32, input, rows, dim, workspace))


def linearArgmaxWorkspaceBytes(tensor_type: int, in_dim: int, out_dim: int) -> int:
    return _lib.lib().afhip_linear_argmax_workspace_bytes(tensor_type, in_dim, out_dim)


def launchLinearArgmaxLastRowF32(stream, tensor_type, layout, token_u32: Buffer, token_f32: Buffer, input: Buffer,
                                 weight: Buffer, rows, in_dim, out_dim, workspace: Buffer) -> None:
    """argmax(X[rows-1] @ W^T) without the logits matrix (lm_head of a greedy decode step)."""
    check(_lib.lib().afhip_launch_linear_argmax_last_row_f32(stream, tensor_type, layout, token_u32, token_f32, input,
                                                             weight, rows, in_dim, out_dim, workspace))


def launchEmbeddingLookupF32(stream, tensor_type, layout, dst: Buffer, weight: Buffer, ids_i64: Buffer, total, dim,
                             vocab) -> None:
    """get_rows: dst f32 [total, dim] = dequantized rows ids[t] of a [vocab, dim] table (ids: int64 on the device)."""
    check(_lib.lib().afhip_launch_embedding_lookup_f32(stream, tensor_type, layout, dst, weight, ids_i64, total, dim,
                                                       vocab))


def launchDequantizeF32(stream, tensor_type, layout, dst: Buffer, weight: Buffer, rows, dim) -> None:
    """cpy_q_to_f32: the whole [rows, dim] tensor as f32."""
    check(_lib.lib().afhip_launch_dequantize_f32(stream, tensor_type, layout, dst, weight, rows, dim))


def launchQuantizeRows(stream, tensor_type, dst_raw: Buffer, input: Buffer, rows, dim, row_ids_i64: Buffer = NO_BUFFER,
                       dst_rows=None) -> None:
    """cpy_f32_to_q (no ids) / set_rows (row t of input -> row ids[t] of the destination): f32 -> raw GGUF blocks."""
    check(_lib.lib().afhip_launch_quantize_rows(stream, tensor_type, dst_raw, input, row_ids_i64, rows, dim,
                                                rows if dst_rows is None else dst_rows))


def launchDecodeFp16(stream, dst_f32: Buffer, src_u16: Buffer, n: int) -> None:
    check(_lib.lib().afhip_launch_decode_fp16(stream, dst_f32, src_u16, n))


def launchStreamRead(stream, src: Buffer, sink: Buffer) -> None:
    check(_lib.lib().afhip_launch_stream_read(stream, src, sink))


def launchStreamCopy(stream, src: Buffer, dst: Buffer) -> None:
    check(_lib.lib().afhip_launch_stream_copy(stream, src, dst))


def smokeQ8_0() -> None:
    check(_lib.lib().afhip_smoke_q8_0())


def smokeQ4_0() -> None:
    check(_lib.lib().afhip_smoke_q4_0())
