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


def launchLinearPairF32(stream, tensor_type, layout, dst_a: Buffer, dst_b: Buffer, input: Buffer, weight_a: Buffer,
                        weight_b: Buffer, rows, in_dim, out_dim, workspace: Buffer = NO_BUFFER,
                        dispatch: int = -1) -> None:
    """Two matmuls of one shape that share X (gate + up): X is quantized once."""
    check(_lib.lib().afhip_launch_linear_pair_f32(stream, tensor_type, layout, dst_a, dst_b, input, weight_a, weight_b,
                                                  rows, in_dim, out_dim, workspace, dispatch))


def launchLinearQ8_0F32(stream, dst: Buffer, input: Buffer, weight_raw: Buffer, rows, in_dim, out_dim,
                        workspace: Buffer = NO_BUFFER) -> None:
    check(_lib.lib().afhip_launch_linear_q8_0_f32(stream, dst, input, weight_raw, rows, in_dim, out_dim, workspace))


def launchLinearQ4_0F32(stream, dst: Buffer, input: Buffer, weight_raw: Buffer, rows, in_dim, out_dim,
                        workspace: Buffer = NO_BUFFER) -> None:
    check(_lib.lib().afhip_launch_linear_q4_0_f32(stream, dst, input, weight_raw, rows, in_dim, out_dim, workspace))


def launchPrepareWeight(stream, tensor_type, dst_prepared: Buffer, src_raw: Buffer, out_dim, in_dim) -> None:
    check(_lib.lib().afhip_launch_prepare_weight(stream, tensor_type, dst_prepared, src_raw, out_dim, in_dim))


def launchQuantizeActivations(stream, input: Buffer, rows, in_dim, q: Buffer, scales: Buffer,
                              sums: Buffer = NO_BUFFER) -> None:
    check(_lib.lib().afhip_launch_quantize_activations(stream, input, rows, in_dim, q, scales, sums))


def launchBlockDots(stream, tensor_type, layout, dots: Buffer, input: Buffer, weight: Buffer, rows, in_dim, out_dim,
                    workspace: Buffer = NO_BUFFER, dispatch: int = -1) -> None:
    check(_lib.lib().afhip_launch_block_dots(stream, tensor_type, layout, dots, input, weight, rows, in_dim, out_dim,
                                             workspace, dispatch))


def launchDecodeFp16(stream, dst_f32: Buffer, src_u16: Buffer, n: int) -> None:
    check(_lib.lib().afhip_launch_decode_fp16(stream, dst_f32, src_u16, n))


def launchStreamRead(stream, src: Buffer, sink: Buffer) -> None:
    check(_lib.lib().afhip_launch_stream_read(stream, src, sink))


def smokeQ8_0() -> None:
    check(_lib.lib().afhip_smoke_q8_0())


def smokeQ4_0() -> None:
    check(_lib.lib().afhip_smoke_q4_0())
