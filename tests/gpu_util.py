"""Helpers for the GPU tests: torch is only the allocator and the stream."""
import numpy as np
import torch

from antfly_amd import _lib, kernels
from antfly_amd._lib import Buffer

DEV = "cuda:0"


def buf(t: torch.Tensor) -> Buffer:
    return Buffer(t.data_ptr(), t.numel() * t.element_size())


def stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def to_dev(a: np.ndarray) -> torch.Tensor:
    return torch.from_numpy(np.ascontiguousarray(a)).to(DEV)


def prepare(fmt: int, w_raw: np.ndarray, out_dim: int, in_dim: int) -> torch.Tensor:
    raw = to_dev(w_raw)
    prepared = torch.empty(kernels.preparedWeightBytes(fmt, out_dim, in_dim), dtype=torch.uint8, device=DEV)
    kernels.launchPrepareWeight(stream(), fmt, buf(prepared), buf(raw), out_dim, in_dim)
    torch.cuda.synchronize()
    return prepared


def numpy_prepare(fmt: int, w_raw: np.ndarray, out_dim: int, in_dim: int) -> np.ndarray:
    """The PREPARED layout of a Q4_0 / Q8_0 weight: quant bytes of every block, the fp16 scales in
    block order, zero padding to 16 bytes, then the scales once more in wavefront-tile order (one
    tile = the columns of one GEMV wavefront x 128 blocks; 64 lane entries of 8 / 4 halves; entries
    of blocks or columns past the matrix are zero)."""
    q4 = fmt == _lib.TYPE_Q4_0
    bb = 18 if q4 else 34
    kb = in_dim // 32
    blocks = np.asarray(w_raw, np.uint8).reshape(out_dim * kb, bb)
    scales = blocks[:, :2].copy().view(np.uint16).reshape(out_dim, kb)
    cols, per_lane = (4, 8) if q4 else (2, 4)
    groups, slices = (out_dim + cols - 1) // cols, (kb + 127) // 128
    tiles = np.zeros((groups, slices, 64, per_lane), np.uint16)
    o, k = np.meshgrid(np.arange(out_dim), np.arange(kb), indexing="ij")
    ks = k % 128
    if q4:
        lane, inner = ks % 64, (ks // 64) * 4 + o % 4
    else:
        step = ks // 32
        lane, inner = (ks % 32) * 2 + (step >> 1), (step & 1) * 2 + o % 2
    tiles[o // cols, k // 128, lane, inner] = scales
    head = np.concatenate([blocks[:, 2:].reshape(-1), blocks[:, :2].reshape(-1)])
    pad = np.zeros((-head.size) % 16, np.uint8)
    return np.concatenate([head, pad, tiles.reshape(-1).view(np.uint8)])


def numpy_prepare_q4k(w_raw: np.ndarray, out_dim: int, in_dim: int) -> np.ndarray:
    """The tile-major Q4_K layout: per tile of 32 columns and super-block, 32 headers of 16 bytes, then for
    each 32-byte chunk of nibbles lane c + 32 g holds bytes 16 g .. 16 g + 15 of column c; columns past
    out_dim are zero."""
    kb = in_dim // 256
    tiles = (out_dim + 31) // 32
    blocks = np.zeros((tiles * 32, kb, 144), np.uint8)
    blocks[:out_dim] = np.asarray(w_raw, np.uint8).reshape(out_dim, kb, 144)
    blocks = blocks.reshape(tiles, 32, kb, 144).transpose(0, 2, 1, 3)          # [tile][sb][c][144]
    headers = blocks[..., :16].reshape(tiles, kb, 512)
    quants = blocks[..., 16:].reshape(tiles, kb, 32, 4, 2, 16).transpose(0, 1, 3, 4, 2, 5)  # [tile][sb][chunk][g][c][16]
    return np.concatenate([headers, quants.reshape(tiles, kb, 4096)], axis=2).reshape(-1)


def linear(fmt, layout, x: np.ndarray, w_dev: torch.Tensor, rows, in_dim, out_dim, dispatch=-1) -> np.ndarray:
    xd = to_dev(x.astype(np.float32))
    y = torch.full((rows, out_dim), float("nan"), dtype=torch.float32, device=DEV)
    ws_bytes = kernels.workspaceBytes(fmt, rows, in_dim, out_dim)
    ws = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device=DEV)
    kernels.launchLinearF32(stream(), fmt, layout, buf(y), buf(xd), buf(w_dev), rows, in_dim, out_dim, buf(ws), dispatch)
    torch.cuda.synchronize()
    return y.cpu().numpy()


def linear_pair(fmt, layout, x: np.ndarray, wa_dev: torch.Tensor, wb_dev: torch.Tensor, rows, in_dim, out_dim, dispatch=-1):
    xd = to_dev(x.astype(np.float32))
    ya = torch.full((rows, out_dim), float("nan"), dtype=torch.float32, device=DEV)
    yb = torch.full((rows, out_dim), float("nan"), dtype=torch.float32, device=DEV)
    ws_bytes = kernels.workspaceBytes(fmt, rows, in_dim, out_dim)
    ws = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device=DEV)
    kernels.launchLinearPairF32(stream(), fmt, layout, buf(ya), buf(yb), buf(xd), buf(wa_dev), buf(wb_dev), rows, in_dim,
                                out_dim, buf(ws), dispatch)
    torch.cuda.synchronize()
    return ya.cpu().numpy(), yb.cpu().numpy()


def linear_bias(fmt, layout, x: np.ndarray, w_dev: torch.Tensor, bias: np.ndarray, rows, in_dim, out_dim,
                dispatch=-1) -> np.ndarray:
    xd, bd = to_dev(x.astype(np.float32)), to_dev(bias.astype(np.float32))
    y = torch.full((rows, out_dim), float("nan"), dtype=torch.float32, device=DEV)
    ws = torch.empty(max(kernels.workspaceBytes(fmt, rows, in_dim, out_dim), 16), dtype=torch.uint8, device=DEV)
    kernels.launchLinearBiasF32(stream(), fmt, layout, buf(y), buf(xd), buf(w_dev), buf(bd), rows, in_dim, out_dim,
                                buf(ws), dispatch)
    torch.cuda.synchronize()
    return y.cpu().numpy()


def linear_pair_bias(fmt, layout, x: np.ndarray, wa_dev, ba: np.ndarray, wb_dev, bb: np.ndarray, rows, in_dim, out_dim,
                     dispatch=-1):
    xd, bad, bbd = to_dev(x.astype(np.float32)), to_dev(ba.astype(np.float32)), to_dev(bb.astype(np.float32))
    ya = torch.full((rows, out_dim), float("nan"), dtype=torch.float32, device=DEV)
    yb = torch.full((rows, out_dim), float("nan"), dtype=torch.float32, device=DEV)
    ws = torch.empty(max(kernels.workspaceBytes(fmt, rows, in_dim, out_dim), 16), dtype=torch.uint8, device=DEV)
    kernels.launchLinearPairBiasF32(stream(), fmt, layout, buf(ya), buf(yb), buf(xd), buf(wa_dev), buf(bad), buf(wb_dev),
                                    buf(bbd), rows, in_dim, out_dim, buf(ws), dispatch)
    torch.cuda.synchronize()
    return ya.cpu().numpy(), yb.cpu().numpy()


def block_dots(fmt, layout, x: np.ndarray, w_dev: torch.Tensor, rows, in_dim, out_dim, dispatch=-1) -> np.ndarray:
    xd = to_dev(x.astype(np.float32))
    d = torch.full((rows, out_dim, in_dim // 32), -(2 ** 31), dtype=torch.int32, device=DEV)
    ws_bytes = kernels.workspaceBytes(fmt, rows, in_dim, out_dim)
    ws = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device=DEV)
    kernels.launchBlockDots(stream(), fmt, layout, buf(d), buf(xd), buf(w_dev), rows, in_dim, out_dim, buf(ws), dispatch)
    torch.cuda.synchronize()
    return d.cpu().numpy()


def max_rel_err(got: np.ndarray, want: np.ndarray) -> float:
    """Largest |got - want| relative to the largest |want| of the same output row.

    The gate is normalised by the row maximum, not element by element: an output is a sum of
    in_dim/32 signed terms, so an element near zero is the difference of large partial sums and
    its own magnitude says nothing about the rounding error it carries."""
    scale = np.abs(want).max(axis=-1, keepdims=True)
    scale = np.where(scale == 0, 1.0, scale)
    return float((np.abs(got.astype(np.float64) - want) / scale).max())


def elementwise_rel_err(got: np.ndarray, want: np.ndarray, floor: float = 1e-3) -> float:
    """Largest |got - want| / |want| over the outputs whose |want| is above `floor` times the
    largest |want| of their row (reported next to the row-normalised figure, for information)."""
    want = np.asarray(want, np.float64)
    scale = np.abs(want).max(axis=-1, keepdims=True)
    keep = np.abs(want) > floor * np.where(scale == 0, 1.0, scale)
    if not keep.any():
        return 0.0
    err = np.abs(got.astype(np.float64) - want)
    return float((err[keep] / np.abs(want[keep])).max())
