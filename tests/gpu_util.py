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


def numpy_prepare(fmt: int, w_raw: np.ndarray) -> np.ndarray:
    bb = 18 if fmt == _lib.TYPE_Q4_0 else 34
    blocks = np.asarray(w_raw, np.uint8).reshape(-1, bb)
    return np.concatenate([blocks[:, 2:].reshape(-1), blocks[:, :2].reshape(-1)])


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
    """Largest |got - want| relative to the largest |want| of the same output row."""
    scale = np.abs(want).max(axis=-1, keepdims=True)
    scale = np.where(scale == 0, 1.0, scale)
    return float((np.abs(got.astype(np.float64) - want) / scale).max())
