"""Seeded synthetic inputs for the quantized-matmul benchmarks and parity tests.

Everything derives from one counter-based generator (SplitMix64 over the element
index), so the CPU checker and the GPU harness see the same bits whatever order
or chunking they are produced in.

Shapes and distributions follow the benchmark definition:
  x          f32 [M, K] ~ N(0, 1)
  Q8_0 W     32 int8 uniform in [-127, 127] per block, scale fp16(|N(0, 0.02)| / 127)
  Q4_0 W     16 bytes of two uniform nibbles 0..15 (value = nibble - 8, low nibbles
             are elements 0..15 and high nibbles 16..31), scale fp16(|N(0, 0.02)| / 7)
  Q4_K W     144-byte super-blocks of 256 weights: d = fp16(|N(0, 0.02)| / 240),
             dmin = fp16(|N(0, 0.02)| / 64), 12 uniform bytes of packed 6-bit scales and
             mins, 128 uniform bytes of nibbles
Block layouts are GGUF's: [fp16 scale, little endian][quants], 34 / 18 bytes.
"""
from __future__ import annotations

import numpy as np

Q4_0 = 2  # GGUF tensor-type ids
Q8_0 = 8
Q4_K = 12
BLOCK_VALUES = 32
BLOCK_BYTES = {Q4_0: 18, Q8_0: 34}
Q4_K_BLOCK_VALUES, Q4_K_BLOCK_BYTES = 256, 144

_GOLDEN = np.uint64(0x9E3779B97F4A7C15)
_M1 = np.uint64(0xBF58476D1CE4E5B9)
_M2 = np.uint64(0x94D049BB133111EB)


def splitmix64(seed: int, start: int, count: int) -> np.ndarray:
    """count 64-bit outputs for counters start .. start+count-1 of stream `seed`."""
    with np.errstate(over="ignore"):
        idx = np.arange(start + 1, start + count + 1, dtype=np.uint64)
        z = np.uint64(seed & 0xFFFFFFFFFFFFFFFF) + idx * _GOLDEN
        z = (z ^ (z >> np.uint64(30))) * _M1
        z = (z ^ (z >> np.uint64(27))) * _M2
        return z ^ (z >> np.uint64(31))


def uniform01(seed: int, start: int, count: int) -> np.ndarray:
    """float64 uniform in (0, 1), 53 bits."""
    return ((splitmix64(seed, start, count) >> np.uint64(11)).astype(np.float64) + 0.5) * (1.0 / (1 << 53))


def normal(seed: int, count: int) -> np.ndarray:
    """float64 standard normal via Box-Muller on counters (2i, 2i+1)."""
    u = uniform01(seed, 0, 2 * count)
    r = np.sqrt(-2.0 * np.log(u[0::2]))
    return r * np.cos(2.0 * np.pi * u[1::2])


def activations(seed: int, rows: int, in_dim: int) -> np.ndarray:
    return normal(seed, rows * in_dim).astype(np.float32).reshape(rows, in_dim)


def weights_q4_k(seed: int, out_dim: int, in_dim: int) -> np.ndarray:
    """Raw GGUF Q4_K bytes for W[out_dim, in_dim], flat uint8."""
    if in_dim % Q4_K_BLOCK_VALUES:
        raise ValueError("in_dim must be a multiple of 256")
    nb = out_dim * (in_dim // Q4_K_BLOCK_VALUES)
    out = np.empty((nb, Q4_K_BLOCK_BYTES), dtype=np.uint8)
    d = (np.abs(normal(seed ^ 0x5CA1E, nb)) * 0.02 / 240.0).astype(np.float16)
    dmin = (np.abs(normal(seed ^ 0xD317, nb)) * 0.02 / 64.0).astype(np.float16)
    out[:, 0:2] = d.view(np.uint8).reshape(nb, 2)
    out[:, 2:4] = dmin.view(np.uint8).reshape(nb, 2)
    raw = splitmix64(seed, 0, nb * 18)  # 140 of the 144 random bytes per block are used
    out[:, 4:] = raw.view(np.uint8).reshape(nb, 144)[:, :140]
    return out.reshape(-1)


def weights(fmt: int, seed: int, out_dim: int, in_dim: int) -> np.ndarray:
    """Raw GGUF block bytes for W[out_dim, in_dim], flat uint8."""
    if fmt == Q4_K:
        return weights_q4_k(seed, out_dim, in_dim)
    if in_dim % BLOCK_VALUES:
        raise ValueError("in_dim must be a multiple of 32")
    nb = out_dim * (in_dim // BLOCK_VALUES)
    bb = BLOCK_BYTES[fmt]
    out = np.empty((nb, bb), dtype=np.uint8)
    div = 127.0 if fmt == Q8_0 else 7.0
    scale = (np.abs(normal(seed ^ 0x5CA1E, nb)) * 0.02 / div).astype(np.float16)
    out[:, 0:2] = scale.view(np.uint8).reshape(nb, 2)  # little endian host
    if fmt == Q8_0:
        raw = splitmix64(seed, 0, nb * 32)
        q = (raw % np.uint64(255)).astype(np.int16) - 127
        out[:, 2:] = q.astype(np.int8).view(np.uint8).reshape(nb, 32)
    else:
        raw = splitmix64(seed, 0, nb * 2)  # 16 random bytes per block
        out[:, 2:] = raw.view(np.uint8).reshape(nb, 16)
    return out.reshape(-1)


def weight_bytes(fmt: int, out_dim: int, in_dim: int) -> int:
    return out_dim * (in_dim // BLOCK_VALUES) * BLOCK_BYTES[fmt]
