"""Seeded synthetic operands for the GEMM parity tests and the benchmark.

A counter-based splitmix64 stream, so that every box generates bit-identical
matrices from (seed, shape) with vectorised numpy and no state to carry:
element number i of a stream is mix(seed + (i+1)*GAMMA).
"""
from __future__ import annotations

import numpy as np

_GAMMA = np.uint64(0x9E3779B97F4A7C15)
_M1 = np.uint64(0xBF58476D1CE4E5B9)
_M2 = np.uint64(0x94D049BB133111EB)


def _splitmix64(seed: int, start: int, count: int) -> np.ndarray:
    with np.errstate(over="ignore"):
        idx = np.arange(start + 1, start + count + 1, dtype=np.uint64)
        z = np.uint64(seed) + idx * _GAMMA
        z = (z ^ (z >> np.uint64(30))) * _M1
        z = (z ^ (z >> np.uint64(27))) * _M2
        z = z ^ (z >> np.uint64(31))
    return z


def _unit(seed: int, start: int, count: int) -> np.ndarray:
    """Doubles in [0, 1) with 53 random bits."""
    return (_splitmix64(seed, start, count) >> np.uint64(11)).astype(np.float64) * (1.0 / 9007199254740992.0)


def uniform(seed: int, count: int, dtype=np.float64, chunk: int = 1 << 24) -> np.ndarray:
    """count values i.i.d. uniform on [-1, 1)."""
    out = np.empty(count, dtype=dtype)
    for s in range(0, count, chunk):
        c = min(chunk, count - s)
        out[s:s + c] = 2.0 * _unit(seed, s, c) - 1.0
    return out


def normal(seed: int, count: int, dtype=np.float32, chunk: int = 1 << 23) -> np.ndarray:
    """count values i.i.d. N(0, 1) by Box-Muller on pairs of the stream."""
    out = np.empty(count, dtype=dtype)
    for s in range(0, count, chunk):
        c = min(chunk, count - s)
        half = (c + 1) // 2
        # pair p of the chunk starting at element s uses stream elements 2*(s/2+p), +1
        u = _unit(seed, (s // 2) * 2, 2 * half)
        u1 = 1.0 - u[0::2]            # (0, 1]
        u2 = u[1::2]
        r = np.sqrt(-2.0 * np.log(u1))
        z = np.empty(2 * half, dtype=np.float64)
        z[0::2] = r * np.cos(2.0 * np.pi * u2)
        z[1::2] = r * np.sin(2.0 * np.pi * u2)
        out[s:s + c] = z[:c]
    return out


def matrix(seed: int, rows: int, cols: int, ld: int | None = None, dist: str = "uniform", dtype=np.float64,
           sentinel: float | None = None) -> np.ndarray:
    """A column-major (ld x cols) window, Fortran-ordered, whose leading
    rows x cols part is random and whose padding rows hold `sentinel`
    (default: -2560000000.0, the gap filler of the ATLAS tester)."""
    ld = rows if ld is None else ld
    if ld < max(1, rows):
        raise ValueError("ld < rows")
    gen = uniform if dist == "uniform" else normal
    body = gen(seed, rows * cols, dtype=dtype).reshape((rows, cols), order="F")
    if ld == rows:
        return np.asfortranarray(body)
    out = np.full((ld, cols), -2560000000.0 if sentinel is None else sentinel, dtype=dtype, order="F")
    out[:rows, :] = body
    return out
