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


def _unit_bits(seed: int, start: int, count: int) -> np.ndarray:
    """The top 53 bits of `count` stream elements from `start`, as uint64."""
    with np.errstate(over="ignore"):
        z = np.arange(start + 1, start + count + 1, dtype=np.uint64)
        z *= _GAMMA
        z += np.uint64(seed)
        t = z >> np.uint64(30)
        z ^= t
        z *= _M1
        np.right_shift(z, np.uint64(27), out=t)
        z ^= t
        z *= _M2
        np.right_shift(z, np.uint64(31), out=t)
        z ^= t
        z >>= np.uint64(11)
    return z


def _unit(seed: int, start: int, count: int) -> np.ndarray:
    """Doubles in [0, 1) with 53 random bits."""
    u = _unit_bits(seed, start, count).astype(np.float64)
    u *= 1.0 / 9007199254740992.0
    return u


_CHUNK = 1 << 20            # elements per work item; even, so normal() pairs never straddle chunks


def _fill(out: np.ndarray, fn) -> np.ndarray:
    """out[s:s+c] = fn(s, c) over chunks, on a few threads (numpy releases the
    GIL inside its loops); the result does not depend on the thread count."""
    count = out.shape[0]
    starts = range(0, count, _CHUNK)

    def work(s):
        c = min(_CHUNK, count - s)
        out[s:s + c] = fn(s, c)

    if count <= 4 * _CHUNK:
        for s in starts:
            work(s)
    else:
        from concurrent.futures import ThreadPoolExecutor
        import os
        with ThreadPoolExecutor(max_workers=min(8, os.cpu_count() or 1)) as pool:
            list(pool.map(work, starts))
    return out


def uniform(seed: int, count: int, dtype=np.float64) -> np.ndarray:
    """count values i.i.d. uniform on [-1, 1)."""
    def fn(s, c):
        u = _unit(seed, s, c)
        u *= 2.0
        u -= 1.0
        return u
    return _fill(np.empty(count, dtype=dtype), fn)


def normal(seed: int, count: int, dtype=np.float32) -> np.ndarray:
    """count values i.i.d. N(0, 1) by Box-Muller: elements 2p and 2p+1 come
    from stream elements 2p (radius) and 2p+1 (angle)."""
    def fn(s, c):                       # s is even
        half = (c + 1) // 2
        u = _unit(seed, s, 2 * half)
        r = np.sqrt(-2.0 * np.log(1.0 - u[0::2]))      # 1-u in (0, 1]
        phi = (2.0 * np.pi) * u[1::2]
        z = np.empty(2 * half, dtype=np.float64)
        z[0::2] = r * np.cos(phi)
        z[1::2] = r * np.sin(phi)
        return z[:c]
    return _fill(np.empty(count, dtype=dtype), fn)


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


# ---------------------------------------------------------------------------
# The same streams generated where the benchmark needs them: in device memory.
# ---------------------------------------------------------------------------
def _device_unit(seed: int, start: int, count: int):
    """_unit on the current torch device.  int64 arithmetic wraps like uint64;
    the logical right shifts are arithmetic shifts with the sign bits masked."""
    import torch
    def i64(x):         # a 64-bit pattern as the int64 that has it
        x &= (1 << 64) - 1
        return x - (1 << 64) if x >= (1 << 63) else x

    def lsr(z, s):
        return torch.bitwise_and(torch.bitwise_right_shift(z, s), (1 << (64 - s)) - 1)

    z = torch.arange(start + 1, start + count + 1, dtype=torch.int64, device="cuda")
    z *= i64(int(_GAMMA))
    z += i64(seed)
    z ^= lsr(z, 30)
    z *= i64(int(_M1))
    z ^= lsr(z, 27)
    z *= i64(int(_M2))
    z ^= lsr(z, 31)
    z = lsr(z, 11)
    u = z.to(torch.float64)
    u *= 1.0 / 9007199254740992.0
    return u


def device_matrix(seed: int, rows: int, cols: int, ld: int | None = None, dist: str = "uniform", dtype=np.float64,
                  sentinel: float | None = None):
    """matrix() as a torch tensor on the current device, with the memory image
    of the column-major (ld x cols) window (shape (cols, ld), contiguous),
    generated there.  Uniform values are bit-identical to matrix()'s; normal
    values go through the device's log / sqrt / cos / sin and may differ from
    the host's in the last place."""
    import torch
    ld = rows if ld is None else ld
    if ld < max(1, rows):
        raise ValueError("ld < rows")
    tdt = torch.float64 if np.dtype(dtype) == np.float64 else torch.float32
    out = torch.full((cols, ld), -2560000000.0 if sentinel is None else sentinel, dtype=tdt, device="cuda")
    per = max(1, (1 << 25) // max(1, rows))                  # columns per pass: 32M elements of temporaries
    per += per % 2 if rows % 2 else 0                        # normal(): pairs (2p, 2p+1) never straddle passes
    for c0 in range(0, cols, per):
        nc = min(per, cols - c0)
        s, c = c0 * rows, nc * rows
        if dist == "uniform":
            v = _device_unit(seed, s, c)
            v *= 2.0
            v -= 1.0
        else:
            half = (c + 1) // 2
            u = _device_unit(seed, s, 2 * half)
            r = torch.sqrt(-2.0 * torch.log(1.0 - u[0::2]))
            phi = (2.0 * np.pi) * u[1::2]
            v = torch.empty(2 * half, dtype=torch.float64, device="cuda")
            v[0::2] = r * torch.cos(phi)
            v[1::2] = r * torch.sin(phi)
            v = v[:c]
        out[c0:c0 + nc, :rows] = v.reshape(nc, rows).to(tdt)
    return out
