"""Seeded synthetic tensors for the benchmark configurations.

Counter-based SplitMix64: element i of stream (seed, tag) is mix(mix(seed, tag) + (i + 1) * GOLDEN),
so any slice can be generated independently and the bytes do not depend on a numpy or torch RNG
version. Uniforms use the top 24 bits (exact in f32); normals are Box-Muller in f64, rounded once.
"""
from __future__ import annotations

import zlib

import numpy as np

_GOLDEN = np.uint64(0x9E3779B97F4A7C15)
_M1 = np.uint64(0xBF58476D1CE4E5B9)
_M2 = np.uint64(0x94D049BB133111EB)


def _mix(z: np.ndarray) -> np.ndarray:
    z = (z ^ (z >> np.uint64(30))) * _M1
    z = (z ^ (z >> np.uint64(27))) * _M2
    return z ^ (z >> np.uint64(31))


def _stream_key(seed: int, tag: str) -> np.uint64:
    t = np.uint64(zlib.crc32(tag.encode()) | (len(tag) << 32))
    with np.errstate(over="ignore"):
        return _mix(np.array([np.uint64(seed) * _GOLDEN + t], dtype=np.uint64))[0]


_CHUNK = 1 << 20


def _chunks(n: int):
    return [(s, min(n, s + _CHUNK)) for s in range(0, n, _CHUNK)]


def _parallel(fn, n: int) -> None:
    """Runs fn(start, end) over 1 Mi-element chunks on a thread pool (numpy releases the GIL)."""
    import concurrent.futures
    import os

    spans = _chunks(n)
    workers = max(1, min(16, os.cpu_count() or 1, len(spans)))
    if workers == 1:
        for s, e in spans:
            fn(s, e)
        return
    with concurrent.futures.ThreadPoolExecutor(max_workers=workers) as pool:
        list(pool.map(lambda se: fn(*se), spans))


def _bits_span(key: np.uint64, s: int, e: int) -> np.ndarray:
    with np.errstate(over="ignore"):
        idx = np.arange(s + 1, e + 1, dtype=np.uint64)
        return _mix(key + idx * _GOLDEN)


def uniform(seed: int, tag: str, shape, lo: float = 0.0, hi: float = 1.0, dtype=np.float32) -> np.ndarray:
    n = int(np.prod(shape, dtype=np.int64))
    key = _stream_key(seed, tag)
    out = np.empty(n, dtype=dtype)
    f32 = np.dtype(dtype) == np.float32

    def fill(s, e):
        b = _bits_span(key, s, e)
        if f32:
            u = (b >> np.uint64(40)).astype(np.float64) * (1.0 / (1 << 24))
        else:
            u = (b >> np.uint64(11)).astype(np.float64) * (1.0 / (1 << 53))
        out[s:e] = (lo + (hi - lo) * u).astype(dtype)

    _parallel(fill, n)
    return out.reshape(shape)


def normal(seed: int, tag: str, shape, mean: float = 0.0, std: float = 1.0, dtype=np.float32) -> np.ndarray:
    """Box-Muller on the two 32-bit halves of one 64-bit draw per element."""
    n = int(np.prod(shape, dtype=np.int64))
    key = _stream_key(seed, tag)
    out = np.empty(n, dtype=dtype)

    def fill(s, e):
        b = _bits_span(key, s, e)
        u1 = ((b >> np.uint64(32)).astype(np.float64) + 1.0) * (1.0 / (1 << 32))            # (0, 1]
        u2 = (b & np.uint64(0xFFFFFFFF)).astype(np.float64) * (1.0 / (1 << 32))             # [0, 1)
        z = np.sqrt(-2.0 * np.log(u1)) * np.cos(2.0 * np.pi * u2)
        out[s:e] = (mean + std * z).astype(dtype)

    _parallel(fill, n)
    return out.reshape(shape)


def token_ids(seed: int, tag: str, shape, vocab: int) -> np.ndarray:
    """Uniform ids in [0, vocab) as f64 VALUES (indices are float-valued tensors in the reference)."""
    n = int(np.prod(shape, dtype=np.int64))
    key = _stream_key(seed, tag)
    ids = (_bits_span(key, 0, n) >> np.uint64(11)) % np.uint64(vocab)
    return ids.astype(np.float64).reshape(shape)
