"""Host-side packing of weights into the library's interchange layout (NumPy).

Layout: element k of row n is the field at bit (k % (32/bits)) * bits of word
k // (32/bits), least-significant field first; one float16 scale per `group`
consecutive k.  q4f16 uses the symmetric zero point 7, q8f16 none.
"""
from __future__ import annotations

import numpy as np


def pack_q4(w: np.ndarray) -> np.ndarray:
    """Integers 0..15 of shape [N, K] -> uint32 [N, K/8]."""
    w = np.asarray(w)
    n, k = w.shape
    if k % 8:
        raise ValueError("K must be a multiple of 8")
    if w.size and (w.min() < 0 or w.max() > 15):
        raise ValueError("int4 fields must lie in 0..15")
    f = w.astype(np.uint32).reshape(n, k // 8, 8)
    shifts = (4 * np.arange(8, dtype=np.uint32))[None, None, :]
    return np.bitwise_or.reduce(f << shifts, axis=2).astype(np.uint32)


def pack_q8(w: np.ndarray) -> np.ndarray:
    """Integers -128..127 of shape [N, K] -> uint32 [N, K/4] (two's-complement bytes)."""
    w = np.asarray(w)
    n, k = w.shape
    if k % 4:
        raise ValueError("K must be a multiple of 4")
    if w.size and (w.min() < -128 or w.max() > 127):
        raise ValueError("int8 fields must lie in -128..127")
    f = (w.astype(np.int64) & 0xFF).astype(np.uint32).reshape(n, k // 4, 4)
    shifts = (8 * np.arange(4, dtype=np.uint32))[None, None, :]
    return np.bitwise_or.reduce(f << shifts, axis=2).astype(np.uint32)


def quantize_q4f16(w: np.ndarray, group: int = 32):
    """Float weights [N, K] -> (wq uint32 [N, K/8], scales float16 [N, K/group]), zero point 7."""
    w = np.asarray(w, dtype=np.float32)
    n, k = w.shape
    if k % group:
        raise ValueError("K must be a multiple of the group size")
    g = w.reshape(n, k // group, group)
    amax = np.abs(g).max(axis=2)
    scales = np.maximum(amax / 7.0, 1e-8).astype(np.float16)
    q = np.clip(np.rint(g / scales.astype(np.float32)[:, :, None]) + 7, 0, 15).astype(np.int64)
    return pack_q4(q.reshape(n, k)), scales


def quantize_q8f16(w: np.ndarray, group: int = 128):
    """Float weights [N, K] -> (wq uint32 [N, K/4], scales float16 [N, K/group])."""
    w = np.asarray(w, dtype=np.float32)
    n, k = w.shape
    if k % group:
        raise ValueError("K must be a multiple of the group size")
    g = w.reshape(n, k // group, group)
    amax = np.abs(g).max(axis=2)
    scales = np.maximum(amax / 127.0, 1e-8).astype(np.float16)
    q = np.clip(np.rint(g / scales.astype(np.float32)[:, :, None]), -127, 127).astype(np.int64)
    return pack_q8(q.reshape(n, k)), scales
