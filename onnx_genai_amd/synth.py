"""Seeded synthetic MatMulNBits operands, shared by the parity tests and the benchmark.

Layouts are the ORT contrib-op ones: B uint8 [N, kb, bs/2] with the low nibble holding the
even element, scales [N, kb] in the activation dtype (or f32), zero points uint8
[N, ceil(kb/2)] packed the same way (absent = 8).
"""
from __future__ import annotations

import numpy as np

F32, U8, I32, F16, BF16 = 1, 2, 6, 10, 16
ITEMSIZE = {F32: 4, F16: 2, BF16: 2, U8: 1, I32: 4}


def f32_to_bf16_bits(x: np.ndarray) -> np.ndarray:
    """Round-to-nearest-even f32 -> bf16, returned as uint16 bit patterns."""
    u = np.ascontiguousarray(x, np.float32).view(np.uint32)
    nan = (u & 0x7FFFFFFF) > 0x7F800000
    r = ((u >> 16) & 1) + 0x7FFF
    out = ((u + r) >> 16).astype(np.uint16)
    out[nan] = ((u[nan] >> 16) | 0x40).astype(np.uint16)
    return out


def bf16_bits_to_f32(x: np.ndarray) -> np.ndarray:
    return (np.ascontiguousarray(x, np.uint16).astype(np.uint32) << 16).view(np.float32)


def to_dtype(x: np.ndarray, code: int) -> np.ndarray:
    """f32 array -> storage array of dtype `code` (bf16 as uint16 bits)."""
    if code == F32:
        return np.ascontiguousarray(x, np.float32)
    if code == F16:
        return np.ascontiguousarray(x, np.float32).astype(np.float16)
    if code == BF16:
        return f32_to_bf16_bits(x)
    raise ValueError(code)


def to_f32(x: np.ndarray, code: int) -> np.ndarray:
    if code == BF16:
        return bf16_bits_to_f32(x)
    return np.asarray(x).astype(np.float32)


def pack_nibbles(q: np.ndarray) -> np.ndarray:
    """[..., 2j] values in 0..15 -> [..., j] bytes, even element in the low nibble."""
    q = np.asarray(q, np.uint8)
    if q.shape[-1] % 2:
        q = np.concatenate([q, np.zeros(q.shape[:-1] + (1,), np.uint8)], axis=-1)
    return (q[..., 0::2] | (q[..., 1::2] << 4)).astype(np.uint8)


def unpack_nibbles(p: np.ndarray, count: int) -> np.ndarray:
    p = np.asarray(p, np.uint8)
    out = np.empty(p.shape[:-1] + (p.shape[-1] * 2,), np.uint8)
    out[..., 0::2] = p & 0x0F
    out[..., 1::2] = p >> 4
    return out[..., :count]


def make_weights(n, k, bs, seed, *, zero_points: bool, scale_lo: float, scale_hi: float, scale_dtype: int):
    """Random nibbles, uniform scales in [lo, hi] rounded to `scale_dtype`, optional random zero points."""
    rng = np.random.default_rng(seed)
    kb = -(-k // bs)
    q = rng.integers(0, 16, size=(n, kb, bs), dtype=np.uint8)
    b = pack_nibbles(q)
    scales = to_dtype(rng.uniform(scale_lo, scale_hi, size=(n, kb)).astype(np.float32), scale_dtype)
    zp = None
    if zero_points:
        zq = rng.integers(0, 16, size=(n, kb), dtype=np.uint8)
        zp = pack_nibbles(zq)
    return b, scales, zp


def make_weights_bits(n, k, bs, bits, seed, *, zero_points: bool, scale_lo: float, scale_hi: float, scale_dtype: int):
    """The same for 2- or 8-bit weights: random bytes are uniform fields of any width; zero points packed alike."""
    rng = np.random.default_rng(seed)
    kb = -(-k // bs)
    b = rng.integers(0, 256, size=(n, kb, bs * bits // 8), dtype=np.uint8)
    scales = to_dtype(rng.uniform(scale_lo, scale_hi, size=(n, kb)).astype(np.float32), scale_dtype)
    zp = rng.integers(0, 256, size=(n, -(-kb * bits // 8)), dtype=np.uint8) if zero_points else None
    return b, scales, zp


def make_activation(m, k, seed, dtype: int, dist: str = "normal"):
    rng = np.random.default_rng(seed + 7919)
    a = rng.standard_normal((m, k)).astype(np.float32) if dist == "normal" else rng.uniform(-1, 1, (m, k)).astype(np.float32)
    return to_dtype(a, dtype)


def algorithmic_bytes(m, n, k, bs, *, a_dtype: int, scale_dtype: int, zero_points: bool, y_dtype: int | None = None) -> int:
    """Bytes one call must move: packed B + scales + zero points + A + Y."""
    kb = -(-k // bs)
    y_dtype = a_dtype if y_dtype is None else y_dtype
    total = n * kb * (bs // 2) + n * kb * ITEMSIZE[scale_dtype]
    if zero_points:
        total += n * (-(-kb // 2))
    return total + m * k * ITEMSIZE[a_dtype] + m * n * ITEMSIZE[y_dtype]


def matmul_flops(m, n, k) -> int:
    return 2 * m * n * k
