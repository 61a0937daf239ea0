"""Input generators restated from the reference's own tests, and error metrics."""
from __future__ import annotations

import numpy as np

from onnx_genai_amd import synth


def rel_l2(x, ref) -> float:
    x = np.asarray(x, np.float64).ravel()
    ref = np.asarray(ref, np.float64).ravel()
    d = np.linalg.norm(ref)
    return float(np.linalg.norm(x - ref) / d) if d else float(np.linalg.norm(x))


def max_rel_to_peak(x, ref) -> float:
    """max |x - ref| / max |ref| — the error measure of matmul_nbits.rs:11045-11068."""
    ref = np.asarray(ref, np.float64)
    return float(np.abs(np.asarray(x, np.float64) - ref).max() / np.abs(ref).max())


def quantize_blockwise(weights_nk: np.ndarray, bs: int, asymmetric: bool):
    """The reference tests' block quantizer (matmul_nbits.rs:11447-11491, mlas-sys/src/lib.rs quantize_int4).

    -> packed B [N, kb, bs/2], f32 scales [N, kb], packed zero points or None, dequantized f32 [N, K]."""
    w = np.asarray(weights_nk, np.float32)
    n, k = w.shape
    kb = -(-k // bs)
    q_all = np.zeros((n, kb, bs), np.uint8)
    scales = np.zeros((n, kb), np.float32)
    zps = np.full((n, kb), 8, np.uint8)
    deq = np.zeros((n, k), np.float32)
    for blk in range(kb):
        lo, hi = blk * bs, min((blk + 1) * bs, k)
        v = w[:, lo:hi]
        if asymmetric:
            mn, mx = v.min(axis=1), v.max(axis=1)
            s = np.maximum(((mx - mn) / np.float32(15.0)).astype(np.float32), np.float32(1e-6))
            z = np.clip(_round_half_away((-mn / s).astype(np.float32)), 0, 15).astype(np.uint8)
        else:
            s = np.maximum((np.abs(v).max(axis=1) / np.float32(7.0)).astype(np.float32), np.float32(1e-6))
            z = np.full(n, 8, np.uint8)
        q = np.clip(_round_half_away((v / s[:, None] + z[:, None].astype(np.float32)).astype(np.float32)), 0, 15).astype(np.uint8)
        q_all[:, blk, : hi - lo] = q
        scales[:, blk] = s
        zps[:, blk] = z
        deq[:, lo:hi] = (q.astype(np.float32) - z[:, None].astype(np.float32)) * s[:, None]
    packed = synth.pack_nibbles(q_all)
    zp_packed = synth.pack_nibbles(zps) if asymmetric else None
    return packed, scales, zp_packed, deq


def _round_half_away(x):
    return np.sign(x) * np.floor(np.abs(x) + np.float32(0.5))


def envelope_fixture():
    """matmul_nbits.rs:10986-10997: K=1024, N=128, block 32, asymmetric."""
    k, n, bs = 1024, 128, 32
    i = np.arange(n * k, dtype=np.uint64)
    weights = (((i * np.uint64(2654435761)) % np.uint64(1000)).astype(np.float32) / np.float32(500.0) - np.float32(1.0)).reshape(n, k)
    j = np.arange(k, dtype=np.uint64)
    act = (((j * np.uint64(40503)) % np.uint64(1000)).astype(np.float32) / np.float32(500.0) - np.float32(1.0)).reshape(1, k)
    return k, n, bs, weights, act


def sqnbit_fixture(m, n, k):
    """mlas-sys/src/lib.rs:3027-3036 (check_sqnbit): trig-formula weights, activations and bias."""
    i = np.arange(n * k, dtype=np.float32)
    weights = np.sin(i * np.float32(0.017) + np.float32(0.3)).astype(np.float32).reshape(n, k)
    j = np.arange(m * k, dtype=np.float32)
    a = (np.cos(j * np.float32(0.011) + np.float32(0.7)) * np.float32(0.5)).astype(np.float32).reshape(m, k)
    bias = np.sin(np.arange(n, dtype=np.float32) * np.float32(0.03)).astype(np.float32)
    return weights, a, bias
