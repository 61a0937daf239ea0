"""Full-size calls of the benchmark configurations against the CPU oracle on a sample of output columns (and rows).

The oracle cannot afford 152064 columns x 8192 rows, and does not need to: an output element depends only on its own
row of A and its own rows of B / scales / zero points, so the full-size call is made on the GPU and the oracle runs on
the weight rows of ~250 columns spread over N (always including the last 16: the ragged end of the grid) and, for tall
calls, on a few dozen rows of A spread over M (always including the last ones). Bars as everywhere: rel-L2 <= 5e-3 for
16-bit outputs, <= 1e-5 for accuracy_level 4 against the oracle's own integer path.
"""
import numpy as np
import pytest

import oracle
from onnx_genai_amd import ep as E
from onnx_genai_amd import synth
from tests import helpers

pytestmark = pytest.mark.gpu

TOL_F32 = 1e-5
TOL_HALF = 5e-3


def random_weights(n, k, bs, seed, zero_points, dtype, scale_lo, scale_hi):
    """Random bytes are uniform nibbles: no unpacked intermediate for tensors of hundreds of megabytes."""
    rng = np.random.default_rng(seed)
    kb = -(-k // bs)
    b = rng.integers(0, 256, size=(n, kb, bs // 2), dtype=np.uint8)
    s = synth.to_dtype(rng.uniform(scale_lo, scale_hi, size=(n, kb)).astype(np.float32), dtype)
    zp = rng.integers(0, 256, size=(n, (kb + 1) // 2), dtype=np.uint8) if zero_points else None
    return b, s, zp


def spread(count, want):
    """`want` indices spread over 0..count-1, always with the last 16."""
    idx = np.concatenate([np.linspace(0, count - 1, min(want, count)).astype(np.int64), np.arange(max(count - 16, 0), count)])
    return np.unique(idx)


def sampled_f64(port, a_f32, b, s_f32, zp, cols, k, bs, rows=None):
    """f64 product of the sampled rows of A with the dequantized sampled columns (the oracle's bit-exact dequantization, then
    a double-precision GEMM)."""
    bc, sc = np.ascontiguousarray(b[cols]), np.ascontiguousarray(s_f32[cols])
    zc = np.ascontiguousarray(zp[cols]) if zp is not None else None
    w = port.dequantize_nk(bc, sc, zc, len(cols), k, bs).astype(np.float64)
    a = a_f32 if rows is None else a_f32[rows]
    return a.astype(np.float64) @ w.T


DECODE_SHAPES = [
    # name, dtype, block, zero points, K, N, rows, scale range
    ("7b lm_head", E.BF16, 128, True, 3584, 152064, (1, 4, 8, 16), (0.002, 0.01)),
    ("7b down", E.BF16, 128, True, 18944, 3584, (1, 4, 5, 8, 16), (0.002, 0.01)),
    ("7b qkv", E.BF16, 128, True, 3584, 4608, (1, 4, 8, 9, 16), (0.002, 0.01)),
    ("7b o", E.BF16, 128, True, 3584, 3584, (1, 4, 8, 16), (0.002, 0.01)),
    ("7b gate_up", E.BF16, 128, True, 3584, 37888, (1, 4, 8, 16), (0.002, 0.01)),
    ("0.5b lm_head", E.F16, 32, True, 896, 151936, (1,), (0.002, 0.01)),
]


@pytest.mark.parametrize("name,dt,bs,zero_points,k,n,rows,scale_range", DECODE_SHAPES, ids=[s[0] for s in DECODE_SHAPES])
def test_decode_configs_at_full_size(ep, port, name, dt, bs, zero_points, k, n, rows, scale_range):
    """configs[1] and configs[2] at their real shapes, through the default dispatch over constant weights."""
    b, s, zp = random_weights(n, k, bs, 1234 + n, zero_points, dt, *scale_range)
    sf = synth.to_f32(s, dt)
    cols = spread(n, 240)
    ops = E.DeviceOperands(ep, b, s, dt, zp, n, k, bs)
    try:
        for m in rows:
            a = synth.make_activation(m, k, 77 + m, dt)
            ab, yb = ep.upload(a), ep.allocate(m * n * 2)
            try:
                ops.run(ab, dt, m, yb)
                y = synth.to_f32(ep.download(yb, (m, n), np.uint16 if dt == E.BF16 else np.float16), dt)
            finally:
                ep.deallocate(ab)
                ep.deallocate(yb)
            want = sampled_f64(port, synth.to_f32(a, dt), b, sf, zp, cols, k, bs)
            assert ops.kernel.last_variant().startswith("decode_mfma"), ops.kernel.last_variant()
            assert np.isfinite(y).all()
            assert helpers.rel_l2(y[:, cols], want) <= TOL_HALF, (name, m)
    finally:
        ops.free()


PREFILL_SHAPES = [(4096, 14336, 512), (14336, 4096, 512), (4096, 14336, 2048), (14336, 4096, 2048), (4096, 14336, 8192), (14336, 4096, 8192)]


@pytest.mark.parametrize("route", ["hand_written", "default"])
@pytest.mark.parametrize("k,n,m", PREFILL_SHAPES)
def test_prefill_configs_at_full_size(ep, ep_tiled, port, route, k, n, m):
    """configs[3]: fp16, block 32, no zero points, Llama-3-8B MLP shapes, on the hand-written tiled kernel and on whatever the
    default dispatch picks at that height."""
    provider = ep_tiled if route == "hand_written" else ep
    if route == "default" and m == 512:
        pytest.skip("the default dispatch runs the same kernel as the hand-written route at this height")
    dt, bs = E.F16, 32
    b, s, _ = random_weights(n, k, bs, 4321 + n, False, dt, 0.001, 0.01)
    a = synth.make_activation(m, k, 99, dt)
    cols, rows = spread(n, 200), spread(m, 48)
    ops = E.DeviceOperands(provider, b, s, dt, None, n, k, bs)
    ab, yb = provider.upload(a), provider.allocate(m * n * 2)
    try:
        ops.run(ab, dt, m, yb)
        y = provider.download(yb, (m, n), np.float16)
        variant = ops.kernel.last_variant()
    finally:
        provider.deallocate(ab)
        provider.deallocate(yb)
        ops.free()
    if route == "hand_written":
        assert variant == "prefill_mfma_lds"
    want = sampled_f64(port, a.astype(np.float32), b, s.astype(np.float32), None, cols, k, bs, rows=rows)
    assert np.isfinite(y.astype(np.float32)).all()
    assert helpers.rel_l2(y[np.ix_(rows, cols)].astype(np.float64), want) <= TOL_HALF, variant


ACC4_SHAPES = [(8192, 28672, 1), (8192, 28672, 8), (28672, 8192, 16), (8192, 28672, 256), (28672, 8192, 1), (28672, 8192, 256), (8192, 10240, 4096),
               (8192, 28672, 4096), (28672, 8192, 4096), (8192, 10240, 1), (8192, 10240, 256)]


@pytest.mark.parametrize("k,n,m", ACC4_SHAPES)
def test_acc4_configs_at_full_size(ep, port, k, n, m):
    """configs[4]: fp16, block 64, zero points, accuracy_level 4, 70B-class shapes. f32 output against the oracle's integer
    path on sampled rows and columns (the quantizer works row by row, so a row sample is a faithful sub-problem)."""
    dt, bs = E.F16, 64
    b, s, zp = random_weights(n, k, bs, 2468 + n, True, dt, 0.002, 0.01)
    a = synth.make_activation(m, k, 55, dt)
    cols, rows = spread(n, 200), spread(m, 24)
    ops = E.DeviceOperands(ep, b, s, dt, zp, n, k, bs, accuracy_level=4)
    ab, yb = ep.upload(a), ep.allocate(m * n * 4)
    try:
        ops.run(ab, dt, m, yb, E.F32)
        y = ep.download(yb, (m, n), np.float32)
        variant = ops.kernel.last_variant()
    finally:
        ep.deallocate(ab)
        ep.deallocate(yb)
        ops.free()
    assert variant.startswith("acc4_mfma_i8"), variant
    af = np.ascontiguousarray(a.astype(np.float32)[rows])
    want = port.matmul_acc4_f32(af, np.ascontiguousarray(b[cols]), np.ascontiguousarray(s.astype(np.float32)[cols]), np.ascontiguousarray(zp[cols]),
                                len(cols), k, bs, oracle.ROUND_HALF_EVEN)
    assert np.isfinite(y).all()
    assert helpers.rel_l2(y[np.ix_(rows, cols)], want) <= TOL_F32


def _random_decode_cases(count, seed):
    """Seeded decode calls at model widths: 64 .. 3200 column groups (some ragged), 1 .. 37 tile groups of K (some ending inside a
    tile group), 1 .. 16 rows, block 32 / 64 / 128, f16 / bf16 with 16-bit or f32 scales, float and accuracy_level 4 - the ranges
    over which the launchers pick wave counts, register sets, row builds and kernels."""
    rng = np.random.default_rng(seed)
    cases = []
    for _ in range(count):
        a_dt = int(rng.choice([E.F16, E.BF16]))
        s_dt = a_dt if rng.random() < 0.8 else E.F32
        bs = int(rng.choice([32, 64, 128]))
        zero_points = bool(rng.random() < 0.6)
        m = int(rng.choice([1, 1, 2, 3, 4, 4, 5, 6, 8, 9, 12, 16]))
        k = int(rng.integers(1, 38)) * 512 - (int(rng.integers(0, 512 // bs)) * bs if rng.random() < 0.4 else 0)
        k = max(k, bs)
        n = int(np.exp(rng.uniform(np.log(64), np.log(3200)))) * 16 - (int(rng.integers(0, 16)) if rng.random() < 0.4 else 0)
        while n * k > 3.0e8:
            n //= 2
        cases.append((a_dt, s_dt, bs, zero_points, m, max(n, 17), k, 4 if rng.random() < 0.35 else 0, bool(rng.random() < 0.5)))
    return cases


@pytest.mark.parametrize("a_dt,s_dt,bs,zero_points,m,n,k,acc,with_bias", _random_decode_cases(80, 20260214))
def test_random_decode_shapes_at_model_widths(ep, port, a_dt, s_dt, bs, zero_points, m, n, k, acc, with_bias):
    """Whatever wave count, register-set build, row build or kernel the launcher picks for the shape: f32 output against the
    oracle on a column sample, and the second call (what a graph replays) equal to the first (which repacks) bit for bit."""
    b, s, zp = random_weights(n, k, bs, 900 + n + k, zero_points, s_dt, 0.002, 0.01)
    a = synth.make_activation(m, k, 900 + m, a_dt)
    bias = synth.to_dtype(np.random.default_rng(n).standard_normal(n).astype(np.float32), a_dt) if with_bias else None
    cols = spread(n, 160)
    ops = E.DeviceOperands(ep, b, s, s_dt, zp, n, k, bs, accuracy_level=acc, bias=bias, bias_dtype=a_dt)
    ab, yb = ep.upload(a), ep.allocate(m * n * 4)
    try:
        ys = []
        for _ in range(2):
            ops.run(ab, a_dt, m, yb, E.F32)
            ys.append(ep.download(yb, (m, n), np.float32).copy())
        variant = ops.kernel.last_variant()
    finally:
        ep.deallocate(ab)
        ep.deallocate(yb)
        ops.free()
    assert variant == ("acc4_mfma_i8_packed" if acc == 4 else "decode_mfma_packed")
    assert np.isfinite(ys[1]).all()
    assert np.array_equal(ys[0], ys[1])
    af, sf = synth.to_f32(a, a_dt), synth.to_f32(s, s_dt)
    bc, sc = np.ascontiguousarray(b[cols]), np.ascontiguousarray(sf[cols])
    zc = np.ascontiguousarray(zp[cols]) if zp is not None else None
    bf = None if bias is None else np.ascontiguousarray(synth.to_f32(bias, a_dt)[cols])
    if acc == 4:
        want = port.matmul_acc4_f32(af, bc, sc, zc, len(cols), k, bs, oracle.ROUND_HALF_EVEN, bias=bf)
        assert helpers.rel_l2(ys[1][:, cols], want) <= TOL_F32
    else:
        want = port.matmul_f64(af, bc, sc, zc, len(cols), k, bs, bias=bf)
        assert helpers.rel_l2(ys[1][:, cols], want) <= 1e-4
