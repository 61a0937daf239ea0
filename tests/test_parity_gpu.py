"""Parity of the HIP path with the CPU oracle, called through the C ABI of libnxrt_ep_rocm.so.

Bars (from the parity contract of this build):
  * dequantized weights ........................ bit-exact
  * accuracy_level=4 codes and int32 block sums  bit-exact
  * outputs, f32 activations ................... rel-L2 <= 1e-5
  * outputs, f16/bf16 activations .............. rel-L2 <= 5e-3
"""
import os

import numpy as np
import pytest

import oracle
from onnx_genai_amd import ep as E
from onnx_genai_amd import synth
from tests import helpers

pytestmark = pytest.mark.gpu

TOL_F32 = 1e-5
TOL_HALF = 5e-3
NPDT = {E.F32: np.float32, E.F16: np.float16, E.BF16: np.uint16}


def run_op(ep, a, a_dt, b, s, s_dt, zp, n, k, bs, **kw):
    return E.matmul_nbits(ep, a, a_dt, b, s, s_dt, zp, n, k, bs, **kw)


def oracle_f64(port, a, a_dt, b, s, s_dt, zp, n, k, bs, bias=None, bias_dt=E.F32):
    af = synth.to_f32(a, a_dt)
    sf = synth.to_f32(s, s_dt)
    bf = None if bias is None else synth.to_f32(bias, bias_dt)
    return port.matmul_f64(af, b, sf, zp, n, k, bs, bias=bf)


# ---------------------------------------------------------------------------------------------
# dequantization: bit-exact
# ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("bs", [16, 32, 64, 128, 256])
@pytest.mark.parametrize("zero_points", [False, True])
@pytest.mark.parametrize("s_dt", [E.F32, E.F16, E.BF16])
def test_dequantize_bit_exact(ep, port, bs, zero_points, s_dt):
    n, k = 75, 3 * bs + (bs // 2 if bs >= 32 else 0)      # ragged N, partial last block
    b, s, zp = synth.make_weights(n, k, bs, 11 + bs, zero_points=zero_points, scale_lo=0.002, scale_hi=0.02, scale_dtype=s_dt)
    want = port.dequantize_nk(b, synth.to_f32(s, s_dt), zp, n, k, bs)
    bb, sb = ep.upload(b), ep.upload(s)
    zb = ep.upload(zp) if zp is not None else None
    out = ep.allocate(n * k * 4)
    ep.dequantize(bb, sb, s_dt, zb, n, k, bs, out)
    got = ep.download(out, (n, k), np.float32)
    for buf in (bb, sb, zb, out):
        if buf is not None:
            ep.deallocate(buf)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_dequantize_all_nibble_zero_point_pairs(ep, port):
    """Every (q, zp) pair against scales with awkward bit patterns."""
    bs, kb = 16, 16
    n = 16
    q = np.tile(np.arange(16, dtype=np.uint8), (n, kb, 1))
    b = synth.pack_nibbles(q)
    zq = np.tile(np.arange(16, dtype=np.uint8)[:, None], (1, kb))
    zp = synth.pack_nibbles(zq)
    rng = np.random.default_rng(5)
    s = rng.uniform(1e-4, 3.0, size=(n, kb)).astype(np.float32)
    s.view(np.uint32)[:, ::2] |= 0x7FF                      # low mantissa bits set: products must round once
    want = port.dequantize_nk(b, s, zp, n, kb * bs, bs)
    bb, sb, zb, out = ep.upload(b), ep.upload(s), ep.upload(zp), ep.allocate(n * kb * bs * 4)
    ep.dequantize(bb, sb, E.F32, zb, n, kb * bs, bs, out)
    got = ep.download(out, (n, kb * bs), np.float32)
    for buf in (bb, sb, zb, out):
        ep.deallocate(buf)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


# ---------------------------------------------------------------------------------------------
# known answers held by the reference's own tests
# ---------------------------------------------------------------------------------------------
def test_low_nibble_before_high_nibble(ep):
    """matmul_nbits.rs:18702-18722: packed[0]=0xe1, A=[1,10,0...] -> (1-8)*1 + (14-8)*10 = 53."""
    k = 16
    a = np.zeros((1, k), np.float32)
    a[0, 0], a[0, 1] = 1.0, 10.0
    b = np.full((1, 1, 8), 0x88, np.uint8)
    b[0, 0, 0] = 0xE1
    y, _ = run_op(ep, a, E.F32, b, np.ones((1, 1), np.float32), E.F32, None, 1, k, 16)
    assert y.tolist() == [[53.0]]


def test_accuracy_envelope_against_f64(ep, port):
    """matmul_nbits.rs:10986-11068: level 0 error < 1e-5, level 4 error inside [1e-4, 1e-2)."""
    k, n, bs, weights, act = helpers.envelope_fixture()
    b, s, zp, _ = helpers.quantize_blockwise(weights, bs, True)
    want = port.matmul_f64(act, b, s, zp, n, k, bs)
    assert np.abs(want).max() > 1.0
    y0, _ = run_op(ep, act, E.F32, b, s, E.F32, zp, n, k, bs, accuracy_level=0)
    y4, _ = run_op(ep, act, E.F32, b, s, E.F32, zp, n, k, bs, accuracy_level=4)
    exact, reduced = helpers.max_rel_to_peak(y0, want), helpers.max_rel_to_peak(y4, want)
    assert exact < 1e-5
    assert reduced > 10 * exact
    assert 1e-4 <= reduced < 1e-2


# ---------------------------------------------------------------------------------------------
# f32 activations (f32 FMA streaming kernel; the scalar catch-all below block size 32 or odd K): rel-L2 <= 1e-5
# ---------------------------------------------------------------------------------------------
def test_config1_qwen_mlp_shape_f32(ep, port, ref):
    m, k, n, bs = 1, 896, 4864, 32
    b, s, _ = synth.make_weights(n, k, bs, 1, zero_points=False, scale_lo=0.005, scale_hi=0.02, scale_dtype=E.F32)
    a = synth.make_activation(m, k, 1, E.F32, dist="uniform")
    y, variant = run_op(ep, a, E.F32, b, s, E.F32, None, n, k, bs)
    assert variant == "gemv_f32_valu"
    want = port.matmul_f64(a, b, s, None, n, k, bs)
    assert helpers.rel_l2(y, want) <= TOL_F32
    y_ref = ref.matmul(a, b, s, None, n, k, bs, ref.COMP_FP32)
    assert helpers.rel_l2(y, y_ref) <= TOL_F32


@pytest.mark.parametrize("m", [1, 5])
@pytest.mark.parametrize("bs", [32, 64, 128])
@pytest.mark.parametrize("asym", [False, True])
def test_sqnbit_grid_f32(ep, port, ref, m, bs, asym):
    """mlas-sys/src/lib.rs:3268-3285 grid: n=96, k=256."""
    n, k = 96, 256
    w, a, bias = helpers.sqnbit_fixture(m, n, k)
    b, s, zp, deq = helpers.quantize_blockwise(w, bs, asym)
    y, _ = run_op(ep, a, E.F32, b, s, E.F32, zp, n, k, bs, bias=bias)
    want = port.matmul_f64(a, b, s, zp, n, k, bs, bias=bias)
    assert helpers.rel_l2(y, want) <= TOL_F32
    y_ref = ref.matmul(a, b, s, zp, n, k, bs, ref.COMP_FP32, bias=bias)
    assert helpers.rel_l2(y, y_ref) <= TOL_F32
    assert np.abs(y - port.matmul_dequant_f32(a, deq, bias)).max() <= 2e-2       # the reference test's own tolerance


@pytest.mark.parametrize("k,bs", [(40, 16), (100, 32), (72, 64), (130, 128)])
def test_ragged_k_f32(ep, port, k, bs):
    """K not a multiple of the block size (partial last block) and of 8."""
    n, m = 37, 3
    b, s, zp = synth.make_weights(n, k, bs, 3, zero_points=True, scale_lo=0.01, scale_hi=0.05, scale_dtype=E.F32)
    a = synth.make_activation(m, k, 3, E.F32)
    y, _ = run_op(ep, a, E.F32, b, s, E.F32, zp, n, k, bs)
    assert helpers.rel_l2(y, port.matmul_f64(a, b, s, zp, n, k, bs)) <= TOL_F32


F32_CASES = [
    # s_dt, bs, zp, m, n, k      (K windows of 2048, steps of 512: whole, ragged and multi-window spans)
    (E.F32, 32, True, 1, 896, 896),
    (E.F32, 32, False, 2, 33, 4096),
    (E.F32, 64, True, 3, 100, 4100),
    (E.F32, 128, True, 4, 257, 8192),
    (E.F16, 128, True, 1, 64, 18944),
    (E.BF16, 64, False, 5, 31, 1000),
    (E.F32, 32, True, 9, 65, 516),
    (E.F32, 256, True, 1, 40, 3584),
    (E.F32, 128, True, 64, 32, 640),
    (E.F32, 32, True, 65, 16, 512),       # beyond 64 rows: the catch-all
    (E.F32, 16, True, 1, 48, 512),        # block size 16: the catch-all
    (E.F32, 32, True, 1, 48, 130),        # K % 4 != 0: the catch-all
]


@pytest.mark.parametrize("s_dt,bs,zero_points,m,n,k", F32_CASES)
def test_f32_activations_match_oracle(ep, port, s_dt, bs, zero_points, m, n, k):
    b, s, zp = synth.make_weights(n, k, bs, 7 + n + k, zero_points=zero_points, scale_lo=0.002, scale_hi=0.01, scale_dtype=s_dt)
    a = synth.make_activation(m, k, n, E.F32)
    bias = np.random.default_rng(n).standard_normal(n).astype(np.float32)
    y, variant = run_op(ep, a, E.F32, b, s, s_dt, zp, n, k, bs, bias=bias)
    assert variant == ("gemv_f32_valu" if m <= 64 and bs >= 32 and k % 4 == 0 else "gemv_generic_f32")
    want = oracle_f64(port, a, E.F32, b, s, s_dt, zp, n, k, bs, bias, E.F32)
    assert helpers.rel_l2(y, want) <= TOL_F32


# ---------------------------------------------------------------------------------------------
# decode path (f16 / bf16 activations, M <= 16)
# ---------------------------------------------------------------------------------------------
DECODE_CASES = [
    # a_dt, s_dt, bs, zp, m, n, k
    (E.BF16, E.BF16, 128, True, 1, 512, 3584),
    (E.BF16, E.BF16, 128, True, 4, 500, 3584),
    (E.BF16, E.BF16, 128, True, 8, 96, 1024),
    (E.BF16, E.BF16, 128, True, 16, 1000, 2048),
    (E.BF16, E.F32, 128, False, 3, 64, 512),
    (E.F16, E.F16, 32, True, 1, 896, 896),
    (E.F16, E.F16, 32, True, 1, 128, 896),
    (E.F16, E.F16, 32, False, 7, 130, 4864),
    (E.F16, E.F16, 64, True, 2, 257, 1024),
    (E.BF16, E.BF16, 64, True, 16, 48, 8192),
    (E.F16, E.F32, 128, True, 5, 80, 1536),
    (E.BF16, E.BF16, 32, False, 1, 33, 768),
    (E.BF16, E.BF16, 32, True, 13, 100, 1000),
    (E.F16, E.F16, 128, True, 12, 40, 18944),
    (E.F16, E.F16, 32, True, 9, 17, 72),        # K = 72: multiple of 8, not of the block size
    (E.BF16, E.BF16, 128, True, 2, 20, 200),    # partial last block
    (E.F16, E.F16, 64, True, 1, 1, 64),
    (E.F16, E.F32, 64, True, 1, 100, 64 * 21),  # f32 scales, odd block count, tile groups padded
    (E.BF16, E.F32, 32, True, 3, 50, 32 * 19),
    (E.BF16, E.BF16, 64, False, 4, 70, 4096),
    # many columns and several rows: activations shared through LDS, one wave per 16 columns
    (E.BF16, E.BF16, 128, True, 16, 16400, 3584),
    (E.F16, E.F16, 32, True, 5, 16384, 1000),
    (E.F16, E.F32, 64, False, 6, 20000, 64 * 21),
    (E.BF16, E.BF16, 128, True, 8, 37888, 3584),
    (E.F16, E.F16, 128, True, 13, 16385, 2048 + 8),
    (E.BF16, E.BF16, 128, True, 9, 98400, 512),         # three or more workgroups per CU: the variant with the second MFMA
    (E.F16, E.F16, 64, True, 16, 98304, 256),
    (E.BF16, E.BF16, 128, True, 12, 98400, 1536),       # the same over three tile groups: a pair of passes and a peeled one
    (E.BF16, E.BF16, 128, True, 16, 14336, 1024),       # the narrowest shape the shared-activation kernel takes (fewer workgroups than CUs)
    (E.F16, E.F16, 64, True, 11, 14400, 512),
    (E.F16, E.F16, 32, True, 9, 14336, 512),
    (E.BF16, E.BF16, 64, True, 8, 37888, 1024 + 64),    # block 64, between one and 1.5 workgroups per CU: ten waves a workgroup, second-MFMA build with weights ahead
    (E.F16, E.F16, 64, True, 16, 32784, 512),           # the same with nine waves and a ragged last workgroup
    (E.F16, E.F16, 32, True, 12, 37888, 512),           # block 32 never takes the sums build (here: 296 workgroups of eight waves)
    (E.BF16, E.F32, 32, True, 7, 20000, 32 * 19),       # ... nor with f32 scales; a partial last tile group
    (E.F16, E.F32, 128, True, 4, 18432, 512),           # four rows at block 128 from 18432 columns: the shared-activation kernel with one block of rows
    (E.BF16, E.BF16, 128, False, 4, 18450, 1024 + 128),  # ... a ragged last workgroup
    (E.BF16, E.BF16, 128, True, 4, 18431, 512),         # one column short of it: the four-row split-K build
    (E.BF16, E.BF16, 128, True, 17, 16400, 3584),       # up to 64 rows ride on one pass over the weights
    (E.F16, E.F16, 64, True, 40, 16384, 1024 + 64),     # block size 64 stops at 32 rows per pass: the tiled kernel takes this one
    (E.F16, E.F16, 64, True, 25, 16384, 1024 + 64),
    (E.BF16, E.F32, 128, False, 64, 16390, 2048),
    (E.F16, E.F16, 32, True, 30, 16384, 1000),
]


@pytest.mark.parametrize("a_dt,s_dt,bs,zero_points,m,n,k", DECODE_CASES)
@pytest.mark.parametrize("prepack", [True, False])
def test_decode_matches_oracle(ep, ep_unpacked, port, prepack, a_dt, s_dt, bs, zero_points, m, n, k):
    ep = ep if prepack else ep_unpacked
    b, s, zp = synth.make_weights(n, k, bs, 100 + n + k, zero_points=zero_points, scale_lo=0.002, scale_hi=0.01, scale_dtype=s_dt)
    a = synth.make_activation(m, k, n, a_dt)
    bias = synth.to_dtype(np.random.default_rng(n).standard_normal(n).astype(np.float32), a_dt)
    want64 = oracle_f64(port, a, a_dt, b, s, s_dt, zp, n, k, bs, bias, a_dt)

    # f32 output: the arithmetic itself, before any narrowing
    y32, variant = run_op(ep, a, a_dt, b, s, s_dt, zp, n, k, bs, bias=bias, bias_dtype=a_dt, y_dtype=E.F32)
    if m <= 16:
        # up to 16 rows read the repacked stream at every width (the split-K kernel, or the shared-activation kernel where the call is wide enough)
        assert variant == ("decode_mfma_packed" if prepack else "decode_mfma_splitk")
    else:
        # m <= 32: two row blocks through the decode kernel where that beats the tiled kernel (block 128, few columns or rows)
        row_blocks = m <= 32 and (k % 64 != 0 or (bs >= 128 and (n <= 8192 or m <= 20)))
        unpacked = "decode_mfma_splitk" if row_blocks else "prefill_mfma_lds" if k % 64 == 0 else "gemv_generic_f32"
        # rows per pass over the repacked weights: 16 at block size 32 (17..32 rows go as two such passes), 32 at 64, 64 at 128
        packed_rows = 32 if bs <= 64 else 64
        assert variant == ("decode_mfma_packed" if prepack and m <= packed_rows else unpacked)
    # The kernel carries each weight as (2^10 + q) in f16 or (2^7 + q) in bf16 and cancels the offset inside the
    # f32 accumulator, which costs 10 (7) of its 24 bits: a few 1e-5 on outputs that themselves cancel.
    # (The tiled kernel, which serves these row counts when nothing is repacked, rounds weights to 16 bits in LDS.)
    assert helpers.rel_l2(y32, want64) <= (TOL_HALF if variant == "prefill_mfma_lds" else 1e-4)

    # output in the activation dtype, against the oracle's whole-operator result
    y, _ = run_op(ep, a, a_dt, b, s, s_dt, zp, n, k, bs, bias=bias, bias_dtype=a_dt)
    want = port.matmul_nbits(a, a_dt, b, s, s_dt, zp, bias, a_dt, a_dt, m, n, k, bs)
    assert helpers.rel_l2(synth.to_f32(y, a_dt), synth.to_f32(want, a_dt)) <= TOL_HALF
    assert helpers.rel_l2(synth.to_f32(y, a_dt), want64) <= TOL_HALF

    # dtype contract (matmul_nbits.rs:17197-17281): compute in f32, narrow once
    assert np.array_equal(np.asarray(y).view(np.uint16), np.asarray(port.narrow(y32, a_dt)).view(np.uint16))


@pytest.mark.parametrize("waves,cg", [(1, 1), (3, 2), (16, 4), (7, 1)])
def test_decode_launch_shapes_agree(port, waves, cg):
    """Every split of the work over waves and column groups gives the same answer (to f32 rounding)."""
    provider = E.RocmExecutionProvider(0, {"decode_waves": waves, "decode_col_groups": cg, "prepack": "0"})
    try:
        a_dt, bs, m, n, k = E.BF16, 128, 6, 200, 3584
        b, s, zp = synth.make_weights(n, k, bs, 77, zero_points=True, scale_lo=0.002, scale_hi=0.01, scale_dtype=a_dt)
        a = synth.make_activation(m, k, 77, a_dt)
        y32, variant = run_op(provider, a, a_dt, b, s, a_dt, zp, n, k, bs, y_dtype=E.F32)
        assert variant == "decode_mfma_splitk"
        assert helpers.rel_l2(y32, oracle_f64(port, a, a_dt, b, s, a_dt, zp, n, k, bs)) <= 2e-5
    finally:
        provider.shutdown()


@pytest.mark.parametrize("waves", [1, 3, 8])
def test_packed_decode_wave_counts_agree(port, waves):
    provider = E.RocmExecutionProvider(0, {"decode_waves": waves})
    try:
        a_dt, bs, n, k = E.BF16, 128, 200, 3584
        b, s, zp = synth.make_weights(n, k, bs, 78, zero_points=True, scale_lo=0.002, scale_hi=0.01, scale_dtype=a_dt)
        for m in (1, 3, 7, 16):
            a = synth.make_activation(m, k, 78 + m, a_dt)
            y32, variant = run_op(provider, a, a_dt, b, s, a_dt, zp, n, k, bs, y_dtype=E.F32)
            assert variant == "decode_mfma_packed"
            assert helpers.rel_l2(y32, oracle_f64(port, a, a_dt, b, s, a_dt, zp, n, k, bs)) <= 2e-5
    finally:
        provider.shutdown()


@pytest.mark.parametrize("prepack", [True, False])
@pytest.mark.parametrize("m", [17, 25, 32])
def test_row_blocks_through_the_decode_kernels(ep, ep_unpacked, port, prepack, m):
    """17..32 rows at a shape without many columns: a block of 16 rows and a remainder through the decode kernels."""
    ep = ep if prepack else ep_unpacked
    a_dt, bs, n, k = E.BF16, 128, 300, 1024
    b, s, zp = synth.make_weights(n, k, bs, 55, zero_points=True, scale_lo=0.002, scale_hi=0.01, scale_dtype=a_dt)
    a = synth.make_activation(m, k, 55 + m, a_dt)
    bias = synth.to_dtype(np.linspace(-2, 2, n).astype(np.float32), a_dt)
    y32, variant = run_op(ep, a, a_dt, b, s, a_dt, zp, n, k, bs, bias=bias, bias_dtype=a_dt, y_dtype=E.F32)
    # with the repacked copy, both row blocks read it
    assert variant == ("decode_mfma_packed" if prepack else "decode_mfma_splitk")
    assert helpers.rel_l2(y32, oracle_f64(port, a, a_dt, b, s, a_dt, zp, n, k, bs, bias, a_dt)) <= 1e-4
    y, _ = run_op(ep, a, a_dt, b, s, a_dt, zp, n, k, bs, bias=bias, bias_dtype=a_dt)
    assert np.array_equal(np.asarray(y).view(np.uint16), np.asarray(port.narrow(y32, a_dt)).view(np.uint16))


def test_block_32_between_14336_and_16384_columns(ep, port):
    """Block size 32 at 14336 columns: up to 16 rows ride the shared-activation kernel; 17..32 rows go to the tiled kernel,
    not to two repacked passes."""
    a_dt, bs, n, k = E.F16, 32, 14336, 256
    b, s, zp = synth.make_weights(n, k, bs, 77, zero_points=True, scale_lo=0.002, scale_hi=0.01, scale_dtype=a_dt)
    for m, expected in ((16, "decode_mfma_packed"), (24, "prefill_mfma_lds")):
        a = synth.make_activation(m, k, 77 + m, a_dt)
        y32, variant = run_op(ep, a, a_dt, b, s, a_dt, zp, n, k, bs, y_dtype=E.F32)
        assert variant == expected
        assert helpers.rel_l2(y32, oracle_f64(port, a, a_dt, b, s, a_dt, zp, n, k, bs)) <= TOL_HALF


GRAPH_CASES = [
    # a_dt, bs, accuracy_level, m, n, k, what runs
    (E.BF16, 128, 0, 1, 300, 3584),        # one-row decode over the repacked stream
    (E.BF16, 128, 0, 8, 16400, 1024),      # shared-activation decode
    (E.F16, 32, 0, 40, 200, 1024),         # tiled kernel
    (E.F16, 64, 0, 100, 130, 4096),        # tiled kernel over slices of K: partial sums in the kernel's own scratch + reduce
    (E.F32, 32, 0, 3, 100, 1000),          # f32 activations
    (E.F16, 64, 4, 1, 160, 1024),          # accuracy_level 4, one row: quantized inside the kernel, no workspace
    (E.F16, 64, 4, 5, 96, 512),            # accuracy_level 4 with the caller's workspace: quantizer + int8 MFMA
    (E.F16, 64, 4, 130, 200, 576),
    (E.F16, 64, 4, 130, 200, 2048),        # the same over slices of K: partial sums in the workspace + reduce
    (E.BF16, 128, 0, 1024, 136, 512),      # tall call: the tiled kernel in 256-row tiles (the library GEMM route is opt-in)
]


@pytest.mark.parametrize("a_dt,bs,acc,m,n,k", GRAPH_CASES)
def test_graph_replays_match_eager(ep, a_dt, bs, acc, m, n, k):
    """A call recorded into a HIP graph gives, on every replay, bit for bit what the eager call gave - with other eager
    work and synchronisations between the replays, and after the input has changed."""
    s_dt = a_dt
    b, s, zp = synth.make_weights(n, k, bs, 61 + n, zero_points=True, scale_lo=0.002, scale_hi=0.01, scale_dtype=s_dt)
    ops = E.DeviceOperands(ep, b, s, s_dt, zp, n, k, bs, accuracy_level=acc, rows=m, a_dtype=a_dt)
    y_dt = a_dt
    elem = 4 if y_dt == E.F32 else 2
    np_y = np.float32 if y_dt == E.F32 else np.uint16
    inputs = [synth.make_activation(m, k, 70 + i, a_dt) for i in range(3)]
    ab, yb = ep.upload(inputs[0]), ep.allocate(m * n * elem)
    scratch_y = ep.allocate(m * n * elem)
    workspace = None
    if acc == 4:
        need, _ = ops.kernel.workspace_requirement([((m, k), a_dt)])
        workspace = ep.allocate(need)
    out = [E.TensorView(yb.ptr, y_dt, (m, n), device_index=ep.device_index)]
    other = [E.TensorView(scratch_y.ptr, y_dt, (m, n), device_index=ep.device_index)]

    def run(target):
        ops.kernel.execute(ops.views(ab, a_dt, m), target, workspace=workspace)

    eager = []
    for a in inputs:                                   # eager results for each input (the first call also repacks / allocates)
        ep.copy_from_host(ab, a)
        run(out)
        eager.append(ep.download(yb, (m, n), np_y).copy())
    ep.sync()
    ep.capture_begin()
    try:
        run(out)
    finally:
        graph = ep.capture_end()
    try:
        for i, a in enumerate(inputs):
            ep.copy_from_host(ab, a)
            run(other)                                 # eager work of the same kernel object between replays
            ep.sync()
            ep.copy_from_host(yb, np.full(m * n * elem, 0xFF, np.uint8))     # a replay must overwrite all of Y
            graph.replay()
            got = ep.download(yb, (m, n), np_y)
            assert np.array_equal(got.view(np.uint8), eager[i].view(np.uint8)), "replay %d differs from the eager result" % i
    finally:
        graph.release()
        for buf in (ab, yb, scratch_y, workspace):
            if buf is not None:
                ep.deallocate(buf)
        ops.free()


def test_graph_survives_a_later_larger_call(ep_tiled):
    """A graph recorded while the kernel's own scratch had one size still replays correctly after a later, taller call made
    the kernel grow that scratch (the outgrown buffer stays allocated for the graphs that name it)."""
    ep = ep_tiled
    a_dt, bs, n, k = E.F16, 64, 130, 4096                      # few tiles of Y, long K: K in slices, partial sums in scratch
    b, s, zp = synth.make_weights(n, k, bs, 63, zero_points=True, scale_lo=0.002, scale_hi=0.01, scale_dtype=a_dt)
    ops = E.DeviceOperands(ep, b, s, a_dt, zp, n, k, bs)
    small, tall = 100, 400
    a1 = ep.upload(synth.make_activation(small, k, 64, a_dt))
    a2 = ep.upload(synth.make_activation(tall, k, 65, a_dt))
    y1, y2 = ep.allocate(small * n * 2), ep.allocate(tall * n * 2)
    try:
        ops.run(a1, a_dt, small, y1)
        eager = ep.download(y1, (small, n), np.uint16).copy()
        ep.capture_begin()
        try:
            ops.run(a1, a_dt, small, y1)
        finally:
            graph = ep.capture_end()
        ops.run(a2, a_dt, tall, y2)                              # needs more scratch than the recorded call had
        ep.sync()
        ep.copy_from_host(y1, np.full(small * n * 2, 0xFF, np.uint8))
        graph.replay()
        assert np.array_equal(ep.download(y1, (small, n), np.uint16), eager)
        graph.release()
    finally:
        for buf in (a1, a2, y1, y2):
            ep.deallocate(buf)
        ops.free()


def test_packed_copy_follows_the_weights(port):
    """One kernel object, two weight tensors in turn: the repacked copy is rebuilt when the pointers change. The replaced
    copy is freed while the provider has recorded no graph, and kept once it has (a graph may replay through it)."""
    ep = E.RocmExecutionProvider(0)
    a_dt, bs, m, n, k = E.F16, 128, 1, 96, 1024
    a = synth.make_activation(m, k, 5, a_dt)
    ab, yb, yg = ep.upload(a), ep.allocate(m * n * 4), ep.allocate(m * n * 4)
    b1, s1, zp1 = synth.make_weights(n, k, bs, 31, zero_points=True, scale_lo=0.002, scale_hi=0.01, scale_dtype=a_dt)
    first = E.DeviceOperands(ep, b1, s1, a_dt, zp1, n, k, bs)
    b2, s2, zp2 = synth.make_weights(n, k, bs, 32, zero_points=True, scale_lo=0.002, scale_hi=0.01, scale_dtype=a_dt)
    other = [ep.upload(b2), ep.upload(s2), ep.upload(zp2)]
    kb = k // bs
    views1 = first.views(ab, a_dt, m)
    views2 = [E.TensorView(ab.ptr, a_dt, (m, k)), E.TensorView(other[0].ptr, E.U8, (n, kb, bs // 2)),
              E.TensorView(other[1].ptr, a_dt, (n, kb)), E.TensorView(other[2].ptr, E.U8, (n, (kb + 1) // 2))]
    want1 = oracle_f64(port, a, a_dt, b1, s1, a_dt, zp1, n, k, bs)
    want2 = oracle_f64(port, a, a_dt, b2, s2, a_dt, zp2, n, k, bs)
    first.kernel.execute(views1, [E.TensorView(yb.ptr, E.F32, (m, n))])
    assert helpers.rel_l2(ep.download(yb, (m, n), np.float32), want1) <= 1e-4
    for _ in range(3):                        # back and forth without a graph: every replaced copy is freed
        first.kernel.execute(views2, [E.TensorView(yb.ptr, E.F32, (m, n))])
        assert first.kernel.last_variant() == "decode_mfma_packed"
        assert helpers.rel_l2(ep.download(yb, (m, n), np.float32), want2) <= 1e-4
        first.kernel.execute(views1, [E.TensorView(yb.ptr, E.F32, (m, n))])
        assert helpers.rel_l2(ep.download(yb, (m, n), np.float32), want1) <= 1e-4
    assert first.kernel.retired_buffers() == 0
    ep.sync()
    ep.capture_begin()
    try:
        first.kernel.execute(views1, [E.TensorView(yg.ptr, E.F32, (m, n))])
    finally:
        graph = ep.capture_end()
    # the graph reads the copy made from the first weights: a call with the second keeps that copy
    first.kernel.execute(views2, [E.TensorView(yb.ptr, E.F32, (m, n))])
    assert first.kernel.retired_buffers() == 1
    assert helpers.rel_l2(ep.download(yb, (m, n), np.float32), want2) <= 1e-4
    graph.replay()
    ep.sync()
    assert helpers.rel_l2(ep.download(yg, (m, n), np.float32), want1) <= 1e-4
    graph.release()
    for buf in other + [ab, yb, yg]:
        ep.deallocate(buf)
    first.free()
    ep.shutdown()


def test_decode_is_deterministic(ep):
    a_dt, bs, m, n, k = E.F16, 32, 4, 300, 4864
    b, s, zp = synth.make_weights(n, k, bs, 9, zero_points=True, scale_lo=0.002, scale_hi=0.01, scale_dtype=a_dt)
    a = synth.make_activation(m, k, 9, a_dt)
    y1, _ = run_op(ep, a, a_dt, b, s, a_dt, zp, n, k, bs)
    y2, _ = run_op(ep, a, a_dt, b, s, a_dt, zp, n, k, bs)
    assert np.array_equal(y1.view(np.uint16), y2.view(np.uint16))


def test_linearity_at_full_7b_shape(ep):
    """Size-independent property at a full 7B decode shape: Y(A1 + A2) = Y(A1) + Y(A2) when the sum is exact."""
    a_dt, bs, n, k = E.BF16, 128, 4608, 3584
    b, s, zp = synth.make_weights(n, k, bs, 21, zero_points=True, scale_lo=0.002, scale_hi=0.01, scale_dtype=a_dt)
    rng = np.random.default_rng(21)
    a1 = rng.integers(-8, 9, size=(1, k)).astype(np.float32)          # small integers: sums stay exact in bf16
    a2 = rng.integers(-8, 9, size=(1, k)).astype(np.float32)
    ys = []
    for a in (a1, a2, a1 + a2):
        y, _ = run_op(ep, synth.to_dtype(a, a_dt), a_dt, b, s, a_dt, zp, n, k, bs, y_dtype=E.F32)
        ys.append(y.astype(np.float64))
    assert helpers.rel_l2(ys[0] + ys[1], ys[2]) <= 1e-5


# ---------------------------------------------------------------------------------------------
# prefill path (f16 / bf16 activations, M > 16)
# ---------------------------------------------------------------------------------------------
PREFILL_CASES = [
    # a_dt, s_dt, bs, zp, m, n, k
    (E.F16, E.F16, 32, False, 512, 256, 4096),
    (E.F16, E.F16, 32, True, 300, 200, 512),
    (E.F16, E.F16, 64, True, 17, 128, 64),
    (E.F16, E.F16, 128, True, 64, 130, 1024),
    (E.F16, E.F32, 32, True, 100, 96, 256),
    (E.BF16, E.BF16, 128, True, 257, 384, 3584),
    (E.BF16, E.BF16, 32, False, 33, 100, 128),
    (E.BF16, E.F32, 64, True, 1030, 128, 512),
    (E.F16, E.F16, 64, True, 49, 128, 64),
    (E.BF16, E.BF16, 32, False, 60, 100, 128),
]


@pytest.mark.parametrize("a_dt,s_dt,bs,zero_points,m,n,k", PREFILL_CASES)
def test_prefill_matches_oracle(ep_tiled, port, a_dt, s_dt, bs, zero_points, m, n, k):
    ep = ep_tiled
    b, s, zp = synth.make_weights(n, k, bs, 200 + n + k, zero_points=zero_points, scale_lo=0.001, scale_hi=0.01, scale_dtype=s_dt)
    a = synth.make_activation(m, k, n, a_dt)
    bias = synth.to_dtype(np.random.default_rng(n).standard_normal(n).astype(np.float32), a_dt)
    want64 = oracle_f64(port, a, a_dt, b, s, s_dt, zp, n, k, bs, bias, a_dt)
    y32, variant = run_op(ep, a, a_dt, b, s, s_dt, zp, n, k, bs, bias=bias, bias_dtype=a_dt, y_dtype=E.F32)
    assert variant == "prefill_mfma_lds" if m > 32 else variant in ("prefill_mfma_lds", "decode_mfma_splitk", "decode_mfma_packed")   # up to 32 rows: row blocks through the decode kernels where they pay
    assert helpers.rel_l2(y32, want64) <= TOL_HALF
    y, _ = run_op(ep, a, a_dt, b, s, s_dt, zp, n, k, bs, bias=bias, bias_dtype=a_dt)
    assert helpers.rel_l2(synth.to_f32(y, a_dt), want64) <= TOL_HALF
    assert np.array_equal(np.asarray(y).view(np.uint16), np.asarray(port.narrow(y32, a_dt)).view(np.uint16))


@pytest.mark.parametrize("tile", [1, 2, 3, 4])
@pytest.mark.parametrize("a_dt,s_dt,bs,zero_points", [(E.F16, E.F16, 32, True), (E.BF16, E.F32, 128, False), (E.BF16, E.BF16, 64, True)])
@pytest.mark.parametrize("n", [520, 515])
def test_prefill_tile_shapes_agree(port, tile, a_dt, s_dt, bs, zero_points, n):
    """Every workgroup tile (128 x 128, 256 x 128, 256 x 256, 128 x 64) on a shape with ragged edges in M and N. With N a
    multiple of 8 the 16-bit outputs leave through the wide stores (16 bytes per lane after a turn through LDS), otherwise
    element by element: both against the same expectations."""
    m, k = 300, 1024
    provider = E.RocmExecutionProvider(0, {"prefill_tile": str(tile)})
    try:
        b, s, zp = synth.make_weights(n, k, bs, 41, zero_points=zero_points, scale_lo=0.002, scale_hi=0.01, scale_dtype=s_dt)
        a = synth.make_activation(m, k, 41, a_dt)
        y32, variant = run_op(provider, a, a_dt, b, s, s_dt, zp, n, k, bs, y_dtype=E.F32)
        assert variant == "prefill_mfma_lds"
        assert helpers.rel_l2(y32, oracle_f64(port, a, a_dt, b, s, s_dt, zp, n, k, bs)) <= TOL_HALF
        # The epilogue forms of each tile against that f32 output, bit for bit: a bias per column, a residual per element
        # (added before the one rounding) and a folded residual (added after the accumulator was rounded).
        o_dt = {E.F16: oracle.F16, E.BF16: oracle.BF16}[a_dt]
        bits = lambda t: np.asarray(t).view(np.uint16)
        rng = np.random.default_rng(tile)
        bias = synth.to_dtype(rng.standard_normal(n).astype(np.float32), a_dt)
        residual = synth.to_dtype((rng.standard_normal((m, n)) * 0.5).astype(np.float32), a_dt)
        y, _ = run_op(provider, a, a_dt, b, s, s_dt, zp, n, k, bs, bias=bias, bias_dtype=a_dt)
        assert np.array_equal(bits(y), bits(port.narrow(y32 + synth.to_f32(bias, a_dt)[None, :], o_dt)))
        y, _ = run_op(provider, a, a_dt, b, s, s_dt, zp, n, k, bs, bias=residual, bias_dtype=a_dt)
        assert np.array_equal(bits(y), bits(port.narrow(y32 + synth.to_f32(residual, a_dt), o_dt)))
        y, _ = run_op(provider, a, a_dt, b, s, s_dt, zp, n, k, bs, bias=residual, bias_dtype=a_dt, folded_bias=1)
        rounded = synth.to_f32(port.narrow(y32, o_dt), a_dt)
        assert np.array_equal(bits(y), bits(port.narrow(rounded + synth.to_f32(residual, a_dt), o_dt)))
    finally:
        provider.shutdown()


@pytest.mark.parametrize("bs,zero_points", [(32, True), (64, False), (128, True)])
def test_prefill_weight_tiles_are_f16_of_f32_dequant(ep, port, bs, zero_points):
    """One-hot activation rows read single weights back out of the GEMM: with f16 scales each must equal the f32
    dequantized weight rounded once to f16, bit for bit."""
    m, n, k = 64, 256, 256
    b, s, zp = synth.make_weights(n, k, bs, 300 + bs, zero_points=zero_points, scale_lo=0.001, scale_hi=0.01, scale_dtype=E.F16)
    ks = (np.arange(m) * 37) % k
    a = np.zeros((m, k), np.float16)
    a[np.arange(m), ks] = 1.0
    y, variant = run_op(ep, a, E.F16, b, s, E.F16, zp, n, k, bs)
    assert variant == "prefill_mfma_lds"
    w = port.dequantize_nk(b, synth.to_f32(s, E.F16), zp, n, k, bs)            # f32 [N, K], bit-exact reference definition
    want = port.narrow(np.ascontiguousarray(w[:, ks].T), oracle.F16)
    assert np.array_equal(y.view(np.uint16), want.view(np.uint16))


# ---------------------------------------------------------------------------------------------
# folded bias: a standalone Add folded into the bias input keeps the two nodes' two roundings
# ---------------------------------------------------------------------------------------------
FOLDED_BIAS_CASES = [
    # a_dt, bs, accuracy_level, m, n, k: one per kernel family
    (E.BF16, 128, 0, 1, 300, 3584),        # one row over the repacked stream
    (E.F16, 32, 0, 4, 130, 896),           # four rows over the repacked stream
    (E.BF16, 128, 0, 8, 16400, 1024),      # shared-activation kernel
    (E.F16, 64, 0, 16, 100, 2048),         # split-K kernel
    (E.F16, 32, 0, 200, 136, 512),         # tiled kernel
    (E.F16, 64, 0, 100, 130, 4096),        # tiled kernel, K in slices: the reduce kernel adds the bias
    (E.F16, 32, 0, 1100, 136, 512),        # tall call
    (E.BF16, 16, 0, 3, 40, 64),            # catch-all kernel
    (E.F16, 64, 4, 1, 160, 1024),          # accuracy_level 4, one row
    (E.F16, 64, 4, 5, 96, 512),            # accuracy_level 4, split-K
    (E.BF16, 128, 4, 130, 200, 2560),      # accuracy_level 4, tiled, K in slices
    (E.F16, 16, 4, 20, 64, 256),           # accuracy_level 4, catch-all
]


@pytest.mark.parametrize("a_dt,bs,acc,m,n,k", FOLDED_BIAS_CASES)
def test_folded_bias_rounds_twice(ep_tiled, port, a_dt, bs, acc, m, n, k):
    """folded_bias = 1 on a 16-bit output gives round(round(acc) + bias), i.e. exactly what the same kernel without a bias
    followed by a 16-bit Add gives (onnx-runtime-ep-cuda/src/kernels/matmul_nbits.rs:1189-1212); without the marker the
    bias joins the accumulator before the one rounding."""
    ep = ep_tiled                                    # with and without a bias the same hand-written kernel must serve the call
    b, s, zp = synth.make_weights(n, k, bs, 700 + n, zero_points=True, scale_lo=0.002, scale_hi=0.01, scale_dtype=a_dt)
    a = synth.make_activation(m, k, 700 + m, a_dt)
    bias = synth.to_dtype((np.random.default_rng(n).standard_normal(n) * 0.37).astype(np.float32), a_dt)
    o_dt = oracle.F16 if a_dt == E.F16 else oracle.BF16
    common = dict(accuracy_level=acc)
    plain, v0 = run_op(ep, a, a_dt, b, s, a_dt, zp, n, k, bs, **common)
    folded, v1 = run_op(ep, a, a_dt, b, s, a_dt, zp, n, k, bs, bias=bias, bias_dtype=a_dt, folded_bias=1, **common)
    fused, _ = run_op(ep, a, a_dt, b, s, a_dt, zp, n, k, bs, bias=bias, bias_dtype=a_dt, **common)
    fused32, _ = run_op(ep, a, a_dt, b, s, a_dt, zp, n, k, bs, bias=bias, bias_dtype=a_dt, y_dtype=E.F32, **common)
    assert v0 == v1
    want = port.narrow(synth.to_f32(plain, a_dt) + synth.to_f32(bias, a_dt)[None, :], o_dt)
    assert np.array_equal(np.asarray(folded).view(np.uint16), np.asarray(want).view(np.uint16))
    assert np.array_equal(np.asarray(fused).view(np.uint16), np.asarray(port.narrow(fused32, o_dt)).view(np.uint16))
    assert not np.array_equal(np.asarray(folded).view(np.uint16), np.asarray(fused).view(np.uint16)) or m * n < 2000


@pytest.mark.parametrize("folded", [1, None])
@pytest.mark.parametrize("a_dt,bs,acc,m,n,k", [c for c in FOLDED_BIAS_CASES if c[3] > 1] + [(E.F16, 32, 0, 25, 130, 896), (E.F32, 32, 0, 7, 100, 256)])
def test_residual_in_the_bias_slot(ep_tiled, port, folded, a_dt, bs, acc, m, n, k):
    """A bias of Y's shape is a per-token residual (row stride N) - what the CUDA provider's folded residual epilogue passes
    (kernels/matmul_nbits.rs:7891-7897). With folded_bias it is added after the accumulator was rounded, else before."""
    ep = ep_tiled
    b, s, zp = synth.make_weights(n, k, bs, 710 + n, zero_points=True, scale_lo=0.002, scale_hi=0.01, scale_dtype=a_dt)
    a = synth.make_activation(m, k, 710 + m, a_dt)
    residual = synth.to_dtype((np.random.default_rng(n + m).standard_normal((m, n)) * 0.5).astype(np.float32), a_dt)
    o_dt = {E.F16: oracle.F16, E.BF16: oracle.BF16, E.F32: oracle.F32}[a_dt]
    got, v1 = run_op(ep, a, a_dt, b, s, a_dt, zp, n, k, bs, accuracy_level=acc, bias=residual, bias_dtype=a_dt, folded_bias=folded)
    if folded and a_dt != E.F32:
        plain, v0 = run_op(ep, a, a_dt, b, s, a_dt, zp, n, k, bs, accuracy_level=acc)
        want = port.narrow(synth.to_f32(plain, a_dt) + synth.to_f32(residual, a_dt), o_dt)
    else:
        plain32, v0 = run_op(ep, a, a_dt, b, s, a_dt, zp, n, k, bs, accuracy_level=acc, y_dtype=E.F32)
        want = port.narrow(plain32 + synth.to_f32(residual, a_dt), o_dt) if a_dt != E.F32 else plain32 + residual
    assert v0 == v1
    if a_dt == E.F32:
        assert np.array_equal(np.asarray(got), np.asarray(want))
    else:
        assert np.array_equal(np.asarray(got).view(np.uint16), np.asarray(want).view(np.uint16))


@pytest.mark.parametrize("folded", [1, None])
@pytest.mark.parametrize("bias_shape", ["[1, N]", "[1, 1, N]"])
@pytest.mark.parametrize("a_dt,bs,acc,n,k", [(E.BF16, 128, 0, 300, 3584), (E.F16, 64, 4, 160, 1024), (E.F32, 32, 0, 100, 256)])
def test_one_row_residual_in_the_bias_slot(ep, port, folded, bias_shape, a_dt, bs, acc, n, k):
    """A one-row decode step passes its residual as [1, N] or [1, 1, N]: N elements, so it broadcasts like a bias [N]
    (the CUDA provider accepts the bias slot by element count, kernels/matmul_nbits.rs:7728-7735, 7891-7897)."""
    b, s, zp = synth.make_weights(n, k, bs, 720 + n, zero_points=True, scale_lo=0.002, scale_hi=0.01, scale_dtype=a_dt)
    a = synth.make_activation(1, k, 721, a_dt)
    residual = synth.to_dtype((np.random.default_rng(n).standard_normal(n) * 0.5).astype(np.float32), a_dt)
    shape = (1, n) if bias_shape == "[1, N]" else (1, 1, n)
    common = dict(accuracy_level=acc, bias=residual, bias_dtype=a_dt, folded_bias=folded)
    got, v1 = run_op(ep, a, a_dt, b, s, a_dt, zp, n, k, bs, bias_shape=shape, **common)
    flat, v0 = run_op(ep, a, a_dt, b, s, a_dt, zp, n, k, bs, **common)            # the same values declared as [N]
    assert v0 == v1
    view = np.float32 if a_dt == E.F32 else np.uint16
    assert np.array_equal(np.asarray(got).view(view), np.asarray(flat).view(view))
    with pytest.raises(E.EpError) as e:
        run_op(ep, a, a_dt, b, s, a_dt, zp, n, k, bs, bias_shape=(n - 1,), **common)
    assert f"bias must have {n} elements" in str(e.value)


def test_folded_bias_keeps_tall_calls_off_the_library_gemm(ep_dense):
    """The library's epilogue adds a bias before the one rounding, so a folded bias stays on the hand-written kernel even
    where the opt-in dense route is on."""
    ep = ep_dense
    a_dt, bs, m, n, k = E.F16, 32, 1100, 136, 512
    b, s, zp = synth.make_weights(n, k, bs, 5, zero_points=False, scale_lo=0.002, scale_hi=0.01, scale_dtype=a_dt)
    a = synth.make_activation(m, k, 5, a_dt)
    bias = synth.to_dtype(np.linspace(-1, 1, n).astype(np.float32), a_dt)
    _, variant = run_op(ep, a, a_dt, b, s, a_dt, zp, n, k, bs, bias=bias, bias_dtype=a_dt, folded_bias=1)
    assert variant == "prefill_mfma_lds"
    _, variant = run_op(ep, a, a_dt, b, s, a_dt, zp, n, k, bs, bias=bias, bias_dtype=a_dt)
    assert variant == "dense_transient_blaslt"


# ---------------------------------------------------------------------------------------------
# bits = 2 and 8: the CPU provider's other widths, on the plain kernels and the dense route
# ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("bits", [2, 8])
@pytest.mark.parametrize("bs,zero_points,s_dt", [(16, True, E.F32), (32, False, E.F16), (128, True, E.BF16)])
def test_dequantize_bits_bit_exact(ep, port, bits, bs, zero_points, s_dt):
    n, k = 37, 5 * bs - 8
    b, s, zp = synth.make_weights_bits(n, k, bs, bits, 40 + bits, zero_points=zero_points, scale_lo=0.001, scale_hi=0.05, scale_dtype=s_dt)
    bb, sb, zb, ob = ep.upload(b), ep.upload(s), ep.upload(zp) if zp is not None else None, ep.allocate(n * k * 4)
    try:
        ep.dequantize(bb, sb, s_dt, zb, n, k, bs, ob, bits=bits)
        got = ep.download(ob, (n, k), np.float32)
        assert np.array_equal(got, port.dequantize_nk_bits(b, synth.to_f32(s, s_dt), zp, n, k, bs, bits))
    finally:
        for buf in (bb, sb, zb, ob):
            if buf is not None:
                ep.deallocate(buf)


NBITS_CASES = [
    # a_dt, s_dt, bs, zp, m, n, k
    (E.F32, E.F32, 32, True, 1, 300, 896),
    (E.F16, E.F16, 32, False, 1, 130, 1024),
    (E.BF16, E.BF16, 128, True, 5, 200, 3584),
    (E.F16, E.F32, 16, True, 13, 64, 200),        # K ends inside a block
    (E.F16, E.F16, 64, True, 40, 136, 512),       # tall enough for the dense route at these widths
    (E.F16, E.F16, 32, True, 9, 100, 640),        # nine rows: the tiled kernel over the dense copy by default (from five)
    (E.BF16, E.BF16, 128, True, 300, 256, 1024),
    (E.F32, E.F16, 64, True, 20, 72, 256),        # f32 activations stay on the plain kernel at any height
    (E.BF16, E.BF16, 128, True, 1, 1030, 3584),   # 8 bits: the 16-byte-load GEMV (one row), ragged column count
    (E.F16, E.F16, 16, False, 4, 70, 1040),       # 8 bits: four rows, a K that leaves the last step half empty
    (E.F16, E.F16, 32, True, 3, 40, 72),          # K % 16 != 0: the plain kernel
    (E.F16, E.F16, 32, True, 3, 72, 1024),        # 2 bits: three rows through the 16-byte-load GEMV (K % 64 == 0)
    (E.BF16, E.F32, 16, True, 2, 50, 4096 + 64),  # ... block 16: four blocks per load, f32 scales
]


@pytest.mark.parametrize("route", ["default", "library"])
@pytest.mark.parametrize("bits", [2, 8])
@pytest.mark.parametrize("a_dt,s_dt,bs,zero_points,m,n,k", NBITS_CASES)
def test_other_bit_widths_match_oracle(ep, ep_dense, port, route, bits, a_dt, s_dt, bs, zero_points, m, n, k):
    """bits = 2 and 8. Up to four rows (and f32 activations, or K not a multiple of 64, at any height) the plain kernel; taller 16-bit calls expand the weights
    to the activations' type and run this provider's tiled kernel over the dense copy - or, where the provider was created with
    the opt-in library route, the library GEMM."""
    tall = a_dt != E.F32 and m >= (32 if route == "library" else 5) and k % 64 == 0
    if route == "library":
        if not tall:
            pytest.skip("the library route only differs on tall calls")
        ep = ep_dense
    b, s, zp = synth.make_weights_bits(n, k, bs, bits, 50 + bits + n, zero_points=zero_points, scale_lo=0.002 if bits == 8 else 0.02,
                                       scale_hi=0.004 if bits == 8 else 0.04, scale_dtype=s_dt)
    a = synth.make_activation(m, k, 51 + m, a_dt)
    bias = synth.to_dtype(np.linspace(-1, 1, n).astype(np.float32), a_dt)
    y, variant = run_op(ep, a, a_dt, b, s, s_dt, zp, n, k, bs, bias=bias, bias_dtype=a_dt, bits=bits)
    assert variant == (("dense_transient_blaslt" if route == "library" else "dense_transient_tiled") if tall else "gemv_nbits_f32")
    want = port.matmul_f64_bits(synth.to_f32(a, a_dt), b, synth.to_f32(s, s_dt), zp, n, k, bs, bits, bias=synth.to_f32(bias, a_dt))
    assert helpers.rel_l2(synth.to_f32(y, a_dt), want) <= (TOL_F32 if a_dt == E.F32 else TOL_HALF)


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("a_dt,bs,zero_points,m,n,k,with_bias", [
    (E.F32, 32, True, 1, 100, 256, False),
    (E.F16, 32, False, 3, 130, 1024, True),
    (E.BF16, 128, True, 16, 72, 1024, False),
    (E.F16, 64, True, 48, 136, 512, True),          # tall: dense route over weights expanded with their groups
])
@pytest.mark.parametrize("route", ["default", "library"])
def test_g_idx_matches_oracle(ep, ep_dense, port, route, bits, a_dt, bs, zero_points, m, n, k, with_bias):
    """Act-order weights (g_idx at input 4): scale and zero point of element k come from group g_idx[k] (matmul_nbits.rs:3636-3658).
    Tall 16-bit calls expand the weights with their groups and run the tiled kernel over the dense copy (default) or the
    library GEMM (opt-in)."""
    tall = m >= (32 if route == "library" else 5) and a_dt != E.F32 and k % 64 == 0
    if route == "library":
        if not tall:
            pytest.skip("the library route only differs on tall calls")
        ep = ep_dense
    kb = k // bs
    if bits == 4:
        b, s, zp = synth.make_weights(n, k, bs, 60 + n, zero_points=zero_points, scale_lo=0.005, scale_hi=0.02, scale_dtype=a_dt)
    else:
        b, s, zp = synth.make_weights_bits(n, k, bs, bits, 60 + n, zero_points=zero_points, scale_lo=0.001, scale_hi=0.003, scale_dtype=a_dt)
    g = np.random.default_rng(k + bits).integers(0, kb, size=k).astype(np.int32)
    a = synth.make_activation(m, k, 61 + m, a_dt)
    bias = synth.to_dtype(np.linspace(-1, 1, n).astype(np.float32), a_dt) if with_bias else None
    y, variant = run_op(ep, a, a_dt, b, s, a_dt, zp, n, k, bs, bias=bias, bias_dtype=a_dt, bits=bits, g_idx=g)
    assert variant == (("dense_transient_blaslt" if route == "library" else "dense_transient_tiled") if tall else "gemv_nbits_f32")
    w = port.dequantize_nk_gidx(b, synth.to_f32(s, a_dt), zp, g, n, k, bs, bits).astype(np.float64)
    want = synth.to_f32(a, a_dt).astype(np.float64) @ w.T + (synth.to_f32(bias, a_dt).astype(np.float64) if with_bias else 0.0)
    assert helpers.rel_l2(synth.to_f32(y, a_dt), want) <= (TOL_F32 if a_dt == E.F32 else TOL_HALF)
    if m == 1:                                         # the identity grouping is the plain operator
        ident = (np.arange(k) // bs).astype(np.int32)
        y0, _ = run_op(ep, a, a_dt, b, s, a_dt, zp, n, k, bs, bits=bits, g_idx=ident)
        plain = port.matmul_f64_bits(synth.to_f32(a, a_dt), b, synth.to_f32(s, a_dt), zp, n, k, bs, bits)
        assert helpers.rel_l2(synth.to_f32(y0, a_dt), plain) <= TOL_F32


def test_g_idx_out_of_range_is_an_error(ep):
    a_dt, bs, n, k = E.F16, 32, 16, 128
    b, s, zp = synth.make_weights(n, k, bs, 3, zero_points=True, scale_lo=0.005, scale_hi=0.02, scale_dtype=a_dt)
    g = (np.arange(k) // bs).astype(np.int32)
    g[77] = k // bs
    with pytest.raises(E.EpError, match=r"g_idx\[77\] is outside 0\.\.4"):
        run_op(ep, synth.make_activation(1, k, 1, a_dt), a_dt, b, s, a_dt, zp, n, k, bs, g_idx=g)
    with pytest.raises(E.EpError, match="accuracy_level=4 does not take g_idx"):
        run_op(ep, synth.make_activation(1, k, 1, a_dt), a_dt, b, s, a_dt, zp, n, k, bs, g_idx=(np.arange(k) // bs).astype(np.int32), accuracy_level=4)


def test_other_bit_widths_validation(ep):
    with pytest.raises(E.EpError, match="bits in {2, 4, 8}"):
        ep.get_kernel({"K": 64, "N": 8, "bits": 3, "block_size": 32})
    with pytest.raises(E.EpError, match="accuracy_level=4 is implemented for bits=4 only"):
        ep.get_kernel({"K": 64, "N": 8, "bits": 8, "block_size": 32, "accuracy_level": 4})
    n, k, bs = 8, 64, 32
    b4, s, _ = synth.make_weights(n, k, bs, 1, zero_points=False, scale_lo=0.01, scale_hi=0.02, scale_dtype=E.F16)
    a = synth.make_activation(1, k, 1, E.F16)
    ops = E.DeviceOperands(ep, b4, s, E.F16, None, n, k, bs, bits=8)       # 4-bit sized B on an 8-bit node
    ab, yb = ep.upload(a), ep.allocate(n * 2)
    try:
        views = ops.views(ab, E.F16, 1)
        views[1] = E.TensorView(ops.b.ptr, E.U8, (n, k // bs, bs // 2), device_index=ep.device_index)
        with pytest.raises(E.EpError, match=r"B must have shape \[8, 2, 32\]"):
            ops.kernel.execute(views, [E.TensorView(yb.ptr, E.F16, (1, n), device_index=ep.device_index)])
    finally:
        ep.deallocate(ab)
        ep.deallocate(yb)
        ops.free()


# ---------------------------------------------------------------------------------------------
# fused gate/up node: silu(gate) * up over both projections, rounded as the separate nodes round
# ---------------------------------------------------------------------------------------------
SWIGLU_CASES = [
    # a_dt, s_dt, bs, zero points, m, n, k, decomposed
    (E.F16, E.F16, 32, False, 1, 300, 896, False),
    (E.F16, E.F16, 32, True, 1, 4864, 896, True),
    (E.BF16, E.BF16, 128, True, 1, 1000, 3584, False),
    (E.BF16, E.BF16, 128, True, 4, 520, 1024, True),
    (E.F16, E.F32, 64, True, 3, 130, 512, False),
    (E.F16, E.F16, 32, True, 16, 200, 1024, False),
    (E.BF16, E.BF16, 128, False, 8, 16400, 512, False),
    (E.F16, E.F16, 64, True, 100, 136, 1024, False),
    (E.F16, E.F16, 32, False, 1100, 136, 512, True),
]


@pytest.mark.parametrize("a_dt,s_dt,bs,zero_points,m,n,k,decomposed", SWIGLU_CASES)
def test_gate_up_swiglu(ep_unpacked, port, a_dt, s_dt, bs, zero_points, m, n, k, decomposed):
    """The fused node equals, bit for bit, the oracle's epilogue applied to this provider's own two projections (the node's
    contract: 'identical to the separate kernels'), and is within the 16-bit bar of the epilogue applied to f64 projections.
    Run without repacked copies: over those a pair splits K as one launch of twice the columns would, which a projection
    launched alone does not (test_gate_up_swiglu_single_launch covers that path)."""
    ep = ep_unpacked
    gate = synth.make_weights(n, k, bs, 810 + n, zero_points=zero_points, scale_lo=0.004, scale_hi=0.02, scale_dtype=s_dt)
    up = synth.make_weights(n, k, bs, 811 + n, zero_points=zero_points, scale_lo=0.004, scale_hi=0.02, scale_dtype=s_dt)
    a = synth.make_activation(m, k, 812 + m, a_dt)
    o_dt = oracle.F16 if a_dt == E.F16 else oracle.BF16
    y, variant = E.gate_up_swiglu(ep, a, a_dt, gate, up, s_dt, n, k, bs, decomposed=decomposed)
    assert variant.startswith("gate_up_swiglu")
    g16, _ = run_op(ep, a, a_dt, gate[0], gate[1], s_dt, gate[2], n, k, bs)
    u16, _ = run_op(ep, a, a_dt, up[0], up[1], s_dt, up[2], n, k, bs)
    want = port.swiglu(g16, u16, o_dt, decomposed)
    assert np.array_equal(np.asarray(y).view(np.uint16), np.asarray(want).view(np.uint16))
    g64 = oracle_f64(port, a, a_dt, gate[0], gate[1], s_dt, gate[2], n, k, bs)
    u64 = oracle_f64(port, a, a_dt, up[0], up[1], s_dt, up[2], n, k, bs)
    ideal = g64 / (1.0 + np.exp(-g64)) * u64
    assert helpers.rel_l2(synth.to_f32(y, a_dt), ideal) <= 2 * TOL_HALF


@pytest.mark.parametrize("a_dt,s_dt,bs,zero_points,m,n,k,decomposed", [c for c in SWIGLU_CASES if c[4] <= 4] + [
    (E.BF16, E.BF16, 128, True, 1, 18944, 3584, False),      # the 7B gate/up pair at full size: seven waves per projection
    (E.F16, E.F16, 32, True, 2, 96, 4096, False),            # more waves per projection than half a workgroup holds: each takes half, two tile groups a wave
    (E.BF16, E.BF16, 64, True, 1, 520, 8192 + 64, True),     # ... five tile groups a wave, the last one partial
    (E.F16, E.F16, 32, True, 2, 96, 16384, False),           # eight tile groups a wave would be too many: stays on two launches
])
def test_gate_up_swiglu_single_launch(ep, port, a_dt, s_dt, bs, zero_points, m, n, k, decomposed):
    """From the second call on, up to four rows over constant weights run as one launch over both repacked copies, with
    the result of the first call (two launches and the epilogue) bit for bit - also when replayed from a HIP graph."""
    gate = synth.make_weights(n, k, bs, 810 + n, zero_points=zero_points, scale_lo=0.004, scale_hi=0.02, scale_dtype=s_dt)
    up = synth.make_weights(n, k, bs, 811 + n, zero_points=zero_points, scale_lo=0.004, scale_hi=0.02, scale_dtype=s_dt)
    a = synth.make_activation(m, k, 812 + m, a_dt)
    ops = E.GateUpOperands(ep, gate, up, s_dt, n, k, bs, decomposed=decomposed)
    ab, yb = ep.upload(a), ep.allocate(m * n * 2)
    try:
        ops.run(ab, a_dt, m, yb)
        first = ep.download(yb, (m, n), np.uint16).copy()
        assert ops.kernel.last_variant() == "gate_up_swiglu[decode_mfma_packed]"
        ep.copy_from_host(yb, np.full(m * n * 2, 0xFF, np.uint8))
        ops.run(ab, a_dt, m, yb)
        half_workgroup = 8 if bs == 128 and s_dt != E.F32 else 4           # waves a projection may take in the paired launch
        single = -(-(-(-k // 512)) // half_workgroup) <= 5
        assert ops.kernel.last_variant() == ("gate_up_swiglu_packed" if single else "gate_up_swiglu[decode_mfma_packed]")
        assert np.array_equal(ep.download(yb, (m, n), np.uint16), first)
        ep.sync()
        ep.capture_begin()
        try:
            ops.run(ab, a_dt, m, yb)
        finally:
            graph = ep.capture_end()
        ep.copy_from_host(yb, np.full(m * n * 2, 0xFF, np.uint8))
        graph.replay()
        assert np.array_equal(ep.download(yb, (m, n), np.uint16), first)
        graph.release()
        g64 = oracle_f64(port, a, a_dt, gate[0], gate[1], s_dt, gate[2], n, k, bs)
        u64 = oracle_f64(port, a, a_dt, up[0], up[1], s_dt, up[2], n, k, bs)
        ideal = g64 / (1.0 + np.exp(-g64)) * u64
        assert helpers.rel_l2(synth.to_f32(first.view(NPDT[a_dt]), a_dt), ideal) <= 2 * TOL_HALF
    finally:
        ep.deallocate(ab)
        ep.deallocate(yb)
        ops.free()


@pytest.mark.parametrize("a_dt,s_dt,bs,m,n,k,decomposed", [
    (E.BF16, E.BF16, 128, 16, 18944, 3584, False),    # the 7B pair: fewer workgroups than CUs per projection alone (weights and windows ahead)
    (E.BF16, E.BF16, 128, 4, 18944, 3584, True),      # four rows at block 128 with 18432 .. 49151 columns in the pair: this kernel too
    (E.F16, E.F16, 128, 4, 9216, 512, False),          # ... its lower edge
    (E.BF16, E.BF16, 128, 2, 18944, 1024, False),     # ... a pair from two rows
    (E.F16, E.F32, 128, 3, 9300, 640, True),
    (E.BF16, E.BF16, 128, 5, 14336, 512, True),
    (E.F16, E.F16, 64, 9, 14400, 640, False),         # ragged: the last workgroup's waves run out of column groups
    (E.F16, E.F32, 32, 16, 14336, 256, False),
    (E.BF16, E.BF16, 128, 8, 98400, 256, False),      # three or more workgroups per CU: the build with the second MFMA
    (E.BF16, E.BF16, 32, 6, 18944, 512, False),       # block 32: the second-MFMA build with weights ahead, in both projections and in the pair
    (E.F16, E.F16, 64, 8, 37888, 256, True),          # block 64 where one projection alone gets a balanced grid (second MFMA): the pair follows it
])
def test_gate_up_swiglu_single_launch_at_5_to_16_rows(ep, port, a_dt, s_dt, bs, m, n, k, decomposed):
    """5 to 16 rows where both projections are wide enough for the shared-activation kernel: from the second call on one
    launch whose workgroups hold four column groups of each projection; the result of the first call (two launches and the
    epilogue) bit for bit, also replayed from a HIP graph, and the oracle's SwiGLU of the two projections rounded to 16 bits."""
    gate = synth.make_weights(n, k, bs, 850 + m, zero_points=True, scale_lo=0.004, scale_hi=0.02, scale_dtype=s_dt)
    up = synth.make_weights(n, k, bs, 851 + m, zero_points=True, scale_lo=0.004, scale_hi=0.02, scale_dtype=s_dt)
    a = synth.make_activation(m, k, 852 + m, a_dt)
    ops = E.GateUpOperands(ep, gate, up, s_dt, n, k, bs, decomposed=decomposed)
    ab, yb = ep.upload(a), ep.allocate(m * n * 2)
    try:
        ops.run(ab, a_dt, m, yb)
        first = ep.download(yb, (m, n), np.uint16).copy()
        assert ops.kernel.last_variant() == "gate_up_swiglu[decode_mfma_packed]"
        ep.copy_from_host(yb, np.full(m * n * 2, 0xFF, np.uint8))
        ops.run(ab, a_dt, m, yb)
        assert ops.kernel.last_variant() == "gate_up_swiglu_packed"
        assert np.array_equal(ep.download(yb, (m, n), np.uint16), first)
        ep.sync()
        ep.capture_begin()
        try:
            ops.run(ab, a_dt, m, yb)
        finally:
            graph = ep.capture_end()
        ep.copy_from_host(yb, np.full(m * n * 2, 0xFF, np.uint8))
        graph.replay()
        assert np.array_equal(ep.download(yb, (m, n), np.uint16), first)
        graph.release()
        # against the oracle on a sample of columns (the last 16 included): each projection rounded to 16 bits, then the epilogue
        cols = np.unique(np.concatenate([np.linspace(0, n - 1, 64).astype(np.int64), np.arange(n - 16, n)]))
        o_dt = oracle.F16 if a_dt == E.F16 else oracle.BF16
        sub = lambda w: (np.ascontiguousarray(w[0][cols]), np.ascontiguousarray(w[1][cols]), np.ascontiguousarray(w[2][cols]))
        g16, _ = run_op(ep, a, a_dt, *sub(gate)[:2], s_dt, sub(gate)[2], len(cols), k, bs)
        u16, _ = run_op(ep, a, a_dt, *sub(up)[:2], s_dt, sub(up)[2], len(cols), k, bs)
        want = port.swiglu(g16, u16, o_dt, decomposed)
        got = first.reshape(m, n)[:, cols]
        # the narrow sub-problem runs another kernel (other summation order): compare in value, not in bits
        assert helpers.rel_l2(synth.to_f32(got.view(NPDT[a_dt]), a_dt), synth.to_f32(np.asarray(want), a_dt)) <= 2 * TOL_HALF
        g64 = oracle_f64(port, a, a_dt, *sub(gate)[:2], s_dt, sub(gate)[2], len(cols), k, bs)
        u64 = oracle_f64(port, a, a_dt, *sub(up)[:2], s_dt, sub(up)[2], len(cols), k, bs)
        ideal = g64 / (1.0 + np.exp(-g64)) * u64
        assert helpers.rel_l2(synth.to_f32(got.view(NPDT[a_dt]), a_dt), ideal) <= 2 * TOL_HALF
    finally:
        ep.deallocate(ab)
        ep.deallocate(yb)
        ops.free()


RMSNORM_CASES = [
    # a_dt, gamma dtype, bs, m, n, k, epsilon
    (E.F16, E.F16, 32, 1, 300, 896, 1e-6),
    (E.F16, E.F32, 32, 3, 136, 1024, 1e-5),
    (E.BF16, E.BF16, 128, 1, 520, 3584, 1e-6),
    (E.BF16, E.F32, 128, 16, 200, 1024, 1e-5),
    (E.F16, E.F16, 64, 100, 136, 512, 1e-5),
    # up to four rows over constant weights: normalized inside the decode kernel - one row and four, both gamma types, every
    # block size, K over several waves, few and many workgroups (with and without the second register set)
    (E.BF16, E.F32, 128, 1, 4608, 3584, 1e-6),
    (E.BF16, E.BF16, 128, 4, 520, 3584, 1e-6),
    (E.F16, E.F32, 64, 2, 333, 2048, 1e-5),
    (E.F16, E.F16, 64, 1, 24576, 512, 1e-5),
    (E.F16, E.F16, 32, 4, 24576, 512, 1e-6),
    (E.BF16, E.F32, 32, 3, 100, 128 * 9, 1e-5),
    (E.F16, E.F32, 128, 4, 77, 128 * 40, 1e-5),
]


def test_gate_up_swiglu_at_accuracy_level_4_stays_on_the_int8_kernels(ep):
    """A fused gate/up node with accuracy_level 4 runs both projections through the int8 path on every call: the float
    single-launch form (which the repacked copies of the first call would make available) must not take later calls."""
    a_dt, bs, m, n, k = E.F16, 64, 1, 160, 1024
    gate = synth.make_weights(n, k, bs, 801, zero_points=True, scale_lo=0.002, scale_hi=0.01, scale_dtype=a_dt)
    up = synth.make_weights(n, k, bs, 802, zero_points=True, scale_lo=0.002, scale_hi=0.01, scale_dtype=a_dt)
    a = synth.make_activation(m, k, 803, a_dt)
    ops = E.GateUpOperands(ep, gate, up, a_dt, n, k, bs, accuracy_level=4)
    ab, yb = ep.upload(a), ep.allocate(m * n * 2)
    try:
        outs, variants = [], []
        for _ in range(3):
            ops.run(ab, a_dt, m, yb)
            outs.append(ep.download(yb, (m, n), np.uint16).copy())
            variants.append(ops.kernel.last_variant())
        assert variants[0] == variants[1] == variants[2] == "gate_up_swiglu[acc4_mfma_i8_packed]", variants
        assert np.array_equal(outs[0], outs[1]) and np.array_equal(outs[0], outs[2])
    finally:
        ep.deallocate(ab)
        ep.deallocate(yb)
        ops.free()


@pytest.mark.parametrize("a_dt,g_dt,bs,m,n,k,eps", RMSNORM_CASES)
def test_rmsnorm_prologue(ep, ep_unpacked, port, a_dt, g_dt, bs, m, n, k, eps):
    """A node with the RMS-normalization prologue gives, bit for bit, what the same node without it gives on activations the
    oracle normalized: the prologue's kernel equals the oracle's restatement (sums in the reference's order) on every element
    that matters to the product."""
    b, s, zp = synth.make_weights(n, k, bs, 820 + n, zero_points=True, scale_lo=0.002, scale_hi=0.01, scale_dtype=a_dt)
    a = synth.make_activation(m, k, 821 + m, a_dt)
    gamma = synth.to_dtype((1.0 + 0.25 * np.random.default_rng(k).standard_normal(k)).astype(np.float32), g_dt)
    o_dt = oracle.F16 if a_dt == E.F16 else oracle.BF16
    g_code = oracle.F32 if g_dt == E.F32 else o_dt
    normalized = port.rmsnorm16(np.asarray(a).reshape(m, k), gamma, g_code, eps, o_dt)
    y, variant = run_op(ep, a, a_dt, b, s, a_dt, zp, n, k, bs, gamma=gamma, gamma_dtype=g_dt, rmsnorm_epsilon=eps)
    want, plain_variant = run_op(ep, normalized, a_dt, b, s, a_dt, zp, n, k, bs)
    # up to four rows over the repacked stream, up to 8192 columns: the decode kernel normalizes the rows itself; otherwise a
    # launch of its own does
    assert variant == ("rmsnorm[decode_mfma_packed]" if m <= 4 and n <= 8192 else "rmsnorm+" + plain_variant)
    assert np.array_equal(np.asarray(y).view(np.uint16), np.asarray(want).view(np.uint16))
    if m <= 4 and n > 8192:
        # the in-kernel form at this width too, where the setting allows it
        wide = E.RocmExecutionProvider(0, {"rmsnorm_in_kernel_max_cols": str(n)})
        try:
            y3, variant3 = run_op(wide, a, a_dt, b, s, a_dt, zp, n, k, bs, gamma=gamma, gamma_dtype=g_dt, rmsnorm_epsilon=eps)
        finally:
            wide.shutdown()
        assert variant3 == "rmsnorm[decode_mfma_packed]"
        assert np.array_equal(np.asarray(y3).view(np.uint16), np.asarray(want).view(np.uint16))
    if m <= 4:
        # the same node where nothing is repacked: the separate normalization launch, the same bits
        y2, variant2 = run_op(ep_unpacked, a, a_dt, b, s, a_dt, zp, n, k, bs, gamma=gamma, gamma_dtype=g_dt, rmsnorm_epsilon=eps)
        assert variant2 == "rmsnorm+decode_mfma_splitk"
        assert helpers.rel_l2(synth.to_f32(y2, a_dt), synth.to_f32(want, a_dt)) <= TOL_HALF
    # and the normalization is one: mean square of the normalized row over gamma^2 is 1 within the 16-bit roundings
    nf = synth.to_f32(normalized, a_dt) / synth.to_f32(gamma, g_dt)[None, :]
    assert np.allclose(np.mean(nf.astype(np.float64) ** 2, axis=1), 1.0, rtol=2e-2)


def test_rmsnorm_prologue_on_the_fused_gate_up_node(ep, port):
    a_dt, bs, m, n, k, eps = E.F16, 32, 2, 200, 1024, 1e-6
    gate = synth.make_weights(n, k, bs, 830, zero_points=True, scale_lo=0.004, scale_hi=0.02, scale_dtype=a_dt)
    up = synth.make_weights(n, k, bs, 831, zero_points=True, scale_lo=0.004, scale_hi=0.02, scale_dtype=a_dt)
    a = synth.make_activation(m, k, 832, a_dt)
    gamma = (1.0 + 0.25 * np.random.default_rng(7).standard_normal(k)).astype(np.float32)
    normalized = port.rmsnorm16(np.asarray(a).reshape(m, k), gamma, oracle.F32, eps, oracle.F16)
    y, variant = E.gate_up_swiglu(ep, a, a_dt, gate, up, a_dt, n, k, bs, gamma=gamma, gamma_dtype=E.F32, rmsnorm_epsilon=eps)
    want, _ = E.gate_up_swiglu(ep, normalized, a_dt, gate, up, a_dt, n, k, bs)
    assert variant.startswith("rmsnorm+gate_up_swiglu")
    assert np.array_equal(np.asarray(y).view(np.uint16), np.asarray(want).view(np.uint16))


@pytest.mark.parametrize("a_dt,g_dt,bs,m,n,k", [(E.F16, E.F32, 32, 2, 200, 1024), (E.BF16, E.BF16, 128, 1, 2368, 3584), (E.BF16, E.F32, 128, 4, 300, 3584),
                                                (E.F16, E.F16, 64, 3, 100, 512)])
def test_rmsnorm_prologue_inside_the_single_launch_gate_up_node(ep, port, a_dt, g_dt, bs, m, n, k):
    """Calls after the first (which repacks both projections) run normalization, both projections and the SwiGLU epilogue as
    one launch; the result equals, bit for bit, the first call's (separate normalization launch, separate projections) and
    the node without the prologue on rows the oracle normalized."""
    eps = 1e-6
    gate = synth.make_weights(n, k, bs, 840, zero_points=True, scale_lo=0.004, scale_hi=0.02, scale_dtype=a_dt)
    up = synth.make_weights(n, k, bs, 841, zero_points=True, scale_lo=0.004, scale_hi=0.02, scale_dtype=a_dt)
    a = synth.make_activation(m, k, 842, a_dt)
    gamma = synth.to_dtype((1.0 + 0.25 * np.random.default_rng(8).standard_normal(k)).astype(np.float32), g_dt)
    o_dt = oracle.F16 if a_dt == E.F16 else oracle.BF16
    normalized = port.rmsnorm16(np.asarray(a).reshape(m, k), gamma, oracle.F32 if g_dt == E.F32 else o_dt, eps, o_dt)
    want, _ = E.gate_up_swiglu(ep, normalized, a_dt, gate, up, a_dt, n, k, bs)
    ops = E.GateUpOperands(ep, gate, up, a_dt, n, k, bs, gamma=gamma, gamma_dtype=g_dt, rmsnorm_epsilon=eps)
    ab, yb = ep.upload(a), ep.allocate(m * n * 2)
    try:
        outs, variants = [], []
        for _ in range(3):
            ops.run(ab, a_dt, m, yb)
            outs.append(ep.download(yb, (m, n), np.uint16).copy())
            variants.append(ops.kernel.last_variant())
        assert variants[0].startswith("rmsnorm+gate_up_swiglu[")
        assert variants[1] == variants[2] == "rmsnorm[gate_up_swiglu_packed]", variants
        for got in outs:
            assert np.array_equal(got, np.asarray(want).view(np.uint16))
    finally:
        ep.deallocate(ab)
        ep.deallocate(yb)
        ops.free()


def test_rmsnorm_prologue_validation(ep):
    a_dt, bs, n = E.F16, 32, 64
    for k, match in ((192, "multiple of 128"), (256, "normalization weight at input 6")):
        b, s, zp = synth.make_weights(n, k, bs, 1, zero_points=True, scale_lo=0.004, scale_hi=0.02, scale_dtype=a_dt)
        ops = E.DeviceOperands(ep, b, s, a_dt, zp, n, k, bs, gamma=np.ones(k, np.float32), gamma_dtype=E.F32)
        a, y = ep.upload(synth.make_activation(2, k, 3, a_dt)), ep.allocate(2 * n * 2)
        try:
            views = ops.views(a, a_dt, 2)
            out = [E.TensorView(y.ptr, a_dt, (2, n), device_index=ep.device_index)]
            with pytest.raises(E.EpError, match=match):
                ops.kernel.execute(views if k == 192 else views[:6], out)
        finally:
            ep.deallocate(a)
            ep.deallocate(y)
            ops.free()


def test_gate_up_swiglu_validation(ep):
    a_dt, bs, n, k = E.F16, 32, 64, 128
    gate = synth.make_weights(n, k, bs, 1, zero_points=True, scale_lo=0.004, scale_hi=0.02, scale_dtype=a_dt)
    up = synth.make_weights(n, k, bs, 2, zero_points=True, scale_lo=0.004, scale_hi=0.02, scale_dtype=a_dt)
    ops = E.GateUpOperands(ep, gate, up, a_dt, n, k, bs)
    a, y = ep.upload(synth.make_activation(2, k, 3, a_dt)), ep.allocate(2 * n * 2)
    try:
        assert ops.kernel.workspace_requirement([((2, k), a_dt)])[0] == 2 * 256
        views = ops.views(a, a_dt, 2)
        out = [E.TensorView(y.ptr, a_dt, (2, n), device_index=ep.device_index)]
        with pytest.raises(E.EpError, match="both projections or neither"):
            ops.kernel.execute(views[:7], out)
        with pytest.raises(E.EpError, match="expects 5 to 8 inputs"):
            ops.kernel.execute(views[:4], out)
        gamma = list(views)
        gamma[5] = E.TensorView(a.ptr, a_dt, (k,), device_index=ep.device_index)
        with pytest.raises(E.EpError, match="no RMS-norm prologue marker"):
            ops.kernel.execute(gamma, out)
        with pytest.raises(E.EpError, match="Y must have dtype"):
            ops.kernel.execute(views, [E.TensorView(y.ptr, E.F32, (2, n), device_index=ep.device_index)])
        ops.kernel.execute(views, out)                       # and the well-formed call goes through
    finally:
        ep.deallocate(a)
        ep.deallocate(y)
        ops.free()


# ---------------------------------------------------------------------------------------------
# dense route: weights expanded to 16 bits, then the library GEMM (tall calls)
# ---------------------------------------------------------------------------------------------
DENSE_CASES = [
    # a_dt, s_dt, bs, zp, m, n, k, bias dtype (None = no bias)
    (E.F16, E.F16, 32, False, 200, 256, 512, E.F16),
    (E.F16, E.F32, 64, True, 96, 120, 256, None),
    (E.F16, E.F16, 128, True, 1030, 136, 1024, E.F32),
    (E.BF16, E.BF16, 128, True, 130, 384, 3584, E.F32),
    (E.BF16, E.BF16, 32, False, 64, 100, 128, E.BF16),
    (E.BF16, E.F32, 16, True, 257, 72, 136, None),
]


@pytest.mark.parametrize("mode", ["transient", "resident"])
@pytest.mark.parametrize("a_dt,s_dt,bs,zero_points,m,n,k,bias_dt", DENSE_CASES)
def test_dense_route_matches_oracle(port, mode, a_dt, s_dt, bs, zero_points, m, n, k, bias_dt):
    provider = E.RocmExecutionProvider(0, {"dense_gemm_min_rows": "64", "dense_weights": mode})
    try:
        b, s, zp = synth.make_weights(n, k, bs, 500 + n + k, zero_points=zero_points, scale_lo=0.001, scale_hi=0.01, scale_dtype=s_dt)
        a = synth.make_activation(m, k, n, a_dt)
        bias = None if bias_dt is None else synth.to_dtype(np.random.default_rng(n).standard_normal(n).astype(np.float32), bias_dt)
        want64 = oracle_f64(port, a, a_dt, b, s, s_dt, zp, n, k, bs, bias, bias_dt if bias_dt is not None else E.F32)
        y, variant = run_op(provider, a, a_dt, b, s, s_dt, zp, n, k, bs, bias=bias, bias_dtype=bias_dt if bias_dt is not None else E.F32)
        assert variant == "dense_%s_blaslt" % mode
        assert helpers.rel_l2(synth.to_f32(y, a_dt), want64) <= TOL_HALF
    finally:
        provider.shutdown()


@pytest.mark.parametrize("a_dt,s_dt", [(E.F16, E.F16), (E.BF16, E.BF16), (E.BF16, E.F32)])
@pytest.mark.parametrize("bs,zero_points", [(32, True), (128, False)])
def test_dense_weights_are_the_f32_dequant_rounded_once(port, a_dt, s_dt, bs, zero_points):
    """One-hot activation rows read single weights back out of the library GEMM: each must equal the f32 dequantized
    weight rounded once to the 16-bit type, bit for bit (a product by 1 and sums with zeros are exact)."""
    m, n, k = 64, 256, 256
    provider = E.RocmExecutionProvider(0, {"dense_gemm_min_rows": "64"})
    try:
        b, s, zp = synth.make_weights(n, k, bs, 300 + bs, zero_points=zero_points, scale_lo=0.001, scale_hi=0.01, scale_dtype=s_dt)
        ks = (np.arange(m) * 37) % k
        a32 = np.zeros((m, k), np.float32)
        a32[np.arange(m), ks] = 1.0
        y, variant = run_op(provider, synth.to_dtype(a32, a_dt), a_dt, b, s, s_dt, zp, n, k, bs)
        assert variant == "dense_transient_blaslt"
        w = port.dequantize_nk(b, synth.to_f32(s, s_dt), zp, n, k, bs)            # f32 [N, K], bit-exact reference definition
        want = port.narrow(np.ascontiguousarray(w[:, ks].T), oracle.F16 if a_dt == E.F16 else oracle.BF16)
        assert np.array_equal(np.asarray(y).view(np.uint16), np.asarray(want).view(np.uint16))
    finally:
        provider.shutdown()


def test_dense_route_declines_what_it_cannot_take(port):
    """f32 outputs, short calls and weights beyond the configured size stay on the hand-written kernels; so does a first
    use while a graph capture is open (the route may not allocate then), and the captured call still gives the result."""
    a_dt, bs, m, n, k = E.F16, 32, 128, 128, 256
    b, s, zp = synth.make_weights(n, k, bs, 77, zero_points=True, scale_lo=0.002, scale_hi=0.01, scale_dtype=a_dt)
    a = synth.make_activation(m, k, 77, a_dt)
    want = oracle_f64(port, a, a_dt, b, s, a_dt, zp, n, k, bs)
    provider = E.RocmExecutionProvider(0, {"dense_gemm_min_rows": "64"})
    small = E.RocmExecutionProvider(0, {"dense_gemm_min_rows": "64", "dense_gemm_max_mb": "0"})
    try:
        y32, variant = run_op(provider, a, a_dt, b, s, a_dt, zp, n, k, bs, y_dtype=E.F32)
        assert variant == "prefill_mfma_lds" and helpers.rel_l2(y32, want) <= TOL_HALF
        _, variant = run_op(provider, a[:48], a_dt, b, s, a_dt, zp, n, k, bs)
        assert variant == "prefill_mfma_lds"
        _, variant = run_op(small, a, a_dt, b, s, a_dt, zp, n, k, bs)
        assert variant == "prefill_mfma_lds"
        # first use inside a capture
        fresh = E.RocmExecutionProvider(0, {"dense_gemm_min_rows": "64"})
        try:
            ops = E.DeviceOperands(fresh, b, s, a_dt, zp, n, k, bs)
            ab, yb = fresh.upload(a), fresh.allocate(m * n * 2)
            fresh.sync()
            fresh.capture_begin()
            try:
                ops.run(ab, a_dt, m, yb)
            finally:
                graph = fresh.capture_end()
            assert ops.kernel.last_variant() == "prefill_mfma_lds"
            graph.replay()
            got = fresh.download(yb, (m, n), np.float16)
            assert helpers.rel_l2(got.astype(np.float32), want) <= TOL_HALF
            graph.release()
            ops.run(ab, a_dt, m, yb)                     # outside the capture the route sets itself up
            assert ops.kernel.last_variant() == "dense_transient_blaslt"
            assert helpers.rel_l2(fresh.download(yb, (m, n), np.float16).astype(np.float32), want) <= TOL_HALF
            fresh.deallocate(ab)
            fresh.deallocate(yb)
            ops.free()
        finally:
            fresh.shutdown()
    finally:
        provider.shutdown()
        small.shutdown()


# ---------------------------------------------------------------------------------------------
# accuracy_level = 4
# ---------------------------------------------------------------------------------------------
def _tie_heavy_activation(m, k, bs, seed, dtype):
    """N(0,1) rows plus blocks built to hit exact .5 ties, all-zero blocks and +-max codes."""
    rng = np.random.default_rng(seed)
    a = rng.standard_normal((m, k)).astype(np.float32)
    blocks = k // bs
    if blocks >= 3:
        a[0, 0:bs] = 0.0                                              # all-zero block: scale 0, codes 0
        a[0, bs:2 * bs] = (rng.integers(-253, 254, size=bs) * 0.5).astype(np.float32)
        a[0, bs] = 127.0                                              # max = 127 -> inv = 1 -> halves are exact ties
        a[0, bs + 1] = -127.0
        a[0, 2 * bs:3 * bs] = np.float32(3.0)                         # every element is the maximum
    return synth.to_dtype(a, dtype)


@pytest.mark.parametrize("a_dt", [E.F32, E.F16, E.BF16])
@pytest.mark.parametrize("bs", [16, 32, 64, 128])
@pytest.mark.parametrize("rounding", [oracle.ROUND_HALF_EVEN, oracle.ROUND_HALF_AWAY])
def test_quantize_a_bit_exact(ep, port, ref, a_dt, bs, rounding):
    m, k = 5, 4 * bs + (bs // 2)
    a = _tie_heavy_activation(m, k, bs, 40 + bs, a_dt)
    af = synth.to_f32(a, a_dt)
    kb = -(-k // bs)
    want_q, want_s = port.quantize_a(af, k, bs, rounding)
    ab, qb, sb = ep.upload(a), ep.allocate(m * kb * bs), ep.allocate(m * kb * 4)
    ep.quantize_a(ab, a_dt, m, k, bs, rounding, qb, sb)
    got_q = ep.download(qb, (m, kb * bs), np.int8)
    got_s = ep.download(sb, (m, kb), np.float32)
    for buf in (ab, qb, sb):
        ep.deallocate(buf)
    assert np.array_equal(got_q, want_q)
    assert np.array_equal(got_s.view(np.uint32), want_s.view(np.uint32))
    if rounding == oracle.ROUND_HALF_EVEN:                            # the reference's compiled MLAS quantizer
        r = ref.quantize_a(af, k, bs)
        assert r is not None
        assert np.array_equal(got_q, r[0]) and np.array_equal(got_s.view(np.uint32), r[1].view(np.uint32))
    assert (want_q != port.quantize_a(af, k, bs, 1 - rounding)[0]).any()   # the fixture does separate the two rules


@pytest.mark.parametrize("bs,zero_points", [(16, True), (32, False), (64, True), (128, True)])
def test_block_accumulators_bit_exact(ep, port, bs, zero_points):
    m, n, k = 6, 50, 5 * bs
    b, _, zp = synth.make_weights(n, k, bs, 60 + bs, zero_points=zero_points, scale_lo=0.01, scale_hi=0.02, scale_dtype=E.F32)
    a = synth.make_activation(m, k, 60, E.F32)
    qa, _ = port.quantize_a(a, k, bs, oracle.ROUND_HALF_EVEN)
    want = port.block_acc_i32(qa, b, zp, n, k, bs)
    kb = k // bs
    qb, bb = ep.upload(qa), ep.upload(b)
    zb = ep.upload(zp) if zp is not None else None
    acc = ep.allocate(m * n * kb * 4)
    ep.block_acc(qb, bb, zb, m, n, k, bs, acc)
    got = ep.download(acc, (m, n, kb), np.int32)
    for buf in (qb, bb, zb, acc):
        if buf is not None:
            ep.deallocate(buf)
    assert np.array_equal(got, want)
    # independent integer check of the oracle itself on the same operands
    q = synth.unpack_nibbles(b.reshape(n, kb, bs // 2), bs).astype(np.int64)
    z = synth.unpack_nibbles(zp, kb).astype(np.int64) if zp is not None else np.full((n, kb), 8, np.int64)
    brute = np.einsum("mbk,nbk->mnb", qa.reshape(m, kb, bs).astype(np.int64), q - z[:, :, None])
    assert np.array_equal(want.astype(np.int64), brute)


def _production_block_acc(provider, port, a, a_dt, bs, zero_points, n, k, rounding, seed):
    """Runs one accuracy_level=4 call with the accumulator probe set; returns (probe contents, oracle accumulators, y32, oracle y, variant)."""
    m = a.shape[0]
    kb = -(-k // bs)
    b, s, zp = synth.make_weights(n, k, bs, seed, zero_points=zero_points, scale_lo=0.002, scale_hi=0.01, scale_dtype=a_dt)
    ops = E.DeviceOperands(provider, b, s, a_dt, zp, n, k, bs, accuracy_level=4)
    probe = provider.upload(np.full(m * n * kb, 0x7FFFFFFF, np.int32))                     # a sentinel no accumulator can reach
    ab, yb = provider.upload(a), provider.allocate(m * n * 4)
    try:
        ops.kernel.set_block_acc_probe(probe)
        ops.run(ab, a_dt, m, yb, E.F32)
        got = provider.download(probe, (m, n, kb), np.int32)
        y32 = provider.download(yb, (m, n), np.float32)
        variant = ops.kernel.last_variant()
        ops.kernel.set_block_acc_probe(None)
        provider.copy_from_host(probe, np.full(m * n * kb, 0x7FFFFFFF, np.int32))
        ops.run(ab, a_dt, m, yb, E.F32)                                                      # without the probe: same result, nothing stored
        assert np.array_equal(provider.download(yb, (m, n), np.float32), y32)
        assert (provider.download(probe, (m, n, kb), np.int32) == 0x7FFFFFFF).all()
    finally:
        for buf in (probe, ab, yb):
            provider.deallocate(buf)
        ops.free()
    af, sf = synth.to_f32(a, a_dt), synth.to_f32(s, a_dt)
    qa, _ = port.quantize_a(af, k, bs, rounding)
    want = port.block_acc_i32(qa, b, zp, n, k, bs)
    return got, want, y32, port.matmul_acc4_f32(af, b, sf, zp, n, k, bs, rounding), variant


PRODUCTION_ACC_CASES = [
    # bs, zero points, m, n, k, prepack - one row and 5 / 16 rows over the repacked stream and over the caller's layout (the
    # split-K kernel), the tiled kernel at 40; each with K short (one wave / one slice) and long (several waves / K in slices)
    (32, True, 1, 100, 32 * 11, True), (64, True, 1, 333, 64 * 37, True), (128, False, 1, 160, 128 * 40, True),
    (32, False, 1, 48, 32 * 9, False), (64, True, 1, 100, 64 * 50, False), (128, True, 1, 64, 128 * 24, False),
    (32, True, 5, 48, 32 * 9, True), (64, True, 5, 100, 64 * 50, True), (128, False, 5, 77, 128 * 33, True), (64, True, 16, 40, 200, True),
    (32, True, 2, 100, 32 * 37, True), (128, True, 16, 33, 128 * 21, True),
    # two to four 16-bit rows on a short call: quantized inside the kernel when no probe is set (the helper compares that run with the probing one bit for bit)
    (64, True, 3, 100, 64 * 50, True), (128, False, 4, 77, 128 * 33, True), (32, True, 4, 130, 32 * 21 + 8, True),
    (32, True, 5, 48, 32 * 9, False), (64, True, 5, 100, 64 * 50, False), (128, False, 5, 77, 128 * 33, False), (64, True, 16, 40, 200, False),
    (32, True, 40, 96, 32 * 35, True), (64, True, 40, 96, 64 * 17, True), (128, True, 130, 200, 128 * 20, True), (64, False, 40, 200, 64 * 3, True),
    (256, True, 40, 96, 256 * 3, True), (32, False, 33, 64, 200, True),
]


@pytest.mark.parametrize("a_dt", [E.F16, E.BF16, E.F32])
@pytest.mark.parametrize("bs,zero_points,m,n,k,prepack", PRODUCTION_ACC_CASES)
def test_production_kernels_block_accumulators_bit_exact(port, a_dt, bs, zero_points, m, n, k, prepack):
    """The int32 block accumulators as the production int8 matrix-core kernels hold them when they scale them into the result
    (matmul_nbits.rs:9159-9177; canonical form acc[m,n,b] = sum_k code[m,k] * (q[n,k] - zp[n,b])): read out of the one-row
    kernel over the repacked stream (with its fused quantizer for 16-bit rows), the split-K kernel and the tiled kernel, and
    compared bit for bit with the oracle's integers."""
    provider = E.RocmExecutionProvider(0, {"prepack": "1" if prepack else "0"})
    try:
        a = _tie_heavy_activation(m, k, bs, 300 + m, a_dt) if k % bs == 0 else synth.make_activation(m, k, 300 + m, a_dt)
        got, want, y32, y_want, variant = _production_block_acc(provider, port, a, a_dt, bs, zero_points, n, k, oracle.ROUND_HALF_EVEN, 310 + n)
        assert variant == ("acc4_mfma_i8_packed" if prepack and m <= 16 else "acc4_mfma_i8")
        assert not (got == 0x7FFFFFFF).any(), "an accumulator was never stored"
        assert np.array_equal(got, want)
        assert helpers.rel_l2(y32, y_want) <= TOL_F32
    finally:
        provider.shutdown()


@pytest.mark.parametrize("a_dt", [E.F16, E.BF16])
@pytest.mark.parametrize("bs", [32, 64, 128])
@pytest.mark.parametrize("rounding", ["mlas", "native"])
def test_fused_quantizer_on_ties_zero_blocks_and_extremes(port, a_dt, bs, rounding):
    """The quantizer inside the one-row kernel over the repacked stream (every f16 / bf16 decode call at accuracy_level 4 over
    constant weights) on the fixture that separates the two rounding rules: exact .5 ties, an all-zero block (scale 0, codes
    0, no division by zero), +-max codes. Codes are checked through the integers they produce, bit for bit."""
    n, k = 96, bs * 6
    provider = E.RocmExecutionProvider(0, {"acc4_rounding": rounding})
    try:
        rule = oracle.ROUND_HALF_EVEN if rounding == "mlas" else oracle.ROUND_HALF_AWAY
        a = _tie_heavy_activation(1, k, bs, 400 + bs, a_dt)
        got, want, y32, y_want, variant = _production_block_acc(provider, port, a, a_dt, bs, True, n, k, rule, 410 + bs)
        assert variant == "acc4_mfma_i8_packed"
        assert np.array_equal(got, want)
        assert (got[0, :, 0] == 0).all()                                   # the all-zero block
        assert np.isfinite(y32).all() and helpers.rel_l2(y32, y_want) <= TOL_F32
        af = synth.to_f32(a, a_dt)
        other = port.quantize_a(af, k, bs, 1 - rule)[0]
        assert (other != port.quantize_a(af, k, bs, rule)[0]).any()        # the fixture does separate the two rules
    finally:
        provider.shutdown()


ACC4_CASES = [
    (E.F16, 64, True, 1, 160, 1024),
    (E.F16, 64, True, 5, 96, 512),
    (E.F32, 32, False, 1, 128, 1024),
    (E.BF16, 128, True, 3, 77, 1024),
    (E.F16, 32, True, 20, 64, 256),
    (E.F32, 16, True, 2, 40, 80),
    (E.F16, 64, True, 1, 333, 64 * 37),       # odd block count, ragged N, several waves per workgroup
    (E.BF16, 32, True, 16, 48, 32 * 9),
    (E.F32, 128, False, 2, 17, 128 * 3),
    (E.F16, 64, True, 1, 64, 200),            # K ends inside a block
    (E.F16, 32, False, 7, 130, 4096),
    (E.F16, 128, True, 1, 512, 8192),
    (E.BF16, 128, True, 9, 100, 128 * 5 + 64),
    (E.BF16, 32, True, 1, 100, 32 * 11),      # one bf16 row: quantized inside the kernel, blocks of 4 lanes
    (E.BF16, 128, False, 1, 64, 1024),
    (E.F16, 32, False, 1, 48, 4100),          # K % 8 != 0: the separate quantizer serves the row
    # M > 16: tiled int8 MFMA kernel
    (E.F16, 64, True, 130, 200, 64 * 9),      # ragged M and N tiles
    (E.F16, 32, True, 33, 64, 32 * 7),        # K ends in the middle of a 64-code step
    (E.BF16, 128, False, 64, 128, 128 * 6),
    (E.F32, 256, True, 40, 96, 256 * 3),
    (E.F16, 64, True, 256, 256, 2048),        # few tiles of Y, long K: K in four slices + reduce
    (E.BF16, 128, True, 130, 200, 128 * 20),  # five slices of whole blocks (two steps per block)
    (E.F16, 256, False, 64, 130, 256 * 9),    # slices rounded up to whole blocks of four steps
    (E.F16, 64, True, 40, 96, 64 * 17),       # two unequal slices
    (E.F16, 32, True, 130, 200, 32 * 80),     # block size 32 (two blocks per step): five slices
    (E.BF16, 32, False, 40, 96, 32 * 35),     # block size 32, two slices, K ends in the middle of a step
    (E.F16, 32, False, 17, 130, 200),         # K ends inside a block
    (E.F16, 16, True, 20, 64, 256),           # block size 16: not a matrix-core shape
]


# every case under both rounding rules; the cases of up to 16 rows once more with the repacked path turned off
ACC4_RUNS = [case + (rounding, True) for case in ACC4_CASES for rounding in ("mlas", "native")] + \
            [case + ("mlas", False) for case in ACC4_CASES if case[3] <= 16]


@pytest.mark.parametrize("a_dt,bs,zero_points,m,n,k,rounding,prepack", ACC4_RUNS)
def test_acc4_outputs(port, ref, a_dt, bs, zero_points, m, n, k, rounding, prepack):
    provider = E.RocmExecutionProvider(0, {"acc4_rounding": rounding, "prepack": "1" if prepack else "0"})
    try:
        b, s, zp = synth.make_weights(n, k, bs, 80 + n, zero_points=zero_points, scale_lo=0.002, scale_hi=0.01, scale_dtype=a_dt)
        a = synth.make_activation(m, k, 80, a_dt)
        bias = synth.to_dtype(np.linspace(-1, 1, n).astype(np.float32), a_dt)
        y32, variant = run_op(provider, a, a_dt, b, s, a_dt, zp, n, k, bs, accuracy_level=4, bias=bias, bias_dtype=a_dt, y_dtype=E.F32)
        on_matrix_cores = bs in (32, 64, 128) if m <= 16 else bs >= 32
        expected = "acc4_mfma_i8" if on_matrix_cores else "acc4_gemv_dot4"
        if prepack and m <= 16 and on_matrix_cores:
            expected = "acc4_mfma_i8_packed"                            # constant weights: the repacked stream
        assert variant == expected
        rnd = oracle.ROUND_HALF_EVEN if rounding == "mlas" else oracle.ROUND_HALF_AWAY
        af, sf, bf = synth.to_f32(a, a_dt), synth.to_f32(s, a_dt), synth.to_f32(bias, a_dt)
        want = port.matmul_acc4_f32(af, b, sf, zp, n, k, bs, rnd, bias=bf)
        assert helpers.rel_l2(y32, want) <= TOL_F32                   # same codes, same integers: only f32 summation order differs
        if rounding == "mlas":
            y_ref = ref.matmul(af, b, sf, zp, n, k, bs, ref.COMP_INT8, bias=bf)
            if y_ref is not None:
                assert helpers.rel_l2(y32, y_ref) <= TOL_F32
        y, _ = run_op(provider, a, a_dt, b, s, a_dt, zp, n, k, bs, accuracy_level=4, bias=bias, bias_dtype=a_dt)
        assert np.array_equal(np.asarray(y).view(NPDT[a_dt] if a_dt != E.F32 else np.float32), np.asarray(port.narrow(y32, a_dt)))
    finally:
        provider.shutdown()


@pytest.mark.parametrize("m,rule", [(2, oracle.ROUND_HALF_AWAY), (4, oracle.ROUND_HALF_EVEN), (40, oracle.ROUND_HALF_EVEN)])
def test_acc4_rounding_route_follows_row_count(port, m, rule):
    """acc4_rounding = auto: fewer rows than the crossover round the native way, the rest the MLAS way
    (matmul_nbits.rs:640-660, where the crossover is NXRT_SQNBIT_DECODE_MIN or twice the decode threads)."""
    bs, n, k = 64, 48, 64 * 6
    provider = E.RocmExecutionProvider(0, {"acc4_rounding": "auto", "acc4_native_below": "4"})
    try:
        b, s, zp = synth.make_weights(n, k, bs, 91, zero_points=True, scale_lo=0.002, scale_hi=0.01, scale_dtype=E.F32)
        a = _tie_heavy_activation(m, k, bs, 92, E.F32)
        y, _ = run_op(provider, a, E.F32, b, s, E.F32, zp, n, k, bs, accuracy_level=4)
        assert helpers.rel_l2(y, port.matmul_acc4_f32(a, b, s, zp, n, k, bs, rule)) <= TOL_F32
        assert helpers.rel_l2(y, port.matmul_acc4_f32(a, b, s, zp, n, k, bs, 1 - rule)) > 10 * TOL_F32   # the other rule is told apart
    finally:
        provider.shutdown()


@pytest.mark.parametrize("waves", [1, 3, 8])
@pytest.mark.parametrize("s_dt", [E.F32, E.F16])
@pytest.mark.parametrize("prepack", [True, False])
def test_acc4_decode_wave_counts_agree(port, waves, s_dt, prepack):
    a_dt, bs, n, k = E.F16, 64, 100, 64 * 50
    provider = E.RocmExecutionProvider(0, {"decode_waves": str(waves), "prepack": "1" if prepack else "0"})
    try:
        b, s, zp = synth.make_weights(n, k, bs, 95, zero_points=True, scale_lo=0.002, scale_hi=0.01, scale_dtype=s_dt)
        for m in (1, 6):
            a = synth.make_activation(m, k, 95 + m, a_dt)
            y32, variant = run_op(provider, a, a_dt, b, s, s_dt, zp, n, k, bs, accuracy_level=4, y_dtype=E.F32)
            assert variant == ("acc4_mfma_i8_packed" if prepack else "acc4_mfma_i8")
            want = port.matmul_acc4_f32(synth.to_f32(a, a_dt), b, synth.to_f32(s, s_dt), zp, n, k, bs, oracle.ROUND_HALF_EVEN)
            assert helpers.rel_l2(y32, want) <= TOL_F32
    finally:
        provider.shutdown()


def test_acc4_power_of_two_scaling_at_full_70b_shape(ep):
    """Size-independent property at a full 70B-class shape: doubling A doubles every block scale and leaves the int8
    codes alone, so Y doubles exactly (f32 output, no bias) - on the decode kernel and on the tiled kernel."""
    a_dt, bs, n, k = E.F16, 64, 10240, 8192
    b, s, zp = synth.make_weights(n, k, bs, 23, zero_points=True, scale_lo=0.002, scale_hi=0.01, scale_dtype=a_dt)
    ops = E.DeviceOperands(ep, b, s, a_dt, zp, n, k, bs, accuracy_level=4)
    for m in (1, 8, 40):
        a = np.random.default_rng(m).uniform(-1.0, 1.0, size=(m, k)).astype(np.float16)
        ys = []
        for scale in (1.0, 2.0):
            ab, yb = ep.upload((a * np.float16(scale)).astype(np.float16)), ep.allocate(m * n * 4)
            ops.run(ab, a_dt, m, yb, E.F32)
            ys.append(ep.download(yb, (m, n), np.float32))
            ep.deallocate(ab)
            ep.deallocate(yb)
        assert ops.kernel.last_variant() == ("acc4_mfma_i8_packed" if m <= 16 else "acc4_mfma_i8")
        assert np.isfinite(ys[0]).all() and np.abs(ys[0]).max() > 0
        assert np.array_equal(ys[1], 2.0 * ys[0])
    ops.free()


def test_prefill_linearity_at_full_8b_shape(ep):
    """Size-independent property at a full Llama-3-8B MLP shape: with small-integer activations every product and
    partial sum of A1 + A2 is the sum of those of A1 and A2 up to f32 rounding of the accumulation."""
    a_dt, bs, m, n, k = E.F16, 32, 512, 14336, 4096
    b, s, _ = synth.make_weights(n, k, bs, 29, zero_points=False, scale_lo=0.001, scale_hi=0.01, scale_dtype=a_dt)
    ops = E.DeviceOperands(ep, b, s, a_dt, None, n, k, bs)
    rng = np.random.default_rng(29)
    a1 = rng.integers(-8, 9, size=(m, k)).astype(np.float16)
    a2 = rng.integers(-8, 9, size=(m, k)).astype(np.float16)
    ys = []
    for a in (a1, a2, (a1 + a2).astype(np.float16)):
        ab, yb = ep.upload(a), ep.allocate(m * n * 4)
        ops.run(ab, a_dt, m, yb, E.F32)
        ys.append(ep.download(yb, (m, n), np.float32).astype(np.float64))
        ep.deallocate(ab)
        ep.deallocate(yb)
    assert ops.kernel.last_variant() == "prefill_mfma_lds"
    assert helpers.rel_l2(ys[0] + ys[1], ys[2]) <= 1e-5
    ops.free()


def test_acc4_with_caller_workspace(ep, port):
    a_dt, bs, m, n, k = E.F16, 64, 4, 64, 512
    b, s, zp = synth.make_weights(n, k, bs, 91, zero_points=True, scale_lo=0.002, scale_hi=0.01, scale_dtype=a_dt)
    a = synth.make_activation(m, k, 91, a_dt)
    ops = E.DeviceOperands(ep, b, s, a_dt, zp, n, k, bs, accuracy_level=4)
    need, align = ops.kernel.workspace_requirement([((m, k), a_dt)])
    assert need > 0 and align == 256
    ws, ab, yb = ep.allocate(need), ep.upload(a), ep.allocate(m * n * 2)
    ops.kernel.execute(ops.views(ab, a_dt, m), [E.TensorView(yb.ptr, a_dt, (m, n))], workspace=ws)
    y = ep.download(yb, (m, n), np.float16)
    want = port.matmul_nbits(a, a_dt, b, s, a_dt, zp, None, E.F32, a_dt, m, n, k, bs, accuracy_level=4, rounding=oracle.ROUND_HALF_EVEN)
    assert helpers.rel_l2(y.astype(np.float32), want.astype(np.float32)) <= TOL_HALF
    for buf in (ws, ab, yb):
        ep.deallocate(buf)
    ops.free()


# ---------------------------------------------------------------------------------------------
# interface behaviour through the C ABI
# ---------------------------------------------------------------------------------------------
def test_provider_identity(ep):
    assert ep.name() == "RocmExecutionProvider"
    assert ep.device_type() == 2 and ep.device_id() == 0 and ep.memory_vendor_id() == 0x1002
    info = ep.device_info()
    assert info["arch"].startswith("gfx950") and info["compute_units"] >= 200


def test_execute_validation_messages(ep):
    """Same checks, same words as the reference's Kernel::execute (matmul_nbits.rs:1490-1572)."""
    n, k, bs = 8, 64, 32
    b, s, zp = synth.make_weights(n, k, bs, 1, zero_points=True, scale_lo=0.01, scale_hi=0.02, scale_dtype=E.F32)
    ops = E.DeviceOperands(ep, b, s, E.F32, zp, n, k, bs)
    ab, yb = ep.upload(np.zeros((2, k), np.float32)), ep.allocate(2 * n * 4)
    good_in = ops.views(ab, E.F32, 2)
    good_out = [E.TensorView(yb.ptr, E.F32, (2, n))]

    def fails(inputs, outputs, text):
        with pytest.raises(E.EpError) as e:
            ops.kernel.execute(inputs, outputs)
        assert text in str(e.value), str(e.value)

    fails(good_in[:2], good_out, "MatMulNBits: expected 3..=6 inputs, got 2")
    bad = list(good_in)
    bad[0] = E.TensorView(ab.ptr, E.F32, (2, k - 1))
    fails(bad, good_out, f"MatMulNBits: A must have rank >= 1 and last dimension K={k}, got [2, {k - 1}]")
    bad = list(good_in)
    bad[1] = E.TensorView(ops.b.ptr, E.I8, (n, 2, 16))
    fails(bad, good_out, "MatMulNBits: B must have dtype Uint8, got Int8")
    bad = list(good_in)
    bad[1] = E.TensorView(ops.b.ptr, E.U8, (n, 2, 15))
    fails(bad, good_out, f"MatMulNBits: B must have shape [{n}, 2, 16], got [{n}, 2, 15]")
    bad = list(good_in)
    bad[2] = E.TensorView(ops.scales.ptr, E.F32, (n, 3))
    fails(bad, good_out, f"MatMulNBits: scales must have shape [{n * 2}] or [{n}, 2], got [{n}, 3]")
    fails(good_in, [E.TensorView(yb.ptr, E.F32, (2, n + 1))], f"MatMulNBits: Y must have shape [2, {n}], got [2, {n + 1}]")
    fails(good_in, [E.TensorView(yb.ptr, E.I32, (2, n))], "MatMulNBits: Y must have dtype Float32, Float16, or BFloat16, got Int32")
    bad = list(good_in)
    bad[0] = E.TensorView(ab.ptr, E.F32, (2, k), strides=(2 * k, 1))
    fails(bad, good_out, "MatMulNBits: A must be contiguous on the ROCm execution provider")
    bad = list(good_in) + [E.TensorView(ops.b.ptr, E.I32, (k,))]
    fails(bad, good_out, "] is outside 0..2")                    # 256 random weight bytes read as 64 group indices: far out of range
    bad = list(good_in)
    bad[0] = E.TensorView(ab.ptr, E.F32, (2, k), device_type=0)
    fails(bad, good_out, "must live on ROCm device 0")

    # a required tensor without memory behind it is refused before anything is launched
    launches = ep.kernel_launch_count()
    for slot, name in ((0, "A"), (1, "B"), (2, "scales")):
        bad = list(good_in)
        bad[slot] = E.TensorView(None, good_in[slot].dtype, good_in[slot].shape)
        fails(bad, good_out, f"MatMulNBits: {name} has a null data pointer")
    fails(good_in, [E.TensorView(None, E.F32, (2, n))], "MatMulNBits: Y has a null data pointer")
    assert ep.kernel_launch_count() == launches

    # flat scales / zero points are accepted, as in the reference
    flat = list(good_in)
    flat[2] = E.TensorView(ops.scales.ptr, E.F32, (n * 2,))
    flat[3] = E.TensorView(ops.zp.ptr, E.U8, (n * 1,))
    ops.kernel.execute(flat, good_out)
    # rank-3 A: Y = A.shape[:-1] + [N]
    ops.kernel.execute([E.TensorView(ab.ptr, E.F32, (2, 1, k))] + good_in[1:], [E.TensorView(yb.ptr, E.F32, (2, 1, n))])
    # empty A is a no-op
    ops.kernel.execute([E.TensorView(ab.ptr, E.F32, (0, k))] + good_in[1:], [E.TensorView(yb.ptr, E.F32, (0, n))])
    ep.sync()
    for buf in (ab, yb):
        ep.deallocate(buf)
    ops.free()


def test_last_call_metrics_follow_the_reference_count(ep):
    """record_kernel_metrics (onnx-runtime-ep-api/src/kernel.rs:243-267, matmul_nbits.rs:1588-1597): bytes = every present input's
    bytes plus the output's; flops = 2 M N K, plus M N with a bias."""
    a_dt, bs, m, n, k = E.BF16, 128, 3, 80, 512
    kb = k // bs
    b, s, zp = synth.make_weights(n, k, bs, 35, zero_points=True, scale_lo=0.002, scale_hi=0.01, scale_dtype=a_dt)
    bias = synth.to_dtype(np.linspace(-1, 1, n).astype(np.float32), a_dt)
    for with_bias in (False, True):
        ops = E.DeviceOperands(ep, b, s, a_dt, zp, n, k, bs, bias=bias if with_bias else None, bias_dtype=a_dt)
        assert ops.kernel.last_metrics() == (0, 0)
        ab, yb = ep.upload(synth.make_activation(m, k, 36, a_dt)), ep.allocate(m * n * 2)
        try:
            ops.run(ab, a_dt, m, yb)
            ep.sync()
            flops, nbytes = ops.kernel.last_metrics()
        finally:
            ep.deallocate(ab)
            ep.deallocate(yb)
            ops.free()
        want_bytes = m * k * 2 + n * kb * (bs // 2) + n * kb * 2 + n * ((kb + 1) // 2) + (n * 2 if with_bias else 0) + m * n * 2
        assert flops == 2 * m * n * k + (m * n if with_bias else 0)
        assert nbytes == want_bytes


def test_kernel_vtable_execute(ep, port):
    """The nxrt kernel vtable (raw pointers only) runs the same kernel with the create-time shapes."""
    import ctypes as C
    a_dt, bs, m, n, k = E.F16, 32, 2, 64, 256
    b, s, zp = synth.make_weights(n, k, bs, 33, zero_points=True, scale_lo=0.002, scale_hi=0.01, scale_dtype=a_dt)
    a = synth.make_activation(m, k, 33, a_dt)
    ops = E.DeviceOperands(ep, b, s, a_dt, zp, n, k, bs, rows=m, a_dtype=a_dt)
    assert ops.kernel.estimated_flops() == 2 * m * n * k
    ab, yb = ep.upload(a), ep.allocate(m * n * 2)

    class KernelVtable(C.Structure):
        _fields_ = [("struct_size", C.c_uint32), ("_pad", C.c_uint32),
                    ("execute", C.CFUNCTYPE(E.NxrtStatus, C.c_void_p, C.POINTER(C.c_void_p), C.c_uint32, C.POINTER(C.c_void_p), C.c_uint32)),
                    ("release", C.CFUNCTYPE(None, C.c_void_p)), ("ctx", C.c_void_p)]

    vt = C.c_void_p()
    ep.lib.nxrt_rocm_matmul_nbits_as_vtable(ops.kernel.handle, C.byref(vt)).check()
    table = C.cast(vt, C.POINTER(KernelVtable)).contents
    assert table.struct_size == C.sizeof(KernelVtable)
    ins = (C.c_void_p * 4)(ab.ptr, ops.b.ptr, ops.scales.ptr, ops.zp.ptr)
    outs = (C.c_void_p * 1)(yb.ptr)
    table.execute(table.ctx, ins, 4, outs, 1).check()
    y = ep.download(yb, (m, n), np.float16)
    want = port.matmul_nbits(a, a_dt, b, s, a_dt, zp, None, E.F32, a_dt, m, n, k, bs)
    assert helpers.rel_l2(y.astype(np.float32), want.astype(np.float32)) <= TOL_HALF
    for buf in (ab, yb):
        ep.deallocate(buf)
    ops.free()


def _random_cases(count, seed):
    rng = np.random.default_rng(seed)
    cases = []
    for _ in range(count):
        bs = int(rng.choice([16, 32, 64, 128, 256]))
        a_dt = int(rng.choice([E.F32, E.F16, E.BF16]))
        s_dt = a_dt if rng.random() < 0.7 else E.F32
        m = int(rng.choice([1, 2, 3, 4, 5, 8, 13, 16, 17, 24, 32, 33, 50, 64, 65, 130, 300]))
        n = int(rng.integers(1, 700)) if rng.random() < 0.8 else int(rng.integers(16384, 17000))
        blocks = int(rng.integers(1, 40))
        k = blocks * bs - (int(rng.integers(0, bs // 8)) * 8 if rng.random() < 0.3 else 0)
        acc = 4 if rng.random() < 0.35 else 0
        cases.append((a_dt, s_dt, bs, bool(rng.random() < 0.6), m, n, max(k, 8), acc, bool(rng.random() < 0.5)))
    return cases


@pytest.mark.parametrize("a_dt,s_dt,bs,zero_points,m,n,k,acc,with_bias", _random_cases(60, 20260101))
def test_random_shapes_against_oracle(ep, port, a_dt, s_dt, bs, zero_points, m, n, k, acc, with_bias):
    """Seeded random shapes over every dispatch path (whatever kernel the shape lands on) against the CPU oracle."""
    b, s, zp = synth.make_weights(n, k, bs, 900 + n + k, zero_points=zero_points, scale_lo=0.002, scale_hi=0.01, scale_dtype=s_dt)
    a = synth.make_activation(m, k, 900 + m, a_dt)
    bias = synth.to_dtype(np.random.default_rng(n).standard_normal(n).astype(np.float32), a_dt) if with_bias else None
    y32, variant = run_op(ep, a, a_dt, b, s, s_dt, zp, n, k, bs, accuracy_level=acc, bias=bias, bias_dtype=a_dt, y_dtype=E.F32)
    af, sf = synth.to_f32(a, a_dt), synth.to_f32(s, s_dt)
    bf = None if bias is None else synth.to_f32(bias, a_dt)
    if acc == 4:
        want = port.matmul_acc4_f32(af, b, sf, zp, n, k, bs, oracle.ROUND_HALF_EVEN, bias=bf)
        assert variant.startswith("acc4_")
        assert helpers.rel_l2(y32, want) <= TOL_F32, variant
    else:
        want = port.matmul_f64(af, b, sf, zp, n, k, bs, bias=bf)
        tol = TOL_F32 if a_dt == E.F32 else TOL_HALF
        assert helpers.rel_l2(y32, want) <= tol, variant


def test_concurrent_dense_calls_share_one_buffer(port):
    """Two host threads drive two kernels whose tall calls expand their weights into the provider's one dense buffer: the
    expansion and the GEMM of a call are enqueued as a pair, so neither call multiplies by the other's weights."""
    import threading
    provider = E.RocmExecutionProvider(0, {"dense_gemm_min_rows": "64"})
    a_dt, bs, m, n, k = E.F16, 32, 96, 136, 512
    sets = []
    try:
        for i in range(2):
            b, s, zp = synth.make_weights(n, k, bs, 90 + i, zero_points=True, scale_lo=0.002, scale_hi=0.01, scale_dtype=a_dt)
            a = synth.make_activation(m, k, 92 + i, a_dt)
            ops = E.DeviceOperands(provider, b, s, a_dt, zp, n, k, bs)
            ops.kernel.set_constant_inputs([False] * 6)          # weights not constant: every call refills the shared buffer
            sets.append((ops, a, b, s, zp, provider.upload(a), provider.allocate(m * n * 2)))
        for ops, a, _, _, _, ab, yb in sets:                     # first calls, one after the other: set-up happens here
            ops.run(ab, a_dt, m, yb)
        provider.sync()
        errors = []

        def work(item):
            try:
                ops, _, _, _, _, ab, yb = item
                for _ in range(50):
                    ops.run(ab, a_dt, m, yb)
            except Exception as exc:                               # noqa: BLE001 - reported below
                errors.append(exc)

        threads = [threading.Thread(target=work, args=(item,)) for item in sets]
        for t in threads:
            t.start()
        for t in threads:
            t.join()
        provider.sync()
        assert not errors, errors
        for ops, a, b, s, zp, ab, yb in sets:
            assert ops.kernel.last_variant() == "dense_transient_blaslt"
            got = synth.to_f32(provider.download(yb, (m, n), np.float16), a_dt)
            assert helpers.rel_l2(got, oracle_f64(port, a, a_dt, b, s, a_dt, zp, n, k, bs)) <= TOL_HALF
    finally:
        for ops, _, _, _, _, ab, yb in sets:
            provider.deallocate(ab)
            provider.deallocate(yb)
            ops.free()
        provider.shutdown()


def test_concurrent_execute_on_one_kernel(ep, port):
    """Two host threads drive the same kernel object (the plugin contract asks for thread-safe vtables): every call
    must see consistent per-object state (repacked copy, scratch) and produce its own result."""
    import threading
    a_dt, bs, n, k = E.F16, 64, 160, 1024
    b, s, zp = synth.make_weights(n, k, bs, 71, zero_points=True, scale_lo=0.002, scale_hi=0.01, scale_dtype=a_dt)
    ops = E.DeviceOperands(ep, b, s, a_dt, zp, n, k, bs, accuracy_level=4)
    jobs = []
    for i, m in enumerate((1, 3, 20, 1, 40, 2)):
        a = synth.make_activation(m, k, 700 + i, a_dt)
        jobs.append((m, a, ep.upload(a), ep.allocate(m * n * 4)))
    errors = []

    def work(part):
        try:
            for _ in range(10):
                for m, _, ab, yb in part:
                    ops.run(ab, a_dt, m, yb, E.F32)
        except Exception as exc:                                   # noqa: BLE001 - reported below
            errors.append(exc)

    threads = [threading.Thread(target=work, args=(jobs[i::2],)) for i in range(2)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    ep.sync()
    assert not errors, errors
    for m, a, ab, yb in jobs:
        got = ep.download(yb, (m, n), np.float32)
        want = port.matmul_acc4_f32(synth.to_f32(a, a_dt), b, synth.to_f32(s, a_dt), zp, n, k, bs, oracle.ROUND_HALF_EVEN)
        assert helpers.rel_l2(got, want) <= TOL_F32
        ep.deallocate(ab)
        ep.deallocate(yb)
    ops.free()


def test_plain_c_host_roundtrip():
    """tests/harness/nxrt_roundtrip.c: a host in plain C loads the library the way the reference's loader does, runs
    MatMulNBits through the plugin allocator and the kernel mirror, and checks the result itself."""
    import subprocess
    here = os.path.dirname(os.path.abspath(__file__))
    exe = os.path.join(here, "harness", "nxrt_roundtrip")
    assert os.path.exists(exe), "tests/harness/nxrt_roundtrip is built by __graft_entry__.build()"
    run = subprocess.run([exe, E.LIB_PATH], capture_output=True, text=True, timeout=100)
    assert run.returncode == 0, run.stdout + run.stderr
    assert "roundtrip ok" in run.stdout and "accuracy_level 4" in run.stdout and "nxmem unload report: nothing live" in run.stdout


def test_launch_counter_proves_native_path(ep):
    before = ep.kernel_launch_count()
    test_low_nibble_before_high_nibble(ep)
    assert ep.kernel_launch_count() == before + 1
