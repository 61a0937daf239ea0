"""The entry point that allocates nothing (nxrt_rocm_matmul_nbits_execute_static) against nxrt_rocm_matmul_nbits_execute.

Collected last on purpose (the file name sorts after every other test file): the round-end run stops at the first
failure, and a failure here should not hide the parity tests.
"""
import numpy as np
import pytest

from onnx_genai_amd import ep as E
from onnx_genai_amd import synth

pytestmark = pytest.mark.gpu


def _both_ways(provider, a_dt, bs, acc, m, n, k, y_dt, seed):
    """One node, the same inputs through execute and through execute_static; returns both outputs, the variant of each, and
    the number of device allocations the static call made."""
    lib = provider.lib
    b, s, zp = synth.make_weights(n, k, bs, seed, zero_points=True, scale_lo=0.002, scale_hi=0.01, scale_dtype=a_dt)
    a = synth.make_activation(m, k, seed + 1, a_dt)
    bias = synth.to_dtype(np.linspace(-1, 1, n).astype(np.float32), a_dt)
    ops = E.DeviceOperands(provider, b, s, a_dt, zp, n, k, bs, accuracy_level=acc, bias=bias, bias_dtype=a_dt)
    item = 4 if y_dt == E.F32 else 2
    np_dt = np.float32 if y_dt == E.F32 else np.uint16
    ab, y1, y2 = provider.upload(a), provider.allocate(m * n * item), provider.allocate(m * n * item)
    try:
        views = ops.views(ab, a_dt, m)
        ops.kernel.execute(views, [E.TensorView(y1.ptr, y_dt, (m, n))])
        v1 = ops.kernel.last_variant()
        want = provider.download(y1, (m, n), np_dt)
        provider.copy_from_host(y2, np.full(m * n * item, 0xEE, np.uint8))
        before = lib.nxrt_rocm_device_allocation_count()
        ops.kernel.execute_static(views, [E.TensorView(y2.ptr, y_dt, (m, n))])
        allocations = lib.nxrt_rocm_device_allocation_count() - before
        v2 = ops.kernel.last_variant()
        got = provider.download(y2, (m, n), np_dt)
    finally:
        for buf in (ab, y1, y2):
            provider.deallocate(buf)
        ops.free()
    return want, got, v1, v2, allocations


def test_execute_static_matches_execute_and_allocates_nothing():
    # weights streamed as given (no repacked copy, no dense copy): both entry points then run the same kernels
    provider = E.RocmExecutionProvider(0, {"prepack": "0", "dense_gemm_min_rows": "0"})
    try:
        calls = [
            # a_dt, block, accuracy_level, m, n, k, y dtype - each pair: a larger call, then a smaller one over the same scratch
            (E.F16, 64, 4, 40, 96, 64 * 17, E.F32),       # int8 tiled kernel, K in two slices: codes, scales and partial sums in scratch
            (E.F16, 64, 4, 3, 50, 256, E.F32),            # int8 split-K kernel, a few KB of codes
            (E.F16, 64, 0, 100, 130, 4096, E.F16),        # float tiled kernel, K in slices: f32 partial sums in scratch
            (E.BF16, 128, 0, 40, 72, 2048, E.BF16),       # the same kernel, smaller, fewer slices
            (E.F16, 32, 4, 1, 48, 4100, E.F32),           # one row, K % 8 != 0: the separate quantizer fills the scratch
            (E.BF16, 128, 0, 4, 300, 3584, E.BF16),       # a decode call: no scratch at all
        ]
        for i, (a_dt, bs, acc, m, n, k, y_dt) in enumerate(calls):
            want, got, v1, v2, allocations = _both_ways(provider, a_dt, bs, acc, m, n, k, y_dt, 900 + i)
            assert v1 == v2, (calls[i], v1, v2)
            assert allocations == 0, (calls[i], allocations)
            assert np.array_equal(want, got), (calls[i], v1)            # same kernels, same order of summation: the same bits
    finally:
        provider.shutdown()


def test_execute_static_on_a_default_provider_after_the_copy_exists():
    """The default configuration: execute makes the repacked copy of the constant weights on its first call; from then on the
    static entry point runs the same kernels over that copy - the one-row and few-row decode builds, accuracy_level 4 with the
    row quantized inside the kernel, and with the codes of 2 .. 16 rows written into the static scratch in the copy's order."""
    provider = E.RocmExecutionProvider(0)
    try:
        calls = [
            (E.BF16, 128, 0, 1, 304, 3584, E.BF16),       # one row over the repacked stream
            (E.F16, 32, 0, 4, 528, 2048, E.F16),          # four rows
            (E.BF16, 128, 0, 16, 272, 3584, E.BF16),      # sixteen rows: the build that stages them per wave
            (E.F16, 64, 4, 1, 320, 8192, E.F32),          # accuracy_level 4, one row quantized in the kernel
            (E.F16, 64, 4, 8, 320, 4096, E.F32),          # accuracy_level 4, eight rows: codes and pairs in the static scratch
            (E.F16, 64, 4, 3, 96, 1024, E.F32),           # the same, smaller, over the same scratch
        ]
        for i, (a_dt, bs, acc, m, n, k, y_dt) in enumerate(calls):
            want, got, v1, v2, allocations = _both_ways(provider, a_dt, bs, acc, m, n, k, y_dt, 970 + i)
            assert v1 == v2 and ("packed" in v1), (calls[i], v1, v2)
            assert allocations == 0, (calls[i], allocations)
            assert np.array_equal(want, got), (calls[i], v1)
    finally:
        provider.shutdown()


def test_execute_static_with_fewer_slices_than_execute(port):
    """A tall call whose preferred K slices want more partial sums than the static scratch holds runs with fewer slices: another
    order of summation than execute's, so the two are held to the oracle's bar, not to each other's bits."""
    from tests import helpers
    provider = E.RocmExecutionProvider(0, {"prepack": "0", "dense_gemm_min_rows": "0"})
    try:
        a_dt, bs, m, n, k = E.F16, 32, 300, 2048, 16384
        b, s, zp = synth.make_weights(n, k, bs, 990, zero_points=True, scale_lo=0.002, scale_hi=0.01, scale_dtype=a_dt)
        a = synth.make_activation(m, k, 991, a_dt)
        ops = E.DeviceOperands(provider, b, s, a_dt, zp, n, k, bs)
        need, _ = ops.kernel.workspace_requirement([((m, k), a_dt)])
        assert need > 8 << 20, need                                  # the preferred plan does not fit the 8 MiB array
        ab, y1, y2 = provider.upload(a), provider.allocate(m * n * 2), provider.allocate(m * n * 2)
        try:
            views = ops.views(ab, a_dt, m)
            ops.kernel.execute(views, [E.TensorView(y1.ptr, a_dt, (m, n))])
            before = provider.lib.nxrt_rocm_device_allocation_count()
            ops.kernel.execute_static(views, [E.TensorView(y2.ptr, a_dt, (m, n))])
            assert provider.lib.nxrt_rocm_device_allocation_count() == before
            assert ops.kernel.last_variant() == "prefill_mfma_lds"
            got1, got2 = provider.download(y1, (m, n), np.float16), provider.download(y2, (m, n), np.float16)
        finally:
            for buf in (ab, y1, y2):
                provider.deallocate(buf)
            ops.free()
        cols = np.unique(np.linspace(0, n - 1, 96).astype(np.int64))
        w = port.dequantize_nk(np.ascontiguousarray(b[cols]), np.ascontiguousarray(s.astype(np.float32)[cols]), np.ascontiguousarray(zp[cols]), len(cols), k, bs)
        want = a.astype(np.float64) @ w.astype(np.float64).T
        assert helpers.rel_l2(got1[:, cols], want) <= 5e-3
        assert helpers.rel_l2(got2[:, cols], want) <= 5e-3
    finally:
        provider.shutdown()


def test_execute_static_refuses_what_does_not_fit():
    provider = E.RocmExecutionProvider(0, {"prepack": "0", "dense_gemm_min_rows": "0"})
    try:
        a_dt, bs, m, n, k = E.F16, 64, 2048, 64, 8192                    # 16 MiB of activation codes: beyond the 8 MiB array
        b, s, zp = synth.make_weights(n, k, bs, 950, zero_points=True, scale_lo=0.002, scale_hi=0.01, scale_dtype=a_dt)
        ops = E.DeviceOperands(provider, b, s, a_dt, zp, n, k, bs, accuracy_level=4)
        ab, yb = provider.upload(synth.make_activation(m, k, 951, a_dt)), provider.allocate(m * n * 2)
        try:
            launches = provider.kernel_launch_count()
            with pytest.raises(E.EpError) as e:
                ops.kernel.execute_static(ops.views(ab, a_dt, m), [E.TensorView(yb.ptr, a_dt, (m, n))])
            assert "bytes of scratch and the static scratch of execute_static holds 8388608" in str(e.value)
            assert provider.kernel_launch_count() == launches
            ops.kernel.execute(ops.views(ab, a_dt, m), [E.TensorView(yb.ptr, a_dt, (m, n))])          # the allocating entry point takes it
        finally:
            provider.deallocate(ab)
            provider.deallocate(yb)
            ops.free()
        fused = E.GateUpOperands(provider, synth.make_weights(32, 128, 32, 1, zero_points=False, scale_lo=0.01, scale_hi=0.02, scale_dtype=E.F16),
                                 synth.make_weights(32, 128, 32, 2, zero_points=False, scale_lo=0.01, scale_hi=0.02, scale_dtype=E.F16), E.F16, 32, 128, 32)
        ab, yb = provider.upload(synth.make_activation(1, 128, 3, E.F16)), provider.allocate(64)
        try:
            with pytest.raises(E.EpError) as e:
                fused.kernel.execute_static(fused.views(ab, E.F16, 1), [E.TensorView(yb.ptr, E.F16, (1, 32))])
            assert "execute_static serves plain MatMulNBits nodes" in str(e.value)
        finally:
            provider.deallocate(ab)
            provider.deallocate(yb)
            fused.free()
    finally:
        provider.shutdown()


def test_static_calls_through_two_providers_of_one_gpu_do_not_race():
    """Two providers share the GPU's static scratch and have a stream each. Calls that use the scratch heavily (int8 codes
    of a tall accuracy_level 4 call) are made through both in turn without any host synchronization in between; each must
    give what it gives alone. The library chains them on the GPU (an event recorded behind each call, waited for by the next
    call on another stream)."""
    p1, p2 = E.RocmExecutionProvider(0, {"prepack": "0"}), E.RocmExecutionProvider(0, {"prepack": "0"})
    try:
        jobs = []
        for i, (prov, m, n, k) in enumerate([(p1, 96, 256, 8192), (p2, 80, 320, 8192)]):
            a_dt, bs = E.F16, 64
            b, s, zp = synth.make_weights(n, k, bs, 990 + i, zero_points=True, scale_lo=0.002, scale_hi=0.01, scale_dtype=a_dt)
            a = synth.make_activation(m, k, 995 + i, a_dt)
            ops = E.DeviceOperands(prov, b, s, a_dt, zp, n, k, bs, accuracy_level=4)
            ab, y_ref, y = prov.upload(a), prov.allocate(m * n * 4), prov.allocate(m * n * 4)
            views = ops.views(ab, a_dt, m)
            ops.kernel.execute_static(views, [E.TensorView(y_ref.ptr, E.F32, (m, n))])
            prov.sync()
            jobs.append((prov, ops, views, ab, y_ref, y, m, n))
        alone = [job[0].download(job[4], (job[6], job[7]), np.float32) for job in jobs]
        before = p1.lib.nxrt_rocm_device_allocation_count()
        for _ in range(20):                                    # 40 calls, alternating providers, no synchronization in between
            for prov, ops, views, ab, y_ref, y, m, n in jobs:
                ops.kernel.execute_static(views, [E.TensorView(y.ptr, E.F32, (m, n))])
        assert p1.lib.nxrt_rocm_device_allocation_count() == before
        p1.sync()
        p2.sync()
        for (prov, ops, views, ab, y_ref, y, m, n), want in zip(jobs, alone):
            assert np.array_equal(prov.download(y, (m, n), np.float32), want)
        for prov, ops, views, ab, y_ref, y, m, n in jobs:
            for buf in (ab, y_ref, y):
                prov.deallocate(buf)
            ops.free()
    finally:
        p1.shutdown()
        p2.shutdown()

