"""What can be checked of the C ABI without a GPU: the library loads, exports every symbol its headers declare,
keeps the wire layouts, and fails closed. No compute call is made here."""
import ctypes as C
import os
import re

import pytest

from onnx_genai_amd import ep as E

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
INCLUDE = os.path.join(ROOT, "include")


@pytest.fixture(scope="module")
def lib():
    if not os.path.exists(E.LIB_PATH):
        from onnx_genai_amd import build
        build.build()
    return E.load_library()


def declared_symbols():
    names = set()
    for header in sorted(os.listdir(INCLUDE)):
        text = open(os.path.join(INCLUDE, header)).read()
        text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
        for m in re.finditer(r"^[A-Za-z_][\w\s\*]*?\b((?:nxrt_rocm_|Nxrt|Nxmem)\w+|CreateEpFactories|ReleaseEpFactory)\s*\(", text, flags=re.M):
            line_start = text.rfind("\n", 0, m.start()) + 1
            if text[line_start:m.start()].strip().startswith("typedef"):
                continue
            names.add(m.group(1))
    return sorted(names)


def test_every_declared_symbol_is_exported(lib):
    names = declared_symbols()
    assert len(names) >= 40 and "NxrtNegotiate" in names and "nxrt_rocm_matmul_nbits_execute" in names and "NxmemQueryUnloadReadiness" in names
    assert "CreateEpFactories" in names and "ReleaseEpFactory" in names               # the ORT plugin-EP export
    missing = [n for n in names if not hasattr(lib, n)]
    assert not missing, missing


def test_headers_compile_as_c_and_cxx():
    import subprocess
    for lang, std in (("c", "-std=c11"), ("c++", "-std=c++17")):
        for header in ("nxrt_ep_rocm.h", "nxrt_ort_plugin.h", "ort_plugin_ep_subset.h"):
            subprocess.run(["gcc", "-fsyntax-only", "-x", lang, std, "-Wall", "-Werror", os.path.join(INCLUDE, header)], check=True)


class VersionRange(C.Structure):
    _fields_ = [("major_min", C.c_uint32), ("major_max", C.c_uint32), ("minor_max", C.c_uint32)]


class NegotiateRequest(C.Structure):
    _fields_ = [("struct_size", C.c_uint32), ("host_range", VersionRange)]


class NegotiateResponse(C.Structure):
    _fields_ = [("struct_size", C.c_uint32), ("agreed_major", C.c_uint32), ("agreed_minor", C.c_uint32),
                ("plugin_range", VersionRange), ("capability_flags", C.c_uint64)]


class FactoryVtable(C.Structure):
    _fields_ = [("struct_size", C.c_uint32), ("num_devices", C.c_uint32), ("name", C.c_char_p),
                ("create_ep", C.CFUNCTYPE(E.NxrtStatus, C.c_void_p, C.c_uint32, C.POINTER(C.c_void_p))),
                ("release", C.CFUNCTYPE(None, C.c_void_p)), ("ctx", C.c_void_p)]


def test_status_and_negotiate_layouts():
    """crates/onnx-runtime-ep-nxrt-abi/src/status.rs:105-119 (264 bytes) and version.rs:40-78."""
    assert C.sizeof(E.NxrtStatus) == 264
    assert C.sizeof(NegotiateRequest) == 16 and C.sizeof(NegotiateResponse) == 32
    assert C.sizeof(E.NxrtTensorDesc) == 24 and C.sizeof(FactoryVtable) == 40


def negotiate(lib, major_min, major_max, minor_max):
    lib.NxrtNegotiate.restype = E.NxrtStatus
    lib.NxrtNegotiate.argtypes = [C.c_void_p, C.c_void_p]
    req = NegotiateRequest(C.sizeof(NegotiateRequest), VersionRange(major_min, major_max, minor_max))
    resp = NegotiateResponse()
    return lib.NxrtNegotiate(C.byref(req), C.byref(resp)), resp


def test_negotiate_same_version(lib):
    """version.rs tests: negotiate_success_same_version, negotiate_agrees_on_min_minor."""
    st, resp = negotiate(lib, 1, 1, 0)
    assert st.code == 0 and (resp.agreed_major, resp.agreed_minor) == (1, 0)
    assert resp.capability_flags & ~0xF == 0 and resp.capability_flags & 1      # only known bits; device enumeration offered
    st, resp = negotiate(lib, 1, 1, 5)
    assert st.code == 0 and resp.agreed_minor == 0


def test_negotiate_rejects_incompatible_major(lib):
    """version.rs: negotiate_rejects_incompatible_major — VersionMismatch, message names the plugin major, range reported."""
    st, resp = negotiate(lib, 99, 99, 0)
    assert st.code == 1 and "plugin major version 1 outside host range [99, 99]" in st.text()
    assert (resp.plugin_range.major_min, resp.plugin_range.major_max) == (1, 1)
    lib.NxrtNegotiate.argtypes = [C.c_void_p, C.c_void_p]
    st = lib.NxrtNegotiate(None, None)
    assert st.code == 3 and "null request or response pointer" in st.text()


def test_create_factories_lifecycle_without_gpu(lib):
    """vtable.rs tests: null / zero max rejected; a factory is created even when no device is visible and its
    create_ep then reports a device error instead of crashing (fail closed)."""
    lib.NxrtCreateEpFactories.restype = E.NxrtStatus
    lib.NxrtCreateEpFactories.argtypes = [C.POINTER(C.c_void_p), C.c_size_t, C.POINTER(C.c_size_t)]
    n = C.c_size_t(99)
    st = lib.NxrtCreateEpFactories(None, 1, C.byref(n))
    assert st.code == 3 and "null pointer or zero max_factories" in st.text() and n.value == 0
    out = (C.c_void_p * 1)()
    st = lib.NxrtCreateEpFactories(out, 0, C.byref(n))
    assert st.code == 3
    st = lib.NxrtCreateEpFactories(out, 1, C.byref(n))
    assert st.code == 0 and n.value == 1 and out[0]
    factory = C.cast(out[0], C.POINTER(FactoryVtable)).contents
    assert factory.struct_size == C.sizeof(FactoryVtable) and factory.name == b"RocmExecutionProvider"
    if factory.num_devices == 0:
        vt = C.c_void_p()
        st = factory.create_ep(factory.ctx, 0, C.byref(vt))
        assert st.code == 6 and not vt.value and "no HIP device is visible" in st.text()
        assert lib.nxrt_rocm_live_provider_count() == 0
    factory.release(factory.ctx)


class NxmemStatus(C.Structure):
    _fields_ = [("code", C.c_uint32), ("message_len", C.c_uint32), ("message", C.c_uint8 * 256)]


class NxmemVersionRange(C.Structure):
    _fields_ = [("major_min", C.c_uint32), ("major_max", C.c_uint32), ("minor_min", C.c_uint32), ("minor_max", C.c_uint32)]


class NxmemNegotiateRequest(C.Structure):
    _fields_ = [("struct_size", C.c_uint32), ("reserved", C.c_uint32), ("host_range", NxmemVersionRange), ("host_capability_flags", C.c_uint64)]


class NxmemNegotiateResponse(C.Structure):
    _fields_ = [("struct_size", C.c_uint32), ("agreed_major", C.c_uint32), ("agreed_minor", C.c_uint32), ("reserved", C.c_uint32),
                ("plugin_range", NxmemVersionRange), ("capability_flags", C.c_uint64)]


class NxmemUnloadReport(C.Structure):
    _fields_ = [("struct_size", C.c_uint32), ("reserved", C.c_uint32), ("live_allocators", C.c_uint64), ("live_allocations", C.c_uint64),
                ("live_views", C.c_uint64), ("live_capabilities", C.c_uint64), ("queued_releases", C.c_uint64)]


def test_nxmem_negotiate_and_unload_report(lib):
    """nxmem_memory_abi.h:664-718: sizes 32 / 40 / 48; capabilities are a subset of what the host offered; short
    structs, foreign majors and a host that does not offer plain allocation are refused."""
    assert (C.sizeof(NxmemNegotiateRequest), C.sizeof(NxmemNegotiateResponse), C.sizeof(NxmemUnloadReport)) == (32, 40, 48)
    lib.NxmemNegotiate.restype = NxmemStatus
    lib.NxmemNegotiate.argtypes = [C.c_void_p, C.c_void_p]
    resp = NxmemNegotiateResponse()
    req = NxmemNegotiateRequest(32, 0, NxmemVersionRange(1, 1, 0, 1), 0x1F)
    st = lib.NxmemNegotiate(C.byref(req), C.byref(resp))
    assert st.code == 0 and resp.agreed_major == 1 and resp.agreed_minor == 0 and resp.capability_flags == 1
    req.struct_size = 8
    assert lib.NxmemNegotiate(C.byref(req), C.byref(resp)).code == 2            # SHORT_STRUCT
    req = NxmemNegotiateRequest(32, 0, NxmemVersionRange(2, 3, 0, 0), 1)
    assert lib.NxmemNegotiate(C.byref(req), C.byref(resp)).code == 1            # VERSION_MISMATCH
    req = NxmemNegotiateRequest(32, 0, NxmemVersionRange(1, 1, 0, 1), 0x2)
    assert lib.NxmemNegotiate(C.byref(req), C.byref(resp)).code == 3            # UNSUPPORTED_CAPABILITY
    assert lib.NxmemNegotiate(None, None).code == 4
    lib.NxmemQueryUnloadReadiness.restype = NxmemStatus
    lib.NxmemQueryUnloadReadiness.argtypes = [C.c_void_p]
    report = NxmemUnloadReport()
    assert lib.NxmemQueryUnloadReadiness(C.byref(report)).code == 0 and report.struct_size == 48 and report.live_allocations == 0
    lib.NxmemCreateAllocatorFactories.restype = NxmemStatus
    lib.NxmemCreateAllocatorFactories.argtypes = [C.POINTER(C.c_void_p), C.c_uint64, C.POINTER(C.c_uint64)]
    out, n = (C.c_void_p * 4)(), C.c_uint64(7)
    assert lib.NxmemCreateAllocatorFactories(out, 0, C.byref(n)).code == 4
    assert lib.NxmemCreateAllocatorFactories(out, 4, C.byref(n)).code == 0 and n.value <= 4


def create_status(lib, **attrs):
    a = E.make_attrs(**attrs)
    h = C.c_void_p()
    return lib.nxrt_rocm_matmul_nbits_create(None, C.byref(a), None, 0, C.byref(h)), h


def test_attribute_validation_messages(lib):
    """KernelFactory::create, matmul_nbits.rs:1410-1445 + 10258-10277: checks run before anything touches a device."""
    cases = [
        (dict(N=8, bits=4, block_size=32), "MatMulNBits: missing required integer attribute 'K'"),
        (dict(K=64, bits=4, block_size=32), "MatMulNBits: missing required integer attribute 'N'"),
        (dict(K=0, N=8, block_size=32), "MatMulNBits: attribute 'K' must be positive, got 0"),
        (dict(K=64, N=-3, block_size=32), "MatMulNBits: attribute 'N' must be positive, got -3"),
        (dict(K=64, N=8), "MatMulNBits: missing required integer attribute 'block_size'"),
        (dict(K=64, N=8, block_size=8), "MatMulNBits: block_size must be a power of two and at least 16, got 8"),
        (dict(K=64, N=8, block_size=48), "MatMulNBits: block_size must be a power of two and at least 16, got 48"),
        (dict(K=64, N=8, block_size=32, weight_prepacked=2), "weight_prepacked must be 0 (standard ONNX layout) or 1 (MLAS SQNBit packed layout), got 2"),
        (dict(K=64, N=8, block_size=32, weight_prepacked=1), "weight_prepacked=1 holds the MLAS SQNBit CPU layout"),
        (dict(K=64, N=8, block_size=32, bits=3), "MatMulNBits ROCm supports bits in {2, 4, 8}, got bits=3"),
        (dict(K=64, N=8, block_size=32, bits=16), "MatMulNBits ROCm supports bits in {2, 4, 8}, got bits=16"),
        (dict(K=64, N=8, block_size=32, bits=8, accuracy_level=4), "accuracy_level=4 is implemented for bits=4 only, got bits=8"),
    ]
    for attrs, text in cases:
        st, h = create_status(lib, **attrs)
        assert st.code == 3 and text in st.text() and not h.value, (attrs, st.text())
    st, h = create_status(lib, K=64, N=8, block_size=32)            # bits defaults to 4; only the provider is missing
    assert st.code == 3 and st.text() == "MatMulNBits: null provider"


def test_supports_op_declines_with_reasons(lib):
    reason = C.create_string_buffer(512)
    a = E.make_attrs(K=64, N=8, bits=3, block_size=32)
    assert lib.nxrt_rocm_ep_supports_matmul_nbits(None, C.byref(a), None, 0, reason, 512) == 0 and b"How to fix" in reason.value
    a = E.make_attrs(K=64, N=8, bits=8, block_size=32)
    assert lib.nxrt_rocm_ep_supports_matmul_nbits(None, C.byref(a), None, 0, reason, 512) == 1 and reason.value == b""
    a = E.make_attrs(K=64, N=8, bits=4, block_size=32)
    assert lib.nxrt_rocm_ep_supports_matmul_nbits(None, C.byref(a), None, 0, reason, 512) == 1 and reason.value == b""
    descs, keep = E.make_descs([((1, 64), E.F16), ((8, 2, 16), E.U8), ((8, 2), E.F16), (None, 0), ((64,), E.I32)])
    assert lib.nxrt_rocm_ep_supports_matmul_nbits(None, C.byref(a), descs, 5, reason, 512) == 1                      # act-order weights are taken
    a4 = E.make_attrs(K=64, N=8, bits=4, block_size=32, accuracy_level=4)
    assert lib.nxrt_rocm_ep_supports_matmul_nbits(None, C.byref(a4), descs, 5, reason, 512) == 0 and b"does not take g_idx" in reason.value
    descs, keep = E.make_descs([((1, 64), E.I32), ((8, 2, 16), E.U8), ((8, 2), E.F16)])
    assert lib.nxrt_rocm_ep_supports_matmul_nbits(None, C.byref(a), descs, 3, reason, 512) == 0
    assert reason.value == b"MatMulNBits: A must have dtype Float32, Float16, or BFloat16, got Int32"


def test_provider_creation_fails_loudly_without_gpu(lib):
    import torch
    if torch.cuda.is_available():
        pytest.skip("a GPU is visible here")
    with pytest.raises(E.EpError) as e:
        E.RocmExecutionProvider(0)
    assert e.value.code == 6 and "no HIP device is visible" in str(e.value)


def test_bench_refuses_more_than_one_gpu():
    import subprocess
    import sys
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert r.returncode != 0 and "one GPU only" in (r.stderr + r.stdout)


def test_build_reads_kernel_resource_remarks():
    """The build refuses kernels that use scratch memory; this pins how it reads the compiler's resource remarks."""
    from onnx_genai_amd import build
    tag = "[" + build.REMARKS + "]"
    err = "\n".join([
        "k.hip:25:1: remark: Function Name: kernel_a " + tag,
        "   25 | {",
        "      | ^",
        "k.hip:25:1: remark:     VGPRs: 17 " + tag,
        "k.hip:25:1: remark:     ScratchSize [bytes/lane]: 0 " + tag,
        "k.hip:25:1: remark:     VGPRs Spill: 0 " + tag,
        "k.hip:90:1: remark: Function Name: kernel_b " + tag,
        "k.hip:90:1: remark:     VGPRs: 256 " + tag,
        "k.hip:90:1: remark:     ScratchSize [bytes/lane]: 524 " + tag,
        "k.hip:90:1: remark:     VGPRs Spill: 158 " + tag,
        "k.hip:3:1: warning: unused variable 'x'",
        "    3 | int x;",
        "      | ^",
    ])
    usage = build._resource_usage(err)
    assert usage["kernel_a"] == {"VGPRs": 17, "ScratchSize [bytes/lane]": 0, "VGPRs Spill": 0}
    assert usage["kernel_b"]["ScratchSize [bytes/lane]"] == 524 and usage["kernel_b"]["VGPRs Spill"] == 158
    assert build._diagnostics(err) == "k.hip:3:1: warning: unused variable 'x'\n    3 | int x;\n      | ^"


def test_launcher_occupancy_table_matches_the_build():
    """The split-K launcher sizes mid-size launches by the waves per SIMD of the one-set builds: the figures it assumes are
    the ones the build reported for those kernels."""
    from onnx_genai_amd import build
    report = os.path.join(build.OBJ, "kernel_resources.txt")
    if not os.path.exists(report):
        pytest.skip("no build report in this tree")
    lib = C.CDLL(build.LIB)
    lib.rocm_decode_packed_waves_per_simd.restype = C.c_int
    lib.rocm_decode_packed_waves_per_simd.argtypes = [C.c_int, C.c_int, C.c_int, C.c_int]
    # _ZN3mnb20decode_packed_kernelILb<bf16>ELi<block>ELi<rows staged>E<t|f: scale type>Li<sets>ELb<pair>ELb<norm>EEEv...
    pat = re.compile(r"decode_packed_kernelILb([01])ELi(\d+)ELi(\d+)E([tf])Li1ELb0ELb0EEE\S* .*Occupancy \[waves/SIMD\]=(\d+)")
    seen = 0
    for line in open(report).read().splitlines():
        m = pat.search(line)
        if m:
            bf16, bs, rows, f32, built = int(m.group(1)), int(m.group(2)), int(m.group(3)), m.group(4) == "f", int(m.group(5))
            assert lib.rocm_decode_packed_waves_per_simd(bs, rows, int(f32), bf16) == built, line
            seen += 1
    assert seen == 2 * 3 * 4 * 2


class _FfiArgs(C.Structure):
    """RocmMatMulNBitsArgs of csrc/hip_ffi.h (the internal kernel-launch interface), for the calls below that do no GPU work."""
    _fields_ = [("a", C.c_void_p), ("b", C.c_void_p), ("scales", C.c_void_p), ("zp", C.c_void_p), ("bias", C.c_void_p), ("y", C.c_void_p),
                ("a_dtype", C.c_int), ("scale_dtype", C.c_int), ("bias_dtype", C.c_int), ("y_dtype", C.c_int),
                ("m", C.c_int64), ("n", C.c_int64), ("k", C.c_int64), ("block_size", C.c_int),
                ("g_idx", C.c_void_p), ("acc_probe", C.c_void_p), ("gamma", C.c_void_p), ("gamma_dtype", C.c_int), ("norm_epsilon", C.c_float)]


def _prefill_plan(lib, m, n, k, bf16=True, scratch=1 << 40):
    args = _FfiArgs()
    args.a, args.b, args.scales, args.y = 0x10000, 0x20000, 0x30000, 0x40000         # never dereferenced: alignment only
    args.a_dtype = args.scale_dtype = args.y_dtype = 16 if bf16 else 10
    args.m, args.n, args.k, args.block_size = m, n, k, 128
    rows, cols, slices = C.c_int(), C.c_int(), C.c_int()
    assert lib.rocm_prefill_mfma_plan(C.byref(args), 0, C.c_uint64(scratch), C.byref(rows), C.byref(cols), C.byref(slices)) == 0
    return rows.value, cols.value, slices.value


def test_prefill_plan_slices_long_k_on_short_grids():
    """The tiled prefill kernel's planner: tall calls on wide shapes take whole 256 x 256 tiles; a long K on a short grid takes
    the larger tiles over slices of K instead of small unsliced ones; without scratch nothing is sliced."""
    from onnx_genai_amd import build
    lib = C.CDLL(build.LIB)
    lib.rocm_prefill_mfma_plan.restype = C.c_int
    lib.rocm_prefill_mfma_plan.argtypes = [C.c_void_p, C.c_int, C.c_uint64, C.POINTER(C.c_int), C.POINTER(C.c_int), C.POINTER(C.c_int)]
    assert _prefill_plan(lib, 8192, 14336, 4096) == (256, 256, 1)
    assert _prefill_plan(lib, 4096, 37888, 3584) == (256, 256, 1)
    rows, cols, slices = _prefill_plan(lib, 1536, 3584, 18944)            # 336 tiles of 128 x 128 would run in two rounds on 256 CUs
    assert rows == 256 and slices >= 3
    rows, cols, slices = _prefill_plan(lib, 1536, 3584, 18944, scratch=0)
    assert slices == 1
    # every plan covers K: the slices are whole 64-element steps
    for m, n, k in [(256, 4096, 14336), (512, 3584, 18944), (3072, 4096, 14336), (300, 1000, 4160)]:
        rows, cols, slices = _prefill_plan(lib, m, n, k)
        assert rows in (128, 256) and cols in (64, 128, 256) and 1 <= slices <= 16 and slices <= k // 64


def test_built_kernels_use_no_scratch():
    """The report the last build wrote lists every kernel with zero scratch bytes and zero spilled registers."""
    from onnx_genai_amd import build
    report = os.path.join(build.OBJ, "kernel_resources.txt")
    if not os.path.exists(report):
        pytest.skip("no build report in this tree")
    lines = [l for l in open(report).read().splitlines() if l.strip()]
    assert len(lines) > 100
    for line in lines:
        assert "ScratchSize [bytes/lane]=0" in line and "VGPRs Spill=0" in line, line
