"""Host-side mirror of the reference's ExecutionProvider / Kernel interface for MatMulNBits,
bound to libnxrt_ep_rocm.so through its C ABI (include/nxrt_ep_rocm.h).

Names follow the reference (crates/onnx-runtime-ep-api): ExecutionProvider.allocate / deallocate /
copy_from_host / copy_to_host / sync / supports_op / get_kernel, Kernel.set_constant_inputs /
workspace_requirement / execute, TensorView, DeviceBuffer, EpError::KernelFailed. There is no CPU
fallback: if the library is missing or no GPU is visible, construction raises.
"""
from __future__ import annotations

import ctypes as C
import os
from dataclasses import dataclass

import numpy as np

from . import synth

F32, U8, I8, I32, F16, BF16 = 1, 2, 3, 6, 10, 16
DEVICE_ROCM = 2
_ITEM = {F32: 4, U8: 1, I8: 1, I32: 4, F16: 2, BF16: 2}

LIB_PATH = os.environ.get("NXRT_ROCM_LIBRARY") or os.path.join(os.path.dirname(os.path.abspath(__file__)), "lib", "libnxrt_ep_rocm.so")


class EpError(RuntimeError):
    """EpError from the reference's ep-api: carries the nxrt status code and message."""

    def __init__(self, code: int, message: str):
        super().__init__(message)
        self.code = code
        self.message = message


class NxrtStatus(C.Structure):
    _fields_ = [("code", C.c_uint32), ("message_len", C.c_uint32), ("message", C.c_uint8 * 256)]

    def text(self) -> str:
        return bytes(self.message[: self.message_len]).decode("utf-8", "replace")

    def check(self):
        if self.code != 0:
            raise EpError(self.code, self.text())


class NxrtTensorDesc(C.Structure):
    _fields_ = [("ndim", C.c_uint32), ("_pad", C.c_uint32), ("dims", C.POINTER(C.c_int64)), ("dtype", C.c_uint32), ("_pad2", C.c_uint32)]


class Attrs(C.Structure):
    _fields_ = [("struct_size", C.c_uint32), ("present", C.c_uint32), ("K", C.c_int64), ("N", C.c_int64), ("bits", C.c_int64),
                ("block_size", C.c_int64), ("accuracy_level", C.c_int64), ("weight_prepacked", C.c_int64), ("folded_bias", C.c_int64),
                ("gate_up_swiglu", C.c_int64), ("decomposed_silu", C.c_int64), ("rmsnorm_prologue", C.c_int64), ("rmsnorm_epsilon", C.c_double)]


class CTensorView(C.Structure):
    _fields_ = [("data", C.c_void_p), ("dtype", C.c_uint32), ("ndim", C.c_uint32), ("shape", C.POINTER(C.c_uint64)),
                ("strides", C.POINTER(C.c_int64)), ("byte_offset", C.c_uint64), ("device_type", C.c_uint32), ("device_index", C.c_uint32)]


class WorkspaceRequirement(C.Structure):
    _fields_ = [("bytes", C.c_uint64), ("alignment", C.c_uint64)]


_ATTR_BITS = {"K": 0, "N": 1, "bits": 2, "block_size": 3, "accuracy_level": 4, "weight_prepacked": 5, "folded_bias": 6, "gate_up_swiglu": 7,
              "decomposed_silu": 8, "rmsnorm_prologue": 9, "rmsnorm_epsilon": 10}
_lib = None


def load_library() -> C.CDLL:
    """dlopen the in-tree provider library and declare its entry points. Raises if it is not built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise FileNotFoundError(f"{LIB_PATH} is not built; run `python -m onnx_genai_amd.build` (needs hipcc)")
    L = C.CDLL(LIB_PATH)
    v, u32, u64, sz, S = C.c_void_p, C.c_uint32, C.c_uint64, C.c_size_t, NxrtStatus
    L.nxrt_rocm_ep_create.restype = S
    L.nxrt_rocm_ep_create.argtypes = [u32, C.POINTER(C.c_char_p), C.POINTER(C.c_char_p), u32, C.POINTER(v)]
    L.nxrt_rocm_ep_release.restype = None
    L.nxrt_rocm_ep_release.argtypes = [v]
    L.nxrt_rocm_ep_name.restype = C.c_char_p
    L.nxrt_rocm_ep_name.argtypes = [v]
    for fn in ("nxrt_rocm_ep_device_type", "nxrt_rocm_ep_device_id", "nxrt_rocm_ep_memory_vendor_id"):
        getattr(L, fn).restype = u32
        getattr(L, fn).argtypes = [v]
    L.nxrt_rocm_ep_device_info.restype = S
    L.nxrt_rocm_ep_device_info.argtypes = [v, C.c_char_p, sz, C.POINTER(u32), C.POINTER(u64)]
    L.nxrt_rocm_ep_allocate.restype = S
    L.nxrt_rocm_ep_allocate.argtypes = [v, sz, sz, C.POINTER(v)]
    L.nxrt_rocm_ep_deallocate.restype = S
    L.nxrt_rocm_ep_deallocate.argtypes = [v, v]
    L.nxrt_rocm_ep_copy_from_host.restype = S
    L.nxrt_rocm_ep_copy_from_host.argtypes = [v, v, v, sz]
    L.nxrt_rocm_ep_copy_to_host.restype = S
    L.nxrt_rocm_ep_copy_to_host.argtypes = [v, v, v, sz]
    L.nxrt_rocm_ep_copy.restype = S
    L.nxrt_rocm_ep_copy.argtypes = [v, v, v, sz]
    L.nxrt_rocm_ep_read_probe.restype = S
    L.nxrt_rocm_ep_read_probe.argtypes = [v, v, sz]
    L.nxrt_rocm_ep_lds_probe.restype = S
    L.nxrt_rocm_ep_lds_probe.argtypes = [v, u32, u32, u32, C.POINTER(C.c_double)]
    L.nxrt_rocm_ep_sync.restype = S
    L.nxrt_rocm_ep_sync.argtypes = [v]
    L.nxrt_rocm_ep_from_vtable.restype = v
    L.nxrt_rocm_ep_from_vtable.argtypes = [v]
    L.nxrt_rocm_ep_supports_matmul_nbits.restype = C.c_int
    L.nxrt_rocm_ep_supports_matmul_nbits.argtypes = [v, C.POINTER(Attrs), C.POINTER(NxrtTensorDesc), u32, C.c_char_p, sz]
    L.nxrt_rocm_matmul_nbits_create.restype = S
    L.nxrt_rocm_matmul_nbits_create.argtypes = [v, C.POINTER(Attrs), C.POINTER(NxrtTensorDesc), u32, C.POINTER(v)]
    L.nxrt_rocm_matmul_nbits_set_constant_inputs.restype = None
    L.nxrt_rocm_matmul_nbits_set_constant_inputs.argtypes = [v, C.POINTER(C.c_uint8), u32]
    L.nxrt_rocm_matmul_nbits_workspace_requirement.restype = S
    L.nxrt_rocm_matmul_nbits_workspace_requirement.argtypes = [v, C.POINTER(NxrtTensorDesc), u32, C.POINTER(WorkspaceRequirement)]
    L.nxrt_rocm_matmul_nbits_execute.restype = S
    L.nxrt_rocm_matmul_nbits_execute.argtypes = [v, C.POINTER(CTensorView), u32, C.POINTER(CTensorView), u32, v, u64]
    L.nxrt_rocm_matmul_nbits_execute_static.restype = S
    L.nxrt_rocm_matmul_nbits_execute_static.argtypes = [v, C.POINTER(CTensorView), u32, C.POINTER(CTensorView), u32]
    L.nxrt_rocm_device_allocation_count.restype = u64
    L.nxrt_rocm_device_allocation_count.argtypes = []
    L.nxrt_rocm_matmul_nbits_estimated_flops.restype = u64
    L.nxrt_rocm_matmul_nbits_estimated_flops.argtypes = [v]
    L.nxrt_rocm_matmul_nbits_last_variant.restype = C.c_char_p
    L.nxrt_rocm_matmul_nbits_last_variant.argtypes = [v]
    L.nxrt_rocm_matmul_nbits_last_metrics.restype = None
    L.nxrt_rocm_matmul_nbits_last_metrics.argtypes = [v, C.POINTER(u64), C.POINTER(u64)]
    L.nxrt_rocm_matmul_nbits_release.restype = None
    L.nxrt_rocm_matmul_nbits_release.argtypes = [v]
    L.nxrt_rocm_matmul_nbits_set_block_acc_probe.restype = S
    L.nxrt_rocm_matmul_nbits_set_block_acc_probe.argtypes = [v, v, u64]
    L.nxrt_rocm_matmul_nbits_retired_buffers.restype = u64
    L.nxrt_rocm_matmul_nbits_retired_buffers.argtypes = [v]
    L.nxrt_rocm_matmul_nbits_as_vtable.restype = S
    L.nxrt_rocm_matmul_nbits_as_vtable.argtypes = [v, C.POINTER(v)]
    L.nxrt_rocm_matmul_nbits_dequantize.restype = S
    L.nxrt_rocm_matmul_nbits_dequantize.argtypes = [v, v, v, u32, v, u64, u64, u32, v]
    L.nxrt_rocm_matmul_nbits_dequantize_bits.restype = S
    L.nxrt_rocm_matmul_nbits_dequantize_bits.argtypes = [v, v, v, u32, v, u64, u64, u32, u32, v]
    L.nxrt_rocm_matmul_nbits_quantize_a.restype = S
    L.nxrt_rocm_matmul_nbits_quantize_a.argtypes = [v, v, u32, u64, u64, u32, u32, v, v]
    L.nxrt_rocm_matmul_nbits_block_acc.restype = S
    L.nxrt_rocm_matmul_nbits_block_acc.argtypes = [v, v, v, v, u64, u64, u64, u32, v]
    L.nxrt_rocm_ep_event_create.restype = S
    L.nxrt_rocm_ep_event_create.argtypes = [v, C.POINTER(v)]
    L.nxrt_rocm_ep_event_record.restype = S
    L.nxrt_rocm_ep_event_record.argtypes = [v, v]
    L.nxrt_rocm_ep_event_elapsed_ms.restype = S
    L.nxrt_rocm_ep_event_elapsed_ms.argtypes = [v, v, v, C.POINTER(C.c_float)]
    L.nxrt_rocm_ep_event_destroy.restype = None
    L.nxrt_rocm_ep_event_destroy.argtypes = [v, v]
    L.nxrt_rocm_ep_capture_begin.restype = S
    L.nxrt_rocm_ep_capture_begin.argtypes = [v]
    L.nxrt_rocm_ep_capture_end.restype = S
    L.nxrt_rocm_ep_capture_end.argtypes = [v, C.POINTER(v), C.POINTER(u64)]
    L.nxrt_rocm_ep_graph_replay.restype = S
    L.nxrt_rocm_ep_graph_replay.argtypes = [v, v]
    L.nxrt_rocm_ep_graph_release.restype = None
    L.nxrt_rocm_ep_graph_release.argtypes = [v, v]
    L.nxrt_rocm_ep_kernel_launch_count.restype = u64
    L.nxrt_rocm_ep_kernel_launch_count.argtypes = [v]
    L.nxrt_rocm_live_provider_count.restype = u64
    L.nxrt_rocm_live_provider_count.argtypes = []
    _lib = L
    return L


def make_attrs(**kw) -> Attrs:
    """Node attributes; only the names passed are marked present (a missing K must be reported as missing)."""
    a = Attrs()
    a.struct_size = C.sizeof(Attrs)
    for name, value in kw.items():
        if value is None:
            continue
        a.present |= 1 << _ATTR_BITS[name]
        setattr(a, name, float(value) if name == "rmsnorm_epsilon" else int(value))
    return a


def make_descs(shapes_dtypes):
    """[(shape or None, dtype)] -> (array of NxrtTensorDesc, keep-alive list)."""
    n = len(shapes_dtypes)
    arr = (NxrtTensorDesc * max(n, 1))()
    keep = []
    for i, (shape, dtype) in enumerate(shapes_dtypes):
        if shape is None:
            arr[i].ndim = 0
            arr[i].dtype = 0
            continue
        dims = (C.c_int64 * max(len(shape), 1))(*[int(d) for d in shape])
        keep.append(dims)
        arr[i].ndim = len(shape)
        arr[i].dims = C.cast(dims, C.POINTER(C.c_int64))
        arr[i].dtype = dtype
    return arr, keep


@dataclass
class DeviceBuffer:
    """DeviceBuffer of the reference: a raw device allocation owned by one provider."""
    ptr: int
    nbytes: int


@dataclass
class TensorView:
    """TensorView / TensorMut of the reference (ep-api tensor.rs:132-143). data=None marks an absent optional input."""
    data: int | None
    dtype: int
    shape: tuple
    strides: tuple | None = None
    byte_offset: int = 0
    device_type: int = DEVICE_ROCM
    device_index: int = 0

    @staticmethod
    def absent(dtype: int = 0) -> "TensorView":
        return TensorView(None, dtype, ())


def _c_views(views):
    arr = (CTensorView * max(len(views), 1))()
    keep = []
    for i, t in enumerate(views):
        shape = (C.c_uint64 * max(len(t.shape), 1))(*[int(d) for d in t.shape])
        keep.append(shape)
        arr[i].data = t.data
        arr[i].dtype = t.dtype
        arr[i].ndim = len(t.shape)
        arr[i].shape = C.cast(shape, C.POINTER(C.c_uint64))
        if t.strides is not None:
            st = (C.c_int64 * max(len(t.strides), 1))(*[int(s) for s in t.strides])
            keep.append(st)
            arr[i].strides = C.cast(st, C.POINTER(C.c_int64))
        arr[i].byte_offset = t.byte_offset
        arr[i].device_type = t.device_type
        arr[i].device_index = t.device_index
    return arr, keep


class RocmExecutionProvider:
    """ExecutionProvider for one MI355X. `config` is the reference's EpConfig string map."""

    def __init__(self, device_ordinal: int = 0, config: dict | None = None):
        self.lib = load_library()
        config = config or {}
        n = len(config)
        keys = (C.c_char_p * max(n, 1))(*[k.encode() for k in config])
        vals = (C.c_char_p * max(n, 1))(*[str(v).encode() for v in config.values()])
        handle = C.c_void_p()
        self.lib.nxrt_rocm_ep_create(device_ordinal, keys, vals, n, C.byref(handle)).check()
        self.handle = handle
        self.device_index = device_ordinal

    # -- identity ---------------------------------------------------------------------------------
    def name(self) -> str:
        return self.lib.nxrt_rocm_ep_name(self.handle).decode()

    def device_type(self) -> int:
        return self.lib.nxrt_rocm_ep_device_type(self.handle)

    def device_id(self) -> int:
        return self.lib.nxrt_rocm_ep_device_id(self.handle)

    def memory_vendor_id(self) -> int:
        return self.lib.nxrt_rocm_ep_memory_vendor_id(self.handle)

    def device_info(self) -> dict:
        arch = C.create_string_buffer(64)
        cus, mem = C.c_uint32(), C.c_uint64()
        self.lib.nxrt_rocm_ep_device_info(self.handle, arch, 64, C.byref(cus), C.byref(mem)).check()
        return {"arch": arch.value.decode(), "compute_units": cus.value, "total_memory": mem.value}

    # -- memory -----------------------------------------------------------------------------------
    def allocate(self, size: int, align: int = 256) -> DeviceBuffer:
        p = C.c_void_p()
        self.lib.nxrt_rocm_ep_allocate(self.handle, size, align, C.byref(p)).check()
        return DeviceBuffer(p.value, size)

    def deallocate(self, buf: DeviceBuffer) -> None:
        self.lib.nxrt_rocm_ep_deallocate(self.handle, buf.ptr).check()

    def copy_from_host(self, dst: DeviceBuffer | int, src: np.ndarray, offset: int = 0) -> None:
        src = np.ascontiguousarray(src)
        ptr = (dst.ptr if isinstance(dst, DeviceBuffer) else dst) + offset
        self.lib.nxrt_rocm_ep_copy_from_host(self.handle, ptr, src.ctypes.data, src.nbytes).check()

    def copy_to_host(self, dst: np.ndarray, src: DeviceBuffer | int, offset: int = 0) -> None:
        assert dst.flags["C_CONTIGUOUS"]
        ptr = (src.ptr if isinstance(src, DeviceBuffer) else src) + offset
        self.lib.nxrt_rocm_ep_copy_to_host(self.handle, dst.ctypes.data, ptr, dst.nbytes).check()

    def copy(self, dst: DeviceBuffer, src: DeviceBuffer, nbytes: int) -> None:
        self.lib.nxrt_rocm_ep_copy(self.handle, dst.ptr, src.ptr, nbytes).check()

    def read_probe(self, src: DeviceBuffer, nbytes: int) -> None:
        """Enqueues a plain read of `nbytes` of `src` (a benchmark's yardstick: the least time a kernel can take to pull them)."""
        self.lib.nxrt_rocm_ep_read_probe(self.handle, src.ptr, nbytes).check()

    def lds_probe(self, mode: int, waves: int, iters: int = 2000) -> float:
        """Bytes per clock one CU's LDS moves (mode 0 reads, 1 writes, 2 global memory straight into LDS, 3 reads and writes mixed)."""
        out = C.c_double()
        self.lib.nxrt_rocm_ep_lds_probe(self.handle, mode, waves, iters, C.byref(out)).check()
        return out.value

    def sync(self) -> None:
        self.lib.nxrt_rocm_ep_sync(self.handle).check()

    def upload(self, arr: np.ndarray) -> DeviceBuffer:
        arr = np.ascontiguousarray(arr)
        buf = self.allocate(max(arr.nbytes, 1))
        if arr.nbytes:
            self.copy_from_host(buf, arr)
        return buf

    def download(self, buf: DeviceBuffer, shape, np_dtype) -> np.ndarray:
        out = np.empty(shape, np_dtype)
        if out.nbytes:
            self.copy_to_host(out, buf)
        return out

    # -- operator ---------------------------------------------------------------------------------
    def supports_op(self, attrs: dict, inputs=None):
        """-> (True, "") or (False, reason). inputs: [(shape or None, dtype)] for A, B, scales, ..."""
        a = make_attrs(**attrs)
        reason = C.create_string_buffer(512)
        if inputs is None:
            ok = self.lib.nxrt_rocm_ep_supports_matmul_nbits(self.handle, C.byref(a), None, 0, reason, 512)
        else:
            descs, keep = make_descs(inputs)
            ok = self.lib.nxrt_rocm_ep_supports_matmul_nbits(self.handle, C.byref(a), descs, len(inputs), reason, 512)
        return bool(ok), reason.value.decode()

    def get_kernel(self, attrs: dict, input_shapes=None) -> "MatMulNBitsKernel":
        return MatMulNBitsKernel(self, attrs, input_shapes)

    # -- pieces -----------------------------------------------------------------------------------
    def dequantize(self, b: DeviceBuffer, scales: DeviceBuffer, scale_dtype: int, zp: DeviceBuffer | None, n, k, bs, out: DeviceBuffer, bits: int = 4) -> None:
        if bits == 4:
            self.lib.nxrt_rocm_matmul_nbits_dequantize(self.handle, b.ptr, scales.ptr, scale_dtype, zp.ptr if zp else None, n, k, bs, out.ptr).check()
        else:
            self.lib.nxrt_rocm_matmul_nbits_dequantize_bits(self.handle, b.ptr, scales.ptr, scale_dtype, zp.ptr if zp else None, n, k, bs, bits, out.ptr).check()

    def quantize_a(self, a: DeviceBuffer, a_dtype: int, m, k, bs, rounding: int, qa: DeviceBuffer, qscale: DeviceBuffer) -> None:
        self.lib.nxrt_rocm_matmul_nbits_quantize_a(self.handle, a.ptr, a_dtype, m, k, bs, rounding, qa.ptr, qscale.ptr).check()

    def block_acc(self, qa: DeviceBuffer, b: DeviceBuffer, zp: DeviceBuffer | None, m, n, k, bs, acc: DeviceBuffer) -> None:
        self.lib.nxrt_rocm_matmul_nbits_block_acc(self.handle, qa.ptr, b.ptr, zp.ptr if zp else None, m, n, k, bs, acc.ptr).check()

    # -- graph capture ----------------------------------------------------------------------------
    def capture_begin(self) -> None:
        self.lib.nxrt_rocm_ep_capture_begin(self.handle).check()

    def capture_end(self) -> "Graph":
        h, nodes = C.c_void_p(), C.c_uint64()
        self.lib.nxrt_rocm_ep_capture_end(self.handle, C.byref(h), C.byref(nodes)).check()
        return Graph(self, h, nodes.value)

    # -- timing -----------------------------------------------------------------------------------
    def event(self) -> "Event":
        return Event(self)

    def kernel_launch_count(self) -> int:
        return self.lib.nxrt_rocm_ep_kernel_launch_count(self.handle)

    def shutdown(self) -> None:
        if self.handle:
            self.lib.nxrt_rocm_ep_release(self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.shutdown()
        except Exception:
            pass


class Graph:
    """A recorded sequence of launches on the provider's stream (a HIP graph)."""

    def __init__(self, ep, handle, num_nodes):
        self.ep, self.handle, self.num_nodes = ep, handle, num_nodes

    def replay(self) -> None:
        self.ep.lib.nxrt_rocm_ep_graph_replay(self.ep.handle, self.handle).check()

    def release(self) -> None:
        if self.handle and self.ep.handle:
            self.ep.lib.nxrt_rocm_ep_graph_release(self.ep.handle, self.handle)
        self.handle = None

    def __del__(self):
        try:
            self.release()
        except Exception:
            pass


class Event:
    """A HIP event on the provider's stream."""

    def __init__(self, ep: RocmExecutionProvider):
        self.ep = ep
        h = C.c_void_p()
        ep.lib.nxrt_rocm_ep_event_create(ep.handle, C.byref(h)).check()
        self.handle = h

    def record(self) -> None:
        self.ep.lib.nxrt_rocm_ep_event_record(self.ep.handle, self.handle).check()

    def elapsed_ms(self, stop: "Event") -> float:
        ms = C.c_float()
        self.ep.lib.nxrt_rocm_ep_event_elapsed_ms(self.ep.handle, self.handle, stop.handle, C.byref(ms)).check()
        return ms.value

    def __del__(self):
        try:
            if self.handle and self.ep.handle:
                self.ep.lib.nxrt_rocm_ep_event_destroy(self.ep.handle, self.handle)
        except Exception:
            pass


class MatMulNBitsKernel:
    """Kernel of the reference (ep-api kernel.rs:548-706) for one MatMulNBits node."""

    def __init__(self, ep: RocmExecutionProvider, attrs: dict, input_shapes=None):
        self.ep = ep
        self.lib = ep.lib
        a = make_attrs(**attrs)
        h = C.c_void_p()
        if input_shapes is None:
            st = self.lib.nxrt_rocm_matmul_nbits_create(ep.handle, C.byref(a), None, 0, C.byref(h))
        else:
            descs, keep = make_descs(input_shapes)
            st = self.lib.nxrt_rocm_matmul_nbits_create(ep.handle, C.byref(a), descs, len(input_shapes), C.byref(h))
        st.check()
        self.handle = h

    def set_constant_inputs(self, flags) -> None:
        arr = (C.c_uint8 * max(len(flags), 1))(*[1 if f else 0 for f in flags])
        self.lib.nxrt_rocm_matmul_nbits_set_constant_inputs(self.handle, arr, len(flags))

    def workspace_requirement(self, input_shapes) -> tuple[int, int]:
        descs, keep = make_descs(input_shapes)
        out = WorkspaceRequirement()
        self.lib.nxrt_rocm_matmul_nbits_workspace_requirement(self.handle, descs, len(input_shapes), C.byref(out)).check()
        return out.bytes, out.alignment

    def execute(self, inputs, outputs, workspace: DeviceBuffer | None = None) -> None:
        cin, k1 = _c_views(inputs)
        cout, k2 = _c_views(outputs)
        self.lib.nxrt_rocm_matmul_nbits_execute(self.handle, cin, len(inputs), cout, len(outputs),
                                                workspace.ptr if workspace else None, workspace.nbytes if workspace else 0).check()

    def execute_static(self, inputs, outputs) -> None:
        """execute without any device allocation: scratch comes from the library's static per-GPU array."""
        cin, k1 = _c_views(inputs)
        cout, k2 = _c_views(outputs)
        self.lib.nxrt_rocm_matmul_nbits_execute_static(self.handle, cin, len(inputs), cout, len(outputs)).check()

    def estimated_flops(self) -> int:
        return self.lib.nxrt_rocm_matmul_nbits_estimated_flops(self.handle)

    def last_variant(self) -> str:
        return self.lib.nxrt_rocm_matmul_nbits_last_variant(self.handle).decode()

    def last_metrics(self) -> tuple[int, int]:
        """(flops, bytes) of the last plain call, by the reference's count (record_kernel_metrics)."""
        flops, nbytes = C.c_uint64(), C.c_uint64()
        self.lib.nxrt_rocm_matmul_nbits_last_metrics(self.handle, C.byref(flops), C.byref(nbytes))
        return flops.value, nbytes.value

    def set_block_acc_probe(self, buf: DeviceBuffer | None) -> None:
        """accuracy_level 4: later executes also store their int32 block accumulators [M, N, kb] into `buf` (None clears)."""
        self.lib.nxrt_rocm_matmul_nbits_set_block_acc_probe(self.handle, buf.ptr if buf else None, buf.nbytes // 4 if buf else 0).check()

    def retired_buffers(self) -> int:
        return self.lib.nxrt_rocm_matmul_nbits_retired_buffers(self.handle)

    def release(self) -> None:
        if self.handle:
            self.lib.nxrt_rocm_matmul_nbits_release(self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.release()              # safe after the provider's own release: the kernel holds a reference to it
        except Exception:
            pass


_NP = {F32: np.float32, F16: np.float16, BF16: np.uint16, U8: np.uint8, I8: np.int8, I32: np.int32}


class DeviceOperands:
    """The device-resident operands of one MatMulNBits node plus its kernel; what a session would hold."""

    def __init__(self, ep, b, scales, scale_dtype, zp, n, k, bs, *, accuracy_level=0, bias=None, bias_dtype=F32, rows=None, a_dtype=None,
                 folded_bias=None, gamma=None, gamma_dtype=F32, rmsnorm_epsilon=None, bits=4, g_idx=None, bias_shape=None):
        self.ep, self.n, self.k, self.bs, self.bits = ep, n, k, bs, bits
        self.bias_shape = bias_shape                                          # the shape the bias view declares (default: [N], or [M, N] for a residual)
        self.g_idx = ep.upload(np.ascontiguousarray(g_idx, np.int32)) if g_idx is not None else None      # act-order groups, input 4
        self.kb = -(-k // bs)
        self.scale_dtype, self.bias_dtype = scale_dtype, bias_dtype
        self.b = ep.upload(np.asarray(b, np.uint8))
        self.scales = ep.upload(scales)
        self.zp = ep.upload(np.asarray(zp, np.uint8)) if zp is not None else None
        self.bias = ep.upload(bias) if bias is not None else None
        self.bias_per_row = bias is not None and np.asarray(bias).size != n      # a folded residual [M, N] in the bias slot
        self.gamma = ep.upload(gamma) if gamma is not None else None        # RMS-normalization prologue: gamma [K] at input 6
        self.gamma_dtype = gamma_dtype
        shapes = None
        if rows is not None and a_dtype is not None:
            shapes = [((rows, k), a_dtype), ((n, self.kb, bs * bits // 8), U8), ((n, self.kb), scale_dtype)]
        self.kernel = ep.get_kernel({"K": k, "N": n, "bits": bits, "block_size": bs, "accuracy_level": accuracy_level, "folded_bias": folded_bias,
                                     "rmsnorm_prologue": 1 if gamma is not None else None, "rmsnorm_epsilon": rmsnorm_epsilon}, shapes)
        self.kernel.set_constant_inputs([False, True, True, True, True, True, True])

    def views(self, a_buf: DeviceBuffer, a_dtype: int, m: int):
        dev = self.ep.device_index
        ins = [TensorView(a_buf.ptr, a_dtype, (m, self.k), device_index=dev),
               TensorView(self.b.ptr, U8, (self.n, self.kb, self.bs * self.bits // 8), device_index=dev),
               TensorView(self.scales.ptr, self.scale_dtype, (self.n, self.kb), device_index=dev)]
        if self.zp is not None or self.bias is not None or self.gamma is not None or self.g_idx is not None:
            ins.append(TensorView(self.zp.ptr, U8, (self.n, (self.kb * self.bits + 7) // 8), device_index=dev) if self.zp is not None else TensorView.absent(U8))
        if self.g_idx is not None and self.bias is None and self.gamma is None:
            ins.append(TensorView(self.g_idx.ptr, I32, (self.k,), device_index=dev))
        if self.bias is not None or self.gamma is not None:
            ins.append(TensorView(self.g_idx.ptr, I32, (self.k,), device_index=dev) if self.g_idx is not None else TensorView.absent(I32))
            bias_shape = self.bias_shape or ((m, self.n) if self.bias_per_row else (self.n,))
            ins.append(TensorView(self.bias.ptr, self.bias_dtype, bias_shape, device_index=dev) if self.bias is not None else TensorView.absent(F32))
        if self.gamma is not None:
            ins.append(TensorView(self.gamma.ptr, self.gamma_dtype, (self.k,), device_index=dev))
        return ins

    def run(self, a_buf: DeviceBuffer, a_dtype: int, m: int, y_buf: DeviceBuffer, y_dtype: int | None = None) -> None:
        y_dtype = a_dtype if y_dtype is None else y_dtype
        out = [TensorView(y_buf.ptr, y_dtype, (m, self.n), device_index=self.ep.device_index)]
        self.kernel.execute(self.views(a_buf, a_dtype, m), out)

    def free(self) -> None:
        self.kernel.release()
        for buf in (self.b, self.scales, self.zp, self.bias, self.gamma, self.g_idx):
            if buf is not None:
                self.ep.deallocate(buf)


def matmul_nbits(ep, a, a_dtype, b, scales, scale_dtype, zp, n, k, bs, *, accuracy_level=0, bias=None, bias_dtype=F32, y_dtype=None, folded_bias=None,
                 gamma=None, gamma_dtype=F32, rmsnorm_epsilon=None, bits=4, g_idx=None, bias_shape=None):
    """One-shot helper: upload, execute through the C ABI, download. Returns (Y as numpy, variant name)."""
    y_dtype = a_dtype if y_dtype is None else y_dtype
    a = np.ascontiguousarray(a)
    m = a.size // k
    ops = DeviceOperands(ep, b, scales, scale_dtype, zp, n, k, bs, accuracy_level=accuracy_level, bias=bias, bias_dtype=bias_dtype, folded_bias=folded_bias,
                         gamma=gamma, gamma_dtype=gamma_dtype, rmsnorm_epsilon=rmsnorm_epsilon, bits=bits, g_idx=g_idx, bias_shape=bias_shape)
    a_buf = ep.upload(a)
    y_buf = ep.allocate(max(m * n * _ITEM[y_dtype], 1))
    try:
        ops.run(a_buf, a_dtype, m, y_buf, y_dtype)
        y = ep.download(y_buf, (m, n), _NP[y_dtype])
        variant = ops.kernel.last_variant()
    finally:
        ep.deallocate(a_buf)
        ep.deallocate(y_buf)
        ops.free()
    return y, variant


class GateUpOperands:
    """Device-resident operands of the fused gate/up node (inputs [x, W_gate, scales_gate, W_up, scales_up, -, zp_gate, zp_up])."""

    def __init__(self, ep, gate, up, scale_dtype, n, k, bs, *, decomposed=False, rows=None, a_dtype=None, gamma=None, gamma_dtype=F32, rmsnorm_epsilon=None,
                 accuracy_level=None):
        self.ep, self.n, self.k, self.bs, self.scale_dtype = ep, n, k, bs, scale_dtype
        self.kb = -(-k // bs)
        self.bufs = []
        for b, s, zp in (gate, up):
            self.bufs.append((ep.upload(np.asarray(b, np.uint8)), ep.upload(s), ep.upload(np.asarray(zp, np.uint8)) if zp is not None else None))
        shapes = [((rows, k), a_dtype)] if rows is not None and a_dtype is not None else None
        self.gamma = ep.upload(gamma) if gamma is not None else None
        self.gamma_dtype = gamma_dtype
        self.kernel = ep.get_kernel({"K": k, "N": n, "bits": 4, "block_size": bs, "gate_up_swiglu": 1, "decomposed_silu": 1 if decomposed else None,
                                     "accuracy_level": accuracy_level, "rmsnorm_prologue": 1 if gamma is not None else None, "rmsnorm_epsilon": rmsnorm_epsilon}, shapes)
        self.kernel.set_constant_inputs([False, True, True, True, True, True, True, True])

    def views(self, a_buf: DeviceBuffer, a_dtype: int, m: int):
        dev = self.ep.device_index
        (bg, sg, zg), (bu, su, zu) = self.bufs
        w_shape, s_shape, z_shape = (self.n, self.kb, self.bs // 2), (self.n, self.kb), (self.n, (self.kb + 1) // 2)
        ins = [TensorView(a_buf.ptr, a_dtype, (m, self.k), device_index=dev),
               TensorView(bg.ptr, U8, w_shape, device_index=dev), TensorView(sg.ptr, self.scale_dtype, s_shape, device_index=dev),
               TensorView(bu.ptr, U8, w_shape, device_index=dev), TensorView(su.ptr, self.scale_dtype, s_shape, device_index=dev)]
        gamma = TensorView(self.gamma.ptr, self.gamma_dtype, (self.k,), device_index=dev) if self.gamma is not None else None
        if zg is not None:
            ins += [gamma or TensorView.absent(F32), TensorView(zg.ptr, U8, z_shape, device_index=dev), TensorView(zu.ptr, U8, z_shape, device_index=dev)]
        elif gamma is not None:
            ins.append(gamma)
        return ins

    def run(self, a_buf: DeviceBuffer, a_dtype: int, m: int, y_buf: DeviceBuffer, workspace: DeviceBuffer | None = None) -> None:
        out = [TensorView(y_buf.ptr, a_dtype, (m, self.n), device_index=self.ep.device_index)]
        self.kernel.execute(self.views(a_buf, a_dtype, m), out, workspace=workspace)

    def free(self) -> None:
        self.kernel.release()
        for group in self.bufs + [(self.gamma,)]:
            for buf in group:
                if buf is not None:
                    self.ep.deallocate(buf)


def gate_up_swiglu(ep, a, a_dtype, gate, up, scale_dtype, n, k, bs, *, decomposed=False, gamma=None, gamma_dtype=F32, rmsnorm_epsilon=None):
    """One-shot helper for the fused gate/up node: gate and up are (B, scales, zero_points or None). Returns (Y, variant)."""
    a = np.ascontiguousarray(a)
    m = a.size // k
    ops = GateUpOperands(ep, gate, up, scale_dtype, n, k, bs, decomposed=decomposed, gamma=gamma, gamma_dtype=gamma_dtype, rmsnorm_epsilon=rmsnorm_epsilon)
    a_buf = ep.upload(a)
    y_buf = ep.allocate(max(m * n * 2, 1))
    try:
        ops.run(a_buf, a_dtype, m, y_buf)
        y = ep.download(y_buf, (m, n), _NP[a_dtype])
        variant = ops.kernel.last_variant()
    finally:
        ep.deallocate(a_buf)
        ep.deallocate(y_buf)
        ops.free()
    return y, variant


__all__ = ["RocmExecutionProvider", "GateUpOperands", "gate_up_swiglu", "MatMulNBitsKernel", "TensorView", "DeviceBuffer", "DeviceOperands", "EpError", "matmul_nbits",
           "load_library", "make_attrs", "make_descs", "synth", "F32", "U8", "I8", "I32", "F16", "BF16"]
