"""ctypes bindings for the two CPU checkers of the int4 MatMulNBits path.

TEST INFRASTRUCTURE ONLY. `port` is this repository's plain-C restatement
(oracle/matmul_nbits_oracle.c); `ref` is the reference's own vendored MLAS + plain-C shim
(crates/mlas-sys/vendor) compiled by oracle/Makefile into oracle/_ref/libmlas_ref.so.
Only tests, the smoke check and the benchmark's cpu_baseline leg import this module; the
product package never does.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
PORT_SO = os.path.join(_HERE, "liboracle_port.so")
REF_SO = os.path.join(_HERE, "_ref", "libmlas_ref.so")

ROUND_HALF_EVEN = 0  # MLAS rule
ROUND_HALF_AWAY = 1  # native Rust rule

F32, U8, I32, F16, BF16 = 1, 2, 6, 10, 16
_NP_DT = {F32: np.float32, F16: np.float16, BF16: np.uint16}


def build(ref: bool | None = None) -> None:
    """Compile the C restatement, and the reference MLAS when its sources are present."""
    subprocess.run(["make", "-s", "-C", _HERE, "port"], check=True)
    if ref is None:
        ref = os.path.isdir("/root/reference/crates/mlas-sys/vendor")
    if ref:
        subprocess.run(["make", "-s", "-j8", "-C", _HERE, "ref"], check=True)


def _ptr(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def _c(a, dtype):
    return None if a is None else np.ascontiguousarray(a, dtype=dtype)


def dtype_code(arr: np.ndarray, bf16: bool = False) -> int:
    if arr.dtype == np.float32:
        return F32
    if arr.dtype == np.float16:
        return F16
    if arr.dtype == np.uint16 and bf16:
        return BF16
    raise TypeError(f"unsupported dtype {arr.dtype}")


class Port:
    """The repo's C restatement (matmul_nbits_oracle.h)."""

    def __init__(self):
        if not os.path.exists(PORT_SO):
            build(ref=False)
        self.lib = C.CDLL(PORT_SO)
        L = self.lib
        L.mnb_f16_to_f32.restype = C.c_float
        L.mnb_f16_to_f32.argtypes = [C.c_uint16]
        L.mnb_f32_to_f16.restype = C.c_uint16
        L.mnb_f32_to_f16.argtypes = [C.c_float]
        L.mnb_bf16_to_f32.restype = C.c_float
        L.mnb_bf16_to_f32.argtypes = [C.c_uint16]
        L.mnb_f32_to_bf16.restype = C.c_uint16
        L.mnb_f32_to_bf16.argtypes = [C.c_float]
        z = C.c_size_t
        v = C.c_void_p
        L.mnb_widen.argtypes = [v, C.c_int, z, v]
        L.mnb_narrow.argtypes = [v, z, C.c_int, v]
        L.mnb_dequantize_nk.argtypes = [v, v, v, z, z, z, v]
        L.mnb_matmul_dequant_f32.argtypes = [v, v, v, z, z, z, v]
        L.mnb_matmul_f64.argtypes = [v, v, v, v, v, z, z, z, z, v]
        L.mnb_matmul_blocksum_f32.argtypes = [v, v, v, v, v, z, z, z, z, v]
        L.mnb_quantize_a.argtypes = [v, z, z, z, C.c_int, v, v]
        L.mnb_block_acc_i32.argtypes = [v, v, v, z, z, z, z, v]
        L.mnb_matmul_acc4_f32.argtypes = [v, v, v, v, v, z, z, z, z, C.c_int, v]
        L.mnb_swiglu_silu.restype = C.c_float
        L.mnb_swiglu_silu.argtypes = [C.c_float]
        L.mnb_swiglu_silu_decomposed.restype = C.c_float
        L.mnb_swiglu_silu_decomposed.argtypes = [C.c_float, C.c_int]
        L.mnb_swiglu.argtypes = [v, v, z, C.c_int, C.c_int, v]
        L.mnb_rmsnorm16.argtypes = [v, v, C.c_int, z, z, C.c_float, C.c_int, v]
        L.mnb_dequantize_nk_bits.argtypes = [v, v, v, z, z, z, C.c_int, v]
        L.mnb_matmul_f64_bits.argtypes = [v, v, v, v, v, z, z, z, z, C.c_int, v]
        L.mnb_dequantize_nk_gidx.restype = C.c_long
        L.mnb_dequantize_nk_gidx.argtypes = [v, v, v, v, z, z, z, C.c_int, v]
        L.mnb_matmul_nbits.restype = C.c_int
        L.mnb_matmul_nbits.argtypes = [v, C.c_int, v, v, C.c_int, v, v, C.c_int, v, C.c_int, z, z, z, z, C.c_int, C.c_int]

    # -- conversions -------------------------------------------------------------------------
    def widen(self, src: np.ndarray, code: int) -> np.ndarray:
        src = np.ascontiguousarray(src)
        out = np.empty(src.shape, np.float32)
        self.lib.mnb_widen(_ptr(src), code, src.size, _ptr(out))
        return out

    def narrow(self, src: np.ndarray, code: int) -> np.ndarray:
        src = _c(src, np.float32)
        out = np.empty(src.shape, _NP_DT[code])
        self.lib.mnb_narrow(_ptr(src), src.size, code, _ptr(out))
        return out

    # -- the CUDA provider's fused gate/up epilogue ------------------------------------------------
    def swiglu(self, gate16: np.ndarray, up16: np.ndarray, code: int, decomposed: bool = False) -> np.ndarray:
        """round16(silu(gate) * up) on 16-bit inputs (f16 arrays, or bf16 bit patterns as uint16)."""
        gate16, up16 = np.ascontiguousarray(gate16), np.ascontiguousarray(up16)
        out = np.empty(gate16.shape, _NP_DT[code])
        self.lib.mnb_swiglu(_ptr(gate16), _ptr(up16), gate16.size, code, int(decomposed), _ptr(out))
        return out

    # -- bits 2 / 4 / 8 ---------------------------------------------------------------------------
    def dequantize_nk_bits(self, b, scales, zp, n, k, bs, bits) -> np.ndarray:
        b, scales, zp = _c(b, np.uint8), _c(scales, np.float32), _c(zp, np.uint8)
        out = np.empty((n, k), np.float32)
        self.lib.mnb_dequantize_nk_bits(_ptr(b), _ptr(scales), _ptr(zp), n, k, bs, bits, _ptr(out))
        return out

    def matmul_f64_bits(self, a, b, scales, zp, n, k, bs, bits, bias=None) -> np.ndarray:
        a, b, scales, zp, bias = _c(a, np.float32), _c(b, np.uint8), _c(scales, np.float32), _c(zp, np.uint8), _c(bias, np.float32)
        m = a.size // k
        y = np.empty((m, n), np.float64)
        self.lib.mnb_matmul_f64_bits(_ptr(a), _ptr(b), _ptr(scales), _ptr(zp), _ptr(bias), m, n, k, bs, bits, _ptr(y))
        return y

    def dequantize_nk_gidx(self, b, scales, zp, g_idx, n, k, bs, bits=4) -> np.ndarray:
        """Dequantized [N, K] with scale / zero point of element k taken from group g_idx[k]; raises on an index outside 0..kb."""
        b, scales, zp, g_idx = _c(b, np.uint8), _c(scales, np.float32), _c(zp, np.uint8), _c(g_idx, np.int32)
        out = np.empty((n, k), np.float32)
        rc = self.lib.mnb_dequantize_nk_gidx(_ptr(b), _ptr(scales), _ptr(zp), _ptr(g_idx), n, k, bs, bits, _ptr(out))
        if rc != 0:
            raise ValueError("g_idx[%d] is outside 0..kb" % (-1 - rc))
        return out

    def rmsnorm16(self, a16: np.ndarray, gamma: np.ndarray, gamma_code: int, epsilon: float, code: int) -> np.ndarray:
        """The RMS-normalization prologue on 16-bit rows [rows, K] (K % 128 == 0); gamma 16-bit of the same type or f32."""
        a16, gamma = np.ascontiguousarray(a16), np.ascontiguousarray(gamma)
        rows, k = a16.shape
        assert k % 128 == 0 and gamma.size == k
        out = np.empty(a16.shape, _NP_DT[code])
        self.lib.mnb_rmsnorm16(_ptr(a16), _ptr(gamma), gamma_code, rows, k, float(epsilon), code, _ptr(out))
        return out

    # -- operator pieces -----------------------------------------------------------------------
    def dequantize_nk(self, b, scales, zp, n, k, bs) -> np.ndarray:
        b, scales, zp = _c(b, np.uint8), _c(scales, np.float32), _c(zp, np.uint8)
        out = np.empty((n, k), np.float32)
        self.lib.mnb_dequantize_nk(_ptr(b), _ptr(scales), _ptr(zp), n, k, bs, _ptr(out))
        return out

    def matmul_dequant_f32(self, a, w_nk, bias=None) -> np.ndarray:
        a, w_nk, bias = _c(a, np.float32), _c(w_nk, np.float32), _c(bias, np.float32)
        m, k = a.shape
        n = w_nk.shape[0]
        y = np.empty((m, n), np.float32)
        self.lib.mnb_matmul_dequant_f32(_ptr(a), _ptr(w_nk), _ptr(bias), m, n, k, _ptr(y))
        return y

    def matmul_f64(self, a, b, scales, zp, n, k, bs, bias=None) -> np.ndarray:
        a, b, scales, zp, bias = _c(a, np.float32), _c(b, np.uint8), _c(scales, np.float32), _c(zp, np.uint8), _c(bias, np.float32)
        m = a.size // k
        y = np.empty((m, n), np.float64)
        self.lib.mnb_matmul_f64(_ptr(a), _ptr(b), _ptr(scales), _ptr(zp), _ptr(bias), m, n, k, bs, _ptr(y))
        return y

    def matmul_blocksum_f32(self, a, b, scales, zp, n, k, bs, bias=None) -> np.ndarray:
        a, b, scales, zp, bias = _c(a, np.float32), _c(b, np.uint8), _c(scales, np.float32), _c(zp, np.uint8), _c(bias, np.float32)
        m = a.size // k
        y = np.empty((m, n), np.float32)
        self.lib.mnb_matmul_blocksum_f32(_ptr(a), _ptr(b), _ptr(scales), _ptr(zp), _ptr(bias), m, n, k, bs, _ptr(y))
        return y

    def quantize_a(self, a, k, bs, rounding):
        a = _c(a, np.float32)
        m = a.size // k
        kb = -(-k // bs)
        qa = np.empty((m, kb * bs), np.int8)
        qs = np.empty((m, kb), np.float32)
        self.lib.mnb_quantize_a(_ptr(a), m, k, bs, rounding, _ptr(qa), _ptr(qs))
        return qa, qs

    def block_acc_i32(self, qa, b, zp, n, k, bs) -> np.ndarray:
        qa, b, zp = _c(qa, np.int8), _c(b, np.uint8), _c(zp, np.uint8)
        kb = -(-k // bs)
        m = qa.size // (kb * bs)
        acc = np.empty((m, n, kb), np.int32)
        self.lib.mnb_block_acc_i32(_ptr(qa), _ptr(b), _ptr(zp), m, n, k, bs, _ptr(acc))
        return acc

    def matmul_acc4_f32(self, a, b, scales, zp, n, k, bs, rounding, bias=None) -> np.ndarray:
        a, b, scales, zp, bias = _c(a, np.float32), _c(b, np.uint8), _c(scales, np.float32), _c(zp, np.uint8), _c(bias, np.float32)
        m = a.size // k
        y = np.empty((m, n), np.float32)
        self.lib.mnb_matmul_acc4_f32(_ptr(a), _ptr(b), _ptr(scales), _ptr(zp), _ptr(bias), m, n, k, bs, rounding, _ptr(y))
        return y

    def matmul_nbits(self, a, a_code, b, scales, s_code, zp, bias, bias_code, y_code, m, n, k, bs, accuracy_level=0, rounding=ROUND_HALF_EVEN) -> np.ndarray:
        a, scales = np.ascontiguousarray(a), np.ascontiguousarray(scales)
        b, zp = _c(b, np.uint8), _c(zp, np.uint8)
        bias = None if bias is None else np.ascontiguousarray(bias)
        y = np.empty((m, n), _NP_DT[y_code])
        rc = self.lib.mnb_matmul_nbits(_ptr(a), a_code, _ptr(b), _ptr(scales), s_code, _ptr(zp), _ptr(bias), bias_code or F32, _ptr(y), y_code, m, n, k, bs, accuracy_level, rounding)
        if rc != 0:
            raise MemoryError("oracle allocation failed")
        return y


class Ref:
    """The reference's CPU path itself: vendored MLAS through crates/mlas-sys/vendor/shim.cpp:304-432."""

    COMP_FP32 = 0
    COMP_INT8 = 3

    def __init__(self):
        if not os.path.exists(REF_SO):
            raise FileNotFoundError(REF_SO)
        self.lib = C.CDLL(REF_SO)
        L = self.lib
        z, v, i = C.c_size_t, C.c_void_p, C.c_int
        L.mlas_qnbit_gemm_available.restype = i
        L.mlas_qnbit_gemm_available.argtypes = [z, z, i]
        L.mlas_qnbit_gemm_pack_b_size.restype = z
        L.mlas_qnbit_gemm_pack_b_size.argtypes = [z, z, z, z, i, i]
        L.mlas_qnbit_gemm_pack_b.restype = None
        L.mlas_qnbit_gemm_pack_b.argtypes = [z, z, z, z, i, v, v, v, i, v]
        L.mlas_qnbit_gemm_workspace_size.restype = z
        L.mlas_qnbit_gemm_workspace_size.argtypes = [z, z, z, z, z, i, i]
        L.mlas_qnbit_gemm.restype = None
        L.mlas_qnbit_gemm.argtypes = [z, z, z, z, z, i, v, z, v, v, i, v, v, v, z, v, i]
        L.mlas_ref_quantize_a_rows.restype = i
        L.mlas_ref_quantize_a_rows.argtypes = [z, z, z, v, z, v, v, v]
        L.mlas_ref_qnbit_dispatch_id.restype = i

    @staticmethod
    def available() -> bool:
        return os.path.exists(REF_SO)

    def dispatch_id(self) -> int:
        return self.lib.mlas_ref_qnbit_dispatch_id()

    @staticmethod
    def _aligned(nbytes: int, align: int = 64) -> np.ndarray:
        raw = np.zeros(nbytes + align, np.uint8)
        off = (-raw.ctypes.data) % align
        return raw[off:off + nbytes]

    def pack(self, b, scales, zp, n, k, bs, comp):
        """mlas-sys/src/lib.rs:2030-2060: pack once; 64-byte aligned buffer."""
        b, scales, zp = _c(b, np.uint8), _c(scales, np.float32), _c(zp, np.uint8)
        if not self.lib.mlas_qnbit_gemm_available(4, bs, comp):
            return None
        size = self.lib.mlas_qnbit_gemm_pack_b_size(n, k, 4, bs, int(zp is not None), comp)
        if size == 0:
            return None
        packed = self._aligned(size)
        self.lib.mlas_qnbit_gemm_pack_b(n, k, 4, bs, comp, _ptr(b), _ptr(packed), _ptr(scales), int(zp is not None), _ptr(zp))
        return {"packed": packed, "scales": scales, "zp": zp, "n": n, "k": k, "bs": bs, "comp": comp}

    def gemm(self, pk, a, bias=None, multithread=0, out=None, workspace=None) -> np.ndarray:
        """mlas-sys/src/lib.rs:2307-2352: f32 activations in, f32 out; workspace +64 bytes, aligned."""
        a, bias = _c(a, np.float32), _c(bias, np.float32)
        n, k, bs, comp = pk["n"], pk["k"], pk["bs"], pk["comp"]
        m = a.size // k
        y = out if out is not None else np.empty((m, n), np.float32)
        if workspace is None:
            ws = self.lib.mlas_qnbit_gemm_workspace_size(m, n, k, 4, bs, int(pk["zp"] is not None), comp)
            workspace = self._aligned(ws + 64) if ws else None
        self.lib.mlas_qnbit_gemm(m, n, k, 4, bs, comp, _ptr(a), k, _ptr(pk["packed"]), _ptr(pk["scales"]), int(pk["zp"] is not None), _ptr(pk["zp"]), _ptr(bias), _ptr(y), n, _ptr(workspace), multithread)
        return y

    def workspace(self, pk, m):
        ws = self.lib.mlas_qnbit_gemm_workspace_size(m, pk["n"], pk["k"], 4, pk["bs"], int(pk["zp"] is not None), pk["comp"])
        return self._aligned(ws + 64) if ws else None

    def matmul(self, a, b, scales, zp, n, k, bs, comp, bias=None) -> np.ndarray | None:
        pk = self.pack(b, scales, zp, n, k, bs, comp)
        return None if pk is None else self.gemm(pk, a, bias)

    def quantize_a(self, a, k, bs):
        a = _c(a, np.float32)
        m = a.size // k
        kb = -(-k // bs)
        qa = np.zeros((m, kb * bs), np.int8)
        qs = np.zeros((m, kb), np.float32)
        bsum = np.zeros((m, kb), np.float32)
        rc = self.lib.mlas_ref_quantize_a_rows(m, k, bs, _ptr(a), k, _ptr(qa), _ptr(qs), _ptr(bsum))
        if rc != 0:
            return None
        return qa, qs, bsum
