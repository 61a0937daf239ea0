"""Writes tests/golden/dispatch_table.json: what the launchers plan for the benchmark configurations' shapes on 256 CUs.

No GPU work: the planning entry points of the built library only do arithmetic on shapes. Run after a deliberate change of a
launcher's rules (`python tests/golden/make_dispatch_table.py`) and review the diff; tests/test_dispatch_cpu.py holds the
library against the committed file.
"""
import ctypes as C
import json
import os
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from onnx_genai_amd import build  # noqa: E402

F16, BF16, F32 = 10, 16, 1
CUS = 256


class FfiArgs(C.Structure):
    """RocmMatMulNBitsArgs of csrc/hip_ffi.h."""
    _fields_ = [("a", C.c_void_p), ("b", C.c_void_p), ("scales", C.c_void_p), ("zp", C.c_void_p), ("bias", C.c_void_p), ("y", C.c_void_p),
                ("a_dtype", C.c_int), ("scale_dtype", C.c_int), ("bias_dtype", C.c_int), ("y_dtype", C.c_int),
                ("m", C.c_int64), ("n", C.c_int64), ("k", C.c_int64), ("block_size", C.c_int),
                ("g_idx", C.c_void_p), ("acc_probe", C.c_void_p), ("gamma", C.c_void_p), ("gamma_dtype", C.c_int), ("norm_epsilon", C.c_float)]


class DecodePlan(C.Structure):
    """RocmDecodePackedPlan of csrc/hip_ffi.h."""
    _fields_ = [("shared_activations", C.c_int), ("rows_build", C.c_int), ("waves", C.c_int), ("groups_per_wave", C.c_int),
                ("register_sets", C.c_int), ("activation_sums", C.c_int), ("workgroups", C.c_int64)]


# (configuration, name, dtype, block, zero points, K, N)
DECODE = [
    ("configs[1]", "q/o", F16, 32, True, 896, 896), ("configs[1]", "k/v", F16, 32, True, 896, 128), ("configs[1]", "gate/up", F16, 32, True, 896, 4864),
    ("configs[1]", "down", F16, 32, True, 4864, 896), ("configs[1]", "lm_head", F16, 32, True, 896, 151936),
    ("configs[2]", "qkv", BF16, 128, True, 3584, 4608), ("configs[2]", "o", BF16, 128, True, 3584, 3584), ("configs[2]", "gate_up", BF16, 128, True, 3584, 37888),
    ("configs[2]", "down", BF16, 128, True, 18944, 3584), ("configs[2]", "lm_head", BF16, 128, True, 3584, 152064),
]
PREFILL = [("configs[3]", F16, 32, 4096, 14336), ("configs[3]", F16, 32, 14336, 4096)]
ACC4 = [("configs[4]", F16, 64, 8192, 28672), ("configs[4]", F16, 64, 28672, 8192), ("configs[4]", F16, 64, 8192, 10240)]


def load():
    lib = C.CDLL(build.LIB)
    lib.rocm_decode_packed_plan.restype = C.c_int
    lib.rocm_decode_packed_plan.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_void_p]
    lib.rocm_acc4_packed_plan.restype = C.c_int
    lib.rocm_acc4_packed_plan.argtypes = [C.c_void_p, C.c_int, C.c_int, C.POINTER(C.c_int), C.POINTER(C.c_int), C.POINTER(C.c_int)]
    lib.rocm_prefill_mfma_plan.restype = C.c_int
    lib.rocm_prefill_mfma_plan.argtypes = [C.c_void_p, C.c_int, C.c_uint64, C.POINTER(C.c_int), C.POINTER(C.c_int), C.POINTER(C.c_int)]
    return lib


def ffi_args(dt, bs, zero_points, m, n, k):
    a = FfiArgs()
    a.a, a.b, a.scales, a.y = 0x10000, 0x20000, 0x30000, 0x40000          # never dereferenced: alignment only
    a.zp = 0x50000 if zero_points else None
    a.a_dtype = a.scale_dtype = a.y_dtype = dt
    a.m, a.n, a.k, a.block_size = m, n, k, bs
    return a


def table(lib):
    rows = []
    for cfg, name, dt, bs, zp, k, n in DECODE:
        for m in (1, 4, 8, 16):
            plan = DecodePlan()
            rc = lib.rocm_decode_packed_plan(C.byref(ffi_args(dt, bs, zp, m, n, k)), 0, 0, CUS, C.byref(plan))
            row = {"config": cfg, "shape": name, "k": k, "n": n, "m": m, "route": "decode_packed" if rc == 0 else "other"}
            if rc == 0:
                row.update({f: getattr(plan, f) for f, _ in DecodePlan._fields_})
            rows.append(row)
    for cfg, dt, bs, k, n in PREFILL:
        for m in (512, 2048, 8192):
            tr, tc, sl = C.c_int(), C.c_int(), C.c_int()
            rc = lib.rocm_prefill_mfma_plan(C.byref(ffi_args(dt, bs, False, m, n, k)), 0, C.c_uint64(1 << 40), C.byref(tr), C.byref(tc), C.byref(sl))
            rows.append({"config": cfg, "shape": "mlp", "k": k, "n": n, "m": m, "route": "prefill_mfma" if rc == 0 else "other",
                         "tile_rows": tr.value, "tile_cols": tc.value, "slices": sl.value})
    for cfg, dt, bs, k, n in ACC4:
        w, g, sets = C.c_int(), C.c_int(), C.c_int()
        rc = lib.rocm_acc4_packed_plan(C.byref(ffi_args(dt, bs, True, 1, n, k)), 0, CUS, C.byref(w), C.byref(g), C.byref(sets))
        rows.append({"config": cfg, "shape": "acc4", "k": k, "n": n, "m": 1, "route": "acc4_packed" if rc == 0 else "other",
                     "waves": w.value, "groups_per_wave": g.value, "register_sets": sets.value})
    return rows


if __name__ == "__main__":
    out = os.path.join(HERE, "dispatch_table.json")
    with open(out, "w") as f:
        f.write("[\n" + ",\n".join(" " + json.dumps(r) for r in table(load())) + "\n]\n")
    print("wrote", out)
