"""Builds libnxrt_ep_rocm.so in-tree: every HIP kernel for gfx950 plus the host side of the C ABI."""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(HERE, "build")
LIB = os.path.join(HERE, "lib", "libnxrt_ep_rocm.so")
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")

HIP_SOURCES = [
    "hip_ffi.hip",
    "kernels/dequant.hip",
    "kernels/gemv_generic.hip",
    "kernels/gemv_nbits.hip",
    "kernels/gemv_f32.hip",
    "kernels/decode_mfma.hip",
    "kernels/decode_packed.hip",
    "kernels/prefill_mfma.hip",
    "kernels/dense_gemm.hip",
    "kernels/swiglu.hip",
    "kernels/acc4.hip",
    "kernels/acc4_mfma.hip",
]
HOST_SOURCES = ["ep/provider.cpp", "ep/matmul_nbits.cpp", "ep/nxrt_plugin.cpp", "ep/nxmem_plugin.cpp"]

# packed-fp32 VALU forms are kept off for all device code
DEVICE_FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]
HOST_FLAGS = ["-O2", "-std=c++17", "-fPIC", "-Wall", "-Wextra", "-Wno-unused-parameter"]


def _run(cmd):
    r = subprocess.run(cmd, capture_output=True, text=True)
    err = "\n".join(l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l)
    if r.returncode != 0:
        raise RuntimeError("command failed: " + " ".join(cmd) + "\n" + err)
    if err.strip():
        sys.stderr.write(err + "\n")


def build(force: bool = True) -> str:
    os.makedirs(OBJ, exist_ok=True)
    os.makedirs(os.path.dirname(LIB), exist_ok=True)
    jobs, objs = [], []
    for src in HIP_SOURCES:
        obj = os.path.join(OBJ, src.replace("/", "_") + ".o")
        objs.append(obj)
        jobs.append([HIPCC, *DEVICE_FLAGS, "-c", os.path.join(CSRC, src), "-o", obj])
    for src in HOST_SOURCES:
        obj = os.path.join(OBJ, src.replace("/", "_") + ".o")
        objs.append(obj)
        jobs.append(["g++", *HOST_FLAGS, "-c", os.path.join(CSRC, src), "-o", obj])
    with ThreadPoolExecutor(max_workers=8) as pool:
        list(pool.map(_run, jobs))
    _run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB, *objs, "-L/opt/rocm/lib", "-lhipblaslt", "-Wl,-z,defs", "-Wl,--exclude-libs,ALL"])
    return LIB


if __name__ == "__main__":
    print(build())
