"""Builds libnxrt_ep_rocm.so in-tree: every HIP kernel for gfx950 plus the host side of the C ABI."""
from __future__ import annotations

import os
import re
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
HOST_SOURCES = ["ep/provider.cpp", "ep/matmul_nbits.cpp", "ep/nxrt_plugin.cpp", "ep/nxmem_plugin.cpp", "ep/ort_plugin.cpp"]

# packed-fp32 VALU forms are kept off for all device code
DEVICE_FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]
HOST_FLAGS = ["-O2", "-std=c++17", "-fPIC", "-Wall", "-Wextra", "-Wno-unused-parameter"]


REMARKS = "-Rpass-analysis=kernel-resource-usage"


def _resource_usage(stderr):
    """Per kernel, the registers and scratch bytes per lane that the compiler's resource remarks report."""
    usage, name = {}, None
    for line in stderr.splitlines():
        if REMARKS not in line or "remark:" not in line:
            continue
        text = line.split("remark:", 1)[1].replace("[" + REMARKS + "]", "").strip()
        key, _, value = text.partition(":")
        if key == "Function Name":
            name = value.strip()
            usage[name] = {}
        elif name is not None and key in ("VGPRs", "AGPRs", "ScratchSize [bytes/lane]", "VGPRs Spill", "Occupancy [waves/SIMD]"):
            usage[name][key] = int(value)
    return usage


def _diagnostics(stderr):
    """Compiler output without the resource remarks (some are followed by a source line and a caret line) and the feature note."""
    out, after_remark = [], 0
    for line in stderr.splitlines():
        if REMARKS in line:
            after_remark = 1
            continue
        if after_remark == 1 and re.match(r"\s*\d+ \|", line):
            after_remark = 2
            continue
        if after_remark == 2 and re.match(r"\s*\|\s*\^", line):
            after_remark = 0
            continue
        after_remark = 0
        if "packed-fp32-ops" not in line:
            out.append(line)
    return "\n".join(out)


def _run(cmd):
    r = subprocess.run(cmd, capture_output=True, text=True)
    err = _diagnostics(r.stderr)
    if r.returncode != 0:
        raise RuntimeError("command failed: " + " ".join(cmd) + "\n" + err)
    if err.strip():
        sys.stderr.write(err + "\n")
    return _resource_usage(r.stderr)


def build(force: bool = True) -> str:
    os.makedirs(OBJ, exist_ok=True)
    os.makedirs(os.path.dirname(LIB), exist_ok=True)
    jobs, objs = [], []
    for src in HIP_SOURCES:
        obj = os.path.join(OBJ, src.replace("/", "_") + ".o")
        objs.append(obj)
        jobs.append([HIPCC, *DEVICE_FLAGS, REMARKS, "-c", os.path.join(CSRC, src), "-o", obj])
    for src in HOST_SOURCES:
        obj = os.path.join(OBJ, src.replace("/", "_") + ".o")
        objs.append(obj)
        jobs.append(["g++", *HOST_FLAGS, "-c", os.path.join(CSRC, src), "-o", obj])
    with ThreadPoolExecutor(max_workers=8) as pool:
        usage = {}
        for part in pool.map(_run, jobs):
            usage.update(part)
    # No kernel here is meant to touch scratch memory: an accumulator array that the compiler could not keep in
    # registers (a loop over it that did not unroll) shows up here, long before it shows up as a slow kernel.
    with open(os.path.join(OBJ, "kernel_resources.txt"), "w") as f:
        for name in sorted(usage):
            f.write(name + " " + " ".join(f"{k}={v}" for k, v in usage[name].items()) + "\n")
    spilled = {n: u for n, u in usage.items() if u.get("ScratchSize [bytes/lane]", 0) or u.get("VGPRs Spill", 0)}
    if spilled:
        raise RuntimeError("kernels that use scratch memory:\n" + "\n".join(f"  {n}: {u}" for n, u in sorted(spilled.items())))
    _run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB, *objs, "-ldl", "-Wl,-z,defs", "-Wl,--exclude-libs,ALL"])
    return LIB


if __name__ == "__main__":
    print(build())
