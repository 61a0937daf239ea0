"""Writes tests/golden/mlas_vectors.npz: inputs and outputs of the reference's own compiled CPU path
(oracle/_ref/libmlas_ref.so, built by oracle/Makefile from crates/mlas-sys/vendor) on the grid of the reference's
check_sqnbit tests (crates/mlas-sys/src/lib.rs:3268-3285: m in {1,5}, n=96, k=256, block 32/64/128, symmetric and
asymmetric, plus m=4 n=128 k=512 block 32 with bias), and its activation codes on a tie-heavy fixture.

Run from the repository root in the build container:  python tests/golden/make_mlas_vectors.py
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

import oracle  # noqa: E402
from tests import helpers  # noqa: E402


def main():
    ref = oracle.Ref()
    out = {"dispatch_id": np.int32(ref.dispatch_id())}
    cases = [(m, 96, 256, bs, asym, False) for m in (1, 5) for bs in (32, 64, 128) for asym in (False, True)]
    cases.append((4, 128, 512, 32, True, True))
    names = []
    for m, n, k, bs, asym, with_bias in cases:
        w, a, bias = helpers.sqnbit_fixture(m, n, k)
        b, s, zp, _ = helpers.quantize_blockwise(w, bs, asym)
        bias = bias if with_bias else None
        tag = f"m{m}_n{n}_k{k}_b{bs}_{'asym' if asym else 'sym'}{'_bias' if with_bias else ''}"
        names.append(tag)
        out[tag + "_b"] = b
        out[tag + "_s"] = s
        if zp is not None:
            out[tag + "_zp"] = zp
        out[tag + "_a"] = a
        if bias is not None:
            out[tag + "_bias"] = bias
        out[tag + "_y_fp32"] = ref.matmul(a, b, s, zp, n, k, bs, ref.COMP_FP32, bias=bias)
        out[tag + "_y_int8"] = ref.matmul(a, b, s, zp, n, k, bs, ref.COMP_INT8, bias=bias)
    out["cases"] = np.array(names)
    # activation quantizer: N(0,1) rounded to f16 plus exact ties, a zero block and +-max
    rng = np.random.default_rng(2024)
    for bs in (32, 64, 128):
        k = 4 * bs
        a = rng.standard_normal((3, k)).astype(np.float16).astype(np.float32)
        a[0, :bs] = 0.0
        a[0, bs:2 * bs] = (rng.integers(-253, 254, size=bs) * 0.5).astype(np.float32)
        a[0, bs], a[0, bs + 1] = 127.0, -127.0
        qa, qs, bsum = ref.quantize_a(a, k, bs)
        out[f"quant_b{bs}_a"] = a
        out[f"quant_b{bs}_codes"] = qa
        out[f"quant_b{bs}_scales"] = qs
        out[f"quant_b{bs}_blksum"] = bsum
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "mlas_vectors.npz")
    np.savez_compressed(path, **out)
    print(path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
