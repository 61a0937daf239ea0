"""Which build, wave count and register sets the launchers pick for the benchmark configurations' shapes, held against the
committed table tests/golden/dispatch_table.json (no GPU work: the planning entry points only do arithmetic on shapes).

The launch rules hold dozens of measured thresholds; correctness of whatever they pick is covered by the GPU tests, but
nothing else would notice a rule tuned for one shape quietly moving a benchmark shape to another build.
"""
import ctypes as C
import json
import os

import pytest

from onnx_genai_amd import build
from tests.golden import make_dispatch_table as T

HERE = os.path.dirname(os.path.abspath(__file__))


@pytest.fixture(scope="module")
def lib():
    if not os.path.exists(build.LIB):
        pytest.skip("library not built")
    return T.load()


def test_benchmark_shapes_keep_their_launch_plans(lib):
    with open(os.path.join(HERE, "golden", "dispatch_table.json")) as f:
        want = json.load(f)
    got = T.table(lib)
    assert len(got) == len(want) == 4 * 10 + 6 + 3
    for g, w in zip(got, want):
        assert g == w, f"launch plan moved:\n  now  {g}\n  was  {w}\n(if intended: python tests/golden/make_dispatch_table.py, and review the diff)"


def test_headline_decode_step_plans(lib):
    """The five calls of the Qwen2.5-7B decode step at one row, spelled out: one tile group of 512 k per wave (three on the
    long K), one register set, the activation-sums form, sixteen columns per workgroup."""
    rows = {(r["shape"], r["m"]): r for r in T.table(lib) if r["config"] == "configs[2]"}
    for shape, waves, groups, workgroups in [("qkv", 7, 1, 288), ("o", 7, 1, 224), ("gate_up", 7, 1, 2368), ("down", 13, 3, 224), ("lm_head", 7, 1, 9504)]:
        r = rows[(shape, 1)]
        assert (r["shared_activations"], r["rows_build"], r["waves"], r["groups_per_wave"], r["register_sets"], r["activation_sums"], r["workgroups"]) == \
            (0, 1, waves, groups, 1, 1, workgroups), r
    # 16 rows: the wide shapes share one LDS copy of the activations; gate/up spreads its 2368 column groups over one workgroup per CU
    r = rows[("gate_up", 16)]
    assert r["shared_activations"] == 1 and r["waves"] == 10 and r["workgroups"] == 237
    assert rows[("lm_head", 16)]["shared_activations"] == 1 and rows[("down", 16)]["shared_activations"] == 0


def test_plans_follow_the_compute_unit_count(lib):
    """The CU count is an input of the plan, not a literal: on a chip of 304 CUs the gate/up grid at 16 rows is no longer
    'between one and one and a half workgroups per CU' and keeps eight waves a workgroup."""
    a = T.ffi_args(T.BF16, 128, True, 16, 37888, 3584)
    p256, p304 = T.DecodePlan(), T.DecodePlan()
    assert lib.rocm_decode_packed_plan(C.byref(a), 0, 0, 256, C.byref(p256)) == 0
    assert lib.rocm_decode_packed_plan(C.byref(a), 0, 0, 304, C.byref(p304)) == 0
    assert (p256.waves, p256.workgroups) == (10, 237)
    assert (p304.waves, p304.workgroups) == (8, 296)
    # a mid-size split-K grid fits more waves on more CUs
    b = T.ffi_args(T.BF16, 128, True, 16, 13824, 5120)
    q128, q256 = T.DecodePlan(), T.DecodePlan()
    assert lib.rocm_decode_packed_plan(C.byref(b), 0, 0, 128, C.byref(q128)) == 0
    assert lib.rocm_decode_packed_plan(C.byref(b), 0, 0, 256, C.byref(q256)) == 0
    assert q128.waves <= q256.waves and q128.waves * q128.groups_per_wave >= 10 and q256.waves * q256.groups_per_wave >= 10
    assert lib.rocm_decode_packed_plan(C.byref(a), 0, 0, 0, C.byref(p256)) == -1
