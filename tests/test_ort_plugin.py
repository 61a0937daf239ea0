"""The ORT plugin execution-provider export (CreateEpFactories / ReleaseEpFactory) against a mock of ONNX Runtime's side.

tests/harness/ort_mock_host.cpp plays the host: it loads the library by path, resolves the two symbols by name, serves the
OrtApi / OrtEpApi members the plugin calls, and checks every answer of the lifecycle a session walks through - the
reference's own coverage of this path (crates/onnx-runtime-ep-plugin/src/factory.rs tests, lib.rs:190-236) restated for a
C host. No ONNX Runtime exists in this image: what these tests pin is the plugin's behaviour behind the tables, not the
tables' offsets in a real onnxruntime build.
"""
import os
import subprocess

import pytest

from onnx_genai_amd import ep as E

HERE = os.path.dirname(os.path.abspath(__file__))
HOST = os.path.join(HERE, "harness", "ort_mock_host")


def run_host(*args):
    assert os.path.exists(HOST), "tests/harness/ort_mock_host is built by __graft_entry__.build()"
    return subprocess.run([HOST, E.LIB_PATH, *args], capture_output=True, text=True, timeout=100)


def test_lifecycle_without_a_gpu():
    """Entry-point argument checks, factory identity, device selection (AMD GPUs only), EP creation, GetCapability over a graph
    of supported and unsupported MatMulNBits nodes (per-slot dtype rule, attribute checks), Compile, allocator and data
    transfer creation, and release in the host's order and in a wrong one - none of which may touch a GPU."""
    run = run_host()
    assert run.returncode == 0, run.stdout + run.stderr
    assert "ort plugin lifecycle ok" in run.stdout


@pytest.mark.gpu
def test_compute_through_the_ort_tables():
    """The same, plus one compiled node run on the GPU: tensors from the plugin's allocator, filled through its data transfer,
    Compute through a mock kernel context, result within 1e-5 (rel-L2, f32) of a double-precision product computed by the host."""
    run = run_host("--gpu")
    assert run.returncode == 0, run.stdout + run.stderr
    assert "ort plugin lifecycle ok (with compute)" in run.stdout
