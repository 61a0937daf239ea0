import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def port():
    import oracle
    return oracle.Port()


@pytest.fixture(scope="session")
def ref():
    """The reference's own compiled CPU path (oracle/_ref). Built here from /root/reference; prebuilt on the GPU box."""
    import oracle
    if not oracle.Ref.available():
        if os.path.isdir("/root/reference/crates/mlas-sys/vendor"):
            oracle.build(ref=True)
        else:
            pytest.skip("oracle/_ref/libmlas_ref.so is not built and /root/reference is absent")
    return oracle.Ref()


@pytest.fixture(scope="session")
def ep():
    """One provider for the whole GPU session. No fallback: a missing library or GPU is a hard failure."""
    from onnx_genai_amd.ep import RocmExecutionProvider
    provider = RocmExecutionProvider(0)
    info = provider.device_info()
    assert info["arch"].startswith("gfx950"), info
    yield provider
    provider.shutdown()


@pytest.fixture(scope="session")
def ep_unpacked():
    """A provider that never repacks constant weights: decode calls stream the caller's tensors as they are."""
    from onnx_genai_amd.ep import RocmExecutionProvider
    provider = RocmExecutionProvider(0, {"prepack": "0"})
    yield provider
    provider.shutdown()


@pytest.fixture(scope="session")
def ep_tiled():
    """A provider whose tall 16-bit calls stay on the hand-written tiled kernel (no dense copy, no library GEMM) - the
    default, spelled out."""
    from onnx_genai_amd.ep import RocmExecutionProvider
    provider = RocmExecutionProvider(0, {"dense_gemm_min_rows": "0"})
    yield provider
    provider.shutdown()


@pytest.fixture(scope="session")
def ep_dense():
    """A provider with the opt-in dense route on: from 1024 rows (32 for bit widths and act-order weights that have no tiled
    kernel) a 16-bit call expands the weights and runs the library GEMM."""
    from onnx_genai_amd.ep import RocmExecutionProvider
    provider = RocmExecutionProvider(0, {"dense_gemm_min_rows": "1024"})
    yield provider
    provider.shutdown()
