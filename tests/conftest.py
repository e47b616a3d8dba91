import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


def _has_gpu():
    try:
        import torch
        return torch.cuda.is_available()
    except Exception:
        return False


def pytest_collection_modifyitems(config, items):
    if _has_gpu():
        return
    skip = pytest.mark.skip(reason="no GPU in this container")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(scope="session")
def lib():
    from daceml_amd import _lib
    return _lib.load()


@pytest.fixture(autouse=True)
def _reset_diagnostic_switches():
    """A test that pins a tile configuration and fails midway must not leave the pin set for the tests after it."""
    yield
    from daceml_amd import _lib
    lib = _lib._lib
    if lib is not None:
        lib.dmlhip_debug_force_gemm_config(-1)
        lib.dmlhip_debug_gemm_direct_lds(1)
        lib.dmlhip_debug_force_fused_strip(0)
        lib.dmlhip_debug_fused_rolling(0, 8)
        lib.dmlhip_debug_gemm_trace(None)
        lib.dmlhip_debug_attention_trace(None)
