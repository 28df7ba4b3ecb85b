import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


def _gpu_present() -> bool:
    try:
        import torch
        return torch.cuda.is_available()
    except Exception:
        return False


def pytest_collection_modifyitems(config, items):
    if _gpu_present():
        return
    skip = pytest.mark.skip(reason="no GPU in this environment")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(scope="session")
def oracle():
    """The C oracle, built on demand (gcc)."""
    from oracle import moe_ref
    moe_ref.lib()
    return moe_ref


@pytest.fixture(scope="session", autouse=True)
def built_library():
    """The tests load the library that is built in-tree; only when there is none do they build it
    (hipcc cross-compiles gfx950 without a GPU)."""
    from aristos_amd import _capi, build
    if not os.path.exists(_capi.LIB_PATH):
        build.build_library()
    return _capi.LIB_PATH
