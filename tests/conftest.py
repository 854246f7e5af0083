import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def _has_gpu() -> bool:
    try:
        import torch
        return torch.cuda.is_available()
    except Exception:
        return False


def pytest_collection_modifyitems(config, items):
    if _has_gpu():
        return
    skip = pytest.mark.skip(reason="no GPU in this environment")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(scope="session", autouse=True)
def _built_libraries():
    """The tests load what is built; only when nothing is do they build it (in-tree, with
    hipcc cross-compiling for gfx950: no GPU is needed for that)."""
    import importlib
    g2 = importlib.import_module("cuda-gpt2-inference_amd")
    if not os.path.exists(g2.LIB_PATH):
        import __graft_entry__
        __graft_entry__.build()
    yield
