import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: test needs a real MI355X (run with -m gpu)")


def pytest_collection_modifyitems(config, items):
    # GPU tests are skipped (not failed) where no device exists, so a plain `pytest tests/`
    # on a CPU-only machine stays green.
    try:
        import torch
        have_gpu = torch.cuda.is_available()
    except Exception:
        have_gpu = False
    if have_gpu:
        return
    skip = pytest.mark.skip(reason="no GPU in this environment")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(autouse=True)
def held_workspace_off():
    """The plain entry points take a workspace from the library's own cache where that pays
    (adr_set_held_workspace_limit).  Most tests here name the kernel a product runs on
    (adr_matmul_f16_plan) and then call the plain entry point to test THAT kernel, so the cache is
    off unless a test switches it on (tests/test_gpu_held_workspace.py and the randomised tests do)."""
    from adrastea_amd import _ffi
    lib = _ffi.lib()
    before = lib.adr_held_workspace_limit()
    lib.adr_set_held_workspace_limit(0)
    yield
    lib.adr_set_held_workspace_limit(before)
