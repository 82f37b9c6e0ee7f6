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
def held_workspace_off(request):
    """The plain entry points take a workspace from the library's own pool where that pays
    (adr_set_held_workspace_limit).  Most GPU tests here name the kernel a product runs on
    (adr_matmul_f16_plan) and then call the plain entry point to test THAT kernel, so the pool is
    off unless a test switches it on (tests/test_gpu_held_workspace.py, the randomised tests and the
    full-size tests parametrised over it do).  Tests without the gpu marker are left alone (they
    must not need the built library just to be set up)."""
    if "gpu" not in request.keywords:
        yield
        return
    from adrastea_amd import _ffi
    lib = _ffi.lib()
    before = lib.adr_held_workspace_limit()
    lib.adr_set_held_workspace_limit(0)
    yield
    lib.adr_set_held_workspace_limit(before)


WORKSPACE_MODES = ["pool_off", "shipped_default", "u8_dequantise_first"]


@pytest.fixture
def workspace_mode(request):
    """How the plain entry points are configured for a test (indirect parameter):
    "pool_off": adr_set_held_workspace_limit(0), what most tests here run with;
    "shipped_default": the library as a drop-in caller finds it (pool on at its default limit,
    u8 products on the fused kernels) -- what bench.py measures;
    "u8_dequantise_first": the pool on and adr_set_u8_dequantise_first(1)."""
    from adrastea_amd import _ffi
    lib = _ffi.lib()
    mode = request.param
    assert mode in WORKSPACE_MODES
    lib.adr_set_held_workspace_limit(0 if mode == "pool_off" else _ffi.HELD_WORKSPACE_DEFAULT_BYTES)
    lib.adr_set_u8_dequantise_first(1 if mode == "u8_dequantise_first" else 0)
    yield mode
    lib.adr_set_held_workspace_limit(0)
    lib.adr_set_u8_dequantise_first(0)
