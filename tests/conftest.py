import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


def pytest_collection_modifyitems(config, items):
    """GPU tests are skipped, not failed, where no GPU exists."""
    try:
        import torch
        has_gpu = torch.cuda.is_available()
    except Exception:
        has_gpu = False
    if has_gpu:
        return
    skip = pytest.mark.skip(reason="no GPU in this environment")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(scope="session")
def oracle():
    from oracle import oracle as O
    O.lib()
    return O


@pytest.fixture(scope="session")
def golden():
    import json
    with open(os.path.join(ROOT, "tests", "golden", "hash_golden.json")) as f:
        return json.load(f)


@pytest.fixture
def force_general_hash_loader():
    """Switches the block-key kernel to the loader form it uses when a workgroup's requests span 4 GiB or more, through
    the library's test hook (an exported symbol that no header declares); restores the previous setting afterwards."""
    import ctypes
    from tair_kvcache_amd import _lib
    hook = _lib.lib().kvcm_test_hook_hash_force_global_loads
    hook.restype, hook.argtypes = ctypes.c_int32, [ctypes.c_int32]
    state = {"previous": None}

    def switch(on):
        previous = hook(1 if on else 0)
        if state["previous"] is None:
            state["previous"] = previous

    yield switch
    if state["previous"] is not None:
        hook(state["previous"])
