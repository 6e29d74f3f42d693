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


class _GeneralLoaderLib:
    """The shipped library with its three block-key entry points replaced by those of
    tests/libkvcm_hash_general_loader.so: the same source built with KVCM_TEST_FORCE_GENERAL_LOADER=1, in which every
    launch takes the loader form of a workgroup whose requests span 4 GiB or more."""
    _SWAPPED = ("kvcm_hip_hash_tokens", "kvcm_hip_hash_tokens_i32", "kvcm_hip_prefix_chain")

    def __init__(self):
        import ctypes
        from tair_kvcache_amd import _lib, build
        if not os.path.exists(build.TEST_HOOK_LIB_PATH):
            raise _lib.KvcmLibraryError(f"{build.TEST_HOOK_LIB_PATH} is not built; run `python -m tair_kvcache_amd.build`")
        self._shipped = _lib.lib()
        general = ctypes.CDLL(build.TEST_HOOK_LIB_PATH)
        for name in self._SWAPPED:
            fn = getattr(general, name)
            fn.restype, fn.argtypes = _lib.SIGNATURES[name]
            setattr(self, name, fn)

    def __getattr__(self, name):  # everything else is the shipped library's
        return getattr(self._shipped, name)


@pytest.fixture
def force_general_hash_loader(monkeypatch):
    """switch(True) makes tair_kvcache_amd.hashing launch the block-key kernels of the general-loader build for the
    rest of the test; switch(False) goes back to the shipped library."""
    from tair_kvcache_amd import _torch_util, hashing
    state = {}

    def switch(on):
        if on:
            if "lib" not in state:
                state["lib"] = _GeneralLoaderLib()
            monkeypatch.setattr(hashing, "lib", lambda: state["lib"])
        else:
            monkeypatch.setattr(hashing, "lib", _torch_util.lib)

    yield switch
