"""The C-ABI library builds, loads and exports every symbol include/kvcm_hip.h declares (no GPU, no compute)."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "kvcm_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(kvcm_(?:hip_)?[a-z0-9_]+)\s*\(", text)))


def test_header_declares_the_expected_entry_points():
    names = declared_symbols()
    for must in ("kvcm_hip_hash_tokens", "kvcm_hip_hash_tokens_i32", "kvcm_hip_prefix_chain",
                 "kvcm_hip_sha256_first8_be", "kvcm_hip_batch_gather", "kvcm_hip_batch_scatter",
                 "kvcm_hip_batch_gather_host_idx", "kvcm_hip_batch_scatter_host_idx",
                 "kvcm_hip_paged_gather", "kvcm_hip_paged_scatter", "kvcm_hip_gather_ex", "kvcm_hip_scatter_ex",
                 "kvcm_hip_generate_blocks_idx", "kvcm_hip_iov_crc32", "kvcm_blocks_hash_from_crcs",
                 "kvcm_hip_first_occurrence", "kvcm_hip_first_occurrence_workspace_bytes",
                 "kvcm_hip_mask_to_indices", "kvcm_hip_mask_to_indices_workspace_bytes",
                 "kvcm_file_store_create", "kvcm_file_store_destroy", "kvcm_file_store_put", "kvcm_file_store_get",
                 "kvcm_copy_iovs"):
        assert must in names


def test_library_exports_every_declared_symbol():
    from tair_kvcache_amd import _lib
    L = _lib.lib()
    for name in declared_symbols():
        assert hasattr(L, name), name
        assert name in _lib.SIGNATURES, f"{name} has no ctypes signature"
    assert L.kvcm_hip_version() >= 100


def test_every_prototype_cites_the_reference():
    text = open(os.path.join(ROOT, "include", "kvcm_hip.h")).read()
    for anchor in ("cache_manager.cc:76-87", "hash_util.h:8-24", "trace_util.cc:47-56", "connector.py:397-415",
                   "batch_gather_scatter_helper.py:33-136", "batch_gather_scatter_helper.py:139-248",
                   "v1_connector.py:308-320", "sdk_buffer_check_util.cu:21-44", "sdk_buffer_check_util.cc:56-60",
                   "v1_connector.py:835-850", "cache_manager.cc:589-635", "local_file_sdk.cc:68-85",
                   "local_file_sdk.cc:161-260", "hf3fs_usrbio_client.cc:478-505", "common.h:102-110"):
        assert anchor in text, anchor


def test_argument_validation_needs_no_device():
    from tair_kvcache_amd import _lib
    L = _lib.lib()
    one = ctypes.c_int64(0)
    p = ctypes.addressof(one)
    # rejected before any HIP call
    assert L.kvcm_hip_batch_gather(p, 0, p, 64, p, None, 1, 16, 64, 0, None) == _lib.ERR_INVALID_ARG  # P = 0
    assert L.kvcm_hip_batch_gather(p, 2, p, 64, p, None, -1, 16, 64, 0, None) == _lib.ERR_INVALID_ARG  # B < 0
    assert L.kvcm_hip_batch_gather(p, 2, p, 64, p, None, 1, 16, 64, 0, None) == _lib.ERR_INVALID_ARG  # slot too small
    assert L.kvcm_hip_batch_gather(None, 2, p, 2 * 16 * 64, p, None, 1, 16, 64, 0, None) == _lib.ERR_INVALID_ARG
    assert L.kvcm_hip_paged_gather(p, 2, p, 2 * 16 * 64, p, 3, None, 1, 16, 64, 0, None) == _lib.ERR_INVALID_ARG
    # a staging block of 2 GiB or more cannot be numbered with 31-bit chunk indices
    assert L.kvcm_hip_batch_scatter(p, 2, p, 1 << 34, p, None, 1, 1 << 20, 1 << 12, 0, None) == _lib.ERR_TOO_LARGE
    # nothing to do is not an error
    assert L.kvcm_hip_batch_gather(p, 2, p, 2 * 16 * 64, p, None, 0, 16, 64, 0, None) == _lib.OK
    assert L.kvcm_hip_hash_tokens(p, p, 0, 16, 0, p, None, None) == _lib.OK
    assert L.kvcm_hip_hash_tokens(p, p, 1, 0, 0, p, None, None) == _lib.ERR_INVALID_ARG
    assert L.kvcm_hip_hash_tokens(None, p, 1, 16, 0, p, None, None) == _lib.ERR_INVALID_ARG
    assert L.kvcm_hip_sha256_first8_be(None, None, 0, None, None) == _lib.OK
    assert L.kvcm_hip_iov_crc32(None, 1, None, 4, None) == _lib.ERR_INVALID_ARG
    assert L.kvcm_hip_generate_blocks_idx(p, 1, p, 1, 0, 16, p, None, None) == _lib.ERR_INVALID_ARG
    assert L.kvcm_hip_first_occurrence_workspace_bytes(0) == 4096 and L.kvcm_hip_first_occurrence_workspace_bytes(513) == 2048 * 4
    assert L.kvcm_hip_first_occurrence_workspace_bytes((1 << 30) + 1) == _lib.ERR_TOO_LARGE
    assert L.kvcm_hip_first_occurrence(None, 0, None, 0, None, None, None) == _lib.OK
    assert L.kvcm_hip_first_occurrence(None, 5, p, 1 << 20, p, None, None) == _lib.ERR_INVALID_ARG
    assert L.kvcm_hip_first_occurrence(p, 5, p, 8, p, None, None) == _lib.ERR_INVALID_ARG  # workspace too small
    assert L.kvcm_hip_mask_to_indices_workspace_bytes(1025) == 3 * 4
    assert L.kvcm_hip_mask_to_indices(p, None, 5, p, 1 << 20, p, None, None) == _lib.ERR_INVALID_ARG  # no count
    assert L.kvcm_hip_mask_to_indices(p, None, (1 << 30) + 1, p, 1 << 20, p, p, None) == _lib.ERR_TOO_LARGE
    # host index lists: the walk over the lists refuses a wild index before any HIP call
    T = 16
    tok = (ctypes.c_int32 * (2 * T))(*range(2 * T))
    sl = (ctypes.c_int32 * 2)(0, 1)
    host_idx = L.kvcm_hip_batch_gather_host_idx
    assert host_idx(p, 2, p, 2 * T * 64, 2, tok, sl, 2, T, 64, 2 * T - 1, 0, None) == _lib.ERR_OUT_OF_RANGE  # token slot
    assert host_idx(p, 2, p, 2 * T * 64, 1, tok, sl, 2, T, 64, 0, 0, None) == _lib.ERR_OUT_OF_RANGE  # staging slot
    assert host_idx(p, 2, p, 2 * T * 64, 1, tok, None, 2, T, 64, 0, 0, None) == _lib.ERR_OUT_OF_RANGE  # implied slot 1
    sl[1] = -1
    assert L.kvcm_hip_batch_scatter_host_idx(p, 2, p, 2 * T * 64, 0, tok, sl, 2, T, 64, 0, 0, None) == _lib.ERR_OUT_OF_RANGE
    assert host_idx(p, 2, p, 2 * T * 64, 2, None, sl, 2, T, 64, 0, 0, None) == _lib.ERR_INVALID_ARG
    assert host_idx(p, 2, p, 2 * T * 64, 2, tok, sl, 0, T, 64, 0, 0, None) == _lib.OK
    wide = (ctypes.c_int32 * 1024)(*range(0, 2048, 2))  # 1024 runs in one block: more than an argument block holds
    assert host_idx(p, 2, p, 2 * 1024 * 64, 1, wide, None, 1, 1024, 64, 0, 0, None) == _lib.ERR_TOO_LARGE
    assert _lib.error_string(_lib.ERR_OUT_OF_RANGE) == "index out of range"
    assert _lib.error_string(_lib.ERR_INVALID_ARG) == "invalid argument"
    assert _lib.error_string(0) == "ok"


def test_host_helper_blocks_hash(oracle):
    import numpy as np
    from tair_kvcache_amd import buffer_check
    rng = np.random.default_rng(4)
    crcs = rng.integers(0, 2**32, size=12, dtype=np.uint64).astype(np.uint32)
    assert buffer_check.blocks_hash_from_crcs(crcs.tolist(), 4) == oracle.blocks_hash_from_crcs(crcs, 4).tolist()


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    from tair_kvcache_amd import _lib
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", str(tmp_path / "nope.so"))
    with pytest.raises(_lib.KvcmLibraryError):
        _lib.lib()


def test_header_is_plain_c(tmp_path):
    """A cgo / FFI binding includes the header from C: it must compile as C99 with warnings on, without HIP headers."""
    import shutil
    import subprocess
    if shutil.which("gcc") is None:
        pytest.skip("no gcc")
    src = tmp_path / "use_header.c"
    src.write_text('#include "kvcm_hip.h"\n'
                   "int main(void) { kvcm_iov v; v.type = KVCM_MEMORY_GPU; v.ignore = 0; v.base = 0; v.size = 0;\n"
                   "  return (int)v.size + (KVCM_ERR_IO == -4 ? 0 : 1); }\n")
    subprocess.run(["gcc", "-std=c99", "-Wall", "-Wextra", "-Werror", "-pedantic", "-I", os.path.join(ROOT, "include"),
                    "-c", str(src), "-o", str(tmp_path / "use_header.o")], check=True)
