"""ctypes binding of libkvcm_hip.so, the C-ABI declared in include/kvcm_hip.h.

There is no fallback: when the shared library is missing or does not export a declared symbol the import of
any operator fails with KvcmLibraryError, so a run can never pass silently on something that is not the HIP path.
"""
import ctypes as C
import os
import threading

from .build import LIB_PATH


class KvcmLibraryError(RuntimeError):
    pass


class KvcmError(RuntimeError):
    """A non-zero return code of a kvcm_hip_* entry point."""

    def __init__(self, code, what):
        self.code = code
        super().__init__(f"{what} failed with code {code}: {error_string(code)}")


OK = 0
ERR_INVALID_ARG = -1
ERR_ALIGNMENT = -2
ERR_TOO_LARGE = -3
ERR_IO = -4
ERR_OUT_OF_RANGE = -5

i32, i64, vp, sz = C.c_int32, C.c_int64, C.c_void_p, C.c_size_t


class CopyDesc(C.Structure):
    """struct kvcm_copy_desc."""
    _fields_ = [
        ("d_ptr_table", vp), ("P", i32), ("ptrs_per_entry", i32), ("entry_stride_bytes", i64),
        ("d_staging", vp), ("staging_block_stride_bytes", i64), ("staging_tile_stride_bytes", i64),
        ("d_run_start", vp), ("d_staging_idx", vp), ("B", i32), ("T", i32), ("run_tokens", i32),
        ("slot_limit", i32), ("row_bytes", i64), ("d_trailer_ptr_table", vp), ("d_trailer_idx", vp),
        ("trailer_bytes", i32), ("max_workgroups", i32),
    ]


class IovDevice(C.Structure):
    """struct kvcm_iov_device."""
    _fields_ = [("base", vp), ("size", sz)]


# symbol -> (restype, argtypes); every prototype of include/kvcm_hip.h
SIGNATURES = {
    "kvcm_hip_version": (i32, []),
    "kvcm_hip_error_string": (C.c_char_p, [i32]),
    "kvcm_hip_hash_tokens": (i32, [vp, vp, i32, i32, i64, vp, vp, vp]),
    "kvcm_hip_hash_tokens_i32": (i32, [vp, vp, i32, i32, i64, vp, vp, vp]),
    "kvcm_hip_prefix_chain": (i32, [vp, vp, i32, vp, vp]),
    "kvcm_hip_sha256_first8_be": (i32, [vp, vp, i32, vp, vp]),
    "kvcm_hip_batch_gather": (i32, [vp, i32, vp, i64, vp, vp, i32, i32, i64, i32, vp]),
    "kvcm_hip_batch_scatter": (i32, [vp, i32, vp, i64, vp, vp, i32, i32, i64, i32, vp]),
    "kvcm_hip_batch_gather_host_idx": (i32, [vp, i32, vp, i64, i64, vp, vp, i32, i32, i64, i64, i32, vp]),
    "kvcm_hip_batch_scatter_host_idx": (i32, [vp, i32, vp, i64, i64, vp, vp, i32, i32, i64, i64, i32, vp]),
    "kvcm_hip_paged_gather": (i32, [vp, i32, vp, i64, vp, i32, vp, i32, i32, i64, i32, vp]),
    "kvcm_hip_paged_scatter": (i32, [vp, i32, vp, i64, vp, i32, vp, i32, i32, i64, i32, vp]),
    "kvcm_hip_gather_ex": (i32, [C.POINTER(CopyDesc), vp]),
    "kvcm_hip_scatter_ex": (i32, [C.POINTER(CopyDesc), vp]),
    "kvcm_hip_generate_blocks_idx": (i32, [vp, i32, vp, i32, i32, i32, vp, vp, vp]),
    "kvcm_hip_first_occurrence_workspace_bytes": (i64, [i64]),
    "kvcm_hip_first_occurrence": (i32, [vp, i64, vp, i64, vp, vp, vp]),
    "kvcm_hip_first_occurrence_static_max_keys": (i64, []),
    "kvcm_hip_first_occurrence_static": (i32, [vp, i64, vp, vp, vp]),
    "kvcm_hip_mask_to_indices_workspace_bytes": (i64, [i64]),
    "kvcm_hip_mask_to_indices": (i32, [vp, vp, i64, vp, i64, vp, vp, vp]),
    "kvcm_hip_iov_crc32": (i32, [vp, i32, vp, sz, vp]),
    "kvcm_blocks_hash_from_crcs": (i32, [vp, i64, i32, vp]),
    "kvcm_file_store_create": (i32, [i64, i64, i32, i32, C.POINTER(vp)]),
    "kvcm_file_store_destroy": (None, [vp]),
    "kvcm_file_store_put": (i32, [vp, C.c_char_p, vp, vp, vp, vp, i32]),
    "kvcm_file_store_get": (i32, [vp, C.c_char_p, vp, vp, vp, vp, i32]),
    "kvcm_copy_iovs": (i32, [vp, sz, vp, i32, i32, vp]),
}

_lock = threading.Lock()
_lib = None


def lib():
    """The loaded library (thread-safe, loaded once)."""
    global _lib
    if _lib is None:
        with _lock:
            if _lib is None:
                if not os.path.exists(LIB_PATH):
                    raise KvcmLibraryError(
                        f"{LIB_PATH} is not built; run `python -m tair_kvcache_amd.build` (needs hipcc). "
                        "There is no CPU fallback.")
                # torch first: it brings its own copy of the HIP runtime, and a process must end up with ONE runtime.
                # Loaded after torch, this library binds to the runtime torch has already loaded; loaded before it,
                # the library pulls in the system's copy, torch then loads its own, and the kernels registered with
                # one runtime are launched on streams of the other ("no ROCm-capable device is detected").
                import torch  # noqa: F401
                try:
                    L = C.CDLL(LIB_PATH)
                except OSError as e:
                    raise KvcmLibraryError(f"cannot load {LIB_PATH}: {e}") from e
                for name, (res, args) in SIGNATURES.items():
                    try:
                        fn = getattr(L, name)
                    except AttributeError as e:
                        raise KvcmLibraryError(f"{LIB_PATH} does not export {name}") from e
                    fn.restype = res
                    fn.argtypes = args
                _lib = L
    return _lib


def error_string(code):
    return lib().kvcm_hip_error_string(int(code)).decode()


def check(code, what):
    if code != OK:
        raise KvcmError(code, what)
