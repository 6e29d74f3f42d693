"""ctypes doors onto the C oracle (libkvcm_oracle.so), onto the reference-source build (oracle/_ref) when it
exists, and a second, independent restatement in NumPy / Python integers used to cross-check the C one.

TEST INFRASTRUCTURE ONLY: imported by tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg.

Reference lines followed (paths relative to the reference root):
  hash step            kv_cache_manager/manager/hash_util.h:8-12
  GenKeyVector         kv_cache_manager/manager/cache_manager.cc:76-87
  ApplyPrefixHash      kv_cache_manager/optimizer/trace_converter/trace_util.cc:47-56
  _sha256_to_int64     kv_cache_manager/py_connector/sglang/connector.py:397-401
  gather/scatter       kv_cache_manager/py_connector/kernel/batch_gather_scatter_helper.py:49-98,155-205
  legacy gather        kv_cache_manager/py_connector/kernel/gather_scatter_helper.py:10-107
  generate_blocks_idx  kv_cache_manager/py_connector/vllm/v1_connector.py:308-320
  iov CRC              kv_cache_manager/client/src/internal/sdk/sdk_buffer_check_util.cu:10-44
  mask -> save indices kv_cache_manager/py_connector/vllm/v1_connector.py:835-850
  block files          kv_cache_manager/client/src/internal/sdk/local_file_sdk.cc:161-364
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libkvcm_oracle.so")
_REF_PATH = os.path.join(_HERE, "_ref", "libkvcm_refhash.so")

GOLDEN = 0x9E3779B97F4A7C15
_M64 = (1 << 64) - 1


def build(force=False):
    """Compile the C oracle (and oracle/_ref when the reference tree is present) with oracle/Makefile."""
    if force:
        subprocess.check_call(["make", "-C", _HERE, "clean"], stdout=subprocess.DEVNULL)
    subprocess.check_call(["make", "-C", _HERE], stdout=subprocess.DEVNULL)


class CopyDesc(C.Structure):
    _fields_ = [
        ("ptr_table", C.c_void_p),
        ("P", C.c_int32),
        ("ptrs_per_entry", C.c_int32),
        ("entry_stride_bytes", C.c_int64),
        ("staging", C.c_void_p),
        ("staging_block_stride_bytes", C.c_int64),
        ("staging_tile_stride_bytes", C.c_int64),
        ("run_start", C.c_void_p),
        ("staging_idx", C.c_void_p),
        ("B", C.c_int32),
        ("T", C.c_int32),
        ("run_tokens", C.c_int32),
        ("slot_limit", C.c_int32),
        ("row_bytes", C.c_int64),
        ("trailer_ptr_table", C.c_void_p),
        ("trailer_idx", C.c_void_p),
        ("trailer_bytes", C.c_int32),
        ("max_workgroups", C.c_int32),
    ]


class Iov(C.Structure):
    _fields_ = [("base", C.c_void_p), ("size", C.c_size_t)]


_lib = None
_ref = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        L = C.CDLL(_LIB_PATH)
        i64, i32, vp = C.c_int64, C.c_int32, C.c_void_p
        L.kvcm_ref_hash_step.restype = i64
        L.kvcm_ref_hash_step.argtypes = [i64, i64]
        L.kvcm_ref_hash_array.restype = i64
        L.kvcm_ref_hash_array.argtypes = [i64, vp, vp]
        L.kvcm_ref_gen_key_vector.restype = i64
        L.kvcm_ref_gen_key_vector.argtypes = [vp, i64, i64, i64, vp]
        L.kvcm_ref_hash_tokens.restype = i32
        L.kvcm_ref_hash_tokens.argtypes = [vp, vp, i32, i32, i64, vp, vp]
        L.kvcm_ref_hash_tokens_i32.restype = i32
        L.kvcm_ref_hash_tokens_i32.argtypes = [vp, vp, i32, i32, i64, vp, vp]
        L.kvcm_ref_hash_tokens_mt.restype = i32
        L.kvcm_ref_hash_tokens_mt.argtypes = [vp, vp, i32, i32, i64, vp, vp, i32]
        L.kvcm_ref_prefix_chain.restype = i32
        L.kvcm_ref_prefix_chain.argtypes = [vp, vp, i32, vp]
        L.kvcm_ref_sha256.restype = None
        L.kvcm_ref_sha256.argtypes = [vp, C.c_size_t, vp]
        L.kvcm_ref_sha256_first8_be.restype = i32
        L.kvcm_ref_sha256_first8_be.argtypes = [vp, vp, i32, vp]
        for name in ("kvcm_ref_gather_ex", "kvcm_ref_scatter_ex"):
            getattr(L, name).restype = i32
            getattr(L, name).argtypes = [C.POINTER(CopyDesc)]
        for name in ("kvcm_ref_gather_ex_mt", "kvcm_ref_scatter_ex_mt"):
            getattr(L, name).restype = i32
            getattr(L, name).argtypes = [C.POINTER(CopyDesc), i32]
        for name in ("kvcm_ref_batch_gather", "kvcm_ref_batch_scatter"):
            getattr(L, name).restype = i32
            getattr(L, name).argtypes = [vp, i32, vp, i64, vp, vp, i32, i32, i64]
        L.kvcm_ref_generate_blocks_idx.restype = i32
        L.kvcm_ref_generate_blocks_idx.argtypes = [vp, i32, vp, i32, i32, i32, vp]
        L.kvcm_ref_iov_crc32.restype = i32
        L.kvcm_ref_iov_crc32.argtypes = [vp, i32, vp, C.c_size_t]
        L.kvcm_ref_blocks_hash_from_crcs.restype = i32
        L.kvcm_ref_blocks_hash_from_crcs.argtypes = [vp, i64, i32, vp]
        for name in ("kvcm_ref_file_put", "kvcm_ref_file_get"):
            getattr(L, name).restype = i32
            getattr(L, name).argtypes = [C.c_char_p, i64, vp, vp, vp, vp, i32]
        L.kvcm_ref_copy_iovs.restype = i64
        L.kvcm_ref_copy_iovs.argtypes = [vp, vp, i32, i32]
        L.kvcm_ref_first_occurrence.restype = i32
        L.kvcm_ref_first_occurrence.argtypes = [vp, i64, vp, vp]
        L.kvcm_ref_mask_to_indices.restype = i64
        L.kvcm_ref_mask_to_indices.argtypes = [vp, vp, i64, vp]
        _lib = L
    return _lib


def ref_available():
    return os.path.exists(_REF_PATH)


def ref():
    """The reference's own headers compiled by oracle/Makefile (None when oracle/_ref was not built)."""
    global _ref
    if _ref is None and ref_available():
        L = C.CDLL(_REF_PATH)
        i64, i32, vp = C.c_int64, C.c_int32, C.c_void_p
        L.kvcm_refsrc_hash_step.restype = i64
        L.kvcm_refsrc_hash_step.argtypes = [i64, i64]
        L.kvcm_refsrc_hash_array.restype = i64
        L.kvcm_refsrc_hash_array.argtypes = [i64, vp, vp]
        L.kvcm_refsrc_gen_key_vector.restype = i64
        L.kvcm_refsrc_gen_key_vector.argtypes = [vp, i64, i64, vp]
        L.kvcm_refsrc_hash_tokens.restype = i32
        L.kvcm_refsrc_hash_tokens.argtypes = [vp, vp, i32, i32, vp, vp]
        L.kvcm_refsrc_prefix_chain.restype = None
        L.kvcm_refsrc_prefix_chain.argtypes = [vp, i64, vp]
        L.kvcm_refsrc_hash_u32_array.restype = i64
        L.kvcm_refsrc_hash_u32_array.argtypes = [vp, vp, i64]
        _ref = L
    return _ref


def _p(a):
    return a.ctypes.data if a is not None else None


# ---------------------------------------------------------------------------------------------- hashing (C)

def hash_step(h, v):
    return lib().kvcm_ref_hash_step(int(h), int(v))


def _offsets_uniform(R, L):
    return np.arange(R + 1, dtype=np.int64) * L


def hash_tokens(tokens, block_size, token_offsets=None, seed=0, threads=1):
    """tokens: int64/int32 array [R, L] (uniform) or flat with token_offsets [R+1]. Returns (keys, key_offsets)."""
    tokens = np.ascontiguousarray(tokens)
    if token_offsets is None:
        assert tokens.ndim == 2
        R, L = tokens.shape
        token_offsets = _offsets_uniform(R, L)
    token_offsets = np.ascontiguousarray(token_offsets, dtype=np.int64)
    R = len(token_offsets) - 1
    counts = (token_offsets[1:] - token_offsets[:-1]) // block_size
    key_offsets = np.zeros(R + 1, dtype=np.int64)
    np.cumsum(counts, out=key_offsets[1:])
    keys = np.zeros(int(key_offsets[-1]), dtype=np.int64)
    flat = tokens.reshape(-1)
    if flat.dtype == np.int32:
        rc = lib().kvcm_ref_hash_tokens_i32(_p(flat), _p(token_offsets), R, block_size, seed, _p(keys),
                                            _p(key_offsets))
    else:
        assert flat.dtype == np.int64
        if threads > 1:
            rc = lib().kvcm_ref_hash_tokens_mt(_p(flat), _p(token_offsets), R, block_size, seed, _p(keys),
                                               _p(key_offsets), threads)
        else:
            rc = lib().kvcm_ref_hash_tokens(_p(flat), _p(token_offsets), R, block_size, seed, _p(keys),
                                            _p(key_offsets))
    assert rc == 0, rc
    return keys, key_offsets


def gen_key_vector(tokens, block_size, seed=0):
    tokens = np.ascontiguousarray(tokens, dtype=np.int64)
    keys = np.zeros(max(len(tokens) // block_size, 0), dtype=np.int64)
    n = lib().kvcm_ref_gen_key_vector(_p(tokens), len(tokens), block_size, seed, _p(keys))
    assert n == len(keys)
    return keys


def prefix_chain(digests, offsets=None):
    digests = np.ascontiguousarray(digests, dtype=np.int64)
    if offsets is None:
        offsets = np.array([0, len(digests)], dtype=np.int64)
    offsets = np.ascontiguousarray(offsets, dtype=np.int64)
    keys = np.zeros_like(digests)
    rc = lib().kvcm_ref_prefix_chain(_p(digests), _p(offsets), len(offsets) - 1, _p(keys))
    assert rc == 0
    return keys


def pack_strings(strings):
    """UTF-8 bytes of every string back to back, plus int64 offsets [N+1]."""
    enc = [s.encode("utf-8") if isinstance(s, str) else bytes(s) for s in strings]
    offsets = np.zeros(len(enc) + 1, dtype=np.int64)
    np.cumsum([len(e) for e in enc], out=offsets[1:])
    data = np.frombuffer(b"".join(enc) + b"\0", dtype=np.uint8).copy()
    return data, offsets


def sha256_first8_be(strings):
    data, offsets = pack_strings(strings)
    out = np.zeros(len(strings), dtype=np.int64)
    rc = lib().kvcm_ref_sha256_first8_be(_p(data), _p(offsets), len(strings), _p(out))
    assert rc == 0
    return out


def sha256(msg):
    buf = np.frombuffer(bytes(msg) + b"\0", dtype=np.uint8).copy()
    dg = np.zeros(32, dtype=np.uint8)
    lib().kvcm_ref_sha256(_p(buf), len(msg), _p(dg))
    return dg.tobytes()


# ---------------------------------------------------------------------------------------------- hashing (Python ints)

def py_hash_step(h, v):
    """hash_util.h:10 on Python integers; h and v are signed 64-bit values."""
    hu = h & _M64
    sar = (h >> 32) & _M64  # Python's >> on a negative int is arithmetic
    out = hu ^ (((v & _M64) + GOLDEN + ((hu << 12) & _M64) + sar) & _M64)
    return out - (1 << 64) if out >> 63 else out


def py_gen_key_vector(tokens, block_size, seed=0):
    keys = []
    h = seed
    n = len(tokens) // block_size
    for i in range(n):
        for v in tokens[i * block_size:(i + 1) * block_size]:
            h = py_hash_step(h, int(v))
        keys.append(h)
    return keys


# ---------------------------------------------------------------------------------------------- gather / scatter (C)

def _ptr_table(arrays):
    return np.array([a.ctypes.data for a in arrays], dtype=np.uint64)


def make_desc(pool_arrays, staging, run_start, staging_idx, B, T, row_bytes, run_tokens=1, ptrs_per_entry=1,
              entry_stride_bytes=0, slot_limit=0, tile_stride=None, block_stride=None, trailers=None,
              trailer_idx=None, trailer_bytes=0):
    """Builds a CopyDesc over NumPy arrays; returns (desc, keepalive)."""
    table = _ptr_table(pool_arrays)
    P = len(pool_arrays) * ptrs_per_entry
    tile_stride = T * row_bytes + trailer_bytes if tile_stride is None else tile_stride
    block_stride = P * tile_stride if block_stride is None else block_stride
    run_start = np.ascontiguousarray(run_start, dtype=np.int32)
    sidx = None if staging_idx is None else np.ascontiguousarray(staging_idx, dtype=np.int32)
    ttable = None if trailers is None else _ptr_table(trailers)
    tidx = None if trailer_idx is None else np.ascontiguousarray(trailer_idx, dtype=np.int32)
    d = CopyDesc(_p(table), P, ptrs_per_entry, entry_stride_bytes, _p(staging), block_stride, tile_stride,
                 _p(run_start), _p(sidx), B, T, run_tokens, slot_limit, row_bytes, _p(ttable), _p(tidx),
                 trailer_bytes, 0)
    return d, (table, run_start, sidx, ttable, tidx, pool_arrays, staging, trailers)


def gather_ex(desc, threads=1):
    rc = lib().kvcm_ref_gather_ex_mt(C.byref(desc), threads) if threads > 1 else lib().kvcm_ref_gather_ex(C.byref(desc))
    assert rc == 0, rc


def scatter_ex(desc, threads=1):
    rc = lib().kvcm_ref_scatter_ex_mt(C.byref(desc), threads) if threads > 1 else lib().kvcm_ref_scatter_ex(C.byref(desc))
    assert rc == 0, rc


def batch_gather(pool_arrays, staging, token_idx, staging_idx, T, row_bytes):
    """pool_arrays: list of P C-contiguous arrays; staging: array of slots [S, P*T*row_bytes] bytes."""
    table = _ptr_table(pool_arrays)
    token_idx = np.ascontiguousarray(token_idx, dtype=np.int32)
    B = token_idx.size // T
    sidx = None if staging_idx is None else np.ascontiguousarray(staging_idx, dtype=np.int32)
    stride = len(pool_arrays) * T * row_bytes
    rc = lib().kvcm_ref_batch_gather(_p(table), len(pool_arrays), _p(staging), stride, _p(token_idx), _p(sidx), B,
                                     T, row_bytes)
    assert rc == 0, rc


def batch_scatter(pool_arrays, staging, token_idx, staging_idx, T, row_bytes):
    table = _ptr_table(pool_arrays)
    token_idx = np.ascontiguousarray(token_idx, dtype=np.int32)
    B = token_idx.size // T
    sidx = None if staging_idx is None else np.ascontiguousarray(staging_idx, dtype=np.int32)
    stride = len(pool_arrays) * T * row_bytes
    rc = lib().kvcm_ref_batch_scatter(_p(table), len(pool_arrays), _p(staging), stride, _p(token_idx), _p(sidx), B,
                                      T, row_bytes)
    assert rc == 0, rc


def generate_blocks_idx(manager_block_idxes, local_block_ids, T_mgr, T_eng):
    m = np.ascontiguousarray(manager_block_idxes, dtype=np.int32)
    l = np.ascontiguousarray(local_block_ids, dtype=np.int32)
    out = np.zeros((len(m), T_mgr), dtype=np.int32)
    bad = lib().kvcm_ref_generate_blocks_idx(_p(m), len(m), _p(l), len(l), T_mgr, T_eng, _p(out))
    return out, bad


# ---------------------------------------------------------------------------------------------- gather / scatter (NumPy)

def np_batch_gather(pools, staging, token_idx, staging_idx, T):
    """pools: list of P arrays [slots, D]; staging: [S, P, T, D]. batch_gather_scatter_helper.py:57-97."""
    token_idx = np.asarray(token_idx).reshape(-1, T)
    sb = np.arange(len(token_idx)) if staging_idx is None else np.asarray(staging_idx)
    for p, pool in enumerate(pools):
        staging[sb, p] = pool[token_idx]


def np_batch_scatter(pools, staging, token_idx, staging_idx, T):
    """batch_gather_scatter_helper.py:163-205."""
    token_idx = np.asarray(token_idx).reshape(-1, T)
    sb = np.arange(len(token_idx)) if staging_idx is None else np.asarray(staging_idx)
    for p, pool in enumerate(pools):
        pool[token_idx] = staging[sb, p]


def py_generate_blocks_idx(manager_block_idxes, local_block_ids, T_mgr, T_eng):
    """v1_connector.py:308-320, the same double loop."""
    out = []
    for m in manager_block_idxes:
        row = []
        for i in range(T_mgr):
            tok = m * T_mgr + i
            row.append(local_block_ids[tok // T_eng] * T_eng + tok % T_eng)
        out.append(row)
    return out


# ---------------------------------------------------------------------------------------------- which blocks to save

def first_occurrence(keys):
    """first_idx[i] = smallest j with keys[j] == keys[i]; is_repeat[i] = first_idx[i] != i."""
    k = np.ascontiguousarray(keys, dtype=np.int64)
    first = np.zeros(len(k), dtype=np.int32)
    rep = np.zeros(len(k), dtype=np.uint8)
    rc = lib().kvcm_ref_first_occurrence(_p(k), len(k), _p(first), _p(rep))
    assert rc == 0, rc
    return first, rep


def mask_to_indices(mask, mask2=None):
    """Indices whose mask entries are all false (v1_connector.py:835-850, bool_masks branch)."""
    a = np.ascontiguousarray(mask, dtype=np.uint8)
    b = None if mask2 is None else np.ascontiguousarray(mask2, dtype=np.uint8)
    out = np.zeros(len(a), dtype=np.int32)
    n = lib().kvcm_ref_mask_to_indices(_p(a), _p(b), len(a), _p(out))
    return out[:n]


def py_parse_block_mask_to_save_indices(response, target_save_num):
    """v1_connector.py:835-850 on the response dict, both branches."""
    block_mask = response.get("block_mask", {})
    save_indices = []
    if "offset" in block_mask:
        for idx in range(block_mask["offset"], target_save_num):
            save_indices.append(idx)
    else:
        for idx, is_saved in enumerate(block_mask.get("bool_masks", {}).get("values", [])):
            if not is_saved:
                save_indices.append(idx)
    return save_indices


# ---------------------------------------------------------------------------------------------- block files

class FileIov(C.Structure):
    """struct kvcm_ref_fiov."""
    _fields_ = [("type", C.c_uint8), ("ignore", C.c_uint8), ("base", C.c_void_p), ("size", C.c_size_t)]


def _file_call(fn, path, bsz, blocks, sizes=None):
    """blocks: list of (blkid, [iov, ...]); an iov is a NumPy uint8 array (moved), an int n (n ignored bytes) or
    ("null", n) (null base of n bytes). sizes: the URI `size` per block (default bsz)."""
    n = len(blocks)
    blkids = np.array([b[0] for b in blocks], dtype=np.uint64)
    sz = np.array([bsz] * n if sizes is None else sizes, dtype=np.uint64)
    counts = np.array([len(b[1]) for b in blocks], dtype=np.int32)
    flat = [v for b in blocks for v in b[1]]
    iovs = (FileIov * max(len(flat), 1))()
    for k, v in enumerate(flat):
        if isinstance(v, np.ndarray):
            iovs[k] = FileIov(0, 0, v.ctypes.data, v.nbytes)
        elif isinstance(v, tuple):
            iovs[k] = FileIov(0, 0, None, int(v[1]))
        else:
            iovs[k] = FileIov(0, 1, 1, int(v))   # ignored: the base is never touched
    return fn(os.fsencode(path), int(bsz), _p(blkids), _p(sz), _p(counts), C.addressof(iovs), n)


def file_put(path, bsz, blocks, sizes=None):
    """LocalFileSdk::DoPut on host iovs (local_file_sdk.cc:262-364). Returns 0 / -1 invalid / -4 file I/O."""
    return _file_call(lib().kvcm_ref_file_put, path, bsz, blocks, sizes)


def file_get(path, bsz, blocks, sizes=None):
    """LocalFileSdk::DoGet on host iovs (local_file_sdk.cc:161-260)."""
    return _file_call(lib().kvcm_ref_file_get, path, bsz, blocks, sizes)


def copy_iovs(host_buffer, pieces, load):
    """Hf3fsUsrbioClient::CopyIovs on host iovs (hf3fs_usrbio_client.cc:478-505). pieces: NumPy uint8 arrays, or an
    int n for an ignored iov of n bytes. Returns the bytes used in host_buffer."""
    iovs = (FileIov * max(len(pieces), 1))()
    for k, v in enumerate(pieces):
        iovs[k] = FileIov(0, 0, v.ctypes.data, v.nbytes) if isinstance(v, np.ndarray) else FileIov(0, 1, 1, int(v))
    return lib().kvcm_ref_copy_iovs(host_buffer.ctypes.data, C.addressof(iovs), len(pieces), int(load))


# ---------------------------------------------------------------------------------------------- buffer check

def iov_crc32(buffers, cal_bytes):
    """buffers: list of NumPy uint8 arrays (one iov each)."""
    iovs = (Iov * len(buffers))(*[Iov(b.ctypes.data, b.nbytes) for b in buffers])
    out = np.zeros(len(buffers), dtype=np.uint32)
    rc = lib().kvcm_ref_iov_crc32(C.cast(iovs, C.c_void_p), len(buffers), _p(out), cal_bytes)
    assert rc == 0
    return out


def blocks_hash_from_crcs(crcs, iovs_per_block):
    crcs = np.ascontiguousarray(crcs, dtype=np.uint32)
    out = np.zeros(len(crcs) // iovs_per_block, dtype=np.int64)
    rc = lib().kvcm_ref_blocks_hash_from_crcs(_p(crcs), len(crcs), iovs_per_block, _p(out))
    assert rc == 0
    return out
