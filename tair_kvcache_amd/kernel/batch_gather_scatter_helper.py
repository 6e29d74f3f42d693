"""batch_gather_kv_caches / batch_scatter_kv_caches on MI355X.

Drop-in for kv_cache_manager/py_connector/kernel/batch_gather_scatter_helper.py:101-136,208-248: same names,
same positional order, same defaults. Differences a caller can rely on:
  - index arguments may also be int32 tensors (CPU or device); device tensors are used without a copy;
  - index arguments in host memory (Python lists, CPU tensors) are not uploaded at all: they are walked once on the
    calling thread -- range checks, and the discovery that a block's slots are consecutive, which turns the launch
    into the block-table form -- and travel to the kernel inside its argument block (kvcm_hip_batch_*_host_idx);
  - `pool_token_slots` (keyword only) = token slots per pool array: with it, a token slot beyond the pool raises
    ValueError before anything is launched (the reference checks nothing; a wild slot is a GPU memory fault);
  - the staging tensor may live in HBM or in pinned host memory;
  - `sm_count` (the reference's 3-program PCIe throttle, :110,:115) is accepted and ignored unless
    SM_COUNT_IS_CAP is set, in which case it caps the number of workgroups;
  - shape mismatches raise ValueError before anything is launched (the reference lets Triton fail).
The launch is asynchronous on the current torch stream and never synchronises, like the reference's.
"""
from array import array
from typing import List, Sequence, Union

import torch

from .. import _lib
from .._torch_util import as_device_i32, lib, ptr, require_cuda, stream_handle

try:  # one C loop over a list (flat or nested); absent only when the package was not built with its build.py
    from .._kvcm_pylist import blocks_idx as _blocks_idx_c, pack_i32 as _pack_i32
except ImportError:  # host-side convenience only: the lists then go through array('i'), three times slower
    _pack_i32 = _blocks_idx_c = None

IndexArg = Union[List[int], Sequence[int], torch.Tensor]

# When True, `sm_count` caps the grid as in the reference; when False the device is filled.
SM_COUNT_IS_CAP = False


def _geometry(kv_caches_ptrs_tensor, staging, num_tokens_per_block, dim_size_per_token_per_layer, run_tokens=1):
    require_cuda(kv_caches_ptrs_tensor, "kv_caches_ptrs_tensor")
    if kv_caches_ptrs_tensor.dtype != torch.int64 or kv_caches_ptrs_tensor.dim() != 1:
        raise ValueError("kv_caches_ptrs_tensor must be a 1-D int64 tensor of device pointers")
    if not kv_caches_ptrs_tensor.is_contiguous():
        raise ValueError("kv_caches_ptrs_tensor must be contiguous")
    if not isinstance(staging, torch.Tensor) or not staging.is_contiguous():
        raise ValueError("the staging tensor must be a contiguous tensor")
    if not staging.is_cuda and not staging.is_pinned():
        raise ValueError("the staging tensor must be on the GPU or in pinned host memory")
    T, D = int(num_tokens_per_block), int(dim_size_per_token_per_layer)
    if T <= 0 or D <= 0 or run_tokens <= 0 or T % run_tokens != 0:
        raise ValueError("num_tokens_per_block and dim_size_per_token_per_layer must be positive")
    P = kv_caches_ptrs_tensor.numel()
    if P == 0:
        raise ValueError("kv_caches_ptrs_tensor is empty")
    esz = staging.element_size()
    row_bytes = D * esz
    block_bytes = P * T * row_bytes
    nbytes = staging.numel() * esz
    if nbytes == 0 or nbytes % block_bytes != 0:
        raise ValueError(
            f"staging tensor of {staging.numel()} elements is not a whole number of [P={P}, T={T}, D={D}] blocks")
    return kv_caches_ptrs_tensor.device, P, T, row_bytes, block_bytes, nbytes // block_bytes


def _prepare(kv_caches_ptrs_tensor, staging, block_token_indices, block_indices, num_tokens_per_block,
             dim_size_per_token_per_layer, run_tokens=1):
    device, P, T, row_bytes, block_bytes, slots = _geometry(
        kv_caches_ptrs_tensor, staging, num_tokens_per_block, dim_size_per_token_per_layer, run_tokens)
    sidx = as_device_i32(block_indices, device, "block indices")
    B = sidx.numel()
    tidx = as_device_i32(block_token_indices, device, "block_token_indices")
    if tidx.numel() != B * (T // run_tokens):
        raise ValueError(
            f"block_token_indices has {tidx.numel()} entries, expected {B} blocks x {T // run_tokens}")
    if not isinstance(block_indices, torch.Tensor) and B > 0:
        if min(block_indices) < 0 or max(block_indices) >= slots:
            raise ValueError(f"staging block index out of range [0, {slots})")
    return device, P, T, row_bytes, block_bytes, tidx, sidx, B


def pack_index_list(values, name="index list"):
    """A Python list of ints -- flat, or nested as generate_blocks_idx returns it in the reference (one list per
    block) -- as packed int32 in host memory: bytes, or an array('i') when the C helper is not built."""
    try:
        if _pack_i32 is not None and isinstance(values, (list, tuple)):
            return _pack_i32(values)
        if isinstance(values, (list, tuple)) and len(values) > 0 and isinstance(values[0], (list, tuple)):
            flat = array("i")
            for row in values:
                flat.extend(row)
            return flat
        return array("i", values)
    except (TypeError, OverflowError) as e:
        raise ValueError(f"{name} must be a list of ints that fit 32 bits, or an integer tensor: {e}") from e


def _host_i32(values, name):
    """(address, count, keep-alive) of `values` as int32 in host memory, or None when `values` lives on the GPU."""
    if isinstance(values, torch.Tensor):
        if values.is_cuda:
            return None
        t = values.reshape(-1)
        if t.dtype != torch.int32 or not t.is_contiguous():
            t = t.to(torch.int32).contiguous()
        return t.data_ptr(), t.numel(), t
    packed = getattr(values, "packed_int32", None)  # a HostBlockIndex of tair_kvcache_amd.connector
    if packed is not None:
        values = packed
    if isinstance(values, bytes):  # already packed by pack_index_list
        return values, len(values) // 4, values
    if not (isinstance(values, array) and values.typecode == "i"):
        values = pack_index_list(values, name)
        if isinstance(values, bytes):
            return values, len(values) // 4, values
    return values.buffer_info()[0], len(values), values


def _stream(stream, device):
    """`stream` of a call: None = the current torch stream of `device`, else a torch.cuda.Stream or a raw handle."""
    if stream is None:
        return stream_handle(device)
    return getattr(stream, "cuda_stream", stream)


def _run(host_fn, device_fn, kv_caches_ptrs_tensor, staging, block_token_indices, block_indices,
         num_tokens_per_block, dim_size_per_token_per_layer, sm_count, pool_token_slots, stream=None):
    """Host index lists take the entry point that carries them in the kernel's argument block; anything on the GPU
    (or a block of more runs than an argument block holds) takes the device-index entry point."""
    tok = _host_i32(block_token_indices, "block_token_indices")
    sl = _host_i32(block_indices, "block indices") if tok is not None else None
    if tok is not None and sl is not None:
        device, P, T, row_bytes, block_bytes, slots = _geometry(
            kv_caches_ptrs_tensor, staging, num_tokens_per_block, dim_size_per_token_per_layer)
        B = sl[1]
        if tok[1] != B * T:
            raise ValueError(f"block_token_indices has {tok[1]} entries, expected {B} blocks x {T}")
        rc = host_fn(ptr(kv_caches_ptrs_tensor), P, ptr(staging), block_bytes, slots, tok[0], sl[0], B, T, row_bytes,
                     int(pool_token_slots or 0), _cap(sm_count), _stream(stream, device))
        if rc == _lib.ERR_OUT_OF_RANGE:
            raise ValueError(f"index out of range: staging slots must lie in [0, {slots}), token slots below "
                             f"pool_token_slots ({pool_token_slots})")
        if rc != _lib.ERR_TOO_LARGE:
            _lib.check(rc, host_fn.__name__)
            return
    if hasattr(stream, "cuda_stream"):
        # list arguments are uploaded on torch's current stream: that has to be the stream of the launch
        with torch.cuda.stream(stream):
            device, P, T, row_bytes, block_bytes, tidx, sidx, B = _prepare(
                kv_caches_ptrs_tensor, staging, block_token_indices, block_indices, num_tokens_per_block,
                dim_size_per_token_per_layer)
    else:
        device, P, T, row_bytes, block_bytes, tidx, sidx, B = _prepare(
            kv_caches_ptrs_tensor, staging, block_token_indices, block_indices, num_tokens_per_block,
            dim_size_per_token_per_layer)
    rc = device_fn(ptr(kv_caches_ptrs_tensor), P, ptr(staging), block_bytes, ptr(tidx), ptr(sidx), B, T, row_bytes,
                   _cap(sm_count), _stream(stream, device))
    _lib.check(rc, device_fn.__name__)


def _cap(sm_count):
    return int(sm_count) if SM_COUNT_IS_CAP and sm_count and sm_count > 0 else 0


def batch_gather_kv_caches(
        kv_caches_ptrs_tensor: torch.Tensor,  # int64 [P] device pointers, one per layer and K/V
        dst_tensor: torch.Tensor,  # [block_num, P, num_tokens_per_block, dim_size_per_token_per_layer]
        block_token_indices: IndexArg,  # flat B*T token slots
        dst_block_indices: IndexArg,  # B staging slots
        num_tokens_per_block: int,
        dim_size_per_token_per_layer: int,
        sm_count: int = 3,
        *, pool_token_slots: int = 0, stream=None):
    """dst[sb[b], p, t, :] = pool_p[idx[b*T + t], :]  (batch_gather_scatter_helper.py:49-98).
    `stream` (keyword only): a torch.cuda.Stream to launch on instead of torch's current one."""
    L = lib()
    _run(L.kvcm_hip_batch_gather_host_idx, L.kvcm_hip_batch_gather, kv_caches_ptrs_tensor, dst_tensor,
         block_token_indices, dst_block_indices, num_tokens_per_block, dim_size_per_token_per_layer, sm_count,
         pool_token_slots, stream)


def batch_scatter_kv_caches(
        kv_caches_ptrs_tensor: torch.Tensor,
        src_tensor: torch.Tensor,  # [block_num, P, num_tokens_per_block, dim_size_per_token_per_layer]
        block_token_indices: IndexArg,
        src_block_indices: IndexArg,
        num_tokens_per_block: int,
        dim_size_per_token_per_layer: int,
        sm_count: int = 3,
        *, pool_token_slots: int = 0, stream=None):
    """pool_p[idx[b*T + t], :] = src[sb[b], p, t, :]  (batch_gather_scatter_helper.py:155-205).

    Two work blocks that name the same pool row race; callers must not pass duplicates."""
    L = lib()
    _run(L.kvcm_hip_batch_scatter_host_idx, L.kvcm_hip_batch_scatter, kv_caches_ptrs_tensor, src_tensor,
         block_token_indices, src_block_indices, num_tokens_per_block, dim_size_per_token_per_layer, sm_count,
         pool_token_slots, stream)


def paged_gather_kv_caches(kv_caches_ptrs_tensor, dst_tensor, run_start_slots: IndexArg,
                           dst_block_indices: IndexArg, num_tokens_per_block: int,
                           dim_size_per_token_per_layer: int, run_tokens: int, sm_count: int = 0):
    """Block-table fast path: every entry of run_start_slots names `run_tokens` consecutive token slots
    (engine_block_id * engine_block_size + offset), so no per-token index is built or uploaded."""
    device, P, T, row_bytes, block_bytes, ridx, sidx, B = _prepare(
        kv_caches_ptrs_tensor, dst_tensor, run_start_slots, dst_block_indices, num_tokens_per_block,
        dim_size_per_token_per_layer, run_tokens)
    rc = lib().kvcm_hip_paged_gather(ptr(kv_caches_ptrs_tensor), P, ptr(dst_tensor), block_bytes, ptr(ridx),
                                     int(run_tokens), ptr(sidx), B, T, row_bytes, _cap(sm_count),
                                     stream_handle(device))
    _lib.check(rc, "kvcm_hip_paged_gather")


def paged_scatter_kv_caches(kv_caches_ptrs_tensor, src_tensor, run_start_slots: IndexArg,
                            src_block_indices: IndexArg, num_tokens_per_block: int,
                            dim_size_per_token_per_layer: int, run_tokens: int, sm_count: int = 0):
    device, P, T, row_bytes, block_bytes, ridx, sidx, B = _prepare(
        kv_caches_ptrs_tensor, src_tensor, run_start_slots, src_block_indices, num_tokens_per_block,
        dim_size_per_token_per_layer, run_tokens)
    rc = lib().kvcm_hip_paged_scatter(ptr(kv_caches_ptrs_tensor), P, ptr(src_tensor), block_bytes, ptr(ridx),
                                      int(run_tokens), ptr(sidx), B, T, row_bytes, _cap(sm_count),
                                      stream_handle(device))
    _lib.check(rc, "kvcm_hip_paged_scatter")
