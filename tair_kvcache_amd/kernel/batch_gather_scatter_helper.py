"""batch_gather_kv_caches / batch_scatter_kv_caches on MI355X.

Drop-in for kv_cache_manager/py_connector/kernel/batch_gather_scatter_helper.py:101-136,208-248: same names,
same positional order, same defaults. Differences a caller can rely on:
  - index arguments may also be int32 tensors (CPU or device); device tensors are used without a copy;
  - the staging tensor may live in HBM or in pinned host memory;
  - `sm_count` (the reference's 3-program PCIe throttle, :110,:115) is accepted and ignored unless
    SM_COUNT_IS_CAP is set, in which case it caps the number of workgroups;
  - shape mismatches raise ValueError before anything is launched (the reference lets Triton fail).
The launch is asynchronous on the current torch stream and never synchronises, like the reference's.
"""
from typing import List, Sequence, Union

import torch

from .. import _lib
from .._torch_util import as_device_i32, lib, ptr, require_cuda, stream_handle

IndexArg = Union[List[int], Sequence[int], torch.Tensor]

# When True, `sm_count` caps the grid as in the reference; when False the device is filled.
SM_COUNT_IS_CAP = False


def _prepare(kv_caches_ptrs_tensor, staging, block_token_indices, block_indices, num_tokens_per_block,
             dim_size_per_token_per_layer, run_tokens=1):
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
    device = kv_caches_ptrs_tensor.device
    P = kv_caches_ptrs_tensor.numel()
    if P == 0:
        raise ValueError("kv_caches_ptrs_tensor is empty")
    row_bytes = D * staging.element_size()
    block_bytes = P * T * row_bytes
    if staging.numel() == 0 or (staging.numel() * staging.element_size()) % block_bytes != 0:
        raise ValueError(
            f"staging tensor of {staging.numel()} elements is not a whole number of [P={P}, T={T}, D={D}] blocks")
    slots = staging.numel() * staging.element_size() // block_bytes
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


def _cap(sm_count):
    return int(sm_count) if SM_COUNT_IS_CAP and sm_count and sm_count > 0 else 0


def batch_gather_kv_caches(
        kv_caches_ptrs_tensor: torch.Tensor,  # int64 [P] device pointers, one per layer and K/V
        dst_tensor: torch.Tensor,  # [block_num, P, num_tokens_per_block, dim_size_per_token_per_layer]
        block_token_indices: IndexArg,  # flat B*T token slots
        dst_block_indices: IndexArg,  # B staging slots
        num_tokens_per_block: int,
        dim_size_per_token_per_layer: int,
        sm_count: int = 3):
    """dst[sb[b], p, t, :] = pool_p[idx[b*T + t], :]  (batch_gather_scatter_helper.py:49-98)."""
    device, P, T, row_bytes, block_bytes, tidx, sidx, B = _prepare(
        kv_caches_ptrs_tensor, dst_tensor, block_token_indices, dst_block_indices, num_tokens_per_block,
        dim_size_per_token_per_layer)
    rc = lib().kvcm_hip_batch_gather(ptr(kv_caches_ptrs_tensor), P, ptr(dst_tensor), block_bytes, ptr(tidx),
                                     ptr(sidx), B, T, row_bytes, _cap(sm_count), stream_handle(device))
    _lib.check(rc, "kvcm_hip_batch_gather")


def batch_scatter_kv_caches(
        kv_caches_ptrs_tensor: torch.Tensor,
        src_tensor: torch.Tensor,  # [block_num, P, num_tokens_per_block, dim_size_per_token_per_layer]
        block_token_indices: IndexArg,
        src_block_indices: IndexArg,
        num_tokens_per_block: int,
        dim_size_per_token_per_layer: int,
        sm_count: int = 3):
    """pool_p[idx[b*T + t], :] = src[sb[b], p, t, :]  (batch_gather_scatter_helper.py:155-205).

    Two work blocks that name the same pool row race; callers must not pass duplicates."""
    device, P, T, row_bytes, block_bytes, tidx, sidx, B = _prepare(
        kv_caches_ptrs_tensor, src_tensor, block_token_indices, src_block_indices, num_tokens_per_block,
        dim_size_per_token_per_layer)
    rc = lib().kvcm_hip_batch_scatter(ptr(kv_caches_ptrs_tensor), P, ptr(src_tensor), block_bytes, ptr(tidx),
                                      ptr(sidx), B, T, row_bytes, _cap(sm_count), stream_handle(device))
    _lib.check(rc, "kvcm_hip_batch_scatter")


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
