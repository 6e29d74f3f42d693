"""Single-block gather/scatter over one [2, total_tokens, hidden] tensor per layer, and the staging-slot pool.

Drop-in for kv_cache_manager/py_connector/kernel/gather_scatter_helper.py: gather_kv_caches (:143-172),
scatter_kv_caches (:110-140) and CopyBufferAllocator (:175-252) keep their names, argument order and error
behaviour. The two kernels run through the same HIP tile mover as the batch operators (one launch over
2*num_layers tiles) instead of a (num_layers, num_tokens) grid of tiny programs.
"""
import threading
from typing import List, Sequence, Union

import torch

from .. import _lib
from .._torch_util import as_device_i32, lib, ptr, require_cuda, stream_handle


class LayerMismatchError(AssertionError, ValueError):
    """The reference asserts on this condition (gather_scatter_helper.py:117,150)."""


def _legacy_desc(kv_caches_ptrs, total_token_in_kvcache, staging, token_indices):
    require_cuda(kv_caches_ptrs, "kv_caches_ptrs")
    if kv_caches_ptrs.dtype != torch.int64 or kv_caches_ptrs.dim() != 1 or not kv_caches_ptrs.is_contiguous():
        raise ValueError("kv_caches_ptrs must be a contiguous 1-D int64 tensor of device pointers")
    if kv_caches_ptrs.shape[0] != staging.shape[0]:
        raise LayerMismatchError("Number of layers mismatch")
    if staging.dim() != 4 or staging.shape[1] != 2 or not staging.is_contiguous():
        raise ValueError("the staging tensor must be contiguous [num_layers, 2, num_tokens_in_block, hidden_size]")
    if not staging.is_cuda and not staging.is_pinned():
        raise ValueError("the staging tensor must be on the GPU or in pinned host memory")
    device = kv_caches_ptrs.device
    idx = as_device_i32(token_indices, device, "token_indices")
    T = idx.numel()
    if T != staging.shape[2]:
        raise ValueError(f"{T} token indices for a staging tensor of {staging.shape[2]} tokens")
    if int(total_token_in_kvcache) <= 0:
        raise ValueError("total_token_in_kvcache must be positive")
    L = kv_caches_ptrs.shape[0]
    row_bytes = staging.shape[3] * staging.element_size()
    d = _lib.CopyDesc()
    d.d_ptr_table = ptr(kv_caches_ptrs)
    d.P = 2 * L
    d.ptrs_per_entry = 2  # K at offset 0, V at total_tokens * hidden (gather_scatter_helper.py:96-97)
    d.entry_stride_bytes = int(total_token_in_kvcache) * row_bytes
    d.d_staging = ptr(staging)
    d.staging_tile_stride_bytes = T * row_bytes
    d.staging_block_stride_bytes = 2 * L * T * row_bytes
    d.d_run_start = ptr(idx)
    d.d_staging_idx = None
    d.B = 1
    d.T = T
    d.run_tokens = 1
    d.slot_limit = int(total_token_in_kvcache)  # rows with idx >= total are skipped (:37-38,:88-89)
    d.row_bytes = row_bytes
    d.d_trailer_ptr_table = None
    d.d_trailer_idx = None
    d.trailer_bytes = 0
    d.max_workgroups = 0
    return d, idx, device


def scatter_kv_caches(
        kv_caches_ptrs: torch.Tensor,  # int64 [num_layers]; each points at [2, total_token_in_kvcache, hidden]
        total_token_in_kvcache: int,
        src_tensor: torch.Tensor,  # [num_layers, 2, num_tokens_in_block, hidden_size]
        token_indices: Union[List[int], Sequence[int], torch.Tensor]):
    """cache_l[kv, idx[t], :] = src[l, kv, t, :]; rows with idx[t] >= total_token_in_kvcache are skipped."""
    if len(token_indices) == 0:
        return
    d, idx, device = _legacy_desc(kv_caches_ptrs, total_token_in_kvcache, src_tensor, token_indices)
    rc = lib().kvcm_hip_scatter_ex(d, stream_handle(device))
    _lib.check(rc, "kvcm_hip_scatter_ex")


def gather_kv_caches(
        kv_caches_ptrs: torch.Tensor,
        total_token_in_kvcache: int,
        dst_tensor: torch.Tensor,  # [num_layers, 2, num_tokens_in_block, hidden_size]
        token_indices: Union[List[int], Sequence[int], torch.Tensor]):
    """dst[l, kv, t, :] = cache_l[kv, idx[t], :]; rows with idx[t] >= total_token_in_kvcache are skipped."""
    if len(token_indices) == 0:
        return
    d, idx, device = _legacy_desc(kv_caches_ptrs, total_token_in_kvcache, dst_tensor, token_indices)
    rc = lib().kvcm_hip_gather_ex(d, stream_handle(device))
    _lib.check(rc, "kvcm_hip_gather_ex")


class CopyBufferAllocator:
    """A fixed pool of `max_count` staging slots of `shape` carved out of one tensor.

    Behaviour of the reference class (gather_scatter_helper.py:175-252): one zero-filled backing tensor
    `_raw_buffer` of shape [max_count] + shape, pinned when it lives on the CPU; slots are handed out from the
    tail of the free list; alloc_buffer_idx_blocking waits on a condition until enough slots are free;
    free_buffer wakes every waiter. ValueError for a bad count or slot index, RuntimeError when more slots are
    returned than are in use.
    """

    def __init__(self, device, dtype, shape: List[int], max_count: int):
        if max_count <= 0:
            raise ValueError("max_count must be positive")
        self.max_count = max_count
        self.device = torch.device(device)
        self.dtype = dtype
        self._cond = threading.Condition()
        # host staging is pinned so that the GPU (and the storage SDK's DMA) can address it directly
        need_pin = self.device.type == "cpu" and torch.cuda.is_available()
        self._raw_buffer = torch.zeros([max_count] + list(shape), dtype=dtype, device=self.device,
                                       pin_memory=need_pin)
        self._free_idx_list = list(range(max_count))
        self._free_buffer_list = [self._raw_buffer[i] for i in range(max_count)]
        self.shape = self._free_buffer_list[0].shape
        self._inuse_count = 0

    @property
    def slot_nbytes(self):
        return self._raw_buffer[0].numel() * self._raw_buffer.element_size()

    def alloc_buffer_idx_blocking(self, count: int) -> List[int]:
        if count <= 0:
            raise ValueError("count must be positive")
        if count > self.max_count:
            raise ValueError(f"count ({count}) exceeds max_count ({self.max_count})")
        with self._cond:
            self._cond.wait_for(lambda: self._inuse_count + count <= self.max_count)
            self._inuse_count += count
            taken = self._free_idx_list[-count:]
            del self._free_idx_list[-count:]
            return taken

    def get_buffer_by_idx(self, indices: List[int]):
        return [self._free_buffer_list[i] for i in indices]

    def free_buffer(self, buffers: List[int]):
        if not buffers:
            return
        with self._cond:
            for idx in buffers:
                if idx >= self.max_count or idx < 0:
                    raise ValueError(f"Buffer idx {idx} wrong")
            n = len(buffers)
            if self._inuse_count < n:
                raise RuntimeError(f"Trying to free {n} buffers, but only {self._inuse_count} are in use")
            self._inuse_count -= n
            self._free_idx_list.extend(buffers)
            self._cond.notify_all()
