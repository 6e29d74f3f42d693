"""Which blocks of a batch have to be saved, decided on the GPU.

    parse_block_mask_to_save_indices   TairKvCacheConnector.parse_block_mask_to_save_indices
                                       kv_cache_manager/py_connector/vllm/v1_connector.py:835-850
    first_occurrence                   no counterpart: the manager filters shared blocks per request
                                       (FilterWriteCache, kv_cache_manager/manager/cache_manager.cc:589-635)
    select_save_indices                both combined, for a whole batch of requests

The index tensors stay on the device and feed `connector.generate_blocks_idx` / `generate_run_starts` directly.
"""
from typing import Optional, Tuple

import torch

from . import _lib
from ._torch_util import lib, ptr, require_cuda, stream_handle


def _as_mask(mask, name):
    require_cuda(mask, name)
    if mask.dtype == torch.bool:
        mask = mask.view(torch.uint8)
    if mask.dtype != torch.uint8 or mask.dim() != 1:
        raise ValueError(f"{name} must be a 1-D bool or uint8 tensor")
    return mask.contiguous()


def first_occurrence(keys: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """(first_idx int32 [n], is_repeat bool [n]): first_idx[i] = smallest j with keys[j] == keys[i];
    is_repeat[i] = a smaller index holds the same key. Asynchronous on the current stream."""
    require_cuda(keys, "keys")
    if keys.dtype != torch.int64 or keys.dim() != 1:
        raise ValueError("keys must be a 1-D int64 tensor")
    keys = keys.contiguous()
    n = keys.numel()
    first = torch.empty(n, dtype=torch.int32, device=keys.device)
    rep = torch.empty(n, dtype=torch.uint8, device=keys.device)
    if n:
        ws_bytes = lib().kvcm_hip_first_occurrence_workspace_bytes(n)
        if ws_bytes < 0:
            raise _lib.KvcmError(int(ws_bytes), "kvcm_hip_first_occurrence_workspace_bytes")
        ws = torch.empty(ws_bytes // 4, dtype=torch.int32, device=keys.device)
        rc = lib().kvcm_hip_first_occurrence(ptr(keys), n, ptr(ws), ws_bytes, ptr(first), ptr(rep),
                                             stream_handle(keys.device))
        _lib.check(rc, "kvcm_hip_first_occurrence")
    return first, rep.view(torch.bool)


def mask_to_indices(mask: torch.Tensor, mask2: Optional[torch.Tensor] = None) -> Tuple[torch.Tensor, torch.Tensor]:
    """(indices int32 [n], count int32 [1]) on the device: indices[:count] are the positions, ascending, where mask
    (and mask2) are false. No synchronisation: read `count` when the list's length is needed on the host."""
    a = _as_mask(mask, "mask")
    b = None if mask2 is None else _as_mask(mask2, "mask2")
    if b is not None and b.numel() != a.numel():
        raise ValueError("mask and mask2 differ in length")
    n = a.numel()
    indices = torch.empty(n, dtype=torch.int32, device=a.device)
    count = torch.empty(1, dtype=torch.int32, device=a.device)
    ws_bytes = lib().kvcm_hip_mask_to_indices_workspace_bytes(n)
    if ws_bytes < 0:
        raise _lib.KvcmError(int(ws_bytes), "kvcm_hip_mask_to_indices_workspace_bytes")
    ws = torch.empty(ws_bytes // 4, dtype=torch.int32, device=a.device)
    rc = lib().kvcm_hip_mask_to_indices(ptr(a) if n else None, ptr(b) if (b is not None and n) else None, n, ptr(ws),
                                        ws_bytes, ptr(indices) if n else None, ptr(count), stream_handle(a.device))
    _lib.check(rc, "kvcm_hip_mask_to_indices")
    return indices, count


def parse_block_mask_to_save_indices(response: dict, target_save_num: int, device="cuda") -> list:
    """The reference's method, same argument and result (a Python list); the bool mask goes through the device
    kernel, the offset branch is a range."""
    block_mask = response.get("block_mask", {})
    if "offset" in block_mask:
        return list(range(block_mask["offset"], target_save_num))
    values = block_mask.get("bool_masks", {}).get("values", [])
    if not values:
        return []
    mask = torch.tensor([bool(v) for v in values], dtype=torch.bool).to(device)
    indices, count = mask_to_indices(mask)
    return indices[:int(count.item())].tolist()


def select_save_indices(keys: torch.Tensor, saved_mask: Optional[torch.Tensor] = None) -> Tuple[torch.Tensor, torch.Tensor]:
    """Positions in a batch's flat key list that have to be saved: the first occurrence of every key that the
    manager's mask (true = already stored) does not cover. Returns (indices, count) as mask_to_indices."""
    _, rep = first_occurrence(keys)
    if saved_mask is None:
        return mask_to_indices(rep)
    return mask_to_indices(saved_mask, rep)
