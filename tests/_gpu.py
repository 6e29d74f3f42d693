"""Helpers of the GPU parity tests: NumPy inputs -> device tensors, pointer tables, byte views."""
import numpy as np
import torch


def dev(a, device="cuda"):
    """NumPy array -> device tensor of the same bytes (uint16 travels as int16)."""
    a = np.ascontiguousarray(a)
    if a.dtype == np.uint16:
        return torch.from_numpy(a.view(np.int16)).to(device)
    if a.dtype == np.uint32:
        return torch.from_numpy(a.view(np.int32)).to(device)
    return torch.from_numpy(a).to(device)


def host(t, dtype):
    """Device tensor -> NumPy array reinterpreted as `dtype`."""
    return t.detach().cpu().contiguous().numpy().view(dtype)


def ptr_table(tensors, device="cuda"):
    return torch.tensor([t.data_ptr() for t in tensors], dtype=torch.int64, device=device)


def sync():
    torch.cuda.synchronize()
