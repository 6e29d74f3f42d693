"""Small helpers shared by the operator modules: torch is used for device memory and streams only."""
import torch

from . import _lib


def stream_handle(device):
    """The current torch stream of `device` as the void* the C-ABI takes."""
    return torch.cuda.current_stream(device).cuda_stream


def require_cuda(t, name):
    if not isinstance(t, torch.Tensor) or not t.is_cuda:
        raise ValueError(f"{name} must be a tensor on the GPU")


def as_device_i32(values, device, name):
    """int32 device tensor from a Python list, a CPU tensor or a device tensor (device tensors: no copy).

    The reference uploads its index lists from pageable memory with non_blocking=True
    (kv_cache_manager/py_connector/kernel/batch_gather_scatter_helper.py:118-121); the copy is ordered on the
    current stream before the kernel, and the caching allocator keeps the buffer until that stream has passed.
    """
    if isinstance(values, torch.Tensor):
        t = values
        if t.dtype != torch.int32:
            t = t.to(torch.int32)
        t = t.reshape(-1)
        if t.device != device:
            t = t.to(device, non_blocking=True)
        return t.contiguous()
    try:
        t = torch.tensor(values, dtype=torch.int32, device="cpu").reshape(-1)
    except (TypeError, ValueError, RuntimeError) as e:
        raise ValueError(f"{name} must be a list of ints or an integer tensor: {e}") from e
    return t.to(device, non_blocking=True)


def ptr(t):
    return None if t is None else t.data_ptr()


def lib():
    return _lib.lib()
