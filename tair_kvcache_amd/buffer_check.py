"""Buffer check of the transfer client on the GPU: a CRC-32 of the head and tail bytes of every iov, folded
per block with the hashInt64 chain.

    get_iovs_crc     SdkBufferCheckUtil::GetIovsCrc   kv_cache_manager/client/src/internal/sdk/sdk_buffer_check_util.cu:50-69
    get_blocks_hash  SdkBufferCheckUtil::GetBlocksHash kv_cache_manager/client/src/internal/sdk/sdk_buffer_check_util.cc:35-61
"""
import ctypes
import os
from typing import List, Optional, Sequence, Tuple

import torch

from . import _lib
from ._torch_util import lib, ptr, stream_handle

IovLike = Tuple[int, int]  # (device address, size in bytes)


def min_cal_byte_size() -> int:
    """KVCM_CHECK_IOV_BYTE_SIZE, default 4 (sdk_buffer_check_util.cu:6)."""
    return int(os.environ.get("KVCM_CHECK_IOV_BYTE_SIZE", "4"))


def get_iovs_crc(iovs: Sequence[IovLike], device="cuda", cal_byte_size: Optional[int] = None) -> List[int]:
    """CRC-32 over head||tail bytes of each iov. The number of bytes per end is
    min(cal_byte_size, iovs[0].size // 2) -- taken from the FIRST iov, as the reference does (.cu:52) -- and
    an empty list is returned when that is 0."""
    if len(iovs) == 0:
        return []
    limit = min_cal_byte_size() if cal_byte_size is None else int(cal_byte_size)
    cal = min(limit, int(iovs[0][1]) // 2)
    if cal == 0:
        return []
    n = len(iovs)
    for i, (base, size) in enumerate(iovs):
        # the count of bytes comes from the first iov only; the reference would read past a shorter iov's end
        if int(base) == 0 or int(size) < cal:
            raise ValueError(f"iov {i} (base {int(base):#x}, size {int(size)}) cannot supply {cal} bytes per end")
    table = (_lib.IovDevice * n)(*[_lib.IovDevice(int(b), int(s)) for b, s in iovs])
    raw = torch.frombuffer(bytearray(bytes(table)), dtype=torch.uint8)
    d_iovs = raw.to(device)
    d_crc = torch.empty(n, dtype=torch.int32, device=device)
    rc = lib().kvcm_hip_iov_crc32(ptr(d_iovs), n, ptr(d_crc), cal, stream_handle(d_crc.device))
    _lib.check(rc, "kvcm_hip_iov_crc32")
    return [int(v) & 0xFFFFFFFF for v in d_crc.tolist()]  # .tolist() waits for the stream, like the reference


def blocks_hash_from_crcs(crcs: Sequence[int], iovs_per_block: int) -> List[int]:
    n = len(crcs)
    arr = (ctypes.c_uint32 * max(n, 1))(*[int(c) & 0xFFFFFFFF for c in crcs])
    out = (ctypes.c_int64 * max(n // iovs_per_block, 1))()
    rc = lib().kvcm_blocks_hash_from_crcs(ctypes.cast(arr, ctypes.c_void_p), n, int(iovs_per_block),
                                          ctypes.cast(out, ctypes.c_void_p))
    _lib.check(rc, "kvcm_blocks_hash_from_crcs")
    return [int(out[i]) for i in range(n // iovs_per_block)]


def get_blocks_hash(block_buffers: Sequence[Sequence[IovLike]], device="cuda",
                    max_iov_num: Optional[int] = None) -> List[int]:
    """One int64 per block buffer: the hash chain (seed 0) over the CRCs of its iovs. With max_iov_num, whole
    blocks are added only while the iov count stays within it (sdk_buffer_check_util.cc:43-53)."""
    if len(block_buffers) == 0:
        return []
    iov_num = len(block_buffers[0])
    flat = []
    for bb in block_buffers:
        if len(bb) != iov_num:
            raise ValueError("every block buffer must hold the same number of iovs")
        if max_iov_num is not None and len(flat) + len(bb) > max_iov_num:
            break
        flat.extend(bb)
    crcs = get_iovs_crc(flat, device=device)
    return blocks_hash_from_crcs(crcs, iov_num) if crcs else []
