"""The value types a transfer client exchanges with the connector, as plain Python.

Field names and enum values follow kv_cache_manager/client/include/common.h:11-63,94-118 and the pybind module
kvcm_py_client (kv_cache_manager/client/pybind/py_client_binding.cc:17-125), so a DataTransferManager built with
this module or with the real kvcm_py_client behaves the same.
"""
import enum
from dataclasses import dataclass, field
from typing import List


class MemoryType(enum.IntEnum):
    CPU = 0
    GPU = 1


class ClientErrorCode(enum.IntEnum):
    ER_OK = 0
    ER_INVALID_PARAMS = 3
    ER_INVALID_SDKBACKEND_CONFIG = 8
    ER_SDK_TIMEOUT = 100
    ER_SDKREAD_ERROR = 104
    ER_SDKWRITE_ERROR = 105
    ER_SDKALLOC_ERROR = 106
    ER_INVALID_LOCAL_BUFFERS = 108
    ER_FILE_IO_ERROR = 111


@dataclass
class Iov:
    type: MemoryType = MemoryType.GPU
    base: int = 0
    size: int = 0
    ignore: bool = False


@dataclass
class BlockBuffer:
    iovs: List[Iov] = field(default_factory=list)
