"""Block files on a local or network file system, for staging slots in HBM or host memory.

    StandardUri              kv_cache_manager/common/standard_uri.cc:16-140
    LocalFileSdk             kv_cache_manager/client/src/internal/sdk/local_file_sdk.cc:61-364
                             (SplitByPath: kv_cache_manager/client/src/internal/sdk/sdk_interface.cc:5-17)
    copy_iovs                Hf3fsUsrbioClient::CopyIovs
                             kv_cache_manager/client/src/internal/sdk/hf3fs_usrbio_client.cc:478-505
    LocalFileTransferClient  the TransferClient surface the connector calls
                             (kv_cache_manager/client/include/transfer_client.h:19-21,
                              kv_cache_manager/client/src/transfer_client_impl.cc:119-161) over one LocalFileSdk

The byte movement is native (`kvcm_file_store_*` of libkvcm_hip.so); this module parses URIs, groups blocks by file
and maps return codes as the reference's classes do. `Iov.type = MemoryType.GPU` is served through pinned bounce
buffers, so `DataTransferManager` can keep its staging pool in HBM.
"""
import ctypes as C
import os
from typing import Dict, List, Sequence, Tuple

from . import _lib, client_types
from ._torch_util import lib


class StandardUri:
    """protocol://[user@]host[:port][/path][?k=v&k2=v2]; parameters are kept sorted by key like the std::map."""

    def __init__(self, uri: str = ""):
        self.protocol, self.user_info, self.hostname, self.port, self.path = "", "", "", 0, ""
        self.params: Dict[str, str] = {}
        if uri:
            self.parse(uri)

    def parse(self, uri: str) -> bool:
        self.__init__()
        end = uri.find("://")
        if end < 0:
            return False
        self.protocol = uri[:end]
        authority = end + 3
        host_start = authority
        at = uri.find("@", authority)
        if at >= 0:
            self.user_info = uri[authority:at]
            host_start = at + 1
        path_start = uri.find("/", authority)
        query_start = uri.find("?", authority)
        host_end = min(path_start if path_start >= 0 else len(uri), query_start if query_start >= 0 else len(uri))
        host_port = uri[host_start:host_end]
        colon = host_port.find(":")
        if colon < 0:
            self.hostname = host_port
        else:
            self.hostname = host_port[:colon]
            try:
                self.port = int(host_port[colon + 1:])
            except ValueError:
                return False
        if path_start >= 0:
            if query_start >= 0 and path_start < query_start:
                self.path = uri[path_start:query_start]
                self._parse_params(uri[query_start + 1:])
            else:
                self.path = uri[path_start:]
        elif query_start >= 0:
            self._parse_params(uri[query_start + 1:])
        return True

    def _parse_params(self, query: str):
        start = 0
        while start < len(query):
            end = query.find("&", start)
            if end < 0:
                end = len(query)
            eq = query.find("=", start)
            if 0 <= eq < end:
                self.params[query[start:eq]] = query[eq + 1:end]
            else:
                self.params[query[start:end]] = ""
            start = end + 1

    @classmethod
    def from_uri(cls, source: str) -> "StandardUri":
        """An empty (invalid) URI when `source` does not parse (standard_uri.cc:126-132)."""
        out = cls()
        if not out.parse(source):
            return cls()
        return out

    def valid(self) -> bool:
        return bool(self.protocol)

    def get_param(self, key: str) -> str:
        return self.params.get(key, "")

    def get_param_as_uint(self, key: str, default: int = 0) -> int:
        """GetParamAs<uint64_t>: the whole value must be decimal digits, otherwise the default stays."""
        val = self.get_param(key)
        return int(val) if val.isascii() and val.isdigit() else default

    def set_param(self, key: str, value: str):
        self.params[key] = value

    def to_uri_string(self) -> str:
        if not self.valid():
            return ""
        out = self.protocol + "://"
        if self.user_info:
            out += self.user_info + "@"
        out += self.hostname
        if self.port > 0:
            out += f":{self.port}"
        out += self.path
        if self.params:
            out += "?" + "&".join(f"{k}={self.params[k]}" for k in sorted(self.params))
        return out


class _Iov(C.Structure):
    """struct kvcm_iov."""
    _fields_ = [("type", C.c_uint8), ("ignore", C.c_uint8), ("base", C.c_void_p), ("size", C.c_size_t)]


def copy_iovs(host_buffer_ptr: int, host_buffer_size: int, iovs, load: bool, stream_handle=None) -> int:
    """iovs <-> one contiguous host buffer, pieces back to back, ignored iovs taking no room
    (Hf3fsUsrbioClient::CopyIovs, kv_cache_manager/client/src/internal/sdk/hf3fs_usrbio_client.cc:478-505).
    `iovs` are objects with type / base / size / ignore. Returns the library's code (0 = done and synchronised)."""
    arr = (_Iov * max(len(iovs), 1))()
    for k, iov in enumerate(iovs):
        arr[k].type = int(iov.type)
        arr[k].ignore = 1 if iov.ignore else 0
        arr[k].base = int(iov.base) or None
        arr[k].size = int(iov.size)
    return lib().kvcm_copy_iovs(host_buffer_ptr, host_buffer_size, arr, len(iovs), 1 if load else 0, stream_handle)


def _as_uri(u) -> StandardUri:
    return u if isinstance(u, StandardUri) else StandardUri(str(u))


class LocalFileSdk:
    """Put / Get of blocks in files, `file_offset = blkid * byte_size_per_block`."""

    def __init__(self, client_module=client_types):
        self._cm = client_module
        self._store = None
        self._byte_size_per_block = 0

    def Init(self, byte_size_per_block, bounce_bytes: int = 0, sync_on_put: bool = True, io_threads: int = 0):
        """Returns ER_INVALID_SDKBACKEND_CONFIG (8) for a missing or non-positive block size (local_file_sdk.cc:70-78),
        and for a negative bounce size or more than 32 I/O threads. `io_threads` (0 = 4) is how many threads share the
        device iovs of one Get."""
        bad_config = getattr(self._cm.ClientErrorCode, "ER_INVALID_SDKBACKEND_CONFIG", 8)
        if byte_size_per_block is None or int(byte_size_per_block) <= 0:
            return bad_config
        self.close()
        handle = C.c_void_p()
        rc = lib().kvcm_file_store_create(int(byte_size_per_block), int(bounce_bytes), int(bool(sync_on_put)),
                                          int(io_threads), C.byref(handle))
        if rc == _lib.ERR_INVALID_ARG:
            return bad_config
        _lib.check(rc, "kvcm_file_store_create")
        self._store = handle
        self._byte_size_per_block = int(byte_size_per_block)
        return self._cm.ClientErrorCode.ER_OK

    def close(self):
        if self._store is not None:
            lib().kvcm_file_store_destroy(self._store)
            self._store = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    @staticmethod
    def _split_by_path(uris: Sequence[StandardUri], buffers) -> Dict[str, Tuple[list, list]]:
        groups: Dict[str, Tuple[list, list]] = {}
        for uri, buf in zip(uris, buffers):
            g = groups.setdefault(uri.path, ([], []))
            g[0].append(uri)
            g[1].append(buf)
        return groups

    def _call(self, fn, uris, buffers) -> int:
        n = len(uris)
        for u in uris:
            if not u.path:
                return _lib.ERR_INVALID_ARG
        blkids = (C.c_uint64 * n)(*[u.get_param_as_uint("blkid") for u in uris])
        sizes = (C.c_uint64 * n)(*[u.get_param_as_uint("size") for u in uris])
        counts = (C.c_int32 * n)(*[len(b.iovs) for b in buffers])
        total = sum(counts)
        iovs = (_Iov * max(total, 1))()
        k = 0
        for b in buffers:
            for iov in b.iovs:
                iovs[k].type = int(iov.type)
                iovs[k].ignore = 1 if iov.ignore else 0
                iovs[k].base = int(iov.base) or None
                iovs[k].size = int(iov.size)
                k += 1
        return fn(self._store, uris[0].path.encode(), blkids, sizes, counts, iovs, n)

    def Put(self, remote_uris, local_buffers):
        """(code, actual_remote_uris). Blocks are grouped by file; any failing group ends the call with
        ER_SDKWRITE_ERROR, an unequal number of URIs and buffers with ER_INVALID_PARAMS (local_file_sdk.cc:105-134)."""
        ec = self._cm.ClientErrorCode
        actual: List[StandardUri] = []
        if self._store is None or len(remote_uris) != len(local_buffers):
            return ec.ER_INVALID_PARAMS, actual
        uris = [_as_uri(u) for u in remote_uris]
        for _, (g_uris, g_bufs) in self._split_by_path(uris, local_buffers).items():
            actual.extend(g_uris)
            if self._call(lib().kvcm_file_store_put, g_uris, g_bufs) != _lib.OK:
                return ec.ER_SDKWRITE_ERROR, actual
        return ec.ER_OK, actual

    def Get(self, remote_uris, local_buffers):
        ec = self._cm.ClientErrorCode
        if self._store is None or len(remote_uris) != len(local_buffers):
            return ec.ER_INVALID_PARAMS
        uris = [_as_uri(u) for u in remote_uris]
        for _, (g_uris, g_bufs) in self._split_by_path(uris, local_buffers).items():
            if self._call(lib().kvcm_file_store_get, g_uris, g_bufs) != _lib.OK:
                return ec.ER_SDKREAD_ERROR
        return ec.ER_OK


class LocalFileTransferClient:
    """SaveKvCaches / LoadKvCaches over block files; what `DataTransferManager` needs from a transfer client."""

    def __init__(self, byte_size_per_block: int, client_module=client_types, bounce_bytes: int = 0,
                 sync_on_put: bool = True, io_threads: int = 0):
        self._cm = client_module
        self._sdk = LocalFileSdk(client_module)
        code = self._sdk.Init(byte_size_per_block, bounce_bytes, sync_on_put, io_threads)
        if code != client_module.ClientErrorCode.ER_OK:
            raise ValueError(f"LocalFileSdk.Init failed with code {int(code)}")

    def SaveKvCaches(self, uri_str_vec, block_buffers):
        code, actual = self._sdk.Put([StandardUri(u) for u in uri_str_vec], block_buffers)
        if code != self._cm.ClientErrorCode.ER_OK:
            return code, []
        return code, [u.to_uri_string() for u in actual]

    def LoadKvCaches(self, uri_str_vec, block_buffers):
        return self._sdk.Get([StandardUri(u) for u in uri_str_vec], block_buffers)

    def close(self):
        self._sdk.close()
