"""The callers on either side of the gather/scatter kernels, as the vLLM connector arranges them.

    generate_blocks_idx   TairKvCacheConnector.generate_blocks_idx  kv_cache_manager/py_connector/vllm/v1_connector.py:308-320
    generate_blocks_idx_host, HostBlockIndex   the same on the host, packed (for callers that work with Python lists)
    register_kv_caches    TairKvCacheConnector.register_kv_caches   kv_cache_manager/py_connector/vllm/v1_connector.py:360-445
    KVCacheInfo           kv_cache_manager/py_connector/common/types.py:9-23
    MultiResult           kv_cache_manager/py_connector/vllm/data_transfer.py:18-36
    DataTransferManager   kv_cache_manager/py_connector/vllm/data_transfer.py:39-278 (constructor :47-78, load_task
                          :108-158, create_load_done_callback :160-188, save_task :190-244,
                          create_save_done_callback :246-278)

What is not here: the engine plugin classes, the HTTP manager client and the ZMQ coordinator (control plane).
The transfer client is whatever object offers SaveKvCaches(uris, buffers) -> (code, uris) and
LoadKvCaches(uris, buffers) -> code (kv_cache_manager/client/include/transfer_client.h:19-21); the coordinator client
is whatever object offers send(bytes) (TpCoordinatorClient, kv_cache_manager/py_connector/common/tp_coordinator.py).
"""
import math
import threading
import time
from concurrent.futures import ThreadPoolExecutor
from dataclasses import dataclass
from typing import Any, Callable, Dict, List, Optional, Sequence, Tuple

import torch

from . import _lib, client_types, coordinator_messages
from ._torch_util import as_device_i32, lib, ptr, stream_handle
from .kernel import batch_gather_scatter_helper
from .kernel.gather_scatter_helper import CopyBufferAllocator


# How a worker thread waits for its copy: True = the thread sleeps until the event has happened (hipEventBlockingSync),
# False = it spins on the event as a plain torch.cuda.Event() does (the reference's). The connector keeps 32 worker
# threads; spinning, they occupy every host core a GPU has here (16) while the threads that have launches to issue wait
# for a core: 133-159 us per task of 128 blocks spinning against 124-132 us sleeping on a busy host, 97 against 100 us
# on an idle one.
_EVENT_BLOCKING = True
_blocks_idx_error_flags: Dict[Any, torch.Tensor] = {}
_blocks_idx_error_lock = threading.Lock()


def _default_error_flag(device: torch.device) -> torch.Tensor:
    """The int32 flag that generate_blocks_idx raises for tensor arguments when the caller passes none: one per
    device, created on first use, read and cleared by blocks_idx_error()."""
    key = (device.type, device.index if device.index is not None else torch.cuda.current_device())
    flag = _blocks_idx_error_flags.get(key)
    if flag is None:
        with _blocks_idx_error_lock:
            flag = _blocks_idx_error_flags.get(key)
            if flag is None:
                flag = torch.zeros(1, dtype=torch.int32, device=device)
                _blocks_idx_error_flags[key] = flag
    return flag


def blocks_idx_error(device="cuda", clear: bool = True) -> bool:
    """True when a generate_blocks_idx call with tensor arguments (and no error_flag of its own) on `device` has met a
    manager block that reaches beyond local_block_ids since the last call of this function. Reads the flag back, so
    it waits for the device: call it at a point where the caller waits anyway (DataTransferManager.save_task does,
    after the event it waits for and before the staged blocks are handed to the transfer client)."""
    device = torch.device(device)
    key = (device.type, device.index if device.index is not None else torch.cuda.current_device())
    flag = _blocks_idx_error_flags.get(key)
    if flag is None:
        return False
    raised = bool(flag.item())
    if raised and clear:
        flag.zero_()
    return raised


def generate_blocks_idx(manager_block_idxes: Sequence[int], local_block_ids: Sequence[int],
                        manager_block_size: int, local_block_size: int, device="cuda",
                        error_flag: Optional[torch.Tensor] = None) -> torch.Tensor:
    """int32 device tensor [B, manager_block_size]:
    out[b][i] = local_block_ids[tok // local_block_size] * local_block_size + tok % local_block_size with
    tok = manager_block_idxes[b] * manager_block_size + i. The reference builds this as nested Python lists;
    here it is one kernel and the result never visits the host.

    A manager block that reaches beyond local_block_ids: with Python sequences this raises AssertionError before
    anything is launched, as the reference's assert does. With tensor arguments nothing is read back (no
    synchronisation): the kernel writes -1 for such entries, which the gather/scatter kernels skip, and raises an
    int32 flag on the device to 1 -- `error_flag` if the caller passes one, otherwise a flag the module keeps per
    device, which blocks_idx_error() reads and clears. The error is never dropped: DataTransferManager.save_task looks
    at that flag before it lets the transfer client save what was gathered."""
    T_mgr, T_eng = int(manager_block_size), int(local_block_size)
    B = len(manager_block_idxes)
    out = torch.empty((B, T_mgr), dtype=torch.int32, device=device)
    if B == 0:
        return out
    if not isinstance(manager_block_idxes, torch.Tensor):
        lo, hi = min(manager_block_idxes), max(manager_block_idxes)
        if lo < 0 or (hi * T_mgr + T_mgr - 1) // T_eng >= len(local_block_ids):
            raise AssertionError("manager block reaches beyond local_block_ids")
    if error_flag is not None and (not error_flag.is_cuda or error_flag.dtype != torch.int32 or error_flag.numel() < 1):
        raise ValueError("error_flag must be an int32 tensor on the GPU")
    if error_flag is None and isinstance(manager_block_idxes, torch.Tensor):
        error_flag = _default_error_flag(out.device)
    m = as_device_i32(manager_block_idxes, out.device, "manager_block_idxes")
    l = as_device_i32(local_block_ids, out.device, "local_block_ids")
    rc = lib().kvcm_hip_generate_blocks_idx(ptr(m), B, ptr(l), l.numel(), T_mgr, T_eng, ptr(out), ptr(error_flag),
                                            stream_handle(out.device))
    _lib.check(rc, "kvcm_hip_generate_blocks_idx")
    return out


class HostBlockIndex:
    """Token slots of manager blocks, int32 [B][T] packed in host memory: what generate_blocks_idx_host returns. It
    slices by block like the nested list the reference's generate_blocks_idx returns (`blocks_idx[i:end]`,
    kv_cache_manager/py_connector/vllm/v1_connector.py:515), an integer index gives one block's list of slots, and the
    gather/scatter operators take it as it is (no conversion, no upload: the host-list entry points)."""
    __slots__ = ("packed_int32", "tokens_per_block")

    def __init__(self, packed_int32: bytes, tokens_per_block: int):
        self.packed_int32 = packed_int32
        self.tokens_per_block = int(tokens_per_block)

    def __len__(self):
        return len(self.packed_int32) // (4 * self.tokens_per_block)

    def __getitem__(self, key):
        row = 4 * self.tokens_per_block
        if isinstance(key, slice):
            start, stop, step = key.indices(len(self))
            if step != 1:
                raise ValueError("a HostBlockIndex is sliced in steps of one block")
            return HostBlockIndex(self.packed_int32[start * row:max(start, stop) * row], self.tokens_per_block)
        b = key + len(self) if key < 0 else key
        if not 0 <= b < len(self):
            raise IndexError("block index out of range")
        return memoryview(self.packed_int32)[b * row:(b + 1) * row].cast("i").tolist()

    def tolist(self):
        return [self[b] for b in range(len(self))]


def generate_blocks_idx_host(manager_block_idxes: Sequence[int], local_block_ids: Sequence[int],
                             manager_block_size: int, local_block_size: int) -> HostBlockIndex:
    """generate_blocks_idx for callers that hold their block lists as Python lists and hand the result to
    DataTransferManager task by task, as the reference connector does (v1_connector.py:455,499-515): the same values
    as the reference's Python double loop (:308-320), computed in one C loop (2 us for 128 blocks of 16 tokens instead
    of 258 us) and kept packed, so that every task's slice goes to the host-list gather/scatter entry points as it is
    -- no device kernel, no upload, and whole-block tasks take the block-table form of the copy kernel.
    AssertionError when a manager block reaches beyond local_block_ids, like the reference's assert."""
    T_mgr, T_eng = int(manager_block_size), int(local_block_size)
    if T_mgr <= 0 or T_eng <= 0:
        raise ValueError("block sizes must be positive")
    c_loop = batch_gather_scatter_helper._blocks_idx_c
    if c_loop is not None and isinstance(manager_block_idxes, (list, tuple)) and \
            isinstance(local_block_ids, (list, tuple)):
        try:
            packed = c_loop(manager_block_idxes, local_block_ids, T_mgr, T_eng)
        except (TypeError, OverflowError) as e:
            raise ValueError(f"block lists must hold ints that fit 32 bits: {e}") from e
        if packed is None:
            raise AssertionError("manager block reaches beyond local_block_ids")
        return HostBlockIndex(packed, T_mgr)
    flat = []
    for m in manager_block_idxes:  # the reference's loop, for anything that is not a plain list
        for i in range(T_mgr):
            tok = int(m) * T_mgr + i
            assert 0 <= tok // T_eng < len(local_block_ids), "manager block reaches beyond local_block_ids"
            flat.append(int(local_block_ids[tok // T_eng]) * T_eng + tok % T_eng)
    packed = batch_gather_scatter_helper.pack_index_list(flat, "block indices")
    return HostBlockIndex(bytes(packed) if not isinstance(packed, bytes) else packed, T_mgr)


def generate_run_starts(manager_block_idxes: Sequence[int], local_block_ids: Sequence[int],
                        manager_block_size: int, local_block_size: int, device="cuda"):
    """Block-table form of generate_blocks_idx: (run_start [B, manager_block_size // g], g) with
    g = gcd(manager_block_size, local_block_size). A run of g tokens that starts at a multiple of g never
    crosses an engine block, so run_start[b][j] = generate_blocks_idx(...)[b][j * g] describes the same rows."""
    T_mgr, T_eng = int(manager_block_size), int(local_block_size)
    g = math.gcd(T_mgr, T_eng)
    groups = generate_blocks_idx(manager_block_idxes, local_block_ids, T_mgr // g, T_eng // g, device)
    return groups * g, g


@dataclass(frozen=True)
class KVCacheInfo:
    """What register_kv_caches derives from the engine's cache tensors: the reference's value class, same field names
    and positional order (kv_cache_manager/py_connector/common/types.py:9-23; built positionally at
    kv_cache_manager/py_connector/vllm/v1_connector.py:416-430)."""
    tp_rank: int
    world_size: int
    kvcaches: Dict[str, torch.Tensor]
    kvcache_ptr_tensor_cpu: torch.Tensor
    kvcache_ptr_tensor_gpu: torch.Tensor
    all_kvcache_ptr_tensor_gpu: torch.Tensor
    layer_num: int
    local_token_num: int
    per_manager_block_shape: Tuple[int, ...]
    per_manager_block_byte_size: int
    per_token_per_layer_dim_size: int
    device: torch.device
    dtype: torch.dtype


def register_kv_caches(kv_caches: Dict[str, torch.Tensor], manager_block_size: int, local_block_size: int,
                       use_mla: bool = False, tp_rank: int = 0, world_size: int = 1) -> KVCacheInfo:
    """Pointer tables and staging geometry for per-layer caches [2, block_num, block_size, kv_heads, head_dim]
    (MLA: [block_num, block_size, latent_dim], one pointer per layer).

    Order of the pointer table: layer-major, K before V (v1_connector.py:405-413); staging slot shape
    [layers, 2, manager_block_size, kv_heads * head_dim] (:376-388) whose byte size is the location-spec size
    the manager and the storage backends use as the per-block file stride."""
    if len(kv_caches) == 0:
        raise ValueError("kv_caches is empty")
    first = next(iter(kv_caches.values()))
    kv_dim = 1 if use_mla else 2
    tok_axis = 1 if use_mla else 2
    assert local_block_size == first.shape[tok_axis], "kv cache shape error"
    for t in kv_caches.values():
        assert t.is_contiguous(), "kv cache must be contiguous"
        assert t.shape == first.shape and t.dtype == first.dtype, "kv cache shape error"
    block_num = first.shape[tok_axis - 1]
    dim = math.prod(first.shape[tok_axis + 1:])
    itemsize = first.element_size()
    layer_shape = [kv_dim, manager_block_size, dim]
    row = first[0] if use_mla else first[0][0]  # [block_size, ...] of the first block
    assert dim * itemsize == row[1].data_ptr() - row[0].data_ptr(), "kv cache shape error"
    spec_shape = [len(kv_caches)] + layer_shape
    spec_bytes = math.prod(spec_shape) * itemsize
    names = list(kv_caches)
    ptr_cpu = torch.tensor([kv_caches[n].data_ptr() for n in names], dtype=torch.int64)
    if use_mla:
        all_ptrs = [kv_caches[n].data_ptr() for n in names]
    else:
        all_ptrs = []
        for n in names:
            all_ptrs.append(kv_caches[n][0].data_ptr())
            all_ptrs.append(kv_caches[n][1].data_ptr())
    device = first.device
    return KVCacheInfo(tp_rank, world_size, kv_caches, ptr_cpu, ptr_cpu.to(device),
                       torch.tensor(all_ptrs, dtype=torch.int64).to(device), len(kv_caches),
                       block_num * local_block_size, tuple(spec_shape), spec_bytes, dim, device, first.dtype)


class MultiResult:
    """Collects the results of `size` tasks and calls `callback(results)` once, from the thread that
    delivers the last one (data_transfer.py:18-36)."""

    def __init__(self, size: int, callback: Callable[[list], Any]):
        self._size = size
        self._results = [None] * size
        self._lock = threading.Lock()
        self._finished_num = 0
        self._finished_callback = callback

    def submit_result(self, idx: int, result):
        with self._lock:
            assert self._results[idx] is None
            self._results[idx] = result
            self._finished_num += 1
            done = self._finished_num == self._size
        if done:
            self._finished_callback(self._results)


class DataTransferManager:
    """save_task: wait for the KV cache -> gather blocks into staging slots -> hand the slots to the transfer
    client. load_task: let the transfer client fill staging slots -> scatter them into the KV cache.

    Stream/event choreography and failure behaviour follow data_transfer.py: one save and one load stream;
    the gather waits for `kvcache_ready_event`; the calling thread waits for the copy with an event, not a
    device-wide sync; when the client reports an error on load the scatter is NOT launched (:137-156); staging
    slots are always returned; every block of a task gets the task's result code.
    `block_token_indices` may be nested lists (as generate_blocks_idx returns in the reference), a flat list
    or an int32 tensor.
    """

    def __init__(self, kvcache_info: KVCacheInfo, manager_block_size: int,
                 copy_buffer_allocator: CopyBufferAllocator, transfer_client: Any,
                 coordinator_client: Any = None, extra_config: Any = None, *,
                 client_module: Any = client_types, message_module: Any = coordinator_messages,
                 max_workers: int = 32):
        """The six positional arguments are the reference's (data_transfer.py:47-53; call site
        kv_cache_manager/py_connector/vllm/v1_connector.py:435-442). Keyword-only extras: `client_module` supplies
        Iov / BlockBuffer / MemoryType / ClientErrorCode (the pybind module kvcm_py_client, or the plain-Python twin),
        `message_module` the coordinator message classes and their serialiser, `max_workers` the size of the I/O
        thread pool (32 in the reference, :89-93)."""
        self._kvcache_info = kvcache_info
        self._manager_block_size = manager_block_size
        self._copy_buffer_allocator = copy_buffer_allocator
        self._transfer_client = transfer_client
        self._coordinator_client = coordinator_client
        self._extra_config = extra_config
        self._cm = client_module
        self._mm = message_module
        device = kvcache_info.device

        def init_worker():
            torch.cuda.set_device(device)

        self._io_executor = ThreadPoolExecutor(max_workers=max_workers, thread_name_prefix="kvcm_io_",
                                               initializer=init_worker)
        # one save and one load stream (data_transfer.py:77-78), made when the first task needs them so that the
        # object, its callbacks and its result plumbing can be built and tested where there is no GPU
        self._stream_lock = threading.Lock()
        self._streams: Dict[str, Any] = {}
        self._slot_buffer_cache: Dict[int, Any] = {}
        self._tls = threading.local()

    def _stream(self, which: str):
        s = self._streams.get(which)
        if s is None:
            with self._stream_lock:
                s = self._streams.get(which)
                if s is None:
                    with torch.cuda.device(self._kvcache_info.device):
                        s = torch.cuda.Stream()
                    self._streams[which] = s
        return s

    @property
    def _save_stream(self):
        return self._stream("save")

    @property
    def _load_stream(self):
        return self._stream("load")

    def _thread_event(self):
        """The event a worker thread waits for its copy with: one per thread, recorded anew for every task (a thread
        has one task at a time)."""
        ev = getattr(self._tls, "event", None)
        if ev is None:
            ev = self._tls.event = torch.cuda.Event(blocking=_EVENT_BLOCKING)
        return ev

    def submit_task(self, func, *args, **kwargs):
        return self._io_executor.submit(func, *args, **kwargs)

    def shutdown(self):
        self._io_executor.shutdown(wait=True)

    @staticmethod
    def _flat_indices(block_token_indices):
        if isinstance(block_token_indices, (torch.Tensor, HostBlockIndex)):
            return block_token_indices
        if len(block_token_indices) > 0 and isinstance(block_token_indices[0], (list, tuple)):
            # nested, one list per block, as generate_blocks_idx returns it in the reference: packed in one C loop
            return batch_gather_scatter_helper.pack_index_list(block_token_indices, "block_token_indices")
        return block_token_indices

    def _slot_buffers(self, slot_indices):
        """One BlockBuffer of one Iov per staging slot (data_transfer.py:124-135,218-229). A slot's address and size
        never change, so its buffer object is built once and handed out again: building 128 Iov and BlockBuffer objects
        per task costs more interpreter time than everything else a task does on the host."""
        cache = self._slot_buffer_cache
        missing = [i for i in slot_indices if i not in cache]
        if missing:
            on_gpu = self._copy_buffer_allocator.device.type != "cpu"
            mem = self._cm.MemoryType.GPU if on_gpu else self._cm.MemoryType.CPU
            for i, slot in zip(missing, self._copy_buffer_allocator.get_buffer_by_idx(missing)):
                iov = self._cm.Iov()
                iov.type = mem
                iov.base = slot.data_ptr()
                iov.size = slot.numel() * slot.element_size()
                iov.ignore = False
                buf = self._cm.BlockBuffer()
                buf.iovs = [iov]
                cache[i] = buf  # a dict store is atomic; two threads that build the same slot build equal objects
        return [cache[i] for i in slot_indices]

    def load_task(self, multi_result: MultiResult, task_idx: int, remote_uris: List[str], block_token_indices):
        ok = self._cm.ClientErrorCode.ER_OK
        slots = self._copy_buffer_allocator.alloc_buffer_idx_blocking(len(remote_uris))
        try:
            result = self._transfer_client.LoadKvCaches(remote_uris, self._slot_buffers(slots))
            if result == ok:
                # launched on the load stream by handing the stream over, not by making it torch's current one:
                # entering a stream context and building an event object are interpreter time, which the worker
                # threads serialise
                stream = self._load_stream
                batch_gather_scatter_helper.batch_scatter_kv_caches(
                    self._kvcache_info.all_kvcache_ptr_tensor_gpu, self._copy_buffer_allocator._raw_buffer,
                    self._flat_indices(block_token_indices), slots, self._manager_block_size,
                    self._kvcache_info.per_token_per_layer_dim_size,
                    pool_token_slots=self._kvcache_info.local_token_num, stream=stream)
                done = self._thread_event()
                done.record(stream)
                done.synchronize()
        finally:
            self._copy_buffer_allocator.free_buffer(slots)
        multi_result.submit_result(task_idx, [result] * len(remote_uris))

    def create_load_done_callback(self, req_id, tp_rank, epoch, local_block_ids):
        """Callback for a MultiResult of load tasks (data_transfer.py:160-188): walks the per-block result codes of all
        tasks in order, collects local_block_ids[i] for every block i whose code is not ER_OK, and sends a
        LoadBlockFinishedEvent with that list to the coordinator."""
        ok = self._cm.ClientErrorCode.ER_OK

        def generate_message(task_results):
            failed_block_idxs = []
            idx = 0
            for task_result in task_results:
                for block_result in task_result:
                    if block_result != ok:
                        failed_block_idxs.append(local_block_ids[idx])
                    idx += 1
            event = self._mm.LoadBlockFinishedEvent(request_id=req_id, tp_rank=tp_rank, epoch=epoch,
                                                    failed_block_idxs=failed_block_idxs)
            self._send(self._mm.CoordinateMessage(time.time(), event))

        return generate_message

    def create_save_done_callback(self, req_id, tp_rank, write_session_id):
        """Callback for a MultiResult of save tasks (data_transfer.py:246-278): one success flag per block, in task
        order, sent to the coordinator as a SendBlockFinishedEvent."""
        ok = self._cm.ClientErrorCode.ER_OK

        def generate_message(task_results):
            is_successes = [block_result == ok for task_result in task_results for block_result in task_result]
            event = self._mm.SendBlockFinishedEvent(request_id=req_id, tp_rank=tp_rank,
                                                    write_session_id=write_session_id, is_success_list=is_successes)
            self._send(self._mm.CoordinateMessage(time.time(), event))

        return generate_message

    def _send(self, message):
        if self._coordinator_client is None:
            raise RuntimeError("DataTransferManager was built without a coordinator client: nothing to send to")
        self._coordinator_client.send(self._mm.CoordinateMsgSerializer.dumps(message))

    def save_task(self, multi_result: MultiResult, task_idx: int, remote_uris: List[str], block_token_indices,
                  kvcache_ready_event: Optional[torch.cuda.Event] = None):
        slots = None
        try:
            stream = self._save_stream
            if kvcache_ready_event is not None:
                kvcache_ready_event.wait(stream)
            slots = self._copy_buffer_allocator.alloc_buffer_idx_blocking(len(remote_uris))
            batch_gather_scatter_helper.batch_gather_kv_caches(
                self._kvcache_info.all_kvcache_ptr_tensor_gpu, self._copy_buffer_allocator._raw_buffer,
                self._flat_indices(block_token_indices), slots, self._manager_block_size,
                self._kvcache_info.per_token_per_layer_dim_size,
                pool_token_slots=self._kvcache_info.local_token_num, stream=stream)
            done = self._thread_event()
            done.record(stream)
            done.synchronize()
            if isinstance(block_token_indices, torch.Tensor) and block_token_indices.is_cuda and \
                    blocks_idx_error(block_token_indices.device):
                # indices built on the device named a block beyond the request's block list: those rows were skipped
                # by the gather, so the staged bytes are not the request's KV cache and must not be saved
                result = (self._cm.ClientErrorCode.ER_INVALID_PARAMS, [])
            else:
                result = self._transfer_client.SaveKvCaches(remote_uris, self._slot_buffers(slots))
        finally:
            if slots is not None:
                self._copy_buffer_allocator.free_buffer(slots)
        multi_result.submit_result(task_idx, [result[0]] * len(remote_uris))
