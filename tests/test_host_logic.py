"""Host-side mirror of the reference's Python interface: staging-slot pool, result fan-in, argument checks (no GPU)."""
import inspect
import threading
import time

import pytest
import torch

from tair_kvcache_amd.connector import MultiResult
from tair_kvcache_amd.kernel import batch_gather_scatter_helper as bgs
from tair_kvcache_amd.kernel import gather_scatter_helper as gsh
from tair_kvcache_amd.kernel.gather_scatter_helper import CopyBufferAllocator


def test_allocator_shape_and_zero_fill():
    a = CopyBufferAllocator(torch.device("cpu"), torch.bfloat16, [4, 2, 16, 8], 6)
    assert a._raw_buffer.shape == (6, 4, 2, 16, 8) and a.shape == (4, 2, 16, 8)
    assert not a._raw_buffer.any()
    assert a.slot_nbytes == 4 * 2 * 16 * 8 * 2


def test_allocator_takes_from_the_tail_and_validates():
    a = CopyBufferAllocator(torch.device("cpu"), torch.float16, [2], 8)
    assert a.alloc_buffer_idx_blocking(3) == [5, 6, 7]  # gather_scatter_helper.py:224-225
    assert a.alloc_buffer_idx_blocking(2) == [3, 4]
    bufs = a.get_buffer_by_idx([3, 7])
    assert bufs[0].data_ptr() == a._raw_buffer[3].data_ptr() and bufs[1].data_ptr() == a._raw_buffer[7].data_ptr()
    a.free_buffer([6, 3])
    assert a.alloc_buffer_idx_blocking(2) == [6, 3]
    for bad in (0, -1):
        with pytest.raises(ValueError):
            a.alloc_buffer_idx_blocking(bad)
    with pytest.raises(ValueError):
        a.alloc_buffer_idx_blocking(9)
    with pytest.raises(ValueError):
        a.free_buffer([8])
    with pytest.raises(ValueError):
        a.free_buffer([-1])
    a.free_buffer([])  # no-op
    a.free_buffer([5, 6, 7, 3, 4])
    with pytest.raises(RuntimeError):
        a.free_buffer([0])
    with pytest.raises(ValueError):
        CopyBufferAllocator(torch.device("cpu"), torch.float16, [2], 0)


def test_allocator_blocks_until_slots_return():
    a = CopyBufferAllocator(torch.device("cpu"), torch.float16, [2], 4)
    first = a.alloc_buffer_idx_blocking(3)
    got = []

    def waiter():
        got.append(a.alloc_buffer_idx_blocking(3))

    t = threading.Thread(target=waiter)
    t.start()
    time.sleep(0.2)
    assert not got and t.is_alive()  # 1 free < 3 wanted
    a.free_buffer(first[:1])
    time.sleep(0.2)
    assert not got  # 2 free, still waiting
    a.free_buffer(first[1:])
    t.join(5)
    assert not t.is_alive() and len(got[0]) == 3 and len(set(got[0])) == 3


def test_allocator_many_threads_never_oversubscribe():
    a = CopyBufferAllocator(torch.device("cpu"), torch.float16, [2], 16)
    in_use = set()
    lock = threading.Lock()
    errors = []

    def worker(seed):
        for i in range(50):
            n = 1 + (seed + i) % 5
            idx = a.alloc_buffer_idx_blocking(n)
            with lock:
                if in_use & set(idx):
                    errors.append("slot handed out twice")
                in_use.update(idx)
            with lock:
                in_use.difference_update(idx)
            a.free_buffer(idx)

    ts = [threading.Thread(target=worker, args=(s,)) for s in range(8)]
    [t.start() for t in ts]
    [t.join(30) for t in ts]
    assert not errors and a._inuse_count == 0 and sorted(a._free_idx_list) == list(range(16))


def test_multi_result_calls_back_once_with_all_results():
    seen = []
    m = MultiResult(3, seen.append)
    m.submit_result(2, ["c"])
    m.submit_result(0, ["a"])
    assert not seen
    m.submit_result(1, ["b"])
    assert seen == [[["a"], ["b"], ["c"]]]
    with pytest.raises(AssertionError):
        m.submit_result(1, ["again"])


def test_operators_reject_host_tensors_before_touching_the_device():
    ptrs = torch.zeros(4, dtype=torch.int64)
    st = torch.zeros(2, 4, 16, 8, dtype=torch.float16)
    with pytest.raises(ValueError):
        bgs.batch_gather_kv_caches(ptrs, st, [0] * 32, [0, 1], 16, 8)
    with pytest.raises(ValueError):
        bgs.batch_scatter_kv_caches(ptrs, st, [0] * 32, [0, 1], 16, 8)
    with pytest.raises(ValueError):
        gsh.gather_kv_caches(ptrs, 128, torch.zeros(4, 2, 16, 8), list(range(16)))


def test_signatures_match_the_reference_operators():
    import inspect
    def positional(sig):  # what a reference call site can reach; extras of this port are keyword-only
        return [n for n, p in sig.parameters.items() if p.kind is not inspect.Parameter.KEYWORD_ONLY]

    sig = inspect.signature(bgs.batch_gather_kv_caches)
    assert positional(sig) == ["kv_caches_ptrs_tensor", "dst_tensor", "block_token_indices", "dst_block_indices",
                               "num_tokens_per_block", "dim_size_per_token_per_layer", "sm_count"]
    assert sig.parameters["sm_count"].default == 3
    assert sig.parameters["pool_token_slots"].default == 0
    sig = inspect.signature(bgs.batch_scatter_kv_caches)
    assert positional(sig) == ["kv_caches_ptrs_tensor", "src_tensor", "block_token_indices", "src_block_indices",
                               "num_tokens_per_block", "dim_size_per_token_per_layer", "sm_count"]
    assert list(inspect.signature(gsh.gather_kv_caches).parameters) == ["kv_caches_ptrs", "total_token_in_kvcache",
                                                                         "dst_tensor", "token_indices"]
    assert list(inspect.signature(gsh.scatter_kv_caches).parameters) == ["kv_caches_ptrs", "total_token_in_kvcache",
                                                                          "src_tensor", "token_indices"]
    assert list(inspect.signature(CopyBufferAllocator.__init__).parameters) == ["self", "device", "dtype", "shape",
                                                                                "max_count"]


def _vllm_caches(L=3, nblk=8, T=16, H=2, hd=64, dtype=torch.float16):
    return {f"model.layers.{l}.attn": torch.zeros(2, nblk, T, H, hd, dtype=dtype) for l in range(L)}


def test_register_kv_caches_pointer_order_and_spec_size():
    # v1_connector.py:360-445: layer-major, K before V; slot shape [layers, 2, manager_block, heads*dim]
    from tair_kvcache_amd import connector
    kv = _vllm_caches()
    info = connector.register_kv_caches(kv, manager_block_size=64, local_block_size=16, tp_rank=1, world_size=2)
    want = []
    for t in kv.values():
        want += [t[0].data_ptr(), t[1].data_ptr()]
    assert info.all_kvcache_ptr_tensor_gpu.tolist() == want
    assert info.kvcache_ptr_tensor_cpu.tolist() == [t.data_ptr() for t in kv.values()]
    assert info.per_manager_block_shape == (3, 2, 64, 128)
    assert info.per_manager_block_byte_size == 3 * 2 * 64 * 128 * 2
    assert info.per_token_per_layer_dim_size == 128 and info.local_token_num == 8 * 16
    assert (info.layer_num, info.tp_rank, info.world_size, info.dtype) == (3, 1, 2, torch.float16)
    # V of a layer sits block_num * block_size rows after K: the legacy [2, total, H] view of the same tensor
    assert want[1] - want[0] == 8 * 16 * 128 * 2


def test_register_kv_caches_mla_one_pointer_per_layer():
    from tair_kvcache_amd import connector
    kv = {f"l{l}": torch.zeros(32, 128, 576, dtype=torch.uint8) for l in range(4)}
    info = connector.register_kv_caches(kv, manager_block_size=128, local_block_size=128, use_mla=True)
    assert info.all_kvcache_ptr_tensor_gpu.tolist() == [t.data_ptr() for t in kv.values()]
    assert info.per_manager_block_shape == (4, 1, 128, 576)
    assert info.per_manager_block_byte_size == 4 * 128 * 576
    assert info.local_token_num == 32 * 128


def test_register_kv_caches_rejects_what_the_reference_asserts_on():
    from tair_kvcache_amd import connector
    kv = _vllm_caches()
    with pytest.raises(AssertionError):  # engine block size mismatch (v1_connector.py:365)
        connector.register_kv_caches(kv, 16, 32)
    bad = dict(kv)
    bad["x"] = torch.zeros(2, 8, 16, 2, 128, dtype=torch.float16)[..., :64]  # not contiguous (:367)
    with pytest.raises(AssertionError):
        connector.register_kv_caches(bad, 16, 16)
    with pytest.raises(ValueError):
        connector.register_kv_caches({}, 16, 16)


def test_generate_blocks_idx_bounds_check_runs_on_the_host():
    # the reference asserts per token (v1_connector.py:315); here the same condition is checked before any launch
    from tair_kvcache_amd import connector
    with pytest.raises(AssertionError):
        connector.generate_blocks_idx([4], [0, 1, 2, 3], 64, 16, device="cpu")  # tokens 256..319 need block 16
    with pytest.raises(AssertionError):
        connector.generate_blocks_idx([-1], [0, 1, 2, 3], 16, 16, device="cpu")
    assert connector.generate_blocks_idx([], [0], 16, 16, device="cpu").shape == (0, 16)


class _FakeCoordinator:
    """Stands in for TpCoordinatorClient (kv_cache_manager/py_connector/common/tp_coordinator.py): keeps what it is sent."""

    def __init__(self):
        self.sent = []

    def send(self, data):
        assert isinstance(data, bytes)
        self.sent.append(data)


class _ExtraConfig:
    block_per_save_task = 128
    block_per_load_task = 2


def _manager_as_the_connector_builds_it(coordinator):
    """register_kv_caches' tail, v1_connector.py:416-442: KVCacheInfo and DataTransferManager, all arguments positional."""
    from tair_kvcache_amd import connector
    from tair_kvcache_amd.kernel.gather_scatter_helper import CopyBufferAllocator
    kv = _vllm_caches()
    ptrs = torch.tensor([t.data_ptr() for t in kv.values()], dtype=torch.int64)
    all_ptrs = torch.tensor([p for t in kv.values() for p in (t[0].data_ptr(), t[1].data_ptr())], dtype=torch.int64)
    shape = [3, 2, 16, 128]
    info = connector.KVCacheInfo(1, 2, kv, ptrs, ptrs, all_ptrs, len(kv), 8 * 16, tuple(shape), 3 * 2 * 16 * 128 * 2, 128,
                                 torch.device("cpu"), torch.float16)
    alloc = CopyBufferAllocator(torch.device("cpu"), torch.float16, shape, 4)
    transfer_client = object()
    mgr = connector.DataTransferManager(info, 16, alloc, transfer_client, coordinator, _ExtraConfig())
    return info, mgr


def test_kvcache_info_is_the_reference_value_class():
    # kv_cache_manager/py_connector/common/types.py:9-23: names, order, frozen
    import dataclasses
    from tair_kvcache_amd import connector
    assert [f.name for f in dataclasses.fields(connector.KVCacheInfo)] == [
        "tp_rank", "world_size", "kvcaches", "kvcache_ptr_tensor_cpu", "kvcache_ptr_tensor_gpu",
        "all_kvcache_ptr_tensor_gpu", "layer_num", "local_token_num", "per_manager_block_shape",
        "per_manager_block_byte_size", "per_token_per_layer_dim_size", "device", "dtype"]
    info, _ = _manager_as_the_connector_builds_it(_FakeCoordinator())
    with pytest.raises(dataclasses.FrozenInstanceError):
        info.tp_rank = 0


def test_data_transfer_manager_takes_the_reference_constructor_call():
    # data_transfer.py:47-53 and its call at v1_connector.py:435-442
    from tair_kvcache_amd import connector
    params = list(inspect.signature(connector.DataTransferManager.__init__).parameters.values())
    assert [p.name for p in params[:7]] == ["self", "kvcache_info", "manager_block_size", "copy_buffer_allocator",
                                            "transfer_client", "coordinator_client", "extra_config"]
    assert all(p.kind is inspect.Parameter.KEYWORD_ONLY for p in params[7:])
    coord = _FakeCoordinator()
    info, mgr = _manager_as_the_connector_builds_it(coord)
    assert mgr._coordinator_client is coord and isinstance(mgr._extra_config, _ExtraConfig)
    assert mgr._kvcache_info is info and mgr._manager_block_size == 16
    assert list(inspect.signature(mgr.create_load_done_callback).parameters) == ["req_id", "tp_rank", "epoch",
                                                                                 "local_block_ids"]
    assert list(inspect.signature(mgr.create_save_done_callback).parameters) == ["req_id", "tp_rank", "write_session_id"]
    mgr.shutdown()


def test_load_done_callback_reports_failed_local_blocks_like_start_load_kv():
    """The loop of start_load_kv (v1_connector.py:448-475) with block_per_load_task = 2 over five blocks: three tasks,
    the second one fails => the local block ids at positions 2 and 3 are reported (data_transfer.py:172-186)."""
    import copy
    import json
    import math
    from tair_kvcache_amd import client_types as ct, connector, coordinator_messages as cm
    coord = _FakeCoordinator()
    info, mgr = _manager_as_the_connector_builds_it(coord)
    local_block_ids = [40, 41, 42, 43, 44]
    block_token_indices = [[b * 16 + i for i in range(16)] for b in local_block_ids]
    per_task_size = mgr._extra_config.block_per_load_task
    task_num = math.ceil(len(block_token_indices) / per_task_size)
    done_callback = mgr.create_load_done_callback("req-7", info.tp_rank, 3, copy.copy(local_block_ids))
    multi_result = connector.MultiResult(task_num, done_callback)
    codes = [ct.ClientErrorCode.ER_OK, ct.ClientErrorCode.ER_SDKREAD_ERROR, ct.ClientErrorCode.ER_OK]
    task_idx = 0
    for i in range(0, len(block_token_indices), per_task_size):
        end_idx = min(len(block_token_indices), i + per_task_size)
        # what load_task submits: the task's code once per block of the task (data_transfer.py:158)
        assert not coord.sent
        multi_result.submit_result(task_idx, [codes[task_idx]] * (end_idx - i))
        task_idx += 1
    assert len(coord.sent) == 1
    msg = cm.CoordinateMsgSerializer.loads(coord.sent[0])
    assert isinstance(msg.content, cm.LoadBlockFinishedEvent)
    assert (msg.content.request_id, msg.content.tp_rank, msg.content.epoch) == ("req-7", 1, 3)
    assert msg.content.failed_block_idxs == [42, 43]
    wire = json.loads(coord.sent[0])
    assert list(wire) == ["send_time", "content", "create_time"]
    assert list(wire["content"]) == ["request_id", "tp_rank", "epoch", "failed_block_idxs", "type"]
    assert wire["content"]["type"] == "LoadBlockFinishedEvent"
    mgr.shutdown()


def test_save_done_callback_reports_one_flag_per_block_like_wait_for_save():
    """wait_for_save's loop (v1_connector.py:486-519): 300 blocks in tasks of 128 => three tasks; the last one fails."""
    import json
    import math
    from tair_kvcache_amd import client_types as ct, connector, coordinator_messages as cm
    coord = _FakeCoordinator()
    info, mgr = _manager_as_the_connector_builds_it(coord)
    n = 300
    per_task_size = mgr._extra_config.block_per_save_task
    task_num = math.ceil(n / per_task_size)
    multi_result = connector.MultiResult(task_num, mgr.create_save_done_callback("req-9", info.tp_rank, "ws-1"))
    # tasks finish out of order on the 32-thread pool
    for task_idx in (2, 0, 1):
        size = min(n, (task_idx + 1) * per_task_size) - task_idx * per_task_size
        code = ct.ClientErrorCode.ER_SDKWRITE_ERROR if task_idx == 2 else ct.ClientErrorCode.ER_OK
        multi_result.submit_result(task_idx, [code] * size)
    assert len(coord.sent) == 1
    msg = cm.CoordinateMsgSerializer.loads(coord.sent[0])
    assert isinstance(msg.content, cm.SendBlockFinishedEvent)
    assert (msg.content.request_id, msg.content.tp_rank, msg.content.write_session_id) == ("req-9", 1, "ws-1")
    assert msg.content.is_success_list == [True] * 256 + [False] * 44
    wire = json.loads(coord.sent[0])
    assert list(wire["content"]) == ["request_id", "tp_rank", "write_session_id", "is_success_list", "remote_uris", "type"]
    assert wire["content"]["remote_uris"] == [] and msg.send_time <= msg.create_time + 1.0
    mgr.shutdown()


def test_done_callback_without_a_coordinator_says_so():
    from tair_kvcache_amd import connector
    from tair_kvcache_amd.kernel.gather_scatter_helper import CopyBufferAllocator
    info, _ = _manager_as_the_connector_builds_it(_FakeCoordinator())
    mgr = connector.DataTransferManager(info, 16, CopyBufferAllocator(torch.device("cpu"), torch.float16, [1], 1), object())
    with pytest.raises(RuntimeError):
        mgr.create_save_done_callback("r", 0, "w")([[0]])
    mgr.shutdown()


def test_hashing_and_buffer_check_reject_bad_arguments_before_any_launch():
    from tair_kvcache_amd import buffer_check, hashing
    with pytest.raises(ValueError):
        hashing.hash_tokens(torch.zeros(2, 32, dtype=torch.int64), 16)             # tokens not on the GPU
    with pytest.raises(ValueError):
        hashing.apply_prefix_hash(torch.zeros(8, dtype=torch.int64))
    with pytest.raises(ValueError):   # an iov shorter than the bytes taken from the first iov's size
        buffer_check.get_iovs_crc([(0x1000, 64), (0x2000, 3)], device="cpu")
    with pytest.raises(ValueError):   # an iov without an address
        buffer_check.get_iovs_crc([(0x1000, 64), (0, 64)], device="cpu")
    assert buffer_check.get_iovs_crc([(0x1000, 1)], device="cpu") == []            # size 1 -> nothing to hash


def test_index_lists_are_packed_in_c_flat_and_nested():
    """pack_index_list: the C helper and the array('i') path it replaces give the same bytes; what is not an integer
    that fits 32 bits is refused with ValueError either way."""
    from array import array
    import numpy as np
    assert bgs._pack_i32 is not None, "tair_kvcache_amd/_kvcm_pylist is not built (python -m tair_kvcache_amd.build)"
    flat = [(i * 7919) % 500000 - 3 for i in range(2048)]
    nested = [flat[i * 16:(i + 1) * 16] for i in range(128)]
    want = array("i", flat).tobytes()
    for form in (flat, tuple(flat), nested, [tuple(r) for r in nested], tuple(nested)):
        assert bgs.pack_index_list(form) == want
    assert bgs.pack_index_list([np.int64(5), True, -2 ** 31, 2 ** 31 - 1]) == array("i", [5, 1, -2 ** 31, 2 ** 31 - 1]).tobytes()
    assert bgs.pack_index_list([]) == b"" and bgs.pack_index_list([[], []]) == b""
    for bad in ([1.5], [2 ** 31], [-2 ** 31 - 1], ["7"], [[1], 2], [None], [[1.0]]):
        with pytest.raises(ValueError):
            bgs.pack_index_list(bad)
    # the same without the C helper
    helper, bgs._pack_i32 = bgs._pack_i32, None
    try:
        assert bytes(bgs.pack_index_list(flat)) == want and bgs.pack_index_list(nested).tobytes() == want
        assert bgs.pack_index_list(range(5)).tolist() == [0, 1, 2, 3, 4]
        for bad in ([1.5], [2 ** 31], ["7"], [[1], 2]):
            with pytest.raises(ValueError):
                bgs.pack_index_list(bad)
    finally:
        bgs._pack_i32 = helper


def test_generate_blocks_idx_host_equals_the_reference_loop(oracle):
    """generate_blocks_idx_host: the values of the reference's Python double loop (v1_connector.py:308-320) and of the
    oracle, for manager blocks smaller than, equal to and larger than engine blocks; slices by block like the nested
    list the reference returns; asserts like the reference when a manager block reaches beyond the block list."""
    import numpy as np
    from tair_kvcache_amd import connector

    def reference_loop(manager_block_idxes, local_block_ids, T_mgr, T_eng):
        blocks_idx = []
        for m in manager_block_idxes:
            row = []
            for i in range(T_mgr):
                tok = m * T_mgr + i
                assert tok // T_eng < len(local_block_ids)
                row.append(local_block_ids[tok // T_eng] * T_eng + tok % T_eng)
            blocks_idx.append(row)
        return blocks_idx

    rng = np.random.default_rng(3)
    for T_mgr, T_eng in ((16, 16), (64, 16), (16, 64), (24, 16), (1, 1), (128, 128)):
        local = rng.permutation(5000)[:300].tolist()
        n_mgr = len(local) * T_eng // T_mgr
        mgr = rng.integers(0, n_mgr, size=77).tolist()
        want = reference_loop(mgr, local, T_mgr, T_eng)
        got = connector.generate_blocks_idx_host(mgr, local, T_mgr, T_eng)
        assert len(got) == 77 and got.tolist() == want
        idx, bad = oracle.generate_blocks_idx(np.array(mgr, dtype=np.int32), np.array(local, dtype=np.int32), T_mgr, T_eng)
        assert bad == 0 and idx.tolist() == want
        assert got[10:20].tolist() == want[10:20] and got[5] == want[5] and got[-1] == want[-1]
        assert len(got[70:200]) == 7 and len(got[80:90]) == 0
        assert bgs._host_i32(got[3:9], "x")[1] == 6 * T_mgr
        # tuples, and anything that is not a plain list (the Python loop)
        assert connector.generate_blocks_idx_host(tuple(mgr), tuple(local), T_mgr, T_eng).tolist() == want
        assert connector.generate_blocks_idx_host(np.array(mgr), local, T_mgr, T_eng).tolist() == want
    with pytest.raises(AssertionError):
        connector.generate_blocks_idx_host([19], list(range(19)), 16, 16)
    with pytest.raises(AssertionError):
        connector.generate_blocks_idx_host([-1], list(range(19)), 16, 16)
    with pytest.raises(ValueError):
        connector.generate_blocks_idx_host([0], [2 ** 31], 16, 16)
    with pytest.raises(ValueError):
        connector.generate_blocks_idx_host([0], [1.5], 16, 16)
    with pytest.raises(ValueError):
        connector.generate_blocks_idx_host([0], [2 ** 30], 16, 16)  # the slot itself does not fit 32 bits
    assert len(connector.generate_blocks_idx_host([], [1, 2], 16, 16)) == 0
