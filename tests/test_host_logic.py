"""Host-side mirror of the reference's Python interface: staging-slot pool, result fan-in, argument checks (no GPU)."""
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
    sig = inspect.signature(bgs.batch_gather_kv_caches)
    assert list(sig.parameters) == ["kv_caches_ptrs_tensor", "dst_tensor", "block_token_indices", "dst_block_indices",
                                    "num_tokens_per_block", "dim_size_per_token_per_layer", "sm_count"]
    assert sig.parameters["sm_count"].default == 3
    sig = inspect.signature(bgs.batch_scatter_kv_caches)
    assert list(sig.parameters) == ["kv_caches_ptrs_tensor", "src_tensor", "block_token_indices", "src_block_indices",
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
    info = connector.register_kv_caches(kv, manager_block_size=64, local_block_size=16, tp_rank=1, tp_size=2)
    want = []
    for t in kv.values():
        want += [t[0].data_ptr(), t[1].data_ptr()]
    assert info.all_kvcache_ptr_tensor_gpu.tolist() == want
    assert info.kvcache_ptr_tensor_cpu.tolist() == [t.data_ptr() for t in kv.values()]
    assert info.per_manager_location_spec_shape == (3, 2, 64, 128)
    assert info.per_manager_location_spec_byte_size == 3 * 2 * 64 * 128 * 2
    assert info.per_token_per_layer_dim_size == 128 and info.local_token_num == 8 * 16
    assert (info.layer_num, info.tp_rank, info.tp_size, info.dtype) == (3, 1, 2, torch.float16)
    # V of a layer sits block_num * block_size rows after K: the legacy [2, total, H] view of the same tensor
    assert want[1] - want[0] == 8 * 16 * 128 * 2


def test_register_kv_caches_mla_one_pointer_per_layer():
    from tair_kvcache_amd import connector
    kv = {f"l{l}": torch.zeros(32, 128, 576, dtype=torch.uint8) for l in range(4)}
    info = connector.register_kv_caches(kv, manager_block_size=128, local_block_size=128, use_mla=True)
    assert info.all_kvcache_ptr_tensor_gpu.tolist() == [t.data_ptr() for t in kv.values()]
    assert info.per_manager_location_spec_shape == (4, 1, 128, 576)
    assert info.per_manager_location_spec_byte_size == 4 * 128 * 576
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
