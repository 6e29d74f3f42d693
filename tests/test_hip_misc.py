"""GPU parity: buffer check (iov CRC + block fold) and the save/load choreography around the kernels."""
import threading
import zlib

import numpy as np
import pytest
import torch

import _cases as cases
from _gpu import dev, host, ptr_table, sync

pytestmark = pytest.mark.gpu


def test_iov_crc_reference_known_answers():
    # kv_cache_manager/client/src/internal/sdk/test/sdk_buffer_check_util_test.cc:13-74
    from tair_kvcache_amd import buffer_check as bc
    s = torch.frombuffer(bytearray(b"1234xxxxxxxx5678"), dtype=torch.uint8).cuda()
    assert bc.get_iovs_crc([(s.data_ptr(), 16)], cal_byte_size=8) == [0xDE28307C]
    assert bc.get_iovs_crc([(s.data_ptr(), 16)], cal_byte_size=4) == [0x9AE0DAAF]
    s2 = torch.frombuffer(bytearray(b"1278"), dtype=torch.uint8).cuda()
    assert bc.get_iovs_crc([(s2.data_ptr(), 4)], cal_byte_size=4) == [0xF639698C]
    s3 = torch.frombuffer(bytearray(b"1"), dtype=torch.uint8).cuda()
    assert bc.get_iovs_crc([(s3.data_ptr(), 1)], cal_byte_size=4) == []


def test_iov_crc_and_block_hash_match_oracle(oracle):
    from tair_kvcache_amd import buffer_check as bc
    rng = np.random.default_rng(8)
    data = rng.integers(0, 256, size=(6, 4, 1024), dtype=np.uint8)  # 6 blocks x 4 iovs
    d = dev(data)
    blocks = [[(d[b, i].data_ptr(), 1024) for i in range(4)] for b in range(6)]
    flat = [iov for bb in blocks for iov in bb]
    crcs = bc.get_iovs_crc(flat)
    want = [zlib.crc32(data[b, i, :4].tobytes() + data[b, i, -4:].tobytes()) for b in range(6) for i in range(4)]
    assert crcs == want
    assert crcs == oracle.iov_crc32([data[b, i] for b in range(6) for i in range(4)], 4).tolist()
    hashes = bc.get_blocks_hash(blocks)
    assert hashes == oracle.blocks_hash_from_crcs(np.array(want, dtype=np.uint32), 4).tolist()
    assert len(bc.get_blocks_hash(blocks, max_iov_num=10)) == 2  # whole blocks only (.cc:43-47)
    same = bc.get_blocks_hash([blocks[0], blocks[0]])
    assert same[0] == same[1]


class FakeTransferClient:
    """Keeps blocks in a dict keyed by URI; stands in for TransferClient (transfer_client.h:19-21)."""

    def __init__(self, fail_load=False, fail_save=False):
        self.store = {}
        self.fail_load = fail_load
        self.fail_save = fail_save
        self.lock = threading.Lock()

    def SaveKvCaches(self, uris, buffers):
        from tair_kvcache_amd.client_types import ClientErrorCode
        if len(uris) != len(buffers) or not uris:
            return (ClientErrorCode.ER_INVALID_PARAMS, [])
        if self.fail_save:
            return (ClientErrorCode.ER_SDKWRITE_ERROR, [])
        import ctypes
        with self.lock:
            for uri, buf in zip(uris, buffers):
                iov = buf.iovs[0]
                self.store[uri] = ctypes.string_at(iov.base, iov.size)
        return (ClientErrorCode.ER_OK, list(uris))

    def LoadKvCaches(self, uris, buffers):
        from tair_kvcache_amd.client_types import ClientErrorCode
        if self.fail_load:
            return ClientErrorCode.ER_SDKREAD_ERROR
        import ctypes
        for uri, buf in zip(uris, buffers):
            iov = buf.iovs[0]
            ctypes.memmove(iov.base, self.store[uri], iov.size)
        return ClientErrorCode.ER_OK


def test_save_then_load_through_the_transfer_manager(oracle):
    """register_kv_caches -> generate_blocks_idx -> save_task (gather + client) -> load_task (client + scatter) on
    vLLM-shaped caches [2, blocks, block_size, heads, dim]; stored bytes equal the oracle's staging layout."""
    from tair_kvcache_amd import connector
    from tair_kvcache_amd.client_types import ClientErrorCode
    from tair_kvcache_amd.kernel.gather_scatter_helper import CopyBufferAllocator
    L, nblk, T, H, hd = 4, 64, 16, 2, 64
    rng = np.random.default_rng(1)
    np_caches = [rng.integers(0, 65536, size=(2, nblk, T, H, hd), dtype=np.uint16) for _ in range(L)]
    kv = {f"layer{l}": dev(np_caches[l]).view(torch.bfloat16) for l in range(L)}
    info = connector.register_kv_caches(kv, manager_block_size=T, local_block_size=T)
    assert info.per_manager_block_shape == (L, 2, T, H * hd)
    assert info.per_manager_block_byte_size == L * 2 * T * H * hd * 2
    assert info.all_kvcache_ptr_tensor_gpu.tolist() == [x for l in range(L) for x in
                                                        (kv[f"layer{l}"][0].data_ptr(), kv[f"layer{l}"][1].data_ptr())]
    alloc = CopyBufferAllocator(torch.device("cpu"), torch.bfloat16, list(info.per_manager_block_shape), 32)
    client = FakeTransferClient()
    mgr = connector.DataTransferManager(info, T, alloc, client, max_workers=4)
    local_block_ids = cases.block_table(nblk, 24).tolist()
    manager_blocks = list(range(24))
    idx = connector.generate_blocks_idx(manager_blocks, local_block_ids, T, T)
    sync()
    idx_h = host(idx, np.int32)
    done = threading.Event()
    results = []
    multi = connector.MultiResult(2, lambda r: (results.append(r), done.set()))
    ready = torch.cuda.Event()
    ready.record()
    uris = [f"file:///kv/blk?blkid={i}&size={info.per_manager_block_byte_size}" for i in range(24)]
    mgr.submit_task(mgr.save_task, multi, 0, uris[:12], idx_h[:12].tolist(), ready)
    mgr.submit_task(mgr.save_task, multi, 1, uris[12:], idx[12:], ready)
    assert done.wait(60)
    assert results[0] == [[ClientErrorCode.ER_OK] * 12] * 2
    assert alloc._inuse_count == 0
    # stored bytes = oracle staging
    pools = [np_caches[l][kvi].reshape(nblk * T, H * hd) for l in range(L) for kvi in (0, 1)]
    want = np.zeros((24, 2 * L, T, H * hd), dtype=np.uint16)
    oracle.batch_gather(pools, want, idx_h, None, T, H * hd * 2)
    for i, uri in enumerate(uris):
        assert client.store[uri] == want[i].tobytes()
    # load into zeroed caches
    kv2 = {k: torch.zeros_like(v) for k, v in kv.items()}
    info2 = connector.register_kv_caches(kv2, T, T)
    mgr2 = connector.DataTransferManager(info2, T, alloc, client, max_workers=4)
    done2 = threading.Event()
    res2 = []
    multi2 = connector.MultiResult(1, lambda r: (res2.append(r), done2.set()))
    mgr2.submit_task(mgr2.load_task, multi2, 0, uris, idx_h.tolist())
    assert done2.wait(60)
    assert res2[0] == [[ClientErrorCode.ER_OK] * 24]
    touched = np.array(local_block_ids)
    rest = np.setdiff1d(np.arange(nblk), touched)
    for l in range(L):
        g = host(kv2[f"layer{l}"].view(torch.int16), np.uint16)
        assert (g[:, touched] == np_caches[l][:, touched]).all()
        assert not g[:, rest].any()
    # a failed load launches no scatter and still returns the slots
    kv3 = {k: torch.zeros_like(v) for k, v in kv.items()}
    mgr3 = connector.DataTransferManager(connector.register_kv_caches(kv3, T, T), T, alloc,
                                         FakeTransferClient(fail_load=True), max_workers=2)
    done3 = threading.Event()
    res3 = []
    mgr3.submit_task(mgr3.load_task, connector.MultiResult(1, lambda r: (res3.append(r), done3.set())), 0, uris[:4],
                     idx_h[:4].tolist())
    assert done3.wait(60)
    assert res3[0] == [[ClientErrorCode.ER_SDKREAD_ERROR] * 4] and alloc._inuse_count == 0
    sync()
    assert all(not v.view(torch.int16).any() for v in kv3.values())
    # a failed save reports the client's code for every block of the task and returns the slots
    mgr4 = connector.DataTransferManager(info, T, alloc, FakeTransferClient(fail_save=True), max_workers=2)
    done4 = threading.Event()
    res4 = []
    mgr4.submit_task(mgr4.save_task, connector.MultiResult(1, lambda r: (res4.append(r), done4.set())), 0, uris[:3],
                     idx_h[:3].tolist(), None)
    assert done4.wait(60)
    assert res4[0] == [[ClientErrorCode.ER_SDKWRITE_ERROR] * 3] and alloc._inuse_count == 0
    for m in (mgr, mgr2, mgr3, mgr4):
        m.shutdown()


class FakeCoordinatorClient:
    """Stands in for TpCoordinatorClient: records the messages and says when one has arrived."""

    def __init__(self):
        self.sent = []
        self.arrived = threading.Event()

    def send(self, data):
        self.sent.append(data)
        self.arrived.set()

    def take(self):
        assert self.arrived.wait(60)
        self.arrived.clear()
        return self.sent.pop()


def test_worker_loops_of_the_connector_run_on_the_manager_unchanged(oracle):
    """wait_for_save and start_load_kv as the reference writes them (v1_connector.py:448-475,486-519): the manager is
    built with the six positional arguments, tasks of block_per_*_task blocks go to the thread pool, the done
    callbacks fold the per-block codes into the message for the coordinator. One load task is made to fail: its local
    block ids come back in failed_block_idxs and its blocks stay untouched."""
    import copy
    import math
    from tair_kvcache_amd import connector, coordinator_messages as cm
    from tair_kvcache_amd.client_types import ClientErrorCode
    from tair_kvcache_amd.kernel.gather_scatter_helper import CopyBufferAllocator

    class ExtraConfig:
        block_per_save_task = 8
        block_per_load_task = 6

    L, nblk, T, H, hd = 3, 64, 16, 2, 64
    rng = np.random.default_rng(3)
    np_caches = [rng.integers(0, 65536, size=(2, nblk, T, H, hd), dtype=np.uint16) for _ in range(L)]
    kv = {f"layer{l}": dev(np_caches[l]).view(torch.bfloat16) for l in range(L)}
    info = connector.register_kv_caches(kv, T, T, tp_rank=0, world_size=1)
    alloc = CopyBufferAllocator(torch.device("cuda"), torch.bfloat16, list(info.per_manager_block_shape), 16)
    client, coord, extra = FakeTransferClient(), FakeCoordinatorClient(), ExtraConfig()

    # the staging pool is in HBM: this fake client finds the slot tensor behind an iov's address
    def slot_of(iov):
        raw = alloc._raw_buffer
        k, rem = divmod(iov.base - raw.data_ptr(), raw[0].numel() * raw.element_size())
        assert rem == 0 and iov.size == raw[0].numel() * raw.element_size()
        return raw[k]

    def save(uris, buffers):
        for uri, buf in zip(uris, buffers):
            client.store[uri] = slot_of(buf.iovs[0]).view(torch.int16).cpu().numpy().tobytes()
        return (ClientErrorCode.ER_OK, list(uris))

    def load(uris, buffers):
        if any("blkid=7&" in u for u in uris):
            return ClientErrorCode.ER_SDKREAD_ERROR
        for uri, buf in zip(uris, buffers):
            slot = slot_of(buf.iovs[0])
            data = torch.frombuffer(bytearray(client.store[uri]), dtype=torch.int16).view(slot.shape)
            slot.view(torch.int16).copy_(data)
        return ClientErrorCode.ER_OK

    client.SaveKvCaches, client.LoadKvCaches = save, load
    data_transfer = connector.DataTransferManager(info, T, alloc, client, coord, extra)

    local_block_ids = cases.block_table(nblk, 20).tolist()
    manager_block_idxes = list(range(20))
    all_remote_uris = [f"file:///kv/f?blkid={i}&size={info.per_manager_block_byte_size}" for i in range(20)]

    # ---- wait_for_save ----
    kvcache_ready_event = torch.cuda.Event()
    kvcache_ready_event.record(torch.cuda.current_stream())
    blocks_idx = connector.generate_blocks_idx(manager_block_idxes, local_block_ids, T, T)
    per_task_size = extra.block_per_save_task
    task_num = math.ceil(len(blocks_idx) / per_task_size)
    done_callback = data_transfer.create_save_done_callback("req-1", info.tp_rank, "session-1")
    multi_result = connector.MultiResult(task_num, done_callback)
    task_idx = 0
    for i in range(0, len(blocks_idx), per_task_size):
        end_idx = min(len(blocks_idx), i + per_task_size)
        data_transfer.submit_task(data_transfer.save_task, multi_result, task_idx, all_remote_uris[i:end_idx],
                                  blocks_idx[i:end_idx], kvcache_ready_event)
        task_idx += 1
    msg = cm.CoordinateMsgSerializer.loads(coord.take())
    assert isinstance(msg.content, cm.SendBlockFinishedEvent) and msg.content.is_success_list == [True] * 20
    assert (msg.content.request_id, msg.content.write_session_id) == ("req-1", "session-1")
    idx_h = host(blocks_idx, np.int32)
    pools = [np_caches[l][kvi].reshape(nblk * T, H * hd) for l in range(L) for kvi in (0, 1)]
    want = np.zeros((20, 2 * L, T, H * hd), dtype=np.uint16)
    oracle.batch_gather(pools, want, idx_h, None, T, H * hd * 2)
    for i, uri in enumerate(all_remote_uris):
        assert client.store[uri] == want[i].tobytes()

    # ---- start_load_kv into an empty cache; the task that holds block 7 fails ----
    kv2 = {k: torch.zeros_like(v) for k, v in kv.items()}
    info2 = connector.register_kv_caches(kv2, T, T)
    data_transfer2 = connector.DataTransferManager(info2, T, alloc, client, coord, extra)
    block_token_indices = idx_h.tolist()   # the reference's nested Python lists
    per_task_size = extra.block_per_load_task
    task_num = math.ceil(len(block_token_indices) / per_task_size)
    done_callback = data_transfer2.create_load_done_callback("req-1", info2.tp_rank, 5, copy.copy(local_block_ids))
    multi_result = connector.MultiResult(task_num, done_callback)
    task_idx = 0
    for i in range(0, len(block_token_indices), per_task_size):
        end_idx = min(len(block_token_indices), i + per_task_size)
        data_transfer2.submit_task(data_transfer2.load_task, multi_result, task_idx, all_remote_uris[i:end_idx],
                                   block_token_indices[i:end_idx])
        task_idx += 1
    msg = cm.CoordinateMsgSerializer.loads(coord.take())
    assert isinstance(msg.content, cm.LoadBlockFinishedEvent) and msg.content.epoch == 5
    assert msg.content.failed_block_idxs == local_block_ids[6:12]   # the second task of six blocks
    sync()
    assert alloc._inuse_count == 0
    loaded = np.array(local_block_ids[:6] + local_block_ids[12:])
    rest = np.setdiff1d(np.arange(nblk), loaded)
    for l in range(L):
        g = host(kv2[f"layer{l}"].view(torch.int16), np.uint16)
        assert (g[:, loaded] == np_caches[l][:, loaded]).all()
        assert not g[:, rest].any()
    data_transfer.shutdown()
    data_transfer2.shutdown()


def test_entry_points_can_be_captured_in_a_hip_graph(oracle):
    """The C-ABI neither allocates nor synchronises, so a transfer task (hash + gather + scatter on device-resident
    indices) can be captured once and replayed; every replay is checked against the eager result on fresh data, with
    eager work and synchronisations between replays."""
    from tair_kvcache_amd import hashing
    from tair_kvcache_amd.kernel import batch_gather_scatter_helper as bgs
    P, T, D, nblk, B = 16, 16, 256, 256, 64
    rng = np.random.default_rng(1)
    pool = torch.zeros((P, nblk * T, D), dtype=torch.int16, device="cuda")
    pool2 = torch.zeros_like(pool)
    table, table2 = ptr_table([pool[p] for p in range(P)]), ptr_table([pool2[p] for p in range(P)])
    blocks = cases.block_table(nblk, B)
    runs = dev((blocks * T).astype(np.int32))
    slots = torch.arange(B, dtype=torch.int32, device="cuda")
    staging = torch.zeros((B, P, T, D), dtype=torch.int16, device="cuda")
    tokens = torch.zeros((8, 256), dtype=torch.int64, device="cuda")
    toff = torch.arange(9, dtype=torch.int64, device="cuda") * 256
    koff = torch.arange(9, dtype=torch.int64, device="cuda") * 16
    keys = torch.zeros(8 * 16, dtype=torch.int64, device="cuda")

    def task():
        hashing.hash_tokens(tokens, 16, token_offsets=toff, keys=keys, key_offsets=koff)
        bgs.paged_gather_kv_caches(table, staging, runs, slots, T, D, T)
        bgs.paged_scatter_kv_caches(table2, staging, runs, slots, T, D, T)

    task()  # warm-up outside the capture
    sync()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        task()
    for it in range(4):
        new_pool = rng.integers(0, 65536, size=(P, nblk * T, D), dtype=np.uint16)
        new_tok = rng.integers(0, 128256, size=(8, 256), dtype=np.int64)
        pool.copy_(dev(new_pool))
        tokens.copy_(dev(new_tok))
        pool2.zero_()
        staging.zero_()
        keys.zero_()
        sync()
        graph.replay()
        sync()
        want = np.zeros((B, P, T, D), dtype=np.uint16)
        tidx = cases.token_idx_from_blocks(blocks, T)
        oracle.batch_gather([new_pool[p] for p in range(P)], want, tidx, None, T, D * 2)
        assert (host(staging, np.uint16) == want).all(), it
        touched = tidx.reshape(-1)
        got2 = host(pool2, np.uint16)
        assert (got2[:, touched] == new_pool[:, touched]).all(), it
        wkeys, _ = oracle.hash_tokens(new_tok, 16)
        assert (host(keys, np.int64) == wkeys).all(), it


def test_concurrent_callers_on_their_own_streams(oracle):
    """Sixteen host threads, each with its own stream, staging slots and index set, call gather, scatter and the hash at
    once (the reference drives its kernels from a 32-thread pool, data_transfer.py:80-93). The library keeps no
    mutable state, so every thread must get exactly its own answer."""
    from concurrent.futures import ThreadPoolExecutor
    from tair_kvcache_amd import hashing
    from tair_kvcache_amd.kernel import batch_gather_scatter_helper as bgs
    P, T, D, nblk, n_threads, per = 8, 16, 128, 512, 16, 24
    pools = cases.pool_u16(P, nblk * T, D)
    d_pools = [dev(p) for p in pools]
    table = ptr_table(d_pools)
    perm = cases.block_table(nblk, n_threads * per)
    staging = torch.zeros((n_threads * per, P, T, D), dtype=torch.int16, device="cuda")
    fresh = [torch.zeros_like(t) for t in d_pools]
    table2 = ptr_table(fresh)
    toks = cases.tokens(n_threads * 4, 512, 32000, seed=9)
    d_toks = dev(toks)
    keys_out = [None] * n_threads
    sync()

    def worker(i):
        torch.cuda.set_device(0)
        stream = torch.cuda.Stream()
        blocks = perm[i * per:(i + 1) * per]
        slots = list(range(i * per, (i + 1) * per))
        tidx = cases.token_idx_from_blocks(blocks, T).reshape(-1).tolist()
        with torch.cuda.stream(stream):
            for _ in range(5):
                bgs.batch_gather_kv_caches(table, staging, tidx, slots, T, D)
                bgs.batch_scatter_kv_caches(table2, staging, tidx, slots, T, D)
                keys_out[i], _ = hashing.hash_tokens(d_toks[i * 4:(i + 1) * 4], 16)
        stream.synchronize()
        return i

    with ThreadPoolExecutor(max_workers=n_threads) as ex:
        assert sorted(ex.map(worker, range(n_threads))) == list(range(n_threads))
    sync()
    tidx_all = cases.token_idx_from_blocks(perm, T)
    want = np.zeros((n_threads * per, P, T, D), dtype=np.uint16)
    oracle.batch_gather(pools, want, tidx_all, None, T, D * 2)
    assert (host(staging, np.uint16) == want).all()
    touched = np.zeros(nblk * T, dtype=bool)
    touched[tidx_all.reshape(-1)] = True
    for p in range(P):
        g = host(fresh[p], np.uint16)
        assert (g[touched] == pools[p][touched]).all() and not g[~touched].any()
    wkeys, _ = oracle.hash_tokens(toks, 16)
    for i in range(n_threads):
        assert (host(keys_out[i], np.int64) == wkeys[i * 128:(i + 1) * 128]).all()


class DeviceStagingClient:
    """A transfer client for staging slots that live in HBM: iovs arrive as MemoryType.GPU and are resolved back to
    slots of the allocator's backing tensor (a real SDK would hipMemcpyAsync from iov.base)."""

    def __init__(self, alloc):
        self.alloc = alloc
        self.store = {}

    def _slot(self, iov):
        from tair_kvcache_amd.client_types import MemoryType
        assert iov.type == MemoryType.GPU and iov.size == self.alloc.slot_nbytes
        off = iov.base - self.alloc._raw_buffer.data_ptr()
        assert off % self.alloc.slot_nbytes == 0
        return off // self.alloc.slot_nbytes

    def SaveKvCaches(self, uris, buffers):
        from tair_kvcache_amd.client_types import ClientErrorCode
        for uri, buf in zip(uris, buffers):
            self.store[uri] = self.alloc._raw_buffer[self._slot(buf.iovs[0])].cpu().clone()
        return (ClientErrorCode.ER_OK, list(uris))

    def LoadKvCaches(self, uris, buffers):
        from tair_kvcache_amd.client_types import ClientErrorCode
        for uri, buf in zip(uris, buffers):
            self.alloc._raw_buffer[self._slot(buf.iovs[0])].copy_(self.store[uri])
        torch.cuda.synchronize()
        return ClientErrorCode.ER_OK


def test_transfer_manager_with_staging_in_hbm(oracle):
    """The same save/load choreography with the staging pool on the GPU: slots are handed over as GPU iovs."""
    from tair_kvcache_amd import connector
    from tair_kvcache_amd.client_types import ClientErrorCode
    from tair_kvcache_amd.kernel.gather_scatter_helper import CopyBufferAllocator
    L, nblk, T_eng, T_mgr, H, hd = 3, 64, 16, 32, 4, 32
    rng = np.random.default_rng(4)
    np_caches = [rng.integers(0, 65536, size=(2, nblk, T_eng, H, hd), dtype=np.uint16) for _ in range(L)]
    kv = {f"layer{l}": dev(np_caches[l]).view(torch.float16) for l in range(L)}
    info = connector.register_kv_caches(kv, manager_block_size=T_mgr, local_block_size=T_eng)
    alloc = CopyBufferAllocator(torch.device("cuda"), torch.float16, list(info.per_manager_block_shape), 16)
    client = DeviceStagingClient(alloc)
    mgr = connector.DataTransferManager(info, T_mgr, alloc, client, max_workers=2)
    local_block_ids = cases.block_table(nblk, 24).tolist()  # 24 engine blocks = 12 manager blocks of 32 tokens
    idx = connector.generate_blocks_idx(list(range(12)), local_block_ids, T_mgr, T_eng)
    uris = [f"mem://blk{i}" for i in range(12)]
    done = threading.Event()
    res = []
    mgr.submit_task(mgr.save_task, connector.MultiResult(1, lambda r: (res.append(r), done.set())), 0, uris, idx, None)
    assert done.wait(60) and res[0] == [[ClientErrorCode.ER_OK] * 12]
    pools = [np_caches[l][k].reshape(nblk * T_eng, H * hd) for l in range(L) for k in (0, 1)]
    want = np.zeros((12, 2 * L, T_mgr, H * hd), dtype=np.uint16)
    oracle.batch_gather(pools, want, host(idx, np.int32), None, T_mgr, H * hd * 2)
    for i, uri in enumerate(uris):
        assert (client.store[uri].view(torch.int16).numpy().view(np.uint16).reshape(2 * L, T_mgr, H * hd) == want[i]).all()
    kv2 = {k: torch.zeros_like(v) for k, v in kv.items()}
    mgr2 = connector.DataTransferManager(connector.register_kv_caches(kv2, T_mgr, T_eng), T_mgr, alloc, client,
                                         max_workers=2)
    done2 = threading.Event()
    res2 = []
    mgr2.submit_task(mgr2.load_task, connector.MultiResult(1, lambda r: (res2.append(r), done2.set())), 0, uris, idx)
    assert done2.wait(60) and res2[0] == [[ClientErrorCode.ER_OK] * 12]
    touched = np.array(local_block_ids)
    for l in range(L):
        g = host(kv2[f"layer{l}"].view(torch.int16), np.uint16)
        assert (g[:, touched] == np_caches[l][:, touched]).all()
    assert alloc._inuse_count == 0
    mgr.shutdown()
    mgr2.shutdown()


def test_device_built_indices_that_leave_the_block_list_are_not_saved():
    """generate_blocks_idx with tensor arguments never reads back; a manager block beyond local_block_ids (the reference
    asserts, v1_connector.py:316) raises the module's per-device flag instead, and save_task, which waits for its gather
    anyway, looks at the flag before it hands the staged blocks to the transfer client."""
    from tair_kvcache_amd import connector
    from tair_kvcache_amd.client_types import ClientErrorCode
    from tair_kvcache_amd.kernel.gather_scatter_helper import CopyBufferAllocator
    L, nblk, T, H, hd = 2, 16, 16, 2, 32
    kv = {f"layer{l}": torch.ones(2, nblk, T, H, hd, dtype=torch.bfloat16, device="cuda") for l in range(L)}
    info = connector.register_kv_caches(kv, T, T)
    # pinned host staging: the fake client reads the slots with the CPU
    alloc = CopyBufferAllocator(torch.device("cpu"), torch.bfloat16, list(info.per_manager_block_shape), 8)
    client = FakeTransferClient()
    mgr = connector.DataTransferManager(info, T, alloc, client, max_workers=2)
    connector.blocks_idx_error("cuda")  # whatever an earlier test left behind
    assert connector.blocks_idx_error("cuda") is False
    local = torch.tensor([3, 5, 7], dtype=torch.int32, device="cuda")
    good = connector.generate_blocks_idx(torch.tensor([0, 2], dtype=torch.int32, device="cuda"), local, T, T)
    assert connector.blocks_idx_error("cuda") is False
    bad = connector.generate_blocks_idx(torch.tensor([1, 3], dtype=torch.int32, device="cuda"), local, T, T)
    sync()
    assert host(bad, np.int32)[1].tolist() == [-1] * T and host(good, np.int32)[1, 0] == 7 * T
    for idx, want in ((bad, ClientErrorCode.ER_INVALID_PARAMS), (good, ClientErrorCode.ER_OK)):
        done, out = threading.Event(), []
        multi = connector.MultiResult(1, lambda r: (out.append(r), done.set()))
        uris = [f"file:///kv/err?blkid={i}&size={info.per_manager_block_byte_size}" for i in range(2)]
        mgr.submit_task(mgr.save_task, multi, 0, uris, idx)
        assert done.wait(60)
        assert out[0] == [[want] * 2]
        assert alloc._inuse_count == 0
        assert (want == ClientErrorCode.ER_OK) == all(u in client.store for u in uris)
    assert connector.blocks_idx_error("cuda") is False  # read and cleared by the task that met it
    mgr.shutdown()


def test_host_built_block_index_through_the_transfer_manager(oracle):
    """generate_blocks_idx_host (the reference's list flow, v1_connector.py:308-320, without the Python double loop)
    -> slices of it handed to save_task and load_task; manager blocks of 64 tokens over engine blocks of 16. Stored
    bytes equal the oracle's staging layout and the caches come back byte for byte."""
    from tair_kvcache_amd import connector
    from tair_kvcache_amd.client_types import ClientErrorCode
    from tair_kvcache_amd.kernel.gather_scatter_helper import CopyBufferAllocator
    L, nblk, T_eng, T_mgr, H, hd = 3, 96, 16, 64, 2, 64
    rng = np.random.default_rng(5)
    np_caches = [rng.integers(0, 65536, size=(2, nblk, T_eng, H, hd), dtype=np.uint16) for _ in range(L)]
    kv = {f"layer{l}": dev(np_caches[l]).view(torch.bfloat16) for l in range(L)}
    info = connector.register_kv_caches(kv, manager_block_size=T_mgr, local_block_size=T_eng)
    alloc = CopyBufferAllocator(torch.device("cpu"), torch.bfloat16, list(info.per_manager_block_shape), 16)
    client = FakeTransferClient()
    mgr = connector.DataTransferManager(info, T_mgr, alloc, client, max_workers=2)
    local_block_ids = cases.block_table(nblk, 40).tolist()  # 40 engine blocks = 10 manager blocks
    manager_blocks = [9, 0, 3, 4, 5, 7]
    idx = connector.generate_blocks_idx_host(manager_blocks, local_block_ids, T_mgr, T_eng)
    idx_np, bad = oracle.generate_blocks_idx(np.array(manager_blocks, dtype=np.int32),
                                             np.array(local_block_ids, dtype=np.int32), T_mgr, T_eng)
    assert bad == 0 and idx.tolist() == idx_np.tolist()
    n = len(manager_blocks)
    print(f"host-built index: {n} manager blocks of {T_mgr} over engine blocks of {T_eng}", flush=True)
    uris = [f"file:///kv/h?blkid={i}" for i in range(n)]
    done, results = threading.Event(), []
    multi = connector.MultiResult(2, lambda r: (results.append(r), done.set()))
    mgr.submit_task(mgr.save_task, multi, 0, uris[:4], idx[:4], None)
    mgr.submit_task(mgr.save_task, multi, 1, uris[4:], idx[4:], None)
    assert done.wait(60)
    assert results[0] == [[ClientErrorCode.ER_OK] * 4, [ClientErrorCode.ER_OK] * 2]
    pools = [np_caches[l][kvi].reshape(nblk * T_eng, H * hd) for l in range(L) for kvi in (0, 1)]
    want = np.zeros((n, 2 * L, T_mgr, H * hd), dtype=np.uint16)
    oracle.batch_gather(pools, want, idx_np, None, T_mgr, H * hd * 2)
    for i, uri in enumerate(uris):
        assert client.store[uri] == want[i].tobytes(), i
    kv2 = {k: torch.zeros_like(v) for k, v in kv.items()}
    mgr2 = connector.DataTransferManager(connector.register_kv_caches(kv2, T_mgr, T_eng), T_mgr, alloc, client,
                                         max_workers=2)
    done2, res2 = threading.Event(), []
    mgr2.submit_task(mgr2.load_task, connector.MultiResult(1, lambda r: (res2.append(r), done2.set())), 0, uris, idx)
    assert done2.wait(60)
    assert res2[0] == [[ClientErrorCode.ER_OK] * n] and alloc._inuse_count == 0
    sync()
    touched = np.unique(idx_np // T_eng)
    rest = np.setdiff1d(np.arange(nblk), touched)
    for l in range(L):
        g = host(kv2[f"layer{l}"].view(torch.int16), np.uint16)
        assert (g[:, touched] == np_caches[l][:, touched]).all()
        assert not g[:, rest].any()
    mgr.shutdown()
    mgr2.shutdown()
