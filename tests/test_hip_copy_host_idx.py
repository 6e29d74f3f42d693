"""GPU parity of the entry points that take their index lists in HOST memory (kvcm_hip_batch_gather_host_idx /
kvcm_hip_batch_scatter_host_idx: the form in which the reference's operators receive them,
batch_gather_scatter_helper.py:101-136,208-248), against the CPU oracle, byte-exact, through the C-ABI and through the
operator module. The lists are chosen so that every way the host walk can classify them is met: whole engine blocks
(one run per block), manager blocks of several engine blocks (runs of g slots), unrelated slots (runs of 1), rows to
skip (negative slots), and more blocks than one argument block holds (several launches per call)."""
from array import array

import numpy as np
import pytest
import torch

import _cases as cases
from _gpu import dev, host, ptr_table, sync

pytestmark = pytest.mark.gpu

GUARD = 0x5A5A


def _ops():
    from tair_kvcache_amd.kernel import batch_gather_scatter_helper as bgs
    return bgs


def _index_lists(kind, B, T, n_slots, rng):
    if kind == "whole_blocks":  # T consecutive slots per block: block-table form, one run per block
        return cases.token_idx_from_blocks(rng.permutation(n_slots // T)[:B].astype(np.int32), T)
    if kind == "runs_of_4":  # a manager block = T/4 engine blocks of 4 slots
        starts = rng.permutation(n_slots // 4)[:B * (T // 4)].reshape(B, T // 4).astype(np.int64) * 4
        return (starts[:, :, None] + np.arange(4)[None, None, :]).reshape(B, T).astype(np.int32)
    if kind == "unrelated":  # page size 1
        return rng.permutation(n_slots)[:B * T].reshape(B, T).astype(np.int32)
    if kind == "one_break":  # every block consecutive but ONE block with a break at an odd position: runs of 1
        idx = cases.token_idx_from_blocks(rng.permutation(n_slots // T)[:B].astype(np.int32), T)
        idx[B // 2, 3:] = idx[B // 2, 3:][::-1].copy()
        return idx
    if kind == "with_skips":  # negative slots: those rows stay as they are, their neighbours move
        idx = cases.token_idx_from_blocks(rng.permutation(n_slots // T)[:B].astype(np.int32), T)
        idx[1, 5] = -1
        idx[2, :] = -1
        idx[3, 0] = -7
        return idx
    raise AssertionError(kind)


@pytest.mark.parametrize("kind,B,T,D", [
    ("whole_blocks", 128, 16, 1024),  # one transfer task of the Llama-3-8B layout (P scaled down)
    ("whole_blocks", 500, 16, 128),   # more than the 416 blocks one launch holds
    ("runs_of_4", 40, 16, 256),
    ("unrelated", 100, 16, 512),      # 48 blocks per launch: three launches
    ("unrelated", 7, 24, 64),         # a block size that is not a power of two, 128-byte rows
    ("one_break", 33, 16, 256),
    ("with_skips", 9, 16, 128),
])
def test_host_lists_match_oracle(oracle, kind, B, T, D):
    bgs = _ops()
    P, slots = 6, B + 5
    n_slots = max(2 * B * T, 64 * T)
    rng = np.random.default_rng(11)
    print(f"kind={kind} B={B} T={T} D={D} P={P}", flush=True)
    tidx = _index_lists(kind, B, T, n_slots, rng)
    sidx = rng.permutation(slots)[:B].astype(np.int32)
    pools = cases.pool_u16(P, n_slots, D)
    want = np.full((slots, P, T, D), GUARD, dtype=np.uint16)
    oracle.batch_gather(pools, want, tidx, sidx, T, D * 2)
    d_pools = [dev(p) for p in pools]
    table = ptr_table(d_pools)
    d_all = torch.full((slots + 2, P, T, D), GUARD, dtype=torch.int16, device="cuda")
    d_st = d_all[1:-1]
    bgs.batch_gather_kv_caches(table, d_st, tidx.reshape(-1).tolist(), sidx.tolist(), T, D, pool_token_slots=n_slots)
    sync()
    got = host(d_all, np.uint16)
    assert (got[1:-1] == want).all()
    assert (got[0] == GUARD).all() and (got[-1] == GUARD).all()
    # back into pools full of guard values, this time from CPU tensors (host memory as well)
    want_pools = [np.full_like(p, GUARD) for p in pools]
    oracle.batch_scatter(want_pools, want, tidx, sidx, T, D * 2)
    d_fresh = [torch.full((n_slots + 2, D), GUARD, dtype=torch.int16, device="cuda") for _ in range(P)]
    table2 = ptr_table([t[1:] for t in d_fresh])
    bgs.batch_scatter_kv_caches(table2, d_st, torch.from_numpy(tidx), torch.from_numpy(sidx), T, D,
                                pool_token_slots=n_slots)
    sync()
    for p in range(P):
        g = host(d_fresh[p], np.uint16)
        assert (g[1:-1] == want_pools[p]).all(), p
        assert (g[0] == GUARD).all() and (g[-1] == GUARD).all()


def test_c_abi_null_staging_list_and_array_argument(oracle):
    """Straight through the C-ABI: h_staging_idx = NULL means slot b; the lists may be freed right after the call."""
    from tair_kvcache_amd import _lib
    L = _lib.lib()
    P, T, D, B, n_slots = 4, 16, 256, 450, 16 * 1024
    pools = cases.pool_u16(P, n_slots, D)
    tidx = cases.token_idx_from_blocks(cases.block_table(n_slots // T, B), T)
    want = np.zeros((B, P, T, D), dtype=np.uint16)
    oracle.batch_gather(pools, want, tidx, None, T, D * 2)
    d_pools = [dev(p) for p in pools]
    table = ptr_table(d_pools)
    st = torch.zeros((B, P, T, D), dtype=torch.int16, device="cuda")
    lst = array("i", tidx.reshape(-1).tolist())
    rc = L.kvcm_hip_batch_gather_host_idx(table.data_ptr(), P, st.data_ptr(), P * T * D * 2, B, lst.buffer_info()[0],
                                          None, B, T, D * 2, n_slots, 0, torch.cuda.current_stream().cuda_stream)
    assert rc == 0
    for i in range(len(lst)):  # the call has returned: the list is the caller's again
        lst[i] = -1
    del lst
    sync()
    assert (host(st, np.uint16) == want).all()


def test_out_of_range_indices_are_refused_before_anything_is_launched():
    bgs = _ops()
    P, T, D, n_slots = 2, 16, 64, 1024
    pool = torch.zeros((P, n_slots, D), dtype=torch.int16, device="cuda")
    table = ptr_table([pool[0], pool[1]])
    st = torch.full((4, P, T, D), 7, dtype=torch.int16, device="cuda")
    good = list(range(T))
    with pytest.raises(ValueError):
        bgs.batch_gather_kv_caches(table, st, good[:-1] + [n_slots], [0], T, D, pool_token_slots=n_slots)
    with pytest.raises(ValueError):
        bgs.batch_gather_kv_caches(table, st, good, [4], T, D)
    with pytest.raises(ValueError):
        bgs.batch_scatter_kv_caches(table, st, good, [-1], T, D)
    with pytest.raises(ValueError):
        bgs.batch_gather_kv_caches(table, st, good + [1], [0], T, D)  # 17 entries for one block
    with pytest.raises(ValueError):
        bgs.batch_gather_kv_caches(table, st, good[:-1] + [2 ** 40], [0], T, D)
    with pytest.raises(ValueError):
        bgs.batch_gather_kv_caches(table, st, good[:-1] + ["x"], [0], T, D)
    sync()
    assert bool((st == 7).all()) and not bool(pool.any())


def test_a_block_of_more_runs_than_an_argument_block_holds_is_uploaded(oracle):
    """T = 1024 unrelated slots per block: 1024 runs do not fit the kernel's argument block; the operator falls back to
    uploading the list, with the same result."""
    bgs = _ops()
    P, T, D, B, n_slots = 2, 1024, 32, 3, 8192
    rng = np.random.default_rng(5)
    tidx = rng.permutation(n_slots)[:B * T].reshape(B, T).astype(np.int32)
    pools = cases.pool_u16(P, n_slots, D)
    want = np.zeros((B, P, T, D), dtype=np.uint16)
    oracle.batch_gather(pools, want, tidx, None, T, D * 2)
    d_pools = [dev(p) for p in pools]
    table = ptr_table(d_pools)
    st = torch.zeros((B, P, T, D), dtype=torch.int16, device="cuda")
    bgs.batch_gather_kv_caches(table, st, tidx.reshape(-1).tolist(), list(range(B)), T, D)
    sync()
    assert (host(st, np.uint16) == want).all()


def test_host_list_call_can_be_captured_and_replayed(oracle):
    """The host-list entry points launch kernels and nothing else (no upload, no allocation, no memset): a captured
    call carries its index tables inside the graph. Replayed three times with other pool contents each time, with eager
    work and synchronisations in between, every replay against the oracle."""
    bgs = _ops()
    P, T, D, B, n_slots = 4, 16, 256, 100, 4096
    rng = np.random.default_rng(21)
    tidx = rng.permutation(n_slots)[:B * T].reshape(B, T).astype(np.int32)   # unrelated slots: three launches per call
    lst, slots = tidx.reshape(-1).tolist(), list(range(B))
    pool = torch.zeros((P, n_slots, D), dtype=torch.int16, device="cuda")
    table = ptr_table([pool[p] for p in range(P)])
    st = torch.zeros((B, P, T, D), dtype=torch.int16, device="cuda")
    bgs.batch_gather_kv_caches(table, st, lst, slots, T, D)  # eager once: the library and its kernels are loaded
    sync()
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.graph(graph, stream=side):
        bgs.batch_gather_kv_caches(table, st, lst, slots, T, D, pool_token_slots=n_slots)
    lst[:] = [0] * len(lst)  # the lists are the caller's again: the graph must not look at them
    for rep in range(3):
        pools = cases.pool_u16(P, n_slots, D, seed=100 + rep)
        pool.copy_(torch.stack([dev(p) for p in pools]))
        st.fill_(-1)
        sync()
        graph.replay()
        sync()
        want = np.zeros((B, P, T, D), dtype=np.uint16)
        oracle.batch_gather(pools, want, tidx, None, T, D * 2)
        assert (host(st, np.uint16) == want).all(), rep


@pytest.mark.parametrize("form", ["lists", "device_tensors", "list_and_tensor"])
def test_stream_argument_launches_on_that_stream(oracle, form):
    """`stream=` hands the launch a stream of the caller's instead of torch's current one (what DataTransferManager's
    worker threads do): the copy is ordered behind work queued on that stream before it, whichever way the indices
    arrive -- host lists, device tensors, or a list that has to be uploaded on that stream first."""
    bgs = _ops()
    P, T, D, B, n_slots = 4, 16, 512, 64, 4096
    pools = cases.pool_u16(P, n_slots, D)
    tidx = cases.token_idx_from_blocks(cases.block_table(n_slots // T, B), T)
    sidx = np.arange(B, dtype=np.int32)
    want = np.zeros((B, P, T, D), dtype=np.uint16)
    oracle.batch_gather(pools, want, tidx, sidx, T, D * 2)
    pool = torch.zeros((P, n_slots, D), dtype=torch.int16, device="cuda")
    table = ptr_table([pool[p] for p in range(P)])
    st = torch.zeros((B, P, T, D), dtype=torch.int16, device="cuda")
    fresh = torch.stack([dev(p) for p in pools])
    d_tidx, d_sidx = dev(tidx.reshape(-1)), dev(sidx)
    sync()
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        filler = torch.empty(256 << 20, dtype=torch.uint8, device="cuda")
        for _ in range(20):
            filler.add_(1)          # work in front of ...
        pool.copy_(fresh)           # ... the copy that fills the pool, all on the side stream
    # torch's current stream is the default one here: only the stream argument orders the gather behind the fill
    if form == "lists":
        bgs.batch_gather_kv_caches(table, st, tidx.reshape(-1).tolist(), sidx.tolist(), T, D, stream=side)
    elif form == "device_tensors":
        bgs.batch_gather_kv_caches(table, st, d_tidx, d_sidx, T, D, stream=side)
    else:
        bgs.batch_gather_kv_caches(table, st, tidx.reshape(-1).tolist(), d_sidx, T, D, stream=side)
    side.synchronize()
    assert (host(st, np.uint16) == want).all()
