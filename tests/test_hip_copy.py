"""GPU parity: the HIP gather/scatter path, called through the C-ABI, against the CPU oracle. Byte-exact."""
import numpy as np
import pytest
import torch

import _cases as cases
from _gpu import dev, host, ptr_table, sync

pytestmark = pytest.mark.gpu

GUARD = 0x6B6B


def _ops():
    from tair_kvcache_amd.kernel import batch_gather_scatter_helper as bgs
    return bgs


def _case_inputs(name):
    c = cases.SMALL_CONFIGS[name]
    P, T, D = c["L"] * c["kv"], c["T"], c["D"]
    rng = np.random.default_rng(2)
    if name == "c5_page1_scaled":
        n_slots = 4096
        tidx = rng.permutation(n_slots)[:c["B"] * T].reshape(c["B"], T).astype(np.int32)
    else:
        n_slots = c["pool_blocks"] * T
        tidx = cases.token_idx_from_blocks(cases.block_table(c["pool_blocks"], c["B"]), T)
    pools = cases.pool_u16(P, n_slots, D)
    sidx = rng.permutation(c["slots"])[:c["B"]].astype(np.int32)
    return c, P, T, D, n_slots, pools, tidx, sidx


@pytest.mark.parametrize("name", list(cases.SMALL_CONFIGS))
def test_gather_then_scatter_matches_oracle(oracle, name):
    bgs = _ops()
    c, P, T, D, n_slots, pools, tidx, sidx = _case_inputs(name)
    print(f"case={name} P={P} T={T} D={D} B={c['B']}", flush=True)
    # oracle
    want = np.full((c["slots"], P, T, D), GUARD, dtype=np.uint16)
    oracle.batch_gather(pools, want, tidx, sidx, T, D * 2)
    # device: one guard slot before and after the staging pool
    d_pools = [dev(p) for p in pools]
    table = ptr_table(d_pools)
    d_st_all = torch.full((c["slots"] + 2, P, T, D), GUARD, dtype=torch.int16, device="cuda")
    d_st = d_st_all[1:-1]
    bgs.batch_gather_kv_caches(table, d_st, tidx.reshape(-1).tolist(), sidx.tolist(), T, D)
    sync()
    got = host(d_st_all, np.uint16)
    assert (got[1:-1] == want).all()
    assert (got[0] == GUARD).all() and (got[-1] == GUARD).all()
    # scatter back into pools full of guard values
    want_pools = [np.full_like(p, GUARD) for p in pools]
    oracle.batch_scatter(want_pools, want, tidx, sidx, T, D * 2)
    d_fresh = [torch.full((n_slots + 2, D), GUARD, dtype=torch.int16, device="cuda") for _ in range(P)]
    table2 = ptr_table([t[1:] for t in d_fresh])
    bgs.batch_scatter_kv_caches(table2, d_st, dev(tidx), dev(sidx), T, D)  # tensor index arguments
    sync()
    for p in range(P):
        g = host(d_fresh[p], np.uint16)
        assert (g[1:-1] == want_pools[p]).all(), p
        assert (g[0] == GUARD).all() and (g[-1] == GUARD).all()


def test_reference_edge_one_token_one_block(oracle):
    # test_batch_gather_scatter.py:221-298,499-577
    bgs = _ops()
    rng = np.random.default_rng(42)
    cache = rng.integers(0, 65536, size=(2, 32, 64), dtype=np.uint16)
    d_cache = dev(cache)
    table = ptr_table([d_cache[0], d_cache[1]])
    dst = torch.zeros(1, 2, 1, 64, dtype=torch.int16, device="cuda")
    bgs.batch_gather_kv_caches(table, dst, [5], [0], 1, 64, 2)
    sync()
    got = host(dst, np.uint16)
    assert (got[0, 0, 0] == cache[0, 5]).all() and (got[0, 1, 0] == cache[1, 5]).all()
    d_cache2 = torch.zeros_like(d_cache)
    table2 = ptr_table([d_cache2[0], d_cache2[1]])
    bgs.batch_scatter_kv_caches(table2, dst, [9], [0], 1, 64, 2)
    sync()
    g2 = host(d_cache2, np.uint16)
    assert (g2[0, 9] == cache[0, 5]).all() and (g2[1, 9] == cache[1, 5]).all()
    g2[:, 9] = 0
    assert not g2.any()


def test_ramp_pool_and_bf16_dtype():
    """Typed tensors (bf16) move as bytes; a ramp pool names the slot every staged row came from."""
    bgs = _ops()
    P, T, D, slots = 6, 16, 128, 2048
    pool = (torch.arange(slots, device="cuda", dtype=torch.float32) % 256)[None, :, None].expand(P, slots, D)
    pool = (pool + torch.arange(P, device="cuda", dtype=torch.float32)[:, None, None] * 256).to(torch.bfloat16).contiguous()
    table = ptr_table([pool[p] for p in range(P)])
    blocks = cases.block_table(slots // T, 40)
    tidx = cases.token_idx_from_blocks(blocks, T)
    st = torch.zeros(40, P, T, D, dtype=torch.bfloat16, device="cuda")
    bgs.batch_gather_kv_caches(table, st, tidx.reshape(-1).tolist(), list(range(40)), T, D)
    sync()
    want = pool[:, torch.from_numpy(tidx.astype(np.int64)).cuda()]  # [P, B, T, D]
    assert torch.equal(st, want.permute(1, 0, 2, 3))


def test_paged_runs_equal_token_granular(oracle):
    bgs = _ops()
    from tair_kvcache_amd import connector
    P, T_mgr, T_eng, D = 8, 64, 16, 256
    n_eng = 128
    pools = cases.pool_u16(P, n_eng * T_eng, D)
    local = cases.block_table(n_eng, 64)
    mgr = [3, 0, 7, 12, 5]
    idx, bad = oracle.generate_blocks_idx(np.array(mgr, dtype=np.int32), local, T_mgr, T_eng)
    assert bad == 0
    want = np.zeros((5, P, T_mgr, D), dtype=np.uint16)
    oracle.batch_gather(pools, want, idx, None, T_mgr, D * 2)
    d_pools = [dev(p) for p in pools]
    table = ptr_table(d_pools)
    # CL1 on device equals the oracle's double loop
    d_idx = connector.generate_blocks_idx(mgr, local.tolist(), T_mgr, T_eng)
    runs, g = connector.generate_run_starts(mgr, local.tolist(), T_mgr, T_eng)
    sync()
    assert (host(d_idx, np.int32) == idx).all()
    assert g == 16 and (host(runs, np.int32) == idx[:, ::16]).all()
    a = torch.zeros(5, P, T_mgr, D, dtype=torch.int16, device="cuda")
    b = torch.zeros_like(a)
    bgs.batch_gather_kv_caches(table, a, d_idx, list(range(5)), T_mgr, D)
    bgs.paged_gather_kv_caches(table, b, runs, list(range(5)), T_mgr, D, g)
    sync()
    assert (host(a, np.uint16) == want).all() and (host(b, np.uint16) == want).all()
    # manager block smaller than the engine block
    runs2, g2 = connector.generate_run_starts([5, 2], local.tolist(), 8, 16)
    idx2, _ = oracle.generate_blocks_idx(np.array([5, 2], dtype=np.int32), local, 8, 16)
    sync()
    assert g2 == 8 and (host(runs2, np.int32)[:, 0] == idx2[:, 0]).all()
    with pytest.raises(AssertionError):
        connector.generate_blocks_idx([1000], local.tolist(), T_mgr, T_eng)
    # scatter through the paged entry point
    fresh = [torch.zeros_like(t) for t in d_pools]
    bgs.paged_scatter_kv_caches(ptr_table(fresh), b, runs, list(range(5)), T_mgr, D, g)
    sync()
    want_pools = [np.zeros_like(p) for p in pools]
    oracle.batch_scatter(want_pools, want, idx, None, T_mgr, D * 2)
    for p in range(P):
        assert (host(fresh[p], np.uint16) == want_pools[p]).all()


@pytest.mark.parametrize("row_bytes,base_off", [(64, 0), (36, 0), (36, 4), (37, 0), (48, 4), (64, 1), (2048, 0), (272, 0)])
def test_alignment_classes(oracle, row_bytes, base_off):
    """16-byte, dword and byte paths, and pool bases that are themselves misaligned."""
    from tair_kvcache_amd import _lib
    P, T, B, slots = 5, 4, 9, 40
    rng = np.random.default_rng(row_bytes * 7 + base_off)
    pools = [rng.integers(0, 256, size=(slots, row_bytes), dtype=np.uint8) for _ in range(P)]
    tidx = rng.permutation(slots)[:B * T].reshape(B, T).astype(np.int32)
    want = np.zeros((B, P * T * row_bytes), dtype=np.uint8)
    oracle.batch_gather(pools, want, tidx, None, T, row_bytes)
    backing = [torch.zeros(slots * row_bytes + 64, dtype=torch.uint8, device="cuda") for _ in range(P)]
    views = []
    for p in range(P):
        v = backing[p][base_off:base_off + slots * row_bytes]
        v.copy_(torch.from_numpy(pools[p].reshape(-1)))
        views.append(v)
    table = ptr_table(views)
    st = torch.zeros(B, P * T * row_bytes, dtype=torch.uint8, device="cuda")
    d_tidx = dev(tidx)
    rc = _lib.lib().kvcm_hip_batch_gather(table.data_ptr(), P, st.data_ptr(), P * T * row_bytes, d_tidx.data_ptr(), None,
                                          B, T, row_bytes, 0, torch.cuda.current_stream().cuda_stream)
    assert rc == 0
    sync()
    assert (host(st, np.uint8) == want).all()
    for v in views:
        v.zero_()
    rc = _lib.lib().kvcm_hip_batch_scatter(table.data_ptr(), P, st.data_ptr(), P * T * row_bytes, d_tidx.data_ptr(), None,
                                           B, T, row_bytes, 0, torch.cuda.current_stream().cuda_stream)
    assert rc == 0
    sync()
    want_pools = [np.zeros_like(p) for p in pools]
    oracle.batch_scatter(want_pools, want, tidx, None, T, row_bytes)
    for p in range(P):
        assert (host(views[p], np.uint8).reshape(slots, row_bytes) == want_pools[p]).all()
        assert not host(backing[p], np.uint8)[:base_off].any()


def test_mla_fp8_with_interleaved_scales(oracle):
    """Config-4 shape, scaled: one latent pool per layer (576 bytes/token), 128-token blocks, one fp32 scale per
    (layer, block) appended to every layer record; the record stride is only 4-byte aligned."""
    from tair_kvcache_amd import _lib
    L, T, row, nblocks, B = 7, 128, 576, 24, 10
    rng = np.random.default_rng(1)
    codes = np.array([c for c in range(256) if c not in (0x7F, 0xFF)], dtype=np.uint8)
    pools = [codes[rng.integers(0, 254, size=(nblocks * T, row))] for _ in range(L)]
    scales = [rng.standard_normal(nblocks).astype(np.float32) for _ in range(L)]
    blocks = cases.block_table(nblocks, B)
    rec = T * row + 4
    want = np.full((B, L * rec), 0xEE, dtype=np.uint8)
    d, keep = oracle.make_desc(pools, want, blocks * T, None, B, T, row, run_tokens=T, trailers=scales,
                               trailer_idx=blocks, trailer_bytes=4)
    oracle.gather_ex(d)
    d_pools = [dev(p) for p in pools]
    d_scales = [dev(s) for s in scales]
    st = torch.full((B, L * rec), 0xEE, dtype=torch.uint8, device="cuda")
    run_start = dev((blocks * T).astype(np.int32))
    tr_idx = dev(blocks)
    table, ttable = ptr_table(d_pools), ptr_table(d_scales)

    def desc(pool_table, trailer_table):
        x = _lib.CopyDesc()
        x.d_ptr_table, x.P, x.ptrs_per_entry, x.entry_stride_bytes = pool_table.data_ptr(), L, 1, 0
        x.d_staging, x.staging_block_stride_bytes, x.staging_tile_stride_bytes = st.data_ptr(), L * rec, rec
        x.d_run_start, x.d_staging_idx, x.B, x.T, x.run_tokens = run_start.data_ptr(), None, B, T, T
        x.slot_limit, x.row_bytes = 0, row
        x.d_trailer_ptr_table, x.d_trailer_idx, x.trailer_bytes = trailer_table.data_ptr(), tr_idx.data_ptr(), 4
        x.max_workgroups = 0
        return x

    rc = _lib.lib().kvcm_hip_gather_ex(desc(table, ttable), torch.cuda.current_stream().cuda_stream)
    assert rc == 0
    sync()
    got = host(st, np.uint8)
    assert (got == want).all()
    assert got[0, T * row:rec].tobytes() == scales[0][blocks[0]:blocks[0] + 1].tobytes()
    pools2 = [torch.zeros_like(t) for t in d_pools]
    scales2 = [torch.zeros_like(t) for t in d_scales]
    rc = _lib.lib().kvcm_hip_scatter_ex(desc(ptr_table(pools2), ptr_table(scales2)),
                                        torch.cuda.current_stream().cuda_stream)
    assert rc == 0
    sync()
    for l in range(L):
        g = host(pools2[l], np.uint8).reshape(nblocks, T * row)
        w = pools[l].reshape(nblocks, T * row)
        assert (g[blocks] == w[blocks]).all()
        rest = np.setdiff1d(np.arange(nblocks), blocks)
        assert not g[rest].any()
        gs = host(scales2[l], np.float32)
        assert (gs[blocks] == scales[l][blocks]).all() and not gs[rest].any()
    # a negative trailer index skips a block's trailers, a negative run start its rows: against the oracle, both ways
    tr_np = blocks.astype(np.int32).copy()
    tr_np[[0, 3]] = -1
    runs_np = (blocks * T).astype(np.int32)
    runs_np[[3, 5]] = -1
    want2 = np.full((B, L * rec), 0xEE, dtype=np.uint8)
    d, keep = oracle.make_desc(pools, want2, runs_np, None, B, T, row, run_tokens=T, trailers=scales, trailer_idx=tr_np,
                               trailer_bytes=4)
    oracle.gather_ex(d)
    st.fill_(0xEE)
    run_start, tr_idx = dev(runs_np), dev(tr_np)
    assert _lib.lib().kvcm_hip_gather_ex(desc(table, ttable), torch.cuda.current_stream().cuda_stream) == 0
    sync()
    assert (host(st, np.uint8) == want2).all()
    w_pools, w_scales = [np.zeros_like(p) for p in pools], [np.zeros_like(x) for x in scales]
    d, keep = oracle.make_desc(w_pools, want2, runs_np, None, B, T, row, run_tokens=T, trailers=w_scales,
                               trailer_idx=tr_np, trailer_bytes=4)
    oracle.scatter_ex(d)
    pools3 = [torch.zeros_like(t) for t in d_pools]
    scales3 = [torch.zeros_like(t) for t in d_scales]
    assert _lib.lib().kvcm_hip_scatter_ex(desc(ptr_table(pools3), ptr_table(scales3)),
                                          torch.cuda.current_stream().cuda_stream) == 0
    sync()
    for l in range(L):
        assert (host(pools3[l], np.uint8) == w_pools[l]).all()
        assert host(scales3[l], np.float32).tobytes() == w_scales[l].tobytes()


def test_legacy_single_block_operators(oracle):
    """gather_kv_caches / scatter_kv_caches at the reference main()'s shape (gather_scatter_helper.py:279-317)."""
    from tair_kvcache_amd.kernel import gather_scatter_helper as gsh
    L, total, T, H = 4, 128, 32, 512
    rng = np.random.default_rng(42)
    caches = [rng.standard_normal((2, total, H)).astype(np.float32) for _ in range(L)]
    src = rng.standard_normal((L, 2, T, H)).astype(np.float32)
    idx = rng.permutation(total)[:T]
    d_caches = [dev(c) for c in caches]
    table = ptr_table(d_caches)
    gsh.scatter_kv_caches(table, total, dev(src), idx.tolist())
    sync()
    for l in range(L):
        want = caches[l].copy()
        want[:, idx, :] = src[l]  # reference_impl (:273-276)
        assert (host(d_caches[l], np.float32) == want).all()
    dst = torch.zeros(L, 2, T, H, dtype=torch.float32, device="cuda")
    gsh.gather_kv_caches(table, total, dst, idx.tolist())
    sync()
    assert (host(dst, np.float32) == src).all()
    # out-of-range indices are skipped
    idx2 = idx.copy()
    idx2[[0, 3]] = [total, total + 9]
    dst2 = torch.full((L, 2, T, H), 7.0, dtype=torch.float32, device="cuda")
    gsh.gather_kv_caches(table, total, dst2, idx2.tolist())
    sync()
    g = host(dst2, np.float32)
    assert (g[:, :, [0, 3]] == 7.0).all() and (g[:, :, 1] == src[:, :, 1]).all()
    with pytest.raises(AssertionError):
        gsh.gather_kv_caches(table, total, torch.zeros(L + 1, 2, T, H, device="cuda"), idx.tolist())


def test_pinned_host_staging_and_workgroup_cap(oracle):
    """Staging in pinned host memory (the reference's CopyBufferAllocator default) and a capped grid (sm_count)."""
    bgs = _ops()
    from tair_kvcache_amd.kernel.gather_scatter_helper import CopyBufferAllocator
    P, T, D = 8, 16, 128
    pools = cases.pool_u16(P, 64 * T, D)
    tidx = cases.token_idx_from_blocks(cases.block_table(64, 12), T)
    alloc = CopyBufferAllocator(torch.device("cpu"), torch.int16, [P // 2, 2, T, D], 16)
    assert alloc._raw_buffer.is_pinned()
    slots = alloc.alloc_buffer_idx_blocking(12)
    want = np.zeros((16, P, T, D), dtype=np.uint16)
    oracle.batch_gather(pools, want, tidx, np.array(slots, dtype=np.int32), T, D * 2)
    table = ptr_table([dev(p) for p in pools])
    keep = [dev(p) for p in pools]
    table = ptr_table(keep)
    bgs.SM_COUNT_IS_CAP = True
    try:
        bgs.batch_gather_kv_caches(table, alloc._raw_buffer, tidx.reshape(-1).tolist(), slots, T, D)  # sm_count = 3
    finally:
        bgs.SM_COUNT_IS_CAP = False
    sync()
    assert (alloc._raw_buffer.numpy().view(np.uint16).reshape(16, P, T, D) == want).all()
    alloc.free_buffer(slots)


def test_shape_errors_raise_value_error():
    bgs = _ops()
    t = torch.zeros(4, 16 * 8, dtype=torch.int16, device="cuda")
    table = ptr_table([t[i] for i in range(4)])
    st = torch.zeros(2, 4, 16, 8, dtype=torch.int16, device="cuda")
    with pytest.raises(ValueError):
        bgs.batch_gather_kv_caches(table, st, [0] * 31, [0, 1], 16, 8)  # wrong index count
    with pytest.raises(ValueError):
        bgs.batch_gather_kv_caches(table, st, [0] * 32, [0, 2], 16, 8)  # staging slot out of range
    with pytest.raises(ValueError):
        bgs.batch_gather_kv_caches(table, st[:, :3], [0] * 32, [0, 1], 16, 8)  # not contiguous
    with pytest.raises(ValueError):
        bgs.batch_gather_kv_caches(table, st, [0] * 32, [0, 1], 16, 7)  # staging is not whole blocks
    bgs.batch_gather_kv_caches(table, st, [], [], 16, 8)  # empty batch is a no-op
    sync()


def test_block_major_pools_are_the_one_array_case(oracle):
    """Engines whose pool is already block-major -- TRT-LLM's [blocks, layers, K|V, heads*dim*tokens]
    (trtllm/connector.py:173-179) or a page-first host pool -- need no transposition: the pool is ONE array whose
    'rows' are whole blocks, so the same entry point moves them with P = 1, T = 1 and block ids as slots."""
    bgs = _ops()
    nblk, layers, kvf, block_elems, B = 96, 4, 2, 8 * 64 * 32, 40
    rng = np.random.default_rng(1)
    pool = rng.integers(0, 65536, size=(nblk, layers * kvf * block_elems), dtype=np.uint16)
    ids = cases.block_table(nblk, B)
    want = np.zeros((B, 1, 1, pool.shape[1]), dtype=np.uint16)
    oracle.batch_gather([pool], want, ids, None, 1, pool.shape[1] * 2)
    assert (want[:, 0, 0] == pool[ids]).all()
    d_pool = dev(pool)
    table = ptr_table([d_pool])
    st = torch.zeros((B, 1, 1, pool.shape[1]), dtype=torch.int16, device="cuda")
    bgs.batch_gather_kv_caches(table, st, ids.tolist(), list(range(B)), 1, pool.shape[1])
    sync()
    assert (host(st, np.uint16) == want).all()
    fresh = torch.zeros_like(d_pool)
    bgs.batch_scatter_kv_caches(ptr_table([fresh]), st, ids.tolist(), list(range(B)), 1, pool.shape[1])
    sync()
    g = host(fresh, np.uint16)
    rest = np.setdiff1d(np.arange(nblk), ids)
    assert (g[ids] == pool[ids]).all() and not g[rest].any()
