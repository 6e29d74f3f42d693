"""Pins the gather/scatter oracle (no GPU): a permutation copy checked against NumPy indexing written from the
reference's index algebra, the reference kernel test's own expected-value loops, self-identifying ramp pools,
round trips and guard bands."""
import numpy as np
import pytest

import _cases as cases


def _staging(slots, P, T, D, fill=0):
    return np.full((slots, P, T, D), fill, dtype=np.uint16)


@pytest.mark.parametrize("name", ["c1_qwen05b", "c2_llama8b_scaled", "ref_test_shape"])
def test_gather_matches_numpy(oracle, name):
    c = cases.SMALL_CONFIGS[name]
    P, T, D = c["L"] * c["kv"], c["T"], c["D"]
    pools = cases.pool_u16(P, c["pool_blocks"] * T, D)
    rng = np.random.default_rng(2)
    # token-granular indices: any slot, as in the reference test (randperm per block)
    tidx = np.stack([rng.permutation(c["pool_blocks"] * T)[:T] for _ in range(c["B"])]).astype(np.int32)
    sidx = rng.permutation(c["slots"])[:c["B"]].astype(np.int32)
    got = _staging(c["slots"], P, T, D, 0xABCD)
    want = got.copy()
    oracle.batch_gather(pools, got, tidx, sidx, T, D * 2)
    oracle.np_batch_gather(pools, want, tidx, sidx, T)
    assert (got == want).all()
    untouched = np.setdiff1d(np.arange(c["slots"]), sidx)
    assert (got[untouched] == 0xABCD).all()


def test_reference_test_expected_loops(oracle):
    """The per-element expectation of test_batch_gather_scatter.py:91-114 at its own shape, on a sample."""
    c = cases.SMALL_CONFIGS["ref_test_shape"]
    L, T, D = c["L"], c["T"], c["D"]
    total_tokens = 10240
    rng = np.random.default_rng(42)
    caches = [rng.integers(0, 65536, size=(2, total_tokens, D), dtype=np.uint16) for _ in range(L)]
    pools = []
    for cache in caches:
        pools += [cache[0], cache[1]]
    tidx = np.concatenate([rng.permutation(total_tokens)[:T] for _ in range(c["B"])]).astype(np.int32)
    sidx = rng.permutation(c["slots"])[:c["B"]].astype(np.int32)
    dst = _staging(c["slots"], 2 * L, T, D)
    oracle.batch_gather(pools, dst, tidx, sidx, T, D * 2)
    for block_idx in range(0, c["B"], 7):
        for token_pos in range(T):
            token_idx = tidx[block_idx * T + token_pos]
            for layer_idx in range(L):
                assert (dst[sidx[block_idx], layer_idx * 2, token_pos] == caches[layer_idx][0][token_idx]).all()
                assert (dst[sidx[block_idx], layer_idx * 2 + 1, token_pos] == caches[layer_idx][1][token_idx]).all()


def test_edge_one_token_one_block(oracle):
    # test_batch_gather_scatter.py:221-298: 1 layer, 32 tokens in the cache, T = 1, D = 64, token 5 -> slot 0
    rng = np.random.default_rng(42)
    cache = rng.integers(0, 65536, size=(2, 32, 64), dtype=np.uint16)
    dst = _staging(1, 2, 1, 64)
    oracle.batch_gather([cache[0], cache[1]], dst, [5], [0], 1, 128)
    assert (dst[0, 0, 0] == cache[0, 5]).all() and (dst[0, 1, 0] == cache[1, 5]).all()
    cache2 = np.zeros_like(cache)
    oracle.batch_scatter([cache2[0], cache2[1]], dst, [9], [0], 1, 128)
    assert (cache2[0, 9] == cache[0, 5]).all() and (cache2[1, 9] == cache[1, 5]).all()
    cache2[:, 9] = 0
    assert not cache2.any()


def test_ramp_pool_names_its_rows(oracle):
    P, T, D, slots = 6, 16, 32, 512
    pools = cases.ramp_pool_u16(P, slots, D)
    blocks = cases.block_table(slots // T, 20)
    tidx = cases.token_idx_from_blocks(blocks, T)
    st = _staging(20, P, T, D)
    oracle.batch_gather(pools, st, tidx, None, T, D * 2)
    for p in range(P):
        want = ((p * 131 + tidx) % 65536).astype(np.uint16)
        assert (st[:, p, :, 0] == want).all() and (st[:, p, :, D - 1] == want).all()


def test_scatter_inverts_gather_and_spares_the_rest(oracle):
    c = cases.SMALL_CONFIGS["c1_qwen05b"]
    P, T, D = c["L"] * c["kv"], c["T"], c["D"]
    pools = cases.pool_u16(P, c["pool_blocks"] * T, D)
    blocks = cases.block_table(c["pool_blocks"], c["B"])
    tidx = cases.token_idx_from_blocks(blocks, T)
    st = _staging(c["slots"], P, T, D)
    oracle.batch_gather(pools, st, tidx, None, T, D * 2)
    fresh = [np.full_like(p, 0x5A5A) for p in pools]
    oracle.batch_scatter(fresh, st, tidx, None, T, D * 2)
    touched = np.zeros(c["pool_blocks"] * T, dtype=bool)
    touched[tidx.reshape(-1)] = True
    for p in range(P):
        assert (fresh[p][touched] == pools[p][touched]).all()
        assert (fresh[p][~touched] == 0x5A5A).all()
    want = [np.full_like(p, 0x5A5A) for p in pools]
    oracle.np_batch_scatter(want, st, tidx, None, T)
    assert all((a == b).all() for a, b in zip(fresh, want))


def test_paged_runs_equal_token_indices(oracle):
    """run_tokens > 1 (block-table fast path) moves the same bytes as the expanded per-token index."""
    P, T_mgr, T_eng, D = 4, 64, 16, 40
    n_eng_blocks = 64
    pools = cases.pool_u16(P, n_eng_blocks * T_eng, D)
    local = cases.block_table(n_eng_blocks, 32)
    mgr = np.array([3, 0, 5], dtype=np.int32)
    idx, bad = oracle.generate_blocks_idx(mgr, local, T_mgr, T_eng)
    assert bad == 0 and idx.tolist() == oracle.py_generate_blocks_idx(mgr.tolist(), local.tolist(), T_mgr, T_eng)
    a = _staging(3, P, T_mgr, D)
    oracle.batch_gather(pools, a, idx, None, T_mgr, D * 2)
    b = _staging(3, P, T_mgr, D)
    d, keep = oracle.make_desc(pools, b, idx[:, ::T_eng], None, 3, T_mgr, D * 2, run_tokens=T_eng)
    oracle.gather_ex(d)
    assert (a == b).all()
    # manager block smaller than the engine block: one run inside an engine block
    idx2, bad = oracle.generate_blocks_idx(np.array([5, 2], dtype=np.int32), local, 8, 16)
    assert bad == 0 and idx2.tolist() == oracle.py_generate_blocks_idx([5, 2], local.tolist(), 8, 16)
    assert idx2[0, 0] == local[2] * 16 + 8
    # reaching beyond the local blocks is flagged, the reference asserts there (v1_connector.py:315)
    _, bad = oracle.generate_blocks_idx(np.array([100], dtype=np.int32), local, 64, 16)
    assert bad == 1


def test_legacy_layout_equals_batch_on_views(oracle):
    """gather_scatter_helper.py:61-107: one [2, total, H] tensor per layer, staging [L, 2, T, H], idx >= total skipped."""
    L, total, H, T = 3, 128, 48, 32
    rng = np.random.default_rng(42)
    caches = [rng.integers(0, 65536, size=(2, total, H), dtype=np.uint16) for _ in range(L)]
    idx = rng.permutation(total)[:T].astype(np.int32)
    dst = np.zeros((L, 2, T, H), dtype=np.uint16)
    d, keep = oracle.make_desc(caches, dst, idx, None, 1, T, H * 2, ptrs_per_entry=2,
                               entry_stride_bytes=total * H * 2, slot_limit=total)
    oracle.gather_ex(d)
    for l in range(L):
        assert (dst[l] == caches[l][:, idx, :]).all()
    views = []
    for cch in caches:
        views += [cch[0], cch[1]]
    dst2 = np.zeros((1, 2 * L, T, H), dtype=np.uint16)
    oracle.batch_gather(views, dst2, idx, None, T, H * 2)
    assert (dst2.reshape(L, 2, T, H) == dst).all()
    # reference_impl of the file's own main(): kv_caches[l][:, token_indices, :] = source[l] (:273-276)
    src = rng.integers(0, 65536, size=(L, 2, T, H), dtype=np.uint16)
    got = [c.copy() for c in caches]
    want = [c.copy() for c in caches]
    d, keep = oracle.make_desc(got, src, idx, None, 1, T, H * 2, ptrs_per_entry=2, entry_stride_bytes=total * H * 2,
                               slot_limit=total)
    oracle.scatter_ex(d)
    for l in range(L):
        want[l][:, idx, :] = src[l]
        assert (got[l] == want[l]).all()
    # out-of-range rows are skipped in both directions
    idx_oob = idx.copy()
    idx_oob[[1, 7]] = [total, total + 5]
    dst3 = np.full((L, 2, T, H), 0x7777, dtype=np.uint16)
    d, keep = oracle.make_desc(caches, dst3, idx_oob, None, 1, T, H * 2, ptrs_per_entry=2,
                               entry_stride_bytes=total * H * 2, slot_limit=total)
    oracle.gather_ex(d)
    assert (dst3[:, :, [1, 7]] == 0x7777).all() and (dst3[:, :, 0] == np.stack([c[:, idx[0]] for c in caches])).all()
    # negative rows (the -1 that generate_blocks_idx writes past the local blocks) are skipped too, limit or not
    for limit in (total, 0):
        idx_neg = idx.copy()
        idx_neg[[0, 9]] = [-1, -7]
        dst4 = np.full((L, 2, T, H), 0x3333, dtype=np.uint16)
        d, keep = oracle.make_desc(caches, dst4, idx_neg, None, 1, T, H * 2, ptrs_per_entry=2,
                                   entry_stride_bytes=total * H * 2, slot_limit=limit)
        oracle.gather_ex(d)
        assert (dst4[:, :, [0, 9]] == 0x3333).all()
        assert (np.delete(dst4, [0, 9], axis=2) == np.delete(dst, [0, 9], axis=2)).all()


def test_trailer_interleave_bruteforce(oracle):
    """fp8 latent cache with one fp32 scale per (layer, block): record = payload then 4 scale bytes."""
    L, T, row, nblocks = 5, 8, 36, 16  # row of 36 bytes: 4-byte aligned only
    rng = np.random.default_rng(1)
    pools = [rng.integers(0, 254, size=(nblocks * T, row), dtype=np.uint8) for _ in range(L)]
    scales = [rng.standard_normal(nblocks).astype(np.float32) for _ in range(L)]
    blocks = cases.block_table(nblocks, 6)
    rec = T * row + 4
    st = np.full((6, L * rec), 0xEE, dtype=np.uint8)
    d, keep = oracle.make_desc(pools, st, blocks * T, None, 6, T, row, run_tokens=T, trailers=scales,
                               trailer_idx=blocks, trailer_bytes=4)
    oracle.gather_ex(d)
    for b, blk in enumerate(blocks):
        for l in range(L):
            base = l * rec
            assert (st[b, base:base + T * row] == pools[l][blk * T:(blk + 1) * T].reshape(-1)).all()
            assert st[b, base + T * row:base + rec].tobytes() == scales[l][blk:blk + 1].tobytes()
    pools2 = [np.zeros_like(p) for p in pools]
    scales2 = [np.zeros_like(s) for s in scales]
    d, keep = oracle.make_desc(pools2, st, blocks * T, None, 6, T, row, run_tokens=T, trailers=scales2,
                               trailer_idx=blocks, trailer_bytes=4)
    oracle.scatter_ex(d)
    for l in range(L):
        for blk in blocks:
            assert (pools2[l][blk * T:(blk + 1) * T] == pools[l][blk * T:(blk + 1) * T]).all()
            assert scales2[l][blk] == scales[l][blk]
        rest = np.setdiff1d(np.arange(nblocks), blocks)
        assert not scales2[l][rest].any()


def test_threaded_copy_equals_serial(oracle):
    P, T, D = 8, 16, 64
    pools = cases.pool_u16(P, 64 * T, D)
    tidx = cases.token_idx_from_blocks(cases.block_table(64, 40), T)
    a = _staging(40, P, T, D)
    b = _staging(40, P, T, D)
    d, keep = oracle.make_desc(pools, a, tidx, None, 40, T, D * 2)
    oracle.gather_ex(d)
    d2, keep2 = oracle.make_desc(pools, b, tidx, None, 40, T, D * 2)
    oracle.gather_ex(d2, threads=4)
    assert (a == b).all()


def test_trailer_is_skipped_for_negative_trailer_index_bruteforce(oracle):
    """trailer_idx[b] < 0 = no trailer for block b: on gather its staging trailer bytes keep their fill, on scatter no
    scale is written; a block whose rows are skipped (run start < 0) still moves its trailer when the index is valid."""
    L, T, row, nblocks = 3, 4, 16, 8
    rng = np.random.default_rng(8)
    pools = [rng.integers(0, 254, size=(nblocks * T, row), dtype=np.uint8) for _ in range(L)]
    scales = [rng.standard_normal(nblocks).astype(np.float32) for _ in range(L)]
    runs = np.array([5 * T, -1, 2 * T], dtype=np.int32)      # block 1: rows skipped
    tr_idx = np.array([-1, 6, 2], dtype=np.int32)              # block 0: trailer skipped
    rec = T * row + 4
    st = np.full((3, L * rec), 0xEE, dtype=np.uint8)
    d, keep = oracle.make_desc(pools, st, runs, None, 3, T, row, run_tokens=T, trailers=scales, trailer_idx=tr_idx,
                               trailer_bytes=4)
    oracle.gather_ex(d)
    for l in range(L):
        base = l * rec
        assert (st[0, base:base + T * row] == pools[l][5 * T:6 * T].reshape(-1)).all()
        assert (st[0, base + T * row:base + rec] == 0xEE).all()                              # no trailer moved
        assert (st[1, base:base + T * row] == 0xEE).all()                                    # rows skipped
        assert st[1, base + T * row:base + rec].tobytes() == scales[l][6:7].tobytes()        # trailer still moved
        assert st[2, base + T * row:base + rec].tobytes() == scales[l][2:3].tobytes()
    pools2 = [np.zeros_like(p) for p in pools]
    scales2 = [np.zeros_like(s) for s in scales]
    d, keep = oracle.make_desc(pools2, st, runs, None, 3, T, row, run_tokens=T, trailers=scales2, trailer_idx=tr_idx,
                               trailer_bytes=4)
    oracle.scatter_ex(d)
    for l in range(L):
        assert scales2[l][6] == scales[l][6] and scales2[l][2] == scales[l][2]
        assert not np.delete(scales2[l], [6, 2]).any()
        for blk in (5, 2):
            assert (pools2[l][blk * T:(blk + 1) * T] == pools[l][blk * T:(blk + 1) * T]).all()
        assert not np.delete(pools2[l].reshape(nblocks, -1), [5, 2], axis=0).any()
