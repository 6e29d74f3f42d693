"""GPU parity of the general copy entry points on many small random shapes against the CPU oracle: every chunk size
(16 / 4 / 1 byte), runs of several tokens, two pointers per table entry, skipped slots, trailers of odd sizes,
misaligned pool bases, scrambled staging slots with padding between tiles and blocks, capped grids. Byte-exact,
both directions, guard bytes around everything."""
import numpy as np
import pytest
import torch

from _gpu import ptr_table, sync

pytestmark = pytest.mark.gpu

ROWS = [1, 3, 4, 12, 16, 20, 36, 48, 64, 100, 256, 272, 1000, 1024, 4096]


def _case(rng):
    row = int(rng.choice(ROWS))
    run_tokens = int(rng.choice([1, 1, 2, 4]))
    T = run_tokens * int(rng.integers(1, 7))
    ppe = int(rng.choice([1, 1, 2]))
    entries = int(rng.integers(1, 6))
    P = entries * ppe
    B = int(rng.integers(0, 10))
    slots_pool = int(rng.integers(T * 2, T * 12))
    trailer = int(rng.choice([0, 0, 0, 4, 3, 8]))
    align = 4 if row % 4 == 0 and trailer % 4 == 0 else 1
    pad_tile = int(rng.choice([0, 0, 16 if align == 4 else 5]))
    tile_stride = T * row + trailer + pad_tile
    block_stride = P * tile_stride + int(rng.choice([0, 0, 32 if align == 4 else 7]))
    n_slots = B + int(rng.integers(0, 4))
    base_off = int(rng.choice([0, 0, 0, 4, 1])) if row % 4 == 0 else int(rng.choice([0, 1, 2]))
    limit = int(rng.choice([0, 0, slots_pool // 2]))
    cap = int(rng.choice([0, 0, 1, 3]))
    return dict(row=row, run_tokens=run_tokens, T=T, ppe=ppe, entries=entries, P=P, B=B, slots_pool=slots_pool,
                trailer=trailer, tile_stride=tile_stride, block_stride=block_stride, n_slots=n_slots,
                base_off=base_off, limit=limit, cap=cap)


def _run_case(oracle, c, rng, direction):
    from tair_kvcache_amd import _lib
    row, T, P, B, ppe = c["row"], c["T"], c["P"], c["B"], c["ppe"]
    runs = T // c["run_tokens"]
    entry_stride = c["slots_pool"] * row if ppe == 2 else 0
    entry_bytes = c["slots_pool"] * row * ppe
    # host data: pool entries, trailer arrays (one per p, indexed by a per-block id), staging
    pools = [rng.integers(0, 256, size=entry_bytes, dtype=np.uint8) for _ in range(c["entries"])]
    n_tr = 16
    trailers = [rng.integers(0, 256, size=n_tr * max(c["trailer"], 1), dtype=np.uint8) for _ in range(P)]
    staging = rng.integers(0, 256, size=max(c["n_slots"], 1) * c["block_stride"], dtype=np.uint8)
    max_start = c["slots_pool"] - c["run_tokens"]
    # distinct runs (scatter must not see duplicates); a few negative entries are skipped by contract
    starts = (rng.permutation(max_start // c["run_tokens"] + 1)[:B * runs] * c["run_tokens"]).astype(np.int32)
    if len(starts) < B * runs:
        return False
    if B * runs > 2 and rng.random() < 0.3:
        starts[int(rng.integers(0, B * runs))] = -1
    sidx = rng.permutation(max(c["n_slots"], 1))[:B].astype(np.int32)
    tr_idx = rng.permutation(n_tr)[:B].astype(np.int32)   # distinct: two blocks scattering into one trailer row race

    def make(o_pools, o_staging, o_trailers):
        d, keep = oracle.make_desc(o_pools, o_staging, starts, sidx, B, T, row, run_tokens=c["run_tokens"],
                                   ptrs_per_entry=ppe, entry_stride_bytes=entry_stride, slot_limit=c["limit"],
                                   tile_stride=c["tile_stride"], block_stride=c["block_stride"],
                                   trailers=o_trailers if c["trailer"] else None,
                                   trailer_idx=tr_idx if c["trailer"] else None, trailer_bytes=c["trailer"])
        return d, keep

    w_pools = [p.copy() for p in pools]
    w_staging = staging.copy()
    w_trailers = [t.copy() for t in trailers]
    d, keep = make(w_pools, w_staging, w_trailers)
    (oracle.scatter_ex if direction == "scatter" else oracle.gather_ex)(d)

    # device copies with guard bytes and an optional misalignment of every pool base
    GUARD = 64
    off = c["base_off"]
    d_pools_back = [torch.full((entry_bytes + 2 * GUARD + 8,), 0xA5, dtype=torch.uint8, device="cuda") for _ in pools]
    d_pools = []
    for back, p in zip(d_pools_back, pools):
        view = back[GUARD + off:GUARD + off + entry_bytes]
        view.copy_(torch.from_numpy(p))
        d_pools.append(view)
    d_trailers = [torch.from_numpy(t).cuda() for t in trailers]
    d_staging_back = torch.full((len(staging) + 2 * GUARD,), 0x5A, dtype=torch.uint8, device="cuda")
    d_staging = d_staging_back[GUARD:GUARD + len(staging)]
    d_staging.copy_(torch.from_numpy(staging))
    d_starts = torch.from_numpy(starts).cuda() if B else torch.zeros(1, dtype=torch.int32, device="cuda")
    d_sidx = torch.from_numpy(sidx).cuda() if B else torch.zeros(1, dtype=torch.int32, device="cuda")
    d_tr_idx = torch.from_numpy(tr_idx).cuda() if B else torch.zeros(1, dtype=torch.int32, device="cuda")
    table, ttable = ptr_table(d_pools), ptr_table(d_trailers)
    x = _lib.CopyDesc()
    x.d_ptr_table, x.P, x.ptrs_per_entry, x.entry_stride_bytes = table.data_ptr(), P, ppe, entry_stride
    x.d_staging, x.staging_block_stride_bytes, x.staging_tile_stride_bytes = (d_staging.data_ptr(), c["block_stride"],
                                                                               c["tile_stride"])
    x.d_run_start, x.d_staging_idx, x.B, x.T, x.run_tokens = d_starts.data_ptr(), d_sidx.data_ptr(), B, T, c["run_tokens"]
    x.slot_limit, x.row_bytes = c["limit"], row
    x.d_trailer_ptr_table = ttable.data_ptr() if c["trailer"] else None
    x.d_trailer_idx = d_tr_idx.data_ptr() if c["trailer"] else None
    x.trailer_bytes, x.max_workgroups = c["trailer"], c["cap"]
    fn = _lib.lib().kvcm_hip_scatter_ex if direction == "scatter" else _lib.lib().kvcm_hip_gather_ex
    rc = fn(x, torch.cuda.current_stream().cuda_stream)
    assert rc == 0, (rc, c)
    sync()
    assert (d_staging.cpu().numpy() == w_staging).all(), c
    for back, view, want in zip(d_pools_back, d_pools, w_pools):
        assert (view.cpu().numpy() == want).all(), c
        b = back.cpu().numpy()
        assert (b[:GUARD + off] == 0xA5).all() and (b[GUARD + off + entry_bytes:] == 0xA5).all(), c
    if c["trailer"]:
        for t, want in zip(d_trailers, w_trailers):
            assert (t.cpu().numpy() == want).all(), c
    sb = d_staging_back.cpu().numpy()
    assert (sb[:GUARD] == 0x5A).all() and (sb[GUARD + len(staging):] == 0x5A).all(), c
    return True


@pytest.mark.parametrize("direction", ["gather", "scatter"])
def test_random_small_shapes(oracle, direction):
    rng = np.random.default_rng(2024 if direction == "gather" else 4202)
    done = 0
    for i in range(90):
        c = _case(rng)
        print(f"random copy case {i} {direction}: {c}", flush=True)
        done += bool(_run_case(oracle, c, rng, direction))
    assert done >= 60
