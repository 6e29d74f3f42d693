"""GPU parity at the benchmark configurations' full sizes, through properties that need no host copy of the data:
the pool holds a pattern that is a function of (array, slot, element), so every staged row and every loaded row can
be recomputed on the device from the index alone; untouched memory must keep its fill value.
Bit-exact (integer patterns)."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _bgs():
    from tair_kvcache_amd.kernel import batch_gather_scatter_helper as bgs
    return bgs


def pattern(p, slots, D, device):
    """int16 [len(slots), D]: a different value for every (array p, slot, element)."""
    s = slots.to(torch.int64)[:, None]
    d = torch.arange(D, device=device, dtype=torch.int64)[None, :]
    return ((s * 40503 + d * 31 + p * 7919 + ((s >> 7) ^ d)) & 0xFFFF).to(torch.int16)


def fill_pool(pool):
    P, n_slots, D = pool.shape
    step = 1 << 18
    for p in range(P):
        for s0 in range(0, n_slots, step):
            sl = torch.arange(s0, min(s0 + step, n_slots), device=pool.device)
            pool[p, s0:s0 + len(sl)] = pattern(p, sl, D, pool.device)


def free():
    torch.cuda.synchronize()
    torch.cuda.empty_cache()


def test_config2_llama3_8b_save_and_load():
    """32 layers x K/V, 8 x 128 bf16, 16-token blocks, pool of 32768 blocks; 12416 unique blocks of 64 requests."""
    bgs = _bgs()
    dev = torch.device("cuda")
    P, T, D, nblk, B = 64, 16, 1024, 32768, 12416
    pool = torch.empty((P, nblk * T, D), dtype=torch.int16, device=dev)
    fill_pool(pool)
    table = torch.tensor([pool[p].data_ptr() for p in range(P)], dtype=torch.int64, device=dev)
    perm = np.random.default_rng(2).permutation(nblk).astype(np.int32)
    save_b, load_b = perm[:B], perm[B:2 * B]
    staging = torch.zeros((B, P, T, D), dtype=torch.int16, device=dev)
    runs = torch.from_numpy(save_b * T).to(dev)
    slots = torch.arange(B, dtype=torch.int32, device=dev)
    print("config2 gather", flush=True)
    bgs.paged_gather_kv_caches(table, staging, runs, slots, T, D, T)
    tok = (torch.from_numpy(save_b.astype(np.int64)).to(dev)[:, None] * T + torch.arange(T, device=dev)[None, :]).reshape(-1)
    for p in range(P):
        assert torch.equal(staging[:, p].reshape(B * T, D), pattern(p, tok, D, dev)), p
    # the per-token form of the same call gives the same staging
    staging2 = torch.zeros((256, P, T, D), dtype=torch.int16, device=dev)
    bgs.batch_gather_kv_caches(table, staging2, tok[:256 * T].to(torch.int32), slots[:256], T, D)
    assert torch.equal(staging2, staging[:256])
    del staging2
    print("config2 scatter", flush=True)
    load_runs = torch.from_numpy(load_b * T).to(dev)
    bgs.paged_scatter_kv_caches(table, staging, load_runs, slots, T, D, T)
    ltok = (torch.from_numpy(load_b.astype(np.int64)).to(dev)[:, None] * T + torch.arange(T, device=dev)[None, :]).reshape(-1)
    rest = torch.from_numpy(np.sort(perm[2 * B:]).astype(np.int64)).to(dev)
    rtok = (rest[:, None] * T + torch.arange(T, device=dev)[None, :]).reshape(-1)
    for p in range(P):
        assert torch.equal(pool[p][ltok], pattern(p, tok, D, dev)), p      # loaded rows = the staged rows
        assert torch.equal(pool[p][tok], pattern(p, tok, D, dev)), p       # sources untouched
    for p in (0, 31, 63):
        assert torch.equal(pool[p][rtok], pattern(p, rtok, D, dev)), p     # bystanders untouched
    del pool, staging
    free()


def test_config3_long_context_load():
    """80 layers, 64-token blocks of 8 x 128 bf16, pool of 8192 blocks; the 25 % missed blocks of 32 requests
    (2048 blocks, 40 GiB of staging [block][layer][K|V][64][8][128]) are scattered into a zeroed pool."""
    bgs = _bgs()
    dev = torch.device("cuda")
    P, T, D, nblk, B = 160, 64, 1024, 8192, 2048
    pool = torch.zeros((P, nblk * T, D), dtype=torch.int16, device=dev)
    table = torch.tensor([pool[p].data_ptr() for p in range(P)], dtype=torch.int64, device=dev)
    staging = torch.empty((B, P, T, D), dtype=torch.int16, device=dev)
    rows = torch.arange(B * T, device=dev)
    for p in range(P):
        staging[:, p] = pattern(p, rows, D, dev).reshape(B, T, D)
    perm = np.random.default_rng(2).permutation(nblk).astype(np.int32)
    # per request: 256 blocks, the last 64 are misses
    miss = np.concatenate([perm[r * 256 + 192:(r + 1) * 256] for r in range(32)])
    runs = torch.from_numpy(miss * T).to(dev)
    print("config3 scatter", flush=True)
    bgs.paged_scatter_kv_caches(table, staging, runs, torch.arange(B, dtype=torch.int32, device=dev), T, D, T)
    tok = (torch.from_numpy(miss.astype(np.int64)).to(dev)[:, None] * T + torch.arange(T, device=dev)[None, :]).reshape(-1)
    touched = torch.zeros(nblk * T, dtype=torch.bool, device=dev)
    touched[tok] = True
    for p in range(P):
        assert torch.equal(pool[p][tok], staging[:, p].reshape(B * T, D)), p
    for p in (0, 79, 159):
        assert not pool[p][~touched].any(), p
    del pool, staging
    free()


def test_config4_mla_fp8_latent_with_scales():
    """61 layers, one 576-byte e4m3 latent per token, 128-token blocks, pool of 4096 blocks, one fp32 scale per
    (layer, block); one full permutation of the pool is gathered into records of 73 728 payload + 4 scale bytes."""
    from tair_kvcache_amd import _lib
    dev = torch.device("cuda")
    L, T, row, nblk = 61, 128, 576, 4096
    rec = T * row + 4
    g = torch.Generator(device=dev)
    g.manual_seed(1)
    codes = torch.tensor([c for c in range(256) if c not in (0x7F, 0xFF)], dtype=torch.uint8, device=dev)
    pool = torch.empty((L, nblk * T, row), dtype=torch.uint8, device=dev)
    for l in range(L):
        pool[l] = codes[torch.randint(0, 254, (nblk * T, row), device=dev, generator=g)]
    scales = torch.randn((L, nblk), dtype=torch.float32, device=dev, generator=g)
    table = torch.tensor([pool[l].data_ptr() for l in range(L)], dtype=torch.int64, device=dev)
    ttable = torch.tensor([scales[l].data_ptr() for l in range(L)], dtype=torch.int64, device=dev)
    blocks = np.random.default_rng(2).permutation(nblk).astype(np.int32)
    d_blocks = torch.from_numpy(blocks).to(dev)
    runs = d_blocks * T
    staging = torch.full((nblk, L * rec), 0xEE, dtype=torch.uint8, device=dev)

    def desc(pt, tt):
        x = _lib.CopyDesc()
        x.d_ptr_table, x.P, x.ptrs_per_entry, x.entry_stride_bytes = pt.data_ptr(), L, 1, 0
        x.d_staging, x.staging_block_stride_bytes, x.staging_tile_stride_bytes = staging.data_ptr(), L * rec, rec
        x.d_run_start, x.d_staging_idx, x.B, x.T, x.run_tokens = runs.data_ptr(), None, nblk, T, T
        x.slot_limit, x.row_bytes = 0, row
        x.d_trailer_ptr_table, x.d_trailer_idx, x.trailer_bytes = tt.data_ptr(), d_blocks.data_ptr(), 4
        x.max_workgroups = 0
        return x

    print("config4 gather", flush=True)
    rc = _lib.lib().kvcm_hip_gather_ex(desc(table, ttable), torch.cuda.current_stream().cuda_stream)
    assert rc == 0
    st = staging.view(nblk, L, rec)
    idx = d_blocks.to(torch.int64)
    for l in range(L):
        assert torch.equal(st[:, l, :T * row], pool[l].view(nblk, T * row)[idx]), l
        assert torch.equal(st[:, l, T * row:].contiguous().view(torch.float32).reshape(-1), scales[l][idx]), l
    print("config4 scatter", flush=True)
    pool2 = torch.zeros_like(pool)
    scales2 = torch.zeros_like(scales)
    rc = _lib.lib().kvcm_hip_scatter_ex(
        desc(torch.tensor([pool2[l].data_ptr() for l in range(L)], dtype=torch.int64, device=dev),
             torch.tensor([scales2[l].data_ptr() for l in range(L)], dtype=torch.int64, device=dev)),
        torch.cuda.current_stream().cuda_stream)
    assert rc == 0
    torch.cuda.synchronize()
    assert torch.equal(pool2, pool) and torch.equal(scales2, scales)  # a full permutation: everything comes back
    del pool, pool2, staging
    free()


def test_config5_token_granular_paging():
    """Page size 1: 28 layers x K/V of 4 x 128 fp16; 1 048 576 random slots of a 2 M-slot pool gathered into 65 536
    storage blocks of 16 tokens (staging [65536][56][16][512])."""
    bgs = _bgs()
    dev = torch.device("cuda")
    P, T, D, n_slots, B = 56, 16, 512, 2 * 1024 * 1024, 65536
    pool = torch.empty((P, n_slots, D), dtype=torch.int16, device=dev)
    fill_pool(pool)
    table = torch.tensor([pool[p].data_ptr() for p in range(P)], dtype=torch.int64, device=dev)
    perm = np.random.default_rng(2).permutation(n_slots).astype(np.int32)
    idx = torch.from_numpy(perm[:B * T]).to(dev)
    staging = torch.zeros((B, P, T, D), dtype=torch.int16, device=dev)
    slots = torch.arange(B, dtype=torch.int32, device=dev)
    print("config5 gather", flush=True)
    bgs.batch_gather_kv_caches(table, staging, idx, slots, T, D)
    for p in range(P):
        assert torch.equal(staging[:, p].reshape(B * T, D), pattern(p, idx, D, dev)), p
    print("config5 scatter", flush=True)
    idx2 = torch.from_numpy(perm[B * T:]).to(dev)  # the other million slots
    bgs.batch_scatter_kv_caches(table, staging, idx2, slots, T, D)
    for p in range(P):
        assert torch.equal(pool[p][idx2.to(torch.int64)], pattern(p, idx, D, dev)), p
        assert torch.equal(pool[p][idx.to(torch.int64)], pattern(p, idx, D, dev)), p
    del pool, staging
    free()
