"""GPU parity of the save-selection entry points (first occurrence of block keys in a batch, mask -> ascending index
list) against the CPU oracle. Integer work: exact."""
import numpy as np
import pytest
import torch

import _cases as cases
from _gpu import sync

pytestmark = pytest.mark.gpu


def _keys_with_repeats(rng, n, distinct):
    base = rng.integers(-2**63, 2**63 - 1, size=max(distinct, 1), dtype=np.int64)
    return base[rng.integers(0, max(distinct, 1), size=n)]


@pytest.mark.parametrize("n,distinct", [(1, 1), (2, 1), (63, 5), (64, 64), (1000, 1), (1025, 700), (8192, 8192), (16383, 16383),
                                        (16384, 12416), (16384, 16384), (16385, 9000), (65536, 300), (300000, 150000), (1 << 20, 1 << 20)])
def test_first_occurrence_matches_oracle(oracle, n, distinct):
    from tair_kvcache_amd import save_selection
    rng = np.random.default_rng(n * 7 + distinct)
    keys = _keys_with_repeats(rng, n, distinct)
    if n >= 8:   # extremes and values that differ only in the high or only in the low half
        keys[:8] = [-2**63, 2**63 - 1, 0, -1, 1 << 32, 1, (1 << 32) + 1, -2**63]
    print(f"first_occurrence n={n} distinct={distinct}", flush=True)
    first, rep = save_selection.first_occurrence(torch.from_numpy(keys).cuda())
    sync()
    w_first, w_rep = oracle.first_occurrence(keys)
    assert (first.cpu().numpy() == w_first).all()
    assert (rep.cpu().numpy().astype(np.uint8) == w_rep).all()


def test_first_occurrence_sequential_and_clustered_keys(oracle):
    """Keys that would pile up in a table indexed by low bits: small consecutive integers and multiples of 2^20."""
    from tair_kvcache_amd import save_selection
    for keys in (np.arange(50000, dtype=np.int64) % 20000, (np.arange(50000, dtype=np.int64) % 777) << 20,
                 np.zeros(4096, dtype=np.int64)):
        first, _ = save_selection.first_occurrence(torch.from_numpy(keys).cuda())
        sync()
        assert (first.cpu().numpy() == oracle.first_occurrence(keys)[0]).all()


@pytest.mark.parametrize("n", [0, 1, 63, 64, 1023, 1024, 1025, 4096, 16384, 65535, 65536, 65537, 100000, (1 << 20) + 3, 3 << 20])
@pytest.mark.parametrize("density", [0.0, 0.3, 1.0])
def test_mask_to_indices_matches_oracle(oracle, n, density):
    from tair_kvcache_amd import save_selection
    rng = np.random.default_rng(n + int(density * 10))
    mask = (rng.random(n) < density)
    mask2 = (rng.random(n) < 0.2) if n % 2 else None
    print(f"mask_to_indices n={n} density={density}", flush=True)
    idx, count = save_selection.mask_to_indices(torch.from_numpy(mask).cuda(),
                                                None if mask2 is None else torch.from_numpy(mask2).cuda())
    sync()
    want = oracle.mask_to_indices(mask, mask2)
    assert int(count.item()) == len(want)
    assert (idx[:len(want)].cpu().numpy() == want).all()


def test_parse_block_mask_to_save_indices_like_the_reference(oracle):
    from tair_kvcache_amd import save_selection
    rng = np.random.default_rng(5)
    values = (rng.random(300) < 0.5).tolist()
    for response, target in (({"block_mask": {"bool_masks": {"values": values}}}, 300),
                             ({"block_mask": {"offset": 17}}, 64), ({"block_mask": {"offset": 64}}, 64),
                             ({"block_mask": {"bool_masks": {"values": []}}}, 0), ({}, 9)):
        assert (save_selection.parse_block_mask_to_save_indices(response, target)
                == oracle.py_parse_block_mask_to_save_indices(response, target))


def test_config2_batch_keys_to_unique_blocks(oracle):
    """Llama-3-8B batch: 64 requests x 4096 tokens, 32 of them share a 2048-token prefix => of the 16 384 block keys
    12 416 are first occurrences. Keys, dedup and index list all computed on the device."""
    from tair_kvcache_amd import hashing, save_selection
    toks = cases.tokens(64, 4096, 128256, shared_rows=32, shared_len=2048)
    keys, _ = hashing.hash_tokens(torch.from_numpy(toks).cuda(), 16)
    saved = torch.zeros(keys.numel(), dtype=torch.bool, device="cuda")
    saved[5000:5100] = True   # the manager says these are stored already
    idx, count = save_selection.select_save_indices(keys, saved)
    idx_all, count_all = save_selection.select_save_indices(keys)
    sync()
    assert int(count_all.item()) == 12416
    w_keys = np.concatenate([np.array(oracle.gen_key_vector(t, 16), dtype=np.int64) for t in toks])
    assert (keys.cpu().numpy() == w_keys).all()
    _, w_rep = oracle.first_occurrence(w_keys)
    assert (idx_all[:12416].cpu().numpy() == oracle.mask_to_indices(w_rep)).all()
    want = oracle.mask_to_indices(saved.cpu().numpy(), w_rep)
    assert int(count.item()) == len(want) and (idx[:len(want)].cpu().numpy() == want).all()


def test_workspace_is_checked():
    from tair_kvcache_amd import _lib
    L = _lib.lib()
    keys = torch.zeros(4096, dtype=torch.int64, device="cuda")
    out = torch.zeros(4096, dtype=torch.int32, device="cuda")
    need = L.kvcm_hip_first_occurrence_workspace_bytes(4096)
    assert need == 8192 * 4
    ws = torch.zeros(need // 4, dtype=torch.int32, device="cuda")
    assert L.kvcm_hip_first_occurrence(keys.data_ptr(), 4096, ws.data_ptr(), need - 4, out.data_ptr(), None,
                                       None) == _lib.ERR_INVALID_ARG
    assert L.kvcm_hip_first_occurrence(keys.data_ptr(), 4096, ws.data_ptr() + 2, need, out.data_ptr(), None,
                                       None) == _lib.ERR_ALIGNMENT
    assert L.kvcm_hip_first_occurrence(keys.data_ptr(), 4096, ws.data_ptr(), need, out.data_ptr(), None, None) == 0
    sync()
    assert (out == 0).all()


def test_config5_zipf_shared_prefixes_hash_dedup_gather(oracle):
    """The page-size-1 configuration's key workload at its own sharing pattern and scale: 1024 requests x 1024 tokens
    whose shared prefixes are Zipf(1.2)-distributed over 16 templates -> 65 536 keys -> first occurrence of every key
    -> ascending save list -> gather of exactly those storage blocks (token-granular index). Keys, masks and index
    list are compared with the oracle, the staged rows with the pool rows they name. Exact."""
    import bench
    from tair_kvcache_amd import hashing, save_selection
    from tair_kvcache_amd.kernel import batch_gather_scatter_helper as bgs
    toks, which, plen = bench.zipf_prefix_tokens(np)
    assert toks.shape == (1024, 1024) and len(set(which.tolist())) > 4 and plen.min() >= 64 and plen.max() <= 1024
    print("config5 zipf: hash", flush=True)
    keys, koff = hashing.hash_tokens(torch.from_numpy(toks).cuda(), 16)
    first, rep = save_selection.first_occurrence(keys)
    idx, count = save_selection.select_save_indices(keys)
    sync()
    w_keys, _ = oracle.hash_tokens(toks, 16)
    assert (keys.cpu().numpy() == w_keys).all()
    w_first, w_rep = oracle.first_occurrence(w_keys)
    assert (first.cpu().numpy() == w_first).all() and (rep.cpu().numpy().astype(np.uint8) == w_rep).all()
    want_idx = oracle.mask_to_indices(w_rep)
    n = int(count.item())
    assert n == len(want_idx) and (idx[:n].cpu().numpy() == want_idx).all()
    # what the sharing pattern implies, derived from the generator's own draws and not from any hash: a block is new
    # unless an earlier request uses the same template at least that far
    expect_new = 0
    longest = {}
    for r in range(1024):
        t, blocks = int(which[r]), int(plen[r]) // 16
        expect_new += 64 - min(blocks, longest.get(t, 0))
        longest[t] = max(longest.get(t, 0), blocks)
    assert n == expect_new and n < 65536
    # gather the blocks to save: storage block k of the batch = 16 token slots of a 2^20-slot pool (4 arrays, 1 KiB rows)
    P, D, n_slots = 4, 512, 1 << 20
    pool = torch.randint(-32768, 32767, (P, n_slots, D), dtype=torch.int16, device="cuda")
    table = torch.tensor([pool[p].data_ptr() for p in range(P)], dtype=torch.int64, device="cuda")
    slot_of_token = torch.from_numpy(np.random.default_rng(2).permutation(n_slots).astype(np.int32)).cuda()
    tidx = slot_of_token.view(65536, 16)[idx[:n].long()].contiguous()      # [n, 16] token slots of the blocks to save
    staging = torch.zeros((n, P, 16, D), dtype=torch.int16, device="cuda")
    print(f"config5 zipf: gather {n} of 65536 blocks", flush=True)
    bgs.batch_gather_kv_caches(table, staging, tidx, torch.arange(n, dtype=torch.int32, device="cuda"), 16, D)
    sync()
    for p in range(P):
        assert torch.equal(staging[:, p].reshape(n * 16, D), pool[p][tidx.reshape(-1).long()]), p
