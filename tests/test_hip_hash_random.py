"""GPU parity of the block-key kernel on many random batches against the CPU oracle: request counts around the
64-request workgroup size, lengths around the 64-token tile size and its multiples, every kind of block size (1, odd,
multiples of 8, larger than a tile, larger than most requests), both token widths, both loader forms, seeds of either
sign, every launch repeated so that a result that depends on timing shows up. Bit-exact int64."""
import numpy as np
import pytest

from _gpu import dev, host, sync

pytestmark = pytest.mark.gpu


def _case(rng):
    R = int(rng.choice([1, 2, 63, 64, 65, 127, 128, 129, int(rng.integers(1, 400))]))
    base = int(rng.choice([0, 1, 63, 64, 65, 127, 128, 129, 191, 192, 193, 320, 383, 384, 385, 448, 1000, 2050]))
    ragged = bool(rng.random() < 0.6)
    if ragged:
        lens = np.maximum(0, base + rng.integers(-70, 71, size=R)).astype(np.int64)
        if rng.random() < 0.3:
            lens[rng.integers(0, R)] = 0
    else:
        lens = np.full(R, base, dtype=np.int64)
    bs = int(rng.choice([1, 2, 3, 7, 8, 16, 16, 16, 24, 31, 32, 64, 72, 128, 200]))
    seed = int(rng.choice([0, 0, 1, -1, 2**62, -2**63]))
    dtype = np.int32 if rng.random() < 0.3 else np.int64
    return R, lens, bs, seed, dtype


@pytest.mark.parametrize("force_global", ["0", "1"])
def test_random_batches(oracle, force_general_hash_loader, force_global):
    from tair_kvcache_amd import hashing
    force_general_hash_loader(force_global == "1")
    rng = np.random.default_rng(77 + int(force_global))
    for i in range(70 if force_global == "0" else 30):
        R, lens, bs, seed, dtype = _case(rng)
        total = int(lens.sum())
        if dtype == np.int32:
            flat = rng.integers(-2**31, 2**31 - 1, size=total, dtype=np.int64).astype(np.int32)
        else:
            flat = rng.integers(-2**63, 2**63 - 1, size=total, dtype=np.int64)
        toff = np.zeros(R + 1, dtype=np.int64)
        np.cumsum(lens, out=toff[1:])
        print(f"hash random case {i} global={force_global}: R={R} lens~{int(lens.mean()) if R else 0} bs={bs} seed={seed} "
              f"{np.dtype(dtype).name}", flush=True)
        want, woff = oracle.hash_tokens(flat, bs, token_offsets=toff, seed=seed)
        d_flat = dev(flat if total else np.zeros(1, dtype=dtype))
        d_toff = dev(toff)
        for rep in range(2):
            keys, off = hashing.hash_tokens(d_flat, bs, token_offsets=d_toff, seed=seed)
            sync()
            assert (host(off, np.int64) == woff).all(), (i, rep)
            assert (host(keys, np.int64) == want).all(), (i, rep, R, bs, seed)


def test_random_launches_of_many_requests(oracle):
    """The same against the oracle for launches of thousands of requests, on both sides of every request count at which
    the way keys reach memory changes, for the block sizes that have staged forms; lengths of one to a few groups of
    tiles, ragged, some requests empty or short, key ranges with gaps."""
    from tair_kvcache_amd import hashing
    rng = np.random.default_rng(123)
    for i in range(18):
        bs = int(rng.choice([1, 8, 16, 16, 32, 64, 128]))
        R = int(rng.choice([1023, 1024, 2047, 2048, 4100, 8191, 8192, 10239, 10240, 12287, 12288, 16390]))
        dtype = np.int32 if rng.random() < 0.4 else np.int64
        group_tokens = 64 * bs if bs > 1 else 64
        top = int(min(max(2.5 * group_tokens, 300), 24_000_000 // R))
        lens = rng.integers(top // 3, top + 1, size=R).astype(np.int64)
        lens[rng.random(R) < 0.05] = rng.integers(0, 40)
        toff = np.zeros(R + 1, dtype=np.int64)
        np.cumsum(lens, out=toff[1:])
        flat = rng.integers(-2**31, 2**31 - 1, size=int(toff[-1]), dtype=np.int64).astype(dtype)
        seed = int(rng.choice([0, -1, 2**62]))
        print(f"hash random large case {i}: R={R} lens {top // 3}..{top} bs={bs} seed={seed} {np.dtype(dtype).name}", flush=True)
        want, woff = oracle.hash_tokens(flat, bs, token_offsets=toff, seed=seed, threads=8)
        counts = lens // bs
        koff = np.zeros(R + 1, dtype=np.int64)
        koff[1:] = np.cumsum(counts + rng.integers(0, 3, size=R))
        import torch
        keys = torch.full((int(koff[-1]) + 16,), -7, dtype=torch.int64, device="cuda")
        got, _ = hashing.hash_tokens(dev(flat), bs, token_offsets=dev(toff), seed=seed, keys=keys, key_offsets=dev(koff))
        sync()
        got = host(got, np.int64)
        expect = np.full(got.shape, -7, dtype=np.int64)
        idx = np.repeat(koff[:-1] - woff[:-1], counts) + np.arange(len(want))
        expect[idx] = want
        assert (got == expect).all(), (i, R, bs, seed)
