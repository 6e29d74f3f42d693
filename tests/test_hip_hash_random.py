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
