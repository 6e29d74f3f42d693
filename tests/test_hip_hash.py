"""GPU parity: block keys from the HIP kernels, through the C-ABI, against the golden vectors and the CPU oracle.
Bit-exact int64."""
import hashlib

import numpy as np
import pytest
import torch

import _cases as cases
from _gpu import dev, host, sync

pytestmark = pytest.mark.gpu


def _h():
    from tair_kvcache_amd import hashing
    return hashing


def test_golden_c1(golden):
    tok = cases.tokens(4, 512, 151936, shared_rows=4, shared_len=256, seed=0)
    assert tok[0, :8].tolist() == golden["c1"]["tokens_row0_first8"]
    keys, off = _h().hash_tokens(dev(tok), 16)
    sync()
    assert host(off, np.int64).tolist() == [0, 32, 64, 96, 128]
    assert host(keys, np.int64).reshape(4, 32).tolist() == golden["c1"]["keys"]
    keys32, _ = _h().hash_tokens(dev(tok.astype(np.int32)), 16)
    sync()
    assert host(keys32, np.int64).reshape(4, 32).tolist() == golden["c1"]["keys"]


def test_golden_cases_single_requests(golden):
    for case in golden["cases"]:
        got = _h().gen_key_vector(case["tokens"], case["block_size"])
        assert got == case["keys"], case["name"]


def test_golden_prefix_chains(golden):
    for ch in golden["prefix_chains"]:
        if not ch["ids"]:
            continue
        got = _h().apply_prefix_hash(torch.tensor(ch["ids"], dtype=torch.int64, device="cuda"))
        sync()
        assert got.tolist() == ch["keys"]


@pytest.mark.parametrize("R,L,bs", [(64, 4096, 16), (1, 16, 16), (3, 1000, 16), (65, 256, 64), (130, 96, 8),
                                    (32, 1024, 128), (7, 333, 7), (5, 64, 1), (200, 40, 24)])
def test_uniform_batches_match_oracle(oracle, R, L, bs):
    print(f"hash case R={R} L={L} bs={bs}", flush=True)
    rng = np.random.default_rng(R * 1000 + L + bs)
    tok = rng.integers(-2**63, 2**63 - 1, size=(R, L), dtype=np.int64)  # full int64 range, both signs
    want, woff = oracle.hash_tokens(tok, bs)
    keys, off = _h().hash_tokens(dev(tok), bs)
    sync()
    assert (host(off, np.int64) == woff).all()
    assert (host(keys, np.int64) == want).all()


def test_ragged_batch_and_seed(oracle):
    rng = np.random.default_rng(3)
    lens = [0, 5, 16, 17, 160, 33, 1024, 31, 4096, 15, 48] + [int(x) for x in rng.integers(0, 700, size=120)]
    toks = [rng.integers(0, 152064, size=n, dtype=np.int64) for n in lens]
    flat = np.concatenate(toks)
    toff = np.zeros(len(lens) + 1, dtype=np.int64)
    np.cumsum(lens, out=toff[1:])
    for bs, seed in [(16, 0), (16, 12345), (5, -7), (64, 0)]:
        want, woff = oracle.hash_tokens(flat, bs, token_offsets=toff, seed=seed)
        keys, off = _h().hash_tokens(dev(flat), bs, token_offsets=dev(toff), seed=seed)
        sync()
        assert (host(off, np.int64) == woff).all()
        assert (host(keys, np.int64) == want).all(), (bs, seed)
    # int32 tokens, ragged (request starts at odd element offsets: 16-byte loads at 4-byte alignment)
    flat32 = flat.astype(np.int32)
    want, _ = oracle.hash_tokens(flat32, 16, token_offsets=toff)
    keys, _ = _h().hash_tokens(dev(flat32), 16, token_offsets=dev(toff))
    sync()
    assert (host(keys, np.int64) == want).all()


@pytest.mark.parametrize("dtype", [np.int64, np.int32])
def test_general_loader_path(oracle, force_general_hash_loader, dtype):
    """The loader form used when a workgroup's requests span 4 GiB or more (32-bit buffer offsets cannot reach),
    taken here from the test-only build in which every launch uses it, on a ragged batch whose last request ends exactly at the end of the buffer."""
    force_general_hash_loader(True)
    rng = np.random.default_rng(17)
    lens = [int(x) for x in rng.integers(0, 900, size=150)] + [64]
    flat = rng.integers(-2**31, 2**31 - 1, size=sum(lens), dtype=np.int64).astype(dtype)
    toff = np.zeros(len(lens) + 1, dtype=np.int64)
    np.cumsum(lens, out=toff[1:])
    want, woff = oracle.hash_tokens(flat, 16, token_offsets=toff)
    keys, off = _h().hash_tokens(dev(flat), 16, token_offsets=dev(toff))
    sync()
    assert (host(keys, np.int64) == want).all()


def test_config2_batch_prefix_property(oracle):
    """64 x 4096 tokens, half the requests share a 2048-token prefix: 128 leading keys shared, the rest distinct."""
    tok = cases.tokens(64, 4096, 128256, shared_rows=32, shared_len=2048, seed=0)
    keys, _ = _h().hash_tokens(dev(tok), 16)
    sync()
    k = host(keys, np.int64).reshape(64, 256)
    want, _ = oracle.hash_tokens(tok, 16)
    assert (k == want.reshape(64, 256)).all()
    assert (k[:32, :128] == k[0, :128]).all()
    assert len(np.unique(k[:, 128])) == 64 and len(np.unique(k[32:, 0])) == 32


@pytest.mark.parametrize("R,L,bs,vocab", [(32, 16384, 64, 152064), (128, 8192, 128, 129280)])
def test_config3_and_config4_batches(oracle, R, L, bs, vocab):
    tok = cases.tokens(R, L, vocab, shared_rows=R // 2, shared_len=(L * 3 // 4 // bs) * bs, seed=0)
    keys, _ = _h().hash_tokens(dev(tok), bs)
    sync()
    want, _ = oracle.hash_tokens(tok, bs, threads=8)
    assert (host(keys, np.int64) == want).all()


def test_config5_many_requests(oracle):
    tok = cases.tokens(1024, 1024, 152064, seed=0)
    keys, _ = _h().hash_tokens(dev(tok), 16)
    sync()
    want, _ = oracle.hash_tokens(tok, 16, threads=8)
    assert (host(keys, np.int64) == want).all()


def test_sha256_keys(oracle):
    rng = np.random.default_rng(6)
    strs = ["", "abc", "é-ü-漢字", "x" * 55, "y" * 56, "z" * 64, "w" * 119, "v" * 120, "u" * 1000]
    strs += ["%064x" % int(x) for x in rng.integers(0, 2**62, size=300)]
    got = _h().sha256_to_int64(strs).tolist()
    want = [int.from_bytes(hashlib.sha256(s.encode("utf-8")).digest()[:8], "big", signed=True) for s in strs]
    assert got == want
    assert got == oracle.sha256_first8_be(strs).tolist()
    keys, n_prefix, n_new = _h().prepare_block_keys(strs[10:20], prefix_keys=strs[:3])
    assert (n_prefix, n_new) == (3, 10) and keys == want[:3] + want[10:20]
    assert _h().prepare_block_keys([], None) == ([], 0, 0)


def test_bad_buffers_are_refused_on_the_host():
    """Short key buffers, offsets of the wrong type, length or device would be out-of-bounds device accesses: ValueError."""
    h = _h()
    tok = torch.zeros(4, 64, dtype=torch.int64, device="cuda")
    with pytest.raises(ValueError):
        h.hash_tokens(tok, 16, keys=torch.empty(15, dtype=torch.int64, device="cuda"))       # 16 keys needed
    with pytest.raises(ValueError):
        h.hash_tokens(tok, 16, keys=torch.empty(16, dtype=torch.int32, device="cuda"))
    with pytest.raises(ValueError):
        h.hash_tokens(tok, 16, keys=torch.empty(16, dtype=torch.int64))                      # keys on the host
    flat = tok.reshape(-1)
    off = torch.arange(5, dtype=torch.int64, device="cuda") * 64
    with pytest.raises(ValueError):
        h.hash_tokens(flat, 16, token_offsets=off.cpu())
    with pytest.raises(ValueError):
        h.hash_tokens(flat, 16, token_offsets=off.to(torch.int32))
    with pytest.raises(ValueError):
        h.hash_tokens(flat, 16, token_offsets=off, key_offsets=torch.zeros(4, dtype=torch.int64, device="cuda"))
    with pytest.raises(ValueError):
        h.apply_prefix_hash(flat, offsets=torch.tensor([0, 256], dtype=torch.int64))         # offsets on the host
    keys, _ = h.hash_tokens(flat, 16, token_offsets=off)                                     # and the good call works
    sync()
    assert keys.numel() == 16


@pytest.mark.parametrize("dtype", [np.int64, np.int32])
@pytest.mark.parametrize("shape", ["uniform", "uniform_odd_count", "ragged", "ragged_short", "two_lengths",
                                   "workgroup_on_every_cu", "every_cu_ragged", "every_cu_two_lengths",
                                   "short_and_long_workgroups"])
def test_many_requests_take_the_staged_key_path(oracle, dtype, shape):
    """In launches of thousands of requests the keys of 16-token blocks are collected in LDS and written out as
    512-byte rows by the loader waves: a sixteenth of a group per tile and the rest after the loop (8-byte tokens, 2048
    to 10 239 requests; workgroups whose requests are shorter than 32 tiles store directly), or a whole group right
    after the barrier that closes it (8-byte tokens from 10 240 requests, 4-byte tokens from 12 288). Groups of tiles in
    which some request has run out, requests past a multiple of 64, and whatever does not fill a group of sixteen tiles
    go the direct way. Every mixture against the oracle, exact."""
    rng = np.random.default_rng(5)
    lens = {
        "uniform": np.full(8192, 2048),                                # two whole groups per request
        "uniform_odd_count": np.full(8192 + 37, 1024 + 64 * 3 + 5),    # one group + three tiles + a tail; last workgroup partial
        "ragged": rng.integers(1100, 3000, size=8300),                 # first group whole for everyone, later ones not
        "ragged_short": rng.integers(0, 1500, size=9000),              # many workgroups with no whole group at all
        "two_lengths": np.where(np.arange(8192) % 64 < 32, 4096, 2048),  # half of every workgroup ends after two groups
        "workgroup_on_every_cu": np.full(16384 + 70, 1024 + 100),      # one group + a tile + a tail; last workgroup partial
        "every_cu_ragged": rng.integers(1100, 3000, size=16384 + 70),
        "every_cu_two_lengths": np.where(np.arange(16384) % 64 < 32, 3072, 1024),
        # workgroups of short requests (direct), of long ones (staged) and of both in one launch of the spread kernel
        "short_and_long_workgroups": np.where((np.arange(4096) // 64) % 3 == 0, 1536, np.where(np.arange(4096) % 5 == 0, 1024, 2560)),
    }[shape].astype(np.int64)
    toff = np.zeros(len(lens) + 1, dtype=np.int64)
    np.cumsum(lens, out=toff[1:])
    if dtype == np.int32:
        flat = rng.integers(-2**31, 2**31 - 1, size=int(toff[-1]), dtype=np.int64).astype(np.int32)
    else:
        flat = rng.integers(-2**63, 2**63 - 1, size=int(toff[-1]), dtype=np.int64)
    print(f"staged keys case {shape} {np.dtype(dtype).name}: {len(lens)} requests, {int(toff[-1])} tokens", flush=True)
    want, woff = oracle.hash_tokens(flat, 16, token_offsets=toff, seed=3, threads=8)
    keys = torch.full((len(want) + 64,), -7, dtype=torch.int64, device="cuda")    # room behind the keys: must stay untouched
    d_koff = dev(woff)
    got, off = _h().hash_tokens(dev(flat), 16, token_offsets=dev(toff), seed=3, keys=keys, key_offsets=d_koff)
    sync()
    assert (host(got, np.int64)[:len(want)] == want).all()
    assert (host(got, np.int64)[len(want):] == -7).all()


@pytest.mark.parametrize("dtype,R,bs", [(np.int64, 16384 + 70, 16), (np.int64, 8300, 16), (np.int32, 12288 + 70, 16),
                                         (np.int64, 300, 1), (np.int64, 2100, 8)])
def test_staged_keys_with_the_general_loader(oracle, force_general_hash_loader, dtype, R, bs):
    """The staged-key forms (spread and burst) are loader code as well: both with the loader that a workgroup spanning
    4 GiB of tokens would take, ragged requests, exact."""
    force_general_hash_loader(True)
    rng = np.random.default_rng(23)
    lens = rng.integers(1030, 2300, size=R).astype(np.int64)
    toff = np.zeros(R + 1, dtype=np.int64)
    np.cumsum(lens, out=toff[1:])
    flat = rng.integers(-2**31, 2**31 - 1, size=int(toff[-1]), dtype=np.int64).astype(dtype)
    print(f"staged keys, general loader: {R} requests of {np.dtype(dtype).name}, block size {bs}, {int(toff[-1])} tokens", flush=True)
    want, woff = oracle.hash_tokens(flat, bs, token_offsets=toff, threads=8)
    keys, off = _h().hash_tokens(dev(flat), bs, token_offsets=dev(toff))
    sync()
    assert (host(keys, np.int64) == want).all()



@pytest.mark.parametrize("dtype,R", [(np.int64, 2048 + 9), (np.int64, 10240 + 9), (np.int32, 12288 + 9), (np.int64, 2047)])
def test_key_offsets_with_gaps_and_odd_starts(oracle, dtype, R):
    """Keys go where key_offsets says, wherever that is: odd first positions (a request's 512-byte rows then start on
    8-byte boundaries only) and gaps between the requests' ranges, which must stay untouched -- on both sides of the
    request counts at which the way keys are written changes."""
    rng = np.random.default_rng(31)
    lens = rng.integers(2100, 2300, size=R).astype(np.int64)
    lens[::7] = 1024 + 48                                                # some requests end early in every workgroup
    toff = np.zeros(R + 1, dtype=np.int64)
    np.cumsum(lens, out=toff[1:])
    flat = rng.integers(-2**31, 2**31 - 1, size=int(toff[-1]), dtype=np.int64).astype(dtype)
    want, woff = oracle.hash_tokens(flat, 16, token_offsets=toff, seed=-5, threads=8)
    counts = lens // 16
    gaps = rng.integers(0, 4, size=R)
    koff = np.zeros(R + 1, dtype=np.int64)
    koff[0] = 1
    koff[1:] = 1 + np.cumsum(counts + gaps)
    print(f"gapped key offsets: {R} requests of {np.dtype(dtype).name}, {int(koff[-1])} key slots", flush=True)
    keys = torch.full((int(koff[-1]) + 64,), -7, dtype=torch.int64, device="cuda")
    got, _ = _h().hash_tokens(dev(flat), 16, token_offsets=dev(toff), seed=-5, keys=keys, key_offsets=dev(koff))
    sync()
    got = host(got, np.int64)
    expect = np.full(got.shape, -7, dtype=np.int64)
    for r in range(R):
        expect[koff[r]:koff[r] + counts[r]] = want[woff[r]:woff[r + 1]]
    assert (got == expect).all()


@pytest.mark.parametrize("bs,dtype", [(1, np.int64), (8, np.int64), (32, np.int64), (64, np.int64), (8, np.int32),
                                      (1, np.int32), (128, np.int64)])
def test_staged_keys_at_other_block_sizes(oracle, bs, dtype):
    """In launches of many requests the keys of 1-, 8-, 32-, 64- and 128-token blocks are staged too (a group is as many
    tiles as yield 64 keys per request: 1, 8, 32, 64, 128 tiles) and leave a group at a time. Ragged requests of one to three
    groups, some ending early, the last workgroup partial; exact against the oracle, spare key slots untouched."""
    group_tokens = 64 * max(bs, 1) if bs > 1 else 64
    rng = np.random.default_rng(41 + bs)
    R = (10240 if dtype == np.int64 else 12288) + 37   # past every threshold of the launch rule
    lens = rng.integers(group_tokens + 70, (3 if bs < 128 else 1.5) * group_tokens, size=R).astype(np.int64)
    lens[::9] = group_tokens // 2 + 5
    toff = np.zeros(R + 1, dtype=np.int64)
    np.cumsum(lens, out=toff[1:])
    flat = rng.integers(-2**31, 2**31 - 1, size=int(toff[-1]), dtype=np.int64).astype(dtype)
    print(f"staged keys, block size {bs}: {R} requests of {np.dtype(dtype).name}, {int(toff[-1])} tokens", flush=True)
    want, woff = oracle.hash_tokens(flat, bs, token_offsets=toff, seed=11, threads=8)
    keys = torch.full((len(want) + 64,), -7, dtype=torch.int64, device="cuda")
    got, off = _h().hash_tokens(dev(flat), bs, token_offsets=dev(toff), seed=11, keys=keys, key_offsets=dev(woff))
    sync()
    got = host(got, np.int64)
    assert (got[:len(want)] == want).all()
    assert (got[len(want):] == -7).all()


@pytest.mark.parametrize("general_loader", [False, True])
@pytest.mark.parametrize("bs", [8, 16, 32, 64, 128])
def test_raw_tiles_of_4_byte_tokens(oracle, force_general_hash_loader, bs, general_loader):
    """Launches of 12 288 requests or more of 4-byte tokens use tiles of 128 RAW tokens per request (the chain wave
    sign-extends and adds the constant itself) and write their keys as whole rows. Request lengths sit on and around
    the tile width (64, 127, 128, 129, 192, 256, ...), on multiples of a key group, and in between; every workgroup
    mixes them; tokens cover the whole signed 32-bit range. Both loaders. Exact against the oracle."""
    force_general_hash_loader(general_loader)
    rng = np.random.default_rng(41 + bs)
    R = 12288 + 77                                   # the last workgroup is partial
    group = 64 * bs                                  # tokens that yield one group of staged keys
    menu = np.array([0, 1, bs - 1, bs, 63, 64, 65, 127, 128, 129, 191, 192, 193, 255, 256, 257, 384, 511, 512,
                     group - 1, group, group + 1, group + 128, group + 129, 2 * group, 2 * group + 64 + bs])
    lens = menu[rng.integers(0, len(menu), size=R)].astype(np.int64)
    lens[rng.random(R) < 0.3] = rng.integers(0, 2 * group + 300)      # and anything in between
    lens[:64] = 2 * group + 128                      # one workgroup of equal, whole requests: every group staged
    lens[64:128] = np.where(np.arange(64) % 2 == 0, group + 128, 2 * group)
    scale = max(1, int(lens.sum() // 40_000_000) + 1)                 # keep the launch under ~160 MB of tokens
    if scale > 1:
        lens[128:] = lens[128:] // scale
    toff = np.zeros(R + 1, dtype=np.int64)
    np.cumsum(lens, out=toff[1:])
    flat = rng.integers(-2**31, 2**31, size=int(toff[-1]), dtype=np.int64).astype(np.int32)
    flat[:16] = [-2**31, 2**31 - 1, -1, 0, 1, -2, 2**31 - 2, -2**31 + 1] * 2
    print(f"raw tiles: bs={bs} general_loader={general_loader} R={R} tokens={int(toff[-1])}", flush=True)
    want, woff = oracle.hash_tokens(flat, bs, token_offsets=toff, seed=-3)
    keys = torch.full((len(want) + 64,), -7, dtype=torch.int64, device="cuda")
    got, off = _h().hash_tokens(dev(flat), bs, token_offsets=dev(toff), seed=-3, keys=keys, key_offsets=dev(woff))
    sync()
    got = host(got, np.int64)
    assert (got[:len(want)] == want).all()
    assert (got[len(want):] == -7).all()
