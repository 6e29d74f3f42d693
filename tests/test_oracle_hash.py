"""Pins the hash functions of the CPU oracle (no GPU).

Sources of truth, none of which is the oracle's own formula:
  * tests/golden/hash_golden.json -- written by the reference's hash headers compiled as they lie
    (tests/golden/make_hash_golden.py);
  * oracle/_ref -- the same build, live, when it exists in this checkout (random inputs);
  * the closed form of the first step, sign/shift special cases, and a restatement on Python big integers.
"""
import numpy as np
import pytest

C = 0x9E3779B97F4A7C15
M = (1 << 64) - 1


def s64(x):
    x &= M
    return x - (1 << 64) if x >> 63 else x


def test_golden_steps(oracle, golden):
    for st in golden["steps"]:
        assert oracle.hash_step(st["h"], st["v"]) == st["out"], st
        assert oracle.py_hash_step(st["h"], st["v"]) == st["out"], st


def test_golden_cases(oracle, golden):
    for case in golden["cases"]:
        keys = oracle.gen_key_vector(np.array(case["tokens"], dtype=np.int64), case["block_size"])
        assert keys.tolist() == case["keys"], case["name"]


def test_golden_c1_batched(oracle, golden):
    rng = np.random.default_rng(0)
    tok = rng.integers(0, 151936, size=(4, 512), dtype=np.int64)
    tok[:, :256] = tok[0, :256]
    assert tok[0, :8].tolist() == golden["c1"]["tokens_row0_first8"]  # the recipe regenerates the same inputs
    keys, off = oracle.hash_tokens(tok, 16)
    assert off.tolist() == [0, 32, 64, 96, 128]
    assert keys.reshape(4, 32).tolist() == golden["c1"]["keys"]
    # 256 shared tokens = 16 shared blocks
    k = keys.reshape(4, 32)
    assert (k[:, :16] == k[0, :16]).all() and len({int(x) for x in k[:, 16]}) == 4
    # int32 tokens and the threaded variant give the same keys
    k32, _ = oracle.hash_tokens(tok.astype(np.int32), 16)
    kmt, _ = oracle.hash_tokens(tok, 16, threads=3)
    assert (k32 == keys).all() and (kmt == keys).all()


def test_golden_prefix_chains_and_folds(oracle, golden):
    for ch in golden["prefix_chains"]:
        got = oracle.prefix_chain(np.array(ch["ids"], dtype=np.int64))
        assert got.tolist() == ch["keys"]
    for f in golden["u32_folds"]:
        got = oracle.blocks_hash_from_crcs(np.array(f["crcs"], dtype=np.uint32), len(f["crcs"]))
        assert got.tolist() == [f["hash"]]


def test_known_answers_of_the_compiled_reference_header(oracle):
    keys = oracle.gen_key_vector(np.arange(64, dtype=np.int64), 16)
    assert [int(k) & M for k in keys] == [0x5AFC88D355FF4B7B, 0x10B81CF351F85B40, 0x9663CF74B462B173,
                                          0x253717686B900F1B]
    assert oracle.gen_key_vector(np.array([-1, -2**63, 2**63 - 1], dtype=np.int64), 3).tolist() == [
        8024479189367639538]


def test_closed_forms(oracle):
    # from h = 0 both shift terms vanish: H(0, v) = v + C (mod 2^64)
    for v in (0, 1, 456, -1, 2**63 - 1, -2**63):
        assert oracle.hash_step(0, v) == s64(v + C)
    assert oracle.hash_step(0, 456) == -7046029254386352675
    # h = -1: (h << 12) = -4096, arithmetic (h >> 32) = -1; a logical shift would give 2^32 - 1 instead
    assert oracle.hash_step(-1, 0) == s64(M ^ ((C - 4096 - 1) & M))
    assert oracle.hash_step(-1, 0) != s64(M ^ ((C - 4096 + (1 << 32) - 1) & M))
    # h = 2^32: (h >> 32) = 1, (h << 12) = 2^44
    assert oracle.hash_step(1 << 32, 7) == s64((1 << 32) ^ ((7 + C + (1 << 44) + 1) & M))
    # top bits shifted out: h = 2^52 -> (h << 12) = 0 mod 2^64, (h >> 32) = 2^20
    assert oracle.hash_step(1 << 52, 0) == s64((1 << 52) ^ ((C + (1 << 20)) & M))


def test_against_python_bigints(oracle):
    rng = np.random.default_rng(7)
    for n, bs in [(1, 1), (17, 4), (200, 16), (129, 64)]:
        tok = rng.integers(-2**63, 2**63 - 1, size=n, dtype=np.int64)
        assert oracle.gen_key_vector(tok, bs).tolist() == oracle.py_gen_key_vector(tok.tolist(), bs)


def test_invariants(oracle):
    rng = np.random.default_rng(11)
    tok = rng.integers(0, 128256, size=1000, dtype=np.int64)
    keys = oracle.gen_key_vector(tok, 16)
    assert len(keys) == 62  # trailing 8 tokens dropped (cache_manager.cc:78)
    # key i depends on tokens [0, 16(i+1)) only
    t2 = tok.copy()
    t2[16 * 30] += 1
    k2 = oracle.gen_key_vector(t2, 16)
    assert (k2[:30] == keys[:30]).all() and (k2[30:] != keys[30:]).all()
    # key i equals the plain fold of the prefix
    for i in (0, 5, 61):
        acc = 0
        for v in tok[:16 * (i + 1)]:
            acc = oracle.hash_step(acc, int(v))
        assert acc == keys[i]
    # ApplyPrefixHash is GenKeyVector with block_size 1
    assert (oracle.prefix_chain(tok) == oracle.gen_key_vector(tok, 1)).all()
    # shorter than a block, and empty
    assert len(oracle.gen_key_vector(tok[:15], 16)) == 0
    assert len(oracle.gen_key_vector(tok[:0], 16)) == 0
    # seed: continuing from key 9 reproduces the tail
    tail = oracle.gen_key_vector(tok[160:], 16, seed=int(keys[9]))
    assert (tail == keys[10:]).all()


def test_ragged_batch(oracle):
    rng = np.random.default_rng(3)
    lens = [0, 5, 16, 17, 160, 33, 1024, 31]
    toks = [rng.integers(0, 1000, size=n, dtype=np.int64) for n in lens]
    flat = np.concatenate(toks)
    off = np.zeros(len(lens) + 1, dtype=np.int64)
    np.cumsum(lens, out=off[1:])
    keys, koff = oracle.hash_tokens(flat, 16, token_offsets=off)
    assert koff.tolist() == [0, 0, 0, 1, 2, 12, 14, 78, 79]
    for r, t in enumerate(toks):
        assert keys[koff[r]:koff[r + 1]].tolist() == oracle.py_gen_key_vector(t.tolist(), 16)


def test_against_reference_source_build(oracle):
    """Live comparison with the reference headers; skipped where oracle/_ref was not built."""
    ref = oracle.ref()
    if ref is None:
        pytest.skip("oracle/_ref not built in this checkout")
    rng = np.random.default_rng(99)
    for _ in range(200):
        h, v = (int(x) for x in rng.integers(-2**63, 2**63 - 1, size=2, dtype=np.int64))
        assert oracle.hash_step(h, v) == ref.kvcm_refsrc_hash_step(h, v)
    for n, bs in [(4096, 16), (1000, 7), (64, 64), (5, 8)]:
        tok = rng.integers(-2**63, 2**63 - 1, size=n, dtype=np.int64)
        want = np.zeros(n // bs, dtype=np.int64)
        ref.kvcm_refsrc_gen_key_vector(tok.ctypes.data, n, bs, want.ctypes.data)
        assert (oracle.gen_key_vector(tok, bs) == want).all()
        chain = np.zeros(n, dtype=np.int64)
        ref.kvcm_refsrc_prefix_chain(tok.ctypes.data, n, chain.ctypes.data)
        assert (oracle.prefix_chain(tok) == chain).all()
    crcs = rng.integers(0, 2**32, size=96, dtype=np.uint64).astype(np.uint32)
    want = ref.kvcm_refsrc_hash_u32_array(crcs.ctypes.data, crcs.ctypes.data + 4 * 96, 0)
    assert oracle.blocks_hash_from_crcs(crcs, 96).tolist() == [want]
