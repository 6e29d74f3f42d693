"""Pins the oracle's SHA-256 key mapping and iov CRC (no GPU): hashlib / zlib and the reference's known answers."""
import hashlib
import zlib

import numpy as np


def test_sha256_fips_vectors(oracle):
    vectors = {
        b"": "e3b0c44298fc1c149afbf4c8996fb92427ae41e4649b934ca495991b7852b855",
        b"abc": "ba7816bf8f01cfea414140de5dae2223b00361a396177a9cb410ff61f20015ad",
        b"abcdbcdecdefdefgefghfghighijhijkijkljklmklmnlmnomnopnopq":
            "248d6a61d20638b8e5c026930c3e6039a33ce45964ff2167f6ecedd419db06c1",
    }
    for msg, hexd in vectors.items():
        assert oracle.sha256(msg).hex() == hexd
    assert oracle.sha256(b"a" * 1000).hex() == hashlib.sha256(b"a" * 1000).hexdigest()


def test_sha256_every_length_across_padding(oracle):
    rng = np.random.default_rng(5)
    for n in list(range(0, 130)) + [183, 184, 185, 247, 248, 249, 1000]:
        msg = rng.integers(0, 256, size=n, dtype=np.uint8).tobytes()
        assert oracle.sha256(msg) == hashlib.sha256(msg).digest(), n


def test_sha256_to_int64(oracle):
    # sglang/connector.py:397-401: first 8 digest bytes, big endian, signed
    rng = np.random.default_rng(6)
    keys = ["", "abc", "é-ü-漢字"] + ["%064x" % int(x) for x in rng.integers(0, 2**62, size=50)]
    want = [int.from_bytes(hashlib.sha256(k.encode("utf-8")).digest()[:8], "big", signed=True) for k in keys]
    got = oracle.sha256_first8_be(keys).tolist()
    assert got == want
    assert any(w < 0 for w in want) and any(w > 0 for w in want)


def _buf(s):
    return np.frombuffer(s, dtype=np.uint8).copy()


def test_crc_reference_known_answers(oracle):
    # kv_cache_manager/client/src/internal/sdk/test/sdk_buffer_check_util_test.cc:13-59
    s = b"1234xxxxxxxx5678"
    assert oracle.iov_crc32([_buf(s)], 8).tolist() == [0xDE28307C]  # whole string
    assert oracle.iov_crc32([_buf(s)], 4).tolist() == [0x9AE0DAAF]  # crc32("12345678")
    assert oracle.iov_crc32([_buf(b"1278")], 2).tolist() == [0xF639698C]  # min(4, 4 // 2) = 2 bytes per end
    assert zlib.crc32(b"1234xxxxxxxx5678") == 0xDE28307C and zlib.crc32(b"12345678") == 0x9AE0DAAF


def test_crc_against_zlib(oracle):
    rng = np.random.default_rng(8)
    bufs = [rng.integers(0, 256, size=n, dtype=np.uint8) for n in (2, 8, 9, 1024, 4097)]
    for cal in (1, 4, 8):
        usable = [b for b in bufs if b.nbytes >= 2 * cal or b.nbytes >= cal]
        got = oracle.iov_crc32(usable, cal)
        for b, g in zip(usable, got):
            raw = b.tobytes()
            assert int(g) == zlib.crc32(raw[:cal] + raw[len(raw) - cal:])


def test_blocks_hash_fold(oracle):
    crcs = np.array([1, 2, 3, 4, 5, 6], dtype=np.uint32)
    got = oracle.blocks_hash_from_crcs(crcs, 3).tolist()
    want = []
    for blk in (crcs[:3], crcs[3:]):
        h = 0
        for c in blk:
            h = oracle.py_hash_step(h, int(c))
        want.append(h)
    assert got == want
    # CRCs enter zero-extended, never sign-extended
    big = np.array([0xFFFFFFFF], dtype=np.uint32)
    assert oracle.blocks_hash_from_crcs(big, 1).tolist() == [oracle.py_hash_step(0, 0xFFFFFFFF)]
