"""Block files: the URI parser against the reference's own known answers (common/test/standard_uri_test.cc), the
reference's LocalFileSdk unit tests restated on host iovs (client/src/internal/sdk/test/local_file_sdk_test.cc:26-95),
and the product's files byte for byte against the oracle's restatement of DoPut / DoGet. No GPU: host iovs never
touch the device runtime."""
import os

import numpy as np
import pytest

from tair_kvcache_amd import client_types as ct
from tair_kvcache_amd.local_file_sdk import LocalFileSdk, LocalFileTransferClient, StandardUri, copy_iovs

EC = ct.ClientErrorCode


def test_uri_known_answers_of_the_reference():
    u = StandardUri.from_uri("redis://user:pw@127.0.0.1:6379/abc/def?retry_count=2&timeout_ms=2000")
    assert (u.protocol, u.user_info, u.hostname, u.port, u.path) == ("redis", "user:pw", "127.0.0.1", 6379, "/abc/def")
    assert u.get_param("retry_count") == "2" and u.get_param("timeout_ms") == "2000"
    u = StandardUri.from_uri("redis://127.0.0.1:6379/")
    assert (u.user_info, u.hostname, u.port, u.path, u.get_param("retry_count")) == ("", "127.0.0.1", 6379, "/", "")
    u = StandardUri.from_uri("file:///tmp/kvcm")
    assert (u.protocol, u.hostname, u.port, u.path) == ("file", "", 0, "/tmp/kvcm")
    u = StandardUri.from_uri("file://nfs_01/tmp/test1/test.txt?offset=1&length=2")
    assert u.valid() and (u.hostname, u.path) == ("nfs_01", "/tmp/test1/test.txt")
    u.set_param("new_param", "v1")
    r = StandardUri.from_uri(u.to_uri_string())
    assert (r.hostname, r.path, r.get_param("offset"), r.get_param("length"), r.get_param("new_param")) == (
        "nfs_01", "/tmp/test1/test.txt", "1", "2", "v1")
    assert u.to_uri_string() == "file://nfs_01/tmp/test1/test.txt?length=2&new_param=v1&offset=1"   # std::map order
    u = StandardUri.from_uri("file://?offset=1&length=2")
    assert u.valid() and (u.hostname, u.path, u.get_param("offset"), u.get_param("length")) == ("", "", "1", "2")
    u = StandardUri.from_uri("file:///?offset=1&length=2")
    assert (u.hostname, u.path, u.get_param("length")) == ("", "/", "2")
    u = StandardUri.from_uri("file:///tmp/file?param1=&param2&param3=val3")
    assert (u.path, u.get_param("param1"), u.get_param("param2"), u.get_param("param3")) == ("/tmp/file", "", "", "val3")
    u = StandardUri.from_uri("redis://user:pw@127.0.0.1")
    assert (u.user_info, u.hostname, u.port) == ("user:pw", "127.0.0.1", 0)
    assert not StandardUri.from_uri("redis://user:pw@127.0.0.1:abcd/").valid()
    assert not StandardUri.from_uri("no-protocol-here").valid()
    # GetParamAs<uint64_t>: only a value that is a number from end to end replaces the default
    u = StandardUri("file:///f?blkid=12&size=12x")
    assert u.get_param_as_uint("blkid") == 12 and u.get_param_as_uint("size", 7) == 7 and u.get_param_as_uint("no") == 0


def _iov(arr, ignore=False):
    return ct.Iov(type=ct.MemoryType.CPU, base=arr.ctypes.data, size=arr.nbytes, ignore=ignore)


def _uri(path, blkid, size):
    return f"file://{path}?blkid={blkid}&size={size}"


def test_init_like_the_reference():
    sdk = LocalFileSdk()
    assert sdk.Init(None) == EC.ER_INVALID_SDKBACKEND_CONFIG
    assert sdk.Init(-1) == EC.ER_INVALID_SDKBACKEND_CONFIG
    assert sdk.Init(1024, io_threads=33) == EC.ER_INVALID_SDKBACKEND_CONFIG
    assert sdk.Init(1024, io_threads=-1) == EC.ER_INVALID_SDKBACKEND_CONFIG
    assert sdk.Init(1024) == EC.ER_OK
    sdk.close()


def test_put_get_with_cpu_like_the_reference(tmp_path):
    sdk = LocalFileSdk()
    assert sdk.Init(1024) == EC.ER_OK
    path = str(tmp_path / "local_file" / "test.txt")
    uri, invalid_uri = _uri(path, 0, 1024), _uri(path, 0, 1023)
    d1 = np.frombuffer(b"this is local file test", dtype=np.uint8).copy()
    d2 = np.frombuffer(b"and this is another local file test", dtype=np.uint8).copy()
    buf = ct.BlockBuffer(iovs=[_iov(d1), _iov(d2)])
    code, actual = sdk.Put([invalid_uri], [buf])
    assert code == EC.ER_SDKWRITE_ERROR
    code, actual = sdk.Put([uri], [buf])
    assert code == EC.ER_OK and len(actual) == 1
    assert actual[0].to_uri_string() == StandardUri(uri).to_uri_string()
    assert os.path.getsize(path) == 1024
    raw = open(path, "rb").read()
    assert raw[:len(d1) + len(d2)] == d1.tobytes() + d2.tobytes() and set(raw[len(d1) + len(d2):]) == {0}
    g1, g2 = np.zeros_like(d1), np.zeros_like(d2)
    gbuf = ct.BlockBuffer(iovs=[_iov(g1), _iov(g2)])
    assert sdk.Get([invalid_uri], [gbuf]) == EC.ER_SDKREAD_ERROR
    assert sdk.Get([uri], [gbuf]) == EC.ER_OK
    assert (g1 == d1).all() and (g2 == d2).all()
    # counts must agree; a file that is not there cannot be read
    assert sdk.Get([uri, uri], [gbuf]) == EC.ER_INVALID_PARAMS
    assert sdk.Put([uri, uri], [buf])[0] == EC.ER_INVALID_PARAMS
    assert sdk.Get([_uri(str(tmp_path / "missing"), 0, 1024)], [gbuf]) == EC.ER_SDKREAD_ERROR
    sdk.close()


def _random_blocks(rng, bsz, n_blocks, max_blkid):
    """(blkid, [iov spec]) with iov specs as oracle._file_call takes them; total size per block <= bsz."""
    blkids = rng.permutation(max_blkid + 1)[:n_blocks]
    blocks = []
    for blkid in blkids:
        left, iovs = bsz, []
        while left > 0 and len(iovs) < 6:
            size = int(rng.integers(1, left + 1))
            kind = rng.random()
            if kind < 0.7:
                iovs.append(rng.integers(0, 256, size=size, dtype=np.uint8))
            elif kind < 0.85:
                iovs.append(size)              # ignored
            else:
                iovs.append(("null", size))    # null base
            left -= size
            if rng.random() < 0.2:
                break
        blocks.append((int(blkid), iovs))
    return blocks


def _buffers(blocks, out=False):
    bufs = []
    for _, iovs in blocks:
        items = []
        for v in iovs:
            if isinstance(v, np.ndarray):
                items.append(_iov(v))
            elif isinstance(v, tuple):
                items.append(ct.Iov(type=ct.MemoryType.CPU, base=0, size=v[1], ignore=False))
            else:
                items.append(ct.Iov(type=ct.MemoryType.CPU, base=1, size=v, ignore=True))
        bufs.append(ct.BlockBuffer(iovs=items))
    return bufs


@pytest.mark.parametrize("seed", range(6))
def test_files_equal_the_oracles_byte_for_byte(oracle, tmp_path, seed):
    rng = np.random.default_rng(seed)
    bsz = int(rng.choice([64, 1000, 4096]))
    sdk = LocalFileSdk()
    assert sdk.Init(bsz, sync_on_put=bool(seed % 2)) == EC.ER_OK
    ours, theirs = str(tmp_path / "deep" / "dir" / "ours.bin"), str(tmp_path / "theirs.bin")
    for round_ in range(3):   # later puts overwrite some blocks and grow the file
        blocks = _random_blocks(rng, bsz, int(rng.integers(1, 12)), 8 + 8 * round_)
        assert oracle.file_put(theirs, bsz, blocks) == 0
        code, _ = sdk.Put([_uri(ours, b, bsz) for b, _ in blocks], _buffers(blocks))
        assert code == EC.ER_OK
        assert open(ours, "rb").read() == open(theirs, "rb").read()
    # read back through the other implementation, with fresh destination arrays of the same shapes
    mine = [(b, [np.zeros_like(v) if isinstance(v, np.ndarray) else v for v in iovs]) for b, iovs in blocks]
    ref = [(b, [np.zeros_like(v) if isinstance(v, np.ndarray) else v for v in iovs]) for b, iovs in blocks]
    assert oracle.file_get(ours, bsz, ref) == 0
    assert sdk.Get([_uri(theirs, b, bsz) for b, _ in mine], _buffers(mine)) == EC.ER_OK
    for (_, src), (_, a), (_, b) in zip(blocks, mine, ref):
        for s, x, y in zip(src, a, b):
            if isinstance(s, np.ndarray):
                assert (x == s).all() and (y == s).all()
    sdk.close()


def test_refusals_match_the_oracle(oracle, tmp_path):
    bsz = 256
    sdk = LocalFileSdk()
    sdk.Init(bsz)
    ours, theirs = str(tmp_path / "o.bin"), str(tmp_path / "t.bin")
    big = np.arange(300, dtype=np.uint8)
    ok = np.arange(200, dtype=np.uint8)
    # an iov that reaches beyond (max blkid + 1) * bsz is refused ...
    assert oracle.file_put(theirs, bsz, [(0, [big])]) == -1
    assert sdk.Put([_uri(ours, 0, bsz)], [ct.BlockBuffer(iovs=[_iov(big)])])[0] == EC.ER_SDKWRITE_ERROR
    # ... but a block may spill into the next one when the file is long enough (no per-block bound in the reference)
    blocks = [(0, [big]), (3, [ok])]
    assert oracle.file_put(theirs, bsz, blocks) == 0
    assert sdk.Put([_uri(ours, 0, bsz), _uri(ours, 3, bsz)], _buffers(blocks))[0] == EC.ER_OK
    assert open(ours, "rb").read() == open(theirs, "rb").read() and os.path.getsize(ours) == 4 * bsz
    # get beyond the end of the file
    dst = np.zeros(200, dtype=np.uint8)
    assert oracle.file_get(theirs, bsz, [(4, [dst])]) == -1
    assert sdk.Get([_uri(ours, 4, bsz)], [ct.BlockBuffer(iovs=[_iov(dst)])]) == EC.ER_SDKREAD_ERROR
    # the URI's size must be the store's block size
    assert oracle.file_put(theirs, bsz, [(0, [ok])], sizes=[255]) == -1
    assert oracle.file_get(theirs, bsz, [(0, [dst])], sizes=[255]) == -1
    # a size that would wrap the offset arithmetic is refused like any other that reaches beyond the file
    huge = ct.Iov(type=ct.MemoryType.CPU, base=ok.ctypes.data, size=2**64 - 8, ignore=False)
    assert sdk.Put([_uri(ours, 0, bsz)], [ct.BlockBuffer(iovs=[_iov(ok[:16]), huge])])[0] == EC.ER_SDKWRITE_ERROR
    assert sdk.Get([_uri(ours, 0, bsz)], [ct.BlockBuffer(iovs=[_iov(dst[:16]), huge])]) == EC.ER_SDKREAD_ERROR
    # a put never shrinks a file
    assert sdk.Put([_uri(ours, 1, bsz)], [ct.BlockBuffer(iovs=[_iov(ok)])])[0] == EC.ER_OK
    assert os.path.getsize(ours) == 4 * bsz
    sdk.close()


def test_blocks_are_grouped_by_file(tmp_path):
    bsz = 128
    client = LocalFileTransferClient(bsz)
    a, b = str(tmp_path / "a.bin"), str(tmp_path / "b.bin")
    data = [np.full(bsz, i + 1, dtype=np.uint8) for i in range(4)]
    uris = [_uri(a, 1, bsz), _uri(b, 0, bsz), _uri(a, 0, bsz), _uri(b, 2, bsz)]
    code, actual = client.SaveKvCaches(uris, [ct.BlockBuffer(iovs=[_iov(d)]) for d in data])
    assert code == EC.ER_OK and sorted(actual) == sorted(StandardUri(u).to_uri_string() for u in uris)
    assert open(a, "rb").read() == bytes([3] * bsz + [1] * bsz)
    assert open(b, "rb").read() == bytes([2] * bsz + [0] * bsz + [4] * bsz)
    back = [np.zeros(bsz, dtype=np.uint8) for _ in range(4)]
    assert client.LoadKvCaches(uris, [ct.BlockBuffer(iovs=[_iov(d)]) for d in back]) == EC.ER_OK
    assert all((x == y).all() for x, y in zip(back, data))
    code, actual = client.SaveKvCaches([_uri(a, 0, bsz + 1)], [ct.BlockBuffer(iovs=[_iov(data[0])])])
    assert code == EC.ER_SDKWRITE_ERROR and actual == []
    client.close()


def test_sglang_page_first_pool_goes_to_files_without_a_gather(oracle, tmp_path):
    """SGLang's host pool in the page_first_direct layout, (2, pages, layers, page_size, heads, dim)
    (py_connector/sglang/test.py:48,146-151): a page's K and V are one contiguous piece each, so the connector hands
    the transfer client two iovs per block (_prepare_buffers, sglang/connector.py:426-440) and nothing is gathered.
    The pool is filled as the reference's test fills it (value = token index)."""
    pages, layers, page_size, heads, dim = 12, 3, 8, 2, 16
    pool = np.zeros((2, pages, layers, page_size, heads, dim), dtype=np.uint16)
    for i in range(pages * page_size):
        pool[:, i // page_size, :, i % page_size] = i
    piece = layers * page_size * heads * dim * 2          # bytes of one page's K (or V)
    bsz = 2 * piece                                       # location_spec_size = size per token * page_size
    client = LocalFileTransferClient(bsz)
    page_ids = [7, 0, 3, 11]

    def buffers(arr):
        out = []
        for pg in page_ids:
            iovs = [ct.Iov(type=ct.MemoryType.CPU, base=arr[kv, pg].ctypes.data, size=piece, ignore=False)
                    for kv in (0, 1)]
            out.append(ct.BlockBuffer(iovs=iovs))
        return out

    path = str(tmp_path / "hicache" / "blocks")
    uris = [_uri(path, i, bsz) for i in range(len(page_ids))]
    code, _ = client.SaveKvCaches(uris, buffers(pool))
    assert code == EC.ER_OK
    raw = np.frombuffer(open(path, "rb").read(), dtype=np.uint16).reshape(len(page_ids), 2, layers, page_size, heads, dim)
    for i, pg in enumerate(page_ids):
        assert (raw[i, 0] == pool[0, pg]).all() and (raw[i, 1] == pool[1, pg]).all()
    theirs = str(tmp_path / "oracle_blocks")
    blocks = [(i, [pool[0, pg].reshape(-1).view(np.uint8), pool[1, pg].reshape(-1).view(np.uint8)])
              for i, pg in enumerate(page_ids)]
    assert oracle.file_put(theirs, bsz, blocks) == 0
    assert open(path, "rb").read() == open(theirs, "rb").read()
    back = np.zeros_like(pool)
    assert client.LoadKvCaches(uris, buffers(back)) == EC.ER_OK
    for pg in range(pages):
        assert (back[:, pg] == (pool[:, pg] if pg in page_ids else 0)).all()
    client.close()


def test_copy_iovs_packs_like_the_oracle(oracle):
    """iovs <-> one I/O buffer (the 3FS client's CopyIovs): ignored iovs take no room, pieces keep their order."""
    rng = np.random.default_rng(31)
    for trial in range(20):
        pieces, iovs = [], []
        for _ in range(int(rng.integers(0, 9))):
            n = int(rng.integers(1, 3000))
            if rng.random() < 0.25:
                pieces.append(n)
                iovs.append(ct.Iov(type=ct.MemoryType.CPU, base=1, size=n, ignore=True))
            else:
                a = rng.integers(0, 256, size=n, dtype=np.uint8)
                pieces.append(a)
                iovs.append(_iov(a))
        need = sum(p.nbytes for p in pieces if isinstance(p, np.ndarray))
        theirs = np.full(need + 64, 0xEE, dtype=np.uint8)
        ours = np.full(need + 64, 0xEE, dtype=np.uint8)
        assert oracle.copy_iovs(theirs, pieces, load=False) == need
        assert copy_iovs(ours.ctypes.data, ours.nbytes, iovs, load=False) == 0
        assert (ours == theirs).all() and (ours[need:] == 0xEE).all()
        # and back out of the buffer into fresh arrays
        outs = [np.zeros_like(p) if isinstance(p, np.ndarray) else p for p in pieces]
        o_iovs = [_iov(o) if isinstance(o, np.ndarray) else ct.Iov(type=ct.MemoryType.CPU, base=1, size=o, ignore=True)
                  for o in outs]
        assert copy_iovs(theirs.ctypes.data, theirs.nbytes, o_iovs, load=True) == 0
        for p, o in zip(pieces, outs):
            if isinstance(p, np.ndarray):
                assert (p == o).all()
        # a buffer that is too small is refused before anything moves
        if need > 1:
            small = np.full(need - 1, 0xEE, dtype=np.uint8)
            assert copy_iovs(small.ctypes.data, small.nbytes, iovs, load=False) == -1
            assert (small == 0xEE).all()
