"""GPU parity of the staging-slot <-> block-file hop: device iovs through the library against the oracle's restatement
of the reference's DoPut / DoGet run on host copies of the same bytes (files compared byte for byte), the reference's
own GPU unit test restated (local_file_sdk_test.cc:97-172), and the whole save -> files -> load path of
DataTransferManager with the staging pool in HBM."""
import os
import threading

import numpy as np
import pytest
import torch

import _cases as cases
from _gpu import dev, host, sync

pytestmark = pytest.mark.gpu


def _uri(path, blkid, size):
    return f"file://{path}?blkid={blkid}&size={size}"


def _giov(t, ignore=False):
    from tair_kvcache_amd import client_types as ct
    return ct.Iov(type=ct.MemoryType.GPU, base=t.data_ptr(), size=t.numel() * t.element_size(), ignore=ignore)


def test_put_get_with_gpu_like_the_reference(tmp_path):
    from tair_kvcache_amd import client_types as ct
    from tair_kvcache_amd.local_file_sdk import LocalFileSdk, StandardUri
    EC = ct.ClientErrorCode
    sdk = LocalFileSdk()
    assert sdk.Init(1024) == EC.ER_OK
    path = str(tmp_path / "local_file" / "test_gpu.txt")
    uri, invalid_uri = _uri(path, 0, 1024), _uri(path, 0, 1023)
    d1, d2 = b"this is local file test", b"and this is another local file test"
    gpu_put = torch.frombuffer(bytearray(d1 + d2), dtype=torch.uint8).cuda()
    buf = ct.BlockBuffer(iovs=[_giov(gpu_put[:len(d1)]), _giov(gpu_put[len(d1):])])
    assert sdk.Put([invalid_uri], [buf])[0] == EC.ER_SDKWRITE_ERROR
    code, actual = sdk.Put([uri], [buf])
    assert code == EC.ER_OK and [u.to_uri_string() for u in actual] == [StandardUri(uri).to_uri_string()]
    gpu_get = torch.zeros(len(d1) + len(d2), dtype=torch.uint8, device="cuda")
    gbuf = ct.BlockBuffer(iovs=[_giov(gpu_get[:len(d1)]), _giov(gpu_get[len(d1):])])
    assert sdk.Get([invalid_uri], [gbuf]) == EC.ER_SDKREAD_ERROR
    assert sdk.Get([uri], [gbuf]) == EC.ER_OK
    assert bytes(gpu_get.cpu().numpy()) == d1 + d2
    sdk.close()


@pytest.mark.parametrize("seed,bounce", [(0, 4096), (1, 4096), (2, 1000), (3, 0), (4, 64), (5, 1 << 20)])
def test_device_iovs_write_the_oracles_file(oracle, tmp_path, seed, bounce):
    """Random blocks of 1-5 iovs each, device and host iovs mixed, some ignored; bounce buffers far smaller than a
    block so that every segment is cut into many chunks."""
    from tair_kvcache_amd import client_types as ct
    from tair_kvcache_amd.local_file_sdk import LocalFileSdk
    EC = ct.ClientErrorCode
    rng = np.random.default_rng(100 + seed)
    bsz = int(rng.choice([4096, 10000, 65536 + 12]))
    sdk = LocalFileSdk()
    assert sdk.Init(bsz, bounce_bytes=bounce, sync_on_put=False) == EC.ER_OK
    ours, theirs = str(tmp_path / "ours.bin"), str(tmp_path / "theirs.bin")
    n_blocks = int(rng.integers(1, 20))
    blkids = rng.permutation(40)[:n_blocks]
    if seed % 2:
        blkids = np.sort(blkids)
    # one device arena; blocks with consecutive ids that are also neighbours in the arena get merged by the library
    arena = rng.integers(0, 256, size=n_blocks * bsz, dtype=np.uint8)
    d_arena = torch.from_numpy(arena).cuda()
    o_blocks, bufs, pieces = [], [], []
    for j, blkid in enumerate(blkids):
        cuts = np.sort(rng.choice(np.arange(1, bsz), size=int(rng.integers(0, 5)), replace=False))
        edges = [0] + cuts.tolist() + [bsz]
        o_iovs, iovs = [], []
        for a, b in zip(edges[:-1], edges[1:]):
            lo, hi = j * bsz + a, j * bsz + b
            kind = rng.random()
            if kind < 0.7:
                o_iovs.append(arena[lo:hi])
                iovs.append(_giov(d_arena[lo:hi]))
                pieces.append(("device", lo, hi, None))
            elif kind < 0.85:
                h = arena[lo:hi].copy()
                o_iovs.append(h)
                iovs.append(ct.Iov(type=ct.MemoryType.CPU, base=h.ctypes.data, size=h.nbytes, ignore=False))
                pieces.append(("host", lo, hi, h))
            else:
                o_iovs.append(hi - lo)
                iovs.append(_giov(d_arena[lo:hi], ignore=True))
                pieces.append(("ignored", lo, hi, None))
        o_blocks.append((int(blkid), o_iovs))
        bufs.append(ct.BlockBuffer(iovs=iovs))
    uris = [_uri(ours, int(b), bsz) for b in blkids]
    print(f"file store case seed={seed} bsz={bsz} bounce={bounce} blocks={n_blocks}", flush=True)
    assert oracle.file_put(theirs, bsz, o_blocks) == 0
    assert sdk.Put(uris, bufs)[0] == EC.ER_OK
    assert open(ours, "rb").read() == open(theirs, "rb").read()
    # back up into a cleared arena (ignored pieces must stay zero), from the ORACLE's file
    d_arena.zero_()
    for kind, lo, hi, h in pieces:
        if kind == "host":
            h[:] = 0
    assert sdk.Get([_uri(theirs, int(b), bsz) for b in blkids], bufs) == EC.ER_OK
    sync()
    got = d_arena.cpu().numpy()
    for kind, lo, hi, h in pieces:
        if kind == "device":
            assert (got[lo:hi] == arena[lo:hi]).all()
        else:
            assert not got[lo:hi].any()
            if kind == "host":
                assert (h == arena[lo:hi]).all()
    sdk.close()


def test_large_merged_run_of_staging_slots(oracle, tmp_path):
    """48 consecutive 1 MiB slots with consecutive block ids are one 48 MiB segment: 6 chunks per bounce buffer."""
    from tair_kvcache_amd import client_types as ct
    from tair_kvcache_amd.local_file_sdk import LocalFileSdk
    bsz, n = 1 << 20, 48
    rng = np.random.default_rng(9)
    data = rng.integers(0, 256, size=n * bsz, dtype=np.uint8)
    d = torch.from_numpy(data).cuda()
    sdk = LocalFileSdk()
    sdk.Init(bsz)
    ours, theirs = str(tmp_path / "big_ours.bin"), str(tmp_path / "big_theirs.bin")
    bufs = [ct.BlockBuffer(iovs=[_giov(d[i * bsz:(i + 1) * bsz])]) for i in range(n)]
    assert sdk.Put([_uri(ours, 5 + i, bsz) for i in range(n)], bufs)[0] == ct.ClientErrorCode.ER_OK
    assert oracle.file_put(theirs, bsz, [(5 + i, [data[i * bsz:(i + 1) * bsz]]) for i in range(n)]) == 0
    assert open(ours, "rb").read() == open(theirs, "rb").read()
    back = torch.zeros_like(d)
    bufs = [ct.BlockBuffer(iovs=[_giov(back[i * bsz:(i + 1) * bsz])]) for i in range(n)]
    assert sdk.Get([_uri(theirs, 5 + i, bsz) for i in range(n)], bufs) == ct.ClientErrorCode.ER_OK
    assert torch.equal(back, d)
    sdk.close()


def test_helper_threads_share_one_get(oracle, tmp_path):
    """A Get of many chunks is split among the store's helper threads: every split (1, 2, 3, 8 and the maximum of 32
    threads; 38 chunks of an odd size, so the ranges are ragged and the last chunk is short) reads the same bytes, a
    second Get reuses the started helpers, and a Get from three callers at once divides them."""
    from tair_kvcache_amd import client_types as ct
    from tair_kvcache_amd.local_file_sdk import LocalFileSdk
    EC = ct.ClientErrorCode
    bsz, n, bounce = 100_000, 37, 99_993  # the 3.7 MB run of slots is one segment of 37 full chunks + 259 bytes
    rng = np.random.default_rng(12)
    data = rng.integers(0, 256, size=n * bsz, dtype=np.uint8)
    theirs = str(tmp_path / "helpers.bin")
    assert oracle.file_put(theirs, bsz, [(i, [data[i * bsz:(i + 1) * bsz]]) for i in range(n)]) == 0
    d = torch.from_numpy(data).cuda()
    uris = [_uri(theirs, i, bsz) for i in range(n)]
    for io in (1, 2, 3, 8, 32):
        sdk = LocalFileSdk()
        assert sdk.Init(bsz, bounce_bytes=bounce, sync_on_put=False, io_threads=io) == EC.ER_OK
        for _ in range(2):
            back = torch.zeros_like(d)
            bufs = [ct.BlockBuffer(iovs=[_giov(back[i * bsz:(i + 1) * bsz])]) for i in range(n)]
            assert sdk.Get(uris, bufs) == EC.ER_OK
            assert torch.equal(back, d), io
        backs = [torch.zeros_like(d) for _ in range(3)]
        codes = [None] * 3

        def reader(k):
            torch.cuda.set_device(0)
            bufs = [ct.BlockBuffer(iovs=[_giov(backs[k][i * bsz:(i + 1) * bsz])]) for i in range(n)]
            codes[k] = sdk.Get(uris, bufs)

        threads = [threading.Thread(target=reader, args=(k,)) for k in range(3)]
        for t in threads:
            t.start()
        for t in threads:
            t.join(120)
        assert codes == [EC.ER_OK] * 3 and all(torch.equal(b, d) for b in backs), io
        sdk.close()


def test_many_threads_share_one_store(oracle, tmp_path):
    """The connector calls its transfer client from a thread pool: every caller gets its own stream and buffers."""
    from tair_kvcache_amd import client_types as ct
    from tair_kvcache_amd.local_file_sdk import LocalFileTransferClient
    bsz, per, n_threads = 256 * 1024, 6, 8
    rng = np.random.default_rng(10)
    data = rng.integers(0, 256, size=(n_threads, per, bsz), dtype=np.uint8)
    d = torch.from_numpy(data).cuda()
    back = torch.zeros_like(d)
    client = LocalFileTransferClient(bsz, bounce_bytes=64 * 1024, sync_on_put=False)
    errors = []

    def worker(i):
        try:
            torch.cuda.set_device(0)
            uris = [_uri(str(tmp_path / f"t{i}.bin"), k, bsz) for k in range(per)]
            code, _ = client.SaveKvCaches(uris, [ct.BlockBuffer(iovs=[_giov(d[i, k])]) for k in range(per)])
            assert code == ct.ClientErrorCode.ER_OK
            code = client.LoadKvCaches(uris, [ct.BlockBuffer(iovs=[_giov(back[i, k])]) for k in range(per)])
            assert code == ct.ClientErrorCode.ER_OK
        except Exception as e:  # noqa: BLE001
            errors.append((i, repr(e)))

    threads = [threading.Thread(target=worker, args=(i,)) for i in range(n_threads)]
    for t in threads:
        t.start()
    for t in threads:
        t.join(120)
    assert not errors, errors
    assert torch.equal(back, d)
    for i in range(n_threads):
        assert open(tmp_path / f"t{i}.bin", "rb").read() == data[i].tobytes()
    client.close()


def test_save_to_files_then_load_through_the_transfer_manager(oracle, tmp_path):
    """tokens -> pool -> gather -> HBM staging -> block files -> HBM staging -> scatter, files checked against the
    oracle's gather written by the oracle's DoPut."""
    from tair_kvcache_amd import connector
    from tair_kvcache_amd.client_types import ClientErrorCode
    from tair_kvcache_amd.kernel.gather_scatter_helper import CopyBufferAllocator
    from tair_kvcache_amd.local_file_sdk import LocalFileTransferClient
    L, nblk, T_eng, T_mgr, H, hd = 3, 64, 16, 32, 4, 32
    rng = np.random.default_rng(4)
    np_caches = [rng.integers(0, 65536, size=(2, nblk, T_eng, H, hd), dtype=np.uint16) for _ in range(L)]
    kv = {f"layer{l}": dev(np_caches[l]).view(torch.float16) for l in range(L)}
    info = connector.register_kv_caches(kv, manager_block_size=T_mgr, local_block_size=T_eng)
    alloc = CopyBufferAllocator(torch.device("cuda"), torch.float16, list(info.per_manager_block_shape), 16)
    bsz = alloc.slot_nbytes
    client = LocalFileTransferClient(bsz, bounce_bytes=32 * 1024)
    mgr = connector.DataTransferManager(info, T_mgr, alloc, client, max_workers=2)
    local_block_ids = cases.block_table(nblk, 24).tolist()
    idx = connector.generate_blocks_idx(list(range(12)), local_block_ids, T_mgr, T_eng)
    # two files of 6 blocks, as the storage backend lays keys out (key_count_per_file blocks per file)
    uris = [_uri(str(tmp_path / "kv" / f"file{i // 6}"), i % 6, bsz) for i in range(12)]
    done, res = threading.Event(), []
    mgr.submit_task(mgr.save_task, connector.MultiResult(1, lambda r: (res.append(r), done.set())), 0, uris, idx, None)
    assert done.wait(60) and res[0] == [[ClientErrorCode.ER_OK] * 12]
    pools = [np_caches[l][k].reshape(nblk * T_eng, H * hd) for l in range(L) for k in (0, 1)]
    want = np.zeros((12, 2 * L, T_mgr, H * hd), dtype=np.uint16)
    oracle.batch_gather(pools, want, host(idx, np.int32), None, T_mgr, H * hd * 2)
    for f in range(2):
        theirs = str(tmp_path / f"oracle_file{f}")
        blocks = [(i, [want[f * 6 + i].reshape(-1).view(np.uint8)]) for i in range(6)]
        assert oracle.file_put(theirs, bsz, blocks) == 0
        assert open(tmp_path / "kv" / f"file{f}", "rb").read() == open(theirs, "rb").read()
    kv2 = {k: torch.zeros_like(v) for k, v in kv.items()}
    mgr2 = connector.DataTransferManager(connector.register_kv_caches(kv2, T_mgr, T_eng), T_mgr, alloc, client,
                                         max_workers=2)
    done2, res2 = threading.Event(), []
    mgr2.submit_task(mgr2.load_task, connector.MultiResult(1, lambda r: (res2.append(r), done2.set())), 0, uris, idx)
    assert done2.wait(60) and res2[0] == [[ClientErrorCode.ER_OK] * 12]
    touched = np.array(local_block_ids)
    for l in range(L):
        g = host(kv2[f"layer{l}"].view(torch.int16), np.uint16)
        assert (g[:, touched] == np_caches[l][:, touched]).all()
    # a missing file fails the load task, and the slots are returned
    done3, res3 = threading.Event(), []
    bad = [_uri(str(tmp_path / "kv" / "nope"), 0, bsz)]
    mgr2.submit_task(mgr2.load_task, connector.MultiResult(1, lambda r: (res3.append(r), done3.set())), 0, bad, idx[:1])
    assert done3.wait(60) and res3[0] == [[ClientErrorCode.ER_SDKREAD_ERROR]]
    assert alloc._inuse_count == 0
    mgr.shutdown()
    mgr2.shutdown()
    client.close()


def test_sglang_page_first_pool_on_the_device(oracle, tmp_path):
    """The page_first_direct pool of py_connector/sglang/test.py:146-151 kept in HBM: two device iovs per block, no
    gather, files equal to the oracle's DoPut of the same bytes."""
    from tair_kvcache_amd import client_types as ct
    from tair_kvcache_amd.local_file_sdk import LocalFileTransferClient
    pages, layers, page_size, heads, dim = 40, 4, 64, 8, 128
    rng = np.random.default_rng(21)
    pool = rng.integers(0, 65536, size=(2, pages, layers, page_size, heads, dim), dtype=np.uint16)
    d_pool = dev(pool)
    piece = layers * page_size * heads * dim * 2
    bsz = 2 * piece
    client = LocalFileTransferClient(bsz, sync_on_put=False)
    page_ids = rng.permutation(pages)[:16].tolist()

    def buffers(t):
        return [ct.BlockBuffer(iovs=[ct.Iov(type=ct.MemoryType.GPU, base=t[kv, pg].data_ptr(), size=piece, ignore=False)
                                     for kv in (0, 1)]) for pg in page_ids]

    path = str(tmp_path / "hicache" / "blocks")
    uris = [_uri(path, i, bsz) for i in range(len(page_ids))]
    code, _ = client.SaveKvCaches(uris, buffers(d_pool))
    assert code == ct.ClientErrorCode.ER_OK
    theirs = str(tmp_path / "oracle_blocks")
    blocks = [(i, [pool[0, pg].reshape(-1).view(np.uint8), pool[1, pg].reshape(-1).view(np.uint8)])
              for i, pg in enumerate(page_ids)]
    assert oracle.file_put(theirs, bsz, blocks) == 0
    assert open(path, "rb").read() == open(theirs, "rb").read()
    back = torch.zeros_like(d_pool)
    assert client.LoadKvCaches([_uri(theirs, i, bsz) for i in range(len(page_ids))], buffers(back)) == 0
    got = host(back, np.uint16)
    for pg in range(pages):
        assert (got[:, pg] == (pool[:, pg] if pg in page_ids else 0)).all()
    client.close()


def test_trtllm_block_major_pool_on_the_device(oracle, tmp_path):
    """TensorRT-LLM's pool is block-major, {blocks, layers, K|V, block_size} (py_connector/trtllm/connector.py:173-179):
    a block is contiguous, the reference copies it to the host (`kv_cache_tensor[block_id].cpu()`, :261-279) and hands
    over a host iov. Here the block leaves as one device iov and comes back the same way."""
    from tair_kvcache_amd import client_types as ct
    from tair_kvcache_amd.local_file_sdk import LocalFileTransferClient
    blocks_n, layers, kv, block_elems = 64, 6, 2, 32 * 4 * 64   # tokens_per_block * heads * head_dim
    rng = np.random.default_rng(22)
    pool = rng.integers(0, 65536, size=(blocks_n, layers, kv, block_elems), dtype=np.uint16)
    d_pool = dev(pool)
    bsz = layers * kv * block_elems * 2                        # location_spec_size (:180)
    client = LocalFileTransferClient(bsz, bounce_bytes=1 << 20, sync_on_put=False)
    block_ids = rng.permutation(blocks_n)[:20].tolist()

    def buffers(t):
        return [ct.BlockBuffer(iovs=[ct.Iov(type=ct.MemoryType.GPU, base=t[b].data_ptr(), size=bsz, ignore=False)])
                for b in block_ids]

    path = str(tmp_path / "trt" / "blocks")
    uris = [_uri(path, i, bsz) for i in range(len(block_ids))]
    assert client.SaveKvCaches(uris, buffers(d_pool))[0] == ct.ClientErrorCode.ER_OK
    theirs = str(tmp_path / "oracle_blocks")
    assert oracle.file_put(theirs, bsz, [(i, [pool[b].reshape(-1).view(np.uint8)]) for i, b in enumerate(block_ids)]) == 0
    assert open(path, "rb").read() == open(theirs, "rb").read()
    back = torch.zeros_like(d_pool)
    assert client.LoadKvCaches([_uri(theirs, i, bsz) for i in range(len(block_ids))], buffers(back)) == 0
    got = host(back, np.uint16)
    for b in range(blocks_n):
        assert (got[b] == (pool[b] if b in block_ids else 0)).all()
    client.close()


def test_copy_iovs_with_device_pieces(oracle):
    """The 3FS client's CopyIovs with device iovs: packed into a pinned I/O buffer and unpacked into fresh device
    memory, against the oracle run on host copies."""
    from tair_kvcache_amd import client_types as ct
    from tair_kvcache_amd.local_file_sdk import copy_iovs
    rng = np.random.default_rng(32)
    arena = rng.integers(0, 256, size=1 << 20, dtype=np.uint8)
    d_arena = torch.from_numpy(arena).cuda()
    cuts = np.sort(rng.choice(np.arange(1, arena.size), size=9, replace=False)).tolist()
    edges = [0] + cuts + [arena.size]
    pieces, iovs = [], []
    for j, (a, b) in enumerate(zip(edges[:-1], edges[1:])):
        if j % 4 == 3:
            pieces.append(b - a)
            iovs.append(_giov(d_arena[a:b], ignore=True))
        elif j % 4 == 1:
            h = arena[a:b].copy()
            pieces.append(h)
            iovs.append(ct.Iov(type=ct.MemoryType.CPU, base=h.ctypes.data, size=h.nbytes, ignore=False))
        else:
            pieces.append(arena[a:b])
            iovs.append(_giov(d_arena[a:b]))
    need = sum(p.nbytes for p in pieces if isinstance(p, np.ndarray))
    theirs = np.zeros(need, dtype=np.uint8)
    assert oracle.copy_iovs(theirs, pieces, load=False) == need
    pinned = torch.zeros(need, dtype=torch.uint8).pin_memory()
    stream = torch.cuda.Stream()
    assert copy_iovs(pinned.data_ptr(), need, iovs, load=False, stream_handle=stream.cuda_stream) == 0
    assert (pinned.numpy() == theirs).all()
    pageable = np.zeros(need, dtype=np.uint8)
    assert copy_iovs(pageable.ctypes.data, need, iovs, load=False) == 0 and (pageable == theirs).all()
    # unpack into a cleared arena: ignored ranges stay zero
    d_arena.zero_()
    assert copy_iovs(pinned.data_ptr(), need, iovs, load=True, stream_handle=stream.cuda_stream) == 0
    got = d_arena.cpu().numpy()
    for j, (a, b) in enumerate(zip(edges[:-1], edges[1:])):
        if j % 4 == 3 or j % 4 == 1:
            assert not got[a:b].any()
        else:
            assert (got[a:b] == arena[a:b]).all()
