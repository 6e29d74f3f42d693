#!/usr/bin/env python3
"""bench.py -- the save/load hot path at the Llama-3-8B KV layout on one MI355X.

One "step" = one pass of the hot path over one batch of synthetic input, inputs resident in HBM:
    hash   block keys of 64 requests x 4096 tokens (16-token blocks -> 16 384 keys)
    save   gather the batch's 12 416 unique KV blocks (32 layers x K/V, 8 heads x 128 dims, bf16) from the paged
           pool (32 768 blocks per layer) into block-major staging
    load   scatter the same staged blocks into 12 416 other free blocks of the pool
`value` = algorithmic bytes of one step / wall time of one step, in GB/s (1e9). Per-kernel durations come from
events recorded on the launch stream inside the timed region.

After the timed steps the same process measures, outside `value`: the block-key kernel at other chain counts, the
reference-signature call (Python-list indices, one transfer task of 128 blocks, index upload inside the timed
region), the kernel on one contiguous buffer (the chip's own read+write ceiling), the other four benchmark
configurations at their full sizes (key `configs`), and the CPU path on this host's cores (key `cpu_baseline`).

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--pool-blocks N] [--no-cpu-baseline] [--no-configs]

Prints ONE JSON line. Runs on one GPU only.
"""
import argparse
import hashlib
import itertools
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0  # MI355X HBM3E, published peak

# HBM bytes per launch from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, scaled by a plain 8 GiB copy in the same run
# (profiles/copy_span_llama3_8b_hbm_traffic.md, profiles/hash_tokens_16384_chains_hbm_traffic.md). Counters cannot be
# read from inside this process, so the figures are carried here together with the digest of the kernel sources they
# were measured on: a run whose sources differ reports traffic null and says why.
KERNEL_SOURCES = ("tair_kvcache_amd/csrc/kvcm_copy.hip", "tair_kvcache_amd/csrc/kvcm_hash.hip",
                  "tair_kvcache_amd/csrc/kvcm_internal.h", "tair_kvcache_amd/csrc/kvcm_host_idx.h")
MEASURED_TRAFFIC = {"sources_sha256": "b62a6cdaebc73c73", "unique_blocks": 12416, "gather": 52076736287,
                    "scatter": 52076206605, "hash_saturated": 571049774, "hash_saturated_i32": 302690688, "prefix_chain": 1074210200}

# Llama-3-8B KV layout: the configuration the headline metric is quoted on
LAYERS, KV_HEADS, HEAD_DIM, ITEMSIZE = 32, 8, 128, 2
T = 16
REQUESTS, TOKENS_PER_REQ, VOCAB = 64, 4096, 128256
SHARED_REQS, SHARED_TOKENS = 32, 2048
TASK_BLOCKS = 128  # block_per_save_task / block_per_load_task of the reference connector (vllm/config.py:23-24)

# Dependent VALU instructions of one wave issue 3.65 ns apart on this chip (measured) and one step of the recurrence
# is three of them deep, so one request of n tokens cannot be hashed in less than n x 10.95 ns.
HASH_STEP_FLOOR_NS = 10.95


def kernel_sources_digest():
    h = hashlib.sha256()
    for rel in KERNEL_SOURCES:
        with open(os.path.join(ROOT, rel), "rb") as f:
            h.update(f.read())
    return h.hexdigest()[:16]


def zipf_prefix_tokens(np, requests=1024, length=1024, vocab=152064, block=16, templates=16, s=1.2, seed=0):
    """Token IDs of the page-size-1 configuration: every request starts with a prefix of one of `templates` shared
    sequences and goes on with tokens of its own. The template is drawn Zipf(s) over the template ranks and the prefix
    length Zipf(s) over 4, 8, 12, ... blocks (capped at the request), so a few prefixes are shared by many requests
    and most shared prefixes are short. Returns (tokens int64 [requests, length], template id, prefix length)."""
    rng = np.random.default_rng(seed)
    tok = rng.integers(0, vocab, size=(requests, length), dtype=np.int64)
    shared = rng.integers(0, vocab, size=(templates, length), dtype=np.int64)
    ranks = np.arange(1, templates + 1, dtype=np.float64)
    p_template = ranks ** -s / np.sum(ranks ** -s)
    which = rng.choice(templates, size=requests, p=p_template)
    max_units = length // (4 * block)
    units = np.arange(1, max_units + 1, dtype=np.float64)
    p_len = units ** -s / np.sum(units ** -s)
    plen = rng.choice(max_units, size=requests, p=p_len) + 1
    plen = plen * 4 * block
    for r in range(requests):
        tok[r, :plen[r]] = shared[which[r], :plen[r]]
    return tok, which, plen


def build_inputs(torch, np, pool_blocks, device):
    P = LAYERS * 2
    D = KV_HEADS * HEAD_DIM
    row_bytes = D * ITEMSIZE
    # pool: P arrays [pool_blocks * T, D] bf16 ~ N(0,1), generated on the device (a 64 GiB upload would take minutes)
    pool = torch.empty((P, pool_blocks * T, D), dtype=torch.bfloat16, device=device)
    gen = torch.Generator(device=device)
    gen.manual_seed(1)
    for p in range(P):
        pool[p].normal_(0.0, 1.0, generator=gen)
    ptr_table = torch.tensor([pool[p].data_ptr() for p in range(P)], dtype=torch.int64, device=device)

    rng = np.random.default_rng(0)
    tok = rng.integers(0, VOCAB, size=(REQUESTS, TOKENS_PER_REQ), dtype=np.int64)
    tok[:SHARED_REQS, :SHARED_TOKENS] = tok[0, :SHARED_TOKENS]

    # block tables: disjoint slices of one permutation of the pool; the shared prefix maps to the same blocks
    blocks_per_req = TOKENS_PER_REQ // T
    shared_blocks = SHARED_TOKENS // T
    perm = np.random.default_rng(2).permutation(pool_blocks).astype(np.int32)
    unique = shared_blocks + SHARED_REQS * (blocks_per_req - shared_blocks) + (REQUESTS - SHARED_REQS) * blocks_per_req
    if 2 * unique > pool_blocks:
        raise SystemExit(f"--pool-blocks {pool_blocks} is too small: the workload needs {2 * unique} blocks")
    save_blocks = perm[:unique]            # blocks the batch occupies (gather sources)
    load_blocks = perm[unique:2 * unique]  # other free blocks (scatter targets)
    return dict(P=P, D=D, row_bytes=row_bytes, pool=pool, ptr_table=ptr_table, tokens=tok, unique=unique,
                save_blocks=save_blocks, load_blocks=load_blocks)


def gpu_ms(torch, fn, reps, warm=2):
    """Average milliseconds of one call of fn, from events on the stream the kernels are launched on."""
    for _ in range(warm):
        fn()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(reps):
        fn()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / reps


def copy_figures(ms, nbytes):
    gbps = nbytes / (ms * 1e-3) / 1e9
    return {"ms": round(ms, 4), "GBps": round(gbps, 1), "frac_of_hbm_peak": round(gbps / HBM_PEAK_GBPS, 4)}


def hash_figures(torch, hashing, tokens, block, reps):
    R, L = tokens.shape
    toff = torch.arange(R + 1, dtype=torch.int64, device=tokens.device) * L
    koff = torch.arange(R + 1, dtype=torch.int64, device=tokens.device) * (L // block)
    keys = torch.empty(R * (L // block), dtype=torch.int64, device=tokens.device)
    hashing.hash_tokens(tokens, block, token_offsets=toff, keys=keys, key_offsets=koff)  # the wrapper's checks, once
    from tair_kvcache_amd import _lib
    args = (tokens.data_ptr(), toff.data_ptr(), R, block, 0, keys.data_ptr(), koff.data_ptr(),
            torch.cuda.current_stream().cuda_stream)

    def once():  # straight through the C-ABI: short launches queue up faster than they run
        rc = _lib.lib().kvcm_hip_hash_tokens(*args)
        if rc != 0:
            raise SystemExit(f"bench.py: kvcm_hip_hash_tokens failed with code {rc}")

    ms = gpu_ms(torch, once, reps)
    ms_cold = cold_ms(torch, once, tokens.device)
    return keys, {"hash_chains": R, "tokens_per_chain": L, "block_tokens": block, "keys": keys.numel(),
                  "hash_ms": round(ms, 4), "keys_per_s": round(keys.numel() / (ms * 1e-3)),
                  "hash_ms_cold": round(ms_cold, 4), "keys_per_s_cold": round(keys.numel() / (ms_cold * 1e-3)),
                  "hash_floor_ms": round(L * HASH_STEP_FLOOR_NS * 1e-6, 4)}


def cold_batches_ms(torch, _lib, tokens, token_off, key_off, keys_expected, R, block, n=10, reps=7, sweep_gib=2):
    """(a) Mean milliseconds per launch of n one-batch launches in a row on n DIFFERENT copies of the batch, none of them
    read since a pass over `sweep_gib` GiB of other memory, one pair of events around the n launches: every launch reads
    its tokens from HBM, and no pair of events sits around a single launch. (b) What a pair of events around a single
    launch adds to that launch's reading: per-launch time with an event after every launch minus the mean without, on
    the resident batch. The n key arrays must equal keys_expected (the batch's keys, already checked)."""
    device = tokens.device
    copies = [tokens.clone() for _ in range(n)]
    outs = [torch.zeros_like(keys_expected) for _ in range(n)]
    stream = torch.cuda.current_stream().cuda_stream
    argsets = [(c.data_ptr(), token_off.data_ptr(), R, block, 0, o.data_ptr(), key_off.data_ptr(), stream)
               for c, o in zip(copies, outs)]

    def launch(a):
        rc = _lib.lib().kvcm_hip_hash_tokens(*a)
        if rc != 0:
            raise SystemExit(f"bench.py: kvcm_hip_hash_tokens failed with code {rc}")

    sweep = torch.zeros(sweep_gib * 2**30, dtype=torch.uint8, device=device)
    means = []
    for _ in range(reps):
        sweep.add_(1)
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for a in argsets:
            launch(a)
        e1.record()
        torch.cuda.synchronize()
        means.append(e0.elapsed_time(e1) / n)
    del sweep
    for o in outs:
        if not torch.equal(o, keys_expected):
            raise SystemExit("bench.py: a copy of the batch hashed to other keys than the batch")
    plain, single = [], []
    for _ in range(reps):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(n):
            launch(argsets[0])
        e1.record()
        ev = [torch.cuda.Event(enable_timing=True) for _ in range(n + 1)]
        ev[0].record()
        for i in range(n):
            launch(argsets[0])
            ev[i + 1].record()
        torch.cuda.synchronize()
        plain.append(e0.elapsed_time(e1) / n)
        single.append(sorted(ev[i].elapsed_time(ev[i + 1]) for i in range(n))[n // 2])
    med = lambda v: sorted(v)[len(v) // 2]
    return med(means), med(single) - med(plain)


def cold_ms(torch, fn, device, reps=7, sweep_gib=2):
    """Median milliseconds of one call of fn when every call follows a read-modify-write pass over `sweep_gib` GiB of
    other memory: the 256 MiB memory-side cache and the L2 then hold someone else's dirty lines and the call's inputs
    come from HBM, as they do for tokens that have just arrived (a launch repeated on the same few MiB reads caches)."""
    sweep = torch.zeros(sweep_gib * 2**30, dtype=torch.uint8, device=device)
    times = []
    for _ in range(reps):
        sweep.add_(1)
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        fn()
        e1.record()
        torch.cuda.synchronize()
        times.append(e0.elapsed_time(e1))
    del sweep
    return sorted(times)[len(times) // 2]


def other_configs(torch, np, device, reps=5):
    """Benchmark configurations 1, 3, 4 and 5 (BASELINE.json) at their full sizes, one after the other (memory is released in between):
    save (gather) and load (scatter) milliseconds, GB/s of read+written bytes and the fraction of the HBM peak, and the
    block-key kernel at the configuration's own request count. A sample of every result is checked on the device."""
    from tair_kvcache_amd import _lib, hashing, save_selection
    from tair_kvcache_amd.kernel import batch_gather_scatter_helper as bgs
    out = {}

    def release():
        torch.cuda.synchronize()
        torch.cuda.empty_cache()

    def sample_blocks(B, n=64):  # first, last and a seeded sample: what every configuration's result is checked on
        picks = np.random.default_rng(6).choice(B, size=min(n, B), replace=False).tolist()
        return sorted(set(picks + [0, B - 1]))

    def tokens_uniform(R, L, vocab, seed=0):
        return torch.from_numpy(np.random.default_rng(seed).integers(0, vocab, size=(R, L), dtype=np.int64)).to(device)

    def paged(name, workload, P, D, Tb, pool_blocks, save_b, load_b, tok, hash_block, sets=1):
        """`sets` > 1 (launches of a few microseconds): save_b / load_b hold that many disjoint sets of blocks and every
        launch takes the next set and a staging buffer of its own -- a 48 MiB launch repeated on the same blocks is
        served by the caches (the memory-side cache holds 256 MiB), which is not how a connector's tasks arrive."""
        row_bytes = D * 2
        pool = torch.empty((P, pool_blocks * Tb, D), dtype=torch.int16, device=device)
        pool.random_(-32768, 32767)
        table = torch.tensor([pool[p].data_ptr() for p in range(P)], dtype=torch.int64, device=device)
        B = len(save_b) // sets
        staging = torch.empty((sets, B, P, Tb, D), dtype=torch.int16, device=device)
        slots = torch.arange(B, dtype=torch.int32, device=device)
        d_save = [torch.from_numpy(save_b[i * B:(i + 1) * B] * Tb).to(device) for i in range(sets)]
        d_load = [torch.from_numpy(load_b[i * B:(i + 1) * B] * Tb).to(device) for i in range(sets)]
        nbytes = 2 * B * P * Tb * row_bytes
        # straight through the C-ABI: a 10 us launch must not be timed at the pace of the Python wrapper around it
        L, stream = _lib.lib(), torch.cuda.current_stream().cuda_stream
        tail = (Tb, slots.data_ptr(), B, Tb, row_bytes, 0, stream)
        turn = itertools.count()

        def launch(fn, runs, rotate=True):
            i = next(turn) % sets if rotate else 0
            rc = fn(table.data_ptr(), P, staging[i].data_ptr(), P * Tb * row_bytes, runs[i].data_ptr(), *tail)
            if rc != 0:
                raise SystemExit(f"bench.py: copy launch failed with code {rc}")

        n = reps if nbytes > (1 << 30) else 48
        ms_g = gpu_ms(torch, lambda: launch(L.kvcm_hip_paged_gather, d_save), n, warm=sets)
        ms_s = gpu_ms(torch, lambda: launch(L.kvcm_hip_paged_scatter, d_load), n, warm=sets)
        ok = True
        for i in range(sets):
            for b in sample_blocks(B, 64 // sets + 1):
                s0, l0 = int(save_b[i * B + b]) * Tb, int(load_b[i * B + b]) * Tb
                ok &= bool(torch.equal(staging[i, b], pool[:, s0:s0 + Tb]))
                ok &= bool(torch.equal(staging[i, b], pool[:, l0:l0 + Tb]))
        _, hf = hash_figures(torch, hashing, tok, hash_block, 10)
        out[name] = dict({"workload": workload, "blocks": B, "tile_bytes": Tb * row_bytes,
                          "algorithmic_bytes_per_launch": nbytes, "save": copy_figures(ms_g, nbytes),
                          "load": copy_figures(ms_s, nbytes), "sample_verified": ok}, **hf)
        if sets > 1:  # what the same launch measures when it is repeated on one set of blocks (cache-resident)
            out[name]["block_sets_rotated"] = sets
            out[name]["save_repeated_on_one_set"] = copy_figures(
                gpu_ms(torch, lambda: launch(L.kvcm_hip_paged_gather, d_save, False), n), nbytes)
            out[name]["load_repeated_on_one_set"] = copy_figures(
                gpu_ms(torch, lambda: launch(L.kvcm_hip_paged_scatter, d_load, False), n), nbytes)
        del pool, staging
        release()

    # C1: Qwen2-0.5B-like, 24 layers x K/V, 2 x 64 bf16, 1024-block pool, 128 blocks; 4 x 512 tokens, 256 shared
    perm = np.random.default_rng(2).permutation(1024).astype(np.int32)
    tok = np.random.default_rng(0).integers(0, 151936, size=(4, 512), dtype=np.int64)
    tok[:, :256] = tok[0, :256]
    paged("C1", "Qwen2-0.5B-like: 24 layers x K/V, 2 KV heads x 64, bf16, 16-token blocks, pool of 1024 blocks, 128 "
          "blocks moved (2 x 24 MiB per launch: launch-latency bound), every launch another 128 of the pool's blocks "
          "(four sets each way); 4 requests x 512 tokens hashed",
          48, 128, 16, 1024, perm[:512], perm[512:], torch.from_numpy(tok).to(device), 16, sets=4)

    # C2 under tensor parallelism 8: one rank's share of the Llama-3-8B cache, 1 KV head = 256-byte rows, 4 KiB tiles
    perm = np.random.default_rng(2).permutation(32768).astype(np.int32)
    tok = np.random.default_rng(0).integers(0, VOCAB, size=(REQUESTS, TOKENS_PER_REQ), dtype=np.int64)
    paged("C2_tp8", "Llama-3-8B layout as one rank of TP8 sees it: 32 layers x K/V, 1 KV head x 128, bf16 (256-byte rows, "
          "4 KiB tiles), 16-token blocks, pool of 32768 blocks; 12416 blocks saved and loaded (2 x 3.03 GiB per launch); "
          "the keys are the request's, computed once, not per rank", 64, 128, 16, 32768, perm[:12416], perm[12416:24832],
          torch.from_numpy(tok).to(device), 16)

    # C3: 72B-class, 80 layers x K/V, 8 x 128 bf16, 64-token blocks, 8192-block pool; the 25 % missed blocks of
    # 32 requests x 16384 tokens (2048 blocks, 40 GiB staged)
    perm = np.random.default_rng(2).permutation(8192).astype(np.int32)
    miss = np.concatenate([perm[r * 256 + 192:(r + 1) * 256] for r in range(32)])
    hits = np.concatenate([perm[r * 256:r * 256 + 64] for r in range(32)])
    paged("C3", "72B-class long context: 80 layers x K/V, 8 KV heads x 128, bf16, 64-token blocks, pool of 8192 blocks; "
          "the 2048 missed blocks of 32 requests x 16384 tokens (75 % prefix hits) loaded from 40 GiB of staging "
          "(load is the direction the configuration asks for; save of as many blocks beside it); 32 x 16384 tokens "
          "hashed in 64-token blocks", 160, 1024, 64, 8192, hits, miss, tokens_uniform(32, 16384, 152064), 64)

    # C4: MLA latent cache in fp8 with one fp32 scale per (layer, block) interleaved into the staged record
    L4, T4, row4, nblk4 = 61, 128, 576, 4096
    rec = T4 * row4 + 4
    pool = torch.empty((L4, nblk4 * T4, row4), dtype=torch.uint8, device=device)
    pool.random_(0, 126)  # finite e4m3 codes
    scales = torch.randn((L4, nblk4), dtype=torch.float32, device=device)
    table = torch.tensor([pool[l].data_ptr() for l in range(L4)], dtype=torch.int64, device=device)
    ttable = torch.tensor([scales[l].data_ptr() for l in range(L4)], dtype=torch.int64, device=device)
    blocks = np.random.default_rng(2).permutation(nblk4).astype(np.int32)
    d_blocks = torch.from_numpy(blocks).to(device)
    runs = d_blocks * T4
    staging = torch.empty((nblk4, L4 * rec), dtype=torch.uint8, device=device)
    desc = _lib.CopyDesc()
    desc.d_ptr_table, desc.P, desc.ptrs_per_entry, desc.entry_stride_bytes = table.data_ptr(), L4, 1, 0
    desc.d_staging, desc.staging_block_stride_bytes, desc.staging_tile_stride_bytes = staging.data_ptr(), L4 * rec, rec
    desc.d_run_start, desc.d_staging_idx, desc.B, desc.T, desc.run_tokens = runs.data_ptr(), None, nblk4, T4, T4
    desc.slot_limit, desc.row_bytes = 0, row4
    desc.d_trailer_ptr_table, desc.d_trailer_idx, desc.trailer_bytes = ttable.data_ptr(), d_blocks.data_ptr(), 4
    desc.max_workgroups = 0
    stream = torch.cuda.current_stream().cuda_stream

    def launch(fn):
        rc = fn(desc, stream)
        if rc != 0:
            raise SystemExit(f"bench.py: copy with trailers failed with code {rc}")

    nbytes = 2 * nblk4 * L4 * rec
    ms_g = gpu_ms(torch, lambda: launch(_lib.lib().kvcm_hip_gather_ex), reps)
    ms_s = gpu_ms(torch, lambda: launch(_lib.lib().kvcm_hip_scatter_ex), reps)  # a full permutation: writes every row back
    st = staging.view(nblk4, L4, rec)
    ok = True
    for b in sample_blocks(nblk4):  # payload and the 4 scale bytes behind every tile, both directions (a full permutation)
        s0 = int(blocks[b]) * T4
        ok &= bool(torch.equal(st[b, :, :T4 * row4], pool[:, s0:s0 + T4].reshape(L4, T4 * row4)))
        ok &= bool(torch.equal(st[b, :, T4 * row4:].contiguous().view(torch.float32).reshape(-1), scales[:, int(blocks[b])]))
    _, hf = hash_figures(torch, hashing, tokens_uniform(128, 8192, 129280), 128, 10)
    out["C4"] = dict({"workload": "DeepSeek-V3-style MLA latent cache: 61 layers, 576 e4m3 bytes per token, 128-token "
                                  "blocks, pool of 4096 blocks, one fp32 scale per (layer, block) interleaved behind "
                                  "every 73 728-byte tile (records only 4-byte aligned); one full permutation of the "
                                  "pool (4096 blocks) saved and loaded; 128 requests x 8192 tokens hashed in 128-token "
                                  "blocks", "blocks": nblk4, "tile_bytes": rec, "algorithmic_bytes_per_launch": nbytes,
                      "save": copy_figures(ms_g, nbytes), "load": copy_figures(ms_s, nbytes), "sample_verified": ok}, **hf)
    del pool, staging, scales
    release()

    # C5: page size 1 (token-granular radix-style paging), 28 layers x K/V, 4 x 128 fp16; 1 048 576 random slots of a
    # 2 M-slot pool <-> 65 536 storage blocks of 16 tokens; keys of 1024 requests with Zipf-distributed shared prefixes
    P5, D5, n_slots, B5 = 56, 512, 2 * 1024 * 1024, 65536
    pool = torch.empty((P5, n_slots, D5), dtype=torch.int16, device=device)
    pool.random_(-32768, 32767)
    table = torch.tensor([pool[p].data_ptr() for p in range(P5)], dtype=torch.int64, device=device)
    perm = np.random.default_rng(2).permutation(n_slots).astype(np.int32)
    idx_g, idx_s = torch.from_numpy(perm[:B5 * 16]).to(device), torch.from_numpy(perm[B5 * 16:]).to(device)
    staging = torch.empty((B5, P5, 16, D5), dtype=torch.int16, device=device)
    slots = torch.arange(B5, dtype=torch.int32, device=device)
    nbytes = 2 * B5 * P5 * 16 * D5 * 2
    ms_g = gpu_ms(torch, lambda: bgs.batch_gather_kv_caches(table, staging, idx_g, slots, 16, D5), reps)
    ms_s = gpu_ms(torch, lambda: bgs.batch_scatter_kv_caches(table, staging, idx_s, slots, 16, D5), reps)
    ok = True
    for b in sample_blocks(B5):
        gi, si = idx_g[b * 16:(b + 1) * 16].long(), idx_s[b * 16:(b + 1) * 16].long()
        ok &= bool(torch.equal(staging[b], pool[:, gi])) and bool(torch.equal(staging[b], pool[:, si]))
    tok5, _, _ = zipf_prefix_tokens(np)
    keys5, hf = hash_figures(torch, hashing, torch.from_numpy(tok5).to(device), 16, 10)
    ms_sel = gpu_ms(torch, lambda: save_selection.select_save_indices(keys5), 10)
    _, count = save_selection.select_save_indices(keys5)
    out["C5"] = dict({"workload": "page size 1 (Qwen2.5-7B layout: 28 layers x K/V, 4 KV heads x 128, fp16): 1 048 576 "
                                  "randomly scattered token slots of a 2 M-slot pool <-> 65 536 storage blocks of 16 tokens "
                                  "(token-granular index, 1 KiB rows); keys of 1024 requests x 1024 tokens with "
                                  "Zipf(1.2)-distributed shared prefixes, then first occurrences -> save list on the "
                                  "device", "blocks": B5, "tile_bytes": 16 * D5 * 2, "algorithmic_bytes_per_launch": nbytes,
                      "save": copy_figures(ms_g, nbytes), "load": copy_figures(ms_s, nbytes), "sample_verified": ok,
                      "dedup_ms": round(ms_sel, 4), "unique_keys": int(count.item())}, **hf)
    del pool, staging
    release()
    return out


def cpu_baseline(np, O, threads, host_cores):
    """The CPU path timed on this host: one memcpy per contiguous chunk between a host-resident pool and
    block-major staging (what the reference's storage SDKs do per Iov), and GenKeyVector per request."""
    P, D = LAYERS * 2, KV_HEADS * HEAD_DIM
    row_bytes = D * ITEMSIZE
    pool_blocks, B = 2048, 1024  # 64 arrays x 64 MiB = 4 GiB pool (DRAM-bound), 2 GiB staged
    pools = [np.empty((pool_blocks * T, D), dtype=np.uint16) for _ in range(P)]
    for i, p in enumerate(pools):
        p.fill(i + 1)  # first touch
    staging = np.zeros((B, P * T * D), dtype=np.uint16)
    perm = np.random.default_rng(2).permutation(pool_blocks).astype(np.int32)
    run_g = (perm[:B] * T).astype(np.int32)
    run_s = (perm[B:2 * B] * T).astype(np.int32)
    dg, keep_g = O.make_desc(pools, staging, run_g, None, B, T, row_bytes, run_tokens=T)
    ds, keep_s = O.make_desc(pools, staging, run_s, None, B, T, row_bytes, run_tokens=T)
    moved = 2 * B * P * T * row_bytes  # read + write, one direction

    cpu_seconds = [0.0]

    def timed(fn, seconds):
        """Best of as many repetitions as fit into `seconds` (at least two): about 15 s of CPU work over all legs."""
        best, spent, reps = float("inf"), 0.0, 0
        while reps < 2 or spent < seconds:
            t0 = time.perf_counter()
            fn()
            dt = time.perf_counter() - t0
            best, spent, reps = min(best, dt), spent + dt, reps + 1
        cpu_seconds[0] += spent
        return best

    O.gather_ex(dg, threads=threads)  # warm
    g1 = timed(lambda: O.gather_ex(dg), 2.5)
    s1 = timed(lambda: O.scatter_ex(ds), 2.5)
    gn = timed(lambda: O.gather_ex(dg, threads=threads), 2.5)
    sn = timed(lambda: O.scatter_ex(ds, threads=threads), 2.5)
    del pools, staging

    rng = np.random.default_rng(0)
    tok = rng.integers(0, VOCAB, size=(REQUESTS, TOKENS_PER_REQ), dtype=np.int64)
    nkeys = REQUESTS * (TOKENS_PER_REQ // T)
    h1 = timed(lambda: O.hash_tokens(tok, T), 1.0)
    hn = timed(lambda: O.hash_tokens(tok, T, threads=threads), 1.0)
    # one request per core is only a fair figure on a job that outlasts the start of the threads: 4096 requests of
    # the same shape (128 MiB of tokens), the 64-request batch 64 times over
    big_R = 4096
    big = rng.integers(0, VOCAB, size=(big_R, TOKENS_PER_REQ), dtype=np.int64)
    big_keys = big_R * (TOKENS_PER_REQ // T)
    hb = timed(lambda: O.hash_tokens(big, T, threads=threads), 1.5)
    out = {
        "value": round(2 * moved / (gn + sn) / 1e9, 2), "unit": "GB/s", "cores": threads, "kind": "port",
        "host_cores": host_cores, "threads": threads,
        "thread_cap": "16 = the CPU share of one GPU on these hosts, whatever the core count of the machine",
        "sample": (f"save+load of {B} blocks (2 GiB staged) between a 4 GiB host pool at the same layout and host "
                   f"staging, one memcpy per 32 KiB (layer,K/V,block) chunk, {threads} threads; hash: the 64x4096-token "
                   f"batch on 1 thread and on {threads}, and {big_R} requests of 4096 tokens on {threads} threads; best of "
                   f"the repetitions that fit 2.5 s (copies) or 1-1.5 s (hash) per leg"),
        "save_GBps_1thr": round(moved / g1 / 1e9, 2), "load_GBps_1thr": round(moved / s1 / 1e9, 2),
        "save_GBps": round(moved / gn / 1e9, 2), "load_GBps": round(moved / sn / 1e9, 2),
        "hash_keys_per_s_1thr": round(nkeys / h1), "hash_keys_per_s": round(nkeys / hn),
        "hash_keys_per_s_4096_requests": round(big_keys / hb),
    }
    ref = O.ref()
    if ref is not None:  # the reference's own header, compiled where it lay (oracle/_ref), one request after another
        flat = np.ascontiguousarray(tok).reshape(-1)
        toff = np.arange(REQUESTS + 1, dtype=np.int64) * TOKENS_PER_REQ
        koff = np.arange(REQUESTS + 1, dtype=np.int64) * (TOKENS_PER_REQ // T)
        keys = np.zeros(nkeys, dtype=np.int64)
        hr = timed(lambda: ref.kvcm_refsrc_hash_tokens(flat.ctypes.data, toff.ctypes.data, REQUESTS, T,
                                                      keys.ctypes.data, koff.ctypes.data), 1.0)
        out["hash_keys_per_s_reference_1thr"] = round(nkeys / hr)
    out["cpu_seconds"] = round(cpu_seconds[0], 1)
    return out


def manager_figures(torch, np, inp, pool_blocks, task_bytes, n_tasks, device, workers=32):
    """The connector's own arrangement (data_transfer.py:39-244): DataTransferManager with its 32 worker threads, one
    save and one load stream, every task = nested index lists of 128 blocks -> staging slots from CopyBufferAllocator
    -> gather (scatter) -> event wait -> transfer client. The transfer client here does nothing (returns ER_OK), so
    what is timed is this library's part plus the interpreter lock the 32 threads share."""
    import threading
    from tair_kvcache_amd import client_types, connector
    from tair_kvcache_amd.kernel.gather_scatter_helper import CopyBufferAllocator
    P, D = inp["P"], inp["D"]

    class NullClient:
        def SaveKvCaches(self, uris, buffers):
            return client_types.ClientErrorCode.ER_OK, uris

        def LoadKvCaches(self, uris, buffers):
            return client_types.ClientErrorCode.ER_OK

    info = connector.KVCacheInfo(0, 1, {}, None, None, inp["ptr_table"], LAYERS, pool_blocks * T, (LAYERS, 2, T, D),
                                 P * T * D * ITEMSIZE, D, device, torch.bfloat16)
    alloc = CopyBufferAllocator(device, torch.bfloat16, [P, T, D], workers * TASK_BLOCKS)
    mgr = connector.DataTransferManager(info, T, alloc, NullClient(), max_workers=workers)
    uris = [f"file:///bench?blkid={i}&size={P * T * D * ITEMSIZE}" for i in range(TASK_BLOCKS)]

    def nested(blocks):  # what generate_blocks_idx returns in the reference: one list of T slots per block
        return [[[int(b) * T + t for t in range(T)] for b in blocks[i * TASK_BLOCKS:(i + 1) * TASK_BLOCKS]]
                for i in range(n_tasks)]

    save_idx, load_idx = nested(inp["save_blocks"]), nested(inp["load_blocks"])

    def run(task_fn, idx):
        done = threading.Event()
        mr = connector.MultiResult(n_tasks, lambda results: done.set())
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for i in range(n_tasks):
            mgr.submit_task(task_fn, mr, i, uris, idx[i])
        done.wait()
        return time.perf_counter() - t0

    run(mgr.save_task, save_idx)  # threads, streams and the slot buffer objects come into being here
    run(mgr.load_task, load_idx)
    t_save = min(run(mgr.save_task, save_idx) for _ in range(3))
    t_load = min(run(mgr.load_task, load_idx) for _ in range(3))
    mgr.shutdown()
    del alloc, mgr
    torch.cuda.synchronize()
    torch.cuda.empty_cache()
    moved = n_tasks * task_bytes
    return {"worker_threads": workers, "tasks": n_tasks, "blocks_per_task": TASK_BLOCKS,
            "transfer_client": "none (returns ER_OK): the storage hop is not part of this figure",
            "save_us_per_task": round(t_save / n_tasks * 1e6, 1), "save_GBps": round(moved / t_save / 1e9, 1),
            "save_frac_of_hbm_peak": round(moved / t_save / 1e9 / HBM_PEAK_GBPS, 4),
            "load_us_per_task": round(t_load / n_tasks * 1e6, 1), "load_GBps": round(moved / t_load / 1e9, 1),
            "load_frac_of_hbm_peak": round(moved / t_load / 1e9 / HBM_PEAK_GBPS, 4)}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=2)
    ap.add_argument("--pool-blocks", type=int, default=32768, help="blocks per layer in the paged pool")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-configs", action="store_true", help="skip configurations 1, 3, 4 and 5")
    ap.add_argument("--no-verify", action="store_true")
    ap.add_argument("--calibrate-copy-gib", type=float, default=0.0,
                    help="also run one plain device-to-device copy of this many GiB after the timed region, so that a "
                         "rocprofv3 --pmc run of this command holds a copy kernel of known size to scale counters by")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py measures one GPU: this path has no collectives and every box here has one GPU; "
              "run it with --gpus 1", file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import torch
    from tair_kvcache_amd import _lib, hashing
    from tair_kvcache_amd.kernel import batch_gather_scatter_helper as bgs

    _lib.lib()  # fails loudly when the HIP library is not built
    if not torch.cuda.is_available():
        raise SystemExit("bench.py needs a GPU")
    device = torch.device("cuda:0")
    torch.cuda.set_device(device)

    inp = build_inputs(torch, np, args.pool_blocks, device)
    P, D, row_bytes, unique = inp["P"], inp["D"], inp["row_bytes"], inp["unique"]
    staging = torch.empty((unique, P, T, D), dtype=torch.bfloat16, device=device)
    d_tokens = torch.from_numpy(inp["tokens"]).to(device)
    d_token_off = torch.arange(REQUESTS + 1, dtype=torch.int64, device=device) * TOKENS_PER_REQ
    d_key_off = torch.arange(REQUESTS + 1, dtype=torch.int64, device=device) * (TOKENS_PER_REQ // T)
    d_keys = torch.empty(REQUESTS * (TOKENS_PER_REQ // T), dtype=torch.int64, device=device)
    # device-resident block tables (run start = block id * block size; one run of 16 tokens per block)
    d_save_runs = torch.from_numpy(inp["save_blocks"] * T).to(device)
    d_load_runs = torch.from_numpy(inp["load_blocks"] * T).to(device)
    d_slots = torch.arange(unique, dtype=torch.int32, device=device)

    copy_bytes = 2 * unique * P * T * row_bytes            # read + write, one direction
    hash_bytes = REQUESTS * TOKENS_PER_REQ * 8 + d_keys.numel() * 8
    step_bytes = 2 * copy_bytes + hash_bytes

    def step(ev=None):
        if ev:
            ev[0].record()
        hashing.hash_tokens(d_tokens, T, token_offsets=d_token_off, keys=d_keys, key_offsets=d_key_off)
        if ev:
            ev[1].record()
        bgs.paged_gather_kv_caches(inp["ptr_table"], staging, d_save_runs, d_slots, T, D, T)
        if ev:
            ev[2].record()
        bgs.paged_scatter_kv_caches(inp["ptr_table"], staging, d_load_runs, d_slots, T, D, T)
        if ev:
            ev[3].record()

    # the one batch of the configuration, launched back to back straight through the C-ABI (so that the launches queue
    # up faster than they run), twice: here, before the chip has been streaming for seconds, and after the steps
    hash_args = (d_tokens.data_ptr(), d_token_off.data_ptr(), REQUESTS, T, 0, d_keys.data_ptr(), d_key_off.data_ptr(),
                 torch.cuda.current_stream().cuda_stream)

    def hash_once():
        rc = _lib.lib().kvcm_hip_hash_tokens(*hash_args)
        if rc != 0:
            raise SystemExit(f"bench.py: kvcm_hip_hash_tokens failed with code {rc}")

    torch.cuda.synchronize()
    ms_hash_b2b_first = gpu_ms(torch, hash_once, 20)

    for _ in range(args.warmup):
        step()
    events = [[torch.cuda.Event(enable_timing=True) for _ in range(4)] for _ in range(args.steps)]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for k in range(args.steps):
        step(events[k])
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0

    ms_hash = sum(e[0].elapsed_time(e[1]) for e in events) / args.steps
    ms_gather = sum(e[1].elapsed_time(e[2]) for e in events) / args.steps
    ms_scatter = sum(e[2].elapsed_time(e[3]) for e in events) / args.steps
    ms_step = wall * 1e3 / args.steps

    def spread(i):  # minimum and median over the steps, beside the average that the figures above are built on
        v = sorted(e[i].elapsed_time(e[i + 1]) for e in events)
        return {"min": round(v[0], 4), "median": round(v[len(v) // 2], 4), "max": round(v[-1], 4)}

    per_step = {"hash_ms": spread(0), "save_ms": spread(1), "load_ms": spread(2)}

    if args.calibrate_copy_gib > 0:
        n = int(args.calibrate_copy_gib * 2**30)
        src = staging.view(torch.uint8).reshape(-1)[:n]
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        del dst

    verified = None
    if not args.no_verify:
        # staged bytes of a sample of blocks against the pool rows they came from, and loaded rows against staging
        sample = np.random.default_rng(3).choice(unique, size=64, replace=False)
        ok = True
        for b in sample:
            src = int(inp["save_blocks"][b]) * T
            dst = int(inp["load_blocks"][b]) * T
            ok &= bool(torch.equal(staging[b], inp["pool"][:, src:src + T, :]))
            ok &= bool(torch.equal(staging[b], inp["pool"][:, dst:dst + T, :]))
        from oracle import oracle as O  # the checker, not the measured path
        want, _ = O.hash_tokens(inp["tokens"], T)
        ok &= bool((d_keys.cpu().numpy() == want).all())
        verified = ok
        if not ok:
            raise SystemExit("bench.py: results differ from the oracle; refusing to report a number")

    # ---- the reference-signature call: what data_transfer.py:139-146,206-213 issues per transfer task. Indices are
    # Python lists of B*T token slots and B staging slots; list -> tensor -> device is inside the timed region. Calls are
    # issued back to back (the connector keeps 32 of them in flight from its thread pool); `latency` is one call plus
    # the wait for its completion.
    # Every call takes the next 128 blocks of the save (load) list and the next 128 staging slots, as the connector's
    # tasks do: a task that moved the same 512 MiB over and over would be served by the 256 MiB memory-side cache.
    n_tasks = unique // TASK_BLOCKS

    def task_lists(blocks):
        return [(blocks[i * TASK_BLOCKS:(i + 1) * TASK_BLOCKS, None].astype(np.int64) * T +
                 np.arange(T)[None, :]).reshape(-1).tolist() for i in range(n_tasks)]

    task_tok, task_tok_load = task_lists(inp["save_blocks"]), task_lists(inp["load_blocks"])
    task_slots = [list(range(i * TASK_BLOCKS, (i + 1) * TASK_BLOCKS)) for i in range(n_tasks)]
    task_bytes = 2 * TASK_BLOCKS * P * T * row_bytes
    turn = itertools.count()

    def wall_us(fn, reps):
        fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(reps):
            fn()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / reps * 1e6

    def one_and_wait(fn):
        def f():
            fn()
            torch.cuda.synchronize()
        return f

    def ref_gather():
        i = next(turn) % n_tasks
        bgs.batch_gather_kv_caches(inp["ptr_table"], staging, task_tok[i], task_slots[i], T, D)

    def ref_scatter():
        i = next(turn) % n_tasks
        bgs.batch_scatter_kv_caches(inp["ptr_table"], staging, task_tok_load[i], task_slots[i], T, D)

    d_task_runs = [d_save_runs[i * TASK_BLOCKS:(i + 1) * TASK_BLOCKS].contiguous() for i in range(n_tasks)]
    d_task_slots = [d_slots[i * TASK_BLOCKS:(i + 1) * TASK_BLOCKS].contiguous() for i in range(n_tasks)]

    def fast_gather():
        i = next(turn) % n_tasks
        bgs.paged_gather_kv_caches(inp["ptr_table"], staging, d_task_runs[i], d_task_slots[i], T, D, T)

    us_ref_g, us_ref_s = wall_us(ref_gather, 50), wall_us(ref_scatter, 50)
    reference_signature = {
        "call": "batch_gather_kv_caches / batch_scatter_kv_caches(ptrs, staging, List[int] of 2048 token slots, "
                "List[int] of 128 staging slots, 16, 1024): one transfer task, the lists walked (range checks, run "
                "discovery) and handed to the kernel inside the timed region; every call moves the next 128 of the "
                "12 416 blocks",
        "blocks_per_task": TASK_BLOCKS, "bytes_per_task": task_bytes,
        "save_us_per_task": round(us_ref_g, 1), "save_GBps": round(task_bytes / us_ref_g / 1e3, 1),
        "save_frac_of_hbm_peak": round(task_bytes / us_ref_g / 1e3 / HBM_PEAK_GBPS, 4),
        "load_us_per_task": round(us_ref_s, 1), "load_GBps": round(task_bytes / us_ref_s / 1e3, 1),
        "load_frac_of_hbm_peak": round(task_bytes / us_ref_s / 1e3 / HBM_PEAK_GBPS, 4),
        "save_latency_us": round(wall_us(one_and_wait(ref_gather), 20), 1),
        "load_latency_us": round(wall_us(one_and_wait(ref_scatter), 20), 1),
        "save_us_per_task_device_block_table": round(wall_us(fast_gather, 50), 1),
        "save_kernel_us": round(gpu_ms(torch, fast_gather, 50) * 1e3, 1),
    }
    # host time of one call alone (no GPU wait in it): the list walk, the ctypes call and the launch
    t0 = time.perf_counter()
    for _ in range(200):
        ref_gather()
    reference_signature["save_host_us_per_call"] = round((time.perf_counter() - t0) / 200 * 1e6, 1)
    torch.cuda.synchronize()
    if not args.no_verify:
        # every task once through the list-argument call, gather then scatter, against the device-side answer
        staging.zero_()
        checked = np.random.default_rng(4).choice(n_tasks * TASK_BLOCKS, size=64, replace=False)
        for b in checked:  # the rows these blocks are loaded into start from zero
            dst = int(inp["load_blocks"][b]) * T
            inp["pool"][:, dst:dst + T, :] = 0
        for i in range(n_tasks):
            bgs.batch_gather_kv_caches(inp["ptr_table"], staging, task_tok[i], task_slots[i], T, D,
                                       pool_token_slots=args.pool_blocks * T)
        for i in range(n_tasks):
            bgs.batch_scatter_kv_caches(inp["ptr_table"], staging, task_tok_load[i], task_slots[i], T, D,
                                        pool_token_slots=args.pool_blocks * T)
        torch.cuda.synchronize()
        ok = True
        for b in checked:
            src, dst = int(inp["save_blocks"][b]) * T, int(inp["load_blocks"][b]) * T
            ok &= bool(torch.equal(staging[b], inp["pool"][:, src:src + T, :]))
            ok &= bool(torch.equal(staging[b], inp["pool"][:, dst:dst + T, :]))
        reference_signature["verified"] = ok
        if not ok:
            raise SystemExit("bench.py: the list-argument call moved wrong bytes; refusing to report a number")
    reference_signature["through_DataTransferManager"] = manager_figures(
        torch, np, inp, args.pool_blocks, task_bytes, n_tasks, device)

    # ---- the per-token-index form of the same workload: 16 x 12 416 unrelated token slots, every row (2 KiB) from
    # a place of its own -- what page size 1 makes of this layout, and what the reference's index format always is
    perm_slots = np.random.default_rng(7).permutation(args.pool_blocks * T).astype(np.int32)
    tg_save = torch.from_numpy(perm_slots[:unique * T]).to(device)
    tg_load = torch.from_numpy(perm_slots[unique * T:2 * unique * T]).to(device)
    ms_tg_g = gpu_ms(torch, lambda: bgs.batch_gather_kv_caches(inp["ptr_table"], staging, tg_save, d_slots, T, D), 5)
    ms_tg_s = gpu_ms(torch, lambda: bgs.batch_scatter_kv_caches(inp["ptr_table"], staging, tg_load, d_slots, T, D), 5)
    tg_ok = None
    if not args.no_verify:
        tg_ok = True
        for b in np.random.default_rng(10).choice(unique, size=64, replace=False):
            gi, si = tg_save[b * T:(b + 1) * T].long(), tg_load[b * T:(b + 1) * T].long()
            tg_ok &= bool(torch.equal(staging[b], inp["pool"][:, gi])) and bool(torch.equal(staging[b], inp["pool"][:, si]))
        if not tg_ok:
            raise SystemExit("bench.py: token-granular copy moved wrong bytes; refusing to report a number")
    token_granular = {"workload": f"{unique * T} unrelated token slots of the same pool <-> the same {unique} staging "
                                  "blocks (device-resident int32 index, one entry per token, 2 KiB rows)",
                      "algorithmic_bytes_per_launch": copy_bytes + 4 * unique * T, "save": copy_figures(ms_tg_g, copy_bytes),
                      "load": copy_figures(ms_tg_s, copy_bytes), "sample_verified": tg_ok}
    del tg_save, tg_load

    # ---- the copy kernel on ONE contiguous buffer of the same size (one array, identity block table): what this chip
    # gives a read+write stream, the ceiling the random-block figures are to be read against
    flat_src = inp["pool"].view(torch.int16).reshape(-1)[:unique * P * T * D].view(1, unique * P * T, D)
    flat_table = torch.tensor([flat_src.data_ptr()], dtype=torch.int64, device=device)
    ident = torch.arange(unique, dtype=torch.int32, device=device) * (P * T)
    ms_flat = gpu_ms(torch, lambda: bgs.paged_gather_kv_caches(flat_table, staging.view(unique, 1, P * T, D), ident,
                                                               d_slots, P * T, D, P * T), 5)
    del flat_src
    contiguous = copy_figures(ms_flat, copy_bytes)

    # ---- the block-key kernel at other chain counts
    # 256 batches of the same shape = 16 384 requests (512 MiB of tokens): the HBM-bound regime
    sat_R = 16384
    g = torch.Generator(device=device)
    g.manual_seed(5)
    sat_tokens = torch.randint(0, VOCAB, (sat_R, TOKENS_PER_REQ), dtype=torch.int64, device=device, generator=g)
    sat_keys = torch.empty(sat_R * (TOKENS_PER_REQ // T), dtype=torch.int64, device=device)
    sat_toff = torch.arange(sat_R + 1, dtype=torch.int64, device=device) * TOKENS_PER_REQ
    sat_koff = torch.arange(sat_R + 1, dtype=torch.int64, device=device) * (TOKENS_PER_REQ // T)
    ms_sat = gpu_ms(torch, lambda: hashing.hash_tokens(sat_tokens, T, token_offsets=sat_toff, keys=sat_keys,
                                                       key_offsets=sat_koff), 10, warm=2)
    sat_keys_per_s = sat_keys.numel() / (ms_sat * 1e-3)
    sat_alg_bytes = sat_R * TOKENS_PER_REQ * 8 + (sat_R + 1) * 8 * 2 + sat_keys.numel() * 8
    kpr = TOKENS_PER_REQ // T  # keys per request

    def check_key_sample(tokens, keys, rows, what):
        """Keys of a seeded sample of requests of a big launch against the oracle (outside every timed region)."""
        if args.no_verify:
            return None
        from oracle import oracle as O
        pick = np.sort(np.random.default_rng(8).choice(tokens.shape[0], size=rows, replace=False))
        d_pick = torch.from_numpy(pick).to(device)
        want, _ = O.hash_tokens(tokens[d_pick].cpu().numpy().astype(np.int64), T, threads=min(os.cpu_count() or 1, 16))
        got = keys.view(-1, kpr)[d_pick].cpu().numpy().reshape(-1)
        if not bool((got == want).all()):
            raise SystemExit(f"bench.py: {what}: keys differ from the oracle; refusing to report a number")
        return True

    sat_verified = check_key_sample(sat_tokens, sat_keys, 256, "saturated int64 launch")
    # the same launch on 4-byte token IDs, the width engines hold them in (16 384 x 4096 x 4 B = 256 MiB of tokens)
    sat_tokens32 = sat_tokens.to(torch.int32)
    sat_keys.fill_(0)
    ms_sat32 = gpu_ms(torch, lambda: hashing.hash_tokens(sat_tokens32, T, token_offsets=sat_toff, keys=sat_keys,
                                                         key_offsets=sat_koff), 10, warm=2)
    sat32_args = (sat_tokens32.data_ptr(), sat_toff.data_ptr(), sat_R, T, 0, sat_keys.data_ptr(), sat_koff.data_ptr(),
                  torch.cuda.current_stream().cuda_stream)

    def sat32_once():  # straight through the C-ABI: between the two events there must be the kernel, not the wrapper
        rc = _lib.lib().kvcm_hip_hash_tokens_i32(*sat32_args)
        if rc != 0:
            raise SystemExit(f"bench.py: kvcm_hip_hash_tokens_i32 failed with code {rc}")

    ms_sat32_cold = cold_ms(torch, sat32_once, device)
    sat32_verified = check_key_sample(sat_tokens32, sat_keys, 256, "saturated int32 launch")
    sat32_alg_bytes = sat_R * TOKENS_PER_REQ * 4 + (sat_R + 1) * 8 * 2 + sat_keys.numel() * 8
    roof_hash32 = {"bound": "hbm", "achieved": round(sat32_alg_bytes / (ms_sat32 * 1e-3) / 1e9, 1),
                   "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                   "frac": round(sat32_alg_bytes / (ms_sat32 * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4), "traffic": "filled in below",
                   "kernel": "hash_tokens_kernel<int, 8, 16>", "ms_per_launch": round(ms_sat32, 4),
                   "ms_per_launch_cold": round(ms_sat32_cold, 4),
                   "frac_cold": round(sat32_alg_bytes / (ms_sat32_cold * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4),
                   "algorithmic_bytes_per_launch": sat32_alg_bytes,
                   "keys_per_s": round(sat_keys.numel() / (ms_sat32 * 1e-3)), "verified_against_oracle": sat32_verified,
                   "note": "ms_per_launch repeats the launch on the same 256 MiB of tokens (the loads are non-temporal, "
                           "so they do not stay in the 256 MiB memory-side cache); ms_per_launch_cold follows a pass "
                           "over 2 GiB of other memory"}
    del sat_tokens32
    # four batches of the configuration in one launch (256 chains): the smallest launch that is past 1e9 keys/s, since
    # one batch alone is bound by the latency of its 4096 dependent steps
    few_R = 4 * REQUESTS
    few_keys = few_R * (TOKENS_PER_REQ // T)
    ms_few = gpu_ms(torch, lambda: hashing.hash_tokens(sat_tokens[:few_R], T, token_offsets=sat_toff[:few_R + 1],
                                                       keys=sat_keys[:few_keys], key_offsets=sat_koff[:few_R + 1]), 10)
    few_args = (sat_tokens.data_ptr(), sat_toff.data_ptr(), few_R, T, 0, sat_keys.data_ptr(), sat_koff.data_ptr(),
                torch.cuda.current_stream().cuda_stream)

    def few_once():  # straight through the C-ABI: between the two events there must be the kernel, not the wrapper
        rc = _lib.lib().kvcm_hip_hash_tokens(*few_args)
        if rc != 0:
            raise SystemExit(f"bench.py: kvcm_hip_hash_tokens failed with code {rc}")

    ms_few_cold = cold_ms(torch, few_once, device)
    check_key_sample(sat_tokens[:few_R], sat_keys[:few_keys], few_R, "four batches in one launch")
    # the one batch of the configuration launched back to back: the step's own pair of events also times the
    # hand-over from the 8 ms load kernel before it
    ms_hash_b2b = gpu_ms(torch, hash_once, 20)
    ms_hash_cold = cold_ms(torch, hash_once, device)
    ms_hash_cold_ten, ms_event_pair = cold_batches_ms(torch, _lib, d_tokens, d_token_off, d_key_off, d_keys, REQUESTS, T)
    # ApplyPrefixHash (kv_cache_manager/optimizer/trace_converter/trace_util.cc:47-56) on as many chains: the same
    # 16 384 x 4096 values taken as digests, a key after every step (as many bytes written as read)
    del sat_keys
    chain_keys = torch.empty(sat_R * TOKENS_PER_REQ, dtype=torch.int64, device=device)
    chain_args = (sat_tokens.data_ptr(), sat_toff.data_ptr(), sat_R, chain_keys.data_ptr(),
                  torch.cuda.current_stream().cuda_stream)

    def chain_once():
        rc = _lib.lib().kvcm_hip_prefix_chain(*chain_args)
        if rc != 0:
            raise SystemExit(f"bench.py: kvcm_hip_prefix_chain failed with code {rc}")

    ms_chain = gpu_ms(torch, chain_once, 5, warm=2)
    chain_verified = None
    if not args.no_verify:
        from oracle import oracle as O
        pick = np.sort(np.random.default_rng(9).choice(sat_R, size=256, replace=False))
        d_pick = torch.from_numpy(pick).to(device)
        digests = sat_tokens[d_pick].cpu().numpy()
        want, _ = O.hash_tokens(digests, 1, threads=min(os.cpu_count() or 1, 16))  # block size 1 = the prefix chain
        chain_verified = bool((chain_keys.view(sat_R, TOKENS_PER_REQ)[d_pick].cpu().numpy().reshape(-1) == want).all())
        if not chain_verified:
            raise SystemExit("bench.py: prefix chain: keys differ from the oracle; refusing to report a number")
    chain_bytes = 2 * sat_R * TOKENS_PER_REQ * 8 + (sat_R + 1) * 8
    prefix_chain = {"chains": sat_R, "digests_per_chain": TOKENS_PER_REQ, "ms_per_launch": round(ms_chain, 4),
                    "keys_per_s": round(chain_keys.numel() / (ms_chain * 1e-3)),
                    "algorithmic_bytes_per_launch": chain_bytes,
                    "GBps": round(chain_bytes / (ms_chain * 1e-3) / 1e9, 1),
                    "frac_of_hbm_peak": round(chain_bytes / (ms_chain * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4),
                    "verified_against_oracle": chain_verified}
    del sat_tokens, chain_keys

    digest = kernel_sources_digest()
    traffic_ok = digest == MEASURED_TRAFFIC["sources_sha256"]

    def traffic(which, same_workload):
        if traffic_ok and same_workload:
            return MEASURED_TRAFFIC[which], None
        why = ("the kernel sources differ from the ones the counters were read on" if not traffic_ok
               else "the counters were read on the default workload")
        return None, why

    def roof(ms, which):
        achieved = copy_bytes / (ms * 1e-3) / 1e9
        tr, why = traffic(which, unique == MEASURED_TRAFFIC["unique_blocks"])
        r = {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
             "frac": round(achieved / HBM_PEAK_GBPS, 4), "traffic": tr}
        if why:
            r["traffic_null_because"] = why
        return r

    roof_g, roof_s = roof(ms_gather, "gather"), roof(ms_scatter, "scatter")
    slower_is_gather = ms_gather >= ms_scatter
    dominant = dict(roof_g if slower_is_gather else roof_s,
                    kernel="copy_span_kernel<16, gather>" if slower_is_gather else "copy_span_kernel<16, scatter>",
                    ms_per_launch=round(max(ms_gather, ms_scatter), 4), algorithmic_bytes_per_launch=copy_bytes)
    roof_hash32["traffic"] = traffic("hash_saturated_i32", True)[0]
    prefix_chain["traffic"] = traffic("prefix_chain", True)[0]
    sat_traffic, sat_why = traffic("hash_saturated", True)
    roof_hash = {"bound": "hbm", "achieved": round(sat_alg_bytes / (ms_sat * 1e-3) / 1e9, 1),
                 "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                 "frac": round(sat_alg_bytes / (ms_sat * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4), "traffic": sat_traffic,
                 "kernel": "hash_tokens_kernel<long, 8, 16>", "ms_per_launch": round(ms_sat, 4),
                 "algorithmic_bytes_per_launch": sat_alg_bytes, "verified_against_oracle": sat_verified}
    if sat_why:
        roof_hash["traffic_null_because"] = sat_why

    result = {
        "metric": "KV save/load GB/s (% of HBM peak) + block-keys/s, Llama-3-8B layout, 1 GPU",
        "value": round(step_bytes / (ms_step * 1e-3) / 1e9, 1),
        "unit": "GB/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_step, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "u8", "data": "synthetic",
        "config": {"workload": "Llama-3-8B KV layout (BASELINE configs[1]): 32 layers x K/V, 8 KV heads x 128, bf16, "
                               "16-token blocks; 64 requests x 4096 tokens, 32 share a 2048-token prefix; "
                               "12416 unique blocks saved (gather) and loaded (scatter), 16384 keys hashed",
                   "pool_blocks": args.pool_blocks, "unique_blocks": unique, "staging_GiB": round(copy_bytes / 2 / 2**30, 2),
                   "requests": REQUESTS, "tokens_per_request": TOKENS_PER_REQ, "block_tokens": T},
        "save_GBps": roof_g["achieved"], "save_frac_of_hbm_peak": roof_g["frac"], "save_ms": round(ms_gather, 4),
        "load_GBps": roof_s["achieved"], "load_frac_of_hbm_peak": roof_s["frac"], "load_ms": round(ms_scatter, 4),
        "per_step": per_step,
        "contiguous_copy_same_kernel": contiguous,
        "token_granular_index": token_granular,
        "keys_per_s": round(d_keys.numel() / (ms_hash * 1e-3)), "hash_ms": round(ms_hash, 4), "hash_chains": REQUESTS,
        "hash_ms_back_to_back": round(ms_hash_b2b, 4),
        "keys_per_s_back_to_back": round(d_keys.numel() / (ms_hash_b2b * 1e-3)),
        "hash_ms_back_to_back_before_the_steps": round(ms_hash_b2b_first, 4),
        "hash_ms_cold": round(ms_hash_cold, 4),
        "hash_ms_cold_ten_batches": round(ms_hash_cold_ten, 4),
        "event_pair_around_one_launch_us": round(ms_event_pair * 1e3, 2),
        "hash_floor_us": round(TOKENS_PER_REQ * HASH_STEP_FLOOR_NS * 1e-3, 2),
        "hash_note": "one request is a serial chain of 4096 dependent steps, three dependent VALU instructions each at "
                     "3.65 ns: 64 chains cannot finish in less than hash_floor_us; more than 1e9 keys/s needs 256 or more "
                     "chains in flight (keys_per_s_4_batches). hash_ms is the launch inside the step, behind the 8 ms load kernel; "
                     "the back-to-back figures repeat the launch on tokens that then sit in the caches; hash_ms_cold "
                     "follows a pass over 2 GiB of other memory, which is how a batch that has just arrived is hashed. hash_ms and "
                     "hash_ms_cold are each one launch between its own pair of events, which reads "
                     "event_pair_around_one_launch_us more than the launch takes; hash_ms_cold_ten_batches is the mean of "
                     "ten launches in a row on ten copies of the batch, none read since such a pass, one pair of events "
                     "around the ten",
        "keys_per_s_4_batches": round(few_keys / (ms_few * 1e-3)), "hash_chains_4_batches": few_R,
        "hash_ms_4_batches": round(ms_few, 4), "hash_ms_4_batches_cold": round(ms_few_cold, 4),
        "keys_per_s_4_batches_cold": round(few_keys / (ms_few_cold * 1e-3)),
        "keys_per_s_saturated": round(sat_keys_per_s), "hash_chains_saturated": sat_R,
        "hash_saturated_GBps": round(sat_R * TOKENS_PER_REQ * 8.5 / (ms_sat * 1e-3) / 1e9, 1),
        "verified_against_oracle": verified,
        "roofline": dominant,
        "roofline_hash_saturated": roof_hash,
        "roofline_hash_saturated_i32": roof_hash32,
        "prefix_chain_saturated": prefix_chain,
        "roofline_save": roof_g, "roofline_load": roof_s,
        "reference_signature": reference_signature,
        "kernel_sources_sha256": digest,
    }
    del staging, inp
    torch.cuda.synchronize()
    torch.cuda.empty_cache()
    if not args.no_configs:
        result["configs"] = other_configs(torch, np, device)
    if not args.no_cpu_baseline:
        from oracle import oracle as O
        host_cores = os.cpu_count() or 1
        result["cpu_baseline"] = cpu_baseline(np, O, min(host_cores, 16), host_cores)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
