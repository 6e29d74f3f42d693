#!/usr/bin/env python3
"""bench.py -- the save/load hot path at the Llama-3-8B KV layout on one MI355X.

One "step" = one pass of the hot path over one batch of synthetic input, inputs resident in HBM:
    hash   block keys of 64 requests x 4096 tokens (16-token blocks -> 16 384 keys)
    save   gather the batch's 12 416 unique KV blocks (32 layers x K/V, 8 heads x 128 dims, bf16) from the paged
           pool (32 768 blocks per layer) into block-major staging
    load   scatter the same staged blocks into 12 416 other free blocks of the pool
`value` = algorithmic bytes of one step / wall time of one step, in GB/s (1e9). Per-kernel durations come from
events recorded on the launch stream inside the timed region.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--pool-blocks N] [--no-cpu-baseline]

Prints ONE JSON line. Runs on one GPU only.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0  # MI355X HBM3E, published peak

# HBM bytes per launch of the two copy kernels at the default workload, from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE
# scaled by a plain 8 GiB copy in the same run (profiles/copy_span_llama3_8b_hbm_traffic.md). Counters cannot be read
# from inside this process, so the figures are carried here and reported only for the workload they were taken on.
MEASURED_TRAFFIC = {"unique_blocks": 12416, "gather": 52077746636, "scatter": 52079466648,
                    "hash_saturated": int((512.6 + 38.4) * 2**20)}

# Llama-3-8B KV layout: the configuration the headline metric is quoted on
LAYERS, KV_HEADS, HEAD_DIM, ITEMSIZE = 32, 8, 128, 2
T = 16
REQUESTS, TOKENS_PER_REQ, VOCAB = 64, 4096, 128256
SHARED_REQS, SHARED_TOKENS = 32, 2048


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


def cpu_baseline(np, O, cores):
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

    O.gather_ex(dg, threads=cores)  # warm
    g1 = timed(lambda: O.gather_ex(dg), 2.5)
    s1 = timed(lambda: O.scatter_ex(ds), 2.5)
    gn = timed(lambda: O.gather_ex(dg, threads=cores), 2.5)
    sn = timed(lambda: O.scatter_ex(ds, threads=cores), 2.5)

    rng = np.random.default_rng(0)
    tok = rng.integers(0, VOCAB, size=(REQUESTS, TOKENS_PER_REQ), dtype=np.int64)
    nkeys = REQUESTS * (TOKENS_PER_REQ // T)
    h1 = timed(lambda: O.hash_tokens(tok, T), 1.5)
    hn = timed(lambda: O.hash_tokens(tok, T, threads=cores), 1.5)
    out = {
        "value": round(2 * moved / (gn + sn) / 1e9, 2), "unit": "GB/s", "cores": cores, "kind": "port",
        "sample": (f"save+load of {B} blocks (2 GiB staged) between a 4 GiB host pool at the same layout and host "
                   f"staging, one memcpy per 32 KiB (layer,K/V,block) chunk, {cores} threads; 64x4096-token hash batch; "
                   f"best of the repetitions that fit 2.5 s (copies) or 1.5 s (hash) per leg"),
        "save_GBps_1thr": round(moved / g1 / 1e9, 2), "load_GBps_1thr": round(moved / s1 / 1e9, 2),
        "save_GBps": round(moved / gn / 1e9, 2), "load_GBps": round(moved / sn / 1e9, 2),
        "hash_keys_per_s_1thr": round(nkeys / h1), "hash_keys_per_s": round(nkeys / hn),
    }
    ref = O.ref()
    if ref is not None:  # the reference's own header, compiled where it lay (oracle/_ref), one request after another
        flat = np.ascontiguousarray(tok).reshape(-1)
        toff = np.arange(REQUESTS + 1, dtype=np.int64) * TOKENS_PER_REQ
        koff = np.arange(REQUESTS + 1, dtype=np.int64) * (TOKENS_PER_REQ // T)
        keys = np.zeros(nkeys, dtype=np.int64)
        hr = timed(lambda: ref.kvcm_refsrc_hash_tokens(flat.ctypes.data, toff.ctypes.data, REQUESTS, T,
                                                      keys.ctypes.data, koff.ctypes.data), 1.5)
        out["hash_keys_per_s_reference_1thr"] = round(nkeys / hr)
    out["cpu_seconds"] = round(cpu_seconds[0], 1)
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=2)
    ap.add_argument("--pool-blocks", type=int, default=32768, help="blocks per layer in the paged pool")
    ap.add_argument("--no-cpu-baseline", action="store_true")
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
        sample = np.random.default_rng(3).choice(unique, size=16, replace=False)
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

    # hash throughput with many chains in flight: 256 batches of the same shape = 16 384 requests (512 MiB of tokens)
    sat_R = 16384
    g = torch.Generator(device=device)
    g.manual_seed(5)
    sat_tokens = torch.randint(0, VOCAB, (sat_R, TOKENS_PER_REQ), dtype=torch.int64, device=device, generator=g)
    sat_keys = torch.empty(sat_R * (TOKENS_PER_REQ // T), dtype=torch.int64, device=device)
    sat_toff = torch.arange(sat_R + 1, dtype=torch.int64, device=device) * TOKENS_PER_REQ
    sat_koff = torch.arange(sat_R + 1, dtype=torch.int64, device=device) * (TOKENS_PER_REQ // T)
    hashing.hash_tokens(sat_tokens, T, token_offsets=sat_toff, keys=sat_keys, key_offsets=sat_koff)
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(3):
        hashing.hash_tokens(sat_tokens, T, token_offsets=sat_toff, keys=sat_keys, key_offsets=sat_koff)
    e1.record()
    torch.cuda.synchronize()
    ms_sat = e0.elapsed_time(e1) / 3
    sat_keys_per_s = sat_keys.numel() / (ms_sat * 1e-3)
    sat_alg_bytes = sat_R * TOKENS_PER_REQ * 8 + (sat_R + 1) * 8 * 2 + sat_keys.numel() * 8
    # ... and with four batches of the configuration hashed in one launch (256 chains): the smallest launch that is
    # past 1e9 keys/s, since one batch alone is bound by the latency of its 4096 dependent steps
    few_R = 4 * REQUESTS
    few_keys = few_R * (TOKENS_PER_REQ // T)
    e0.record()
    for _ in range(10):
        hashing.hash_tokens(sat_tokens[:few_R], T, token_offsets=sat_toff[:few_R + 1], keys=sat_keys[:few_keys],
                            key_offsets=sat_koff[:few_R + 1])
    e1.record()
    torch.cuda.synchronize()
    few_keys_per_s = few_keys / (e0.elapsed_time(e1) / 10 * 1e-3)
    # ... and the one batch of the configuration launched ten times back to back: the step's own pair of events also
    # times the hand-over from the 8 ms load kernel before it
    e0.record()
    for _ in range(10):
        hashing.hash_tokens(d_tokens, T, token_offsets=d_token_off, keys=d_keys, key_offsets=d_key_off)
    e1.record()
    torch.cuda.synchronize()
    ms_hash_b2b = e0.elapsed_time(e1) / 10
    del sat_tokens, sat_keys

    def roof(ms, which):
        achieved = copy_bytes / (ms * 1e-3) / 1e9
        traffic = MEASURED_TRAFFIC[which] if unique == MEASURED_TRAFFIC["unique_blocks"] else None
        return {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                "frac": round(achieved / HBM_PEAK_GBPS, 4), "traffic": traffic}

    roof_g, roof_s = roof(ms_gather, "gather"), roof(ms_scatter, "scatter")
    slower_is_gather = ms_gather >= ms_scatter
    dominant = dict(roof_g if slower_is_gather else roof_s,
                    kernel="copy_span_kernel<16, gather>" if slower_is_gather else "copy_span_kernel<16, scatter>",
                    ms_per_launch=round(max(ms_gather, ms_scatter), 4), algorithmic_bytes_per_launch=copy_bytes)

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
        "keys_per_s": round(d_keys.numel() / (ms_hash * 1e-3)), "hash_ms": round(ms_hash, 4), "hash_chains": REQUESTS,
        "hash_ms_back_to_back": round(ms_hash_b2b, 4),
        "keys_per_s_4_batches": round(few_keys_per_s), "hash_chains_4_batches": few_R,
        "keys_per_s_saturated": round(sat_keys_per_s), "hash_chains_saturated": sat_R,
        "hash_saturated_GBps": round(sat_R * TOKENS_PER_REQ * 8.5 / (ms_sat * 1e-3) / 1e9, 1),
        "verified_against_oracle": verified,
        "roofline": dominant,
        # the block-key kernel at 16 384 chains: tokens + offsets read, keys written; traffic from the same two
        # rocprofv3 --pmc runs as the copy kernels (512.6 MiB read + 38.4 MiB written)
        "roofline_hash_saturated": {"bound": "hbm",
                                    "achieved": round(sat_alg_bytes / (ms_sat * 1e-3) / 1e9, 1),
                                    "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                                    "frac": round(sat_alg_bytes / (ms_sat * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4),
                                    "traffic": MEASURED_TRAFFIC["hash_saturated"] if sat_R == 16384 else None,
                                    "kernel": "hash_tokens_kernel<long, 8, 16>", "ms_per_launch": round(ms_sat, 4),
                                    "algorithmic_bytes_per_launch": sat_alg_bytes},
        "roofline_save": roof_g, "roofline_load": roof_s,
    }
    if not args.no_cpu_baseline:
        from oracle import oracle as O
        cores = min(os.cpu_count() or 1, 16)
        result["cpu_baseline"] = cpu_baseline(np, O, cores)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
