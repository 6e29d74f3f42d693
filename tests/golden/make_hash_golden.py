"""Writes tests/golden/hash_golden.json from the REFERENCE's own hash headers.

Run in the build container only (the reference tree must be present):
    make -C oracle ref && python tests/golden/make_hash_golden.py

Every expected value below is produced by oracle/_ref/libkvcm_refhash.so, i.e. by
kv_cache_manager/manager/hash_util.h and kv_cache_manager/common/hash_util.h compiled as they lie; the
restatement in oracle/kvcm_oracle.c is never consulted here. The fixture holds inputs (or the seed and recipe
that regenerate them with NumPy) and expected outputs only.
"""
import ctypes
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)
from oracle import oracle as O  # noqa: E402


def c1_tokens():
    """Tokens of the smallest benchmark configuration: 4 requests x 512, uniform in [0,151936), first 256 shared. Seed 0."""
    rng = np.random.default_rng(0)
    tok = rng.integers(0, 151936, size=(4, 512), dtype=np.int64)
    tok[:, :256] = tok[0, :256]
    return tok


def ref_keys(ref, tokens, block_size):
    tokens = np.ascontiguousarray(tokens, dtype=np.int64)
    keys = np.zeros(len(tokens) // block_size, dtype=np.int64)
    n = ref.kvcm_refsrc_gen_key_vector(tokens.ctypes.data, len(tokens), block_size, keys.ctypes.data)
    assert n == len(keys)
    return [int(k) for k in keys]


def main():
    ref = O.ref()
    if ref is None:
        raise SystemExit("oracle/_ref is not built: run `make -C oracle ref` where the reference tree is present")
    out = {"generator": "tests/golden/make_hash_golden.py", "source": "oracle/_ref (reference hash_util.h compiled)"}

    tok = c1_tokens()
    out["c1"] = {
        "recipe": "rng=np.random.default_rng(0); tok=rng.integers(0,151936,(4,512),dtype=int64); tok[:,:256]=tok[0,:256]",
        "block_size": 16,
        "tokens_row0_first8": [int(x) for x in tok[0, :8]],
        "keys": [ref_keys(ref, tok[r], 16) for r in range(4)],
    }

    cases = []
    rng = np.random.default_rng(1234)
    explicit = [
        ("ramp64_bs16", list(range(64)), 16),
        ("extremes_bs3", [-1, -2**63, 2**63 - 1], 3),
        ("extremes_bs1", [-1, -2**63, 2**63 - 1, 0, 1, -2], 1),
        ("single_456_bs1", [456], 1),
        ("partial_tail_bs4", list(range(100, 110)), 4),
        ("shorter_than_block", [1, 2, 3], 4),
        ("empty", [], 16),
        ("zeros_bs2", [0] * 12, 2),
    ]
    for name, toks, bs in explicit:
        cases.append({"name": name, "tokens": toks, "block_size": bs, "keys": ref_keys(ref, toks, bs)})
    for i, (n, bs) in enumerate([(33, 1), (97, 7), (256, 16), (130, 64), (640, 128), (50, 50)]):
        toks = [int(x) for x in rng.integers(-2**63, 2**63 - 1, size=n, dtype=np.int64)]
        cases.append({"name": f"rand_full_range_{i}", "tokens": toks, "block_size": bs, "keys": ref_keys(ref, toks, bs)})
    out["cases"] = cases

    # single steps, incl. states with the sign bit set (arithmetic shift) -- hashInt64Func itself
    steps = []
    for h, v in [(0, 0), (0, 456), (-1, 0), (-1, -1), (2**63 - 1, 1), (-2**63, -2**63), (0x0123456789ABCDEF, 77),
                 (-0x0123456789ABCDEF, -77)]:
        steps.append({"h": h, "v": v, "out": int(ref.kvcm_refsrc_hash_step(h, v))})
    for _ in range(32):
        h, v = (int(x) for x in rng.integers(-2**63, 2**63 - 1, size=2, dtype=np.int64))
        steps.append({"h": h, "v": v, "out": int(ref.kvcm_refsrc_hash_step(h, v))})
    out["steps"] = steps

    # ApplyPrefixHash loop over the real hashInt64Func
    chains = []
    for n in (0, 1, 5, 64):
        ids = [int(x) for x in rng.integers(-2**63, 2**63 - 1, size=n, dtype=np.int64)]
        a = np.array(ids, dtype=np.int64)
        k = np.zeros(n, dtype=np.int64)
        ref.kvcm_refsrc_prefix_chain(a.ctypes.data, n, k.ctypes.data)
        chains.append({"ids": ids, "keys": [int(x) for x in k]})
    out["prefix_chains"] = chains

    # HashIntArray<uint32_t> (buffer-check fold)
    folds = []
    for n in (1, 2, 64, 128):
        crcs = rng.integers(0, 2**32, size=n, dtype=np.uint64).astype(np.uint32)
        h = ref.kvcm_refsrc_hash_u32_array(crcs.ctypes.data, crcs.ctypes.data + 4 * n, 0)
        folds.append({"crcs": [int(x) for x in crcs], "hash": int(h)})
    out["u32_folds"] = folds

    path = os.path.join(HERE, "hash_golden.json")
    with open(path, "w") as f:
        json.dump(out, f, indent=0, separators=(",", ":"))
        f.write("\n")
    print("wrote", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
