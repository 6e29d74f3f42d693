"""Seeded synthetic inputs shaped like the benchmark configurations, shared by the CPU and GPU tests.

Seeds: 0 tokens, 1 KV values, 2 block tables.
"""
import numpy as np


def tokens(R, L, vocab, shared_rows=0, shared_len=0, seed=0, dtype=np.int64):
    rng = np.random.default_rng(seed)
    tok = rng.integers(0, vocab, size=(R, L), dtype=np.int64)
    if shared_rows and shared_len:
        tok[:shared_rows, :shared_len] = tok[0, :shared_len]
    return tok.astype(dtype)


def pool_u16(P, slots, D, seed=1):
    """P pool arrays [slots, D] of 16-bit patterns (bf16/fp16 payloads are opaque bytes to the copy path)."""
    rng = np.random.default_rng(seed)
    return [rng.integers(0, 65536, size=(slots, D), dtype=np.uint16) for _ in range(P)]


def ramp_pool_u16(P, slots, D):
    """value = (p * 131 + slot) mod 65536 in every element of the row: a misplaced row names where it came from."""
    out = []
    for p in range(P):
        col = ((p * 131 + np.arange(slots)) % 65536).astype(np.uint16)
        out.append(np.repeat(col[:, None], D, axis=1).copy())
    return out


def block_table(n_pool_blocks, n_take, seed=2):
    rng = np.random.default_rng(seed)
    return rng.permutation(n_pool_blocks)[:n_take].astype(np.int32)


def token_idx_from_blocks(block_ids, T):
    """[B, T] token slots of whole engine blocks."""
    return (block_ids[:, None].astype(np.int64) * T + np.arange(T)[None, :]).astype(np.int32)


# name -> (layers, kv, D elements, itemsize, T, pool blocks, work blocks, staging slots)
SMALL_CONFIGS = {
    "c1_qwen05b": dict(L=24, kv=2, D=128, itemsize=2, T=16, pool_blocks=1024, B=128, slots=128),
    "c2_llama8b_scaled": dict(L=32, kv=2, D=1024, itemsize=2, T=16, pool_blocks=96, B=48, slots=64),
    "c3_72b_scaled": dict(L=80, kv=2, D=1024, itemsize=2, T=64, pool_blocks=12, B=5, slots=8),
    "c5_page1_scaled": dict(L=28, kv=2, D=512, itemsize=2, T=16, pool_blocks=0, B=64, slots=64),
    "ref_test_shape": dict(L=4, kv=2, D=1024, itemsize=2, T=16, pool_blocks=640, B=128, slots=1024),
}
