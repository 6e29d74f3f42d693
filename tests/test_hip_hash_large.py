"""GPU parity of the hash kernel on batches beyond 4 GiB of tokens, where 32-bit buffer offsets stop reaching:
(1) many workgroups, each well under 4 GiB, the batch as a whole above it (per-workgroup buffer bases);
(2) one workgroup whose 64 requests span more than 4 GiB (the kernel must pick its general loader by itself)."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _check(oracle, R, L, bs, seed):
    from tair_kvcache_amd import hashing
    g = torch.Generator(device="cuda")
    g.manual_seed(seed)
    tok = torch.randint(-2**40, 2**40, (R, L), dtype=torch.int64, device="cuda", generator=g)
    print(f"large hash case R={R} L={L} bs={bs}: {tok.numel() * 8 / 2**30:.2f} GiB of tokens", flush=True)
    keys, off = hashing.hash_tokens(tok, bs)
    torch.cuda.synchronize()
    got = keys.cpu().numpy()
    host_tok = tok.cpu().numpy()
    del tok
    want, woff = oracle.hash_tokens(host_tok, bs, threads=16)
    assert (off.cpu().numpy() == woff).all()
    assert (got == want).all()
    torch.cuda.empty_cache()


def test_batch_above_4gib_many_workgroups(oracle):
    _check(oracle, R=1200, L=500_032, bs=64, seed=11)  # 4.47 GiB in 19 workgroups of <= 239 MiB each


def test_one_workgroup_spanning_more_than_4gib(oracle):
    _check(oracle, R=70, L=8_400_000, bs=128, seed=12)  # first workgroup: 64 x 8.4 M tokens = 4.0 GiB + ...
