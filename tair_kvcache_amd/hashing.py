"""Block keys on the GPU: the manager's token hashing and its siblings, batched.

    hash_tokens / gen_key_vector   GenKeyVector        kv_cache_manager/manager/cache_manager.cc:76-87
                                   hashInt64Array      kv_cache_manager/manager/hash_util.h:14-24
    apply_prefix_hash              ApplyPrefixHash     kv_cache_manager/optimizer/trace_converter/trace_util.cc:47-56
    sha256_to_int64                _sha256_to_int64    kv_cache_manager/py_connector/sglang/connector.py:397-401
    prepare_block_keys             _prepare_block_keys kv_cache_manager/py_connector/sglang/connector.py:403-415

A connector that computes keys here can send `block_keys` instead of `token_ids`; the manager prefers them
(kv_cache_manager/manager/cache_manager.cc:306-318) and the keys are bit-identical to the ones it would compute.
"""
from typing import List, Optional, Sequence, Tuple

import torch

from . import _lib
from ._torch_util import lib, ptr, require_cuda, stream_handle


def _offsets_for(tokens, token_offsets):
    if token_offsets is None:
        if tokens.dim() != 2:
            raise ValueError("tokens must be [R, L] when token_offsets is not given")
        R, L = tokens.shape
        off = torch.arange(R + 1, dtype=torch.int64, device=tokens.device) * L
        return off, R
    _require_offsets(token_offsets, "token_offsets", tokens.device)
    return token_offsets.contiguous(), token_offsets.numel() - 1


def _require_offsets(t, name, device, entries=None):
    """Offsets are read by the kernel as they are: int64, 1-D, on the tokens' device, R+1 entries."""
    require_cuda(t, name)
    if t.dtype != torch.int64 or t.dim() != 1 or t.numel() < 1:
        raise ValueError(f"{name} must be a 1-D int64 tensor of R+1 entries")
    if t.device != device:
        raise ValueError(f"{name} is on {t.device}, the tokens on {device}")
    if entries is not None and t.numel() != entries:
        raise ValueError(f"{name} has {t.numel()} entries, expected {entries}")


def hash_tokens(tokens: torch.Tensor, block_size: int, token_offsets: Optional[torch.Tensor] = None,
                seed: int = 0, keys: Optional[torch.Tensor] = None,
                key_offsets: Optional[torch.Tensor] = None) -> Tuple[torch.Tensor, torch.Tensor]:
    """Parent-chained block keys of R requests in one launch.

    tokens: int64 or int32 device tensor, [R, L] (uniform lengths) or flat with token_offsets [R+1].
    Returns (keys, key_offsets): request r owns keys[key_offsets[r]:key_offsets[r+1]], len_r // block_size of
    them (a trailing partial block yields no key, cache_manager.cc:78). Asynchronous on the current stream when
    `keys` and `key_offsets` are passed in (or the batch is a 2-D tensor); otherwise the key offsets are computed with
    torch and the total is read back to size `keys`, which costs a synchronisation (about 30 us on an idle MI355X).
    """
    require_cuda(tokens, "tokens")
    if tokens.dtype not in (torch.int64, torch.int32):
        raise ValueError("tokens must be int64 or int32")
    if int(block_size) <= 0:
        raise ValueError("block_size must be positive")
    tokens = tokens.contiguous()
    off, R = _offsets_for(tokens, token_offsets)
    if key_offsets is not None:
        _require_offsets(key_offsets, "key_offsets", tokens.device, R + 1)
        key_offsets = key_offsets.contiguous()
    if keys is not None:
        require_cuda(keys, "keys")
        if keys.dtype != torch.int64 or keys.device != tokens.device or not keys.is_contiguous():
            raise ValueError("keys must be a contiguous int64 tensor on the tokens' device")
        if token_offsets is None and keys.numel() < R * (tokens.shape[1] // int(block_size)):
            raise ValueError(f"keys holds {keys.numel()} entries, the batch yields "
                             f"{R * (tokens.shape[1] // int(block_size))}")
    if key_offsets is None:
        counts = (off[1:] - off[:-1]) // int(block_size)
        key_offsets = torch.zeros(R + 1, dtype=torch.int64, device=tokens.device)
        torch.cumsum(counts, 0, out=key_offsets[1:])
    if keys is None:
        if token_offsets is None:
            total = R * (tokens.shape[1] // int(block_size))
        else:
            total = int(key_offsets[-1].item())
        keys = torch.empty(total, dtype=torch.int64, device=tokens.device)
        if total == 0:  # no request holds a full block: nothing to launch (GenKeyVector returns an empty vector)
            return keys, key_offsets
    fn = lib().kvcm_hip_hash_tokens if tokens.dtype == torch.int64 else lib().kvcm_hip_hash_tokens_i32
    rc = fn(ptr(tokens), ptr(off), R, int(block_size), int(seed), ptr(keys), ptr(key_offsets),
            stream_handle(tokens.device))
    _lib.check(rc, "kvcm_hip_hash_tokens")
    return keys, key_offsets


def gen_key_vector(tokens, block_size: int, device=None) -> List[int]:
    """GenKeyVector for one request, with the reference's list-in / list-out shape."""
    if isinstance(tokens, torch.Tensor):
        t = tokens.reshape(1, -1)
        if not t.is_cuda:
            t = t.to(device or "cuda")
    else:
        t = torch.tensor(list(tokens), dtype=torch.int64, device=device or "cuda").reshape(1, -1)
    if t.shape[1] < block_size:
        return []
    keys, _ = hash_tokens(t, block_size)
    return keys.tolist()


def apply_prefix_hash(hash_ids: torch.Tensor, offsets: Optional[torch.Tensor] = None) -> torch.Tensor:
    """keys[i] = fold of hash_ids[0..i] per sequence (sequence r = hash_ids[offsets[r]:offsets[r+1]])."""
    require_cuda(hash_ids, "hash_ids")
    if hash_ids.dtype != torch.int64:
        raise ValueError("hash_ids must be int64")
    ids = hash_ids.contiguous().reshape(-1)
    if offsets is None:
        offsets = torch.tensor([0, ids.numel()], dtype=torch.int64, device=ids.device)
    else:
        _require_offsets(offsets, "offsets", ids.device)
        offsets = offsets.contiguous()
    keys = torch.empty_like(ids)
    rc = lib().kvcm_hip_prefix_chain(ptr(ids), ptr(offsets), offsets.numel() - 1, ptr(keys),
                                     stream_handle(ids.device))
    _lib.check(rc, "kvcm_hip_prefix_chain")
    return keys.reshape(hash_ids.shape)


def sha256_to_int64(data: Sequence[str], device="cuda") -> torch.Tensor:
    """int.from_bytes(sha256(s.encode('utf-8')).digest()[:8], 'big', signed=True) for every string, on the GPU."""
    enc = [s.encode("utf-8") if isinstance(s, str) else bytes(s) for s in data]
    n = len(enc)
    if n == 0:
        return torch.empty(0, dtype=torch.int64, device=device)
    lens = torch.tensor([len(e) for e in enc], dtype=torch.int64)
    off = torch.zeros(n + 1, dtype=torch.int64)
    torch.cumsum(lens, 0, out=off[1:])
    blob = torch.frombuffer(bytearray(b"".join(enc) + b"\0"), dtype=torch.uint8)
    d_blob = blob.to(device)
    d_off = off.to(device)
    out = torch.empty(n, dtype=torch.int64, device=device)
    rc = lib().kvcm_hip_sha256_first8_be(ptr(d_blob), ptr(d_off), n, ptr(out), stream_handle(out.device))
    _lib.check(rc, "kvcm_hip_sha256_first8_be")
    return out


def prepare_block_keys(keys: List[str], prefix_keys: Optional[List[str]] = None,
                       device="cuda") -> Tuple[List[int], int, int]:
    """(int64 keys of prefix_keys + keys, len(prefix_keys), len(keys)) -- sglang/connector.py:403-415."""
    prefix_keys = list(prefix_keys) if prefix_keys is not None else []
    block_keys = sha256_to_int64(prefix_keys + list(keys), device=device).tolist()
    return block_keys, len(prefix_keys), len(keys)
