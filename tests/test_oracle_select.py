"""What pins the oracle's save-selection functions: brute force on small inputs, NumPy's np.unique on larger ones,
and the reference's own parsing loop (v1_connector.py:835-850) restated line by line in Python."""
import numpy as np

import _cases as cases


def _brute_first(keys):
    return [min(j for j in range(len(keys)) if keys[j] == k) for k in keys]


def test_first_occurrence_brute_force(oracle):
    rng = np.random.default_rng(11)
    for n in (0, 1, 2, 7, 64, 300):
        keys = rng.integers(-5, 6, size=n, dtype=np.int64)
        first, rep = oracle.first_occurrence(keys)
        assert first.tolist() == _brute_first(keys.tolist())
        assert rep.tolist() == [int(f != i) for i, f in enumerate(first.tolist())]
    # extreme values compare as signed 64-bit integers, not as anything narrower
    keys = np.array([-2**63, 2**63 - 1, 0, -2**63, 2**32, 0, 2**63 - 1, 1 << 32], dtype=np.int64)
    assert oracle.first_occurrence(keys)[0].tolist() == [0, 1, 2, 0, 4, 2, 1, 4]


def test_first_occurrence_against_numpy_unique(oracle):
    rng = np.random.default_rng(12)
    keys = rng.integers(-2**63, 2**63 - 1, size=20000, dtype=np.int64)
    keys[rng.integers(0, 20000, size=15000)] = keys[rng.integers(0, 500, size=15000)]
    first, rep = oracle.first_occurrence(keys)
    uniq, idx, inv = np.unique(keys, return_index=True, return_inverse=True)
    assert (first == idx[inv]).all()
    assert int((rep == 0).sum()) == len(uniq)


def test_shared_prefix_batch_config1(oracle):
    """Config 1: 4 requests x 32 keys, first 16 keys of every request equal => 16 + 4*16 = 80 blocks to save."""
    tokens = cases.tokens(4, 512, 151936, shared_rows=4, shared_len=256)
    keys = np.concatenate([np.array(oracle.gen_key_vector(t, 16), dtype=np.int64) for t in tokens])
    first, rep = oracle.first_occurrence(keys)
    save = oracle.mask_to_indices(rep)
    assert len(save) == 80
    assert save.tolist() == list(range(32)) + [r * 32 + b for r in range(1, 4) for b in range(16, 32)]
    assert (first[32:48] == np.arange(16)).all()


def test_mask_to_indices_is_the_reference_loop(oracle):
    rng = np.random.default_rng(13)
    for n in (0, 1, 5, 1023, 1024, 1025, 5000):
        values = (rng.random(n) < 0.4).tolist()
        want = oracle.py_parse_block_mask_to_save_indices({"block_mask": {"bool_masks": {"values": values}}}, n)
        got = oracle.mask_to_indices(np.array(values, dtype=np.uint8))
        assert got.tolist() == want
        assert want == np.flatnonzero(~np.array(values, dtype=bool)).tolist()
    # the offset branch equals the mask that is true below the offset
    want = oracle.py_parse_block_mask_to_save_indices({"block_mask": {"offset": 7}}, 20)
    assert oracle.mask_to_indices((np.arange(20) < 7).astype(np.uint8)).tolist() == want == list(range(7, 20))
    # two masks: saved by the manager OR repeated inside the batch
    a = np.array([1, 0, 0, 1, 0, 0], dtype=np.uint8)
    b = np.array([0, 0, 1, 1, 0, 2], dtype=np.uint8)
    assert oracle.mask_to_indices(a, b).tolist() == [1, 4]
    # an empty response saves nothing
    assert oracle.py_parse_block_mask_to_save_indices({}, 5) == []
