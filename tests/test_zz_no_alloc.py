"""The entry point that allocates nothing (kvcm_hip_first_occurrence_static: table in a device array of the library)
gives the results of kvcm_hip_first_occurrence (caller's workspace), called through the C-ABI on two calls in a row,
the second with a smaller input, so that the table still holds the first call's entries. Integer work: exact."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _keys(rng, n, distinct):
    base = rng.integers(-2**63, 2**63 - 1, size=distinct, dtype=np.int64)
    return base[rng.integers(0, distinct, size=n)]


def _both(L, keys_np):
    """(first, repeat) from the workspace entry point and from the static one, same stream."""
    n = len(keys_np)
    keys = torch.from_numpy(keys_np).cuda()
    stream = torch.cuda.current_stream().cuda_stream
    out = []
    need = L.kvcm_hip_first_occurrence_workspace_bytes(n)
    ws = torch.empty(need // 4, dtype=torch.int32, device="cuda")
    for static in (False, True):
        first = torch.full((n,), -7, dtype=torch.int32, device="cuda")
        rep = torch.full((n,), 9, dtype=torch.uint8, device="cuda")
        if static:
            rc = L.kvcm_hip_first_occurrence_static(keys.data_ptr(), n, first.data_ptr(), rep.data_ptr(), stream)
        else:
            rc = L.kvcm_hip_first_occurrence(keys.data_ptr(), n, ws.data_ptr(), need, first.data_ptr(), rep.data_ptr(),
                                             stream)
        assert rc == 0, rc
        torch.cuda.synchronize()
        out.append((first.cpu().numpy(), rep.cpu().numpy()))
    return out


def test_static_first_occurrence_equals_the_workspace_form_twice_in_a_row(oracle):
    from tair_kvcache_amd import _lib
    L = _lib.lib()
    assert L.kvcm_hip_first_occurrence_static_max_keys() == 1 << 20
    rng = np.random.default_rng(77)
    for n, distinct in ((65536, 40000), (5000, 1200), (1 << 20, 1 << 19), (3, 2)):
        print(f"first_occurrence_static n={n} distinct={distinct}", flush=True)
        keys = _keys(rng, n, distinct)
        (f_ws, r_ws), (f_st, r_st) = _both(L, keys)
        assert (f_st == f_ws).all() and (r_st == r_ws).all()
        w_first, w_rep = oracle.first_occurrence(keys)
        assert (f_st == w_first).all() and (r_st == w_rep).all()


def test_static_first_occurrence_rejects_what_it_cannot_hold():
    from tair_kvcache_amd import _lib
    L = _lib.lib()
    keys = torch.zeros(8, dtype=torch.int64, device="cuda")
    out = torch.zeros(8, dtype=torch.int32, device="cuda")
    assert L.kvcm_hip_first_occurrence_static(keys.data_ptr(), (1 << 20) + 1, out.data_ptr(), None,
                                              None) == _lib.ERR_TOO_LARGE
    assert L.kvcm_hip_first_occurrence_static(keys.data_ptr(), -1, out.data_ptr(), None, None) == _lib.ERR_INVALID_ARG
    assert L.kvcm_hip_first_occurrence_static(None, 8, out.data_ptr(), None, None) == _lib.ERR_INVALID_ARG
    assert L.kvcm_hip_first_occurrence_static(None, 0, None, None, None) == 0   # set-up only
    assert L.kvcm_hip_first_occurrence_static(keys.data_ptr(), 8, out.data_ptr(), None, None) == 0
    torch.cuda.synchronize()
    assert (out == 0).all()
