"""rgs_sort_pairs_static, the entry point that allocates nothing (its scratch is an array the library
holds on the device), against rgs_sort_pairs with a caller's workspace: same results bit for bit, on
two calls in a row of which the second is smaller, and a refusal beyond the stated maximum."""
import ctypes as C

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _sort(fn_static, keys, vals, end_bit):
    from retinags_amd import _capi
    n = keys.shape[0]
    k_in = torch.from_numpy(keys.view(np.int64).copy()).to(DEV)
    v_in = torch.from_numpy(vals.view(np.int32).copy()).to(DEV)
    k_out, v_out = torch.empty_like(k_in), torch.empty_like(v_in)
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    if fn_static:
        _capi.check(_capi.lib.rgs_sort_pairs_static(_capi.ptr(k_in), _capi.ptr(k_out), _capi.ptr(v_in), _capi.ptr(v_out), n,
                                                    end_bit, stream))
    else:
        temp = torch.empty(max(_capi.lib.rgs_sort_temp_bytes(n), 4), dtype=torch.uint8, device=DEV)
        _capi.check(_capi.lib.rgs_sort_pairs(_capi.ptr(k_in), _capi.ptr(k_out), _capi.ptr(v_in), _capi.ptr(v_out), n,
                                             end_bit, _capi.ptr(temp), stream))
    torch.cuda.synchronize()
    return k_out.cpu().numpy().view(np.uint64), v_out.cpu().numpy().view(np.uint32)


def test_sort_without_a_workspace_matches_the_sort_with_one_twice_in_a_row():
    from retinags_amd import _capi
    g = np.random.default_rng(17)
    # the second call is smaller and has another pass count (odd, then even): what the first left in
    # the shared scratch must not matter
    for n, end_bit in ((3_000_001, 45), (70_001, 49), (5, 64), (0, 45)):
        keys = g.integers(0, 2 ** 63, size=n, dtype=np.uint64)
        if n > 10:
            keys[: n // 3] &= np.uint64(0xFFFFF)      # many equal compared bits: stability matters
        vals = g.integers(0, 2 ** 32, size=n, dtype=np.uint32)
        k_ws, v_ws = _sort(False, keys, vals, end_bit)
        k_st, v_st = _sort(True, keys, vals, end_bit)
        assert np.array_equal(k_st, k_ws) and np.array_equal(v_st, v_ws)
        mask = np.uint64((1 << end_bit) - 1) if end_bit < 64 else np.uint64(0xFFFFFFFFFFFFFFFF)
        order = np.argsort(keys & mask, kind="stable")
        assert np.array_equal(k_st, keys[order]) and np.array_equal(v_st, vals[order])
    # beyond the maximum the call refuses (nothing is launched; the pointers are not touched)
    n = _capi.STATIC_SORT_MAX_PAIRS + 1
    rc = _capi.lib.rgs_sort_pairs_static(C.c_void_p(256), C.c_void_p(256), C.c_void_p(256), C.c_void_p(256), n, 45,
                                         C.c_void_p(torch.cuda.current_stream().cuda_stream))
    assert rc != 0 and b"exceed" in _capi.lib.rgs_last_error()
    assert _capi.lib.rgs_sort_fault(C.c_void_p(torch.cuda.current_stream().cuda_stream)) == 0


def test_sort_without_a_workspace_takes_no_device_memory():
    """Free device memory as the driver reports it (hipMemGetInfo: it sees every allocation of the process, the
    library's included, not only those of torch's caching allocator) is the same before and after a call, once the
    library's code and its scratch array are resident (a first call brings them in)."""
    from retinags_amd import _capi
    g = np.random.default_rng(3)
    n = 1_000_003
    k_in = torch.from_numpy(g.integers(0, 2 ** 62, size=n, dtype=np.int64)).to(DEV)
    v_in = torch.arange(n, dtype=torch.int32, device=DEV)
    k_out, v_out = torch.empty_like(k_in), torch.empty_like(v_in)
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    call = lambda: _capi.check(_capi.lib.rgs_sort_pairs_static(_capi.ptr(k_in), _capi.ptr(k_out), _capi.ptr(v_in),
                                                               _capi.ptr(v_out), n, 45, stream))
    call()
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    call()
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before


def test_sort_without_a_workspace_reports_a_sort_that_gave_up():
    """With the look-backs told to give up at once (from the host: every kernel still runs to its end), the static
    entry's report reaches rgs_sort_fault although no pinned report word need exist; the report is cleared by the
    read, and a normal sort afterwards is clean and correct."""
    from retinags_amd import _capi
    g = np.random.default_rng(5)
    n = 40_000     # several tiles of the sort, so that there is a look-back to give up
    keys = g.integers(0, 2 ** 40, size=n, dtype=np.uint64)
    vals = np.arange(n, dtype=np.uint32)
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    assert _capi.lib.rgs_sort_fault(stream) == 0
    _capi.lib.rgs_set_lookback_spin_limit(-1)
    try:
        _sort(True, keys, vals, 40)
    finally:
        _capi.lib.rgs_set_lookback_spin_limit(0)
    assert _capi.lib.rgs_sort_fault(stream) != 0 and b"gave up" in _capi.lib.rgs_last_error()
    assert _capi.lib.rgs_sort_fault(stream) == 0
    k, v = _sort(True, keys, vals, 40)
    order = np.argsort(keys, kind="stable")
    assert np.array_equal(k, keys[order]) and np.array_equal(v, vals[order])
    assert _capi.lib.rgs_sort_fault(stream) == 0
