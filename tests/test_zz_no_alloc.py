"""dali_hip_argsort_i32_noalloc against dali_hip_argsort_i32, through the C ABI.

The entry point that allocates nothing orders keys with the same kernel as dali_hip_argsort_i32 but keeps the kernel's
tickets and counts in a device array built into the library. Results must be bit-equal (index work), on calls in a row
that share the array, the later ones on smaller inputs; the bank and the driver must see no allocation.
"""
import ctypes as C

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

LIMIT = 16384


def _dev(hip, nbytes):
    p = C.c_void_p()
    assert hip.dali_hip_malloc(C.byref(p), max(nbytes, 4)) == 0
    return p


def _run(hip, fn, keys, limit, dk, ds, dp):
    n = keys.size
    poison = np.full(n, -7, np.int32)
    for d in (ds, dp):
        assert hip.dali_hip_memcpy_h2d(d, poison.ctypes.data_as(C.c_void_p), n * 4) == 0
    assert hip.dali_hip_memcpy_h2d(dk, keys.ctypes.data_as(C.c_void_p), n * 4) == 0
    assert fn(dk, n, limit, ds, dp) == 0, hip.dali_hip_last_error()
    sk, pm = np.empty(n, np.int32), np.empty(n, np.int32)
    assert hip.dali_hip_memcpy_d2h(sk.ctypes.data_as(C.c_void_p), ds, n * 4) == 0
    assert hip.dali_hip_memcpy_d2h(pm.ctypes.data_as(C.c_void_p), dp, n * 4) == 0
    return sk, pm


def test_argsort_noalloc_equals_argsort_on_calls_in_a_row(gpu):
    hip = gpu
    rng = np.random.RandomState(77)
    dk, ds, dp = (_dev(hip, LIMIT * 4) for _ in range(3))
    parked, live = C.c_size_t(), C.c_size_t()
    assert hip.dali_hip_bank_stats(C.byref(parked), C.byref(live)) == 0
    bank_before = (parked.value, live.value)
    # the second and later calls are smaller than the first: they find the array as the earlier call left it
    cases = [(LIMIT, 32000), (5000, 32000), (8192, 0), (777, 1 << 30), (1, 0), (LIMIT, 2), (300, 1000)]
    for n, limit in cases:
        if limit > 0:
            keys = rng.randint(0, limit, n).astype(np.int32)
        else:
            keys = rng.randint(-50, 50, n).astype(np.int32)
            keys[rng.randint(0, n, max(1, n // 10))] = np.iinfo(np.int32).max
            keys[rng.randint(0, n, max(1, n // 10))] = np.iinfo(np.int32).min
        want_sk, want_pm = _run(hip, hip.dali_hip_argsort_i32, keys, limit, dk, ds, dp)
        got_sk, got_pm = _run(hip, hip.dali_hip_argsort_i32_noalloc, keys, limit, dk, ds, dp)
        assert np.array_equal(got_pm, want_pm) and np.array_equal(got_sk, want_sk), (n, limit)
        order = np.argsort(keys, kind="stable")
        assert np.array_equal(got_pm, order) and np.array_equal(got_sk, keys[order]), (n, limit)
    assert hip.dali_hip_bank_stats(C.byref(parked), C.byref(live)) == 0
    assert (parked.value, live.value) == bank_before  # nothing taken from or returned to the bank
    # beyond the limit: a clear error, nothing launched, outputs untouched
    assert hip.dali_hip_argsort_i32_noalloc(dk, LIMIT + 1, 0, ds, dp) != 0
    msg = hip.dali_hip_last_error().decode()
    assert "exceed the limit of 16384 keys" in msg
    assert hip.dali_hip_argsort_i32_noalloc(dk, -1, 0, ds, dp) != 0
    assert hip.dali_hip_argsort_i32_noalloc(dk, 0, 0, ds, dp) == 0
    assert hip.dali_hip_argsort_i32_noalloc(None, 5, 0, ds, dp) != 0
    for p in (dk, ds, dp):
        assert hip.dali_hip_free(p) == 0


def test_argsort_noalloc_inside_a_capture(gpu):
    """The call is legal while the library stream is being captured; replays give the eager result every time."""
    hip = gpu
    rng = np.random.RandomState(78)
    n = 6000
    dk, ds, dp = (_dev(hip, n * 4) for _ in range(3))
    keys = rng.randint(0, 500, n).astype(np.int32)
    assert hip.dali_hip_memcpy_h2d(dk, keys.ctypes.data_as(C.c_void_p), n * 4) == 0
    graph = C.c_void_p()
    assert hip.dali_hip_capture_begin() == 0
    status = hip.dali_hip_argsort_i32_noalloc(dk, n, 500, ds, dp)
    assert hip.dali_hip_capture_end(C.byref(graph)) == 0
    assert status == 0, hip.dali_hip_last_error()
    pm = np.empty(n, np.int32)
    for rep in range(3):
        keys = rng.randint(0, 500, n).astype(np.int32)
        assert hip.dali_hip_memcpy_h2d(dk, keys.ctypes.data_as(C.c_void_p), n * 4) == 0
        assert hip.dali_hip_graph_launch(graph) == 0
        assert hip.dali_hip_memcpy_d2h(pm.ctypes.data_as(C.c_void_p), dp, n * 4) == 0
        assert np.array_equal(pm, np.argsort(keys, kind="stable")), rep
    assert hip.dali_hip_graph_destroy(graph) == 0
    for p in (dk, ds, dp):
        assert hip.dali_hip_free(p) == 0
