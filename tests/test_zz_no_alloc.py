"""endia_hip_col_sum_static, the entry point that allocates nothing, against endia_hip_reduce_add (ndim 2, mask 1).

Two calls in a row share the device's one static scratch array, the second with a smaller input: the second result
must not see what the first call left there. The pool's count of device allocations must not move across the calls.
"""
import ctypes

import numpy as np
import pytest

from conftest import assert_close
from endia_amd import _lib as L

pytestmark = pytest.mark.gpu


def _same_plan(R, C):
    """Bit equality with endia_hip_reduce_add holds when both cut the rows the same way, i.e. when the 262144 floats of
    static scratch do not force fewer row splits than the unlimited workspace gets (never on a 256-CU device; the plan
    query says so for whatever device this is, and tests/test_abi.py checks the clamp itself on the CPU)."""
    _, cus, _ = L.device_info()
    plans = []
    for scratch in (0, 1 << 18):
        S, rows = ctypes.c_int64(), ctypes.c_int64()
        L.call("endia_hip_col_sum_plan", R, C, cus, scratch, 1, ctypes.byref(S), ctypes.byref(rows))
        plans.append((S.value, rows.value))
    return plans[0] == plans[1]


def _both(dev, x, scale=1.0):
    R, C = x.shape
    dx = dev.put(x)
    ref, out = dev.alloc(4 * C), dev.alloc(4 * C)
    dev.call("endia_hip_fill", out, C, float("nan"))
    dev.call("endia_hip_reduce_add", 2, L.i64_array([R, C]), 1, dx, ref, scale, 0)
    n0, n1 = ctypes.c_int64(), ctypes.c_int64()
    dev.call("endia_hip_pool_stats", None, None, ctypes.byref(n0))
    dev.call("endia_hip_col_sum_static", R, C, dx, out, scale)
    dev.call("endia_hip_pool_stats", None, None, ctypes.byref(n1))
    assert n1.value == n0.value
    return dev.get(out, (C,)), dev.get(ref, (C,))


def test_col_sum_static_matches_reduce_add_twice_in_a_row(dev):
    rng = np.random.default_rng(11)
    big = rng.standard_normal((4096, 4096)).astype(np.float32)      # the wide MLP's bias gradient: two stages, 64 row splits
    small = rng.standard_normal((5000, 772)).astype(np.float32)    # smaller, still two stages (more than 4096 rows)
    for x, scale in ((big, 1.0), (small, 0.5)):
        got, ref = _both(dev, x, scale)
        if _same_plan(*x.shape):
            assert np.array_equal(got, ref), "static-scratch column sums differ from endia_hip_reduce_add"
        assert_close(got, ref, tol=1e-6, what="static scratch vs reduce_add")
        assert_close(got, scale * x.astype(np.float64).sum(axis=0), what="column sums %s" % (x.shape,))
    for shape in ((40, 96), (1024, 2048)):                          # the single-launch paths (no scratch at all): small, mid-size
        tiny = rng.standard_normal(shape).astype(np.float32)
        got, ref = _both(dev, tiny)
        assert np.array_equal(got, ref)
        assert_close(got, tiny.astype(np.float64).sum(axis=0), what="column sums %s" % (shape,))


def test_col_sum_static_widest_input(dev):
    """262144 columns, the maximum: one row split, whose partial sums fill the static array exactly."""
    rng = np.random.default_rng(12)
    x = rng.standard_normal((24, 1 << 18)).astype(np.float32)
    got, ref = _both(dev, x)
    if _same_plan(*x.shape):
        assert np.array_equal(got, ref)
    assert_close(got, ref, tol=1e-6, what="static scratch vs reduce_add")
    assert_close(got, x.astype(np.float64).sum(axis=0), what="widest column sums")


def test_col_sum_static_limits_and_edges(dev):
    lib = L.lib()
    p = dev.alloc(16)
    assert lib.endia_hip_col_sum_static(4, (1 << 18) + 4, p, p, ctypes.c_float(1.0)) == L.ERR_INVALID
    assert b"maximum" in lib.endia_hip_last_error()
    assert lib.endia_hip_col_sum_static(-1, 4, p, p, ctypes.c_float(1.0)) == L.ERR_INVALID
    assert lib.endia_hip_col_sum_static(4, 0, None, None, ctypes.c_float(1.0)) == 0
    out = dev.alloc(4 * 8)
    dev.call("endia_hip_fill", out, 8, 3.0)
    dev.call("endia_hip_col_sum_static", 0, 8, None, out, 1.0)  # empty sum
    assert np.array_equal(dev.get(out, (8,)), np.zeros(8, np.float32))
