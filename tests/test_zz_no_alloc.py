"""The allocation-free prefix sum (tfhip_scan_inclusive_u32_static) against the ordinary entry point and the oracle.

Collected last on purpose (file name): a failure here must not hide the other GPU tests behind `pytest -x`.
"""
import numpy as np
import pytest

from oracle import oracle
from tensorfrost_amd._lib import TFHipError, call

pytestmark = pytest.mark.gpu


def _scan_both(rt, x):
    n = x.size
    xb = rt.DeviceBuffer.from_numpy(x)
    ref_b = rt.DeviceBuffer(n)
    got_b = rt.DeviceBuffer(n)
    got_b.fill(0xDEADBEEF)
    call("tfhip_scan_inclusive_u32", xb.ptr, ref_b.ptr, n)
    call("tfhip_scan_inclusive_u32_static", xb.ptr, got_b.ptr, n)
    rt.synchronize()
    return got_b.numpy(np.uint32), ref_b.numpy(np.uint32)


def test_two_calls_in_a_row_the_second_smaller(rt):
    """Bit-exact against the allocating entry point and the CPU oracle, twice in a row; the second call is smaller, so
    it meets the status words the first call left behind in the shared array."""
    rng = np.random.default_rng(77)
    for n in (5 * 32768 * 20 + 123, 3 * 32768 + 1, 1000):
        x = rng.integers(0, 2**32, n, dtype=np.uint32)
        got, ref = _scan_both(rt, x)
        assert np.array_equal(got, ref), f"n={n}: differs from tfhip_scan_inclusive_u32"
        assert np.array_equal(got, oracle.scan_inclusive(x)), f"n={n}: differs from the oracle"


def test_in_place_and_limits(rt):
    x = np.arange(1, 70001, dtype=np.uint32)
    xb = rt.DeviceBuffer.from_numpy(x)
    call("tfhip_scan_inclusive_u32_static", xb.ptr, xb.ptr, x.size)
    rt.synchronize()
    assert np.array_equal(xb.numpy(np.uint32), np.cumsum(x, dtype=np.uint64).astype(np.uint32))
    call("tfhip_scan_inclusive_u32_static", xb.ptr, xb.ptr, 0)  # no-op
    with pytest.raises(TFHipError, match="at most"):
        call("tfhip_scan_inclusive_u32_static", xb.ptr, xb.ptr, 2**30 + 1)
