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


def _scratch_info():
    import ctypes as C
    vals = [C.c_size_t() for _ in range(3)]
    call("tfhip_scratch_info", *[C.byref(v) for v in vals])
    return tuple(v.value for v in vals)


def test_the_static_entry_point_leaves_the_library_scratch_alone(rt):
    """What the entry point promises: it allocates nothing. The allocating scan sizes the library's scratch buffer by the
    number of tiles; a static call on a size that buffer has never been grown for must leave its size, and the count of
    retired buffers, as they were -- so the static call comes FIRST here, before any allocating call of that size."""
    n = 32768 * 7000 + 5  # about 229 M elements: 7001 tiles, more than any other test scans
    x = np.full(n, 3, dtype=np.uint32)
    xb = rt.DeviceBuffer.from_numpy(x)
    out = rt.DeviceBuffer(n)
    rt.synchronize()
    before = _scratch_info()
    call("tfhip_scan_inclusive_u32_static", xb.ptr, out.ptr, n)
    rt.synchronize()
    assert _scratch_info() == before
    got = out.numpy(np.uint32)
    assert np.array_equal(got, (np.arange(1, n + 1, dtype=np.uint64) * 3).astype(np.uint32))
    xb.free()
    out.free()


def test_the_static_entry_point_inside_a_recorded_graph(rt):
    """Usable where nothing may be allocated: recorded into a HIP graph and replayed, with other work and waits between
    the replays, each replay bit-exact (the entry point clears its own counters with a kernel, not with a memset node)."""
    rng = np.random.default_rng(5)
    n = 32768 * 9 + 77
    x = rng.integers(0, 2**32, n, dtype=np.uint32)
    xb = rt.DeviceBuffer.from_numpy(x)
    out = rt.DeviceBuffer(n)
    other = rt.DeviceBuffer(n)
    g = rt.Graph()
    before = _scratch_info()
    with g:
        call("tfhip_scan_inclusive_u32_static", xb.ptr, out.ptr, n)
    assert _scratch_info()[:2] == before[:2]
    want = oracle.scan_inclusive(x)
    for replay in range(4):
        out.fill(0)
        g.launch()
        rt.synchronize()
        assert np.array_equal(out.numpy(np.uint32), want), f"replay {replay}"
        # eager work of the same kind between replays: it shares the static array with the graph
        call("tfhip_scan_inclusive_u32_static", xb.ptr, other.ptr, n - replay * 1000)
        rt.synchronize()
        assert np.array_equal(other.numpy(np.uint32)[: n - replay * 1000], want[: n - replay * 1000])
        # new input for the next replay
        x = rng.integers(0, 2**32, n, dtype=np.uint32)
        xb.write(x)
        want = oracle.scan_inclusive(x)
    g.destroy()
    for b in (xb, out, other):
        b.free()
