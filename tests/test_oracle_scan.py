"""Pins the CPU oracle's prefix sums against NumPy."""
import numpy as np
import pytest

from oracle import oracle


@pytest.mark.parametrize("n", [1, 2, 255, 256, 4097, 100_003])
def test_scan_u32_wraps_like_numpy(n):
    rng = np.random.default_rng(3)
    x = rng.integers(0, 2**32, n, dtype=np.uint64).astype(np.uint32)
    assert np.array_equal(oracle.scan_inclusive(x), np.cumsum(x, dtype=np.uint64).astype(np.uint32))


def test_scan_i32_and_lines():
    rng = np.random.default_rng(4)
    x = rng.integers(-2**31, 2**31, (37, 129), dtype=np.int64).astype(np.int32)
    ref = np.cumsum(x.astype(np.int64), axis=1).astype(np.int32)  # wraps modulo 2^32
    assert np.array_equal(oracle.scan_inclusive(x), ref)


def test_scan_f32():
    rng = np.random.default_rng(5)
    x = rng.normal(size=50_000).astype(np.float32)
    got = oracle.scan_inclusive(x)
    ref = np.cumsum(x.astype(np.float64))
    assert np.max(np.abs(got - ref) / np.cumsum(np.abs(x.astype(np.float64)))) < 1e-6
    assert got[0] == x[0]  # inclusive, starts from 0
