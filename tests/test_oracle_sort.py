"""Pins the CPU oracle's radix sort (a restatement of TensorFrost's sort.py) against a stable argsort."""
import numpy as np
import pytest

from oracle import oracle


def _check(keys):
    vals = np.arange(keys.size, dtype=np.uint32)
    k, v = oracle.radix_sort_kv(keys, vals)
    order = np.argsort(keys, kind="stable")
    assert np.array_equal(k.view(np.uint32), keys[order].view(np.uint32))
    assert np.array_equal(v, order.astype(np.uint32))  # payload pins stability


@pytest.mark.parametrize("n", [1, 2, 127, 128, 129, 8191, 8192, 8193, 100_003])
def test_uniform_u32(n):
    rng = np.random.default_rng(31)
    _check(rng.integers(0, 2**32, n, dtype=np.uint64).astype(np.uint32))


@pytest.mark.parametrize("n", [1000, 70_001])
def test_low_entropy_u32(n):
    rng = np.random.default_rng(32)
    _check(rng.integers(0, 1024, n, dtype=np.uint64).astype(np.uint32))
    _check(np.zeros(n, np.uint32))
    _check(np.full(n, 0xFFFFFFFF, np.uint32))


def test_int_and_float_keys():
    rng = np.random.default_rng(33)
    _check(rng.integers(-2**31, 2**31, 50_000, dtype=np.int64).astype(np.int32))
    f = rng.normal(size=50_000).astype(np.float32)
    f[:8] = [0.0, -0.0, np.inf, -np.inf, 1e-45, -1e-45, 3.4e38, -3.4e38]
    k, v = oracle.radix_sort_kv(f, np.arange(f.size, dtype=np.uint32))
    assert np.all(np.diff(k.astype(np.float64)) >= 0)
    assert np.array_equal(np.sort(f.view(np.uint32)), np.sort(k.view(np.uint32)))  # a permutation
    assert np.array_equal(f[v], k)


def test_float_map_is_monotone_bijection():
    specials = np.array([0.0, -0.0, np.inf, -np.inf, 1e-45, -1e-45, 1.0, -1.0, 3.4028235e38, -3.4028235e38, 1.17549435e-38], np.float32)
    rng = np.random.default_rng(34)
    f = np.concatenate([specials, rng.normal(size=2000).astype(np.float32) * np.float32(1e10) ** rng.integers(-3, 4, 2000)]).astype(np.float32)
    u = oracle.map_float_to_uint(f.view(np.uint32))
    assert np.array_equal(oracle.map_uint_to_float(u), f.view(np.uint32))
    order = np.argsort(u, kind="stable")
    assert np.all(np.diff(f[order].astype(np.float64)) >= 0)
    # -0.0 sorts strictly before +0.0 under the map
    assert u[1] < u[0]
