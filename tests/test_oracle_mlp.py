"""Pins the CPU oracle's matmul (and, below, the MLP pieces built on it) against float64 NumPy."""
import numpy as np
import pytest

from conftest import sum_err
from oracle import oracle


@pytest.mark.parametrize("layout", ["nn", "nt", "tn"])
@pytest.mark.parametrize("mnk", [(1, 1, 1), (5, 7, 3), (33, 17, 65), (128, 40, 100)])
def test_matmul_layouts(layout, mnk):
    m, n, k = mnk
    rng = np.random.default_rng(71)
    a = rng.normal(size=(m, k)).astype(np.float32)
    b = rng.normal(size=(k, n)).astype(np.float32)
    ref = a.astype(np.float64) @ b.astype(np.float64)
    scale = np.abs(a).astype(np.float64) @ np.abs(b).astype(np.float64)
    aa = a.T.copy() if layout == "tn" else a
    bb = b.T.copy() if layout == "nt" else b
    assert sum_err(oracle.matmul(aa, bb, layout), ref, scale) < 1e-6


def test_matmul_identity_and_outer_product():
    rng = np.random.default_rng(72)
    a = rng.normal(size=(9, 9)).astype(np.float32)
    assert np.array_equal(oracle.matmul(a, np.eye(9, dtype=np.float32)), a)
    u, v = rng.normal(size=(6, 1)).astype(np.float32), rng.normal(size=(1, 4)).astype(np.float32)
    assert np.array_equal(oracle.matmul(u, v), u * v)
