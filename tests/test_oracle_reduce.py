"""Pins the CPU oracle's reductions and softmax against float64 NumPy closed forms."""
import numpy as np
import pytest

from oracle import oracle
from conftest import rel_err, sum_err

# (rows, cols): unsplit (<1024), split with a multiple of 128, split with a ragged last chunk.
SHAPES = [(1, 1), (3, 7), (37, 100), (5, 1023), (9, 1024), (33, 4096), (7, 1300), (300, 257)]


@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("op", ["sum", "max", "min"])
def test_reduce_rows(shape, op):
    rng = np.random.default_rng(11)
    x = rng.uniform(-4, 4, shape).astype(np.float32)
    ref = getattr(np, op)(x.astype(np.float64), axis=1)
    if op != "sum" and shape[1] >= 1024 and shape[1] % 128:
        # The reference pads the ragged last chunk of a split axis with 0 (Implementations.cpp:56-69), so
        # max/min see an extra 0 there.
        ref = getattr(np, "maximum" if op == "max" else "minimum")(ref, 0.0)
    got = oracle.reduce_rows(op, x)
    if op == "sum":
        assert sum_err(got, ref, np.abs(x).sum(axis=1)) < 1e-6
    else:
        assert np.array_equal(got, ref.astype(np.float32))


@pytest.mark.parametrize("shape", [(s[1], s[0]) for s in SHAPES])
@pytest.mark.parametrize("op", ["sum", "max", "min"])
def test_reduce_cols(shape, op):
    rng = np.random.default_rng(12)
    x = rng.uniform(-4, 4, shape).astype(np.float32)
    ref = getattr(np, op)(x.astype(np.float64), axis=0)
    if op != "sum" and shape[0] >= 1024 and shape[0] % 128:
        ref = getattr(np, "maximum" if op == "max" else "minimum")(ref, 0.0)
    got = oracle.reduce_cols(op, x)
    if op == "sum":
        assert sum_err(got, ref, np.abs(x).sum(axis=0)) < 1e-6
    else:
        assert np.array_equal(got, ref.astype(np.float32))


@pytest.mark.parametrize("shape", [(1, 1), (4, 10), (17, 1000), (8, 1024), (5, 4096), (3, 1500)])
def test_softmax_rows(shape):
    rng = np.random.default_rng(13)
    x = rng.uniform(-4, 4, shape).astype(np.float32)
    x64 = x.astype(np.float64)
    m = x64.max(axis=1, keepdims=True)
    if shape[1] >= 1024 and shape[1] % 128:
        m = np.maximum(m, 0.0)  # zero padding of the ragged chunk enters the row max (cancels in the ratio)
    e = np.exp(x64 - m)
    ref = e / e.sum(axis=1, keepdims=True)
    got = oracle.softmax_rows(x)
    assert rel_err(got, ref) < 1e-5
    assert np.allclose(got.sum(axis=1), 1.0, atol=1e-5)


def test_reduce_detects_structure():
    """A distinguishable value in every position: a dropped chunk or transposed index changes the sum."""
    R, K = 5, 2048
    x = (np.arange(R * K, dtype=np.float64).reshape(R, K) % 251) * (1 + np.arange(R)[:, None])
    assert rel_err(oracle.reduce_rows("sum", x.astype(np.float32)), x.sum(axis=1)) < 1e-6
    assert rel_err(oracle.reduce_cols("sum", x.T.copy().astype(np.float32)), x.sum(axis=1)) < 1e-6
