"""Pins the CPU oracle's N-body step against float64 direct summation and conservation laws."""
import numpy as np

from oracle import oracle


def accel64(x, m, eps):
    x = x.astype(np.float64)
    d = x[None, :, :] - x[:, None, :]                 # d[i, j] = x_j - x_i
    r2 = (d ** 2).sum(-1) + eps ** 2
    w = m.astype(np.float64)[None, :] / r2 ** 1.5
    a = (w[:, :, None] * d).sum(1)
    scale = (np.abs(w)[:, :, None] * np.abs(d)).sum(1)  # sum of term magnitudes
    return a, scale


def test_matches_direct_sum():
    x, v, m = oracle.nbody_inputs(700)
    dt, eps = 1e-3, 1e-3
    xn, vn = oracle.nbody_step(x, v, m, dt, eps)
    a, scale = accel64(x, m, eps)
    v_ref = v.astype(np.float64) + a * dt
    x_ref = x.astype(np.float64) + v_ref * dt
    assert np.max(np.abs(vn - v_ref) / (np.abs(v) + scale * dt)) < 1e-5
    assert np.max(np.abs(xn - x_ref) / (np.abs(x) + 1e-6)) < 1e-5


def test_momentum_is_conserved():
    x, v, m = oracle.nbody_inputs(512, seed=7)
    _, vn = oracle.nbody_step(x, v, m, 1e-3, 1e-3)
    dv = vn.astype(np.float64) - v.astype(np.float64)
    dp = (m[:, None].astype(np.float64) * dv).sum(0)
    scale = (m[:, None] * np.abs(dv)).sum(0)
    assert np.all(np.abs(dp) < 1e-4 * scale)


def test_two_bodies_closed_form():
    x = np.array([[0, 0, 0], [2, 0, 0]], np.float32)
    v = np.zeros((2, 3), np.float32)
    m = np.array([3.0, 5.0], np.float32)
    eps, dt = 0.5, 0.1
    _, vn = oracle.nbody_step(x, v, m, dt, eps)
    r2 = 4 + eps ** 2
    assert np.allclose(vn[0], [5.0 * 2 / r2 ** 1.5 * dt, 0, 0], rtol=1e-6)
    assert np.allclose(vn[1], [-3.0 * 2 / r2 ** 1.5 * dt, 0, 0], rtol=1e-6)
