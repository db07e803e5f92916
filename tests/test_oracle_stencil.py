"""Pins the CPU oracle's sine-Gordon step against float64 closed forms."""
import numpy as np

from conftest import sum_err
from oracle import oracle


def term_scale(u, v, dt):
    """Sum of magnitudes of the terms that make up v_new and u_new: the scale against which a correctly
    rounded fp32 evaluation (in any order, with or without FMA) errs by a few 1e-8 -- the update cancels
    (lap subtracts 4u from its neighbours), so error relative to the RESULT is unbounded near zeros."""
    a = np.abs(u.astype(np.float64))
    taps = np.roll(a, 1, 0) + np.roll(a, -1, 0) + np.roll(a, 1, 1) + np.roll(a, -1, 1) + 4 * a
    sv = np.abs(v.astype(np.float64)) + dt * (taps + np.abs(np.sin(u.astype(np.float64))))
    return a + dt * sv, sv


def _step64(u, v, dt):
    u = u.astype(np.float64)
    v = v.astype(np.float64)
    lap = np.roll(u, 1, 0) + np.roll(u, -1, 0) + np.roll(u, 1, 1) + np.roll(u, -1, 1) - 4 * u
    v = v + dt * (lap - np.sin(u))
    return u + dt * v, v


def test_matches_np_roll_closed_form():
    rng = np.random.default_rng(51)
    for shape in [(16, 16), (37, 53), (1, 7), (130, 64)]:
        u = rng.normal(size=shape).astype(np.float32)
        v = rng.normal(size=shape).astype(np.float32)
        gu, gv = oracle.wave_eq(u, v, 0.1, 1)
        ru, rv = _step64(u, v, np.float32(0.1))
        su, sv = term_scale(u, v, 0.1)
        assert sum_err(gu, ru, su) < 1e-6 and sum_err(gv, rv, sv) < 1e-6


def test_constant_field_has_zero_laplacian():
    u = np.full((40, 24), 0.7, np.float32)
    v = np.zeros_like(u)
    gu, gv = oracle.wave_eq(u, v, 0.1, 1)
    assert np.allclose(gv, -0.1 * np.sin(0.7), rtol=1e-6)
    assert np.allclose(gu, 0.7 + 0.1 * gv, rtol=1e-6)


def test_plane_wave_eigenvalue():
    """For u = eps*cos(kx*j + ky*i) the discrete Laplacian is -(4 - 2cos kx - 2cos ky) u exactly; rows and
    columns use different wavenumbers so a transposed index shows."""
    N, M, eps = 48, 64, 1e-3
    ky, kx = 2 * np.pi * 3 / N, 2 * np.pi * 5 / M
    i, j = np.mgrid[0:N, 0:M]
    u = (eps * np.cos(kx * j + ky * i)).astype(np.float32)
    v = np.zeros_like(u)
    _, gv = oracle.wave_eq(u, v, 0.1, 1)
    lam = 4 - 2 * np.cos(kx) - 2 * np.cos(ky)
    expect = 0.1 * (-lam * u.astype(np.float64) - np.sin(u.astype(np.float64)))
    assert np.max(np.abs(gv - expect)) < 2e-9 + 1e-5 * np.max(np.abs(expect))


def test_many_steps_track_float64():
    u = oracle.sine_gordon_initial_field(96, 96)
    v = np.zeros_like(u)
    gu, gv = oracle.wave_eq(u, v, 0.1, 50)
    ru, rv = u.astype(np.float64), v.astype(np.float64)
    for _ in range(50):
        ru, rv = _step64(ru, rv, 0.1)
    assert np.max(np.abs(gu - ru)) < 1e-4 * np.max(np.abs(ru))
