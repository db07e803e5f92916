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


# ---- the MLP training step ------------------------------------------------------------------------------
def features64(coords):
    c = coords.astype(np.float64)
    out = np.empty((c.shape[0], 64))
    for f in range(64):
        axis, k, s = f // 32, (f % 32) // 2, f % 2
        arg = np.float64(np.float32(np.float32(1 << k) * np.float32(3.14159274))) * c[:, axis]
        out[:, f] = np.sin(arg) if s == 0 else np.cos(arg)
    return out


def forward64(F, params):
    h = F
    acts = [F]
    for l in range(3):
        h = np.maximum(h @ params[2 * l] + params[2 * l + 1], 0.0)
        acts.append(h)
    return h @ params[6] + params[7], acts


def loss64(F, params, target):
    y, _ = forward64(F, params)
    return np.mean((y - target) ** 2)


def step64(coords, target, params, m, v, t, lr=1e-3, b1=0.9, b2=0.999, eps=1e-8):
    F = features64(coords)
    P = [p.astype(np.float64) for p in params]
    y, acts = forward64(F, P)
    T = target.astype(np.float64)
    loss = np.mean((y - T) ** 2)
    up = 2 * (y - T) / y.size
    grads = [None] * 8
    for l in range(3, -1, -1):
        grads[2 * l] = acts[l].T @ up
        grads[2 * l + 1] = up.sum(0)
        if l > 0:
            up = (up @ P[2 * l].T) * (acts[l] > 0)
    t = t + 1
    outs = []
    for i in range(8):
        g = grads[i]
        mm = b1 * m[i] + (1 - b1) * g
        vv = b2 * v[i] + (1 - b2) * g * g
        outs.append((P[i] - lr * (mm / (1 - b1 ** t)) / (np.sqrt(vv / (1 - b2 ** t)) + eps), mm, vv))
    return loss, outs, grads


def test_fourier_features():
    coords = np.random.default_rng(73).uniform(0, 1, (100, 2)).astype(np.float32)
    got = oracle.fourier_features(coords)
    # the argument reaches 2^15 * pi: an fp32 argument is only good to ~1e-3 rad there, so compare the
    # low frequencies tightly and the high ones against fp32-rounded arguments
    ref = features64(coords)
    assert np.max(np.abs(got[:, :8] - ref[:, :8])) < 1e-6
    arg32 = lambda f: np.float32(np.float32(1 << ((f % 32) // 2)) * np.float32(3.14159274)) * coords[:, f // 32]
    for f in range(64):
        r = np.sin(arg32(f).astype(np.float64)) if f % 2 == 0 else np.cos(arg32(f).astype(np.float64))
        assert np.max(np.abs(got[:, f] - r)) < 2e-6


def test_mlp_step_matches_float64_and_finite_differences():
    B = 64
    coords, target, params, m, v = oracle.mlp_inputs(B, seed=5)
    rng = np.random.default_rng(6)
    for i in (1, 3, 5, 7):
        params[i] = rng.normal(size=params[i].shape).astype(np.float32) * 0.1  # non-zero biases
    m = [rng.normal(size=p.shape).astype(np.float32) * 0.01 for p in params]
    v = [np.abs(rng.normal(size=p.shape)).astype(np.float32) * 1e-4 for p in params]
    loss, p_out, m_out, v_out, grads = oracle.mlp_step(coords, target, params, m, v, t=3.0)
    # float64 restatement on the oracle's own fp32 features (the argument rounding is pinned separately)
    ref_loss, outs, ref_grads = step64(coords, target, params, m, v, 3.0)
    F32 = oracle.fourier_features(coords).astype(np.float64)
    assert abs(loss - loss64(F32, [p.astype(np.float64) for p in params], target.astype(np.float64))) < 1e-5 * ref_loss
    P = [p.astype(np.float64) for p in params]
    # gradients by central differences of the float64 loss: pins the backward formulas themselves
    for i in (0, 3, 6, 7):
        flat_idx = rng.integers(0, params[i].size, 4)
        for j in flat_idx:
            d = 1e-5
            Pp = [q.copy() for q in P]; Pm = [q.copy() for q in P]
            Pp[i].flat[j] += d; Pm[i].flat[j] -= d
            fd = (loss64(F32, Pp, target.astype(np.float64)) - loss64(F32, Pm, target.astype(np.float64))) / (2 * d)
            assert abs(grads[i].flat[j] - fd) < 1e-4 * max(abs(fd), 1e-3)
    # Adam against the textbook update, fed with the oracle's own gradients
    for i in range(8):
        g = grads[i].astype(np.float64)
        mm = 0.9 * m[i] + 0.1 * g
        vv = 0.999 * v[i] + 0.001 * g * g
        p_ref = params[i] - 1e-3 * (mm / (1 - 0.9 ** 4)) / (np.sqrt(vv / (1 - 0.999 ** 4)) + 1e-8)
        assert np.allclose(m_out[i], mm, rtol=1e-4, atol=1e-6 * np.abs(mm).max())
        assert np.allclose(v_out[i], vv, rtol=1e-4, atol=1e-6 * np.abs(vv).max())
        assert np.allclose(p_out[i], p_ref, rtol=1e-4, atol=1e-6 * max(np.abs(p_ref).max(), 1e-3))
