"""TEST INFRASTRUCTURE: ctypes loader for liboracle.so plus NumPy-facing wrappers.

The shared object is built by `make -C oracle` (also done by __graft_entry__.build()).
"""
from __future__ import annotations

import ctypes as C
import subprocess
from pathlib import Path

import numpy as np

HERE = Path(__file__).resolve().parent
LIB_PATH = HERE / "liboracle.so"
_lib = None

_OPS = {"sum": 0, "max": 1, "min": 2}
_f32p = np.ctypeslib.ndpointer(dtype=np.float32, flags="C_CONTIGUOUS")
_u32p = np.ctypeslib.ndpointer(dtype=np.uint32, flags="C_CONTIGUOUS")


def build() -> Path:
    subprocess.run(["make", "-C", str(HERE), "-B", "liboracle.so"], check=True, stdout=subprocess.PIPE, stderr=subprocess.STDOUT)
    return LIB_PATH


def load() -> C.CDLL:
    global _lib
    if _lib is None:
        if not LIB_PATH.exists():
            build()
        lib = C.CDLL(str(LIB_PATH))
        lib.oracle_reduce_partial_words.restype = C.c_size_t
        lib.oracle_reduce_partial_words.argtypes = [C.c_size_t, C.c_size_t]
        lib.oracle_reduce_rows_f32.argtypes = [C.c_int, _f32p, _f32p, _f32p, C.c_int, C.c_int]
        lib.oracle_reduce_cols_f32.argtypes = [C.c_int, _f32p, _f32p, _f32p, C.c_int, C.c_int]
        lib.oracle_softmax_rows_f32.argtypes = [_f32p, _f32p, _f32p, _f32p, _f32p, C.c_int, C.c_int]
        _lib = lib
    return _lib


def reduce_rows(op: str, x: np.ndarray) -> np.ndarray:
    lib = load()
    x = np.ascontiguousarray(x, dtype=np.float32)
    R, K = x.shape
    out = np.empty(R, np.float32)
    partial = np.empty(lib.oracle_reduce_partial_words(R, K), np.float32)
    assert lib.oracle_reduce_rows_f32(_OPS[op], x, out, partial, R, K) == 0
    return out


def reduce_cols(op: str, x: np.ndarray) -> np.ndarray:
    lib = load()
    x = np.ascontiguousarray(x, dtype=np.float32)
    K, Cc = x.shape
    out = np.empty(Cc, np.float32)
    partial = np.empty(lib.oracle_reduce_partial_words(Cc, K), np.float32)
    assert lib.oracle_reduce_cols_f32(_OPS[op], x, out, partial, K, Cc) == 0
    return out


def softmax_rows(x: np.ndarray) -> np.ndarray:
    lib = load()
    x = np.ascontiguousarray(x, dtype=np.float32)
    R, K = x.shape
    y = np.empty_like(x)
    row_max = np.empty(R, np.float32)
    row_sum = np.empty(R, np.float32)
    partial = np.empty(lib.oracle_reduce_partial_words(R, K), np.float32)
    assert lib.oracle_softmax_rows_f32(x, y, row_max, row_sum, partial, R, K) == 0
    return y


def scan_inclusive(x: np.ndarray) -> np.ndarray:
    """Inclusive prefix sum along the last axis of a 1-D or 2-D u32 / i32 / f32 array."""
    lib = load()
    x = np.ascontiguousarray(x)
    lines, n = (1, x.shape[0]) if x.ndim == 1 else x.shape
    out = np.empty_like(x)
    fn = {"u": lib.oracle_scan_inclusive_u32, "i": lib.oracle_scan_inclusive_i32, "f": lib.oracle_scan_inclusive_f32}[x.dtype.kind]
    fn.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.c_int]
    assert x.dtype.itemsize == 4
    assert fn(x.ctypes.data, out.ctypes.data, lines, n) == 0
    return out


_KEY_KINDS = {"u": 0, "i": 1, "f": 2}


def radix_sort_kv(keys: np.ndarray, vals: np.ndarray | None = None):
    """Stable key(/value) sort with the reference's 6x6-bit histogram radix sort. Returns (keys, vals)."""
    lib = load()
    keys = np.ascontiguousarray(keys)
    assert keys.dtype.itemsize == 4 and keys.ndim == 1
    n = keys.shape[0]
    kout, ktmp = np.empty_like(keys), np.empty_like(keys)
    fn = lib.oracle_radix_sort_kv
    fn.argtypes = [C.c_int] + [C.c_void_p] * 6 + [C.c_int]
    if vals is None:
        assert fn(_KEY_KINDS[keys.dtype.kind], keys.ctypes.data, None, kout.ctypes.data, None, ktmp.ctypes.data, None, n) == 0
        return kout, None
    vals = np.ascontiguousarray(vals)
    assert vals.dtype.itemsize == 4 and vals.shape == keys.shape
    vout, vtmp = np.empty_like(vals), np.empty_like(vals)
    assert fn(_KEY_KINDS[keys.dtype.kind], keys.ctypes.data, vals.ctypes.data, kout.ctypes.data, vout.ctypes.data, ktmp.ctypes.data, vtmp.ctypes.data, n) == 0
    return kout, vout


def ops(x, y, a, b, u, w):
    """Every scalar op of the op table once, as the C++ backend evaluates it: returns F[42,n], I[28,n], U[16,n]."""
    lib = load()
    i32p = np.ctypeslib.ndpointer(dtype=np.int32, flags="C_CONTIGUOUS")
    lib.oracle_ops.argtypes = [_f32p, _f32p, i32p, i32p, _u32p, _u32p, C.c_int, _f32p, i32p, _u32p]
    n = x.size
    F = np.empty((lib.oracle_ops_float_rows(), n), np.float32)
    I = np.empty((lib.oracle_ops_int_rows(), n), np.int32)
    U = np.empty((lib.oracle_ops_uint_rows(), n), np.uint32)
    lib.oracle_ops(np.ascontiguousarray(x, np.float32), np.ascontiguousarray(y, np.float32), np.ascontiguousarray(a, np.int32),
                   np.ascontiguousarray(b, np.int32), np.ascontiguousarray(u, np.uint32), np.ascontiguousarray(w, np.uint32), n, F, I, U)
    return F, I, U


def ops_inputs(n: int, seed: int = 77):
    """Inputs of the op-table program: floats in (-3, 3) with exact zeros, small and extreme ints, full-range uints."""
    rng = np.random.default_rng(seed)
    x = rng.uniform(-3, 3, n).astype(np.float32)
    y = rng.uniform(-3, 3, n).astype(np.float32)
    y[::17] = 0.0
    x[5::29] = np.float32(0.0)
    x[7::31] = np.round(x[7::31])           # integers and half-way cases for round / floor / ceil / frac
    x[11::37] = np.round(x[11::37]) + 0.5
    a = rng.integers(-1000, 1000, n).astype(np.int32)
    b = rng.integers(-40, 40, n).astype(np.int32)
    a[3::23] = rng.integers(-2**31, 2**31 - 1, a[3::23].size).astype(np.int32)
    a[::101] = 0
    u = rng.integers(0, 2**32, n, dtype=np.uint64).astype(np.uint32)
    w = rng.integers(0, 2**32, n, dtype=np.uint64).astype(np.uint32)
    w[::13] = rng.integers(0, 50, w[::13].size).astype(np.uint32)
    return x, y, a, b, u, w


def map_float_to_uint(bits: np.ndarray) -> np.ndarray:
    lib = load()
    lib.oracle_map_float_to_uint.restype = C.c_uint32
    lib.oracle_map_float_to_uint.argtypes = [C.c_uint32]
    return np.array([lib.oracle_map_float_to_uint(int(b)) for b in np.asarray(bits, dtype=np.uint32)], dtype=np.uint32)


def map_uint_to_float(bits: np.ndarray) -> np.ndarray:
    lib = load()
    lib.oracle_map_uint_to_float.restype = C.c_uint32
    lib.oracle_map_uint_to_float.argtypes = [C.c_uint32]
    return np.array([lib.oracle_map_uint_to_float(int(b)) for b in np.asarray(bits, dtype=np.uint32)], dtype=np.uint32)


def wave_eq(u: np.ndarray, v: np.ndarray, dt: float = 0.1, steps: int = 1):
    """`steps` sine-Gordon leapfrog steps on a periodic grid; returns (u, v) after the last step."""
    lib = load()
    u = np.array(u, dtype=np.float32, order="C", copy=True)
    v = np.array(v, dtype=np.float32, order="C", copy=True)
    N, M = u.shape
    fn = lib.oracle_wave_eq_run
    fn.argtypes = [_f32p, _f32p, _f32p, _f32p, C.c_int, C.c_int, C.c_float, C.c_int]
    assert fn(u, v, np.empty_like(u), np.empty_like(v), N, M, dt, steps) == 0
    return u, v


def sine_gordon_initial_field(n: int, m: int, seed: int = 1235) -> np.ndarray:
    """benchmark config 1 initial condition: seeded sum of 16 Gaussians, amplitude U(0.5,2), sigma U(8,64) px."""
    rng = np.random.default_rng(seed)
    amp = rng.uniform(0.5, 2.0, 16)
    sigma = rng.uniform(8.0, 64.0, 16)
    cy = rng.uniform(0, n, 16)
    cx = rng.uniform(0, m, 16)
    y = np.arange(n, dtype=np.float64)[:, None]
    x = np.arange(m, dtype=np.float64)[None, :]
    u = np.zeros((n, m), np.float64)
    for k in range(16):
        u += amp[k] * np.exp(-((x - cx[k]) ** 2 + (y - cy[k]) ** 2) / (2 * sigma[k] ** 2))
    return u.astype(np.float32)


def nbody_step(x: np.ndarray, v: np.ndarray, m: np.ndarray, dt: float = 1e-3, eps: float = 1e-3):
    """One symplectic-Euler step of the softened all-pairs system; returns (x_new, v_new)."""
    lib = load()
    x = np.ascontiguousarray(x, dtype=np.float32)
    v = np.ascontiguousarray(v, dtype=np.float32)
    m = np.ascontiguousarray(m, dtype=np.float32)
    n = x.shape[0]
    assert x.shape == (n, 3) and v.shape == (n, 3) and m.shape == (n,)
    xn, vn = np.empty_like(x), np.empty_like(v)
    fn = lib.oracle_nbody_step
    fn.argtypes = [_f32p, _f32p, _f32p, _f32p, _f32p, C.c_int, C.c_float, C.c_float]
    assert fn(x, v, m, xn, vn, n, dt, eps) == 0
    return xn, vn


def nbody_inputs(n: int, seed: int = 1238):
    """benchmark config 4 inputs: X ~ U[-1,1]^3, V ~ N(0, 0.01), masses ~ lognormal(0, 0.5)."""
    rng = np.random.default_rng(seed)
    x = rng.uniform(-1, 1, (n, 3)).astype(np.float32)
    v = rng.normal(0, 0.01, (n, 3)).astype(np.float32)
    m = rng.lognormal(0.0, 0.5, n).astype(np.float32)
    return x, v, m


def matmul(a: np.ndarray, b: np.ndarray, layout: str = "nn") -> np.ndarray:
    """C = op(A) op(B): 'nn' A[M,K] B[K,N]; 'nt' A[M,K] B[N,K]; 'tn' A[K,M] B[K,N]."""
    lib = load()
    a = np.ascontiguousarray(a, dtype=np.float32)
    b = np.ascontiguousarray(b, dtype=np.float32)
    if layout == "nn":
        (m, k), (k2, n) = a.shape, b.shape
    elif layout == "nt":
        (m, k), (n, k2) = a.shape, b.shape
    else:
        (k, m), (k2, n) = a.shape, b.shape
    assert k == k2
    c = np.empty((m, n), np.float32)
    fn = lib.oracle_matmul_f32
    fn.argtypes = [C.c_int, _f32p, _f32p, _f32p, C.c_int, C.c_int, C.c_int]
    assert fn({"nn": 0, "nt": 1, "tn": 2}[layout], a, b, c, m, n, k) == 0
    return c


MLP_SHAPES = [(64, 256), (256,), (256, 256), (256,), (256, 256), (256,), (256, 3), (3,)]


def mlp_inputs(batch: int, seed: int = 1239):
    """benchmark config 5 inputs: coords U[0,1]^2, target U[0,1]^3, He-normal weights, zero biases and Adam state."""
    rng = np.random.default_rng(seed)
    coords = rng.uniform(0, 1, (batch, 2)).astype(np.float32)
    target = rng.uniform(0, 1, (batch, 3)).astype(np.float32)
    params = []
    for shp in MLP_SHAPES:
        if len(shp) == 2:
            params.append((rng.normal(size=shp) * np.sqrt(2.0 / shp[0])).astype(np.float32))
        else:
            params.append(np.zeros(shp, np.float32))
    m = [np.zeros_like(p) for p in params]
    v = [np.zeros_like(p) for p in params]
    return coords, target, params, m, v


def mlp_step(coords, target, params, m, v, t=0.0, lr=1e-3, b1=0.9, b2=0.999, eps=1e-8):
    """One forward + backward + Adam step; returns (loss, params', m', v', grads)."""
    lib = load()
    B = coords.shape[0]
    arr = lambda xs: (C.c_void_p * 8)(*[x.ctypes.data for x in xs])
    cont = lambda xs: [np.ascontiguousarray(x, dtype=np.float32) for x in xs]
    params, m, v = cont(params), cont(m), cont(v)
    coords = np.ascontiguousarray(coords, dtype=np.float32)
    target = np.ascontiguousarray(target, dtype=np.float32)
    p_out = [np.empty_like(p) for p in params]
    m_out = [np.empty_like(p) for p in params]
    v_out = [np.empty_like(p) for p in params]
    g_out = [np.empty_like(p) for p in params]
    fn = lib.oracle_mlp_step
    fn.restype = C.c_float
    fn.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_float, C.c_float, C.c_float, C.c_float, C.c_float,
                   C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p]
    loss = fn(coords.ctypes.data, target.ctypes.data, B, arr(params), arr(m), arr(v), t, lr, b1, b2, eps, arr(p_out), arr(m_out), arr(v_out), arr(g_out))
    return float(loss), p_out, m_out, v_out, g_out


def fourier_features(coords: np.ndarray) -> np.ndarray:
    lib = load()
    coords = np.ascontiguousarray(coords, dtype=np.float32)
    out = np.empty((coords.shape[0], 64), np.float32)
    lib.oracle_fourier_features.argtypes = [_f32p, _f32p, C.c_int]
    lib.oracle_fourier_features(coords, out, coords.shape[0])
    return out
