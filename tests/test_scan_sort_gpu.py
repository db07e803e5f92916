"""Parity of the HIP prefix scan and radix sort (through the C ABI) with the CPU oracle: bit-exact."""
import numpy as np
import pytest

from oracle import oracle

pytestmark = pytest.mark.gpu


# ---- scan ------------------------------------------------------------------------------------------
@pytest.mark.parametrize("n", [1, 2, 63, 64, 65, 4095, 4096, 4097, 8191, 100_003, 1 << 20, (1 << 22) + 5])
def test_scan_u32_bit_exact(rt, n):
    rng = np.random.default_rng(41)
    x = rng.integers(0, 2**32, n, dtype=np.uint64).astype(np.uint32)
    xb = rt.DeviceBuffer.from_numpy(x)
    ob = rt.DeviceBuffer(n)
    rt.scan_inclusive(xb, ob, n, np.uint32)
    got = ob.numpy(np.uint32)
    assert np.array_equal(got, oracle.scan_inclusive(x))
    rt.scan_inclusive(xb, xb, n, np.uint32)  # in place
    assert np.array_equal(xb.numpy(np.uint32), got)


def test_scan_i32_bit_exact(rt):
    rng = np.random.default_rng(42)
    x = rng.integers(-1000, 1000, 300_001, dtype=np.int64).astype(np.int32)
    xb = rt.DeviceBuffer.from_numpy(x)
    ob = rt.DeviceBuffer(x.size)
    rt.scan_inclusive(xb, ob, x.size, np.int32)
    assert np.array_equal(ob.numpy(np.int32), oracle.scan_inclusive(x))


def test_scan_unaligned_views(rt):
    """Input/output that do not start on a 16-byte boundary take the scalar load path."""
    from tensorfrost_amd._lib import call

    x = np.arange(1, 10_001, dtype=np.uint32)
    xb = rt.DeviceBuffer.from_numpy(np.concatenate([[0], x]).astype(np.uint32))
    ob = rt.DeviceBuffer(x.size + 3)
    call("tfhip_scan_inclusive_u32", xb.ptr + 4, ob.ptr + 12, x.size)
    assert np.array_equal(ob.numpy(np.uint32, (x.size,), offset_words=3), np.cumsum(x, dtype=np.uint64).astype(np.uint32))


@pytest.mark.parametrize("n", [1, 100, 4096, 4097, 1 << 20, (1 << 24) + 3])
def test_scan_f32(rt, n):
    rng = np.random.default_rng(43)
    x = rng.uniform(0, 1, n).astype(np.float32)
    xb = rt.DeviceBuffer.from_numpy(x)
    ob = rt.DeviceBuffer(n)
    rt.scan_inclusive(xb, ob, n, np.float32)
    got = ob.numpy(np.float32)
    ref = np.cumsum(x.astype(np.float64))
    assert np.max(np.abs(got - ref) / ref) < 1e-4  # north-star tolerance for reductions
    if n <= 1 << 20:
        orc = oracle.scan_inclusive(x)
        assert np.max(np.abs(got - orc) / np.maximum(np.abs(orc), 1e-30)) < 1e-4
    rt.scan_inclusive(xb, ob, n, np.float32)
    assert np.array_equal(ob.numpy(np.float32), got), "f32 scan must be reproducible run to run"


ROW_SHAPES = [(1, 1), (5, 3), (17, 100), (1000, 64), (333, 257), (64, 1024), (100, 1028), (37, 5000), (3, 70000), (20, 65536), (2, 1 << 20),
              (4096, 4096), (25 * 61, 153),
              # lane groups of 1 .. 32 for short aligned rows; segments for few long rows (ragged last segment, unaligned rows)
              (1000, 4), (777, 8), (5000, 16), (4099, 20), (2049, 100), (1025, 128), (7, 100003), (64, 40000), (1, (1 << 22) + 8), (3, 1 << 22)]  # the last one is the reference's scan example (examples/Algorithms/scan.ipynb)


@pytest.mark.parametrize("shape", ROW_SHAPES)
def test_scan_rows_u32_bit_exact(rt, shape):
    """Prefix sums along the last axis, every row on its own: one wave per short row, four per long row, unaligned
    rows (cols % 4 != 0), ragged row counts, few very long rows (device-wide scan per row); in place."""
    rng = np.random.default_rng(shape[0] + shape[1])
    x = rng.integers(0, 2**32, shape, dtype=np.uint64).astype(np.uint32)
    xb = rt.DeviceBuffer.from_numpy(x)
    ob = rt.DeviceBuffer(x.size)
    rt.scan_inclusive_rows(xb, ob, shape[0], shape[1], np.uint32)
    got = ob.numpy(np.uint32, shape)
    assert np.array_equal(got, np.cumsum(x, axis=1, dtype=np.uint32))
    for r in (0, shape[0] - 1):
        assert np.array_equal(got[r], oracle.scan_inclusive(x[r]))
    rt.scan_inclusive_rows(xb, xb, shape[0], shape[1], np.uint32)
    assert np.array_equal(xb.numpy(np.uint32, shape), got)


@pytest.mark.parametrize("shape", ROW_SHAPES)
def test_scan_rows_f32(rt, shape):
    """f32 rows: the additions of a row are grouped by lane and wave, so results are compared at 1e-4 of the running
    sum of magnitudes (the bound for any order of fp32 additions is n * eps of it)."""
    rng = np.random.default_rng(shape[0] * 3 + shape[1])
    x = rng.uniform(-1, 1, shape).astype(np.float32)
    xb = rt.DeviceBuffer.from_numpy(x)
    ob = rt.DeviceBuffer(x.size)
    rt.scan_inclusive_rows(xb, ob, shape[0], shape[1], np.float32)
    got = ob.numpy(np.float32, shape)
    want = np.cumsum(x.astype(np.float64), axis=1)
    scale = np.cumsum(np.abs(x).astype(np.float64), axis=1)
    assert np.max(np.abs(got - want) / scale) < 1e-4
    r = shape[0] // 2
    assert np.max(np.abs(got[r] - oracle.scan_inclusive(x[r])) / scale[r]) < 1e-4


def test_scan_rows_integer_values_in_f32_are_exact(rt):
    x = np.random.default_rng(8).integers(-8, 9, (300, 3000)).astype(np.float32)
    xb = rt.DeviceBuffer.from_numpy(x)
    rt.scan_inclusive_rows(xb, xb, 300, 3000, np.float32)
    assert np.array_equal(xb.numpy(np.float32, (300, 3000)), np.cumsum(x, axis=1, dtype=np.float32))


COL_SHAPES = [(1, 1, 1), (1, 5, 3), (1, 1000, 64), (1, 131072, 64), (3, 17, 100), (1024, 128, 32), (1, 100003, 7), (2, 4096, 1000), (1, 16, 70000),
              (25, 61, 153)]


@pytest.mark.parametrize("shape", COL_SHAPES)
def test_scan_cols_u32_bit_exact(rt, shape):
    """Prefix sums down the columns of a batch of matrices (an axis that is not the last): slabs of rows with a carry,
    narrow matrices sharing a wave, a single slab, in place."""
    b, r, c = shape
    rng = np.random.default_rng(b + r + c)
    x = rng.integers(0, 2**32, shape, dtype=np.uint64).astype(np.uint32)
    xb = rt.DeviceBuffer.from_numpy(x)
    ob = rt.DeviceBuffer(x.size)
    rt.scan_inclusive_cols(xb, ob, b, r, c, np.uint32)
    got = ob.numpy(np.uint32, shape)
    assert np.array_equal(got, np.cumsum(x, axis=1, dtype=np.uint32))
    assert np.array_equal(got[-1, :, c // 2], oracle.scan_inclusive(np.ascontiguousarray(x[-1, :, c // 2])))
    rt.scan_inclusive_cols(xb, xb, b, r, c, np.uint32)
    assert np.array_equal(xb.numpy(np.uint32, shape), got)


@pytest.mark.parametrize("shape", COL_SHAPES)
def test_scan_cols_f32(rt, shape):
    b, r, c = shape
    rng = np.random.default_rng(b * 5 + r + c)
    x = rng.uniform(-1, 1, shape).astype(np.float32)
    xb = rt.DeviceBuffer.from_numpy(x)
    ob = rt.DeviceBuffer(x.size)
    rt.scan_inclusive_cols(xb, ob, b, r, c, np.float32)
    got = ob.numpy(np.float32, shape)
    want = np.cumsum(x.astype(np.float64), axis=1)
    scale = np.cumsum(np.abs(x).astype(np.float64), axis=1)
    assert np.max(np.abs(got - want) / scale) < 1e-4


def test_scan_rows_and_cols_at_2_pow_28_elements(rt):
    """Size-independent properties at 2^28 elements: the last element of every scanned row (column) is the row's
    (column's) sum, computed independently with NumPy in 64 bits and wrapped; first differences give the input back."""
    rows, cols = 1 << 14, 1 << 14
    rng = np.random.default_rng(2028)
    x = rng.integers(0, 2**32, (rows, cols), dtype=np.uint64).astype(np.uint32)
    xb = rt.DeviceBuffer.from_numpy(x)
    ob = rt.DeviceBuffer(x.size)
    rt.scan_inclusive_rows(xb, ob, rows, cols, np.uint32)
    got = ob.numpy(np.uint32, (rows, cols))
    assert np.array_equal(got[:, -1], (x.sum(axis=1, dtype=np.uint64) & 0xFFFFFFFF).astype(np.uint32))
    assert np.array_equal(got[:, 0], x[:, 0])
    assert np.array_equal(got[:, 1:] - got[:, :-1], x[:, 1:])  # uint32 differences wrap like the sums
    rt.scan_inclusive_cols(xb, ob, 1, rows, cols, np.uint32)
    got = ob.numpy(np.uint32, (rows, cols))
    assert np.array_equal(got[-1], (x.sum(axis=0, dtype=np.uint64) & 0xFFFFFFFF).astype(np.uint32))
    assert np.array_equal(got[1:] - got[:-1], x[1:])
    for r in (0, 5000, rows - 1):
        assert np.array_equal(got[:, r], oracle.scan_inclusive(np.ascontiguousarray(x[:, r])))


def test_scan_empty_is_a_noop(rt):
    b = rt.DeviceBuffer(4)
    rt.scan_inclusive(b, b, 0)


# ---- sort ------------------------------------------------------------------------------------------
def _sort(rt, keys, with_vals=True):
    n = keys.size
    kb = rt.DeviceBuffer.from_numpy(keys.view(np.uint32))
    ko = rt.DeviceBuffer(n)
    if with_vals:
        vb = rt.DeviceBuffer.from_numpy(np.arange(n, dtype=np.uint32))
        vo = rt.DeviceBuffer(n)
        rt.radix_sort_kv(kb, vb, ko, vo, n, keys.dtype)
        out = ko.numpy(keys.dtype), vo.numpy(np.uint32)
    else:
        rt.radix_sort_kv(kb, None, ko, None, n, keys.dtype)
        out = ko.numpy(keys.dtype), None
    assert np.array_equal(kb.numpy(keys.dtype).view(np.uint32), keys.view(np.uint32)), "input must not be modified"
    return out


@pytest.mark.parametrize("n", [1, 2, 63, 64, 65, 8191, 8192, 8193, 100_003, 1 << 20])
@pytest.mark.parametrize("dist", ["uniform", "low_entropy"])
def test_sort_kv_matches_oracle(rt, n, dist):
    rng = np.random.default_rng(1234 + 3)
    hi = 2**32 if dist == "uniform" else 1024
    keys = rng.integers(0, hi, n, dtype=np.uint64).astype(np.uint32)
    k, v = _sort(rt, keys)
    ok, ov = oracle.radix_sort_kv(keys, np.arange(n, dtype=np.uint32))
    assert np.array_equal(k, ok)
    assert np.array_equal(v, ov)  # stability: equal keys keep their original order
    order = np.argsort(keys, kind="stable")
    assert np.array_equal(v, order.astype(np.uint32))


def test_sort_degenerate_inputs(rt):
    for keys in (np.zeros(50_000, np.uint32), np.full(50_000, 0xFFFFFFFF, np.uint32),
                 np.arange(50_000, dtype=np.uint32), np.arange(50_000, dtype=np.uint32)[::-1].copy()):
        k, v = _sort(rt, keys)
        order = np.argsort(keys, kind="stable")
        assert np.array_equal(k, keys[order]) and np.array_equal(v, order.astype(np.uint32))


def test_sort_keys_only_and_caller_tmp(rt):
    rng = np.random.default_rng(44)
    keys = rng.integers(0, 2**32, 300_000, dtype=np.uint64).astype(np.uint32)
    k, _ = _sort(rt, keys, with_vals=False)
    assert np.array_equal(k, np.sort(keys))
    n = keys.size
    kb, vb = rt.DeviceBuffer.from_numpy(keys), rt.DeviceBuffer.from_numpy(np.arange(n, dtype=np.uint32))
    ko, vo, kt, vt = (rt.DeviceBuffer(n) for _ in range(4))
    rt.radix_sort_kv(kb, vb, ko, vo, n, np.uint32, keys_tmp=kt, vals_tmp=vt)
    assert np.array_equal(ko.numpy(np.uint32), np.sort(keys))
    assert np.array_equal(vo.numpy(np.uint32), np.argsort(keys, kind="stable").astype(np.uint32))


def test_sort_int_and_float_keys(rt):
    rng = np.random.default_rng(45)
    ki = rng.integers(-2**31, 2**31, 200_000, dtype=np.int64).astype(np.int32)
    k, v = _sort(rt, ki)
    ok, ov = oracle.radix_sort_kv(ki, np.arange(ki.size, dtype=np.uint32))
    assert np.array_equal(k, ok) and np.array_equal(v, ov)
    kf = rng.normal(size=200_000).astype(np.float32)
    kf[:8] = [0.0, -0.0, np.inf, -np.inf, 1e-45, -1e-45, 3.4e38, -3.4e38]
    k, v = _sort(rt, kf)
    ok, ov = oracle.radix_sort_kv(kf, np.arange(kf.size, dtype=np.uint32))
    assert np.array_equal(k.view(np.uint32), ok.view(np.uint32)) and np.array_equal(v, ov)


def test_sort_argument_errors(rt):
    b = rt.DeviceBuffer(16)
    c = rt.DeviceBuffer(16)
    with pytest.raises(rt.TFHipError):
        rt.radix_sort_kv(b, None, b, None, 16)  # in place is refused
    with pytest.raises(rt.TFHipError):
        rt.radix_sort_kv(b, b, c, None, 16)  # payload in without payload out
    rt.radix_sort_kv(b, None, c, None, 0)  # empty: no-op


@pytest.mark.parametrize("dist", ["uniform", "low_entropy"])
def test_sort_2_pow_24(rt, dist):
    """benchmark config 3 middle size; checked against NumPy's stable argsort (the oracle agrees with it on
    the smaller sizes above)."""
    n = 1 << 24
    rng = np.random.default_rng(1234 + 3)
    keys = rng.integers(0, 2**32 if dist == "uniform" else 1024, n, dtype=np.uint64).astype(np.uint32)
    k, v = _sort(rt, keys)
    order = np.argsort(keys, kind="stable")
    assert np.array_equal(k, keys[order])
    assert np.array_equal(v, order.astype(np.uint32))


@pytest.mark.parametrize("dist", ["uniform", "low_entropy"])
def test_sort_2_pow_28_properties(rt, dist):
    """benchmark config 3 full size (2^28 keys + payload), checked through size-independent properties:
    keys non-decreasing, payload a permutation that maps input keys to output keys, and ties in payload
    order (stability)."""
    n = 1 << 28
    rng = np.random.default_rng(1234 + 3)
    keys = rng.integers(0, 2**32 if dist == "uniform" else 1024, n, dtype=np.uint32)
    k, v = _sort(rt, keys)
    d = np.diff(k.astype(np.int64))
    assert np.all(d >= 0), "keys not sorted"
    assert np.array_equal(keys[v], k), "payload does not carry keys to their sorted places"
    ties = d == 0
    assert np.all(v[1:][ties] > v[:-1][ties]), "equal keys are not in original order"
    seen = np.zeros(n, np.bool_)
    seen[v] = True
    assert seen.all(), "payload is not a permutation"


def test_sort_rejects_overlapping_buffers(rt):
    """Every pass scatters into one buffer while other tiles still read another, so no two of the six n-word buffers
    may overlap (the two inputs, which are only read, may be one array). Argument checks only: nothing is launched."""
    from tensorfrost_amd._lib import TFHipError

    n = 1000
    a, b, c, d, e, f = (rt.DeviceBuffer(n) for _ in range(6))
    cases = [
        dict(keys=a, vals=b, keys_out=c, vals_out=d, keys_tmp=a, vals_tmp=f),   # keys_tmp is keys_in
        dict(keys=a, vals=b, keys_out=c, vals_out=d, keys_tmp=c, vals_tmp=f),   # keys_tmp is keys_out
        dict(keys=a, vals=b, keys_out=c, vals_out=d, keys_tmp=e, vals_tmp=b),   # vals_tmp is vals_in
        dict(keys=a, vals=b, keys_out=c, vals_out=d, keys_tmp=e, vals_tmp=d),   # vals_tmp is vals_out
        dict(keys=a, vals=b, keys_out=c, vals_out=c, keys_tmp=e, vals_tmp=f),   # keys_out is vals_out
        dict(keys=a, vals=b, keys_out=c, vals_out=a, keys_tmp=e, vals_tmp=f),   # vals_out is keys_in
    ]
    for kw in cases:
        with pytest.raises(TFHipError, match="overlap|must differ"):
            rt.radix_sort_kv(kw["keys"], kw["vals"], kw["keys_out"], kw["vals_out"], n, keys_tmp=kw["keys_tmp"], vals_tmp=kw["vals_tmp"])
    # a partial overlap: two windows of one allocation
    import ctypes as C

    from tensorfrost_amd._lib import call

    big = rt.DeviceBuffer(3 * n)
    with pytest.raises(TFHipError, match="overlap"):
        call("tfhip_radix_sort_kv", 0, C.c_void_p(big.ptr), None, C.c_void_p(big.ptr + 4 * (n // 2)), None, None, None, n)
    # keys sorted with themselves as payload: the inputs may be one array
    keys = np.random.default_rng(3).integers(0, 1 << 32, n, dtype=np.uint32)
    kb = rt.DeviceBuffer.from_numpy(keys)
    rt.radix_sort_kv(kb, kb, c, d, n)
    assert np.array_equal(c.numpy(np.uint32), np.sort(keys)) and np.array_equal(d.numpy(np.uint32), np.sort(keys))
