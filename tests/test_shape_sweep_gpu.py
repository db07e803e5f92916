"""Seeded random shapes around the boundaries the kernels switch on (tile, wave, slab and chunk sizes, +-1), for
the primitives through the C ABI and for the emitted reduction loops through the program driver. Operands are small
integers wherever that makes every fp32 intermediate exact: the expected result is then the same in any summation
order, it comes from numpy in float64 / uint64, and the comparison is bit-exact, so a wrong index, a dropped tail
or a tile written twice shows as a wrong number instead of hiding inside a tolerance. On integer operands the CPU oracle
gives the same bits too, and is compared as well (the products up to 2^27 multiply-adds). One case per seed; the
assertion message names the shape."""
import numpy as np
import pytest

from oracle import oracle

pytestmark = pytest.mark.gpu

EDGE = [1, 2, 3, 4, 5, 7, 8, 15, 16, 17, 31, 32, 33, 63, 64, 65, 96, 127, 128, 129, 130, 255, 256, 257, 383, 384, 385, 511, 512, 513,
        1023, 1024, 1025, 2047, 2048, 2049, 4095, 4096, 4097, 8191, 8192, 8193, 16384, 32768, 65536, 65537, 131072, 262144]


def _pick(rng, limit):
    limit = max(1, int(limit))
    if rng.random() < 0.6:
        return int(rng.choice([x for x in EDGE if x <= limit]))
    return int(rng.integers(1, limit + 1))


@pytest.fixture(scope="module")
def tf():
    import tensorfrost_amd.host as tfh

    tfh.initialize(tfh.hip)
    yield tfh
    tfh.synchronize()


@pytest.mark.parametrize("seed", range(40))
def test_sgemm_exact_on_integer_operands(rt, seed):
    """Every layout, the three fused tails and the column sums beside the tn product, operands in -3..3
    (|sum| <= 9 K < 2^24: exact)."""
    rng = np.random.default_rng(1000 + seed)
    layout = str(rng.choice(["nn", "nt", "tn"]))
    m = _pick(rng, 300000)
    n = _pick(rng, min(8192, (1 << 23) // m))
    k = _pick(rng, min((1 << 24) // max(m, n), (1 << 31) // (m * n), 300000))
    tail = [None, "bias", "bias_relu", "mask_positive", "colsum"][int(rng.integers(0, 5))]
    if tail == "colsum":
        layout = "tn"
    case = f"{layout} M={m} N={n} K={k} tail={tail}"
    a = rng.integers(-3, 4, (m, k)).astype(np.float32)
    b = rng.integers(-3, 4, (k, n)).astype(np.float32)
    aa = np.ascontiguousarray(a.T) if layout == "tn" else a
    bb = np.ascontiguousarray(b.T) if layout == "nt" else b
    ab, bbuf, cb = rt.DeviceBuffer.from_numpy(aa), rt.DeviceBuffer.from_numpy(bb), rt.DeviceBuffer(m * n)
    want = a.astype(np.float64) @ b.astype(np.float64)
    if tail == "colsum":
        sums = rt.DeviceBuffer(n)
        rt.call("tfhip_sgemm_tn_colsum", ab.ptr, bbuf.ptr, cb.ptr, sums.ptr, m, n, k)
        assert np.array_equal(sums.numpy(np.float32), b.sum(axis=0, dtype=np.float64).astype(np.float32)), case
        sums.free()
    elif tail is None:
        rt.sgemm(layout, ab, bbuf, cb, m, n, k)
    else:
        if tail == "mask_positive":
            aux = rng.integers(-1, 2, (m, n)).astype(np.float32)
            want = np.where(aux > 0, want, 0)
        else:
            aux = rng.integers(-5, 6, n).astype(np.float32)
            want = want + aux
            if tail == "bias_relu":
                want = np.maximum(want, 0)
        xb = rt.DeviceBuffer.from_numpy(aux)
        rt.sgemm(layout, ab, bbuf, cb, m, n, k, epilogue=tail, aux=xb)
        xb.free()
    got = cb.numpy(np.float32, (m, n))
    assert np.array_equal(got, want.astype(np.float32)), case
    if tail in (None, "colsum") and m * n * k <= 1 << 27:
        assert np.array_equal(got, oracle.matmul(aa, bb, layout)), case
    for z in (ab, bbuf, cb):
        z.free()


@pytest.mark.parametrize("seed", range(25))
def test_reductions_and_softmax_over_random_shapes(rt, seed):
    """sum / max / min along both axes exact on integers in -100..100; the fused softmax and log-softmax against float64
    (1e-6 absolute on probabilities, 1e-5 on log-probabilities), the row maxima exact."""
    rng = np.random.default_rng(2000 + seed)
    R = _pick(rng, 200000)
    C = _pick(rng, min(200000, (1 << 24) // R))
    case = f"R={R} C={C}"
    x = rng.integers(-100, 101, (R, C)).astype(np.float32)
    xb, orow, ocol = rt.DeviceBuffer.from_numpy(x), rt.DeviceBuffer(R), rt.DeviceBuffer(C)
    x64 = x.astype(np.float64)
    for op, f in (("sum", np.sum), ("max", np.max), ("min", np.min)):
        rt.reduce_rows(op, xb, orow, R, C)
        rt.reduce_cols(op, xb, ocol, R, C)
        assert np.array_equal(orow.numpy(np.float32), f(x64, axis=1).astype(np.float32)), f"rows {op} {case}"
        assert np.array_equal(ocol.numpy(np.float32), f(x64, axis=0).astype(np.float32)), f"cols {op} {case}"
        assert np.array_equal(orow.numpy(np.float32), oracle.reduce_rows(op, x)) and np.array_equal(ocol.numpy(np.float32), oracle.reduce_cols(op, x)), f"{op} {case}"
    xs = (x / np.float32(16)).astype(np.float32)
    xb.write(xs)
    yb, mb, sb = rt.DeviceBuffer(R * C), rt.DeviceBuffer(R), rt.DeviceBuffer(R)
    rt.softmax_rows(xb, yb, R, C, mb, sb)
    x64 = xs.astype(np.float64)
    mx = x64.max(axis=1, keepdims=True)
    e = np.exp(x64 - mx)
    z = e.sum(axis=1, keepdims=True)
    assert np.array_equal(mb.numpy(np.float32), mx[:, 0].astype(np.float32)), case
    assert np.max(np.abs(sb.numpy(np.float32) - z[:, 0]) / z[:, 0]) < 2e-5, case
    assert np.max(np.abs(yb.numpy(np.float32, (R, C)) - e / z)) < 1e-6, case
    assert np.max(np.abs(yb.numpy(np.float32, (R, C)) - oracle.softmax_rows(xs))) < 1e-6, case
    rt.log_softmax_rows(xb, yb, R, C)
    assert np.max(np.abs(yb.numpy(np.float32, (R, C)) - ((x64 - mx) - np.log(z)))) < 1e-5, case
    for b in (xb, orow, ocol, yb, mb, sb):
        b.free()


@pytest.mark.parametrize("seed", range(25))
def test_prefix_sums_over_random_shapes(rt, seed):
    """Flat, row-wise and column-wise inclusive sums: u32 in wrap-around arithmetic, f32 on integers in -4..4 (exact)."""
    rng = np.random.default_rng(3000 + seed)
    n = _pick(rng, 1 << 24)
    u = rng.integers(0, 2**32, n, dtype=np.uint64).astype(np.uint32)
    ub, ob = rt.DeviceBuffer.from_numpy(u), rt.DeviceBuffer(n)
    rt.scan_inclusive(ub, ob, n)
    assert np.array_equal(ob.numpy(np.uint32), np.cumsum(u, dtype=np.uint64).astype(np.uint32)), f"u32 n={n}"
    assert np.array_equal(ob.numpy(np.uint32), oracle.scan_inclusive(u)), f"u32 n={n}"
    f = rng.integers(-4, 5, n).astype(np.float32)
    ub.write(f)
    rt.scan_inclusive(ub, ob, n, np.float32)
    assert np.array_equal(ob.numpy(np.float32), np.cumsum(f, dtype=np.float64).astype(np.float32)), f"f32 n={n}"
    assert np.array_equal(ob.numpy(np.float32), oracle.scan_inclusive(f)), f"f32 n={n}"
    ub.free()
    ob.free()
    R = _pick(rng, 100000)
    C = _pick(rng, min(100000, (1 << 22) // R))
    case = f"R={R} C={C}"
    u = rng.integers(0, 2**32, (R, C), dtype=np.uint64).astype(np.uint32)
    ub, ob = rt.DeviceBuffer.from_numpy(u), rt.DeviceBuffer(R * C)
    rt.scan_inclusive_rows(ub, ob, R, C)
    assert np.array_equal(ob.numpy(np.uint32, (R, C)), np.cumsum(u, axis=1, dtype=np.uint64).astype(np.uint32)), "rows u32 " + case
    rt.scan_inclusive_cols(ub, ob, 1, R, C)
    assert np.array_equal(ob.numpy(np.uint32, (R, C)), np.cumsum(u, axis=0, dtype=np.uint64).astype(np.uint32)), "cols u32 " + case
    f = rng.integers(-4, 5, (R, C)).astype(np.float32)
    ub.write(f)
    rt.scan_inclusive_rows(ub, ob, R, C, np.float32)
    assert np.array_equal(ob.numpy(np.float32, (R, C)), np.cumsum(f, axis=1, dtype=np.float64).astype(np.float32)), "rows f32 " + case
    rt.scan_inclusive_cols(ub, ob, 1, R, C, np.float32)
    assert np.array_equal(ob.numpy(np.float32, (R, C)), np.cumsum(f, axis=0, dtype=np.float64).astype(np.float32)), "cols f32 " + case
    ub.free()
    ob.free()


@pytest.mark.parametrize("seed", range(20))
def test_sort_over_random_sizes_key_types_and_entropies(rt, seed):
    """Key + payload sorts of u32 / i32 / f32 keys with 32, 8 or 3 random bits (many equal keys: stability shows in the
    payload), against numpy's stable argsort; float keys in the total order of their bit patterns (-0 before +0)."""
    rng = np.random.default_rng(4000 + seed)
    n = _pick(rng, 1 << 22)
    kind = [np.uint32, np.int32, np.float32][int(rng.integers(0, 3))]
    bits = int(rng.choice([32, 32, 8, 3]))
    raw = rng.integers(0, 2**bits, n, dtype=np.uint64).astype(np.uint32)
    if kind is np.float32:
        keys = raw.view(np.float32).copy()
        keys[np.isnan(keys)] = 0.5
    else:
        keys = raw.view(kind)
    vals = rng.integers(0, 2**32, n, dtype=np.uint64).astype(np.uint32)
    kb, vb, ko, vo = rt.DeviceBuffer.from_numpy(keys), rt.DeviceBuffer.from_numpy(vals), rt.DeviceBuffer(n), rt.DeviceBuffer(n)
    rt.radix_sort_kv(kb, vb, ko, vo, n, key_dtype=kind)
    if kind is np.float32:
        u = keys.view(np.uint32)
        order = np.argsort(np.where(u >> 31, ~u, u | np.uint32(0x80000000)).astype(np.uint32), kind="stable")
    else:
        order = np.argsort(keys, kind="stable")
    case = f"n={n} {kind.__name__} bits={bits}"
    assert np.array_equal(ko.numpy(np.uint32), keys[order].view(np.uint32)), case
    assert np.array_equal(vo.numpy(np.uint32), vals[order]), case
    o_keys, o_vals = oracle.radix_sort_kv(keys, vals)
    assert np.array_equal(ko.numpy(np.uint32), o_keys.view(np.uint32)) and np.array_equal(vo.numpy(np.uint32), o_vals), case
    for b in (kb, vb, ko, vo):
        b.free()


@pytest.mark.parametrize("seed", range(25))
def test_emitted_reduction_loops_over_random_shapes(tf, seed):
    """The programs whose loops no primitive serves (five fused loops down the columns; integer sums, maxima and minima
    along the rows), whatever mapping the dispatch picks for the shape: loops shared by a wave, sliced among the waves of
    a group, shared by several groups, or thread-serial. Integer results exact, float sums to 1e-5 of the sum of
    magnitudes."""
    rng = np.random.default_rng(5000 + seed)
    R = _pick(rng, 200000)
    C = _pick(rng, max(1, min(70000, (1 << 24) // R)))
    case = f"R={R} C={C}"
    x = rng.uniform(-3, 5, (R, C)).astype(np.float32)
    u = rng.integers(0, 2**32, (R, C), dtype=np.uint64).astype(np.uint32)
    i = rng.integers(-2**31, 2**31, (R, C), dtype=np.int64).astype(np.int32)
    prog = tf.compile("column_statistics")
    outs = prog(x, u)
    s, mx, mn, norm, su = (o.numpy for o in outs)
    x64 = x.astype(np.float64)
    assert np.max(np.abs(s - x64.sum(axis=0)) / np.abs(x64).sum(axis=0)) < 1e-5, case
    assert np.array_equal(mx, x.max(axis=0)) and np.array_equal(mn, x.min(axis=0)), case
    assert np.max(np.abs(norm - np.sqrt((x64 * x64).sum(axis=0))) / np.sqrt((x64 * x64).sum(axis=0))) < 1e-5, case
    assert np.array_equal(su, (u.astype(np.uint64).sum(axis=0) & 0xFFFFFFFF).astype(np.uint32)), case
    for o in outs:
        o.release()
    prog.destroy()
    prog = tf.compile("integer_reductions")
    outs = prog(u, i)
    sum_u, max_u, sum_i, min_i = (o.numpy for o in outs)
    assert np.array_equal(sum_u, (u.astype(np.uint64).sum(axis=1) & 0xFFFFFFFF).astype(np.uint32)), case
    assert np.array_equal(max_u, u.max(axis=1)) and np.array_equal(min_i, i.min(axis=1)), case
    assert np.array_equal(sum_i.view(np.uint32), (i.astype(np.int64).sum(axis=1) & 0xFFFFFFFF).astype(np.uint32)), case
    for o in outs:
        o.release()
    prog.destroy()
