"""Parity of the HIP reductions and fused softmax (through the C ABI) with the CPU oracle.

Tolerances (benchmark targets): reductions 1e-4 relative; max/min select an input value, so they are
compared exactly. Sums of signed values can cancel, so their error is also bounded relative to the sum
of magnitudes (1e-6), the measure that does not blow up on a near-zero result.
"""
import numpy as np
import pytest

from conftest import rel_err, sum_err
from oracle import oracle

pytestmark = pytest.mark.gpu

# Edge cases: single element, short rows (thread-per-row path), unaligned (cols % 4 != 0), one wave,
# split in the oracle (>=1024), few long rows (segmented path), ragged everything.
SHAPES = [(1, 1), (1, 33), (5, 3), (1000, 32), (37, 100), (64, 256), (33, 4096), (9, 1027), (3, 70000), (2, 1 << 20), (513, 1280),
          # many medium rows (lane-group path): 8, 16 and 32 lanes per row, ragged row count, the split-stage shape
          (5000, 36), (4097, 128), (2048, 260), (1025, 512), (65536, 128),
          # many short rows: 1, 2 and 4 lanes per row when aligned, a thread per row otherwise (transposed: narrow matrices)
          (70001, 4), (40000, 8), (100003, 16), (30000, 20), (50000, 3), (20011, 10), (16384, 63)]


def _run(rt, fn, op, x, out_words):
    xb = rt.DeviceBuffer.from_numpy(x)
    ob = rt.DeviceBuffer(out_words)
    fn(op, xb, ob, x.shape[0], x.shape[1])
    return ob.numpy(np.float32)


@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("op", ["sum", "max", "min"])
def test_reduce_rows_matches_oracle(rt, shape, op):
    rng = np.random.default_rng(21)
    x = rng.uniform(-4, 4, shape).astype(np.float32)
    got = _run(rt, rt.reduce_rows, op, x, shape[0])
    ref = getattr(np, op)(x.astype(np.float64), axis=1)
    if op == "sum":
        orc = oracle.reduce_rows(op, x)
        assert sum_err(got, orc, np.abs(x).sum(axis=1)) < 1e-6
        assert sum_err(got, ref, np.abs(x).sum(axis=1)) < 1e-6
        assert rel_err(got, orc) < 1e-4 or sum_err(got, orc, np.abs(x).sum(axis=1)) < 5e-7  # rows that cancel to nearly zero
    else:
        assert np.array_equal(got, ref.astype(np.float32))
        if not (shape[1] >= 1024 and shape[1] % 128):  # the reference zero-pads a ragged split chunk
            assert np.array_equal(got, oracle.reduce_rows(op, x))


@pytest.mark.parametrize("shape", [(s[1], s[0]) for s in SHAPES] + [(4096, 4096), (100, 1000)])
@pytest.mark.parametrize("op", ["sum", "max", "min"])
def test_reduce_cols_matches_oracle(rt, shape, op):
    rng = np.random.default_rng(22)
    x = rng.uniform(-4, 4, shape).astype(np.float32)
    got = _run(rt, rt.reduce_cols, op, x, shape[1])
    ref = getattr(np, op)(x.astype(np.float64), axis=0)
    if op == "sum":
        orc = oracle.reduce_cols(op, x)
        assert sum_err(got, orc, np.abs(x).sum(axis=0)) < 1e-6
        assert sum_err(got, ref, np.abs(x).sum(axis=0)) < 1e-6
    else:
        assert np.array_equal(got, ref.astype(np.float32))
        if not (shape[0] >= 1024 and shape[0] % 128):
            assert np.array_equal(got, oracle.reduce_cols(op, x))


@pytest.mark.parametrize("shape", [(16384, 4096), (16390, 4096), (70001, 1024), (40003, 2048), (4100, 16384), (8200, 8192), (2050, 32768), (1030, 65536),
                                   (4096, 16384), (16384, 1024), (5461, 12288),
                                   # narrow matrices: whole rows side by side in one group's loads, up to 256 columns
                                   (300001, 132), (70001, 64), (16385, 256), (20000, 200), (100003, 16), (50000, 3), (16384, 255)])
def test_large_matrices_with_one_group_per_compute_unit(rt, shape):
    """Matrices of tens to hundreds of MiB whose rows are whole 4 KiB pieces: the column reductions' first pass and, from
    256 MiB on, the row reductions run one group per compute unit, each walking through its own stretch of rows. Row
    counts that do not divide among the groups, slabs of exactly 64 rows, 1 to 16 column tiles. Integers in -8..8, so
    sums are exact in any order: bit-exact against numpy and the oracle."""
    R, C = shape
    x = np.random.default_rng(R + C).integers(-8, 9, shape).astype(np.float32)
    xb, orow, ocol = rt.DeviceBuffer.from_numpy(x), rt.DeviceBuffer(R), rt.DeviceBuffer(C)
    for op in ("sum", "max", "min"):
        rt.reduce_rows(op, xb, orow, R, C)
        rt.reduce_cols(op, xb, ocol, R, C)
        assert np.array_equal(orow.numpy(np.float32), getattr(np, op)(x, axis=1, dtype=np.float64).astype(np.float32) if op == "sum" else getattr(np, op)(x, axis=1)), (op, shape)
        assert np.array_equal(ocol.numpy(np.float32), getattr(np, op)(x, axis=0, dtype=np.float64).astype(np.float32) if op == "sum" else getattr(np, op)(x, axis=0)), (op, shape)
        assert np.array_equal(orow.numpy(np.float32), oracle.reduce_rows(op, x)) and np.array_equal(ocol.numpy(np.float32), oracle.reduce_cols(op, x)), (op, shape)
    for b in (xb, orow, ocol):
        b.free()


@pytest.mark.parametrize("op", ["sum", "max", "min"])
def test_reduce_cols_in_one_launch_over_several_slabs(rt, op):
    """Wide matrices (8192 columns and more, a multiple of 256, at least 512 rows) that the one-group-per-unit form does
    not take are reduced by one launch: groups of sixteen waves per 256 columns and slab of rows, per-slab results through
    device memory, the last group of each 256 columns adds them up and clears its ticket. Shapes with one slab and with
    several, ragged last slabs, beside shapes that take the other forms; the same shapes again in other orders, so that
    every call finds the tickets of the call before it at zero and partial results of an earlier call in the scratch
    buffer."""
    rng = np.random.default_rng(24)
    shapes = [(4096, 16384), (16384, 4096), (513, 8192), (1000, 256), (2048, 32768), (600, 8448), (5000, 1024), (1024, 65536), (4097, 8192), (700, 12288), (600, 131072), (3000, 8448)]
    for shape in shapes + shapes[::-1] + shapes[::2]:
        x = rng.uniform(-4, 4, shape).astype(np.float32)
        got = _run(rt, rt.reduce_cols, op, x, shape[1])
        ref = getattr(np, op)(x.astype(np.float64), axis=0)
        if op == "sum":
            assert sum_err(got, ref, np.abs(x).sum(axis=0)) < 1e-6, shape
        else:
            assert np.array_equal(got, ref.astype(np.float32)), shape


@pytest.mark.parametrize("shape", [(1, 1), (7, 5), (64, 256), (33, 1000), (100, 4096), (5, 4100), (3, 10001), (2, 65536),
                                   # a group per row with the row in registers (256, 512 and 1024 threads), ragged vector counts
                                   (300, 4100), (256, 8192), (260, 12004), (257, 32768), (256, 20000),
                                   # segments of 8192 with two reads: few long rows, unaligned rows, a ragged last segment
                                   (8, 40000), (4, 1 << 20), (3, 100003), (300, 40004), (1, 8193),
                                   # short rows: lane groups of 1 .. 32 (aligned), a thread per row (ten class scores)
                                   (1000, 4), (777, 8), (5000, 16), (4099, 20), (3000, 64), (2049, 100), (1025, 128), (60000, 10), (100, 31), (20000, 256), (16385, 200), (70001, 132)])
def test_softmax_rows_matches_oracle(rt, shape):
    rng = np.random.default_rng(23)
    x = rng.uniform(-4, 4, shape).astype(np.float32)
    xb = rt.DeviceBuffer.from_numpy(x)
    yb = rt.DeviceBuffer(x.size)
    rt.softmax_rows(xb, yb, *shape)
    got = yb.numpy(np.float32, shape)
    assert rel_err(got, oracle.softmax_rows(x)) < 1e-5
    assert np.allclose(got.sum(axis=1, dtype=np.float64), 1.0, atol=1e-5)
    # in place
    rt.softmax_rows(xb, xb, *shape)
    assert np.array_equal(xb.numpy(np.float32, shape), got)


@pytest.mark.parametrize("shape", [(1000, 10), (4096, 64), (70, 4), (512, 1000), (5, 4096), (300, 5000), (300, 20000), (64, 5120), (3, 100000), (77, 333), (2, 2049), (20000, 256), (16385, 200)])
def test_softmax_with_row_statistics(rt, shape):
    """tfhip_softmax_rows_stats_f32: the same y as tfhip_softmax_rows_f32 bit for bit, plus the rows' maxima (exact) and
    the sums of exp(x - max) (1e-5 relative), from every kernel the row length can select."""
    rows, cols = shape
    x = np.random.default_rng(rows * 7 + cols).normal(0, 3, shape).astype(np.float32)
    xb = rt.DeviceBuffer.from_numpy(x)
    y0, y1 = rt.DeviceBuffer(x.size), rt.DeviceBuffer(x.size)
    m, z = rt.DeviceBuffer(rows), rt.DeviceBuffer(rows)
    rt.softmax_rows(xb, y0, rows, cols)
    rt.softmax_rows(xb, y1, rows, cols, m, z)
    assert np.array_equal(y0.numpy(np.float32), y1.numpy(np.float32))
    assert np.array_equal(m.numpy(np.float32), x.max(axis=1))
    want = np.exp(x.astype(np.float64) - x.max(axis=1, keepdims=True)).sum(axis=1)
    assert np.max(np.abs(z.numpy(np.float32) - want) / want) < 1e-5
    # statistics only (no y): the same maxima and sums, nothing written anywhere else
    m2, z2 = rt.DeviceBuffer(rows), rt.DeviceBuffer(rows)
    rt.call("tfhip_softmax_rows_stats_f32", xb.ptr, None, m2.ptr, z2.ptr, rows, cols)
    assert np.array_equal(m2.numpy(np.float32), m.numpy(np.float32)) and np.array_equal(z2.numpy(np.float32), z.numpy(np.float32))
    with pytest.raises(rt.TFHipError, match="null pointer"):
        rt.call("tfhip_softmax_rows_stats_f32", xb.ptr, y1.ptr, None, z.ptr, rows, cols)


@pytest.mark.parametrize("shape", [(1, 1), (7, 5), (64, 256), (33, 1000), (100, 4096), (2048, 4096), (5, 4100), (3, 10001), (300, 4100), (256, 8192), (260, 12004),
                                   (257, 32768), (8, 40000), (3, 100003), (1, 8193), (1000, 4), (777, 8), (5000, 16), (4099, 20), (3000, 64), (1025, 128), (60000, 10), (100, 31), (20000, 256), (16390, 136)])
def test_log_softmax_rows(rt, shape):
    """tfhip_log_softmax_rows_f32 through every kernel a row length selects: (x - max) - log(sum(exp(x - max))) against
    float64 (1e-5 of the largest magnitude, element-wise), the rows' maxima and sums as the softmax leaves them, in place."""
    rows, cols = shape
    x = np.random.default_rng(rows * 3 + cols).normal(0, 3, shape).astype(np.float32)
    x64 = x.astype(np.float64)
    shifted = x64 - x64.max(axis=1, keepdims=True)
    want = shifted - np.log(np.exp(shifted).sum(axis=1, keepdims=True))
    xb = rt.DeviceBuffer.from_numpy(x)
    yb, m, z = rt.DeviceBuffer(x.size), rt.DeviceBuffer(rows), rt.DeviceBuffer(rows)
    rt.log_softmax_rows(xb, yb, rows, cols)
    got = yb.numpy(np.float32, shape)
    assert np.max(np.abs(got - want)) < 1e-5 * max(1.0, np.abs(want).max())
    assert np.allclose(np.exp(got.astype(np.float64)).sum(axis=1), 1.0, atol=1e-4)
    y2 = rt.DeviceBuffer(x.size)
    rt.log_softmax_rows(xb, y2, rows, cols, m, z)
    assert np.array_equal(y2.numpy(np.float32), yb.numpy(np.float32))
    assert np.array_equal(m.numpy(np.float32), x.max(axis=1))
    zs = np.exp(shifted).sum(axis=1)
    assert np.max(np.abs(z.numpy(np.float32) - zs) / zs) < 1e-5
    rt.log_softmax_rows(xb, xb, rows, cols)  # in place
    assert np.array_equal(xb.numpy(np.float32, shape), got)
    with pytest.raises(rt.TFHipError, match="null pointer"):
        rt.call("tfhip_log_softmax_rows_stats_f32", xb.ptr, None, m.ptr, z.ptr, rows, cols)


def test_log_softmax_extreme_rows(rt):
    """Where the softmax underflows the log form does not: x itself is kept, not exp(x - max)."""
    x = np.zeros((4, 512), np.float32)
    x[0] = 80.0
    x[1, 7] = 100.0
    x[2] = np.linspace(-100, 100, 512)
    x[3] = -1e4
    xb = rt.DeviceBuffer.from_numpy(x)
    yb = rt.DeviceBuffer(x.size)
    rt.log_softmax_rows(xb, yb, 4, 512)
    got = yb.numpy(np.float32, (4, 512))
    x64 = x.astype(np.float64)
    shifted = x64 - x64.max(axis=1, keepdims=True)
    want = shifted - np.log(np.exp(shifted).sum(axis=1, keepdims=True))
    assert np.all(np.isfinite(got))
    assert np.max(np.abs(got - want)) < 1e-5 * np.abs(want).max()
    assert got[2, 0] < -199.0  # exp(-200) is zero in fp32; its logarithm is not taken


def test_softmax_extreme_rows(rt):
    """Large spread and constant rows: shifting by the row max keeps exp in range."""
    x = np.zeros((4, 512), np.float32)
    x[0] = 80.0
    x[1, 7] = 100.0
    x[2] = np.linspace(-100, 100, 512)
    x[3] = -1e4
    xb = rt.DeviceBuffer.from_numpy(x)
    yb = rt.DeviceBuffer(x.size)
    rt.softmax_rows(xb, yb, 4, 512)
    got = yb.numpy(np.float32, (4, 512))
    assert np.all(np.isfinite(got))
    assert rel_err(got[:3], oracle.softmax_rows(x)[:3]) < 1e-5
    assert np.allclose(got[3], 1 / 512)


def test_config2_full_size_properties(rt):
    """benchmark config 2 at its real shape [16384, 4096]: size-independent properties plus the oracle on
    a row subset."""
    R, C = 16384, 4096
    rng = np.random.default_rng(1236)
    x = rng.uniform(-4, 4, (R, C)).astype(np.float32)
    xb = rt.DeviceBuffer.from_numpy(x)
    row = rt.DeviceBuffer(R)
    col = rt.DeviceBuffer(C)
    rt.reduce_rows("sum", xb, row, R, C)
    rs = row.numpy(np.float32)
    rt.reduce_cols("sum", xb, col, R, C)
    cs = col.numpy(np.float32)
    # the sum of row sums equals the sum of column sums (a checksum of checksums)
    total = x.sum(dtype=np.float64)
    assert abs(rs.sum(dtype=np.float64) - total) < 1e-6 * np.abs(x).sum(dtype=np.float64)
    assert abs(cs.sum(dtype=np.float64) - total) < 1e-6 * np.abs(x).sum(dtype=np.float64)
    assert sum_err(rs, x.sum(axis=1, dtype=np.float64), np.abs(x).sum(axis=1)) < 1e-6
    assert sum_err(cs, x.sum(axis=0, dtype=np.float64), np.abs(x).sum(axis=0)) < 1e-6
    rt.reduce_rows("max", xb, row, R, C)
    assert np.array_equal(row.numpy(np.float32), x.max(axis=1))
    rt.reduce_cols("max", xb, col, R, C)
    assert np.array_equal(col.numpy(np.float32), x.max(axis=0))
    yb = rt.DeviceBuffer(R * C)
    rt.softmax_rows(xb, yb, R, C)
    y = yb.numpy(np.float32, (R, C))
    assert np.allclose(y.sum(axis=1, dtype=np.float64), 1.0, atol=1e-5)
    assert np.array_equal(y.argmax(axis=1), x.argmax(axis=1))
    sub = slice(0, R, 512)
    assert rel_err(y[sub], oracle.softmax_rows(x[sub])) < 1e-5


def test_softmax_long_and_short_rows_at_full_size(rt):
    """256 MiB matrices in the other shapes: few long rows (segments, two reads), rows held by one group, short rows
    handled by lane groups. Rows sum to one, the largest element stays the largest, a row subset against the oracle."""
    for shape in [(64, 1 << 20), (2048, 32768), (1 << 22, 16)]:
        rows, cols = shape
        x = np.random.default_rng(rows % 1000 + cols % 1000).uniform(-4, 4, shape).astype(np.float32)
        xb = rt.DeviceBuffer.from_numpy(x)
        yb = rt.DeviceBuffer(x.size)
        rt.softmax_rows(xb, yb, rows, cols)
        y = yb.numpy(np.float32, shape)
        assert np.allclose(y.sum(axis=1, dtype=np.float64), 1.0, atol=1e-5)
        assert np.array_equal(y.argmax(axis=1), x.argmax(axis=1))
        sub = slice(0, rows, max(1, rows // 16))
        assert rel_err(y[sub], oracle.softmax_rows(x[sub])) < 1e-5
        xb.free()
        yb.free()


def test_argument_errors(rt):
    xb = rt.DeviceBuffer(16)
    with pytest.raises(rt.TFHipError):
        rt.reduce_rows("sum", xb, xb, 0, 4)
    with pytest.raises(rt.TFHipError):
        rt.softmax_rows(xb, xb, 4, 0)
    with pytest.raises(ValueError):
        rt.DeviceBuffer(0)


@pytest.mark.parametrize("op", ["sum", "max", "min"])
@pytest.mark.parametrize("rows,cols,per", [(1024, 512, 128), (1000, 300, 128), (16384, 4096, 128), (5, 7, 2), (129, 1024, 128)])
def test_reduce_cols_slabs(rt, op, rows, cols, per):
    """out[s, c] = op over the s-th slab of rows: every slab against the oracle's column reduction of that slab."""
    rng = np.random.default_rng(rows + cols)
    x = rng.uniform(-4, 4, (rows, cols)).astype(np.float32)
    slabs = (rows + per - 1) // per
    xb = rt.DeviceBuffer.from_numpy(x)
    ob = rt.DeviceBuffer(slabs * cols)
    rt.reduce_cols_slabs(op, xb, ob, rows, cols, per)
    got = ob.numpy(np.float32, (slabs, cols))
    for s in ([0, slabs - 1] if slabs > 4 else range(slabs)):
        block = x[s * per:(s + 1) * per]
        want = oracle.reduce_cols(op, block)
        if op == "sum":
            assert sum_err(got[s], want, np.abs(block).astype(np.float64).sum(0)) < 1e-4
        else:
            assert np.array_equal(got[s], want)
