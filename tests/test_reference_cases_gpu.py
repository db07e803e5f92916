"""The cases the reference's own test files hold for this path, with their sizes, value ranges and acceptance
criteria, run through this backend:

    tests/sorting_test.py:33-72          radix sort of 2^20 uint keys below 2^31 - 1 and of 2^20 float keys in [0, 1),
                                         with random payloads; accepted when sum |sorted - keys[argsort(keys)]| == 0
    tests/sorting_test.py:14-18,49-54    tf.sort.bitonic (sort.py:4-35) on the same 2^20 uint keys: two nested host loops,
                                         one dispatch per stage of the network, swaps behind an `if`; same criterion
    tests/reshape_reduction_test.py      A = rand(10, 5, 6, 7) reshaped to [10, 210]: max, min, sum, mean, norm over the
                                         last axis, the max of the maxima and min of the minima, the mean over axis 0;
                                         np.allclose
    tests/autograd_test.py:29-31         log_softmax(X) = (X - max) - log(sum(exp(X - max))) over class scores
    tests/autograd_test.py:233-237       network outputs atol 1e-5, gradients atol 1e-3: here the dense layer's forward
                                         product with bias and the two gradient products, at those tolerances
    tests/autograd_test.py:33-108,210-232 the test network's forward pass and loss (convolutions as sums over gathered
                                         indices, max pooling, GELU, dense layers, grouped products with tanh and a
                                         residual, log_softmax loss) at batch 64 against PyTorch: loss 1e-5, logits
                                         atol 1e-5
    tests/split_dim_test.py:13-24        split_dim(data, 32, 0) and merge_dim(splitted, axis = 1) on int32 (128, 128, 32):
                                         merged equals data exactly, shapes [4, 32, 128, 32] and [128, 128, 32]
    tests/linalg_test.py:87-112          Gram-Schmidt QR in a host loop over the columns, the inverse of the triangular
                                         factor in a second host loop, R_inv @ Q^T, on rand(5, 5): |Q R - Q'R'| < 1e-5,
                                         |R_inv - R_inv'| < 5e-3, |A_inv - A_inv'| < 5e-3 (Frobenius) against NumPy

The reference's tests draw unseeded random data; the seeds here are fixed."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def tf():
    import tensorfrost_amd.host as tfh

    tfh.initialize(tfh.hip)
    yield tfh
    tfh.synchronize()


@pytest.mark.parametrize("program", ["radix_sort", "radix_sort_ir"], ids=["onesweep_primitive", "reference_composition"])
def test_sorting_test_radix_uint_and_float(tf, program):
    n = 2 ** 20
    rng = np.random.default_rng(20)
    keys = rng.integers(0, 2 ** 31 - 1, n).astype(np.uint32)
    values = rng.integers(0, 2 ** 31 - 1, n).astype(np.uint32)
    prog = tf.compile(program, [tf.uint32])
    sorted_keys, sorted_values = (t.numpy for t in prog(keys, values))
    order = np.argsort(keys, kind="stable")
    assert np.sum(np.abs(sorted_keys.astype(np.int64) - keys[order].astype(np.int64))) == 0
    assert np.array_equal(sorted_values, values[order])  # the reference checks the keys only; the sort is stable
    prog.destroy()

    keys = rng.random(n).astype(np.float32)
    values = rng.random(n).astype(np.float32)
    prog = tf.compile(program, [tf.float32])
    sorted_keys, sorted_values = (t.numpy for t in prog(keys, values.view(np.uint32)))
    order = np.argsort(keys, kind="stable")
    assert np.sum(np.abs(sorted_keys.view(np.float32) - keys[order])) == 0
    assert np.array_equal(sorted_values.view(np.float32), values[order])
    prog.destroy()


def test_reshape_reduction_test(rt):
    a = np.random.default_rng(21).random((10, 5, 6, 7)).astype(np.float32)
    ar = a.reshape(10, -1)
    rows, cols = ar.shape
    xb = rt.DeviceBuffer.from_numpy(ar)
    sq = rt.DeviceBuffer.from_numpy(ar * ar)  # tf.norm is sqrt(sum(x * x)): the square is element-wise work
    out = rt.DeviceBuffer(rows)

    def reduced(op, src=xb):
        rt.reduce_rows(op, src, out, rows, cols)
        return out.numpy(np.float32).copy()

    max_val, min_val, total = reduced("max"), reduced("min"), reduced("sum")
    assert np.allclose(max_val, ar.max(axis=1)) and np.allclose(min_val, ar.min(axis=1))
    assert np.allclose(total, ar.sum(axis=1)) and np.allclose(total / cols, ar.mean(axis=1))
    assert np.allclose(np.sqrt(reduced("sum", sq)), np.linalg.norm(ar, axis=1))
    one = rt.DeviceBuffer(1)
    rt.reduce_rows("max", rt.DeviceBuffer.from_numpy(max_val), one, 1, rows)
    assert np.allclose(one.numpy(np.float32)[0], ar.max())
    rt.reduce_rows("min", rt.DeviceBuffer.from_numpy(min_val), one, 1, rows)
    assert np.allclose(one.numpy(np.float32)[0], ar.min())
    col = rt.DeviceBuffer(cols)
    rt.reduce_cols("sum", xb, col, rows, cols)  # mean over axis 0 of A, viewed as [10, 5 * 6 * 7]
    assert np.allclose(col.numpy(np.float32).reshape(5, 6, 7) / rows, a.mean(axis=0))


@pytest.mark.parametrize("shape", [(10, 5, 6, 7), (3, 1, 1, 5), (64, 16, 16, 16), (1000, 3, 7, 11), (5000, 4, 4, 8), (70000, 1, 2, 3)])
def test_reshape_reduction_test_as_lowered_kernels(tf, shape):
    """The same reference test (tests/reshape_reduction_test.py:5-21) as the kernels its passes produce: the five
    reductions over the reshaped view fused into one kernel (mean's division and norm's square and square root on the
    GPU), the totals over the row results, the mean over axis 0. Nothing here is one of the whole-kernel idioms, so
    every loop runs as emitted: the five loops over a row as one loop that a wave shares, the loop down the columns
    sliced among the waves of a group and, for the tall shapes, among several groups. The reference's own criterion
    is np.allclose; here the sums are held to 1e-4 of the sum of magnitudes of their terms and max / min are exact."""
    a = np.random.default_rng(21).random(shape).astype(np.float32) - np.float32(0.25)
    prog = tf.compile("reshape_reduction")
    assert "primitive" not in " ".join(k["mapping"] for k in prog.kernels())
    before = tf.dispatch_stats()["served_by_primitives"]
    outs = prog(a)
    assert tf.dispatch_stats()["served_by_primitives"] == before
    max_val, min_val, total, mean, norm, total_max, total_min, mean_block = (o.numpy for o in outs)
    ar = a.reshape(shape[0], -1).astype(np.float64)
    m = ar.shape[1]
    magnitudes = np.abs(ar).sum(axis=1)
    assert np.array_equal(max_val, a.reshape(shape[0], -1).max(axis=1)) and np.array_equal(min_val, a.reshape(shape[0], -1).min(axis=1))
    assert np.max(np.abs(total - ar.sum(axis=1)) / magnitudes) < 1e-4
    assert np.max(np.abs(mean - ar.mean(axis=1)) / (magnitudes / m)) < 1e-4
    assert np.max(np.abs(norm - np.linalg.norm(ar, axis=1)) / np.linalg.norm(ar, axis=1)) < 1e-4
    assert total_max[0] == a.max() and total_min[0] == a.min()
    assert mean_block.shape == shape[1:]
    assert np.max(np.abs(mean_block - a.astype(np.float64).mean(axis=0)) / (np.abs(a).astype(np.float64).sum(axis=0) / shape[0])) < 1e-4
    # the reference's own acceptance criterion (relative to the result, so among tens of thousands of short rows one whose
    # terms cancel fails it in any fp32 summation order: held only at the reference's scale)
    if shape[0] <= 5000:
        assert np.allclose(total, ar.sum(axis=1)) and np.allclose(mean, ar.mean(axis=1)) and np.allclose(norm, np.linalg.norm(ar, axis=1))
    for o in outs:
        o.release()
    prog.destroy()


@pytest.mark.parametrize("shape", [(1, 1), (7, 130), (300, 4096), (4096, 33)])
def test_integer_reductions_as_lowered_kernels(tf, shape):
    """dim_sum / dim_max / dim_min of uint and int tensors (Compiler/Operations.cpp: dim_sum u_u, i_i) as emitted loops:
    bit-exact, sums in wrap-around arithmetic."""
    rng = np.random.default_rng(23)
    u = rng.integers(0, 2**32, shape, dtype=np.uint32)
    i = rng.integers(-2**31, 2**31, shape, dtype=np.int64).astype(np.int32)
    prog = tf.compile("integer_reductions")
    outs = prog(u, i)
    sum_u, max_u, sum_i, min_i = (o.numpy for o in outs)
    assert np.array_equal(sum_u, (u.astype(np.uint64).sum(axis=1) & 0xFFFFFFFF).astype(np.uint32))
    assert np.array_equal(max_u, u.max(axis=1))
    assert np.array_equal(sum_i.view(np.uint32), (i.astype(np.int64).sum(axis=1) & 0xFFFFFFFF).astype(np.uint32))
    assert np.array_equal(min_i, i.min(axis=1))
    for o in outs:
        o.release()
    prog.destroy()


@pytest.mark.parametrize("shape", [(1, 1), (130, 7), (300, 4096), (5000, 64), (20000, 300), (70000, 16), (1200, 70000)])
def test_fused_reductions_over_axis_0_as_lowered_kernels(tf, shape):
    """sum, max, min, norm of a float tensor and the wrap-around sum of a uint tensor over axis 0, five loops down the
    columns in one kernel (tensors of unknown shape: no 128-chunk split). The emitter fuses the loops into one, slices
    it among the waves of a group and, for tall tensors with few columns, among several groups with five partial
    results per thread; tensors with many columns and short loops take the thread-serial twin. Integer sums and
    max / min are exact whatever the order."""
    R, C = shape
    rng = np.random.default_rng(R * 7 + C)
    x = rng.uniform(-3, 5, shape).astype(np.float32)
    u = rng.integers(0, 2**32, shape, dtype=np.uint64).astype(np.uint32)
    prog = tf.compile("column_statistics")
    kinds = [k["mapping"] for k in prog.kernels()]
    assert kinds == ["reduction:block", "flat:vec4"]
    for _ in range(2):  # the second execution finds the ticket counters of the first at zero again
        outs = prog(x, u)
        s, mx, mn, norm, su = (o.numpy for o in outs)
        x64 = x.astype(np.float64)
        assert np.max(np.abs(s - x64.sum(axis=0)) / np.abs(x64).sum(axis=0)) < 1e-5
        assert np.array_equal(mx, x.max(axis=0)) and np.array_equal(mn, x.min(axis=0))
        assert np.max(np.abs(norm - np.sqrt((x64 * x64).sum(axis=0))) / np.sqrt((x64 * x64).sum(axis=0))) < 1e-5
        assert np.array_equal(su, (u.astype(np.uint64).sum(axis=0) & 0xFFFFFFFF).astype(np.uint32))
        for o in outs:
            o.release()
    prog.destroy()


@pytest.mark.parametrize("batch,classes", [(64, 10), (1000, 10), (256, 1000)])
def test_autograd_test_log_softmax(rt, batch, classes):
    x = np.random.default_rng(22).normal(0, 2, (batch, classes)).astype(np.float32)
    xb = rt.DeviceBuffer.from_numpy(x)
    yb, m, z = rt.DeviceBuffer(x.size), rt.DeviceBuffer(batch), rt.DeviceBuffer(batch)
    rt.softmax_rows(xb, yb, batch, classes, m, z)
    got = (x - m.numpy(np.float32)[:, None]) - np.log(z.numpy(np.float32))[:, None]
    x64 = x.astype(np.float64)
    shifted = x64 - x64.max(axis=1, keepdims=True)
    want = shifted - np.log(np.exp(shifted).sum(axis=1, keepdims=True))
    assert np.allclose(got, want, atol=1e-5)
    assert np.allclose(np.log(yb.numpy(np.float32, x.shape)), want, atol=1e-5)


def test_autograd_test_dense_layer_forward_and_gradients(tf):
    """A dense layer of the reference's test networks (flattened 28 x 28 input, as in TestModule1): output at atol 1e-5
    per unit of its scale, gradient products at atol 1e-3, through the lowered matmul loops."""
    rng = np.random.default_rng(23)
    m, k, n = 64, 784, 128
    x = rng.random((m, k)).astype(np.float32)
    w = (rng.normal(size=(k, n)) / np.sqrt(k)).astype(np.float32)
    bias = rng.normal(size=n).astype(np.float32) * 0.1
    g = rng.normal(size=(m, n)).astype(np.float32)
    prog = tf.compile("dense_layer")
    h, y, dx = (t.numpy for t in prog(x, w, bias, g))
    y64 = x.astype(np.float64) @ w.astype(np.float64) + bias
    assert np.allclose(y, y64, atol=1e-5 * max(1.0, np.abs(y64).max()))
    assert np.allclose(h, np.maximum(y64, 0), atol=1e-5 * max(1.0, np.abs(y64).max()))
    assert np.allclose(dx, np.where(x > 0, g.astype(np.float64) @ w.astype(np.float64).T, 0.0), atol=1e-3)
    prog.destroy()


@pytest.mark.parametrize("shape", [(128, 128, 32), (100, 7, 5), (1, 1, 1), (33, 2, 129)], ids=str)
def test_split_dim_test(tf, shape):
    """tests/split_dim_test.py:13-24 at its own size, and at sizes whose first extent is no multiple of 32: the split pads
    with zeros (ConstantOutOfBounds, Compiler/Implementations.cpp:56-69) and the merge keeps the padding."""
    data = np.random.default_rng(31).integers(0, 100, shape, dtype=np.int32)
    prog = tf.compile("split_merge")
    merged, splitted = prog(data)
    groups = (shape[0] + 31) // 32
    assert list(splitted.shape) == [groups, 32, shape[1], shape[2]]
    assert list(merged.shape) == [groups * 32, shape[1], shape[2]]
    padded = np.zeros((groups * 32,) + shape[1:], np.int32)
    padded[: shape[0]] = data
    assert np.sum(np.abs(padded - merged.numpy)) == 0
    assert np.array_equal(splitted.numpy, padded.reshape(groups, 32, shape[1], shape[2]))
    for t in (merged, splitted):
        t.release()
    prog.destroy()


def _gram_schmidt(a):
    """Column by column: normalise, project the remaining columns on it, subtract (float64)."""
    a = a.astype(np.float64).copy()
    m, n = a.shape
    q, r = np.zeros((m, n)), np.zeros((n, n))
    for i in range(n):
        r[i, i] = np.sqrt(np.sum(a[:, i] ** 2))
        q[:, i] = a[:, i] / r[i, i]
        r[i, i + 1:] = q[:, i] @ a[:, i + 1:]
        a[:, i + 1:] -= q[:, i:i + 1] * r[i:i + 1, i + 1:]
    return q, r


def _upper_triangular_inverse(r):
    """Forward substitution on the transpose, row by row, transposed back."""
    low = r.T
    n = low.shape[0]
    x = np.zeros((n, n))
    for i in range(n):
        x[i, i] = 1.0 / low[i, i]
        x[i, :i] = -(low[i, :i] @ x[:i, :i]) / low[i, i]
    return x.T


@pytest.mark.parametrize("shape", [(5, 5), (8, 8), (16, 16), (12, 7), (1, 1), (40, 40)], ids=str)
def test_linalg_test_qr_inversion(tf, shape):
    """tests/linalg_test.py:87-112 at its own size and tolerances, then at other sizes (a tall matrix gives the
    pseudo-inverse) with the properties the factors must have. Every kernel's extent depends on the host loop's
    variable; the last iterations dispatch kernels with zero threads."""
    m, n = shape
    a = np.random.default_rng(32 + m).random((m, n)).astype(np.float32)
    if m > 8:
        a += np.eye(m, n, dtype=np.float32) * 2  # keep larger random matrices well conditioned
    prog = tf.compile("qr_inversion")
    q, r, r_inv, a_inv = (t.numpy for t in prog(a))
    q64, r64 = _gram_schmidt(a)
    r_inv64 = _upper_triangular_inverse(r64)
    a_inv64 = r_inv64 @ q64.T
    assert np.linalg.norm(q64 @ r64 - q.astype(np.float64) @ r.astype(np.float64)) < 1e-5 * max(1.0, np.linalg.norm(a) / 2.5)
    assert np.linalg.norm(r_inv64 - r_inv) < 5e-3
    assert np.linalg.norm(a_inv64 - a_inv) < 5e-3
    # what the factors are: R upper triangular with a positive diagonal, Q's columns orthonormal, A_inv A = I
    assert np.all(np.tril(r, -1) == 0) and np.all(np.diag(r) > 0)
    assert np.allclose(q.T @ q, np.eye(n), atol=1e-4)
    assert np.allclose(a_inv.astype(np.float64) @ a, np.eye(n), atol=5e-3)
    prog.destroy()


@pytest.mark.parametrize("batch", [64, 5])
def test_autograd_test_network_forward_and_loss(tf, batch):
    """tests/autograd_test.py: TestModule1.forward and .loss (:73-108) against the same network in PyTorch (:110-186),
    with the reference's acceptance bounds for the loss (1e-5, :231) and the network outputs (atol 1e-5, :233). The
    gradients of that test come from the compiler's autodiff, which is upstream of this backend."""
    import torch
    import torch.nn.functional as F

    rng = np.random.default_rng(41)
    f32 = np.float32
    x = rng.random((batch, 784)).astype(f32)
    labels = rng.integers(0, 10, batch)
    y = np.eye(10, dtype=f32)[labels]
    conv1 = (rng.normal(size=(16, 1, 5, 5)) * np.sqrt(0.1 / 25)).astype(f32)
    conv2 = (rng.normal(size=(64, 16, 5, 5)) * np.sqrt(0.1 / (25 * 16))).astype(f32)
    fc1 = (rng.normal(size=(1024, 64)) / np.sqrt(1024)).astype(f32)
    fc1_bias = (rng.normal(size=64) * 0.1).astype(f32)
    sum1 = (rng.normal(size=(16, 8)) * 0.1).astype(f32)
    sum1_bias = (rng.normal(size=8) * 0.1).astype(f32)
    sum2 = (rng.normal(size=(8, 16)) * 0.1).astype(f32)
    sum2_bias = (rng.normal(size=16) * 0.1).astype(f32)
    fc2 = (rng.normal(size=(64, 10)) / np.sqrt(64)).astype(f32)
    fc2_bias = (rng.normal(size=10) * 0.1).astype(f32)
    params = [conv1, conv2, fc1, fc1_bias, sum1, sum1_bias, sum2, sum2_bias, fc2, fc2_bias]

    prog = tf.compile("autograd_network_forward")
    loss_t, logits_t = prog(x, y, *params)
    loss, logits = float(loss_t.numpy[0]), logits_t.numpy

    t = lambda a: torch.from_numpy(a.astype(np.float64))
    gelu = lambda v: 0.5 * v * (1.0 + torch.tanh(np.sqrt(2.0 / np.pi) * (v + 0.044715 * (v * v * v))))
    h = t(x).reshape(batch, 1, 28, 28)
    h = gelu(F.max_pool2d(F.conv2d(h, t(conv1)), 2))
    h = gelu(F.max_pool2d(F.conv2d(h, t(conv2)), 2))
    h = gelu(h.reshape(batch, 1024) @ t(fc1) + t(fc1_bias))
    h = h.reshape(batch, 4, 16)
    r = torch.tanh(h @ t(sum1) + t(sum1_bias)).sum(dim=1).unsqueeze(1)
    h = (h + torch.tanh(r @ t(sum2) + t(sum2_bias))).reshape(batch, 64)
    want_logits = h @ t(fc2) + t(fc2_bias)
    shifted = want_logits - want_logits.max(dim=-1, keepdim=True).values
    log_softmax = shifted - torch.log(torch.exp(shifted).sum(dim=-1, keepdim=True))
    want_loss = float((-t(y) * log_softmax).sum(dim=-1).mean())
    assert np.allclose(logits, want_logits.numpy(), atol=1e-5)
    assert abs(loss - want_loss) < 1e-5
    for o in (loss_t, logits_t):
        o.release()
    prog.destroy()


@pytest.mark.parametrize("n", [1 << 20, 1000, (1 << 16) + 3, 2, 1])
def test_sorting_test_bitonic(tf, n):
    """tests/sorting_test.py:33-54 for tf.sort.bitonic: 2^20 uint keys below 2^31 - 1, accepted when
    sum |sorted - keys[argsort(keys)]| == 0. The network is not stable and the reference never compares the values; here
    the values are the keys' original positions, so every value must still point at its key. Sizes that are no power of
    two exercise the bounds tests of the swap (the network runs over the next power of two)."""
    rng = np.random.default_rng(n)
    keys = rng.integers(0, 2**31 - 1, n).astype(np.uint32)
    values = np.arange(n, dtype=np.uint32)
    prog = tf.compile("bitonic_sort")
    before = tf.dispatch_stats()["dispatches"]
    sorted_keys, sorted_values = prog(keys, values)
    stages = int(np.ceil(np.log2(np.float32(n)))) if n > 1 else 0
    assert tf.dispatch_stats()["dispatches"] - before == 2 + stages * (stages + 1) // 2
    got_k, got_v = sorted_keys.numpy, sorted_values.numpy
    want = keys[np.argsort(keys, kind="stable")]
    assert np.sum(np.abs(got_k.astype(np.int64) - want.astype(np.int64))) == 0
    assert np.array_equal(keys[got_v], got_k) and np.array_equal(np.sort(got_v), values)
    for t in (sorted_keys, sorted_values):
        t.release()
    prog.destroy()
