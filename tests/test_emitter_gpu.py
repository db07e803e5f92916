"""Emitted HIP kernels, op by op and construct by construct, against the CPU oracle: every scalar op of the op
table, atomics, group memory with a barrier, per-thread arrays, and the thread-serial reduction / scan / matmul
loops in the forms the reference's lowering leaves (run through the emitter, not through the primitives)."""
import numpy as np
import pytest

from conftest import sum_err
from oracle import oracle
from test_oracle_ops import FLOAT_OPS, INT_OPS, UINT_OPS, float_row_errors

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def tf():
    import tensorfrost_amd.host as tfh

    tfh.initialize(tfh.hip)
    yield tfh
    tfh.synchronize()


# 5000: the scalar entry point; 300001: the four-wide entry point with a ragged tail; 1 and 3: less than one quad
@pytest.mark.parametrize("n", [5000, 300001, 1, 3, 1 << 20])
def test_every_scalar_op(tf, n):
    inputs = oracle.ops_inputs(n, seed=n)
    prog = tf.compile("ops")
    F, I, U = (t.numpy for t in prog(*inputs))
    Fo, Io, Uo = oracle.ops(*inputs)
    for k, name in enumerate(INT_OPS):
        assert np.array_equal(I[k], Io[k]), f"int op {name}"
    for k, name in enumerate(UINT_OPS):
        if name == "from_float":
            continue  # checked below: the product of the cast's argument may round differently by one ulp
        assert np.array_equal(U[k], Uo[k]), f"uint op {name}"
    assert np.max(np.abs(U[UINT_OPS.index("from_float")].astype(np.int64) - Uo[UINT_OPS.index("from_float")].astype(np.int64))) <= 1
    err = float_row_errors(F, Fo.astype(np.float64))
    for k, name in enumerate(FLOAT_OPS):
        assert err[k] < 1e-5, f"float op {name}: {err[k]:.3g}"  # element-wise tolerance 1e-5
    prog.destroy()


@pytest.mark.parametrize("n,bins", [(100000, 16), (777, 5), (1 << 20, 256)])
def test_atomics(tf, n, bins):
    rng = np.random.default_rng(n)
    keys = rng.integers(0, bins, n).astype(np.uint32)
    vals = rng.normal(size=n).astype(np.float32)
    ints = rng.integers(-2**31, 2**31 - 1, n).astype(np.int32)
    prog = tf.compile("atomics", [bins])
    hist, fsum, imax, imin, bits, tickets, fmax, fmin = (t.numpy for t in prog(keys, vals, ints))
    assert np.array_equal(hist, np.bincount(keys, minlength=bins).astype(np.uint32))
    want_sum = np.zeros(bins, np.float64)
    np.add.at(want_sum, keys, vals.astype(np.float64))
    abs_sum = np.zeros(bins, np.float64)
    np.add.at(abs_sum, keys, np.abs(vals).astype(np.float64))
    assert sum_err(fsum, want_sum, abs_sum) < 1e-4  # float atomics add in arrival order: reduction tolerance
    for b in range(bins):
        sel = keys == b
        if sel.any():
            assert imax[b] == ints[sel].max() and imin[b] == ints[sel].min()
            assert fmax[b] == vals[sel].max() and fmin[b] == vals[sel].min()
    assert bits[0] == np.bitwise_and.reduce(keys | np.uint32(0xFFFFFF00))
    assert bits[1] == np.bitwise_or.reduce(keys)
    assert bits[2] == np.bitwise_xor.reduce(keys)
    # InterlockedAdd_Prev on one counter hands every thread a distinct ticket
    assert np.array_equal(np.sort(tickets), np.arange(n, dtype=np.uint32))
    prog.destroy()


@pytest.mark.parametrize("groups", [1, 7, 4096])
def test_group_memory_barrier_and_local_array(tf, groups):
    rng = np.random.default_rng(groups)
    data = rng.normal(size=(groups, 128)).astype(np.float32)
    prog = tf.compile("group_reverse")
    out = prog(data)
    # the per-thread array holds 0, .25, .5, .75 -> total 1.5, exact in fp32
    assert np.array_equal(out.numpy, data[:, ::-1] + np.float32(1.5))
    kernel = prog.kernels()[0]
    assert kernel["mapping"] == "group" and "__shared__ float tile[128]" in kernel["source"]
    prog.destroy()


@pytest.mark.parametrize("n,k", [(64, 64), (100, 36), (4, 260), (1028, 772)])
def test_tiled_kernel_threads_sit_where_the_reference_puts_them(tf, n, k):
    """Kernel of shape [N/4, K/4] with 16x16 groups (the frame of the reference's tiled matrix product): element
    (i1, i0) is written by the thread with index_1 = i1, index_0 = i0, and its tile origin, passed through group
    memory, is (i1 - i1 % 16, i0 - i0 % 16) -- tx = block_thread_id1 walks index_1, ty = block_thread_id0 index_0, as
    in the kernel text the reference printed (tests/golden/tiled_kernel_index_header.json)."""
    prog = tf.compile("tile_indices")
    ids, tiles = (t.numpy for t in prog(np.zeros((n, k), np.float32)))
    i1, i0 = np.meshgrid(np.arange(n // 4), np.arange(k // 4), indexing="ij")
    assert np.array_equal(ids, i1 * 65536 + i0)
    assert np.array_equal(tiles, (i1 - i1 % 16) * 65536 + (i0 - i0 % 16))
    prog.destroy()


@pytest.mark.parametrize("n,m,k", [(64, 64, 64), (128, 192, 64), (256, 64, 320), (1024, 512, 768)])
def test_reference_tiled_matmul_example_through_the_emitter(tf, n, m, k):
    """The reference's hand-tiled matrix product (two 64x64 group buffers, two barriers per panel, 4x4 results per
    thread) as an emitted user kernel, against the oracle's matmul (tolerance 1e-4 of the sum of magnitudes)."""
    rng = np.random.default_rng(n + m + k)
    a = rng.normal(size=(n, m)).astype(np.float32)
    b = rng.normal(size=(m, k)).astype(np.float32)
    prog = tf.compile("tiled_matmul_ir")
    (kernel,) = prog.kernels()
    assert kernel["mapping"] == "group" and "__shared__ float A_group_tile[4096]" in kernel["source"]
    c = prog(a, b).numpy
    want = oracle.matmul(a, b)
    scale = np.abs(a).astype(np.float64) @ np.abs(b).astype(np.float64)
    assert np.max(np.abs(c - want) / scale) < 1e-4
    assert np.max(np.abs(c - a.astype(np.float64) @ b.astype(np.float64)) / scale) < 1e-6
    with pytest.raises(tf.TFHostError, match="multiple of 64"):
        prog(a[:, :-1], b[:-1])
    prog.destroy()


@pytest.mark.parametrize("primitives", [False, True], ids=["emitted", "primitives"])
@pytest.mark.parametrize("R,C,N", [(64, 1024, 32), (100, 300, 7), (3, 128, 1), (1, 5, 5), (517, 2048, 20), (2, 70000, 3), (1280, 384, 4), (256, 130, 2), (4096, 256, 3), (20000, 100, 2)])
def test_lowered_reduction_scan_matmul_loops(tf, monkeypatch, R, C, N, primitives):
    """The same lowered loops twice: as emitted kernels, and with the kernels that are exactly one reduction /
    prefix-sum / matmul loop served by the hand-written primitives (the default)."""
    if not primitives:
        monkeypatch.setenv("TFHIP_NO_IDIOMS", "1")
    rng = np.random.default_rng(R * 1000 + C)
    X = rng.normal(size=(R, C)).astype(np.float32)
    W = rng.normal(size=(C, N)).astype(np.float32)
    prog = tf.compile("lowered_idioms")
    # the three reductions down the columns come in two forms (sliced among waves, thread-serial): three more kernels
    assert [k["mapping"].partition("+")[2] for k in prog.kernels()] == ["reduce"] * 6 + ["scan", "matmul"] + [""] * 3
    before = tf.dispatch_stats()
    sum_last, max_last, sum_first, scanned, product, max_first = (t.numpy for t in prog(X, W))
    after = tf.dispatch_stats()
    assert after["dispatches"] - before["dispatches"] == 8
    # The first stage of a split reduction is served only when the chunks tile the axis exactly (otherwise the emitted
    # kernel keeps the reference's zero padding); the prefix sum along the last axis goes to the row-wise scan.
    served = 6 + (C % 128 == 0) + (R % 128 == 0)
    assert after["served_by_primitives"] - before["served_by_primitives"] == (served if primitives else 0)
    absX = np.abs(X).astype(np.float64)
    assert sum_err(sum_last, oracle.reduce_rows("sum", X), absX.sum(1)) < 1e-4
    # the 128-chunk split pads the last chunk with zeros (the reference's SplitDim), so a row of negatives maxes to 0
    want_max = oracle.reduce_rows("max", X)
    if C % 128:
        want_max = np.maximum(want_max, np.float32(0))
    assert np.array_equal(max_last, want_max)
    want_max0 = oracle.reduce_cols("max", X)
    if R % 128:
        want_max0 = np.maximum(want_max0, np.float32(0))
    assert np.array_equal(max_first, want_max0)
    assert sum_err(sum_first, oracle.reduce_cols("sum", X), absX.sum(0)) < 1e-4
    assert sum_err(scanned, oracle.scan_inclusive(X), np.cumsum(absX, axis=1)) < 1e-4
    scale = absX @ np.abs(W).astype(np.float64)
    assert sum_err(product, oracle.matmul(X, W), scale) < 1e-4
    prog.destroy()


@pytest.mark.parametrize("primitives", [False, True], ids=["emitted", "primitives"])
@pytest.mark.parametrize("M,K,N", [(256, 64, 128), (100, 33, 7), (1000, 256, 3), (1, 1, 1), (300, 200, 260)])
def test_dense_layer_kernels_with_fused_tails(tf, monkeypatch, M, K, N, primitives):
    """Matmul loop + bias / ReLU / mask in one kernel, as kernel fusion leaves a dense layer: emitted as is, and
    served by the matmul primitive with the matching fused tail. Integer-valued operands make both paths exact."""
    if not primitives:
        monkeypatch.setenv("TFHIP_NO_IDIOMS", "1")
    rng = np.random.default_rng(M + K + N)
    X = rng.integers(-3, 4, (M, K)).astype(np.float32)
    W = rng.integers(-3, 4, (K, N)).astype(np.float32)
    bias = rng.integers(-5, 6, N).astype(np.float32)
    G = rng.integers(-3, 4, (M, N)).astype(np.float32)
    prog = tf.compile("dense_layer")
    assert [k["mapping"].partition("+")[2] for k in prog.kernels()] == ["matmul", "matmul", "matmul"]
    before = tf.dispatch_stats()["served_by_primitives"]
    H, Y, dX = (t.numpy for t in prog(X, W, bias, G))
    assert tf.dispatch_stats()["served_by_primitives"] - before == (3 if primitives else 0)
    Z = oracle.matmul(X, W) + bias
    assert np.array_equal(Y, Z)
    assert np.array_equal(H, np.maximum(Z, 0))
    assert np.array_equal(dX, np.where(X > 0, oracle.matmul(G, W, "nt"), 0))
    prog.destroy()


@pytest.mark.parametrize("primitives", [False, True], ids=["emitted", "primitives"])
@pytest.mark.parametrize("M,K,N", [(64, 32, 48), (100, 70, 33), (1, 5, 3), (2048, 256, 128), (300, 1, 260)])
def test_matmul_loops_with_any_elementwise_tail(tf, monkeypatch, M, K, N, primitives):
    """Matmul loops whose tails are none of the fixed fused forms (two stores with a tanh and a residual; a product
    with loaded values and a host scalar): emitted as is, or split into the matmul primitive writing a pooled temporary
    plus the same kernel without its loop. Matmul tolerance 1e-4 of the sum of magnitudes; the tail is element-wise."""
    if not primitives:
        monkeypatch.setenv("TFHIP_NO_IDIOMS", "1")
    rng = np.random.default_rng(M * 7 + K + N)
    X = rng.uniform(-1, 1, (M, K)).astype(np.float32)
    W = rng.normal(size=(K, N)).astype(np.float32)
    bias = rng.normal(size=N).astype(np.float32)
    R = rng.normal(size=(M, N)).astype(np.float32)
    G = rng.normal(size=(M, N)).astype(np.float32)
    prog = tf.compile("dense_tanh")
    kernels = prog.kernels()
    # the two kernels of the program, then the two tail kernels built from them (one more read-only buffer each)
    assert [k["mapping"].partition("+")[2] for k in kernels] == ["matmul", "matmul", "", ""]
    assert all("matmul_product_mem" in k["source"] and "for (int vloop" not in k["source"] for k in kernels[2:])
    assert all("for (int vloop" in k["source"] for k in kernels[:2])
    before = tf.dispatch_stats()
    created = tf.memory_stats()["buffers_created"]
    Z, H, dX = (t.numpy for t in prog(X, W, bias, R, G))
    after = tf.dispatch_stats()
    assert after["dispatches"] - before["dispatches"] == 2
    assert after["served_by_primitives"] - before["served_by_primitives"] == (2 if primitives else 0)
    z64 = X.astype(np.float64) @ W.astype(np.float64) + bias
    scale = np.abs(X).astype(np.float64) @ np.abs(W).astype(np.float64) + np.abs(bias)
    assert np.max(np.abs(Z - z64) / scale) < 1e-4
    assert np.max(np.abs(Z - (oracle.matmul(X, W) + bias)) / scale) < 1e-4
    # tanh has slope <= 1: H inherits Z's error plus the element-wise 1e-5
    assert np.max(np.abs(H - (np.tanh(z64) + R)) / (scale + np.abs(R) + 1)) < 1e-4
    assert np.max(np.abs(H - (np.tanh(Z.astype(np.float64)) + R))) < 1e-5 * (1 + np.abs(R).max())
    g64 = G.astype(np.float64) @ W.astype(np.float64).T
    gscale = np.abs(G).astype(np.float64) @ np.abs(W).astype(np.float64).T
    want = g64 * (1 - X.astype(np.float64) ** 2) * 0.5
    assert np.max(np.abs(dX - want) / (gscale + 1e-30)) < 1e-4
    if primitives:
        # the product temporaries come from the pool and go back to it: a second call creates no buffer
        created = tf.memory_stats()["buffers_created"]
        for t in prog(X, W, bias, R, G):
            t.release()
        for t in prog(X, W, bias, R, G):
            t.release()
        assert tf.memory_stats()["buffers_created"] - created <= 3
    prog.destroy()


@pytest.mark.parametrize("primitives", [False, True], ids=["emitted", "primitives"])
@pytest.mark.parametrize("T,M,K,N", [(3, 64, 32, 48), (5, 100, 70, 33), (1, 7, 5, 3), (16, 256, 128, 160), (40, 9, 16, 20)])
def test_matmul_with_a_leading_batch_dimension(tf, monkeypatch, T, M, K, N, primitives):
    """The reference's matmul carries batch dimensions through its loop: both operands batched, and one shared by the
    batch. As emitted loops, and as one batched launch of the matmul primitive."""
    if not primitives:
        monkeypatch.setenv("TFHIP_NO_IDIOMS", "1")
    rng = np.random.default_rng(T + M + K + N)
    A = rng.normal(size=(T, M, K)).astype(np.float32)
    B = rng.normal(size=(T, K, N)).astype(np.float32)
    W = rng.normal(size=(K, N)).astype(np.float32)
    prog = tf.compile("batched_matmul")
    assert [k["mapping"].partition("+")[2] for k in prog.kernels()] == ["matmul", "matmul"]
    before = tf.dispatch_stats()["served_by_primitives"]
    P, Q = (t.numpy for t in prog(A, B, W))
    assert tf.dispatch_stats()["served_by_primitives"] - before == (2 if primitives else 0)
    a64, b64, w64 = A.astype(np.float64), B.astype(np.float64), W.astype(np.float64)
    assert np.max(np.abs(P - a64 @ b64) / (np.abs(a64) @ np.abs(b64))) < 1e-4
    assert np.max(np.abs(Q - a64 @ w64) / (np.abs(a64) @ np.abs(w64))) < 1e-4
    for t in (0, T - 1):
        scale = np.abs(a64[t]) @ np.abs(b64[t])
        assert np.max(np.abs(P[t] - oracle.matmul(A[t], B[t])) / scale) < 1e-4
    prog.destroy()


@pytest.mark.parametrize("n,K,first", [(1000, 500, 0), (64, 5, 0), (70000, 4099, 17), (1, 16, 3), (130, 33, 33)])
def test_loops_over_a_shared_table_are_split_among_waves(tf, n, K, first):
    """Loops whose loads are the same in every thread: the waves of a HIP group take slices of the loop and combine
    in group memory. Three accumulators of different types and operations, a run-time first index, empty slices."""
    rng = np.random.default_rng(n + K)
    x = rng.normal(size=n).astype(np.float32)
    a = rng.integers(-100, 100, n).astype(np.int32)
    table = rng.normal(size=K).astype(np.float32)
    itable = rng.integers(-100, 100, K).astype(np.int32)
    prog = tf.compile("broadcast_loops")
    assert prog.kernels()[0]["mapping"] == "reduction:block"
    s, m, c = (t.numpy for t in prog(x, a, table, itable, np.array([first], np.int32)))
    t64 = table[first:].astype(np.float64)
    assert sum_err(s, t64.sum() * x, np.abs(t64).sum() * np.abs(x) + 1e-30) < 1e-4
    want_max = (table[first:, None] - x[None, :]).max(0) if K > first else np.full(n, -3.402823466e+38, np.float32)
    assert np.array_equal(m, want_max.astype(np.float32))
    assert np.array_equal(c, (itable[first:, None] > a[None, :]).sum(0).astype(np.int32))
    prog.destroy()


@pytest.mark.parametrize("dims,shape", [(3, (1, 5, 9, 13)), (3, (1, 8, 8, 8)), (3, (1, 33, 20, 100)), (3, (1, 1, 1, 1)), (3, (1, 64, 64, 64)),
                                        (4, (3, 5, 9, 13)), (4, (2, 16, 8, 32)), (4, (7, 1, 3, 2))])
def test_index_decoding_of_3d_and_4d_kernels(tf, dims, shape):
    """block_id -> per-dimension block index -> index_k with 8x8x8 groups and an ungrouped outer dimension; clamped,
    periodic and transposed addresses checked against NumPy indexing."""
    B, D, H, W = shape
    rng = np.random.default_rng(sum(shape))
    data = rng.normal(size=shape).astype(np.float32)
    prog = tf.compile("indexing", [dims])
    shifted, transposed, ids = (t.numpy for t in prog(data))
    z = np.clip(np.arange(D) - 1, 0, D - 1)
    y = (np.arange(H) + 1) % H
    x = np.clip(np.arange(W) + 2, 0, W - 1)
    assert np.array_equal(shifted, data[:, z][:, :, y][:, :, :, x])
    assert np.array_equal(transposed, data.transpose(0, 3, 2, 1))
    assert np.array_equal(ids, np.arange(data.size, dtype=np.int32).reshape(shape))
    prog.destroy()


@pytest.mark.parametrize("n,shift", [(128, 0), (128 * 37, 6), (128 * 5 + 100, 12), (1 << 20, 26)])
def test_reference_gpu_sort_scatter_kernel_runs_as_emitted(tf, n, shift):
    """One pass of the reference's radix sort, GPU branch (sort.py:133-169): group buffers, barriers, a packed atomic add on
    group memory and a run-time loop, emitted with the IR's own 128-thread group. The histogram scans the kernel consumes
    are made with NumPy; the result must be the stable partition of keys and payload by the 6-bit digit."""
    rng = np.random.default_rng(n + shift)
    keys = rng.integers(0, 2**32, n, dtype=np.uint64).astype(np.uint32)
    values = np.arange(n, dtype=np.uint32)
    digits = ((keys >> np.uint32(shift)) & np.uint32(63)).astype(np.int64)
    groups = (n + 127) // 128
    hist = np.zeros((groups, 64), np.uint32)
    np.add.at(hist, (np.arange(n) // 128, digits), 1)
    scan = np.cumsum(hist, axis=0, dtype=np.uint32)
    total = np.cumsum(scan[-1], dtype=np.uint32)
    prog = tf.compile("radix_scatter_pass", [shift])
    assert prog.kernels()[0]["mapping"] == "group"
    keys_out, values_out = (t.numpy for t in prog(keys, values, scan, total))
    order = np.argsort(digits, kind="stable")
    assert np.array_equal(keys_out, keys[order])
    assert np.array_equal(values_out, values[order])
    prog.destroy()


def test_emitted_source_is_hip_with_the_reference_statement_forms(tf):
    """Statement forms of the generator: loads as asfloat(X_mem[addr]), stores as X_mem[addr] = asuint(v),
    casts as ((T)(x)), loops as for (int i = a; i < b; i += s)."""
    prog = tf.compile("lowered_idioms")
    src = prog.kernels()[6]["source"]  # the scan kernel
    # a word that only this thread reads, and only at this step, is fetched past the caches; any other load is X_mem[addr]
    assert "asfloat(tf_stream_load(X_mem + ((index_0 * var.C) + vloop)))" in src
    matmul = prog.kernels()[7]["source"]
    assert "asfloat(X_mem[" in matmul and "asfloat(W_mem[" in matmul and "tf_stream_load(X_mem" not in matmul
    assert "scanned_mem[(index_0 * var.C) + vloop] = asuint(prefix_sum);" in src
    assert "for (int vloop = 0; vloop < var.C; vloop += 1)" in src
    prog.destroy()
