"""Recorded graphs: a sequence of launches recorded once and replayed with one call must give what the same
calls give when issued one by one. Every graph is replayed several times, with ordinary work, host copies and
synchronisation between the replays, and every replay is checked (bit-exact: the same kernels run on the same data)."""
import numpy as np
import pytest

from oracle import oracle

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def tf():
    import tensorfrost_amd.host as tfh

    tfh.initialize(tfh.hip)
    yield tfh
    tfh.synchronize()


def _eager_steps(tf, prog, u, v, steps):
    ut, vt = tf.tensor(u), tf.tensor(v)
    for _ in range(steps):
        v2, u2 = prog(ut, vt)
        ut.release(); vt.release()
        ut, vt = u2, v2
    out = ut.numpy, vt.numpy
    ut.release(); vt.release()
    return out


@pytest.mark.parametrize("shape,repeat", [((64, 96), 1), ((257, 1000), 5), ((2048, 2048), 10)])
def test_stencil_iteration_recorded_with_feedback(tf, shape, repeat):
    """wave_eq(u, v) -> (v', u'): `repeat` steps per graph, outputs fed back (u <- output 1, v <- output 0)."""
    u0 = oracle.sine_gordon_initial_field(*shape)
    v0 = np.zeros_like(u0)
    prog = tf.compile("wave_eq")
    u, v = tf.tensor(u0), tf.tensor(v0)
    graph = prog.record(u, v, repeat=repeat, feedback=(1, 0))
    assert graph.nodes >= repeat
    # the ordinary run that sizes the pool and the recording itself leave the inputs untouched
    assert np.array_equal(u.numpy, u0) and np.array_equal(v.numpy, v0)
    other = tf.compile("wave_eq")
    for replay in range(1, 4):
        graph.replay()
        # ordinary work between the replays: another program on other buffers, a readback, a synchronisation
        a, b = other(u0, v0)
        a.numpy
        a.release(); b.release()
        tf.synchronize()
        eu, ev = _eager_steps(tf, prog, u0, v0, repeat * replay)
        assert np.array_equal(graph.outputs[1].numpy, eu) and np.array_equal(graph.outputs[0].numpy, ev)
        assert np.array_equal(u.numpy, eu) and np.array_equal(v.numpy, ev)  # the feedback copy
    # one oracle step from the state the graph left is what one more eager step gives (ties the chain to the oracle)
    ou, ov = oracle.wave_eq(u0, v0, 0.1, repeat * 3)
    assert np.max(np.abs(u.numpy - ou)) < 1e-4 * max(np.max(np.abs(ou)), 1.0)
    graph.destroy()
    other.destroy()
    prog.destroy()


def test_new_inputs_between_replays_and_primitives_inside_a_graph(tf):
    """The lowered reductions of config 2's form (served by the reduction primitives, which use the scratch buffer):
    one recorded execution, inputs rewritten in place between replays."""
    shape = (1024, 1280)
    rng = np.random.default_rng(5)
    prog = tf.compile("reductions_ir")
    x = tf.tensor(np.zeros(shape, np.float32))
    graph = prog.record(x)
    for _ in range(3):
        data = rng.uniform(-4, 4, shape).astype(np.float32)
        x.write(data)
        graph.replay()
        eager = prog(data)
        for got, want in zip(graph.outputs, eager):
            assert np.array_equal(got.numpy, want.numpy)
            want.release()
        assert np.array_equal(graph.outputs[1].numpy, data.max(axis=1))
    graph.destroy()
    prog.destroy()


def test_a_loop_shared_by_several_groups_inside_a_graph(tf):
    """The mean over axis 0 of a tall tensor with few columns is a loop down the columns that several HIP groups share
    slab by slab (per-slab results in a pooled temporary, a ticket per group of 64 threads that the last group resets):
    recorded once, replayed on new data, equal to the call-by-call results bit for bit every time."""
    shape = (6000, 4, 4, 8)
    rng = np.random.default_rng(12)
    prog = tf.compile("reshape_reduction")
    a = tf.tensor(np.zeros(shape, np.float32))
    graph = prog.record(a)
    for _ in range(3):
        data = rng.uniform(-1, 3, shape).astype(np.float32)
        a.write(data)
        graph.replay()
        eager = prog(data)
        for got, want in zip(graph.outputs, eager):
            assert np.array_equal(got.numpy, want.numpy)
            want.release()
        mean_block = graph.outputs[-1].numpy
        assert np.allclose(mean_block, data.astype(np.float64).mean(axis=0), rtol=1e-5, atol=1e-6)
    graph.destroy()
    prog.destroy()


@pytest.mark.parametrize("emitted", [True, False], ids=["kernels_as_emitted", "region_served_by_onesweep"])
def test_reference_sort_composition_as_one_graph(tf, emitted, monkeypatch):
    """The reference's sort composition recorded once, bit-exact on every replay: as its six passes of emitted kernels
    with group memory, barriers and atomics (recognition switched off while recording), and as the one onesweep call
    that serves the recognised `Radix sort` region (a handful of nodes)."""
    if emitted:
        monkeypatch.setenv("TFHIP_NO_IDIOMS", "1")
    n = 50000
    rng = np.random.default_rng(6)
    prog = tf.compile("radix_sort_ir", [tf.uint32])
    keys = tf.tensor(np.zeros(n, np.uint32))
    vals = tf.tensor(np.arange(n, dtype=np.uint32))
    graph = prog.record(keys, vals)
    assert graph.nodes >= 40 if emitted else graph.nodes <= 12
    for _ in range(3):
        k = rng.integers(0, 2**32, n, dtype=np.uint64).astype(np.uint32)
        k[::3] %= 7
        keys.write(k)
        graph.replay()
        tf.synchronize()
        order = np.argsort(k, kind="stable")
        assert np.array_equal(graph.outputs[0].numpy, k[order])
        assert np.array_equal(graph.outputs[1].numpy, order.astype(np.uint32))
    graph.destroy()
    prog.destroy()


def test_split_matmul_tails_and_row_scans_inside_a_graph(tf):
    """Kernels that the dispatcher splits (matmul primitive into a pooled temporary + emitted tail kernel) and the
    row-wise scan primitive, recorded: the temporaries belong to the graph, replays match call-by-call results."""
    M, K, N = 300, 64, 128
    rng = np.random.default_rng(11)
    prog = tf.compile("dense_tanh")
    ins = [tf.tensor(np.zeros(s, np.float32)) for s in [(M, K), (K, N), (N,), (M, N), (M, N)]]
    graph = prog.record(*ins)
    for _ in range(3):
        data = [rng.uniform(-1, 1, t.shape).astype(np.float32) for t in ins]
        for t, d in zip(ins, data):
            t.write(d)
        graph.replay()
        eager = prog(*data)
        for got, want in zip(graph.outputs, eager):
            assert np.array_equal(got.numpy, want.numpy)
            want.release()
    graph.destroy()
    prog.destroy()
    prog = tf.compile("lowered_idioms")
    X, W = tf.tensor(np.zeros((64, 1024), np.float32)), tf.tensor(np.zeros((1024, 32), np.float32))
    graph = prog.record(X, W)
    for _ in range(2):
        x, w = rng.normal(size=(64, 1024)).astype(np.float32), rng.normal(size=(1024, 32)).astype(np.float32)
        X.write(x)
        W.write(w)
        graph.replay()
        eager = prog(x, w)
        for got, want in zip(graph.outputs, eager):
            assert np.array_equal(got.numpy, want.numpy)
            want.release()
    graph.destroy()
    prog.destroy()


def test_graph_buffers_leave_and_rejoin_the_pool(tf):
    prog = tf.compile("wave_eq")
    u, v = tf.tensor(np.ones((300, 300), np.float32)), tf.tensor(np.zeros((300, 300), np.float32))
    graph = prog.record(u, v, repeat=3, feedback=(1, 0))
    unused_with_graph = tf.memory_stats()["unused_words"]
    # releasing an output handle does not hand the graph's buffer to the pool
    graph.outputs[0].release()
    assert tf.memory_stats()["unused_words"] == unused_with_graph
    graph.replay()
    graph.destroy()
    assert tf.memory_stats()["unused_words"] >= unused_with_graph + 2 * 300 * 300
    prog.destroy()


def test_record_argument_errors(tf):
    prog = tf.compile("wave_eq")
    u, v = tf.tensor(np.ones((8, 8), np.float32)), tf.tensor(np.zeros((8, 8), np.float32))
    with pytest.raises(tf.TFHostError, match="feedback"):
        prog.record(u, v, repeat=2)
    with pytest.raises(tf.TFHostError, match="names output"):
        prog.record(u, v, feedback=(2, 0))
    with pytest.raises(tf.TFHostError, match="zero executions"):
        prog.record(u, v, repeat=0)
    with pytest.raises(TypeError):
        prog.record(np.ones((8, 8), np.float32), v)
    # nothing is left in recording mode: ordinary execution still works
    a, b = prog(u, v)
    assert np.all(np.isfinite(a.numpy))
    prog.destroy()


def test_primitives_recorded_through_the_c_abi(rt):
    """Sort, prefix sum and softmax recorded back to back; replays against the same calls issued one by one."""
    n, rows, cols = 1 << 18, 512, 1000
    rng = np.random.default_rng(7)
    keys, vals = rt.DeviceBuffer(n), rt.DeviceBuffer.from_numpy(np.arange(n, dtype=np.uint32))
    ko, vo, sc = rt.DeviceBuffer(n), rt.DeviceBuffer(n), rt.DeviceBuffer(n)
    x, y = rt.DeviceBuffer(rows * cols), rt.DeviceBuffer(rows * cols)

    def work():
        rt.radix_sort_kv(keys, vals, ko, vo, n)
        rt.scan_inclusive(ko, sc, n)
        rt.softmax_rows(x, y, rows, cols)

    keys.write(rng.integers(0, 1000, n).astype(np.uint32))
    x.write(rng.uniform(-4, 4, rows * cols).astype(np.float32))
    work()  # sizes the scratch buffer
    rt.synchronize()
    graph = rt.Graph()
    with graph:
        work()
    assert graph.nodes >= 3
    for _ in range(3):
        k = rng.integers(0, 1000, n).astype(np.uint32)
        xs = rng.uniform(-4, 4, rows * cols).astype(np.float32)
        keys.write(k)
        x.write(xs)
        graph.launch()
        got = [b.numpy(np.uint32) for b in (ko, vo, sc)] + [y.numpy(np.float32)]
        for b in (ko, vo, sc, y):
            b.fill(0)
        work()
        want = [b.numpy(np.uint32) for b in (ko, vo, sc)] + [y.numpy(np.float32)]
        for g, w in zip(got, want):
            assert np.array_equal(g, w)
        order = np.argsort(k, kind="stable")
        assert np.array_equal(got[0], k[order]) and np.array_equal(got[1], order.astype(np.uint32))
        assert np.array_equal(got[2], np.cumsum(k[order], dtype=np.uint32))
    graph.destroy()


def test_calls_that_wait_are_refused_while_recording(rt):
    buf = rt.DeviceBuffer.from_numpy(np.arange(16, dtype=np.uint32))
    graph = rt.Graph()
    with pytest.raises(rt.TFHipError, match="while a graph is being recorded"):
        with graph:
            buf.fill(3)
            buf.numpy(np.uint32)
    assert graph.handle is None
    with pytest.raises(rt.TFHipError, match="no graph is being recorded"):
        rt.call("tfhip_graph_end", None)
    # the abandoned recording ran nothing, and ordinary work goes on
    assert np.array_equal(buf.numpy(np.uint32), np.arange(16, dtype=np.uint32))
    buf.fill(3)
    assert np.all(buf.numpy(np.uint32) == 3)
