"""The drop-in path on the GPU: host program -> TFRuntime callbacks -> pooled hipMalloc tensors ->
emitted HIP kernels compiled by hiprtc, checked against the CPU oracle."""
import numpy as np
import pytest

from conftest import sum_err
from oracle import oracle
from test_oracle_stencil import term_scale

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def tf():
    import tensorfrost_amd.host as tfh

    tfh.initialize(tfh.hip)
    yield tfh
    tfh.synchronize()


def test_tensor_roundtrip_and_coercion(tf):
    a = np.arange(24, dtype=np.float64).reshape(2, 3, 4)
    t = tf.tensor(a)
    assert t.shape == (2, 3, 4) and t.type == tf.float32
    assert np.array_equal(t.numpy, a.astype(np.float32))
    assert tf.tensor(np.array([-3, 5])).numpy.dtype == np.int32
    assert tf.tensor(np.array([True, False, True])).numpy.tolist() == [True, False, True]
    with pytest.raises(tf.TFHostError, match="size 0"):
        tf.tensor(np.zeros((0, 4), np.float32))


@pytest.mark.parametrize("shape", [(16, 16), (37, 53), (1, 7), (130, 64), (257, 1000)])
def test_wave_eq_single_step_matches_oracle(tf, shape):
    rng = np.random.default_rng(61)
    u = rng.normal(size=shape).astype(np.float32)
    v = rng.normal(size=shape).astype(np.float32)
    prog = tf.compile("wave_eq")
    v_new, u_new = prog(u, v)
    gu, gv = u_new.numpy, v_new.numpy
    ou, ov = oracle.wave_eq(u, v, 0.1, 1)
    su, sv = term_scale(u, v, 0.1)
    # 1e-5 of the scale of the terms (elementwise / stencil tolerance of the north star)
    assert sum_err(gu, ou, su) < 1e-5 and sum_err(gv, ov, sv) < 1e-5
    prog.destroy()


def test_wave_eq_config1_shape_and_drift(tf):
    """benchmark config 1: 2048x2048, seeded 16-Gaussian field. Single step from identical state against
    the oracle; then 100 steps, comparing norm-wise (1-ulp differences compound over steps)."""
    n = 2048
    u0 = oracle.sine_gordon_initial_field(n, n)
    v0 = np.zeros_like(u0)
    prog = tf.compile("wave_eq")
    v1, u1 = prog(u0, v0)
    ou, ov = oracle.wave_eq(u0, v0, 0.1, 1)
    su, sv = term_scale(u0, v0, 0.1)
    assert sum_err(u1.numpy, ou, su) < 1e-5 and sum_err(v1.numpy, ov, sv) < 1e-5
    u, v = u1, v1
    created_before = tf.memory_stats()["buffers_created"]
    for _ in range(99):
        v2, u2 = prog(u, v)
        u.release(); v.release()
        u, v = u2, v2
    ou, ov = oracle.wave_eq(u0, v0, 0.1, 100)
    gu = u.numpy
    assert np.max(np.abs(gu - ou)) < 1e-4 * np.max(np.abs(ou))
    # energy-like invariant of the linearised system stays bounded: the field does not blow up
    assert np.max(np.abs(gu)) < 2 * np.max(np.abs(u0)) + 1
    # steady state allocates at most one more pair: outputs ping-pong through the pool
    assert tf.memory_stats()["buffers_created"] - created_before <= 2
    prog.destroy()


def test_input_checks_raise_like_the_reference(tf):
    prog = tf.compile("wave_eq")
    u = np.zeros((8, 8), np.float32)
    with pytest.raises(tf.TFHostError, match="Invalid number of inputs for TensorProgram. Expected 2, got 1"):
        prog(u)
    with pytest.raises(tf.TFHostError, match="Invalid shape for dimension 1 in v. Expected 8, got 9"):
        prog(u, np.zeros((8, 9), np.float32))
    with pytest.raises(tf.TFHostError, match="Invalid type for v. Expected Float, got Int"):
        prog(u, np.zeros((8, 8), np.int32))
    with pytest.raises(tf.TFHostError, match="Invalid number of dimensions for u"):
        prog(np.zeros(8, np.float32), np.zeros(8, np.float32))
    prog.destroy()


def test_pool_reuses_buffers(tf):
    """First fit in [n, 16n] (TensorMemory.cpp:182-224): a released buffer serves a slightly smaller request,
    but not one more than 16 times smaller."""
    a = tf.tensor(np.ones(100_003, np.float32))
    pa = a.device_pointer
    a.release()
    b = tf.tensor(np.ones(90_001, np.float32))
    assert b.device_pointer == pa
    assert b.numpy.sum() == 90_001
    b.release()
    c = tf.tensor(np.ones(5_000, np.float32))  # 16 * 5000 < 100003
    assert c.device_pointer != pa
    d = tf.tensor(np.ones(99_999, np.float32))
    assert d.device_pointer == pa
    c.release(); d.release()


def _nbody_scale(x, m, eps):
    """Sum of magnitudes of the force terms per body (float64), the scale a 65536-term fp32 sum errs against."""
    from test_oracle_nbody import accel64

    return accel64(x, m, eps)


@pytest.mark.parametrize("n", [1, 2, 255, 1000, 4096])
def test_nbody_step_matches_oracle(tf, n):
    x, v, m = oracle.nbody_inputs(n)
    dt, eps = np.float32(1e-3), np.float32(1e-3)
    prog = tf.compile("nbody")
    x_new, v_new = prog(x, v, m, np.array([dt]), np.array([eps]))
    gx, gv = x_new.numpy, v_new.numpy
    ox, ov = oracle.nbody_step(x, v, m, dt, eps)
    a, scale = _nbody_scale(x, m, eps)
    # reductions: 1e-4, measured against the sum of magnitudes of the accumulated terms
    assert np.max(np.abs(gv - ov) / (np.abs(v) + scale * dt + 1e-30)) < 1e-4
    # x' = x + v' dt: element-wise 1e-5 of |x| on top of dt times the velocity tolerance
    assert np.all(np.abs(gx - ox) <= 1e-5 * np.abs(x) + dt * 1e-4 * (np.abs(v) + scale * dt) + 1e-30)
    prog.destroy()


def test_nbody_config4_full_size(tf):
    """benchmark config 4: N = 65536. Against the oracle on every body, plus momentum conservation."""
    n = 65536
    x, v, m = oracle.nbody_inputs(n)
    dt, eps = np.float32(1e-3), np.float32(1e-3)
    prog = tf.compile("nbody")
    x_new, v_new = prog(x, v, m, np.array([dt]), np.array([eps]))
    gv = v_new.numpy
    ox, ov = oracle.nbody_step(x, v, m, dt, eps)
    dv_scale = np.abs(ov - v).max()
    assert np.max(np.abs(gv - ov)) < 1e-4 * dv_scale
    assert np.max(np.abs(x_new.numpy - ox)) < 1e-6 + dt * 1e-4 * dv_scale  # x inherits dt times the velocity error
    dv = gv.astype(np.float64) - v
    dp = (m[:, None] * dv).sum(0)
    assert np.all(np.abs(dp) < 1e-4 * (m[:, None] * np.abs(dv)).sum(0))
    prog.destroy()


def _run_mlp(tf, prog, coords, target, params, m, v, t):
    ins = [coords, target] + params + m + v + [np.array([t], np.float32)]
    outs = prog(*ins)
    vals = [o.numpy for o in outs]
    for o in outs:
        o.release()
    return float(vals[0][0]), vals[1:9], vals[9:17], vals[17:25], float(vals[25][0])


@pytest.mark.parametrize("unfused", [0, 1, 2], ids=["fused_tails", "separate_kernels", "lowered_loops"])
@pytest.mark.parametrize("batch", [64, 1000, 4096])
def test_mlp_step_matches_oracle(tf, batch, unfused):
    """Forward + backward + Adam of the coordinate MLP against the CPU oracle: matmul / reduction tolerance 1e-4,
    measured per tensor against its largest magnitude (gradients are long signed sums). In the third form every matmul
    and sum is the lowered loop kernel itself and reaches the primitives only by being recognised."""
    coords, target, params, m, v = oracle.mlp_inputs(batch, seed=9)
    rng = np.random.default_rng(10)
    for i in (1, 3, 5, 7):
        params[i] = (rng.normal(size=params[i].shape) * 0.1).astype(np.float32)
    m = [(rng.normal(size=p.shape) * 0.01).astype(np.float32) for p in params]
    v = [(np.abs(rng.normal(size=p.shape)) * 1e-4).astype(np.float32) for p in params]
    prog = tf.compile("mlp", [unfused])
    before = tf.dispatch_stats()
    loss, p_new, m_new, v_new, t_new = _run_mlp(tf, prog, coords, target, params, m, v, 2.0)
    after = tf.dispatch_stats()
    # every layer's weight gradient X^T dY and bias gradient (column sums of dY) are dispatched one after the other and
    # served by one call that reads dY once, whether the program names the primitives or dispatches the lowered loops
    assert after["fused_chains"] - before["fused_chains"] == 4
    # the eight Adam kernels (one per parameter tensor, disjoint buffers apart from the step count they all read) leave as
    # one launch; the gradients the program releases between them return to the pool after it
    assert after["batched_launches"] - before["batched_launches"] >= 1
    assert after["batched_dispatches"] - before["batched_dispatches"] >= 8
    if unfused == 2:
        assert "primitive" not in " ".join(k["mapping"] for k in prog.kernels())
        # 4 forward products, 4 weight gradients, 3 input gradients, 4 bias gradients, the loss sum
        assert after["served_by_primitives"] - before["served_by_primitives"] == 16
    o_loss, o_p, o_m, o_v, _ = oracle.mlp_step(coords, target, params, m, v, t=2.0)
    assert t_new == 3.0
    assert abs(loss - o_loss) < 1e-4 * abs(o_loss)
    for i in range(8):
        assert np.max(np.abs(m_new[i] - o_m[i])) < 1e-4 * np.max(np.abs(o_m[i]))
        # v' = lerp(g*g, v, beta2) = g*g + (v - g*g)*0.999 cancels where g*g >> v: any fp32 evaluation (with or
        # without FMA) is only good to eps/(1 - beta2) ~ 6e-5 of g*g there, so v is compared at 1e-3
        assert np.max(np.abs(v_new[i] - o_v[i])) < 1e-3 * np.max(np.abs(o_v[i]))
        # the parameter moves by lr * mhat / (sqrt(vhat) + eps): compare the UPDATE, not the parameter
        upd, o_upd = p_new[i] - params[i], o_p[i] - params[i]
        assert np.max(np.abs(upd - o_upd)) < 2e-3 * np.max(np.abs(o_upd)) + 1e-9
        assert np.max(np.abs(p_new[i] - o_p[i])) < 1e-5 * max(np.max(np.abs(o_p[i])), 1e-3)
    prog.destroy()


@pytest.mark.parametrize("form", [0, 2], ids=["named_primitives", "lowered_loops"])
def test_mlp_step_with_bias_gradients_dispatched_first(tf, form):
    """Which of a layer's two gradients autodiff emits first is not fixed. With db = column sums of dY dispatched BEFORE
    dW = X^T dY the pair is still one call that reads dY once (the column sums are held for one dispatch); the step's
    results are those of the other order."""
    batch = 4096
    coords, target, params, m, v = oracle.mlp_inputs(batch, seed=21)
    results = []
    for order in (0, 1):
        prog = tf.compile("mlp", [form, order])
        before = tf.dispatch_stats()
        results.append(_run_mlp(tf, prog, coords, target, params, m, v, 1.0))
        after = tf.dispatch_stats()
        # the lowered column sums are recognised kernels and can be held; a program that NAMES the reduction primitive
        # dispatches it at once, so there the reversed order pairs nothing
        assert after["fused_chains"] - before["fused_chains"] == (4 if form == 2 or order == 0 else 0)
        prog.destroy()
    (loss0, p0, m0, v0, _), (loss1, p1, m1, v1, _) = results
    assert loss0 == loss1
    for i in range(8):
        if form == 2:
            assert np.array_equal(p0[i], p1[i]) and np.array_equal(m0[i], m1[i]) and np.array_equal(v0[i], v1[i])
        else:
            assert np.max(np.abs(m0[i] - m1[i])) < 1e-5 * np.max(np.abs(m0[i]))


@pytest.fixture(scope="module")
def mlp_benchmark_case():
    """Inputs of benchmark config 5 at its real batch and what the oracle says about them. The loss is a mean over rows
    and every gradient is the mean of the gradients of equal chunks, so the oracle runs on the 64 chunks of 4096 rows
    (the size the other tests pin it at) and the chunk results are averaged in float64."""
    batch, chunk = 262144, 4096
    coords, target, params, m, v = oracle.mlp_inputs(batch, seed=1239)
    rng = np.random.default_rng(12)
    for i in (1, 3, 5, 7):
        params[i] = (rng.normal(size=params[i].shape) * 0.1).astype(np.float32)
    want_loss = 0.0
    want_grads = [np.zeros(p.shape, np.float64) for p in params]
    chunks = batch // chunk
    for c in range(chunks):
        rows = slice(c * chunk, (c + 1) * chunk)
        o_loss, _, _, _, o_grads = oracle.mlp_step(coords[rows], target[rows], params, m, v, t=0.0)
        want_loss += o_loss / chunks
        for i in range(8):
            want_grads[i] += o_grads[i].astype(np.float64) / chunks
    return coords, target, params, m, v, want_loss, want_grads


@pytest.mark.parametrize("form", [0, 2], ids=["fused_tails", "lowered_loops"])
def test_mlp_step_at_the_benchmark_batch(tf, mlp_benchmark_case, form):
    """Benchmark config 5 at its real batch of 262144, where the products pick other kernels than at 4096 (K-sliced and
    direct weight gradients, skinny layers, long column sums). With m = v = 0 and t = 0 the step's first moments are
    (1 - beta1) times the gradients. Tolerance: 1e-4 of each tensor's largest magnitude (matmul / reduction bar)."""
    coords, target, params, m, v, want_loss, want_grads = mlp_benchmark_case
    prog = tf.compile("mlp", [form])
    loss, p_new, m_new, v_new, t_new = _run_mlp(tf, prog, coords, target, params, m, v, 0.0)
    prog.destroy()
    assert t_new == 1.0
    assert abs(loss - want_loss) < 1e-4 * abs(want_loss)
    for i in range(8):
        got = m_new[i].astype(np.float64) / (1.0 - 0.9)
        assert np.max(np.abs(got - want_grads[i])) < 1e-4 * np.max(np.abs(want_grads[i])), f"gradient {i}"
        # first Adam step from zero moments: the update is lr * g / (|g| + eps'), i.e. lr against the gradient's sign
        upd = p_new[i] - params[i]
        big = np.abs(want_grads[i]) > 1e-3 * np.max(np.abs(want_grads[i]))
        assert np.all(np.sign(upd[big]) == -np.sign(want_grads[i][big]))
        assert np.max(np.abs(np.abs(upd[big]) - 1e-3)) < 2e-5


def test_mlp_training_reduces_the_loss(tf):
    """A few steps at the reference hyper-parameters: the loss goes down and stays finite."""
    coords, target, params, m, v = oracle.mlp_inputs(8192, seed=11)
    prog = tf.compile("mlp")
    t = 0.0
    losses = []
    for _ in range(8):
        loss, params, m, v, t = _run_mlp(tf, prog, coords, target, params, m, v, t)
        losses.append(loss)
    assert np.all(np.isfinite(losses)) and losses[-1] < losses[0]
    prog.destroy()


@pytest.mark.parametrize("shape", [(16384, 4096), (1024, 1280), (1000, 300), (130, 1024)])
def test_config2_reductions_in_the_lowered_split_form(tf, shape):
    """Sum and max over both axes as OptimizeReductions leaves them (128-chunk first stage behind the dim_split
    view, second stage over the partials). Stages whose chunks tile the axis go to the primitives; ragged ones run
    as emitted kernels and keep the reference's zero padding of the last chunk."""
    R, C = shape
    x = np.random.default_rng(1234 + 2).uniform(-4, 4, shape).astype(np.float32)
    prog = tf.compile("reductions_ir")
    kinds = [k["mapping"] for k in prog.kernels()]
    assert all(k.endswith("+reduce") for k in kinds[:8]) and kinds[8:] == ["flat:vec4"] * 4  # thread-serial twins of the column stages
    before = tf.dispatch_stats()
    s_last, m_last, s_first, m_first = (t.numpy for t in prog(x))
    after = tf.dispatch_stats()
    assert after["dispatches"] - before["dispatches"] == 8
    assert after["served_by_primitives"] - before["served_by_primitives"] == 4 + 2 * (C % 128 == 0) + 2 * (R % 128 == 0)
    # both stages of a split whose chunks tile the axis become one call of the reduction primitive on X itself, once
    # the program has released the chunk results
    assert after["fused_chains"] - before["fused_chains"] == 2 * (C % 128 == 0) + 2 * (R % 128 == 0)
    absx = np.abs(x).astype(np.float64)
    assert sum_err(s_last, oracle.reduce_rows("sum", x), absx.sum(1)) < 1e-4
    assert sum_err(s_first, oracle.reduce_cols("sum", x), absx.sum(0)) < 1e-4
    # x is in (-4, 4): every row and column holds positive values, so the zero padding never wins the max
    assert np.array_equal(m_last, oracle.reduce_rows("max", x))
    assert np.array_equal(m_first, oracle.reduce_cols("max", x))
    prog.destroy()


def _softmax_close(got, want):
    return np.max(np.abs(got - want) / np.maximum(np.abs(want), 1e-6 * np.abs(want).max())) < 1e-5


def test_split_reductions_whose_chunk_results_stay_alive(tf):
    """The chunk tensors are released only at the end of the program. For the first three reductions another dispatch
    arrives while the chunk results are still alive, so their stages run one by one (each served on its own); the last
    pair is still held when the releases come, nothing has read its chunk results, and it becomes one call on X."""
    R, C = 1024, 1280
    x = np.random.default_rng(77).uniform(-4, 4, (R, C)).astype(np.float32)
    prog = tf.compile("reductions_ir", [1])
    before, pool_before = tf.dispatch_stats(), tf.memory_stats()
    outs = prog(x)
    after = tf.dispatch_stats()
    assert after["fused_chains"] - before["fused_chains"] == 1
    assert after["served_by_primitives"] - before["served_by_primitives"] == 8 and after["dispatches"] - before["dispatches"] == 8
    s_last, m_last, s_first, m_first = (t.numpy for t in outs)
    absx = np.abs(x).astype(np.float64)
    assert sum_err(s_last, oracle.reduce_rows("sum", x), absx.sum(1)) < 1e-4 and sum_err(s_first, oracle.reduce_cols("sum", x), absx.sum(0)) < 1e-4
    assert np.array_equal(m_last, x.max(axis=1)) and np.array_equal(m_first, x.max(axis=0))
    for t in outs:
        t.release()
    pool_after = tf.memory_stats()
    assert pool_after["allocated_words"] - pool_after["unused_words"] == pool_before["allocated_words"] - pool_before["unused_words"]
    prog.destroy()


@pytest.mark.parametrize("primitives", [False, True], ids=["emitted", "primitives"])
@pytest.mark.parametrize("shape", [(16384, 4096), (1000, 1280), (37, 1027), (5, 128), (300, 5000), (64, 5120)])
def test_softmax_as_the_reference_composes_it(tf, monkeypatch, shape, primitives):
    """max / exp / sum / divide as five lowered kernels (both reductions split into 128-chunks, exp fused into the sum's
    first stage and into the final element-wise kernel): element-wise tolerance 1e-5 against the oracle's softmax.
    When the chunks tile the rows the kernel manager recognises the five dispatches as one softmax and runs the fused
    primitive once; otherwise (the last chunk is padded with zeros) the plain reduction kernels of the second stages go
    to the reduction primitives and the rest runs as emitted."""
    if not primitives:
        monkeypatch.setenv("TFHIP_NO_IDIOMS", "1")
    R, C = shape
    x = np.random.default_rng(R + C).uniform(-4, 4, shape).astype(np.float32)
    prog = tf.compile("softmax_ir")
    assert [k["mapping"].partition("+")[2] for k in prog.kernels()] == ["reduce", "reduce", "expsum", "reduce", "normalise"]
    before = tf.dispatch_stats()
    y = prog(x)
    got = y.numpy
    after = tf.dispatch_stats()
    assert after["dispatches"] - before["dispatches"] == 5
    fused = primitives and C % 128 == 0
    assert after["fused_chains"] - before["fused_chains"] == (1 if fused else 0)
    assert after["served_by_primitives"] - before["served_by_primitives"] == (5 if fused else 2 if primitives else 0)
    assert _softmax_close(got, oracle.softmax_rows(x))
    assert np.allclose(got.sum(axis=1, dtype=np.float64), 1.0, atol=1e-5)
    y.release()
    prog.destroy()


@pytest.mark.parametrize("split", [True, False], ids=["split", "unsplit"])
@pytest.mark.parametrize("shape", [(16384, 4096), (1000, 1280), (37, 1027), (300, 640)])
def test_softmax_whose_exponentials_are_a_tensor_of_their_own(tf, monkeypatch, shape, split):
    """Whether exp(x - m) is recomputed inside the kernels that use it or kept as a tensor E is the passes' decision. In the
    second cut the composition is: row maxima (one or two kernels), E = exp(x - m) (element-wise), row sums of E (a plain
    reduction, one or two kernels), Y = E / z (element-wise), E released. The chain of dispatches is recognised all the
    same -- by the two element-wise kernels' computations and the buffers they share -- and served by the one fused call,
    which never writes E; with recognition off the kernels run as emitted and give the same softmax."""
    R, C = shape
    x = np.random.default_rng(R * 7 + C).uniform(-4, 4, shape).astype(np.float32)
    flags = 32 | (0 if split else 1)
    prog = tf.compile("softmax_ir", [flags])
    kinds = [k["mapping"].partition("+")[2] for k in prog.kernels()]
    assert "expdiff" in kinds and "dividerows" in kinds  # (the program also builds the kernels of the other cut; it dispatches none of them)
    before = tf.dispatch_stats()
    y = prog(x)
    got = y.numpy
    after = tf.dispatch_stats()
    n = 6 if split else 4
    assert after["dispatches"] - before["dispatches"] == n
    fused = (not split) or C % 128 == 0  # a padded last chunk keeps the reference's zero padding, i.e. the emitted kernels
    assert after["fused_chains"] - before["fused_chains"] == (1 if fused else 0)
    if fused:
        assert after["served_by_primitives"] - before["served_by_primitives"] == n
    assert _softmax_close(got, oracle.softmax_rows(x))
    y.release()
    # E kept as an output: the program reads it, so every kernel runs (the reductions still go to their primitives)
    prog2 = tf.compile("softmax_ir", [flags | 64])
    before = tf.dispatch_stats()
    y2, e2 = prog2(x)
    after = tf.dispatch_stats()
    assert after["fused_chains"] - before["fused_chains"] == 0  # held to the end in case E is released, then run one by one
    e_want = np.exp(x - x.max(axis=1, keepdims=True))
    assert np.allclose(e2.numpy, e_want, rtol=2e-6, atol=1e-12)
    assert _softmax_close(y2.numpy, oracle.softmax_rows(x))
    y2.release()
    e2.release()
    prog2.destroy()
    # and as emitted
    monkeypatch.setenv("TFHIP_NO_IDIOMS", "1")
    y3 = prog(x)
    assert _softmax_close(y3.numpy, oracle.softmax_rows(x))
    y3.release()
    prog.destroy()


@pytest.mark.parametrize("shape", [(4096, 512), (1000, 10), (77, 333), (3, 1000), (100000, 64)])
def test_softmax_with_unsplit_reductions_is_one_primitive_call(tf, shape):
    """Rows shorter than 1024 keep whole-row reductions: three kernels (max, sum of exp(x - max), normalise), recognised
    as one softmax for any row length. The maxima and sums are outputs here: the fused call has to write them too."""
    R, C = shape
    x = np.random.default_rng(R * 3 + C).normal(0, 3, shape).astype(np.float32)
    prog = tf.compile("softmax_ir", [1 | 2])
    assert [k["mapping"].partition("+")[2] for k in prog.kernels()] == ["reduce", "expsum", "normalise"]
    before = tf.dispatch_stats()
    y, m, z = prog(x)
    after = tf.dispatch_stats()
    assert after["fused_chains"] - before["fused_chains"] == 1 and after["served_by_primitives"] - before["served_by_primitives"] == 3
    assert _softmax_close(y.numpy, oracle.softmax_rows(x))
    assert np.array_equal(m.numpy, x.max(axis=1))
    want_z = np.exp(x.astype(np.float64) - x.max(axis=1, keepdims=True)).sum(axis=1)
    assert np.max(np.abs(z.numpy - want_z) / want_z) < 1e-5
    for t in (y, m, z):
        t.release()
    prog.destroy()


def test_softmax_chain_keeps_its_intermediates_when_the_program_still_holds_them(tf):
    """Split form with maxima and sums as outputs: still one fused call (it writes both). With the chunk tensors released
    only after the last kernel the chain cannot tell that they are dead: every kernel runs as dispatched, in order."""
    R, C = 512, 2048
    x = np.random.default_rng(99).uniform(-6, 6, (R, C)).astype(np.float32)
    want_z = np.exp(x.astype(np.float64) - x.max(axis=1, keepdims=True)).sum(axis=1)
    for flags, fused in [(2, 1), (2 | 4, 0)]:
        prog = tf.compile("softmax_ir", [flags])
        pool_before = tf.memory_stats()
        before = tf.dispatch_stats()
        y, m, z = prog(x)
        after = tf.dispatch_stats()
        assert after["fused_chains"] - before["fused_chains"] == fused
        assert after["dispatches"] - before["dispatches"] == 5
        assert after["served_by_primitives"] - before["served_by_primitives"] == (5 if fused else 3)
        assert _softmax_close(y.numpy, oracle.softmax_rows(x))
        assert np.array_equal(m.numpy, x.max(axis=1))
        assert np.max(np.abs(z.numpy - want_z) / want_z) < 1e-5
        for t in (y, m, z):
            t.release()
        # every buffer the program took has gone back to the pool (the frees held back with the chain included)
        pool_after = tf.memory_stats()
        assert pool_after["allocated_words"] - pool_after["unused_words"] == pool_before["allocated_words"] - pool_before["unused_words"]
        prog.destroy()


def _log_softmax64(x):
    x64 = x.astype(np.float64)
    shifted = x64 - x64.max(axis=1, keepdims=True)
    return shifted - np.log(np.exp(shifted).sum(axis=1, keepdims=True))


@pytest.mark.parametrize("flags,shape", [(8, (2048, 1024)), (8, (16384, 4096)), (1 | 8, (1000, 10)), (1 | 8, (4096, 512)), (8, (300, 5000)), (8, (64, 8192)), (1 | 8, (5, 40000))])
def test_log_softmax_as_the_reference_composes_it_is_one_call(tf, flags, shape):
    """log_softmax(X) = (X - max) - log(sum(exp(X - max))) (the reference's tests/autograd_test.py:29-31): the max and
    sum kernels are those of a softmax and the last kernel is (x - m) - log(z). The whole sequence is recognised and
    served by the fused log-softmax: one read and one write of X."""
    R, C = shape
    x = np.random.default_rng(R + C + flags).normal(0, 3, shape).astype(np.float32)
    prog = tf.compile("softmax_ir", [flags])
    assert prog.kernels()[-1]["mapping"].endswith("+normalise")
    before = tf.dispatch_stats()
    y = prog(x)
    got = y.numpy
    after = tf.dispatch_stats()
    split = not (flags & 1)
    fused = not split or C % 128 == 0
    assert after["dispatches"] - before["dispatches"] == (5 if split else 3)
    assert after["fused_chains"] - before["fused_chains"] == (1 if fused else 0)
    assert after["served_by_primitives"] - before["served_by_primitives"] == ((5 if split else 3) if fused else 2)
    want = _log_softmax64(x)
    assert np.allclose(got, want, atol=1e-5 * max(1.0, np.abs(want).max()))
    y.release()
    prog.destroy()


@pytest.mark.parametrize("flags,shape", [(8 | 16, (2048, 1024)), (8 | 16, (16384, 4096)), (1 | 8 | 16, (1000, 10)), (1 | 8 | 16, (4096, 512)), (8 | 16, (300, 5000))])
def test_another_last_kernel_still_gets_both_row_statistics_from_one_read(tf, flags, shape):
    """The same max and sum kernels followed by a last kernel that is neither a softmax's nor a log-softmax's (the
    log-softmax scaled by -1/C, as a fused cross-entropy term would be). When it arrives, the two (four, when split)
    reduction dispatches that were held back are served by one statistics-only call: one read of X instead of two;
    the last kernel runs as emitted."""
    R, C = shape
    x = np.random.default_rng(R + C + flags).normal(0, 3, shape).astype(np.float32)
    prog = tf.compile("softmax_ir", [flags])
    before = tf.dispatch_stats()
    y = prog(x)
    got = y.numpy
    after = tf.dispatch_stats()
    split = not (flags & 1)
    fused = not split or C % 128 == 0
    assert after["dispatches"] - before["dispatches"] == (5 if split else 3)
    assert after["fused_chains"] - before["fused_chains"] == (1 if fused else 0)
    assert after["served_by_primitives"] - before["served_by_primitives"] == ((4 if split else 2) if fused else 2)
    want = _log_softmax64(x) * (-1.0 / C)
    assert np.allclose(got, want, atol=1e-5 * max(1.0 / C, np.abs(want).max()))
    y.release()
    prog.destroy()


@pytest.mark.parametrize("lengths", [(1000, 37, 5000), (1, 1, 1), (70000, 3, 129), (300000, 300000, 8)], ids=str)
def test_small_dispatches_on_disjoint_buffers_leave_as_one_launch(tf, lengths):
    """Seven dispatches of one kernel: three independent ones, one that reads an earlier result, a temporary that is
    written, read and released, one more independent one. Independent neighbours share a launch (grid.y picks the
    dispatch), a dependent one waits for what it reads, and the results are those of running them one by one. Dispatches
    large enough to fill the chip by themselves are launched on their own."""
    rng = np.random.default_rng(sum(lengths))
    a, b, c = (rng.normal(size=n).astype(np.float32) for n in lengths)
    shift = np.array([0.25], np.float32)
    prog = tf.compile("gathered_updates")
    before = tf.dispatch_stats()
    outs = prog(tf.tensor(a), tf.tensor(b), tf.tensor(c), tf.tensor(shift))
    after = tf.dispatch_stats()
    got = [o.numpy for o in outs]
    f = np.float32
    want = [a * f(2) + shift, b * f(3) + shift, c * f(4) + shift, (a * f(2) + shift) * f(5) + shift, (b * f(7) + shift) * f(1.5) + shift, -c + shift]
    for g, w in zip(got, want):
        assert np.allclose(g, w, rtol=1e-6, atol=1e-6)  # a fused multiply-add may round once instead of twice
    assert after["dispatches"] - before["dispatches"] == 7
    if max(lengths) < 100000:
        # {o1, o2, o3}, {o4, tmp}, {o5, o6}
        assert after["batched_launches"] - before["batched_launches"] == 3
        assert after["batched_dispatches"] - before["batched_dispatches"] == 7
    else:
        # a and b are launched alone; {tmp} is; only c's two are small, and they are not neighbours
        assert after["batched_launches"] - before["batched_launches"] == 0
    for o in outs:
        o.release()
    prog.destroy()


def test_gathering_can_be_switched_off(tf, monkeypatch):
    """TFHIP_NO_GATHER=1 (for a host that does not pass the written tensors first): the same seven dispatches leave as
    seven launches, with the same results."""
    monkeypatch.setenv("TFHIP_NO_GATHER", "1")
    rng = np.random.default_rng(9)
    a, b, c = (rng.normal(size=n).astype(np.float32) for n in (1000, 37, 5000))
    shift = np.array([0.25], np.float32)
    prog = tf.compile("gathered_updates")
    before = tf.dispatch_stats()
    outs = prog(tf.tensor(a), tf.tensor(b), tf.tensor(c), tf.tensor(shift))
    after = tf.dispatch_stats()
    f = np.float32
    want = [a * f(2) + shift, b * f(3) + shift, c * f(4) + shift, (a * f(2) + shift) * f(5) + shift, (b * f(7) + shift) * f(1.5) + shift, -c + shift]
    for o, w in zip(outs, want):
        assert np.allclose(o.numpy, w, rtol=1e-6, atol=1e-6)
    assert after["dispatches"] - before["dispatches"] == 7
    assert after["batched_launches"] - before["batched_launches"] == 0
    for o in outs:
        o.release()
    prog.destroy()


def test_gathered_dispatches_inside_a_recorded_graph(tf):
    rng = np.random.default_rng(77)
    prog = tf.compile("gathered_updates")
    ins = [tf.tensor(np.zeros(n, np.float32)) for n in (1000, 37, 5000)] + [tf.tensor(np.array([0.5], np.float32))]
    graph = prog.record(*ins)
    assert graph.nodes == 3
    for _ in range(3):
        data = [rng.normal(size=n).astype(np.float32) for n in (1000, 37, 5000)]
        for t, d in zip(ins, data):
            t.write(d)
        graph.replay()
        a, b, c = data
        f, s = np.float32, np.float32(0.5)
        want = [a * f(2) + s, b * f(3) + s, c * f(4) + s, (a * f(2) + s) * f(5) + s, (b * f(7) + s) * f(1.5) + s, -c + s]
        for o, w in zip(graph.outputs, want):
            assert np.allclose(o.numpy, w, rtol=1e-6, atol=1e-6)
    graph.destroy()
    prog.destroy()


def test_softmax_chain_inside_a_recorded_graph(tf):
    R, C = 2048, 1024
    rng = np.random.default_rng(5)
    prog = tf.compile("softmax_ir")
    x = tf.tensor(np.zeros((R, C), np.float32))
    graph = prog.record(x)
    assert graph.nodes <= 2  # one kernel for the whole chain
    for _ in range(3):
        data = rng.uniform(-5, 5, (R, C)).astype(np.float32)
        x.write(data)
        graph.replay()
        assert _softmax_close(graph.outputs[0].numpy, oracle.softmax_rows(data))
    graph.destroy()
    prog.destroy()


def _sort_keys(kind, n, low_entropy=False):
    rng = np.random.default_rng(n)
    if kind == "u32":
        keys = rng.integers(0, 1024 if low_entropy else 2**32, n, dtype=np.uint64).astype(np.uint32)
        keys[::3] = keys[::3] % 7  # duplicates: an unstable scatter would show in the payload
    elif kind == "i32":
        keys = rng.integers(-512 if low_entropy else -2**31, 512 if low_entropy else 2**31, n).astype(np.int32)
        keys[::3] = keys[::3] % 5 - 2
    else:
        keys = rng.normal(size=n).astype(np.float32)
        keys[::4] = np.round(keys[::4])
        keys[:8] = np.array([0.0, -0.0, np.inf, -np.inf, 1e-40, -1e-40, 3.4e38, -3.4e38], np.float32)[: min(8, n)]
    return keys


def _check_sorted(keys, values, ks, vs, kind):
    ok, ov = oracle.radix_sort_kv(keys, values)
    assert np.array_equal(ks.view(np.uint32), ok.view(np.uint32)) and np.array_equal(vs, ov)
    if kind != "f32":
        order = np.argsort(keys, kind="stable")
        assert np.array_equal(ks, keys[order]) and np.array_equal(vs, values[order])


_TYPES = {"u32": "uint32", "i32": "int32", "f32": "float32"}


@pytest.mark.parametrize("kind", ["u32", "i32", "f32"])
@pytest.mark.parametrize("n", [1, 127, 128, 1000, 8192 + 77, 1 << 20])
def test_reference_sort_composition_through_the_emitter(tf, n, kind, monkeypatch):
    """tf.sort.radix as the reference composes it (six 6-bit passes; packed group histograms, grouped prefix sums, the
    group-buffer scatter kernel), every kernel emitted (region recognition switched off): bit-exact and stable against
    the oracle's restatement of the same algorithm and against NumPy's stable argsort."""
    monkeypatch.setenv("TFHIP_NO_IDIOMS", "1")
    keys = _sort_keys(kind, n)
    values = np.arange(n, dtype=np.uint32)
    prog = tf.compile("radix_sort_ir", [getattr(tf, _TYPES[kind])])
    before = tf.dispatch_stats()
    ks, vs = (t.numpy for t in prog(keys, values))
    after = tf.dispatch_stats()
    assert after["fused_chains"] == before["fused_chains"]
    _check_sorted(keys, values, ks, vs, kind)
    prog.destroy()


def _composition_dispatches(flags, bits=6):
    """Dispatches of radix_sort_ir inside the region: the prologue copies and, per pass, the composition's kernels."""
    passes = (32 + bits - 1) // bits // 2 * 2
    return (1 if flags & 2 else 2) + passes * (7 + (1 if flags & 16 else 0) - (1 if flags & 8 else 0))


@pytest.mark.parametrize("kind", ["u32", "i32", "f32"])
@pytest.mark.parametrize("n,low_entropy", [(1, False), (127, False), (129, True), (8192 + 77, False), (1 << 20, False), (1 << 20, True)])
def test_the_radix_sort_region_is_served_by_one_onesweep_call(tf, n, low_entropy, kind):
    """The unchanged composition between region_begin('Radix sort') and region_end('Radix sort') (Python/TensorFrost/
    sort.py:74-176) is recognised and served by ONE call of the onesweep sort: 2 + 6 x 7 dispatches held, none launched,
    `fused_chains` counts one more; the result is what the 44 kernels leave (bit-exact, stable), the mapped-to-uint key
    buffer included, since the program's own un-map kernel runs on it afterwards."""
    keys = _sort_keys(kind, n, low_entropy)
    values = np.arange(n, dtype=np.uint32)[::-1].copy()  # any payload, not only the index
    prog = tf.compile("radix_sort_ir", [getattr(tf, _TYPES[kind])])
    before = tf.dispatch_stats()
    ks, vs = (t.numpy for t in prog(keys, values))
    after = tf.dispatch_stats()
    assert after["fused_chains"] == before["fused_chains"] + 1
    assert after["dispatches"] - before["dispatches"] == 45  # the composition's 44 + the un-map kernel after the region
    assert after["served_by_primitives"] - before["served_by_primitives"] == 44
    _check_sorted(keys, values, ks, vs, kind)
    # twice in a row on pooled buffers
    ks2, vs2 = (t.numpy for t in prog(keys, values))
    assert np.array_equal(ks2.view(np.uint32), ks.view(np.uint32)) and np.array_equal(vs2, vs)
    prog.destroy()


SORT_CUTS = [(2, "the two copies fused into one kernel"), (4, "the shift, not the pass index, as the kernels' scalar"),
             (8, "group_histogram never stored: unpacked inside the kernels that read it"), (16, "the digits of a pass as a tensor of their own"),
             (32, "separate kernels for the two SortIteration calls of a host-loop iteration"), (2 | 4 | 8 | 16 | 32, "all of these at once")]


@pytest.mark.parametrize("flags,what", SORT_CUTS, ids=[str(f) for f, _ in SORT_CUTS])
@pytest.mark.parametrize("kind,n,low_entropy", [("u32", 129, False), ("f32", 8192 + 77, False), ("u32", 1 << 20, False), ("i32", 1 << 20, True)])
def test_the_sort_region_is_served_however_the_passes_cut_it_into_kernels(tf, flags, what, kind, n, low_entropy):
    """Which operations of sort.py share a kernel is the compiler's decision (Compiler/Graph/Scope.cpp:5-35,165-188), and so
    is the form in which a host scalar reaches a kernel. The region is followed by its data flow and by what its kernels
    compute (copies, digit extraction, the scatter), so each of these other cuts of the same composition is served by the
    one onesweep call too -- and, with recognition switched off, still sorts when run kernel by kernel as emitted."""
    keys = _sort_keys(kind, n, low_entropy)
    values = np.arange(n, dtype=np.uint32)[::-1].copy()
    prog = tf.compile("radix_sort_ir", [getattr(tf, _TYPES[kind]), 6, flags])
    before = tf.dispatch_stats()
    ks, vs = (t.numpy for t in prog(keys, values))
    after = tf.dispatch_stats()
    held = _composition_dispatches(flags)
    assert after["fused_chains"] == before["fused_chains"] + 1, what
    assert after["dispatches"] - before["dispatches"] == held + 1
    assert after["served_by_primitives"] - before["served_by_primitives"] == held
    _check_sorted(keys, values, ks, vs, kind)
    prog.destroy()


@pytest.mark.parametrize("flags", [f for f, _ in SORT_CUTS])
def test_every_cut_of_the_sort_composition_sorts_as_emitted(tf, monkeypatch, flags):
    monkeypatch.setenv("TFHIP_NO_IDIOMS", "1")
    n = 40_000 + 13
    keys = _sort_keys("f32", n)
    values = np.arange(n, dtype=np.uint32)
    prog = tf.compile("radix_sort_ir", [tf.float32, 6, flags])
    before = tf.dispatch_stats()
    ks, vs = (t.numpy for t in prog(keys, values))
    assert tf.dispatch_stats()["fused_chains"] == before["fused_chains"]
    _check_sorted(keys, values, ks, vs, "f32")
    prog.destroy()


@pytest.mark.parametrize("bits", [8, 7, 4])
def test_other_digit_widths_that_cover_the_key_are_served_too(tf, bits):
    """sort.py's bits_per_pass is a parameter: any number of passes whose digits cover the 32 key bits gives the stable
    order of the whole key (7 bits: (32 + 6) // 7 = 5 iterations, of which the host loop runs 4 = 28 bits -- not served)."""
    n = 70_001
    keys = _sort_keys("u32", n)
    values = np.arange(n, dtype=np.uint32)
    prog = tf.compile("radix_sort_ir", [tf.uint32, bits])
    before = tf.dispatch_stats()
    ks, vs = (t.numpy for t in prog(keys, values))
    after = tf.dispatch_stats()
    passes = (32 + bits - 1) // bits // 2 * 2
    covered = passes * bits >= 32
    assert after["fused_chains"] == before["fused_chains"] + (1 if covered else 0)
    if covered:
        _check_sorted(keys, values, ks, vs, "u32")
    else:
        order = np.argsort(keys & np.uint32((1 << (passes * bits)) - 1), kind="stable")
        assert np.array_equal(ks, keys[order]) and np.array_equal(vs, values[order])
    prog.destroy()


@pytest.mark.parametrize("params,why", [([None, 6, 1], "one more dispatch inside the region: a copy sort.py does not make"),
                                        ([None, 5], "5-bit digits: 6 passes cover 30 bits only"),
                                        ([None, 6, 64], "a kernel of an iteration reads a buffer from outside the region"),
                                        ([None, 6, 128], "a buffer the skipped kernels would have written stays alive")])
def test_a_perturbed_sort_region_runs_as_dispatched(tf, params, why):
    """A `Radix sort` region whose data flow does not prove it to be the whole-key sort is not substituted: its kernels run
    as emitted, and the result is that composition's own (bit-exact against the oracle for the full-width variants)."""
    n = 50_000
    keys = _sort_keys("u32", n)
    values = np.arange(n, dtype=np.uint32)
    params = [tf.uint32] + params[1:]
    prog = tf.compile("radix_sort_ir", params)
    before = tf.dispatch_stats()
    outputs = [t.numpy for t in prog(keys, values)]
    ks, vs = outputs[0], outputs[1]
    after = tf.dispatch_stats()
    assert after["fused_chains"] == before["fused_chains"], why
    if params[1] == 5:
        # (32 + 4) // 5 = 7 iterations, 7 // 2 * 2 = 6 passes: stable order of the low 30 bits, as sort.py would give
        order = np.argsort(keys & np.uint32((1 << 30) - 1), kind="stable")
        assert np.array_equal(ks, keys[order]) and np.array_equal(vs, values[order])
    else:
        _check_sorted(keys, values, ks, vs, "u32")
    if len(outputs) == 3:
        # the kept tensor holds what the last pass's kernels wrote: inclusive counts of the top digit (6 bits of which 2 exist)
        top = keys >> np.uint32(30)
        assert np.array_equal(outputs[2][:4], np.cumsum(np.bincount(top, minlength=4)).astype(np.uint32))
    prog.destroy()


def test_precise_math_option_in_a_process_of_its_own():
    """`-DTF_PRECISE_MATH` in the backend options (a hiprtc option) selects IEEE division / square roots and the written
    order of float sums in emitted kernels. Backend options are per process, so a child process compiles and runs the
    N-body step (division by d2 * sqrt(d2), a reordered sum of squares) and the op table with it."""
    import subprocess
    import sys
    from pathlib import Path

    script = r"""
import sys
import numpy as np
sys.path.insert(0, sys.argv[1])
sys.path.insert(0, sys.argv[1] + "/tests")
import tensorfrost_amd.host as tf
from oracle import oracle
tf.initialize(tf.hip, "-DTF_PRECISE_MATH")
rng = np.random.default_rng(3)
n = 2048
x = rng.uniform(-1, 1, (n, 3)).astype(np.float32); v = (rng.normal(size=(n, 3)) * 0.01).astype(np.float32)
m = rng.lognormal(0, 0.5, n).astype(np.float32)
dt, eps = 1e-3, 1e-3
prog = tf.compile("nbody")
src = prog.kernels()[0]["source"]
assert "TF_REASSOC(" in src and "tf_div_by_pow_3_2(" in src
x_new, v_new = prog(x, v, m, np.array([dt], np.float32), np.array([eps], np.float32))
ox, ov = oracle.nbody_step(x, v, m, dt, eps)
dv_scale = np.abs(ov - v).max()
assert np.max(np.abs(v_new.numpy - ov)) < 1e-4 * dv_scale
a = rng.uniform(0.5, 4, 1000).astype(np.float32); b = rng.uniform(0.5, 4, 1000).astype(np.float32)
print("ok")
"""
    root = str(Path(__file__).resolve().parents[1])
    out = subprocess.run([sys.executable, "-c", script, root], capture_output=True, text=True, timeout=110)
    assert out.returncode == 0 and out.stdout.strip().endswith("ok"), out.stdout + out.stderr


def test_large_copies_survive_a_restart_of_the_backend(tf):
    """Copies of a megabyte and more are cut into slices that helper threads copy beside the caller; stopping the
    backend ends those threads and the next large copy starts new ones, which must serve that copy and no earlier
    one (a helper that began at request zero once copied a finished request's slice again, into memory long freed)."""
    rng = np.random.default_rng(99)
    for round_ in range(3):
        data = rng.integers(0, 2**32, (3 << 20) + 12345 * round_, dtype=np.uint64).astype(np.uint32)
        t = tf.tensor(data)
        assert np.array_equal(t.numpy, data)
        small = tf.tensor(data[:1000])
        assert np.array_equal(small.numpy, data[:1000])
        t.release()
        small.release()
        tf.initialize(tf.hip)  # stops the running backend (and the library under it) and starts both again
