#!/usr/bin/env python3
"""Benchmark of the MI355X backend's hot path on one GPU.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu] [--no-extras] [--no-graphs]

Workload (the second benchmark configuration, row reductions and softmax): X[16384, 4096] fp32 ~ U(-4, 4), seeded. One step = tf.sum, tf.max
and a fused softmax along the last axis, then tf.sum and tf.max along axis 0 -- five primitive calls
through the C ABI, inputs resident in HBM. `value` is algorithmic bytes per step / time per step.

Prints ONE JSON line. `roofline` is for the dominant kernel of the step (the fused softmax: 8 B per
element), timed with HIP events on the library's own stream inside the timed region; the other four
calls are timed the same way in a second pass (`kernels`), so that their events (about 3 us of stream
time each) do not stretch the step that `value` is computed from; `cpu_baseline` is the CPU oracle (a
restatement of the reference's generated OpenMP kernels) on the host cores of the same machine.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

import numpy as np

R, C = 16384, 4096
HBM_PEAK_GBS = 8000.0

# Algorithmic bytes per call: inputs read once, outputs written once.
BYTES = {
    "sum_rows": 4 * R * C + 4 * R,
    "max_rows": 4 * R * C + 4 * R,
    "softmax_rows": 8 * R * C,
    "sum_cols": 4 * R * C + 4 * C,
    "max_cols": 4 * R * C + 4 * C,
}
STEP_BYTES = sum(BYTES.values())


def softmax_traffic_bytes():
    """HBM bytes one launch of the softmax kernel moves, from the committed counter summary (FETCH_SIZE and WRITE_SIZE
    of `python bench.py --pmc-probe`, scaled by the same counters of a plain copy of known size)."""
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "profiles", "config2_softmax_hbm_traffic.json")
    try:
        with open(path) as f:
            return int(json.load(f)["softmax_rows_block_kernel<512, 2>"]["traffic_bytes_per_launch"])
    except (OSError, KeyError, ValueError):
        return None


def make_input() -> np.ndarray:
    rng = np.random.default_rng(1234 + 2)
    return rng.uniform(-4.0, 4.0, (R, C)).astype(np.float32)


N_SETS = 8  # copies of X (and half as many outputs) that the calls rotate over: 2 GiB + 1 GiB, eight times the last-level cache


def _timed_steps(rt, calls_of_step, steps: int, dominant: int):
    """K steps between two synchronisations, host clock. Inside the region only the dominant kernel (the softmax) is
    bracketed by events on the library's stream; an event costs about 3 us of stream time, so bracketing all five
    calls would add 7 % to the step being measured. Returns (ms per step, ms per dominant call)."""
    events = [(rt.Event(), rt.Event()) for _ in range(steps)]
    rt.synchronize()
    t0 = time.perf_counter()
    for s in range(steps):
        for i, fn in enumerate(calls_of_step(s)):
            if i == dominant:
                events[s][0].record()
                fn()
                events[s][1].record()
            else:
                fn()
    rt.synchronize()
    t1 = time.perf_counter()
    return (t1 - t0) * 1e3 / steps, sum(a.elapsed_ms(b) for a, b in events) / steps


def _per_call_ms(rt, calls_of_step, names, steps: int) -> dict:
    """Per-call durations of all five, from a separate pass of K steps with an event before every call."""
    events = [[rt.Event() for _ in range(len(names) + 1)] for _ in range(steps)]
    for s in range(steps):
        for i, fn in enumerate(calls_of_step(s)):
            events[s][i].record()
            fn()
        events[s][len(names)].record()
    rt.synchronize()
    out = {name: 0.0 for name in names}
    for s in range(steps):
        for i, name in enumerate(names):
            out[name] += events[s][i].elapsed_ms(events[s][i + 1])
    return {k: v / steps for k, v in out.items()}


def gpu_leg(x: np.ndarray, steps: int, warmup: int) -> dict:
    """Two timings of the same step. The headline (`value`, `roofline`) comes from the run in which every call reads a
    copy of X that no call has touched for the last 2 GiB of traffic, so nothing can be served by the 256 MiB last-level
    cache: call j of step s reads copy (5 s + j) mod 8 and the softmax writes output (s mod 4). The run on ONE copy of X,
    in which X (exactly the size of that cache) is read by five calls in a row, is reported beside it as `llc_assisted`."""
    from tensorfrost_amd import runtime as rt
    from tensorfrost_amd._lib import call

    rt.initialize(0)
    xs = [rt.DeviceBuffer.from_numpy(x)]
    for _ in range(N_SETS - 1):
        b = rt.DeviceBuffer(R * C)
        call("tfhip_d2d", b.ptr, xs[0].ptr, R * C)
        xs.append(b)
    ys = [rt.DeviceBuffer(R * C) for _ in range(N_SETS // 2)]
    row = rt.DeviceBuffer(R)
    col = rt.DeviceBuffer(C)
    names = ["sum_rows", "max_rows", "softmax_rows", "sum_cols", "max_cols"]
    dominant = names.index("softmax_rows")

    def calls_on(xb, yb):
        return [
            lambda: rt.reduce_rows("sum", xb, row, R, C),
            lambda: rt.reduce_rows("max", xb, row, R, C),
            lambda: rt.softmax_rows(xb, yb, R, C),
            lambda: rt.reduce_cols("sum", xb, col, R, C),
            lambda: rt.reduce_cols("max", xb, col, R, C),
        ]

    per_set = [[calls_on(xb, yb) for yb in ys] for xb in xs]

    def rotating(s):  # every call on the copy of X that was touched longest ago
        return [per_set[(5 * s + j) % N_SETS][s % len(ys)][j] for j in range(5)]

    def resident(s):  # one X, one Y: the input stays in the last-level cache from call to call
        return per_set[0][0]

    result = {}
    for mode, calls_of_step in (("hbm", rotating), ("llc_assisted", resident)):
        for s in range(warmup):
            for fn in calls_of_step(s):
                fn()
        rt.synchronize()
        ms_step, ms_dominant = _timed_steps(rt, calls_of_step, steps, dominant)
        per_call = _per_call_ms(rt, calls_of_step, names, steps)
        per_call["softmax_rows"] = ms_dominant  # the figure from the timed region
        result[mode] = {"ms_per_step": ms_step, "per_call_ms": per_call}

    # quick self-check so that a broken kernel cannot post a number: every output buffer, a few rows each
    e = np.exp(x[:4].astype(np.float64) - x[:4].max(axis=1, keepdims=True))
    for yb in ys:
        y0 = yb.numpy(np.float32, (4, C), offset_words=0)
        if not np.allclose(y0, e / e.sum(axis=1, keepdims=True), rtol=1e-4, atol=1e-9):
            raise RuntimeError("softmax self-check failed; refusing to report a throughput")
    for b in xs[1:] + ys[1:]:
        b.free()

    result["device"] = rt.device_info()
    return result


def cpu_leg(x: np.ndarray) -> dict:
    """Times the CPU oracle on the same step (the whole matrix: a step takes the host cores well under a second),
    as bytes/s of the same algorithmic bytes."""
    from oracle import oracle

    oracle.load()
    threads = int(os.environ.get("OMP_NUM_THREADS", "0")) or (os.cpu_count() or 1)
    rows = R
    xs = np.ascontiguousarray(x[:rows])
    sample_bytes = (2 * (4 * rows * C + 4 * rows) + 8 * rows * C + 2 * (4 * rows * C + 4 * C))

    def step():
        oracle.reduce_rows("sum", xs)
        oracle.reduce_rows("max", xs)
        oracle.softmax_rows(xs)
        oracle.reduce_cols("sum", xs)
        oracle.reduce_cols("max", xs)

    step()  # warm-up: page in, spin up the OpenMP team
    t0 = time.perf_counter()
    step()
    one = time.perf_counter() - t0
    reps = int(max(1, min(20, 15.0 / max(one, 1e-3))))
    times = []
    for _ in range(reps):
        t0 = time.perf_counter()
        step()
        times.append(time.perf_counter() - t0)
    med = float(np.median(times))
    return {
        "parity_vs_gpu": parity_on_sample(xs, oracle),
        "value": round(sample_bytes / med / 1e9, 3),
        "unit": "GB/s",
        "cores": threads,
        "kind": "port",
        "sample": f"the same five calls on the whole matrix ([{rows},{C}] fp32), median of {reps} runs after one warm-up, "
                  f"g++ -O3 -ffast-math -fopenmp restatement of the reference's generated kernels",
    }


def parity_on_sample(xs: np.ndarray, oracle) -> dict:
    """The five calls on the GPU and in the CPU oracle on the same sample, in the same run: sums against the sum of
    magnitudes (tolerance 1e-4), softmax element-wise relative (1e-5), maxima exact."""
    from tensorfrost_amd import runtime as rt

    rows, cols = xs.shape
    xb = rt.DeviceBuffer.from_numpy(xs)
    yb, row, col = rt.DeviceBuffer(xs.size), rt.DeviceBuffer(rows), rt.DeviceBuffer(cols)
    out = {}
    mag = np.abs(xs).astype(np.float64)
    rt.reduce_rows("sum", xb, row, rows, cols)
    out["sum_rows_err_over_sum_of_magnitudes"] = float(np.max(np.abs(row.numpy(np.float32) - oracle.reduce_rows("sum", xs)) / mag.sum(axis=1)))
    rt.reduce_rows("max", xb, row, rows, cols)
    out["max_rows_exact"] = bool(np.array_equal(row.numpy(np.float32), oracle.reduce_rows("max", xs)))
    rt.softmax_rows(xb, yb, rows, cols)
    ref = oracle.softmax_rows(xs)
    out["softmax_rows_max_rel_err"] = float(np.max(np.abs(yb.numpy(np.float32, xs.shape) - ref) / np.maximum(np.abs(ref), 1e-6 * np.abs(ref).max())))
    rt.reduce_cols("sum", xb, col, rows, cols)
    out["sum_cols_err_over_sum_of_magnitudes"] = float(np.max(np.abs(col.numpy(np.float32) - oracle.reduce_cols("sum", xs)) / mag.sum(axis=0)))
    rt.reduce_cols("max", xb, col, rows, cols)
    out["max_cols_exact"] = bool(np.array_equal(col.numpy(np.float32), oracle.reduce_cols("max", xs)))
    ok = (out["sum_rows_err_over_sum_of_magnitudes"] < 1e-4 and out["sum_cols_err_over_sum_of_magnitudes"] < 1e-4 and out["softmax_rows_max_rel_err"] < 1e-5
          and out["max_rows_exact"] and out["max_cols_exact"])
    if not ok:
        raise RuntimeError(f"GPU and CPU oracle disagree on the sample: {out}")
    return {k: (v if isinstance(v, bool) else float(f"{v:.3g}")) for k, v in out.items()}


def cpu_others_leg() -> dict:
    """The CPU oracle on bounded samples of the other configs (one warm-up, median of up to three runs each)."""
    from oracle import oracle

    def timed(fn):
        fn()
        times = []
        for _ in range(3):
            t0 = time.perf_counter()
            fn()
            times.append(time.perf_counter() - t0)
            if sum(times) > 6.0:
                break
        return float(np.median(times))

    out = {}
    rng = np.random.default_rng(7)
    n = 1 << 20
    keys, vals = rng.integers(0, 2**32, n, dtype=np.uint32), np.arange(n, dtype=np.uint32)
    t = timed(lambda: oracle.radix_sort_kv(keys, vals))
    out["radix_sort_kv_u32"] = {"value": round(n / t / 1e9, 4), "unit": "Gkeys/s", "sample": "2^20 uniform keys + payload, the reference's 6 x 6-bit histogram sort"}
    u = oracle.sine_gordon_initial_field(2048, 2048)
    v = np.zeros_like(u)
    t = timed(lambda: oracle.wave_eq(u, v, 0.1, 10)) / 10
    out["sine_gordon_2048x2048"] = {"value": round(16 * 2048 * 2048 / t / 1e9, 2), "unit": "GB/s", "sample": "10 steps of the full grid"}
    x, vel, mass = oracle.nbody_inputs(8192)
    t = timed(lambda: oracle.nbody_step(x, vel, mass, np.float32(1e-3), np.float32(1e-3)))
    out["nbody"] = {"value": round(20.0 * 8192 * 8192 / t / 1e12, 4), "unit": "TFLOP/s", "sample": "N = 8192 (1/64 of the pair interactions)"}
    a = rng.normal(size=(4096, 256)).astype(np.float32)
    b = rng.normal(size=(256, 256)).astype(np.float32)
    t = timed(lambda: oracle.matmul(a, b))
    out["sgemm_nn"] = {"value": round(2.0 * 4096 * 256 * 256 / t / 1e12, 4), "unit": "TFLOP/s", "sample": "[4096,256] x [256,256] (1/64 of the rows)"}
    coords, target, params, m, vv = oracle.mlp_inputs(4096)
    t = timed(lambda: oracle.mlp_step(coords, target, params, m, vv, t=0.0))
    out["mlp_step"] = {"value": round(t * 1e3 * 64, 1), "unit": "ms per 262144-sample step (scaled from the sample)", "sample": "batch 4096 (1/64 of the batch)"}
    return out


def _time_events(rt, fn, reps: int, warm: int = 2, warm_ms: float = 0.0) -> float:
    """Average milliseconds per call of fn, from events on the library's stream. warm_ms: keep the GPU busy with fn for
    at least that long first (compute-bound kernels reach their steady clock only after some hundred milliseconds of
    load: the 256-wide sgemm runs at 100 TFLOP/s in its first 10 ms and at 117-120 from 100 ms on)."""
    for _ in range(warm):
        fn()
    rt.synchronize()
    if warm_ms > 0:
        t_end = time.perf_counter() + warm_ms * 1e-3
        while time.perf_counter() < t_end:
            for _ in range(10):
                fn()
            rt.synchronize()
    e0, e1 = rt.Event(), rt.Event()
    e0.record()
    for _ in range(reps):
        fn()
    e1.record()
    return e0.elapsed_ms(e1) / reps


def _mlp_float64(features: np.ndarray, target: np.ndarray, params) -> tuple:
    """The benchmark MLP's loss and gradients at the full batch in float64 (textbook forward and backward of four dense
    layers with ReLU and a mean-squared error), from the float32 Fourier features."""
    w = [p.astype(np.float64) for p in params]
    acts = [features.astype(np.float64)]
    for l in range(3):
        acts.append(np.maximum(acts[-1] @ w[2 * l] + w[2 * l + 1], 0.0))
    y = acts[-1] @ w[6] + w[7]
    diff = y - target
    loss = float(np.mean(diff * diff))
    up = diff * (2.0 / diff.size)
    grads = [None] * 8
    for l in range(3, -1, -1):
        grads[2 * l] = acts[l].T @ up
        grads[2 * l + 1] = up.sum(0)
        if l > 0:
            up = (up @ w[2 * l].T) * (acts[l] > 0)
    return loss, grads


def _check_mlp(prog, ins, want, label: str) -> None:
    """One more step on the timed inputs (zero moments, t = 0: the first moments it returns are (1 - beta1) times the
    gradients), compared with the float64 evaluation at the matmul / reduction bar of 1e-4 of each tensor's magnitude."""
    outs = prog(*ins)
    loss = float(outs[0].numpy[0])
    grads = [outs[9 + i].numpy.astype(np.float64) / (1.0 - 0.9) for i in range(8)]
    for o in outs:
        o.release()
    want_loss, want_grads = want
    bad = [i for i in range(8) if np.max(np.abs(grads[i] - want_grads[i])) > 1e-4 * np.max(np.abs(want_grads[i]))]
    if abs(loss - want_loss) > 1e-4 * abs(want_loss) or bad:
        raise RuntimeError(f"{label}: self-check against the float64 evaluation failed (loss {loss} vs {want_loss}, gradients {bad}); refusing to report a throughput")


def extras_leg(graphs: bool = True) -> dict:
    """The other benchmark configs, each at its full size, as secondary numbers (same process, after the
    timed region of the headline metric)."""
    from tensorfrost_amd import runtime as rt
    import tensorfrost_amd.host as tf
    from oracle import oracle as orc  # input generators only; nothing below is computed by the oracle

    out = {}
    # config 3: key/value radix sort, 2^28 uint32 keys + uint32 payload, uniform and low-entropy keys
    n = 1 << 28
    rng = np.random.default_rng(1234 + 3)
    vb = rt.DeviceBuffer.from_numpy(np.arange(n, dtype=np.uint32))
    ko, vo, kt, vt = (rt.DeviceBuffer(n) for _ in range(4))
    for dist, hi in (("uniform", 2 ** 32), ("low_entropy", 1024)):
        keys_np = rng.integers(0, hi, n, dtype=np.uint32)
        kb = rt.DeviceBuffer.from_numpy(keys_np)
        ms = _time_events(rt, lambda: rt.radix_sort_kv(kb, vb, ko, vo, n, np.uint32, keys_tmp=kt, vals_tmp=vt), reps=5, warm=1)
        # the whole result: ascending, every payload still points at its key, equal keys in their original order
        # (the payload is the original index, so key and payload together must ascend strictly)
        ks, vs = ko.numpy(np.uint32, (n,)), vo.numpy(np.uint32, (n,))
        if not (np.all(ks[1:] >= ks[:-1]) and np.array_equal(keys_np[vs], ks) and np.all((ks[1:] > ks[:-1]) | (vs[1:] > vs[:-1]))):
            raise RuntimeError(f"radix sort ({dist}): self-check of the whole result failed; refusing to report a throughput")
        del ks, vs, keys_np
        out[f"radix_sort_kv_u32_2^28_{dist}"] = {"ms": round(ms, 3), "Gkeys/s": round(n / ms / 1e6, 2), "GB/s_at_68B_per_key": round(68 * n / ms / 1e6, 1)}
        kb.free()
    # prefix sums over the same 2^28 elements, reusing two of the buffers (u32: one-pass chained scan, 8 B per
    # element; f32: tile sums + scan of sums + rescan, 12 B per element, reproducible summation order)
    ko.fill(1)
    ms = _time_events(rt, lambda: rt.scan_inclusive(ko, vo, n, np.uint32), reps=5, warm=1)
    if vo.numpy(np.uint32, (4,), offset_words=n - 4).tolist() != [n - 3, n - 2, n - 1, n]:
        raise RuntimeError("scan self-check failed")
    out["scan_u32_2^28"] = {"ms": round(ms, 3), "GB/s_at_8B_per_element": round(8 * n / ms / 1e6, 1), "frac_of_hbm_peak": round(8 * n / ms / 1e6 / HBM_PEAK_GBS, 3)}
    ko.fill(0x3F800000)
    ms = _time_events(rt, lambda: rt.scan_inclusive(ko, vo, n, np.float32), reps=5, warm=1)
    # ones: element i must hold i + 1 to the reduction bar (in fact to one rounding: tile offsets are exact multiples of the tile)
    got = vo.numpy(np.float32, (n,)).astype(np.float64)
    want = np.arange(1, n + 1, dtype=np.float64)
    if not np.all(np.abs(got - want) <= 1e-6 * want):
        raise RuntimeError("scan (f32): self-check of the whole result failed; refusing to report a throughput")
    del got, want
    out["scan_f32_2^28"] = {"ms": round(ms, 3), "GB/s_at_12B_per_element": round(12 * n / ms / 1e6, 1), "frac_of_hbm_peak": round(12 * n / ms / 1e6 / HBM_PEAK_GBS, 3)}
    for b in (vb, ko, vo, kt, vt):
        b.free()

    # tf.matmul on the config-5 hidden-layer shape and a large square
    # Operands matter: constant fills toggle few bits, draw less power and run several percent faster than random
    # data. The hidden-layer shape gets what that layer sees in config 5 -- activations after a ReLU (half zeros) and
    # He-normal weights N(0, 2/fan_in) -- the square gets standard normal operands.
    rng_g = np.random.default_rng(1234 + 5)
    for (m, nn, k) in ((262144, 256, 256), (8192, 8192, 8192)):
        an = rng_g.standard_normal((m, k), dtype=np.float32)
        bn = rng_g.standard_normal((k, nn), dtype=np.float32)
        if m == 262144:
            np.maximum(an, 0.0, out=an)
            bn *= np.float32(np.sqrt(2.0 / k))
        a = rt.DeviceBuffer.from_numpy(an)
        b = rt.DeviceBuffer.from_numpy(bn)
        c = rt.DeviceBuffer(m * nn)
        ms = _time_events(rt, lambda: rt.sgemm("nn", a, b, c, m, nn, k), reps=20, warm=5, warm_ms=300)
        # sampled rows of the product against float64, at the matmul bar of 1e-4 of the row's largest magnitude
        for row in sorted({0, 1, m // 3, m // 2 + 77, m - 129, m - 1}):
            got_row = c.numpy(np.float32, (nn,), offset_words=row * nn).astype(np.float64)
            want_row = an[row].astype(np.float64) @ bn.astype(np.float64)
            if not np.max(np.abs(got_row - want_row)) <= 1e-4 * np.max(np.abs(want_row)):
                raise RuntimeError(f"sgemm {m}x{nn}x{k}: row {row} differs from the float64 product; refusing to report a throughput")
        tfl = 2.0 * m * nn * k / ms / 1e9
        out[f"sgemm_nn_{m}x{nn}x{k}"] = {"ms": round(ms, 4), "TFLOP/s": round(tfl, 1), "frac_of_fp32_mfma_peak_157.3": round(tfl / 157.3, 3),
                                          "operands": "relu(N(0,1)) x N(0,2/K)" if m == 262144 else "N(0,1) x N(0,1)"}
        for x in (a, b, c):
            x.free()

    tf.initialize(tf.hip)
    # config 1: 2048^2 sine-Gordon, 1000 steps through the host path (pool, dispatch, emitted kernel)
    u0 = orc.sine_gordon_initial_field(2048, 2048)
    prog = tf.compile("wave_eq")
    state = [tf.tensor(u0), tf.tensor(np.zeros_like(u0))]

    def wave_steps(steps):
        for _ in range(steps):
            v2, u2 = prog(state[0], state[1])
            state[0].release()
            state[1].release()
            state[0], state[1] = u2, v2

    # one repetition = 1000 steps; one untimed repetition, then the median of 10 (the first thousands of
    # launches run a few percent slower than the steady state)
    wave_steps(1000)
    tf.synchronize()
    reps = []
    for _ in range(10):
        e0, e1 = rt.Event(), rt.Event()
        e0.record()
        wave_steps(1000)
        e1.record()
        reps.append(e0.elapsed_ms(e1))  # ms per 1000 steps == us per step
    ms = float(np.median(reps))
    out["sine_gordon_2048x2048_1000_steps"] = {"us_per_step": round(ms, 3), "us_per_step_min_max_of_10_reps": [round(min(reps), 3), round(max(reps), 3)],
                                                "GB/s_at_16B_per_cell": round(16 * 2048 * 2048 * 1000 / ms / 1e6, 1),
                                                "frac_of_hbm_peak": round(16 * 2048 * 2048 * 1000 / ms / 1e6 / HBM_PEAK_GBS, 3)}
    # the same step on an 8192^2 grid: 1 GiB of state per step (u, v read; u, v written), four times the last-level cache,
    # so this one is an HBM figure, while the 2048^2 set (64 MiB) above stays resident in that cache
    big = np.random.default_rng(1).standard_normal((8192, 8192), dtype=np.float32)
    for t in state:
        t.release()
    state[:] = [tf.tensor(big), tf.tensor(np.zeros_like(big))]
    del big
    wave_steps(20)
    tf.synchronize()
    reps = []
    for _ in range(5):
        e0, e1 = rt.Event(), rt.Event()
        e0.record()
        wave_steps(100)
        e1.record()
        reps.append(e0.elapsed_ms(e1) * 10.0)  # ms per 100 steps -> us per step
    us = float(np.median(reps))
    out["sine_gordon_8192x8192_beyond_the_last_level_cache"] = {"us_per_step": round(us, 2), "GB/s_at_16B_per_cell": round(16 * 8192 * 8192 / us / 1e3, 1),
                                                                "frac_of_hbm_peak": round(16 * 8192 * 8192 / us / 1e3 / HBM_PEAK_GBS, 3)}
    out["sine_gordon_2048x2048_1000_steps"]["note"] = "64 MiB working set: resident in the 256 MiB last-level cache, not an HBM figure"
    # the same iteration on a 512^2 grid, where the kernel is shorter than the host work of one dispatch: issued call by
    # call through the host path, and as ten replays of a recorded graph of 100 steps (outputs fed back to the inputs)
    small = orc.sine_gordon_initial_field(512, 512)
    for t in state:
        t.release()
    state[:] = [tf.tensor(small), tf.tensor(np.zeros_like(small))]
    wave_steps(1000)
    tf.synchronize()
    e0, e1 = rt.Event(), rt.Event()
    e0.record()
    wave_steps(1000)
    e1.record()
    eager_us = e0.elapsed_ms(e1)
    out["sine_gordon_512x512_1000_steps"] = {"us_per_step_call_by_call": round(eager_us, 3)}
    if graphs:
        graph = prog.record(state[0], state[1], repeat=100, feedback=(1, 0))
        graph.replay()
        tf.synchronize()
        e0, e1 = rt.Event(), rt.Event()
        e0.record()
        for _ in range(10):
            graph.replay()
        e1.record()
        out["sine_gordon_512x512_1000_steps"]["us_per_step_recorded_graph_of_100_steps"] = round(e0.elapsed_ms(e1), 3)
        graph.destroy()
    prog.destroy()

    # the reference's hand-tiled matrix product example (group buffers, barriers, 4x4 results per thread) as an emitted
    # user kernel, at the example's own size 4096^3 (its notebook prints 8.74 TFLOP/s for the run kept there)
    tiled = tf.compile("tiled_matmul_ir")
    rng_t = np.random.default_rng(7)
    ta, tb = tf.tensor(rng_t.random((4096, 4096), dtype=np.float32)), tf.tensor(rng_t.random((4096, 4096), dtype=np.float32))

    def tiled_step():
        tiled(ta, tb).release()

    ms = _time_events(rt, tiled_step, reps=10, warm=3, warm_ms=200)
    out["tiled_matmul_example_4096^3_emitted_user_kernel"] = {"ms": round(ms, 3), "TFLOP/s": round(2 * 4096**3 / ms / 1e9, 1),
                                                              "frac_of_fp32_valu_peak_78.6": round(2 * 4096**3 / ms / 1e9 / 78.6, 3)}
    for t in (ta, tb):
        t.release()
    tiled.destroy()

    # config 2 once more, this time as the reference's passes hand it to a backend: eight kernels in lowered IR form
    # (128-chunk split reductions behind the dim_split view), recognised and served by the reductions of libtfhip;
    # and the same program with the recognition switched off, i.e. the emitter's own kernels
    xr = tf.tensor(make_input())
    prog = tf.compile("reductions_ir")

    def reductions_step():
        for o in prog(xr):
            o.release()

    four_calls = BYTES["sum_rows"] + BYTES["max_rows"] + BYTES["sum_cols"] + BYTES["max_cols"]
    ms = _time_events(rt, reductions_step, reps=20, warm=20)  # the upload of X leaves the GPU idle: reach the steady state first
    out["config2_sum_max_both_axes_from_lowered_ir"] = {"ms": round(ms, 4), "GB/s": round(four_calls / ms / 1e6, 1), "frac_of_hbm_peak": round(four_calls / ms / 1e6 / HBM_PEAK_GBS, 3)}
    os.environ["TFHIP_NO_IDIOMS"] = "1"
    ms = _time_events(rt, reductions_step, reps=20, warm=3)
    del os.environ["TFHIP_NO_IDIOMS"]
    out["config2_sum_max_both_axes_emitted_kernels_only"] = {"ms": round(ms, 4), "GB/s": round(four_calls / ms / 1e6, 1), "frac_of_hbm_peak": round(four_calls / ms / 1e6 / HBM_PEAK_GBS, 3)}
    prog.destroy()
    # the softmax of the same config as the reference composes it: five lowered kernels. The kernel manager recognises the
    # sequence and runs the fused primitive once (one read); with that switched off the kernels run as dispatched (three reads)
    sm = tf.compile("softmax_ir")

    def softmax_step():
        sm(xr).release()

    def softmax_entry(ms):
        return {"ms": round(ms, 4), "GB/s_at_8B_per_element": round(BYTES["softmax_rows"] / ms / 1e6, 1),
                "frac_of_hbm_peak": round(BYTES["softmax_rows"] / ms / 1e6 / HBM_PEAK_GBS, 3)}

    chains = tf.dispatch_stats()["fused_chains"]
    out["config2_softmax_from_lowered_ir_recognised_as_one_softmax"] = softmax_entry(_time_events(rt, softmax_step, reps=20, warm=10))
    assert tf.dispatch_stats()["fused_chains"] - chains == 30, "the lowered softmax was not served as one chain"
    os.environ["TFHIP_NO_IDIOMS"] = "1"
    out["config2_softmax_from_lowered_ir_five_emitted_kernels"] = softmax_entry(_time_events(rt, softmax_step, reps=20, warm=10))
    del os.environ["TFHIP_NO_IDIOMS"]
    sm.destroy()
    # log_softmax(X) = (X - max) - log(sum(exp(X - max))), as the reference's tests compose it: recognised like the softmax
    # and served by the fused log-softmax (one read, one write)
    sm = tf.compile("softmax_ir", [8])
    out["config2_log_softmax_from_lowered_ir"] = softmax_entry(_time_events(rt, softmax_step, reps=20, warm=10))
    os.environ["TFHIP_NO_IDIOMS"] = "1"
    out["config2_log_softmax_from_lowered_ir_five_emitted_kernels"] = softmax_entry(_time_events(rt, softmax_step, reps=20, warm=10))
    del os.environ["TFHIP_NO_IDIOMS"]
    sm.destroy()
    # a last kernel that is neither (the log-softmax scaled, as a fused cross-entropy term): the four reduction dispatches
    # held back are served by one statistics-only call (one read) and the last kernel runs as emitted (a second read, one write)
    sm = tf.compile("softmax_ir", [8 | 16])
    out["config2_scaled_log_softmax_from_lowered_ir_statistics_in_one_read"] = softmax_entry(_time_events(rt, softmax_step, reps=20, warm=10))
    sm.destroy()
    xr.release()

    # reductions that are none of the fixed primitives, as the emitter runs them (the reference's reshape_reduction_test
    # and integer dim_sum / dim_max / dim_min in lowered form; the programs live with the test suite's programs): five
    # row statistics fused into one loop that a wave shares, a total over the row results, the mean over axis 0 as a loop
    # down the columns shared by the waves of a group and by several groups; four integer reductions of two tensors
    test_programs = os.path.join(os.path.dirname(os.path.abspath(__file__)), "tests", "programs", "libtftestprograms.so")
    if os.path.exists(test_programs):
        tf.load_programs(test_programs)
        rng_r = np.random.default_rng(1234 + 6)
        a4 = rng_r.random((16384, 16, 16, 16), dtype=np.float32) - np.float32(0.25)
        rr = tf.compile("reshape_reduction")
        ta4 = tf.tensor(a4)

        def rr_step():
            for o in rr(ta4):
                o.release()

        ms = _time_events(rt, rr_step, reps=20, warm=5)
        out["reshape_reduction_16384x4096_five_row_statistics_totals_and_column_mean_emitted"] = {
            "ms": round(ms, 4), "kernels": 3, "GB/s_at_two_reads_of_the_input": round(2 * a4.nbytes / ms / 1e6, 1),
            "frac_of_hbm_peak": round(2 * a4.nbytes / ms / 1e6 / HBM_PEAK_GBS, 3)}
        ta4.release()
        rr.destroy()
        del a4
        ir = tf.compile("integer_reductions")
        u2 = rng_r.integers(0, 2 ** 32, (16384, 4096), dtype=np.uint64).astype(np.uint32)
        i2 = rng_r.integers(-2 ** 31, 2 ** 31, (16384, 4096), dtype=np.int64).astype(np.int32)
        tu2, ti2 = tf.tensor(u2), tf.tensor(i2)

        def ir_step():
            for o in ir(tu2, ti2):
                o.release()

        ms = _time_events(rt, ir_step, reps=20, warm=5)
        out["integer_reductions_16384x4096_sum_max_u32_sum_min_i32_emitted"] = {
            "ms": round(ms, 4), "kernels": 1, "GB/s_at_one_read_of_each_input": round((u2.nbytes + i2.nbytes) / ms / 1e6, 1),
            "frac_of_hbm_peak": round((u2.nbytes + i2.nbytes) / ms / 1e6 / HBM_PEAK_GBS, 3)}
        tu2.release()
        ti2.release()
        ir.destroy()
        del u2, i2

    # config 3 once more, as an unchanged TensorFrost program reaches this backend: the reference's own composition of
    # tf.sort.radix (six 6-bit passes of seven kernels between region_begin / region_end 'Radix sort'), dispatched
    # kernel by kernel through the host path. The kernel manager recognises the region and serves it with one onesweep
    # call; with recognition switched off every kernel runs as emitted. `radix_sort` is the program that names the primitive.
    sort_rng = np.random.default_rng(1234 + 3)
    for log_n in (24, 28):
        n_keys = 1 << log_n
        host_keys = sort_rng.integers(0, 2 ** 32, n_keys, dtype=np.uint64).astype(np.uint32)
        keys_t = tf.tensor(host_keys)
        vals_t = tf.tensor(np.arange(n_keys, dtype=np.uint32))
        # (program, parameters, run as emitted, tag). The second and third entries are the same composition cut into kernels in
        # other ways the compiler's passes may choose (the two copies fused; every cut at once: shift as the kernels'
        # scalar, the group histogram never stored, the digits a tensor of their own, separate kernels per SortIteration call)
        variants = [("radix_sort_ir", [], False, "reference_composition"),
                    ("radix_sort_ir", [1, 6, 2], False, "reference_composition_copies_fused"),
                    ("radix_sort_ir", [1, 6, 2 | 4 | 8 | 16 | 32], False, "reference_composition_every_other_cut"),
                    ("radix_sort", [], False, "onesweep_through_host_path")]
        if log_n == 24:
            variants.insert(1, ("radix_sort_ir", [], True, "reference_composition_emitted"))
        for name, prog_params, emitted, tag in variants:
            prog = tf.compile(name, prog_params) if prog_params else tf.compile(name)
            last = []

            def sort_step():
                for o in last:
                    o.release()
                last[:] = prog(keys_t, vals_t)

            if emitted:
                os.environ["TFHIP_NO_IDIOMS"] = "1"
            chains = tf.dispatch_stats()["fused_chains"]
            ms = _time_events(rt, sort_step, reps=3, warm=2)
            if emitted:
                del os.environ["TFHIP_NO_IDIOMS"]
            served = tf.dispatch_stats()["fused_chains"] - chains
            if name == "radix_sort_ir" and served != (0 if emitted else 5):
                raise RuntimeError(f"the 'Radix sort' region was served by the onesweep sort {served} times out of 5")
            # self-check on the whole result of the last call: ascending, every payload points at its key, equal keys in
            # their original order (the payload is the original index)
            got_k = last[0].numpy
            got_v = last[1].numpy
            if not (np.all(got_k[1:] >= got_k[:-1]) and np.array_equal(host_keys[got_v], got_k) and np.all((got_k[1:] > got_k[:-1]) | (got_v[1:] > got_v[:-1]))):
                raise RuntimeError(f"sort self-check failed ({name} {prog_params}, 2^{log_n}); refusing to report a throughput")
            del got_k, got_v
            for o in last:
                o.release()
            out[f"radix_sort_kv_u32_2^{log_n}_{tag}"] = {"ms": round(ms, 3), "Gkeys/s": round(n_keys / ms / 1e6, 2)}
            prog.destroy()
        keys_t.release()
        vals_t.release()
        del host_keys

    # config 4: all-pairs N-body, N = 65536
    x, v, mass = orc.nbody_inputs(65536)
    prog = tf.compile("nbody")
    X, V, M = tf.tensor(x), tf.tensor(v), tf.tensor(mass)
    dt, eps = tf.tensor(np.array([1e-3], np.float32)), tf.tensor(np.array([1e-3], np.float32))

    def nbody_step():
        a, b = prog(X, V, M, dt, eps)
        a.release()
        b.release()

    ms = _time_events(rt, nbody_step, reps=10, warm=5, warm_ms=200)
    # self-check on the timed shape: 64 bodies against a float64 direct sum over all 65536, tolerance 1e-4 of the sum of
    # magnitudes of the force terms (the bar of a 65536-term fp32 sum)
    x_new, v_new = prog(X, V, M, dt, eps)
    got_v = v_new.numpy
    x_new.release()
    v_new.release()
    probe = np.random.default_rng(3).choice(65536, 64, replace=False)
    d = x.astype(np.float64)[None, :, :] - x.astype(np.float64)[probe, None, :]
    d2 = (d * d).sum(-1) + 1e-3 ** 2
    w = mass.astype(np.float64)[None, :] / (d2 * np.sqrt(d2))
    acc = (w[:, :, None] * d).sum(1)
    scale = (w[:, :, None] * np.abs(d)).sum(1)
    if not np.all(np.abs(got_v[probe] - (v[probe] + acc * 1e-3)) <= 1e-4 * scale * 1e-3 + 1e-6 * np.abs(v[probe])):
        raise RuntimeError("N-body self-check failed; refusing to report a throughput")
    tfl = 20.0 * 65536 * 65536 / ms / 1e9
    out["nbody_65536"] = {"ms_per_step": round(ms, 3), "TFLOP/s_at_20_flop_per_pair": round(tfl, 2), "frac_of_fp32_valu_peak_78.6": round(tfl / 78.6, 3)}
    prog.destroy()

    # config 5: coordinate-MLP training step, batch 262144
    B = 262144
    coords, target, params, m_, v_ = orc.mlp_inputs(B)
    prog = tf.compile("mlp")
    ins = [tf.tensor(a) for a in [coords, target] + params + m_ + v_ + [np.zeros(1, np.float32)]]

    def mlp_step():
        for o in prog(*ins):
            o.release()

    ms = _time_events(rt, mlp_step, reps=20, warm=5, warm_ms=400)  # the uploads leave the GPU idle: reach the steady state first
    flop = 2.0 * (148224 + 280064) * B
    want = _mlp_float64(orc.fourier_features(coords), target, params)
    _check_mlp(prog, ins, want, "mlp")
    out["mlp_step_batch_262144"] = {"ms_per_step": round(ms, 3), "TFLOP/s_gemm_flop_over_step_time": round(flop / ms / 1e9, 1)}
    prog.destroy()
    # the same step with every matmul and sum as the lowered loop kernel of the reference (no primitive named by the
    # program): the primitives are reached by recognition alone
    prog = tf.compile("mlp", [2])
    ms = _time_events(rt, mlp_step, reps=20, warm=5, warm_ms=400)
    _check_mlp(prog, ins, want, "mlp from lowered loops")
    out["mlp_step_batch_262144_from_lowered_ir"] = {"ms_per_step": round(ms, 3), "TFLOP/s_gemm_flop_over_step_time": round(flop / ms / 1e9, 1)}
    prog.destroy()
    return out


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU-oracle baseline leg")
    ap.add_argument("--no-extras", action="store_true", help="skip the secondary numbers for the other benchmark configs")
    ap.add_argument("--no-graphs", action="store_true", help="skip the recorded-graph comparison (for runs under a kernel tracer)")
    ap.add_argument("--pmc-probe", action="store_true",
                    help="for counter collection: 7 device-to-device copies of X (a plain copy of known size, the calibration for "
                         "FETCH_SIZE / WRITE_SIZE) followed by 3 steps in which every call reads another copy of X, as in the timed run; prints nothing to time")
    ap.add_argument("--pmc-probe-sgemm", action="store_true",
                    help="for counter collection: 3 calls of tfhip_sgemm_nn on the config-5 hidden-layer shape [262144,256] x [256,256] "
                         "with normally distributed operands; prints nothing to time")
    ap.add_argument("--pmc-probe-sgemm-square", action="store_true",
                    help="for counter collection: 3 calls of tfhip_sgemm_nn on 4096 x 4096 x 4096 with normally distributed operands; prints nothing to time")
    ap.add_argument("--pmc-probe-sort", action="store_true",
                    help="for counter collection: one 1 GiB device copy (calibration), then two key-value sorts and two u32 prefix sums "
                         "of 2^28 elements; prints nothing to time")
    ap.add_argument("--pmc-probe-nbody", action="store_true",
                    help="for counter collection: 3 steps of the all-pairs N-body program (config 4, N = 65536) through the host path, "
                         "no warm-up (counters are per dispatch); prints nothing to time")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this backend runs on ONE GPU; --gpus must be 1 (multi-GPU sharding is a design note, not built)", file=sys.stderr)
        return 2

    if args.pmc_probe_sgemm or args.pmc_probe_sgemm_square:
        from tensorfrost_amd import runtime as rt

        rt.initialize(0)
        rng_g = np.random.default_rng(1234 + 5)
        m, n, k = (4096, 4096, 4096) if args.pmc_probe_sgemm_square else (262144, 256, 256)
        a = rt.DeviceBuffer.from_numpy(rng_g.standard_normal((m, k), dtype=np.float32))
        b = rt.DeviceBuffer.from_numpy(rng_g.standard_normal((k, n), dtype=np.float32))
        c = rt.DeviceBuffer(m * n)
        for _ in range(3):
            rt.sgemm("nn", a, b, c, m, n, k)
        rt.synchronize()
        print(json.dumps({"pmc_probe": "done", "flop_per_call": 2 * m * n * k}))
        return 0
    if args.pmc_probe_nbody:
        import tensorfrost_amd.host as tf
        from oracle import oracle as orc  # input generator only

        tf.initialize(tf.hip)
        xb, vb, mb = orc.nbody_inputs(65536)
        prog = tf.compile("nbody")
        X, V, M = tf.tensor(xb), tf.tensor(vb), tf.tensor(mb)
        dt, eps = tf.tensor(np.array([1e-3], np.float32)), tf.tensor(np.array([1e-3], np.float32))
        for _ in range(3):
            a, b = prog(X, V, M, dt, eps)
            a.release()
            b.release()
        tf.synchronize()
        print(json.dumps({"pmc_probe": "done", "pairs_per_step": 65536 * 65536, "flop_per_step_at_20_per_pair": 20 * 65536 * 65536}))
        return 0
    if args.pmc_probe_sort:
        from tensorfrost_amd import runtime as rt
        from tensorfrost_amd._lib import call

        rt.initialize(0)
        n = 1 << 28
        rng_s = np.random.default_rng(1234 + 3)
        keys = rt.DeviceBuffer.from_numpy(rng_s.integers(0, 2 ** 32, n, dtype=np.uint64).astype(np.uint32))
        vals = rt.DeviceBuffer(n)
        call("tfhip_d2d", vals.ptr, keys.ptr, n)  # the calibration copy: 1 GiB each way
        keys_out, vals_out = rt.DeviceBuffer(n), rt.DeviceBuffer(n)
        for _ in range(2):
            rt.radix_sort_kv(keys, vals, keys_out, vals_out, n)
        for _ in range(2):
            rt.scan_inclusive(keys, keys_out, n, np.uint32)
        rt.synchronize()
        print(json.dumps({"pmc_probe": "done", "copy_bytes_each_way": 4 * n, "keys": n}))
        return 0
    x = make_input()
    if args.pmc_probe:
        from tensorfrost_amd import runtime as rt
        from tensorfrost_amd._lib import call

        rt.initialize(0)
        xs = [rt.DeviceBuffer.from_numpy(x)]
        for _ in range(N_SETS - 1):
            xs.append(rt.DeviceBuffer(R * C))
        ys = [rt.DeviceBuffer(R * C) for _ in range(N_SETS // 2)]
        row, col = rt.DeviceBuffer(R), rt.DeviceBuffer(C)
        # the calibration copies double as the initialisation of the other copies of X (7 copies of 256 MiB each way)
        for b in xs[1:]:
            call("tfhip_d2d", b.ptr, xs[0].ptr, R * C)
        for s in range(3):
            at = lambda j: xs[(5 * s + j) % N_SETS]
            rt.reduce_rows("sum", at(0), row, R, C)
            rt.reduce_rows("max", at(1), row, R, C)
            rt.softmax_rows(at(2), ys[s % len(ys)], R, C)
            rt.reduce_cols("sum", at(3), col, R, C)
            rt.reduce_cols("max", at(4), col, R, C)
        rt.synchronize()
        print(json.dumps({"pmc_probe": "done", "copy_bytes_each_way": 4 * R * C}))
        return 0
    gpu = gpu_leg(x, args.steps, args.warmup)
    dom = "softmax_rows"

    def summary(mode):
        ms = gpu[mode]["ms_per_step"]
        per_call = gpu[mode]["per_call_ms"]
        return {
            "GB/s": round(STEP_BYTES / (ms * 1e-3) / 1e9, 2),
            "ms_per_step": round(ms, 5),
            "pct_of_hbm_peak": round(100.0 * STEP_BYTES / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 2),
            "kernels": {k: {"ms": round(v, 5), "GB/s": round(BYTES[k] / (v * 1e-3) / 1e9, 1)} for k, v in per_call.items()},
        }

    hbm = summary("hbm")
    ms = gpu["hbm"]["ms_per_step"]
    dom_ms = gpu["hbm"]["per_call_ms"][dom]
    achieved = BYTES[dom] / (dom_ms * 1e-3) / 1e9
    line = {
        "metric": "fused-kernel HBM GB/s",
        "value": hbm["GB/s"],
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": hbm["ms_per_step"],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {
            "workload": "row reductions + softmax: X[16384,4096] fp32 U(-4,4); sum, max, fused softmax along axis -1, then sum, max along axis 0; "
                        f"every call reads one of {N_SETS} copies of X in rotation (2 GiB between two reads of the same copy), so no read is served by the 256 MiB last-level cache",
            "rows": R, "cols": C, "bytes_per_step": STEP_BYTES, "device": gpu["device"]["name"],
        },
        "pct_of_hbm_peak": hbm["pct_of_hbm_peak"],
        "kernels": hbm["kernels"],
        "kernels_timing": "softmax_rows: events inside the timed region; the other calls: events in a second pass of the same steps",
        # the same step with all five calls on ONE copy of X (256 MiB, the size of the last-level cache) and one output:
        # part of the reads are served from that cache, so this is not an HBM figure
        "llc_assisted": summary("llc_assisted"),
        "roofline": {
            "kernel": "softmax_rows_block_kernel<512, 2>",
            "bound": "hbm",
            "achieved": round(achieved, 1),
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": round(achieved / HBM_PEAK_GBS, 4),
            # HBM bytes per launch of this kernel from FETCH_SIZE + WRITE_SIZE, each scaled by what the same counter
            # reads for a 256 MiB device-to-device copy; collected with --pmc-probe (same rotation over copies of X)
            # and kept in the counter summary under profiles/ (null when that file is absent)
            "traffic": softmax_traffic_bytes(),
        },
    }
    if not args.no_cpu:
        line["cpu_baseline"] = cpu_leg(x)
        if not args.no_extras:
            line["cpu_baseline"]["other_configs"] = cpu_others_leg()
    if not args.no_extras:
        line["extras"] = extras_leg(graphs=not args.no_graphs)
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())
