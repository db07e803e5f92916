"""Kernels that runs of the reference printed, executed: the text of tests/golden/reference_kernel_text.json is parsed
into a kernel tree (tests/programs/kernel_text.cpp), emitted by the HIP emitter, dispatched through the host path on
the MI355X, and the result is compared with what the kernel is known to compute -- a 1024-point FFT against numpy's,
the hand-tiled matrix product against a float64 product, the Buddhabrot tone-mapping and clearing kernels and the
fluid solver's divergence / curl stencil against NumPy restatements of the printed statements. Each kernel runs twice:
emitted verbatim (the form the text comparison checks) and emitted the way any program's kernel is (four-wide
mapping, range-based simplifications), so the optimised emission is tied to the same printed kernels."""
import ctypes

import numpy as np
import pytest

from test_reference_kernel_text import KERNELS

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def tf():
    import tensorfrost_amd.host as tfh

    tfh.initialize(tfh.hip)
    yield tfh
    tfh.synchronize()


@pytest.fixture(scope="module")
def set_text():
    from conftest import TEST_PROGRAMS

    lib = ctypes.CDLL(str(TEST_PROGRAMS), mode=ctypes.RTLD_GLOBAL)
    fn = lib.tftest_set_kernel_text
    fn.restype = ctypes.c_long
    fn.argtypes = [ctypes.c_char_p, ctypes.POINTER(ctypes.c_int), ctypes.c_char_p, ctypes.c_char_p, ctypes.c_size_t]

    def run(kernel):
        out = ctypes.create_string_buffer(1 << 16)
        n = fn("\n".join(kernel["body"]).encode(), (ctypes.c_int * 3)(*kernel["group_size"]), "\n".join(kernel["shared"]).encode(), out, len(out))
        text = out.value.decode()
        if n < 0:
            raise RuntimeError(text)
        buffers, variables = text.split("|")
        return [b for b in buffers.split(",") if b], [v for v in variables.split(",") if v]

    return run


def kernel_of(notebook, index):
    found = [k for k in KERNELS if notebook in k["from"] and k["from"].endswith(f"kernel {index}")]
    assert len(found) == 1
    return found[0]


def run_kernel(tf, set_text, kernel, shape, buffers, variables, as_any_kernel):
    """buffers: name -> array of 32-bit words; variables: name -> int. Returns name -> array after the dispatch."""
    names, var_names = set_text(kernel)
    assert sorted(names) == sorted(buffers) and sorted(var_names) == sorted(variables), (names, var_names)
    prog = tf.compile("kernel_text", [int(as_any_kernel), len(shape), *shape, *[variables[v] for v in var_names]])
    tensors = [tf.tensor(np.ascontiguousarray(buffers[n]).view(np.uint32).reshape(-1)) for n in names]
    prog(*tensors).release()
    out = {n: t.numpy.view(buffers[n].dtype).reshape(buffers[n].shape) for n, t in zip(names, tensors)}
    for t in tensors:
        t.release()
    prog.destroy()
    return out


@pytest.mark.parametrize("as_any_kernel", [False, True], ids=["verbatim", "optimised"])
def test_fft_group_kernel_computes_the_fft(tf, set_text, as_any_kernel):
    rng = np.random.default_rng(11)
    z = (rng.normal(size=1024) + 1j * rng.normal(size=1024)).astype(np.complex64)
    a = np.stack([z.real, z.imag], axis=1).astype(np.float32)
    # one group of 512 threads transforms all 1024 points (two per thread) in group memory
    out = run_kernel(tf, set_text, kernel_of("fft_group", 0), [512], {"A": a}, {}, as_any_kernel)["A"]
    got = out[:, 0] + 1j * out[:, 1]
    want = np.fft.fft(z.astype(np.complex128))
    assert np.max(np.abs(got - want)) < 1e-4 * np.abs(z).sum()  # every output is a sum of all 1024 inputs


@pytest.mark.parametrize("as_any_kernel", [False, True], ids=["verbatim", "optimised"])
def test_tiled_matrix_product_kernel_computes_the_product(tf, set_text, as_any_kernel):
    n = 128  # the printed kernel walks the inner dimension up to var.K: square operands
    rng = np.random.default_rng(12)
    a = rng.normal(size=(n, n)).astype(np.float32)
    b = rng.normal(size=(n, n)).astype(np.float32)
    c = np.zeros((n, n), np.float32)
    out = run_kernel(tf, set_text, kernel_of("matrix_mul", 0), [n // 4, n // 4], {"C": c, "A": a, "B": b}, {"N": n, "M": n, "K": n}, as_any_kernel)["C"]
    scale = np.abs(a).astype(np.float64) @ np.abs(b).astype(np.float64)
    assert np.max(np.abs(out - a.astype(np.float64) @ b.astype(np.float64)) / scale) < 1e-6


def smoothstep(lo, hi, x):
    t = np.clip((x - lo) / (hi - lo), 0.0, 1.0)
    return t * t * (3.0 - 2.0 * t)


@pytest.mark.parametrize("as_any_kernel", [False, True], ids=["verbatim", "optimised"])
def test_buddhabrot_kernels(tf, set_text, as_any_kernel):
    rng = np.random.default_rng(13)
    counts = rng.integers(0, 3000, (1024, 1024, 3)).astype(np.int32)
    # kernel 0 clears the hit counters (3-D dispatch, 3 x 8 x 8 groups)
    cleared = run_kernel(tf, set_text, kernel_of("buddhabrot", 0), [1024, 1024, 3], {"atomic_canvas": counts.copy()}, {}, as_any_kernel)["atomic_canvas"]
    assert not cleared.any()
    # kernel 3: m1 = frame_id + 1 (one thread)
    out = run_kernel(tf, set_text, kernel_of("buddhabrot", 3), [1], {"m1": np.zeros(1, np.int32), "frame_id": np.array([41], np.int32)}, {}, as_any_kernel)
    assert out["m1"][0] == 42
    # kernel 2: tone mapping of the counters, averaged with the previous frame
    prev = rng.random((1024, 1024, 3), dtype=np.float32)
    fid = 7
    out = run_kernel(tf, set_text, kernel_of("buddhabrot", 2), [1024, 1024],
                     {"canvas": np.zeros((1024, 1024, 3), np.float32), "atomic_canvas": counts, "frame_id": np.array([fid], np.int32), "prev_frame": prev}, {}, as_any_kernel)["canvas"]
    x, y, rz = (counts[..., k].astype(np.float64) for k in range(3))
    rx, ry = x + y + rz, y + rz
    want = np.stack([(prev[..., k].astype(np.float64) * fid + smoothstep(0.0, 1.0, 2.5 * np.power(r / 800.0, e))) / (fid + 1.0)
                     for k, (r, e) in enumerate(((rx, np.float32(0.9)), (ry, np.float32(0.65)), (rz, np.float32(0.5))))], axis=-1)
    assert np.max(np.abs(out - want)) < 1e-5  # element-wise tolerance (values in [0, 1])


@pytest.mark.parametrize("as_any_kernel", [False, True], ids=["verbatim", "optimised"])
@pytest.mark.parametrize("n1,m1", [(540, 960), (17, 33)])
def test_fluid_divergence_and_curl_kernel(tf, set_text, as_any_kernel, n1, m1):
    rng = np.random.default_rng(n1)
    vx = rng.normal(size=(n1, m1)).astype(np.float32)
    vy = rng.normal(size=(n1, m1)).astype(np.float32)
    kernel = kernel_of("fluid_simulation", 1)
    assert "curl_mem" in "\n".join(kernel["body"])
    out = run_kernel(tf, set_text, kernel, [n1, m1],
                     {"div": np.zeros((n1, m1), np.float32), "curl": np.zeros((n1, m1), np.float32), "vx_2": vx, "vy_2": vy}, {"M1": m1, "N1": n1}, as_any_kernel)
    i, j = np.meshgrid(np.arange(n1), np.arange(m1), indexing="ij")

    def at(f, di, dj):  # clamped taps, as the printed loads index them
        return f[np.clip(i + di, 0, n1 - 1), np.clip(j + dj, 0, m1 - 1)].astype(np.float64)

    div = (((at(vx, 1, 0) - at(vx, -1, 0)) + at(vy, 0, 1)) - at(vy, 0, -1)) / 2.0
    curl = np.abs(((at(vy, 1, 0) - at(vy, -1, 0)) - at(vx, 0, 1)) + at(vx, 0, -1)) / 2.0
    assert np.max(np.abs(out["div"] - div)) < 1e-5
    assert np.max(np.abs(out["curl"] - curl)) < 1e-5


@pytest.mark.parametrize("as_any_kernel", [False, True], ids=["verbatim", "optimised"])
def test_fluid_red_black_pressure_kernel(tf, set_text, as_any_kernel):
    """One half-sweep of the pressure solver: zero outside the 540 x 960 grid (the constants are in the printed text),
    over-relaxation 1.2 on the cells whose index sum is even, the other cells copied."""
    n1, m1 = 540, 960
    rng = np.random.default_rng(14)
    p0 = rng.normal(size=(n1, m1)).astype(np.float32)
    div = rng.normal(size=(n1, m1)).astype(np.float32)
    out = run_kernel(tf, set_text, kernel_of("fluid_simulation", 3), [n1, m1],
                     {"pressure2": np.zeros((n1, m1), np.float32), "pressure0": p0, "div_3": div}, {"v7_1": m1, "v7_0": n1}, as_any_kernel)["pressure2"]
    padded = np.pad(p0.astype(np.float64), 1)
    neighbours = padded[:-2, 1:-1] + padded[2:, 1:-1] + padded[1:-1, :-2] + padded[1:-1, 2:]
    relaxed = p0 + ((neighbours - div) / 4.0 - p0) * np.float64(np.float32(1.2))
    i, j = np.meshgrid(np.arange(n1), np.arange(m1), indexing="ij")
    want = np.where((i + j) % 2 == 0, relaxed, p0)
    assert np.max(np.abs(out - want)) < 1e-5 * (1.0 + np.abs(want).max())


def test_buddhabrot_orbit_kernel(tf, set_text):
    """The kernel with everything in it: a pcg random stream kept in a modified variable, two nested escape-time loops with
    break and continue, a chained ternary and integer atomics into a clamped canvas. Every orbit point is added at
    (y, x) and at (1023 - y, x), so the canvas must mirror itself exactly; integer atomics make the result independent
    of timing, so the verbatim and the optimised emission must agree in every counter."""
    kernel = kernel_of("buddhabrot", 1)
    inputs = {"atomic_canvas": np.zeros((1024, 1024, 3), np.int32), "m0": np.array([0.7], np.float32), "frame_id": np.array([3], np.int32)}
    plain = run_kernel(tf, set_text, kernel, [1024, 1024], inputs, {}, False)["atomic_canvas"]
    assert plain.sum() > 1_000_000 and plain.min() >= 0
    assert np.array_equal(plain, plain[::-1])
    assert plain[..., 2].sum() > 0 and plain[..., 1].sum() > 0  # short and medium orbits both occur
    optimised = run_kernel(tf, set_text, kernel, [1024, 1024], inputs, {}, True)["atomic_canvas"]
    assert np.array_equal(plain, optimised)


@pytest.mark.parametrize("index", range(14))
def test_fluid_kernels_give_the_same_results_verbatim_and_optimised(tf, set_text, index):
    """All 14 kernels of the fluid solver (advection with bilinear taps, divergence, multigrid restriction, red-black
    sweeps, prolongation, the final projection and rendering): emitted verbatim and emitted with the four-wide
    mapping, interior / border variants and range-based simplifications, on the same random fields, they must agree.
    Every extent is 48 and every buffer holds 48^3 words, which covers the largest index any of the printed address
    expressions can form (clamped taps, 2 i + 1 restriction taps, three channels per pixel)."""
    kernel = kernel_of("fluid_simulation", index)
    names, var_names = set_text(kernel)
    extent = 48
    rng = np.random.default_rng(100 + index)
    buffers = {n: rng.random(extent**3, dtype=np.float32) for n in names}
    variables = {v: extent for v in var_names}
    plain = run_kernel(tf, set_text, kernel, [extent, extent], buffers, variables, False)
    optimised = run_kernel(tf, set_text, kernel, [extent, extent], buffers, variables, True)
    changed = False
    for n in names:
        assert np.all(np.isfinite(plain[n]))
        assert np.allclose(plain[n], optimised[n], rtol=1e-5, atol=1e-6), n
        changed |= not np.array_equal(plain[n], buffers[n])
    assert changed  # the kernel wrote something
