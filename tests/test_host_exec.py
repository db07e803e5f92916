"""The host interpreter without a GPU: host programs run against a TFRuntime that only logs its six callbacks
(tests/host_exec_driver.cpp), and the host's scalar evaluator is compared op by op with NumPy.

What is pinned: the call sequence a program makes through the callback table (the contract of the generated `main`,
TensorFrost/Backend/CodeGen/Langs/CPP.cpp:678-718), the group count of a dispatch (CPP.cpp:503-515, closed form computed
here), the trailing block-offset word and the read-write-only tensor list (CPP.cpp:482-501), the error texts of the
input checks (CPP.cpp:431-448), and host control flow (loop / break / continue / if / set)."""
import shutil
import subprocess
from pathlib import Path

import numpy as np
import pytest

ROOT = Path(__file__).resolve().parent.parent
HOST = ROOT / "tensorfrost_amd" / "csrc" / "host"
LIB = ROOT / "tensorfrost_amd" / "lib"
TESTLIB = ROOT / "tests" / "programs"


@pytest.fixture(scope="module")
def driver(tmp_path_factory):
    if shutil.which("g++") is None:
        pytest.skip("g++ not available")
    exe = tmp_path_factory.mktemp("host_exec") / "driver"
    cmd = ["g++", "-O1", "-g", "-std=c++17", f"-I{ROOT / 'include'}", f"-I{ROOT / 'tensorfrost_amd' / 'csrc'}", f"-I{HOST}",
           str(Path(__file__).with_name("host_exec_driver.cpp")), f"-L{LIB}", f"-L{TESTLIB}", "-Wl,--no-as-needed", "-ltftestprograms", "-ltfhost", "-ltfhip",
           f"-Wl,-rpath,{LIB}", f"-Wl,-rpath,{TESTLIB}", "-Wl,-rpath,/opt/rocm/lib", "-o", str(exe)]
    build = subprocess.run(cmd, capture_output=True, text=True)
    assert build.returncode == 0, build.stderr[-4000:]
    return exe


def run(driver, scenario):
    out = subprocess.run([str(driver), "run", scenario], capture_output=True, text=True, timeout=300)
    assert out.returncode == 0, out.stdout + out.stderr
    return out.stdout.splitlines()


def f32_bits(x):
    return int(np.float32(x).view(np.uint32))


def test_wave_eq_call_sequence(driver):
    groups = -(-37 // 16) * -(-100 // 16)  # innermost two extents in groups of 16, rounded up
    assert run(driver, "wave_eq") == [
        "begin WaveEq",
        "alloc v_new [100,37] Float",
        "alloc u_new [100,37] Float",
        # all tensors in the read-write list, written ones (marked stale for the host: *) first; variables N, M, then the block offset 0
        f"dispatch k0 tensors v_new* u_new* u v ro=0 vars 100 37 0 groups {groups}",
        "end WaveEq",
        "out 0 v_new [100,37] Float",
        "out 1 u_new [100,37] Float",
    ]


@pytest.mark.parametrize("scenario, message", [
    ("wave_eq_bad_shape", "error Invalid shape for dimension 1 in v. Expected 37, got 38"),
    ("wave_eq_bad_type", "error Invalid type for v. Expected Float, got Int"),
    ("wave_eq_bad_dims", "error Invalid number of dimensions for u. Expected 2, got 1"),
    ("tiled_bad", "error Assertion failed: tiled_matmul_ir: every dimension must be a multiple of 64"),
])
def test_input_checks_fail_with_the_reference_texts_before_any_allocation(driver, scenario, message):
    log = run(driver, scenario)
    assert log[-1] == message
    assert not [l for l in log if l.startswith(("alloc", "dispatch"))]


def test_scalar_tensors_reach_the_kernel_as_buffers_without_a_readback(driver):
    log = run(driver, "nbody")
    assert not [l for l in log if l.startswith("read")]
    assert f"dispatch k0 tensors x_new* v_new* X V M dt eps ro=0 vars 1000 0 groups {-(-1000 // 256)}" in log


def test_a_scalar_read_back_by_the_host_becomes_a_kernel_variable(driver):
    log = run(driver, "broadcast_loops")
    assert "read first 0" in log
    (dispatch,) = [l for l in log if l.startswith("dispatch")]
    assert dispatch == f"dispatch k0 tensors out_sum* out_max* out_count* x a table itable ro=0 vars 500 7 40 0 groups {-(-500 // 256)}"


def test_four_dimensional_dispatch_counts_outer_extents_whole(driver):
    log = run(driver, "indexing4")
    groups = 3 * -(-9 // 8) * -(-10 // 8) * -(-17 // 8)  # the outermost extent has no group size
    (dispatch,) = [l for l in log if l.startswith("dispatch")]
    assert dispatch == f"dispatch k0 tensors shifted* transposed* ids* data ro=0 vars 3 9 10 17 0 groups {groups}"
    assert "alloc transposed [3,17,10,9] Float" in log


def test_sort_composition_call_sequence(driver):
    """tf.sort.radix on 1000 keys: the copies, then six passes of seven kernels between region markers, every
    intermediate released inside its pass (Python/TensorFrost/sort.py:76-176)."""
    log = run(driver, "radix_sort_ir")
    n, group, hist = 1000, 128, 64
    G = -(-n // group)
    chunks = -(-G // 64)
    assert log[0] == "begin Radix sort"
    assert log.count("begin Radix sort iteration") == 6 and log.count("end Radix sort iteration") == 6
    dispatches = [l for l in log if l.startswith("dispatch")]
    assert len(dispatches) == 2 + 6 * 7 + 1
    first_pass = log[log.index("begin Radix sort iteration"):log.index("end Radix sort iteration") + 1]
    assert first_pass == [
        "begin Radix sort iteration",
        f"alloc group_histogram_packed [{G},{hist // 4}] Uint",
        f"dispatch k3 tensors group_histogram_packed* keys ro=0 vars {n} {G} 0 0 groups {-(-(hist // 4) // 16) * -(-G // 16)}",
        f"alloc group_histogram [{G},{hist}] Uint",
        f"dispatch k4 tensors group_histogram* group_histogram_packed ro=0 vars {G} 0 groups {-(-hist // 16) * -(-G // 16)}",
        "dealloc group_histogram_packed",
        f"alloc chunk_scan [{chunks},{hist}] Uint",
        f"dispatch k5 tensors chunk_scan* group_histogram ro=0 vars {G} {chunks} 0 groups {-(-hist // 16) * -(-chunks // 16)}",
        f"alloc chunk_scan_out [{chunks},{hist}] Uint",
        f"dispatch k6 tensors chunk_scan_out* chunk_scan ro=0 vars {chunks} 0 groups 1",
        "dealloc chunk_scan",
        f"alloc group_histogram_scan [{G},{hist}] Uint",
        f"dispatch k7 tensors group_histogram_scan* group_histogram chunk_scan_out ro=0 vars {G} {chunks} 0 groups {-(-hist // 16) * -(-chunks // 16)}",
        "dealloc group_histogram",
        "dealloc chunk_scan_out",
        f"alloc total_bit_histogram [{hist}] Uint",
        f"dispatch k8 tensors total_bit_histogram* group_histogram_scan ro=0 vars {G} 0 groups 1",
        # the scatter kernel: shape [G, 128] with one group dimension of 128
        f"dispatch k9 tensors keys1* values1* keys values group_histogram_scan total_bit_histogram ro=0 vars {n} {G} 0 0 groups {G}",
        "dealloc group_histogram_scan",
        "dealloc total_bit_histogram",
        "end Radix sort iteration",
    ]
    # the second pass reads what the first one wrote
    second = [l for l in dispatches if l.startswith("dispatch k9")][1]
    assert second == f"dispatch k9 tensors keys* values* keys1 values1 group_histogram_scan total_bit_histogram ro=0 vars {n} {G} 1 0 groups {G}"
    assert log[-2:] == ["out 0 keys_sorted [1000] Uint", "out 1 values [1000] Uint"]


def test_host_control_flow(driver):
    """counts = [3, 5, -2, 300, 7, 9]: counts[0] bounds the trips; trip 1 adds 5, trip 2 is skipped by `continue`
    (negative), trip 3 adds 300, trip 4 leaves through `break`."""
    log = run(driver, "control")
    body = log[:log.index("listing")]
    total = 305
    assert body == [
        "read counts 0",
        "read counts 1",
        "alloc step [5] Float",
        f"dispatch k0 tensors step* ro=0 vars 5 {f32_bits(0.5)} 0 groups 1",
        "dealloc step",
        "read counts 2",
        "read counts 3",
        "alloc step [300] Float",
        f"dispatch k0 tensors step* ro=0 vars 300 {f32_bits(1.5)} 0 groups 2",
        "dealloc step",
        f"write counts 0 {total}",
        f"alloc grid [{total},2] Float",
        # the reshaped view shares grid's buffer; 1 / float(total) is evaluated in fp32 on the host
        f"dispatch k0 tensors grid* ro=0 vars {2 * total} {f32_bits(np.float32(1.0) / np.float32(total))} 0 groups {-(-2 * total // 256)}",
        f"out 0 grid [{total},2] Float",
        f"out 1 grid [{2 * total}] Float",
    ]
    listing = log[log.index("listing") + 1:]
    assert any("tf.reshape(" in l for l in listing) and any("tf.assert_tensor(" in l for l in listing)


def test_assert_value_stops_the_program(driver):
    log = run(driver, "control_assert")
    body = log[:log.index("listing")]
    assert body[-1] == "error Assertion failed: total is positive"
    assert not [l for l in body if l.startswith(("alloc", "dispatch", "write"))]


# ---- the scalar evaluator ------------------------------------------------------------------------------------------

def evaluate(driver, rows):
    text = "".join(f"{op} {src} {dst} {a:08x} {b:08x} {c:08x}\n" for op, src, dst, a, b, c in rows)
    out = subprocess.run([str(driver), "scalar"], input=text, capture_output=True, text=True, timeout=300)
    assert out.returncode == 0, out.stderr
    lines = out.stdout.splitlines()
    assert len(lines) == len(rows)
    return lines


def test_integer_and_bit_operations_are_exact(driver):
    rng = np.random.default_rng(5)
    a = np.concatenate([rng.integers(-2**31, 2**31, 200), [0, 1, -1, 2**31 - 1, -2**31, 7, -7]]).astype(np.int64)
    b = np.concatenate([rng.integers(-2**31, 2**31, 200), [3, -3, 5, 1, -1, -2, 2]]).astype(np.int64)
    b[::5] = rng.integers(-40, 40, b[::5].size)
    b[b == 0] = 9
    c = np.minimum(np.maximum(a, b) + 11, 2**31 - 1)
    wrap = lambda v: int(v) & 0xFFFFFFFF
    trunc_div = lambda x, y: int(abs(x) // abs(y)) * (1 if (x >= 0) == (y > 0) else -1)
    rows, want = [], []
    for x, y, z in zip(a, b, c):
        x, y, z = int(x), int(y), int(z)
        ux, uy = x & 0xFFFFFFFF, y & 0xFFFFFFFF
        sh = uy & 31
        q = trunc_div(x, y) if not (x == -2**31 and y == -1) else x
        cases = [
            ("add", "i", "i", wrap(x + y)), ("sub", "i", "i", wrap(x - y)), ("mul", "i", "i", wrap(x * y)), ("div", "i", "i", wrap(q)),
            ("mod", "i", "i", wrap(x - trunc_div(x, y) * y) if y != -1 else 0), ("lshift", "i", "i", wrap(ux << sh)), ("rshift", "i", "i", wrap(x >> sh)),
            ("and", "i", "i", ux & uy), ("or", "i", "i", ux | uy), ("xor", "i", "i", ux ^ uy), ("not", "i", "i", wrap(~x)), ("neg", "i", "i", wrap(-x)),
            ("min", "i", "i", wrap(min(x, y))), ("max", "i", "i", wrap(max(x, y))), ("abs", "i", "i", wrap(abs(x))), ("sign", "i", "i", wrap(-1 if x < 0 else 1)),
            ("lt", "i", "b", int(x < y)), ("lte", "i", "b", int(x <= y)), ("gt", "i", "b", int(x > y)), ("gte", "i", "b", int(x >= y)),
            ("eq", "i", "b", int(x == y)), ("neq", "i", "b", int(x != y)),
            ("add", "u", "u", wrap(ux + uy)), ("mul", "u", "u", wrap(ux * uy)), ("div", "u", "u", ux // uy), ("mod", "u", "u", ux % uy),
            ("rshift", "u", "u", ux >> sh), ("lshift", "u", "u", wrap(ux << sh)), ("min", "u", "u", min(ux, uy)), ("lt", "u", "b", int(ux < uy)),
            ("asint", "u", "i", ux), ("asuint", "i", "u", ux), ("asfloat", "u", "f", ux), ("uint", "i", "u", ux), ("int", "u", "i", ux),
            ("bool", "i", "b", int(x != 0)), ("notb", "b", "b", int(not (x & 1))),
            ("reversebits", "u", "u", int(f"{ux:032b}"[::-1], 2)),
        ]
        for op, src, dst, expected in cases:
            rows.append((op, src, dst, ux if src != "b" else x & 1, uy, 0))
            want.append(expected)
        lo, hi = min(y, z), max(y, z)
        rows.append(("clamp", "i", "i", ux, wrap(lo), wrap(hi)))
        want.append(wrap(min(max(x, lo), hi)))
        rows.append(("ternary", "i", "i", x & 1, uy, wrap(z)))
        want.append(uy if x & 1 else wrap(z))
    # PCG-RXS-M-XS 32 (O'Neill 2014) on 64-bit integers with explicit masks
    for v in [0, 1, 12345, 0xFFFFFFFF, 0xDEADBEEF]:
        state = (v * 747796405 + 2891336453) & 0xFFFFFFFF
        word = (((state >> ((state >> 28) + 4)) ^ state) * 277803737) & 0xFFFFFFFF
        rows.append(("pcg", "u", "u", v, 0, 0))
        want.append((word >> 22) ^ word)
    got = evaluate(driver, rows)
    wrong = [(r, g, f"{w:08x}") for r, g, w in zip(rows, got, want) if g != f"{w:08x}"]
    assert not wrong, wrong[:10]


def test_division_by_zero_is_an_error_of_the_program(driver):
    got = evaluate(driver, [("div", "i", "i", 5, 0, 0), ("mod", "u", "u", 5, 0, 0)])
    assert got == ["error Host program: integer division by zero", "error Host program: integer remainder by zero"]


def test_float_operations(driver):
    rng = np.random.default_rng(6)
    x = np.concatenate([rng.uniform(-3, 3, 120), [0.0, 1.0, -1.0, 0.5, 2.5, -2.5, 1e-3]]).astype(np.float32)
    y = np.concatenate([rng.uniform(-3, 3, 120), [1.0, -2.0, 3.0, 0.25, -0.75, 1.5, 2.0]]).astype(np.float32)
    y[np.abs(y) < 0.05] = 0.7
    z = rng.uniform(0, 1, x.size).astype(np.float32)
    X, Y, Z = x.astype(np.float64), y.astype(np.float64), z.astype(np.float64)
    ax = np.abs(X) + 0.5
    unit = np.clip(X / 3.0, -1, 1)
    t = np.clip((Z - X) / (Y - X), 0, 1)
    exact = {  # correctly rounded in fp32: compared bit for bit
        "add": x + y, "sub": x - y, "mul": x * y, "div": x / y, "neg": -x, "min": np.minimum(x, y), "max": np.maximum(x, y), "abs": np.abs(x),
        "ceil": np.ceil(x), "floor": np.floor(x), "sqrt": np.sqrt(np.abs(x)), "sign": np.where(x < 0, np.float32(-1), np.float32(1)),
        "round": np.where(x >= 0, np.floor(x + np.float32(0.5)), np.ceil(x - np.float32(0.5))).astype(np.float32),
        "step": (y >= x).astype(np.float32), "frac": (x - np.floor(x)).astype(np.float32),
    }
    unary_input = {"sqrt": np.abs(x)}
    close = {  # library functions: within a few ulp of the float64 value
        "exp": (x, np.exp(X)), "exp2": (x, np.exp2(X)), "log": (ax.astype(np.float32), None), "log2": (ax.astype(np.float32), None),
        "sin": (x, np.sin(X)), "cos": (x, np.cos(X)), "tan": (unit.astype(np.float32), None), "asin": (unit.astype(np.float32), None),
        "acos": (unit.astype(np.float32), None), "atan": (x, np.arctan(X)), "sinh": (x, np.sinh(X)), "cosh": (x, np.cosh(X)), "tanh": (x, np.tanh(X)),
        "rsqrt": (ax.astype(np.float32), None), "rcp": (y, 1.0 / Y),
    }
    f64 = {"log": np.log, "log2": np.log2, "tan": np.tan, "asin": np.arcsin, "acos": np.arccos, "rsqrt": lambda v: 1 / np.sqrt(v)}
    rows, want, tol = [], [], []
    bits = lambda v: v.astype(np.float32).view(np.uint32)
    for op, expected in exact.items():
        a = unary_input.get(op, x)
        for k in range(x.size):
            rows.append((op, "f", "f", int(bits(a)[k]), int(bits(y)[k]), 0))
            want.append(float(expected[k]))
            tol.append(0.0)
    for op, (arg, expected) in close.items():
        if expected is None:
            expected = f64[op](arg.astype(np.float64))
        for k in range(x.size):
            rows.append((op, "f", "f", int(bits(arg)[k]), 0, 0))
            want.append(float(expected[k]))
            tol.append(4e-7)
    binary = {"pow": (ax.astype(np.float32), y, np.power(ax.astype(np.float32).astype(np.float64), Y)), "atan2": (x, y, np.arctan2(X, Y)),
              "modf": (x, y, np.fmod(X, Y)), "mod": (x, y, np.fmod(X, Y))}
    for op, (p, q, expected) in binary.items():
        for k in range(x.size):
            rows.append((op, "f", "f", int(bits(p)[k]), int(bits(q)[k]), 0))
            want.append(float(expected[k]))
            tol.append(4e-7)
    lo, hi = np.minimum(y, z), np.maximum(y, z)
    ternary = {"clamp": (x, lo, hi, np.clip(X, lo.astype(np.float64), hi.astype(np.float64)), 0.0), "lerp": (x, y, z, X + (Y - X) * Z, 1e-6),
               "fma": (x, y, z, X * Y + Z, 2e-7), "smoothstep": (x, y, z, t * t * (3 - 2 * t), 2e-6)}
    for op, (p, q, r, expected, tolerance) in ternary.items():
        for k in range(x.size):
            rows.append((op, "f", "f", int(bits(p)[k]), int(bits(q)[k]), int(bits(r)[k])))
            want.append(float(expected[k]))
            tol.append(tolerance)
    # conversions
    for k in range(x.size):
        v = np.float32(x[k] * 1000)
        rows.append(("int", "f", "i", int(v.view(np.uint32)), 0, 0))
        want.append(("bits", int(np.trunc(np.float64(v))) & 0xFFFFFFFF))
        tol.append(0.0)
        i = int(np.trunc(np.float64(v)))
        rows.append(("float", "i", "f", i & 0xFFFFFFFF, 0, 0))
        want.append(float(np.float32(i)))
        tol.append(0.0)
        rows.append(("float", "u", "f", i & 0xFFFFFFFF, 0, 0))
        want.append(float(np.float32(i & 0xFFFFFFFF)))
        tol.append(0.0)
        rows.append(("uint", "f", "u", int(np.abs(v).view(np.uint32)), 0, 0))
        want.append(("bits", int(np.trunc(np.float64(np.abs(v))))))
        tol.append(0.0)
    got = evaluate(driver, rows)
    wrong = []
    for row, g, w, e in zip(rows, got, want, tol):
        if isinstance(w, tuple):
            ok = int(g, 16) == w[1]
        else:
            value = float(np.uint32(int(g, 16)).view(np.float32))
            ok = (value == w) if e == 0.0 else abs(value - w) <= e * max(abs(w), 1.0)
        if not ok:
            wrong.append((row, g, w))
    assert not wrong, wrong[:10]
