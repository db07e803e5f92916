"""Pins the oracle's op-table kernel (oracle/ops.cpp) to independent NumPy formulations: integer and bit rows
bit-for-bit, float rows against float64 evaluations of the textbook definitions."""
import numpy as np

from oracle import oracle

FLOAT_OPS = ["add", "sub", "mul", "div", "neg", "min", "max", "abs", "sign", "ceil", "floor", "round", "frac", "exp", "exp2", "log", "log2",
             "sqrt", "rsqrt", "rcp", "sin", "cos", "tan", "asin", "acos", "atan", "sinh", "cosh", "tanh", "pow", "atan2", "modf", "step",
             "clamp", "lerp", "fma", "smoothstep", "fmod_op", "ternary", "from_int", "from_uint", "pcgf"]
INT_OPS = ["add", "sub", "mul", "div", "mod", "lshift", "rshift", "and", "or", "xor", "not", "neg", "min", "max", "abs", "sign", "clamp", "lt",
           "lte", "gt", "gte", "eq", "neq", "from_float", "and_bool", "or_bool", "notb", "reversebits"]
UINT_OPS = ["add", "mul", "div", "mod", "lshift", "rshift", "and", "or", "xor", "not", "pcg", "reversebits", "asuint", "min", "max", "from_float"]


def _pcg(u):
    """PCG-RXS-M-XS 32 output function as published (O'Neill 2014), on uint64 with explicit masking."""
    m = np.uint64(0xFFFFFFFF)
    state = (u.astype(np.uint64) * np.uint64(747796405) + np.uint64(2891336453)) & m
    word = (((state >> ((state >> np.uint64(28)) + np.uint64(4))) ^ state) * np.uint64(277803737)) & m
    return ((word >> np.uint64(22)) ^ word).astype(np.uint32)


def _reverse_bits(u):
    bits = np.unpackbits(u.astype(">u4").view(np.uint8).reshape(-1, 4), axis=1)
    return np.packbits(bits[:, ::-1], axis=1).view(">u4").reshape(-1).astype(np.uint32)


def numpy_ops(x, y, a, b, u, w):
    """Independent evaluation: floats in float64 from the float32 inputs, integers in int64 wrapped to 32 bits."""
    X, Y = x.astype(np.float64), y.astype(np.float64)
    ynz = np.where(Y == 0, 1.0, Y)
    ax = np.abs(X)
    unit = np.clip(X, -1, 1)
    t = np.clip((X + 1.0) / 3.0, 0, 1)
    F = [X + Y, X - Y, X * Y, X / ynz, -X, np.minimum(X, Y), np.maximum(X, Y), ax, np.where(X < 0, -1.0, 1.0), np.ceil(X), np.floor(X),
         np.where(X >= 0, np.floor(X + 0.5), np.ceil(X - 0.5)), X - np.floor(X), np.exp(X), np.exp2(X), np.log(ax + 0.5), np.log2(ax + 0.5),
         np.sqrt(ax), 1 / np.sqrt(ax + 0.5), 1 / ynz, np.sin(X), np.cos(X), np.tan(unit), np.arcsin(unit), np.arccos(unit), np.arctan(X),
         np.sinh(X), np.cosh(X), np.tanh(X), np.power(ax + 0.5, Y), np.arctan2(X, Y), np.fmod(X, ynz), (X >= Y).astype(np.float64),
         np.clip(X, -0.5, 0.75), X + (Y - X) * 0.25, X * Y + 1.5, t * t * (3 - 2 * t), np.fmod(X, ynz), np.where(X > Y, X, Y),
         a.astype(np.float64), u.astype(np.float64), _pcg(u).astype(np.float64) / float(0xFFFFFFFF)]
    A, B = a.astype(np.int64), b.astype(np.int64)
    wrap = lambda v: (v & 0xFFFFFFFF).astype(np.uint32).view(np.int32)
    sh = B & 7
    bnz = np.where(B == 0, 1, B)
    trunc_div = (np.abs(A) // np.abs(bnz)) * np.sign(A) * np.sign(bnz)
    xi = np.trunc((x * np.float32(100.0)).astype(np.float64)).astype(np.int64)
    I = [wrap(A + B), wrap(A - B), wrap(A * B), wrap(trunc_div), wrap(A - trunc_div * bnz), wrap(A << sh), wrap(A >> sh), wrap(A & B),
         wrap(A | B), wrap(A ^ B), wrap(~A), wrap(-A), wrap(np.minimum(A, B)), wrap(np.maximum(A, B)), wrap(np.abs(A)),
         wrap(np.where(A < 0, -1, 1)), wrap(np.clip(A, -100, 1000)), wrap((A < B) * 1), wrap((A <= B) * 1), wrap((A > B) * 1),
         wrap((A >= B) * 1), wrap((A == B) * 1), wrap((A != B) * 1), wrap(xi), wrap(((A < B) & (x < y)) * 1), wrap(((A < B) | (x < y)) * 1),
         wrap((~(A < B)) * 1), _reverse_bits(a.view(np.uint32)).view(np.int32)]
    Uu, W = u.astype(np.uint64), w.astype(np.uint64)
    uw = lambda v: (v & np.uint64(0xFFFFFFFF)).astype(np.uint32)
    shu = W & np.uint64(7)
    wnz = np.where(W == 0, np.uint64(1), W)
    U = [uw(Uu + W), uw(Uu * W), uw(Uu // wnz), uw(Uu % wnz), uw(Uu << shu), uw(Uu >> shu), uw(Uu & W), uw(Uu | W), uw(Uu ^ W),
         uw(~Uu), _pcg(u), _reverse_bits(u), x.view(np.uint32), np.minimum(u, w), np.maximum(u, w),
         np.trunc((np.abs(x) * np.float32(1000.0)).astype(np.float64)).astype(np.uint32)]
    return np.stack(F), np.stack(I), np.stack(U)


def float_row_errors(got, want):
    """Largest error of each float row relative to max(1, |expected|)."""
    return np.max(np.abs(got.astype(np.float64) - want) / np.maximum(1.0, np.abs(want)), axis=1)


def test_op_lists_match_row_counts():
    lib = oracle.load()
    assert (lib.oracle_ops_float_rows(), lib.oracle_ops_int_rows(), lib.oracle_ops_uint_rows()) == (len(FLOAT_OPS), len(INT_OPS), len(UINT_OPS))


def test_oracle_ops_against_numpy():
    inputs = oracle.ops_inputs(5000)
    F, I, U = oracle.ops(*inputs)
    Fn, In, Un = numpy_ops(*inputs)
    for k, name in enumerate(INT_OPS):
        assert np.array_equal(I[k], In[k]), f"int op {name}"
    for k, name in enumerate(UINT_OPS):
        assert np.array_equal(U[k], Un[k]), f"uint op {name}"
    err = float_row_errors(F, Fn)
    for k, name in enumerate(FLOAT_OPS):
        # 1e-5 of max(1, |value|): element-wise tolerance; the oracle is built with -ffast-math like the reference's kernels
        assert err[k] < 1e-5, f"float op {name}: {err[k]:.3g}"


def test_known_answers():
    """Hand-derived values: pcg(0) from the published output function, bit reversal, C truncation of / and %."""
    x = np.array([2.5, -2.5, -0.0, 1.0], np.float32)
    y = np.array([0.0, 2.0, -1.0, 1.0], np.float32)
    a = np.array([-7, 7, -2**31 + 1, 5], np.int32)
    b = np.array([2, -2, 3, 0], np.int32)
    u = np.array([0, 1, 0x80000000, 0xFFFFFFFF], np.uint32)
    w = np.array([0, 3, 1, 2], np.uint32)
    F, I, U = oracle.ops(x, y, a, b, u, w)
    assert I[INT_OPS.index("div")].tolist() == [-3, -3, -715827882, 5]
    assert I[INT_OPS.index("mod")].tolist() == [-1, 1, -1, 0]
    assert F[FLOAT_OPS.index("round")].tolist() == [3.0, -3.0, 0.0, 1.0]
    assert F[FLOAT_OPS.index("sign")].tolist() == [1.0, -1.0, 1.0, 1.0]       # sign(0) = 1 in the C++ prelude
    assert U[UINT_OPS.index("reversebits")].tolist() == [0, 0x80000000, 1, 0xFFFFFFFF]
    # pcg(0): state = 2891336453; shift = (state >> 28) + 4 = 14; word = ((state >> 14) ^ state) * 277803737 mod 2^32; out = (word >> 22) ^ word
    state = 2891336453
    word = (((state >> ((state >> 28) + 4)) ^ state) * 277803737) & 0xFFFFFFFF
    assert int(U[UINT_OPS.index("pcg")][0]) == ((word >> 22) ^ word)
