"""Pins the oracle's restatement of the generated-kernel prelude (CPP.cpp:31-271) and of the dispatch
arithmetic (CPP.cpp:503-515) against independent formulations."""
import ctypes as C
import itertools
import struct

import numpy as np
import pytest

from oracle import oracle


@pytest.fixture(scope="module")
def lib():
    lib = oracle.load()
    lib.oracle_pcg.restype = C.c_uint32
    lib.oracle_pcg.argtypes = [C.c_uint32]
    lib.oracle_pcgf.restype = C.c_float
    lib.oracle_pcgf.argtypes = [C.c_uint32]
    lib.oracle_reversebits.restype = C.c_uint32
    lib.oracle_reversebits.argtypes = [C.c_uint32]
    for name in ("oracle_sign_f",):
        getattr(lib, name).restype = C.c_float
        getattr(lib, name).argtypes = [C.c_float]
    lib.oracle_sign_i.argtypes = [C.c_int]
    lib.oracle_clamp_i.argtypes = [C.c_int] * 3
    for name in ("oracle_clamp_f", "oracle_lerp", "oracle_smoothstep"):
        getattr(lib, name).restype = C.c_float
        getattr(lib, name).argtypes = [C.c_float] * 3
    for name in ("oracle_max_f", "oracle_min_f"):
        getattr(lib, name).restype = C.c_float
        getattr(lib, name).argtypes = [C.c_float] * 2
    lib.oracle_asuint_f.restype = C.c_uint32
    lib.oracle_asuint_f.argtypes = [C.c_float]
    lib.oracle_asfloat_u.restype = C.c_float
    lib.oracle_asfloat_u.argtypes = [C.c_uint32]
    lib.oracle_work_group_count.restype = C.c_size_t
    lib.oracle_work_group_count.argtypes = [C.POINTER(C.c_size_t), C.c_size_t, C.POINTER(C.c_size_t), C.c_size_t]
    return lib


def pcg_bigint(v: int) -> int:
    """The PCG RXS-M-XS output permutation in unbounded Python integers with explicit 32-bit masks: a different
    arithmetic from C's wrapping uint32, so a dropped wrap, a signed shift or a wrong shift amount shows."""
    M = 0xFFFFFFFF
    state = (v * 747796405 + 2891336453) & M
    word = (((state >> ((state >> 28) + 4)) ^ state) * 277803737) & M
    return ((word >> 22) ^ word) & M


def test_pcg_matches_unbounded_arithmetic_and_is_a_bijection(lib):
    rng = np.random.default_rng(1)
    for v in [0, 1, 2, 0x7FFFFFFF, 0x80000000, 0xFFFFFFFF] + [int(x) for x in rng.integers(0, 2**32, 2000)]:
        assert lib.oracle_pcg(v) == pcg_bigint(v)
    # RXS-M-XS is a permutation of the 32-bit integers: no two of 2^17 consecutive inputs collide
    outs = {lib.oracle_pcg(v) for v in range(1 << 17)}
    assert len(outs) == 1 << 17


def test_pcgf_is_pcg_over_2_32_minus_1_in_float(lib):
    for v in (0, 5, 123456789, 0xFFFFFFFF):
        expect = np.float32(np.float32(pcg_bigint(v)) / np.float32(0xFFFFFFFF))
        assert lib.oracle_pcgf(v) == expect
        assert 0.0 <= lib.oracle_pcgf(v) <= 1.0  # 1.0 is reachable: float(0xffffffff) rounds up


def test_reversebits_is_string_reversal(lib):
    rng = np.random.default_rng(2)
    for v in [0, 1, 0x80000000, 0xFFFFFFFF, 0x12345678] + [int(x) for x in rng.integers(0, 2**32, 500)]:
        assert lib.oracle_reversebits(v) == int(format(v, "032b")[::-1], 2)


def test_sign_of_zero_is_plus_one(lib):
    assert lib.oracle_sign_f(0.0) == 1.0 and lib.oracle_sign_f(-0.0) == 1.0
    assert lib.oracle_sign_f(-2.5) == -1.0 and lib.oracle_sign_f(3.0) == 1.0
    assert lib.oracle_sign_i(0) == 1 and lib.oracle_sign_i(-7) == -1


def test_clamp_lerp_smoothstep_closed_forms(lib):
    assert [lib.oracle_clamp_i(x, 0, 9) for x in (-5, 0, 4, 9, 12)] == [0, 0, 4, 9, 9]
    assert lib.oracle_clamp_f(1.5, 0.0, 1.0) == 1.0 and lib.oracle_clamp_f(-1.5, 0.0, 1.0) == 0.0
    assert lib.oracle_lerp(2.0, 10.0, 0.25) == 4.0      # a + (b - a) t
    assert lib.oracle_lerp(2.0, 10.0, 0.0) == 2.0 and lib.oracle_lerp(2.0, 10.0, 1.0) == 10.0
    assert lib.oracle_smoothstep(0.0, 1.0, 0.5) == 0.5  # 3t^2 - 2t^3
    assert lib.oracle_smoothstep(0.0, 2.0, 0.5) == pytest.approx(3 * 0.25**2 - 2 * 0.25**3)
    assert lib.oracle_smoothstep(0.0, 1.0, -3.0) == 0.0 and lib.oracle_smoothstep(0.0, 1.0, 7.0) == 1.0


def test_max_min_nan_order(lib):
    """max(a, b) = a > b ? a : b: a NaN in the second slot wins, in the first it loses."""
    nan = float("nan")
    assert np.isnan(lib.oracle_max_f(1.0, nan)) and lib.oracle_max_f(nan, 1.0) == 1.0
    assert np.isnan(lib.oracle_min_f(1.0, nan)) and lib.oracle_min_f(nan, 1.0) == 1.0


def test_reinterpretation_is_bitwise(lib):
    for f in (0.0, -0.0, 1.0, -2.5, 3.4028235e38, 1e-45):
        bits = struct.unpack("<I", struct.pack("<f", f))[0]
        assert lib.oracle_asuint_f(f) == bits
        assert struct.pack("<f", lib.oracle_asfloat_u(bits)) == struct.pack("<f", f)


@pytest.mark.parametrize("shape,group", [((5,), (256,)), ((1000,), (256,)), ((17, 33), (16, 16)), ((3, 40, 9), (8, 8, 8)),
                                          ((4, 5, 17, 33), (8, 8, 8)), ((7, 100), (128,)), ((2, 3), (3, 16))])
def test_work_group_count_by_brute_force(lib, shape, group):
    """Count the distinct thread-groups that the threads of the dispatch fall into: outer dimensions are not
    grouped, group[i] tiles shape[dim-1-i]."""
    dim, gdim = len(shape), len(group)
    groups = set()
    for idx in itertools.product(*[range(s) for s in shape]):
        key = tuple(idx[: dim - gdim]) + tuple(idx[dim - 1 - i] // group[i] for i in range(gdim))
        groups.add(key)
    got = lib.oracle_work_group_count((C.c_size_t * dim)(*shape), dim, (C.c_size_t * gdim)(*group), gdim)
    assert got == len(groups)
