"""What the code generator finds in the kernels of tf.sort.radix (csrc/host/sort_features.cpp), without a GPU.

The `Radix sort` region (Python/TensorFrost/sort.py:74-176) is served by one onesweep call when its data flow and three
kinds of computation in its kernels show that it is a least-significant-digit radix sort over the whole key
(shim/hip_sort_region.cpp). These tests pin the per-kernel half of that: element-wise copies and key maps are
recognised by EVALUATING what a kernel stores as a function of what it loads, digit extractions by their form
(load >> shift) & mask with the shift as a polynomial of the kernel's host scalars, the scatter by its effects. They are
found in the composition however it is cut into kernels, and a scatter kernel that moves anything else is refused."""
import ctypes
import re

import pytest

from conftest import TEST_PROGRAMS

UINT, INT, FLOAT = 1, 2, 0  # TFType values


@pytest.fixture(scope="module")
def features():
    import tensorfrost_amd.host  # noqa: F401  (loads libtfhost, which the test library links against)
    lib = ctypes.CDLL(str(TEST_PROGRAMS), mode=ctypes.RTLD_GLOBAL)
    lib.tftest_sort_features.restype = ctypes.c_long
    lib.tftest_sort_features.argtypes = [ctypes.c_char_p, ctypes.POINTER(ctypes.c_int64), ctypes.c_size_t, ctypes.c_int, ctypes.c_char_p, ctypes.c_size_t]

    def run(name, params, mutate=0):
        out = ctypes.create_string_buffer(1 << 16)
        arr = (ctypes.c_int64 * max(1, len(params)))(*params)
        n = lib.tftest_sort_features(name.encode(), arr, len(params), mutate, out, len(out))
        assert n >= 0, out.value.decode()
        return out.value.decode().strip().split("\n")

    return run


def _scatters(lines):
    return [l for l in lines if "scatter=1" in l]


@pytest.mark.parametrize("key_type,map_in,map_out", [(UINT, 0, 0), (FLOAT, 1, 3), (INT, 2, 2)])
def test_copies_and_key_maps_are_recognised_by_what_they_compute(features, key_type, map_in, map_out):
    lines = features("radix_sort_ir", [key_type, 6, 0])
    # kernel 0: the plain copy; kernel 1: keys = map(copy(keys)); kernel 2: the un-map after the region
    assert "copies=[0<-1 map0 n=1*v0] only=1" in lines[0]
    assert f"copies=[0<-1 map{map_in} n=1*v0] only=1" in lines[1]
    assert f"copies=[0<-1 map{map_out} n=1*v0] only=1" in lines[2]
    # fused into one kernel: two copies, still nothing else
    fused = features("radix_sort_ir", [key_type, 6, 2])
    assert f"copies=[0<-2 map{map_in} n=1*v0][1<-3 map0 n=1*v0] only=1" in fused[1]


@pytest.mark.parametrize("flags", [0, 4, 8, 16, 32, 2 | 4 | 8 | 16 | 32])
@pytest.mark.parametrize("bits", [6, 8, 4])
def test_digit_and_scatter_are_found_however_the_passes_cut_the_composition(features, flags, bits):
    lines = features("radix_sort_ir", [UINT, bits, flags])
    mask = (1 << bits) - 1
    shift = r"1\*v\d" if flags & 4 else rf"{bits}\*v\d"
    scatters = _scatters(lines)
    assert len(scatters) == (2 if flags & 32 else 1)
    for s in scatters:
        assert re.search(rf"scatter=1\[k0<-2 v1<-3 >>{shift}&{mask} n=1\*v0\]", s), s
    # besides the scatter, exactly one kernel per pass set takes a digit of the keys it reads: the histogram, or the
    # kernel that writes the digits as a tensor
    takers = [l for l in lines if re.search(rf"digits=\[b1>>{shift}&{mask}\]", l) and "scatter=0" in l]
    assert len(takers) == (2 if flags & 32 else 1), lines
    # nothing else looks like a copy, a digit or a scatter (the unpack's (word >> 8 * (i % 4)) & 0xFF moves with the thread)
    others = [l for l in lines if l not in scatters and l not in takers and "only=1" not in l]
    assert all("digits= scatter=0" in l and "copies= only=0" in l for l in others), others


@pytest.mark.parametrize("mutate,what", [(1, "values stored at their own element"), (2, "both stores write the value"), (3, "the key is changed on the way"),
                                        (4, "an atomic instead of a store")])
def test_a_kernel_that_does_not_just_move_the_element_is_no_scatter(features, mutate, what):
    assert len(_scatters(features("radix_sort_ir", [UINT, 6, 0]))) == 1
    assert _scatters(features("radix_sort_ir", [UINT, 6, 0], mutate)) == [], what


def test_other_programs_have_no_scatter_and_only_true_copies(features):
    for name, params in [("wave_eq", []), ("mlp", [2]), ("softmax_ir", []), ("reductions_ir", []), ("nbody", []), ("ops", []), ("bitonic_sort", []), ("atomics", []),
                         ("group_reverse", []), ("gathered_updates", [])]:
        lines = features(name, params)
        assert _scatters(lines) == [], name
        # an element-wise kernel that computes anything is no copy: `only=1` needs every store to be map(load) of the same element
        for l in lines:
            if "only=1" in l:
                assert re.search(r"copies=(\[\d+<-\d+ map\d n=[^\]]+\])+ only=1", l), (name, l)
