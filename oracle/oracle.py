"""TEST INFRASTRUCTURE: ctypes loader for liboracle.so plus NumPy-facing wrappers.

The shared object is built by `make -C oracle` (also done by __graft_entry__.build()).
"""
from __future__ import annotations

import ctypes as C
import subprocess
from pathlib import Path

import numpy as np

HERE = Path(__file__).resolve().parent
LIB_PATH = HERE / "liboracle.so"
_lib = None

_OPS = {"sum": 0, "max": 1, "min": 2}
_f32p = np.ctypeslib.ndpointer(dtype=np.float32, flags="C_CONTIGUOUS")
_u32p = np.ctypeslib.ndpointer(dtype=np.uint32, flags="C_CONTIGUOUS")


def build() -> Path:
    subprocess.run(["make", "-C", str(HERE), "-B", "liboracle.so"], check=True, stdout=subprocess.PIPE, stderr=subprocess.STDOUT)
    return LIB_PATH


def load() -> C.CDLL:
    global _lib
    if _lib is None:
        if not LIB_PATH.exists():
            build()
        lib = C.CDLL(str(LIB_PATH))
        lib.oracle_reduce_partial_words.restype = C.c_size_t
        lib.oracle_reduce_partial_words.argtypes = [C.c_size_t, C.c_size_t]
        lib.oracle_reduce_rows_f32.argtypes = [C.c_int, _f32p, _f32p, _f32p, C.c_int, C.c_int]
        lib.oracle_reduce_cols_f32.argtypes = [C.c_int, _f32p, _f32p, _f32p, C.c_int, C.c_int]
        lib.oracle_softmax_rows_f32.argtypes = [_f32p, _f32p, _f32p, _f32p, _f32p, C.c_int, C.c_int]
        _lib = lib
    return _lib


def reduce_rows(op: str, x: np.ndarray) -> np.ndarray:
    lib = load()
    x = np.ascontiguousarray(x, dtype=np.float32)
    R, K = x.shape
    out = np.empty(R, np.float32)
    partial = np.empty(lib.oracle_reduce_partial_words(R, K), np.float32)
    assert lib.oracle_reduce_rows_f32(_OPS[op], x, out, partial, R, K) == 0
    return out


def reduce_cols(op: str, x: np.ndarray) -> np.ndarray:
    lib = load()
    x = np.ascontiguousarray(x, dtype=np.float32)
    K, Cc = x.shape
    out = np.empty(Cc, np.float32)
    partial = np.empty(lib.oracle_reduce_partial_words(Cc, K), np.float32)
    assert lib.oracle_reduce_cols_f32(_OPS[op], x, out, partial, K, Cc) == 0
    return out


def softmax_rows(x: np.ndarray) -> np.ndarray:
    lib = load()
    x = np.ascontiguousarray(x, dtype=np.float32)
    R, K = x.shape
    y = np.empty_like(x)
    row_max = np.empty(R, np.float32)
    row_sum = np.empty(R, np.float32)
    partial = np.empty(lib.oracle_reduce_partial_words(R, K), np.float32)
    assert lib.oracle_softmax_rows_f32(x, y, row_max, row_sum, partial, R, K) == 0
    return y
