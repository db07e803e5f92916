"""Python face of the device runtime: buffers of 32-bit words, JIT kernels, events, primitives.

Everything here is a thin, typed view of the C ABI in include/tfhip.h; it holds no compute of its
own. Buffers follow the reference's memory model: flat arrays of 32-bit words whose element kind
(float32 / int32 / uint32 / bool-as-word) is only a reinterpretation
(TensorFrost/Backend/CodeGen/Generators.cpp:406-426; upload coercions as
TensorFrost/Frontend/Python/PyTensorMemory.cpp:21-63: f64->f32, i64->i32, u64->u32, bool->u32).
"""
from __future__ import annotations

import ctypes as C

import numpy as np

from . import _lib
from ._lib import TFHipError, call

REDUCE_SUM, REDUCE_MAX, REDUCE_MIN = 0, 1, 2
_REDUCE_OPS = {"sum": REDUCE_SUM, "max": REDUCE_MAX, "min": REDUCE_MIN}

_initialized = False


def initialize(device: int = 0) -> None:
    """Binds the library to one GPU (idempotent)."""
    global _initialized
    call("tfhip_init", device)
    _initialized = True


def shutdown() -> None:
    global _initialized
    call("tfhip_shutdown")
    _initialized = False


def device_info() -> dict:
    name = C.create_string_buffer(256)
    cus, mem = C.c_int(0), C.c_size_t(0)
    call("tfhip_device_info", name, 256, C.byref(cus), C.byref(mem))
    return {"name": name.value.decode(), "compute_units": cus.value, "hbm_bytes": mem.value}


def synchronize() -> None:
    call("tfhip_sync")


def _coerce(arr: np.ndarray) -> np.ndarray:
    """Host array -> contiguous array of a 32-bit element kind, as the reference's upload does."""
    arr = np.asarray(arr)
    k = arr.dtype.kind
    if k == "f":
        arr = arr.astype(np.float32, copy=False)
    elif k == "i":
        arr = arr.astype(np.int32, copy=False)
    elif k == "u":
        arr = arr.astype(np.uint32, copy=False)
    elif k == "b":
        arr = arr.astype(np.uint32)
    else:
        raise TypeError(f"unsupported dtype {arr.dtype}")
    return np.ascontiguousarray(arr)


class DeviceBuffer:
    """An owned device allocation of `n_words` 32-bit words."""

    def __init__(self, n_words: int):
        if n_words <= 0:
            raise ValueError("Trying to allocate a tensor with size 0")
        ptr = C.c_void_p()
        call("tfhip_malloc", C.byref(ptr), n_words)
        self.ptr = ptr.value
        self.n_words = int(n_words)

    @classmethod
    def from_numpy(cls, arr) -> "DeviceBuffer":
        arr = _coerce(arr)
        buf = cls(arr.size)
        buf.write(arr)
        return buf

    def write(self, arr, offset_words: int = 0) -> None:
        arr = _coerce(arr)
        if offset_words + arr.size > self.n_words:
            raise ValueError("write past the end of the buffer")
        call("tfhip_h2d", self.ptr, offset_words, arr.ctypes.data, arr.size)

    def numpy(self, dtype=np.float32, shape=None, offset_words: int = 0) -> np.ndarray:
        dtype = np.dtype(dtype)
        if dtype.itemsize != 4:
            raise TypeError("buffers hold 32-bit words")
        count = self.n_words - offset_words if shape is None else int(np.prod(shape))
        if offset_words + count > self.n_words:
            raise ValueError("read past the end of the buffer")
        out = np.empty(count, dtype=dtype)
        call("tfhip_d2h", out.ctypes.data, self.ptr, offset_words, count)
        return out if shape is None else out.reshape(shape)

    def fill(self, word: int) -> None:
        call("tfhip_fill_u32", self.ptr, word & 0xFFFFFFFF, self.n_words)

    def free(self) -> None:
        if self.ptr:
            ptr, self.ptr = self.ptr, None  # the memory is gone even when the call reports an earlier kernel's error
            call("tfhip_free", ptr)

    def __del__(self):
        try:
            if getattr(self, "ptr", None) and _initialized:
                self.free()
        except Exception:
            pass


class Event:
    def __init__(self):
        h = C.c_void_p()
        call("tfhip_event_create", C.byref(h))
        self.handle = h.value

    def record(self) -> None:
        call("tfhip_event_record", self.handle)

    def elapsed_ms(self, stop: "Event") -> float:
        ms = C.c_float()
        call("tfhip_event_elapsed_ms", self.handle, stop.handle, C.byref(ms))
        return ms.value

    def __del__(self):
        try:
            if getattr(self, "handle", None):
                _lib.load().tfhip_event_destroy(self.handle)
        except Exception:
            pass


class Graph:
    """Everything issued inside the `with` block is recorded instead of run; launch() then enqueues it at once.

        g = Graph()
        with g:
            sort_kv(...)
        g.launch()

    Host copies, synchronize() and free are refused while recording; the recorded work keeps using the same buffers.
    """

    def __init__(self):
        self.handle = None

    def __enter__(self):
        call("tfhip_graph_begin")
        return self

    def __exit__(self, exc_type, exc, tb):
        if exc_type is not None:
            _lib.load().tfhip_graph_end(None)  # abandon the recording, keep the original error
            return False
        h = C.c_void_p()
        call("tfhip_graph_end", C.byref(h))
        self.handle = h.value
        return False

    @property
    def nodes(self) -> int:
        n = C.c_size_t()
        call("tfhip_graph_node_count", self.handle, C.byref(n))
        return n.value

    def launch(self) -> None:
        call("tfhip_graph_launch", self.handle)

    def destroy(self) -> None:
        if self.handle:
            call("tfhip_graph_destroy", self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.destroy()
        except Exception:
            pass


class Kernel:
    """A hiprtc-compiled `extern "C" __global__` function (buffers..., vars struct)."""

    def __init__(self, source: str, name: str, options: str = ""):
        h = C.c_void_p()
        call("tfhip_module_compile", source.encode(), name.encode(), options.encode(), C.byref(h))
        self.handle = h.value
        self.name = name

    def launch(self, grid: int, block, buffers, variables=()) -> None:
        bx, by, bz = (list(block) + [1, 1])[:3]
        ptrs = (C.c_void_p * max(1, len(buffers)))(*[b.ptr if isinstance(b, DeviceBuffer) else b for b in buffers])
        words = np.asarray(list(variables), dtype=np.uint32)
        vars_arr = (C.c_uint32 * max(1, len(words)))(*[int(w) for w in words])
        call("tfhip_launch", self.handle, grid, bx, by, bz, ptrs, len(buffers), vars_arr, len(words))

    def __del__(self):
        try:
            if getattr(self, "handle", None):
                _lib.load().tfhip_module_unload(self.handle)
        except Exception:
            pass


# ---- primitives ---------------------------------------------------------------------------------

def reduce_rows(op: str, x: DeviceBuffer, out: DeviceBuffer, rows: int, cols: int) -> None:
    """out[r] = op over the last axis of the [rows, cols] fp32 matrix in x."""
    call("tfhip_reduce_rows_f32", _REDUCE_OPS[op], x.ptr, out.ptr, rows, cols)


def reduce_cols(op: str, x: DeviceBuffer, out: DeviceBuffer, rows: int, cols: int) -> None:
    """out[c] = op over axis 0 of the [rows, cols] fp32 matrix in x."""
    call("tfhip_reduce_cols_f32", _REDUCE_OPS[op], x.ptr, out.ptr, rows, cols)


def reduce_cols_slabs(op: str, x: DeviceBuffer, out: DeviceBuffer, rows: int, cols: int, rows_per_slab: int) -> None:
    """out[s, c] = op over rows [s*rows_per_slab, (s+1)*rows_per_slab) of column c."""
    call("tfhip_reduce_cols_slabs_f32", _REDUCE_OPS[op], x.ptr, out.ptr, rows, cols, rows_per_slab)


def softmax_rows(x: DeviceBuffer, y: DeviceBuffer, rows: int, cols: int, row_max: DeviceBuffer = None, row_sum: DeviceBuffer = None) -> None:
    """y = softmax of every row of x[rows, cols]; with row_max and row_sum also the rows' maxima and sums of exp(x - max)."""
    if row_max is None and row_sum is None:
        call("tfhip_softmax_rows_f32", x.ptr, y.ptr, rows, cols)
    else:
        call("tfhip_softmax_rows_stats_f32", x.ptr, y.ptr, row_max.ptr if row_max else None, row_sum.ptr if row_sum else None, rows, cols)


def log_softmax_rows(x: DeviceBuffer, y: DeviceBuffer, rows: int, cols: int, row_max: DeviceBuffer = None, row_sum: DeviceBuffer = None) -> None:
    """y = (x - max) - log(sum(exp(x - max))) along every row of x[rows, cols]; with row_max and row_sum also those two."""
    if row_max is None and row_sum is None:
        call("tfhip_log_softmax_rows_f32", x.ptr, y.ptr, rows, cols)
    else:
        call("tfhip_log_softmax_rows_stats_f32", x.ptr, y.ptr, row_max.ptr if row_max else None, row_sum.ptr if row_sum else None, rows, cols)


def scan_inclusive(x: DeviceBuffer, out: DeviceBuffer, n: int, dtype=np.uint32) -> None:
    """out[i] = x[0] + ... + x[i]; dtype picks the u32 / i32 / f32 entry point."""
    kind = np.dtype(dtype).kind
    name = {"u": "tfhip_scan_inclusive_u32", "i": "tfhip_scan_inclusive_i32", "f": "tfhip_scan_inclusive_f32"}[kind]
    call(name, x.ptr, out.ptr, n)


def sgemm_batched(layout: str, a: DeviceBuffer, b: DeviceBuffer, c: DeviceBuffer, m: int, n: int, k: int, batch: int,
                  stride_a: int, stride_b: int, stride_c: int) -> None:
    """`batch` products in one launch; a stride of 0 shares that operand across the batch."""
    call("tfhip_sgemm_batched", {"nn": 0, "nt": 1, "tn": 2}[layout], a.ptr, b.ptr, c.ptr, m, n, k, batch, stride_a, stride_b, stride_c)


def scan_inclusive_cols(x: DeviceBuffer, out: DeviceBuffer, batch: int, rows: int, cols: int, dtype=np.uint32) -> None:
    """Prefix sums down the columns of `batch` row-major [rows, cols] matrices."""
    name = "tfhip_scan_inclusive_cols_f32" if np.dtype(dtype).kind == "f" else "tfhip_scan_inclusive_cols_u32"
    call(name, x.ptr, out.ptr, batch, rows, cols)


def scan_inclusive_rows(x: DeviceBuffer, out: DeviceBuffer, rows: int, cols: int, dtype=np.uint32) -> None:
    """Prefix sums along the last axis of a row-major [rows, cols] matrix, every row on its own."""
    name = "tfhip_scan_inclusive_rows_f32" if np.dtype(dtype).kind == "f" else "tfhip_scan_inclusive_rows_u32"
    call(name, x.ptr, out.ptr, rows, cols)


_KEY_KINDS = {"u": 0, "i": 1, "f": 2}


def radix_sort_kv(keys: DeviceBuffer, vals, keys_out: DeviceBuffer, vals_out, n: int, key_dtype=np.uint32,
                  keys_tmp: DeviceBuffer | None = None, vals_tmp: DeviceBuffer | None = None) -> None:
    """Stable ascending key(/payload) sort; vals / vals_out may be None for a keys-only sort."""
    p = lambda b: b.ptr if b is not None else None
    call("tfhip_radix_sort_kv", _KEY_KINDS[np.dtype(key_dtype).kind], keys.ptr, p(vals), keys_out.ptr, p(vals_out), p(keys_tmp), p(vals_tmp), n)


_EPILOGUES = {None: 0, "bias_relu": 1, "bias": 2, "mask_positive": 3}


def sgemm(layout: str, a: DeviceBuffer, b: DeviceBuffer, c: DeviceBuffer, m: int, n: int, k: int, epilogue=None, aux=None) -> None:
    """C[m,n] = op(A) op(B); layout 'nn' (A[m,k] B[k,n]), 'nt' (A[m,k] B[n,k]) or 'tn' (A[k,m] B[k,n]).
    epilogue: None | 'bias' | 'bias_relu' (aux = bias[n]) | 'mask_positive' (aux[m,n]: keep where aux > 0)."""
    if epilogue is None:
        call({"nn": "tfhip_sgemm_nn", "nt": "tfhip_sgemm_nt", "tn": "tfhip_sgemm_tn"}[layout], a.ptr, b.ptr, c.ptr, m, n, k)
    else:
        call("tfhip_sgemm_fused", {"nn": 0, "nt": 1, "tn": 2}[layout], a.ptr, b.ptr, c.ptr, m, n, k, _EPILOGUES[epilogue], aux.ptr if aux is not None else None)


__all__ = [
    "initialize", "shutdown", "device_info", "synchronize", "DeviceBuffer", "Event", "Kernel",
    "reduce_rows", "reduce_cols", "reduce_cols_slabs", "softmax_rows", "log_softmax_rows", "scan_inclusive", "radix_sort_kv", "sgemm", "TFHipError",
]
