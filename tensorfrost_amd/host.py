"""Python face of libtfhost.so: the calls a TensorFrost user makes, routed to the HIP backend.

    import tensorfrost_amd.host as tf
    tf.initialize(tf.hip)                       # tf.initialize(tf.cpu) in the reference
    wave = tf.compile("wave_eq")                # tf.compile(WaveEq): programs come from a built-in registry
    v, u = wave(v, u)                           # TensorProgram.__call__; numpy arrays are uploaded on the fly
    u.numpy                                     # readback

Mirrors TensorFrost/Frontend/Python/PybindModule.cpp:112-115 (initialize),
Definitions/TensorProgram.cpp:12-150 (compile, __call__), Definitions/TensorMemory.cpp:24-69 (tensor, numpy,
allocated_memory). No computation happens here, and nothing falls back to the CPU.
"""
from __future__ import annotations

import ctypes as C
import re
from pathlib import Path

import numpy as np

from . import _lib

PKG = Path(__file__).resolve().parent
LIB_PATH = PKG / "lib" / "libtfhost.so"
HEADER = PKG.parent / "include" / "tfhost.h"

hip = 0
codegen = 1

float32, uint32, int32, bool32 = 0, 1, 2, 3
_NP_OF_TYPE = {0: np.float32, 1: np.uint32, 2: np.int32, 3: np.uint32}

_lib_host = None


class TFHostError(RuntimeError):
    pass


def declared_symbols() -> list[str]:
    text = re.sub(r"/\*.*?\*/", "", HEADER.read_text(), flags=re.S)
    return sorted(set(re.findall(r"\b(tfhost_[a-z0-9_]+)\s*\(", text)))


def load() -> C.CDLL:
    global _lib_host
    if _lib_host is not None:
        return _lib_host
    _lib.load()  # libtfhip.so first (RTLD_GLOBAL), libtfhost.so links against it
    if not LIB_PATH.exists():
        raise ImportError(f"{LIB_PATH} is missing: build it with `python -m tensorfrost_amd.build`")
    lib = C.CDLL(str(LIB_PATH))
    lib.tfhost_last_error.restype = C.c_char_p
    vp, sz = C.c_void_p, C.c_size_t
    sigs = {
        "tfhost_initialize": [C.c_int, C.c_char_p],
        "tfhost_shutdown": [],
        "tfhost_sync": [],
        "tfhost_program_create": [C.c_char_p, C.POINTER(C.c_int64), sz, C.POINTER(vp)],
        "tfhost_program_destroy": [vp],
        "tfhost_program_kernel_count": [vp, C.POINTER(sz)],
        "tfhost_program_kernel_info": [vp, sz, C.POINTER(C.c_char_p), C.POINTER(C.c_char_p), C.POINTER(C.c_int), C.POINTER(sz)],
        "tfhost_program_host_code": [vp, C.POINTER(C.c_char_p)],
        "tfhost_program_compile_times": [vp, C.POINTER(C.c_float), C.POINTER(C.c_float), C.POINTER(C.c_float)],
        "tfhost_load_programs": [C.c_char_p],
        "tfhost_program_execute": [vp, C.POINTER(vp), sz, C.POINTER(vp), sz, C.POINTER(sz)],
        "tfhost_tensor_create": [C.POINTER(sz), sz, C.c_int, vp, C.POINTER(vp)],
        "tfhost_tensor_info": [vp, C.POINTER(sz), sz, C.POINTER(sz), C.POINTER(C.c_int), C.POINTER(sz)],
        "tfhost_tensor_read": [vp, vp, sz],
        "tfhost_tensor_write": [vp, vp, sz],
        "tfhost_program_record": [vp, C.POINTER(vp), sz, sz, C.POINTER(C.c_int), C.POINTER(vp), sz, C.POINTER(sz), C.POINTER(vp)],
        "tfhost_graph_replay": [vp],
        "tfhost_graph_node_count": [vp, C.POINTER(sz)],
        "tfhost_graph_destroy": [vp],
        "tfhost_tensor_device_pointer": [vp, C.POINTER(vp)],
        "tfhost_tensor_release": [vp],
        "tfhost_memory_stats": [C.POINTER(sz)] * 4,
        "tfhost_dispatch_stats": [C.POINTER(sz)] * 2,
        "tfhost_fused_chain_count": [C.POINTER(sz)],
        "tfhost_batched_launch_stats": [C.POINTER(sz), C.POINTER(sz)],
    }
    for name, argtypes in sigs.items():
        fn = getattr(lib, name)
        fn.restype = C.c_int
        fn.argtypes = argtypes
    _lib_host = lib
    return lib


def _call(name: str, *args) -> None:
    lib = load()
    if getattr(lib, name)(*args) != 0:
        raise TFHostError(lib.tfhost_last_error().decode("utf-8", "replace"))


def initialize(backend: int = hip, kernel_compile_options: str = "") -> None:
    _call("tfhost_initialize", backend, kernel_compile_options.encode())


def shutdown() -> None:
    _call("tfhost_shutdown")


def synchronize() -> None:
    _call("tfhost_sync")


class Tensor:
    """A device tensor (the reference's TensorMemory): shape, 32-bit element kind, pooled buffer."""

    def __init__(self, handle):
        self._h = handle

    @property
    def _info(self):
        shape = (C.c_size_t * 8)()
        dim, words, typ = C.c_size_t(), C.c_size_t(), C.c_int()
        _call("tfhost_tensor_info", self._h, shape, 8, C.byref(dim), C.byref(typ), C.byref(words))
        return tuple(shape[i] for i in range(dim.value)), typ.value, words.value

    @property
    def shape(self):
        return self._info[0]

    @property
    def type(self):
        return self._info[1]

    @property
    def numpy(self) -> np.ndarray:
        shape, typ, words = self._info
        out = np.empty(words, dtype=_NP_OF_TYPE[typ])
        _call("tfhost_tensor_read", self._h, out.ctypes.data, words)
        out = out.reshape(shape)
        return out.astype(bool) if typ == bool32 else out

    def write(self, arr) -> None:
        """Overwrites the tensor in place (same element count; the array is converted to the tensor's 32-bit type)."""
        shape, typ, words = self._info
        arr = np.ascontiguousarray(np.asarray(arr).astype(_NP_OF_TYPE[typ], copy=False))
        if arr.size != words:
            raise ValueError(f"tensor holds {words} elements, array has {arr.size}")
        _call("tfhost_tensor_write", self._h, arr.ctypes.data, words)

    @property
    def device_pointer(self) -> int:
        p = C.c_void_p()
        _call("tfhost_tensor_device_pointer", self._h, C.byref(p))
        return p.value

    def release(self) -> None:
        if self._h:
            _call("tfhost_tensor_release", self._h)
            self._h = None

    def __del__(self):
        try:
            self.release()
        except Exception:
            pass


def tensor(arr) -> Tensor:
    """Uploads a host array (f64->f32, i64->i32, u64->u32, bool->u32, as the reference's upload does)."""
    arr = np.asarray(arr)
    kind = arr.dtype.kind
    if kind == "f":
        arr, typ = arr.astype(np.float32, copy=False), float32
    elif kind == "i":
        arr, typ = arr.astype(np.int32, copy=False), int32
    elif kind == "u":
        arr, typ = arr.astype(np.uint32, copy=False), uint32
    elif kind == "b":
        arr, typ = arr.astype(np.uint32), bool32
    else:
        raise TypeError(f"unsupported dtype {arr.dtype}")
    arr = np.ascontiguousarray(arr)
    shape = (C.c_size_t * max(1, arr.ndim))(*arr.shape)
    h = C.c_void_p()
    _call("tfhost_tensor_create", shape, arr.ndim, typ, arr.ctypes.data, C.byref(h))
    return Tensor(h.value)


class TensorProgram:
    def __init__(self, name: str, params=()):
        p = (C.c_int64 * max(1, len(params)))(*params)
        h = C.c_void_p()
        _call("tfhost_program_create", name.encode(), p, len(params), C.byref(h))
        self._h = h.value
        self.name = name

    def kernels(self) -> list[dict]:
        n = C.c_size_t()
        _call("tfhost_program_kernel_count", self._h, C.byref(n))
        out = []
        for i in range(n.value):
            src, mapping, threads, kid = C.c_char_p(), C.c_char_p(), C.c_int(), C.c_size_t()
            _call("tfhost_program_kernel_info", self._h, i, C.byref(src), C.byref(mapping), C.byref(threads), C.byref(kid))
            out.append({"source": src.value.decode(), "mapping": mapping.value.decode(), "hip_threads": threads.value, "kernel_id": kid.value})
        return out

    def host_code(self) -> str:
        """The host program (checks, allocations, host scalars, dispatches) as the interpreter's instruction list."""
        text = C.c_char_p()
        _call("tfhost_program_host_code", self._h, C.byref(text))
        return text.value.decode()

    def compile_times(self) -> dict:
        """Seconds tf.compile spent building the tree, generating code and compiling the kernels."""
        v = [C.c_float() for _ in range(3)]
        _call("tfhost_program_compile_times", self._h, *[C.byref(x) for x in v])
        return dict(zip(["trace", "codegen", "kernel_compile"], [x.value for x in v]))

    def __call__(self, *inputs):
        temps = []
        handles = []
        for x in inputs:
            if not isinstance(x, Tensor):
                x = tensor(x)
                temps.append(x)
            handles.append(x._h)
        arr = (C.c_void_p * max(1, len(handles)))(*handles)
        outs = (C.c_void_p * 64)()
        n = C.c_size_t()
        _call("tfhost_program_execute", self._h, arr, len(handles), outs, 64, C.byref(n))
        res = tuple(Tensor(outs[i]) for i in range(n.value))
        for t in temps:
            t.release()
        return res[0] if len(res) == 1 else res

    def record(self, *inputs, repeat: int = 1, feedback=None) -> "RecordedProgram":
        """Records `repeat` executions on these input tensors as one HIP graph. feedback[i] names the output that
        becomes input i in the next execution (-1: the input stays), e.g. (1, 0) for wave_eq(u, v) -> (v, u)."""
        for x in inputs:
            if not isinstance(x, Tensor):
                raise TypeError("record() takes device tensors: the graph keeps using their buffers")
        arr = (C.c_void_p * max(1, len(inputs)))(*[x._h for x in inputs])
        outs = (C.c_void_p * 64)()
        n, g = C.c_size_t(), C.c_void_p()
        fb = None
        if feedback is not None:
            if len(feedback) != len(inputs):
                raise ValueError("feedback needs one entry per input")
            fb = (C.c_int * max(1, len(inputs)))(*feedback)
        _call("tfhost_program_record", self._h, arr, len(inputs), repeat, fb, outs, 64, C.byref(n), C.byref(g))
        return RecordedProgram(g.value, inputs, tuple(Tensor(outs[i]) for i in range(n.value)))

    def destroy(self) -> None:
        if self._h:
            _call("tfhost_program_destroy", self._h)
            self._h = None


class RecordedProgram:
    """A program's dispatch sequence on fixed buffers. `inputs` are the caller's tensors (kept alive here), `outputs`
    the tensors every replay writes; with feedback the inputs also hold the latest state after a replay."""

    def __init__(self, handle, inputs, outputs):
        self._h = handle
        self.inputs = tuple(inputs)
        self.outputs = outputs

    @property
    def nodes(self) -> int:
        n = C.c_size_t()
        _call("tfhost_graph_node_count", self._h, C.byref(n))
        return n.value

    def replay(self) -> None:
        _call("tfhost_graph_replay", self._h)

    def destroy(self) -> None:
        if self._h:
            for t in self.outputs:
                t.release()
            _call("tfhost_graph_destroy", self._h)
            self._h = None


def load_programs(library: str | Path) -> None:
    """Adds the programs a shared library registers (e.g. the test suite's tests/programs/libtftestprograms.so)."""
    _call("tfhost_load_programs", str(library).encode())


def compile(name: str, params=()) -> TensorProgram:  # noqa: A001 - mirrors tf.compile
    return TensorProgram(name, params)


def dispatch_stats() -> dict:
    v = [C.c_size_t() for _ in range(2)]
    _call("tfhost_dispatch_stats", *[C.byref(x) for x in v])
    chains = C.c_size_t()
    _call("tfhost_fused_chain_count", C.byref(chains))
    launches, carried = C.c_size_t(), C.c_size_t()
    _call("tfhost_batched_launch_stats", C.byref(launches), C.byref(carried))
    return dict(zip(["dispatches", "served_by_primitives"], [x.value for x in v]), fused_chains=chains.value,
                batched_launches=launches.value, batched_dispatches=carried.value)


def memory_stats() -> dict:
    v = [C.c_size_t() for _ in range(4)]
    _call("tfhost_memory_stats", *[C.byref(x) for x in v])
    return dict(zip(["allocated_words", "unused_words", "buffers_created", "buffers_removed"], [x.value for x in v]))
