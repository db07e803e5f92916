"""ctypes binding of libtfhip.so (C ABI declared in include/tfhip.h).

There is no fallback: if the shared library is missing, loading raises, and every wrapper raises
TFHipError with the library's own message when a call returns a non-zero status.
"""
from __future__ import annotations

import ctypes as C
import re
from pathlib import Path

PKG = Path(__file__).resolve().parent
LIB_PATH = PKG / "lib" / "libtfhip.so"
HEADER = PKG.parent / "include" / "tfhip.h"

_lib = None


class TFHipError(RuntimeError):
    """A libtfhip call failed; the message is tfhip_last_error()."""

    def __init__(self, func: str, status: int, message: str):
        super().__init__(f"{func} failed with status {status}: {message}")
        self.status = status


def declared_symbols(header: Path | None = None) -> list[str]:
    """Names of every function the C headers of the library declare (tfhip.h and the test hooks of tfhip_test.h), or
    those of one given header."""
    headers = [header] if header is not None else [HEADER, HEADER.with_name("tfhip_test.h")]
    names: set[str] = set()
    for h in headers:
        text = re.sub(r"/\*.*?\*/", "", h.read_text(), flags=re.S)
        text = re.sub(r"//[^\n]*", "", text)
        names.update(re.findall(r"\b(tfhip_[a-z0-9_]+)\s*\(", text))
    return sorted(names)


_vp, _sz, _u32, _i = C.c_void_p, C.c_size_t, C.c_uint32, C.c_int
_SIGNATURES = {
    "tfhip_init": [_i],
    "tfhip_shutdown": [],
    "tfhip_device_info": [C.c_char_p, _sz, C.POINTER(_i), C.POINTER(_sz)],
    "tfhip_malloc": [C.POINTER(_vp), _sz],
    "tfhip_free": [_vp],
    "tfhip_h2d": [_vp, _sz, _vp, _sz],
    "tfhip_d2h": [_vp, _vp, _sz, _sz],
    "tfhip_d2d": [_vp, _vp, _sz],
    "tfhip_fill_u32": [_vp, _u32, _sz],
    "tfhip_module_compile": [C.c_char_p, C.c_char_p, C.c_char_p, C.POINTER(_vp)],
    "tfhip_module_get_kernel": [_vp, C.c_char_p, C.POINTER(_vp)],
    "tfhip_module_unload": [_vp],
    "tfhip_launch": [_vp, _u32, _u32, _u32, _u32, C.POINTER(_vp), _sz, C.POINTER(_u32), _sz],
    "tfhip_launch_batch": [_vp, _u32, _u32, _u32, _vp, _sz],
    "tfhip_sync": [],
    "tfhip_range_push": [C.c_char_p],
    "tfhip_range_pop": [],
    "tfhip_graph_begin": [],
    "tfhip_graph_end": [C.POINTER(_vp)],
    "tfhip_graph_node_count": [_vp, C.POINTER(C.c_size_t)],
    "tfhip_graph_launch": [_vp],
    "tfhip_graph_destroy": [_vp],
    "tfhip_scratch_info": [C.POINTER(_sz), C.POINTER(_sz), C.POINTER(_sz)],
    "tfhip_scratch_reserve": [_sz],
    "tfhip_test_raise_async_error": [_u32],
    "tfhip_test_scan_u32_first_tile_absent": [_vp, _vp, _sz, _u32],
    "tfhip_event_create": [C.POINTER(_vp)],
    "tfhip_event_destroy": [_vp],
    "tfhip_event_record": [_vp],
    "tfhip_event_elapsed_ms": [_vp, _vp, C.POINTER(C.c_float)],
    "tfhip_reduce_rows_f32": [_i, _vp, _vp, _sz, _sz],
    "tfhip_reduce_cols_f32": [_i, _vp, _vp, _sz, _sz],
    "tfhip_reduce_cols_slabs_f32": [C.c_int, _vp, _vp, _sz, _sz, _sz],
    "tfhip_softmax_rows_f32": [_vp, _vp, _sz, _sz],
    "tfhip_softmax_rows_stats_f32": [_vp, _vp, _vp, _vp, _sz, _sz],
    "tfhip_log_softmax_rows_f32": [_vp, _vp, _sz, _sz],
    "tfhip_log_softmax_rows_stats_f32": [_vp, _vp, _vp, _vp, _sz, _sz],
    "tfhip_scan_inclusive_u32": [_vp, _vp, _sz],
    "tfhip_scan_inclusive_i32": [_vp, _vp, _sz],
    "tfhip_scan_inclusive_u32_static": [_vp, _vp, _sz],
    "tfhip_scan_inclusive_f32": [_vp, _vp, _sz],
    "tfhip_scan_inclusive_rows_u32": [_vp, _vp, _sz, _sz],
    "tfhip_scan_inclusive_rows_f32": [_vp, _vp, _sz, _sz],
    "tfhip_scan_inclusive_cols_u32": [_vp, _vp, _sz, _sz, _sz],
    "tfhip_scan_inclusive_cols_f32": [_vp, _vp, _sz, _sz, _sz],
    "tfhip_radix_sort_kv": [_i, _vp, _vp, _vp, _vp, _vp, _vp, _sz],
    "tfhip_radix_sort_kv_u32": [_vp, _vp, _vp, _vp, _vp, _vp, _sz],
    "tfhip_sgemm_nn": [_vp, _vp, _vp, _sz, _sz, _sz],
    "tfhip_sgemm_nt": [_vp, _vp, _vp, _sz, _sz, _sz],
    "tfhip_sgemm_tn": [_vp, _vp, _vp, _sz, _sz, _sz],
    "tfhip_sgemm_tn_colsum": [_vp, _vp, _vp, _vp, _sz, _sz, _sz],
    "tfhip_sgemm_fused": [C.c_int, _vp, _vp, _vp, _sz, _sz, _sz, C.c_int, _vp],
    "tfhip_sgemm_batched": [C.c_int, _vp, _vp, _vp, _sz, _sz, _sz, _sz, _sz, _sz, _sz],
}
for _op in ("sum", "max", "min"):
    for _ax in ("rows", "cols"):
        _SIGNATURES[f"tfhip_reduce_{_op}_f32_{_ax}"] = [_vp, _vp, _sz, _sz]


def load() -> C.CDLL:
    """Loads libtfhip.so once and types its entry points. Raises if the library was not built."""
    global _lib
    if _lib is not None:
        return _lib
    if not LIB_PATH.exists():
        raise ImportError(
            f"{LIB_PATH} is missing: build it with `python -m tensorfrost_amd.build` "
            "(tensorfrost_amd has no CPU or PyTorch fallback)")
    lib = C.CDLL(str(LIB_PATH), mode=C.RTLD_GLOBAL)
    lib.tfhip_last_error.restype = C.c_char_p
    lib.tfhip_last_error.argtypes = []
    for name, argtypes in _SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = _i
        fn.argtypes = argtypes
    _lib = lib
    return lib


def check(func: str, status: int) -> None:
    if status != 0:
        msg = load().tfhip_last_error()
        raise TFHipError(func, status, msg.decode("utf-8", "replace") if msg else "")


def call(func: str, *args) -> None:
    """Calls lib.<func>(*args) and raises TFHipError on a non-zero status."""
    check(func, getattr(load(), func)(*args))
