"""The C-ABI library loads on a machine without a GPU and exports everything the headers declare."""
import ctypes as C
import subprocess
from pathlib import Path

import pytest

from tensorfrost_amd import _lib

ROOT = Path(__file__).resolve().parent.parent


def test_exports_every_declared_symbol():
    lib = _lib.load()
    names = _lib.declared_symbols()
    assert len(names) >= 25
    missing = [n for n in names if not hasattr(lib, n)]
    assert not missing, f"declared in include/tfhip.h but not exported: {missing}"


def test_every_declared_symbol_is_typed():
    untyped = [n for n in _lib.declared_symbols() if n not in _lib._SIGNATURES and n != "tfhip_last_error"]
    assert not untyped, f"no ctypes signature for: {untyped}"


def test_calls_fail_loudly_before_init():
    lib = _lib.load()
    ptr = C.c_void_p()
    status = lib.tfhip_malloc(C.byref(ptr), 16)
    assert status == -4  # TFHIP_ERR_STATE
    assert b"tfhip_init" in lib.tfhip_last_error()
    with pytest.raises(_lib.TFHipError):
        _lib.call("tfhip_sync")


def test_abi_struct_layout_compiles(tmp_path):
    """tf_abi.h carries static_asserts for the struct layout of the reference (TensorMemory.h:19-72)."""
    src = tmp_path / "abi.cpp"
    src.write_text('#include "tf_abi.h"\n#include "tfhip.h"\nint main() { return sizeof(TFTensor) == 40 ? 0 : 1; }\n')
    exe = tmp_path / "abi"
    subprocess.run(["g++", "-std=c++17", f"-I{ROOT / 'include'}", str(src), "-o", str(exe)], check=True)
    assert subprocess.run([str(exe)]).returncode == 0
    csrc = tmp_path / "abi.c"
    csrc.write_text('#include "tf_abi.h"\n#include "tfhip.h"\nint main(void) { return sizeof(TFDispatchInfo) == 64 ? 0 : 1; }\n')
    subprocess.run(["gcc", "-std=c11", f"-I{ROOT / 'include'}", str(csrc), "-o", str(exe)], check=True)
    assert subprocess.run([str(exe)]).returncode == 0


KERNEL = r'''
struct Vars { int n; unsigned _kernel_block_offset; };
extern "C" __global__ void kernel_0(unsigned* out_mem, unsigned* in_mem, Vars var) {
  int i = (int)(blockIdx.x + var._kernel_block_offset) * 256 + (int)threadIdx.x;
  if (i < var.n) out_mem[i] = in_mem[i] * 2u + 1u;
}
'''


def test_hiprtc_compiles_for_gfx950_without_a_gpu(tmp_path, monkeypatch):
    monkeypatch.setenv("TFHIP_CACHE_DIR", str(tmp_path))
    lib = _lib.load()
    h = C.c_void_p()
    _lib.call("tfhip_module_compile", KERNEL.encode(), b"kernel_0", b"", C.byref(h))
    assert h.value
    assert list(tmp_path.glob("*.hsaco")), "code object was not cached"
    lib.tfhip_module_unload(h)
    # second time comes from the cache
    _lib.call("tfhip_module_compile", KERNEL.encode(), b"kernel_0", b"", C.byref(h))
    lib.tfhip_module_unload(h)


def test_hiprtc_error_carries_the_log(tmp_path, monkeypatch):
    monkeypatch.setenv("TFHIP_CACHE_DIR", str(tmp_path))
    h = C.c_void_p()
    with pytest.raises(_lib.TFHipError) as e:
        _lib.call("tfhip_module_compile", b'extern "C" __global__ void k() { not_a_symbol(); }', b"k", b"", C.byref(h))
    assert e.value.status == -2
    assert "not_a_symbol" in str(e.value)
