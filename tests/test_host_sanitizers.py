"""Host C++ under AddressSanitizer and UndefinedBehaviorSanitizer (no GPU): a small driver linked from the host
sources builds every registered program on the code-generation backend -- IR builders, idiom matcher, HIP emitter,
hiprtc acceptance -- and must finish without a sanitizer report."""
import os
import shutil
import subprocess
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
HOST = ROOT / "tensorfrost_amd" / "csrc" / "host"
LIB = ROOT / "tensorfrost_amd" / "lib"


@pytest.mark.skipif(shutil.which("g++") is None, reason="g++ not available")
def test_every_program_builds_cleanly_under_asan_and_ubsan(tmp_path):
    if not (LIB / "libtfhip.so").exists():
        pytest.fail("libtfhip.so has not been built (python __graft_entry__.py)")
    exe = tmp_path / "driver"
    sources = [str(Path(__file__).with_name("host_sanitizer_driver.cpp"))] + sorted(map(str, HOST.rglob("*.cpp"))) + sorted(map(str, (ROOT / "tests" / "programs").glob("*.cpp")))
    cmd = ["g++", "-O1", "-g", "-std=c++17", "-fsanitize=address,undefined", "-fno-sanitize-recover=undefined", "-fno-omit-frame-pointer",
           f"-I{ROOT / 'include'}", f"-I{ROOT / 'tensorfrost_amd' / 'csrc'}", f"-I{HOST}", f"-I{HOST / 'programs'}", f"-I{HOST / 'shim'}", *sources, f"-L{LIB}", "-ltfhip",
           f"-Wl,-rpath,{LIB}", "-Wl,-rpath,/opt/rocm/lib", "-o", str(exe)]
    build = subprocess.run(cmd, capture_output=True, text=True)
    assert build.returncode == 0, build.stderr[-4000:]
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=0:abort_on_error=0", TFHIP_CACHE_DIR=str(tmp_path / "cache"))
    run = subprocess.run([str(exe)], capture_output=True, text=True, env=env, timeout=900)
    report = run.stdout + run.stderr
    assert "runtime error" not in report and "AddressSanitizer" not in report, report[-4000:]
    assert run.returncode == 0, report[-4000:]
    assert "wave_eq(0): 1 kernels" in report and "softmax_ir(0): 5 kernels" in report
