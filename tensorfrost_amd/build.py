"""Builds the native libraries of this package in-tree with hipcc / g++ (no cmake, no JIT cache).

    python -m tensorfrost_amd.build            # everything
    python -m tensorfrost_amd.build --only tfhip

Outputs:
    tensorfrost_amd/lib/libtfhip.so    device runtime + hand-written gfx950 kernels (C ABI: include/tfhip.h)
    tensorfrost_amd/lib/libtfhost.so   C++ host side: memory/kernel managers, HIP emitter, program driver
"""
from __future__ import annotations

import argparse
import concurrent.futures
import os
import shutil
import subprocess
import sys
from pathlib import Path

PKG = Path(__file__).resolve().parent
ROOT = PKG.parent
CSRC = PKG / "csrc"
LIB = PKG / "lib"
OBJ = PKG / "lib" / "obj"
ROCM = Path(os.environ.get("ROCM_PATH", "/opt/rocm"))

# Packed fp32 VALU forms are disabled for every device translation unit.
HIP_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fno-gpu-rdc",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-result", "-Wno-unused-value", "-Wno-unknown-warning-option",
    f"-I{ROOT / 'include'}", f"-I{CSRC}",
]
HOST_FLAGS = ["-O2", "-std=c++17", "-fPIC", "-Wall", "-Wno-unused-function", f"-I{ROOT / 'include'}", f"-I{CSRC}"]


def _hipcc() -> str:
    exe = shutil.which("hipcc") or str(ROCM / "bin" / "hipcc")
    if not Path(exe).exists():
        raise RuntimeError("hipcc not found; the HIP libraries of tensorfrost_amd cannot be built")
    return exe


def _run(cmd: list[str]) -> None:
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        raise RuntimeError("command failed: " + " ".join(cmd) + "\n" + proc.stdout)
    # hipcc's host pass does not know the device-only target feature; that warning is expected.
    noise = ("is not a recognized feature for this target", "warning generated", "warnings generated")
    out = "\n".join(l for l in proc.stdout.splitlines() if l.strip() and not any(n in l for n in noise))
    if out.strip():
        print(out)


def _compile_all(jobs: list[tuple[list[str], Path]], workers: int) -> None:
    with concurrent.futures.ThreadPoolExecutor(max_workers=workers) as pool:
        futs = [pool.submit(_run, cmd) for cmd, _ in jobs]
        for f in futs:
            f.result()


def build_tfhip(workers: int = 8) -> Path:
    """hipcc every csrc/*.hip to an object, then link libtfhip.so."""
    hipcc = _hipcc()
    OBJ.mkdir(parents=True, exist_ok=True)
    srcs = sorted(CSRC.glob("*.hip"))
    jobs = []
    objs = []
    for src in srcs:
        obj = OBJ / (src.stem + ".o")
        objs.append(obj)
        jobs.append(([hipcc, *HIP_FLAGS, "-c", str(src), "-o", str(obj)], obj))
    _compile_all(jobs, workers)
    out = LIB / "libtfhip.so"
    _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", str(out), *map(str, objs),
          f"-L{ROCM / 'lib'}", "-lhiprtc", "-ldl", "-lpthread", f"-Wl,-rpath,{ROCM / 'lib'}"])
    return out


def build_tfhost(workers: int = 8) -> Path | None:
    """g++ every csrc/host/*.cpp and link libtfhost.so against libtfhip.so."""
    host_dir = CSRC / "host"
    srcs = sorted(host_dir.rglob("*.cpp")) if host_dir.exists() else []
    if not srcs:
        return None
    gxx = shutil.which("g++") or "g++"
    obj_dir = OBJ / "host"
    obj_dir.mkdir(parents=True, exist_ok=True)
    jobs, objs = [], []
    for src in srcs:
        obj = obj_dir / ("_".join(src.relative_to(host_dir).with_suffix("").parts) + ".o")
        objs.append(obj)
        jobs.append(([gxx, *HOST_FLAGS, f"-I{host_dir}", "-c", str(src), "-o", str(obj)], obj))
    _compile_all(jobs, workers)
    out = LIB / "libtfhost.so"
    _run([gxx, "-shared", "-fPIC", "-o", str(out), *map(str, objs), f"-L{LIB}", "-ltfhip", "-ldl", "-lpthread",
          "-Wl,-rpath,$ORIGIN", f"-Wl,-rpath,{ROCM / 'lib'}"])
    return out


def build_test_programs(workers: int = 8) -> Path | None:
    """g++ tests/programs/*.cpp (the op-by-op programs of the test suite) into tests/programs/libtftestprograms.so,
    which registers them with libtfhost.so when tfhost_load_programs loads it. Not part of the product library."""
    src_dir = ROOT / "tests" / "programs"
    srcs = sorted(src_dir.glob("*.cpp")) if src_dir.exists() else []
    if not srcs:
        return None
    gxx = shutil.which("g++") or "g++"
    host_dir = CSRC / "host"
    obj_dir = OBJ / "test_programs"
    obj_dir.mkdir(parents=True, exist_ok=True)
    jobs, objs = [], []
    for src in srcs:
        obj = obj_dir / (src.stem + ".o")
        objs.append(obj)
        jobs.append(([gxx, *HOST_FLAGS, f"-I{host_dir}", f"-I{host_dir / 'programs'}", "-c", str(src), "-o", str(obj)], obj))
    _compile_all(jobs, workers)
    out = src_dir / "libtftestprograms.so"
    _run([gxx, "-shared", "-fPIC", "-o", str(out), *map(str, objs), f"-L{LIB}", "-ltfhost", "-ltfhip",
          f"-Wl,-rpath,{LIB}", "-Wl,-rpath,$ORIGIN/../../tensorfrost_amd/lib", f"-Wl,-rpath,{ROCM / 'lib'}"])
    return out


def build_all(workers: int = 8) -> list[Path]:
    outs = [build_tfhip(workers)]
    host = build_tfhost(workers)
    if host:
        outs.append(host)
        tests = build_test_programs(workers)
        if tests:
            outs.append(tests)
    return outs


def main(argv: list[str] | None = None) -> int:
    ap = argparse.ArgumentParser(description=__doc__)
    ap.add_argument("--only", choices=["tfhip", "tfhost"], default=None)
    ap.add_argument("-j", type=int, default=min(8, os.cpu_count() or 1))
    args = ap.parse_args(argv)
    if args.only == "tfhip":
        outs = [build_tfhip(args.j)]
    elif args.only == "tfhost":
        # the test suite's programs are compiled against the host library's headers: they follow every rebuild of it
        outs = [build_tfhost(args.j), build_test_programs(args.j)]
        outs = [o for o in outs if o]
    else:
        outs = build_all(args.j)
    for o in outs:
        print("built", o)
    return 0


if __name__ == "__main__":
    sys.exit(main())
