"""The tensor memory pool against the reference's own object code.

TensorFrost/Backend/TensorMemory.cpp compiles here from its own source file with nothing added, so
oracle/ref/Makefile builds it -- unmodified, where it lies in the reference tree -- together with a small driver into
oracle/_ref/libref_pool.so. The same driver source is compiled here against this repository's restatement of the pool
(tensorfrost_amd/csrc/host/tf_memory.{h,cpp}); both are fed the same random traces of allocations and releases.

Which buffer serves a request depends on the iteration order of std::unordered_set<TFBuffer*>, i.e. on the buffers'
addresses, so the driver puts the n-th buffer a pool creates at arena + n * stride: both pools, run one after the other
on the same arena, see the same addresses and can be compared buffer for buffer -- the ordinal of the buffer that serves
every request, whether it was created for it, which buffers were evicted during the call, every live buffer's
size / used_size / time_since_used, and the pool's allocated and unused totals (TensorMemory.cpp:29-55,104-118,145-224).

Build container only: skipped where neither the reference tree nor a prebuilt oracle/_ref/libref_pool.so is present.
"""
import ctypes
import os
import shutil
import subprocess
from pathlib import Path

import numpy as np
import pytest

ROOT = Path(__file__).resolve().parent.parent
REFERENCE = Path("/root/reference/TensorFrost")
REF_LIB = ROOT / "oracle" / "_ref" / "libref_pool.so"
HOST = ROOT / "tensorfrost_amd" / "csrc" / "host"
SLOTS = 4096


def _bind(path):
    lib = ctypes.CDLL(str(path), mode=os.RTLD_NOW | os.RTLD_LOCAL)
    lib.pool_create.restype = ctypes.c_void_p
    lib.pool_create.argtypes = [ctypes.c_void_p, ctypes.c_size_t, ctypes.c_size_t]
    lib.pool_alloc.restype = ctypes.c_long
    lib.pool_alloc.argtypes = [ctypes.c_void_p, ctypes.c_size_t, ctypes.POINTER(ctypes.c_int), ctypes.POINTER(ctypes.c_long), ctypes.c_size_t,
                               ctypes.POINTER(ctypes.c_size_t)]
    lib.pool_free.restype = None
    lib.pool_free.argtypes = [ctypes.c_void_p, ctypes.c_long]
    lib.pool_buffer.restype = None
    lib.pool_buffer.argtypes = [ctypes.c_void_p, ctypes.c_long] + [ctypes.POINTER(ctypes.c_size_t)] * 3
    for name in ("pool_allocated_words", "pool_unused_words"):
        getattr(lib, name).restype = ctypes.c_size_t
        getattr(lib, name).argtypes = [ctypes.c_void_p]
    lib.pool_buffer_stride.restype = ctypes.c_size_t
    return lib


@pytest.fixture(scope="module")
def reference_pool():
    if (REFERENCE / "Backend" / "TensorMemory.cpp").exists() and shutil.which("make") and shutil.which("g++"):
        run = subprocess.run(["make", "-C", str(ROOT / "oracle" / "ref")], capture_output=True, text=True)
        assert run.returncode == 0, run.stdout[-2000:] + run.stderr[-4000:]
    if not REF_LIB.exists():
        pytest.skip("needs the reference tree (build container) or a prebuilt oracle/_ref/libref_pool.so")
    return _bind(REF_LIB)


@pytest.fixture(scope="module")
def own_pool(tmp_path_factory):
    out = tmp_path_factory.mktemp("pool") / "libown_pool.so"
    cmd = ["g++", "-std=c++17", "-O1", "-g", "-shared", "-fPIC", f"-I{HOST}", f"-I{ROOT / 'include'}", "-o", str(out),
           str(ROOT / "oracle" / "ref" / "pool_trace_driver.cpp"), str(HOST / "tf_memory.cpp")]
    run = subprocess.run(cmd, capture_output=True, text=True)
    assert run.returncode == 0, run.stderr[-4000:]
    return _bind(out)


def make_trace(seed, steps, sizes, live_target, idle_bursts):
    """('alloc', words) / ('free', k-th live buffer in allocation order) steps. `sizes`: the size classes requests are
    drawn from; live_target: how many buffers the trace tends to keep alive; idle_bursts: now and then the trace stops
    using a size for longer than the eviction delay, which is what makes buffers expire and delays adapt."""
    rng = np.random.default_rng(seed)
    if live_target == 0:  # a fixed cycle: allocate every size, release them in allocation order
        cycle = [("alloc", int(s)) for s in sizes] + [("free", 0)] * len(sizes)
        return (cycle * (steps // len(cycle) + 1))[:steps // len(cycle) * len(cycle)]
    trace, live = [], 0
    banned, until = None, 0
    for step in range(steps):
        if idle_bursts and step >= until and rng.random() < 0.01:
            banned, until = int(rng.integers(len(sizes))), step + int(rng.integers(100, 400))
        if step >= until:
            banned = None
        if live and (live >= live_target or rng.random() < 0.45):
            trace.append(("free", int(rng.integers(live))))
            live -= 1
        else:
            k = int(rng.integers(len(sizes)))
            if banned is not None and k == banned:
                k = (k + 1) % len(sizes)
            trace.append(("alloc", int(sizes[k])))
            live += 1
    return trace


def replay(lib, trace, arena, stride):
    """Runs the trace; returns one record per step and the largest number of buffers created."""
    pool = lib.pool_create(ctypes.addressof(arena), stride, SLOTS)
    assert pool
    live, alive, records = [], set(), []
    created = ctypes.c_int()
    evicted = (ctypes.c_long * 256)()
    n_evicted = ctypes.c_size_t()
    a, b, c = ctypes.c_size_t(), ctypes.c_size_t(), ctypes.c_size_t()
    stats = {"created": 0, "reused": 0, "evicted": 0, "reused_larger": 0}
    for op, arg in trace:
        if op == "alloc":
            ordinal = lib.pool_alloc(pool, arg, ctypes.byref(created), evicted, len(evicted), ctypes.byref(n_evicted))
            assert ordinal >= 0, "the pool threw"
            gone = sorted(evicted[i] for i in range(n_evicted.value))
            alive.add(ordinal)
            alive -= set(gone)
            live.append(ordinal)
            stats["created" if created.value else "reused"] += 1
            stats["evicted"] += len(gone)
            record = ["alloc", arg, ordinal, created.value, tuple(gone)]
        else:
            ordinal = live.pop(arg)
            lib.pool_free(pool, ordinal)
            record = ["free", ordinal]
        state = []
        for o in sorted(alive):
            lib.pool_buffer(pool, o, ctypes.byref(a), ctypes.byref(b), ctypes.byref(c))
            state.append((o, a.value, b.value, c.value))
            if op == "alloc" and o == record[2] and a.value > arg:
                stats["reused_larger"] += 1
        record += [tuple(state), lib.pool_allocated_words(pool), lib.pool_unused_words(pool)]
        records.append(tuple(record))
    return records, stats


TRACES = [
    # few size classes, many buffers of each: reuse within a class, ties between unused buffers of different ages
    dict(seed=1, steps=6000, sizes=[64, 64, 4096, 1 << 20], live_target=12, idle_bursts=True),
    # sizes spread over more than 16x: the [n, 16n] window, smallest fitting class first
    dict(seed=2, steps=6000, sizes=[3, 17, 40, 100, 640, 1000, 5000, 16000, 70000, 1 << 18], live_target=10, idle_bursts=True),
    # powers of two and their neighbours: boundaries of the window (n, 16n, 16n + 1)
    dict(seed=3, steps=6000, sizes=[16, 17, 255, 256, 257, 4096, 4097, 65536], live_target=8, idle_bursts=True),
    # a steady loop, as a program that is called again and again: four buffers, created once, nothing ever expires
    dict(seed=4, steps=3000, sizes=[1 << 22, 1 << 22, 1 << 16, 4096], live_target=0, idle_bursts=False),
    # long idle gaps: delays grow (allocation_delay adapts up to 32768), buffers expire, classes are re-created
    dict(seed=5, steps=20000, sizes=[128, 1000, 30000], live_target=5, idle_bursts=True),
]


@pytest.mark.parametrize("spec", TRACES, ids=[f"trace{t['seed']}" for t in TRACES])
def test_the_pool_makes_the_reference_pools_decisions(reference_pool, own_pool, spec):
    stride = reference_pool.pool_buffer_stride()
    assert own_pool.pool_buffer_stride() == stride
    trace = make_trace(**spec)
    arena = ctypes.create_string_buffer(stride * SLOTS + 64)
    want, stats = replay(reference_pool, trace, arena, stride)
    ctypes.memset(arena, 0, len(arena))
    got, _ = replay(own_pool, trace, arena, stride)
    for step, (w, g) in enumerate(zip(want, got)):
        assert w == g, f"step {step} ({trace[step]}):\n  reference: {w[:5]}\n  here:      {g[:5]}\n  reference state: {w[-3]}\n  here:            {g[-3]}"
    # the trace exercised what it is meant to
    if spec["live_target"] == 0:
        assert stats["created"] == len(spec["sizes"]) and stats["evicted"] == 0 and stats["reused"] > 1000
        return
    assert stats["reused"] > 100 and stats["created"] > 5
    assert stats["reused_larger"] > 0 or len(set(spec["sizes"])) <= 3
    assert stats["evicted"] > 0, "no buffer ever expired in this trace"
