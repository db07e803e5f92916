"""Device runtime through the C ABI: memory, JIT kernels with the generated-kernel signature, events."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

KERNEL = r'''
struct Vars { int n; float scale; unsigned _kernel_block_offset; };
extern "C" __global__ void kernel_0(unsigned* out_mem, unsigned* in_mem, Vars var) {
  int block_id = (int)(blockIdx.x + var._kernel_block_offset);
  int i = block_id * 256 + (int)threadIdx.x;
  if (i < var.n) out_mem[i] = __float_as_uint(__uint_as_float(in_mem[i]) * var.scale);
}
'''


def test_device_is_mi355x(rt):
    info = rt.device_info()
    assert "gfx950" in info["name"]
    assert info["compute_units"] >= 200


def test_roundtrip_and_offsets(rt):
    a = np.arange(1000, dtype=np.uint32)
    b = rt.DeviceBuffer.from_numpy(a)
    assert np.array_equal(b.numpy(np.uint32), a)
    b.write(np.array([7, 8, 9], np.uint32), offset_words=10)
    assert list(b.numpy(np.uint32, (5,), offset_words=9)) == [9, 7, 8, 9, 13]
    b.fill(0xDEADBEEF)
    assert np.all(b.numpy(np.uint32) == 0xDEADBEEF)
    # dtype coercions of the upload path: f64->f32, i64->i32, bool->u32
    assert rt.DeviceBuffer.from_numpy(np.array([1.5, 2.5])).numpy(np.float32).tolist() == [1.5, 2.5]
    assert rt.DeviceBuffer.from_numpy(np.array([-1, 2])).numpy(np.int32).tolist() == [-1, 2]
    assert rt.DeviceBuffer.from_numpy(np.array([True, False])).numpy(np.uint32).tolist() == [1, 0]


def test_jit_kernel_launch(rt):
    n = 100_000
    x = np.random.default_rng(1).normal(size=n).astype(np.float32)
    xb = rt.DeviceBuffer.from_numpy(x)
    ob = rt.DeviceBuffer(n)
    k = rt.Kernel(KERNEL, "kernel_0")
    scale = np.float32(2.5)
    k.launch((n + 255) // 256, (256,), [ob, xb], [n, scale.view(np.uint32), 0])
    assert np.array_equal(ob.numpy(np.float32), x * scale)
    # block offset: second half only
    ob.fill(0)
    half = ((n + 255) // 256) // 2
    k.launch((n + 255) // 256 - half, (256,), [ob, xb], [n, scale.view(np.uint32), half])
    got = ob.numpy(np.float32)
    assert np.all(got[: half * 256] == 0) and np.array_equal(got[half * 256:], (x * scale)[half * 256:])


def test_launch_errors(rt):
    k = rt.Kernel(KERNEL, "kernel_0")
    xb = rt.DeviceBuffer(4)
    with pytest.raises(rt.TFHipError):
        k.launch(1, (2048,), [xb, xb], [4, 0, 0])
    with pytest.raises(rt.TFHipError):
        rt.Kernel("this is not HIP", "kernel_0")


def test_events_time_the_stream(rt):
    xb = rt.DeviceBuffer(1 << 24)
    e0, e1 = rt.Event(), rt.Event()
    e0.record()
    for _ in range(10):
        xb.fill(1)
    e1.record()
    ms = e0.elapsed_ms(e1)
    assert 0.0 < ms < 1000.0


def test_out_of_memory_is_an_error_not_a_crash(rt):
    with pytest.raises(rt.TFHipError):
        rt.DeviceBuffer(1 << 40)  # 4 TiB
    # the runtime stays usable
    assert rt.DeviceBuffer.from_numpy(np.ones(4, np.float32)).numpy().sum() == 4


def test_large_copies_through_the_staging_buffers(rt):
    """Copies of 1 MiB and more are cut into 8 MiB chunks through two pinned buffers: odd sizes, an offset, one,
    two and several chunks, and a small copy in between; sizes whose bytes do not divide evenly among the threads that
    copy a chunk's slices (eight by default: 4 bytes over a multiple of 8 x 4096, as a whole copy and as the last chunk
    of 4095 x 4095 words)."""
    rng = np.random.default_rng(5)
    for n_words in (1 << 18, (2 << 20) + 3, (4 << 20) + 1, (11 << 20) + 12345, 8192 * 40 + 1, 4095 * 4095):
        data = rng.integers(0, 2**32, n_words, dtype=np.uint32)
        buf = rt.DeviceBuffer(n_words + 7)
        buf.write(data, offset_words=7)
        buf.write(np.arange(7, dtype=np.uint32))
        assert np.array_equal(buf.numpy(np.uint32, (n_words,), offset_words=7), data)
        assert buf.numpy(np.uint32, (7,)).tolist() == list(range(7))
        assert np.array_equal(buf.numpy(np.uint32), np.concatenate([np.arange(7, dtype=np.uint32), data]))
        buf.free()


def _scratch_info():
    import ctypes as C

    from tensorfrost_amd._lib import call

    b, r, g = C.c_size_t(), C.c_size_t(), C.c_size_t()
    call("tfhip_scratch_info", C.byref(b), C.byref(r), C.byref(g))
    return b.value, r.value, g.value


def test_scratch_that_grows_under_a_live_graph_stays_valid_for_it(rt):
    """A recorded graph carries the scratch address of its day (here the status words of a prefix sum and the
    histograms of a sort). Eager work that outgrows that scratch must not free it while the graph lives: the old
    buffer is parked, the graph replays bit-exact, and the last graph to be destroyed releases it."""
    from tensorfrost_amd._lib import call

    rng = np.random.default_rng(11)
    n = 300_000
    x = rng.integers(0, 2**32, n, dtype=np.uint32)
    keys = rng.integers(0, 2**32, n, dtype=np.uint32)
    xb, ob = rt.DeviceBuffer.from_numpy(x), rt.DeviceBuffer(n)
    kb, vb = rt.DeviceBuffer.from_numpy(keys), rt.DeviceBuffer.from_numpy(np.arange(n, dtype=np.uint32))
    ko, vo = rt.DeviceBuffer(n), rt.DeviceBuffer(n)
    # the same work once, eagerly: sizes the scratch and gives the expected result
    rt.scan_inclusive(xb, ob, n)
    rt.radix_sort_kv(kb, vb, ko, vo, n)
    rt.synchronize()
    want_scan, want_keys, want_vals = ob.numpy(np.uint32), ko.numpy(np.uint32), vo.numpy(np.uint32)
    order = np.argsort(keys, kind="stable")
    assert np.array_equal(want_keys, keys[order]) and np.array_equal(want_vals, order.astype(np.uint32))
    bytes_before, retired_before, graphs_before = _scratch_info()
    g = rt.Graph()
    with g:
        rt.scan_inclusive(xb, ob, n)
        rt.radix_sort_kv(kb, vb, ko, vo, n)
    assert _scratch_info()[2] == graphs_before + 1
    # eager work with a larger need: the scratch buffer moves
    call("tfhip_scratch_reserve", bytes_before + (8 << 20))
    bytes_after, retired_after, _ = _scratch_info()
    assert bytes_after > bytes_before and retired_after == retired_before + 1
    big = rt.DeviceBuffer.from_numpy(rng.integers(0, 2**32, 3_000_000, dtype=np.uint32))
    big_out = rt.DeviceBuffer(big.n_words)
    rt.scan_inclusive(big, big_out, big.n_words)  # eager work in the new scratch
    for _ in range(3):
        ob.fill(0); ko.fill(0); vo.fill(0)
        g.launch()
        rt.synchronize()
        assert np.array_equal(ob.numpy(np.uint32), want_scan)
        assert np.array_equal(ko.numpy(np.uint32), want_keys) and np.array_equal(vo.numpy(np.uint32), want_vals)
    g.destroy()
    if graphs_before == 0:
        assert _scratch_info()[1] == 0  # the last graph released the parked buffers


def test_a_given_up_wait_is_reported_by_every_call_that_waits(rt):
    """The word a look-back kernel sets when it gives up its bounded wait is written through the test hook; each call
    that waits for the stream must report it once and clear it. No kernel waits or misbehaves for this."""
    from tensorfrost_amd._lib import TFHipError, call

    buf = rt.DeviceBuffer.from_numpy(np.arange(16, dtype=np.uint32))
    big = rt.DeviceBuffer(1 << 20)  # 4 MiB: the staged copy path
    host_big = np.zeros(1 << 20, np.uint32)
    ev0, ev1 = rt.Event(), rt.Event()
    ev0.record(); ev1.record()
    waits = {
        "tfhip_sync": lambda: rt.synchronize(),
        "tfhip_d2h": lambda: buf.numpy(np.uint32),
        "tfhip_d2h staged": lambda: big.numpy(np.uint32),
        "tfhip_h2d": lambda: buf.write(np.arange(16, dtype=np.uint32)),
        "tfhip_h2d staged": lambda: big.write(host_big),
        "tfhip_event_elapsed_ms": lambda: ev0.elapsed_ms(ev1),
        "tfhip_free": lambda: rt.DeviceBuffer(64).free(),
    }
    for name, wait in waits.items():
        call("tfhip_test_raise_async_error", 1)
        with pytest.raises(TFHipError, match="gave up a bounded wait"):
            wait()
        wait()  # cleared: the next call is clean
    rt.synchronize()


@pytest.mark.parametrize("n,spins", [(5 * 32768 + 100, 16), (64 * 32768, 1), (2 * 32768, 4096), (40 * 32768 + 7, 4096)])
def test_lookback_gives_up_when_a_tile_never_publishes(rt, n, spins):
    """The bounded wait of the one-pass scan, forced from the host: tickets start at 1, so tile 0 is never published.
    Every look-back that reaches it runs out of polls, reports through the error word and goes on; every group stores
    its tile and exits (nothing hangs), the next waiting call reports the given-up wait once, and the ordinary scan on
    the same buffers is right afterwards."""
    from tensorfrost_amd._lib import TFHipError, call

    tile = 32768  # elements per tile of the one-pass scan (1024 threads x 8 vectors of 4)
    rng = np.random.default_rng(n)
    x = rng.integers(0, 1000, n, dtype=np.uint32)
    src = rt.DeviceBuffer.from_numpy(x)
    out = rt.DeviceBuffer(n)
    out.fill(0xDEADBEEF)
    call("tfhip_test_scan_u32_first_tile_absent", src.ptr, out.ptr, n, spins)
    with pytest.raises(TFHipError, match="gave up a bounded wait"):
        rt.synchronize()
    rt.synchronize()  # reported once
    got = out.numpy(np.uint32)
    assert np.all(got[:tile] == 0xDEADBEEF)  # nobody ran tile 0
    # tile 1 went on with an empty prefix
    assert np.array_equal(got[tile:2 * tile], np.cumsum(x[tile:2 * tile], dtype=np.uint32))
    # its successors store their tiles too: each one's values rise by its own elements from whatever prefix it took
    later = got[2 * tile:].astype(np.int64)
    steps = np.diff(later) % (1 << 32)
    inside = (np.arange(2 * tile + 1, n) % tile) != 0
    assert np.array_equal(steps[inside], x[2 * tile + 1:][inside].astype(np.int64))
    if spins >= 4096:
        # with a wait this long only tile 0 is ever given up on: everything chains on what tile 1 published
        assert np.array_equal(got[tile:], np.cumsum(x[tile:], dtype=np.uint32))
    rt.scan_inclusive(src, out, n)
    rt.synchronize()
    assert np.array_equal(out.numpy(np.uint32), np.cumsum(x, dtype=np.uint32))
    with pytest.raises(TFHipError, match="needs 2"):
        call("tfhip_test_scan_u32_first_tile_absent", src.ptr, out.ptr, tile, spins)
    with pytest.raises(TFHipError, match="spin limit"):
        call("tfhip_test_scan_u32_first_tile_absent", src.ptr, out.ptr, n, 0)
    src.free()
    out.free()


@pytest.mark.parametrize("helpers", [1, 2, 6, 15])
def test_large_copies_with_other_numbers_of_copying_threads(helpers):
    """TFHIP_COPY_HELPERS is read once per process, so each count runs in a process of its own: copies whose bytes do not
    divide among helpers + 1 threads (a remainder of 4 to 60 bytes behind whole 4 KiB slices), both ways, with an offset."""
    import subprocess
    import sys
    from pathlib import Path

    script = r"""
import sys
import numpy as np
sys.path.insert(0, sys.argv[1])
from tensorfrost_amd import runtime as rt
rt.initialize(0)
parts = int(sys.argv[2]) + 1
rng = np.random.default_rng(parts)
for extra_words in (1, 3, 7, 15):
    for base in (4096 * parts * 256 // 4, (9 << 20) // 4 // parts * parts):
        n = base + extra_words
        data = rng.integers(0, 2**32, n, dtype=np.uint32)
        buf = rt.DeviceBuffer(n + 5)
        buf.write(data, offset_words=5)
        assert np.array_equal(buf.numpy(np.uint32, (n,), offset_words=5), data), (parts, n)
        buf.free()
print("ok")
"""
    root = str(Path(__file__).resolve().parents[1])
    env = dict(__import__("os").environ, TFHIP_COPY_HELPERS=str(helpers))
    out = subprocess.run([sys.executable, "-c", script, root, str(helpers)], capture_output=True, text=True, timeout=110, env=env)
    assert out.returncode == 0 and out.stdout.strip().endswith("ok"), out.stdout + out.stderr
