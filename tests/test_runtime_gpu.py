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
    two and several chunks, and a small copy in between."""
    rng = np.random.default_rng(5)
    for n_words in (1 << 18, (2 << 20) + 3, (4 << 20) + 1, (11 << 20) + 12345):
        data = rng.integers(0, 2**32, n_words, dtype=np.uint32)
        buf = rt.DeviceBuffer(n_words + 7)
        buf.write(data, offset_words=7)
        buf.write(np.arange(7, dtype=np.uint32))
        assert np.array_equal(buf.numpy(np.uint32, (n_words,), offset_words=7), data)
        assert buf.numpy(np.uint32, (7,)).tolist() == list(range(7))
        assert np.array_equal(buf.numpy(np.uint32), np.concatenate([np.arange(7, dtype=np.uint32), data]))
        buf.free()
