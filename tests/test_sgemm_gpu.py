"""Parity of the MFMA fp32 matmul (through the C ABI) with the CPU oracle: 1e-4 relative for matmul, measured
against sum_k |a||b| (the scale a K-term fp32 dot product errs against, in any summation order)."""
import numpy as np
import pytest

from conftest import sum_err
from oracle import oracle

pytestmark = pytest.mark.gpu

# (M, N, K): tile-aligned, ragged in every dimension, below one tile, skinny (plain kernel), K slicing, K = 1
SHAPES = [(128, 128, 16), (256, 256, 256), (130, 70, 33), (32, 32, 5), (1000, 257, 129), (64, 3, 256), (3, 64, 100),
          (1, 1, 1), (256, 256, 20000), (40, 50, 8200), (777, 256, 64),
          # skinny N (bandwidth-bound kernels): output layer 256 -> 3 and its weight gradient, N = 8, ragged K
          (1000, 3, 256), (256, 3, 20000), (512, 8, 1001), (10, 5, 17), (260, 2, 64),
          # matrix times a few vectors: a wave per row, and per K segment when rows are few (unaligned and ragged K too)
          (4096, 1, 4096), (1000, 3, 5000), (3, 2, 100003), (5, 8, 65536), (70000, 8, 1024), (33, 1, 4099), (2, 4, 1 << 20),
          # few rows against a wide B (a batch of 1 .. 32 samples): the transposed skinny problem, eight rows at a time
          (1, 4096, 4096), (8, 1000, 513), (5, 1001, 300), (17, 260, 5000), (32, 128, 64), (2, 256, 70000), (9, 12, 16),
          # short K with many rows (B resident in group memory, A streamed): ragged rows and columns, K = 16 .. 128
          (40000, 64, 64), (33000, 64, 128), (32768 + 17, 50, 128), (50000, 32, 16), (70000, 40, 48), (40000, 33, 24),
          # small result, long K (weight gradients of narrow layers; tn reads both operands straight into the matrix
          # instruction): 1 to 4 block columns per wave, an odd K, 96 rows (three block rows: the tiled kernel instead)
          (64, 64, 5000), (128, 128, 4096), (32, 512, 10001), (64, 256, 20001), (128, 96, 8192), (96, 64, 4100), (32, 32, 70000),
          # exactly tiled by 256 x 128 with enough tiles for the wide kernel
          (65536, 256, 48), (32768, 512, 16),
          # many rows, at most eight columns, K <= 256: the lanes of a wave along k, sums across the wave by halving
          (70000, 3, 256), (65536 + 5, 8, 100), (100000, 1, 16), (66000, 5, 252), (131072, 7, 64), (70001, 2, 128), (66000, 4, 200), (66000, 6, 36)]


def _gemm(rt, layout, a, b, m, n, k):
    ab, bb = rt.DeviceBuffer.from_numpy(a), rt.DeviceBuffer.from_numpy(b)
    cb = rt.DeviceBuffer(m * n)
    rt.sgemm(layout, ab, bb, cb, m, n, k)
    return cb.numpy(np.float32, (m, n))


@pytest.mark.parametrize("mnk", SHAPES)
@pytest.mark.parametrize("layout", ["nn", "nt", "tn"])
def test_sgemm_matches_oracle(rt, layout, mnk):
    m, n, k = mnk
    rng = np.random.default_rng(81)
    a = rng.normal(size=(m, k)).astype(np.float32)
    b = rng.normal(size=(k, n)).astype(np.float32)
    aa = np.ascontiguousarray(a.T) if layout == "tn" else a
    bb = np.ascontiguousarray(b.T) if layout == "nt" else b
    got = _gemm(rt, layout, aa, bb, m, n, k)
    scale = np.abs(a).astype(np.float64) @ np.abs(b).astype(np.float64)
    ref = a.astype(np.float64) @ b.astype(np.float64)
    assert sum_err(got, ref, scale) < 1e-5
    if m * n * k <= 1 << 26:
        assert sum_err(got, oracle.matmul(aa, bb, layout), scale) < 1e-4


def test_sgemm_structure(rt):
    """Distinct integers everywhere (exact in fp32): a transposed tile or a swapped accumulator shows as a
    wrong integer, not as rounding."""
    m, n, k = 192, 160, 48
    a = (np.arange(m * k).reshape(m, k) % 7 - 3).astype(np.float32)
    b = (np.arange(k * n).reshape(k, n) % 5 - 2).astype(np.float32)
    assert np.array_equal(_gemm(rt, "nn", a, b, m, n, k), a @ b)
    assert np.array_equal(_gemm(rt, "nt", a, np.ascontiguousarray(b.T), m, n, k), a @ b)
    assert np.array_equal(_gemm(rt, "tn", np.ascontiguousarray(a.T), b, m, n, k), a @ b)


def test_sgemm_k_zero_and_errors(rt):
    c = rt.DeviceBuffer.from_numpy(np.ones(12, np.float32))
    a = rt.DeviceBuffer(4)
    rt.sgemm("nn", a, a, c, 3, 4, 0)
    assert np.all(c.numpy(np.float32) == 0)
    with pytest.raises(rt.TFHipError):
        rt.sgemm("nn", a, a, c, 0, 4, 4)


def test_sgemm_config5_layer_shape(rt):
    """benchmark config 5 hidden layer at full size: [262144,256] x [256,256], checked on sampled rows against
    float64 and through linearity (A(x+y) = Ax + Ay exactly for integer-valued inputs)."""
    m, n, k = 262144, 256, 256
    rng = np.random.default_rng(82)
    a = rng.normal(size=(m, k)).astype(np.float32)
    b = (rng.normal(size=(k, n)) * np.sqrt(2.0 / k)).astype(np.float32)
    got = _gemm(rt, "nn", a, b, m, n, k)
    rows = rng.integers(0, m, 512)
    ref = a[rows].astype(np.float64) @ b.astype(np.float64)
    scale = np.abs(a[rows]).astype(np.float64) @ np.abs(b).astype(np.float64)
    assert sum_err(got[rows], ref, scale) < 1e-5
    ai = rng.integers(-3, 4, (m, k)).astype(np.float32)
    bi = rng.integers(-3, 4, (k, n)).astype(np.float32)
    gi = _gemm(rt, "nn", ai, bi, m, n, k)
    assert np.array_equal(gi[rows], ai[rows] @ bi)
    assert float(gi.sum(dtype=np.float64)) == float((ai.sum(axis=0, dtype=np.float64) @ bi.astype(np.float64)).sum())


@pytest.mark.parametrize("mnk", [(256, 256, 64), (130, 70, 33), (1000, 3, 256), (10, 5, 17), (40, 50, 8200), (33, 40, 0), (512, 8, 1001), (65536, 256, 32),
                                 (700, 3, 2048), (6, 2, 40000), (7, 64, 100), (20, 300, 2048), (1, 256, 256), (40000, 48, 64),
                                 (70000, 3, 256), (66000, 6, 36)])
@pytest.mark.parametrize("layout", ["nn", "nt", "tn"])
@pytest.mark.parametrize("epilogue", ["bias", "bias_relu", "mask_positive"])
def test_sgemm_fused_epilogues(rt, layout, epilogue, mnk):
    """The element-wise tail fused behind the product: integer-valued operands make every path exact, so the
    result must equal the oracle's matmul followed by the same tail bit for bit."""
    m, n, k = mnk
    rng = np.random.default_rng(83)
    a = rng.integers(-3, 4, (m, k)).astype(np.float32)
    b = rng.integers(-3, 4, (k, n)).astype(np.float32)
    aa = np.ascontiguousarray(a.T) if layout == "tn" else a
    bb = np.ascontiguousarray(b.T) if layout == "nt" else b
    aux = rng.integers(-5, 6, n if epilogue != "mask_positive" else (m, n)).astype(np.float32)
    ab, bbuf, auxb = rt.DeviceBuffer.from_numpy(aa if k else np.zeros(1, np.float32)), rt.DeviceBuffer.from_numpy(bb if k else np.zeros(1, np.float32)), rt.DeviceBuffer.from_numpy(aux)
    cb = rt.DeviceBuffer(m * n)
    rt.sgemm(layout, ab, bbuf, cb, m, n, k, epilogue=epilogue, aux=auxb)
    got = cb.numpy(np.float32, (m, n))
    product = oracle.matmul(aa, bb, layout) if k else np.zeros((m, n), np.float32)
    assert np.array_equal(product, a @ b)
    want = {"bias": product + aux, "bias_relu": np.maximum(product + aux, 0), "mask_positive": np.where(aux > 0, product, 0)}[epilogue]
    assert np.array_equal(got, want.astype(np.float32))


def test_sgemm_fused_argument_errors(rt):
    a = rt.DeviceBuffer(64)
    with pytest.raises(rt.TFHipError, match="needs its bias"):
        rt.sgemm("nn", a, a, a, 4, 4, 4, epilogue="bias")


@pytest.mark.parametrize("layout", ["nn", "nt", "tn"])
@pytest.mark.parametrize("batch,m,n,k", [(1, 64, 64, 64), (7, 130, 70, 33), (64, 128, 128, 256), (300, 8, 5, 17), (5, 256, 512, 1000)])
def test_sgemm_batched(rt, layout, batch, m, n, k):
    """A batch of products in one launch, with A batched and B either batched or shared (stride 0)."""
    rng = np.random.default_rng(batch + m + n + k)
    a = rng.normal(size=(batch, m, k)).astype(np.float32)
    b = rng.normal(size=(batch, k, n)).astype(np.float32)
    aa = np.ascontiguousarray(a.transpose(0, 2, 1)) if layout == "tn" else a
    bb = np.ascontiguousarray(b.transpose(0, 2, 1)) if layout == "nt" else b
    ab, bbuf, cb = rt.DeviceBuffer.from_numpy(aa), rt.DeviceBuffer.from_numpy(bb), rt.DeviceBuffer(batch * m * n)
    rt.sgemm_batched(layout, ab, bbuf, cb, m, n, k, batch, m * k, k * n, m * n)
    got = cb.numpy(np.float32, (batch, m, n))
    a64, b64 = a.astype(np.float64), b.astype(np.float64)
    assert np.max(np.abs(got - a64 @ b64) / (np.abs(a64) @ np.abs(b64))) < 1e-5
    rt.sgemm_batched(layout, ab, bbuf, cb, m, n, k, batch, m * k, 0, m * n)  # every product uses the first B
    got = cb.numpy(np.float32, (batch, m, n))
    assert np.max(np.abs(got - a64 @ b64[0]) / (np.abs(a64) @ np.abs(b64[0]))) < 1e-5
    assert sum_err(got[-1], oracle.matmul(a[-1], b[0]), np.abs(a64[-1]) @ np.abs(b64[0])) < 1e-5


def test_sgemm_batched_argument_errors(rt):
    a = rt.DeviceBuffer(64)
    with pytest.raises(rt.TFHipError, match="overlap"):
        rt.sgemm_batched("nn", a, a, a, 4, 4, 4, 2, 16, 16, 8)
    with pytest.raises(rt.TFHipError, match="empty batch"):
        rt.sgemm_batched("nn", a, a, a, 4, 4, 4, 0, 16, 16, 16)


@pytest.mark.parametrize("mnk", [(256, 256, 262144), (128, 128, 4096), (256, 300, 1000), (512, 96, 64), (384, 128, 130), (130, 40, 5000),
                                 # shapes whose product takes another kernel: the sums come from a column reduction beside it
                                 (4, 3, 100), (100, 256, 777), (256, 8, 4096), (3, 200, 50), (96, 64, 8192),
                                 # narrow results with a long K: the sums ride in the kernel that feeds the operands straight from memory
                                 (64, 256, 16384), (64, 256, 262144), (32, 32, 8192), (64, 64, 100001), (32, 128, 4099),
                                 # at most eight columns: the sums ride in the kernel whose lanes share a row of B
                                 (256, 3, 262144), (64, 8, 5000), (8, 5, 300), (1024, 1, 2000), (260, 7, 70000),
                                 # 128 rows of C with a long K: the tiled kernel (slices that are multiples of 16) and the direct kernel
                                 # (slabs that are multiples of 8) would sum in different orders; both calls must take the same one
                                 (128, 128, 100000), (128, 64, 8200), (128, 32, 50000), (128, 96, 12345)])
def test_sgemm_tn_with_the_column_sums_of_b(rt, mnk):
    """tfhip_sgemm_tn_colsum: the weight gradient X^T dY and the bias gradient sum_k dY[k, :] from one call; the product is
    the very product tfhip_sgemm_tn gives (bit for bit), the sums are within the reduction tolerance."""
    m, n, k = mnk
    rng = np.random.default_rng(m + n + k)
    a = rng.normal(size=(k, m)).astype(np.float32)
    b = rng.normal(size=(k, n)).astype(np.float32)
    ab, bb = rt.DeviceBuffer.from_numpy(a), rt.DeviceBuffer.from_numpy(b)
    c0, c1, sums = rt.DeviceBuffer(m * n), rt.DeviceBuffer(m * n), rt.DeviceBuffer(n + 8)
    sums.fill(0x7FC00000)
    rt.sgemm("tn", ab, bb, c0, m, n, k)
    rt.call("tfhip_sgemm_tn_colsum", ab.ptr, bb.ptr, c1.ptr, sums.ptr, m, n, k)
    assert np.array_equal(c0.numpy(np.float32), c1.numpy(np.float32))
    want = b.astype(np.float64).sum(axis=0)
    scale = np.abs(b).astype(np.float64).sum(axis=0)
    assert np.max(np.abs(sums.numpy(np.float32)[:n] - want) / scale) < 1e-4
    assert np.all(sums.numpy(np.uint32)[n:] == 0x7FC00000), "wrote past the n column sums"
    ref = a.astype(np.float64).T @ b.astype(np.float64)
    assert np.max(np.abs(c1.numpy(np.float32, (m, n)) - ref) / (np.abs(a).astype(np.float64).T @ np.abs(b).astype(np.float64))) < 1e-4
    with pytest.raises(rt.TFHipError, match="null pointer"):
        rt.call("tfhip_sgemm_tn_colsum", ab.ptr, bb.ptr, c1.ptr, None, m, n, k)
    for buf in (ab, bb, c0, c1, sums):
        buf.free()
