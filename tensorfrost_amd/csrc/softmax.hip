// Fused row softmax: y = exp(x - rowmax) / rowsum(exp(x - rowmax)), one HBM read and one write.
//
// In the reference a softmax is a user-level composition (tests/autograd_test.py:29-31,
// examples/ML/MNIST/module.py:8-10) that lowers to >= 5 generated kernels: max stage 1/2, exp-sum
// stage 1/2 (TensorFrost/Compiler/Steps/Optimization.cpp:469-510 splits the 4096-long axis) and the
// normalisation, reading the input three times. Here a row of up to 4096 floats lives in the
// registers of one wavefront (64 lanes x 16 float4); rows up to 32768 floats live in the registers of one
// group; longer rows (or few long ones) are cut into segments handled by three kernels with two reads; short
// unaligned rows take a group-per-row path that re-reads the row from cache.

#include "common.h"

namespace tfhip {

static constexpr float kNegMax = -3.402823466e+38f;

// Streaming accesses (common.h): the input is read once and the output is not read again by this kernel, so neither
// should displace anything from the caches.
static __device__ __forceinline__ void store_stream(float4* p, float a, float b, float c, float d) { st4_stream(reinterpret_cast<float*>(p), a, b, c, d); }
static __device__ __forceinline__ float4 load_stream(const float4* p) { return ld4_stream(reinterpret_cast<const float*>(p)); }

// Every kernel below also computes the log-softmax, (x - max) - log(sum), when `log_form` is set (the composition of
// tests/autograd_test.py:29-31): the same read, maximum and sum; only what is written differs. The flag is uniform, and
// the kernels wait for memory, so the selects cost nothing measurable.
// exp(v - m) element-wise; v keeps x in the log form (its output needs x itself) and becomes the exponentials otherwise.
static __device__ __forceinline__ float exp4_sum(float4& v, float m, bool log_form) {
	const float4 e = make_float4(__expf(v.x - m), __expf(v.y - m), __expf(v.z - m), __expf(v.w - m));
	if (!log_form) v = e;
	return (e.x + e.y) + (e.z + e.w);
}
// k = 1 / sum (softmax) or log(sum) (log form)
static __device__ __forceinline__ float finish_factor(float s, bool log_form) { return log_form ? logf(s) : 1.0f / s; }
static __device__ __forceinline__ float finish1(float v, float m, float k, bool log_form) { return log_form ? (v - m) - k : v * k; }
static __device__ __forceinline__ void finish_store(float4* p, float4 v, float m, float k, bool log_form) {
	store_stream(p, finish1(v.x, m, k, log_form), finish1(v.y, m, k, log_form), finish1(v.z, m, k, log_form), finish1(v.w, m, k, log_form));
}

// One wave per row; NV float4 per lane; cols % 4 == 0, cols <= 256*NV.
template <int NV>
__global__ __launch_bounds__(256) void softmax_rows_wave_kernel(const float* x, float* y, size_t rows, size_t cols, float* row_max, float* row_sum, bool log_form) {
	const int lane = threadIdx.x & 63;
	const size_t row = (size_t)blockIdx.x * 4 + (threadIdx.x >> 6);
	if (row >= rows) return;
	const float4* px = reinterpret_cast<const float4*>(x + row * cols);
	float4* py = reinterpret_cast<float4*>(y + row * cols);
	const int nvec = (int)(cols >> 2);
	float4 v[NV];
#pragma unroll
	for (int i = 0; i < NV; i++) {
		int c = lane + 64 * i;
		v[i] = c < nvec ? load_stream(px + c) : make_float4(kNegMax, kNegMax, kNegMax, kNegMax);
	}
	float m = kNegMax;
#pragma unroll
	for (int i = 0; i < NV; i++) m = fmaxf(fmaxf(m, fmaxf(v[i].x, v[i].y)), fmaxf(v[i].z, v[i].w));
	m = wave_reduce(m, OpMax());
	float s = 0.0f;
#pragma unroll
	for (int i = 0; i < NV; i++) s += exp4_sum(v[i], m, log_form);
	s = wave_reduce(s, OpSum());
	if (row_max && lane == 0) {
		row_max[row] = m;
		row_sum[row] = s;
	}
	const float k = finish_factor(s, log_form);
#pragma unroll
	for (int i = 0; i < NV; i++) {
		int c = lane + 64 * i;
		if (y && c < nvec) finish_store(py + c, v[i], m, k, log_form);
	}
}

// Rows of 132 .. 256 floats, many of them: a wave takes four consecutive rows (one float4 per lane and row, all four
// loads in flight before the first maximum), so a group of four waves reads and writes 16 consecutive rows.
__global__ __launch_bounds__(256) void softmax_rows_wave4_kernel(const float* x, float* y, size_t rows, size_t cols, float* row_max, float* row_sum, bool log_form) {
	const int lane = threadIdx.x & 63;
	const size_t row0 = ((size_t)blockIdx.x * 4 + (threadIdx.x >> 6)) * 4;
	const int nvec = (int)(cols >> 2);
	float4 v[4];
#pragma unroll
	for (int r = 0; r < 4; r++)
		v[r] = row0 + r < rows && lane < nvec ? load_stream(reinterpret_cast<const float4*>(x + (row0 + r) * cols) + lane) : make_float4(kNegMax, kNegMax, kNegMax, kNegMax);
#pragma unroll
	for (int r = 0; r < 4; r++) {
		const size_t row = row0 + r;
		if (row >= rows) break;
		const float m = wave_reduce(fmaxf(fmaxf(v[r].x, v[r].y), fmaxf(v[r].z, v[r].w)), OpMax());
		const float s = wave_reduce(exp4_sum(v[r], m, log_form), OpSum());
		if (row_max && lane == 0) {
			row_max[row] = m;
			row_sum[row] = s;
		}
		const float k = finish_factor(s, log_form);
		if (y && lane < nvec) finish_store(reinterpret_cast<float4*>(y + row * cols) + lane, v[r], m, k, log_form);
	}
}

// Short rows (cols <= 128, 16-byte aligned): LANES lanes own a row with one float4 each, so a wave works on 64/LANES
// rows at once and, when cols == 4*LANES, reads and writes whole contiguous kilobytes. Four row groups per trip.
template <int LANES>
__global__ __launch_bounds__(256) void softmax_rows_lanes_kernel(const float* x, float* y, size_t rows, size_t cols, float* row_max, float* row_sum, bool log_form) {
	constexpr int kRowsPerStep = 64 / LANES;
	constexpr int kSteps = 4;
	const int lane = threadIdx.x & 63;
	const int sub = lane % LANES, which = lane / LANES;
	const size_t wave = (size_t)blockIdx.x * 4 + (threadIdx.x >> 6);
	const size_t row0 = wave * (kRowsPerStep * kSteps) + which;
	const bool has = (size_t)sub * 4 < cols;
	float4 v[kSteps];
#pragma unroll
	for (int u = 0; u < kSteps; u++) {
		const size_t row = row0 + (size_t)u * kRowsPerStep;
		v[u] = (has && row < rows) ? ld4_stream(x + row * cols + sub * 4) : make_float4(kNegMax, kNegMax, kNegMax, kNegMax);
	}
#pragma unroll
	for (int u = 0; u < kSteps; u++) {
		float m = fmaxf(fmaxf(v[u].x, v[u].y), fmaxf(v[u].z, v[u].w));
#pragma unroll
		for (int off = LANES / 2; off >= 1; off >>= 1) m = fmaxf(m, __shfl_xor(m, off, 64));
		float s = exp4_sum(v[u], m, log_form);
#pragma unroll
		for (int off = LANES / 2; off >= 1; off >>= 1) s += __shfl_xor(s, off, 64);
		const float k = finish_factor(s, log_form);
		const size_t row = row0 + (size_t)u * kRowsPerStep;
		if (row_max && sub == 0 && row < rows) {
			row_max[row] = m;
			row_sum[row] = s;
		}
		if (y && has && row < rows) finish_store(reinterpret_cast<float4*>(y + row * cols + sub * 4), v[u], m, k, log_form);
	}
}

// Short rows of any length and alignment (cols <= 32, e.g. ten class scores): one thread per row, three sweeps; the
// lines a wave touches stay in cache between the sweeps.
__global__ __launch_bounds__(256) void softmax_rows_thread_kernel(const float* x, float* y, size_t rows, size_t cols, float* row_max, float* row_sum, bool log_form) {
	const size_t row = (size_t)blockIdx.x * 256 + threadIdx.x;
	if (row >= rows) return;
	const float* px = x + row * cols;
	float* py = y + row * cols;
	float m = kNegMax;
	for (size_t c = 0; c < cols; c++) m = fmaxf(m, px[c]);
	float s = 0.0f;
	for (size_t c = 0; c < cols; c++) s += __expf(px[c] - m);
	if (row_max) {
		row_max[row] = m;
		row_sum[row] = s;
	}
	const float k = finish_factor(s, log_form);
	if (y)
		for (size_t c = 0; c < cols; c++) py[c] = log_form ? (px[c] - m) - k : __expf(px[c] - m) * k;
}

// Any cols: one 256-thread group per row, three sweeps (max, sum, write); sweeps two and three hit cache.
__global__ __launch_bounds__(256) void softmax_rows_group_kernel(const float* x, float* y, size_t rows, size_t cols, float* row_max, float* row_sum, bool log_form) {
	__shared__ float red[4];
	const int lane = threadIdx.x & 63;
	const int wave = threadIdx.x >> 6;
	const size_t row = blockIdx.x;
	const float* px = x + row * cols;
	float* py = y + row * cols;

	float m = kNegMax;
	for (size_t c = threadIdx.x; c < cols; c += 256) m = fmaxf(m, px[c]);
	m = wave_reduce(m, OpMax());
	if (lane == 0) red[wave] = m;
	__syncthreads();
	m = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
	__syncthreads();

	float s = 0.0f;
	for (size_t c = threadIdx.x; c < cols; c += 256) s += __expf(px[c] - m);
	s = wave_reduce(s, OpSum());
	if (lane == 0) red[wave] = s;
	__syncthreads();
	s = (red[0] + red[1]) + (red[2] + red[3]);
	if (row_max && threadIdx.x == 0) {
		row_max[row] = m;
		row_sum[row] = s;
	}
	const float k = finish_factor(s, log_form);
	// In-place use (x == y) is safe: each element is read and written by the same thread, and the
	// earlier sweeps over the row ended at the barriers above.
	if (y)
		for (size_t c = threadIdx.x; c < cols; c += 256) py[c] = log_form ? (px[c] - m) - k : __expf(px[c] - m) * k;
}

// Rows of 2049 .. 32768 floats: one group of THREADS threads per row holds the row in registers (NV float4 per
// thread), so the row is still read once; maxima and sums cross the waves through group memory. Few vectors per
// thread and many threads per row is the shape that streams fastest: a 4096-float row as 512 threads x 2 vectors moves
// 6.5 TB/s with nothing cached, as 256 x 4 6.3, as one wave x 16 vectors 5.7.
template <int THREADS, int NV>
__global__ __launch_bounds__(THREADS) void softmax_rows_block_kernel(const float* x, float* y, size_t rows, size_t cols, float* row_max, float* row_sum, bool log_form) {
	constexpr int kWaves = THREADS / 64;
	__shared__ float red[kWaves];
	const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
	const size_t row = blockIdx.x;
	const float4* px = reinterpret_cast<const float4*>(x + row * cols);
	float4* py = reinterpret_cast<float4*>(y + row * cols);
	const int nvec = (int)(cols >> 2);
	float4 v[NV];
#pragma unroll
	for (int i = 0; i < NV; i++) {
		const int c = threadIdx.x + THREADS * i;
		v[i] = c < nvec ? load_stream(px + c) : make_float4(kNegMax, kNegMax, kNegMax, kNegMax);
	}
	float m = kNegMax;
#pragma unroll
	for (int i = 0; i < NV; i++) m = fmaxf(fmaxf(m, fmaxf(v[i].x, v[i].y)), fmaxf(v[i].z, v[i].w));
	m = wave_reduce(m, OpMax());
	if (lane == 0) red[wave] = m;
	__syncthreads();
	m = red[0];
#pragma unroll
	for (int w = 1; w < kWaves; w++) m = fmaxf(m, red[w]);
	__syncthreads();
	float s = 0.0f;
#pragma unroll
	for (int i = 0; i < NV; i++) s += exp4_sum(v[i], m, log_form);
	s = wave_reduce(s, OpSum());
	if (lane == 0) red[wave] = s;
	__syncthreads();
	s = red[0];
#pragma unroll
	for (int w = 1; w < kWaves; w++) s += red[w];
	if (row_max && threadIdx.x == 0) {
		row_max[row] = m;
		row_sum[row] = s;
	}
	const float k = finish_factor(s, log_form);
#pragma unroll
	for (int i = 0; i < NV; i++) {
		const int c = threadIdx.x + THREADS * i;
		if (y && c < nvec) finish_store(py + c, v[i], m, k, log_form);
	}
}

// Longer rows, or few of them: three kernels. (1) every 8192-element segment of a row gives its maximum and the sum of
// exp(x - that maximum) from one read; (2) one thread per row folds the segment pairs into the row's maximum and the
// reciprocal of its sum; (3) y = exp(x - max) / sum from a second read. Two reads and one write of the matrix.
constexpr int kSegLen = 8192;  // 256 threads x 8 float4

template <bool VEC>
__global__ __launch_bounds__(256) void softmax_segment_kernel(const float* __restrict__ x, float2* __restrict__ partial, size_t cols, size_t segs) {
	__shared__ float red[4];
	const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
	const size_t row = blockIdx.x / segs, seg = blockIdx.x % segs;
	const size_t c0 = seg * kSegLen;
	const size_t c1 = c0 + kSegLen < cols ? c0 + kSegLen : cols;
	const float* px = x + row * cols;
	float v[32];
	if (VEC) {
#pragma unroll
		for (int i = 0; i < 8; i++) {
			const size_t c = c0 + ((size_t)threadIdx.x + 256 * i) * 4;
			const float4 t = c < c1 ? *reinterpret_cast<const float4*>(px + c) : make_float4(kNegMax, kNegMax, kNegMax, kNegMax);
			v[4 * i] = t.x;
			v[4 * i + 1] = t.y;
			v[4 * i + 2] = t.z;
			v[4 * i + 3] = t.w;
		}
	} else {
#pragma unroll
		for (int i = 0; i < 32; i++) {
			const size_t c = c0 + threadIdx.x + 256 * (size_t)i;
			v[i] = c < c1 ? px[c] : kNegMax;
		}
	}
	float m = kNegMax;
#pragma unroll
	for (int i = 0; i < 32; i++) m = fmaxf(m, v[i]);
	m = wave_reduce(m, OpMax());
	if (lane == 0) red[wave] = m;
	__syncthreads();
	m = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
	__syncthreads();
	float s = 0.0f;
#pragma unroll
	for (int i = 0; i < 32; i++) s += __expf(v[i] - m);  // padding: exp(-huge) = 0
	s = wave_reduce(s, OpSum());
	if (lane == 0) red[wave] = s;
	__syncthreads();
	if (threadIdx.x == 0) partial[blockIdx.x] = make_float2(m, (red[0] + red[1]) + (red[2] + red[3]));
}

__global__ __launch_bounds__(256) void softmax_fold_kernel(const float2* __restrict__ partial, float2* __restrict__ row_stats, size_t rows, size_t segs, float* row_max, float* row_sum, bool log_form) {
	const int lane = threadIdx.x & 63;
	const size_t row = (size_t)blockIdx.x * 4 + (threadIdx.x >> 6);  // one wave per row
	if (row >= rows) return;
	const float2* p = partial + row * segs;
	float m = kNegMax;
	for (size_t k = lane; k < segs; k += 64) m = fmaxf(m, p[k].x);
	m = wave_reduce(m, OpMax());
	float s = 0.0f;
	for (size_t k = lane; k < segs; k += 64) s += p[k].y * __expf(p[k].x - m);
	s = wave_reduce(s, OpSum());
	if (lane == 0) {
		row_stats[row] = make_float2(m, finish_factor(s, log_form));
		if (row_max) {
			row_max[row] = m;
			row_sum[row] = s;
		}
	}
}

template <bool VEC>
__global__ __launch_bounds__(256) void softmax_apply_kernel(const float* x, float* y, const float2* __restrict__ row_stats, size_t cols, size_t segs, bool log_form) {
	const size_t row = blockIdx.x / segs, seg = blockIdx.x % segs;
	const size_t c0 = seg * kSegLen;
	const size_t c1 = c0 + kSegLen < cols ? c0 + kSegLen : cols;
	const float2 st = row_stats[row];
	const float* px = x + row * cols;
	float* py = y + row * cols;
	if (VEC) {
#pragma unroll
		for (int i = 0; i < 8; i++) {
			const size_t c = c0 + ((size_t)threadIdx.x + 256 * i) * 4;
			if (c < c1) {
				const float4 t = *reinterpret_cast<const float4*>(px + c);
				if (log_form)
					store_stream(reinterpret_cast<float4*>(py + c), (t.x - st.x) - st.y, (t.y - st.x) - st.y, (t.z - st.x) - st.y, (t.w - st.x) - st.y);
				else
					store_stream(reinterpret_cast<float4*>(py + c), __expf(t.x - st.x) * st.y, __expf(t.y - st.x) * st.y, __expf(t.z - st.x) * st.y, __expf(t.w - st.x) * st.y);
			}
		}
	} else {
		for (size_t c = c0 + threadIdx.x; c < c1; c += 256) py[c] = log_form ? (px[c] - st.x) - st.y : __expf(px[c] - st.x) * st.y;
	}
}

static int softmax_three_pass(const float* x, float* y, size_t rows, size_t cols, bool vec, float* row_max, float* row_sum, bool log_form) {
	State& s = state();
	const size_t segs = (cols + kSegLen - 1) / kSegLen;
	if (rows * segs > 0x7FFFFFFFull) return fail(TFHIP_ERR_ARG, "softmax of %zu x %zu is too large", rows, cols);
	const size_t partial_bytes = (rows * segs * sizeof(float2) + 255) & ~size_t(255);
	char* base = (char*)scratch(partial_bytes + rows * sizeof(float2));
	if (!base) return TFHIP_ERR_HIP;
	float2* partial = (float2*)base;
	float2* row_stats = (float2*)(base + partial_bytes);
	const dim3 grid((unsigned)(rows * segs)), block(256);
	if (vec)
		hipLaunchKernelGGL(softmax_segment_kernel<true>, grid, block, 0, s.stream, x, partial, cols, segs);
	else
		hipLaunchKernelGGL(softmax_segment_kernel<false>, grid, block, 0, s.stream, x, partial, cols, segs);
	TFHIP_CHECK_LAUNCH();
	hipLaunchKernelGGL(softmax_fold_kernel, dim3((unsigned)((rows + 3) / 4)), block, 0, s.stream, (const float2*)partial, row_stats, rows, segs, row_max, row_sum, log_form);
	TFHIP_CHECK_LAUNCH();
	if (!y) return TFHIP_OK;  // statistics only
	if (vec)
		hipLaunchKernelGGL(softmax_apply_kernel<true>, grid, block, 0, s.stream, x, y, (const float2*)row_stats, cols, segs, log_form);
	else
		hipLaunchKernelGGL(softmax_apply_kernel<false>, grid, block, 0, s.stream, x, y, (const float2*)row_stats, cols, segs, log_form);
	TFHIP_CHECK_LAUNCH();
	return TFHIP_OK;
}

}  // namespace tfhip

using namespace tfhip;

static int softmax_rows(const float* x, float* y, size_t rows, size_t cols, float* row_max, float* row_sum, bool log_form) {
	TFHIP_REQUIRE_INIT();
	if (!x || (!y && !row_max)) return fail(TFHIP_ERR_ARG, "null pointer passed to the row softmax");
	if (rows == 0 || cols == 0) return fail(TFHIP_ERR_ARG, "softmax over an empty matrix (%zu x %zu)", rows, cols);
	State& s = state();
	const bool vec = (cols % 4 == 0) && (((uintptr_t)x & 15) == 0) && (((uintptr_t)y & 15) == 0);  // y == nullptr: statistics only
	if (vec && cols <= 128 && rows >= 64) {
		const size_t vecs = cols / 4;
		const int lanes = vecs <= 1 ? 1 : vecs <= 2 ? 2 : vecs <= 4 ? 4 : vecs <= 8 ? 8 : vecs <= 16 ? 16 : 32;
		const size_t rows_per_group = (size_t)(64 / lanes) * 4 * 4;
		const size_t blocks = (rows + rows_per_group - 1) / rows_per_group;
		if (blocks > 0x7FFFFFFFull) return fail(TFHIP_ERR_ARG, "too many rows (%zu)", rows);
		dim3 g((unsigned)blocks), b(256);
		switch (lanes) {
			case 1: hipLaunchKernelGGL(softmax_rows_lanes_kernel<1>, g, b, 0, s.stream, x, y, rows, cols, row_max, row_sum, log_form); break;
			case 2: hipLaunchKernelGGL(softmax_rows_lanes_kernel<2>, g, b, 0, s.stream, x, y, rows, cols, row_max, row_sum, log_form); break;
			case 4: hipLaunchKernelGGL(softmax_rows_lanes_kernel<4>, g, b, 0, s.stream, x, y, rows, cols, row_max, row_sum, log_form); break;
			case 8: hipLaunchKernelGGL(softmax_rows_lanes_kernel<8>, g, b, 0, s.stream, x, y, rows, cols, row_max, row_sum, log_form); break;
			case 16: hipLaunchKernelGGL(softmax_rows_lanes_kernel<16>, g, b, 0, s.stream, x, y, rows, cols, row_max, row_sum, log_form); break;
			default: hipLaunchKernelGGL(softmax_rows_lanes_kernel<32>, g, b, 0, s.stream, x, y, rows, cols, row_max, row_sum, log_form); break;
		}
	} else if (!vec && cols <= 32) {
		const size_t blocks = (rows + 255) / 256;
		if (blocks > 0x7FFFFFFFull) return fail(TFHIP_ERR_ARG, "too many rows (%zu)", rows);
		hipLaunchKernelGGL(softmax_rows_thread_kernel, dim3((unsigned)blocks), dim3(256), 0, s.stream, x, y, rows, cols, row_max, row_sum, log_form);
	} else if (vec && cols > 2048 && cols <= 4096 && rows >= (size_t)s.compute_units * 4 && rows <= 0x7FFFFFFFull) {
		hipLaunchKernelGGL((softmax_rows_block_kernel<512, 2>), dim3((unsigned)rows), dim3(512), 0, s.stream, x, y, rows, cols, row_max, row_sum, log_form);
	} else if (vec && cols <= 4096) {
		size_t blocks = (rows + 3) / 4;
		if (blocks > 0x7FFFFFFFull) return fail(TFHIP_ERR_ARG, "too many rows (%zu)", rows);
		dim3 g((unsigned)blocks), b(256);
		if (cols <= 256 && rows >= (size_t)s.compute_units * 64)
			hipLaunchKernelGGL(softmax_rows_wave4_kernel, dim3((unsigned)((rows + 15) / 16)), b, 0, s.stream, x, y, rows, cols, row_max, row_sum, log_form);
		else if (cols <= 256)
			hipLaunchKernelGGL(softmax_rows_wave_kernel<1>, g, b, 0, s.stream, x, y, rows, cols, row_max, row_sum, log_form);
		else if (cols <= 512)
			hipLaunchKernelGGL(softmax_rows_wave_kernel<2>, g, b, 0, s.stream, x, y, rows, cols, row_max, row_sum, log_form);
		else if (cols <= 1024)
			hipLaunchKernelGGL(softmax_rows_wave_kernel<4>, g, b, 0, s.stream, x, y, rows, cols, row_max, row_sum, log_form);
		else if (cols <= 2048)
			hipLaunchKernelGGL(softmax_rows_wave_kernel<8>, g, b, 0, s.stream, x, y, rows, cols, row_max, row_sum, log_form);
		else
			hipLaunchKernelGGL(softmax_rows_wave_kernel<16>, g, b, 0, s.stream, x, y, rows, cols, row_max, row_sum, log_form);
	} else if (vec && cols <= 32768 && rows >= (size_t)s.compute_units && rows <= 0x7FFFFFFFull) {
		// enough rows to give every compute unit one: a group per row, the row in registers
		dim3 g((unsigned)rows);
		if (cols <= 8192)
			hipLaunchKernelGGL((softmax_rows_block_kernel<256, 8>), g, dim3(256), 0, s.stream, x, y, rows, cols, row_max, row_sum, log_form);
		else if (cols <= 16384)
			hipLaunchKernelGGL((softmax_rows_block_kernel<512, 8>), g, dim3(512), 0, s.stream, x, y, rows, cols, row_max, row_sum, log_form);
		else
			hipLaunchKernelGGL((softmax_rows_block_kernel<1024, 8>), g, dim3(1024), 0, s.stream, x, y, rows, cols, row_max, row_sum, log_form);
	} else if (cols > 2048) {
		return softmax_three_pass(x, y, rows, cols, vec, row_max, row_sum, log_form);
	} else {
		if (rows > 0x7FFFFFFFull) return fail(TFHIP_ERR_ARG, "too many rows (%zu)", rows);
		hipLaunchKernelGGL(softmax_rows_group_kernel, dim3((unsigned)rows), dim3(256), 0, s.stream, x, y, rows, cols, row_max, row_sum, log_form);
	}
	TFHIP_CHECK_LAUNCH();
	return TFHIP_OK;
}

extern "C" int tfhip_softmax_rows_f32(const float* x, float* y, size_t rows, size_t cols) { return softmax_rows(x, y, rows, cols, nullptr, nullptr, false); }

extern "C" int tfhip_log_softmax_rows_f32(const float* x, float* y, size_t rows, size_t cols) { return softmax_rows(x, y, rows, cols, nullptr, nullptr, true); }

extern "C" int tfhip_log_softmax_rows_stats_f32(const float* x, float* y, float* row_max, float* row_sum, size_t rows, size_t cols) {
	if (!y || !row_max || !row_sum) return fail(TFHIP_ERR_ARG, "null pointer passed to tfhip_log_softmax_rows_stats_f32");
	return softmax_rows(x, y, rows, cols, row_max, row_sum, true);
}

extern "C" int tfhip_softmax_rows_stats_f32(const float* x, float* y, float* row_max, float* row_sum, size_t rows, size_t cols) {
	if (!row_max || !row_sum) return fail(TFHIP_ERR_ARG, "null pointer passed to tfhip_softmax_rows_stats_f32");
	return softmax_rows(x, y, rows, cols, row_max, row_sum, false);
}
