// Fused row softmax: y = exp(x - rowmax) / rowsum(exp(x - rowmax)), one HBM read and one write.
//
// In the reference a softmax is a user-level composition (tests/autograd_test.py:29-31,
// examples/ML/MNIST/module.py:8-10) that lowers to >= 5 generated kernels: max stage 1/2, exp-sum
// stage 1/2 (TensorFrost/Compiler/Steps/Optimization.cpp:469-510 splits the 4096-long axis) and the
// normalisation, reading the input three times. Here a row of up to 4096 floats lives in the
// registers of one wavefront (64 lanes x 16 float4); longer or unaligned rows take a group-per-row
// path that re-reads the row from cache.

#include "common.h"

namespace tfhip {

static constexpr float kNegMax = -3.402823466e+38f;

typedef float floatx4 __attribute__((ext_vector_type(4)));

// Streaming store: the softmax output is not read again by this kernel, so it should not displace the
// input (which later reductions re-read) from the last-level cache.
static __device__ __forceinline__ void store_stream(float4* p, float a, float b, float c, float d) {
	floatx4 v = {a, b, c, d};
	__builtin_nontemporal_store(v, reinterpret_cast<floatx4*>(p));
}

// One wave per row; NV float4 per lane; cols % 4 == 0, cols <= 256*NV.
template <int NV>
__global__ __launch_bounds__(256) void softmax_rows_wave_kernel(const float* x, float* y, size_t rows, size_t cols) {
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
		v[i] = c < nvec ? px[c] : make_float4(kNegMax, kNegMax, kNegMax, kNegMax);
	}
	float m = kNegMax;
#pragma unroll
	for (int i = 0; i < NV; i++) m = fmaxf(fmaxf(m, fmaxf(v[i].x, v[i].y)), fmaxf(v[i].z, v[i].w));
	m = wave_reduce(m, OpMax());
	float s = 0.0f;
#pragma unroll
	for (int i = 0; i < NV; i++) {
		v[i].x = __expf(v[i].x - m);
		v[i].y = __expf(v[i].y - m);
		v[i].z = __expf(v[i].z - m);
		v[i].w = __expf(v[i].w - m);
		s += (v[i].x + v[i].y) + (v[i].z + v[i].w);
	}
	s = wave_reduce(s, OpSum());
	const float inv = 1.0f / s;
#pragma unroll
	for (int i = 0; i < NV; i++) {
		int c = lane + 64 * i;
		if (c < nvec) store_stream(py + c, v[i].x * inv, v[i].y * inv, v[i].z * inv, v[i].w * inv);
	}
}

// Any cols: one 256-thread group per row, three sweeps (max, sum, write); sweeps two and three hit cache.
__global__ __launch_bounds__(256) void softmax_rows_group_kernel(const float* x, float* y, size_t rows, size_t cols) {
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
	const float inv = 1.0f / s;
	// In-place use (x == y) is safe: each element is read and written by the same thread, and the
	// earlier sweeps over the row ended at the barriers above.
	for (size_t c = threadIdx.x; c < cols; c += 256) py[c] = __expf(px[c] - m) * inv;
}

}  // namespace tfhip

using namespace tfhip;

extern "C" int tfhip_softmax_rows_f32(const float* x, float* y, size_t rows, size_t cols) {
	TFHIP_REQUIRE_INIT();
	if (!x || !y) return fail(TFHIP_ERR_ARG, "null pointer passed to tfhip_softmax_rows_f32");
	if (rows == 0 || cols == 0) return fail(TFHIP_ERR_ARG, "softmax over an empty matrix (%zu x %zu)", rows, cols);
	State& s = state();
	const bool vec = (cols % 4 == 0) && (((uintptr_t)x & 15) == 0) && (((uintptr_t)y & 15) == 0);
	if (vec && cols <= 4096) {
		size_t blocks = (rows + 3) / 4;
		if (blocks > 0x7FFFFFFFull) return fail(TFHIP_ERR_ARG, "too many rows (%zu)", rows);
		dim3 g((unsigned)blocks), b(256);
		if (cols <= 256)
			hipLaunchKernelGGL(softmax_rows_wave_kernel<1>, g, b, 0, s.stream, x, y, rows, cols);
		else if (cols <= 512)
			hipLaunchKernelGGL(softmax_rows_wave_kernel<2>, g, b, 0, s.stream, x, y, rows, cols);
		else if (cols <= 1024)
			hipLaunchKernelGGL(softmax_rows_wave_kernel<4>, g, b, 0, s.stream, x, y, rows, cols);
		else if (cols <= 2048)
			hipLaunchKernelGGL(softmax_rows_wave_kernel<8>, g, b, 0, s.stream, x, y, rows, cols);
		else
			hipLaunchKernelGGL(softmax_rows_wave_kernel<16>, g, b, 0, s.stream, x, y, rows, cols);
	} else {
		if (rows > 0x7FFFFFFFull) return fail(TFHIP_ERR_ARG, "too many rows (%zu)", rows);
		hipLaunchKernelGGL(softmax_rows_group_kernel, dim3((unsigned)rows), dim3(256), 0, s.stream, x, y, rows, cols);
	}
	TFHIP_CHECK_LAUNCH();
	return TFHIP_OK;
}
