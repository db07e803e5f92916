// Internal helpers shared by the translation units of libtfhip.so. Not part of the C ABI.
#pragma once

#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

#include "tfhip.h"
#include "tfhip_test.h"

namespace tfhip {

// Library-wide state (one device, one in-order stream).
struct State {
	bool initialized = false;
	int device = 0;
	hipStream_t stream = nullptr;
	int compute_units = 0;
	// Grow-only device scratch for partial results of the primitives (never shrinks; freed at shutdown).
	void* scratch = nullptr;
	size_t scratch_bytes = 0;
	// Recorded graphs hold the scratch address of their day in kernel arguments. While any graph is alive, a scratch
	// buffer that has to make way for a larger one is parked here instead of freed; the last graph to go frees them.
	size_t live_graphs = 0;
	void* retired_scratch[32] = {};
	size_t retired_scratch_count = 0;
	// One word of pinned host memory that kernels with a bounded wait set when the bound is hit
	// (host view and device view of the same word). Checked by tfhip_sync.
	volatile uint32_t* async_error_host = nullptr;
	uint32_t* async_error_dev = nullptr;
	// Two pinned staging buffers (allocated on the first large host<->device copy) and the events that say
	// when the DMA engine is done with each.
	void* staging[2] = {nullptr, nullptr};
	hipEvent_t staging_done[2] = {nullptr, nullptr};
	// True between tfhip_graph_begin and tfhip_graph_end: the stream records instead of running, so calls that
	// wait for the stream, free memory or move the scratch buffer are refused.
	bool capturing = false;
};

#define TFHIP_REFUSE_WHILE_RECORDING(what)                                                                      \
	do {                                                                                                        \
		if (::tfhip::state().capturing) return ::tfhip::fail(TFHIP_ERR_STATE, what " is not possible while a graph is being recorded"); \
	} while (0)

// Codes a kernel may leave in the async error word.
constexpr uint32_t kAsyncErrLookbackTimeout = 1;

State& state();

// Records msg as the calling thread's last error and returns code.
int fail(int code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));
int fail_hip(hipError_t err, const char* what);

// Returns scratch of at least `bytes` (256-byte aligned) or nullptr after recording the error.
void* scratch(size_t bytes);

// After every wait for the stream: reports (and clears) the word that kernels with a bounded wait set when they give
// up. Returns TFHIP_OK or TFHIP_ERR_HIP with the message recorded.
int check_async_error();

// Finds the device address of the fixed status-word array of the allocation-free scan on `device`, which must be the
// current device (every GPU holds its own copy at its own address). Called by tfhip_init.
int locate_static_scratch(int device);

#define TFHIP_CHECK(expr)                                         \
	do {                                                          \
		hipError_t _e = (expr);                                   \
		if (_e != hipSuccess) return ::tfhip::fail_hip(_e, #expr); \
	} while (0)

#define TFHIP_REQUIRE_INIT()                                                                    \
	do {                                                                                        \
		if (!::tfhip::state().initialized) return ::tfhip::fail(TFHIP_ERR_STATE, "tfhip_init has not been called"); \
	} while (0)

// Checks the launch that was just issued.
#define TFHIP_CHECK_LAUNCH() TFHIP_CHECK(hipGetLastError())

constexpr int kWave = 64;

typedef float floatx4 __attribute__((ext_vector_type(4)));

// 16-byte load / store of data that this kernel touches once (a streamed operand, a result nobody re-reads here):
// marked non-temporal, so the caches do not keep it. Measured on 256 MiB operands that rotate over 2 GiB, i.e. with
// nothing served by the last-level cache: a read stream runs at 6.8 TB/s with these loads against 6.2 TB/s with plain
// ones, a copy at 6.3-6.5 against 5.7 TB/s.
__device__ __forceinline__ float4 ld4_stream(const float* p) {
	const floatx4 v = __builtin_nontemporal_load(reinterpret_cast<const floatx4*>(p));
	return make_float4(v.x, v.y, v.z, v.w);
}
__device__ __forceinline__ void st4_stream(float* p, float a, float b, float c, float d) {
	const floatx4 v = {a, b, c, d};
	__builtin_nontemporal_store(v, reinterpret_cast<floatx4*>(p));
}

// ---- device helpers ---------------------------------------------------------------------------

// Cross-lane reductions over one 64-wide wavefront; every lane returns the full result.
template <class T, class Op>
__device__ __forceinline__ T wave_reduce(T v, Op op) {
#pragma unroll
	for (int off = 32; off >= 1; off >>= 1) v = op(v, __shfl_xor(v, off, 64));
	return v;
}

struct OpSum {
	__device__ __forceinline__ float operator()(float a, float b) const { return a + b; }
	static __device__ __forceinline__ float init() { return 0.0f; }
};
struct OpMax {
	__device__ __forceinline__ float operator()(float a, float b) const { return a > b ? a : b; }
	static __device__ __forceinline__ float init() { return -3.402823466e+38f; }
};
struct OpMin {
	__device__ __forceinline__ float operator()(float a, float b) const { return a < b ? a : b; }
	static __device__ __forceinline__ float init() { return 3.402823466e+38f; }
};

}  // namespace tfhip
