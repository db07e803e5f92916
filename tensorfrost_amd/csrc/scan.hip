// Inclusive prefix sums over a contiguous array.
//
// The reference computes dim_prefix_sum as a serial loop in ONE thread per scan line
// (TensorFrost/Compiler/Implementations.cpp:305-359,447-449: acc += x[k]; out[k] = acc), so a 1-D
// scan runs on a single thread; the two-level grouped form users write around it
// (Python/TensorFrost/sort.py:39-50) still serialises across groups.
//
// u32 (and i32, which is the same bit pattern under two's complement wrap-around): single pass,
// "decoupled look-back". Tiles of 4096 elements take a ticket in start order, publish their
// aggregate, then look back over the published aggregates / inclusive prefixes of earlier tiles,
// 64 tiles per wave step. One read and one write of the data; integer addition is associative, so
// the result is bit-exact whatever the timing.
//
// f32: addition is not associative, and how far a look-back walks depends on timing, so the chained
// scan would not be reproducible run to run. Floats use reduce-then-scan instead: tile sums, a
// (recursive) scan of the tile sums, then a rescan of each tile from its exclusive prefix -- two reads
// and one write, with a summation order fixed by the tiling.

#include "common.h"

namespace tfhip {

constexpr int kScanThreads = 256;
constexpr int kScanVecs = 4;                                  // uint4/float4 per thread
constexpr int kScanTile = kScanThreads * kScanVecs * 4;       // 4096 elements
constexpr uint32_t kSpinLimit = 1u << 22;                     // bounded wait of the look-back

constexpr uint64_t kFlagAggregate = 1ull << 32;
constexpr uint64_t kFlagPrefix = 2ull << 32;

template <class T>
struct alignas(16) Vec4 {
	T x, y, z, w;
};

template <class T>
__device__ __forceinline__ T wave_inclusive_scan(T v) {
	const int lane = threadIdx.x & 63;
#pragma unroll
	for (int off = 1; off < 64; off <<= 1) {
		T o = __shfl_up(v, off, 64);
		if (lane >= off) v += o;
	}
	return v;
}

// Loads the tile in "vector-striped" order: vector k of thread t is vector (k*256 + t) of the tile, so
// every wave instruction reads 1 KiB of consecutive memory.
template <class T>
__device__ __forceinline__ void load_tile(const T* in, size_t base, size_t n, bool aligned, Vec4<T> (&v)[kScanVecs]) {
#pragma unroll
	for (int k = 0; k < kScanVecs; k++) {
		size_t i = base + ((size_t)k * kScanThreads + threadIdx.x) * 4;
		if (aligned && i + 3 < n) {
			v[k] = *reinterpret_cast<const Vec4<T>*>(in + i);
		} else {
			v[k].x = i < n ? in[i] : T(0);
			v[k].y = i + 1 < n ? in[i + 1] : T(0);
			v[k].z = i + 2 < n ? in[i + 2] : T(0);
			v[k].w = i + 3 < n ? in[i + 3] : T(0);
		}
	}
}

template <class T>
__device__ __forceinline__ void store_tile(T* out, size_t base, size_t n, bool aligned, const Vec4<T> (&v)[kScanVecs]) {
#pragma unroll
	for (int k = 0; k < kScanVecs; k++) {
		size_t i = base + ((size_t)k * kScanThreads + threadIdx.x) * 4;
		if (aligned && i + 3 < n) {
			*reinterpret_cast<Vec4<T>*>(out + i) = v[k];
		} else {
			if (i < n) out[i] = v[k].x;
			if (i + 1 < n) out[i + 1] = v[k].y;
			if (i + 2 < n) out[i + 2] = v[k].z;
			if (i + 3 < n) out[i + 3] = v[k].w;
		}
	}
}

// Turns v[] into the inclusive scan of the tile (without any cross-tile prefix) and returns the tile
// total to every thread. lds: kScanVecs*4 + 1 elements.
template <class T>
__device__ __forceinline__ T scan_tile_in_registers(Vec4<T> (&v)[kScanVecs], T* lds) {
	const int lane = threadIdx.x & 63;
	const int wave = threadIdx.x >> 6;
	T excl[kScanVecs];  // sum of the vectors of lower lanes of this wave, same k
#pragma unroll
	for (int k = 0; k < kScanVecs; k++) {
		v[k].y += v[k].x;
		v[k].z += v[k].y;
		v[k].w += v[k].z;
		T incl = wave_inclusive_scan(v[k].w);
		if (lane == 63) lds[k * 4 + wave] = incl;
		T up = __shfl_up(incl, 1, 64);
		excl[k] = lane == 0 ? T(0) : up;
	}
	__syncthreads();
	T total = T(0);
#pragma unroll
	for (int k = 0; k < kScanVecs; k++) {
		T before = total;  // everything in vectors of lower k, then lower waves of this k
#pragma unroll
		for (int w = 0; w < 4; w++) {
			T t = lds[k * 4 + w];
			if (w < wave) before += t;
			total += t;
		}
		T offset = before + excl[k];
		v[k].x += offset;
		v[k].y += offset;
		v[k].z += offset;
		v[k].w += offset;
	}
	return total;
}

__device__ __forceinline__ void status_store(uint64_t* p, uint64_t v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ uint64_t status_load(uint64_t* p) { return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }

// status[tile]: high word = flag (0 none, 1 aggregate, 2 inclusive prefix), low word = value.
// ticket: one counter, zeroed (with status) before the launch.
__global__ __launch_bounds__(kScanThreads) void scan_lookback_u32_kernel(const uint32_t* in, uint32_t* out, size_t n,
                                                                          uint64_t* status, uint32_t* ticket, uint32_t* async_error) {
	__shared__ uint32_t lds[kScanVecs * 4];
	__shared__ uint32_t s_tile;
	__shared__ uint32_t s_prefix;
	if (threadIdx.x == 0) s_tile = atomicAdd(ticket, 1u);
	__syncthreads();
	const uint32_t tile = s_tile;
	const size_t base = (size_t)tile * kScanTile;
	const bool aligned = ((((uintptr_t)in) | ((uintptr_t)out)) & 15) == 0;

	Vec4<uint32_t> v[kScanVecs];
	load_tile(in, base, n, aligned, v);
	const uint32_t total = scan_tile_in_registers(v, lds);

	if (threadIdx.x < 64) {  // wave 0 resolves the tile's exclusive prefix
		const int lane = threadIdx.x;
		if (lane == 0) status_store(&status[tile], (tile == 0 ? kFlagPrefix : kFlagAggregate) | total);
		uint32_t exclusive = 0;
		if (tile > 0) {
			int64_t look = (int64_t)tile - 1;  // lane 0 inspects tile `look`, lane i tile `look - i`
			uint32_t spins = 0;
			bool done = false;
			while (!done) {
				const int64_t t = look - lane;
				uint64_t s = t >= 0 ? status_load(&status[t]) : kFlagPrefix;  // before tile 0: prefix 0
				const uint64_t ready = __ballot((s >> 32) != 0);
				if (ready != ~0ull) {
					if (++spins > kSpinLimit) {  // an earlier tile never published: give up, flag it
						if (lane == 0) *async_error = kAsyncErrLookbackTimeout;
						break;
					}
					__builtin_amdgcn_s_sleep(1);
					continue;
				}
				const uint64_t has_prefix = __ballot((s >> 32) == 2);
				// nearest tile with a full prefix ends the walk; everything nearer contributes its aggregate
				const int stop = has_prefix ? __builtin_ctzll(has_prefix) : 63;
				uint32_t contrib = lane <= stop ? (uint32_t)s : 0u;
				exclusive += wave_reduce(contrib, [](uint32_t a, uint32_t b) { return a + b; });
				if (has_prefix)
					done = true;
				else
					look -= 64;
			}
			if (lane == 0) status_store(&status[tile], kFlagPrefix | (uint64_t)(uint32_t)(exclusive + total));
		}
		if (lane == 0) s_prefix = exclusive;
	}
	__syncthreads();
	const uint32_t prefix = s_prefix;
#pragma unroll
	for (int k = 0; k < kScanVecs; k++) {
		v[k].x += prefix;
		v[k].y += prefix;
		v[k].z += prefix;
		v[k].w += prefix;
	}
	store_tile(out, base, n, aligned, v);
}

// ---- f32: reduce-then-scan ----------------------------------------------------------------------

__global__ __launch_bounds__(kScanThreads) void scan_tile_sums_f32_kernel(const float* __restrict__ in, float* __restrict__ sums, size_t n) {
	__shared__ float lds[kScanVecs * 4];
	const size_t base = (size_t)blockIdx.x * kScanTile;
	const bool aligned = (((uintptr_t)in) & 15) == 0;
	Vec4<float> v[kScanVecs];
	load_tile(in, base, n, aligned, v);
	// Same arithmetic as the rescan below, so that prefix + local scan reproduces these totals exactly.
	const float total = scan_tile_in_registers(v, lds);
	if (threadIdx.x == 0) sums[blockIdx.x] = total;
}

// out = inclusive scan of the tile + exclusive prefix of the tile (prefix[tile-1], 0 for tile 0).
__global__ __launch_bounds__(kScanThreads) void scan_apply_f32_kernel(const float* in, float* out, size_t n,
                                                                       const float* tile_inclusive) {
	__shared__ float lds[kScanVecs * 4];
	const size_t base = (size_t)blockIdx.x * kScanTile;
	const bool aligned = ((((uintptr_t)in) | ((uintptr_t)out)) & 15) == 0;
	Vec4<float> v[kScanVecs];
	load_tile(in, base, n, aligned, v);
	(void)scan_tile_in_registers(v, lds);
	const float prefix = (blockIdx.x == 0 || tile_inclusive == nullptr) ? 0.0f : tile_inclusive[blockIdx.x - 1];
#pragma unroll
	for (int k = 0; k < kScanVecs; k++) {
		v[k].x += prefix;
		v[k].y += prefix;
		v[k].z += prefix;
		v[k].w += prefix;
	}
	store_tile(out, base, n, aligned, v);
}

// level_buf: scratch for all recursion levels, laid out by the caller.
static int scan_f32_recursive(const float* in, float* out, size_t n, float* level_buf) {
	State& s = state();
	const size_t tiles = (n + kScanTile - 1) / kScanTile;
	if (tiles > 0x7FFFFFFFull) return fail(TFHIP_ERR_ARG, "scan of %zu elements is too long", n);
	if (tiles == 1) {
		hipLaunchKernelGGL(scan_apply_f32_kernel, dim3(1), dim3(kScanThreads), 0, s.stream, in, out, n, (const float*)nullptr);
		TFHIP_CHECK_LAUNCH();
		return TFHIP_OK;
	}
	float* sums = level_buf;
	float* next = level_buf + ((tiles + 63) & ~size_t(63));
	hipLaunchKernelGGL(scan_tile_sums_f32_kernel, dim3((unsigned)tiles), dim3(kScanThreads), 0, s.stream, in, sums, n);
	TFHIP_CHECK_LAUNCH();
	int rc = scan_f32_recursive(sums, sums, tiles, next);  // in place: sums -> inclusive tile prefixes
	if (rc) return rc;
	hipLaunchKernelGGL(scan_apply_f32_kernel, dim3((unsigned)tiles), dim3(kScanThreads), 0, s.stream, in, out, n, (const float*)sums);
	TFHIP_CHECK_LAUNCH();
	return TFHIP_OK;
}

}  // namespace tfhip

using namespace tfhip;

extern "C" {

int tfhip_scan_inclusive_u32(const uint32_t* in, uint32_t* out, size_t n) {
	TFHIP_REQUIRE_INIT();
	if (n == 0) return TFHIP_OK;
	if (!in || !out) return fail(TFHIP_ERR_ARG, "null pointer passed to tfhip_scan_inclusive_u32");
	State& s = state();
	const size_t tiles = (n + kScanTile - 1) / kScanTile;
	if (tiles > 0x7FFFFFFFull) return fail(TFHIP_ERR_ARG, "scan of %zu elements is too long", n);
	const size_t status_bytes = (tiles + 1) * sizeof(uint64_t);  // + ticket word
	char* base = (char*)scratch(status_bytes);
	if (!base) return TFHIP_ERR_HIP;
	uint64_t* status = (uint64_t*)base;
	uint32_t* ticket = (uint32_t*)(base + tiles * sizeof(uint64_t));
	int rc = tfhip_fill_u32(base, 0u, status_bytes / 4);
	if (rc) return rc;
	hipLaunchKernelGGL(scan_lookback_u32_kernel, dim3((unsigned)tiles), dim3(kScanThreads), 0, s.stream, in, out, n, status, ticket, s.async_error_dev);
	TFHIP_CHECK_LAUNCH();
	return TFHIP_OK;
}

int tfhip_scan_inclusive_i32(const int32_t* in, int32_t* out, size_t n) {
	return tfhip_scan_inclusive_u32((const uint32_t*)in, (uint32_t*)out, n);
}

int tfhip_scan_inclusive_f32(const float* in, float* out, size_t n) {
	TFHIP_REQUIRE_INIT();
	if (n == 0) return TFHIP_OK;
	if (!in || !out) return fail(TFHIP_ERR_ARG, "null pointer passed to tfhip_scan_inclusive_f32");
	// scratch for every level: tiles, tiles/4096, ... each rounded up to 64 floats
	size_t words = 0;
	for (size_t m = (n + kScanTile - 1) / kScanTile; m > 1; m = (m + kScanTile - 1) / kScanTile) words += (m + 63) & ~size_t(63);
	float* level_buf = nullptr;
	if (words) {
		level_buf = (float*)scratch(words * sizeof(float));
		if (!level_buf) return TFHIP_ERR_HIP;
	}
	return scan_f32_recursive(in, out, n, level_buf);
}

}  // extern "C"
