// Inclusive prefix sums over a contiguous array.
//
// The reference computes dim_prefix_sum as a serial loop in ONE thread per scan line
// (TensorFrost/Compiler/Implementations.cpp:305-359,447-449: acc += x[k]; out[k] = acc), so a 1-D
// scan runs on a single thread; the two-level grouped form users write around it
// (Python/TensorFrost/sort.py:39-50) still serialises across groups.
//
// u32 (and i32, which is the same bit pattern under two's complement wrap-around): single pass,
// "decoupled look-back". Tiles of 32768 elements take a ticket in start order, publish their
// aggregate, then look back over the published aggregates / inclusive prefixes of earlier tiles,
// 64 tiles per wave step. One read and one write of the data; integer addition is associative, so
// the result is bit-exact whatever the timing.
//
// f32: addition is not associative, and how far a look-back walks depends on timing, so the chained
// scan would not be reproducible run to run. Floats use reduce-then-scan instead: tile sums, a
// (recursive) scan of the tile sums, then a rescan of each tile from its exclusive prefix -- two reads
// and one write, with a summation order fixed by the tiling.

#include <type_traits>

#include "common.h"

namespace tfhip {

// Tile geometry: `threads` threads hold `vecs` 4-element vectors each.
template <int THREADS, int VECS>
struct ScanCfg {
	static constexpr int threads = THREADS, vecs = VECS, waves = THREADS / 64, tile = THREADS * VECS * 4;
};
// The single-pass chained scan wants few, large tiles: a tile waits about one coherent round trip for its
// predecessors while it sits in registers (2^28 elements: 512 x 8 vectors 392-399 us, 1024 x 8 vectors 386-388 us).
// The three-kernel form has no such wait and runs best with small groups.
using LookbackCfg = ScanCfg<1024, 8>;  // 32768 elements
using SplitCfg = ScanCfg<256, 4>;     // 4096 elements
constexpr int kPollSleep = 8;                                 // x 64 clocks between two polls of one status word
constexpr uint32_t kSpinLimit = 1u << 22;                     // bounded wait of the look-back

constexpr uint64_t kFlagAggregate = 1ull << 32;
constexpr uint64_t kFlagPrefix = 2ull << 32;

template <class T>
struct alignas(16) Vec4 {
	T x, y, z, w;
};

// 32-bit integers: the cross-lane adds run in the vector ALU's data-parallel-primitive paths (shifts within rows of 16
// lanes, then the last lane of a row broadcast to the rows behind it) instead of through group memory's crossbar.
__device__ __forceinline__ uint32_t wave_inclusive_scan(uint32_t v) {
	int x = (int)v;
	x += __builtin_amdgcn_update_dpp(0, x, 0x111, 0xf, 0xf, false);  // row_shr:1
	x += __builtin_amdgcn_update_dpp(0, x, 0x112, 0xf, 0xf, false);  // row_shr:2
	x += __builtin_amdgcn_update_dpp(0, x, 0x114, 0xf, 0xf, false);  // row_shr:4
	x += __builtin_amdgcn_update_dpp(0, x, 0x118, 0xf, 0xf, false);  // row_shr:8
	x += __builtin_amdgcn_update_dpp(0, x, 0x142, 0xa, 0xf, false);  // row_bcast:15 into rows 1 and 3
	x += __builtin_amdgcn_update_dpp(0, x, 0x143, 0xc, 0xf, false);  // row_bcast:31 into rows 2 and 3
	return (uint32_t)x;
}

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
// FULL: the whole tile lies inside the array and the array is 16-byte aligned (decided once per group, so the
// common case carries no per-element bounds arithmetic).
template <class T>
using NativeVec4 = T __attribute__((ext_vector_type(4)));

// The tile is read once and its result is written once: non-temporal accesses, so that neither stays in the caches.
template <class T>
__device__ __forceinline__ Vec4<T> load_vec4_stream(const T* p) {
	const NativeVec4<T> q = __builtin_nontemporal_load(reinterpret_cast<const NativeVec4<T>*>(p));
	return Vec4<T>{q.x, q.y, q.z, q.w};
}
template <class T>
__device__ __forceinline__ void store_vec4_stream(T* p, const Vec4<T>& v) {
	const NativeVec4<T> q = {v.x, v.y, v.z, v.w};
	__builtin_nontemporal_store(q, reinterpret_cast<NativeVec4<T>*>(p));
}

// STREAM: the tile is not read again by a later kernel of the same call.
template <class C, bool FULL, bool STREAM = true, class T>
__device__ __forceinline__ void load_tile(const T* in, size_t base, size_t n, bool aligned, Vec4<T> (&v)[C::vecs]) {
	if (FULL) {
#pragma unroll
		for (int k = 0; k < C::vecs; k++) {
			const T* p = in + base + ((size_t)k * C::threads + threadIdx.x) * 4;
			v[k] = STREAM ? load_vec4_stream(p) : *reinterpret_cast<const Vec4<T>*>(p);
		}
	} else {
		// the ragged last tile, or an array that is not 16-byte aligned. Unrolled like the full form, so that the tile's
		// registers are never indexed by a run-time value (which would move the whole tile to scratch memory).
		// one 64-bit pointer per thread; everything else is 32-bit arithmetic on offsets inside the tile
		const T* p = in + base + (size_t)threadIdx.x * 4;
		const uint32_t limit = n - base < (size_t)C::tile ? (uint32_t)(n - base) : (uint32_t)C::tile;
		const uint32_t first = threadIdx.x * 4u;
#pragma unroll
		for (int k = 0; k < C::vecs; k++) {
			const uint32_t o = first + (uint32_t)k * C::threads * 4u;
			const T* q = p + k * C::threads * 4;
			if (aligned && o + 4u <= limit) {
				v[k] = *reinterpret_cast<const Vec4<T>*>(q);
			} else {
				v[k].x = o < limit ? q[0] : T(0);
				v[k].y = o + 1u < limit ? q[1] : T(0);
				v[k].z = o + 2u < limit ? q[2] : T(0);
				v[k].w = o + 3u < limit ? q[3] : T(0);
			}
		}
	}
}

template <class C, bool FULL, class T>
__device__ __forceinline__ void store_tile(T* out, size_t base, size_t n, bool aligned, const Vec4<T> (&v)[C::vecs]) {
	if (FULL) {
#pragma unroll
		for (int k = 0; k < C::vecs; k++) store_vec4_stream(out + base + ((size_t)k * C::threads + threadIdx.x) * 4, v[k]);
	} else {
		T* p = out + base + (size_t)threadIdx.x * 4;
		const uint32_t limit = n - base < (size_t)C::tile ? (uint32_t)(n - base) : (uint32_t)C::tile;
		const uint32_t first = threadIdx.x * 4u;
#pragma unroll
		for (int k = 0; k < C::vecs; k++) {
			const uint32_t o = first + (uint32_t)k * C::threads * 4u;
			T* q = p + k * C::threads * 4;
			if (aligned && o + 4u <= limit) {
				*reinterpret_cast<Vec4<T>*>(q) = v[k];
			} else {
				if (o < limit) q[0] = v[k].x;
				if (o + 1u < limit) q[1] = v[k].y;
				if (o + 2u < limit) q[2] = v[k].z;
				if (o + 3u < limit) q[3] = v[k].w;
			}
		}
	}
}

// Turns v[] into the inclusive scan of the tile (without any cross-tile prefix) and returns the tile
// total to every thread. lds: C::vecs * C::waves elements.
struct NoHook {
	template <class T>
	__device__ __forceinline__ void operator()(T) const {}
};

// on_total(total) runs in every thread as soon as the tile's total is known, before the offsets are applied.
template <class C, class T, class Hook = NoHook>
__device__ __forceinline__ T scan_tile_in_registers(Vec4<T> (&v)[C::vecs], T* lds, Hook on_total = Hook()) {
	const int lane = threadIdx.x & 63;
	const int wave = threadIdx.x >> 6;
	T excl[C::vecs];  // sum of the vectors of lower lanes of this wave, same k
#pragma unroll
	for (int k = 0; k < C::vecs; k++) {
		v[k].y += v[k].x;
		v[k].z += v[k].y;
		v[k].w += v[k].z;
		T incl = wave_inclusive_scan(v[k].w);
		if (lane == 63) lds[k * C::waves + wave] = incl;
		if constexpr (std::is_integral<T>::value) {
			excl[k] = incl - v[k].w;  // exact in wrap-around arithmetic
		} else {
			T up = __shfl_up(incl, 1, 64);
			excl[k] = lane == 0 ? T(0) : up;
		}
	}
	__syncthreads();
	if constexpr (std::is_integral<T>::value && C::vecs * C::waves <= 128 && 64 % C::waves == 0) {
		// the vecs * waves partial sums fit one wave (one or two values per lane): every wave scans them in registers and
		// reads the offsets it needs as wave-uniform values
		constexpr int kPartials = C::vecs * C::waves;
		const int uniform_wave = __builtin_amdgcn_readfirstlane(wave);
		const T part = lane < kPartials ? lds[lane] : T(0);
		const T incl = wave_inclusive_scan(part);
		const T before_all = incl - part;
		T total = (T)__builtin_amdgcn_readlane((int)incl, 63);
		T before_upper = T(0);  // the same for partial sums 64 .. 127
		if constexpr (kPartials > 64) {
			const T upper = lane + 64 < kPartials ? lds[64 + lane] : T(0);
			const T upper_incl = wave_inclusive_scan(upper);
			before_upper = upper_incl - upper + total;
			total += (T)__builtin_amdgcn_readlane((int)upper_incl, 63);
		}
		on_total(total);
#pragma unroll
		for (int k = 0; k < C::vecs; k++) {
			// waves divides 64, so the partial sums of one k lie on one side of the split
			const T offset = (k * C::waves < 64 ? (T)__builtin_amdgcn_readlane((int)before_all, (k * C::waves) % 64 + uniform_wave)
			                                    : (T)__builtin_amdgcn_readlane((int)before_upper, (k * C::waves) % 64 + uniform_wave)) +
			                 excl[k];
			v[k].x += offset;
			v[k].y += offset;
			v[k].z += offset;
			v[k].w += offset;
		}
		return total;
	}
	T total = T(0);
#pragma unroll
	for (int k = 0; k < C::vecs; k++) {
		T before = total;  // everything in vectors of lower k, then lower waves of this k
#pragma unroll
		for (int w = 0; w < C::waves; w++) {
			T t = lds[k * C::waves + w];
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
template <class C, bool FULL>
__device__ __forceinline__ void scan_lookback_u32_body(const uint32_t* in, uint32_t* out, size_t n, uint64_t* status, uint32_t* async_error, uint32_t spin_limit,
                                                       uint32_t tile, bool aligned, uint32_t* lds, uint32_t& s_prefix) {
	static_assert(C::vecs * C::waves <= 128 && 64 % C::waves == 0, "the tile's total is taken from the one-wave scan of its partial sums");
	const size_t base = (size_t)tile * C::tile;
	Vec4<uint32_t> v[C::vecs];
	load_tile<C, FULL>(in, base, n, aligned, v);
	// A first look at the predecessors' status words, issued right behind the tile's own loads: the words travel while
	// the tile's data does. Tiles run staggered, so the nearest predecessors have usually published by then and the
	// look-back below finds what it needs without a round trip of its own.
	constexpr int kWidth = 8;  // tiles inspected per look-back step
	uint64_t probe = 0;
	if (threadIdx.x < kWidth && tile > 0) {
		const int64_t t = (int64_t)tile - 1 - (int64_t)threadIdx.x;
		probe = t >= 0 ? status_load(&status[t]) : kFlagPrefix;
	}
	// The tile's total is published the moment it is known (after the first half of the scan): what later tiles wait
	// for is this word. Nothing may delay it, not even the first look above.
	const uint32_t total = scan_tile_in_registers<C>(v, lds, [&](uint32_t tile_total) {
		if (threadIdx.x == 0) status_store(&status[tile], (tile == 0 ? kFlagPrefix : kFlagAggregate) | tile_total);
	});

	if (threadIdx.x < 64) {  // wave 0 resolves the tile's exclusive prefix
		const int lane = threadIdx.x;
		uint32_t exclusive = 0;
		if (tile > 0) {
			uint32_t mine = 0;  // this lane's share of the exclusive prefix; added across the wave once at the end
			int64_t look = (int64_t)tile - 1;
			bool done = false, blocked = false;
			bool have = true;
			// Lane i inspects tile look - i, for i < kWidth. A wider window finds a published prefix in fewer steps but
			// every status word read crosses the fabric beside the data streams: without the first look above, 2^28
			// elements take 434 us with 64 tiles per step, 401 us with 8 or 16, 415 us with 2 and 450 us with 1; several
			// windows fetched at once are slower still (2 x 64: 468 us, 4 x 64: 525 us). With the first look: 392 us;
			// with no look-back at all (wrong results) the kernel moves the data in 365 us.
			uint32_t spins = 0;
			while (!done) {
				// Tile `look` has not published: wait for that one word with one lane, and not too eagerly.
				while (blocked) {
					if (++spins > spin_limit) {  // an earlier tile never published: give up, flag it
						if (lane == 0) *async_error = kAsyncErrLookbackTimeout;
						done = true;
						break;
					}
					__builtin_amdgcn_s_sleep(kPollSleep);
					const uint64_t one = lane == 0 ? status_load(&status[look]) : 0;
					blocked = __ballot((one >> 32) != 0) == 0;
				}
				if (done) break;
				spins = 0;  // the bound is per wait for one tile's word, not for the whole walk
				uint64_t s = probe;  // the first step uses what the first look brought (lanes >= kWidth hold 0)
				if (!have) {
					const int64_t t = look - lane;
					s = lane >= kWidth ? 0 : t >= 0 ? status_load(&status[t]) : kFlagPrefix;  // before tile 0: prefix 0
				}
				have = false;
				const uint64_t not_ready = __ballot((s >> 32) == 0);
				const uint64_t has_prefix = __ballot((s >> 32) == 2);
				// lanes below `usable` have published; the nearest inclusive prefix among them ends the walk,
				// otherwise their aggregates are taken and the walk resumes at the first tile that has not published
				const int usable = not_ready ? __builtin_ctzll(not_ready) : 64;
				const int stop = has_prefix ? __builtin_ctzll(has_prefix) : 64;
				const int take = stop < usable ? stop + 1 : usable;
				if (lane < take) mine += (uint32_t)s;
				if (stop < usable) {
					done = true;
				} else {
					look -= take;
					blocked = take < kWidth;
				}
			}
			exclusive = wave_reduce(mine, [](uint32_t a, uint32_t b) { return a + b; });
			if (lane == 0) status_store(&status[tile], kFlagPrefix | (uint64_t)(uint32_t)(exclusive + total));
		}
		if (lane == 0) s_prefix = exclusive;
	}
	__syncthreads();
	const uint32_t prefix = s_prefix;
#pragma unroll
	for (int k = 0; k < C::vecs; k++) {
		v[k].x += prefix;
		v[k].y += prefix;
		v[k].z += prefix;
		v[k].w += prefix;
	}
	store_tile<C, FULL>(out, base, n, aligned, v);
}

// ---- status words that need no allocation -------------------------------------------------------------------
// The allocation-free entry point keeps its ticket (first 8 bytes) and one status word per tile in this array, which
// every GPU the library runs on holds from load until the process ends. In host code the array's name is only a handle
// for hipGetSymbolAddress; the device address found at set-up is what kernels and fills are given.
constexpr size_t kStaticScanMaxElements = size_t(1) << 30;
constexpr size_t kStaticScanMaxTiles = kStaticScanMaxElements / LookbackCfg::tile;  // 32768
constexpr int kStaticScratchDevices = 64;
static __device__ __align__(256) unsigned char static_scratch[(kStaticScanMaxTiles + 1) * sizeof(uint64_t)];  // 512 KiB + 8 B
static void* g_static_scratch_ptr[kStaticScratchDevices];

int locate_static_scratch(int device) {
	if (device < 0 || device >= kStaticScratchDevices) return TFHIP_OK;  // the entry point reports it when called
	void* ptr = nullptr;
	hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(static_scratch));
	if (e != hipSuccess) return fail_hip(e, "hipGetSymbolAddress(static_scratch)");
	g_static_scratch_ptr[device] = ptr;
	return TFHIP_OK;
}

// Two 1024-thread groups per compute unit (eight waves per SIMD): the tile's registers must stay within 64 per lane.
template <class C>
__global__ __launch_bounds__(C::threads) __attribute__((amdgpu_waves_per_eu(8, 8))) void scan_lookback_u32_kernel(const uint32_t* in, uint32_t* out, size_t n,
                                                                          uint64_t* status, uint32_t* ticket, uint32_t* async_error, uint32_t spin_limit) {
	__shared__ uint32_t lds[C::vecs * C::waves];
	__shared__ uint32_t s_tile;
	__shared__ uint32_t s_prefix;
	if (threadIdx.x == 0) s_tile = atomicAdd(ticket, 1u);
	__syncthreads();
	const uint32_t tile = s_tile;

	const bool aligned = ((((uintptr_t)in) | ((uintptr_t)out)) & 15) == 0;
	if (aligned && ((size_t)tile + 1) * C::tile <= n)
		scan_lookback_u32_body<C, true>(in, out, n, status, async_error, spin_limit, tile, aligned, lds, s_prefix);
	else
		scan_lookback_u32_body<C, false>(in, out, n, status, async_error, spin_limit, tile, aligned, lds, s_prefix);
}

// ---- f32: reduce-then-scan ----------------------------------------------------------------------

// The bodies are instantiated separately for full and ragged tiles so that the full form carries no bounds tests.
template <class C, bool FULL, class T>
__device__ __forceinline__ void scan_tile_sums_body(const T* __restrict__ in, T* __restrict__ sums, size_t n, size_t base, bool aligned, T* lds) {
	Vec4<T> v[C::vecs];
	load_tile<C, FULL, false>(in, base, n, aligned, v);  // the second kernel reads the tile again: leave it to the caches
	// Same arithmetic as the rescan below, so that prefix + local scan reproduces these totals exactly.
	const T total = scan_tile_in_registers<C>(v, lds);
	if (threadIdx.x == 0) sums[blockIdx.x] = total;
}

template <class C, class T>
__global__ __launch_bounds__(C::threads) void scan_tile_sums_kernel(const T* __restrict__ in, T* __restrict__ sums, size_t n) {
	__shared__ T lds[C::vecs * C::waves];
	const size_t base = (size_t)blockIdx.x * C::tile;
	const bool aligned = (((uintptr_t)in) & 15) == 0;
	if (aligned && base + C::tile <= n)
		scan_tile_sums_body<C, true>(in, sums, n, base, aligned, lds);
	else
		scan_tile_sums_body<C, false>(in, sums, n, base, aligned, lds);
}

// out = inclusive scan of the tile + exclusive prefix of the tile (prefix[tile-1], 0 for tile 0).
template <class C, bool FULL, class T>
__device__ __forceinline__ void scan_apply_body(const T* in, T* out, size_t n, const T* tile_inclusive, size_t base, bool aligned, T* lds) {
	Vec4<T> v[C::vecs];
	load_tile<C, FULL>(in, base, n, aligned, v);
	(void)scan_tile_in_registers<C>(v, lds);
	const T prefix = (blockIdx.x == 0 || tile_inclusive == nullptr) ? T(0) : tile_inclusive[blockIdx.x - 1];
#pragma unroll
	for (int k = 0; k < C::vecs; k++) {
		v[k].x += prefix;
		v[k].y += prefix;
		v[k].z += prefix;
		v[k].w += prefix;
	}
	store_tile<C, FULL>(out, base, n, aligned, v);
}

template <class C, class T>
__global__ __launch_bounds__(C::threads) void scan_apply_kernel(const T* in, T* out, size_t n, const T* tile_inclusive) {
	__shared__ T lds[C::vecs * C::waves];
	const size_t base = (size_t)blockIdx.x * C::tile;
	const bool aligned = ((((uintptr_t)in) | ((uintptr_t)out)) & 15) == 0;
	if (aligned && base + C::tile <= n)
		scan_apply_body<C, true>(in, out, n, tile_inclusive, base, aligned, lds);
	else
		scan_apply_body<C, false>(in, out, n, tile_inclusive, base, aligned, lds);
}

// level_buf: scratch for all recursion levels, laid out by the caller.
template <class T>
static int scan_recursive(const T* in, T* out, size_t n, T* level_buf) {
	State& s = state();
	const size_t tiles = (n + SplitCfg::tile - 1) / SplitCfg::tile;
	if (tiles > 0x7FFFFFFFull) return fail(TFHIP_ERR_ARG, "scan of %zu elements is too long", n);
	if (tiles == 1) {
		hipLaunchKernelGGL((scan_apply_kernel<SplitCfg, T>), dim3(1), dim3(SplitCfg::threads), 0, s.stream, in, out, n, (const T*)nullptr);
		TFHIP_CHECK_LAUNCH();
		return TFHIP_OK;
	}
	T* sums = level_buf;
	T* next = level_buf + ((tiles + 63) & ~size_t(63));
	hipLaunchKernelGGL((scan_tile_sums_kernel<SplitCfg, T>), dim3((unsigned)tiles), dim3(SplitCfg::threads), 0, s.stream, in, sums, n);
	TFHIP_CHECK_LAUNCH();
	int rc = scan_recursive<T>(sums, sums, tiles, next);  // in place: sums -> inclusive tile prefixes
	if (rc) return rc;
	hipLaunchKernelGGL((scan_apply_kernel<SplitCfg, T>), dim3((unsigned)tiles), dim3(SplitCfg::threads), 0, s.stream, in, out, n, (const T*)sums);
	TFHIP_CHECK_LAUNCH();
	return TFHIP_OK;
}

template <class T>
static int scan_reduce_then_scan(const T* in, T* out, size_t n) {
	// scratch for every level: tiles, tiles/tile, ... each rounded up to 64 words
	size_t words = 0;
	for (size_t m = (n + SplitCfg::tile - 1) / SplitCfg::tile; m > 1; m = (m + SplitCfg::tile - 1) / SplitCfg::tile) words += (m + 63) & ~size_t(63);
	T* level_buf = nullptr;
	if (words) {
		level_buf = (T*)scratch(words * sizeof(T));
		if (!level_buf) return TFHIP_ERR_HIP;
	}
	return scan_recursive<T>(in, out, n, level_buf);
}

// ---- many rows, each scanned on its own ------------------------------------------------------------------------
//
// A row may be cut into `segs` segments of `seg_len` elements (few long rows: more groups than rows); a segment is
// the unit of work below and segs == 1 the common case.
//
// WAVES waves (one or four) own a segment and walk it in chunks of WAVES * 256 elements, a 16-byte vector per lane,
// two chunks per trip so that the second chunk's loads are in flight while the first is scanned. The running total
// stays in a register; with four waves the wave totals of a chunk cross through group memory (two slots, one barrier
// per chunk). A 256-thread group holds 4 / WAVES segments.
// TOTALS: nothing is stored but the segment's total, totals[segment]. Otherwise `offsets`, if given, holds what
// precedes each segment in its row.
template <class T, int WAVES, bool VEC, bool TOTALS>
__global__ __launch_bounds__(256) void scan_rows_kernel(const T* in, T* out, size_t rows, size_t cols, size_t segs, size_t seg_len, T* totals_out,
                                                        const T* __restrict__ offsets) {
	__shared__ T totals[2][4];
	constexpr int kPerGroup = 4 / WAVES;
	constexpr size_t kChunk = (size_t)WAVES * 256;
	const int lane = threadIdx.x & 63;
	const int wave = threadIdx.x >> 6;
	const int wave_in_row = wave % WAVES;
	const size_t item = (size_t)blockIdx.x * kPerGroup + wave / WAVES;
	const bool active = item < rows * segs;  // WAVES == 4: the whole group shares the segment, so barriers are uniform
	const size_t row = active ? item / segs : 0;
	const size_t first = active ? (item - row * segs) * seg_len : 0;
	const size_t len = active ? (first + seg_len < cols ? seg_len : cols - first) : 0;
	const T* pin = in + row * cols + first;
	T* pout = TOTALS ? nullptr : out + row * cols + first;
	T carry = (!TOTALS && offsets && active) ? offsets[item] : T(0);
	int slot = 0;
	auto load = [&](size_t c) {
		Vec4<T> v = {T(0), T(0), T(0), T(0)};
		if (VEC) {
			if (c < len) v = *reinterpret_cast<const Vec4<T>*>(pin + c);
		} else {
			if (c < len) v.x = pin[c];
			if (c + 1 < len) v.y = pin[c + 1];
			if (c + 2 < len) v.z = pin[c + 2];
			if (c + 3 < len) v.w = pin[c + 3];
		}
		return v;
	};
	auto scan_and_store = [&](Vec4<T> v, size_t c) {
		v.y += v.x;
		v.z += v.y;
		v.w += v.z;
		const T incl = wave_inclusive_scan(v.w);
		const T up = __shfl_up(incl, 1, 64);
		T before = lane == 0 ? T(0) : up;  // lower lanes of this wave
		T chunk_total = __shfl(incl, 63, 64);
		if (WAVES > 1) {
			if (lane == 63) totals[slot][wave_in_row] = incl;
			__syncthreads();
			chunk_total = T(0);
#pragma unroll
			for (int w = 0; w < WAVES; w++) {
				const T t = totals[slot][w];
				if (w < wave_in_row) before += t;
				chunk_total += t;
			}
			slot ^= 1;
		}
		const T offset = carry + before;
		carry += chunk_total;
		if (TOTALS) return;
		v.x += offset;
		v.y += offset;
		v.z += offset;
		v.w += offset;
		if (VEC) {
			if (c < len) *reinterpret_cast<Vec4<T>*>(pout + c) = v;
		} else {
			if (c < len) pout[c] = v.x;
			if (c + 1 < len) pout[c + 1] = v.y;
			if (c + 2 < len) pout[c + 2] = v.z;
			if (c + 3 < len) pout[c + 3] = v.w;
		}
	};
	const size_t mine = ((size_t)wave_in_row * 64 + lane) * 4;
	// with four waves the whole group shares the segment, so `len` and with it the barriers are uniform
	for (size_t base = 0; base < len; base += 2 * kChunk) {
		const Vec4<T> a = load(base + mine);
		const Vec4<T> b = load(base + kChunk + mine);
		scan_and_store(a, base + mine);
		if (base + kChunk < len) scan_and_store(b, base + kChunk + mine);
	}
	if (TOTALS && active && lane == 0 && wave_in_row == 0) totals_out[item] = carry;
}

// Short rows (cols <= 128, 16-byte aligned): LANES lanes own a row with one vector each, so a wave scans 64 / LANES
// rows at once; four such row groups per wave.
template <class T, int LANES>
__global__ __launch_bounds__(256) void scan_rows_lanes_kernel(const T* in, T* out, size_t rows, size_t cols) {
	constexpr int kRowsPerStep = 64 / LANES;
	const int lane = threadIdx.x & 63;
	const int sub = lane % LANES, which = lane / LANES;
	const size_t wave = (size_t)blockIdx.x * 4 + (threadIdx.x >> 6);
	const size_t row0 = wave * (kRowsPerStep * 4) + which;
	const bool has = (size_t)sub * 4 < cols;
	Vec4<T> v[4];
#pragma unroll
	for (int u = 0; u < 4; u++) {
		const size_t row = row0 + (size_t)u * kRowsPerStep;
		v[u] = Vec4<T>{T(0), T(0), T(0), T(0)};
		if (has && row < rows) v[u] = *reinterpret_cast<const Vec4<T>*>(in + row * cols + sub * 4);
	}
#pragma unroll
	for (int u = 0; u < 4; u++) {
		v[u].y += v[u].x;
		v[u].z += v[u].y;
		v[u].w += v[u].z;
		T incl = v[u].w;
#pragma unroll
		for (int off = 1; off < LANES; off <<= 1) {
			const T o = __shfl_up(incl, off, LANES);
			if (sub >= off) incl += o;
		}
		const T up = __shfl_up(incl, 1, LANES);
		const T before = sub == 0 ? T(0) : up;  // the lanes below in this row
		const size_t row = row0 + (size_t)u * kRowsPerStep;
		if (has && row < rows) {
			Vec4<T> r = {v[u].x + before, v[u].y + before, v[u].z + before, v[u].w + before};
			*reinterpret_cast<Vec4<T>*>(out + row * cols + sub * 4) = r;
		}
	}
}

// One wave per row over the totals of its segments: offsets[row, s] = totals[row, 0] + ... + totals[row, s - 1].
template <class T>
__global__ __launch_bounds__(256) void scan_segment_offsets_kernel(const T* __restrict__ totals, T* __restrict__ offsets, size_t rows, size_t segs) {
	const int lane = threadIdx.x & 63;
	const size_t row = (size_t)blockIdx.x * 4 + (threadIdx.x >> 6);
	if (row >= rows) return;
	T carry = T(0);
	for (size_t base = 0; base < segs; base += 64) {
		const size_t i = base + lane;
		const T t = i < segs ? totals[row * segs + i] : T(0);
		const T incl = wave_inclusive_scan(t);
		if (i < segs) offsets[row * segs + i] = carry + (incl - t);
		carry += __shfl(incl, 63, 64);
	}
}

template <class T, bool TOTALS>
static void launch_scan_rows(const T* in, T* out, size_t rows, size_t cols, size_t segs, size_t seg_len, T* totals, const T* offsets, bool vec, bool wide) {
	State& s = state();
	const size_t items = rows * segs;
	const dim3 grid((unsigned)(wide ? items : (items + 3) / 4)), block(256);
	if (wide) {
		if (vec) hipLaunchKernelGGL((scan_rows_kernel<T, 4, true, TOTALS>), grid, block, 0, s.stream, in, out, rows, cols, segs, seg_len, totals, offsets);
		else hipLaunchKernelGGL((scan_rows_kernel<T, 4, false, TOTALS>), grid, block, 0, s.stream, in, out, rows, cols, segs, seg_len, totals, offsets);
	} else {
		if (vec) hipLaunchKernelGGL((scan_rows_kernel<T, 1, true, TOTALS>), grid, block, 0, s.stream, in, out, rows, cols, segs, seg_len, totals, offsets);
		else hipLaunchKernelGGL((scan_rows_kernel<T, 1, false, TOTALS>), grid, block, 0, s.stream, in, out, rows, cols, segs, seg_len, totals, offsets);
	}
}

// ---- prefix sums down the columns of [batch] matrices [rows, cols] ------------------------------------------------
//
// One thread per (matrix, column) keeps neighbouring lanes on neighbouring words. The rows are cut into slabs so that there
// are enough threads: (1) every (slab, column) sums its rows, (2) a thread per column turns the slab sums into what
// precedes each slab, (3) every (slab, column) walks its rows again with that carry. sums: [batch, slabs, cols].
template <class T, bool APPLY>
__global__ __launch_bounds__(256) void scan_cols_kernel(const T* in, T* out, T* sums, size_t batch, size_t rows, size_t cols, size_t slabs, size_t rows_per_slab) {
	const size_t flat = (size_t)blockIdx.x * 256 + threadIdx.x;  // over batch * cols: narrow matrices share a wave
	if (flat >= batch * cols) return;
	const size_t b = flat / cols, col = flat - b * cols;
	const size_t slab = blockIdx.y;
	const size_t r0 = slab * rows_per_slab;
	const size_t r1 = r0 + rows_per_slab < rows ? r0 + rows_per_slab : rows;
	const T* pin = in + (b * rows + r0) * cols + col;
	T carry = (APPLY && sums) ? sums[(b * slabs + slab) * cols + col] : T(0);  // no sums: a single slab
	if (APPLY) {
		T* pout = out + (b * rows + r0) * cols + col;
		size_t r = r0;
		for (; r + 3 < r1; r += 4) {  // four loads in flight
			const T v0 = pin[0], v1 = pin[cols], v2 = pin[2 * cols], v3 = pin[3 * cols];
			carry += v0;
			pout[0] = carry;
			carry += v1;
			pout[cols] = carry;
			carry += v2;
			pout[2 * cols] = carry;
			carry += v3;
			pout[3 * cols] = carry;
			pin += 4 * cols;
			pout += 4 * cols;
		}
		for (; r < r1; r++) {
			carry += *pin;
			*pout = carry;
			pin += cols;
			pout += cols;
		}
	} else {
		T c1 = T(0), c2 = T(0), c3 = T(0);
		size_t r = r0;
		for (; r + 3 < r1; r += 4) {
			carry += pin[0];
			c1 += pin[cols];
			c2 += pin[2 * cols];
			c3 += pin[3 * cols];
			pin += 4 * cols;
		}
		for (; r < r1; r++) {
			carry += *pin;
			pin += cols;
		}
		sums[(b * slabs + slab) * cols + col] = (carry + c1) + (c2 + c3);
	}
}

template <class T>
__global__ __launch_bounds__(256) void scan_cols_offsets_kernel(T* sums, size_t batch, size_t cols, size_t slabs) {
	const size_t flat = (size_t)blockIdx.x * 256 + threadIdx.x;
	if (flat >= batch * cols) return;
	const size_t b = flat / cols, col = flat - b * cols;
	T* p = sums + b * slabs * cols + col;
	T carry = T(0);
	size_t sl = 0;
	for (; sl + 7 < slabs; sl += 8) {  // eight loads in flight before the first store (same array: the compiler keeps their order)
		T t[8];
#pragma unroll
		for (int u = 0; u < 8; u++) t[u] = p[(sl + u) * cols];
#pragma unroll
		for (int u = 0; u < 8; u++) {
			p[(sl + u) * cols] = carry;
			carry += t[u];
		}
	}
	for (; sl < slabs; sl++) {
		const T t = p[sl * cols];
		p[sl * cols] = carry;
		carry += t;
	}
}

template <class T>
static int scan_cols(const T* in, T* out, size_t batch, size_t rows, size_t cols) {
	State& s = state();
	// about 1024 threads per compute unit, slabs of at least 16 rows and at most 65535 of them
	size_t slabs = ((size_t)s.compute_units * 1024 + batch * cols - 1) / (batch * cols);
	if (slabs > rows / 16) slabs = rows / 16;
	if (slabs < 1) slabs = 1;
	if (slabs > 1024) slabs = 1024;
	size_t rows_per_slab = (rows + slabs - 1) / slabs;
	slabs = (rows + rows_per_slab - 1) / rows_per_slab;
	const size_t col_groups = (batch * cols + 255) / 256;
	if (col_groups > 0x7FFFFFFFull) return fail(TFHIP_ERR_ARG, "too many columns (%zu x %zu)", batch, cols);
	T* sums = nullptr;
	if (slabs > 1) {
		sums = (T*)scratch(batch * slabs * cols * sizeof(T));
		if (!sums) return TFHIP_ERR_HIP;
	}
	const dim3 grid((unsigned)col_groups, (unsigned)slabs), block(256);
	if (slabs > 1) {
		hipLaunchKernelGGL((scan_cols_kernel<T, false>), grid, block, 0, s.stream, in, out, sums, batch, rows, cols, slabs, rows_per_slab);
		TFHIP_CHECK_LAUNCH();
		hipLaunchKernelGGL(scan_cols_offsets_kernel<T>, dim3((unsigned)col_groups), block, 0, s.stream, sums, batch, cols, slabs);
		TFHIP_CHECK_LAUNCH();
	}
	hipLaunchKernelGGL((scan_cols_kernel<T, true>), grid, block, 0, s.stream, in, out, sums, batch, rows, cols, slabs, rows_per_slab);
	TFHIP_CHECK_LAUNCH();
	return TFHIP_OK;
}

template <class T>
static int scan_rows(const T* in, T* out, size_t rows, size_t cols) {
	State& s = state();
	const bool vec = (cols % 4 == 0) && (((uintptr_t)in | (uintptr_t)out) & 15) == 0;
	if (vec && cols <= 128 && rows >= 64) {
		const size_t vecs = cols / 4;
		const int lanes = vecs <= 1 ? 1 : vecs <= 2 ? 2 : vecs <= 4 ? 4 : vecs <= 8 ? 8 : vecs <= 16 ? 16 : 32;
		const size_t rows_per_group = (size_t)(64 / lanes) * 16;
		const size_t groups = (rows + rows_per_group - 1) / rows_per_group;
		if (groups > 0x7FFFFFFFull) return fail(TFHIP_ERR_ARG, "too many rows (%zu)", rows);
		const dim3 grid((unsigned)groups), block(256);
		switch (lanes) {
			case 1: hipLaunchKernelGGL((scan_rows_lanes_kernel<T, 1>), grid, block, 0, s.stream, in, out, rows, cols); break;
			case 2: hipLaunchKernelGGL((scan_rows_lanes_kernel<T, 2>), grid, block, 0, s.stream, in, out, rows, cols); break;
			case 4: hipLaunchKernelGGL((scan_rows_lanes_kernel<T, 4>), grid, block, 0, s.stream, in, out, rows, cols); break;
			case 8: hipLaunchKernelGGL((scan_rows_lanes_kernel<T, 8>), grid, block, 0, s.stream, in, out, rows, cols); break;
			case 16: hipLaunchKernelGGL((scan_rows_lanes_kernel<T, 16>), grid, block, 0, s.stream, in, out, rows, cols); break;
			default: hipLaunchKernelGGL((scan_rows_lanes_kernel<T, 32>), grid, block, 0, s.stream, in, out, rows, cols); break;
		}
		TFHIP_CHECK_LAUNCH();
		return TFHIP_OK;
	}
	// Few long rows: cut them so that there are about four groups per compute unit, scan the segments' totals, then
	// scan the segments with what precedes them.
	size_t segs = 1, seg_len = cols;
	const size_t want = (size_t)s.compute_units * 4;
	if (rows < want && cols >= 32768) {
		segs = (want + rows - 1) / rows;
		seg_len = ((cols + segs - 1) / segs + 2047) & ~size_t(2047);  // whole two-chunk trips
		if (seg_len < 8192) seg_len = 8192;
		segs = (cols + seg_len - 1) / seg_len;
	}
	if (rows * segs > 0x7FFFFFFFull) return fail(TFHIP_ERR_ARG, "too many rows (%zu)", rows);
	const bool wide = seg_len > 1024;  // four waves per segment
	if (segs == 1) {
		launch_scan_rows<T, false>(in, out, rows, cols, 1, cols, nullptr, nullptr, vec, wide);
		TFHIP_CHECK_LAUNCH();
		return TFHIP_OK;
	}
	const size_t n = rows * segs;
	const size_t half = (n * sizeof(T) + 255) & ~size_t(255);
	char* base = (char*)scratch(2 * half);
	if (!base) return TFHIP_ERR_HIP;
	T* totals = (T*)base;
	T* offsets = (T*)(base + half);
	launch_scan_rows<T, true>(in, nullptr, rows, cols, segs, seg_len, totals, nullptr, vec, wide);
	TFHIP_CHECK_LAUNCH();
	hipLaunchKernelGGL(scan_segment_offsets_kernel<T>, dim3((unsigned)((rows + 3) / 4)), dim3(256), 0, s.stream, (const T*)totals, offsets, rows, segs);
	TFHIP_CHECK_LAUNCH();
	launch_scan_rows<T, false>(in, out, rows, cols, segs, seg_len, nullptr, (const T*)offsets, vec, wide);
	TFHIP_CHECK_LAUNCH();
	return TFHIP_OK;
}

}  // namespace tfhip

using namespace tfhip;

extern "C" {

// Rows of a [rows, cols] matrix, each scanned on its own. Few long rows go through the device-wide scan one after
// the other; many rows get one or four waves each.
int tfhip_scan_inclusive_rows_u32(const uint32_t* in, uint32_t* out, size_t rows, size_t cols) {
	TFHIP_REQUIRE_INIT();
	if (rows == 0 || cols == 0) return TFHIP_OK;
	if (!in || !out) return fail(TFHIP_ERR_ARG, "null pointer passed to tfhip_scan_inclusive_rows_u32");
	if (rows <= 4 && cols >= ((size_t)1 << 22)) {
		for (size_t r = 0; r < rows; r++) {
			int rc = tfhip_scan_inclusive_u32(in + r * cols, out + r * cols, cols);
			if (rc) return rc;
		}
		return TFHIP_OK;
	}
	return scan_rows<uint32_t>(in, out, rows, cols);
}

int tfhip_scan_inclusive_rows_f32(const float* in, float* out, size_t rows, size_t cols) {
	TFHIP_REQUIRE_INIT();
	if (rows == 0 || cols == 0) return TFHIP_OK;
	if (!in || !out) return fail(TFHIP_ERR_ARG, "null pointer passed to tfhip_scan_inclusive_rows_f32");
	if (rows <= 4 && cols >= ((size_t)1 << 22)) {
		for (size_t r = 0; r < rows; r++) {
			int rc = tfhip_scan_inclusive_f32(in + r * cols, out + r * cols, cols);
			if (rc) return rc;
		}
		return TFHIP_OK;
	}
	return scan_rows<float>(in, out, rows, cols);
}

int tfhip_scan_inclusive_cols_u32(const uint32_t* in, uint32_t* out, size_t batch, size_t rows, size_t cols) {
	TFHIP_REQUIRE_INIT();
	if (batch == 0 || rows == 0 || cols == 0) return TFHIP_OK;
	if (!in || !out) return fail(TFHIP_ERR_ARG, "null pointer passed to tfhip_scan_inclusive_cols_u32");
	return scan_cols<uint32_t>(in, out, batch, rows, cols);
}

int tfhip_scan_inclusive_cols_f32(const float* in, float* out, size_t batch, size_t rows, size_t cols) {
	TFHIP_REQUIRE_INIT();
	if (batch == 0 || rows == 0 || cols == 0) return TFHIP_OK;
	if (!in || !out) return fail(TFHIP_ERR_ARG, "null pointer passed to tfhip_scan_inclusive_cols_f32");
	return scan_cols<float>(in, out, batch, rows, cols);
}

int tfhip_scan_inclusive_u32(const uint32_t* in, uint32_t* out, size_t n) {
	TFHIP_REQUIRE_INIT();
	if (n == 0) return TFHIP_OK;
	if (!in || !out) return fail(TFHIP_ERR_ARG, "null pointer passed to tfhip_scan_inclusive_u32");
	State& s = state();
	const size_t tiles = (n + LookbackCfg::tile - 1) / LookbackCfg::tile;
	if (tiles > 0x7FFFFFFFull) return fail(TFHIP_ERR_ARG, "scan of %zu elements is too long", n);
	const size_t status_bytes = (tiles + 1) * sizeof(uint64_t);  // + ticket word
	char* base = (char*)scratch(status_bytes);
	if (!base) return TFHIP_ERR_HIP;
	uint64_t* status = (uint64_t*)base;
	uint32_t* ticket = (uint32_t*)(base + tiles * sizeof(uint64_t));
	int rc = tfhip_fill_u32(base, 0u, status_bytes / 4);
	if (rc) return rc;
	hipLaunchKernelGGL(scan_lookback_u32_kernel<LookbackCfg>, dim3((unsigned)tiles), dim3(LookbackCfg::threads), 0, s.stream, in, out, n, status, ticket, s.async_error_dev, kSpinLimit);
	TFHIP_CHECK_LAUNCH();
	return TFHIP_OK;
}

// The scan with its first tile missing: tickets start at 1, so nobody publishes tile 0 and every look-back that reaches
// it runs into its spin limit, reports through the error word and carries on with what it has. Every group stores its
// tile and exits; nothing waits without bound.
int tfhip_test_scan_u32_first_tile_absent(const uint32_t* in, uint32_t* out, size_t n, uint32_t spin_limit) {
	TFHIP_REQUIRE_INIT();
	if (!in || !out) return fail(TFHIP_ERR_ARG, "null pointer passed to tfhip_test_scan_u32_first_tile_absent");
	State& s = state();
	const size_t tiles = (n + LookbackCfg::tile - 1) / LookbackCfg::tile;
	if (tiles < 2 || tiles > 32768) return fail(TFHIP_ERR_ARG, "tfhip_test_scan_u32_first_tile_absent needs 2 .. 32768 tiles of %d elements; got %zu", LookbackCfg::tile, tiles);
	if (spin_limit == 0 || spin_limit > 4096) return fail(TFHIP_ERR_ARG, "spin limit %u outside 1 .. 4096", spin_limit);
	const size_t status_bytes = (tiles + 1) * sizeof(uint64_t);
	char* base = (char*)scratch(status_bytes);
	if (!base) return TFHIP_ERR_HIP;
	uint64_t* status = (uint64_t*)base;
	uint32_t* ticket = (uint32_t*)(base + tiles * sizeof(uint64_t));
	int rc = tfhip_fill_u32(base, 0u, status_bytes / 4);
	if (rc) return rc;
	rc = tfhip_fill_u32(ticket, 1u, 1);
	if (rc) return rc;
	hipLaunchKernelGGL(scan_lookback_u32_kernel<LookbackCfg>, dim3((unsigned)(tiles - 1)), dim3(LookbackCfg::threads), 0, s.stream, in, out, n, status, ticket, s.async_error_dev, spin_limit);
	TFHIP_CHECK_LAUNCH();
	return TFHIP_OK;
}

int tfhip_scan_inclusive_i32(const int32_t* in, int32_t* out, size_t n) {
	return tfhip_scan_inclusive_u32((const uint32_t*)in, (uint32_t*)out, n);
}

int tfhip_scan_inclusive_u32_static(const uint32_t* in, uint32_t* out, size_t n) {
	TFHIP_REQUIRE_INIT();
	if (n == 0) return TFHIP_OK;
	if (!in || !out) return fail(TFHIP_ERR_ARG, "null pointer passed to tfhip_scan_inclusive_u32_static");
	if (n > kStaticScanMaxElements)
		return fail(TFHIP_ERR_ARG, "tfhip_scan_inclusive_u32_static takes at most %zu elements (its status words live in a fixed device array); got %zu",
		            kStaticScanMaxElements, n);
	State& s = state();
	if (s.device < 0 || s.device >= kStaticScratchDevices || !g_static_scratch_ptr[s.device])
		return fail(TFHIP_ERR_STATE, "the fixed scratch array of device %d was not located by tfhip_init", s.device);
	// The array keeps what the previous call left: the ticket and the status words of this call's tiles start at zero.
	char* base = (char*)g_static_scratch_ptr[s.device];
	const size_t tiles = (n + LookbackCfg::tile - 1) / LookbackCfg::tile;
	uint32_t* ticket = (uint32_t*)base;
	uint64_t* status = (uint64_t*)(base + sizeof(uint64_t));
	int rc = tfhip_fill_u32(base, 0u, (tiles + 1) * (sizeof(uint64_t) / sizeof(uint32_t)));  // a fill kernel, not a memset node
	if (rc) return rc;
	hipLaunchKernelGGL(scan_lookback_u32_kernel<LookbackCfg>, dim3((unsigned)tiles), dim3(LookbackCfg::threads), 0, s.stream, in, out, n, status, ticket, s.async_error_dev, kSpinLimit);
	TFHIP_CHECK_LAUNCH();
	return TFHIP_OK;
}

int tfhip_scan_inclusive_f32(const float* in, float* out, size_t n) {
	TFHIP_REQUIRE_INIT();
	if (n == 0) return TFHIP_OK;
	if (!in || !out) return fail(TFHIP_ERR_ARG, "null pointer passed to tfhip_scan_inclusive_f32");
	return scan_reduce_then_scan<float>(in, out, n);
}

}  // extern "C"
