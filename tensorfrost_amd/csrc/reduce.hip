// Row (contiguous-axis) and column (strided-axis) reductions of a dense row-major fp32 matrix.
//
// The reference computes dim_sum / dim_max / dim_min as a serial loop in one thread per output
// element (TensorFrost/Compiler/Implementations.cpp:243-303), split for constant axes >= 1024 into two
// such kernels over chunks of 128 (Compiler/Steps/Optimization.cpp:469-510). On a GPU the first stage
// of a last-axis reduction makes neighbouring threads read addresses 512 B apart. Here:
//   rows: one 64-lane wavefront owns a (row, segment); lanes read consecutive float4s (one 1 KiB
//         request per wave instruction), accumulate in registers and finish with cross-lane shuffles.
//         Long rows with few of them are cut into segments and reduced a second time; matrices of 256 MiB and
//         more take one group per compute unit, each walking through its own stretch of rows.
//   cols: a 256-thread group owns a tile of up to 1024 columns and a slab of rows; every lane keeps
//         its own four columns in registers while the group walks down the slab reading up to 4 KiB of
//         contiguous row per instruction; slabs are combined by a second pass over the [slabs, cols]
//         partials (narrow matrices put waves on different rows instead and combine through LDS). Large matrices
//         whose rows are whole 4 KiB pieces take one group per compute unit in the first pass, each walking through
//         one stretch of memory (reduce_cols_wide_kernel). Other wide matrices (8192 columns and more, a multiple
//         of 256, at least 512 rows) take one launch: sixteen waves per 256 columns and slab, the last group of each
//         256 columns adds the slabs up (reduce_cols_folded_kernel).
// HBM traffic is the matrix once plus the (tiny) partials.

#include "common.h"

#include <algorithm>

namespace tfhip {

static __device__ __forceinline__ float4 ld4(const float* p) { return *reinterpret_cast<const float4*>(p); }

// ---- rows -------------------------------------------------------------------------------------

// grid.x = ceil(rows*segs / 4); block = 256 threads = 4 waves; wave -> (row, seg).
// out[row*segs + seg] = reduce x[row, seg*seg_len .. min(cols, (seg+1)*seg_len))
template <class Op, bool VEC4>
__global__ __launch_bounds__(256) void reduce_rows_wave_kernel(const float* __restrict__ x, float* __restrict__ out,
                                                               size_t rows, size_t cols, size_t segs, size_t seg_len) {
	const int lane = threadIdx.x & 63;
	const size_t item = (size_t)blockIdx.x * 4 + (threadIdx.x >> 6);
	if (item >= rows * segs) return;
	const size_t row = item / segs;
	const size_t seg = item - row * segs;
	const size_t c0 = seg * seg_len;
	const size_t c1 = c0 + seg_len < cols ? c0 + seg_len : cols;
	const float* __restrict__ p = x + row * cols;
	Op op;
	float acc = Op::init();
	if (VEC4) {
		// cols % 4 == 0 and seg_len % 4 == 0: every row piece starts on a 16-byte boundary.
		const size_t v0 = c0 >> 2, v1 = c1 >> 2;
		size_t v = v0 + lane;
		float a0 = Op::init(), a1 = Op::init(), a2 = Op::init(), a3 = Op::init();
		for (; v + 7 * 64 < v1; v += 8 * 64) {
			float4 t[8];
#pragma unroll
			for (int u = 0; u < 8; u++) t[u] = ld4_stream(p + ((v + u * 64) << 2));
#pragma unroll
			for (int u = 0; u < 8; u++) {
				a0 = op(a0, t[u].x);
				a1 = op(a1, t[u].y);
				a2 = op(a2, t[u].z);
				a3 = op(a3, t[u].w);
			}
		}
		for (; v < v1; v += 64) {
			float4 t = ld4_stream(p + (v << 2));
			a0 = op(a0, t.x);
			a1 = op(a1, t.y);
			a2 = op(a2, t.z);
			a3 = op(a3, t.w);
		}
		acc = op(op(a0, a1), op(a2, a3));
	} else {
		size_t c = c0 + lane;
		float a0 = Op::init(), a1 = Op::init(), a2 = Op::init(), a3 = Op::init();
		for (; c + 3 * 64 < c1; c += 4 * 64) {
			float t0 = p[c], t1 = p[c + 64], t2 = p[c + 128], t3 = p[c + 192];
			a0 = op(a0, t0);
			a1 = op(a1, t1);
			a2 = op(a2, t2);
			a3 = op(a3, t3);
		}
		for (; c < c1; c += 64) a0 = op(a0, p[c]);
		acc = op(op(a0, a1), op(a2, a3));
	}
	acc = wave_reduce(acc, op);
	if (lane == 0) out[item] = acc;
}

// Short rows (cols <= 32): one thread per row; a wave's 64 rows are one contiguous span of memory, so
// every fetched line is consumed by the wave within a few iterations.
template <class Op>
__global__ __launch_bounds__(256) void reduce_rows_thread_kernel(const float* __restrict__ x, float* __restrict__ out, size_t rows, size_t cols) {
	const size_t row = (size_t)blockIdx.x * 256 + threadIdx.x;
	if (row >= rows) return;
	const float* __restrict__ p = x + row * cols;
	Op op;
	float acc = Op::init();
	for (size_t c = 0; c < cols; c++) acc = op(acc, p[c]);
	out[row] = acc;
}

// Short and medium rows (4 .. 512 columns, 16-byte aligned): LANES lanes own a row, so a wave works on 64/LANES rows at a
// time and the cross-lane finish takes log2(LANES) steps for all of them together. This is the shape of the first
// stage of a split reduction (rows of 128). A wave walks four row groups per trip for loads in flight.
template <class Op, int LANES>
__global__ __launch_bounds__(256) void reduce_rows_group_kernel(const float* __restrict__ x, float* __restrict__ out, size_t rows, size_t cols) {
	constexpr int kRowsPerStep = 64 / LANES;
	constexpr int kSteps = 4;
	const int lane = threadIdx.x & 63;
	const int sub = lane % LANES, which = lane / LANES;
	const size_t wave = (size_t)blockIdx.x * 4 + (threadIdx.x >> 6);
	const size_t row0 = wave * (kRowsPerStep * kSteps) + which;
	const size_t vecs = cols >> 2;
	Op op;
	float acc[kSteps];
#pragma unroll
	for (int u = 0; u < kSteps; u++) {
		const size_t row = row0 + (size_t)u * kRowsPerStep;
		float a0 = Op::init(), a1 = Op::init(), a2 = Op::init(), a3 = Op::init();
		if (row < rows) {
			const float* __restrict__ p = x + row * cols;
			for (size_t v = sub; v < vecs; v += LANES) {
				const float4 t = ld4_stream(p + (v << 2));
				a0 = op(a0, t.x);
				a1 = op(a1, t.y);
				a2 = op(a2, t.z);
				a3 = op(a3, t.w);
			}
		}
		acc[u] = op(op(a0, a1), op(a2, a3));
	}
#pragma unroll
	for (int u = 0; u < kSteps; u++) {
#pragma unroll
		for (int off = LANES / 2; off >= 1; off >>= 1) acc[u] = op(acc[u], __shfl_xor(acc[u], off, 64));
		const size_t row = row0 + (size_t)u * kRowsPerStep;
		if (sub == 0 && row < rows) out[row] = acc[u];
	}
}

// Large matrices (256 MiB and more) with rows of 1024 columns or a multiple of 2048: one group per compute unit
// (two for 1024 columns, where a row is only four loads per lane), each walking through its own stretch of rows, wave
// w taking rows w, w + 4, ... with eight 16-byte loads in flight per lane. Against one wave per row and 4096 groups, by
// events: [16384, 4096] 40.7 against 42.1 us, [32768, 2048] 38.6 / 41.1, [65536, 1024] 38.9 / 43.5, [100000, 1024]
// 59.2 / 65.2, [16384, 8192] 78.6 / 83.1, [4096, 16384] 44.3 / 47.6; no difference at [40000, 4096], [16384, 6144],
// [8192, 8192]; 3 % slower at half that size ([8192, 4096] 22.8 / 22.2), 20-60 % slower with rows of three pieces.
template <class Op, int U>
__global__ __launch_bounds__(256) void reduce_rows_persist_kernel(const float* __restrict__ x, float* __restrict__ out, size_t rows, size_t cols, size_t rows_per_group) {
	const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
	const size_t r0 = (size_t)blockIdx.x * rows_per_group;
	const size_t r1 = r0 + rows_per_group < rows ? r0 + rows_per_group : rows;
	Op op;
	const size_t vecs = cols >> 2;
	for (size_t row = r0 + wave; row < r1; row += 4) {
		const float* __restrict__ p = x + row * cols;
		float a0 = Op::init(), a1 = Op::init(), a2 = Op::init(), a3 = Op::init();
		size_t v = lane;
		for (; v + (U - 1) * 64 < vecs; v += U * 64) {
			float4 t[U];
#pragma unroll
			for (int u = 0; u < U; u++) t[u] = ld4_stream(p + ((v + u * 64) << 2));
#pragma unroll
			for (int u = 0; u < U; u++) {
				a0 = op(a0, t[u].x);
				a1 = op(a1, t[u].y);
				a2 = op(a2, t[u].z);
				a3 = op(a3, t[u].w);
			}
		}
		for (; v < vecs; v += 64) {
			float4 t = ld4_stream(p + (v << 2));
			a0 = op(a0, t.x);
			a1 = op(a1, t.y);
			a2 = op(a2, t.z);
			a3 = op(a3, t.w);
		}
		float acc = wave_reduce(op(op(a0, a1), op(a2, a3)), op);
		if (lane == 0) out[row] = acc;
	}
}

template <class Op>
static int reduce_rows_impl(const float* x, float* out, size_t rows, size_t cols) {
	State& s = state();
	if (cols <= 512 && cols % 4 == 0 && (((uintptr_t)x & 15) == 0) && rows >= 1024) {
		// lanes per row: the smallest power of two that leaves each lane at most four 16-byte loads
		const size_t vecs = cols / 4;
		const int lanes = vecs <= 1 ? 1 : vecs <= 2 ? 2 : vecs <= 4 ? 4 : vecs <= 32 ? 8 : vecs <= 64 ? 16 : 32;
		const size_t rows_per_wave = (size_t)(64 / lanes) * 4;
		const size_t blocks = (rows + rows_per_wave * 4 - 1) / (rows_per_wave * 4);
		if (blocks > 0x7FFFFFFFull) return fail(TFHIP_ERR_ARG, "too many rows (%zu)", rows);
		if (lanes == 1) hipLaunchKernelGGL((reduce_rows_group_kernel<Op, 1>), dim3((unsigned)blocks), dim3(256), 0, s.stream, x, out, rows, cols);
		else if (lanes == 2) hipLaunchKernelGGL((reduce_rows_group_kernel<Op, 2>), dim3((unsigned)blocks), dim3(256), 0, s.stream, x, out, rows, cols);
		else if (lanes == 4) hipLaunchKernelGGL((reduce_rows_group_kernel<Op, 4>), dim3((unsigned)blocks), dim3(256), 0, s.stream, x, out, rows, cols);
		else if (lanes == 8) hipLaunchKernelGGL((reduce_rows_group_kernel<Op, 8>), dim3((unsigned)blocks), dim3(256), 0, s.stream, x, out, rows, cols);
		else if (lanes == 16) hipLaunchKernelGGL((reduce_rows_group_kernel<Op, 16>), dim3((unsigned)blocks), dim3(256), 0, s.stream, x, out, rows, cols);
		else hipLaunchKernelGGL((reduce_rows_group_kernel<Op, 32>), dim3((unsigned)blocks), dim3(256), 0, s.stream, x, out, rows, cols);
		TFHIP_CHECK_LAUNCH();
		return TFHIP_OK;
	}
	if (cols <= 32) {
		size_t blocks = (rows + 255) / 256;
		if (blocks > 0x7FFFFFFFull) return fail(TFHIP_ERR_ARG, "too many rows (%zu)", rows);
		hipLaunchKernelGGL(reduce_rows_thread_kernel<Op>, dim3((unsigned)blocks), dim3(256), 0, s.stream, x, out, rows, cols);
		TFHIP_CHECK_LAUNCH();
		return TFHIP_OK;
	}
	if (rows * cols >= ((size_t)64 << 20) && (cols == 1024 || (cols % 2048 == 0 && cols <= 16384)) && (((uintptr_t)x & 15) == 0)) {
		const size_t groups = (size_t)s.compute_units * (cols == 1024 ? 2 : 1);
		if (rows >= groups * 16) {
			const size_t rpg = ((rows + groups - 1) / groups + 3) & ~(size_t)3;
			const unsigned grid = (unsigned)((rows + rpg - 1) / rpg);
			if (cols == 1024)
				hipLaunchKernelGGL((reduce_rows_persist_kernel<Op, 4>), dim3(grid), dim3(256), 0, s.stream, x, out, rows, cols, rpg);
			else
				hipLaunchKernelGGL((reduce_rows_persist_kernel<Op, 8>), dim3(grid), dim3(256), 0, s.stream, x, out, rows, cols, rpg);
			TFHIP_CHECK_LAUNCH();
			return TFHIP_OK;
		}
	}
	// Enough waves to cover the chip several times over. Few long rows are cut into at most 2048
	// segments of at least 2048 elements; the [rows, segs] partials then take the unsplit path.
	const size_t want_waves = (size_t)s.compute_units * 16;
	size_t segs = 1;
	if (rows < want_waves && cols >= 8192) {
		segs = (want_waves + rows - 1) / rows;
		size_t max_segs = cols / 2048;
		if (segs > max_segs) segs = max_segs;
		if (segs > 2048) segs = 2048;
	}
	size_t seg_len = (cols + segs - 1) / segs;
	seg_len = (seg_len + 255) & ~size_t(255);  // whole 1 KiB wave requests
	segs = (cols + seg_len - 1) / seg_len;
	const bool vec = (cols % 4 == 0) && (((uintptr_t)x & 15) == 0);
	float* stage_out = out;
	if (segs > 1) {
		stage_out = (float*)scratch(rows * segs * sizeof(float));
		if (!stage_out) return TFHIP_ERR_HIP;
	}
	size_t items = rows * segs;
	size_t blocks = (items + 3) / 4;
	if (blocks > 0x7FFFFFFFull) return fail(TFHIP_ERR_ARG, "too many rows (%zu)", rows);
	if (vec)
		hipLaunchKernelGGL((reduce_rows_wave_kernel<Op, true>), dim3((unsigned)blocks), dim3(256), 0, s.stream, x, stage_out, rows, cols, segs, seg_len);
	else
		hipLaunchKernelGGL((reduce_rows_wave_kernel<Op, false>), dim3((unsigned)blocks), dim3(256), 0, s.stream, x, stage_out, rows, cols, segs, seg_len);
	TFHIP_CHECK_LAUNCH();
	if (segs > 1) return reduce_rows_impl<Op>(stage_out, out, rows, segs);  // segs <= 2048: no further split
	return TFHIP_OK;
}

// ---- cols -------------------------------------------------------------------------------------

// block = 256 threads = 4 waves, arranged WC waves across columns x (4/WC) waves across rows.
// Tile = 64*V*WC columns: with WC = 4 a group reads 4 KiB of contiguous row per instruction and no
// cross-wave combine is needed. grid.x = col_tiles * slabs, slab-major so that consecutive groups read
// consecutive row pieces. out[slab*cols + c].
// STREAM: the source is the matrix itself (read once, non-temporal loads, four rows in flight per lane: 6.2 TB/s with
// nothing cached against 5.6 TB/s with plain loads and eight); partial rows of an earlier level come from cache.
template <class Op, int V, int WC, bool STREAM>
__global__ __launch_bounds__(256) void reduce_cols_kernel(const float* __restrict__ x, float* __restrict__ out,
                                                          size_t rows, size_t cols, size_t col_tiles, size_t rows_per_slab) {
	constexpr int WR = 4 / WC;
	__shared__ float lds[4][64 * V];
	const int lane = threadIdx.x & 63;
	const int wave = threadIdx.x >> 6;
	const int wc = wave % WC;   // which 64*V-column piece of the tile
	const int wr = wave / WC;   // row phase
	const size_t tile = blockIdx.x % col_tiles;
	const size_t slab = blockIdx.x / col_tiles;
	const size_t col = ((tile * WC + wc) * 64 + lane) * V;
	const size_t r0 = slab * rows_per_slab;
	const size_t r1 = r0 + rows_per_slab < rows ? r0 + rows_per_slab : rows;
	Op op;
	float acc[V];
#pragma unroll
	for (int k = 0; k < V; k++) acc[k] = Op::init();
	if (col < cols) {
		const float* __restrict__ p = x + col;
		size_t r = r0 + wr;
		if (V == 4) {
			constexpr int U = STREAM ? 4 : 8;
			for (; r + (U - 1) * WR < r1; r += U * WR) {
				float4 t[U];
#pragma unroll
				for (int u = 0; u < U; u++) t[u] = STREAM ? ld4_stream(p + (r + u * WR) * cols) : ld4(p + (r + u * WR) * cols);
#pragma unroll
				for (int u = 0; u < U; u++) {
					acc[0] = op(acc[0], t[u].x);
					acc[1 % V] = op(acc[1 % V], t[u].y);
					acc[2 % V] = op(acc[2 % V], t[u].z);
					acc[3 % V] = op(acc[3 % V], t[u].w);
				}
			}
			for (; r < r1; r += WR) {
				float4 t = STREAM ? ld4_stream(p + r * cols) : ld4(p + r * cols);
				acc[0] = op(acc[0], t.x);
				acc[1 % V] = op(acc[1 % V], t.y);
				acc[2 % V] = op(acc[2 % V], t.z);
				acc[3 % V] = op(acc[3 % V], t.w);
			}
		} else {
			for (; r + 7 * WR < r1; r += 8 * WR) {
				float t[8];
#pragma unroll
				for (int u = 0; u < 8; u++) t[u] = p[(r + u * WR) * cols];
#pragma unroll
				for (int u = 0; u < 8; u++) acc[0] = op(acc[0], t[u]);
			}
			for (; r < r1; r += WR) acc[0] = op(acc[0], p[r * cols]);
		}
	}
	if (WR == 1) {
		if (col < cols) {
#pragma unroll
			for (int k = 0; k < V; k++) out[slab * cols + col + k] = acc[k];
		}
		return;
	}
#pragma unroll
	for (int k = 0; k < V; k++) lds[wave][lane * V + k] = acc[k];
	__syncthreads();
	if (wr == 0 && col < cols) {
#pragma unroll
		for (int k = 0; k < V; k++) {
			float a = lds[wc][lane * V + k];
#pragma unroll
			for (int j = 1; j < WR; j++) a = op(a, lds[wc + j * WC][lane * V + k]);
			out[slab * cols + col + k] = a;
		}
	}
}

// A column reduction in ONE launch. A group of sixteen waves owns 256 columns (a lane four of them, 1 KiB of a row per
// wave instruction) and a slab of rows that its waves take in turn (wave w rows w, w + 16, ... of the slab, four in
// flight per lane); the waves' results meet in group memory. With several slabs per 256 columns every group leaves its
// slab's result in `partial` with device-scope write-through stores, waits for their acknowledgement and takes a
// ticket; the group that takes the last ticket adds the slabs up in a fixed order (each wave its slabs in ascending
// order, then the waves in order), writes the result and leaves the ticket counter at zero for the next launch. No
// fences: a device-scope release or acquire fence writes back or empties a whole L2, which costs tens of microseconds
// per group. Few slabs keep the partial results small (the same fold over 256 slabs of [16384, 4096], 4 MB through
// write-through stores, took 83 us).
static __device__ unsigned fold_tickets[4096];  // one per 256 columns; zero between launches

template <class Op>
__global__ __launch_bounds__(1024) void reduce_cols_folded_kernel(const float* __restrict__ x, float* __restrict__ out, float* partial, size_t rows,
                                                                 size_t cols, unsigned col_groups, unsigned slabs, size_t rows_per_slab) {
	__shared__ float4 part[16][64];
	__shared__ unsigned ticket;
	const int lane = threadIdx.x & 63;
	const int wave = threadIdx.x >> 6;
	const unsigned cg = blockIdx.x % col_groups;
	const unsigned slab = blockIdx.x / col_groups;
	const size_t col = (size_t)cg * 256 + (size_t)lane * 4;
	const size_t r0 = (size_t)slab * rows_per_slab;
	const size_t r1 = r0 + rows_per_slab < rows ? r0 + rows_per_slab : rows;
	Op op;
	float4 acc = make_float4(Op::init(), Op::init(), Op::init(), Op::init());
	auto fold = [&](const float4& t) {
		acc.x = op(acc.x, t.x);
		acc.y = op(acc.y, t.y);
		acc.z = op(acc.z, t.z);
		acc.w = op(acc.w, t.w);
	};
	{
		const float* __restrict__ p = x + col;
		size_t r = r0 + wave;
		for (; r + 48 < r1; r += 64) {
			float4 t[4];
#pragma unroll
			for (int u = 0; u < 4; u++) t[u] = ld4_stream(p + (r + u * 16) * cols);
#pragma unroll
			for (int u = 0; u < 4; u++) fold(t[u]);
		}
		for (; r < r1; r += 16) fold(ld4_stream(p + r * cols));
	}
	part[wave][lane] = acc;
	__syncthreads();
	if (wave == 0) {
		acc = part[0][lane];
#pragma unroll
		for (int w = 1; w < 16; w++) fold(part[w][lane]);
	}
	if (slabs == 1) {
		if (wave == 0) *reinterpret_cast<float4*>(out + col) = acc;
		return;
	}
	if (wave == 0) {
		float* mine = partial + (size_t)slab * cols + col;
		__hip_atomic_store(mine + 0, acc.x, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
		__hip_atomic_store(mine + 1, acc.y, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
		__hip_atomic_store(mine + 2, acc.z, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
		__hip_atomic_store(mine + 3, acc.w, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
		__builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): the stores have been acknowledged
		if (lane == 0) ticket = atomicAdd(&fold_tickets[cg], 1u);
	}
	__syncthreads();
	if (ticket != slabs - 1) return;
	// the last group of these 256 columns
	acc = make_float4(Op::init(), Op::init(), Op::init(), Op::init());
	for (unsigned s = wave; s < slabs; s += 16) {
		const float* theirs = partial + (size_t)s * cols + col;
		float4 t;
		t.x = __hip_atomic_load(theirs + 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
		t.y = __hip_atomic_load(theirs + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
		t.z = __hip_atomic_load(theirs + 2, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
		t.w = __hip_atomic_load(theirs + 3, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
		fold(t);
	}
	part[wave][lane] = acc;
	__syncthreads();
	if (wave == 0) {
		acc = part[0][lane];
#pragma unroll
		for (int w = 1; w < 16; w++) fold(part[w][lane]);
		*reinterpret_cast<float4*>(out + col) = acc;
		if (lane == 0) fold_tickets[cg] = 0;
	}
}

// The last level of a column reduction: a few hundred partial rows (just written, so they come from cache) of many
// columns. A group owns 16 columns: a lane reads four of them (16 bytes) of one row, a wave instruction 16 rows, the
// four waves 64 rows per trip, so [256, 4096] partial rows are finished by 256 groups in four loads per lane
// (the general kernel's one wave per 256 columns gives 16 groups there, each walking 64 rows: 5 us against 2).
template <class Op>
__global__ __launch_bounds__(256) void reduce_cols_last_level_kernel(const float* __restrict__ partial, float* __restrict__ out, size_t rows, size_t cols) {
	__shared__ float4 lds[4][4];
	const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
	const int quad = lane & 3, phase = lane >> 2;  // which four columns, which of 16 rows
	const size_t col = (size_t)blockIdx.x * 16 + quad * 4;
	Op op;
	float4 acc = make_float4(Op::init(), Op::init(), Op::init(), Op::init());
	if (col < cols) {
		for (size_t r = (size_t)wave * 16 + phase; r < rows; r += 64) {
			const float4 t = ld4(partial + r * cols + col);
			acc.x = op(acc.x, t.x);
			acc.y = op(acc.y, t.y);
			acc.z = op(acc.z, t.z);
			acc.w = op(acc.w, t.w);
		}
	}
#pragma unroll
	for (int off = 4; off < 64; off <<= 1) {
		acc.x = op(acc.x, __shfl_xor(acc.x, off, 64));
		acc.y = op(acc.y, __shfl_xor(acc.y, off, 64));
		acc.z = op(acc.z, __shfl_xor(acc.z, off, 64));
		acc.w = op(acc.w, __shfl_xor(acc.w, off, 64));
	}
	if (lane < 4) lds[wave][lane] = acc;
	__syncthreads();
	if (wave == 0 && lane < 4 && col < cols) {
		float4 a = lds[0][lane];
#pragma unroll
		for (int w = 1; w < 4; w++) {
			const float4 b = lds[w][lane];
			a.x = op(a.x, b.x);
			a.y = op(a.y, b.y);
			a.z = op(a.z, b.z);
			a.w = op(a.w, b.w);
		}
		*reinterpret_cast<float4*>(out + col) = a;
	}
}

// Level 0 for large matrices whose rows are whole 4 KiB pieces: as many groups as compute units, no more. A group of
// 256 threads owns T pieces of 1024 columns side by side (T = 4: 16 KiB of a row) and one slab of at least 64 rows, and
// reads U rows at a time (T * U = 8 loads of 16 bytes in flight per lane), so each compute unit walks front to back
// through one stretch of memory: [16384, 4096] level 0 in 39.7 us (6.8 TB/s, kernel trace) against 43.9 us with four groups per unit
// and slabs of 1024 columns; both levels by events 43.1 against 47.3 us, [16384, 8192] 81 against 90 (one launch
// with the fold), [2048, 32768] 45 / 49, [65536, 1024] 43 / 47. One group more than there are units costs a second
// wave of groups (256 -> 320 groups: 43 -> 56 us); slabs shorter than 64 rows lose ([4096, 4096]: 16.3 against 14.8 us).
template <class Op, int T, int U>
__global__ __launch_bounds__(256) void reduce_cols_wide_kernel(const float* __restrict__ x, float* __restrict__ out, size_t rows, size_t cols, size_t col_tiles,
                                                              size_t rows_per_slab) {
	const size_t tile = blockIdx.x % col_tiles;
	const size_t slab = blockIdx.x / col_tiles;
	const size_t col = tile * (1024 * T) + (size_t)threadIdx.x * 4;
	const size_t r0 = slab * rows_per_slab;
	const size_t r1 = r0 + rows_per_slab < rows ? r0 + rows_per_slab : rows;
	Op op;
	float4 acc[T];
#pragma unroll
	for (int t = 0; t < T; t++) acc[t] = make_float4(Op::init(), Op::init(), Op::init(), Op::init());
	const float* __restrict__ p = x + col;
	size_t r = r0;
	for (; r + U <= r1; r += U) {
		float4 v[U][T];
#pragma unroll
		for (int u = 0; u < U; u++)
#pragma unroll
			for (int t = 0; t < T; t++) v[u][t] = ld4_stream(p + (r + u) * cols + t * 1024);
#pragma unroll
		for (int u = 0; u < U; u++)
#pragma unroll
			for (int t = 0; t < T; t++) {
				acc[t].x = op(acc[t].x, v[u][t].x);
				acc[t].y = op(acc[t].y, v[u][t].y);
				acc[t].z = op(acc[t].z, v[u][t].z);
				acc[t].w = op(acc[t].w, v[u][t].w);
			}
	}
	for (; r < r1; r++) {
#pragma unroll
		for (int t = 0; t < T; t++) {
			const float4 v = ld4_stream(p + r * cols + t * 1024);
			acc[t].x = op(acc[t].x, v.x);
			acc[t].y = op(acc[t].y, v.y);
			acc[t].z = op(acc[t].z, v.z);
			acc[t].w = op(acc[t].w, v.w);
		}
	}
#pragma unroll
	for (int t = 0; t < T; t++) *reinterpret_cast<float4*>(out + slab * cols + col + t * 1024) = acc[t];
}

// How a [rows, cols] column reduction is cut: `slabs` groups of `rows_per_slab` rows per column tile.
static void plan_cols(size_t rows, size_t col_tiles, size_t& slabs, size_t& rows_per_slab) {
	// Aim for >= 4 groups per compute unit (more, shorter slabs stream no faster and leave more partial rows to the
	// next level: 16384 x 4096 runs 43 us with 256 or 512 slabs, 46 us with 1024); a slab is at least 32 rows.
	const size_t want_groups = (size_t)state().compute_units * 4;
	slabs = (want_groups + col_tiles - 1) / col_tiles;
	size_t max_slabs = (rows + 31) / 32;
	if (slabs > max_slabs) slabs = max_slabs;
	if (slabs < 1) slabs = 1;
	rows_per_slab = (rows + slabs - 1) / slabs;
	rows_per_slab = (rows_per_slab + 3) & ~size_t(3);
	slabs = (rows + rows_per_slab - 1) / rows_per_slab;
}

template <class Op, int V, int WC>
static void launch_cols(const float* src, float* dst, size_t rows, size_t cols, size_t col_tiles, size_t slabs, size_t rps, bool stream) {
	if (stream)
		hipLaunchKernelGGL((reduce_cols_kernel<Op, V, WC, true>), dim3((unsigned)(col_tiles * slabs)), dim3(256), 0, state().stream, src, dst, rows, cols, col_tiles, rps);
	else
		hipLaunchKernelGGL((reduce_cols_kernel<Op, V, WC, false>), dim3((unsigned)(col_tiles * slabs)), dim3(256), 0, state().stream, src, dst, rows, cols, col_tiles, rps);
}

// Narrow matrices (up to 256 columns, many rows). The matrix is one long contiguous array; a group walks a span
// of whole rows with a stride that is a multiple of the row length, so a thread meets the same column (VEC: the same
// four columns) on every trip and keeps its accumulators in registers. Threads of equal column meet in group memory.
// One group per compute unit, eight non-temporal 16-byte loads in flight per lane: [2097152, 32] 43 us (6.2 TB/s)
// against 59 us with eight groups per unit, four plain loads in flight; [1048576, 64] 43 against 55 and [262144, 256]
// 43 against 46 for the tiled kernel that served them before.
template <class Op, bool VEC>
__global__ __launch_bounds__(256) void reduce_cols_narrow_kernel(const float* __restrict__ x, float* __restrict__ partial,
                                                                 size_t rows, size_t cols, size_t rows_per_group) {
	__shared__ float lds[256 * (VEC ? 4 : 1)];
	const size_t r0 = (size_t)blockIdx.x * rows_per_group;
	const size_t r1 = r0 + rows_per_group < rows ? r0 + rows_per_group : rows;
	const size_t unit = VEC ? cols >> 2 : cols;  // loads per row
	const size_t stride = (256 / unit) * unit;   // active threads
	Op op;
	float a0 = Op::init(), a1 = Op::init(), a2 = Op::init(), a3 = Op::init();
	if (threadIdx.x < stride) {
		size_t i = r0 * unit + threadIdx.x;
		const size_t end = r1 * unit;
		if (VEC) {
			for (; i + 7 * stride < end; i += 8 * stride) {
				float4 t[8];
#pragma unroll
				for (int u = 0; u < 8; u++) t[u] = ld4_stream(x + ((i + u * stride) << 2));
#pragma unroll
				for (int u = 0; u < 8; u++) {
					a0 = op(a0, t[u].x);
					a1 = op(a1, t[u].y);
					a2 = op(a2, t[u].z);
					a3 = op(a3, t[u].w);
				}
			}
			for (; i < end; i += stride) {
				const float4 t = ld4_stream(x + (i << 2));
				a0 = op(a0, t.x);
				a1 = op(a1, t.y);
				a2 = op(a2, t.z);
				a3 = op(a3, t.w);
			}
		} else {
			for (; i + 7 * stride < end; i += 8 * stride) {
				float t[8];
#pragma unroll
				for (int u = 0; u < 8; u++) t[u] = x[i + u * stride];
#pragma unroll
				for (int u = 0; u < 8; u += 4) {
					a0 = op(a0, t[u]);
					a1 = op(a1, t[u + 1]);
					a2 = op(a2, t[u + 2]);
					a3 = op(a3, t[u + 3]);
				}
			}
			for (; i < end; i += stride) a0 = op(a0, x[i]);
			a0 = op(op(a0, a1), op(a2, a3));
		}
	}
	if (VEC) {
		lds[threadIdx.x * 4] = a0;
		lds[threadIdx.x * 4 + 1] = a1;
		lds[threadIdx.x * 4 + 2] = a2;
		lds[threadIdx.x * 4 + 3] = a3;
	} else {
		lds[threadIdx.x] = a0;
	}
	__syncthreads();
	if (threadIdx.x < cols) {
		float acc = Op::init();
		if (VEC) {
			for (size_t t = threadIdx.x >> 2; t < stride; t += unit) acc = op(acc, lds[t * 4 + (threadIdx.x & 3)]);
		} else {
			for (size_t t = threadIdx.x; t < stride; t += unit) acc = op(acc, lds[t]);
		}
		partial[(size_t)blockIdx.x * cols + threadIdx.x] = acc;
	}
}

// One wave per column over a few thousand partial rows.
template <class Op>
__global__ __launch_bounds__(256) void reduce_cols_finish_kernel(const float* __restrict__ partial, float* __restrict__ out, size_t rows, size_t cols) {
	const int lane = threadIdx.x & 63;
	const size_t col = (size_t)blockIdx.x * 4 + (threadIdx.x >> 6);
	if (col >= cols) return;
	Op op;
	float acc = Op::init();
	for (size_t r = lane; r < rows; r += 64) acc = op(acc, partial[r * cols + col]);
	acc = wave_reduce(acc, op);
	if (lane == 0) out[col] = acc;
}

template <class Op>
static int reduce_cols_narrow(const float* x, float* out, size_t rows, size_t cols) {
	State& s = state();
	const bool vec = (cols % 4 == 0) && (((uintptr_t)x & 15) == 0);
	size_t groups = (size_t)s.compute_units;  // one group per compute unit, each walking through its own stretch of rows
	size_t rows_per_group = (rows + groups - 1) / groups;
	if (rows_per_group < 64) rows_per_group = 64;
	groups = (rows + rows_per_group - 1) / rows_per_group;
	float* partial = (float*)scratch(groups * cols * sizeof(float));
	if (!partial) return TFHIP_ERR_HIP;
	if (vec)
		hipLaunchKernelGGL((reduce_cols_narrow_kernel<Op, true>), dim3((unsigned)groups), dim3(256), 0, s.stream, x, partial, rows, cols, rows_per_group);
	else
		hipLaunchKernelGGL((reduce_cols_narrow_kernel<Op, false>), dim3((unsigned)groups), dim3(256), 0, s.stream, x, partial, rows, cols, rows_per_group);
	TFHIP_CHECK_LAUNCH();
	hipLaunchKernelGGL(reduce_cols_finish_kernel<Op>, dim3((unsigned)((cols + 3) / 4)), dim3(256), 0, s.stream, (const float*)partial, out, groups, cols);
	TFHIP_CHECK_LAUNCH();
	return TFHIP_OK;
}

template <class Op>
static int reduce_cols_impl(const float* x, float* out, size_t rows, size_t cols) {
	// up to 256 columns when a row is whole 16-byte loads (then at most 64 loads per row), fewer than 64 otherwise
	if (rows >= 16384 && (cols < 64 || (cols <= 256 && cols % 4 == 0 && (((uintptr_t)x & 15) == 0)))) return reduce_cols_narrow<Op>(x, out, rows, cols);
	const bool vec = (cols % 4 == 0) && (((uintptr_t)x & 15) == 0) && (((uintptr_t)out & 15) == 0);
	// One group per compute unit over whole stretches of rows (reduce_cols_wide_kernel) where a row is one, two or four
	// 4 KiB pieces, or 16 KiB pieces for up to 65536 columns, and the slabs come out at 64 rows or more.
	int wide_t = 0;
	size_t wide_slabs = 0;
	if (vec && (cols == 1024 || cols == 2048 || (cols % 4096 == 0 && cols <= 65536))) {
		wide_t = cols % 4096 == 0 ? 4 : (int)(cols / 1024);
		wide_slabs = (size_t)state().compute_units / (cols / (1024 * (size_t)wide_t));
		if (wide_slabs < 2 || rows / wide_slabs < 64) wide_t = 0;
	}
	if (!wide_t && vec && cols % 256 == 0 && cols >= 8192 && cols / 256 <= 4096 && rows >= 512) {
		// Wide matrices in one launch: enough slabs for three groups of sixteen waves per two compute units, at least 64
		// rows each (where the form above applies it is faster still: [8192, 8192] 44 us, [16384, 8192] 81, [4096, 16384]
		// 44, [2048, 32768] 45; beyond 65536 columns this one wins, [512, 131072] 44 against 49). Against the levelled
		// form below, by events, same process: [4096, 16384] 46 us against 60,
		// [2048, 32768] 50 / 60, [1024, 65536] 47 / 57, [8192, 8192] 47 / 52, [16384, 8192] 90 / 96; with 4096 columns
		// and fewer it needs 24 and more slabs per 256 columns and loses: [16384, 4096] 48 / 47, [65536, 1024] 51 / 47,
		// [262144, 256] 58 / 46. ([16384, 4096] over the number of slabs: 85 us with 4, 51 with 8, 48-49 with 16 to 48,
		// 54-59 with 64 and 128.)
		const size_t col_groups = cols / 256;
		size_t slabs = (3 * (size_t)state().compute_units / 2 + col_groups - 1) / col_groups;
		slabs = std::min(std::min(slabs, rows / 64), (size_t)256);
		slabs = std::max<size_t>(slabs, 1);
		const size_t rps = (rows + slabs - 1) / slabs;
		slabs = (rows + rps - 1) / rps;
		float* partial = nullptr;
		if (slabs > 1) {
			partial = (float*)scratch(slabs * cols * sizeof(float));
			if (!partial) return TFHIP_ERR_HIP;
		}
		hipLaunchKernelGGL(reduce_cols_folded_kernel<Op>, dim3((unsigned)(col_groups * slabs)), dim3(1024), 0, state().stream, x, out, partial, rows, cols, (unsigned)col_groups,
		                   (unsigned)slabs, rps);
		TFHIP_CHECK_LAUNCH();
		return TFHIP_OK;
	}
	const size_t piece = vec ? 256 : 64;  // columns one wave covers
	const int wc = cols >= 4 * piece ? 4 : (cols >= 2 * piece ? 2 : 1);
	const size_t tile_cols = piece * wc;
	const size_t col_tiles = (cols + tile_cols - 1) / tile_cols;
	if (col_tiles > 0x7FFFFFull) return fail(TFHIP_ERR_ARG, "too many columns (%zu)", cols);

	// Plan the levels. Level 0 streams the input with wide tiles; its partial rows (at most a few thousand) are
	// finished with one wave per `piece` of columns, in one pass when that already gives enough groups or few
	// rows are left, otherwise through one intermediate level of at most 256 partial rows.
	struct Level {
		size_t rows, tiles, slabs, rps;
		int wc;
	};
	Level levels[8];
	int n_levels = 0;
	size_t cur_rows = rows;
	for (;;) {
		Level L;
		L.rows = cur_rows;
		L.wc = wc;
		L.tiles = col_tiles;
		plan_cols(cur_rows, col_tiles, L.slabs, L.rps);
		if (n_levels == 0 && wide_t) {
			L.slabs = wide_slabs;
			L.rps = (rows + L.slabs - 1) / L.slabs;
			L.slabs = (rows + L.rps - 1) / L.rps;
		}
		if (n_levels > 0 && cur_rows <= 4096) {
			L.wc = 1;
			L.tiles = (cols + piece - 1) / piece;
			L.slabs = 1;
			if (cur_rows > 256 && L.tiles < 64) {
				L.slabs = (256 + L.tiles - 1) / L.tiles;
				if (L.slabs > cur_rows / 32) L.slabs = cur_rows / 32;
				if (L.slabs < 1) L.slabs = 1;
			}
			L.rps = ((cur_rows + L.slabs - 1) / L.slabs + 3) & ~size_t(3);
			L.slabs = (cur_rows + L.rps - 1) / L.rps;
		}
		if (n_levels == 8) return fail(TFHIP_ERR_STATE, "column reduction does not converge");
		levels[n_levels++] = L;
		if (L.slabs == 1) break;
		cur_rows = L.slabs;
	}
	// Partial rows alternate between two scratch regions: even levels write region A, odd levels region B.
	size_t a_rows = 0, b_rows = 0;
	for (int l = 0; l + 1 < n_levels; l++) {
		size_t& r = (l & 1) ? b_rows : a_rows;
		if (levels[l].slabs > r) r = levels[l].slabs;
	}
	const size_t a_bytes = (a_rows * cols * sizeof(float) + 255) & ~size_t(255);
	const size_t b_bytes = (b_rows * cols * sizeof(float) + 255) & ~size_t(255);
	char* base = nullptr;
	if (a_bytes + b_bytes) {
		base = (char*)scratch(a_bytes + b_bytes);
		if (!base) return TFHIP_ERR_HIP;
	}

	const float* src = x;
	for (int l = 0; l < n_levels; l++) {
		const Level& L = levels[l];
		float* dst = L.slabs > 1 ? (float*)(base + ((l & 1) ? a_bytes : 0)) : out;
		if (vec && l > 0 && L.slabs == 1 && L.rows <= 1024 && cols >= 1024) {
			hipLaunchKernelGGL(reduce_cols_last_level_kernel<Op>, dim3((unsigned)((cols + 15) / 16)), dim3(256), 0, state().stream, src, dst, L.rows, cols);
			TFHIP_CHECK_LAUNCH();
			src = dst;
			continue;
		}
		if (l == 0 && wide_t) {
			const size_t tiles = cols / (1024 * wide_t);
			const unsigned grid = (unsigned)(tiles * L.slabs);
			if (wide_t == 4)
				hipLaunchKernelGGL((reduce_cols_wide_kernel<Op, 4, 2>), dim3(grid), dim3(256), 0, state().stream, src, dst, L.rows, cols, tiles, L.rps);
			else if (wide_t == 2)
				hipLaunchKernelGGL((reduce_cols_wide_kernel<Op, 2, 4>), dim3(grid), dim3(256), 0, state().stream, src, dst, L.rows, cols, tiles, L.rps);
			else
				hipLaunchKernelGGL((reduce_cols_wide_kernel<Op, 1, 8>), dim3(grid), dim3(256), 0, state().stream, src, dst, L.rows, cols, tiles, L.rps);
			TFHIP_CHECK_LAUNCH();
			src = dst;
			continue;
		}
		if (vec) {
			if (L.wc == 4) launch_cols<Op, 4, 4>(src, dst, L.rows, cols, L.tiles, L.slabs, L.rps, l == 0);
			else if (L.wc == 2) launch_cols<Op, 4, 2>(src, dst, L.rows, cols, L.tiles, L.slabs, L.rps, l == 0);
			else launch_cols<Op, 4, 1>(src, dst, L.rows, cols, L.tiles, L.slabs, L.rps, l == 0);
		} else {
			if (L.wc == 4) launch_cols<Op, 1, 4>(src, dst, L.rows, cols, L.tiles, L.slabs, L.rps, l == 0);
			else if (L.wc == 2) launch_cols<Op, 1, 2>(src, dst, L.rows, cols, L.tiles, L.slabs, L.rps, l == 0);
			else launch_cols<Op, 1, 1>(src, dst, L.rows, cols, L.tiles, L.slabs, L.rps, l == 0);
		}
		TFHIP_CHECK_LAUNCH();
		src = dst;
	}
	return TFHIP_OK;
}

// out[s, c] = op over rows [s * rows_per_slab, (s + 1) * rows_per_slab) of column c: the first stage of a split
// axis-0 reduction as one launch (the same kernel the full reduction uses for its first level).
template <class Op>
static int reduce_cols_slabs_impl(const float* x, float* out, size_t rows, size_t cols, size_t rows_per_slab) {
	const bool vec = (cols % 4 == 0) && (((uintptr_t)x & 15) == 0) && (((uintptr_t)out & 15) == 0);
	const size_t piece = vec ? 256 : 64;
	const size_t slabs = (rows + rows_per_slab - 1) / rows_per_slab;
	// the slab height is given, so the width of a group's tile is what sets the number of groups: as wide as
	// still leaves eight groups per compute unit
	int wc = cols >= 4 * piece ? 4 : (cols >= 2 * piece ? 2 : 1);
	while (wc > 1 && ((cols + piece * wc - 1) / (piece * wc)) * slabs < (size_t)state().compute_units * 8) wc /= 2;
	const size_t col_tiles = (cols + piece * wc - 1) / (piece * wc);
	if (col_tiles * slabs > 0x7FFFFFFFull) return fail(TFHIP_ERR_ARG, "too many slabs x column tiles (%zu x %zu)", slabs, col_tiles);
	if (vec) {
		if (wc == 4) launch_cols<Op, 4, 4>(x, out, rows, cols, col_tiles, slabs, rows_per_slab, true);
		else if (wc == 2) launch_cols<Op, 4, 2>(x, out, rows, cols, col_tiles, slabs, rows_per_slab, true);
		else launch_cols<Op, 4, 1>(x, out, rows, cols, col_tiles, slabs, rows_per_slab, true);
	} else {
		if (wc == 4) launch_cols<Op, 1, 4>(x, out, rows, cols, col_tiles, slabs, rows_per_slab, true);
		else if (wc == 2) launch_cols<Op, 1, 2>(x, out, rows, cols, col_tiles, slabs, rows_per_slab, true);
		else launch_cols<Op, 1, 1>(x, out, rows, cols, col_tiles, slabs, rows_per_slab, true);
	}
	TFHIP_CHECK_LAUNCH();
	return TFHIP_OK;
}

static int check_args(const float* x, float* out, size_t rows, size_t cols) {
	if (!x || !out) return fail(TFHIP_ERR_ARG, "null pointer passed to a reduction");
	if (rows == 0 || cols == 0) return fail(TFHIP_ERR_ARG, "reduction over an empty matrix (%zu x %zu)", rows, cols);
	return TFHIP_OK;
}

}  // namespace tfhip

using namespace tfhip;

extern "C" {

int tfhip_reduce_rows_f32(int op, const float* x, float* out, size_t rows, size_t cols) {
	TFHIP_REQUIRE_INIT();
	int rc = check_args(x, out, rows, cols);
	if (rc) return rc;
	switch (op) {
		case TFHIP_REDUCE_SUM: return reduce_rows_impl<OpSum>(x, out, rows, cols);
		case TFHIP_REDUCE_MAX: return reduce_rows_impl<OpMax>(x, out, rows, cols);
		case TFHIP_REDUCE_MIN: return reduce_rows_impl<OpMin>(x, out, rows, cols);
	}
	return fail(TFHIP_ERR_ARG, "unknown reduction op %d", op);
}

int tfhip_reduce_cols_slabs_f32(int op, const float* x, float* out, size_t rows, size_t cols, size_t rows_per_slab) {
	TFHIP_REQUIRE_INIT();
	int rc = check_args(x, out, rows, cols);
	if (rc) return rc;
	if (rows_per_slab == 0) return fail(TFHIP_ERR_ARG, "rows_per_slab must be positive");
	switch (op) {
		case TFHIP_REDUCE_SUM: return reduce_cols_slabs_impl<OpSum>(x, out, rows, cols, rows_per_slab);
		case TFHIP_REDUCE_MAX: return reduce_cols_slabs_impl<OpMax>(x, out, rows, cols, rows_per_slab);
		case TFHIP_REDUCE_MIN: return reduce_cols_slabs_impl<OpMin>(x, out, rows, cols, rows_per_slab);
	}
	return fail(TFHIP_ERR_ARG, "unknown reduction op %d", op);
}

int tfhip_reduce_cols_f32(int op, const float* x, float* out, size_t rows, size_t cols) {
	TFHIP_REQUIRE_INIT();
	int rc = check_args(x, out, rows, cols);
	if (rc) return rc;
	switch (op) {
		case TFHIP_REDUCE_SUM: return reduce_cols_impl<OpSum>(x, out, rows, cols);
		case TFHIP_REDUCE_MAX: return reduce_cols_impl<OpMax>(x, out, rows, cols);
		case TFHIP_REDUCE_MIN: return reduce_cols_impl<OpMin>(x, out, rows, cols);
	}
	return fail(TFHIP_ERR_ARG, "unknown reduction op %d", op);
}

int tfhip_reduce_sum_f32_rows(const float* x, float* out, size_t rows, size_t cols) { return tfhip_reduce_rows_f32(TFHIP_REDUCE_SUM, x, out, rows, cols); }
int tfhip_reduce_max_f32_rows(const float* x, float* out, size_t rows, size_t cols) { return tfhip_reduce_rows_f32(TFHIP_REDUCE_MAX, x, out, rows, cols); }
int tfhip_reduce_min_f32_rows(const float* x, float* out, size_t rows, size_t cols) { return tfhip_reduce_rows_f32(TFHIP_REDUCE_MIN, x, out, rows, cols); }
int tfhip_reduce_sum_f32_cols(const float* x, float* out, size_t rows, size_t cols) { return tfhip_reduce_cols_f32(TFHIP_REDUCE_SUM, x, out, rows, cols); }
int tfhip_reduce_max_f32_cols(const float* x, float* out, size_t rows, size_t cols) { return tfhip_reduce_cols_f32(TFHIP_REDUCE_MAX, x, out, rows, cols); }
int tfhip_reduce_min_f32_cols(const float* x, float* out, size_t rows, size_t cols) { return tfhip_reduce_cols_f32(TFHIP_REDUCE_MIN, x, out, rows, cols); }

}  // extern "C"
