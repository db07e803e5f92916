// fp32 matrix multiplication on the matrix cores: C[M,N] = op(A) * op(B), all operands dense row-major.
//
// The reference lowers tf.matmul to one thread per element of C running a serial loop over K
// (TensorFrost/Compiler/Implementations.cpp:560-646: C = 0; for k: C += A[..,i,k] * B[..,k,j]); a
// transposed operand is an index remap fused into that loop (:451-488) and the backward pass is two more
// such matmuls (:133-135: dA = dC * B^T, dB = A^T * dC). The three operand layouts below are those three.
//
//   nn: A[M,K]   B[K,N]        nt: A[M,K]   B[N,K] (B^T is used)        tn: A[K,M] (A^T is used)   B[K,N]
//
// Kernel: a 256-thread group (4 waves as 2x2) owns a 128x128 tile of C; each wave a 64x64 sub-tile held in
// four 32x32 accumulators of v_mfma_f32_32x32x2_f32. K is walked 16 at a time: the next A and B panels are
// fetched from global memory into registers while the current ones, staged in LDS as As[k][m] and Bs[k][n],
// feed the MFMAs (8 k-pairs x 4 MFMAs per panel and wave). LDS rows are padded to 132 words so that the two
// k-halves of a wave read different banks. Operands whose contiguous axis is k (A of nn/nt, B of nt) are
// transposed on their way into LDS. fp32 MFMA accumulates in fp32; products are not split or rounded to a
// narrower type. A reduction over a very long K with a small C (dW of a dense layer) is cut into K-slices
// whose partial products are summed by the column-reduction kernel.
//
// Products with N <= 8 (the 256 -> 3 output layer and its weight gradient) are bandwidth-bound on streaming A
// once: nn/nt transpose 64-row chunks of A through group memory so that lanes own rows, tn accumulates outer products down slabs of k. Other shapes too small
// for a 128x128 tile to pay (M or N below 32) take a plain kernel with one thread per element of C.

#include "common.h"
#include <type_traits>

extern "C" int tfhip_reduce_cols_f32(int op, const float* x, float* out, size_t rows, size_t cols);

namespace tfhip {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef unsigned uintx4 __attribute__((ext_vector_type(4)));

constexpr int kBM = 128, kBN = 128, kBK = 16;
constexpr int kLdsStride = kBM + 4;  // 132 words: 16-byte aligned rows, k and k+1 rows 4 banks apart

enum Layout { kNN = 0, kNT = 1, kTN = 2 };

struct GemmArgs {
	const float* A;
	const float* B;
	float* C;
	int M, N, K;
	int lda, ldb, ldc;  // leading dimensions (elements) of the arrays as stored
	int k_slices;       // grid.z; slice z covers K range [z*k_per_slice, ...)
	int k_per_slice;    // multiple of kBK
	size_t c_slice_stride;  // elements between partial C matrices
	int epilogue;           // TFHIP_EPILOGUE_*: what happens to an element of the product on its way to C
	const float* aux;       // bias[N] or mask[M,N] of the epilogue
	// A batch of products in one launch (grid.y): elements between consecutive matrices; 0 = the operand is shared.
	size_t batch_a = 0, batch_b = 0, batch_c = 0;
	// tn only: also the column sums of B (the bias gradient beside a weight gradient, both read dY): slice z of K leaves
	// its sums in colsum[z * colsum_stride .. z * colsum_stride + N).
	float* colsum = nullptr;
	size_t colsum_stride = 0;
};

// ---- the sum over K slices ------------------------------------------------------------------------
// Kernels that cut a long K write one partial result per slice: `width` floats every `stride` floats. One launch adds
// them up in a fixed order (a wave takes every WAVES-th slice, then the waves' sums are added in wave order): columns
// below `split` go to out, the others to out2 (the column sums of B, which a slice leaves right behind its product:
// n2 of them, padded to whole vectors in the slices). With few columns and many slices the groups of grid.y first
// sum `per_block` slices each into rows of an intermediate array (out_stride floats apart), which a second launch sums.
template <int WAVES>
__global__ __launch_bounds__(WAVES * 64) void sgemm_sum_slices_kernel(const float* __restrict__ partial, int slices, int per_block, size_t stride, size_t width,
                                                                      float* __restrict__ out, size_t out_stride, size_t split, float* __restrict__ out2, size_t n2) {
	__shared__ float4 red[WAVES][64];
	const int lane = threadIdx.x & 63;
	const int wave = threadIdx.x >> 6;
	const size_t c = ((size_t)blockIdx.x * 64 + lane) * 4;
	const int z_begin = (int)blockIdx.y * per_block;
	const int z_end = z_begin + per_block < slices ? z_begin + per_block : slices;
	out += (size_t)blockIdx.y * out_stride;
	float4 acc = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
	if (c < width) {
		const float* p = partial + c;
		int z = z_begin + wave;
		for (; z + 7 * WAVES < z_end; z += 8 * WAVES) {
			float4 t[8];
#pragma unroll
			for (int u = 0; u < 8; u++) t[u] = *reinterpret_cast<const float4*>(p + (size_t)(z + u * WAVES) * stride);
#pragma unroll
			for (int u = 0; u < 8; u++) {
				acc.x += t[u].x;
				acc.y += t[u].y;
				acc.z += t[u].z;
				acc.w += t[u].w;
			}
		}
		for (; z < z_end; z += WAVES) {
			const float4 t = *reinterpret_cast<const float4*>(p + (size_t)z * stride);
			acc.x += t.x;
			acc.y += t.y;
			acc.z += t.z;
			acc.w += t.w;
		}
	}
	red[wave][lane] = acc;
	__syncthreads();
	if (wave == 0 && c < width) {
#pragma unroll
		for (int w = 1; w < WAVES; w++) {
			const float4 t = red[w][lane];
			acc.x += t.x;
			acc.y += t.y;
			acc.z += t.z;
			acc.w += t.w;
		}
		if (c < split) {
			*reinterpret_cast<float4*>(out + c) = acc;
		} else {
			const size_t c2 = c - split;
			if (c2 + 4 <= n2 && (reinterpret_cast<uintptr_t>(out2) & 15) == 0) {
				*reinterpret_cast<float4*>(out2 + c2) = acc;
			} else {
				const float v[4] = {acc.x, acc.y, acc.z, acc.w};
#pragma unroll
				for (int i = 0; i < 4; i++)
					if (c2 + i < n2) out2[c2 + i] = v[i];
			}
		}
	}
}

// Where the slices of a product [mn floats] and, with `n` > 0, of the column sums [n floats] go in scratch memory.
// merged: a slice's column sums follow its product and one launch of the kernel above finishes both; otherwise (odd
// sizes or addresses) the two sit apart, each dense, and the general column reduction sums them.
struct SlicePlan {
	float* partial = nullptr;
	float* colsum_partial = nullptr;
	size_t stride = 0, colsum_stride = 0;
	bool merged = false;
	// merged, few columns: `blocks` groups of `per_block` slices are summed first, into `level` ([blocks, stride])
	size_t blocks = 1, per_block = 0;
	float* level = nullptr;
};

static int plan_slices(size_t slices, size_t mn, size_t n, const float* C, const float* colsum, SlicePlan& plan) {
	const size_t n_padded = (n + 3) & ~size_t(3);
	plan.merged = (mn & 3) == 0 && (reinterpret_cast<uintptr_t>(C) & 15) == 0 && slices <= 0x7FFFFFFFull && (mn + n_padded + 255) / 256 <= 0x7FFFFFFFull;
	if (plan.merged) {
		plan.stride = plan.colsum_stride = mn + n_padded;
		const size_t groups = (plan.stride + 255) / 256, units = (size_t)state().compute_units;
		if (groups * 4 < units && slices >= 128) {  // too few columns to read the slices with the whole chip: two levels
			plan.blocks = (units + groups - 1) / groups;
			plan.per_block = (slices + plan.blocks - 1) / plan.blocks;
			if (plan.per_block < 16) plan.per_block = 16;
			plan.blocks = (slices + plan.per_block - 1) / plan.per_block;
		}
		const size_t slice_bytes = (slices * plan.stride * sizeof(float) + 255) & ~size_t(255);
		plan.partial = (float*)scratch(slice_bytes + (plan.blocks > 1 ? plan.blocks * plan.stride * sizeof(float) : 0));
		if (!plan.partial) return TFHIP_ERR_HIP;
		if (plan.blocks > 1) plan.level = (float*)((char*)plan.partial + slice_bytes);
		plan.colsum_partial = n ? plan.partial + mn : nullptr;
		return TFHIP_OK;
	}
	// the column reduction that follows takes its own scratch from the same arena: reserve room for both
	const size_t partial_bytes = (slices * mn * sizeof(float) + 255) & ~size_t(255);
	const size_t reduce_bytes = partial_bytes / 16 + (1 << 20);
	const size_t colsum_bytes = (slices * n * sizeof(float) + 255) & ~size_t(255);
	char* base = (char*)scratch(partial_bytes + reduce_bytes + (n ? colsum_bytes : 0));
	if (!base) return TFHIP_ERR_HIP;
	plan.partial = (float*)(base + reduce_bytes);
	plan.stride = mn;
	plan.colsum_partial = n ? (float*)(base + reduce_bytes + partial_bytes) : nullptr;
	plan.colsum_stride = n;
	return TFHIP_OK;
}

static int sum_slices(const SlicePlan& plan, size_t slices, float* C, size_t mn, float* colsum, size_t n) {
	if (plan.merged) {
		const size_t width = mn + ((n + 3) & ~size_t(3));
		const unsigned groups = (unsigned)((width + 255) / 256);
		const float* src = plan.partial;
		if (plan.blocks > 1) {
			hipLaunchKernelGGL(sgemm_sum_slices_kernel<16>, dim3(groups, (unsigned)plan.blocks), dim3(1024), 0, state().stream, src, (int)slices, (int)plan.per_block, plan.stride, width,
			                   plan.level, plan.stride, width, (float*)nullptr, (size_t)0);
			TFHIP_CHECK_LAUNCH();
			src = plan.level;
			slices = plan.blocks;
		}
		// few columns: more waves per group, so that the slices are still read by the whole chip
		if ((size_t)groups * 4 < (size_t)state().compute_units * 8 && slices >= 64)
			hipLaunchKernelGGL(sgemm_sum_slices_kernel<16>, dim3(groups), dim3(1024), 0, state().stream, src, (int)slices, (int)slices, plan.stride, width, C, (size_t)0, mn, colsum, n);
		else
			hipLaunchKernelGGL(sgemm_sum_slices_kernel<4>, dim3(groups), dim3(256), 0, state().stream, src, (int)slices, (int)slices, plan.stride, width, C, (size_t)0, mn, colsum, n);
		TFHIP_CHECK_LAUNCH();
		return TFHIP_OK;
	}
	const int rc = tfhip_reduce_cols_f32(TFHIP_REDUCE_SUM, plan.partial, C, slices, mn);
	if (rc || !n) return rc;
	return tfhip_reduce_cols_f32(TFHIP_REDUCE_SUM, plan.colsum_partial, colsum, slices, n);
}

// The element-wise tail TensorFrost fuses behind a matmul loop: bias add (+ ReLU) of a dense layer, or the
// ReLU mask of the backward pass (keep the product where the forward activation was positive).
__device__ __forceinline__ float apply_epilogue(const GemmArgs& g, size_t row, int col, float v) {
	if (g.epilogue == TFHIP_EPILOGUE_NONE) return v;
	if (g.epilogue == TFHIP_EPILOGUE_MASK_POSITIVE) return g.aux[row * g.ldc + col] > 0.0f ? v : 0.0f;
	v += g.aux[col];
	if (g.epilogue == TFHIP_EPILOGUE_BIAS_RELU) v = v > 0.0f ? v : 0.0f;
	return v;
}

// Fetches this thread's share of the A panel (128 m x 16 k) into 8 registers.
// A_TRANS == false: A is [M,K] (k contiguous). Thread t: row = t/4 (+64), k-quad = t%4.
// A_TRANS == true:  A is [K,M] (m contiguous). Thread t: k = t/32 (+8), m-quad = t%32.
template <bool A_TRANS, bool GUARD>
__device__ __forceinline__ void fetch_a(const GemmArgs& g, int m0, int k0, int k_end, float (&r)[8]) {
	const int t = threadIdx.x;
	if (!A_TRANS) {
#pragma unroll
		for (int h = 0; h < 2; h++) {
			const int m = m0 + (t >> 2) + h * 64;
			const int k = k0 + (t & 3) * 4;
			const float* p = g.A + (size_t)m * g.lda + k;
			if (!GUARD || (m < g.M && k + 3 < k_end && ((g.lda & 3) == 0) && ((reinterpret_cast<uintptr_t>(g.A) & 15) == 0))) {
				const float4 v = *reinterpret_cast<const float4*>(p);
				r[h * 4 + 0] = v.x; r[h * 4 + 1] = v.y; r[h * 4 + 2] = v.z; r[h * 4 + 3] = v.w;
			} else {
#pragma unroll
				for (int j = 0; j < 4; j++) r[h * 4 + j] = (m < g.M && k + j < k_end) ? p[j] : 0.0f;
			}
		}
	} else {
#pragma unroll
		for (int h = 0; h < 2; h++) {
			const int k = k0 + (t >> 5) + h * 8;
			const int m = m0 + (t & 31) * 4;
			const float* p = g.A + (size_t)k * g.lda + m;
			if (!GUARD || (k < k_end && m + 3 < g.M && ((g.lda & 3) == 0) && ((reinterpret_cast<uintptr_t>(g.A) & 15) == 0))) {
				const float4 v = *reinterpret_cast<const float4*>(p);
				r[h * 4 + 0] = v.x; r[h * 4 + 1] = v.y; r[h * 4 + 2] = v.z; r[h * 4 + 3] = v.w;
			} else {
#pragma unroll
				for (int j = 0; j < 4; j++) r[h * 4 + j] = (k < k_end && m + j < g.M) ? p[j] : 0.0f;
			}
		}
	}
}

// Same for the B panel (16 k x 128 n). B_TRANS == false: B is [K,N] (n contiguous); true: B is [N,K].
template <bool B_TRANS, bool GUARD>
__device__ __forceinline__ void fetch_b(const GemmArgs& g, int n0, int k0, int k_end, float (&r)[8]) {
	const int t = threadIdx.x;
	if (!B_TRANS) {
#pragma unroll
		for (int h = 0; h < 2; h++) {
			const int k = k0 + (t >> 5) + h * 8;
			const int n = n0 + (t & 31) * 4;
			const float* p = g.B + (size_t)k * g.ldb + n;
			if (!GUARD || (k < k_end && n + 3 < g.N && ((g.ldb & 3) == 0) && ((reinterpret_cast<uintptr_t>(g.B) & 15) == 0))) {
				const float4 v = *reinterpret_cast<const float4*>(p);
				r[h * 4 + 0] = v.x; r[h * 4 + 1] = v.y; r[h * 4 + 2] = v.z; r[h * 4 + 3] = v.w;
			} else {
#pragma unroll
				for (int j = 0; j < 4; j++) r[h * 4 + j] = (k < k_end && n + j < g.N) ? p[j] : 0.0f;
			}
		}
	} else {
#pragma unroll
		for (int h = 0; h < 2; h++) {
			const int n = n0 + (t >> 2) + h * 64;
			const int k = k0 + (t & 3) * 4;
			const float* p = g.B + (size_t)n * g.ldb + k;
			if (!GUARD || (n < g.N && k + 3 < k_end && ((g.ldb & 3) == 0) && ((reinterpret_cast<uintptr_t>(g.B) & 15) == 0))) {
				const float4 v = *reinterpret_cast<const float4*>(p);
				r[h * 4 + 0] = v.x; r[h * 4 + 1] = v.y; r[h * 4 + 2] = v.z; r[h * 4 + 3] = v.w;
			} else {
#pragma unroll
				for (int j = 0; j < 4; j++) r[h * 4 + j] = (n < g.N && k + j < k_end) ? p[j] : 0.0f;
			}
		}
	}
}

// Writes the fetched registers into the LDS panel S[k][x] (x = m or n). K_CONTIGUOUS: the registers hold 4
// consecutive k of one x (transpose on the way in); otherwise 4 consecutive x of one k.
// Rows 8..15 of a panel are stored eight words further right than rows 0..7 (a panel is 16 rows of 132 words plus
// those eight). In the transposing write a wave's lanes cover 16 columns of four k-quads, i.e. rows 4q + j for
// q = 0..3; with rows 132 words apart the quads q and q + 2 would fall on the same banks (4 * 132 * 2 = 1056 = 0 mod
// 32): a two-way conflict on every one of the eight writes of a panel, 16 cycles per wave and panel by the
// bank-conflict counter. With the shift, quads 2 and 3 land eight banks beside quads 0 and 1. A shift rather than an
// exchange of column blocks, so that a reader's address is one per-lane base plus a compile-time offset in both halves.
__device__ __forceinline__ int lds_shift(int row) { return (row & 8); }
constexpr int kPanelWords = kBK * kLdsStride + 8;

template <bool K_CONTIGUOUS>
__device__ __forceinline__ void stage(float* S, const float (&r)[8]) {
	const int t = threadIdx.x;
	if (K_CONTIGUOUS) {
#pragma unroll
		for (int h = 0; h < 2; h++) {
			const int x = (t >> 2) + h * 64;
			const int k = (t & 3) * 4;
			const int xs = x + lds_shift(k);  // k, k + 1, k + 2, k + 3 lie in the same half of the panel
#pragma unroll
			for (int j = 0; j < 4; j++) S[(k + j) * kLdsStride + xs] = r[h * 4 + j];
		}
	} else {
#pragma unroll
		for (int h = 0; h < 2; h++) {
			const int k = (t >> 5) + h * 8;
			const int x = ((t & 31) * 4) + lds_shift(k);
			*reinterpret_cast<float4*>(&S[k * kLdsStride + x]) = make_float4(r[h * 4 + 0], r[h * 4 + 1], r[h * 4 + 2], r[h * 4 + 3]);
		}
	}
}

// The k loop of one 128x128 tile: register prefetch of the next panels, double-buffered LDS, 32 MFMAs per panel and
// wave. The kernel runs it with GUARD == true for tiles that cross an edge of the matrices, K ranges that are not a
// multiple of the panel depth and unaligned rows; every other tile takes sgemm_mainloop_interior below.
// COLSUM (tn, B is [K, N]): a thread fetches the same four columns of B in every panel (rows t/32 and t/32 + 8), so the
// column sums of the panels it stages accumulate in four registers; `sum_columns` is group-uniform.
template <int LAYOUT, bool GUARD, bool COLSUM>
__device__ __forceinline__ void sgemm_mainloop(const GemmArgs& g, int m0, int n0, int k_begin, int k_end, float (&As)[2][kPanelWords],
                                               float (&Bs)[2][kPanelWords], floatx4 (&acc)[4][4], float* bsum, bool sum_columns) {
	constexpr bool A_TRANS = LAYOUT == kTN;
	constexpr bool B_TRANS = LAYOUT == kNT;
	const int lane = threadIdx.x & 63;
	const int wave = threadIdx.x >> 6;
	const int wm = (wave >> 1) * 64;  // wave's corner inside the tile
	const int wn = (wave & 1) * 64;
	float ra[8], rb[8];
	fetch_a<A_TRANS, GUARD>(g, m0, k_begin, k_end, ra);
	fetch_b<B_TRANS, GUARD>(g, n0, k_begin, k_end, rb);
	stage<!A_TRANS>(As[0], ra);
	stage<B_TRANS>(Bs[0], rb);
	if (COLSUM && sum_columns) {
#pragma unroll
		for (int j = 0; j < 4; j++) bsum[j] += rb[j] + rb[4 + j];
	}
	if (k_begin + kBK < k_end) {
		fetch_a<A_TRANS, GUARD>(g, m0, k_begin + kBK, k_end, ra);
		fetch_b<B_TRANS, GUARD>(g, n0, k_begin + kBK, k_end, rb);
	}
	__syncthreads();

	// Panel i is multiplied out of one LDS buffer while panel i + 1 (fetched during the previous step) is written into
	// the other at the top of the step and panel i + 2 starts its way from memory: a wave leaves the barrier with
	// nothing but its fragment reads between it and the next MFMA burst.
	int buf = 0;
	for (int k0 = k_begin; k0 < k_end; k0 += kBK) {
		if (k0 + kBK < k_end) {
			stage<!A_TRANS>(As[buf ^ 1], ra);
			stage<B_TRANS>(Bs[buf ^ 1], rb);
			if (COLSUM && sum_columns) {
#pragma unroll
				for (int j = 0; j < 4; j++) bsum[j] += rb[j] + rb[4 + j];
			}
			if (k0 + 2 * kBK < k_end) {
				fetch_a<A_TRANS, GUARD>(g, m0, k0 + 2 * kBK, k_end, ra);
				fetch_b<B_TRANS, GUARD>(g, n0, k0 + 2 * kBK, k_end, rb);
			}
		}
		const float* as = As[buf];
		const float* bs = Bs[buf];
		const int kq = lane >> 4;   // which k of the four this lane feeds
		const int x = lane & 15;
#pragma unroll
		for (int kk = 0; kk < kBK; kk += 4) {
			const int xs = x + lds_shift(kk);  // kk is a multiple of four: kk .. kk + 3 share the shift
			float a[4], b[4];
#pragma unroll
			for (int i = 0; i < 4; i++) {
				a[i] = as[(kk + kq) * kLdsStride + wm + 16 * i + xs];
				b[i] = bs[(kk + kq) * kLdsStride + wn + 16 * i + xs];
			}
#pragma unroll
			for (int i = 0; i < 4; i++)
#pragma unroll
				for (int j = 0; j < 4; j++) acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[i], b[j], acc[i][j], 0, 0, 0);
		}
		__syncthreads();
		buf ^= 1;
	}
}

// The interior form of the k loop (whole tile inside the matrices, K range a multiple of the panel depth, 16-byte
// aligned rows), written so that the steady loop holds next to no vector-ALU instructions: with four waves per SIMD
// feeding one matrix pipe, every ordinary vector instruction of one wave (address arithmetic above all) takes an issue
// slot that another wave's next MFMA may be waiting for. So
//   * the panels are fetched through four running pointers, advanced once per panel by a group-uniform step;
//   * every group-memory address is a per-thread base computed before the loop plus a compile-time offset: the loop is
//     unrolled by two panels so that the buffer index is a constant, and the column exchange of rows 8..15 is folded
//     into a second base;
//   * the fragments of k-pair kk + 2 are read while the MFMAs of k-pair kk run (two sets of four registers);
//   * the next panel's way into group memory (8 writes) and the 4 loads of the one after it sit in the middle of the
//     burst of 32 MFMAs, not in front of it: a wave that leaves the barrier starts multiplying at once.
template <int LAYOUT, bool COLSUM>
__device__ __forceinline__ void sgemm_mainloop_interior(const GemmArgs& g, int m0, int n0, int k_begin, int k_end, float (&As)[2][kPanelWords],
                                                        float (&Bs)[2][kPanelWords], floatx4 (&acc)[4][4], float* bsum, bool sum_columns) {
	constexpr bool A_TRANS = LAYOUT == kTN;
	constexpr bool B_TRANS = LAYOUT == kNT;
	const int t = threadIdx.x;
	const int lane = t & 63;
	const int wave = t >> 6;
	const int wm = (wave >> 1) * 64;
	const int wn = (wave & 1) * 64;

	// Where this thread's two 16-byte pieces of a panel come from: a group-uniform base per piece (advanced by scalar
	// instructions) plus one 32-bit byte offset per operand (buffer loads). And where the pieces go (words inside a panel).
	const char* pa[2];
	const char* pb[2];
	unsigned a_off, b_off;
	int wa[2], wb[2];
	{
		const unsigned xk = (unsigned)(t >> 2), kqk = (unsigned)(t & 3) * 4;  // k contiguous in memory: row xk (+ 64), k-quad kqk
		const unsigned kx = (unsigned)(t >> 5), xqx = (unsigned)(t & 31) * 4;  // x contiguous in memory: row kx (+ 8), x-quad xqx
		a_off = A_TRANS ? (kx * (unsigned)g.lda + xqx) * 4u : (xk * (unsigned)g.lda + kqk) * 4u;
		b_off = B_TRANS ? (xk * (unsigned)g.ldb + kqk) * 4u : (kx * (unsigned)g.ldb + xqx) * 4u;
	}
#pragma unroll
	for (int h = 0; h < 2; h++) {
		const int x = (t >> 2) + h * 64, kq = (t & 3) * 4;
		const int k = (t >> 5) + h * 8, xq = (t & 31) * 4;
		if (!A_TRANS) {
			pa[h] = reinterpret_cast<const char*>(g.A + (size_t)(m0 + h * 64) * g.lda + k_begin);
			wa[h] = kq * kLdsStride + x + lds_shift(kq);
		} else {
			pa[h] = reinterpret_cast<const char*>(g.A + (size_t)(k_begin + h * 8) * g.lda + m0);
			wa[h] = k * kLdsStride + xq + lds_shift(k);
		}
		if (B_TRANS) {
			pb[h] = reinterpret_cast<const char*>(g.B + (size_t)(n0 + h * 64) * g.ldb + k_begin);
			wb[h] = kq * kLdsStride + x + lds_shift(kq);
		} else {
			pb[h] = reinterpret_cast<const char*>(g.B + (size_t)(k_begin + h * 8) * g.ldb + n0);
			wb[h] = k * kLdsStride + xq + lds_shift(k);
		}
	}
	const size_t a_step = A_TRANS ? (size_t)kBK * g.lda : (size_t)kBK;
	const size_t b_step = B_TRANS ? (size_t)kBK : (size_t)kBK * g.ldb;
	const int panels = (k_end - k_begin) / kBK;
	// Every panel of the loop below stages the panel after it and fetches the one after that, the last ones too: their
	// fetches read the last panel again (the pointers stop there) and their staging goes to the buffer nobody reads any
	// more. One form of the loop body, nothing kept live for a tail.
	int fetched = 0;
	float va[8], vb[8];
	auto fetch = [&]() {
		const bool more = fetched + 1 < panels;  // group-uniform: the steps below are scalar selects
		const size_t sa = more ? a_step * sizeof(float) : 0, sb = more ? b_step * sizeof(float) : 0;
		fetched++;
#pragma unroll
		for (int h = 0; h < 2; h++) {
			// buffer loads: the address is a scalar descriptor (rebuilt from the advancing base by scalar instructions)
			// plus the thread's 32-bit offset, no 64-bit vector arithmetic and no address registers
			const uintx4 a4 = __builtin_amdgcn_raw_buffer_load_b128(__builtin_amdgcn_make_buffer_rsrc(const_cast<char*>(pa[h]), 0, 0x7FFFFFFF, 0x00020000), (int)a_off, 0, 0);
			const uintx4 b4 = __builtin_amdgcn_raw_buffer_load_b128(__builtin_amdgcn_make_buffer_rsrc(const_cast<char*>(pb[h]), 0, 0x7FFFFFFF, 0x00020000), (int)b_off, 0, 0);
#pragma unroll
			for (int j = 0; j < 4; j++) {
				va[h * 4 + j] = __uint_as_float(a4[j]);
				vb[h * 4 + j] = __uint_as_float(b4[j]);
			}
			pa[h] += sa;
			pb[h] += sb;
		}
	};
	auto stage_one = [&](float* S, int w, const float* v, bool k_contiguous) {
		if (k_contiguous) {
#pragma unroll
			for (int j = 0; j < 4; j++) S[w + j * kLdsStride] = v[j];
		} else {
			*reinterpret_cast<float4*>(&S[w]) = make_float4(v[0], v[1], v[2], v[3]);
		}
	};
	int staged = 0;
	auto stage_panel = [&](float* as, float* bs) {
#pragma unroll
		for (int h = 0; h < 2; h++) {
			stage_one(as, wa[h], &va[h * 4], !A_TRANS);
			stage_one(bs, wb[h], &vb[h * 4], B_TRANS);
		}
		if (COLSUM) {
			// without a branch (the burst around this stays one scheduling region): every group adds, zeros unless it is
			// one of the first tile row and the panel is not one that was fetched twice
			const bool add = sum_columns && staged < panels;
			float4 sums = *reinterpret_cast<float4*>(bsum);
			sums.x += add ? vb[0] + vb[4] : 0.0f;
			sums.y += add ? vb[1] + vb[5] : 0.0f;
			sums.z += add ? vb[2] + vb[6] : 0.0f;
			sums.w += add ? vb[3] + vb[7] : 0.0f;
			*reinterpret_cast<float4*>(bsum) = sums;
		}
		staged++;
	};

	// fragment reads: lane feeds k = kk + lane / 16 of the four, column lane % 16 of each of the wave's four 16-column
	// blocks: one base per operand, everything else (step, block, the shift of rows 8..15) is a compile-time offset
	const int kq = lane >> 4, x = lane & 15;
	const int ra = kq * kLdsStride + wm + x;
	const int rb = kq * kLdsStride + wn + x;
	// Sixteen v_mfma_f32_16x16x4_f32 per step of four k: the 16x16 instruction moves half the accumulator registers per
	// flop of the 32x32x2 one (four in and out per 2048 flop against sixteen per 4096), which leaves the register file
	// more room for the fragments and panels arriving meanwhile (8192^3: 139.7 -> 143 TFLOP/s, timing-only build).
	// The instructions of a step run row by row of the wave's 4x4 blocks: a row's A fragment is free after its four
	// instructions and is read again for the next step at once (twelve instructions ahead of its use); a B fragment is
	// used by every row and free after its instruction of the last row, four instructions ahead of its next use, which
	// is enough while the SIMD's other waves want the matrix pipe too (a second set of B registers changed nothing:
	// 8192^3 150.0 against 149.6 TFLOP/s). So the fragments of a wave are eight registers. Single reads with 16-bit
	// immediate offsets: a paired read reaches 255 words and would need a base register per step and buffer.
	typedef const volatile __attribute__((address_space(3))) float lds_word;
	float fa[4], fb[4];
	auto read_a = [&](const float* as, int kk, int i) { fa[i] = *(lds_word*)(&as[ra + kk * kLdsStride + lds_shift(kk) + 16 * i]); };
	auto read_b = [&](const float* bs, int kk, int j) { fb[j] = *(lds_word*)(&bs[rb + kk * kLdsStride + lds_shift(kk) + 16 * j]); };
	auto step = [&](const float* as, const float* bs, int kk, bool more) {
#pragma unroll
		for (int i = 0; i < 4; i++) {
#pragma unroll
			for (int j = 0; j < 4; j++) {
				acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x4f32(fa[i], fb[j], acc[i][j], 0, 0, 0);
				if (i == 3 && more) {  // the last row: each B fragment is free after its instruction
					__builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
					read_b(bs, kk + 4, j);
					__builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
				}
			}
			if (i < 3 || !more) __builtin_amdgcn_sched_group_barrier(0x008, 4, 0);
			if (more) {
				read_a(as, kk + 4, i);
				__builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
			}
		}
	};
	// One panel out of buffer BUF: half of the burst, the next panel into the other buffer and the one after it on its
	// way from memory, the other half, the barrier. The scheduling barriers pin that order and the read-ahead.
	auto panel = [&](auto buf_c) {
		constexpr int BUF = decltype(buf_c)::value;
		const float* as = As[BUF];
		const float* bs = Bs[BUF];
#pragma unroll
		for (int i = 0; i < 4; i++) {
			read_a(as, 0, i);
			read_b(bs, 0, i);
		}
		__builtin_amdgcn_sched_group_barrier(0x100, 8, 0);
		step(as, bs, 0, true);
		step(as, bs, 4, true);
		__builtin_amdgcn_sched_barrier(0);
		stage_panel(As[BUF ^ 1], Bs[BUF ^ 1]);
		__builtin_amdgcn_sched_barrier(0);  // the loads below reuse the registers just staged: one set, not two
		fetch();
		__builtin_amdgcn_sched_barrier(0);
		step(as, bs, 8, true);
		step(as, bs, 12, false);
		__syncthreads();
	};

	fetch();
	stage_panel(As[0], Bs[0]);
	fetch();
	__syncthreads();
	int i = 0;
	for (; i + 1 < panels; i += 2) {
		panel(std::integral_constant<int, 0>{});
		panel(std::integral_constant<int, 1>{});
	}
	if (i < panels) panel(std::integral_constant<int, 0>{});
}

template <int LAYOUT, bool COLSUM = false>
__global__ __launch_bounds__(256, COLSUM ? 4 : 3) void sgemm_mfma_kernel(GemmArgs g) {
	static_assert(!COLSUM || LAYOUT == kTN, "column sums of B ride in the tn product only");
	g.A += (size_t)blockIdx.y * g.batch_a;
	g.B += (size_t)blockIdx.y * g.batch_b;
	g.C += (size_t)blockIdx.y * g.batch_c;
	__shared__ __attribute__((aligned(16))) float As[2][kPanelWords];
	__shared__ __attribute__((aligned(16))) float Bs[2][kPanelWords];

	const int lane = threadIdx.x & 63;
	const int wave = threadIdx.x >> 6;
	const int wm = (wave >> 1) * 64;
	const int wn = (wave & 1) * 64;
	// Tiles of one row of C (same A panel) are neighbours in the grid, so they run together and share A in L2.
	const int tiles_n = (g.N + kBN - 1) / kBN;
	const int m0 = (blockIdx.x / tiles_n) * kBM;
	const int n0 = (blockIdx.x % tiles_n) * kBN;
	const int k_begin = blockIdx.z * g.k_per_slice;
	const int k_end = k_begin + g.k_per_slice < g.K ? k_begin + g.k_per_slice : g.K;

	floatx4 acc[4][4];  // 16x16 blocks of the wave's 64x64: element e of lane l is row 4 * (l / 16) + e, column l % 16
#pragma unroll
	for (int i = 0; i < 4; i++)
#pragma unroll
		for (int j = 0; j < 4; j++)
#pragma unroll
			for (int e = 0; e < 4; e++) acc[i][j][e] = 0.0f;

	const bool interior = m0 + kBM <= g.M && n0 + kBN <= g.N && ((k_end - k_begin) % kBK) == 0 && k_end > k_begin && ((g.lda | g.ldb) & 3) == 0 &&
	                      g.lda < (1 << 22) && g.ldb < (1 << 22) &&  // a thread's byte offset inside a panel fits 32 bits
	                      ((reinterpret_cast<uintptr_t>(g.A) | reinterpret_cast<uintptr_t>(g.B)) & 15) == 0;
	// Column sums of the panels a thread stages, four per thread, in group memory rather than in registers: the loop is
	// at the register budget of four waves per SIMD, and only the groups of the first tile row add anything here.
	__shared__ __attribute__((aligned(16))) float column_sums[COLSUM ? 1024 : 4];
	float* bsum = &column_sums[COLSUM ? threadIdx.x * 4 : 0];
	if (COLSUM) {
#pragma unroll
		for (int j = 0; j < 4; j++) bsum[j] = 0.0f;
	}
	const bool sum_columns = COLSUM && m0 == 0;  // the groups of the first tile row read every row of B's slice once
	if (interior)
		sgemm_mainloop_interior<LAYOUT, COLSUM>(g, m0, n0, k_begin, k_end, As, Bs, acc, bsum, sum_columns);
	else
		sgemm_mainloop<LAYOUT, true, COLSUM>(g, m0, n0, k_begin, k_end, As, Bs, acc, bsum, sum_columns);
	if (COLSUM && sum_columns) {
		// eight threads (t / 32 = 0 .. 7) hold partial sums of the same four columns; the main loop ended with a barrier
		// behind the last of their additions
		const int t = threadIdx.x;
		if (t < kBN && n0 + t < g.N) {
			float total = 0.0f;
#pragma unroll
			for (int r = 0; r < 8; r++) total += column_sums[(r * 32 + (t >> 2)) * 4 + (t & 3)];
			g.colsum[(size_t)blockIdx.z * g.colsum_stride + n0 + t] = total;
		}
	}

	float* C = g.C + (size_t)blockIdx.z * g.c_slice_stride;
	const bool whole = m0 + kBM <= g.M && n0 + kBN <= g.N && (g.ldc & 3) == 0 && (reinterpret_cast<uintptr_t>(C) & 15) == 0 &&
	                   (g.epilogue == TFHIP_EPILOGUE_NONE || (reinterpret_cast<uintptr_t>(g.aux) & 15) == 0);
	if (whole) {
		// Whole tile inside C: each wave turns its 32x32 blocks through its own corner of group memory (the panels
		// are no longer needed after the loop's last barrier) so that 8 lanes write one 128-byte row segment with
		// 16-byte stores, and the bias / mask of a fused tail is read the same way.
		constexpr int kStride = 36;
		float* T = (wave < 2 ? &As[0][0] : &Bs[0][0]) + (wave & 1) * (32 * kStride);  // 2 x 4608 B in each 16896 B panel array
		const int rr = lane >> 3, c4 = (lane & 7) * 4;
		// The mask of a block is fetched while the block before it is turned and stored: 268 MB of it behind a
		// [262144, 256] product would otherwise be waited for load by load.
		const bool masked = g.epilogue == TFHIP_EPILOGUE_MASK_POSITIVE;
		float4 mask[4];  // row group p of the current block; replaced by the next block's as soon as it has been used
		auto fetch_mask = [&](int i, int j, int p) {
			mask[p] = *reinterpret_cast<const float4*>(g.aux + (size_t)(m0 + wm + i * 32 + rr + 8 * p) * g.ldc + (n0 + wn + j * 32 + c4));
		};
		if (masked) {
#pragma unroll
			for (int p = 0; p < 4; p++) fetch_mask(0, 0, p);
		}
#pragma unroll
		for (int i = 0; i < 2; i++)
#pragma unroll
			for (int j = 0; j < 2; j++) {
#pragma unroll
				for (int a = 0; a < 2; a++)
#pragma unroll
					for (int b = 0; b < 2; b++)
#pragma unroll
						for (int e = 0; e < 4; e++) T[(16 * a + 4 * (lane >> 4) + e) * kStride + 16 * b + (lane & 15)] = acc[2 * i + a][2 * j + b][e];
				__builtin_amdgcn_wave_barrier();  // the wave's own writes, read back by other lanes below
				const int col = n0 + wn + j * 32 + c4;
				float4 bias = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
				if (g.epilogue == TFHIP_EPILOGUE_BIAS || g.epilogue == TFHIP_EPILOGUE_BIAS_RELU) bias = *reinterpret_cast<const float4*>(g.aux + col);
#pragma unroll
				for (int p = 0; p < 4; p++) {
					const size_t row = (size_t)(m0 + wm + i * 32 + rr + 8 * p);
					float4 v = *reinterpret_cast<const float4*>(&T[(rr + 8 * p) * kStride + c4]);
					if (masked) {
						const float4 a = mask[p];
						if (i < 1 || j < 1) fetch_mask(j == 1 ? i + 1 : i, j == 1 ? 0 : 1, p);
						v.x = a.x > 0.0f ? v.x : 0.0f;
						v.y = a.y > 0.0f ? v.y : 0.0f;
						v.z = a.z > 0.0f ? v.z : 0.0f;
						v.w = a.w > 0.0f ? v.w : 0.0f;
					} else if (g.epilogue != TFHIP_EPILOGUE_NONE) {
						v.x += bias.x;
						v.y += bias.y;
						v.z += bias.z;
						v.w += bias.w;
						if (g.epilogue == TFHIP_EPILOGUE_BIAS_RELU) {
							v.x = v.x > 0.0f ? v.x : 0.0f;
							v.y = v.y > 0.0f ? v.y : 0.0f;
							v.z = v.z > 0.0f ? v.z : 0.0f;
							v.w = v.w > 0.0f ? v.w : 0.0f;
						}
					}
					*reinterpret_cast<float4*>(C + row * g.ldc + col) = v;
				}
				__builtin_amdgcn_wave_barrier();
			}
		return;
	}
#pragma unroll
	for (int i = 0; i < 4; i++)
#pragma unroll
		for (int j = 0; j < 4; j++) {
			const int col = n0 + wn + j * 16 + (lane & 15);
#pragma unroll
			for (int e = 0; e < 4; e++) {
				const int row = m0 + wm + i * 16 + 4 * (lane >> 4) + e;
				if (row < g.M && col < g.N) C[(size_t)row * g.ldc + col] = apply_epilogue(g, (size_t)row, col, acc[i][j][e]);
			}
		}
}

// ---- short K (K <= 128): nn / nt products whose whole B fits group memory --------------------------------------------
//
// With so few panels the tiled kernel spends its time filling and draining its pipeline. Here a group keeps a
// [K, NB*32] block of B in group memory for its whole life and every wave streams 32 rows of A straight from memory
// into the matrix instruction's operand layout: the 32x32x2 instruction sums over a pair of k, and since a sum does
// not care about order, lane l pairs k = j with k = K/2 + j (lanes 0-31 feed the first, lanes 32-63 the second), so
// that a lane needs K/2 consecutive floats of its row -- plain 16-byte loads, no group memory, no barrier in the loop.
template <int NB, bool B_TRANS>
__global__ __launch_bounds__(256) void sgemm_short_k_kernel(GemmArgs g, unsigned row_groups) {
	extern __shared__ float bs[];  // [K][NB * 32 + 1 (pad)]
	constexpr int kCols = NB * 32;
	constexpr int kStride = kCols + 1;
	const int lane = threadIdx.x & 63;
	const int wave = threadIdx.x >> 6;
	const int x = lane & 31, h = lane >> 5;
	const int n0 = blockIdx.y * kCols;
	const int half = g.K >> 1;  // a multiple of 4
	for (int i = threadIdx.x; i < g.K * kCols; i += 256) {
		const int k = i / kCols, c = i - k * kCols;
		bs[k * kStride + c] = n0 + c < g.N ? (B_TRANS ? g.B[(size_t)(n0 + c) * g.ldb + k] : g.B[(size_t)k * g.ldb + n0 + c]) : 0.0f;
	}
	__syncthreads();
	const float* b = bs + (h * half) * kStride + x;
	const bool vec_out = (g.N & 3) == 0 && (g.ldc & 3) == 0 && (reinterpret_cast<uintptr_t>(g.C) & 15) == 0;
	// The group keeps its block of B and walks 128-row groups of A; a wave has the next 16 floats of its row in
	// flight while it multiplies the current 16.
	for (unsigned rg = blockIdx.x; rg < row_groups; rg += gridDim.x) {
		const size_t row0 = ((size_t)rg * 4 + wave) * 32;
		if (row0 >= (size_t)g.M) continue;
		const size_t my_row = row0 + x < (size_t)g.M ? row0 + x : (size_t)g.M - 1;  // rows past the end repeat the last one; never stored
		const float* a = g.A + my_row * g.lda + h * half;
		floatx16 acc[NB];
#pragma unroll
		for (int nb = 0; nb < NB; nb++)
#pragma unroll
			for (int e = 0; e < 16; e++) acc[nb][e] = 0.0f;
		float4 cur[4], nxt[4];
#pragma unroll
		for (int q = 0; q < 4; q++) cur[q] = 4 * q < half ? *reinterpret_cast<const float4*>(a + 4 * q) : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
		for (int j = 0; j < half; j += 16) {
#pragma unroll
			for (int q = 0; q < 4; q++) nxt[q] = j + 16 + 4 * q < half ? *reinterpret_cast<const float4*>(a + j + 16 + 4 * q) : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
#pragma unroll
			for (int q = 0; q < 4; q++) {
				if (j + 4 * q < half) {  // uniform
					const float av[4] = {cur[q].x, cur[q].y, cur[q].z, cur[q].w};
#pragma unroll
					for (int jj = 0; jj < 4; jj++) {
#pragma unroll
						for (int nb = 0; nb < NB; nb++)
							acc[nb] = __builtin_amdgcn_mfma_f32_32x32x2f32(av[jj], b[(j + 4 * q + jj) * kStride + nb * 32], acc[nb], 0, 0, 0);
					}
				}
			}
#pragma unroll
			for (int q = 0; q < 4; q++) cur[q] = nxt[q];
		}
		// element e of lane l is row 8*(e/4) + 4*(l/32) + e%4, column l%32
		if (vec_out) {
			// through the wave's own corner of group memory, so that 8 lanes write one 128-byte row segment as 16-byte stores
			constexpr int kT = 36;
			float* T = bs + g.K * kStride + wave * (32 * kT);
			const int rr = lane >> 3, c4 = (lane & 7) * 4;
#pragma unroll
			for (int nb = 0; nb < NB; nb++) {
#pragma unroll
				for (int e = 0; e < 16; e++) T[(8 * (e >> 2) + 4 * h + (e & 3)) * kT + x] = acc[nb][e];
				__builtin_amdgcn_wave_barrier();
				const int col = n0 + nb * 32 + c4;
#pragma unroll
				for (int p = 0; p < 4; p++) {
					const size_t row = row0 + rr + 8 * p;
					if (row < (size_t)g.M && col < g.N) {
						float4 v = *reinterpret_cast<const float4*>(&T[(rr + 8 * p) * kT + c4]);
						v.x = apply_epilogue(g, row, col, v.x);
						v.y = apply_epilogue(g, row, col + 1, v.y);
						v.z = apply_epilogue(g, row, col + 2, v.z);
						v.w = apply_epilogue(g, row, col + 3, v.w);
						*reinterpret_cast<float4*>(g.C + row * g.ldc + col) = v;
					}
				}
				__builtin_amdgcn_wave_barrier();
			}
		} else {
#pragma unroll
			for (int nb = 0; nb < NB; nb++) {
				const int col = n0 + nb * 32 + x;
				if (col < g.N) {
#pragma unroll
					for (int e = 0; e < 16; e++) {
						const size_t row = row0 + 8 * (e >> 2) + 4 * h + (e & 3);
						if (row < (size_t)g.M) g.C[row * g.ldc + col] = apply_epilogue(g, row, col, acc[nb][e]);
					}
				}
			}
		}
	}
}

// One thread per element of C; consecutive threads walk along n. For skinny or tiny products.
template <int LAYOUT>
__global__ __launch_bounds__(256) void sgemm_plain_kernel(GemmArgs g) {
	g.A += (size_t)blockIdx.y * g.batch_a;
	g.B += (size_t)blockIdx.y * g.batch_b;
	g.C += (size_t)blockIdx.y * g.batch_c;
	const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
	if (idx >= (size_t)g.M * g.N) return;
	const int m = (int)(idx / g.N), n = (int)(idx % g.N);
	const int k_begin = blockIdx.z * g.k_per_slice;
	const int k_end = k_begin + g.k_per_slice < g.K ? k_begin + g.k_per_slice : g.K;
	float acc = 0.0f;
	for (int k = k_begin; k < k_end; k++) {
		const float a = LAYOUT == kTN ? g.A[(size_t)k * g.lda + m] : g.A[(size_t)m * g.lda + k];
		const float b = LAYOUT == kNT ? g.B[(size_t)n * g.ldb + k] : g.B[(size_t)k * g.ldb + n];
		acc += a * b;
	}
	(g.C + (size_t)blockIdx.z * g.c_slice_stride)[(size_t)m * g.ldc + n] = apply_epilogue(g, (size_t)m, n, acc);
}

// ---- skinny products: N <= 8 ------------------------------------------------------------------------------
// These are bandwidth-bound on streaming A once; a 128x128 MFMA tile would waste almost all of its columns.

constexpr int kSkinnyN = 8;

// nn / nt with A[M,K]: a 256-thread group owns 64 rows of A and walks K in chunks of 64. A chunk is read
// with 16-byte loads along k (coalesced) and laid into group memory so that lane r can walk row r; wave q then
// multiplies columns [16q, 16q+16) of the chunk with the matching entries of B, which are the same for every
// lane of the wave and come through the scalar unit. The four partial dot products per (row, n) meet in group
// memory and leave as one contiguous block of C.
constexpr int kSkinnyRows = 64, kSkinnyKC = 64, kSkinnyStride = kSkinnyKC + 1;

template <int LAYOUT, int NC>
__global__ __launch_bounds__(256) void sgemm_skinny_rows_kernel(GemmArgs g) {
	__shared__ float tile[kSkinnyRows * kSkinnyStride];
	__shared__ float partial[4 * kSkinnyRows * NC];
	const int t = threadIdx.x;
	const int lane = t & 63;
	const int q = __builtin_amdgcn_readfirstlane(t >> 6);
	const size_t row0 = (size_t)blockIdx.x * kSkinnyRows;
	const bool vec = (g.lda & 3) == 0 && (reinterpret_cast<uintptr_t>(g.A) & 15) == 0;
	// loader: thread t fetches columns [4*(t%16), +4) of rows t/16 + 16*i, i = 0..3
	const int lc = (t & 15) * 4, lr = t >> 4;
	float4 next[4];
	auto fetch = [&](int k0) {
#pragma unroll
		for (int i = 0; i < 4; i++) {
			const size_t row = row0 + lr + 16 * i;
			const int k = k0 + lc;
			const float* p = g.A + row * g.lda + k;
			if (row < (size_t)g.M && vec && k + 3 < g.K) {
				next[i] = *reinterpret_cast<const float4*>(p);
			} else {
				const bool in = row < (size_t)g.M;
				next[i].x = in && k + 0 < g.K ? p[0] : 0.0f;
				next[i].y = in && k + 1 < g.K ? p[1] : 0.0f;
				next[i].z = in && k + 2 < g.K ? p[2] : 0.0f;
				next[i].w = in && k + 3 < g.K ? p[3] : 0.0f;
			}
		}
	};
	float acc[NC];
#pragma unroll
	for (int n = 0; n < NC; n++) acc[n] = 0.0f;
	fetch(0);
	for (int k0 = 0; k0 < g.K; k0 += kSkinnyKC) {
		__syncthreads();  // the previous chunk has been consumed
#pragma unroll
		for (int i = 0; i < 4; i++) {
			float* d = tile + (lr + 16 * i) * kSkinnyStride + lc;
			d[0] = next[i].x;
			d[1] = next[i].y;
			d[2] = next[i].z;
			d[3] = next[i].w;
		}
		__syncthreads();
		if (k0 + kSkinnyKC < g.K) fetch(k0 + kSkinnyKC);
		const float* a = tile + lane * kSkinnyStride + q * 16;
		const int kb = k0 + q * 16;
#pragma unroll
		for (int j = 0; j < 16; j++) {
			const float av = a[j];
			const int k = kb + j;
			if (k < g.K) {  // wave-uniform
#pragma unroll
				for (int n = 0; n < NC; n++) acc[n] += av * (LAYOUT == kNT ? g.B[(size_t)n * g.ldb + k] : g.B[(size_t)k * g.ldb + n]);
			}
		}
	}
#pragma unroll
	for (int n = 0; n < NC; n++) partial[(q * kSkinnyRows + lane) * NC + n] = acc[n];
	__syncthreads();
	for (int e = t; e < kSkinnyRows * NC; e += 256) {
		const size_t row = row0 + e / NC;
		if (row < (size_t)g.M) {
			const float sum = (partial[e] + partial[kSkinnyRows * NC + e]) + (partial[2 * kSkinnyRows * NC + e] + partial[3 * kSkinnyRows * NC + e]);
			g.C[row * g.ldc + e % NC] = apply_epilogue(g, row, e % NC, sum);
		}
	}
}

// nn / nt with K <= 256 and at most eight columns (the last layer of a dense network on a large batch): the lanes of a
// wave lie along k (one 16-byte load per row, the 4 x NC entries of B a lane needs stay in registers for the whole
// kernel), a wave takes R rows per trip and the R * NC partial dot products per lane are summed across the wave by
// halving: at distance 32 a lane keeps half of its values and receives the other lane's partial sums of those, at
// distance 16 half of the rest, ... until one value per lane is left, which the remaining distances sum as usual.
// P (a power of two >= R * NC) values cost P - 1 + log2(64 / P) exchanges instead of 6 * R * NC; lane l ends with the
// sum of value l / (64 / P) (the step at distance d decides one bit of that index by bit d of the lane). No group memory, no barrier: bandwidth-bound on reading A once.
template <int NC>
struct RowsLanesShape {
	static constexpr int R = NC == 1 ? 8 : (16 / NC < 2 ? 2 : 16 / NC);
	static constexpr int V = R * NC;
	static constexpr int P = V <= 8 ? 8 : (V <= 16 ? 16 : 32);
};

// The value of lane ^ DIST for DIST = 8, 2, 1 and of lane ^ 7 for DIST = 4 (also a partner whose bit 2 differs, and the
// distances 2 and 1 that follow close the same groups of eight lanes), read through the data-parallel path of the ALU.
template <int DIST>
__device__ __forceinline__ float lane_partner(float x) {
	constexpr int ctrl = DIST == 8 ? 0x128 /* row_ror:8 */ : DIST == 4 ? 0x141 /* row_half_mirror */ : DIST == 2 ? 0x4e /* quad_perm:[2,3,0,1] */ : 0xb1 /* quad_perm:[1,0,3,2] */;
	return __uint_as_float(__builtin_amdgcn_update_dpp(0u, __float_as_uint(x), ctrl, 0xf, 0xf, false));
}

// One halving step over COUNT values at distance DIST, then the next; with one value left, the plain sums. At distances
// 32 and 16 the swap instructions exchange the upper half of one register with the lower half of another (halves of
// the wave, or odd and even rows of sixteen lanes), which is the whole step: a' + b' is a's sum in the lower lanes and
// b's in the upper ones.
template <int COUNT, int DIST>
__device__ __forceinline__ void sum_by_halving(float* v, int lane) {
	if constexpr (DIST >= 1) {
		constexpr int half = COUNT > 1 ? COUNT / 2 : 1;
#pragma unroll
		for (int e = 0; e < half; e++) {
			const float a = v[e], b = COUNT > 1 ? v[e + COUNT / 2] : v[e];
			if constexpr (DIST == 32) {
				const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(a), __float_as_uint(b), false, false);
				v[e] = __uint_as_float(r[0]) + __uint_as_float(r[1]);
			} else if constexpr (DIST == 16) {
				const auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(a), __float_as_uint(b), false, false);
				v[e] = __uint_as_float(r[0]) + __uint_as_float(r[1]);
			} else if constexpr (COUNT > 1) {
				const bool upper = (lane & DIST) != 0;
				v[e] = (upper ? b : a) + lane_partner<DIST>(upper ? a : b);
			} else {
				v[e] = a + lane_partner<DIST>(a);
			}
		}
		sum_by_halving<(COUNT > 1 ? COUNT / 2 : 1), DIST / 2>(v, lane);
	}
}

template <int LAYOUT, int NC>
__global__ __launch_bounds__(256) void sgemm_rows_lanes_kernel(GemmArgs g, unsigned row_groups) {
	constexpr int R = RowsLanesShape<NC>::R, P = RowsLanesShape<NC>::P, kLanesPerValue = 64 / P;
	const int lane = threadIdx.x & 63;
	const bool active = lane * 4 < g.K;  // K is a multiple of four
	const int k = active ? lane * 4 : 0;
	float b[4][NC];
#pragma unroll
	for (int i = 0; i < 4; i++)
#pragma unroll
		for (int n = 0; n < NC; n++) {
			const float value = LAYOUT == kNT ? g.B[(size_t)n * g.ldb + k + i] : g.B[(size_t)(k + i) * g.ldb + n];
			b[i][n] = active ? value : 0.0f;
		}
	const unsigned waves = gridDim.x * 4;
	const size_t last_row = (size_t)g.M - 1;
	// From the last rows to the first: A is as a rule what the layer before has just written front to back, and of a
	// tensor larger than the 256 MiB last-level cache it is the end that is still there. Inside a training step
	// ([262144, 256] x [256, 3] right behind the product that wrote A): 47.7 us against 58.3 front to back; on an
	// operand that comes from memory either way takes the same time (48.6 / 49.1 us).
	for (unsigned step = blockIdx.x * 4 + (threadIdx.x >> 6); step < row_groups; step += waves) {
		const unsigned rg = row_groups - 1 - step;
		const size_t row0 = (size_t)rg * R;
		float4 a[R];
#pragma unroll
		for (int r = 0; r < R; r++) {  // rows past the end read the last row again; their results are not stored
			const size_t row = row0 + r < last_row ? row0 + r : last_row;
			a[r] = *reinterpret_cast<const float4*>(g.A + row * g.lda + k);
		}
		float v[P];
#pragma unroll
		for (int e = 0; e < P; e++) v[e] = 0.0f;
#pragma unroll
		for (int r = 0; r < R; r++) {
			if (!active) a[r] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
#pragma unroll
			for (int n = 0; n < NC; n++) v[r * NC + n] = (a[r].x * b[0][n] + a[r].y * b[1][n]) + (a[r].z * b[2][n] + a[r].w * b[3][n]);
		}
		sum_by_halving<P, 32>(v, lane);
		const int value = lane / kLanesPerValue;
		const size_t row = row0 + value / NC;
		const int col = value % NC;
		if ((lane & (kLanesPerValue - 1)) == 0 && value < R * NC && row < (size_t)g.M) g.C[row * g.ldc + col] = apply_epilogue(g, row, col, v[0]);
	}
}

template <int LAYOUT>
static void launch_rows_lanes(const GemmArgs& g, hipStream_t stream, int compute_units) {
#define TFHIP_ROWS_LANES(NC)                                                                                                      \
	{                                                                                                                             \
		const size_t row_groups = ((size_t)g.M + RowsLanesShape<NC>::R - 1) / RowsLanesShape<NC>::R;                              \
		size_t groups = (row_groups + 3) / 4;                                                                                     \
		if (groups > (size_t)compute_units * 8) groups = (size_t)compute_units * 8;                                               \
		hipLaunchKernelGGL((sgemm_rows_lanes_kernel<LAYOUT, NC>), dim3((unsigned)groups), dim3(256), 0, stream, g, (unsigned)row_groups); \
	}
	switch (g.N) {
		case 1: TFHIP_ROWS_LANES(1); break;
		case 2: TFHIP_ROWS_LANES(2); break;
		case 3: TFHIP_ROWS_LANES(3); break;
		case 4: TFHIP_ROWS_LANES(4); break;
		case 5: TFHIP_ROWS_LANES(5); break;
		case 6: TFHIP_ROWS_LANES(6); break;
		case 7: TFHIP_ROWS_LANES(7); break;
		default: TFHIP_ROWS_LANES(8); break;
	}
#undef TFHIP_ROWS_LANES
}

template <int LAYOUT>
static void launch_skinny_rows(const GemmArgs& g, unsigned groups, hipStream_t stream) {
	switch (g.N) {
		case 1: hipLaunchKernelGGL((sgemm_skinny_rows_kernel<LAYOUT, 1>), dim3(groups), dim3(256), 0, stream, g); break;
		case 2: hipLaunchKernelGGL((sgemm_skinny_rows_kernel<LAYOUT, 2>), dim3(groups), dim3(256), 0, stream, g); break;
		case 3: hipLaunchKernelGGL((sgemm_skinny_rows_kernel<LAYOUT, 3>), dim3(groups), dim3(256), 0, stream, g); break;
		case 4: hipLaunchKernelGGL((sgemm_skinny_rows_kernel<LAYOUT, 4>), dim3(groups), dim3(256), 0, stream, g); break;
		case 5: hipLaunchKernelGGL((sgemm_skinny_rows_kernel<LAYOUT, 5>), dim3(groups), dim3(256), 0, stream, g); break;
		case 6: hipLaunchKernelGGL((sgemm_skinny_rows_kernel<LAYOUT, 6>), dim3(groups), dim3(256), 0, stream, g); break;
		case 7: hipLaunchKernelGGL((sgemm_skinny_rows_kernel<LAYOUT, 7>), dim3(groups), dim3(256), 0, stream, g); break;
		default: hipLaunchKernelGGL((sgemm_skinny_rows_kernel<LAYOUT, 8>), dim3(groups), dim3(256), 0, stream, g); break;
	}
}

// Skinny products with few rows or a long K (matrix times a few vectors): one wave per (row, K segment). A lane
// walks its row of A in 16-byte steps, 64 lanes one KiB at a time; the matching four rows of B (nn) or four columns
// (nt) are small and stay in cache. Lanes meet in a shuffle reduction. With more than one segment per row the
// partial sums go to scratch, partial[(row * segs + seg) * NC + n], and a second kernel adds them.
template <int LAYOUT, int NC>
__global__ __launch_bounds__(256) void sgemm_rows_wave_kernel(GemmArgs g, int segs, int seg_len, float* partial, long c_row, long c_n) {
	const int lane = threadIdx.x & 63;
	const size_t item = (size_t)blockIdx.x * 4 + (threadIdx.x >> 6);
	if (item >= (size_t)g.M * segs) return;
	const size_t row = item / segs;
	const int seg = (int)(item - row * segs);
	const int k0 = seg * seg_len;
	const int k1 = k0 + seg_len < g.K ? k0 + seg_len : g.K;
	const float* a = g.A + row * g.lda;
	const bool vec = (g.lda & 3) == 0 && (reinterpret_cast<uintptr_t>(g.A) & 15) == 0;  // seg_len is a multiple of 4
	float acc[NC];
#pragma unroll
	for (int n = 0; n < NC; n++) acc[n] = 0.0f;
	auto step = [&](int k, float av) {
#pragma unroll
		for (int n = 0; n < NC; n++) acc[n] += av * (LAYOUT == kNT ? g.B[(size_t)n * g.ldb + k] : g.B[(size_t)k * g.ldb + n]);
	};
	// nt, four consecutive k at once: the values of B they meet are four consecutive elements of each of its NC rows.
	const bool b_vec = (reinterpret_cast<uintptr_t>(g.B) & 15) == 0 && (g.ldb & 3) == 0;
	auto step4 = [&](int k, const float4& av) {
		if (b_vec) {
#pragma unroll
			for (int n = 0; n < NC; n++) {
				const float4 t = *reinterpret_cast<const float4*>(g.B + (size_t)n * g.ldb + k);
				acc[n] += (av.x * t.x + av.y * t.y) + (av.z * t.z + av.w * t.w);
			}
		} else {
			step(k, av.x), step(k + 1, av.y), step(k + 2, av.z), step(k + 3, av.w);
		}
	};
	if (LAYOUT == kNN) {
		// nn: lane l takes k = l, l + 64, ...: neighbouring lanes then read neighbouring rows of B, NC floats each, so
		// the wave's loads of B are one contiguous run (a 16-byte load per lane when NC is 4 or 8 and B has no padding).
		const bool b_rows = g.ldb == NC && (NC % 2 == 0) && (reinterpret_cast<uintptr_t>(g.B) & 15) == 0;
		auto row_of_b = [&](int k, float (&b)[NC]) {
			const float* p = g.B + (size_t)k * g.ldb;
			if (b_rows && NC % 4 == 0) {
#pragma unroll
				for (int q = 0; q < NC / 4; q++) {
					const float4 t = *reinterpret_cast<const float4*>(p + 4 * q);
					b[4 * q] = t.x, b[4 * q + 1] = t.y, b[4 * q + 2] = t.z, b[4 * q + 3] = t.w;
				}
			} else if (b_rows) {
#pragma unroll
				for (int q = 0; q < NC / 2; q++) {
					const float2 t = *reinterpret_cast<const float2*>(p + 2 * q);
					b[2 * q] = t.x, b[2 * q + 1] = t.y;
				}
			} else {
#pragma unroll
				for (int n = 0; n < NC; n++) b[n] = p[n];
			}
		};
		int k = k0 + lane;
		for (; k + 448 < k1; k += 512) {  // eight loads of A in flight
			float av[8];
#pragma unroll
			for (int u = 0; u < 8; u++) av[u] = a[k + 64 * u];
#pragma unroll
			for (int u = 0; u < 8; u++) {
				float b[NC];
				row_of_b(k + 64 * u, b);
#pragma unroll
				for (int n = 0; n < NC; n++) acc[n] += av[u] * b[n];
			}
		}
		for (; k < k1; k += 64) {
			float b[NC];
			row_of_b(k, b);
			const float av = a[k];
#pragma unroll
			for (int n = 0; n < NC; n++) acc[n] += av * b[n];
		}
	} else if (vec) {
		int k = k0 + lane * 4;
		for (; k + 768 + 3 < k1; k += 1024) {  // four vectors in flight
			float4 v[4];
#pragma unroll
			for (int u = 0; u < 4; u++) v[u] = *reinterpret_cast<const float4*>(a + k + 256 * u);
#pragma unroll
			for (int u = 0; u < 4; u++) step4(k + 256 * u, v[u]);
		}
		for (; k < k1; k += 256) {
			if (k + 3 < k1) {
				step4(k, *reinterpret_cast<const float4*>(a + k));
			} else {
				for (int j = k; j < k1; j++) step(j, a[j]);
			}
		}
	} else {
		for (int k = k0 + lane; k < k1; k += 64) step(k, a[k]);
	}
#pragma unroll
	for (int n = 0; n < NC; n++) acc[n] = wave_reduce(acc[n], OpSum());
	if (lane == 0) {
#pragma unroll
		for (int n = 0; n < NC; n++) {
			if (segs == 1)
				g.C[row * c_row + n * c_n] = apply_epilogue(g, row, n, acc[n]);
			else
				partial[item * NC + n] = acc[n];
		}
	}
}

// C[row, n] = tail(sum over segments of partial[(row * segs + seg) * N + n]); one wave per element of C.
__global__ __launch_bounds__(256) void sgemm_rows_combine_kernel(GemmArgs g, int segs, const float* __restrict__ partial, long c_row, long c_n) {
	const int lane = threadIdx.x & 63;
	const size_t e = (size_t)blockIdx.x * 4 + (threadIdx.x >> 6);
	if (e >= (size_t)g.M * g.N) return;
	const size_t row = e / g.N;
	const int n = (int)(e - row * g.N);
	float sum = 0.0f;
	for (int sgm = lane; sgm < segs; sgm += 64) sum += partial[(row * segs + sgm) * g.N + n];
	sum = wave_reduce(sum, OpSum());
	if (lane == 0) g.C[row * c_row + n * c_n] = apply_epilogue(g, row, n, sum);
}

// c_row, c_n: strides of C per row and per column (a transposed result when the product was posed the other way round).
template <int LAYOUT>
static int sgemm_rows_wave(const GemmArgs& g, long c_row = -1, long c_n = 1) {
	State& s = state();
	if (c_row < 0) c_row = g.ldc;
	// enough waves for every SIMD several times over; a segment is at least 2048 long
	const size_t want = (size_t)s.compute_units * 64;
	size_t segs = 1, seg_len = (size_t)g.K;
	if ((size_t)g.M < want && g.K >= 4096) {
		segs = (want + g.M - 1) / g.M;
		if (segs > (size_t)g.K / 2048) segs = (size_t)g.K / 2048;
		if (segs > 4096) segs = 4096;
		seg_len = (((size_t)g.K + segs - 1) / segs + 255) & ~size_t(255);
		segs = ((size_t)g.K + seg_len - 1) / seg_len;
	}
	const size_t items = (size_t)g.M * segs;
	if ((items + 3) / 4 > 0x7FFFFFFFull) return fail(TFHIP_ERR_ARG, "sgemm result too large");
	float* partial = nullptr;
	if (segs > 1) {
		partial = (float*)scratch(items * g.N * sizeof(float));
		if (!partial) return TFHIP_ERR_HIP;
	}
	const dim3 grid((unsigned)((items + 3) / 4)), block(256);
	switch (g.N) {
		case 1: hipLaunchKernelGGL((sgemm_rows_wave_kernel<LAYOUT, 1>), grid, block, 0, s.stream, g, (int)segs, (int)seg_len, partial, c_row, c_n); break;
		case 2: hipLaunchKernelGGL((sgemm_rows_wave_kernel<LAYOUT, 2>), grid, block, 0, s.stream, g, (int)segs, (int)seg_len, partial, c_row, c_n); break;
		case 3: hipLaunchKernelGGL((sgemm_rows_wave_kernel<LAYOUT, 3>), grid, block, 0, s.stream, g, (int)segs, (int)seg_len, partial, c_row, c_n); break;
		case 4: hipLaunchKernelGGL((sgemm_rows_wave_kernel<LAYOUT, 4>), grid, block, 0, s.stream, g, (int)segs, (int)seg_len, partial, c_row, c_n); break;
		case 5: hipLaunchKernelGGL((sgemm_rows_wave_kernel<LAYOUT, 5>), grid, block, 0, s.stream, g, (int)segs, (int)seg_len, partial, c_row, c_n); break;
		case 6: hipLaunchKernelGGL((sgemm_rows_wave_kernel<LAYOUT, 6>), grid, block, 0, s.stream, g, (int)segs, (int)seg_len, partial, c_row, c_n); break;
		case 7: hipLaunchKernelGGL((sgemm_rows_wave_kernel<LAYOUT, 7>), grid, block, 0, s.stream, g, (int)segs, (int)seg_len, partial, c_row, c_n); break;
		default: hipLaunchKernelGGL((sgemm_rows_wave_kernel<LAYOUT, 8>), grid, block, 0, s.stream, g, (int)segs, (int)seg_len, partial, c_row, c_n); break;
	}
	TFHIP_CHECK_LAUNCH();
	if (segs > 1) {
		hipLaunchKernelGGL(sgemm_rows_combine_kernel, dim3((unsigned)(((size_t)g.M * g.N + 3) / 4)), block, 0, s.stream, g, (int)segs, (const float*)partial, c_row, c_n);
		TFHIP_CHECK_LAUNCH();
	}
	return TFHIP_OK;
}

// tn with A[K,M], B[K,N], N <= 8: C[m,n] = sum_k A[k,m] * B[k,n]. A 256-thread group owns a slab of k and a tile
// of 256 m (lane = 4 consecutive m as one float4 of a row of A); the four waves take every fourth k of the slab;
// B[k, :] is the same for all lanes. Slabs write partial C matrices that the column reduction sums.
// B is addressed as B[k * b_k + n * b_n] and C as C[m * c_m + n * c_n], so that the same kernel serves a product with
// few ROWS, C[M,N] = A[M,K] B[K,N] with M <= 8, as the transposed problem (its "A" is then B, its "B" the few rows of A).
// COLSUM: the groups of the first tile also add up the rows of B they walk: the column sums of B over the slab, left in
// g.colsum[slab * g.colsum_stride + n].
template <bool COLSUM, int NC>
__global__ __launch_bounds__(256) void sgemm_skinny_tn_kernel(GemmArgs g, int m_tiles, int k_per_slab, long b_k, long b_n, long c_m, long c_n) {
	__shared__ float lds[4][256 * NC];
	const int lane = threadIdx.x & 63;
	const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);  // the rows of B come through the scalar unit
	const int tile = blockIdx.x % m_tiles;
	const int slab = blockIdx.x / m_tiles;
	const int m = (tile * 64 + lane) * 4;
	const int k0 = slab * k_per_slab;
	const int k1 = k0 + k_per_slab < g.K ? k0 + k_per_slab : g.K;
	float acc[4][NC];
#pragma unroll
	for (int j = 0; j < 4; j++)
#pragma unroll
		for (int n = 0; n < NC; n++) acc[j][n] = 0.0f;
	float bsum[NC];  // the same in every lane of a wave
#pragma unroll
	for (int n = 0; n < NC; n++) bsum[n] = 0.0f;
	// lanes beyond M read the last four rows' worth of A again (M is a multiple of four) and drop the result
	const float* a = g.A + (m < g.M ? m : g.M - 4);
	constexpr int U = 4;  // rows of A in flight per lane
	int k = k0 + wave;
	for (; k + 4 * (U - 1) < k1; k += 4 * U) {
		float4 v[U];
		float bn[U][NC];
#pragma unroll
		for (int u = 0; u < U; u++) {
			v[u] = *reinterpret_cast<const float4*>(a + (size_t)(k + 4 * u) * g.lda);
#pragma unroll
			for (int n = 0; n < NC; n++) bn[u][n] = g.B[(size_t)(k + 4 * u) * b_k + n * b_n];
		}
#pragma unroll
		for (int u = 0; u < U; u++)
#pragma unroll
			for (int n = 0; n < NC; n++) {
				if (COLSUM) bsum[n] += bn[u][n];
				acc[0][n] += v[u].x * bn[u][n];
				acc[1][n] += v[u].y * bn[u][n];
				acc[2][n] += v[u].z * bn[u][n];
				acc[3][n] += v[u].w * bn[u][n];
			}
	}
	for (; k < k1; k += 4) {
		const float4 v = *reinterpret_cast<const float4*>(a + (size_t)k * g.lda);
#pragma unroll
		for (int n = 0; n < NC; n++) {
			const float bn = g.B[(size_t)k * b_k + n * b_n];
			if (COLSUM) bsum[n] += bn;
			acc[0][n] += v.x * bn;
			acc[1][n] += v.y * bn;
			acc[2][n] += v.z * bn;
			acc[3][n] += v.w * bn;
		}
	}
#pragma unroll
	for (int j = 0; j < 4; j++)
#pragma unroll
		for (int n = 0; n < NC; n++) lds[wave][(lane * 4 + j) * NC + n] = acc[j][n];
	__syncthreads();
	if (wave == 0 && m < g.M) {
		float* C = g.C + (size_t)slab * g.c_slice_stride;
#pragma unroll
		for (int j = 0; j < 4; j++)
#pragma unroll
			for (int n = 0; n < NC; n++) {
				const int idx = (lane * 4 + j) * NC + n;
				C[(size_t)(m + j) * c_m + n * c_n] = (lds[0][idx] + lds[1][idx]) + (lds[2][idx] + lds[3][idx]);
			}
	}
	if (COLSUM && tile == 0) {
		__syncthreads();
		if (lane == 0) {
#pragma unroll
			for (int n = 0; n < NC; n++) lds[wave][n] = bsum[n];
		}
		__syncthreads();
		if (threadIdx.x < NC) g.colsum[(size_t)slab * g.colsum_stride + threadIdx.x] = (lds[0][threadIdx.x] + lds[1][threadIdx.x]) + (lds[2][threadIdx.x] + lds[3][threadIdx.x]);
	}
}

template <bool COLSUM>
static void launch_skinny_tn(const GemmArgs& g, unsigned groups, hipStream_t stream, int m_tiles, int k_per_slab, long b_k, long b_n, long c_m, long c_n) {
#define TFHIP_SKINNY_TN(NC) hipLaunchKernelGGL((sgemm_skinny_tn_kernel<COLSUM, NC>), dim3(groups), dim3(256), 0, stream, g, m_tiles, k_per_slab, b_k, b_n, c_m, c_n)
	switch (g.N) {
		case 1: TFHIP_SKINNY_TN(1); break;
		case 2: TFHIP_SKINNY_TN(2); break;
		case 3: TFHIP_SKINNY_TN(3); break;
		case 4: TFHIP_SKINNY_TN(4); break;
		case 5: TFHIP_SKINNY_TN(5); break;
		case 6: TFHIP_SKINNY_TN(6); break;
		case 7: TFHIP_SKINNY_TN(7); break;
		default: TFHIP_SKINNY_TN(8); break;
	}
#undef TFHIP_SKINNY_TN
}

static int sgemm_skinny_tn(GemmArgs g, float* C, long b_k = -1, long b_n = 1, long c_m = -1, long c_n = 1, float* colsum = nullptr) {
	State& s = state();
	if (b_k < 0) b_k = g.ldb;
	if (c_m < 0) c_m = g.ldc;
	const size_t M = g.M, N = g.N, K = g.K;
	const int m_tiles = (int)((M + 255) / 256);
	// enough slabs to fill the chip, at least 64 k per slab
	size_t slabs = ((size_t)s.compute_units * 4 + m_tiles - 1) / m_tiles;
	size_t max_slabs = (K + 63) / 64;
	if (slabs > max_slabs) slabs = max_slabs;
	if (slabs < 1) slabs = 1;
	int k_per_slab = (int)((K + slabs - 1) / slabs);
	k_per_slab = (k_per_slab + 3) & ~3;
	slabs = (K + k_per_slab - 1) / k_per_slab;
	SlicePlan plan;
	plan.partial = C;
	plan.stride = M * N;
	g.colsum = colsum;
	if (slabs > 1) {
		const int rc = plan_slices(slabs, M * N, colsum ? N : 0, C, colsum, plan);
		if (rc) return rc;
		g.colsum = plan.colsum_partial;
		g.colsum_stride = plan.colsum_stride;
	}
	g.C = plan.partial;
	g.c_slice_stride = plan.stride;
	if (colsum)
		launch_skinny_tn<true>(g, (unsigned)(m_tiles * slabs), s.stream, m_tiles, k_per_slab, b_k, b_n, c_m, c_n);
	else
		launch_skinny_tn<false>(g, (unsigned)(m_tiles * slabs), s.stream, m_tiles, k_per_slab, b_k, b_n, c_m, c_n);
	TFHIP_CHECK_LAUNCH();
	if (slabs > 1) return sum_slices(plan, slabs, C, M * N, colsum, colsum ? N : 0);
	return TFHIP_OK;
}

// ---- tn with a small result and a very long K (weight gradients of narrow layers) --------------------------------
//
// C[M, N] = sum_k A[k, m] B[k, n] with M <= 128, M * N <= 16384: both operands are read along their rows, which is
// already the matrix instruction's operand layout (lane l feeds row / column l % 32 of k = pair + l / 32), so the loads
// go straight from memory to the instruction, 128 consecutive bytes per half wave, with no group memory and no
// barrier. A wave owns a slab of k and a slot of C: one row of 32 x 32 blocks and up to four block columns. The four
// waves of a group take the `slots` slots of C, and when C has fewer than four of them, different slabs of k.
// The waves of one slab together cover C once; the column reduction sums the slabs.
// COLSUM: the waves of the first block row also add up the values of B they feed to the instruction: the column sums of
// B over the slab, left in colsum[slab * g.colsum_stride + column] (the bias gradient beside the weight gradient).
template <int QN, bool COLSUM>
__global__ __launch_bounds__(256) void sgemm_tn_direct_kernel(GemmArgs g, int k_per_slab, int ngroups, int slots, int nblocks, float* partial, float* colsum) {
	const int lane = threadIdx.x & 63;
	const int wave = threadIdx.x >> 6;
	const int x = lane & 31, h = lane >> 5;
	const int slot = wave % slots;
	const int mi = slot / ngroups;
	const int ni0 = (slot % ngroups) * QN;
	const int slab = blockIdx.x * (4 / slots) + wave / slots;
	const int k0 = slab * k_per_slab;
	if (k0 >= g.K) return;
	const int k1 = k0 + k_per_slab < g.K ? k0 + k_per_slab : g.K;
	const float* a = g.A + (size_t)(k0 + h) * g.lda + mi * 32 + x;
	const float* b = g.B + (size_t)(k0 + h) * g.ldb + ni0 * 32 + x;
	floatx16 acc[QN];
#pragma unroll
	for (int q = 0; q < QN; q++)
#pragma unroll
		for (int e = 0; e < 16; e++) acc[q][e] = 0.0f;
	// Four pairs of k per trip: (1 + QN) * 4 loads in flight per wave, sixteen waves per compute unit.
	constexpr int kPairs = 4;
	float bsum[QN];
#pragma unroll
	for (int q = 0; q < QN; q++) bsum[q] = 0.0f;
	const bool sum_columns = COLSUM && mi == 0;
	// a block column past the last one reads the last one again (no branch around a load); its products are not stored
	int column[QN];
#pragma unroll
	for (int q = 0; q < QN; q++) column[q] = ((ni0 + q < nblocks ? ni0 + q : nblocks - 1) - ni0) * 32;
	int k = k0;
	for (; k + 2 * kPairs <= k1; k += 2 * kPairs) {
		float av[kPairs], bv[kPairs][QN];
#pragma unroll
		for (int u = 0; u < kPairs; u++) {
			av[u] = a[(size_t)(2 * u) * g.lda];
#pragma unroll
			for (int q = 0; q < QN; q++) bv[u][q] = b[(size_t)(2 * u) * g.ldb + column[q]];
		}
#pragma unroll
		for (int u = 0; u < kPairs; u++)
#pragma unroll
			for (int q = 0; q < QN; q++) acc[q] = __builtin_amdgcn_mfma_f32_32x32x2f32(av[u], bv[u][q], acc[q], 0, 0, 0);
		if (sum_columns) {
#pragma unroll
			for (int u = 0; u < kPairs; u++)
#pragma unroll
				for (int q = 0; q < QN; q++) bsum[q] += bv[u][q];
		}
		a += (size_t)(2 * kPairs) * g.lda;
		b += (size_t)(2 * kPairs) * g.ldb;
	}
	for (; k < k1; k += 2) {  // the last pairs; an odd K leaves half a pair
		const bool in = k + h < k1;
		const float av = in ? a[0] : 0.0f;
#pragma unroll
		for (int q = 0; q < QN; q++) {
			const float bv = in && ni0 + q < nblocks ? b[q * 32] : 0.0f;
			acc[q] = __builtin_amdgcn_mfma_f32_32x32x2f32(av, bv, acc[q], 0, 0, 0);
			if (sum_columns) bsum[q] += bv;
		}
		a += (size_t)2 * g.lda;
		b += (size_t)2 * g.ldb;
	}
	float* out = partial + (size_t)slab * g.c_slice_stride;
#pragma unroll
	for (int q = 0; q < QN; q++) {
		if (ni0 + q < nblocks) {
#pragma unroll
			for (int e = 0; e < 16; e++) out[(size_t)(mi * 32 + 8 * (e >> 2) + 4 * h + (e & 3)) * g.N + (ni0 + q) * 32 + x] = acc[q][e];
		}
	}
	if (sum_columns) {
		// lanes x and x + 32 hold the even and the odd k of the same column
#pragma unroll
		for (int q = 0; q < QN; q++) {
			const float total = bsum[q] + __shfl_xor(bsum[q], 32, 64);
			if (h == 0 && ni0 + q < nblocks) colsum[(size_t)slab * g.colsum_stride + (ni0 + q) * 32 + x] = total;
		}
	}
}

// The same product for M a multiple of 64 and N a multiple of 128, with WIDE loads: a lane reads two consecutive m of a
// row of A (8 bytes) and four consecutive n of a row of B (16 bytes), so one load of each feeds eight matrix
// instructions instead of five narrow loads feeding four, and no element is read by two waves of a group. Component jm
// of the A load and jn of the B load meet in accumulator block (jm, jn), whose row i is m = m0 + 2 i + jm and whose column
// x is n = n0 + 4 x + jn: the interleaving is undone on the way out, where the four jn of a lane are four neighbouring
// columns, i.e. one 16-byte store. A wave owns a slab of k, 64 rows and 128 columns of C; `slots` = (M / 64) * (N / 128)
// waves cover C, the four waves of a group take the slots and, when there are fewer than four, different slabs.
// One wave per SIMD is enough: the operands of the next sixteen k are fetched before this trip's 64 matrix instructions.
template <bool COLSUM>
__global__ __launch_bounds__(256) void sgemm_tn_wide_kernel(GemmArgs g, int k_per_slab, int slots, int n_slots, float* partial, float* colsum) {
	const int lane = threadIdx.x & 63;
	const int wave = threadIdx.x >> 6;
	const int x = lane & 31, h = lane >> 5;
	const int slot = wave % slots;
	const int m0 = (slot / n_slots) * 64, n0 = (slot % n_slots) * 128;
	const int slab = blockIdx.x * (4 / slots) + wave / slots;
	const int k0 = slab * k_per_slab;
	if (k0 >= g.K) return;
	const int k1 = k0 + k_per_slab < g.K ? k0 + k_per_slab : g.K;
	const float* a = g.A + (size_t)(k0 + h) * g.lda + m0 + 2 * x;
	const float* b = g.B + (size_t)(k0 + h) * g.ldb + n0 + 4 * x;
	floatx16 acc[2][4];
#pragma unroll
	for (int jm = 0; jm < 2; jm++)
#pragma unroll
		for (int jn = 0; jn < 4; jn++)
#pragma unroll
			for (int e = 0; e < 16; e++) acc[jm][jn][e] = 0.0f;
	float4 bsum = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
	const bool sum_columns = COLSUM && m0 == 0;
	constexpr int kPairs = 8;
	float2 av0[kPairs], av1[kPairs];
	float4 bv0[kPairs], bv1[kPairs];
	auto fetch = [&](float2 (&av)[kPairs], float4 (&bv)[kPairs]) {
#pragma unroll
		for (int u = 0; u < kPairs; u++) {
			av[u] = *reinterpret_cast<const float2*>(a + (size_t)(2 * u) * g.lda);
			bv[u] = *reinterpret_cast<const float4*>(b + (size_t)(2 * u) * g.ldb);
		}
		a += (size_t)(2 * kPairs) * g.lda;
		b += (size_t)(2 * kPairs) * g.ldb;
	};
	auto multiply_pair = [&](const float2& av, const float4& bv) {
		const float am[2] = {av.x, av.y}, bn[4] = {bv.x, bv.y, bv.z, bv.w};
#pragma unroll
		for (int jm = 0; jm < 2; jm++)
#pragma unroll
			for (int jn = 0; jn < 4; jn++) acc[jm][jn] = __builtin_amdgcn_mfma_f32_32x32x2f32(am[jm], bn[jn], acc[jm][jn], 0, 0, 0);
		if (sum_columns) {
			bsum.x += bv.x;
			bsum.y += bv.y;
			bsum.z += bv.z;
			bsum.w += bv.w;
		}
	};
	auto multiply = [&](const float2 (&av)[kPairs], const float4 (&bv)[kPairs]) {
#pragma unroll
		for (int u = 0; u < kPairs; u++) multiply_pair(av[u], bv[u]);
	};
	const int trips = (k1 - k0) / (2 * kPairs);
	// The loop's body has no branch: a load behind a condition makes the compiler wait as if it had not been issued, i.e.
	// for every load, the early ones included. The scheduler is kept from sinking the early loads down to their uses.
	if (trips > 0) {
		fetch(av0, bv0);
		int fetched = 1;
		for (; fetched + 1 < trips; fetched += 2) {
			__builtin_amdgcn_sched_barrier(0);
			fetch(av1, bv1);
			__builtin_amdgcn_sched_barrier(0);
			multiply(av0, bv0);
			__builtin_amdgcn_sched_barrier(0);
			fetch(av0, bv0);
			__builtin_amdgcn_sched_barrier(0);
			multiply(av1, bv1);
		}
		__builtin_amdgcn_sched_barrier(0);
		if (fetched < trips) {
			fetch(av1, bv1);
			__builtin_amdgcn_sched_barrier(0);
			multiply(av0, bv0);
			multiply(av1, bv1);
		} else {
			multiply(av0, bv0);
		}
	}
	for (int k = k0 + trips * 2 * kPairs; k < k1; k += 2) {  // the last pairs; an odd K leaves half a pair
		const bool in = k + h < k1;
		const float2 av = in ? *reinterpret_cast<const float2*>(a) : make_float2(0.0f, 0.0f);
		const float4 bv = in ? *reinterpret_cast<const float4*>(b) : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
		multiply_pair(av, bv);
		a += (size_t)2 * g.lda;
		b += (size_t)2 * g.ldb;
	}
	float* out = partial + (size_t)slab * g.c_slice_stride;
#pragma unroll
	for (int jm = 0; jm < 2; jm++)
#pragma unroll
		for (int e = 0; e < 16; e++) {
			const int i = 8 * (e >> 2) + 4 * h + (e & 3);
			*reinterpret_cast<float4*>(out + (size_t)(m0 + 2 * i + jm) * g.N + n0 + 4 * x) = make_float4(acc[jm][0][e], acc[jm][1][e], acc[jm][2][e], acc[jm][3][e]);
		}
	if (sum_columns) {
		// lanes x and x + 32 hold the even and the odd k of the same four columns
		bsum.x += __shfl_xor(bsum.x, 32, 64);
		bsum.y += __shfl_xor(bsum.y, 32, 64);
		bsum.z += __shfl_xor(bsum.z, 32, 64);
		bsum.w += __shfl_xor(bsum.w, 32, 64);
		if (h == 0) *reinterpret_cast<float4*>(colsum + (size_t)slab * g.colsum_stride + n0 + 4 * x) = bsum;
	}
}

// Returns 1 when the shape does not fit (the caller goes on).
static int sgemm_tn_direct(GemmArgs g, float* C, float* colsum = nullptr) {
	State& s = state();
	const size_t M = g.M, N = g.N, K = g.K;
	if ((M & 31) || (N & 31) || M > 128 || M * N > 16384 || K < 4096) return 1;
	const int mblocks = (int)(M / 32), nblocks = (int)(N / 32);
	// wide loads: 64 x 128 of C per wave, operands and result addressable as 8- and 16-byte vectors
	const size_t wide_slots = (M / 64) * (N / 128);
	const bool wide = (M % 64) == 0 && (N % 128) == 0 && (wide_slots == 1 || wide_slots == 2 || wide_slots == 4) && (g.lda & 1) == 0 && (g.ldb & 3) == 0 &&
	                  (reinterpret_cast<uintptr_t>(g.A) & 7) == 0 && (reinterpret_cast<uintptr_t>(g.B) & 15) == 0 && (reinterpret_cast<uintptr_t>(C) & 15) == 0 &&
	                  (!colsum || (reinterpret_cast<uintptr_t>(colsum) & 15) == 0);
	if (!wide && mblocks == 3) return 1;
	const int waves_per_m = wide ? 1 : 4 / mblocks;
	const int qn = wide ? 4 : (nblocks + waves_per_m - 1) / waves_per_m;
	if (qn > 4) return 1;
	const int ngroups = (nblocks + qn - 1) / qn;  // wave slots along n
	const int slots = wide ? (int)wide_slots : mblocks * ngroups;  // 1, 2 or 4 (three would leave a wave without work: tiled kernel)
	if (slots == 3) return 1;
	const int slabs_per_group = 4 / slots;
	// sixteen waves per compute unit, at least 256 k per slab
	size_t slabs = (size_t)s.compute_units * 4 * slabs_per_group;
	// the partial results are written and read once more: keep them near a quarter of the operands' bytes, but never
	// fewer than eight waves per compute unit (the loads are narrow: occupancy hides their latency)
	size_t by_traffic = K * (M + N) / (8 * M * N);
	if (by_traffic < (size_t)s.compute_units * 2) by_traffic = (size_t)s.compute_units * 2;
	if (slabs > by_traffic) slabs = by_traffic;
	{  // whole rounds of groups over the compute units: no half-empty last round
		const size_t per_round = (size_t)s.compute_units * slabs_per_group;
		if (slabs > per_round) slabs = slabs / per_round * per_round;
	}
	if (slabs > K / 256) slabs = K / 256;
	if (slabs < 1) slabs = 1;
	size_t k_per_slab = ((K + slabs - 1) / slabs + 7) & ~size_t(7);
	slabs = (K + k_per_slab - 1) / k_per_slab;
	SlicePlan plan;
	{
		const int rc = plan_slices(slabs, M * N, colsum ? N : 0, C, colsum, plan);
		if (rc) return rc;
	}
	g.c_slice_stride = plan.stride;
	g.colsum_stride = plan.colsum_stride;
	float* partial = plan.partial;
	float* colsum_partial = plan.colsum_partial;
	const dim3 grid((unsigned)((slabs + slabs_per_group - 1) / slabs_per_group)), block(256);
	if (wide) {
		// the slices' addresses must allow the 16-byte stores: merged slices keep every stride a multiple of four floats
		if (colsum)
			hipLaunchKernelGGL(sgemm_tn_wide_kernel<true>, grid, block, 0, s.stream, g, (int)k_per_slab, slots, (int)(N / 128), partial, colsum_partial);
		else
			hipLaunchKernelGGL(sgemm_tn_wide_kernel<false>, grid, block, 0, s.stream, g, (int)k_per_slab, slots, (int)(N / 128), partial, (float*)nullptr);
		TFHIP_CHECK_LAUNCH();
		return sum_slices(plan, slabs, C, M * N, colsum, colsum ? N : 0);
	}
#define TFHIP_TN_DIRECT(QN)                                                                                                                                        \
	if (colsum)                                                                                                                                                    \
		hipLaunchKernelGGL((sgemm_tn_direct_kernel<QN, true>), grid, block, 0, s.stream, g, (int)k_per_slab, ngroups, slots, nblocks, partial, colsum_partial);    \
	else                                                                                                                                                           \
		hipLaunchKernelGGL((sgemm_tn_direct_kernel<QN, false>), grid, block, 0, s.stream, g, (int)k_per_slab, ngroups, slots, nblocks, partial, (float*)nullptr)
	switch (qn) {
		case 1: TFHIP_TN_DIRECT(1); break;
		case 2: TFHIP_TN_DIRECT(2); break;
		case 3: TFHIP_TN_DIRECT(3); break;
		default: TFHIP_TN_DIRECT(4); break;
	}
#undef TFHIP_TN_DIRECT
	TFHIP_CHECK_LAUNCH();
	return sum_slices(plan, slabs, C, M * N, colsum, colsum ? N : 0);
}

// The fused tail applied in place to a small C (products that were computed through a transposed formulation).
__global__ __launch_bounds__(256) void sgemm_tail_kernel(GemmArgs g) {
	const size_t e = (size_t)blockIdx.x * 256 + threadIdx.x;
	if (e >= (size_t)g.M * g.N) return;
	const size_t row = e / g.N;
	const int col = (int)(e - row * g.N);
	g.C[row * g.ldc + col] = apply_epilogue(g, row, col, g.C[row * g.ldc + col]);
}

// Few rows (M <= 8) against a wide B, posed as the transposed skinny problem: B is streamed once. Returns TFHIP_OK when handled, 1 when the shape does not fit (the caller goes on).
static int sgemm_few_rows(int layout, const GemmArgs& full) {
	State& s = state();
	const size_t M = full.M, N = full.N;
	const bool b_vec = (reinterpret_cast<uintptr_t>(full.B) & 15) == 0;
	if (layout != kNT && !((N & 3) == 0 && b_vec)) return 1;  // the wide operand is read as 16-byte vectors along N
	for (size_t m0 = 0; m0 < M; m0 += kSkinnyN) {
		const int mc = (int)(M - m0 < (size_t)kSkinnyN ? M - m0 : kSkinnyN);
		GemmArgs g = full;
		g.epilogue = TFHIP_EPILOGUE_NONE;
		g.aux = nullptr;
		g.k_slices = 1;
		int rc;
		if (layout == kNT) {
			// C[m, n] = sum_k A[m, k] B[n, k]: the rows of B against mc rows of A; result element (n, m') goes to C[m0 + m', n]
			g.A = full.B;
			g.lda = full.ldb;
			g.B = full.A + m0 * full.lda;
			g.ldb = full.lda;
			g.M = (int)N;
			g.N = mc;
			g.C = full.C + m0 * full.ldc;
			rc = sgemm_rows_wave<kNT>(g, 1, full.ldc);
		} else {
			// C[m, n] = sum_k A(m, k) B[k, n]: B plays the tall operand [K, N] of the tn kernel, the mc rows of A its few columns
			g.A = full.B;
			g.lda = full.ldb;
			g.B = layout == kNN ? full.A + m0 * full.lda : full.A + m0;
			g.M = (int)N;
			g.N = mc;
			rc = sgemm_skinny_tn(g, full.C + m0 * full.ldc, layout == kNN ? 1 : full.lda, layout == kNN ? full.lda : 1, 1, full.ldc);
		}
		if (rc != TFHIP_OK) return rc;
	}
	if (full.epilogue != TFHIP_EPILOGUE_NONE) {
		hipLaunchKernelGGL(sgemm_tail_kernel, dim3((unsigned)((M * N + 255) / 256)), dim3(256), 0, s.stream, full);
		TFHIP_CHECK_LAUNCH();
	}
	return TFHIP_OK;
}

static int sgemm_impl(int layout, const float* A, const float* B, float* C, size_t M, size_t N, size_t K, int epilogue = TFHIP_EPILOGUE_NONE,
                      const float* aux = nullptr, size_t batch = 1, size_t batch_a = 0, size_t batch_b = 0, size_t batch_c = 0, float* colsum = nullptr) {
	State& s = state();
	if (!A || !B || !C) return fail(TFHIP_ERR_ARG, "null pointer passed to sgemm");

	if (epilogue < TFHIP_EPILOGUE_NONE || epilogue > TFHIP_EPILOGUE_MASK_POSITIVE) return fail(TFHIP_ERR_ARG, "unknown sgemm epilogue %d", epilogue);
	if (epilogue != TFHIP_EPILOGUE_NONE && !aux) return fail(TFHIP_ERR_ARG, "sgemm epilogue %d needs its bias / mask operand", epilogue);
	if (M == 0 || N == 0) return fail(TFHIP_ERR_ARG, "sgemm with an empty result (%zu x %zu)", M, N);
	if (M > 0x7FFFFFFF || N > 0x7FFFFFFF || K > 0x7FFFFFFF) return fail(TFHIP_ERR_ARG, "sgemm dimension beyond 2^31");
	GemmArgs g;
	g.A = A;
	g.B = B;
	g.C = C;
	g.M = (int)M;
	g.N = (int)N;
	g.K = (int)K;
	g.lda = layout == kTN ? (int)M : (int)K;
	g.ldb = layout == kNT ? (int)K : (int)N;
	g.ldc = (int)N;
	g.k_slices = 1;
	g.k_per_slice = (int)((K + kBK - 1) / kBK * kBK);
	g.c_slice_stride = 0;
	g.epilogue = epilogue;
	g.aux = aux;
	if (colsum) {
		// The column sums of B ride in the tiled tn kernel (128-row tiles of C, so that a tile row exists whose groups
		// see all of B), in the direct kernel for narrow results and in the kernel for at most eight columns; every other
		// shape takes its own best kernel for the product and a column reduction beside it.
		const bool plain_tn = layout == kTN && epilogue == TFHIP_EPILOGUE_NONE && batch == 1 && K >= 1;
		// The direct kernels come first, exactly as for the plain product below: C must come out bit-identical to
		// tfhip_sgemm_tn's whether or not the column sums ride along, so both calls have to pick the same kernel.
		if (plain_tn && N > (size_t)kSkinnyN) {
			const int rc = sgemm_tn_direct(g, C, colsum);
			if (rc != 1) return rc;
		}
		const bool rides = plain_tn && M >= (size_t)kBM && N >= 32;
		if (!rides) {
			// the same test that sends the plain product to the kernel for few columns
			if (plain_tn && N <= (size_t)kSkinnyN && K >= 16 && (M & 3) == 0 && (reinterpret_cast<uintptr_t>(A) & 15) == 0)
				return sgemm_skinny_tn(g, C, -1, 1, -1, 1, colsum);
			const int rc = sgemm_impl(layout, A, B, C, M, N, K, epilogue, aux, batch, batch_a, batch_b, batch_c, nullptr);
			if (rc) return rc;
			if (K == 0) return tfhip_fill_u32(colsum, 0u, N);
			return tfhip_reduce_cols_f32(TFHIP_REDUCE_SUM, B, colsum, K, N);
		}
	}
	if (K == 0 && epilogue == TFHIP_EPILOGUE_NONE && batch == 1) return tfhip_fill_u32(C, 0u, M * N);
	if (batch > 1) {
		// One launch for the whole batch (grid.y): the tiled kernel when the matrices are large enough, else a thread
		// per element. The single-product special cases (skinny shapes, K slices) are not batched.
		if (batch > 65535) return fail(TFHIP_ERR_ARG, "more than 65535 products in one batch (%zu)", batch);
		g.batch_a = batch_a;
		g.batch_b = batch_b;
		g.batch_c = batch_c;
		const bool mfma = M >= 32 && N >= 32;
		const size_t groups = mfma ? ((M + kBM - 1) / kBM) * ((N + kBN - 1) / kBN) : (M * N + 255) / 256;
		if (groups > 0x7FFFFFFFull) return fail(TFHIP_ERR_ARG, "sgemm result too large");
		const dim3 grid((unsigned)groups, (unsigned)batch, 1);
		if (mfma) {
			switch (layout) {
				case kNN: hipLaunchKernelGGL(sgemm_mfma_kernel<kNN>, grid, dim3(256), 0, s.stream, g); break;
				case kNT: hipLaunchKernelGGL(sgemm_mfma_kernel<kNT>, grid, dim3(256), 0, s.stream, g); break;
				default: hipLaunchKernelGGL(sgemm_mfma_kernel<kTN>, grid, dim3(256), 0, s.stream, g); break;
			}
		} else {
			switch (layout) {
				case kNN: hipLaunchKernelGGL(sgemm_plain_kernel<kNN>, grid, dim3(256), 0, s.stream, g); break;
				case kNT: hipLaunchKernelGGL(sgemm_plain_kernel<kNT>, grid, dim3(256), 0, s.stream, g); break;
				default: hipLaunchKernelGGL(sgemm_plain_kernel<kTN>, grid, dim3(256), 0, s.stream, g); break;
			}
		}
		TFHIP_CHECK_LAUNCH();
		return TFHIP_OK;
	}

	if (M <= (size_t)kSkinnyN && N > (size_t)kSkinnyN && K >= 16 && M * N <= 0x7FFFFFFFull) {
		const int rc = sgemm_few_rows(layout, g);
		if (rc != 1) return rc;
	}
	if (N <= (size_t)kSkinnyN && K >= 16) {
		if (layout == kTN) {
			// partial products of k-slabs are summed afterwards: no place for an epilogue
			if (epilogue == TFHIP_EPILOGUE_NONE && (M & 3) == 0 && (reinterpret_cast<uintptr_t>(A) & 15) == 0) return sgemm_skinny_tn(g, C);
		} else {
			const size_t groups = (M + kSkinnyRows - 1) / kSkinnyRows;
			// 64-row groups fill the chip only when there are many rows; a long K is better walked by whole waves
			if (K >= 1024 || groups < (size_t)s.compute_units * 4) return layout == kNN ? sgemm_rows_wave<kNN>(g) : sgemm_rows_wave<kNT>(g);
			// a row of A is one 16-byte load per lane of a wave: no detour through group memory
			if (K <= 256 && (K & 3) == 0 && (g.lda & 3) == 0 && (reinterpret_cast<uintptr_t>(A) & 15) == 0 && M <= 0x7FFFFFFFull) {
				if (layout == kNN)
					launch_rows_lanes<kNN>(g, s.stream, s.compute_units);
				else
					launch_rows_lanes<kNT>(g, s.stream, s.compute_units);
				TFHIP_CHECK_LAUNCH();
				return TFHIP_OK;
			}
			if (groups <= 0x7FFFFFFFull) {
				if (layout == kNN)
					launch_skinny_rows<kNN>(g, (unsigned)groups, s.stream);
				else
					launch_skinny_rows<kNT>(g, (unsigned)groups, s.stream);
				TFHIP_CHECK_LAUNCH();
				return TFHIP_OK;
			}
		}
	}

	// Nine to 31 rows still take the matrix-core tiles (mostly padding, but B is streamed once and K is sliced below).
	// Short K, narrow C (at most 64 columns, where the 128-wide tiles would be half empty), many rows: B stays in group
	// memory and A is streamed (nn and nt: A is [M, K] row-major in both, its rows read as 16-byte vectors).
	if ((layout == kNN || layout == kNT) && K >= 16 && K <= 128 && (K & 7) == 0 && N >= 32 && N <= 64 && M >= (size_t)s.compute_units * 128 && (g.lda & 3) == 0 &&
	    (reinterpret_cast<uintptr_t>(A) & 15) == 0) {
		const int nb = N > 32 ? 2 : 1;
		const size_t col_groups = (N + nb * 32 - 1) / (nb * 32);
		const size_t row_groups = (M + 127) / 128;
		if (row_groups <= 0x7FFFFFFFull && col_groups <= 65535) {
			// as many groups as stay resident (the block of B is loaded once per group), each walking row groups
			size_t groups_x = (size_t)s.compute_units * 4 / col_groups;
			if (groups_x < (size_t)s.compute_units) groups_x = (size_t)s.compute_units;
			if (groups_x > row_groups) groups_x = row_groups;
			const dim3 grid((unsigned)groups_x, (unsigned)col_groups), block(256);
			const size_t lds = (K * (nb * 32 + 1) + 4 * 32 * 36) * sizeof(float);  // the block of B, then a 32 x 36 corner per wave for the write-out
			if (layout == kNN) {
				if (nb == 2) hipLaunchKernelGGL((sgemm_short_k_kernel<2, false>), grid, block, lds, s.stream, g, (unsigned)row_groups);
				else hipLaunchKernelGGL((sgemm_short_k_kernel<1, false>), grid, block, lds, s.stream, g, (unsigned)row_groups);
			} else {
				if (nb == 2) hipLaunchKernelGGL((sgemm_short_k_kernel<2, true>), grid, block, lds, s.stream, g, (unsigned)row_groups);
				else hipLaunchKernelGGL((sgemm_short_k_kernel<1, true>), grid, block, lds, s.stream, g, (unsigned)row_groups);
			}
			TFHIP_CHECK_LAUNCH();
			return TFHIP_OK;
		}
	}
	if (layout == kTN && epilogue == TFHIP_EPILOGUE_NONE && N > (size_t)kSkinnyN && !colsum) {
		const int rc = sgemm_tn_direct(g, C);
		if (rc != 1) return rc;
	}
	const bool use_mfma = (M >= 32 || (M > (size_t)kSkinnyN && N >= 128)) && N >= 32;
	const size_t tiles = use_mfma ? ((M + kBM - 1) / kBM) * ((N + kBN - 1) / kBN) : (M * N + 255) / 256;
	if (tiles > 0x7FFFFFFFull) return fail(TFHIP_ERR_ARG, "sgemm result too large");

	// Few tiles and a long K: slice K so that the chip is full; partial products go to scratch and are summed.
	// two groups per compute unit ([262144,256]^T [262144,256] with its column sums: 277 us; three or four: 273-274; six
	// and eight: 290, the partial products grow)
	const size_t want = (size_t)s.compute_units * 2;
	if (tiles < want && K >= 512 && epilogue == TFHIP_EPILOGUE_NONE) {
		size_t slices = (want + tiles - 1) / tiles;
		size_t max_slices = K / 256;
		if (slices > max_slices) slices = max_slices;
		if (slices > 1024) slices = 1024;
		if (slices > 1) {
			size_t per = (K + slices - 1) / slices;
			per = (per + kBK - 1) / kBK * kBK;
			slices = (K + per - 1) / per;
			g.k_slices = (int)slices;
			g.k_per_slice = (int)per;
			g.c_slice_stride = M * N;
		}
	}
	SlicePlan plan;
	g.colsum = colsum;
	if (g.k_slices > 1) {
		const int rc = plan_slices((size_t)g.k_slices, M * N, colsum ? N : 0, C, colsum, plan);
		if (rc) return rc;
		g.C = plan.partial;
		g.c_slice_stride = plan.stride;
		if (colsum) {
			g.colsum = plan.colsum_partial;
			g.colsum_stride = plan.colsum_stride;
		}
	}
	dim3 grid((unsigned)tiles, 1, (unsigned)g.k_slices);
	if (colsum) {
		hipLaunchKernelGGL((sgemm_mfma_kernel<kTN, true>), grid, dim3(256), 0, s.stream, g);
	} else if (use_mfma) {
		switch (layout) {
			case kNN: hipLaunchKernelGGL(sgemm_mfma_kernel<kNN>, grid, dim3(256), 0, s.stream, g); break;
			case kNT: hipLaunchKernelGGL(sgemm_mfma_kernel<kNT>, grid, dim3(256), 0, s.stream, g); break;
			default: hipLaunchKernelGGL(sgemm_mfma_kernel<kTN>, grid, dim3(256), 0, s.stream, g); break;
		}
	} else {
		switch (layout) {
			case kNN: hipLaunchKernelGGL(sgemm_plain_kernel<kNN>, grid, dim3(256), 0, s.stream, g); break;
			case kNT: hipLaunchKernelGGL(sgemm_plain_kernel<kNT>, grid, dim3(256), 0, s.stream, g); break;
			default: hipLaunchKernelGGL(sgemm_plain_kernel<kTN>, grid, dim3(256), 0, s.stream, g); break;
		}
	}
	TFHIP_CHECK_LAUNCH();
	if (g.k_slices > 1) return sum_slices(plan, (size_t)g.k_slices, C, M * N, colsum, colsum ? N : 0);
	return TFHIP_OK;
}

}  // namespace tfhip

using namespace tfhip;

extern "C" {

int tfhip_sgemm_nn(const float* A, const float* B, float* C, size_t M, size_t N, size_t K) {
	TFHIP_REQUIRE_INIT();
	return sgemm_impl(kNN, A, B, C, M, N, K);
}
int tfhip_sgemm_nt(const float* A, const float* B, float* C, size_t M, size_t N, size_t K) {
	TFHIP_REQUIRE_INIT();
	return sgemm_impl(kNT, A, B, C, M, N, K);
}
int tfhip_sgemm_tn(const float* A, const float* B, float* C, size_t M, size_t N, size_t K) {
	TFHIP_REQUIRE_INIT();
	return sgemm_impl(kTN, A, B, C, M, N, K);
}
int tfhip_sgemm_tn_colsum(const float* A, const float* B, float* C, float* colsum_b, size_t M, size_t N, size_t K) {
	TFHIP_REQUIRE_INIT();
	if (!colsum_b) return fail(TFHIP_ERR_ARG, "null pointer passed to tfhip_sgemm_tn_colsum");
	return sgemm_impl(kTN, A, B, C, M, N, K, TFHIP_EPILOGUE_NONE, nullptr, 1, 0, 0, 0, colsum_b);
}
int tfhip_sgemm_batched(int layout, const float* A, const float* B, float* C, size_t M, size_t N, size_t K, size_t batch, size_t stride_a, size_t stride_b,
                        size_t stride_c) {
	TFHIP_REQUIRE_INIT();
	if (layout != TFHIP_GEMM_NN && layout != TFHIP_GEMM_NT && layout != TFHIP_GEMM_TN) return fail(TFHIP_ERR_ARG, "unknown sgemm layout %d", layout);
	if (batch == 0) return fail(TFHIP_ERR_ARG, "sgemm over an empty batch");
	if (batch > 1 && stride_c < M * N) return fail(TFHIP_ERR_ARG, "the results of a batch overlap (stride %zu for %zu x %zu)", stride_c, M, N);
	return sgemm_impl(layout, A, B, C, M, N, K, TFHIP_EPILOGUE_NONE, nullptr, batch, stride_a, stride_b, stride_c);
}

int tfhip_sgemm_fused(int layout, const float* A, const float* B, float* C, size_t M, size_t N, size_t K, int epilogue, const float* aux) {
	TFHIP_REQUIRE_INIT();
	if (layout != TFHIP_GEMM_NN && layout != TFHIP_GEMM_NT && layout != TFHIP_GEMM_TN) return fail(TFHIP_ERR_ARG, "unknown sgemm layout %d", layout);
	return sgemm_impl(layout, A, B, C, M, N, K, epilogue, aux);
}

}  // extern "C"
