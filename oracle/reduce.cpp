// TEST INFRASTRUCTURE -- not part of the product (see prelude.h).
//
// Reductions and softmax as the reference's C++/OpenMP backend executes them: one logical thread per
// OUTPUT element running a serial accumulation loop, threads grouped 256 (1-D) or 16x16 (2-D), groups
// spread over cores with `omp parallel for`, threads of a group run one after the other.
// Follows:
//   TensorFrost/Compiler/Implementations.cpp:243-303   acc = init; for k: acc = op(acc, load(...k...))
//   TensorFrost/Compiler/Implementations.cpp:374-426   initial values (0, -FLT_MAX, FLT_MAX)
//   TensorFrost/Compiler/Steps/Optimization.cpp:469-510 constant axis >= 1024: split into chunks of 128,
//                                                       reduce the chunk axis, then reduce the partials
//   TensorFrost/Compiler/Implementations.cpp:507-527,56-69 split index = outer*128 + inner, out-of-range -> 0
//   TensorFrost/Compiler/Steps/GraphOps.cpp:1091-1186   block_id -> (index_0 innermost, index_1, ...), bounds `if`
//   TensorFrost/Backend/CodeGen/Langs/CPP.cpp:720-779   kernel wrapper
// Softmax is the user-level composition exp(x - max) / sum(exp(x - max)) (tests/autograd_test.py:29-31).
//
// Pins (tests/test_oracle.py): every function here against float64 NumPy (sum/max/min/softmax closed
// forms) on shapes that exercise the split (axis >= 1024, multiple and non-multiple of 128) and
// unsplit paths, both axes; a dropped chunk, a transposed index or a wrong init fails those.
// The exact fp32 summation ORDER of the OpenMP build under -ffast-math is compiler-dependent and is
// not pinned by anything (parity on sums is to 1e-4 relative, not bitwise).

#include <cfloat>

#include "prelude.h"

using namespace tfo;

namespace {

constexpr int kSplit = 128;      // SPLIT_DIM_SIZE
constexpr int kMinSplit = 1024;  // MIN_SPLIT_SIZE

enum Op { kSum = 0, kMax = 1, kMin = 2 };

template <int OP>
inline float op_init() {
	return OP == kSum ? 0.0f : (OP == kMax ? -FLT_MAX : FLT_MAX);
}
template <int OP>
inline float op_apply(float a, float b) {
	return OP == kSum ? a + b : (OP == kMax ? max(a, b) : min(a, b));
}

// Optional element-wise producer fused into the loop by load fusion: exp(x - m[row]).
struct NoFuse {
	inline float operator()(float v, int) const { return v; }
};
struct ExpMinusRowMax {
	const uint* m_mem;
	inline float operator()(float v, int row) const { return expf(v - asfloat(m_mem[row])); }
};

// ---- last-axis reduction, unsplit: kernel shape [R], group {256} ---------------------------------
template <int OP, class Fuse>
void k_reduce_last(const uint* var, uint** mem, uint work_group_count, Fuse fuse) {
	uint* out_mem = mem[0];
	uint* x_mem = mem[1];
	int var_R = asint(var[0]);
	int var_K = asint(var[1]);
	uint var__kernel_block_offset = asuint(var[2]);
#pragma omp parallel for
	for (int block_id = var__kernel_block_offset; block_id < (int)(work_group_count + var__kernel_block_offset); block_id++) {
		for (int block_thread_id0 = 0; block_thread_id0 < 256; block_thread_id0++) {
			int index_0 = (block_id * 256) + block_thread_id0;
			bool is_inside_dispatch = index_0 < var_R;
			if (is_inside_dispatch) {
				float acc = op_init<OP>();
				for (int vloop = 0; vloop < var_K; vloop += 1) {
					float x = asfloat(x_mem[(index_0 * var_K) + vloop]);
					acc = op_apply<OP>(acc, fuse(x, index_0));
				}
				out_mem[index_0] = asuint(acc);
			}
		}
	}
}

// ---- last-axis reduction, stage 1 of the split: kernel shape [R, S], group {16,16} ----------------
// partial[r, s] = reduce_{k<128} (s*128+k < K ? x[r, s*128+k] : 0)
template <int OP, class Fuse>
void k_reduce_last_stage1(const uint* var, uint** mem, uint work_group_count, Fuse fuse) {
	uint* partial_mem = mem[0];
	uint* x_mem = mem[1];
	int var_R = asint(var[0]);
	int var_K = asint(var[1]);
	int var_S = asint(var[2]);
	uint var__kernel_block_offset = asuint(var[3]);
#pragma omp parallel for
	for (int block_id = var__kernel_block_offset; block_id < (int)(work_group_count + var__kernel_block_offset); block_id++) {
		for (int block_thread_id1 = 0; block_thread_id1 < 16; block_thread_id1++)
			for (int block_thread_id0 = 0; block_thread_id0 < 16; block_thread_id0++) {
				int blocks_shape_0 = ((var_S + 16) - 1) / 16;
				int vdiv = block_id / blocks_shape_0;
				int index_0 = ((block_id - (vdiv * blocks_shape_0)) * 16) + block_thread_id0;
				int index_1 = (vdiv * 16) + block_thread_id1;
				bool is_inside_dispatch = (index_0 < var_S) && (index_1 < var_R);
				if (is_inside_dispatch) {
					float acc = op_init<OP>();
					for (int vloop = 0; vloop < kSplit; vloop += 1) {
						int merged = (index_0 * kSplit) + vloop;
						bool out_of_bounds = (merged < 0) || (merged >= var_K);
						float x = asfloat(x_mem[(clamp(index_1, 0, var_R - 1) * var_K) + clamp(merged, 0, var_K - 1)]);
						float split = out_of_bounds ? 0.0f : fuse(x, index_1);
						acc = op_apply<OP>(acc, split);
					}
					partial_mem[(index_1 * var_S) + index_0] = asuint(acc);
				}
			}
	}
}

// ---- axis-0 reduction, unsplit: kernel shape [C], group {256}; x is [K, C] ------------------------
template <int OP>
void k_reduce_first(const uint* var, uint** mem, uint work_group_count) {
	uint* out_mem = mem[0];
	uint* x_mem = mem[1];
	int var_K = asint(var[0]);
	int var_C = asint(var[1]);
	uint var__kernel_block_offset = asuint(var[2]);
#pragma omp parallel for
	for (int block_id = var__kernel_block_offset; block_id < (int)(work_group_count + var__kernel_block_offset); block_id++) {
		for (int block_thread_id0 = 0; block_thread_id0 < 256; block_thread_id0++) {
			int index_0 = (block_id * 256) + block_thread_id0;
			bool is_inside_dispatch = index_0 < var_C;
			if (is_inside_dispatch) {
				float acc = op_init<OP>();
				for (int vloop = 0; vloop < var_K; vloop += 1) {
					float x = asfloat(x_mem[(vloop * var_C) + index_0]);
					acc = op_apply<OP>(acc, x);
				}
				out_mem[index_0] = asuint(acc);
			}
		}
	}
}

// ---- axis-0 reduction, stage 1 of the split: kernel shape [S, C], group {16,16} -------------------
// partial[s, c] = reduce_{k<128} (s*128+k < K ? x[s*128+k, c] : 0)
template <int OP>
void k_reduce_first_stage1(const uint* var, uint** mem, uint work_group_count) {
	uint* partial_mem = mem[0];
	uint* x_mem = mem[1];
	int var_K = asint(var[0]);
	int var_C = asint(var[1]);
	int var_S = asint(var[2]);
	uint var__kernel_block_offset = asuint(var[3]);
#pragma omp parallel for
	for (int block_id = var__kernel_block_offset; block_id < (int)(work_group_count + var__kernel_block_offset); block_id++) {
		for (int block_thread_id1 = 0; block_thread_id1 < 16; block_thread_id1++)
			for (int block_thread_id0 = 0; block_thread_id0 < 16; block_thread_id0++) {
				int blocks_shape_0 = ((var_C + 16) - 1) / 16;
				int vdiv = block_id / blocks_shape_0;
				int index_0 = ((block_id - (vdiv * blocks_shape_0)) * 16) + block_thread_id0;  // column
				int index_1 = (vdiv * 16) + block_thread_id1;                                    // chunk
				bool is_inside_dispatch = (index_0 < var_C) && (index_1 < var_S);
				if (is_inside_dispatch) {
					float acc = op_init<OP>();
					for (int vloop = 0; vloop < kSplit; vloop += 1) {
						int merged = (index_1 * kSplit) + vloop;
						bool out_of_bounds = (merged < 0) || (merged >= var_K);
						float x = asfloat(x_mem[(clamp(merged, 0, var_K - 1) * var_C) + clamp(index_0, 0, var_C - 1)]);
						float split = out_of_bounds ? 0.0f : x;
						acc = op_apply<OP>(acc, split);
					}
					partial_mem[(index_1 * var_C) + index_0] = asuint(acc);
				}
			}
	}
}

// ---- normalisation: kernel shape [R, C], group {16,16}: y = exp(x - m[r]) / s[r] -------------------
void k_softmax_normalise(const uint* var, uint** mem, uint work_group_count) {
	uint* y_mem = mem[0];
	uint* x_mem = mem[1];
	uint* m_mem = mem[2];
	uint* s_mem = mem[3];
	int var_R = asint(var[0]);
	int var_C = asint(var[1]);
	uint var__kernel_block_offset = asuint(var[2]);
#pragma omp parallel for
	for (int block_id = var__kernel_block_offset; block_id < (int)(work_group_count + var__kernel_block_offset); block_id++) {
		for (int block_thread_id1 = 0; block_thread_id1 < 16; block_thread_id1++)
			for (int block_thread_id0 = 0; block_thread_id0 < 16; block_thread_id0++) {
				int blocks_shape_0 = ((var_C + 16) - 1) / 16;
				int vdiv = block_id / blocks_shape_0;
				int index_0 = ((block_id - (vdiv * blocks_shape_0)) * 16) + block_thread_id0;
				int index_1 = (vdiv * 16) + block_thread_id1;
				bool is_inside_dispatch = (index_0 < var_C) && (index_1 < var_R);
				if (is_inside_dispatch) {
					float x = asfloat(x_mem[(index_1 * var_C) + index_0]);
					float m = asfloat(m_mem[index_1]);
					float s = asfloat(s_mem[index_1]);
					y_mem[(index_1 * var_C) + index_0] = asuint(expf(x - m) / s);
				}
			}
	}
}

inline uint groups_1d(size_t n) {
	size_t shape[1] = {n}, group[1] = {256};
	return (uint)work_group_count(shape, 1, group, 1);
}
inline uint groups_2d(size_t outer, size_t inner) {
	size_t shape[2] = {outer, inner}, group[2] = {16, 16};
	return (uint)work_group_count(shape, 2, group, 2);
}

// Host side of a last-axis reduction as the generated `main` would sequence it.
template <int OP, class Fuse>
void reduce_last(const float* x, float* out, float* partial, int R, int K, Fuse fuse) {
	if (K >= kMinSplit) {
		int S = (K + kSplit - 1) / kSplit;
		{
			uint var[4] = {asuint(R), asuint(K), asuint(S), 0u};
			uint* mem[2] = {(uint*)partial, (uint*)x};
			k_reduce_last_stage1<OP>(var, mem, groups_2d(R, S), fuse);
		}
		{
			uint var[3] = {asuint(R), asuint(S), 0u};
			uint* mem[2] = {(uint*)out, (uint*)partial};
			k_reduce_last<OP>(var, mem, groups_1d(R), NoFuse());
		}
	} else {
		uint var[3] = {asuint(R), asuint(K), 0u};
		uint* mem[2] = {(uint*)out, (uint*)x};
		k_reduce_last<OP>(var, mem, groups_1d(R), fuse);
	}
}

template <int OP>
void reduce_first(const float* x, float* out, float* partial, int K, int C) {
	if (K >= kMinSplit) {
		int S = (K + kSplit - 1) / kSplit;
		{
			uint var[4] = {asuint(K), asuint(C), asuint(S), 0u};
			uint* mem[2] = {(uint*)partial, (uint*)x};
			k_reduce_first_stage1<OP>(var, mem, groups_2d(S, C));
		}
		{
			uint var[3] = {asuint(S), asuint(C), 0u};
			uint* mem[2] = {(uint*)out, (uint*)partial};
			k_reduce_first<OP>(var, mem, groups_1d(C));
		}
	} else {
		uint var[3] = {asuint(K), asuint(C), 0u};
		uint* mem[2] = {(uint*)out, (uint*)x};
		k_reduce_first<OP>(var, mem, groups_1d(C));
	}
}

}  // namespace

extern "C" {

// Words of temporary storage the split needs for an axis of length K with `other` outputs.
size_t oracle_reduce_partial_words(size_t other, size_t K) { return K >= (size_t)kMinSplit ? other * ((K + kSplit - 1) / kSplit) : 1; }

// out[r] = op_c x[r, c]; partial holds oracle_reduce_partial_words(R, C) floats.
int oracle_reduce_rows_f32(int op, const float* x, float* out, float* partial, int R, int C) {
	switch (op) {
		case kSum: reduce_last<kSum>(x, out, partial, R, C, NoFuse()); return 0;
		case kMax: reduce_last<kMax>(x, out, partial, R, C, NoFuse()); return 0;
		case kMin: reduce_last<kMin>(x, out, partial, R, C, NoFuse()); return 0;
	}
	return -1;
}

// out[c] = op_r x[r, c]; partial holds oracle_reduce_partial_words(C, R) floats.
int oracle_reduce_cols_f32(int op, const float* x, float* out, float* partial, int R, int C) {
	switch (op) {
		case kSum: reduce_first<kSum>(x, out, partial, R, C); return 0;
		case kMax: reduce_first<kMax>(x, out, partial, R, C); return 0;
		case kMin: reduce_first<kMin>(x, out, partial, R, C); return 0;
	}
	return -1;
}

// y = softmax(x) along the last axis. row_max, row_sum: R floats each; partial as for rows.
int oracle_softmax_rows_f32(const float* x, float* y, float* row_max, float* row_sum, float* partial, int R, int C) {
	reduce_last<kMax>(x, row_max, partial, R, C, NoFuse());
	reduce_last<kSum>(x, row_sum, partial, R, C, ExpMinusRowMax{(const uint*)row_max});
	uint var[3] = {asuint(R), asuint(C), 0u};
	uint* mem[4] = {(uint*)y, (uint*)x, (uint*)row_max, (uint*)row_sum};
	k_softmax_normalise(var, mem, groups_2d(R, C));
	return 0;
}

}  // extern "C"
