// TEST INFRASTRUCTURE -- not part of the product (see prelude.h).
//
// tf.matmul as the reference's C++/OpenMP backend executes it: kernel shape = shape of C, 16x16 thread
// groups, one thread per element running `matmul = 0; for k: matmul = matmul + A[i,k]*B[k,j]`
// (TensorFrost/Compiler/Implementations.cpp:560-646); transposed operands are index remaps fused into the
// loads (:451-488), which gives the nt / tn forms used by the backward pass (:133-135).
//
// Pins (tests/test_oracle_mlp.py): float64 NumPy products on rectangular shapes with M != N != K, so a
// transposed operand or swapped index fails; identity and outer-product special cases.

#include "prelude.h"

using namespace tfo;

namespace {

// layout: 0 = nn (A[M,K], B[K,N]), 1 = nt (A[M,K], B[N,K]), 2 = tn (A[K,M], B[K,N])
template <int LAYOUT>
void k_matmul(const uint* var, uint** mem, uint work_group_count) {
	uint* C_mem = mem[0];
	uint* A_mem = mem[1];
	uint* B_mem = mem[2];
	int var_M = asint(var[0]);
	int var_N = asint(var[1]);
	int var_K = asint(var[2]);
	uint var__kernel_block_offset = asuint(var[3]);
#pragma omp parallel for
	for (int block_id = var__kernel_block_offset; block_id < (int)(work_group_count + var__kernel_block_offset); block_id++) {
		for (int block_thread_id1 = 0; block_thread_id1 < 16; block_thread_id1++)
			for (int block_thread_id0 = 0; block_thread_id0 < 16; block_thread_id0++) {
				int blocks_shape_0 = ((var_N + 16) - 1) / 16;
				int vdiv = block_id / blocks_shape_0;
				int index_0 = ((block_id - (vdiv * blocks_shape_0)) * 16) + block_thread_id0;  // j
				int index_1 = (vdiv * 16) + block_thread_id1;                                    // i
				bool is_inside_dispatch = (index_0 < var_N) && (index_1 < var_M);
				if (is_inside_dispatch) {
					float matmul = 0.0f;
					for (int vloop = 0; vloop < var_K; vloop += 1) {
						float A = LAYOUT == 2 ? asfloat(A_mem[(vloop * var_M) + index_1]) : asfloat(A_mem[(index_1 * var_K) + vloop]);
						float B = LAYOUT == 1 ? asfloat(B_mem[(index_0 * var_K) + vloop]) : asfloat(B_mem[(vloop * var_N) + index_0]);
						matmul = matmul + (A * B);
					}
					C_mem[(index_1 * var_N) + index_0] = asuint(matmul);
				}
			}
	}
}

}  // namespace

extern "C" int oracle_matmul_f32(int layout, const float* A, const float* B, float* C, int M, int N, int K) {
	size_t shape[2] = {(size_t)M, (size_t)N}, group[2] = {16, 16};
	uint var[4] = {asuint(M), asuint(N), asuint(K), 0u};
	uint* mem[3] = {(uint*)C, (uint*)A, (uint*)B};
	uint groups = (uint)work_group_count(shape, 2, group, 2);
	switch (layout) {
		case 0: k_matmul<0>(var, mem, groups); return 0;
		case 1: k_matmul<1>(var, mem, groups); return 0;
		case 2: k_matmul<2>(var, mem, groups); return 0;
	}
	return -1;
}
