// TEST INFRASTRUCTURE -- not part of the product (see prelude.h).
//
// One leapfrog step of the 2-D sine-Gordon equation on a periodic grid as the reference's C++/OpenMP
// backend would run the fused kernel: kernel shape [N, M], thread-groups of 16x16 spread by OpenMP,
// threads of a group run serially, index arithmetic from block_id / block_thread_id, user loads clamped.
// Form follows TensorFrost/Backend/CodeGen/Langs/CPP.cpp:720-779 (wrapper),
// Compiler/Steps/GraphOps.cpp:1091-1186 (indices, bounds `if`), :989-1043 (Clamp indexing, C-order flat
// address); the stencil itself is benchmark config 1 (5-point Laplacian, v += dt*(lap - sin u), u += dt*v).
//
// Pins (tests/test_oracle_stencil.py): float64 np.roll closed form of the same update (1e-6); a constant
// field (lap = 0) and a single-mode plane wave whose discrete Laplacian is known in closed form
// (-(4 - 2cos kx - 2cos ky) u), which a wrong tap, sign or transposed index fails. `sinf` comes from the
// host libm under -ffast-math and is not pinned by any reference test.

#include "prelude.h"

using namespace tfo;

extern "C" void oracle_wave_eq_kernel(const uint* var, uint** mem, uint work_group_count) {
	uint* v_new_mem = mem[0];
	uint* u_new_mem = mem[1];
	uint* u_mem = mem[2];
	uint* v_mem = mem[3];
	int var_N = asint(var[0]);
	int var_M = asint(var[1]);
	float var_dt = asfloat(var[2]);
	uint var__kernel_block_offset = asuint(var[3]);
#pragma omp parallel for
	for (int block_id = var__kernel_block_offset; block_id < (int)(work_group_count + var__kernel_block_offset); block_id++) {
		for (int block_thread_id1 = 0; block_thread_id1 < 16; block_thread_id1++)
			for (int block_thread_id0 = 0; block_thread_id0 < 16; block_thread_id0++) {
				int blocks_shape_0 = ((var_M + 16) - 1) / 16;
				int vdiv = block_id / blocks_shape_0;
				int index_0 = ((block_id - (vdiv * blocks_shape_0)) * 16) + block_thread_id0;
				int index_1 = (vdiv * 16) + block_thread_id1;
				bool is_inside_dispatch = (index_0 < var_M) && (index_1 < var_N);
				if (is_inside_dispatch) {
					float u = asfloat(u_mem[(index_1 * var_M) + index_0]);
					float u_up = asfloat(u_mem[(clamp(((index_1 + var_N) - 1) % var_N, 0, var_N - 1) * var_M) + clamp(index_0, 0, var_M - 1)]);
					float u_down = asfloat(u_mem[(clamp((index_1 + 1) % var_N, 0, var_N - 1) * var_M) + clamp(index_0, 0, var_M - 1)]);
					float u_left = asfloat(u_mem[(clamp(index_1, 0, var_N - 1) * var_M) + clamp(((index_0 + var_M) - 1) % var_M, 0, var_M - 1)]);
					float u_right = asfloat(u_mem[(clamp(index_1, 0, var_N - 1) * var_M) + clamp((index_0 + 1) % var_M, 0, var_M - 1)]);
					float lap = (((u_up + u_down) + u_left) + u_right) - (4.0f * u);
					float v = asfloat(v_mem[(index_1 * var_M) + index_0]);
					float v_new = v + (var_dt * (lap - sinf(u)));
					float u_new = u + (var_dt * v_new);
					v_new_mem[(index_1 * var_M) + index_0] = asuint(v_new);
					u_new_mem[(index_1 * var_M) + index_0] = asuint(u_new);
				}
			}
	}
}

// `steps` leapfrog steps, ping-ponging between (u, v) and (u_tmp, v_tmp); the final state ends in (u, v).
extern "C" int oracle_wave_eq_run(float* u, float* v, float* u_tmp, float* v_tmp, int N, int M, float dt, int steps) {
	size_t shape[2] = {(size_t)N, (size_t)M}, group[2] = {16, 16};
	uint groups = (uint)work_group_count(shape, 2, group, 2);
	uint var[4] = {asuint(N), asuint(M), asuint(dt), 0u};
	float* cur_u = u;
	float* cur_v = v;
	float* nxt_u = u_tmp;
	float* nxt_v = v_tmp;
	for (int s = 0; s < steps; s++) {
		uint* mem[4] = {(uint*)nxt_v, (uint*)nxt_u, (uint*)cur_u, (uint*)cur_v};
		oracle_wave_eq_kernel(var, mem, groups);
		float* t = cur_u; cur_u = nxt_u; nxt_u = t;
		t = cur_v; cur_v = nxt_v; nxt_v = t;
	}
	if (cur_u != u) {
		std::memcpy(u, cur_u, sizeof(float) * (size_t)N * M);
		std::memcpy(v, cur_v, sizeof(float) * (size_t)N * M);
	}
	return 0;
}
