// TEST INFRASTRUCTURE -- not part of the product (see prelude.h).
//
// One symplectic-Euler step of an all-pairs gravitational N-body system as the reference's C++/OpenMP
// backend runs the loop form of the example (examples/Simulation/n-body-benchmark.py:36-65): kernel shape
// [N], thread-groups of 256, one thread per body i running a serial loop over all bodies j with three
// scalar accumulators, then V += a*dt, X += V*dt. benchmark config 4 adds masses and Plummer softening:
//   a_i = sum_j m_j * (x_j - x_i) / (|x_j - x_i|^2 + eps^2)^(3/2)
// User loads index in Clamp mode (Tensor.h:566-567), hence the clamps on j and on the component index.
//
// Pins (tests/test_oracle_nbody.py): float64 NumPy direct summation (1e-5 of the sum of term magnitudes);
// total momentum change sum_i m_i * dV_i == 0 (Newton's third law: fails for a wrong sign or a dropped
// mass); two-body closed form. sqrt and division come from the host toolchain under -ffast-math.

#include "prelude.h"

using namespace tfo;

extern "C" void oracle_nbody_kernel(const uint* var, uint** mem, uint work_group_count) {
	uint* x_new_mem = mem[0];
	uint* v_new_mem = mem[1];
	uint* x_mem = mem[2];
	uint* v_mem = mem[3];
	uint* m_mem = mem[4];
	int var_N = asint(var[0]);
	float var_dt = asfloat(var[1]);
	float var_eps2 = asfloat(var[2]);
	uint var__kernel_block_offset = asuint(var[3]);
#pragma omp parallel for
	for (int block_id = var__kernel_block_offset; block_id < (int)(work_group_count + var__kernel_block_offset); block_id++) {
		for (int block_thread_id0 = 0; block_thread_id0 < 256; block_thread_id0++) {
			int index_0 = (block_id * 256) + block_thread_id0;
			bool is_inside_dispatch = index_0 < var_N;
			if (is_inside_dispatch) {
				float ax = 0.0f;
				float ay = 0.0f;
				float az = 0.0f;
				float x0 = asfloat(x_mem[(clamp(index_0, 0, var_N - 1) * 3) + clamp(0, 0, 2)]);
				float y0 = asfloat(x_mem[(clamp(index_0, 0, var_N - 1) * 3) + clamp(1, 0, 2)]);
				float z0 = asfloat(x_mem[(clamp(index_0, 0, var_N - 1) * 3) + clamp(2, 0, 2)]);
				for (int j = 0; j < var_N; j += 1) {
					float x = asfloat(x_mem[(clamp(j, 0, var_N - 1) * 3) + clamp(0, 0, 2)]);
					float y = asfloat(x_mem[(clamp(j, 0, var_N - 1) * 3) + clamp(1, 0, 2)]);
					float z = asfloat(x_mem[(clamp(j, 0, var_N - 1) * 3) + clamp(2, 0, 2)]);
					float m = asfloat(m_mem[clamp(j, 0, var_N - 1)]);
					float dx = x - x0;
					float dy = y - y0;
					float dz = z - z0;
					float d2 = (((dx * dx) + (dy * dy)) + (dz * dz)) + var_eps2;
					float s = m / (d2 * sqrtf(d2));
					ax = ax + (s * dx);
					ay = ay + (s * dy);
					az = az + (s * dz);
				}
				float vx = asfloat(v_mem[(index_0 * 3) + 0]) + (ax * var_dt);
				float vy = asfloat(v_mem[(index_0 * 3) + 1]) + (ay * var_dt);
				float vz = asfloat(v_mem[(index_0 * 3) + 2]) + (az * var_dt);
				v_new_mem[(index_0 * 3) + 0] = asuint(vx);
				v_new_mem[(index_0 * 3) + 1] = asuint(vy);
				v_new_mem[(index_0 * 3) + 2] = asuint(vz);
				x_new_mem[(index_0 * 3) + 0] = asuint(x0 + (vx * var_dt));
				x_new_mem[(index_0 * 3) + 1] = asuint(y0 + (vy * var_dt));
				x_new_mem[(index_0 * 3) + 2] = asuint(z0 + (vz * var_dt));
			}
		}
	}
}

extern "C" int oracle_nbody_step(const float* x, const float* v, const float* m, float* x_new, float* v_new, int N, float dt, float eps) {
	size_t shape[1] = {(size_t)N}, group[1] = {256};
	uint var[4] = {asuint(N), asuint(dt), asuint(eps * eps), 0u};
	uint* mem[5] = {(uint*)x_new, (uint*)v_new, (uint*)x, (uint*)v, (uint*)m};
	oracle_nbody_kernel(var, mem, (uint)work_group_count(shape, 1, group, 1));
	return 0;
}
