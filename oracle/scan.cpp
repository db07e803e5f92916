// TEST INFRASTRUCTURE -- not part of the product (see prelude.h).
//
// Inclusive prefix sum as the reference's C++/OpenMP backend executes dim_prefix_sum: one logical
// thread per scan LINE runs `acc = acc + x[k]; out[k] = acc` over the axis
// (TensorFrost/Compiler/Implementations.cpp:305-359,447-449). A 1-D array has one line, so the kernel
// shape is [1] (Implementations.cpp:330-333) and a single thread of a single group does all the work.
// A [lines, n] matrix scanned along its last axis has `lines` threads, 256 to a group.
//
// Pins (tests/test_oracle_scan.py): np.cumsum with wrap-around for u32/i32 (exact), float64 cumsum for
// f32 (1e-6 of the running sum of magnitudes); a wrong init, an exclusive instead of inclusive scan or a
// transposed index fails them.

#include "prelude.h"

using namespace tfo;

namespace {

// kernel shape [L], group {256}: line index_0 scans x[index_0, 0..K)
template <class T, class Load, class Store>
void k_prefix_sum_last(const uint* var, uint** mem, uint work_group_count, Load load, Store store) {
	uint* out_mem = mem[0];
	uint* x_mem = mem[1];
	int var_L = asint(var[0]);
	int var_K = asint(var[1]);
	uint var__kernel_block_offset = asuint(var[2]);
#pragma omp parallel for
	for (int block_id = var__kernel_block_offset; block_id < (int)(work_group_count + var__kernel_block_offset); block_id++) {
		for (int block_thread_id0 = 0; block_thread_id0 < 256; block_thread_id0++) {
			int index_0 = (block_id * 256) + block_thread_id0;
			bool is_inside_dispatch = index_0 < var_L;
			if (is_inside_dispatch) {
				T prefix_sum = T(0);
				for (int vloop = 0; vloop < var_K; vloop += 1) {
					T x = load(x_mem[(index_0 * var_K) + vloop]);
					prefix_sum = prefix_sum + x;
					out_mem[(index_0 * var_K) + vloop] = store(prefix_sum);
				}
			}
		}
	}
}

}  // namespace

extern "C" {

int oracle_scan_inclusive_u32(const uint32_t* x, uint32_t* out, int lines, int n) {
	uint var[3] = {asuint(lines), asuint(n), 0u};
	uint* mem[2] = {(uint*)out, (uint*)x};
	size_t shape[1] = {(size_t)lines}, group[1] = {256};
	k_prefix_sum_last<uint>(var, mem, (uint)work_group_count(shape, 1, group, 1), [](uint w) { return w; }, [](uint v) { return v; });
	return 0;
}

int oracle_scan_inclusive_i32(const int32_t* x, int32_t* out, int lines, int n) {
	uint var[3] = {asuint(lines), asuint(n), 0u};
	uint* mem[2] = {(uint*)out, (uint*)x};
	size_t shape[1] = {(size_t)lines}, group[1] = {256};
	k_prefix_sum_last<int>(var, mem, (uint)work_group_count(shape, 1, group, 1), [](uint w) { return asint(w); }, [](int v) { return asuint(v); });
	return 0;
}

int oracle_scan_inclusive_f32(const float* x, float* out, int lines, int n) {
	uint var[3] = {asuint(lines), asuint(n), 0u};
	uint* mem[2] = {(uint*)out, (uint*)x};
	size_t shape[1] = {(size_t)lines}, group[1] = {256};
	k_prefix_sum_last<float>(var, mem, (uint)work_group_count(shape, 1, group, 1), [](uint w) { return asfloat(w); }, [](float v) { return asuint(v); });
	return 0;
}

}  // extern "C"
