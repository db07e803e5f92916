// Programs whose traced function is exactly one of the idioms the backend serves with hand-written
// primitives. The host `main` is what the reference's generator would emit (allocations, shape checks,
// one dispatch per kernel, regions); the kernels are primitive-backed instead of emitted.
//
//   radix_sort   benchmark config 3: keys, values = tf.sort.radix(keys, values)
//                (Python/TensorFrost/sort.py:38-187; the whole `Radix sort` region collapses to one dispatch,
//                 the ping-pong buffers keys1/values1 of sort.py:96-100 are still allocated by the host)
//   reductions   benchmark config 2: tf.sum, tf.max, softmax along the last axis, tf.sum, tf.max along axis 0
//   prefix_sum   tf.prefix_sum of a 1-D uint / int / float tensor
#include "registry.h"

namespace tfhost {

static void BuildRadixSort(Program* program, const std::vector<int64_t>& params) {
	const int key_type = params.empty() ? TFType_Uint : (int)params[0];  // TFType of the keys
	const char* prim = key_type == TFType_Float ? "radix_sort_kv_f32" : key_type == TFType_Int ? "radix_sort_kv_i32" : "radix_sort_kv_u32";
	Kernel* sort = program->AddPrimitive(prim, 6, 1);
	program->input_count = 2;
	program->output_count = 2;
	program->execute_callback = [sort, key_type](TFTensor* in, TFTensor* out, TFRuntime runtime) -> int {
		TFContext tf(runtime);
		TFTensor keys = in[0], values = in[1];
		const TFDataFormat key_format{(TFType)key_type, 32};
		tf.region_begin("Radix sort");
		if (keys.dim != 1) throw std::runtime_error("Invalid number of dimensions for keys. Expected 1, got " + std::to_string(keys.dim));
		int N = (int)keys.shape[0];
		tf.check_tensor(keys, "keys", {(size_t)N}, key_format);
		tf.check_tensor(values, "values", {(size_t)N}, TFTypeUint32);
		TFTensor keys_out = tf.allocate("keys_sorted", {(size_t)N}, key_format);
		TFTensor values_out = tf.allocate("values_sorted", {(size_t)N}, TFTypeUint32);
		TFTensor keys1 = tf.allocate("keys1", {(size_t)N}, key_format);
		TFTensor values1 = tf.allocate("values1", {(size_t)N}, TFTypeUint32);
		tf.dispatch(sort->kernel_id_, {keys_out, values_out, keys1, values1}, {keys, values}, {asuint(N)}, {(size_t)N}, {256});
		tf.deallocate(keys1);
		tf.deallocate(values1);
		tf.region_end("Radix sort");
		out[0] = keys_out;
		out[1] = values_out;
		return 0;
	};
}

static void BuildReductions(Program* program, const std::vector<int64_t>&) {
	Kernel* sum_rows = program->AddPrimitive("reduce_rows_sum", 2, 2);
	Kernel* max_rows = program->AddPrimitive("reduce_rows_max", 2, 2);
	Kernel* softmax = program->AddPrimitive("softmax_rows", 2, 2);
	Kernel* sum_cols = program->AddPrimitive("reduce_cols_sum", 2, 2);
	Kernel* max_cols = program->AddPrimitive("reduce_cols_max", 2, 2);
	program->input_count = 1;
	program->output_count = 5;
	program->execute_callback = [=](TFTensor* in, TFTensor* out, TFRuntime runtime) -> int {
		TFContext tf(runtime);
		TFTensor X = in[0];
		tf.region_begin("Reductions");
		if (X.dim != 2) throw std::runtime_error("Invalid number of dimensions for X. Expected 2, got " + std::to_string(X.dim));
		int R = (int)X.shape[0], C = (int)X.shape[1];
		tf.check_tensor(X, "X", {(size_t)R, (size_t)C}, TFTypeFloat32);
		TFTensor s_last = tf.allocate("sum_last", {(size_t)R}, TFTypeFloat32);
		TFTensor m_last = tf.allocate("max_last", {(size_t)R}, TFTypeFloat32);
		TFTensor sm = tf.allocate("softmax", {(size_t)R, (size_t)C}, TFTypeFloat32);
		TFTensor s_first = tf.allocate("sum_first", {(size_t)C}, TFTypeFloat32);
		TFTensor m_first = tf.allocate("max_first", {(size_t)C}, TFTypeFloat32);
		tf.dispatch(sum_rows->kernel_id_, {s_last}, {X}, {asuint(R), asuint(C)}, {(size_t)R}, {256});
		tf.dispatch(max_rows->kernel_id_, {m_last}, {X}, {asuint(R), asuint(C)}, {(size_t)R}, {256});
		tf.dispatch(softmax->kernel_id_, {sm}, {X}, {asuint(R), asuint(C)}, {(size_t)R, (size_t)C}, {16, 16});
		tf.dispatch(sum_cols->kernel_id_, {s_first}, {X}, {asuint(R), asuint(C)}, {(size_t)C}, {256});
		tf.dispatch(max_cols->kernel_id_, {m_first}, {X}, {asuint(R), asuint(C)}, {(size_t)C}, {256});
		tf.region_end("Reductions");
		out[0] = s_last;
		out[1] = m_last;
		out[2] = sm;
		out[3] = s_first;
		out[4] = m_first;
		return 0;
	};
}

static void BuildPrefixSum(Program* program, const std::vector<int64_t>& params) {
	const int type = params.empty() ? TFType_Uint : (int)params[0];
	const char* prim = type == TFType_Float ? "scan_f32" : type == TFType_Int ? "scan_i32" : "scan_u32";
	Kernel* scan = program->AddPrimitive(prim, 2, 1);
	program->input_count = 1;
	program->output_count = 1;
	program->execute_callback = [scan, type](TFTensor* in, TFTensor* out, TFRuntime runtime) -> int {
		TFContext tf(runtime);
		TFTensor A = in[0];
		const TFDataFormat format{(TFType)type, 32};
		if (A.dim != 1) throw std::runtime_error("Invalid number of dimensions for A. Expected 1, got " + std::to_string(A.dim));
		int N = (int)A.shape[0];
		tf.check_tensor(A, "A", {(size_t)N}, format);
		TFTensor scanned = tf.allocate("prefix_sum", {(size_t)N}, format);
		tf.dispatch(scan->kernel_id_, {scanned}, {A}, {asuint(N)}, {1}, {1});
		out[0] = scanned;
		return 0;
	};
}

static ProgramRegistrar reg_sort("radix_sort", BuildRadixSort);
static ProgramRegistrar reg_reductions("reductions", BuildReductions);
static ProgramRegistrar reg_prefix_sum("prefix_sum", BuildPrefixSum);

}  // namespace tfhost
