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
	const TFType key_type = params.empty() ? TFType_Uint : (TFType)params[0];  // TFType of the keys
	const char* prim = key_type == TFType_Float ? "radix_sort_kv_f32" : key_type == TFType_Int ? "radix_sort_kv_i32" : "radix_sort_kv_u32";
	Kernel* sort = program->AddPrimitive(prim, 6, 1);
	HostBuilder h(program);
	h.RegionBegin("Radix sort");
	V keys = h.Input("keys", {-1}, key_type);
	V n = h.Shape(keys)[0];
	V values = h.Input("values", {n}, TFType_Uint);
	V keys_out = h.Allocate("keys_sorted", {n}, key_type);
	V values_out = h.Allocate("values_sorted", {n}, TFType_Uint);
	V keys1 = h.Allocate("keys1", {n}, key_type);
	V values1 = h.Allocate("values1", {n}, TFType_Uint);
	h.Dispatch(sort, {keys_out, values_out, keys1, values1}, {keys, values}, {n}, {n});
	h.Deallocate(keys1);
	h.Deallocate(values1);
	h.RegionEnd("Radix sort");
	h.Output(keys_out);
	h.Output(values_out);
	h.Finish();
}

static void BuildReductions(Program* program, const std::vector<int64_t>&) {
	Kernel* sum_rows = program->AddPrimitive("reduce_rows_sum", 2, 2);
	Kernel* max_rows = program->AddPrimitive("reduce_rows_max", 2, 2);
	Kernel* softmax = program->AddPrimitive("softmax_rows", 2, 2);
	Kernel* sum_cols = program->AddPrimitive("reduce_cols_sum", 2, 2);
	Kernel* max_cols = program->AddPrimitive("reduce_cols_max", 2, 2);
	HostBuilder h(program);
	h.RegionBegin("Reductions");
	V X = h.Input("X", {-1, -1}, TFType_Float);
	V R = h.Shape(X)[0], C = h.Shape(X)[1];
	V s_last = h.Allocate("sum_last", {R}, TFType_Float);
	V m_last = h.Allocate("max_last", {R}, TFType_Float);
	V sm = h.Allocate("softmax", {R, C}, TFType_Float);
	V s_first = h.Allocate("sum_first", {C}, TFType_Float);
	V m_first = h.Allocate("max_first", {C}, TFType_Float);
	h.Dispatch(sum_rows, {s_last}, {X}, {R, C}, {R});
	h.Dispatch(max_rows, {m_last}, {X}, {R, C}, {R});
	h.Dispatch(softmax, {sm}, {X}, {R, C}, {R, C});
	h.Dispatch(sum_cols, {s_first}, {X}, {R, C}, {C});
	h.Dispatch(max_cols, {m_first}, {X}, {R, C}, {C});
	h.RegionEnd("Reductions");
	for (V out : {s_last, m_last, sm, s_first, m_first}) h.Output(out);
	h.Finish();
}

static void BuildPrefixSum(Program* program, const std::vector<int64_t>& params) {
	const TFType type = params.empty() ? TFType_Uint : (TFType)params[0];
	const char* prim = type == TFType_Float ? "scan_f32" : type == TFType_Int ? "scan_i32" : "scan_u32";
	Kernel* scan = program->AddPrimitive(prim, 2, 1);
	HostBuilder h(program);
	V A = h.Input("A", {-1}, type);
	V n = h.Shape(A)[0];
	V scanned = h.Allocate("prefix_sum", {n}, type);
	h.Dispatch(scan, {scanned}, {A}, {n}, {1});
	h.Output(scanned);
	h.Finish();
}

static ProgramRegistrar reg_sort("radix_sort", BuildRadixSort);
static ProgramRegistrar reg_reductions("reductions", BuildReductions);
static ProgramRegistrar reg_prefix_sum("prefix_sum", BuildPrefixSum);

}  // namespace tfhost
