// benchmark config 2 as the reference's own passes leave it for a tensor of constant shape [R, C]:
// every tf.sum / tf.max over an axis of 1024 or more elements is split by OptimizeReductions into chunks of 128
// (Compiler/Steps/Optimization.cpp:469-510): a first kernel that reduces each chunk, reading the tensor through
// the dim_split view with its out-of-bounds select and clamped load (Compiler/Implementations.cpp:56-69,507-528),
// and a second kernel over the partial results. The kernels below are that IR; nothing names a primitive. The
// backend recognises each of them as a reduction (idiom_matcher.cpp) and serves it with libtfhip's reductions
// when the chunks tile the axis exactly, as they do for [16384, 4096].
//
// The softmax of the same config is a five-kernel composition in user code and is not part of this program.
//
//   params: none.  input X[R, C] float.  outputs: sum and max over the last axis [R], sum and max over axis 0 [C].
#include "registry.h"

namespace tfhost {

namespace {

constexpr float kLowest = -3.402823466e+38f;

struct ReduceOp {
	const char* name;
	float init;
};

V Combine(const ReduceOp& op, V acc, V x) { return std::string(op.name) == "sum" ? acc + x : Fn("max", acc, x); }

// ConstantOutOfBounds: select(false || (i0 < 0 || i0 >= n0) || (i1 < 0 || i1 >= n1), 0, load(clamped indices))
V SplitLoad(KernelBuilder& kb, V X, V row, V col, V R, V C) {
	V oob = kb.Named((kb.ConstB(false) || ((row < kb.Const(0)) || (row >= R))) || ((col < kb.Const(0)) || (col >= C)), "out_of_bounds");
	V x = kb.Load(X, kb.Clamp(row, kb.Const(0), R - kb.Const(1)) * C + kb.Clamp(col, kb.Const(0), C - kb.Const(1)), TFType_Float);
	return kb.Named(Select(oob, kb.Const(0.0f), x), "split");
}

// last axis, stage 1: kernel shape [R, S], partial[r, s] = op_k X[r, s*128 + k]
Kernel* LastAxisStage1(Program* program, const ReduceOp& op) {
	KernelBuilder kb(program, 2);
	V partial = kb.Buffer("partial", false), X = kb.Buffer("X", true);
	V R = kb.Var("R", TFType_Int), C = kb.Var("C", TFType_Int), S = kb.Var("S", TFType_Int);
	std::vector<V> idx = kb.ThreadIndices({S, R});
	V s = idx[0], r = idx[1];
	V acc = kb.Accumulator(op.name, TFType_Float, FloatBits(op.init));
	kb.Loop(kb.Const(0), kb.Const(128), kb.Const(1), [&](V k) { kb.Set(acc, Combine(op, acc, SplitLoad(kb, X, r, s * kb.Const(128) + k, R, C))); });
	kb.Store(partial, r * S + s, acc);
	return kb.Finish();
}

// last axis, stage 2: kernel shape [R], out[r] = op_s partial[r, s]
Kernel* LastAxisStage2(Program* program, const ReduceOp& op) {
	KernelBuilder kb(program, 1);
	V out = kb.Buffer("result", false), partial = kb.Buffer("partial", true);
	V R = kb.Var("R", TFType_Int), S = kb.Var("S", TFType_Int);
	V r = kb.ThreadIndices({R})[0];
	V acc = kb.Accumulator(op.name, TFType_Float, FloatBits(op.init));
	kb.Loop(kb.Const(0), S, kb.Const(1), [&](V k) { kb.Set(acc, Combine(op, acc, kb.Load(partial, r * S + k, TFType_Float))); });
	kb.Store(out, r, acc);
	return kb.Finish();
}

// axis 0, stage 1: kernel shape [S, C], partial[s, c] = op_k X[s*128 + k, c]
Kernel* FirstAxisStage1(Program* program, const ReduceOp& op) {
	KernelBuilder kb(program, 2);
	V partial = kb.Buffer("partial", false), X = kb.Buffer("X", true);
	V R = kb.Var("R", TFType_Int), C = kb.Var("C", TFType_Int), S = kb.Var("S", TFType_Int);
	std::vector<V> idx = kb.ThreadIndices({C, S});
	V c = idx[0], s = idx[1];
	V acc = kb.Accumulator(op.name, TFType_Float, FloatBits(op.init));
	kb.Loop(kb.Const(0), kb.Const(128), kb.Const(1), [&](V k) { kb.Set(acc, Combine(op, acc, SplitLoad(kb, X, s * kb.Const(128) + k, c, R, C))); });
	kb.Store(partial, s * C + c, acc);
	return kb.Finish();
}

// axis 0, stage 2: kernel shape [C], out[c] = op_s partial[s, c]
Kernel* FirstAxisStage2(Program* program, const ReduceOp& op) {
	KernelBuilder kb(program, 1);
	V out = kb.Buffer("result", false), partial = kb.Buffer("partial", true);
	V C = kb.Var("C", TFType_Int), S = kb.Var("S", TFType_Int);
	V c = kb.ThreadIndices({C})[0];
	V acc = kb.Accumulator(op.name, TFType_Float, FloatBits(op.init));
	kb.Loop(kb.Const(0), S, kb.Const(1), [&](V k) { kb.Set(acc, Combine(op, acc, kb.Load(partial, k * C + c, TFType_Float))); });
	kb.Store(out, c, acc);
	return kb.Finish();
}

}  // namespace

static void BuildReductionsIr(Program* program, const std::vector<int64_t>& args) {
	// args[0] = 1: the chunk results are released only at the end of the program, as if something still read them
	const bool late_release = !args.empty() && args[0] == 1;
	const ReduceOp ops[2] = {{"sum", 0.0f}, {"max", kLowest}};
	Kernel *last1[2], *last2[2], *first1[2], *first2[2];
	for (int i = 0; i < 2; i++) {
		last1[i] = LastAxisStage1(program, ops[i]);
		last2[i] = LastAxisStage2(program, ops[i]);
		first1[i] = FirstAxisStage1(program, ops[i]);
		first2[i] = FirstAxisStage2(program, ops[i]);
	}
	program->input_count = 1;
	program->output_count = 4;
	program->execute_callback = [=](TFTensor* in, TFTensor* out, TFRuntime runtime) -> int {
		TFContext tf(runtime);
		TFTensor X = in[0];
		std::vector<TFTensor> kept;
		tf.region_begin("Reductions");
		if (X.dim != 2) throw std::runtime_error("Invalid number of dimensions for X. Expected 2, got " + std::to_string(X.dim));
		const int R = (int)X.shape[0], C = (int)X.shape[1];
		tf.check_tensor(X, "X", {(size_t)R, (size_t)C}, TFTypeFloat32);
		const int SC = (C + 127) / 128, SR = (R + 127) / 128;
		for (int i = 0; i < 2; i++) {
			TFTensor partial = tf.allocate("partial", {(size_t)R, (size_t)SC}, TFTypeFloat32);
			tf.dispatch(last1[i]->kernel_id_, {partial}, {X}, {asuint(R), asuint(C), asuint(SC)}, {(size_t)R, (size_t)SC}, {16, 16});
			TFTensor result = tf.allocate("result", {(size_t)R}, TFTypeFloat32);
			tf.dispatch(last2[i]->kernel_id_, {result}, {partial}, {asuint(R), asuint(SC)}, {(size_t)R}, {256});
			if (late_release) kept.push_back(partial); else tf.deallocate(partial);
			out[i] = result;
		}
		for (int i = 0; i < 2; i++) {
			TFTensor partial = tf.allocate("partial", {(size_t)SR, (size_t)C}, TFTypeFloat32);
			tf.dispatch(first1[i]->kernel_id_, {partial}, {X}, {asuint(R), asuint(C), asuint(SR)}, {(size_t)SR, (size_t)C}, {16, 16});
			TFTensor result = tf.allocate("result", {(size_t)C}, TFTypeFloat32);
			tf.dispatch(first2[i]->kernel_id_, {result}, {partial}, {asuint(C), asuint(SR)}, {(size_t)C}, {256});
			if (late_release) kept.push_back(partial); else tf.deallocate(partial);
			out[2 + i] = result;
		}
		for (TFTensor& t : kept) tf.deallocate(t);
		tf.region_end("Reductions");
		return 0;
	};
}

static ProgramRegistrar reg_reductions_ir("reductions_ir", BuildReductionsIr);

}  // namespace tfhost
