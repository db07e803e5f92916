// Row softmax as the reference composes and lowers it for a tensor of shape [R, C]:
//     m = tf.max(x, axis=-1);  e = tf.exp(x - m);  y = e / tf.sum(e, axis=-1)
// (tests/autograd_test.py:29-31, examples/ML/MNIST/module.py:8-10). With C >= 1024 both reductions are split into
// chunks of 128 (Compiler/Steps/Optimization.cpp:469-510), and kernel fusion puts exp(x - m) into the loop of the
// sum's first stage and into the final element-wise kernel, so the input is read three times:
//   k0  max, stage 1   [R, S]   partial_max[r, s] = max_k X[r, s*128 + k]            (dim_split view, zero padding)
//   k1  max, stage 2   [R]      m[r] = max_s partial_max[r, s]
//   k2  sum, stage 1   [R, S]   partial_sum[r, s] = sum_k exp(X[r, s*128 + k] - m[r])  (zero outside the tensor)
//   k3  sum, stage 2   [R]      z[r] = sum_s partial_sum[r, s]
//   k4  normalise      [R, C]   Y[r, c] = exp(X[r, c] - m[r]) / z[r]
// Nothing names a primitive. k0, k1 and k3 are plain reductions and may be served by libtfhip's; k2 and k4 are emitted.
// For C < 1024 the reductions stay unsplit and the program has three kernels:
//   k0  max        [R]      m[r] = max_c X[r, c]
//   k1  sum        [R]      z[r] = sum_c exp(X[r, c] - m[r])
//   k2  normalise  [R, C]
// The program builds the split form (any C >= 128) or, with bit 0 of its argument set, the unsplit form (any C).
// Bit 1: the row maxima and row sums are outputs as well (Y, m, z) instead of being released. Bit 2 (split form): the
// chunk tensors are released only after the last kernel, as a program would that still reads them. Bit 3: the last
// kernel is that of a log-softmax instead, Y = (X - m) - log(z) (tests/autograd_test.py:29-31). Bit 4 (with bit 3): the
// log-softmax scaled by -1/C, as a cross-entropy against a uniform target would fuse it: a last kernel that is neither.
// Bit 5: e = exp(x - m) is a tensor of its own -- what the passes leave when they do not copy the element-wise value into
// the kernels that load it: one more kernel writes E[R, C], the sum runs over E (split or not, a plain reduction) and the
// last kernel is Y = E / z; E is released behind it. Bit 6 (with bit 5): E is a second output instead (then the program
// still reads it, and nothing may skip writing it).
// When the kernel manager sees the whole sequence arrive on the same tensors (split form: C a multiple of 128, so that
// no padding takes part) it runs the fused softmax primitive instead; otherwise every kernel runs as dispatched.
//
//   input X[R, C] float.  output Y[R, C].
#include "registry.h"

namespace tfhost {

namespace {

constexpr float kLowest = -3.402823466e+38f;

// ConstantOutOfBounds of the dim_split view: select(out of bounds, 0, load(clamped))
V SplitLoad(KernelBuilder& kb, V X, V row, V col, V R, V C) {
	V oob = kb.Named((kb.ConstB(false) || ((row < kb.Const(0)) || (row >= R))) || ((col < kb.Const(0)) || (col >= C)), "out_of_bounds");
	V x = kb.Load(X, kb.Clamp(row, kb.Const(0), R - kb.Const(1)) * C + kb.Clamp(col, kb.Const(0), C - kb.Const(1)), TFType_Float);
	return kb.Named(Select(oob, kb.Const(0.0f), x), "split");
}

}  // namespace

static void BuildSoftmaxIr(Program* program, const std::vector<int64_t>& args) {
	const int64_t flags = args.empty() ? 0 : args[0];
	const bool split = !(flags & 1), keep_stats = flags & 2, late_release = flags & 4, log_form = flags & 8, scaled = flags & 16, separate_exp = flags & 32,
	           keep_exp = flags & 64;
	Kernel* max1 = nullptr;
	if (split) {
		KernelBuilder kb(program, 2);
		V partial = kb.Buffer("partial_max", false), X = kb.Buffer("X", true);
		V R = kb.Var("R", TFType_Int), C = kb.Var("C", TFType_Int), S = kb.Var("S", TFType_Int);
		std::vector<V> idx = kb.ThreadIndices({S, R});
		V s = idx[0], r = idx[1];
		V acc = kb.Accumulator("max", TFType_Float, FloatBits(kLowest));
		kb.Loop(kb.Const(0), kb.Const(128), kb.Const(1), [&](V k) { kb.Set(acc, Fn("max", acc, SplitLoad(kb, X, r, s * kb.Const(128) + k, R, C))); });
		kb.Store(partial, r * S + s, acc);
		max1 = kb.Finish();
	}
	auto stage2 = [&](const char* op, float init, const char* in_name, const char* out_name) {
		KernelBuilder kb(program, 1);
		V out = kb.Buffer(out_name, false), partial = kb.Buffer(in_name, true);
		V R = kb.Var("R", TFType_Int), S = kb.Var("S", TFType_Int);
		V r = kb.ThreadIndices({R})[0];
		V acc = kb.Accumulator(op, TFType_Float, FloatBits(init));
		kb.Loop(kb.Const(0), S, kb.Const(1), [&](V k) {
			V x = kb.Load(partial, r * S + k, TFType_Float);
			kb.Set(acc, std::string(op) == "max" ? Fn("max", acc, x) : acc + x);
		});
		kb.Store(out, r, acc);
		return kb.Finish();
	};
	Kernel* max2 = split ? stage2("max", kLowest, "partial_max", "row_max") : nullptr;
	Kernel* sum1 = nullptr;
	Kernel* max_rows = nullptr;
	Kernel* sum_rows = nullptr;
	if (!split) {
		{
			KernelBuilder kb(program, 1);
			V out = kb.Buffer("row_max", false), X = kb.Buffer("X", true);
			V R = kb.Var("R", TFType_Int), C = kb.Var("C", TFType_Int);
			V r = kb.ThreadIndices({R})[0];
			V acc = kb.Accumulator("max", TFType_Float, FloatBits(kLowest));
			kb.Loop(kb.Const(0), C, kb.Const(1), [&](V k) { kb.Set(acc, Fn("max", acc, kb.Load(X, r * C + k, TFType_Float))); });
			kb.Store(out, r, acc);
			max_rows = kb.Finish();
		}
		{
			KernelBuilder kb(program, 1);
			V out = kb.Buffer("row_sum", false), X = kb.Buffer("X", true), M = kb.Buffer("row_max", true);
			V R = kb.Var("R", TFType_Int), C = kb.Var("C", TFType_Int);
			V r = kb.ThreadIndices({R})[0];
			V acc = kb.Accumulator("sum", TFType_Float, FloatBits(0.0f));
			kb.Loop(kb.Const(0), C, kb.Const(1), [&](V k) { kb.Set(acc, acc + Fn("exp", kb.Load(X, r * C + k, TFType_Float) - kb.Load(M, r, TFType_Float))); });
			kb.Store(out, r, acc);
			sum_rows = kb.Finish();
		}
	}
	if (split) {
		KernelBuilder kb(program, 2);
		V partial = kb.Buffer("partial_sum", false), X = kb.Buffer("X", true), M = kb.Buffer("row_max", true);
		V R = kb.Var("R", TFType_Int), C = kb.Var("C", TFType_Int), S = kb.Var("S", TFType_Int);
		std::vector<V> idx = kb.ThreadIndices({S, R});
		V s = idx[0], r = idx[1];
		V m = kb.Named(kb.Load(M, r, TFType_Float), "m");
		V acc = kb.Accumulator("sum", TFType_Float, FloatBits(0.0f));
		kb.Loop(kb.Const(0), kb.Const(128), kb.Const(1), [&](V k) {
			V col = kb.Named(s * kb.Const(128) + k, "col");
			// the split view pads exp(x - m) itself with zeros: the select wraps the fused element-wise value
			V oob = kb.Named((kb.ConstB(false) || ((r < kb.Const(0)) || (r >= R))) || ((col < kb.Const(0)) || (col >= C)), "out_of_bounds");
			V x = kb.Load(X, kb.Clamp(r, kb.Const(0), R - kb.Const(1)) * C + kb.Clamp(col, kb.Const(0), C - kb.Const(1)), TFType_Float);
			kb.Set(acc, acc + Select(oob, kb.Const(0.0f), Fn("exp", x - m)));
		});
		kb.Store(partial, r * S + s, acc);
		sum1 = kb.Finish();
	}
	Kernel* sum2 = split ? stage2("sum", 0.0f, "partial_sum", "row_sum") : nullptr;
	Kernel* normalise;
	{
		KernelBuilder kb(program, 2);
		V Y = kb.Buffer("Y", false), X = kb.Buffer("X", true), M = kb.Buffer("row_max", true), Z = kb.Buffer("row_sum", true);
		V R = kb.Var("R", TFType_Int), C = kb.Var("C", TFType_Int);
		std::vector<V> idx = kb.ThreadIndices({C, R});
		V c = idx[0], r = idx[1];
		V shifted = kb.Load(X, r * C + c, TFType_Float) - kb.Load(M, r, TFType_Float);
		if (log_form && scaled)
			kb.Store(Y, r * C + c, (shifted - Fn("log", kb.Load(Z, r, TFType_Float))) * (kb.Const(-1.0f) / ToFloat(C)));
		else if (log_form)
			kb.Store(Y, r * C + c, shifted - Fn("log", kb.Load(Z, r, TFType_Float)));
		else
			kb.Store(Y, r * C + c, Fn("exp", shifted) / kb.Load(Z, r, TFType_Float));
		normalise = kb.Finish();
	}
	Kernel *exp_kernel = nullptr, *esum1 = nullptr, *esum_rows = nullptr, *divide = nullptr;
	if (separate_exp) {
		{
			KernelBuilder kb(program, 2);
			V E = kb.Buffer("E", false), X = kb.Buffer("X", true), M = kb.Buffer("row_max", true);
			V R = kb.Var("R", TFType_Int), C = kb.Var("C", TFType_Int);
			std::vector<V> idx = kb.ThreadIndices({C, R});
			V c = idx[0], r = idx[1];
			kb.Store(E, r * C + c, Fn("exp", kb.Load(X, r * C + c, TFType_Float) - kb.Load(M, r, TFType_Float)));
			exp_kernel = kb.Finish();
		}
		if (split) {
			KernelBuilder kb(program, 2);
			V partial = kb.Buffer("partial_sum", false), E = kb.Buffer("E", true);
			V R = kb.Var("R", TFType_Int), C = kb.Var("C", TFType_Int), S = kb.Var("S", TFType_Int);
			std::vector<V> idx = kb.ThreadIndices({S, R});
			V s = idx[0], r = idx[1];
			V acc = kb.Accumulator("sum", TFType_Float, FloatBits(0.0f));
			kb.Loop(kb.Const(0), kb.Const(128), kb.Const(1), [&](V k) { kb.Set(acc, acc + SplitLoad(kb, E, r, s * kb.Const(128) + k, R, C)); });
			kb.Store(partial, r * S + s, acc);
			esum1 = kb.Finish();
		} else {
			KernelBuilder kb(program, 1);
			V out = kb.Buffer("row_sum", false), E = kb.Buffer("E", true);
			V R = kb.Var("R", TFType_Int), C = kb.Var("C", TFType_Int);
			V r = kb.ThreadIndices({R})[0];
			V acc = kb.Accumulator("sum", TFType_Float, FloatBits(0.0f));
			kb.Loop(kb.Const(0), C, kb.Const(1), [&](V k) { kb.Set(acc, acc + kb.Load(E, r * C + k, TFType_Float)); });
			kb.Store(out, r, acc);
			esum_rows = kb.Finish();
		}
		{
			KernelBuilder kb(program, 2);
			V Y = kb.Buffer("Y", false), E = kb.Buffer("E", true), Z = kb.Buffer("row_sum", true);
			V R = kb.Var("R", TFType_Int), C = kb.Var("C", TFType_Int);
			std::vector<V> idx = kb.ThreadIndices({C, R});
			V c = idx[0], r = idx[1];
			kb.Store(Y, r * C + c, kb.Load(E, r * C + c, TFType_Float) / kb.Load(Z, r, TFType_Float));
			divide = kb.Finish();
		}
	}
	HostBuilder h(program);
	h.RegionBegin("Softmax");
	V X = h.Input("X", {-1, -1}, TFType_Float);
	V R = h.Shape(X)[0], C = h.Shape(X)[1];
	V row_max, row_sum, Y, E;
	if (separate_exp) {
		V S = (C + h.Const(127)) / h.Const(128);
		row_max = h.Allocate("row_max", {R}, TFType_Float);
		if (split) {
			V chunk_max = h.Allocate("partial_max", {R, S}, TFType_Float);
			h.Dispatch(max1, {chunk_max}, {X}, {R, C, S}, {R, S});
			h.Dispatch(max2, {row_max}, {chunk_max}, {R, S}, {R});
			h.Deallocate(chunk_max);
		} else {
			h.Dispatch(max_rows, {row_max}, {X}, {R, C}, {R});
		}
		E = h.Allocate("E", {R, C}, TFType_Float);
		h.Dispatch(exp_kernel, {E}, {X, row_max}, {R, C}, {R, C});
		row_sum = h.Allocate("row_sum", {R}, TFType_Float);
		if (split) {
			V chunk_sum = h.Allocate("partial_sum", {R, S}, TFType_Float);
			h.Dispatch(esum1, {chunk_sum}, {E}, {R, C, S}, {R, S});
			h.Dispatch(sum2, {row_sum}, {chunk_sum}, {R, S}, {R});
			h.Deallocate(chunk_sum);
		} else {
			h.Dispatch(esum_rows, {row_sum}, {E}, {R, C}, {R});
		}
		Y = h.Allocate("Y", {R, C}, TFType_Float);
		h.Dispatch(divide, {Y}, {E, row_sum}, {R, C}, {R, C});
		if (!keep_exp) h.Deallocate(E);
	} else if (!split) {
		row_max = h.Allocate("row_max", {R}, TFType_Float);
		h.Dispatch(max_rows, {row_max}, {X}, {R, C}, {R});
		row_sum = h.Allocate("row_sum", {R}, TFType_Float);
		h.Dispatch(sum_rows, {row_sum}, {X, row_max}, {R, C}, {R});
		Y = h.Allocate("Y", {R, C}, TFType_Float);
		h.Dispatch(normalise, {Y}, {X, row_max, row_sum}, {R, C}, {R, C});
	} else {
		V S = (C + h.Const(127)) / h.Const(128);
		V chunk_max = h.Allocate("partial_max", {R, S}, TFType_Float);
		h.Dispatch(max1, {chunk_max}, {X}, {R, C, S}, {R, S});
		row_max = h.Allocate("row_max", {R}, TFType_Float);
		h.Dispatch(max2, {row_max}, {chunk_max}, {R, S}, {R});
		if (!late_release) h.Deallocate(chunk_max);
		V chunk_sum = h.Allocate("partial_sum", {R, S}, TFType_Float);
		h.Dispatch(sum1, {chunk_sum}, {X, row_max}, {R, C, S}, {R, S});
		row_sum = h.Allocate("row_sum", {R}, TFType_Float);
		h.Dispatch(sum2, {row_sum}, {chunk_sum}, {R, S}, {R});
		if (!late_release) h.Deallocate(chunk_sum);
		Y = h.Allocate("Y", {R, C}, TFType_Float);
		h.Dispatch(normalise, {Y}, {X, row_max, row_sum}, {R, C}, {R, C});
		if (late_release) {
			h.Deallocate(chunk_max);
			h.Deallocate(chunk_sum);
		}
	}
	h.Output(Y);
	if (separate_exp && keep_exp) h.Output(E);
	if (keep_stats) {
		h.Output(row_max);
		h.Output(row_sum);
	} else {
		h.Deallocate(row_max);
		h.Deallocate(row_sum);
	}
	h.RegionEnd("Softmax");
	h.Finish();
}

static ProgramRegistrar reg_softmax_ir("softmax_ir", BuildSoftmaxIr);

}  // namespace tfhost
