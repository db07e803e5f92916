// Small programs that exercise the emitter op by op: every operation of the post-lowering op table
// (TensorFrost/Compiler/Operations.cpp:84-178), atomics, group memory with barriers, per-thread arrays, and the
// reference's lowered reduction / scan / matmul loops in the exact forms its passes leave behind
// (Compiler/Implementations.cpp:243-359,560-646; split stage Compiler/Steps/Optimization.cpp:469-510).
#include "registry.h"

namespace tfhost {

namespace {

// Names, in output-row order, of the float / int / uint results the `ops` program produces (the test file holds
// the same lists with their NumPy formulas).
const char* kFloatOps[] = {"add", "sub", "mul", "div", "neg", "min", "max", "abs", "sign", "ceil", "floor", "round", "frac", "exp", "exp2",
                           "log", "log2", "sqrt", "rsqrt", "rcp", "sin", "cos", "tan", "asin", "acos", "atan", "sinh", "cosh", "tanh", "pow",
                           "atan2", "modf", "step", "clamp", "lerp", "fma", "smoothstep", "fmod_op", "ternary", "from_int", "from_uint", "pcgf"};
const char* kIntOps[] = {"add", "sub", "mul", "div", "mod", "lshift", "rshift", "and", "or", "xor", "not", "neg", "min", "max", "abs", "sign",
                         "clamp", "lt", "lte", "gt", "gte", "eq", "neq", "from_float", "and_bool", "or_bool", "notb", "reversebits"};
const char* kUintOps[] = {"add", "mul", "div", "mod", "lshift", "rshift", "and", "or", "xor", "not", "pcg", "reversebits", "asuint", "min", "max", "from_float"};

template <size_t N>
constexpr size_t Count(const char* (&)[N]) {
	return N;
}

}  // namespace

// inputs: x[n], y[n] float; a[n], b[n] int; u[n], w[n] uint.  outputs: F[#float ops, n], I[#int ops, n], U[#uint ops, n]
static void BuildOps(Program* program, const std::vector<int64_t>&) {
	KernelBuilder kb(program, 1);
	V F = kb.Buffer("F", false), I = kb.Buffer("I", false), U = kb.Buffer("U", false);
	V X = kb.Buffer("x", true), Y = kb.Buffer("y", true), A = kb.Buffer("a", true), B = kb.Buffer("b", true), Ub = kb.Buffer("u", true), Wb = kb.Buffer("w", true);
	V n = kb.Var("n", TFType_Int);
	V i = kb.ThreadIndices({n})[0];
	V x = kb.Named(kb.Load(X, i, TFType_Float), "x"), y = kb.Named(kb.Load(Y, i, TFType_Float), "y");
	V a = kb.Named(kb.Load(A, i, TFType_Int), "a"), b = kb.Named(kb.Load(B, i, TFType_Int), "b");
	V u = kb.Named(kb.Load(Ub, i, TFType_Uint), "u"), w = kb.Named(kb.Load(Wb, i, TFType_Uint), "w");
	V ax = kb.Named(Fn("abs", x), "ax");            // non-negative argument for log / sqrt / pow
	V ux = kb.Named(Fn("clamp", x, kb.Const(-1.0f), kb.Const(1.0f)), "unit");  // argument for asin / acos
	V sh = kb.Named(b & kb.Const(7), "shift");
	V shu = kb.Named(w & kb.ConstU(7u), "shiftu");
	V bnz = kb.Named(Select(b == kb.Const(0), kb.Const(1), b), "b_nonzero");
	V wnz = kb.Named(Select(w == kb.ConstU(0u), kb.ConstU(1u), w), "w_nonzero");
	V ynz = kb.Named(Select(y == kb.Const(0.0f), kb.Const(1.0f), y), "y_nonzero");

	std::vector<V> f = {
	    x + y, x - y, x * y, x / ynz, -x, Fn("min", x, y), Fn("max", x, y), Fn("abs", x), Fn("sign", x), Fn("ceil", x), Fn("floor", x), Fn("round", x),
	    Fn("frac", x), Fn("exp", x), Fn("exp2", x), Fn("log", ax + kb.Const(0.5f)), Fn("log2", ax + kb.Const(0.5f)), Fn("sqrt", ax),
	    Fn("rsqrt", ax + kb.Const(0.5f)), Fn("rcp", ynz), Fn("sin", x), Fn("cos", x), Fn("tan", ux), Fn("asin", ux), Fn("acos", ux), Fn("atan", x),
	    Fn("sinh", x), Fn("cosh", x), Fn("tanh", x), Fn("pow", ax + kb.Const(0.5f), y), Fn("atan2", x, y), Fn("modf", x, ynz), Fn("step", y, x),
	    Fn("clamp", x, kb.Const(-0.5f), kb.Const(0.75f)), Fn("lerp", x, y, kb.Const(0.25f)), Fn("fma", x, y, kb.Const(1.5f)),
	    Fn("smoothstep", kb.Const(-1.0f), kb.Const(2.0f), x), x % ynz, Select(x > y, x, y), ToFloat(a), ToFloat(u), Fn("pcgf", u)};
	if (f.size() != Count(kFloatOps)) throw std::runtime_error("float op list out of sync");
	for (size_t k = 0; k < f.size(); k++) kb.Store(F, kb.Const((int)k) * n + i, f[k]);

	auto as_int = [&](V cond) { return Select(cond, kb.Const(1), kb.Const(0)); };
	std::vector<V> g = {
	    a + b, a - b, a * b, a / bnz, a % bnz, a << sh, a >> sh, a & b, a | b, a ^ b, ~a, -a, Fn("min", a, b), Fn("max", a, b), Fn("abs", a), Fn("sign", a),
	    Fn("clamp", a, kb.Const(-100), kb.Const(1000)), as_int(a < b), as_int(a <= b), as_int(a > b), as_int(a >= b), as_int(a == b), as_int(a != b),
	    ToInt(x * kb.Const(100.0f)), as_int((a < b) && (x < y)), as_int((a < b) || (x < y)), as_int(!(a < b)), Fn("reversebits", a)};
	if (g.size() != Count(kIntOps)) throw std::runtime_error("int op list out of sync");
	for (size_t k = 0; k < g.size(); k++) kb.Store(I, kb.Const((int)k) * n + i, g[k]);

	std::vector<V> h = {u + w, u * w, u / wnz, u % wnz, u << shu, u >> shu, u & w, u | w, u ^ w, ~u, Fn("pcg", u), Fn("reversebits", u), AsUint(x),
	                    Fn("min", u, w), Fn("max", u, w), ToUint(ax * kb.Const(1000.0f))};
	if (h.size() != Count(kUintOps)) throw std::runtime_error("uint op list out of sync");
	for (size_t k = 0; k < h.size(); k++) kb.Store(U, kb.Const((int)k) * n + i, h[k]);
	Kernel* kernel = kb.Finish();

	{  // the host part of the tree; its names shadow the kernel's
		HostBuilder h(program);
		const TFType types[6] = {TFType_Float, TFType_Float, TFType_Int, TFType_Int, TFType_Uint, TFType_Uint};
		const char* names[6] = {"x", "y", "a", "b", "u", "w"};
		std::vector<V> in;
		V n;
		for (int t = 0; t < 6; t++) {
			in.push_back(t == 0 ? h.Input(names[t], {-1}, types[t]) : h.Input(names[t], {n}, types[t]));
			if (t == 0) n = h.Shape(in[0])[0];
		}
		V F = h.Allocate("F", {Count(kFloatOps), n}, TFType_Float);
		V I = h.Allocate("I", {Count(kIntOps), n}, TFType_Int);
		V U = h.Allocate("U", {Count(kUintOps), n}, TFType_Uint);
		h.Dispatch(kernel, {F, I, U}, in, {n}, {n});
		for (V out : {F, I, U}) h.Output(out);
		h.Finish();
	}
}

// Scatter atomics. input: keys[n] uint in [0, bins), vals[n] float, ints[n] int.
// outputs: hist[bins] (InterlockedAdd uint), fsum[bins] (float add), imax[bins], imin[bins] (int), bits[3] (and, or, xor of all
// keys), tickets[n] (InterlockedAdd_Prev on one counter: a permutation of 0..n-1), fmax[bins], fmin[bins] (float max/min)
static void BuildAtomics(Program* program, const std::vector<int64_t>& params) {
	const int bins = params.empty() ? 16 : (int)params[0];
	// kernel 0: initialise the outputs
	Kernel* init;
	{
		KernelBuilder kb(program, 1);
		V hist = kb.Buffer("hist", false), fsum = kb.Buffer("fsum", false), imax = kb.Buffer("imax", false), imin = kb.Buffer("imin", false);
		V bits = kb.Buffer("bits", false), counter = kb.Buffer("counter", false), fmax = kb.Buffer("fmax", false), fmin = kb.Buffer("fmin", false);
		V nb = kb.Var("bins", TFType_Int);
		V i = kb.ThreadIndices({nb})[0];
		kb.Store(hist, i, kb.ConstU(0u));
		kb.Store(fsum, i, kb.Const(0.0f));
		kb.Store(imax, i, kb.Const((int)0x80000000));
		kb.Store(imin, i, kb.Const(0x7FFFFFFF));
		kb.Store(fmax, i, kb.Const(-3.402823466e+38f));
		kb.Store(fmin, i, kb.Const(3.402823466e+38f));
		kb.If(i == kb.Const(0), [&] {
			kb.Store(bits, kb.Const(0), kb.ConstU(0xFFFFFFFFu));
			kb.Store(bits, kb.Const(1), kb.ConstU(0u));
			kb.Store(bits, kb.Const(2), kb.ConstU(0u));
			kb.Store(counter, kb.Const(0), kb.ConstU(0u));
		});
		init = kb.Finish();
	}
	Kernel* scatter;
	{
		KernelBuilder kb(program, 1);
		V hist = kb.Buffer("hist", false), fsum = kb.Buffer("fsum", false), imax = kb.Buffer("imax", false), imin = kb.Buffer("imin", false);
		V bits = kb.Buffer("bits", false), counter = kb.Buffer("counter", false), tickets = kb.Buffer("tickets", false);
		V fmax = kb.Buffer("fmax", false), fmin = kb.Buffer("fmin", false);
		V keys = kb.Buffer("keys", true), vals = kb.Buffer("vals", true), ints = kb.Buffer("ints", true);
		V n = kb.Var("n", TFType_Int);
		V i = kb.ThreadIndices({n})[0];
		V key = kb.Named(kb.Load(keys, i, TFType_Uint), "key");
		V bin = kb.Named(ToInt(key), "bin");
		V val = kb.Load(vals, i, TFType_Float);
		V iv = kb.Load(ints, i, TFType_Int);
		kb.Atomic("InterlockedAdd", hist, bin, kb.ConstU(1u));
		kb.Atomic("InterlockedAdd", fsum, bin, val);
		kb.Atomic("InterlockedMax", imax, bin, iv);
		kb.Atomic("InterlockedMin", imin, bin, iv);
		kb.Atomic("InterlockedMax", fmax, bin, val);
		kb.Atomic("InterlockedMin", fmin, bin, val);
		kb.Atomic("InterlockedAnd", bits, kb.Const(0), key | kb.ConstU(0xFFFFFF00u));
		kb.Atomic("InterlockedOr", bits, kb.Const(1), key);
		kb.Atomic("InterlockedXor", bits, kb.Const(2), key);
		V ticket = kb.Atomic("InterlockedAdd_Prev", counter, kb.Const(0), kb.ConstU(1u), true);
		kb.Store(tickets, i, ticket);
		scatter = kb.Finish();
	}
	{  // the host part of the tree; its names shadow the kernel's
		HostBuilder h(program);
		V keys = h.Input("keys", {-1}, TFType_Uint);
		V n = h.Shape(keys)[0];
		V vals = h.Input("vals", {n}, TFType_Float);
		V ints = h.Input("ints", {n}, TFType_Int);
		V hist = h.Allocate("hist", {bins}, TFType_Uint), fsum = h.Allocate("fsum", {bins}, TFType_Float);
		V imax = h.Allocate("imax", {bins}, TFType_Int), imin = h.Allocate("imin", {bins}, TFType_Int);
		V bits = h.Allocate("bits", {3}, TFType_Uint), counter = h.Allocate("counter", {1}, TFType_Uint);
		V tickets = h.Allocate("tickets", {n}, TFType_Uint);
		V fmax = h.Allocate("fmax", {bins}, TFType_Float), fmin = h.Allocate("fmin", {bins}, TFType_Float);
		h.Dispatch(init, {hist, fsum, imax, imin, bits, counter, fmax, fmin}, {}, {h.Const(bins)}, {bins});
		h.Dispatch(scatter, {hist, fsum, imax, imin, bits, counter, tickets, fmax, fmin}, {keys, vals, ints}, {n}, {n});
		h.Deallocate(counter);
		for (V out : {hist, fsum, imax, imin, bits, tickets, fmax, fmin}) h.Output(out);
		h.Finish();
	}
}

// Group memory + barrier + per-thread array: out[g*128 + e] = in[g*128 + 127 - e] + sum of a 4-element local array.
// Kernel shape [G, 128], group {128} as `tf.kernel(shape, group_size=[128])` gives it.
static void BuildGroupReverse(Program* program, const std::vector<int64_t>&) {
	KernelBuilder kb(program, 2, {128});
	V out = kb.Buffer("result", false);
	V in = kb.Buffer("data", true);
	V G = kb.Var("G", TFType_Int);
	std::vector<V> idx = kb.ThreadIndices({kb.Const(128), G});
	V e = idx[0], g = idx[1];
	V tile = kb.GroupMemory("tile", TFType_Float, 128);
	V local = kb.LocalMemory("scratch", TFType_Float, 4);
	V gtid = kb.BlockThreadId(0);
	kb.Store(tile, gtid, kb.Load(in, g * kb.Const(128) + e, TFType_Float));
	kb.Barrier();
	kb.Loop(kb.Const(0), kb.Const(4), kb.Const(1), [&](V k) { kb.Store(local, k, ToFloat(k) * kb.Const(0.25f)); });
	V acc = kb.Accumulator("local_total", TFType_Float, FloatBits(0.0f));
	kb.Loop(kb.Const(0), kb.Const(4), kb.Const(1), [&](V k) { kb.Set(acc, acc + kb.Load(local, k, TFType_Float)); });
	V mirrored = kb.Load(tile, kb.Const(127) - gtid, TFType_Float);
	kb.Store(out, g * kb.Const(128) + e, mirrored + acc);
	Kernel* kernel = kb.Finish();
	{  // the host part of the tree; its names shadow the kernel's
		HostBuilder h(program);
		V data = h.Input("data", {-1, 128}, TFType_Float);
		V groups = h.Shape(data)[0];
		V result = h.Allocate("result", {groups, 128}, TFType_Float);
		h.Dispatch(kernel, {result}, {data}, {groups}, {groups, 128});
		h.Output(result);
		h.Finish();
	}
}

// The frame of the reference's tiled matrix product (examples/Algorithms/matrix_mul.ipynb): a kernel of shape
// [N/4, K/4] with 16x16 groups and group memory, `tf.kernel([N / TBK, K / TBK], group_size=[GK, GK])`. Every thread
// records where it is: ids[i1, i0] = i1 * 65536 + i0 and tiles[i1, i0] = gx * 65536 + gy with gx = i1 - tx, gy = i0 - ty,
// tx = block_thread_index(1), ty = block_thread_index(0), read back through group memory.
static void BuildTileIndices(Program* program, const std::vector<int64_t>&) {
	KernelBuilder kb(program, 2, {16, 16});
	V ids = kb.Buffer("ids", false), tiles = kb.Buffer("tiles", false);
	V N = kb.Var("N", TFType_Int), K = kb.Var("K", TFType_Int);
	V Kq = kb.Named(K / kb.Const(4), "vdiv"), Nq = kb.Named(N / kb.Const(4), "vdiv");
	std::vector<V> idx = kb.ThreadIndices({Kq, Nq});
	V i0 = idx[0], i1 = idx[1];
	V tile = kb.GroupMemory("tile", TFType_Int, 256);
	V tx = kb.Named(kb.BlockThreadId(1), "tx"), ty = kb.Named(kb.BlockThreadId(0), "ty");
	V gx = kb.Named(i1 - tx, "gx"), gy = kb.Named(i0 - ty, "gy");
	kb.Store(tile, tx * kb.Const(16) + ty, gx * kb.Const(65536) + gy);
	kb.Barrier();
	kb.Store(ids, i1 * Kq + i0, i1 * kb.Const(65536) + i0);
	kb.Store(tiles, i1 * Kq + i0, kb.Load(tile, tx * kb.Const(16) + ty, TFType_Int));
	Kernel* kernel = kb.Finish();
	{  // the host part of the tree; its names shadow the kernel's
		HostBuilder h(program);
		V Cm = h.Input("C", {-1, -1}, TFType_Float);
		V n = h.Shape(Cm)[0], k = h.Shape(Cm)[1];
		h.AssertValue("tile_indices: the kernel shape [N/4, K/4] is empty", (n >= h.Const(4)) && (k >= h.Const(4)));
		V nq = n / h.Const(4), kq = k / h.Const(4);
		V ids_t = h.Allocate("ids", {nq, kq}, TFType_Int);
		V tiles_t = h.Allocate("tiles", {nq, kq}, TFType_Int);
		h.Dispatch(kernel, {ids_t, tiles_t}, {}, {n, k}, {nq, kq});
		h.Output(ids_t);
		h.Output(tiles_t);
		h.Finish();
	}
}

// The reference's lowered reductions, scan and matmul on X[R, C], emitted (not served by primitives):
// outputs: sum over the last axis (unsplit loop), max over the last axis via the 128-chunk split (two kernels),
// sum over axis 0 (unsplit, strided loop), prefix sum along the last axis, X * W for W[C, N], max over axis 0 via the split.
static void BuildLoweredIdioms(Program* program, const std::vector<int64_t>&) {
	// k0: sum over the last axis, kernel shape [R]
	Kernel* k_sum_last;
	{
		KernelBuilder kb(program, 1);
		V out = kb.Buffer("sum_last", false), X = kb.Buffer("X", true);
		V R = kb.Var("R", TFType_Int), C = kb.Var("C", TFType_Int);
		V r = kb.ThreadIndices({R})[0];
		V acc = kb.Accumulator("sum", TFType_Float, FloatBits(0.0f));
		kb.Loop(kb.Const(0), C, kb.Const(1), [&](V k) { kb.Set(acc, acc + kb.Load(X, r * C + k, TFType_Float)); });
		kb.Store(out, r, acc);
		k_sum_last = kb.Finish();
	}
	// k1: stage 1 of the split max, kernel shape [R, S] with S = ceil(C/128): partial[r, s] = max_k split(r, s*128+k)
	Kernel* k_max_stage1;
	{
		KernelBuilder kb(program, 2);
		V partial = kb.Buffer("partial", false), X = kb.Buffer("X", true);
		V R = kb.Var("R", TFType_Int), C = kb.Var("C", TFType_Int), S = kb.Var("S", TFType_Int);
		std::vector<V> idx = kb.ThreadIndices({S, R});
		V s = idx[0], r = idx[1];
		V acc = kb.Accumulator("max", TFType_Float, FloatBits(-3.402823466e+38f));
		kb.Loop(kb.Const(0), kb.Const(128), kb.Const(1), [&](V k) {
			V merged = kb.Named(s * kb.Const(128) + k, "merged");
			// ConstantOutOfBounds (Implementations.cpp:56-69): false || (i < 0 || i >= n) for every dimension
			V oob = kb.Named((kb.ConstB(false) || ((r < kb.Const(0)) || (r >= R))) || ((merged < kb.Const(0)) || (merged >= C)), "out_of_bounds");
			V x = kb.Load(X, kb.Clamp(r, kb.Const(0), R - kb.Const(1)) * C + kb.Clamp(merged, kb.Const(0), C - kb.Const(1)), TFType_Float);
			V split = kb.Named(Select(oob, kb.Const(0.0f), x), "split");
			kb.Set(acc, Fn("max", acc, split));
		});
		kb.Store(partial, r * S + s, acc);
		k_max_stage1 = kb.Finish();
	}
	// k2: stage 2, kernel shape [R]: max over the S partials
	Kernel* k_max_stage2;
	{
		KernelBuilder kb(program, 1);
		V out = kb.Buffer("max_last", false), partial = kb.Buffer("partial", true);
		V R = kb.Var("R", TFType_Int), S = kb.Var("S", TFType_Int);
		V r = kb.ThreadIndices({R})[0];
		V acc = kb.Accumulator("max", TFType_Float, FloatBits(-3.402823466e+38f));
		kb.Loop(kb.Const(0), S, kb.Const(1), [&](V k) { kb.Set(acc, Fn("max", acc, kb.Load(partial, r * S + k, TFType_Float))); });
		kb.Store(out, r, acc);
		k_max_stage2 = kb.Finish();
	}
	// k2b/k2c: max over axis 0 through the same split: stage 1 has kernel shape [S0, C] with S0 = ceil(R/128) and walks
	// 128 rows of its chunk; stage 2 reduces the S0 partial rows
	Kernel* k_max0_stage1;
	{
		KernelBuilder kb(program, 2);
		V partial = kb.Buffer("partial0", false), X = kb.Buffer("X", true);
		V R = kb.Var("R", TFType_Int), C = kb.Var("C", TFType_Int), S0 = kb.Var("S0", TFType_Int);
		std::vector<V> idx = kb.ThreadIndices({C, S0});
		V c = idx[0], s = idx[1];
		V acc = kb.Accumulator("max", TFType_Float, FloatBits(-3.402823466e+38f));
		kb.Loop(kb.Const(0), kb.Const(128), kb.Const(1), [&](V k) {
			V merged = kb.Named(s * kb.Const(128) + k, "merged");
			V oob = kb.Named((kb.ConstB(false) || ((merged < kb.Const(0)) || (merged >= R))) || ((c < kb.Const(0)) || (c >= C)), "out_of_bounds");
			V x = kb.Load(X, kb.Clamp(merged, kb.Const(0), R - kb.Const(1)) * C + kb.Clamp(c, kb.Const(0), C - kb.Const(1)), TFType_Float);
			V split = kb.Named(Select(oob, kb.Const(0.0f), x), "split");
			kb.Set(acc, Fn("max", acc, split));
		});
		kb.Store(partial, s * C + c, acc);
		k_max0_stage1 = kb.Finish();
	}
	Kernel* k_max0_stage2;
	{
		KernelBuilder kb(program, 1);
		V out = kb.Buffer("max_first", false), partial = kb.Buffer("partial0", true);
		V C = kb.Var("C", TFType_Int), S0 = kb.Var("S0", TFType_Int);
		V c = kb.ThreadIndices({C})[0];
		V acc = kb.Accumulator("max", TFType_Float, FloatBits(-3.402823466e+38f));
		kb.Loop(kb.Const(0), S0, kb.Const(1), [&](V k) { kb.Set(acc, Fn("max", acc, kb.Load(partial, k * C + c, TFType_Float))); });
		kb.Store(out, c, acc);
		k_max0_stage2 = kb.Finish();
	}
	// k3: sum over axis 0, kernel shape [C]: strided loop
	Kernel* k_sum_first;
	{
		KernelBuilder kb(program, 1);
		V out = kb.Buffer("sum_first", false), X = kb.Buffer("X", true);
		V R = kb.Var("R", TFType_Int), C = kb.Var("C", TFType_Int);
		V c = kb.ThreadIndices({C})[0];
		V acc = kb.Accumulator("sum", TFType_Float, FloatBits(0.0f));
		kb.Loop(kb.Const(0), R, kb.Const(1), [&](V k) { kb.Set(acc, acc + kb.Load(X, k * C + c, TFType_Float)); });
		kb.Store(out, c, acc);
		k_sum_first = kb.Finish();
	}
	// k4: prefix sum along the last axis, kernel shape [R]
	Kernel* k_scan;
	{
		KernelBuilder kb(program, 1);
		V out = kb.Buffer("scanned", false), X = kb.Buffer("X", true);
		V R = kb.Var("R", TFType_Int), C = kb.Var("C", TFType_Int);
		V r = kb.ThreadIndices({R})[0];
		V acc = kb.Accumulator("prefix_sum", TFType_Float, FloatBits(0.0f));
		kb.Loop(kb.Const(0), C, kb.Const(1), [&](V k) {
			kb.Set(acc, acc + kb.Load(X, r * C + k, TFType_Float));
			kb.Store(out, r * C + k, acc);
		});
		k_scan = kb.Finish();
	}
	// k5: matmul X[R,C] * W[C,N], kernel shape [R, N]
	Kernel* k_matmul;
	{
		KernelBuilder kb(program, 2);
		V out = kb.Buffer("product", false), X = kb.Buffer("X", true), W = kb.Buffer("W", true);
		V R = kb.Var("R", TFType_Int), C = kb.Var("C", TFType_Int), N = kb.Var("N", TFType_Int);
		std::vector<V> idx = kb.ThreadIndices({N, R});
		V j = idx[0], i = idx[1];
		V acc = kb.Accumulator("matmul", TFType_Float, FloatBits(0.0f));
		kb.Loop(kb.Const(0), C, kb.Const(1), [&](V k) {
			V a = kb.Load(X, i * C + k, TFType_Float);
			V b = kb.Load(W, k * N + j, TFType_Float);
			kb.Set(acc, acc + a * b);
		});
		kb.Store(out, i * N + j, acc);
		k_matmul = kb.Finish();
	}
	{  // the host part of the tree; its names shadow the kernel's
		HostBuilder h(program);
		V X = h.Input("X", {-1, -1}, TFType_Float);
		V R = h.Shape(X)[0], C = h.Shape(X)[1];
		V W = h.Input("W", {C, -1}, TFType_Float);
		V N = h.Shape(W)[1];
		V S = (C + h.Const(127)) / h.Const(128);
		V sum_last = h.Allocate("sum_last", {R}, TFType_Float);
		h.Dispatch(k_sum_last, {sum_last}, {X}, {R, C}, {R});
		V partial = h.Allocate("partial", {R, S}, TFType_Float);
		h.Dispatch(k_max_stage1, {partial}, {X}, {R, C, S}, {R, S});
		V max_last = h.Allocate("max_last", {R}, TFType_Float);
		h.Dispatch(k_max_stage2, {max_last}, {partial}, {R, S}, {R});
		h.Deallocate(partial);
		V S0 = (R + h.Const(127)) / h.Const(128);
		V partial0 = h.Allocate("partial0", {S0, C}, TFType_Float);
		h.Dispatch(k_max0_stage1, {partial0}, {X}, {R, C, S0}, {S0, C});
		V max_first = h.Allocate("max_first", {C}, TFType_Float);
		h.Dispatch(k_max0_stage2, {max_first}, {partial0}, {C, S0}, {C});
		h.Deallocate(partial0);
		V sum_first = h.Allocate("sum_first", {C}, TFType_Float);
		h.Dispatch(k_sum_first, {sum_first}, {X}, {R, C}, {C});
		V scanned = h.Allocate("scanned", {R, C}, TFType_Float);
		h.Dispatch(k_scan, {scanned}, {X}, {R, C}, {R});
		V product = h.Allocate("product", {R, N}, TFType_Float);
		h.Dispatch(k_matmul, {product}, {X, W}, {R, C, N}, {R, N});
		for (V out : {sum_last, max_last, sum_first, scanned, product, max_first}) h.Output(out);
		h.Finish();
	}
}

// Loops whose loads do not depend on the thread (every thread walks the same table): out_sum[i] = sum_k T[k]*x[i],
// out_max[i] = max_k (T[k] - x[i]), out_count[i] = #{k : Ti[k] > a[i]}, k in [first, K).
static void BuildBroadcastLoops(Program* program, const std::vector<int64_t>&) {
	KernelBuilder kb(program, 1);
	V out_sum = kb.Buffer("out_sum", false), out_max = kb.Buffer("out_max", false), out_count = kb.Buffer("out_count", false);
	V X = kb.Buffer("x", true), A = kb.Buffer("a", true), T = kb.Buffer("table", true), Ti = kb.Buffer("itable", true);
	V n = kb.Var("n", TFType_Int), first = kb.Var("first", TFType_Int), K = kb.Var("K", TFType_Int);
	V i = kb.ThreadIndices({n})[0];
	V x = kb.Named(kb.Load(X, i, TFType_Float), "x"), a = kb.Named(kb.Load(A, i, TFType_Int), "a");
	V sum = kb.Accumulator("total", TFType_Float, FloatBits(0.0f));
	V mx = kb.Accumulator("largest", TFType_Float, FloatBits(-3.402823466e+38f));
	V count = kb.Accumulator("count", TFType_Int, 0);
	kb.Loop(first, K, kb.Const(1), [&](V k) {
		V t = kb.Named(kb.Load(T, k, TFType_Float), "t");
		V ti = kb.Named(kb.Load(Ti, k, TFType_Int), "ti");
		kb.Set(sum, sum + t * x);
		kb.Set(mx, Fn("max", mx, t - x));
		kb.Set(count, count + Select(ti > a, kb.Const(1), kb.Const(0)));
	});
	kb.Store(out_sum, i, sum);
	kb.Store(out_max, i, mx);
	kb.Store(out_count, i, count);
	Kernel* kernel = kb.Finish();
	{  // the host part of the tree; its names shadow the kernel's
		HostBuilder h(program);
		V x = h.Input("x", {-1}, TFType_Float);
		V n = h.Shape(x)[0];
		V a = h.Input("a", {n}, TFType_Int);
		V table = h.Input("table", {-1}, TFType_Float);
		V K = h.Shape(table)[0];
		V itable = h.Input("itable", {K}, TFType_Int);
		V first_t = h.Input("first", {1}, TFType_Int);
		V first = h.Read(first_t, h.Const(0), TFType_Int);
		V s = h.Allocate("out_sum", {n}, TFType_Float), m = h.Allocate("out_max", {n}, TFType_Float);
		V c = h.Allocate("out_count", {n}, TFType_Int);
		h.Dispatch(kernel, {s, m, c}, {x, a, table, itable}, {n, first, K}, {n});
		for (V out : {s, m, c}) h.Output(out);
		h.Finish();
	}
}

// Index decoding of 3-D and 4-D kernels (groups 8x8x8; a fourth, outer dimension has no group extent,
// GraphOps.cpp:1143-1166) with clamped, periodic and transposed addressing.
// input data[B, D, H, W]; outputs: shifted[b,z,y,x] = data[b, clamp(z-1), (y+1)%H, clamp(x+2)],
// transposed[b,x,y,z] = data[b,z,y,x], ids[b,z,y,x] = flat index.  params[0] = 3 or 4 dimensions (3: B must be 1).
static void BuildIndexing(Program* program, const std::vector<int64_t>& params) {
	const int dims = params.empty() ? 3 : (int)params[0];
	if (dims != 3 && dims != 4) throw std::runtime_error("indexing: 3 or 4 dimensions");
	KernelBuilder kb(program, dims);
	V shifted = kb.Buffer("shifted", false), transposed = kb.Buffer("transposed", false), ids = kb.Buffer("ids", false);
	V data = kb.Buffer("data", true);
	V B = kb.Var("B", TFType_Int), D = kb.Var("D", TFType_Int), H = kb.Var("H", TFType_Int), W = kb.Var("W", TFType_Int);
	std::vector<V> shape = {W, H, D};
	if (dims == 4) shape.push_back(B);
	std::vector<V> idx = kb.ThreadIndices(shape);
	V x = idx[0], y = idx[1], z = idx[2];
	V b = dims == 4 ? idx[3] : kb.Const(0);
	auto flat = [&](V bb, V zz, V yy, V xx) { return ((bb * D + zz) * H + yy) * W + xx; };
	V here = kb.Named(flat(b, z, y, x), "here");
	V value = kb.Named(kb.Load(data, here, TFType_Float), "value");
	V zc = kb.Clamp(z - kb.Const(1), kb.Const(0), D - kb.Const(1));
	V yp = (y + kb.Const(1)) % H;
	V xc = kb.Clamp(x + kb.Const(2), kb.Const(0), W - kb.Const(1));
	kb.Store(shifted, here, kb.Load(data, flat(b, zc, yp, xc), TFType_Float));
	kb.Store(transposed, ((b * W + x) * H + y) * D + z, value);
	kb.Store(ids, here, here);
	Kernel* kernel = kb.Finish();
	{  // the host part of the tree; its names shadow the kernel's
		HostBuilder h(program);
		V data_t = h.Input("data", {-1, -1, -1, -1}, TFType_Float);
		std::vector<V> e = h.Shape(data_t);
		V Bn = e[0], Dn = e[1], Hn = e[2], Wn = e[3];
		if (dims == 3) h.AssertValue("indexing: the 3-D form takes B = 1", Bn == h.Const(1));
		V shifted_t = h.Allocate("shifted", {Bn, Dn, Hn, Wn}, TFType_Float);
		V transposed_t = h.Allocate("transposed", {Bn, Wn, Hn, Dn}, TFType_Float);
		V ids_t = h.Allocate("ids", {Bn, Dn, Hn, Wn}, TFType_Int);
		if (dims == 3)
			h.Dispatch(kernel, {shifted_t, transposed_t, ids_t}, {data_t}, {Bn, Dn, Hn, Wn}, {Dn, Hn, Wn});
		else
			h.Dispatch(kernel, {shifted_t, transposed_t, ids_t}, {data_t}, {Bn, Dn, Hn, Wn}, {Bn, Dn, Hn, Wn});
		for (V out : {shifted_t, transposed_t, ids_t}) h.Output(out);
		h.Finish();
	}
}

// A dense layer as kernel fusion leaves it: the matmul loop followed, in the same kernel, by its element-wise tail.
// inputs X[M,K], W[K,N], bias[N], G[M,N] (an upstream gradient).
// outputs: H = max(X W + bias, 0); Y = X W + bias; dX = (G W^T) where X > 0 else 0   (dX[M,K], the mask laid out like dX)
static void BuildDenseLayer(Program* program, const std::vector<int64_t>&) {
	auto forward = [&](bool relu) {
		KernelBuilder kb(program, 2);
		V out = kb.Buffer(relu ? "H" : "Y", false), X = kb.Buffer("X", true), W = kb.Buffer("W", true), bias = kb.Buffer("bias", true);
		V M = kb.Var("M", TFType_Int), N = kb.Var("N", TFType_Int), K = kb.Var("K", TFType_Int);
		std::vector<V> idx = kb.ThreadIndices({N, M});
		V j = idx[0], i = idx[1];
		V acc = kb.Accumulator("matmul", TFType_Float, FloatBits(0.0f));
		kb.Loop(kb.Const(0), K, kb.Const(1), [&](V k) { kb.Set(acc, acc + kb.Load(X, i * K + k, TFType_Float) * kb.Load(W, k * N + j, TFType_Float)); });
		V z = acc + kb.Load(bias, j, TFType_Float);
		kb.Store(out, i * N + j, relu ? Fn("max", z, kb.Const(0.0f)) : z);
		return kb.Finish();
	};
	Kernel* k_relu = forward(true);
	Kernel* k_linear = forward(false);
	Kernel* k_backward;
	{
		KernelBuilder kb(program, 2);
		V dX = kb.Buffer("dX", false), G = kb.Buffer("G", true), W = kb.Buffer("W", true), X = kb.Buffer("X", true);
		V M = kb.Var("M", TFType_Int), N = kb.Var("N", TFType_Int), K = kb.Var("K", TFType_Int);
		std::vector<V> idx = kb.ThreadIndices({K, M});
		V c = idx[0], i = idx[1];
		V acc = kb.Accumulator("matmul", TFType_Float, FloatBits(0.0f));
		kb.Loop(kb.Const(0), N, kb.Const(1), [&](V n) { kb.Set(acc, acc + kb.Load(G, i * N + n, TFType_Float) * kb.Load(W, c * N + n, TFType_Float)); });
		V x = kb.Load(X, i * K + c, TFType_Float);
		kb.Store(dX, i * K + c, Select(x > kb.Const(0.0f), acc, kb.Const(0.0f)));
		k_backward = kb.Finish();
	}
	{  // the host part of the tree; its names shadow the kernel's
		HostBuilder h(program);
		V X = h.Input("X", {-1, -1}, TFType_Float);
		V M = h.Shape(X)[0], K = h.Shape(X)[1];
		V W = h.Input("W", {K, -1}, TFType_Float);
		V N = h.Shape(W)[1];
		V bias = h.Input("bias", {N}, TFType_Float);
		V G = h.Input("G", {M, N}, TFType_Float);
		V H = h.Allocate("H", {M, N}, TFType_Float), Y = h.Allocate("Y", {M, N}, TFType_Float), dX = h.Allocate("dX", {M, K}, TFType_Float);
		h.Dispatch(k_relu, {H}, {X, W, bias}, {M, N, K}, {M, N});
		h.Dispatch(k_linear, {Y}, {X, W, bias}, {M, N, K}, {M, N});
		h.Dispatch(k_backward, {dX}, {G, W, X}, {M, N, K}, {M, K});
		for (V out : {H, Y, dX}) h.Output(out);
		h.Finish();
	}
}

// Matmul with a leading batch dimension as the reference lowers it (Compiler/Implementations.cpp:575-633): kernel
// shape [T, M, N], the batch index appended to the indices of every operand that has the dimension.
// inputs A[T, M, K], B[T, K, N], W[K, N].  outputs: P[t] = A[t] B[t];  Q[t] = A[t] W (W shared by the batch).
static void BuildBatchedMatmul(Program* program, const std::vector<int64_t>&) {
	auto build = [&](bool shared_b) {
		KernelBuilder kb(program, 3);
		V C = kb.Buffer(shared_b ? "Q" : "P", false), A = kb.Buffer("A", true), B = kb.Buffer(shared_b ? "W" : "B", true);
		V T = kb.Var("T", TFType_Int), M = kb.Var("M", TFType_Int), N = kb.Var("N", TFType_Int), K = kb.Var("K", TFType_Int);
		std::vector<V> idx = kb.ThreadIndices({N, M, T});
		V j = idx[0], i = idx[1], t = idx[2];
		V acc = kb.Accumulator("matmul", TFType_Float, FloatBits(0.0f));
		kb.Loop(kb.Const(0), K, kb.Const(1), [&](V k) {
			V a = kb.Load(A, (t * M + i) * K + k, TFType_Float);
			V b = shared_b ? kb.Load(B, k * N + j, TFType_Float) : kb.Load(B, (t * K + k) * N + j, TFType_Float);
			kb.Set(acc, acc + a * b);
		});
		kb.Store(C, (t * M + i) * N + j, acc);
		return kb.Finish();
	};
	Kernel* both = build(false);
	Kernel* shared = build(true);
	{  // the host part of the tree; its names shadow the kernel's
		HostBuilder h(program);
		V A = h.Input("A", {-1, -1, -1}, TFType_Float);
		V T = h.Shape(A)[0], M = h.Shape(A)[1], K = h.Shape(A)[2];
		V B = h.Input("B", {T, K, -1}, TFType_Float);
		V N = h.Shape(B)[2];
		V W = h.Input("W", {K, N}, TFType_Float);
		V P = h.Allocate("P", {T, M, N}, TFType_Float), Q = h.Allocate("Q", {T, M, N}, TFType_Float);
		h.Dispatch(both, {P}, {A, B}, {T, M, N, K}, {T, M, N});
		h.Dispatch(shared, {Q}, {A, W}, {T, M, N, K}, {T, M, N});
		h.Output(P);
		h.Output(Q);
		h.Finish();
	}
}

// A dense layer with a tanh activation, forward and backward, as kernel fusion leaves it: matmul loops followed by
// element-wise tails that are none of the fixed fused forms (two stores; a product with loaded values).
// inputs X[M,K], W[K,N], bias[N], R[M,N] (a residual), G[M,N] (an upstream gradient).
// outputs: Z = X W + bias;  H = tanh(Z) + R  (one kernel, two stores);  dX = (G * (1 - tanh(Z)^2)) W^T is NOT this --
// the backward kernel here is dX[i, c] = (sum_n G[i,n] W[c,n]) * (1 - X[i,c]^2) * scale, scale a host scalar.
static void BuildDenseTanh(Program* program, const std::vector<int64_t>&) {
	Kernel* k_forward;
	{
		KernelBuilder kb(program, 2);
		V Z = kb.Buffer("Z", false), H = kb.Buffer("H", false), X = kb.Buffer("X", true), W = kb.Buffer("W", true), bias = kb.Buffer("bias", true),
		  R = kb.Buffer("R", true);
		V M = kb.Var("M", TFType_Int), N = kb.Var("N", TFType_Int), K = kb.Var("K", TFType_Int);
		std::vector<V> idx = kb.ThreadIndices({N, M});
		V j = idx[0], i = idx[1];
		V acc = kb.Accumulator("matmul", TFType_Float, FloatBits(0.0f));
		kb.Loop(kb.Const(0), K, kb.Const(1), [&](V k) { kb.Set(acc, acc + kb.Load(X, i * K + k, TFType_Float) * kb.Load(W, k * N + j, TFType_Float)); });
		V z = kb.Named(acc + kb.Load(bias, j, TFType_Float), "z");
		kb.Store(Z, i * N + j, z);
		kb.Store(H, i * N + j, Fn("tanh", z) + kb.Load(R, i * N + j, TFType_Float));
		k_forward = kb.Finish();
	}
	Kernel* k_backward;
	{
		KernelBuilder kb(program, 2);
		V dX = kb.Buffer("dX", false), G = kb.Buffer("G", true), W = kb.Buffer("W", true), X = kb.Buffer("X", true);
		V M = kb.Var("M", TFType_Int), N = kb.Var("N", TFType_Int), K = kb.Var("K", TFType_Int), scale = kb.Var("scale", TFType_Float);
		std::vector<V> idx = kb.ThreadIndices({K, M});
		V c = idx[0], i = idx[1];
		V acc = kb.Accumulator("matmul", TFType_Float, FloatBits(0.0f));
		kb.Loop(kb.Const(0), N, kb.Const(1), [&](V n) { kb.Set(acc, acc + kb.Load(G, i * N + n, TFType_Float) * kb.Load(W, c * N + n, TFType_Float)); });
		V x = kb.Load(X, i * K + c, TFType_Float);
		kb.Store(dX, i * K + c, acc * (kb.Const(1.0f) - x * x) * scale);
		k_backward = kb.Finish();
	}
	{  // the host part of the tree; its names shadow the kernel's
		HostBuilder h(program);
		V X = h.Input("X", {-1, -1}, TFType_Float);
		V M = h.Shape(X)[0], K = h.Shape(X)[1];
		V W = h.Input("W", {K, -1}, TFType_Float);
		V N = h.Shape(W)[1];
		V bias = h.Input("bias", {N}, TFType_Float);
		V R = h.Input("R", {M, N}, TFType_Float);
		V G = h.Input("G", {M, N}, TFType_Float);
		V Z = h.Allocate("Z", {M, N}, TFType_Float), H = h.Allocate("H", {M, N}, TFType_Float), dX = h.Allocate("dX", {M, K}, TFType_Float);
		h.Dispatch(k_forward, {Z, H}, {X, W, bias, R}, {M, N, K}, {M, N});
		h.Dispatch(k_backward, {dX}, {G, W, X}, {M, N, K, h.Const(0.5f)}, {M, K});
		for (V out : {Z, H, dX}) h.Output(out);
		h.Finish();
	}
}

// The scatter kernel of one pass of the reference's radix sort, GPU branch (Python/TensorFrost/sort.py:133-169), as its
// tf.kernel(grouped.shape, group_size=[128]) lowers: two group buffers, barriers (the second one inside the bounds
// `if`, as in the reference), a packed scatterAdd on group memory, a run-time loop over the group buffer, two scattered
// stores. params[0] = bit offset of the 6-bit digit. inputs: keys_in[N], values_in[N], group_histogram_scan[G, 64]
// (inclusive over groups), total_bit_histogram[64] (inclusive over digits). outputs: keys_out[N], values_out[N].
static void BuildRadixScatterPass(Program* program, const std::vector<int64_t>& params) {
	const int shift = params.empty() ? 0 : (int)params[0];
	KernelBuilder kb(program, 2, {128});
	V keys_out = kb.Buffer("keys_out", false), values_out = kb.Buffer("values_out", false);
	V keys_in = kb.Buffer("keys_in", true), values_in = kb.Buffer("values_in", true), scan = kb.Buffer("group_histogram_scan", true),
	  total = kb.Buffer("total_bit_histogram", true);
	V N = kb.Var("N", TFType_Int), G = kb.Var("G", TFType_Int);
	std::vector<V> idx = kb.ThreadIndices({kb.Const(128), G});
	V e = idx[0], g = idx[1];
	V temp = kb.GroupMemory("temp", TFType_Uint, 128);
	V half_count = kb.GroupMemory("half_count", TFType_Uint, 64);
	V gtid = kb.BlockThreadId(0);
	kb.If(gtid < kb.Const(64), [&] { kb.Store(half_count, gtid, kb.ConstU(0u)); });
	kb.Barrier();
	V element = kb.Named(g * kb.Const(128) + e, "element");
	kb.If(element < N, [&] {
		V old_key = kb.Named(kb.Load(keys_in, element, TFType_Uint), "old_key");
		V bit = kb.Named((old_key >> kb.ConstU((uint32_t)shift)) & kb.ConstU(63u), "bit");
		V ibit = kb.Named(ToInt(bit), "ibit");
		kb.Store(temp, gtid, bit);
		V quarter = kb.Named(e / kb.Const(32), "quarter_index");
		kb.If(quarter < kb.Const(3), [&] {
			V packed = ToUint(Select(quarter < kb.Const(1), kb.Const(1), kb.Const(0))) | (ToUint(Select(quarter < kb.Const(2), kb.Const(1), kb.Const(0))) << kb.ConstU(8u)) |
			           (ToUint(Select(quarter < kb.Const(3), kb.Const(1), kb.Const(0))) << kb.ConstU(16u));
			kb.Atomic("InterlockedAdd", half_count, ibit, packed);
		});
		kb.Barrier();
		V old_val = kb.Named(kb.Load(values_in, element, TFType_Uint), "old_val");
		V before_groups = Select(g == kb.Const(0), kb.ConstU(0u), kb.Load(scan, kb.Clamp(g - kb.Const(1), kb.Const(0), G - kb.Const(1)) * kb.Const(64) + ibit, TFType_Uint));
		V before_digits = Select(ibit == kb.Const(0), kb.ConstU(0u), kb.Load(total, kb.Clamp(ibit - kb.Const(1), kb.Const(0), kb.Const(63)), TFType_Uint));
		V in_quarters = Select(quarter > kb.Const(0), (kb.Load(half_count, ibit, TFType_Uint) >> ToUint(kb.Const(8) * (quarter - kb.Const(1)))) & kb.ConstU(0xFFu), kb.ConstU(0u));
		V offset = kb.Accumulator("total_offset", TFType_Uint, 0u);
		kb.Set(offset, before_groups + before_digits + in_quarters);
		kb.Loop(quarter * kb.Const(32), e, kb.Const(1), [&](V j) { kb.Set(offset, offset + Select(kb.Load(temp, j, TFType_Uint) == bit, kb.ConstU(1u), kb.ConstU(0u))); });
		V dst = kb.Named(ToInt(offset), "dst");
		kb.Store(keys_out, dst, old_key);
		kb.Store(values_out, dst, old_val);
	});
	Kernel* kernel = kb.Finish();
	{  // the host part of the tree; its names shadow the kernel's
		HostBuilder h(program);
		V keys = h.Input("keys_in", {-1}, TFType_Uint);
		V n = h.Shape(keys)[0];
		V groups = (n + h.Const(127)) / h.Const(128);
		V values = h.Input("values_in", {n}, TFType_Uint);
		V scan_t = h.Input("group_histogram_scan", {groups, 64}, TFType_Uint);
		V total_t = h.Input("total_bit_histogram", {64}, TFType_Uint);
		V keys_sorted = h.Allocate("keys_out", {n}, TFType_Uint), values_sorted = h.Allocate("values_out", {n}, TFType_Uint);
		h.Dispatch(kernel, {keys_sorted, values_sorted}, {keys, values, scan_t, total_t}, {n, groups}, {groups, 128});
		h.Output(keys_sorted);
		h.Output(values_sorted);
		h.Finish();
	}
}

// tests/reshape_reduction_test.py of the reference, as its passes leave it for inputs of unknown shape (no 128-chunk
// split: Compiler/Steps/Optimization.cpp:469-492 splits constant extents >= 1024 only):
//   A[N, Bx, By, Bz]; Ar = reshape(A, [N, M]) with M = Bx*By*Bz (a host-side reshape, the kernel addresses A flat)
//   one kernel of shape [N] with the five fused reductions over the last axis of Ar: max, min, sum,
//   mean = sum / float(M) (Implementations.cpp:370-372), norm = sqrt(sum(x * x)) (:366-368), each its own loop;
//   one kernel of shape [1] with max over the row maxima and min over the row minima;
//   one kernel of shape [Bx, By, Bz] with the mean over axis 0 (a loop of N strided loads, then / float(N)).
static void BuildReshapeReduction(Program* program, const std::vector<int64_t>&) {
	const float lowest = -3.402823466e+38f, highest = 3.402823466e+38f;
	Kernel* rows;
	{
		KernelBuilder kb(program, 1);
		V o_max = kb.Buffer("max_val", false), o_min = kb.Buffer("min_val", false), o_sum = kb.Buffer("sum", false), o_mean = kb.Buffer("mean", false),
		  o_norm = kb.Buffer("norm", false);
		V A = kb.Buffer("Ar", true);
		V N = kb.Var("N", TFType_Int), M = kb.Var("M", TFType_Int);
		V i = kb.ThreadIndices({N})[0];
		V a_max = kb.Accumulator("max", TFType_Float, FloatBits(lowest));
		kb.Loop(kb.Const(0), M, kb.Const(1), [&](V k) { kb.Set(a_max, Fn("max", a_max, kb.Load(A, i * M + k, TFType_Float))); });
		V a_min = kb.Accumulator("min", TFType_Float, FloatBits(highest));
		kb.Loop(kb.Const(0), M, kb.Const(1), [&](V k) { kb.Set(a_min, Fn("min", a_min, kb.Load(A, i * M + k, TFType_Float))); });
		V a_sum = kb.Accumulator("sum", TFType_Float, FloatBits(0.0f));
		kb.Loop(kb.Const(0), M, kb.Const(1), [&](V k) { kb.Set(a_sum, a_sum + kb.Load(A, i * M + k, TFType_Float)); });
		V a_mean = kb.Accumulator("sum", TFType_Float, FloatBits(0.0f));
		kb.Loop(kb.Const(0), M, kb.Const(1), [&](V k) { kb.Set(a_mean, a_mean + kb.Load(A, i * M + k, TFType_Float)); });
		V a_sq = kb.Accumulator("sum", TFType_Float, FloatBits(0.0f));
		kb.Loop(kb.Const(0), M, kb.Const(1), [&](V k) {
			V x = kb.Load(A, i * M + k, TFType_Float);
			kb.Set(a_sq, a_sq + x * x);
		});
		kb.Store(o_max, i, a_max);
		kb.Store(o_min, i, a_min);
		kb.Store(o_sum, i, a_sum);
		kb.Store(o_mean, i, a_mean / ToFloat(M));
		kb.Store(o_norm, i, Fn("sqrt", a_sq));
		rows = kb.Finish();
	}
	Kernel* totals;
	{
		KernelBuilder kb(program, 1);
		V o_max = kb.Buffer("total_max", false), o_min = kb.Buffer("total_min", false);
		V row_max = kb.Buffer("max_val", true), row_min = kb.Buffer("min_val", true);
		V N = kb.Var("N", TFType_Int);
		V t = kb.ThreadIndices({kb.Const(1)})[0];
		V a_max = kb.Accumulator("max", TFType_Float, FloatBits(lowest));
		kb.Loop(kb.Const(0), N, kb.Const(1), [&](V k) { kb.Set(a_max, Fn("max", a_max, kb.Load(row_max, k, TFType_Float))); });
		V a_min = kb.Accumulator("min", TFType_Float, FloatBits(highest));
		kb.Loop(kb.Const(0), N, kb.Const(1), [&](V k) { kb.Set(a_min, Fn("min", a_min, kb.Load(row_min, k, TFType_Float))); });
		kb.Store(o_max, t, a_max);
		kb.Store(o_min, t, a_min);
		totals = kb.Finish();
	}
	Kernel* block;
	{
		KernelBuilder kb(program, 3);
		V o = kb.Buffer("mean_block", false), A = kb.Buffer("A", true);
		V N = kb.Var("N", TFType_Int), Bx = kb.Var("Bx", TFType_Int), By = kb.Var("By", TFType_Int), Bz = kb.Var("Bz", TFType_Int);
		std::vector<V> idx = kb.ThreadIndices({Bz, By, Bx});
		V z = idx[0], y = idx[1], x = idx[2];
		V cell = (x * By + y) * Bz + z;
		V acc = kb.Accumulator("sum", TFType_Float, FloatBits(0.0f));
		kb.Loop(kb.Const(0), N, kb.Const(1), [&](V n) { kb.Set(acc, acc + kb.Load(A, n * ((Bx * By) * Bz) + cell, TFType_Float)); });
		kb.Store(o, cell, acc / ToFloat(N));
		block = kb.Finish();
	}
	{
		HostBuilder h(program);
		V A = h.Input("A", {-1, -1, -1, -1}, TFType_Float);
		std::vector<V> e = h.Shape(A);
		V N = e[0], Bx = e[1], By = e[2], Bz = e[3];
		V M = (Bx * By) * Bz;
		V Ar = h.Reshape(A, "Ar", {N, M}, TFType_Float);
		std::vector<V> row_outputs;
		for (const char* name : {"max_val", "min_val", "sum", "mean", "norm"}) row_outputs.push_back(h.Allocate(name, {N}, TFType_Float));
		h.Dispatch(rows, row_outputs, {Ar}, {N, M}, {N});
		V total_max = h.Allocate("total_max", {1}, TFType_Float), total_min = h.Allocate("total_min", {1}, TFType_Float);
		h.Dispatch(totals, {total_max, total_min}, {row_outputs[0], row_outputs[1]}, {N}, {1});
		V mean_block = h.Allocate("mean_block", {Bx, By, Bz}, TFType_Float);
		h.Dispatch(block, {mean_block}, {A}, {N, Bx, By, Bz}, {Bx, By, Bz});
		for (V out : row_outputs) h.Output(out);
		h.Output(total_max);
		h.Output(total_min);
		h.Output(mean_block);
		h.Finish();
	}
}

// dim_sum / dim_max / dim_min of 32-bit integers over the last axis of [R, C] (Operations.cpp: dim_sum {"u_u", "i_i"}),
// unsplit loops with wrap-around sums. inputs U[R, C] uint, I[R, C] int; outputs sum_u[R], max_u[R], sum_i[R], min_i[R].
static void BuildIntegerReductions(Program* program, const std::vector<int64_t>&) {
	KernelBuilder kb(program, 1);
	V sum_u = kb.Buffer("sum_u", false), max_u = kb.Buffer("max_u", false), sum_i = kb.Buffer("sum_i", false), min_i = kb.Buffer("min_i", false);
	V U = kb.Buffer("U", true), I = kb.Buffer("I", true);
	V R = kb.Var("R", TFType_Int), C = kb.Var("C", TFType_Int);
	V r = kb.ThreadIndices({R})[0];
	V a_su = kb.Accumulator("sum", TFType_Uint, 0u);
	kb.Loop(kb.Const(0), C, kb.Const(1), [&](V k) { kb.Set(a_su, a_su + kb.Load(U, r * C + k, TFType_Uint)); });
	V a_mu = kb.Accumulator("max", TFType_Uint, 0u);
	kb.Loop(kb.Const(0), C, kb.Const(1), [&](V k) { kb.Set(a_mu, Fn("max", a_mu, kb.Load(U, r * C + k, TFType_Uint))); });
	V a_si = kb.Accumulator("sum", TFType_Int, 0u);
	kb.Loop(kb.Const(0), C, kb.Const(1), [&](V k) { kb.Set(a_si, a_si + kb.Load(I, r * C + k, TFType_Int)); });
	V a_mi = kb.Accumulator("min", TFType_Int, 0x7FFFFFFFu);
	kb.Loop(kb.Const(0), C, kb.Const(1), [&](V k) { kb.Set(a_mi, Fn("min", a_mi, kb.Load(I, r * C + k, TFType_Int))); });
	kb.Store(sum_u, r, a_su);
	kb.Store(max_u, r, a_mu);
	kb.Store(sum_i, r, a_si);
	kb.Store(min_i, r, a_mi);
	Kernel* kernel = kb.Finish();
	{
		HostBuilder h(program);
		V Ut = h.Input("U", {-1, -1}, TFType_Uint);
		V rows = h.Shape(Ut)[0], cols = h.Shape(Ut)[1];
		V It = h.Input("I", {rows, cols}, TFType_Int);
		V o_su = h.Allocate("sum_u", {rows}, TFType_Uint), o_mu = h.Allocate("max_u", {rows}, TFType_Uint);
		V o_si = h.Allocate("sum_i", {rows}, TFType_Int), o_mi = h.Allocate("min_i", {rows}, TFType_Int);
		h.Dispatch(kernel, {o_su, o_mu, o_si, o_mi}, {Ut, It}, {rows, cols}, {rows});
		for (V out : {o_su, o_mu, o_si, o_mi}) h.Output(out);
		h.Finish();
	}
}

// Small dispatches of one kernel, some on disjoint buffers and some that depend on an earlier one, with a tensor released
// in between: the kernel manager gathers the independent ones into one launch and must keep the order of the others.
// inputs a, b, c (any lengths), shift[1]; every dispatch computes out[i] = in[i] * scale + shift[0].
// o1 = 2a + s, o2 = 3b + s, o3 = 4c + s | o4 = 5 o1 + s, tmp = 7b + s | o5 = 1.5 tmp + s, o6 = -c + s
static void BuildGatheredUpdates(Program* program, const std::vector<int64_t>&) {
	KernelBuilder kb(program, 1);
	V out = kb.Buffer("result", false);
	V in = kb.Buffer("source", true), shift = kb.Buffer("shift", true);
	V count = kb.Var("count", TFType_Int), scale = kb.Var("scale", TFType_Float);
	V i = kb.ThreadIndices({count})[0];
	kb.Store(out, i, kb.Load(in, i, TFType_Float) * scale + kb.Load(shift, kb.Const(0), TFType_Float));
	Kernel* kernel = kb.Finish();
	HostBuilder h(program);
	V a = h.Input("a", {-1}, TFType_Float), b = h.Input("b", {-1}, TFType_Float), c = h.Input("c", {-1}, TFType_Float);
	V s = h.Input("shift", {1}, TFType_Float);
	V na = h.Shape(a)[0], nb = h.Shape(b)[0], nc = h.Shape(c)[0];
	auto run = [&](V source, V n, float factor, const char* name) {
		V result = h.Allocate(name, {n}, TFType_Float);
		h.Dispatch(kernel, {result}, {source, s}, {n, h.Const(factor)}, {n});
		return result;
	};
	V o1 = run(a, na, 2.0f, "o1");
	V o2 = run(b, nb, 3.0f, "o2");
	V o3 = run(c, nc, 4.0f, "o3");
	V o4 = run(o1, na, 5.0f, "o4");
	V tmp = run(b, nb, 7.0f, "tmp");
	V o5 = run(tmp, nb, 1.5f, "o5");
	h.Deallocate(tmp);
	V o6 = run(c, nc, -1.0f, "o6");
	for (V o : {o1, o2, o3, o4, o5, o6}) h.Output(o);
	h.Finish();
}

// tests/split_dim_test.py of the reference: splitted = tf.split_dim(data, 32, 0); merged = tf.merge_dim(splitted, axis = 1)
// on int32 data[D0, D1, D2]. Both are kernels (Compiler/Implementations.cpp:507-549): the split index is
// outer * 32 + inner, read with the default (clamped) load and replaced by 0 where it lies outside the array
// (ConstantOutOfBounds, :56-69); the merge reads [index % 32, index / 32]. Shapes as Tensor.h:712-755 computes them:
// splitted[ceil(D0 / 32), 32, D1, D2], merged[ceil(D0 / 32) * 32, D1, D2].
static void BuildSplitMerge(Program* program, const std::vector<int64_t>&) {
	const int kSplit = 32;
	Kernel* split_kernel;
	{
		KernelBuilder kb(program, 4);
		V out = kb.Buffer("split", false), data = kb.Buffer("data", true);
		V D0 = kb.Var("D0", TFType_Int), D1 = kb.Var("D1", TFType_Int), D2 = kb.Var("D2", TFType_Int), S = kb.Var("S", TFType_Int);
		std::vector<V> idx = kb.ThreadIndices({D2, D1, kb.Const(kSplit), S});
		V x = idx[0], y = idx[1], inner = idx[2], outer = idx[3];
		V source = kb.Named(outer * kb.Const(kSplit) + inner, "source");
		V outside = kb.Named((source < kb.Const(0)) || (source >= D0), "out_of_bounds");
		V loaded = kb.Load(data, (kb.Clamp(source, kb.Const(0), D0 - kb.Const(1)) * D1 + y) * D2 + x, TFType_Int);
		kb.Store(out, ((outer * kb.Const(kSplit) + inner) * D1 + y) * D2 + x, kb.Named(Select(outside, kb.Const(0), loaded), "split"));
		split_kernel = kb.Finish();
	}
	Kernel* merge_kernel;
	{
		KernelBuilder kb(program, 3);
		V out = kb.Buffer("merged", false), split = kb.Buffer("split", true);
		V D1 = kb.Var("D1", TFType_Int), D2 = kb.Var("D2", TFType_Int), S = kb.Var("S", TFType_Int);
		V M = kb.Named(S * kb.Const(kSplit), "merged_size");
		std::vector<V> idx = kb.ThreadIndices({D2, D1, M});
		V x = idx[0], y = idx[1], m = idx[2];
		V inner = kb.Named(m % kb.Const(kSplit), "inner"), outer = kb.Named(m / kb.Const(kSplit), "outer");
		V outside = kb.Named((inner < kb.Const(0)) || (inner >= kb.Const(kSplit)) || (outer < kb.Const(0)) || (outer >= S), "out_of_bounds");
		V loaded = kb.Load(split, ((kb.Clamp(outer, kb.Const(0), S - kb.Const(1)) * kb.Const(kSplit) + kb.Clamp(inner, kb.Const(0), kb.Const(kSplit - 1))) * D1 + y) * D2 + x, TFType_Int);
		kb.Store(out, (m * D1 + y) * D2 + x, kb.Named(Select(outside, kb.Const(0), loaded), "merged"));
		merge_kernel = kb.Finish();
	}
	HostBuilder h(program);
	V data = h.Input("data", {-1, -1, -1}, TFType_Int);
	std::vector<V> e = h.Shape(data);
	V S = (e[0] + h.Const(kSplit - 1)) / h.Const(kSplit);
	V splitted = h.Allocate("splitted", {S, kSplit, e[1], e[2]}, TFType_Int);
	h.Dispatch(split_kernel, {splitted}, {data}, {e[0], e[1], e[2], S}, {S, kSplit, e[1], e[2]});
	V M = S * h.Const(kSplit);
	V merged = h.Allocate("merged", {M, e[1], e[2]}, TFType_Int);
	h.Dispatch(merge_kernel, {merged}, {splitted}, {e[1], e[2], S}, {M, e[1], e[2]});
	h.Output(merged);
	h.Output(splitted);
	h.Finish();
}

// tests/linalg_test.py of the reference: Q, R = qr_decomposition(A) by Gram-Schmidt in a host loop over the columns, R_inv
// = the inverse of the upper triangular R (row by row in a second host loop, on R transposed), A_inv = R_inv @ Q^T.
// Every statement of the loop bodies is a kernel whose extent depends on the loop variable:
//   R[i, i] = norm(A[:, i])                    one thread walking the column
//   Q[:, i] = A[:, i] / R[i, i]                m threads
//   R[i, k] = sum_p Q[p, i] A[p, k], k > i     n - i - 1 threads, each a loop over the rows (tf.sum(..., axis = 0))
//   A[p, k] -= Q[p, i] R[i, k], k > i          [m, n - i - 1] threads, in place
// and for the inverse (L = R^T, X = its inverse; the program returns X^T):
//   X[i, i] = 1 / L[i, i];  X[i, t] = -sum_{p < i} L[i, p] X[p, t] / L[i, i] for t < i     i threads
// The input is copied first: the program updates A in place.
static void BuildQrInversion(Program* program, const std::vector<int64_t>&) {
	auto finish = [](KernelBuilder& kb) { return kb.Finish(); };
	Kernel *copy, *zero, *norm, *qcol, *dot, *update, *diag, *row, *transpose, *product;
	{
		KernelBuilder kb(program, 1);
		V out = kb.Buffer("copy", false), in = kb.Buffer("source", true);
		V count = kb.Var("count", TFType_Int);
		V i = kb.ThreadIndices({count})[0];
		kb.Store(out, i, kb.Load(in, i, TFType_Float));
		copy = finish(kb);
	}
	{
		KernelBuilder kb(program, 1);
		V out = kb.Buffer("zeros", false);
		V count = kb.Var("count", TFType_Int);
		V i = kb.ThreadIndices({count})[0];
		kb.Store(out, i, kb.Const(0.0f));
		zero = finish(kb);
	}
	{  // R[i, i] = sqrt(sum_j A[j, i]^2)
		KernelBuilder kb(program, 1);
		V R = kb.Buffer("R", false), A = kb.Buffer("A", true);
		V m = kb.Var("m", TFType_Int), n = kb.Var("n", TFType_Int), i = kb.Var("i", TFType_Int);
		kb.ThreadIndices({kb.Const(1)});
		V acc = kb.Accumulator("sum", TFType_Float, 0u);
		kb.Loop(kb.Const(0), m, kb.Const(1), [&](V j) {
			V a = kb.Load(A, j * n + i, TFType_Float);
			kb.Set(acc, acc + a * a);
		});
		kb.Store(R, i * n + i, Fn("sqrt", acc));
		norm = finish(kb);
	}
	{  // Q[j, i] = A[j, i] / R[i, i]
		KernelBuilder kb(program, 1);
		V Q = kb.Buffer("Q", false), A = kb.Buffer("A", true), R = kb.Buffer("R", true);
		V m = kb.Var("m", TFType_Int), n = kb.Var("n", TFType_Int), i = kb.Var("i", TFType_Int);
		V j = kb.ThreadIndices({m})[0];
		kb.Store(Q, j * n + i, kb.Load(A, j * n + i, TFType_Float) / kb.Load(R, i * n + i, TFType_Float));
		qcol = finish(kb);
	}
	{  // R[i, i + 1 + t] = sum_p Q[p, i] * A[p, i + 1 + t]
		KernelBuilder kb(program, 1);
		V R = kb.Buffer("R", false), Q = kb.Buffer("Q", true), A = kb.Buffer("A", true);
		V m = kb.Var("m", TFType_Int), n = kb.Var("n", TFType_Int), i = kb.Var("i", TFType_Int);
		V t = kb.ThreadIndices({n - i - kb.Const(1)})[0];
		V k = kb.Named(t + i + kb.Const(1), "k");
		V acc = kb.Accumulator("sum", TFType_Float, 0u);
		kb.Loop(kb.Const(0), m, kb.Const(1), [&](V p) { kb.Set(acc, acc + kb.Load(Q, p * n + i, TFType_Float) * kb.Load(A, p * n + k, TFType_Float)); });
		kb.Store(R, i * n + k, acc);
		dot = finish(kb);
	}
	{  // A[p, k] -= Q[p, i] * R[i, k] for k > i
		KernelBuilder kb(program, 2);
		V A = kb.Buffer("A", false), Q = kb.Buffer("Q", true), R = kb.Buffer("R", true);
		V m = kb.Var("m", TFType_Int), n = kb.Var("n", TFType_Int), i = kb.Var("i", TFType_Int);
		std::vector<V> idx = kb.ThreadIndices({n - i - kb.Const(1), m});
		V k = kb.Named(idx[0] + i + kb.Const(1), "k"), p = idx[1];
		kb.Store(A, p * n + k, kb.Load(A, p * n + k, TFType_Float) - kb.Load(Q, p * n + i, TFType_Float) * kb.Load(R, i * n + k, TFType_Float));
		update = finish(kb);
	}
	{  // X[i, i] = 1 / L[i, i] with L = R^T
		KernelBuilder kb(program, 1);
		V X = kb.Buffer("X", false), R = kb.Buffer("R", true);
		V n = kb.Var("n", TFType_Int), i = kb.Var("i", TFType_Int);
		kb.ThreadIndices({kb.Const(1)});
		kb.Store(X, i * n + i, kb.Const(1.0f) / kb.Load(R, i * n + i, TFType_Float));
		diag = finish(kb);
	}
	{  // X[i, t] = -sum_{p < i} L[i, p] X[p, t] / L[i, i] for t < i, L[i, p] = R[p, i]
		KernelBuilder kb(program, 1);
		V X = kb.Buffer("X", false), R = kb.Buffer("R", true);
		V n = kb.Var("n", TFType_Int), i = kb.Var("i", TFType_Int);
		V t = kb.ThreadIndices({i})[0];
		V acc = kb.Accumulator("sum", TFType_Float, 0u);
		kb.Loop(kb.Const(0), i, kb.Const(1), [&](V p) { kb.Set(acc, acc + kb.Load(R, p * n + i, TFType_Float) * kb.Load(X, p * n + t, TFType_Float)); });
		kb.Store(X, i * n + t, -acc / kb.Load(R, i * n + i, TFType_Float));
		row = finish(kb);
	}
	{  // out[r, c] = in[c, r]
		KernelBuilder kb(program, 2);
		V out = kb.Buffer("transposed", false), in = kb.Buffer("matrix", true);
		V n = kb.Var("n", TFType_Int);
		std::vector<V> idx = kb.ThreadIndices({n, n});
		kb.Store(out, idx[1] * n + idx[0], kb.Load(in, idx[0] * n + idx[1], TFType_Float));
		transpose = finish(kb);
	}
	{  // A_inv[r, c] = sum_k R_inv[r, k] Q[c, k]   (R_inv @ Q^T, the lowered matmul loop: Implementations.cpp:560-646)
		KernelBuilder kb(program, 2);
		V C = kb.Buffer("C", false), A = kb.Buffer("A", true), B = kb.Buffer("B", true);
		V n = kb.Var("n", TFType_Int), m = kb.Var("m", TFType_Int);
		std::vector<V> idx = kb.ThreadIndices({m, n});
		V c = idx[0], r = idx[1];
		V acc = kb.Accumulator("matmul", TFType_Float, 0u);
		kb.Loop(kb.Const(0), n, kb.Const(1), [&](V k) { kb.Set(acc, acc + kb.Load(A, r * n + k, TFType_Float) * kb.Load(B, c * n + k, TFType_Float)); });
		kb.Store(C, r * m + c, acc);
		product = finish(kb);
	}
	HostBuilder h(program);
	V A_in = h.Input("A", {-1, -1}, TFType_Float);
	std::vector<V> e = h.Shape(A_in);
	V m = e[0], n = e[1];
	V A = h.Allocate("A_work", {m, n}, TFType_Float);
	h.Dispatch(copy, {A}, {A_in}, {m * n}, {m * n});
	V Q = h.Allocate("Q", {m, n}, TFType_Float), R = h.Allocate("R", {n, n}, TFType_Float);
	h.Dispatch(zero, {Q}, {}, {m * n}, {m * n});
	h.Dispatch(zero, {R}, {}, {n * n}, {n * n});
	h.Loop(h.Const(0), n - h.Const(1), h.Const(1), [&](V i) {
		h.Dispatch(norm, {R}, {A}, {m, n, i}, {1});
		h.Dispatch(qcol, {Q}, {A, R}, {m, n, i}, {m});
		h.Dispatch(dot, {R}, {Q, A}, {m, n, i}, {n - i - h.Const(1)});
		h.Dispatch(update, {A}, {Q, R}, {m, n, i}, {m, n - i - h.Const(1)});
	});
	V last = n - h.Const(1);
	h.Dispatch(norm, {R}, {A}, {m, n, last}, {1});
	h.Dispatch(qcol, {Q}, {A, R}, {m, n, last}, {m});
	h.Deallocate(A);
	V X = h.Allocate("inverted", {n, n}, TFType_Float);
	h.Dispatch(zero, {X}, {}, {n * n}, {n * n});
	h.Dispatch(diag, {X}, {R}, {n, h.Const(0)}, {1});
	h.Loop(h.Const(1), n, h.Const(1), [&](V i) {
		h.Dispatch(diag, {X}, {R}, {n, i}, {1});
		h.Dispatch(row, {X}, {R}, {n, i}, {i});
	});
	V R_inv = h.Allocate("R_inv", {n, n}, TFType_Float);
	h.Dispatch(transpose, {R_inv}, {X}, {n}, {n, n});
	h.Deallocate(X);
	V A_inv = h.Allocate("A_inv", {n, m}, TFType_Float);
	h.Dispatch(product, {A_inv}, {R_inv, Q}, {n, m}, {n, m});
	for (V o : {Q, R, R_inv, A_inv}) h.Output(o);
	h.Finish();
}

// The forward pass and loss of the reference's test network (tests/autograd_test.py:33-108, TestModule1): two
// convolutions written as sums over gathered indices, 2 x 2 max pooling, the tanh form of GELU, a dense layer, a small
// matrix product per group of 16 features with tanh, its sum over the groups fed back as a residual, the output layer,
// and the loss mean_b sum_c -Y log_softmax(logits) with log_softmax as :29-31 composes it.
// inputs: X[N, 784], Y[N, 10], conv1[16,1,5,5], conv2[64,16,5,5], fc1[1024,64], fc1_bias[64], sum1[16,8], sum1_bias[8],
// sum2[8,16], sum2_bias[16], fc2[64,10], fc2_bias[10]. outputs: loss[1], logits[N, 10].
static void BuildAutogradNetworkForward(Program* program, const std::vector<int64_t>&) {
	auto gelu = [](KernelBuilder& kb, V x) {
		return kb.Const(0.5f) * x * (kb.Const(1.0f) + Fn("tanh", kb.Const(0.7978845608028654f) * (x + kb.Const(0.044715f) * (x * x * x))));
	};
	// conv[b, co, y, x] = sum_cin sum_it X[b, cin, y + it % w, x + it / w] * W[co, cin, it % w, it / w]   (:73-79: the tap
	// index walks the kernel's first spatial axis fastest, and the same offsets address the image)
	Kernel* conv;
	{
		KernelBuilder kb(program, 4);
		V out = kb.Buffer("conv", false), X = kb.Buffer("X", true), W = kb.Buffer("W", true);
		V N = kb.Var("N", TFType_Int), CIN = kb.Var("CIN", TFType_Int), HI = kb.Var("HI", TFType_Int), WI = kb.Var("WI", TFType_Int), COUT = kb.Var("COUT", TFType_Int),
		  kh = kb.Var("h", TFType_Int), kw = kb.Var("w", TFType_Int);
		V HO = kb.Named(HI - kh + kb.Const(1), "HO"), WO = kb.Named(WI - kw + kb.Const(1), "WO");
		std::vector<V> idx = kb.ThreadIndices({WO, HO, COUT, N});
		V hi = idx[0], wi = idx[1], co = idx[2], b = idx[3];
		V total = kb.Accumulator("sum", TFType_Float, FloatBits(0.0f));
		kb.Loop(kb.Const(0), CIN, kb.Const(1), [&](V cin) {
			V taps = kb.Accumulator("sum", TFType_Float, FloatBits(0.0f));
			kb.Loop(kb.Const(0), kh * kw, kb.Const(1), [&](V it) {
				V i = it % kw, j = it / kw;
				V x = kb.Load(X, ((b * CIN + cin) * HI + (wi + i)) * WI + (hi + j), TFType_Float);
				V w = kb.Load(W, ((co * CIN + cin) * kh + i) * kw + j, TFType_Float);
				kb.Set(taps, taps + x * w);
			});
			kb.Set(total, total + taps);
		});
		kb.Store(out, ((b * COUT + co) * HO + wi) * WO + hi, total);
		conv = kb.Finish();
	}
	// pooled[b, c, y, x] = GELU(max_i max_j X[b, c, 2 y + i, 2 x + j])   (:81-83, :88-91)
	Kernel* pool;
	{
		KernelBuilder kb(program, 4);
		V out = kb.Buffer("pooled", false), X = kb.Buffer("X", true);
		V N = kb.Var("N", TFType_Int), C = kb.Var("C", TFType_Int), H = kb.Var("H", TFType_Int), Wd = kb.Var("W", TFType_Int);
		V HO = kb.Named(H / kb.Const(2), "HO"), WO = kb.Named(Wd / kb.Const(2), "WO");
		std::vector<V> idx = kb.ThreadIndices({WO, HO, C, N});
		V hi = idx[0], wi = idx[1], c = idx[2], b = idx[3];
		V best = kb.Accumulator("max", TFType_Float, FloatBits(-3.402823466e38f));
		kb.Loop(kb.Const(0), kb.Const(2), kb.Const(1), [&](V i) {
			V inner = kb.Accumulator("max", TFType_Float, FloatBits(-3.402823466e38f));
			kb.Loop(kb.Const(0), kb.Const(2), kb.Const(1), [&](V j) {
				kb.Set(inner, Fn("max", inner, kb.Load(X, ((b * C + c) * H + (kb.Const(2) * wi + i)) * Wd + (kb.Const(2) * hi + j), TFType_Float)));
			});
			kb.Set(best, Fn("max", best, inner));
		});
		kb.Store(out, ((b * C + c) * HO + wi) * WO + hi, gelu(kb, best));
		pool = kb.Finish();
	}
	// C[t, i, j] = tail(sum_k A[t, i, k] B[k, j] + bias[j]) (+ R[t, i, j] ...): the lowered matmul loop with the tails the
	// network needs. tail 0: + bias; 1: GELU(+ bias); 2: tanh(+ bias); 3: R[t, i, j] + tanh(+ bias) with A broadcast over i.
	auto dense = [&](int tail) {
		KernelBuilder kb(program, 3);
		V C = kb.Buffer("C", false), A = kb.Buffer("A", true), B = kb.Buffer("B", true), bias = kb.Buffer("bias", true);
		V R = tail == 3 ? kb.Buffer("R", true) : V();
		V T = kb.Var("T", TFType_Int), M = kb.Var("M", TFType_Int), N = kb.Var("N", TFType_Int), K = kb.Var("K", TFType_Int);
		std::vector<V> idx = kb.ThreadIndices({N, M, T});
		V j = idx[0], i = idx[1], t = idx[2];
		V acc = kb.Accumulator("matmul", TFType_Float, FloatBits(0.0f));
		kb.Loop(kb.Const(0), K, kb.Const(1), [&](V k) {
			V a = tail == 3 ? kb.Load(A, t * K + k, TFType_Float) : kb.Load(A, (t * M + i) * K + k, TFType_Float);
			kb.Set(acc, acc + a * kb.Load(B, k * N + j, TFType_Float));
		});
		V z = kb.Named(acc + kb.Load(bias, j, TFType_Float), "z");
		V at = (t * M + i) * N + j;
		if (tail == 0) kb.Store(C, at, z);
		if (tail == 1) kb.Store(C, at, gelu(kb, z));
		if (tail == 2) kb.Store(C, at, Fn("tanh", z));
		if (tail == 3) kb.Store(C, at, kb.Load(R, at, TFType_Float) + Fn("tanh", z));
		return kb.Finish();
	};
	Kernel *dense_bias = dense(0), *dense_gelu = dense(1), *dense_tanh = dense(2), *dense_residual = dense(3);
	// r[b, o] = sum_g x[b, g, o]   (tf.sum(r, axis = 1))
	Kernel* group_sum;
	{
		KernelBuilder kb(program, 2);
		V out = kb.Buffer("summed", false), X = kb.Buffer("X", true);
		V N = kb.Var("N", TFType_Int), G = kb.Var("G", TFType_Int), O = kb.Var("O", TFType_Int);
		std::vector<V> idx = kb.ThreadIndices({O, N});
		V o = idx[0], b = idx[1];
		V acc = kb.Accumulator("sum", TFType_Float, FloatBits(0.0f));
		kb.Loop(kb.Const(0), G, kb.Const(1), [&](V g) { kb.Set(acc, acc + kb.Load(X, (b * G + g) * O + o, TFType_Float)); });
		kb.Store(out, b * O + o, acc);
		group_sum = kb.Finish();
	}
	// row_loss[b] = sum_c -Y[b, c] * ((x - m) - log(sum_c exp(x - m))), m = max_c x[b, c]
	Kernel* row_loss;
	{
		KernelBuilder kb(program, 1);
		V out = kb.Buffer("row_loss", false), X = kb.Buffer("logits", true), Y = kb.Buffer("Y", true);
		V N = kb.Var("N", TFType_Int), C = kb.Var("C", TFType_Int);
		V b = kb.ThreadIndices({N})[0];
		V m = kb.Accumulator("max", TFType_Float, FloatBits(-3.402823466e38f));
		kb.Loop(kb.Const(0), C, kb.Const(1), [&](V c) { kb.Set(m, Fn("max", m, kb.Load(X, b * C + c, TFType_Float))); });
		V z = kb.Accumulator("sum", TFType_Float, FloatBits(0.0f));
		kb.Loop(kb.Const(0), C, kb.Const(1), [&](V c) { kb.Set(z, z + Fn("exp", kb.Load(X, b * C + c, TFType_Float) - m)); });
		V total = kb.Accumulator("sum", TFType_Float, FloatBits(0.0f));
		kb.Loop(kb.Const(0), C, kb.Const(1), [&](V c) {
			V ls = (kb.Load(X, b * C + c, TFType_Float) - m) - Fn("log", z);
			kb.Set(total, total + (-kb.Load(Y, b * C + c, TFType_Float)) * ls);
		});
		kb.Store(out, b, total);
		row_loss = kb.Finish();
	}
	// loss = mean_b row_loss[b]
	Kernel* mean;
	{
		KernelBuilder kb(program, 1);
		V out = kb.Buffer("loss", false), X = kb.Buffer("row_loss", true);
		V N = kb.Var("N", TFType_Int);
		kb.ThreadIndices({kb.Const(1)});
		V acc = kb.Accumulator("sum", TFType_Float, FloatBits(0.0f));
		kb.Loop(kb.Const(0), N, kb.Const(1), [&](V b) { kb.Set(acc, acc + kb.Load(X, b, TFType_Float)); });
		kb.Store(out, kb.Const(0), acc / ToFloat(N));
		mean = kb.Finish();
	}
	HostBuilder h(program);
	V X = h.Input("X", {-1, 784}, TFType_Float);
	V N = h.Shape(X)[0];
	V Y = h.Input("Y", {N, 10}, TFType_Float);
	V conv1 = h.Input("conv1", {16, 1, 5, 5}, TFType_Float), conv2 = h.Input("conv2", {64, 16, 5, 5}, TFType_Float);
	V fc1 = h.Input("fc1", {1024, 64}, TFType_Float), fc1_bias = h.Input("fc1_bias", {64}, TFType_Float);
	V sum1 = h.Input("sum_layer1", {16, 8}, TFType_Float), sum1_bias = h.Input("sum_layer1_bias", {8}, TFType_Float);
	V sum2 = h.Input("sum_layer2", {8, 16}, TFType_Float), sum2_bias = h.Input("sum_layer2_bias", {16}, TFType_Float);
	V fc2 = h.Input("fc2", {64, 10}, TFType_Float), fc2_bias = h.Input("fc2_bias", {10}, TFType_Float);
	auto c = [&](int v) { return h.Const(v); };
	h.RegionBegin("Forward");
	V image = h.Reshape(X, "image", {N, 1, 28, 28}, TFType_Float);
	V x1 = h.Allocate("conv1_out", {N, 16, 24, 24}, TFType_Float);
	h.Dispatch(conv, {x1}, {image, conv1}, {N, c(1), c(28), c(28), c(16), c(5), c(5)}, {N, 16, 24, 24});
	V p1 = h.Allocate("pool1", {N, 16, 12, 12}, TFType_Float);
	h.Dispatch(pool, {p1}, {x1}, {N, c(16), c(24), c(24)}, {N, 16, 12, 12});
	h.Deallocate(x1);
	V x2 = h.Allocate("conv2_out", {N, 64, 8, 8}, TFType_Float);
	h.Dispatch(conv, {x2}, {p1, conv2}, {N, c(16), c(12), c(12), c(64), c(5), c(5)}, {N, 64, 8, 8});
	h.Deallocate(p1);
	V p2 = h.Allocate("pool2", {N, 64, 4, 4}, TFType_Float);
	h.Dispatch(pool, {p2}, {x2}, {N, c(64), c(8), c(8)}, {N, 64, 4, 4});
	h.Deallocate(x2);
	V flat = h.Reshape(p2, "flat", {N, 1024}, TFType_Float);
	V hidden = h.Allocate("hidden", {N, 64}, TFType_Float);
	h.Dispatch(dense_gelu, {hidden}, {flat, fc1, fc1_bias}, {c(1), N, c(64), c(1024)}, {1, N, 64});
	h.Deallocate(p2);
	V grouped = h.Reshape(hidden, "grouped", {N, 4, 16}, TFType_Float);
	V r = h.Allocate("r", {N, 4, 8}, TFType_Float);
	h.Dispatch(dense_tanh, {r}, {grouped, sum1, sum1_bias}, {N, c(4), c(8), c(16)}, {N, 4, 8});
	V rs = h.Allocate("r_sum", {N, 8}, TFType_Float);
	h.Dispatch(group_sum, {rs}, {r}, {N, c(4), c(8)}, {N, 8});
	h.Deallocate(r);
	V mixed = h.Allocate("mixed", {N, 4, 16}, TFType_Float);
	h.Dispatch(dense_residual, {mixed}, {rs, sum2, sum2_bias, grouped}, {N, c(4), c(16), c(8)}, {N, 4, 16});
	h.Deallocate(rs);
	h.Deallocate(hidden);
	V mixed_flat = h.Reshape(mixed, "mixed_flat", {N, 64}, TFType_Float);
	V logits = h.Allocate("logits", {N, 10}, TFType_Float);
	h.Dispatch(dense_bias, {logits}, {mixed_flat, fc2, fc2_bias}, {c(1), N, c(10), c(64)}, {1, N, 10});
	h.Deallocate(mixed);
	h.RegionEnd("Forward");
	V rows = h.Allocate("row_loss", {N}, TFType_Float);
	h.Dispatch(row_loss, {rows}, {logits, Y}, {N, c(10)}, {N});
	V loss = h.Allocate("loss", {1}, TFType_Float);
	h.Dispatch(mean, {loss}, {rows}, {N}, {1});
	h.Deallocate(rows);
	h.Output(loss);
	h.Output(logits);
	h.Finish();
}

// tf.sort.bitonic of the reference (Python/TensorFrost/sort.py:4-35), as tests/sorting_test.py:14-18 uses it: the
// in-place network over 2^ceil(log2 N) / 2 threads in two nested host loops, one dispatch per (k, j); the masks are
// host scalars of the loop variables (shifts, a complement, a select), the count of stages comes from host float
// arithmetic (int(ceil(log2(float(N))))); loads and stores are the user's (clamped), the swap sits behind an `if`.
static void BuildBitonicSort(Program* program, const std::vector<int64_t>&) {
	Kernel* copy;
	{
		KernelBuilder kb(program, 1);
		V out = kb.Buffer("copy", false), in = kb.Buffer("source", true);
		V count = kb.Var("count", TFType_Int);
		V i = kb.ThreadIndices({count})[0];
		kb.Store(out, i, kb.Load(in, i, TFType_Uint));
		copy = kb.Finish();
	}
	Kernel* stage;
	{
		KernelBuilder kb(program, 1);
		V keys = kb.Buffer("keys", false), values = kb.Buffer("values", false);
		V n = kb.Var("element_count", TFType_Int), half = kb.Var("half", TFType_Int), m_inner = kb.Var("m_inner", TFType_Int), m_outer = kb.Var("m_outer", TFType_Int),
		  m_xor = kb.Var("m_xor", TFType_Int);
		V idx = kb.ThreadIndices({half})[0];
		V id1 = kb.Named(kb.Const(2) * (idx & m_outer) + (idx & m_inner), "id1");
		V id2 = kb.Named(id1 ^ m_xor, "id2");
		V last = n - kb.Const(1);
		V at1 = kb.Clamp(id1, kb.Const(0), last), at2 = kb.Clamp(id2, kb.Const(0), last);
		V key1 = kb.Named(kb.Load(keys, at1, TFType_Uint), "key1"), key2 = kb.Named(kb.Load(keys, at2, TFType_Uint), "key2");
		kb.If((key1 >= key2) && (id1 < n) && (id2 < n), [&]() {
			V val1 = kb.Named(kb.Load(values, at1, TFType_Uint), "val1"), val2 = kb.Named(kb.Load(values, at2, TFType_Uint), "val2");
			kb.Store(values, at1, val2);
			kb.Store(values, at2, val1);
			kb.Store(keys, at1, key2);
			kb.Store(keys, at2, key1);
		});
		stage = kb.Finish();
	}
	HostBuilder h(program);
	V keys_in = h.Input("keys", {-1}, TFType_Uint);
	V n = h.Shape(keys_in)[0];
	V values_in = h.Input("values", {n}, TFType_Uint);
	h.RegionBegin("Bitonic sort");
	V keys = h.Allocate("keys", {n}, TFType_Uint), values = h.Allocate("values", {n}, TFType_Uint);
	h.Dispatch(copy, {keys}, {keys_in}, {n}, {n});
	h.Dispatch(copy, {values}, {values_in}, {n}, {n});
	V log2_count = ToInt(Fn("ceil", Fn("log2", ToFloat(n))));
	V count_round = h.Const(1) << log2_count;
	V half = count_round / h.Const(2);
	h.Loop(h.Const(0), log2_count, h.Const(1), [&](V k) {
		h.Loop(h.Const(0), k + h.Const(1), h.Const(1), [&](V j) {
			V s = h.Const(1) << (k - j);
			V m_inner = s - h.Const(1);
			V m_outer = ~m_inner;
			V m_xor = s + Select(j == h.Const(0), m_inner, h.Const(0));
			h.Dispatch(stage, {keys, values}, {}, {n, half, m_inner, m_outer, m_xor}, {half});
		});
	});
	h.RegionEnd("Bitonic sort");
	h.Output(keys);
	h.Output(values);
	h.Finish();
}

// Reductions over axis 0 of [R, C] tensors of unknown shape, fused into one kernel of shape [C] as kernel fusion
// (Compiler/Scope.cpp:165-188) leaves them: sum, max, min of X, the sum of squares of X (norm over axis 0 before its
// square root, Implementations.cpp:366-368) and the wrap-around sum of U, each its own loop of R strided loads.
// inputs X[R, C] float, U[R, C] uint; outputs sum[C], max[C], min[C], norm[C] (float), sum_u[C] (uint).
static void BuildColumnStatistics(Program* program, const std::vector<int64_t>&) {
	const float lowest = -3.402823466e+38f, highest = 3.402823466e+38f;
	KernelBuilder kb(program, 1);
	V o_sum = kb.Buffer("sum", false), o_max = kb.Buffer("max", false), o_min = kb.Buffer("min", false), o_norm = kb.Buffer("norm", false),
	  o_su = kb.Buffer("sum_u", false);
	V X = kb.Buffer("X", true), U = kb.Buffer("U", true);
	V R = kb.Var("R", TFType_Int), C = kb.Var("C", TFType_Int);
	V c = kb.ThreadIndices({C})[0];
	V a_sum = kb.Accumulator("sum", TFType_Float, FloatBits(0.0f));
	kb.Loop(kb.Const(0), R, kb.Const(1), [&](V r) { kb.Set(a_sum, a_sum + kb.Load(X, r * C + c, TFType_Float)); });
	V a_max = kb.Accumulator("max", TFType_Float, FloatBits(lowest));
	kb.Loop(kb.Const(0), R, kb.Const(1), [&](V r) { kb.Set(a_max, Fn("max", a_max, kb.Load(X, r * C + c, TFType_Float))); });
	V a_min = kb.Accumulator("min", TFType_Float, FloatBits(highest));
	kb.Loop(kb.Const(0), R, kb.Const(1), [&](V r) { kb.Set(a_min, Fn("min", a_min, kb.Load(X, r * C + c, TFType_Float))); });
	V a_sq = kb.Accumulator("sum", TFType_Float, FloatBits(0.0f));
	kb.Loop(kb.Const(0), R, kb.Const(1), [&](V r) {
		V x = kb.Load(X, r * C + c, TFType_Float);
		kb.Set(a_sq, a_sq + x * x);
	});
	V a_su = kb.Accumulator("sum", TFType_Uint, 0u);
	kb.Loop(kb.Const(0), R, kb.Const(1), [&](V r) { kb.Set(a_su, a_su + kb.Load(U, r * C + c, TFType_Uint)); });
	kb.Store(o_sum, c, a_sum);
	kb.Store(o_max, c, a_max);
	kb.Store(o_min, c, a_min);
	kb.Store(o_norm, c, Fn("sqrt", a_sq));
	kb.Store(o_su, c, a_su);
	Kernel* kernel = kb.Finish();
	{
		HostBuilder h(program);
		V Xt = h.Input("X", {-1, -1}, TFType_Float);
		V rows = h.Shape(Xt)[0], cols = h.Shape(Xt)[1];
		V Ut = h.Input("U", {rows, cols}, TFType_Uint);
		V sum = h.Allocate("sum", {cols}, TFType_Float), mx = h.Allocate("max", {cols}, TFType_Float), mn = h.Allocate("min", {cols}, TFType_Float),
		  norm = h.Allocate("norm", {cols}, TFType_Float), su = h.Allocate("sum_u", {cols}, TFType_Uint);
		h.Dispatch(kernel, {sum, mx, mn, norm, su}, {Xt, Ut}, {rows, cols}, {cols});
		for (V out : {sum, mx, mn, norm, su}) h.Output(out);
		h.Finish();
	}
}


static ProgramRegistrar reg_ops("ops", BuildOps);
static ProgramRegistrar reg_bitonic("bitonic_sort", BuildBitonicSort);
static ProgramRegistrar reg_autograd_forward("autograd_network_forward", BuildAutogradNetworkForward);
static ProgramRegistrar reg_split_merge("split_merge", BuildSplitMerge);
static ProgramRegistrar reg_qr("qr_inversion", BuildQrInversion);
static ProgramRegistrar reg_gathered("gathered_updates", BuildGatheredUpdates);
static ProgramRegistrar reg_reshape_reduction("reshape_reduction", BuildReshapeReduction);
static ProgramRegistrar reg_integer_reductions("integer_reductions", BuildIntegerReductions);
static ProgramRegistrar reg_column_statistics("column_statistics", BuildColumnStatistics);
static ProgramRegistrar reg_scatter("radix_scatter_pass", BuildRadixScatterPass);
static ProgramRegistrar reg_dense("dense_layer", BuildDenseLayer);
static ProgramRegistrar reg_dense_tanh("dense_tanh", BuildDenseTanh);
static ProgramRegistrar reg_batched_matmul("batched_matmul", BuildBatchedMatmul);
static ProgramRegistrar reg_indexing("indexing", BuildIndexing);
static ProgramRegistrar reg_broadcast("broadcast_loops", BuildBroadcastLoops);
static ProgramRegistrar reg_atomics("atomics", BuildAtomics);
static ProgramRegistrar reg_group("group_reverse", BuildGroupReverse);
static ProgramRegistrar reg_tile_indices("tile_indices", BuildTileIndices);
static ProgramRegistrar reg_idioms("lowered_idioms", BuildLoweredIdioms);

}  // namespace tfhost
