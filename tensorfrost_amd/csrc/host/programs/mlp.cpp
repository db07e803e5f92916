// benchmark config 5: one training step (forward, backward through autodiff, Adam) of a coordinate MLP:
// 2-D coordinates -> 64 Fourier features -> 256 -> 256 -> 256 -> 3 with ReLU, mean-squared error.
// In TensorFrost this is a tf.Module with tf.optimizers.adam (Python/TensorFrost/optimizers.py:104-167)
// compiled into one program whose inputs and outputs are the batch, the parameters, the Adam moments and the
// step counter. After lowering it consists of
//   - element-wise kernels (features, loss gradient, Adam), emitted as HIP, and
//   - matmul / dim_sum idioms (Compiler/Implementations.cpp:560-646, 243-303; VJPs :133-135, :115), which the
//     backend serves with its MFMA sgemm and column-reduction primitives. Kernel fusion leaves the bias add and
//     ReLU of a layer behind the layer's matmul loop, and the ReLU mask of the backward pass behind the loop of
//     dX = dY W^T; those kernels are served by the sgemm with the matching fused tail. params[0] = 1 builds the
//     unfused form instead (separate bias + ReLU and mask kernels), which the tests compare against.
// The host function below sequences them the way the generated `main` would.
#include "registry.h"

namespace tfhost {

namespace {

struct MlpKernels {
	Kernel *fourier, *bias_relu, *bias, *mse_grad, *relu_bwd, *adam, *scale1, *t_inc;
	Kernel *gemm_nn, *gemm_nt, *gemm_tn, *sum_cols, *sum_rows;
	Kernel *gemm_nn_bias_relu, *gemm_nn_bias, *gemm_nt_mask;
};

Kernel* BuildFourier(Program* program) {
	KernelBuilder b(program, 2);
	V F = b.Buffer("features", false);
	V coords = b.Buffer("coords", true);
	V B = b.Var("B", TFType_Int);
	std::vector<V> idx = b.ThreadIndices({b.Const(64), B});
	V f = idx[0], row = idx[1];
	V axis = b.Named(f / b.Const(32), "axis");
	V k = b.Named((f % b.Const(32)) / b.Const(2), "k");
	V c = b.Named(b.Load(coords, b.Clamp(row, b.Const(0), B - b.Const(1)) * b.Const(2) + b.Clamp(axis, b.Const(0), b.Const(1)), TFType_Float), "c");
	V arg = b.Named(ToFloat(b.Const(1) << k) * b.Const(3.14159274f) * c, "arg");
	V val = Select((f % b.Const(2)) == b.Const(0), Fn("sin", arg), Fn("cos", arg));
	b.Store(F, row * b.Const(64) + f, val);
	return b.Finish();
}

Kernel* BuildBiasAct(Program* program, bool relu) {
	KernelBuilder b(program, 2);
	V H = b.Buffer("h", false);
	V Z = b.Buffer("z", true);
	V bias = b.Buffer("bias", true);
	V B = b.Var("B", TFType_Int);
	V N = b.Var("N", TFType_Int);
	std::vector<V> idx = b.ThreadIndices({N, B});
	V j = idx[0], row = idx[1];
	V z = b.Load(Z, row * N + j, TFType_Float) + b.Load(bias, j, TFType_Float);
	b.Store(H, row * N + j, relu ? Fn("max", z, b.Const(0.0f)) : z);
	return b.Finish();
}

Kernel* BuildMseGrad(Program* program) {
	KernelBuilder b(program, 1);
	V dY = b.Buffer("dy", false);
	V sq = b.Buffer("sq", false);
	V Y = b.Buffer("y", true);
	V T = b.Buffer("target", true);
	V count = b.Var("count", TFType_Int);
	V scale = b.Var("scale", TFType_Float);
	V i = b.ThreadIndices({count})[0];
	V d = b.Named(b.Load(Y, i, TFType_Float) - b.Load(T, i, TFType_Float), "d");
	b.Store(sq, i, d * d);
	b.Store(dY, i, d * scale);
	return b.Finish();
}

Kernel* BuildReluBackward(Program* program) {
	KernelBuilder b(program, 1);
	V dZ = b.Buffer("dz", false);
	V dH = b.Buffer("dh", true);
	V H = b.Buffer("h", true);
	V count = b.Var("count", TFType_Int);
	V i = b.ThreadIndices({count})[0];
	V g = b.Load(dH, i, TFType_Float);
	V h = b.Load(H, i, TFType_Float);
	b.Store(dZ, i, Select(h > b.Const(0.0f), g, b.Const(0.0f)));
	return b.Finish();
}

Kernel* BuildAdam(Program* program) {
	KernelBuilder b(program, 1);
	V p_new = b.Buffer("p_new", false);
	V m_new = b.Buffer("m_new", false);
	V v_new = b.Buffer("v_new", false);
	V p = b.Buffer("p", true);
	V g = b.Buffer("g", true);
	V m = b.Buffer("m", true);
	V v = b.Buffer("v", true);
	V t = b.Buffer("t", true);
	V count = b.Var("count", TFType_Int);
	V lr = b.Var("lr", TFType_Float);
	V beta1 = b.Var("beta1", TFType_Float);
	V beta2 = b.Var("beta2", TFType_Float);
	V eps = b.Var("eps", TFType_Float);
	V i = b.ThreadIndices({count})[0];
	V grad = b.Named(b.Load(g, i, TFType_Float), "grad");
	V mm = b.Named(Fn("lerp", grad, b.Load(m, i, TFType_Float), beta1), "m_lerp");
	V vv = b.Named(Fn("lerp", grad * grad, b.Load(v, i, TFType_Float), beta2), "v_lerp");
	V t_val = b.Named(b.Load(t, b.Const(0), TFType_Float), "t_val");
	V mhat = b.Named(mm / (b.Const(1.0f) - Fn("pow", beta1, t_val)), "mhat");
	V vhat = b.Named(vv / (b.Const(1.0f) - Fn("pow", beta2, t_val)), "vhat");
	b.Store(m_new, i, mm);
	b.Store(v_new, i, vv);
	b.Store(p_new, i, b.Load(p, i, TFType_Float) - lr * mhat / (Fn("sqrt", vhat) + eps));
	return b.Finish();
}

// out[0] = in[0] * s  and  out[0] = in[0] + s, on one-element tensors
Kernel* BuildScalarOp(Program* program, bool add) {
	KernelBuilder b(program, 1);
	V out = b.Buffer("result", false);
	V in = b.Buffer("value", true);
	V s = b.Var("s", TFType_Float);
	V i = b.ThreadIndices({b.Const(1)})[0];
	V x = b.Load(in, i, TFType_Float);
	b.Store(out, i, add ? x + s : x * s);
	return b.Finish();
}


// The lowered loops (Compiler/Implementations.cpp:560-646 matmul, :243-303 dim_sum) with the tails kernel fusion leaves.
// C[M,N] = A[M,K] B[K,N] (+ bias[N], optionally through ReLU)
Kernel* BuildMatmulForward(Program* program, int tail) {  // 0 none, 1 bias, 2 bias + ReLU
	KernelBuilder kb(program, 2);
	V C = kb.Buffer("C", false), A = kb.Buffer("A", true), B = kb.Buffer("B", true);
	V bias = tail ? kb.Buffer("bias", true) : V();
	V M = kb.Var("M", TFType_Int), N = kb.Var("N", TFType_Int), K = kb.Var("K", TFType_Int);
	(void)M;
	std::vector<V> idx = kb.ThreadIndices({N, M});
	V j = idx[0], i = idx[1];
	V acc = kb.Accumulator("matmul", TFType_Float, FloatBits(0.0f));
	kb.Loop(kb.Const(0), K, kb.Const(1), [&](V k) { kb.Set(acc, acc + kb.Load(A, i * K + k, TFType_Float) * kb.Load(B, k * N + j, TFType_Float)); });
	if (tail == 0) {
		kb.Store(C, i * N + j, acc);
	} else {
		V z = acc + kb.Load(bias, j, TFType_Float);
		kb.Store(C, i * N + j, tail == 2 ? Fn("max", z, kb.Const(0.0f)) : z);
	}
	return kb.Finish();
}

// dX[M,N] = dY[M,K] W[N,K]^T where act[M,N] > 0, else 0
Kernel* BuildMatmulInputGradient(Program* program) {
	KernelBuilder kb(program, 2);
	V dX = kb.Buffer("dX", false), dY = kb.Buffer("dY", true), W = kb.Buffer("W", true), act = kb.Buffer("act", true);
	V M = kb.Var("M", TFType_Int), N = kb.Var("N", TFType_Int), K = kb.Var("K", TFType_Int);
	(void)M;
	std::vector<V> idx = kb.ThreadIndices({N, M});
	V c = idx[0], i = idx[1];
	V acc = kb.Accumulator("matmul", TFType_Float, FloatBits(0.0f));
	kb.Loop(kb.Const(0), K, kb.Const(1), [&](V n) { kb.Set(acc, acc + kb.Load(dY, i * K + n, TFType_Float) * kb.Load(W, c * K + n, TFType_Float)); });
	V h = kb.Load(act, i * N + c, TFType_Float);
	kb.Store(dX, i * N + c, Select(h > kb.Const(0.0f), acc, kb.Const(0.0f)));
	return kb.Finish();
}

// dW[M,N] = X[K,M]^T dY[K,N]
Kernel* BuildMatmulWeightGradient(Program* program) {
	KernelBuilder kb(program, 2);
	V dW = kb.Buffer("dW", false), X = kb.Buffer("X", true), dY = kb.Buffer("dY", true);
	V M = kb.Var("M", TFType_Int), N = kb.Var("N", TFType_Int), K = kb.Var("K", TFType_Int);
	std::vector<V> idx = kb.ThreadIndices({N, M});
	V j = idx[0], i = idx[1];
	V acc = kb.Accumulator("matmul", TFType_Float, FloatBits(0.0f));
	kb.Loop(kb.Const(0), K, kb.Const(1), [&](V k) { kb.Set(acc, acc + kb.Load(X, k * M + i, TFType_Float) * kb.Load(dY, k * N + j, TFType_Float)); });
	kb.Store(dW, i * N + j, acc);
	return kb.Finish();
}

// out[j] = sum_k x[k, j] over x[R, N] (the bias gradients)    and    out[t] = sum_k x[t, k] over x[T, K] (the loss)
Kernel* BuildSum(Program* program, bool down) {
	KernelBuilder kb(program, 1);
	V out = kb.Buffer("sum", false), x = kb.Buffer("x", true);
	V A = kb.Var(down ? "R" : "T", TFType_Int), B = kb.Var(down ? "N" : "K", TFType_Int);
	V t = kb.ThreadIndices({down ? B : A})[0];
	V acc = kb.Accumulator("sum", TFType_Float, FloatBits(0.0f));
	kb.Loop(kb.Const(0), down ? A : B, kb.Const(1), [&](V k) { kb.Set(acc, acc + kb.Load(x, down ? k * B + t : t * B + k, TFType_Float)); });
	kb.Store(out, t, acc);
	return kb.Finish();
}

}  // namespace

static void BuildMlp(Program* program, const std::vector<int64_t>& build_params) {
	const bool fused = build_params.empty() || build_params[0] != 1;
	const bool lowered = !build_params.empty() && build_params[0] == 2;
	// params[1] = 1: every layer's bias gradient is dispatched before its weight gradient (the order of the two is the
	// order in which autodiff visits the layer's inputs, which nothing fixes)
	const bool bias_gradient_first = build_params.size() > 1 && build_params[1] == 1;
	MlpKernels k;
	k.fourier = BuildFourier(program);
	k.bias_relu = BuildBiasAct(program, true);
	k.bias = BuildBiasAct(program, false);
	k.mse_grad = BuildMseGrad(program);
	k.relu_bwd = BuildReluBackward(program);
	k.adam = BuildAdam(program);
	k.scale1 = BuildScalarOp(program, false);
	k.t_inc = BuildScalarOp(program, true);
	if (lowered) {
		k.gemm_nn = BuildMatmulForward(program, 0);
		k.gemm_nn_bias = BuildMatmulForward(program, 1);
		k.gemm_nn_bias_relu = BuildMatmulForward(program, 2);
		k.gemm_nt = nullptr;  // only the unfused form dispatches it
		k.gemm_nt_mask = BuildMatmulInputGradient(program);
		k.gemm_tn = BuildMatmulWeightGradient(program);
		k.sum_cols = BuildSum(program, true);
		k.sum_rows = BuildSum(program, false);
	} else {
		k.gemm_nn = program->AddPrimitive("sgemm_nn", 3, 3);
		k.gemm_nt = program->AddPrimitive("sgemm_nt", 3, 3);
		k.gemm_tn = program->AddPrimitive("sgemm_tn", 3, 3);
		k.gemm_nn_bias_relu = program->AddPrimitive("sgemm_nn_bias_relu", 4, 3);
		k.gemm_nn_bias = program->AddPrimitive("sgemm_nn_bias", 4, 3);
		k.gemm_nt_mask = program->AddPrimitive("sgemm_nt_mask_positive", 4, 3);
		k.sum_cols = program->AddPrimitive("reduce_cols_sum", 2, 2);
		k.sum_rows = program->AddPrimitive("reduce_rows_sum", 2, 2);
	}

	// inputs: coords, target, 8 parameters, 8 first moments, 8 second moments, t
	// outputs: loss, 8 parameters, 8 first moments, 8 second moments, t
	// The layer loops are Python loops of the traced function, so tracing unrolls them: one set of nodes per layer.
	HostBuilder h(program);
	const float lr = 1e-3f, beta1 = 0.9f, beta2 = 0.999f, eps = 1e-8f;
	const int dims[5] = {64, 256, 256, 256, 3};
	h.RegionBegin("MLPStep");
	V coords = h.Input("coords", {-1, 2}, TFType_Float);
	V B = h.Shape(coords)[0];
	V target = h.Input("target", {B, 3}, TFType_Float);
	V params[8], m[8], v[8];
	for (V* set : {params, m, v}) {
		for (int l = 0; l < 4; l++) {
			set[2 * l] = h.Input("W" + std::to_string(l + 1), {dims[l], dims[l + 1]}, TFType_Float);
			set[2 * l + 1] = h.Input("b" + std::to_string(l + 1), {dims[l + 1]}, TFType_Float);
		}
	}
	V t = h.Input("t", {1}, TFType_Float);
	auto extent = [&](int n) { return h.Const(n); };

	// ---- forward ----
	h.RegionBegin("forward");
	V F = h.Allocate("features", {B, 64}, TFType_Float);
	h.Dispatch(k.fourier, {F}, {coords}, {B}, {B, 64});
	V act[4] = {F, V(), V(), V()};
	for (int l = 0; l < 3; l++) {
		V H = h.Allocate("h" + std::to_string(l + 1), {B, 256}, TFType_Float);
		if (fused) {
			h.Dispatch(k.gemm_nn_bias_relu, {H}, {act[l], params[2 * l], params[2 * l + 1]}, {B, extent(256), extent(dims[l])}, {B, 256});
		} else {
			V Z = h.Allocate("z" + std::to_string(l + 1), {B, 256}, TFType_Float);
			h.Dispatch(k.gemm_nn, {Z}, {act[l], params[2 * l]}, {B, extent(256), extent(dims[l])}, {B, 256});
			h.Dispatch(k.bias_relu, {H}, {Z, params[2 * l + 1]}, {B, extent(256)}, {B, 256});
			h.Deallocate(Z);
		}
		act[l + 1] = H;
	}
	V Y = h.Allocate("y", {B, 3}, TFType_Float);
	if (fused) {
		h.Dispatch(k.gemm_nn_bias, {Y}, {act[3], params[6], params[7]}, {B, extent(3), extent(256)}, {B, 3});
	} else {
		V Z4 = h.Allocate("z4", {B, 3}, TFType_Float);
		h.Dispatch(k.gemm_nn, {Z4}, {act[3], params[6]}, {B, extent(3), extent(256)}, {B, 3});
		h.Dispatch(k.bias, {Y}, {Z4, params[7]}, {B, extent(3)}, {B, 3});
		h.Deallocate(Z4);
	}
	h.RegionEnd("forward");

	// ---- loss and its gradient ----
	V count = B * h.Const(3);
	V dY = h.Allocate("dy", {B, 3}, TFType_Float);
	V sq = h.Allocate("sq", {B, 3}, TFType_Float);
	h.Dispatch(k.mse_grad, {dY, sq}, {Y, target}, {count, h.Const(2.0f) / ToFloat(count)}, {count});
	V loss_sum = h.Allocate("loss_sum", {1}, TFType_Float);
	h.Dispatch(k.sum_rows, {loss_sum}, {sq}, {extent(1), count}, {1});
	V loss = h.Allocate("loss", {1}, TFType_Float);
	h.Dispatch(k.scale1, {loss}, {loss_sum}, {h.Const(1.0f) / ToFloat(count)}, {1});
	h.Deallocate(sq);
	h.Deallocate(loss_sum);
	h.Deallocate(Y);

	// ---- backward ----
	h.RegionBegin("backward");
	V grads[8];
	V upstream = dY;
	for (int l = 3; l >= 0; l--) {
		const int in_n = dims[l], out_n = dims[l + 1];
		grads[2 * l] = h.Allocate("dW" + std::to_string(l + 1), {in_n, out_n}, TFType_Float);
		grads[2 * l + 1] = h.Allocate("db" + std::to_string(l + 1), {out_n}, TFType_Float);
		if (bias_gradient_first) h.Dispatch(k.sum_cols, {grads[2 * l + 1]}, {upstream}, {B, extent(out_n)}, {out_n});
		h.Dispatch(k.gemm_tn, {grads[2 * l]}, {act[l], upstream}, {extent(in_n), extent(out_n), B}, {in_n, out_n});
		if (!bias_gradient_first) h.Dispatch(k.sum_cols, {grads[2 * l + 1]}, {upstream}, {B, extent(out_n)}, {out_n});
		if (l > 0) {
			V dZ = h.Allocate("dz" + std::to_string(l), {B, in_n}, TFType_Float);
			if (fused) {
				h.Dispatch(k.gemm_nt_mask, {dZ}, {upstream, params[2 * l], act[l]}, {B, extent(in_n), extent(out_n)}, {B, in_n});
			} else {
				V dH = h.Allocate("dh" + std::to_string(l), {B, in_n}, TFType_Float);
				h.Dispatch(k.gemm_nt, {dH}, {upstream, params[2 * l]}, {B, extent(in_n), extent(out_n)}, {B, in_n});
				V elements = B * h.Const(in_n);
				h.Dispatch(k.relu_bwd, {dZ}, {dH, act[l]}, {elements}, {elements});
				h.Deallocate(dH);
			}
			h.Deallocate(upstream);
			upstream = dZ;
		}
		h.Deallocate(act[l]);
	}
	h.Deallocate(upstream);
	h.RegionEnd("backward");

	// ---- Adam ----
	h.RegionBegin("adam");
	V t_new = h.Allocate("t", {1}, TFType_Float);
	h.Dispatch(k.t_inc, {t_new}, {t}, {h.Const(1.0f)}, {1});
	V p_out[8], m_out[8], v_out[8];
	for (int i = 0; i < 8; i++) {
		const bool matrix = (i % 2) == 0;
		const int rows = dims[i / 2], cols = dims[i / 2 + 1];
		const int n = matrix ? rows * cols : cols;
		const std::vector<Dim> shape = matrix ? std::vector<Dim>{rows, cols} : std::vector<Dim>{cols};
		p_out[i] = h.Allocate("p", shape, TFType_Float);
		m_out[i] = h.Allocate("m", shape, TFType_Float);
		v_out[i] = h.Allocate("v", shape, TFType_Float);
		h.Dispatch(k.adam, {p_out[i], m_out[i], v_out[i]}, {params[i], grads[i], m[i], v[i], t_new}, {extent(n), h.Const(lr), h.Const(beta1), h.Const(beta2), h.Const(eps)}, {n});
		h.Deallocate(grads[i]);
	}
	h.RegionEnd("adam");
	h.RegionEnd("MLPStep");
	h.Output(loss);
	for (V* set : {p_out, m_out, v_out})
		for (int i = 0; i < 8; i++) h.Output(set[i]);
	h.Output(t_new);
	h.Finish();
}

static ProgramRegistrar reg_mlp("mlp", BuildMlp);

}  // namespace tfhost
