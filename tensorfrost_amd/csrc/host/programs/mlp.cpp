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
	program->input_count = 27;
	program->output_count = 26;
	program->execute_callback = [k, fused](TFTensor* in, TFTensor* out, TFRuntime runtime) -> int {
		TFContext tf(runtime);
		const float lr = 1e-3f, beta1 = 0.9f, beta2 = 0.999f, eps = 1e-8f;
		const size_t dims[5] = {64, 256, 256, 256, 3};
		TFTensor coords = in[0], target = in[1];
		TFTensor* params = in + 2;
		TFTensor* m = in + 10;
		TFTensor* v = in + 18;
		TFTensor t = in[26];
		tf.region_begin("MLPStep");
		if (coords.dim != 2) throw std::runtime_error("Invalid number of dimensions for coords. Expected 2, got " + std::to_string(coords.dim));
		const int B = (int)coords.shape[0];
		const size_t Bs = (size_t)B;
		tf.check_tensor(coords, "coords", {Bs, 2}, TFTypeFloat32);
		tf.check_tensor(target, "target", {Bs, 3}, TFTypeFloat32);
		for (int l = 0; l < 4; l++) {
			for (TFTensor* set : {params, m, v}) {
				tf.check_tensor(set[2 * l], "W" + std::to_string(l + 1), {dims[l], dims[l + 1]}, TFTypeFloat32);
				tf.check_tensor(set[2 * l + 1], "b" + std::to_string(l + 1), {dims[l + 1]}, TFTypeFloat32);
			}
		}
		tf.check_tensor(t, "t", {1}, TFTypeFloat32);

		// ---- forward ----
		tf.region_begin("forward");
		TFTensor F = tf.allocate("features", {Bs, 64}, TFTypeFloat32);
		tf.dispatch(k.fourier->kernel_id_, {F}, {coords}, {asuint(B)}, {Bs, 64}, {16, 16});
		TFTensor act[4] = {F, {}, {}, {}};
		for (int l = 0; l < 3; l++) {
			TFTensor H = tf.allocate("h" + std::to_string(l + 1), {Bs, 256}, TFTypeFloat32);
			if (fused) {
				tf.dispatch(k.gemm_nn_bias_relu->kernel_id_, {H}, {act[l], params[2 * l], params[2 * l + 1]}, {asuint(B), asuint(256), asuint((int)dims[l])}, {Bs, 256}, {16, 16});
			} else {
				TFTensor Z = tf.allocate("z" + std::to_string(l + 1), {Bs, 256}, TFTypeFloat32);
				tf.dispatch(k.gemm_nn->kernel_id_, {Z}, {act[l], params[2 * l]}, {asuint(B), asuint(256), asuint((int)dims[l])}, {Bs, 256}, {16, 16});
				tf.dispatch(k.bias_relu->kernel_id_, {H}, {Z, params[2 * l + 1]}, {asuint(B), asuint(256)}, {Bs, 256}, {16, 16});
				tf.deallocate(Z);
			}
			act[l + 1] = H;
		}
		TFTensor Y = tf.allocate("y", {Bs, 3}, TFTypeFloat32);
		if (fused) {
			tf.dispatch(k.gemm_nn_bias->kernel_id_, {Y}, {act[3], params[6], params[7]}, {asuint(B), asuint(3), asuint(256)}, {Bs, 3}, {16, 16});
		} else {
			TFTensor Z4 = tf.allocate("z4", {Bs, 3}, TFTypeFloat32);
			tf.dispatch(k.gemm_nn->kernel_id_, {Z4}, {act[3], params[6]}, {asuint(B), asuint(3), asuint(256)}, {Bs, 3}, {3, 16});
			tf.dispatch(k.bias->kernel_id_, {Y}, {Z4, params[7]}, {asuint(B), asuint(3)}, {Bs, 3}, {16, 16});
			tf.deallocate(Z4);
		}
		tf.region_end("forward");

		// ---- loss and its gradient ----
		const int count = B * 3;
		TFTensor dY = tf.allocate("dy", {Bs, 3}, TFTypeFloat32);
		TFTensor sq = tf.allocate("sq", {Bs, 3}, TFTypeFloat32);
		tf.dispatch(k.mse_grad->kernel_id_, {dY, sq}, {Y, target}, {asuint(count), asuint(2.0f / (float)count)}, {(size_t)count}, {256});
		TFTensor loss_sum = tf.allocate("loss_sum", {1}, TFTypeFloat32);
		tf.dispatch(k.sum_rows->kernel_id_, {loss_sum}, {sq}, {asuint(1), asuint(count)}, {1}, {256});
		TFTensor loss = tf.allocate("loss", {1}, TFTypeFloat32);
		tf.dispatch(k.scale1->kernel_id_, {loss}, {loss_sum}, {asuint(1.0f / (float)count)}, {1}, {256});
		tf.deallocate(sq);
		tf.deallocate(loss_sum);
		tf.deallocate(Y);

		// ---- backward ----
		tf.region_begin("backward");
		TFTensor grads[8];
		TFTensor upstream = dY;
		for (int l = 3; l >= 0; l--) {
			const size_t in_n = dims[l], out_n = dims[l + 1];
			grads[2 * l] = tf.allocate("dW" + std::to_string(l + 1), {in_n, out_n}, TFTypeFloat32);
			grads[2 * l + 1] = tf.allocate("db" + std::to_string(l + 1), {out_n}, TFTypeFloat32);
			tf.dispatch(k.gemm_tn->kernel_id_, {grads[2 * l]}, {act[l], upstream}, {asuint((int)in_n), asuint((int)out_n), asuint(B)}, {in_n, out_n}, {16, 16});
			tf.dispatch(k.sum_cols->kernel_id_, {grads[2 * l + 1]}, {upstream}, {asuint(B), asuint((int)out_n)}, {out_n}, {256});
			if (l > 0) {
				TFTensor dZ = tf.allocate("dz" + std::to_string(l), {Bs, in_n}, TFTypeFloat32);
				if (fused) {
					tf.dispatch(k.gemm_nt_mask->kernel_id_, {dZ}, {upstream, params[2 * l], act[l]}, {asuint(B), asuint((int)in_n), asuint((int)out_n)}, {Bs, in_n}, {16, 16});
				} else {
					TFTensor dH = tf.allocate("dh" + std::to_string(l), {Bs, in_n}, TFTypeFloat32);
					tf.dispatch(k.gemm_nt->kernel_id_, {dH}, {upstream, params[2 * l]}, {asuint(B), asuint((int)in_n), asuint((int)out_n)}, {Bs, in_n}, {16, 16});
					const int n = B * (int)in_n;
					tf.dispatch(k.relu_bwd->kernel_id_, {dZ}, {dH, act[l]}, {asuint(n)}, {(size_t)n}, {256});
					tf.deallocate(dH);
				}
				tf.deallocate(upstream);
				upstream = dZ;
			}
			tf.deallocate(act[l]);
		}
		tf.deallocate(upstream);
		tf.region_end("backward");

		// ---- Adam ----
		tf.region_begin("adam");
		TFTensor t_new = tf.allocate("t", {1}, TFTypeFloat32);
		tf.dispatch(k.t_inc->kernel_id_, {t_new}, {t}, {asuint(1.0f)}, {1}, {256});
		out[0] = loss;
		for (int i = 0; i < 8; i++) {
			const bool matrix = (i % 2) == 0;
			const size_t rows = dims[i / 2], cols = dims[i / 2 + 1];
			const int n = matrix ? (int)(rows * cols) : (int)cols;
			TFTensor p_new = matrix ? tf.allocate("p", {rows, cols}, TFTypeFloat32) : tf.allocate("p", {cols}, TFTypeFloat32);
			TFTensor m_new = matrix ? tf.allocate("m", {rows, cols}, TFTypeFloat32) : tf.allocate("m", {cols}, TFTypeFloat32);
			TFTensor v_new = matrix ? tf.allocate("v", {rows, cols}, TFTypeFloat32) : tf.allocate("v", {cols}, TFTypeFloat32);
			tf.dispatch(k.adam->kernel_id_, {p_new, m_new, v_new}, {params[i], grads[i], m[i], v[i], t_new},
			            {asuint(n), asuint(lr), asuint(beta1), asuint(beta2), asuint(eps)}, {(size_t)n}, {256});
			tf.deallocate(grads[i]);
			out[1 + i] = p_new;
			out[9 + i] = m_new;
			out[17 + i] = v_new;
		}
		out[25] = t_new;
		tf.region_end("adam");
		tf.region_end("MLPStep");
		return 0;
	};
}

static ProgramRegistrar reg_mlp("mlp", BuildMlp);

}  // namespace tfhost
