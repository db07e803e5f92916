// TEST INFRASTRUCTURE -- not part of the product (see prelude.h).
//
// One training step of the coordinate MLP of benchmark config 5 as the reference's C++/OpenMP backend would
// run it: Fourier features, 64 -> 256 -> 256 -> 256 -> 3 with ReLU, MSE loss, backward pass by the reference's
// VJP rules, Adam. Every piece is one generated-style kernel (one thread per output element, 16x16 or 256
// groups); matmuls are the serial-k kernels of matmul.cpp, bias gradients the axis-0 reductions of reduce.cpp
// (262144 >= 1024, so they take the 128-chunk split).
// Follows:
//   matmul forward / backward   TensorFrost/Compiler/Implementations.cpp:560-646, VJP :133-135 (dA = dC B^T, dB = A^T dC)
//   ReLU as max(z, 0)           VJP of max: select(a > b, grad, 0)   (Implementations.cpp:115)
//   Adam                        Python/TensorFrost/optimizers.py:104-167: t += 1; m = lerp(g, m, b1);
//                               v = lerp(g*g, v, b2); mhat = m / (1 - pow(b1, t)); vhat = v / (1 - pow(b2, t));
//                               p -= lr * mhat / (sqrt(vhat) + eps), with lerp(a, b, t) = a + (b - a) * t (CPP.cpp:103-106)
//   mean-squared error          loss = sum((y - target)^2) / count
//
// Pins (tests/test_oracle_mlp.py): the whole step against a float64 NumPy restatement with gradients checked
// by central finite differences of the float64 loss (so a wrong VJP fails), and Adam against the textbook
// update on hand-sized vectors.

#include <vector>

#include "prelude.h"

using namespace tfo;

extern "C" int oracle_matmul_f32(int layout, const float* A, const float* B, float* C, int M, int N, int K);
extern "C" int oracle_reduce_cols_f32(int op, const float* x, float* out, float* partial, int R, int C);
extern "C" size_t oracle_reduce_partial_words(size_t other, size_t K);

namespace {

#define TFO_2D_PROLOGUE(INNER, OUTER)                                                         \
	int blocks_shape_0 = (((INNER) + 16) - 1) / 16;                                           \
	int vdiv = block_id / blocks_shape_0;                                                     \
	int index_0 = ((block_id - (vdiv * blocks_shape_0)) * 16) + block_thread_id0;             \
	int index_1 = (vdiv * 16) + block_thread_id1;                                             \
	bool is_inside_dispatch = (index_0 < (INNER)) && (index_1 < (OUTER));

template <class Body>
void run_2d(int outer, int inner, Body body) {
	size_t shape[2] = {(size_t)outer, (size_t)inner}, group[2] = {16, 16};
	int groups = (int)work_group_count(shape, 2, group, 2);
#pragma omp parallel for
	for (int block_id = 0; block_id < groups; block_id++)
		for (int block_thread_id1 = 0; block_thread_id1 < 16; block_thread_id1++)
			for (int block_thread_id0 = 0; block_thread_id0 < 16; block_thread_id0++) {
				TFO_2D_PROLOGUE(inner, outer)
				if (is_inside_dispatch) body(index_1, index_0);
			}
}

template <class Body>
void run_1d(int n, Body body) {
	size_t shape[1] = {(size_t)n}, group[1] = {256};
	int groups = (int)work_group_count(shape, 1, group, 1);
#pragma omp parallel for
	for (int block_id = 0; block_id < groups; block_id++)
		for (int block_thread_id0 = 0; block_thread_id0 < 256; block_thread_id0++) {
			int index_0 = (block_id * 256) + block_thread_id0;
			if (index_0 < n) body(index_0);
		}
}

}  // namespace

extern "C" {

// F[b, f]: f = (axis*16 + k)*2 + s -> s == 0 ? sin(2^k pi c[b, axis]) : cos(...)
void oracle_fourier_features(const float* coords, float* F, int B) {
	run_2d(B, 64, [&](int b, int f) {
		int axis = f / 32;
		int k = (f % 32) / 2;
		float arg = ((float)(1 << k) * 3.14159274f) * coords[(b * 2) + axis];
		F[(b * 64) + f] = (f % 2) == 0 ? sinf(arg) : cosf(arg);
	});
}

// H[b, j] = max(Z[b, j] + bias[j], 0)   (relu != 0) or Z + bias
void oracle_bias_act(const float* Z, const float* bias, float* H, int B, int N, int relu) {
	run_2d(B, N, [&](int b, int j) {
		float z = Z[(b * N) + j] + bias[j];
		H[(b * N) + j] = relu ? max(z, 0.0f) : z;
	});
}

// dY = (Y - T) * (2 / count); sq = (Y - T)^2
void oracle_mse_grad(const float* Y, const float* T, float* dY, float* sq, int count) {
	run_1d(count, [&](int i) {
		float d = Y[i] - T[i];
		sq[i] = d * d;
		dY[i] = d * (2.0f / (float)count);
	});
}

// dZ = H > 0 ? dH : 0
void oracle_relu_backward(const float* dH, const float* H, float* dZ, int count) {
	run_1d(count, [&](int i) { dZ[i] = H[i] > 0.0f ? dH[i] : 0.0f; });
}

void oracle_adam(const float* p, const float* g, const float* m, const float* v, float t, float lr, float b1, float b2, float eps,
                 float* p_new, float* m_new, float* v_new, int count) {
	run_1d(count, [&](int i) {
		float grad = g[i];
		float mm = lerp(grad, m[i], b1);
		float vv = lerp(grad * grad, v[i], b2);
		float mhat = mm / (1.0f - powf(b1, t));
		float vhat = vv / (1.0f - powf(b2, t));
		m_new[i] = mm;
		v_new[i] = vv;
		p_new[i] = p[i] - ((lr * mhat) / (sqrtf(vhat) + eps));
	});
}

// One full step. params: W1 b1 W2 b2 W3 b3 W4 b4 (then the same order for m, v and the outputs).
// grads_out (optional): the eight gradients in the same order. Returns the loss.
float oracle_mlp_step(const float* coords, const float* target, int B, const float* const* params, const float* const* m, const float* const* v, float t,
                      float lr, float b1, float b2, float eps, float* const* params_out, float* const* m_out, float* const* v_out, float* const* grads_out) {
	const int dims[5] = {64, 256, 256, 256, 3};
	std::vector<float> F((size_t)B * 64), Z((size_t)B * 256), H[3], Y((size_t)B * 3), dY((size_t)B * 3), sq((size_t)B * 3);
	oracle_fourier_features(coords, F.data(), B);
	const float* act = F.data();
	for (int l = 0; l < 3; l++) {
		H[l].resize((size_t)B * 256);
		oracle_matmul_f32(0, act, params[2 * l], Z.data(), B, 256, dims[l]);
		oracle_bias_act(Z.data(), params[2 * l + 1], H[l].data(), B, 256, 1);
		act = H[l].data();
	}
	std::vector<float> Z4((size_t)B * 3);
	oracle_matmul_f32(0, act, params[6], Z4.data(), B, 3, 256);
	oracle_bias_act(Z4.data(), params[7], Y.data(), B, 3, 0);
	oracle_mse_grad(Y.data(), target, dY.data(), sq.data(), B * 3);
	float loss = 0.0f;
	{
		// tf.sum over all elements of a [count] tensor: a serial loop in one thread (split in chunks of 128 when
		// count >= 1024); the value is reported for monitoring only.
		double acc = 0.0;
		for (size_t i = 0; i < sq.size(); i++) acc += sq[i];
		loss = (float)(acc / (double)(B * 3));
	}

	std::vector<std::vector<float>> grads(8);
	std::vector<float> dH((size_t)B * 256), dZ((size_t)B * 256);
	const float* upstream = dY.data();
	int up_n = 3;
	for (int l = 3; l >= 0; l--) {
		const int in_n = dims[l], out_n = dims[l + 1];
		const float* layer_in = l == 0 ? F.data() : H[l - 1].data();
		grads[2 * l].resize((size_t)in_n * out_n);
		grads[2 * l + 1].resize(out_n);
		oracle_matmul_f32(2, layer_in, upstream, grads[2 * l].data(), in_n, out_n, B);  // dW = X^T dZ
		std::vector<float> partial(oracle_reduce_partial_words(out_n, B));
		oracle_reduce_cols_f32(0, upstream, grads[2 * l + 1].data(), partial.data(), B, out_n);  // db = sum over the batch
		if (l > 0) {
			oracle_matmul_f32(1, upstream, params[2 * l], dH.data(), B, in_n, out_n);  // dX = dZ W^T
			oracle_relu_backward(dH.data(), H[l - 1].data(), dZ.data(), B * in_n);
			upstream = dZ.data();
			up_n = in_n;
		}
	}
	(void)up_n;
	const float t_new = t + 1.0f;
	for (int i = 0; i < 8; i++) {
		const int count = (int)grads[i].size();
		oracle_adam(params[i], grads[i].data(), m[i], v[i], t_new, lr, b1, b2, eps, params_out[i], m_out[i], v_out[i], count);
		if (grads_out) std::memcpy(grads_out[i], grads[i].data(), sizeof(float) * count);
	}
	return loss;
}

}  // extern "C"
