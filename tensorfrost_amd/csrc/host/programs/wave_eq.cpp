// benchmark config 1: one leapfrog step of the 2-D sine-Gordon equation u'' = lap(u) - sin(u) on a periodic
// grid, one fused kernel per step. The traced function would be (TensorFrost Python, cf. README.md:153-166
// and examples/Simulation/wave_simulation.ipynb for the clamped-boundary variant the reference ships):
//
//   def WaveEq():
//       u = tf.input([-1, -1], tf.float32); N, M = u.shape; v = tf.input([N, M], tf.float32)
//       i, j = u.indices
//       lap = u[(i+N-1)%N, j] + u[(i+1)%N, j] + u[i, (j+M-1)%M] + u[i, (j+1)%M] - 4.0*u
//       v_new = v + dt*(lap - tf.sin(u)); u_new = u + dt*v_new
//       return v_new, u_new
//
// User-written loads index in Clamp mode (Tensor.h:566-567), so every tap is clamp(idx, 0, extent-1) on top
// of the explicit non-negative modulus (integer % is emitted verbatim, Operations.cpp:116).
#include "registry.h"

namespace tfhost {

static void BuildWaveEq(Program* program, const std::vector<int64_t>& params) {
	const float dt = params.size() > 0 ? (float)params[0] / 1000.0f : 0.1f;  // params[0] = dt in thousandths

	KernelBuilder b(program, 2);
	V v_new = b.Buffer("v_new", false);
	V u_new = b.Buffer("u_new", false);
	V u = b.Buffer("u", true);
	V v = b.Buffer("v", true);
	V N = b.Var("N", TFType_Int);
	V M = b.Var("M", TFType_Int);
	std::vector<V> idx = b.ThreadIndices({M, N});  // innermost first: index_0 = column j, index_1 = row i
	V j = idx[0], i = idx[1];
	auto tap = [&](V row, V col) {
		V r = b.Clamp(row, b.Const(0), N - b.Const(1));
		V c = b.Clamp(col, b.Const(0), M - b.Const(1));
		return b.Load(u, r * M + c, TFType_Float);
	};
	V centre = b.Named(b.Load(u, i * M + j, TFType_Float), "u");
	V up = tap((i + N - b.Const(1)) % N, j);
	V down = tap((i + b.Const(1)) % N, j);
	V left = tap(i, (j + M - b.Const(1)) % M);
	V right = tap(i, (j + b.Const(1)) % M);
	V lap = b.Named(up + down + left + right - b.Const(4.0f) * centre, "lap");
	V vel = b.Named(b.Load(v, i * M + j, TFType_Float), "v");
	V vn = b.Named(vel + b.Const(dt) * (lap - Fn("sin", centre)), "v_new");
	V un = b.Named(centre + b.Const(dt) * vn, "u_new");
	b.Store(v_new, i * M + j, vn);
	b.Store(u_new, i * M + j, un);
	Kernel* kernel = b.Finish();

	program->input_count = 2;
	program->output_count = 2;
	// Host program in the emitted form (CPP.cpp:678-718): shape reads, input checks, allocations, dispatch.
	program->execute_callback = [kernel](TFTensor* in, TFTensor* out, TFRuntime runtime) -> int {
		TFContext tf(runtime);
		TFTensor u = in[0], v = in[1];
		tf.region_begin("WaveEq");
		if (u.dim != 2) throw std::runtime_error("Invalid number of dimensions for u. Expected 2, got " + std::to_string(u.dim));
		int N = (int)u.shape[0];
		int M = (int)u.shape[1];
		tf.check_tensor(u, "u", {(size_t)N, (size_t)M}, TFTypeFloat32);
		tf.check_tensor(v, "v", {(size_t)N, (size_t)M}, TFTypeFloat32);
		TFTensor v_new = tf.allocate("v_new", {(size_t)N, (size_t)M}, TFTypeFloat32);
		TFTensor u_new = tf.allocate("u_new", {(size_t)N, (size_t)M}, TFTypeFloat32);
		tf.dispatch(kernel->kernel_id_, {v_new, u_new}, {u, v}, {asuint(N), asuint(M)}, {(size_t)N, (size_t)M}, {16, 16});
		tf.region_end("WaveEq");
		out[0] = v_new;
		out[1] = u_new;
		return 0;
	};
}

static ProgramRegistrar reg_wave_eq("wave_eq", BuildWaveEq);

}  // namespace tfhost
