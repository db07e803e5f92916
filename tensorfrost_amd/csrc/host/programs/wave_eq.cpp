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

	// Host part of the tree: u's two extents are open (tf.input([-1, -1])), v must match them.
	HostBuilder h(program);
	h.RegionBegin("WaveEq");
	V u_in = h.Input("u", {-1, -1}, TFType_Float);
	std::vector<V> shape = h.Shape(u_in);
	V v_in = h.Input("v", {shape[0], shape[1]}, TFType_Float);
	V v_out = h.Allocate("v_new", {shape[0], shape[1]}, TFType_Float);
	V u_out = h.Allocate("u_new", {shape[0], shape[1]}, TFType_Float);
	h.Dispatch(kernel, {v_out, u_out}, {u_in, v_in}, {shape[0], shape[1]}, {shape[0], shape[1]});
	h.RegionEnd("WaveEq");
	h.Output(v_out);
	h.Output(u_out);
	h.Finish();
}

static ProgramRegistrar reg_wave_eq("wave_eq", BuildWaveEq);

}  // namespace tfhost
