// benchmark config 4: one symplectic-Euler step of an all-pairs gravitational N-body system, written the way
// the reference's loop-form example is (examples/Simulation/n-body-benchmark.py:36-65) with masses and
// Plummer softening added:
//
//   def NBody():
//       X = tf.input([-1, 3], tf.float32); N = X.shape[0]
//       V = tf.input([N, 3], tf.float32); M = tf.input([N], tf.float32)
//       i, = tf.indices([N])
//       ax, ay, az = tf.const(0.0), tf.const(0.0), tf.const(0.0)
//       x0, y0, z0 = X[i, 0], X[i, 1], X[i, 2]
//       with tf.loop(N) as j:
//           dx, dy, dz = X[j, 0] - x0, X[j, 1] - y0, X[j, 2] - z0
//           d2 = dx*dx + dy*dy + dz*dz + eps*eps
//           s = M[j] / (d2 * tf.sqrt(d2))
//           ax.val += s*dx; ay.val += s*dy; az.val += s*dz
//       Vnew = V + a*dt; Xnew = X + Vnew*dt
//       return Xnew, Vnew
//
// One fused kernel of shape [N]; user loads index in Clamp mode.
#include "registry.h"

namespace tfhost {

static void BuildNBody(Program* program, const std::vector<int64_t>& params) {
	(void)params;
	KernelBuilder b(program, 1);
	V x_new = b.Buffer("x_new", false);
	V v_new = b.Buffer("v_new", false);
	V X = b.Buffer("X", true);
	V Vb = b.Buffer("V", true);
	V Mb = b.Buffer("M", true);
	V dtb = b.Buffer("dt", true);
	V epsb = b.Buffer("eps", true);
	V N = b.Var("N", TFType_Int);
	V i = b.ThreadIndices({N})[0];
	// dt and eps are scalar tensors: a kernel reads such an input from its buffer (a load at address 0), the host
	// never sees the value
	V dt = b.Named(b.Load(dtb, b.Const(0), TFType_Float), "dt");
	V eps = b.Named(b.Load(epsb, b.Const(0), TFType_Float), "eps");
	V eps2 = b.Named(eps * eps, "eps2");

	auto component = [&](V row, int c) {  // X[row, c] with Clamp indexing
		V r = b.Clamp(row, b.Const(0), N - b.Const(1));
		V cc = b.Clamp(b.Const(c), b.Const(0), b.Const(2));
		return b.Load(X, r * b.Const(3) + cc, TFType_Float);
	};
	V ax = b.Accumulator("ax", TFType_Float, FloatBits(0.0f));
	V ay = b.Accumulator("ay", TFType_Float, FloatBits(0.0f));
	V az = b.Accumulator("az", TFType_Float, FloatBits(0.0f));
	V x0 = b.Named(component(i, 0), "x0");
	V y0 = b.Named(component(i, 1), "y0");
	V z0 = b.Named(component(i, 2), "z0");
	b.Loop(b.Const(0), N, b.Const(1), [&](V j) {
		V x = b.Named(component(j, 0), "x");
		V y = b.Named(component(j, 1), "y");
		V z = b.Named(component(j, 2), "z");
		V m = b.Named(b.Load(Mb, b.Clamp(j, b.Const(0), N - b.Const(1)), TFType_Float), "m");
		V dx = b.Named(x - x0, "dx");
		V dy = b.Named(y - y0, "dy");
		V dz = b.Named(z - z0, "dz");
		V d2 = b.Named(dx * dx + dy * dy + dz * dz + eps2, "d2");
		V s = b.Named(m / (d2 * Fn("sqrt", d2)), "s");
		b.Set(ax, ax + s * dx);
		b.Set(ay, ay + s * dy);
		b.Set(az, az + s * dz);
	});
	V a[3] = {ax, ay, az};
	V p0[3] = {x0, y0, z0};
	for (int c = 0; c < 3; c++) {
		V addr = i * b.Const(3) + b.Const(c);
		V vel = b.Load(Vb, addr, TFType_Float) + a[c] * dt;
		b.Store(v_new, addr, vel);
		b.Store(x_new, i * b.Const(3) + b.Const(c), p0[c] + vel * dt);
	}
	Kernel* kernel = b.Finish();

	// Host part: X, V, M, dt, eps (the two scalars as one-element tensors that the kernel itself reads).
	HostBuilder h(program);
	h.RegionBegin("NBody");
	V X_in = h.Input("X", {-1, 3}, TFType_Float);
	V n = h.Shape(X_in)[0];
	V V_in = h.Input("V", {n, 3}, TFType_Float);
	V M_in = h.Input("M", {n}, TFType_Float);
	V dt_in = h.Input("dt", {1}, TFType_Float);
	V eps_in = h.Input("eps", {1}, TFType_Float);
	V x_out = h.Allocate("x_new", {n, 3}, TFType_Float);
	V v_out = h.Allocate("v_new", {n, 3}, TFType_Float);
	h.Dispatch(kernel, {x_out, v_out}, {X_in, V_in, M_in, dt_in, eps_in}, {n}, {n});
	h.RegionEnd("NBody");
	h.Output(x_out);
	h.Output(v_out);
	h.Finish();
}

static ProgramRegistrar reg_nbody("nbody", BuildNBody);

}  // namespace tfhost
