// TEST INFRASTRUCTURE -- not part of the product. Only tests/, __graft_entry__.smoke() and the
// cpu_baseline leg of bench.py may load anything under oracle/.
//
// One kernel in the form the reference's C++ backend gives an element-wise program that uses every
// scalar operation of the op table once (TensorFrost/Compiler/Operations.cpp:84-178): operators are
// written infix (Generators.cpp:474-488), functions by name against the prelude and <cmath>
// (Generators.cpp:489-498; CPP.cpp:31-136), casts as `((T)(x))` (Generators.h:164-167),
// reinterpretations as `asT(x)` (:169-171), the ternary as `c ? a : b` (Generators.cpp:499-505);
// the wrapper is the omp-parallel group loop with serial threads of CPP.cpp:720-779. Signed +, -, * and
// negation are evaluated on the unsigned representation: the same two's-complement result the generated
// `a + b` gives on every target, without leaning on signed-overflow behaviour the C++ standard leaves open.
//
// Pins: the integer and bit rows are checked bit-for-bit against NumPy integer arithmetic, the float rows
// against NumPy float64 evaluations of the textbook definitions (tests/test_oracle_ops.py). rsqrt, rcp,
// frac and step have no definition in the C++ prelude (a program using them does not compile on the
// reference's CPU backend); they follow the GLSL/HLSL built-ins the reference's other backends map them to
// (inversesqrt, 1/x, x - floor(x), x >= edge), and the same test pins them to those closed forms.
#include "prelude.h"

using namespace tfo;

namespace {
inline float rsqrt(float x) { return 1.0f / std::sqrt(x); }
inline float rcp(float x) { return 1.0f / x; }
inline float frac(float x) { return x - std::floor(x); }
inline float step(float edge, float x) { return x >= edge ? 1.0f : 0.0f; }
inline int reversebits(int x) { return (int)tfo::reversebits((uint)x); }
inline uint min(uint a, uint b) { return a < b ? a : b; }
inline uint max(uint a, uint b) { return a > b ? a : b; }
}  // namespace

extern "C" {

int oracle_ops_float_rows() { return 42; }
int oracle_ops_int_rows() { return 28; }
int oracle_ops_uint_rows() { return 16; }

// F[42, n], I[28, n], U[16, n]; row order as in the `ops` program of the host library.
void oracle_ops(const float* x_mem, const float* y_mem, const int* a_mem, const int* b_mem, const uint* u_mem, const uint* w_mem, int n, float* F,
                int* I, uint* U) {
	const int work_group_count = (n + 255) / 256;
#pragma omp parallel for
	for (int block_id = 0; block_id < work_group_count; block_id++)
		for (int block_thread_id0 = 0; block_thread_id0 < 256; block_thread_id0++) {
			int i = block_id * 256 + block_thread_id0;
			if (!(i < n)) continue;
			float x = x_mem[i], y = y_mem[i];
			int a = a_mem[i], b = b_mem[i];
			uint u = u_mem[i], w = w_mem[i];
			float ax = std::abs(x);
			float unit = clamp(x, -1.0f, 1.0f);
			int shift = b & 7;
			uint shiftu = w & 7u;
			int b_nonzero = (b == 0) ? 1 : b;
			uint w_nonzero = (w == 0u) ? 1u : w;
			float y_nonzero = (y == 0.0f) ? 1.0f : y;
			int k = 0;
			auto f = [&](float v) { F[(size_t)(k++) * n + i] = v; };
			f(x + y); f(x - y); f(x * y); f(x / y_nonzero); f(-x); f(min(x, y)); f(max(x, y)); f(std::abs(x)); f(sign(x));
			f(std::ceil(x)); f(std::floor(x)); f(std::round(x)); f(frac(x)); f(std::exp(x)); f(std::exp2(x)); f(std::log(ax + 0.5f));
			f(std::log2(ax + 0.5f)); f(std::sqrt(ax)); f(rsqrt(ax + 0.5f)); f(rcp(y_nonzero)); f(std::sin(x)); f(std::cos(x));
			f(std::tan(unit)); f(std::asin(unit)); f(std::acos(unit)); f(std::atan(x)); f(std::sinh(x)); f(std::cosh(x)); f(std::tanh(x));
			f(std::pow(ax + 0.5f, y)); f(std::atan2(x, y)); f(std::fmod(x, y_nonzero)); f(step(y, x)); f(clamp(x, -0.5f, 0.75f));
			f(lerp(x, y, 0.25f)); f(std::fma(x, y, 1.5f)); f(smoothstep(-1.0f, 2.0f, x)); f(std::fmod(x, y_nonzero)); f(x > y ? x : y);
			f(((float)(a))); f(((float)(u))); f(pcgf(u));
			k = 0;
			auto g = [&](int v) { I[(size_t)(k++) * n + i] = v; };
			g((int)((uint)a + (uint)b)); g((int)((uint)a - (uint)b)); g((int)((uint)a * (uint)b)); g(a / b_nonzero); g(a % b_nonzero);
			g((int)((uint)a << shift)); g(a >> shift); g(a & b); g(a | b); g(a ^ b); g(~a); g((int)(0u - (uint)a)); g(min(a, b)); g(max(a, b));
			g(a < 0 ? (int)(0u - (uint)a) : a); g(sign(a)); g(clamp(a, -100, 1000)); g(a < b ? 1 : 0); g(a <= b ? 1 : 0); g(a > b ? 1 : 0);
			g(a >= b ? 1 : 0); g(a == b ? 1 : 0); g(a != b ? 1 : 0); g(((int)(x * 100.0f))); g(((a < b) && (x < y)) ? 1 : 0);
			g(((a < b) || (x < y)) ? 1 : 0); g(!(a < b) ? 1 : 0); g(reversebits(a));
			k = 0;
			auto h = [&](uint v) { U[(size_t)(k++) * n + i] = v; };
			h(u + w); h(u * w); h(u / w_nonzero); h(u % w_nonzero); h(u << shiftu); h(u >> shiftu); h(u & w); h(u | w); h(u ^ w); h(~u); h(pcg(u));
			h(tfo::reversebits(u)); h(asuint(x)); h(min(u, w)); h(max(u, w)); h(((uint)(ax * 1000.0f)));
		}
}

}  // extern "C"
