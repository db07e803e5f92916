// Scalar operations of the op table evaluated on the host, for host-side nodes of a program (shape arithmetic,
// loop bounds, values read back from tensors). Semantics are those of the C++ the reference generates for the same
// node (Backend/CodeGen/Generators.cpp:474-531: operators in the operand type, casts as C casts, reinterpretation
// as a bit copy) with the helper functions of its prelude (Backend/CodeGen/Langs/CPP.cpp:31-271).
#include <cmath>
#include <cstdint>
#include <cstring>
#include <limits>
#include <stdexcept>
#include <string>
#include <type_traits>
#include <unordered_map>

#include "host_program.h"

namespace tfhost {

namespace {

template <typename T>
inline T From(uint32_t w) {
	T v;
	std::memcpy(&v, &w, 4);
	return v;
}
template <>
inline bool From<bool>(uint32_t w) {
	return w != 0;
}
template <typename T>
inline uint32_t To(T v) {
	uint32_t w;
	std::memcpy(&w, &v, 4);
	return w;
}
template <>
inline uint32_t To<bool>(bool v) {
	return v ? 1u : 0u;
}

inline uint32_t Pcg(uint32_t v) {
	uint32_t state = v * 747796405u + 2891336453u;
	uint32_t word = ((state >> ((state >> 28u) + 4u)) ^ state) * 277803737u;
	return (word >> 22u) ^ word;
}
inline uint32_t ReverseBits(uint32_t x) {
	x = ((x >> 1) & 0x55555555u) | ((x & 0x55555555u) << 1);
	x = ((x >> 2) & 0x33333333u) | ((x & 0x33333333u) << 2);
	x = ((x >> 4) & 0x0F0F0F0Fu) | ((x & 0x0F0F0F0Fu) << 4);
	x = ((x >> 8) & 0x00FF00FFu) | ((x & 0x00FF00FFu) << 8);
	return (x >> 16) | (x << 16);
}

// Integer division and remainder by zero would trap the host; the generated C++ has the same hazard, a GPU
// kernel does not. The host evaluator reports it as an error of the program instead.
template <typename T>
inline T CheckedDiv(T a, T b) {
	if (b == 0) throw std::runtime_error("Host program: integer division by zero");
	if (std::is_signed<T>::value && a == std::numeric_limits<T>::min() && b == (T)-1) return a;
	return a / b;
}
template <typename T>
inline T CheckedMod(T a, T b) {
	if (b == 0) throw std::runtime_error("Host program: integer remainder by zero");
	if (std::is_signed<T>::value && b == (T)-1) return 0;
	return a % b;
}

#define BIN(T, EXPR) [](uint32_t wa, uint32_t wb, uint32_t) -> uint32_t { T a = From<T>(wa), b = From<T>(wb); (void)a; (void)b; return To(EXPR); }
#define UN(T, EXPR) [](uint32_t wa, uint32_t, uint32_t) -> uint32_t { T a = From<T>(wa); (void)a; return To(EXPR); }
#define TER(T, EXPR) [](uint32_t wa, uint32_t wb, uint32_t wc) -> uint32_t { T a = From<T>(wa), b = From<T>(wb), c = From<T>(wc); (void)a; (void)b; (void)c; return To(EXPR); }

using Table = std::unordered_map<std::string, ScalarFn>;

// key: op name + '_' + operand type letter (f, u, i, b)
Table MakeTable() {
	Table t;
#define ARITH(T, L)                          \
	t["add_" L] = BIN(T, (T)(a + b));        \
	t["sub_" L] = BIN(T, (T)(a - b));        \
	t["mul_" L] = BIN(T, (T)(a * b));        \
	t["eq_" L] = BIN(T, (bool)(a == b));     \
	t["neq_" L] = BIN(T, (bool)(a != b));    \
	t["lt_" L] = BIN(T, (bool)(a < b));      \
	t["lte_" L] = BIN(T, (bool)(a <= b));    \
	t["gt_" L] = BIN(T, (bool)(a > b));      \
	t["gte_" L] = BIN(T, (bool)(a >= b));    \
	t["min_" L] = BIN(T, (T)(a < b ? a : b)); \
	t["max_" L] = BIN(T, (T)(a > b ? a : b)); \
	t["clamp_" L] = TER(T, (T)((a > b ? a : b) < c ? (a > b ? a : b) : c)); \
	t["copy_" L] = UN(T, (T)a);
	ARITH(float, "f")
	ARITH(int32_t, "i")
	ARITH(uint32_t, "u")
#undef ARITH
#define INTEGER(T, L)                                   \
	t["div_" L] = BIN(T, CheckedDiv<T>(a, b));          \
	t["mod_" L] = BIN(T, CheckedMod<T>(a, b));          \
	t["lshift_" L] = BIN(T, (T)((uint32_t)a << ((uint32_t)b & 31u))); \
	t["rshift_" L] = BIN(T, (T)(a >> ((uint32_t)b & 31u)));           \
	t["and_" L] = BIN(T, (T)(a & b));                   \
	t["or_" L] = BIN(T, (T)(a | b));                    \
	t["xor_" L] = BIN(T, (T)(a ^ b));                   \
	t["not_" L] = UN(T, (T)(~a));                       \
	t["reversebits_" L] = UN(T, (T)ReverseBits((uint32_t)a));
	INTEGER(int32_t, "i")
	INTEGER(uint32_t, "u")
#undef INTEGER
	t["neg_i"] = UN(int32_t, (int32_t)(0u - (uint32_t)a));
	t["neg_u"] = UN(uint32_t, (uint32_t)(0u - a));
	t["neg_f"] = UN(float, -a);
	t["abs_i"] = UN(int32_t, (int32_t)(a < 0 ? 0u - (uint32_t)a : (uint32_t)a));
	t["abs_u"] = UN(uint32_t, a);
	t["abs_f"] = UN(float, std::fabs(a));
	t["sign_i"] = UN(int32_t, (int32_t)(a < 0 ? -1 : 1));
	t["sign_f"] = UN(float, a < 0.0f ? -1.0f : 1.0f);
	t["pcg_u"] = UN(uint32_t, Pcg(a));
	t["pcgf_u"] = UN(uint32_t, (float)Pcg(a) / (float)0xffffffffu);

	// booleans: stored as 0 / 1 words
	t["and_b"] = BIN(bool, (bool)(a && b));
	t["or_b"] = BIN(bool, (bool)(a || b));
	t["xor_b"] = BIN(bool, (bool)(a != b));
	t["eq_b"] = BIN(bool, (bool)(a == b));
	t["neq_b"] = BIN(bool, (bool)(a != b));
	t["notb_b"] = UN(bool, (bool)!a);
	t["not_b"] = UN(bool, (bool)!a);
	t["copy_b"] = UN(bool, (bool)a);

	// float functions
	t["div_f"] = BIN(float, a / b);
	t["mod_f"] = BIN(float, std::fmod(a, b));
	t["modf_f"] = BIN(float, std::fmod(a, b));
	t["pow_f"] = BIN(float, std::pow(a, b));
	t["atan2_f"] = BIN(float, std::atan2(a, b));
	t["step_f"] = BIN(float, b >= a ? 1.0f : 0.0f);
	t["lerp_f"] = TER(float, a + (b - a) * c);
	t["fma_f"] = TER(float, std::fma(a, b, c));
	t["smoothstep_f"] = [](uint32_t wa, uint32_t wb, uint32_t wc) -> uint32_t {
		float a = From<float>(wa), b = From<float>(wb), x = (From<float>(wc) - a) / (b - a);
		x = x < 0.0f ? 0.0f : x > 1.0f ? 1.0f : x;
		return To(x * x * (3.0f - 2.0f * x));
	};
#define FLOATFN(NAME, EXPR) t[NAME "_f"] = UN(float, (float)(EXPR));
	FLOATFN("ceil", std::ceil(a))
	FLOATFN("floor", std::floor(a))
	FLOATFN("round", std::round(a))
	FLOATFN("frac", a - std::floor(a))
	FLOATFN("exp", std::exp(a))
	FLOATFN("exp2", std::exp2(a))
	FLOATFN("log", std::log(a))
	FLOATFN("log2", std::log2(a))
	FLOATFN("sqrt", std::sqrt(a))
	FLOATFN("rsqrt", 1.0f / std::sqrt(a))
	FLOATFN("rcp", 1.0f / a)
	FLOATFN("sin", std::sin(a))
	FLOATFN("cos", std::cos(a))
	FLOATFN("tan", std::tan(a))
	FLOATFN("asin", std::asin(a))
	FLOATFN("acos", std::acos(a))
	FLOATFN("atan", std::atan(a))
	FLOATFN("sinh", std::sinh(a))
	FLOATFN("cosh", std::cosh(a))
	FLOATFN("tanh", std::tanh(a))
#undef FLOATFN

	// casts ((T)(x), Generators.h:164-167): key = target name + '_' + source type
#define CAST(NAME, T)                                \
	t[NAME "_f"] = UN(float, (T)a);                  \
	t[NAME "_i"] = UN(int32_t, (T)a);                \
	t[NAME "_u"] = UN(uint32_t, (T)a);               \
	t[NAME "_b"] = UN(bool, (T)a);
	CAST("float", float)
	CAST("int", int32_t)
	CAST("uint", uint32_t)
	CAST("bool", bool)
#undef CAST
	// float -> unsigned of a negative value is undefined in C++; the GPU saturates to 0, so does the host
	t["uint_f"] = UN(float, (uint32_t)(a <= 0.0f ? 0u : a >= 4294967296.0f ? 0xffffffffu : (uint32_t)a));
	t["int_f"] = UN(float, (int32_t)(a != a ? 0 : a <= -2147483648.0f ? INT32_MIN : a >= 2147483648.0f ? INT32_MAX : (int32_t)a));

	// reinterpretation: the word itself, except to / from bool (CPP.cpp: asuint(bool) etc. convert)
	for (const char* src : {"f", "i", "u"}) {
		for (const char* dst : {"asfloat", "asint", "asuint"}) t[std::string(dst) + "_" + src] = [](uint32_t a, uint32_t, uint32_t) -> uint32_t { return a; };
		t[std::string("asbool_") + src] = [](uint32_t a, uint32_t, uint32_t) -> uint32_t { return a != 0 ? 1u : 0u; };
	}
	for (const char* dst : {"asint", "asuint", "asbool"}) t[std::string(dst) + "_b"] = [](uint32_t a, uint32_t, uint32_t) -> uint32_t { return a != 0 ? 1u : 0u; };

	// cond ? a : b on words of any type
	for (const char* l : {"f", "i", "u", "b"}) t[std::string("ternary_") + l] = [](uint32_t c, uint32_t a, uint32_t b) -> uint32_t { return c != 0 ? a : b; };
	return t;
}

char TypeLetter(TFType t) {
	switch (t) {
		case TFType_Float: return 'f';
		case TFType_Int: return 'i';
		case TFType_Uint: return 'u';
		case TFType_Bool: return 'b';
		default: return '?';
	}
}

}  // namespace

ScalarFn FindScalarFn(const std::string& op, TFType operand, TFType result) {
	static const Table table = MakeTable();
	// The ternary's first input is the condition; its evaluator does not depend on the value type.
	const TFType key_type = op == "ternary" ? result : operand;
	auto it = table.find(op + "_" + TypeLetter(key_type));
	return it == table.end() ? nullptr : it->second;
}

}  // namespace tfhost
