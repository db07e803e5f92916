#include "hip_generator.h"

#include <cmath>
#include <cstdio>
#include <set>
#include <sstream>
#include <unordered_map>
#include <unordered_set>

namespace tfhost {

static const char* TypeName(TFType t) {
	switch (t) {
		case TFType_Float: return "float";
		case TFType_Uint: return "uint";
		case TFType_Int: return "int";
		case TFType_Bool: return "bool";
		default: return "void";
	}
}

std::string FormatFloat(double value) {
	float f = (float)value;
	if (!std::isfinite(f)) {
		char buf[48];
		snprintf(buf, sizeof(buf), "__uint_as_float(0x%08xu)", FloatBits(f));
		return buf;
	}
	// Nine significant digits reproduce any float exactly.
	char buf[48];
	snprintf(buf, sizeof(buf), "%.9g", (double)f);
	std::string s(buf);
	if (s.find('.') == std::string::npos && s.find('e') == std::string::npos) s += ".0";
	if (s.find('.') == std::string::npos) {  // "1e+10" -> "1.0e+10"
		size_t e = s.find('e');
		s = s.substr(0, e) + ".0" + s.substr(e);
	}
	return s + "f";
}

std::string GetHIPHeader() {
	return R"(typedef unsigned int uint;

// ---- helpers of generated kernels (semantics of the C++/OpenMP backend's prelude) ----
__device__ __forceinline__ int tf_min(int a, int b) { return a < b ? a : b; }
__device__ __forceinline__ int tf_max(int a, int b) { return a > b ? a : b; }
__device__ __forceinline__ uint tf_min(uint a, uint b) { return a < b ? a : b; }
__device__ __forceinline__ uint tf_max(uint a, uint b) { return a > b ? a : b; }
__device__ __forceinline__ float tf_min(float a, float b) { return a < b ? a : b; }
__device__ __forceinline__ float tf_max(float a, float b) { return a > b ? a : b; }
__device__ __forceinline__ float asfloat(uint x) { return __uint_as_float(x); }
__device__ __forceinline__ float asfloat(int x) { return __int_as_float(x); }
__device__ __forceinline__ float asfloat(float x) { return x; }
__device__ __forceinline__ uint asuint(float x) { return __float_as_uint(x); }
__device__ __forceinline__ uint asuint(int x) { return (uint)x; }
__device__ __forceinline__ uint asuint(uint x) { return x; }
__device__ __forceinline__ uint asuint(bool x) { return x ? 1u : 0u; }
__device__ __forceinline__ int asint(uint x) { return (int)x; }
__device__ __forceinline__ int asint(float x) { return __float_as_int(x); }
__device__ __forceinline__ int asint(int x) { return x; }
__device__ __forceinline__ int asint(bool x) { return x ? 1 : 0; }
__device__ __forceinline__ bool asbool(uint x) { return x != 0u; }
__device__ __forceinline__ bool asbool(int x) { return x != 0; }
__device__ __forceinline__ bool asbool(bool x) { return x; }
__device__ __forceinline__ int tf_clamp(int x, int a, int b) { return tf_min(tf_max(x, a), b); }
__device__ __forceinline__ uint tf_clamp(uint x, uint a, uint b) { return tf_min(tf_max(x, a), b); }
__device__ __forceinline__ float tf_clamp(float x, float a, float b) { return tf_min(tf_max(x, a), b); }
__device__ __forceinline__ float tf_lerp(float a, float b, float t) { return a + (b - a) * t; }
__device__ __forceinline__ float tf_smoothstep(float a, float b, float t) {
  t = tf_clamp((t - a) / (b - a), 0.0f, 1.0f);
  return t * t * (3.0f - 2.0f * t);
}
__device__ __forceinline__ float tf_sign(float x) { return x < 0.0f ? -1.0f : 1.0f; }
__device__ __forceinline__ int tf_sign(int x) { return x < 0 ? -1 : 1; }
__device__ __forceinline__ float tf_abs(float x) { return fabsf(x); }
__device__ __forceinline__ int tf_abs(int x) { return x < 0 ? -x : x; }
__device__ __forceinline__ uint tf_abs(uint x) { return x; }
__device__ __forceinline__ uint reversebits(uint x) { return __brev(x); }
__device__ __forceinline__ int reversebits(int x) { return (int)__brev((uint)x); }
__device__ __forceinline__ uint pcg(uint v) {
  uint state = v * 747796405u + 2891336453u;
  uint word = ((state >> ((state >> 28u) + 4u)) ^ state) * 277803737u;
  return (word >> 22u) ^ word;
}
__device__ __forceinline__ float pcgf(uint v) { return (float)pcg(v) / (float)0xffffffffu; }
// Operations the C++ prelude does not define (those programs cannot run on the CPU backend).
__device__ __forceinline__ float tf_rsqrt(float x) { return rsqrtf(x); }
__device__ __forceinline__ float tf_rcp(float x) { return 1.0f / x; }
__device__ __forceinline__ float tf_frac(float x) { return x - floorf(x); }
__device__ __forceinline__ float tf_step(float edge, float x) { return x >= edge ? 1.0f : 0.0f; }
__device__ __forceinline__ void group_barrier() { __syncthreads(); }

// ---- atomics on word buffers ----
__device__ __forceinline__ void InterlockedAdd(int* m, int a, int v) { atomicAdd(m + a, v); }
__device__ __forceinline__ void InterlockedAdd(uint* m, int a, uint v) { atomicAdd(m + a, v); }
__device__ __forceinline__ void InterlockedAdd(float* m, int a, float v) { atomicAdd(m + a, v); }
__device__ __forceinline__ int InterlockedAdd_Prev(int* m, int a, int v) { return atomicAdd(m + a, v); }
__device__ __forceinline__ uint InterlockedAdd_Prev(uint* m, int a, uint v) { return atomicAdd(m + a, v); }
__device__ __forceinline__ float InterlockedAdd_Prev(float* m, int a, float v) { return atomicAdd(m + a, v); }
__device__ __forceinline__ void InterlockedMin(int* m, int a, int v) { atomicMin(m + a, v); }
__device__ __forceinline__ void InterlockedMin(uint* m, int a, uint v) { atomicMin(m + a, v); }
__device__ __forceinline__ void InterlockedMax(int* m, int a, int v) { atomicMax(m + a, v); }
__device__ __forceinline__ void InterlockedMax(uint* m, int a, uint v) { atomicMax(m + a, v); }
__device__ __forceinline__ void InterlockedMin(float* m, int a, float v) {
  uint* p = (uint*)(m + a);
  uint old = *p;
  while (true) {
    float cur = __uint_as_float(old);
    float goal = tf_min(cur, v);
    if (__float_as_uint(goal) == old) break;
    uint seen = atomicCAS(p, old, __float_as_uint(goal));
    if (seen == old) break;
    old = seen;
  }
}
__device__ __forceinline__ void InterlockedMax(float* m, int a, float v) {
  uint* p = (uint*)(m + a);
  uint old = *p;
  while (true) {
    float cur = __uint_as_float(old);
    float goal = tf_max(cur, v);
    if (__float_as_uint(goal) == old) break;
    uint seen = atomicCAS(p, old, __float_as_uint(goal));
    if (seen == old) break;
    old = seen;
  }
}
__device__ __forceinline__ void InterlockedAnd(int* m, int a, int v) { atomicAnd(m + a, v); }
__device__ __forceinline__ void InterlockedAnd(uint* m, int a, uint v) { atomicAnd(m + a, v); }
__device__ __forceinline__ void InterlockedOr(int* m, int a, int v) { atomicOr(m + a, v); }
__device__ __forceinline__ void InterlockedOr(uint* m, int a, uint v) { atomicOr(m + a, v); }
__device__ __forceinline__ void InterlockedXor(int* m, int a, int v) { atomicXor(m + a, v); }
__device__ __forceinline__ void InterlockedXor(uint* m, int a, uint v) { atomicXor(m + a, v); }

// ---- cross-lane finish of a wave-cooperative reduction (64 lanes) ----
#define TF_WAVE_REDUCE(T, NAME, EXPR)                                  \
  __device__ __forceinline__ T NAME(T a) {                             \
    _Pragma("unroll") for (int off = 32; off >= 1; off >>= 1) {        \
      T b = __shfl_xor(a, off, 64);                                    \
      a = (EXPR);                                                      \
    }                                                                  \
    return a;                                                          \
  }
TF_WAVE_REDUCE(float, tf_wave_add, a + b)
TF_WAVE_REDUCE(int, tf_wave_add, a + b)
TF_WAVE_REDUCE(uint, tf_wave_add, a + b)
TF_WAVE_REDUCE(float, tf_wave_mul, a * b)
TF_WAVE_REDUCE(int, tf_wave_mul, a * b)
TF_WAVE_REDUCE(uint, tf_wave_mul, a * b)
TF_WAVE_REDUCE(float, tf_wave_max, tf_max(a, b))
TF_WAVE_REDUCE(int, tf_wave_max, tf_max(a, b))
TF_WAVE_REDUCE(uint, tf_wave_max, tf_max(a, b))
TF_WAVE_REDUCE(float, tf_wave_min, tf_min(a, b))
TF_WAVE_REDUCE(int, tf_wave_min, tf_min(a, b))
TF_WAVE_REDUCE(uint, tf_wave_min, tf_min(a, b))
TF_WAVE_REDUCE(int, tf_wave_and, a & b)
TF_WAVE_REDUCE(uint, tf_wave_and, a & b)
TF_WAVE_REDUCE(int, tf_wave_or, a | b)
TF_WAVE_REDUCE(uint, tf_wave_or, a | b)
__device__ __forceinline__ bool tf_wave_and(bool a) { return __all(a); }
__device__ __forceinline__ bool tf_wave_or(bool a) { return __any(a); }

)";
}

namespace {

struct Line {
	Node* node;
	std::string text;
	int indent;
};

// Names a generated kernel may not use for its own values (C++/HIP keywords and prelude names).
const std::unordered_set<std::string>& ForbiddenNames() {
	static const std::unordered_set<std::string> s = {
	    "unsigned", "input", "output", "max", "min", "exp", "sin", "cos", "if", "else", "while", "for", "switch", "case", "default", "break",
	    "this", "true", "false", "null", "new", "delete", "return", "continue", "goto", "try", "catch", "throw", "const", "static", "extern",
	    "inline", "virtual", "override", "final", "public", "protected", "private", "sample", "asm", "class", "union", "enum", "typedef",
	    "template", "typename", "using", "namespace", "friend", "sizeof", "alignof", "typeid", "auto", "register", "explicit", "mutable",
	    "constexpr", "decltype", "noexcept", "nullptr", "alignas", "and", "or", "not", "xor", "sign", "bool", "char", "int", "uint", "float",
	    "var", "pcg", "pcgf", "abs", "pow", "log", "tan", "floor", "ceil", "round", "sqrt", "clamp", "lerp", "fma", "step", "frac",
	};
	return s;
}

const std::unordered_map<std::string, std::string>& NameMap() {
	static const std::unordered_map<std::string, std::string> m = {
	    {"min", "tf_min"}, {"max", "tf_max"}, {"clamp", "tf_clamp"}, {"lerp", "tf_lerp"}, {"smoothstep", "tf_smoothstep"},
	    {"sign", "tf_sign"}, {"abs", "tf_abs"}, {"rsqrt", "tf_rsqrt"}, {"rcp", "tf_rcp"}, {"frac", "tf_frac"}, {"step", "tf_step"},
	    {"modf", "fmodf"}, {"sqrt", "sqrtf"}, {"exp", "expf"}, {"exp2", "exp2f"}, {"log", "logf"}, {"log2", "log2f"},
	    {"sin", "sinf"}, {"cos", "cosf"}, {"tan", "tanf"}, {"asin", "asinf"}, {"acos", "acosf"}, {"atan", "atanf"},
	    {"sinh", "sinhf"}, {"cosh", "coshf"}, {"tanh", "tanhf"}, {"pow", "powf"}, {"atan2", "atan2f"}, {"ceil", "ceilf"},
	    {"floor", "floorf"}, {"round", "roundf"}, {"fma", "fmaf"},
	};
	return m;
}

bool IsLocalArray(const Node* n) { return std::string(n->op->name) == "group_memory" || std::string(n->op->name) == "local_memory"; }

// ---- reduction idiom ------------------------------------------------------------------------------

struct ReductionLoop {
	Node* accumulator = nullptr;
	Node* loop = nullptr;
	std::string combine;  // tf_wave_add ...
};

bool DependsOn(const Node* n, const Node* target, int depth = 0) {
	if (!n || depth > 64) return false;
	if (n == target) return true;
	for (Node* in : n->inputs)
		if (DependsOn(in, target, depth + 1)) return true;
	if (DependsOn(n->index, target, depth + 1)) return true;
	return false;
}

// address == something_without_loop_var + loop_var  (unit stride in the loop variable)
bool IsUnitStride(const Node* addr, const Node* loop_var) {
	if (!addr) return false;
	if (addr == loop_var) return true;
	if (std::string(addr->op->name) == "add" && addr->inputs.size() == 2) {
		const Node* a = addr->inputs[0];
		const Node* b = addr->inputs[1];
		if (IsUnitStride(a, loop_var) && !DependsOn(b, loop_var)) return true;
		if (IsUnitStride(b, loop_var) && !DependsOn(a, loop_var)) return true;
	}
	return false;
}

// Matches `acc = init; loop(b, e, s) { ...pure...; acc = op(acc, value); }` as the reference lowers dim_sum /
// dim_max / dim_min / dim_prod / dim_any / dim_all (Implementations.cpp:243-303) and checks that a wave
// can run the loop cooperatively: every load in the body is unit-stride in the loop variable, nothing in
// the body writes memory, the accumulator is touched only by its own update.
bool MatchReductionLoop(Node* loop, ReductionLoop& out) {
	if (std::string(loop->op->name) != "loop" || loop->children.empty()) return false;
	Node* last = loop->children.back();
	if (std::string(last->op->name) != "set" || !last->memory || !last->memory->modified) return false;
	Node* acc = last->memory;
	if (std::string(acc->op->name) != "const") return false;
	static const std::set<std::string> idioms = {"sum", "max", "min", "prod", "any", "all"};
	if (!idioms.count(acc->debug_name)) return false;
	Node* update = last->inputs[0];
	const std::string opname = update->op->name;
	if (update->inputs.size() != 2) return false;
	Node* value = nullptr;
	if (update->inputs[0] == acc)
		value = update->inputs[1];
	else if (update->inputs[1] == acc)
		value = update->inputs[0];
	else
		return false;
	if (DependsOn(value, acc)) return false;
	std::string combine;
	if (opname == "add") combine = "tf_wave_add";
	else if (opname == "mul") combine = "tf_wave_mul";
	else if (opname == "max") combine = "tf_wave_max";
	else if (opname == "min") combine = "tf_wave_min";
	else if (opname == "and") combine = "tf_wave_and";
	else if (opname == "or") combine = "tf_wave_or";
	else return false;
	// step must be the constant 1 and the trip count at least one wave when it is a constant
	Node* step = loop->inputs[2];
	if (std::string(step->op->name) != "const" || (int)step->data != 1) return false;
	Node* begin = loop->inputs[0];
	Node* end = loop->inputs[1];
	if (std::string(begin->op->name) == "const" && std::string(end->op->name) == "const" && (int)end->data - (int)begin->data < 64) return false;
	bool has_load = false;
	for (Node* c : loop->children) {
		const std::string n = c->op->name;
		if (c == last) continue;
		if (n == "store" || n == "set" || n == "loop" || n == "if" || n == "break" || n == "continue" || n == "discard" || n == "group_barrier") return false;
		if (c->op->cls == OpClass::Memory && n != "load") return false;  // atomics
		if (n == "load") {
			if (c->local_memory_op) return false;
			// Loads that do not depend on the loop variable are broadcasts (fine); the others must be unit-stride.
			if (DependsOn(c->index, loop)) {
				if (!IsUnitStride(c->index, loop)) return false;
				has_load = true;
			}
		}
		if (c != update && DependsOn(c, acc)) return false;
	}
	if (!has_load) return false;
	out.accumulator = acc;
	out.loop = loop;
	out.combine = combine;
	return true;
}

class HIPGenerator {
 public:
	explicit HIPGenerator(Kernel* kernel) : kernel_(kernel) {
		for (auto& v : kernel->variables) variables_.insert(v.node);
	}

	// wave_cooperative: reduction loops (already matched) are strided over the 64 lanes of a wave.
	void Generate(const std::vector<ReductionLoop>& reductions) {
		for (auto& r : reductions) reduction_of_loop_[r.loop] = r;
		cooperative_ = !reductions.empty();
		for (Node* bufn : kernel_->MemoryBindings()) Rename(bufn);
		for (auto& v : kernel_->variables) v.node->var_name = v.name;
		Walk(kernel_->root, 0, false);
	}

	std::string Assemble(const std::string& base_indent) const {
		std::string code;
		for (auto& l : lines_) {
			if (removed_.count(l.node)) continue;
			code += base_indent;
			for (int i = 0; i < l.indent; i++) code += "  ";
			code += l.text;
			code += "\n";
		}
		return code;
	}

 private:
	Kernel* kernel_;
	std::vector<Line> lines_;
	std::unordered_set<Node*> variables_;
	std::unordered_map<Node*, std::string> expression_;
	std::unordered_map<Node*, bool> needs_parens_;
	std::unordered_set<Node*> removed_;
	std::unordered_map<std::string, int> name_count_;
	std::unordered_map<Node*, ReductionLoop> reduction_of_loop_;
	bool cooperative_ = false;

	static std::string MapName(const std::string& n) {
		auto it = NameMap().find(n);
		return it == NameMap().end() ? n : it->second;
	}

	// Same naming scheme as the reference's RegenerateNodeName (Generators.h:126-149).
	void Rename(Node* node) {
		std::string debug = node->debug_name;
		if (debug.empty()) debug = std::string("v") + node->op->name;
		if (ForbiddenNames().count(debug)) debug += "0";
		auto it = name_count_.find(debug);
		if (it != name_count_.end()) {
			it->second++;
			debug = debug + "_" + std::to_string(it->second);
		} else {
			name_count_[debug] = 1;
		}
		node->var_name = debug;
	}

	std::string ConstantString(const Node* n) const {
		switch (n->type) {
			case TFType_Float: {
				float f;
				std::memcpy(&f, &n->data, 4);
				return FormatFloat(f);
			}
			case TFType_Int: return std::to_string((int)n->data);
			case TFType_Uint: return std::to_string(n->data) + "u";
			case TFType_Bool: return n->data == 0 ? "false" : "true";
			default: throw std::runtime_error("Unsupported constant type");
		}
	}

	// Name under which `arg` appears inside the expression of a user: its variable name, or -- for
	// unnamed single-use pure values -- its whole expression (Generators.h:90-124).
	std::string ArgName(Node* arg, bool parenthesise) {
		if (variables_.count(arg)) return "var." + arg->var_name;
		const std::string opname = arg->op->name;
		const bool is_constant = arg->op->cls == OpClass::Constant;
		const bool is_variable = arg->op->cls == OpClass::Variable;
		std::string expr = expression_[arg];
		if (is_constant && expr.empty()) expr = ConstantString(arg);
		const bool is_static = opname == "loop" || opname == "if" || opname == "InterlockedAdd_Prev" || arg->op->cls == OpClass::Keyword;
		const bool is_memory = opname == "memory" || IsLocalArray(arg) || arg->op->cls == OpClass::Memory;
		const bool single = arg->use_count == 1 || is_constant || is_variable;
		bool reads_modified = false;
		for (Node* in : arg->inputs) reads_modified |= in->modified;
		const bool can_substitute = arg->debug_name.empty() && single && !arg->modified && expr.size() < 100 && !is_static && !is_memory &&
		                            !reads_modified && !expr.empty();
		if (can_substitute) {
			removed_.insert(arg);
			if (parenthesise && needs_parens_[arg]) return "(" + expr + ")";
			return expr;
		}
		return arg->var_name;
	}

	void Emit(Node* node, int indent, const std::string& text) { lines_.push_back({node, text, indent}); }

	void Walk(Node* scope, int indent, bool lane_guard_stores) {
		for (Node* node : scope->children) {
			const std::string opname = node->op->name;
			if (opname == "loop") {
				Rename(node);
				auto red = reduction_of_loop_.find(node);
				std::string b = ArgName(node->inputs[0], false), e = ArgName(node->inputs[1], false), s = ArgName(node->inputs[2], false);
				if (red != reduction_of_loop_.end()) {
					// Lanes of the wave stride the loop; the accumulator of each lane starts from the
					// reduction's identity, so combining the 64 partial results gives the full result.
					Emit(node, indent, "for (int " + node->var_name + " = " + b + " + _lane; " + node->var_name + " < " + e + "; " + node->var_name + " += 64)");
					Emit(nullptr, indent, "{");
					Walk(node, indent + 1, false);
					Emit(nullptr, indent, "}");
					const std::string acc = red->second.accumulator->var_name;
					Emit(nullptr, indent, acc + " = " + red->second.combine + "(" + acc + ");");
				} else {
					Emit(node, indent, "for (int " + node->var_name + " = " + b + "; " + node->var_name + " < " + e + "; " + node->var_name + " += " + s + ")");
					Emit(nullptr, indent, "{");
					Walk(node, indent + 1, lane_guard_stores);
					Emit(nullptr, indent, "}");
				}
				continue;
			}
			if (opname == "if") {
				Emit(node, indent, "if (" + ArgName(node->inputs[0], false) + ")");
				Emit(nullptr, indent, "{");
				// Inside the dispatch guard of a wave-cooperative kernel, writes happen once per logical thread.
				Walk(node, indent + 1, cooperative_ ? true : lane_guard_stores);
				Emit(nullptr, indent, "}");
				continue;
			}
			GenerateLine(node, indent, lane_guard_stores);
		}
	}

	void GenerateLine(Node* node, int indent, bool lane_guard) {
		const std::string opname = node->op->name;
		const OpClass cls = node->op->cls;
		if (opname == "memory" || opname == "variable") return;
		if (opname == "group_memory") {
			Rename(node);
			Emit(node, indent, "// " + std::string(TypeName(node->type)) + " " + node->var_name + "[" + std::to_string(node->data) + "] (declared as __shared__ above)");
			return;
		}
		Rename(node);
		const std::string name = node->var_name;
		const std::string type = TypeName(node->type);
		std::string left, expr, right = ";";
		bool parens = false;
		const std::string guard = lane_guard ? "if (_lane == 0) " : "";

		if (opname == "local_memory") {
			Emit(node, indent, type + " " + name + "[" + std::to_string(node->data) + "];");
			return;
		}
		if (cls == OpClass::Memory) {
			std::string address = node->index ? ArgName(node->index, false) : "0";
			const bool local = node->local_memory_op;
			const std::string mem_name = node->memory->var_name + (local ? "" : "_mem");
			const std::string mem_expr = mem_name + "[" + address + "]";
			const TFType mem_type = local ? node->memory->type : TFType_Uint;
			if (opname == "load") {
				left = type + " " + name + " = ";
				expr = node->type == mem_type ? mem_expr : "as" + type + "(" + mem_expr + ")";
			} else if (opname == "store") {
				Node* value = node->inputs[0];
				const std::string v = ArgName(value, false);
				left = guard;
				expr = mem_expr + " = " + (value->type == mem_type ? v : std::string("as") + TypeName(mem_type) + "(" + v + ")");
			} else {
				Node* value = node->inputs[0];
				const std::string in_type = TypeName(value->type);
				std::string call = opname + "((" + in_type + "*)" + mem_name + ", " + address + ", " + ArgName(value, false) + ")";
				if (node->type != TFType_None) {
					if (lane_guard) throw std::runtime_error("value-returning atomic after a wave-cooperative reduction is not supported");
					left = type + " " + name + " = ";
				} else {
					left = guard;
				}
				expr = call;
			}
		} else if (cls == OpClass::Set) {
			left = node->memory->var_name + " = ";
			expr = ArgName(node->inputs[0], false);
		} else {
			if (node->type != TFType_None) left = type + " " + name + " = ";
			switch (cls) {
				case OpClass::Operator: {
					std::string code = node->op->code;
					if ((code == "&" || code == "|") && node->type == TFType_Bool) code += code;
					if (code == "%" && node->type == TFType_Float) {
						expr = "fmodf(" + ArgName(node->inputs[0], false) + ", " + ArgName(node->inputs[1], false) + ")";
					} else {
						expr = ArgName(node->inputs[0], true) + " " + code + " " + ArgName(node->inputs[1], true);
						parens = true;
					}
					break;
				}
				case OpClass::UnaryOperator:
					expr = node->op->code + ArgName(node->inputs[0], true);
					parens = true;
					break;
				case OpClass::Function: {
					expr = MapName(node->op->code) + "(";
					for (size_t i = 0; i < node->inputs.size(); i++) {
						if (i) expr += ", ";
						expr += ArgName(node->inputs[i], false);
					}
					expr += ")";
					break;
				}
				case OpClass::Copy:
					expr = ArgName(node->inputs[0], false);
					parens = true;
					break;
				case OpClass::Keyword:
					// `discard` ends the logical thread; kernel bodies are emitted inside a lambda per logical thread.
					expr = opname == "discard" ? "return" : node->op->code;
					break;
				case OpClass::DimensionIndex:
					expr = node->op->code + std::to_string(node->data);
					break;
				case OpClass::Variable:
					expr = node->op->code;
					break;
				case OpClass::TypeCast:
					expr = "((" + type + ")(" + ArgName(node->inputs[0], false) + "))";
					break;
				case OpClass::TypeReinterpret:
					expr = "as" + type + "(" + ArgName(node->inputs[0], false) + ")";
					break;
				case OpClass::Constant:
					expr = ConstantString(node);
					break;
				case OpClass::TernaryOperator:
					expr = ArgName(node->inputs[0], true) + " ? " + ArgName(node->inputs[1], true) + " : " + ArgName(node->inputs[2], true);
					parens = true;
					break;
				default:
					throw std::runtime_error("Unknown operation class for " + opname);
			}
		}
		expression_[node] = expr;
		needs_parens_[node] = parens;
		Emit(node, indent, left + expr + right);
	}
};

bool UsesGroupFeatures(const Node* n) {
	const std::string name = n->op->name;
	if (name == "group_barrier" || name == "group_memory") return true;
	for (const Node* c : n->children)
		if (UsesGroupFeatures(c)) return true;
	return false;
}

void CollectLoops(Node* scope, std::vector<Node*>& loops) {
	for (Node* c : scope->children) {
		if (std::string(c->op->name) == "loop") loops.push_back(c);
		if (std::string(c->op->name) == "if") CollectLoops(c, loops);
	}
}

bool HasNestedOrUnmatched(Node* scope, const std::unordered_set<Node*>& matched, bool inside_matched) {
	for (Node* c : scope->children) {
		const std::string n = c->op->name;
		if (n == "loop") {
			if (!matched.count(c)) return true;
			if (inside_matched) return true;
		}
		if (!c->children.empty() && HasNestedOrUnmatched(c, matched, inside_matched || matched.count(c))) return true;
	}
	return false;
}

}  // namespace

void GenerateHIPKernel(Program* program, Kernel* kernel) {
	(void)program;
	if (kernel->kernel_name_.empty()) kernel->kernel_name_ = "kernel_" + std::to_string(kernel->kernel_id_);

	std::vector<int> group = kernel->group_size;
	while (group.size() < 3) group.push_back(1);
	const int group_threads = group[0] * group[1] * group[2];
	if (group_threads < 1 || group_threads > 1024) throw std::runtime_error("group size of " + kernel->kernel_name_ + " is outside 1..1024 threads");
	const bool uses_group = UsesGroupFeatures(kernel->root);

	// Reduction idiom: every loop of the kernel must be a matched reduction, none nested.
	std::vector<ReductionLoop> reductions;
	if (!uses_group) {
		std::vector<Node*> loops;
		CollectLoops(kernel->root, loops);
		std::unordered_set<Node*> matched;
		for (Node* l : loops) {
			ReductionLoop r;
			if (MatchReductionLoop(l, r)) {
				reductions.push_back(r);
				matched.insert(l);
			}
		}
		if (reductions.empty() || HasNestedOrUnmatched(kernel->root, matched, false)) reductions.clear();
	}

	HIPGenerator generator(kernel);
	generator.Generate(reductions);

	// ---- variable block -----------------------------------------------------------------------------
	kernel->var_names.clear();
	kernel->var_types.clear();
	for (auto& v : kernel->variables) {
		kernel->var_names.push_back(v.name);
		kernel->var_types.push_back(TypeName(v.type));
	}
	kernel->var_names.push_back("_kernel_block_offset");
	kernel->var_types.push_back("uint");
	kernel->var_names.push_back("_work_group_count");  // appended by the kernel manager at dispatch
	kernel->var_types.push_back("uint");

	std::string header = GetHIPHeader();
	header += "struct " + kernel->kernel_name_ + "_vars {\n";
	for (size_t i = 0; i < kernel->var_names.size(); i++) header += "  " + kernel->var_types[i] + " " + kernel->var_names[i] + ";\n";
	header += "};\n\n";
	kernel->generated_header_ = header;

	// ---- bindings: one `uint*` per buffer, read-write first ---------------------------------------------
	// Every binding is its own allocation of the memory pool, so the pointers never alias; read-only ones
	// are const, which lets wave-uniform loads from them go through the scalar unit.
	std::string params;
	for (Node* mem : kernel->read_write_memory) params += "uint* __restrict__ " + mem->var_name + "_mem, ";
	for (Node* mem : kernel->read_only_memory) params += "const uint* __restrict__ " + mem->var_name + "_mem, ";
	params += kernel->kernel_name_ + "_vars var";
	kernel->generated_bindings_ = params;

	// ---- thread mapping -------------------------------------------------------------------------------
	std::string main;
	std::string body_indent = "    ";
	if (uses_group) {
		// Kernels with group memory / barriers run with exactly the thread-group the IR chose.
		kernel->hip_threads = group_threads;
		kernel->groups_per_hip_block = 1;
		kernel->idiom = "group";
		main += "extern \"C\" __global__ __launch_bounds__(" + std::to_string(group_threads) + ") void " + kernel->kernel_name_ + "(" + params + ")\n{\n";
		for (Node* gm : kernel->group_memory) {
			// named during generation
			main += "  __shared__ " + std::string(TypeName(gm->type)) + " " + gm->var_name + "[" + std::to_string(gm->data) + "];\n";
		}
		main += "  const int block_id = (int)(blockIdx.x + var._kernel_block_offset);\n";
		main += "  const int block_thread_id0 = (int)threadIdx.x;\n  const int block_thread_id1 = (int)threadIdx.y;\n  const int block_thread_id2 = (int)threadIdx.z;\n";
		main += "  {\n";
		main += generator.Assemble(body_indent);
		main += "  }\n}\n";
	} else if (!reductions.empty()) {
		// One wavefront per logical thread: 4 logical threads per 256-thread HIP group.
		kernel->hip_threads = 256;
		kernel->groups_per_hip_block = 0;  // grid = ceil(work_group_count * group_threads / 4)
		kernel->idiom = "reduction:wave";
		main += "extern \"C\" __global__ __launch_bounds__(256) void " + kernel->kernel_name_ + "(" + params + ")\n{\n";
		main += "  const int _lane = (int)(threadIdx.x & 63u);\n";
		main += "  const long long _logical = (long long)blockIdx.x * 4 + (long long)(threadIdx.x >> 6);\n";
		main += "  const long long _total = (long long)var._work_group_count * " + std::to_string(group_threads) + ";\n";
		main += "  if (_logical < _total)\n  {\n";
		main += "    const int block_id = (int)(_logical / " + std::to_string(group_threads) + ") + (int)var._kernel_block_offset;\n";
		main += "    const int _local = (int)(_logical % " + std::to_string(group_threads) + ");\n";
		main += "    const int block_thread_id0 = _local % " + std::to_string(group[0]) + ";\n";
		main += "    const int block_thread_id1 = (_local / " + std::to_string(group[0]) + ") % " + std::to_string(group[1]) + ";\n";
		main += "    const int block_thread_id2 = _local / " + std::to_string(group[0] * group[1]) + ";\n";
		main += generator.Assemble(body_indent);
		main += "  }\n}\n";
	} else {
		// Flat kernels: a 256-thread HIP group covers Q consecutive IR thread-groups and walks their
		// logical threads so that the 64 lanes of a wave always hold 64 consecutive values of the
		// innermost index (x = q*G0 + t0): one wave instruction touches one contiguous span.
		int q = 1;
		if (group[0] < 64) q = (64 + group[0] - 1) / group[0];
		const int logical = q * group_threads;
		int threads = logical < 256 ? ((logical + 63) / 64) * 64 : 256;
		kernel->hip_threads = threads;
		kernel->groups_per_hip_block = q;
		kernel->idiom = "flat";
		const int width = q * group[0];
		main += "extern \"C\" __global__ __launch_bounds__(" + std::to_string(threads) + ") void " + kernel->kernel_name_ + "(" + params + ")\n{\n";
		main += "  auto _thread = [&](const int block_id, const int block_thread_id0, const int block_thread_id1, const int block_thread_id2)\n  {\n";
		main += generator.Assemble(body_indent);
		main += "  };\n";
		main += "  for (int _l = (int)threadIdx.x; _l < " + std::to_string(logical) + "; _l += " + std::to_string(threads) + ")\n  {\n";
		main += "    const int _x = _l % " + std::to_string(width) + ";\n";
		main += "    const int _r = _l / " + std::to_string(width) + ";\n";
		main += "    const uint _group = blockIdx.x * " + std::to_string(q) + "u + (uint)(_x / " + std::to_string(group[0]) + ");\n";
		main += "    if (_group < var._work_group_count)\n";
		main += "      _thread((int)(_group + var._kernel_block_offset), _x % " + std::to_string(group[0]) + ", _r % " + std::to_string(group[1]) + ", _r / " +
		        std::to_string(group[1]) + ");\n";
		main += "  }\n}\n";
	}
	kernel->generated_main_ = main;
	kernel->full_generated_code_ = kernel->generated_header_ + main;
}

}  // namespace tfhost
