#include "hip_generator.h"
#include "address_poly.h"

#include <functional>

#include <algorithm>
#include <array>
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

namespace {

struct Line {
	Node* node;
	std::string text;
	int indent;
	int variant;  // which emission of the node's scope this line belongs to
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
	    {"modf", "fmodf"}, {"sqrt", "tf_sqrt"}, {"exp", "expf"}, {"exp2", "exp2f"}, {"log", "logf"}, {"log2", "log2f"},
	    {"sin", "sinf"}, {"cos", "cosf"}, {"tan", "tanf"}, {"asin", "asinf"}, {"acos", "acosf"}, {"atan", "atanf"},
	    {"sinh", "sinhf"}, {"cosh", "coshf"}, {"tanh", "tanhf"}, {"pow", "powf"}, {"atan2", "atan2f"}, {"ceil", "ceilf"},
	    {"floor", "floorf"}, {"round", "roundf"}, {"fma", "fmaf"},
	};
	return m;
}

bool IsLocalArray(const Node* n) { return std::string(n->op->name) == "group_memory" || std::string(n->op->name) == "local_memory"; }

// ---- reduction idiom ------------------------------------------------------------------------------

struct ReductionLoop {
	Node* loop = nullptr;
	std::vector<std::pair<Node*, std::string>> accumulators;  // (accumulator, cross-lane combine function)
	// Every load that moves with the loop variable moves by exactly one word per step, and nothing in the body clamps,
	// wraps or selects an index (four consecutive steps then read four consecutive words, whatever the operands are).
	bool unit_stride = false;
	// The same once the index clamps of the body are the identity: clamp(x, lo, hi) with x affine in the loop variable
	// and lo, hi fixed during the loop is the identity over the whole loop if it is at the first and at the last step
	// (the out-of-bounds clamps the reference puts around the loads of reshaped and split tensors, Implementations.cpp:56-69).
	std::vector<Node*> index_clamps;
	// Some load moves with the loop variable by a large or unknown step (a sum down the rows of a matrix, one thread per
	// column: x[i * C + col]; an indirect read): neighbouring lanes cannot share such a loop, neighbouring threads already
	// read neighbouring words. The loop can still be cut into slices that different waves walk for the same threads.
	bool strided = false;
};

bool DependsOn(const Node* n, const Node* target, int depth = 0) {
	if (!n || depth > 64) return false;
	if (n == target) return true;
	for (Node* in : n->inputs)
		if (DependsOn(in, target, depth + 1)) return true;
	if (DependsOn(n->index, target, depth + 1)) return true;
	return false;
}

// Words the address moves per step of the loop variable, if that is a compile-time constant.
bool LoopStride(const Node* addr, const Node* loop_var, long& stride, int depth = 0) {
	if (!addr || depth > 32) return false;
	if (addr == loop_var) {
		stride = 1;
		return true;
	}
	if (!DependsOn(addr, loop_var)) {
		stride = 0;
		return true;
	}
	const std::string op = addr->op->name;
	if ((op == "add" || op == "sub") && addr->inputs.size() == 2) {
		long a, b;
		if (!LoopStride(addr->inputs[0], loop_var, a, depth + 1) || !LoopStride(addr->inputs[1], loop_var, b, depth + 1)) return false;
		stride = op == "add" ? a + b : a - b;
		return true;
	}
	if (op == "mul" && addr->inputs.size() == 2) {
		const Node* x = addr->inputs[0];
		const Node* y = addr->inputs[1];
		if (DependsOn(y, loop_var)) std::swap(x, y);
		if (DependsOn(y, loop_var) || std::string(y->op->name) != "const" || y->modified) return false;
		long a;
		if (!LoopStride(x, loop_var, a, depth + 1)) return false;
		stride = a * (long)(int)y->data;
		return true;
	}
	if (op == "clamp" && addr->inputs.size() == 3 && !DependsOn(addr->inputs[1], loop_var) && !DependsOn(addr->inputs[2], loop_var)) {
		// user-indexed loads: clamp(loop_var, 0, extent-1) moves with the loop variable wherever it is not saturated
		return LoopStride(addr->inputs[0], loop_var, stride, depth + 1);
	}
	if ((op == "int" || op == "uint" || op == "copy") && addr->inputs.size() == 1) return LoopStride(addr->inputs[0], loop_var, stride, depth + 1);
	return false;
}

// Is `bits` the identity of `op` for values of this type (so that every lane may start from it)?
bool IsIdentity(const std::string& op, TFType type, uint32_t bits) {
	if (op == "add" || op == "or") return bits == 0;
	if (op == "mul") return type == TFType_Float ? bits == FloatBits(1.0f) : bits == 1;
	if (op == "and") return type == TFType_Bool ? bits != 0 : bits == 0xFFFFFFFFu;
	if (op == "max") return type == TFType_Float ? bits == FloatBits(-3.402823466e+38f) : type == TFType_Int ? bits == 0x80000000u : bits == 0;
	if (op == "min") return type == TFType_Float ? bits == FloatBits(3.402823466e+38f) : type == TFType_Int ? bits == 0x7FFFFFFFu : bits == 0xFFFFFFFFu;
	return false;
}

// Matches loops of the form `acc_k = init_k; loop(b, e, 1) { ...pure...; acc_k = op_k(acc_k, value_k); ... }`:
// the reference's lowered dim_sum / dim_max / dim_min / dim_prod / dim_any / dim_all
// (Implementations.cpp:243-303) and hand-written accumulation loops (`acc.val += ...`, e.g. the all-pairs
// loop of examples/Simulation/n-body-benchmark.py:36-65). A wave can run such a loop cooperatively when
// every accumulator starts from the identity of its operation, nothing in the body writes memory, the
// accumulators are touched only by their own updates, and the loads that move with the loop variable do so
// by a small constant stride (neighbouring lanes then read neighbouring words).
#ifndef TF_THREADS_PER_LANE_GROUP
#define TF_THREADS_PER_LANE_GROUP 4
#endif
constexpr int kThreadsPerLaneGroup = TF_THREADS_PER_LANE_GROUP;

bool MatchReductionLoop(Node* loop, ReductionLoop& out) {
	if (std::string(loop->op->name) != "loop" || loop->children.empty()) return false;
	Node* step = loop->inputs[2];
	if (std::string(step->op->name) != "const" || (int)step->data != 1) return false;
	Node* begin = loop->inputs[0];
	Node* end = loop->inputs[1];
	if (std::string(begin->op->name) == "const" && std::string(end->op->name) == "const" && (int)end->data - (int)begin->data < 64) return false;

	std::vector<std::pair<Node*, std::string>> accs;
	std::unordered_set<const Node*> updates, acc_set;
	for (Node* c : loop->children) {
		if (std::string(c->op->name) != "set") continue;
		Node* acc = c->memory;
		if (!acc || !acc->modified || std::string(acc->op->name) != "const" || acc_set.count(acc)) return false;
		Node* update = c->inputs[0];
		if (update->inputs.size() != 2) return false;
		Node* value = update->inputs[0] == acc ? update->inputs[1] : update->inputs[1] == acc ? update->inputs[0] : nullptr;
		if (!value) return false;
		const std::string opname = update->op->name;
		static const std::unordered_map<std::string, std::string> combine = {
		    {"add", "tf_wave_add"}, {"mul", "tf_wave_mul"}, {"max", "tf_wave_max"}, {"min", "tf_wave_min"}, {"and", "tf_wave_and"}, {"or", "tf_wave_or"}};
		auto it = combine.find(opname);
		if (it == combine.end() || !IsIdentity(opname, acc->type, acc->data)) return false;
		accs.push_back({acc, it->second});
		acc_set.insert(acc);
		updates.insert(update);
	}
	if (accs.empty()) return false;
	bool has_load = false, unit_stride = true, clamps_ok = true, strided = false, near_load = false;
	std::vector<Node*> index_clamps;
	for (Node* c : loop->children) {
		const std::string n = c->op->name;
		if (n == "set") continue;
		if ((c->type == TFType_Int || c->type == TFType_Uint) && !updates.count(c) && (n == "clamp" || n == "mod" || n == "ternary" || n == "min" || n == "max")) {
			long moves = 0;
			if (n == "clamp" && c->inputs.size() == 3 && LoopStride(c->inputs[0], loop, moves) && !DependsOn(c->inputs[1], loop) && !DependsOn(c->inputs[2], loop))
				index_clamps.push_back(c);
			else
				clamps_ok = false;
		}
		if (n == "store" || n == "loop" || n == "if" || n == "break" || n == "continue" || n == "discard" || n == "group_barrier" || n == "local_memory") return false;
		if (c->op->cls == OpClass::Memory && n != "load") return false;  // atomics
		if (n == "load") {
			if (c->local_memory_op) return false;
			long stride = 0;
			if (!LoopStride(c->index, loop, stride) || std::labs(stride) > 8) {
				strided = true;
				has_load = true;
				unit_stride = false;
			} else if (stride != 0) {
				has_load = true;
				near_load = true;
				unit_stride &= stride == 1;
			}
		}
		if (!updates.count(c))
			for (auto& a : accs)
				if (DependsOn(c, a.first)) return false;
	}
	// the value fed to an update must not read any accumulator either
	for (const Node* u : updates)
		for (Node* in : u->inputs)
			if (!acc_set.count(in))
				for (auto& a : accs)
					if (DependsOn(in, a.first)) return false;
	if (!has_load) return false;
	// one load that lanes could share and one that they cannot (the k loop of a product, A[row, k] * B[k, col]): neither
	// way of sharing the loop fits both, it stays with its thread
	if (strided && near_load) return false;
	out.loop = loop;
	out.accumulators = accs;
	out.unit_stride = unit_stride && clamps_ok && index_clamps.empty();
	if (unit_stride && clamps_ok) out.index_clamps = index_clamps;
	out.strided = strided;
	return true;
}

bool DependsOnThread(const Node* n, int depth = 0) {
	if (!n || depth > 64) return false;
	const std::string op = n->op->name;
	if (op == "block_id" || op == "block_thread_id") return true;
	if (op == "load") return true;  // a loaded value may be anything
	for (Node* in : n->inputs)
		if (DependsOnThread(in, depth + 1)) return true;
	return false;
}

// Do all loads that move with the loop variable read the same words in every thread (an all-pairs loop over a
// second copy of the data, a broadcast table)? Then splitting the loop among lanes would turn one shared word
// into 64 different ones; such loops are split among waves instead and keep their loads wave-uniform.
bool ReadsBroadcast(const ReductionLoop& r) {
	const Node* loop = r.loop;
	if (DependsOnThread(loop->inputs[0]) || DependsOnThread(loop->inputs[1])) return false;
	for (const Node* c : loop->children)
		if (std::string(c->op->name) == "load" && DependsOn(c->index, loop) && DependsOnThread(c->index)) return false;
	return true;
}

// Can the waves of a group share the loop, each walking a slice of it for the same 64 threads? The bounds must be the
// same for every thread. Loops whose loads are shared by all threads are divided that way, and so are loops that no
// wave's lanes can share (ReductionLoop::strided).
bool Sliceable(const ReductionLoop& r) {
	if (ReadsBroadcast(r)) return true;
	return r.strided && !DependsOnThread(r.loop->inputs[0]) && !DependsOnThread(r.loop->inputs[1]);
}

// Do the loads that move with the loop variable ignore the innermost thread index? Then the lanes of a wave that
// differ only in that index read the same words on every trip (the hardware serves them as one request), and the
// plain thread-serial loop is already bandwidth-efficient: e.g. a histogram kernel of shape [groups, digits] in
// which every digit's thread walks the same 128 keys of its group.
bool LoadsIgnoreInnermostIndex(const ReductionLoop& r, const Kernel* kernel) {
	if (kernel->dim < 2 || kernel->index_nodes.empty() || kernel->group_size.empty() || kernel->group_size[0] < 16) return false;
	const Node* innermost = kernel->index_nodes[0];
	auto uses_thread_id0 = [&](const Node* n, auto&& self, int depth) -> bool {
		if (!n || depth > 64) return false;
		if (n == innermost) return true;
		if (std::string(n->op->name) == "block_thread_id" && n->data == 0) return true;
		for (Node* in : n->inputs)
			if (self(in, self, depth + 1)) return true;
		return self(n->index, self, depth + 1);
	};
	bool any = false;
	for (const Node* c : r.loop->children) {
		if (std::string(c->op->name) != "load" || !DependsOn(c->index, r.loop)) continue;
		if (uses_thread_id0(c->index, uses_thread_id0, 0)) return false;
		any = true;
	}
	return any && !uses_thread_id0(r.loop->inputs[0], uses_thread_id0, 0) && !uses_thread_id0(r.loop->inputs[1], uses_thread_id0, 0);
}

// ---- symbolic ranges --------------------------------------------------------------------------------
// Range of an integer value as [lo, hi], both ends of the form a*S + c for ONE symbol S, a kernel extent
// (S >= 1). Enough to see that clamp(index, 0, S-1) is the identity inside the dispatch guard and that
// (index + S - 1) % S needs one conditional subtraction instead of a division.
struct Bound {
	long a = 0, c = 0;
};
struct Range {
	bool known = false;
	const Node* sym = nullptr;
	Bound lo, hi;
};

bool LessEq(const Bound& x, const Bound& y) {  // x <= y for every S >= 1
	const long da = y.a - x.a, dc = y.c - x.c;
	return da >= 0 && da + dc >= 0;
}

class RangeAnalysis {
 public:
	explicit RangeAnalysis(const Kernel* kernel) : kernel_(kernel) {}

	// With a margin m > 0, thread indices are taken to lie in [m, extent-1-m] (the "interior" emission,
	// entered only after a run-time check of exactly that).
	void SetInteriorMargin(int m) {
		margin_ = m;
		memo_.clear();
	}

	Range Get(const Node* n, int depth = 0) {
		auto it = memo_.find(n);
		if (it != memo_.end()) return it->second;
		Range r = Compute(n, depth);
		memo_[n] = r;
		return r;
	}

	static bool Compatible(const Range& a, const Range& b) { return a.known && b.known && (!a.sym || !b.sym || a.sym == b.sym); }

 private:
	const Kernel* kernel_;
	int margin_ = 0;
	std::unordered_map<const Node*, Range> memo_;

	static Range Exact(long a, long c, const Node* sym) {
		Range r;
		r.known = true;
		r.sym = sym;
		r.lo = r.hi = Bound{a, c};
		return r;
	}

	Range Compute(const Node* n, int depth) {
		Range unknown;
		if (!n || depth > 32) return unknown;
		if (n->type != TFType_Int && n->type != TFType_Uint) return unknown;
		const std::string op = n->op->name;
		if (op == "const") {
			if (n->modified) return unknown;
			return Exact(0, n->type == TFType_Int ? (long)(int)n->data : (long)n->data, nullptr);
		}
		for (size_t k = 0; k < kernel_->shape_nodes.size(); k++)
			if (n == kernel_->shape_nodes[k]) return Exact(1, 0, n);
		for (size_t k = 0; k < kernel_->index_nodes.size(); k++) {
			if (n != kernel_->index_nodes[k]) continue;
			Range s = Get(kernel_->shape_nodes[k], depth + 1);
			if (!s.known) return unknown;
			Range r;
			r.known = true;
			r.sym = s.sym;
			r.lo = Bound{0, margin_};
			r.hi = Bound{s.hi.a, s.hi.c - 1 - margin_};
			return r;
		}
		if ((op == "add" || op == "sub") && n->inputs.size() == 2) {
			Range a = Get(n->inputs[0], depth + 1), b = Get(n->inputs[1], depth + 1);
			if (!Compatible(a, b)) return unknown;
			Range r;
			r.known = true;
			r.sym = a.sym ? a.sym : b.sym;
			if (op == "add") {
				r.lo = Bound{a.lo.a + b.lo.a, a.lo.c + b.lo.c};
				r.hi = Bound{a.hi.a + b.hi.a, a.hi.c + b.hi.c};
			} else {
				r.lo = Bound{a.lo.a - b.hi.a, a.lo.c - b.hi.c};
				r.hi = Bound{a.hi.a - b.lo.a, a.hi.c - b.lo.c};
			}
			// stay well inside 32 bits, where the arithmetic of the kernel cannot wrap
			if (std::labs(r.lo.a) > 4 || std::labs(r.hi.a) > 4 || std::labs(r.lo.c) > (1l << 24) || std::labs(r.hi.c) > (1l << 24)) return unknown;
			return r;
		}
		if (op == "mod" && n->inputs.size() == 2) {
			Range x = Get(n->inputs[0], depth + 1), d = Get(n->inputs[1], depth + 1);
			if (!Compatible(x, d) || d.lo.a != d.hi.a || d.lo.c != d.hi.c) return unknown;
			if (!LessEq(Bound{0, 1}, d.lo) || !LessEq(Bound{0, 0}, x.lo)) return unknown;  // divisor >= 1, dividend >= 0
			Range r;
			r.known = true;
			r.sym = d.sym ? d.sym : x.sym;
			if (LessEq(x.hi, Bound{d.lo.a, d.lo.c - 1})) return x;  // already reduced
			if (LessEq(d.lo, x.lo) && LessEq(x.hi, Bound{2 * d.lo.a, 2 * d.lo.c - 1})) {  // exactly one period above
				r.lo = Bound{x.lo.a - d.lo.a, x.lo.c - d.lo.c};
				r.hi = Bound{x.hi.a - d.lo.a, x.hi.c - d.lo.c};
				return r;
			}
			r.lo = Bound{0, 0};
			r.hi = Bound{d.hi.a, d.hi.c - 1};
			return r;
		}
		if (op == "clamp" && n->inputs.size() == 3) {
			Range l = Get(n->inputs[1], depth + 1), h = Get(n->inputs[2], depth + 1);
			if (!Compatible(l, h)) return unknown;
			Range r;
			r.known = true;
			r.sym = l.sym ? l.sym : h.sym;
			r.lo = l.lo;
			r.hi = h.hi;
			return r;
		}
		if ((op == "int" || op == "uint" || op == "copy") && n->inputs.size() == 1) {
			Range x = Get(n->inputs[0], depth + 1);
			if (x.known && LessEq(Bound{0, 0}, x.lo)) return x;  // non-negative values survive the cast
			return unknown;
		}
		if (op == "loop" && n->inputs.size() == 3) {
			// for (i = begin; i < end; i += 1): i in [begin, end - 1] inside the body
			const Node* step = n->inputs[2];
			if (std::string(step->op->name) != "const" || (int)step->data != 1) return unknown;
			Range b = Get(n->inputs[0], depth + 1), e = Get(n->inputs[1], depth + 1);
			if (!Compatible(b, e)) return unknown;
			Range r;
			r.known = true;
			r.sym = b.sym ? b.sym : e.sym;
			r.lo = b.lo;
			r.hi = Bound{e.hi.a, e.hi.c - 1};
			return r;
		}
		return unknown;
	}
};

// ---- generator --------------------------------------------------------------------------------------

// Waves of a HIP group that share the loops of the sliced mapping (1024 threads: four waves per SIMD).
constexpr int kSliceWaves = 16;

using Lanes = std::array<std::string, 4>;

class HIPGenerator {
 public:
	// lanes == 1: one logical thread per emitted body. lanes == 4: four logical threads with consecutive
	// block_thread_id0 per body; values that depend on block_thread_id0 exist once per lane.
	HIPGenerator(Kernel* kernel, int lanes) : kernel_(kernel), lanes_(lanes), ranges_(kernel) {
		for (auto& v : kernel->variables) variables_.insert(v.node);
		if (lanes_ == 4) ComputeVarying(kernel->root);
	}

	// sliced: the matched loops are divided among the waves of a HIP group (each wave holds the same 64 logical
	// threads and walks its own slice); otherwise among the 64 lanes of one wave per logical thread.
	// group_lanes: lanes that share one logical thread in the lane-strided mapping (64 = the whole wave).
	// slabs (sliced only, one loop): several HIP groups may share the 64 threads of a group, each taking one slab of the loop.
	void Generate(const std::vector<ReductionLoop>& reductions, bool sliced = false, int group_lanes = 64, bool slabs = false) {
		for (auto& r : reductions) reduction_of_loop_[r.loop] = r;
		cooperative_ = !reductions.empty();
		sliced_ = sliced;
		slabs_ = slabs;
		group_lanes_ = group_lanes;
		// Buffers appear as <name>_mem, so a value may carry the buffer's own name (the loaded element usually does).
		int next = 0;
		Number(kernel_->root, next);
		read_only_.insert(kernel_->read_only_memory.begin(), kernel_->read_only_memory.end());
		for (auto& v : kernel_->variables) v.node->var_name = v.name;
		Walk(kernel_->root, 0, false);
	}

	void Number(const Node* scope, int& next) {
		for (const Node* c : scope->children) {
			position_[c] = next++;
			if (std::string(c->op->name) == "set" && c->memory) sets_of_[c->memory].push_back(position_[c]);
			if (!c->children.empty()) Number(c, next);
			scope_end_[c] = next - 1;
		}
	}

	// The modified values whose current contents the expression of `n` would read if it were written out at its user.
	void ReadsModified(const Node* n, std::vector<const Node*>& out, int depth = 0) const {
		for (const Node* in : n->inputs) {
			if (in->modified)
				out.push_back(in);
			else if (in->debug_name.empty() && in->use_count == 1 && depth < 64)
				ReadsModified(in, out, depth + 1);
		}
	}

	// Would `arg`, written out inside `user`, read another value of a modified variable than at its own place? That is
	// the case when the variable is set between the two, or when `user` runs in a loop that `arg` lies outside of and
	// that sets the variable.
	bool StaleAt(const Node* arg, const Node* user) const {
		std::vector<const Node*> reads;
		ReadsModified(arg, reads);
		if (reads.empty()) return false;
		auto pa = position_.find(arg), pu = user ? position_.find(user) : position_.end();
		if (pa == position_.end() || pu == position_.end()) return true;  // not placed (a temporary scope): keep the value
		for (const Node* m : reads) {
			auto sets = sets_of_.find(m);
			if (sets == sets_of_.end()) continue;
			for (int at : sets->second) {
				if (at > pa->second && at < pu->second) return true;
				for (const Node* scope = user->parent; scope; scope = scope->parent) {
					if (std::string(scope->op->name) != "loop") continue;
					auto ps = position_.find(scope), pe = scope_end_.find(scope);
					if (ps == position_.end() || pe == scope_end_.end()) return true;
					const bool holds_arg = pa->second > ps->second && pa->second <= pe->second;
					if (!holds_arg && at > ps->second && at <= pe->second) return true;
				}
			}
		}
		return false;
	}

	std::string Assemble(const std::string& base_indent) const {
		std::string code;
		for (auto& l : lines_) {
			if (l.node && removed_.count({l.node, l.variant})) continue;
			code += base_indent;
			for (int i = 0; i < l.indent; i++) code += "  ";
			code += l.text;
			code += "\n";
		}
		return code;
	}

	// Can the kernel be emitted four logical threads at a time? (checked on a lanes == 4 instance)
	int serial_load_loops() const { return serial_load_loops_; }

	bool Vectorizable(std::string* why = nullptr) const {
		auto no = [&](const char* reason) {
			if (why) *why = reason;
			return false;
		};
		if (kernel_->group_size.empty() || kernel_->group_size[0] % 4 != 0) return no("innermost group size is not a multiple of 4");
		if (!kernel_->dispatch_guard || kernel_->root->children.empty() || kernel_->root->children.back() != kernel_->dispatch_guard)
			return no("no dispatch guard at the end of the kernel");
		return CheckScope(kernel_->root, why);
	}

	void SetScalarFallback(const std::string& call_prefix) { scalar_call_prefix_ = call_prefix; }

 private:
	Kernel* kernel_;
	int lanes_;
	RangeAnalysis ranges_;
	std::vector<Line> lines_;
	std::unordered_set<Node*> variables_;
	std::unordered_set<const Node*> varying_;
	std::unordered_map<Node*, Lanes> expression_;
	std::unordered_map<Node*, bool> needs_parens_;
	std::set<std::pair<Node*, int>> removed_;
	int variant_ = 0;
	std::unordered_map<std::string, int> name_count_;
	std::unordered_set<std::string> array_names_;  // group and per-thread arrays: a value of the same name gets a trailing underscore
	// Program order: position of every node, the last position inside every scope, and where each modified value is set.
	std::unordered_map<const Node*, int> position_, scope_end_;
	std::unordered_map<const Node*, std::vector<int>> sets_of_;
	const Node* current_user_ = nullptr;  // the statement whose arguments are being named (nullptr: unknown)
	std::unordered_map<Node*, ReductionLoop> reduction_of_loop_;
	std::unordered_map<const Node*, std::pair<bool, long>> coeff_memo_;
	bool cooperative_ = false;
	bool sliced_ = false;
	bool slabs_ = false;
	int group_lanes_ = 64;
	bool inside_guard_ = false;
	std::vector<const Node*> open_loops_;  // loops whose bodies are being walked, outermost first
	std::unordered_set<const Node*> read_only_;
	int serial_load_loops_ = 0;       // innermost serial loops that read global memory, as emitted so far
	bool index_clamp_macro_ = false;  // integer clamps are printed as TF_INDEX_CLAMP (a loop emitted in two forms is being walked)
	std::string scalar_call_prefix_;

	// a (op) b for the operation whose cross-lane finish is `wave_fn`
	static std::string CombineExpression(const std::string& wave_fn, const std::string& a, const std::string& b) {
		if (wave_fn == "tf_wave_add") return a + " + " + b;
		if (wave_fn == "tf_wave_mul") return a + " * " + b;
		if (wave_fn == "tf_wave_max") return "tf_max(" + a + ", " + b + ")";
		if (wave_fn == "tf_wave_min") return "tf_min(" + a + ", " + b + ")";
		if (wave_fn == "tf_wave_and") return a + " & " + b;
		if (wave_fn == "tf_wave_or") return a + " | " + b;
		throw std::runtime_error("no combine expression for " + wave_fn);
	}

	static std::string MapName(const std::string& n) {
		auto it = NameMap().find(n);
		return it == NameMap().end() ? n : it->second;
	}

	bool IsVarying(const Node* n) const { return lanes_ == 4 && varying_.count(n) != 0; }

	// ---- which values differ between the four logical threads of a body -------------------------------
	void CollectNodes(Node* scope, std::vector<Node*>& out) {
		for (Node* c : scope->children) {
			out.push_back(c);
			if (!c->children.empty()) CollectNodes(c, out);
		}
	}

	void ComputeVarying(Node* root) {
		std::vector<Node*> all;
		CollectNodes(root, all);
		bool changed = true;
		while (changed) {
			changed = false;
			for (Node* n : all) {
				if (varying_.count(n)) continue;
				bool v = false;
				const std::string op = n->op->name;
				if (op == "block_thread_id" && n->data == 0) v = true;
				if (op == "InterlockedAdd_Prev") v = true;
				for (Node* in : n->inputs) v |= varying_.count(in) != 0;
				if (n->index && varying_.count(n->index)) v = true;
				if (op == "load" && n->memory && varying_.count(n->memory)) v = true;
				if (op == "set" && v && n->memory && !varying_.count(n->memory)) {
					varying_.insert(n->memory);
					changed = true;
				}
				if (op == "set" && n->memory && varying_.count(n->memory)) v = true;
				if (v) {
					varying_.insert(n);
					changed = true;
				}
			}
		}
	}

	bool CheckScope(const Node* scope, std::string* why) const {
		for (const Node* c : scope->children) {
			const std::string op = c->op->name;
			auto no = [&](const char* reason) {
				if (why) *why = reason;
				return false;
			};
			if (op == "local_memory" || op == "group_memory" || op == "group_barrier") return no("uses per-thread or group arrays");
			if (op == "discard") return no("uses discard");
			if (op == "loop" && varying_.count(c)) return no("loop bounds differ between neighbouring threads");
			if (op == "if" && c != kernel_->dispatch_guard && varying_.count(c->inputs[0])) return no("branch condition differs between neighbouring threads");
			if (!c->children.empty() && !CheckScope(c, why)) return false;
		}
		return true;
	}

	// clamp(x, lo, hi) with x provably inside [lo, hi] (a thread index against its own extent).
	bool IsIdentityClamp(const Node* n) {
		if (std::string(n->op->name) != "clamp" || n->inputs.size() != 3) return false;
		Range x = ranges_.Get(n->inputs[0]), l = ranges_.Get(n->inputs[1]), h = ranges_.Get(n->inputs[2]);
		return RangeAnalysis::Compatible(x, l) && RangeAnalysis::Compatible(x, h) && RangeAnalysis::Compatible(l, h) && LessEq(l.hi, x.lo) && LessEq(x.hi, h.lo);
	}

	// What an integer remainder x % d reduces to, given the ranges of x and d.
	enum class ModForm { Generic, Identity, SubtractOnce, ConditionalSubtract };
	ModForm ClassifyMod(const Node* n) {
		if (std::string(n->op->name) != "mod" || n->inputs.size() != 2) return ModForm::Generic;
		if (n->type != TFType_Int && n->type != TFType_Uint) return ModForm::Generic;
		Range x = ranges_.Get(n->inputs[0]), d = ranges_.Get(n->inputs[1]);
		if (!RangeAnalysis::Compatible(x, d) || d.lo.a != d.hi.a || d.lo.c != d.hi.c) return ModForm::Generic;
		if (!LessEq(Bound{0, 1}, d.lo) || !LessEq(Bound{0, 0}, x.lo)) return ModForm::Generic;
		if (LessEq(x.hi, Bound{d.lo.a, d.lo.c - 1})) return ModForm::Identity;
		if (!LessEq(x.hi, Bound{2 * d.lo.a, 2 * d.lo.c - 1})) return ModForm::Generic;
		return LessEq(d.lo, x.lo) ? ModForm::SubtractOnce : ModForm::ConditionalSubtract;
	}

	// Coefficient of block_thread_id0 in an integer expression, if the expression is affine in it.
	std::pair<bool, long> Coeff(const Node* n, int depth = 0) {
		if (!n) return {true, 0};
		if (!IsVarying(n)) return {true, 0};
		auto it = coeff_memo_.find(n);
		if (it != coeff_memo_.end()) return it->second;
		std::pair<bool, long> r = {false, 0};
		const std::string op = n->op->name;
		if (depth > 48 || n->modified) {
			r = {false, 0};
		} else if (op == "block_thread_id") {
			r = {true, 1};
		} else if ((op == "add" || op == "sub") && n->inputs.size() == 2) {
			auto a = Coeff(n->inputs[0], depth + 1), b = Coeff(n->inputs[1], depth + 1);
			if (a.first && b.first) r = {true, op == "add" ? a.second + b.second : a.second - b.second};
		} else if (op == "mul" && n->inputs.size() == 2) {
			const Node* x = n->inputs[0];
			const Node* y = n->inputs[1];
			if (IsVarying(y)) std::swap(x, y);  // x varying, y should be a plain constant
			auto a = Coeff(x, depth + 1);
			if (a.first && !IsVarying(y) && std::string(y->op->name) == "const" && !y->modified) r = {true, a.second * (long)(int)y->data};
		} else if ((op == "int" || op == "uint" || op == "copy") && n->inputs.size() == 1) {
			r = Coeff(n->inputs[0], depth + 1);
		} else if (inside_guard_ && IsIdentityClamp(n)) {
			r = Coeff(n->inputs[0], depth + 1);
		} else if (inside_guard_ && op == "mod" && !IsVarying(n->inputs[1])) {
			const ModForm form = ClassifyMod(n);
			if (form == ModForm::Identity || form == ModForm::SubtractOnce) r = Coeff(n->inputs[0], depth + 1);
		}
		coeff_memo_[n] = r;
		return r;
	}

	// x mod d for component `lane` of a quad, when that is the same number in every thread: d divides 4 and the quad's
	// first logical thread has a block_thread_id0 that is a multiple of 4 (the innermost group size is), so the parity of
	// an innermost index -- sine for even, cosine for odd features, red and black cells -- is known per component and the
	// test on it costs nothing, nor does the branch not taken.
	std::pair<bool, long> Residue(const Node* n, long d, int lane, int depth = 0) {
		if (!n || depth > 32 || n->modified || (n->type != TFType_Int && n->type != TFType_Uint)) return {false, 0};
		const std::string op = n->op->name;
		auto norm = [&](long v) { return ((v % d) + d) % d; };
		if (op == "const") return {true, norm(n->type == TFType_Int ? (long)(int)n->data : (long)n->data)};
		if (op == "block_thread_id") return IsVarying(n) ? std::make_pair(true, norm(lane)) : std::make_pair(false, 0l);
		if ((op == "add" || op == "sub") && n->inputs.size() == 2) {
			auto a = Residue(n->inputs[0], d, lane, depth + 1), b = Residue(n->inputs[1], d, lane, depth + 1);
			if (a.first && b.first) return {true, norm(op == "add" ? a.second + b.second : a.second - b.second)};
			return {false, 0};
		}
		if (op == "mul" && n->inputs.size() == 2) {
			auto a = Residue(n->inputs[0], d, lane, depth + 1), b = Residue(n->inputs[1], d, lane, depth + 1);
			if ((a.first && a.second == 0) || (b.first && b.second == 0)) return {true, 0};
			if (a.first && b.first) return {true, norm(a.second * b.second)};
			return {false, 0};
		}
		if ((op == "int" || op == "uint" || op == "copy") && n->inputs.size() == 1) {
			// a cast keeps the residue as long as the value is not negative
			Range x = ranges_.Get(n->inputs[0]);
			if (x.known && LessEq(Bound{0, 0}, x.lo)) return Residue(n->inputs[0], d, lane, depth + 1);
		}
		return {false, 0};
	}

	// Same naming scheme as the reference's RegenerateNodeName (Generators.h:126-149).
	void Rename(Node* node) {
		if (IsLocalArray(node)) {
			// arrays keep their name and only reserve it (RegenerateNodeName's LocalMemory branch)
			node->var_name = node->debug_name;
			array_names_.insert(node->var_name);
			return;
		}
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
		if (array_names_.count(debug)) debug += "_";
		node->var_name = debug;
	}

	std::string LaneName(const Node* n, int lane) const { return IsVarying(n) ? n->var_name + "_v" + std::to_string(lane) : n->var_name; }

	std::string ConstantString(const Node* n) const {
		switch (n->type) {
			case TFType_Float: {
				float f;
				std::memcpy(&f, &n->data, 4);
				return FormatFloat(f);
			}
			case TFType_Int:
				// -2147483648 is not an int literal in C++ (the minus applies to a long)
				return n->data == 0x80000000u ? std::string("(-2147483647 - 1)") : std::to_string((int)n->data);
			case TFType_Uint: return std::to_string(n->data) + "u";
			case TFType_Bool: return n->data == 0 ? "false" : "true";
			default: throw std::runtime_error("Unsupported constant type");
		}
	}

	// Name under which `arg` appears inside the expression of a user: its variable name, or -- for
	// unnamed single-use pure values -- its whole expression (Generators.h:90-124).
	std::string ArgName(Node* arg, bool parenthesise, int lane) {
		if (variables_.count(arg)) return "var." + arg->var_name;
		const std::string opname = arg->op->name;
		const bool is_constant = arg->op->cls == OpClass::Constant;
		const bool is_variable = arg->op->cls == OpClass::Variable;
		const int l = IsVarying(arg) ? lane : 0;
		std::string expr = expression_[arg][l];
		if (is_constant && expr.empty() && !arg->modified) expr = ConstantString(arg);
		const bool is_static = opname == "loop" || opname == "if" || opname == "InterlockedAdd_Prev" || arg->op->cls == OpClass::Keyword;
		const bool is_memory = opname == "memory" || IsLocalArray(arg) || arg->op->cls == OpClass::Memory;
		const bool single = arg->use_count == 1 || is_constant || is_variable;
		// The reference substitutes whatever is unnamed, single-use and short (Generators.h:90-124), also an expression
		// that reads a modified variable; here that is done as long as the variable cannot change on the way.
		const bool can_substitute = arg->debug_name.empty() && single && !arg->modified && expr.size() < 100 && !is_static && !is_memory &&
		                            !expr.empty() && !StaleAt(arg, current_user_);
		if (can_substitute) {
			removed_.insert({arg, variant_});
			if (parenthesise && needs_parens_[arg]) return "(" + expr + ")";
			return expr;
		}
		return LaneName(arg, l);
	}

	void Emit(Node* node, int indent, const std::string& text) { lines_.push_back({node, text, indent, variant_}); }

	static constexpr int kInteriorMargin = 4;

	// Starts another emission of the dispatch-guard body under a different assumption about the indices.
	void BeginVariant(int margin) {
		variant_++;
		ranges_.SetInteriorMargin(margin);
		coeff_memo_.clear();
	}

	static bool HasIndexWrapping(const Node* scope) {
		for (const Node* c : scope->children) {
			const std::string op = c->op->name;
			if ((op == "clamp" || op == "mod") && (c->type == TFType_Int || c->type == TFType_Uint)) return true;
			if (!c->children.empty() && HasIndexWrapping(c)) return true;
		}
		return false;
	}

	// A load inside a loop from a read-only buffer whose address moves with the innermost open loop and with every
	// thread index of the kernel: no other thread and no other step reads the same word (the operand of a reduction),
	// so it is fetched past the caches. A load that ignores a thread index (the operands of a matmul loop) is shared
	// by the threads along that index and stays cached.
	bool StreamsOnce(const Node* load) const {
		if (open_loops_.empty() || !load->index || !read_only_.count(load->memory)) return false;
		if (!DependsOn(load->index, open_loops_.back())) return false;
		for (const Node* idx : kernel_->index_nodes)
			if (!DependsOn(load->index, idx)) return false;
		return !kernel_->index_nodes.empty();
	}

	// The statements of the loop body that the operands of these clamps are computed from, in body order.
	static std::vector<Node*> ClampOperandSlice(const Node* loop, const std::vector<Node*>& clamps) {
		std::unordered_set<const Node*> body(loop->children.begin(), loop->children.end()), needed;
		std::function<void(const Node*)> need = [&](const Node* n) {
			if (!n || !body.count(n) || !needed.insert(n).second) return;
			for (const Node* in : n->inputs) need(in);
			need(n->index);
		};
		for (const Node* c : clamps)
			for (const Node* in : c->inputs) need(in);
		std::vector<Node*> slice;
		for (Node* c : loop->children)
			if (needed.count(c)) slice.push_back(c);
		return slice;
	}

	void Walk(Node* scope, int indent, bool lane_guard_stores) {
		for (Node* node : scope->children) {
			const std::string opname = node->op->name;
			if (opname == "loop") {
				current_user_ = node;
				Rename(node);
				struct OpenLoop {
					std::vector<const Node*>& stack;
					OpenLoop(std::vector<const Node*>& s, const Node* n) : stack(s) { stack.push_back(n); }
					~OpenLoop() { stack.pop_back(); }
				} open_loop(open_loops_, node);
				auto red = reduction_of_loop_.find(node);
				std::string b = ArgName(node->inputs[0], false, 0), e = ArgName(node->inputs[1], false, 0), s = ArgName(node->inputs[2], false, 0);
				if (red != reduction_of_loop_.end() && sliced_) {
					// Every wave of the group walks one contiguous slice of the loop for the same 64 logical threads.
					// Loop bounds and loads that do not depend on the thread are wave-uniform, so they go through the
					// scalar unit; the partial results meet in group memory, and every wave leaves with the total.
					const std::string v = node->var_name;
					if (slabs_) {
						// the groups that share these 64 threads take one slab of the loop each
						Emit(node, indent, "const int " + v + "_all = tf_max((int)((" + e + ") - (" + b + ")), 0);");
						Emit(nullptr, indent, "const int " + v + "_slab = (" + v + "_all + (int)var._slabs - 1) / (int)var._slabs;");
						Emit(nullptr, indent, "const int " + v + "_from = (" + b + ") + (int)_slab * " + v + "_slab;");
						Emit(nullptr, indent, "const int " + v + "_to = tf_min((int)(" + e + "), " + v + "_from + " + v + "_slab);");
						b = v + "_from";
						e = v + "_to";
					}
					if (red->second.strided) {
						// a short walk is not worth sixteen waves' memory latencies: the first wave takes all of it and
						// the others contribute the identity
						Emit(node, indent, "const int " + v + "_trips = tf_max((int)((" + e + ") - (" + b + ")), 0);");
						Emit(nullptr, indent, "const int " + v + "_per = " + v + "_trips < " + std::to_string(kSliceWaves * 8) + " ? " + v + "_trips : (" + v + "_trips + " +
						                          std::to_string(kSliceWaves - 1) + ") / " + std::to_string(kSliceWaves) + ";");
					} else {
						Emit(node, indent, "const int " + v + "_per = ((" + e + ") - (" + b + ") + " + std::to_string(kSliceWaves - 1) + ") / " + std::to_string(kSliceWaves) + ";");
					}
					Emit(nullptr, indent, "const int " + v + "_begin = (" + b + ") + _wave * " + v + "_per;");
					Emit(nullptr, indent, "const int " + v + "_end = tf_min((int)(" + e + "), " + v + "_begin + " + v + "_per);");
					Emit(nullptr, indent, "#pragma unroll 4");
					Emit(nullptr, indent, "for (int " + v + " = " + v + "_begin; " + v + " < " + v + "_end; " + v + " += 1)");
					Emit(nullptr, indent, "{");
					Walk(node, indent + 1, false);
					Emit(nullptr, indent, "}");
					Emit(nullptr, indent, "__syncthreads();");
					int slot = 0;
					for (auto& a : red->second.accumulators)
						Emit(nullptr, indent, "_partials[(" + std::to_string(slot++ * kSliceWaves) + " + _wave) * 64 + _lane] = asuint(" + a.first->var_name + ");");
					Emit(nullptr, indent, "__syncthreads();");
					slot = 0;
					for (auto& a : red->second.accumulators) {
						const std::string t = TypeName(a.first->type);
						const std::string n = a.first->var_name;
						const std::string base = std::to_string(slot++ * kSliceWaves);
						auto partial = [&](const std::string& w) { return "as" + t + "(_partials[(" + base + " + " + w + ") * 64 + _lane])"; };
						Emit(nullptr, indent, n + " = " + partial("0") + ";");
						Emit(nullptr, indent, "for (int _w = 1; _w < " + std::to_string(kSliceWaves) + "; _w++) " + n + " = " + CombineExpression(a.second, n, partial("_w")) + ";");
					}
					if (slabs_) {
						// Every group leaves its slab's results in memory and takes a ticket; the group that takes the last
						// ticket of its 64 threads adds the slabs up in slab order (the same order whichever group it is) and
						// goes on with the rest of the kernel, the others are done. Results are written and read with
						// device-scope atomic accesses (write-through stores, loads that bypass the die's caches), and a
						// group takes its ticket only after its stores have been acknowledged. No fence: a release fence
						// writes the die's whole L2 back and an acquire fence empties it, tens of microseconds per group
						// (measured: the time of a launch grew linearly with the number of groups). The ticket counter is
						// left at zero for the next launch.
						const size_t count = red->second.accumulators.size();
						const std::string words = std::to_string(count * 64);
						Emit(nullptr, indent, "if (var._slabs > 1u)");
						Emit(nullptr, indent, "{");
						Emit(nullptr, indent + 1, "uint* _mine = _slab_partials + ((size_t)_slab * _column_groups + _column_group) * " + words + ";");
						slot = 0;
						for (auto& a : red->second.accumulators)
							Emit(nullptr, indent + 1, "if (_wave == 0) __hip_atomic_store(_mine + " + std::to_string(slot++ * 64) + " + _lane, asuint(" + a.first->var_name +
							                              "), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);");
						Emit(nullptr, indent + 1, "__builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): the write-through stores above have been acknowledged");
						Emit(nullptr, indent + 1, "__syncthreads();");
						Emit(nullptr, indent + 1, "if (_wave == 0 && _lane == (int)__ffsll((unsigned long long)__ballot(1)) - 1) _partials[0] = atomicAdd(_slab_tickets + _column_group, 1u);");
						Emit(nullptr, indent + 1, "__syncthreads();");
						Emit(nullptr, indent + 1, "const uint _ticket = _partials[0];");
						Emit(nullptr, indent + 1, "if (_ticket != var._slabs - 1u) return;");
						Emit(nullptr, indent + 1, "if (_wave == 0 && _lane == (int)__ffsll((unsigned long long)__ballot(1)) - 1) _slab_tickets[_column_group] = 0u;");
						slot = 0;
						for (auto& a : red->second.accumulators) {
							const std::string t = TypeName(a.first->type);
							const std::string n = a.first->var_name;
							const std::string at = std::to_string(slot++ * 64);
							auto partial = [&](const std::string& sl) {
								return "as" + t + "(__hip_atomic_load(_slab_partials + ((size_t)(" + sl + ") * _column_groups + _column_group) * " + words + " + " + at +
								       " + _lane, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT))";
							};
							Emit(nullptr, indent + 1, n + " = " + partial("0") + ";");
							Emit(nullptr, indent + 1, "for (uint _s = 1; _s < var._slabs; _s++) " + n + " = " + CombineExpression(a.second, n, partial("_s")) + ";");
						}
						Emit(nullptr, indent, "}");
					}
				} else if (red != reduction_of_loop_.end()) {
					// Lanes of the wave stride the loop; the accumulator of each lane starts from the
					// reduction's identity, so combining the 64 partial results gives the full result.
					const std::string width = std::to_string(group_lanes_);
					const std::string v = node->var_name;
					// Every load walks its array one word per step: a lane takes four consecutive steps per trip, so
					// that its four loads are one 16-byte access (and a wave instruction covers 1 KiB of consecutive
					// memory); what the trip count leaves over is done a step per lane.
					auto quad_loops = [&](int at) {
						Emit(node, at, "const int " + v + "_trips = tf_max((int)((" + e + ") - (" + b + ")), 0);");
						Emit(nullptr, at, "#pragma unroll 4");
						Emit(nullptr, at, "for (int " + v + "_q = _lane; " + v + "_q < (" + v + "_trips >> 2); " + v + "_q += " + width + ")");
						Emit(nullptr, at, "{");
						Emit(nullptr, at + 1, "#pragma unroll");
						Emit(nullptr, at + 1, "for (int " + v + "_u = 0; " + v + "_u < 4; " + v + "_u++)");
						Emit(nullptr, at + 1, "{");
						Emit(nullptr, at + 2, "const int " + v + " = (" + b + ") + " + v + "_q * 4 + " + v + "_u;");
						variant_++;
						Walk(node, at + 2, false);
						Emit(nullptr, at + 1, "}");
						Emit(nullptr, at, "}");
						Emit(nullptr, at, "for (int " + v + " = (" + b + ") + (" + v + "_trips & ~3) + _lane; " + v + " < " + e + "; " + v + " += " + width + ")");
						Emit(nullptr, at, "{");
						variant_++;
						Walk(node, at + 1, false);
						Emit(nullptr, at, "}");
					};
					auto strided_loop = [&](int at) {
						Emit(nullptr, at, "#pragma unroll 4");
						Emit(node, at, "for (int " + v + " = " + b + " + _lane; " + v + " < " + e + "; " + v + " += " + width + ")");
						Emit(nullptr, at, "{");
						variant_++;
						Walk(node, at + 1, false);
						Emit(nullptr, at, "}");
					};
					if (red->second.unit_stride) {
						quad_loops(indent);
					} else if (!red->second.index_clamps.empty()) {
						// The index clamps of the body are the identity over the whole loop if they are at its first and
						// at its last step (their operands move linearly with the loop variable). Where that holds -- every
						// logical thread except those at a ragged edge -- the loop runs in the four-step form with the
						// clamps compiled out, so that the four loads of a lane are consecutive words again.
						std::vector<Node*> slice = ClampOperandSlice(node, red->second.index_clamps);
						Node scope;
						scope.op = node->op;
						scope.children = slice;
						Emit(nullptr, indent, "bool " + v + "_fast = true;");
						for (int end = 0; end < 2; end++) {
							Emit(nullptr, indent, "{");
							Emit(nullptr, indent + 1, "const int " + v + " = " + (end == 0 ? "(" + b + ")" : "(" + e + ") - 1") + ";");
							variant_++;
							Walk(&scope, indent + 1, false);
							std::string test;
							for (Node* c : red->second.index_clamps) {
								current_user_ = c;
								const std::string x = ArgName(c->inputs[0], true, 0), lo = ArgName(c->inputs[1], true, 0), hi = ArgName(c->inputs[2], true, 0);
								test += " && " + lo + " <= " + x + " && " + x + " <= " + hi;
							}
							Emit(nullptr, indent + 1, v + "_fast = " + v + "_fast" + test + ";");
							Emit(nullptr, indent, "}");
						}
						Emit(nullptr, indent, "if (" + v + "_fast)");
						Emit(nullptr, indent, "{");
						Emit(nullptr, 0, "#undef TF_INDEX_CLAMP");
						Emit(nullptr, 0, "#define TF_INDEX_CLAMP(x, lo, hi) (x)");
						index_clamp_macro_ = true;
						quad_loops(indent + 1);
						Emit(nullptr, 0, "#undef TF_INDEX_CLAMP");
						Emit(nullptr, 0, "#define TF_INDEX_CLAMP(x, lo, hi) tf_clamp(x, lo, hi)");
						Emit(nullptr, indent, "}");
						Emit(nullptr, indent, "else");
						Emit(nullptr, indent, "{");
						strided_loop(indent + 1);
						index_clamp_macro_ = false;
						Emit(nullptr, indent, "}");
					} else {
						strided_loop(indent);
					}
					for (auto& a : red->second.accumulators)
						Emit(nullptr, indent, a.first->var_name + " = " + a.second + "(" + a.first->var_name + (group_lanes_ == 64 ? "" : ", " + width) + ");");
				} else {
					// A serial loop that reads global memory and contains no further loop: unrolled by four, so that the loads of
					// later steps are issued while the first is still in flight (read-only buffers are const __restrict__, so
					// they may move above the loop's stores).
					bool innermost = true, reads = false;
					for (Node* c : node->children) {
						const std::string cn = c->op->name;
						if (cn == "loop") innermost = false;
						if (cn == "load" && !c->local_memory_op) reads = true;
						if (cn == "if")
							for (Node* cc : c->children) {
								if (std::string(cc->op->name) == "loop") innermost = false;
								if (std::string(cc->op->name) == "load" && !cc->local_memory_op) reads = true;
							}
					}
					if (innermost && reads) {
						// Sixteen steps of a quad-wide thread hold 64 registers of loads in flight; the kernel is then
						// compiled for four waves per SIMD instead of eight (see serial_load_loops()).
						Emit(nullptr, indent, "#pragma unroll 16");
						serial_load_loops_++;
					}
					Emit(node, indent, "for (int " + node->var_name + " = " + b + "; " + node->var_name + " < " + e + "; " + node->var_name + " += " + s + ")");
					Emit(nullptr, indent, "{");
					Walk(node, indent + 1, lane_guard_stores);
					Emit(nullptr, indent, "}");
				}
				continue;
			}
			if (opname == "if") {
				current_user_ = node;
				const bool is_guard = node == kernel_->dispatch_guard;
				if (is_guard && lanes_ == 4) {
					// All four logical threads are inside when the first and the last are (index_0 grows with
					// block_thread_id0); otherwise each one goes through the single-thread body with its own guard.
					Emit(node, indent, "if (" + ArgName(node->inputs[0], false, 0) + " && " + ArgName(node->inputs[0], false, 3) + ")");
					Emit(nullptr, indent, "{");
					inside_guard_ = true;
					if (HasIndexWrapping(node)) {
						// Away from the borders (every index at least kInteriorMargin from both ends of its extent)
						// boundary clamps and periodic remainders are the identity or one subtraction, which turns
						// shifted taps into contiguous 16-byte loads; quads near a border keep the general form.
						std::string interior;
						for (size_t k = 0; k < kernel_->index_nodes.size(); k++) {
							Node* idx = kernel_->index_nodes[k];
							Node* ext = kernel_->shape_nodes[k];
							if (!interior.empty()) interior += " && ";
							interior += ArgName(idx, true, 0) + " >= " + std::to_string(kInteriorMargin) + " && " + ArgName(idx, true, 3) + " + " +
							            std::to_string(kInteriorMargin) + " < " + ArgName(ext, true, 0);
						}
						Emit(nullptr, indent + 1, "if (" + interior + ")");
						Emit(nullptr, indent + 1, "{");
						BeginVariant(kInteriorMargin);
						Walk(node, indent + 2, lane_guard_stores);
						Emit(nullptr, indent + 1, "}");
						Emit(nullptr, indent + 1, "else");
						Emit(nullptr, indent + 1, "{");
						BeginVariant(0);
						Walk(node, indent + 2, lane_guard_stores);
						Emit(nullptr, indent + 1, "}");
					} else {
						Walk(node, indent + 1, lane_guard_stores);
					}
					inside_guard_ = false;
					Emit(nullptr, indent, "}");
					Emit(nullptr, indent, "else");
					Emit(nullptr, indent, "{");
					for (int k = 0; k < 4; k++) Emit(nullptr, indent + 1, scalar_call_prefix_ + "block_id, block_thread_id0 + " + std::to_string(k) + ", block_thread_id1, block_thread_id2);");
					Emit(nullptr, indent, "}");
					continue;
				}
				Emit(node, indent, "if (" + ArgName(node->inputs[0], false, 0) + ")");
				Emit(nullptr, indent, "{");
				const bool was_inside = inside_guard_;
				if (is_guard) inside_guard_ = true;
				// Inside the dispatch guard of a wave-cooperative kernel, writes happen once per logical thread.
				Walk(node, indent + 1, cooperative_ ? true : lane_guard_stores);
				inside_guard_ = was_inside;
				Emit(nullptr, indent, "}");
				continue;
			}
			GenerateLine(node, indent, lane_guard_stores);
		}
	}

	// Expression of a pure (non-memory) node for one lane.
	std::string PureExpression(Node* node, int lane, bool& parens) {
		const std::string opname = node->op->name;
		const OpClass cls = node->op->cls;
		const std::string type = TypeName(node->type);
		parens = false;
		auto arg = [&](size_t i, bool p) { return ArgName(node->inputs[i], p, lane); };
		auto as_copy = [&](size_t i) {
			const std::string e = arg(i, false);
			parens = true;  // may be an operator expression
			return e;
		};
		switch (cls) {
			case OpClass::Operator: {
				std::string code = node->op->code;
				if ((code == "&" || code == "|") && node->type == TFType_Bool) code += code;
				if (code == "%" && node->type == TFType_Float) return "fmodf(" + arg(0, false) + ", " + arg(1, false) + ")";
				// float division through the reciprocal instruction, as the reference's -ffast-math build may (Backend.cpp:35)
				if (code == "/" && node->type == TFType_Float) {
					// a / (y * sqrt(y)) (the inverse-cube law of an all-pairs force): one reciprocal square root and
					// three products instead of a square root, a product and a reciprocal.
					const Node* den = node->inputs[1];
					if (!kernel_->verbatim && std::string(den->op->name) == "mul" && den->inputs.size() == 2 && den->use_count == 1 && !den->modified) {
						for (int side = 0; side < 2; side++) {
							const Node* root = den->inputs[side];
							const Node* y = den->inputs[1 - side];
							if (std::string(root->op->name) == "sqrt" && root->inputs.size() == 1 && root->inputs[0] == y && root->use_count == 1 && !root->modified) {
								// the product and the square root are not needed as values of their own
								removed_.insert({const_cast<Node*>(den), variant_});
								removed_.insert({const_cast<Node*>(root), variant_});
								return "tf_div_by_pow_3_2(" + arg(0, false) + ", " + ArgName(const_cast<Node*>(y), false, lane) + ")";
							}
						}
					}
					return "tf_div(" + arg(0, false) + ", " + arg(1, false) + ")";
				}
				if (code == "%" && inside_guard_ && !kernel_->verbatim && lanes_ == 4 && IsVarying(node) && node->type == TFType_Int &&
				    std::string(node->inputs[1]->op->name) == "const" && !node->inputs[1]->modified) {
					// The remainder by 2 or 4 of a value whose residue is fixed per component of the quad: a literal.
					const long d = (long)(int)node->inputs[1]->data;
					Range x = ranges_.Get(node->inputs[0]);
					if ((d == 2 || d == 4) && x.known && LessEq(Bound{0, 0}, x.lo)) {
						auto r = Residue(node->inputs[0], d, lane);
						if (r.first) {
							(void)arg(0, false);
							(void)arg(1, false);
							return std::to_string(r.second);
						}
					}
				}
				if (code == "%" && inside_guard_ && !kernel_->verbatim) {
					// Remainder of a value known to lie in [0, 2d): nothing, or one (conditional) subtraction.
					const ModForm form = ClassifyMod(node);
					if (form == ModForm::Identity) {
						(void)arg(1, false);
						return as_copy(0);
					}
					if (form == ModForm::SubtractOnce) {
						parens = true;
						return arg(0, true) + " - " + arg(1, true);
					}
					if (form == ModForm::ConditionalSubtract) {
						parens = true;
						const std::string a = arg(0, true), b = arg(1, true);
						return a + " >= " + b + " ? " + a + " - " + b + " : " + a;
					}
				}
				if (code == "%" && node->inputs[1]->op->cls != OpClass::Constant) return "tf_mod(" + arg(0, false) + ", " + arg(1, false) + ")";
				if (code == "+" && node->type == TFType_Float && !kernel_->verbatim) {
					// A sum of products and plain terms, e.g. dx*dx + dy*dy + dz*dz + eps: with the plain terms first every
					// product fuses into a multiply-add (three instructions instead of four here). That reorders float
					// additions, which the reference's own kernels are compiled to allow (-ffast-math, Backend.cpp:35);
					// TF_PRECISE_MATH keeps the written order.
					std::vector<Node*> terms, inner;
					std::function<void(Node*)> flatten = [&](Node* n) {
						for (Node* in : n->inputs) {
							const bool chain = std::string(in->op->name) == "add" && in->type == TFType_Float && in->inputs.size() == 2 && in->use_count == 1 &&
							                   in->debug_name.empty() && !in->modified && !variables_.count(in);
							if (chain) {
								inner.push_back(in);
								flatten(in);
							} else {
								terms.push_back(in);
							}
						}
					};
					flatten(node);
					auto is_product = [&](const Node* t) {
						return std::string(t->op->name) == "mul" && t->use_count == 1 && t->debug_name.empty() && !t->modified && !variables_.count(const_cast<Node*>(t));
					};
					bool plain_after_product = false, seen_product = false;
					for (Node* t : terms) {
						if (is_product(t)) seen_product = true;
						else if (seen_product) plain_after_product = true;
					}
					if (terms.size() >= 3 && plain_after_product) {
						const std::string written = arg(0, true) + " + " + arg(1, true);
						std::vector<Node*> order;
						for (Node* t : terms)
							if (!is_product(t)) order.push_back(t);
						for (Node* t : terms)
							if (is_product(t)) order.push_back(t);
						std::string sum = ArgName(order[0], true, lane);
						for (size_t i = 1; i < order.size(); i++) sum = (i > 1 ? "(" + sum + ")" : sum) + " + " + ArgName(order[i], true, lane);
						for (Node* in : inner) removed_.insert({in, variant_});
						return "TF_REASSOC(" + sum + ", " + written + ")";
					}
				}
				parens = true;
				return arg(0, true) + " " + code + " " + arg(1, true);
			}
			case OpClass::UnaryOperator:
				parens = true;
				return node->op->code + arg(0, true);
			case OpClass::Function: {
				if (opname == "clamp" && inside_guard_ && !kernel_->verbatim && node->inputs.size() == 3) {
					// clamp of a value already inside [lo, hi] (thread indices against their own extents)
					if (IsIdentityClamp(node)) {
						// the bounds become unused: drop their lines too
						(void)arg(1, false);
						(void)arg(2, false);
						return as_copy(0);
					}
				}
				const bool index_clamp = index_clamp_macro_ && opname == "clamp" && (node->type == TFType_Int || node->type == TFType_Uint);
				std::string e = (index_clamp ? std::string("TF_INDEX_CLAMP") : MapName(node->op->code)) + "(";
				for (size_t i = 0; i < node->inputs.size(); i++) {
					if (i) e += ", ";
					e += arg(i, false);
				}
				return e + ")";
			}
			case OpClass::Copy: return as_copy(0);
			case OpClass::Keyword: return opname == "discard" ? "return" : node->op->code;
			case OpClass::DimensionIndex: {
				std::string e = node->op->code + std::to_string(node->data);
				if (lane > 0 && IsVarying(node)) {
					parens = true;
					e += " + " + std::to_string(lane);
				}
				return e;
			}
			case OpClass::Variable: return node->op->code;
			case OpClass::TypeCast: return "((" + type + ")(" + arg(0, false) + "))";
			case OpClass::TypeReinterpret: return "as" + type + "(" + arg(0, false) + ")";
			case OpClass::Constant: return ConstantString(node);
			case OpClass::TernaryOperator:
				parens = true;
				return arg(0, true) + " ? " + arg(1, true) + " : " + arg(2, true);
			default: throw std::runtime_error("Unknown operation class for " + opname);
		}
	}

	void GenerateLine(Node* node, int indent, bool lane_guard) {
		current_user_ = node;
		const std::string opname = node->op->name;
		const OpClass cls = node->op->cls;
		if (opname == "memory" || opname == "variable") return;
		if (opname == "group_memory") {
			Rename(node);
			Emit(node, indent, "// " + std::string(TypeName(node->type)) + " " + node->var_name + "[" + std::to_string(node->data) + "] (declared as __shared__ above)");
			return;
		}
		Rename(node);
		const std::string type = TypeName(node->type);
		const std::string guard = !lane_guard ? "" : sliced_ ? "if (_wave == 0) " : "if (_lane == 0) ";
		if (opname == "local_memory") {
			Emit(node, indent, type + " " + node->var_name + "[" + std::to_string(node->data) + "];");
			return;
		}
		const bool varying = IsVarying(node);
		const int n_lanes = varying ? 4 : 1;

		if (cls == OpClass::Memory) {
			const bool local = node->local_memory_op;
			const std::string mem_name = node->memory->var_name + (local ? "" : "_mem");
			const TFType mem_type = local ? node->memory->type : TFType_Uint;
			auto address = [&](int lane) { return node->index ? ArgName(node->index, false, lane) : std::string("0"); };
			auto coeff = Coeff(node->index);
			const bool unit_stride = varying && !local && node->index && IsVarying(node->index) && coeff.first && coeff.second == 1;
			if (opname == "load") {
				if (unit_stride) {
					const std::string q = node->var_name + "_q";
					Emit(node, indent, "const tf_uint4 " + q + " = " + (StreamsOnce(node) ? "tf_load4_stream(" : "tf_load4(") + mem_name + " + (" + address(0) + "));");
					static const char* comp[4] = {".x", ".y", ".z", ".w"};
					for (int k = 0; k < 4; k++) {
						const std::string word = q + comp[k];
						Emit(node, indent, type + " " + LaneName(node, k) + " = " + (node->type == TFType_Uint ? word : "as" + type + "(" + word + ")") + ";");
					}
				} else {
					// Inside a loop that lanes share, a read-only buffer is streamed: each word is read once by this kernel.
					const bool stream = !local && StreamsOnce(node);
					for (int k = 0; k < n_lanes; k++) {
						const std::string mem_expr = stream ? "tf_stream_load(" + mem_name + " + (" + address(k) + "))" : mem_name + "[" + address(k) + "]";
						Emit(node, indent, type + " " + LaneName(node, k) + " = " + (node->type == mem_type ? mem_expr : "as" + type + "(" + mem_expr + ")") + ";");
					}
				}
				for (int k = 0; k < 4; k++) expression_[node][k] = "";
				return;
			}
			Node* value = node->inputs[0];
			if (opname == "store") {
				auto word = [&](int lane) {
					const std::string v = ArgName(value, false, lane);
					return value->type == mem_type ? v : std::string("as") + TypeName(mem_type) + "(" + v + ")";
				};
				if (unit_stride) {
					Emit(node, indent, "tf_store4(" + mem_name + " + (" + address(0) + "), " + word(0) + ", " + word(1) + ", " + word(2) + ", " + word(3) + ");");
				} else {
					for (int k = 0; k < n_lanes; k++) Emit(node, indent, guard + mem_name + "[" + address(k) + "] = " + word(k) + ";");
				}
				return;
			}
			// atomics: once per logical thread, whatever the lanes share
			const std::string in_type = TypeName(value->type);
			const int reps = lanes_;
			if (node->type != TFType_None && lane_guard) throw std::runtime_error("value-returning atomic after a wave-cooperative reduction is not supported");
			for (int k = 0; k < reps; k++) {
				std::string call = opname + "((" + in_type + "*)" + mem_name + ", " + address(k) + ", " + ArgName(value, false, k) + ")";
				if (node->type != TFType_None)
					Emit(node, indent, type + " " + LaneName(node, k) + " = " + call + ";");
				else
					Emit(node, indent, guard + call + ";");
			}
			return;
		}
		if (cls == OpClass::Set) {
			for (int k = 0; k < n_lanes; k++) Emit(node, indent, LaneName(node->memory, k) + " = " + ArgName(node->inputs[0], false, k) + ";");
			return;
		}
		bool parens = false;
		for (int k = 0; k < n_lanes; k++) {
			const std::string expr = PureExpression(node, k, parens);
			expression_[node][k] = expr;
			std::string left;
			if (node->type != TFType_None) left = type + " " + LaneName(node, k) + " = ";
			Emit(node, indent, left + expr + ";");
		}
		needs_parens_[node] = parens;
	}
};

bool UsesGroupFeatures(const Node* n) {
	const std::string name = n->op->name;
	if (name == "group_barrier" || name == "group_memory") return true;
	for (const Node* c : n->children)
		if (UsesGroupFeatures(c)) return true;
	return false;
}

// Sibling accumulation loops over the same range become one loop: the reference's fusion leaves `max`, `min`, `sum`,
// `mean` and `norm` of one tensor as five loops in one kernel (tests/reshape_reduction_test.py:5-21 after
// Compiler/Scope.cpp:165-188), each reading the row again. Fused, the row is read once and the loads that are the same
// word in several bodies are one load. Legal when the later loop and everything between the two can move up: pure
// nodes that do not read the first loop's accumulators.
bool SameValue(const Node* a, const Node* b) {
	if (a == b) return true;
	return a && b && std::string(a->op->name) == "const" && std::string(b->op->name) == "const" && !a->modified && !b->modified && a->type == b->type &&
	       a->data == b->data;
}

void FuseSiblingReductionLoops(Node* scope) {
	for (Node* c : scope->children)
		if (std::string(c->op->name) == "if") FuseSiblingReductionLoops(c);
	auto& list = scope->children;
	for (size_t i = 0; i < list.size(); i++) {
		Node* first = list[i];
		ReductionLoop r1;
		if (std::string(first->op->name) != "loop" || !MatchReductionLoop(first, r1)) continue;
		auto reads_first = [&](const Node* n) {
			for (auto& a : r1.accumulators)
				if (DependsOn(n, a.first)) return true;
			return DependsOn(n, first);
		};
		std::vector<Node*> between;
		size_t j = i + 1;
		while (j < list.size()) {
			Node* n = list[j];
			const std::string name = n->op->name;
			if (name == "loop") {
				ReductionLoop r2;
				bool ok = MatchReductionLoop(n, r2) && r2.strided == r1.strided && SameValue(first->inputs[0], n->inputs[0]) &&
				          SameValue(first->inputs[1], n->inputs[1]) && SameValue(first->inputs[2], n->inputs[2]);
				for (size_t k = 0; ok && k < n->children.size(); k++) {
					const Node* c = n->children[k];
					for (auto& a : r1.accumulators) ok &= !DependsOn(c, a.first) && c->memory != a.first;
				}
				if (!ok) break;
				// what stood between the loops goes in front of the first one, the second body behind the first body
				list.erase(list.begin() + (i + 1), list.begin() + (j + 1));
				list.insert(list.begin() + i, between.begin(), between.end());
				i += between.size();
				between.clear();
				for (Node* c : n->children) {
					for (Node*& in : c->inputs)
						if (in == n) in = first;
					if (c->index == n) c->index = first;
					c->parent = first;
					first->children.push_back(c);
				}
				first->use_count += n->use_count;
				n->children.clear();
				if (!MatchReductionLoop(first, r1)) return;  // cannot happen: both bodies matched and do not touch each other
				j = i + 1;
				continue;
			}
			if (!n->children.empty() || n->op->cls == OpClass::Memory || name == "set" || name == "if" || name == "break" || name == "continue" || name == "discard" ||
			    name == "group_barrier" || reads_first(n))
				break;
			between.push_back(n);
			j++;
		}
	}
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

// Hardware hands consecutive groups to the 8 accelerator dies (XCDs, each with its own L2) in turn. Giving
// die d the d-th contiguous eighth of the tiles instead keeps neighbouring tiles -- which share halo rows of
// stencils -- on one L2. The launch grid is a multiple of 8; tiles past the end are skipped by the caller.
const char* kXcdBand =
    "  const uint _chunk = gridDim.x / 8u;\n"
    "  const uint _hip_block = (blockIdx.x % 8u) * _chunk + blockIdx.x / 8u;\n";

}  // namespace

void GenerateHIPKernel(Program* program, Kernel* kernel) {
	(void)program;
	if (kernel->kernel_name_.empty()) kernel->kernel_name_ = "kernel_" + std::to_string(kernel->kernel_id_);
	const std::string kname = kernel->kernel_name_;

	std::vector<int> group = kernel->group_size;
	while (group.size() < 3) group.push_back(1);
	const int group_threads = group[0] * group[1] * group[2];
	if (group_threads < 1 || group_threads > 1024) throw std::runtime_error("group size of " + kname + " is outside 1..1024 threads");
	const bool uses_group = UsesGroupFeatures(kernel->root);

	// Reduction idiom: every loop of the kernel must be a matched reduction, none nested.
	std::vector<ReductionLoop> reductions;
	if (!uses_group && !kernel->verbatim) FuseSiblingReductionLoops(kernel->root);
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
		// a loop that lanes cannot share runs sliced among waves, which every other loop of the kernel must then allow too
		const bool any_strided = std::any_of(reductions.begin(), reductions.end(), [](const ReductionLoop& r) { return r.strided; });
		if (any_strided && !std::all_of(reductions.begin(), reductions.end(), Sliceable)) reductions.clear();
		kernel->wants_dense_variant = !kernel->serial_loops && !reductions.empty() &&
		                              (any_strided || (!std::all_of(reductions.begin(), reductions.end(), ReadsBroadcast) &&
		                                               std::all_of(reductions.begin(), reductions.end(), [&](const ReductionLoop& r) { return LoadsIgnoreInnermostIndex(r, kernel); })));
		if (kernel->serial_loops) reductions.clear();
	}

	// A kernel of a handful of threads (the total over a vector: shape [1]) whose loops the lanes of a wave can share is
	// better off with a wave per thread than with sixteen waves of which one lane each has a thread.
	bool few_threads = !kernel->shape_nodes.empty();
	{
		long threads = 1;
		for (const Node* extent : kernel->shape_nodes) {
			if (std::string(extent->op->name) != "const" || extent->modified) few_threads = false;
			else threads *= (long)(int)extent->data;
		}
		few_threads = few_threads && threads <= 16;
	}
	const bool any_strided_loop = std::any_of(reductions.begin(), reductions.end(), [](const ReductionLoop& r) { return r.strided; });

	// One sliced loop down the columns, nothing written before it, its trip count a polynomial in the host scalars: HIP
	// groups can then also share the loop slab by slab (few columns and many rows would otherwise leave most of the chip
	// idle: 4096 columns are 64 groups). The dispatch chooses the number of slabs.
	bool slabs = false;
	if (!uses_group && reductions.size() == 1 && reductions[0].strided && Sliceable(reductions[0]) && !(few_threads && !any_strided_loop)) {
		const Node* loop = reductions[0].loop;
		bool writes_before = false;
		std::function<bool(const Node*)> before = [&](const Node* scope) {  // false once the loop is reached
			for (const Node* c : scope->children) {
				if (c == loop) return false;
				const std::string n = c->op->name;
				if (c->op->cls == OpClass::Memory && n != "load") writes_before = true;
				if (n == "set") writes_before = true;
				if (!c->children.empty() && !before(c)) return false;
			}
			return true;
		};
		before(kernel->root);
		address_poly::Matcher m(kernel);
		auto lo = m.ToPoly(loop->inputs[0]), hi = m.ToPoly(loop->inputs[1]);
		if (!writes_before && lo && hi) {
			auto trips = m.ToDim(address_poly::Add(*hi, *lo, -1));
			if (trips) {
				slabs = true;
				kernel->slab_trips = *trips;
				kernel->slab_words_per_thread = (int)reductions[0].accumulators.size();
			}
		}
	}
	kernel->slabs = slabs;

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
	if (slabs) {
		kernel->var_names.push_back("_slabs");  // likewise: HIP groups that share one group of 64 threads
		kernel->var_types.push_back("uint");
	}

	std::string header = GetHIPHeader();
	header += "struct " + kname + "_vars {\n";
	for (size_t i = 0; i < kernel->var_names.size(); i++) header += "  " + kernel->var_types[i] + " " + kernel->var_names[i] + ";\n";
	header += "};\n\n";
	kernel->generated_header_ = header;

	// Buffer names are fixed before any body is generated.
	{
		std::unordered_map<std::string, int> seen;
		for (Node* mem : kernel->MemoryBindings()) {
			std::string n = mem->debug_name.empty() ? "m" : mem->debug_name;
			if (ForbiddenNames().count(n)) n += "0";
			if (seen[n]++) n += "_" + std::to_string(seen[n]);
			mem->var_name = n;
		}
	}
	// Every binding is its own allocation of the memory pool, so the pointers never alias; read-only ones
	// are const, which lets wave-uniform loads from them go through the scalar unit.
	std::string params, args;
	for (Node* mem : kernel->read_write_memory) {
		params += "uint* __restrict__ " + mem->var_name + "_mem, ";
		args += mem->var_name + "_mem, ";
	}
	for (Node* mem : kernel->read_only_memory) {
		params += "const uint* __restrict__ " + mem->var_name + "_mem, ";
		args += mem->var_name + "_mem, ";
	}
	if (slabs) params += "uint* __restrict__ _slab_partials, uint* __restrict__ _slab_tickets, ";  // bound by the kernel manager behind the tensors
	const std::string kernel_params = params + kname + "_vars var";
	kernel->generated_bindings_ = kernel_params;

	std::string main;
	const std::string body_indent = "    ";
	if (uses_group) {
		// Kernels with group memory / barriers run with exactly the thread-group the IR chose.
		HIPGenerator generator(kernel, 1);
		generator.Generate({});
		kernel->hip_threads = group_threads;
		kernel->groups_per_hip_block = 1;
		kernel->idiom = "group";
		main += "extern \"C\" __global__ __launch_bounds__(" + std::to_string(group_threads) + ") void " + kname + "(" + kernel_params + ")\n{\n";
		for (Node* gm : kernel->group_memory) main += "  __shared__ " + std::string(TypeName(gm->type)) + " " + gm->var_name + "[" + std::to_string(gm->data) + "];\n";
		main += "  const int block_id = (int)(blockIdx.x + var._kernel_block_offset);\n";
		main += "  const int block_thread_id0 = (int)threadIdx.x;\n  const int block_thread_id1 = (int)threadIdx.y;\n  const int block_thread_id2 = (int)threadIdx.z;\n";
		main += "  {\n" + generator.Assemble(body_indent) + "  }\n}\n";
	} else if (!reductions.empty() && std::all_of(reductions.begin(), reductions.end(), Sliceable) && !(few_threads && !any_strided_loop)) {
		// 64 logical threads per HIP group, one per lane; the group's waves each walk a slice of the loops.
		HIPGenerator generator(kernel, 1);
		generator.Generate(reductions, true, 64, slabs);
		size_t slots = 0;
		for (auto& r : reductions) slots = std::max(slots, r.accumulators.size());
		kernel->hip_threads = 64 * kSliceWaves;
		kernel->groups_per_hip_block = 0;  // grid = ceil(work_group_count * group_threads / 64)
		kernel->idiom = "reduction:block";
		main += "extern \"C\" __global__ __launch_bounds__(" + std::to_string(64 * kSliceWaves) + ") void " + kname + "(" + kernel_params + ")\n{\n";
		main += "  __shared__ uint _partials[" + std::to_string(slots * kSliceWaves * 64) + "];\n";
		main += "  const int _lane = (int)(threadIdx.x & 63u);\n";
		main += "  const int _wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));\n";
		if (slabs) {
			main += "  const uint _column_groups = gridDim.x / var._slabs;\n";
			main += "  const uint _column_group = blockIdx.x % _column_groups;\n";
			main += "  const uint _slab = blockIdx.x / _column_groups;\n";
			main += "  const long long _logical = (long long)_column_group * 64 + _lane;\n";
		} else {
			main += "  const long long _logical = (long long)blockIdx.x * 64 + _lane;\n";
		}
		main += "  const long long _total = (long long)var._work_group_count * " + std::to_string(group_threads) + ";\n";
		main += "  if (_logical < _total)\n  {\n";
		main += "    const int block_id = (int)(_logical / " + std::to_string(group_threads) + ") + (int)var._kernel_block_offset;\n";
		main += "    const int _local = (int)(_logical % " + std::to_string(group_threads) + ");\n";
		main += "    const int block_thread_id0 = _local % " + std::to_string(group[0]) + ";\n";
		main += "    const int block_thread_id1 = (_local / " + std::to_string(group[0]) + ") % " + std::to_string(group[1]) + ";\n";
		main += "    const int block_thread_id2 = _local / " + std::to_string(group[0] * group[1]) + ";\n";
		main += generator.Assemble(body_indent);
		main += "  }\n}\n";
	} else if (!reductions.empty()) {
		// One wavefront per logical thread (4 logical threads per 256-thread HIP group), or an aligned group of 8 / 16 /
		// 32 lanes per logical thread when every cooperative loop is short and of known length: about four loop steps
		// per lane, and the shuffle finish covers 64 / lanes logical threads at once.
		int lanes = 64;
		{
			long longest = 0;
			bool all_constant = true;
			for (auto& r : reductions) {
				const Node* b = r.loop->inputs[0];
				const Node* e = r.loop->inputs[1];
				if (std::string(b->op->name) == "const" && std::string(e->op->name) == "const" && !b->modified && !e->modified)
					longest = std::max(longest, (long)(int)e->data - (long)(int)b->data);
				else
					all_constant = false;
			}
			if (all_constant && longest > 0) {
				// Loops emitted in the four-step form keep four 16-byte loads per lane in flight: 16 steps per lane
				// (128 steps: 8 lanes). Loops that stay one word per step: 4 steps per lane (128 steps: 32 lanes).
				bool quads = true;
				for (auto& r : reductions) quads &= r.unit_stride || !r.index_clamps.empty();
				const long per_lane = quads ? 16 : 4;
				while (lanes > 8 && (long)lanes * per_lane / 2 >= longest) lanes /= 2;
			}
		}
		const int per_block = 256 / lanes;
		HIPGenerator generator(kernel, 1);
		generator.Generate(reductions, false, lanes);
		kernel->hip_threads = 256;
		kernel->groups_per_hip_block = 0;  // grid = ceil(work_group_count * group_threads / per_block)
		kernel->lanes_per_thread = lanes;
		kernel->idiom = "reduction:wave";
		main += "extern \"C\" __global__ __launch_bounds__(256) void " + kname + "(" + kernel_params + ")\n{\n";
		// Short loops leave a lane with little to do per logical thread: a group of lanes then works through several
		// logical threads one after the other (a wave that lives longer than one kilobyte of loads).
		const int serial = lanes < 64 ? kThreadsPerLaneGroup : 1;
		kernel->threads_per_lane_group = serial;
		main += "  const int _lane = (int)(threadIdx.x & " + std::to_string(lanes - 1) + "u);\n";
		main += "  const long long _total = (long long)var._work_group_count * " + std::to_string(group_threads) + ";\n";
		main += "  #pragma unroll\n";
		main += "  for (int _turn = 0; _turn < " + std::to_string(serial) + "; _turn++)\n  {\n";
		main += "  const long long _logical = ((long long)blockIdx.x * " + std::to_string(serial) + " + _turn) * " + std::to_string(per_block) + " + (long long)(threadIdx.x / " + std::to_string(lanes) + "u);\n";
		main += "  if (_logical < _total)\n  {\n";
		main += "    const int block_id = (int)(_logical / " + std::to_string(group_threads) + ") + (int)var._kernel_block_offset;\n";
		main += "    const int _local = (int)(_logical % " + std::to_string(group_threads) + ");\n";
		main += "    const int block_thread_id0 = _local % " + std::to_string(group[0]) + ";\n";
		main += "    const int block_thread_id1 = (_local / " + std::to_string(group[0]) + ") % " + std::to_string(group[1]) + ";\n";
		main += "    const int block_thread_id2 = _local / " + std::to_string(group[0] * group[1]) + ";\n";
		main += generator.Assemble(body_indent);
		main += "  }\n  }\n}\n";
	} else {
		// Single-thread body as a device function: used directly by the scalar mapping and as the edge path of
		// the four-wide mapping.
		HIPGenerator scalar(kernel, 1);
		scalar.Generate({});
		const std::string thread_fn = kname + "_thread";
		std::string thread_src = "static __device__ __forceinline__ void " + thread_fn + "(" + params + "const " + kname +
		                         "_vars& var, const int block_id, const int block_thread_id0, const int block_thread_id1, const int block_thread_id2)\n{\n" +
		                         scalar.Assemble("  ") + "}\n\n";
		const std::string call_prefix = thread_fn + "(" + args + "var, ";

		HIPGenerator vec(kernel, 4);
		std::string why;
		const bool vectorize = vec.Vectorizable(&why);
		main += thread_src;
		if (vectorize) {
			// Four-wide mapping: a 256-thread HIP group covers Q IR thread-groups side by side; each HIP thread
			// owns 4 consecutive values of the innermost index (one 16-byte access where memory is contiguous in
			// it), consecutive lanes own consecutive quads, and the group walks the remaining rows.
			const int rows = group[1] * group[2];
			const int lanes_x = rows >= 4 ? 64 : (rows == 2 ? 128 : 256);
			const int width = lanes_x * 4;
			int q = width / group[0];
			if (q < 1) q = 1;
			const int real_lanes_x = q * group[0] / 4;  // == lanes_x unless the IR group is wider than the tile
			const int rows_per_pass = 256 / real_lanes_x > 0 ? 256 / real_lanes_x : 1;
			const int passes = (rows + rows_per_pass - 1) / rows_per_pass;
			vec.SetScalarFallback(call_prefix);
			vec.Generate({});
			kernel->hip_threads = real_lanes_x * rows_per_pass;
			kernel->groups_per_hip_block = q;
			kernel->hip_blocks_per_tile = passes;
			kernel->idiom = "flat:vec4";
			// One quad per HIP thread: a tile of Q IR groups is cut into `passes` slabs of rows, each slab a HIP
			// group of its own, so that even small grids fill every compute unit with independent waves.
			// A thread that walks a loop of loads by itself hides memory latency by the loads it has in flight, not by
			// the number of waves: room for 128 registers.
			const std::string occupancy = vec.serial_load_loops() > 0 ? "__attribute__((amdgpu_waves_per_eu(2, 4))) " : "";
			kernel->serial_load_loops = vec.serial_load_loops() > 0;
			main += "extern \"C\" __global__ __launch_bounds__(" + std::to_string(kernel->hip_threads) + ") " + occupancy + "void " + kname + "(" + kernel_params + ")\n{\n";
			main += kXcdBand;
			main += "  const uint _tile = _hip_block / " + std::to_string(passes) + "u;\n";
			main += "  const int _r = (int)((_hip_block % " + std::to_string(passes) + "u) * " + std::to_string(rows_per_pass) + "u + threadIdx.x / " + std::to_string(real_lanes_x) + "u);\n";
			main += "  const int _x = (int)(threadIdx.x % " + std::to_string(real_lanes_x) + "u) * 4;\n";
			main += "  const uint _group = _tile * " + std::to_string(q) + "u + (uint)(_x / " + std::to_string(group[0]) + ");\n";
			main += "  if (_group >= var._work_group_count || _r >= " + std::to_string(rows) + ") return;\n";
			main += "  const int block_id = (int)(_group + var._kernel_block_offset);\n";
			main += "  const int block_thread_id0 = _x % " + std::to_string(group[0]) + ";\n";
			main += "  const int block_thread_id1 = _r % " + std::to_string(group[1]) + ";\n";
			main += "  const int block_thread_id2 = _r / " + std::to_string(group[1]) + ";\n";
			main += "  {\n";
			main += vec.Assemble(body_indent);
			main += "  }\n}\n";
		}
		{
			// Scalar mapping: a 256-thread HIP group covers Q consecutive IR thread-groups and walks their logical
			// threads so that the 64 lanes of a wave hold 64 consecutive values of the innermost index. It is the
			// only entry point of kernels that cannot be emitted four-wide, and a second one (suffix _s) of those
			// that can: dispatches too small to fill the chip with quads use it to get four times the waves.
			int q = 1;
			if (group[0] < 64) q = (64 + group[0] - 1) / group[0];
			const int logical = q * group_threads;
			const int threads = logical < 256 ? ((logical + 63) / 64) * 64 : 256;
			const int width = q * group[0];
			std::string entry = kname;
			if (vectorize) {
				entry = kname + "_s";
				kernel->scalar_entry = entry;
				kernel->scalar_hip_threads = threads;
				kernel->scalar_groups_per_hip_block = q;
			} else {
				kernel->hip_threads = threads;
				kernel->groups_per_hip_block = q;
				kernel->hip_blocks_per_tile = 1;
				kernel->idiom = "flat";
				main += "// not emitted four-wide: " + why + "\n";
			}
			main += "extern \"C\" __global__ __launch_bounds__(" + std::to_string(threads) + ") void " + entry + "(" + kernel_params + ")\n{\n";
			main += kXcdBand;
			main += "  for (int _l = (int)threadIdx.x; _l < " + std::to_string(logical) + "; _l += " + std::to_string(threads) + ")\n  {\n";
			main += "    const int _x = _l % " + std::to_string(width) + ";\n";
			main += "    const int _r = _l / " + std::to_string(width) + ";\n";
			main += "    const uint _group = _hip_block * " + std::to_string(q) + "u + (uint)(_x / " + std::to_string(group[0]) + ");\n";
			main += "    if (_group < var._work_group_count)\n";
			main += "      " + call_prefix + "(int)(_group + var._kernel_block_offset), _x % " + std::to_string(group[0]) + ", _r % " + std::to_string(group[1]) + ", _r / " +
			        std::to_string(group[1]) + ");\n";
			main += "  }\n}\n";

			// Third entry point (suffix _b): several small dispatches of this kernel in one launch. The kernel manager
			// gathers consecutive dispatches that touch disjoint buffers (the per-parameter updates of an optimizer, say);
			// blockIdx.y picks the dispatch, whose arguments sit in one element of the argument array, and the groups of
			// grid.x beyond that dispatch's own count leave at once. Same mapping as the entry point above.
			const size_t call_bytes = ((kernel->read_write_memory.size() + kernel->read_only_memory.size()) * 8 + kernel->var_names.size() * 4 + 4 + 7) / 8 * 8;
			const size_t capacity = std::min<size_t>(16, 3072 / call_bytes);
			const bool words_only = std::none_of(kernel->var_types.begin(), kernel->var_types.end(), [](const std::string& t) { return t == "bool"; });
			if (capacity >= 2 && words_only) {
				kernel->batch_entry = kname + "_b";
				kernel->batch_capacity = (int)capacity;
				kernel->batch_call_bytes = (int)call_bytes;
				main += "\nstruct " + kname + "_call {\n";
				std::string call_args;
				for (Node* mem : kernel->read_write_memory) {
					main += "  uint* " + mem->var_name + "_mem;\n";
					call_args += "_c." + mem->var_name + "_mem, ";
				}
				for (Node* mem : kernel->read_only_memory) {
					main += "  const uint* " + mem->var_name + "_mem;\n";
					call_args += "_c." + mem->var_name + "_mem, ";
				}
				main += "  " + kname + "_vars var;\n  uint _hip_blocks;\n};\n";
				main += "static_assert(sizeof(" + kname + "_call) == " + std::to_string(call_bytes) + ", \"argument layout\");\n";
				main += "struct " + kname + "_batch { " + kname + "_call call[" + std::to_string(capacity) + "]; };\n";
				main += "extern \"C\" __global__ __launch_bounds__(" + std::to_string(threads) + ") void " + kname + "_b(const " + kname + "_batch _batch)\n{\n";
				main += "  const " + kname + "_call& _c = _batch.call[blockIdx.y];\n";
				main += "  if (blockIdx.x >= _c._hip_blocks) return;\n";
				main += "  const uint _chunk = _c._hip_blocks / 8u;\n";
				main += "  const uint _hip_block = (blockIdx.x % 8u) * _chunk + blockIdx.x / 8u;\n";
				main += "  for (int _l = (int)threadIdx.x; _l < " + std::to_string(logical) + "; _l += " + std::to_string(threads) + ")\n  {\n";
				main += "    const int _x = _l % " + std::to_string(width) + ";\n";
				main += "    const int _r = _l / " + std::to_string(width) + ";\n";
				main += "    const uint _group = _hip_block * " + std::to_string(q) + "u + (uint)(_x / " + std::to_string(group[0]) + ");\n";
				main += "    if (_group < _c.var._work_group_count)\n";
				main += "      " + thread_fn + "(" + call_args + "_c.var, (int)(_group + _c.var._kernel_block_offset), _x % " + std::to_string(group[0]) + ", _r % " + std::to_string(group[1]) +
				        ", _r / " + std::to_string(group[1]) + ");\n";
				main += "  }\n}\n";
			}
		}
	}
	kernel->generated_main_ = main;
	kernel->full_generated_code_ = kernel->generated_header_ + main;
}

}  // namespace tfhost
