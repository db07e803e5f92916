// Whole-kernel idioms: kernels that consist of exactly one of the loops the reference's lowering passes
// leave behind for its algorithm ops --
//   dim_sum / dim_max / dim_min   acc = identity; loop k { acc = op(acc, load) }; store acc      (Compiler/Implementations.cpp:243-303)
//   dim_prefix_sum                acc = 0;        loop k { acc += load; store acc }               (:305-359)
//   matmul                        acc = 0;        loop k { acc += load A * load B }; store acc    (:560-646)
//                                 ... or store acc + bias[j], max(acc + bias[j], 0), mask[i,j] > 0 ? acc : 0: the element-wise
//                                 tail kernel fusion leaves behind the loop of a dense layer and of its input gradient
// The addresses of such a kernel are polynomials in the thread indices, the loop variable and the kernel's
// host scalars. The matcher extracts, for every operand, the coefficient of each index as a polynomial in the
// host scalars alone; at dispatch time those evaluate to the strides of the operand, and the kernel manager
// serves the dispatch with libtfhip's reduction / scan / sgemm primitive when they describe a dense row-major
// (or transposed) operand. Anything else -- fused extra arithmetic, offsets, batched forms -- stays with the
// emitted kernel.
#include <algorithm>
#include <map>
#include <optional>
#include <unordered_map>

#include "address_poly.h"
#include "hip_generator.h"

namespace tfhost {

namespace {

using namespace address_poly;

bool IsStatement(const Node* n) {
	const std::string op = n->op->name;
	if (op == "const") return n->modified;
	return op == "loop" || op == "if" || op == "set" || op == "group_barrier" || op == "local_memory" || op == "group_memory" ||
	       n->op->cls == OpClass::Memory || n->op->cls == OpClass::Keyword;
}

uint32_t Bits(float f) { return FloatBits(f); }

}  // namespace

static void MatchLoopIdiom(Kernel* kernel);
static void MatchSoftmaxPiece(Kernel* kernel);

void MatchKernelIdiom(Kernel* kernel) {
	MatchLoopIdiom(kernel);
	if (kernel->match.kind == IdiomMatch::None) MatchSoftmaxPiece(kernel);
}

static void MatchLoopIdiom(Kernel* kernel) {
	kernel->match = IdiomMatch();
	if (!kernel->dispatch_guard || !kernel->group_memory.empty() || kernel->index_nodes.size() != (size_t)kernel->dim) return;

	// Top level of the guarded body: one accumulator, one loop, then loads and stores (and the pure operations
	// between them, which are not statements).
	const Node* acc = nullptr;
	const Node* loop = nullptr;
	const Node* final_store = nullptr;
	std::vector<const Node*> tail_loads;  // operands of an element-wise tail fused behind the loop (bias, mask, ...)
	std::vector<const Node*> tail_stores;
	for (const Node* c : kernel->dispatch_guard->children) {
		if (!IsStatement(c)) continue;
		const std::string op = c->op->name;
		if (op == "const" && !acc && !loop) acc = c;
		else if (op == "loop" && acc && !loop) loop = c;
		else if (op == "load" && loop && !c->local_memory_op) tail_loads.push_back(c);
		else if (op == "store" && loop && !c->local_memory_op) tail_stores.push_back(c);
		else return;
	}
	if (tail_stores.size() == 1) final_store = tail_stores[0];
	// Several stores, or loads after the only store: only a matmul with a general tail can still match.
	bool general_tail = tail_stores.size() > 1;
	{
		bool after_store = false;
		for (const Node* c : kernel->dispatch_guard->children) {
			if (c == final_store) after_store = true;
			else if (after_store && IsStatement(c)) general_tail = true;
		}
	}
	if (!acc || !loop) return;
	const Node* step = loop->inputs[2];
	if (std::string(step->op->name) != "const" || (int)step->data != 1) return;

	// Loop body: loads, one update of the accumulator, for a scan one store of it after the update.
	std::vector<const Node*> loads;
	const Node* update = nullptr;
	const Node* inner_store = nullptr;
	for (const Node* c : loop->children) {
		if (!IsStatement(c)) continue;
		const std::string op = c->op->name;
		if (op == "load" && !c->local_memory_op && !update) loads.push_back(c);
		else if (op == "set" && c->memory == acc && !update) update = c;
		else if (op == "store" && update && !inner_store && !c->local_memory_op) inner_store = c;
		else return;
	}
	if (!update || loads.empty() || loads.size() > 2) return;
	if (inner_store ? !tail_stores.empty() : tail_stores.empty()) return;
	const Node* store = inner_store ? inner_store : tail_stores[0];
	if (store->inputs.size() != 1) return;
	// What is stored: the accumulator itself, or (matmul only) one of the fused tails
	//   acc + bias[j]        max(acc + bias[j], 0)        mask[i, j] > 0 ? acc : 0
	const Node* tail_load = nullptr;
	std::string tail;
	if (!general_tail && !inner_store) {
		auto is_zero = [](const Node* n) { return std::string(n->op->name) == "const" && !n->modified && n->type == TFType_Float && n->data == 0; };
		auto other = [](const Node* n, const Node* x) -> const Node* {
			if (n->inputs.size() != 2) return nullptr;
			return n->inputs[0] == x ? n->inputs[1] : n->inputs[1] == x ? n->inputs[0] : nullptr;
		};
		const Node* v = store->inputs[0];
		const std::string vop = v->op->name;
		if (v == acc) {
		} else if (vop == "add" && other(v, acc) && std::string(other(v, acc)->op->name) == "load") {
			tail = "bias";
			tail_load = other(v, acc);
		} else if (vop == "max" && v->inputs.size() == 2 && (is_zero(v->inputs[0]) || is_zero(v->inputs[1]))) {
			const Node* sum = is_zero(v->inputs[0]) ? v->inputs[1] : v->inputs[0];
			if (std::string(sum->op->name) == "add" && other(sum, acc) && std::string(other(sum, acc)->op->name) == "load") {
				tail = "bias_relu";
				tail_load = other(sum, acc);
			} else {
				general_tail = true;
			}
		} else if (vop == "ternary" && v->inputs.size() == 3 && v->inputs[1] == acc && is_zero(v->inputs[2])) {
			const Node* cond = v->inputs[0];
			if (std::string(cond->op->name) == "gt" && cond->inputs.size() == 2 && std::string(cond->inputs[0]->op->name) == "load" && is_zero(cond->inputs[1])) {
				tail = "mask_positive";
				tail_load = cond->inputs[0];
			} else {
				general_tail = true;
			}
		} else {
			general_tail = true;
		}
		if (!general_tail && (tail_load ? (tail_loads.size() != 1 || tail_loads[0] != tail_load || tail_load->type != TFType_Float) : !tail_loads.empty())) general_tail = true;
		if (general_tail) {
			tail.clear();
			tail_load = nullptr;
		}
	}
	const Node* combine = update->inputs[0];
	if (combine->inputs.size() != 2) return;
	const Node* value = combine->inputs[0] == acc ? combine->inputs[1] : combine->inputs[1] == acc ? combine->inputs[0] : nullptr;
	if (!value) return;
	const std::string cop = combine->op->name;
	Matcher m(kernel);
	m.loop = loop;
	// load wrapped in the reference's out-of-bounds select: ternary(out_of_bounds, constant, load)
	if (std::string(value->op->name) == "ternary" && value->inputs.size() == 3 && loads.size() == 1 && value->inputs[2] == loads[0] &&
	    std::string(value->inputs[1]->op->name) == "const" && m.NeverTrue(value->inputs[0]))
		value = loads[0];
	for (const Node* l : loads) {
		if (l->memory == store->memory) return;  // in place: the primitives assume distinct operands
		for (const Node* st : tail_stores)
			if (l->memory == st->memory) return;
	}

	IdiomMatch match;
	match.type = acc->type;
	match.is_float = acc->type == TFType_Float;
	match.is_float = acc->type == TFType_Float;
	auto K = m.Extent(loop);
	if (!K) return;
	auto dim = [&](const std::optional<Poly>& p) -> bool {
		if (!p) return false;
		auto d = m.ToDim(*p);
		if (!d) return false;
		match.dims.push_back(*d);
		return true;
	};
	auto address = [&](const Node* mem_op) -> std::optional<Poly> {
		if (!mem_op->index) return Constant(0);
		auto p = m.ToPoly(mem_op->index);
		if (!p || !m.Offset(*p).t.empty()) return std::nullopt;
		return p;
	};

	if (loads.size() == 1 && value == loads[0] && (kernel->dim == 1 || kernel->dim == 2) && !tail_load && !general_tail) {
		const Node* t = kernel->index_nodes[0];
		auto in = address(loads[0]), out = address(store);
		auto T = m.Extent(t);
		if (!in || !out || !T) return;
		if (final_store) {
			if (acc->type != TFType_Float) return;
			if (cop == "add" && acc->data == Bits(0.0f)) match.op = "sum";
			else if (cop == "max" && acc->data == Bits(-3.402823466e+38f)) match.op = "max";
			else if (cop == "min" && acc->data == Bits(3.402823466e+38f)) match.op = "min";
			else return;
			match.kind = IdiomMatch::Reduce;
			auto out_k = m.Coefficient(*out, loop);
			if (!out_k || !out_k->t.empty()) return;
			if (!dim(T) || !dim(K) || !dim(m.Coefficient(*in, t)) || !dim(m.Coefficient(*in, loop)) || !dim(m.Coefficient(*out, t))) return;
			if (kernel->dim == 2) {  // second (outer) thread index: its extent and strides
				const Node* t1 = kernel->index_nodes[1];
				if (!dim(m.Extent(t1)) || !dim(m.Coefficient(*in, t1)) || !dim(m.Coefficient(*out, t1))) return;
			}
		} else {
			if (cop != "add" || acc->data != 0) return;  // +0.0f and integer 0 share the all-zero word
			match.kind = IdiomMatch::Scan;
			if (!dim(T) || !dim(K) || !dim(m.Coefficient(*in, t)) || !dim(m.Coefficient(*in, loop)) || !dim(m.Coefficient(*out, t)) ||
			    !dim(m.Coefficient(*out, loop)))
				return;
			if (kernel->dim == 2) {  // second (outer) thread index: a batch of scans
				const Node* t1 = kernel->index_nodes[1];
				if (!dim(m.Extent(t1)) || !dim(m.Coefficient(*in, t1)) || !dim(m.Coefficient(*out, t1))) return;
			}
		}
		match.buffers = {m.BindingOf(store->memory), m.BindingOf(loads[0]->memory)};
	} else if (loads.size() == 2 && !inner_store && (kernel->dim == 2 || (kernel->dim == 3 && !general_tail && !tail_load)) && acc->type == TFType_Float &&
	           cop == "add" && acc->data == Bits(0.0f)) {
		if (std::string(value->op->name) != "mul" || value->inputs.size() != 2) return;
		if (!((value->inputs[0] == loads[0] && value->inputs[1] == loads[1]) || (value->inputs[0] == loads[1] && value->inputs[1] == loads[0]))) return;
		const Node* j = kernel->index_nodes[0];
		const Node* i = kernel->index_nodes[1];
		auto p0 = address(loads[0]), p1 = address(loads[1]);
		std::optional<Poly> pc = general_tail ? std::optional<Poly>(Constant(0)) : address(store);
		if (!p0 || !p1 || !pc) return;
		auto zero = [&](const Poly& p, const Node* leaf) {
			auto c = m.Coefficient(p, leaf);
			return c && c->t.empty();
		};
		const Node* A = loads[0];
		const Node* B = loads[1];
		if (zero(*p0, j) && zero(*p1, i)) {
		} else if (zero(*p1, j) && zero(*p0, i)) {
			std::swap(A, B);
			std::swap(p0, p1);
		} else {
			return;
		}
		if (general_tail) {
			// Any element-wise tail: the product goes to a temporary laid out [M, N] and the kernel without its loop
			// (built by MakeMatmulTailKernel) reads it back, so the addresses of the tail's own loads and stores are free.
			match.kind = IdiomMatch::Matmul;
			match.op = "tail";
			match.accumulator = acc;
			match.loop = loop;
			if (!dim(m.Extent(j)) || !dim(m.Extent(i)) || !dim(K) || !dim(m.Coefficient(*p0, i)) || !dim(m.Coefficient(*p0, loop)) ||
			    !dim(m.Coefficient(*p1, loop)) || !dim(m.Coefficient(*p1, j)))
				return;
			match.buffers = {-1, m.BindingOf(A->memory), m.BindingOf(B->memory)};
			if (match.buffers[1] < 0 || match.buffers[2] < 0) return;
			match.buffers[0] = 0;
			for (auto& c : m.conditions) {
				auto lhs = m.ToDim(c.first), rhs = m.ToDim(c.second);
				if (!lhs || !rhs) return;
				match.conditions.push_back({*lhs, *rhs});
			}
			kernel->match = match;
			return;
		}
		if (!zero(*pc, loop)) return;
		if (tail_load) {
			// bias: one word per column; mask: laid out like C
			if (tail_load->memory == store->memory) return;
			auto pt = address(tail_load);
			if (!pt) return;
			auto ti = m.Coefficient(*pt, i), tj = m.Coefficient(*pt, j), ci = m.Coefficient(*pc, i), cj = m.Coefficient(*pc, j);
			if (!ti || !tj || !ci || !cj) return;
			if (tail == "mask_positive" ? !(*ti == *ci && *tj == *cj) : !(ti->t.empty() && *tj == Constant(1))) return;
			match.op = tail;
		}
		match.kind = IdiomMatch::Matmul;
		if (!dim(m.Extent(j)) || !dim(m.Extent(i)) || !dim(K) || !dim(m.Coefficient(*p0, i)) || !dim(m.Coefficient(*p0, loop)) ||
		    !dim(m.Coefficient(*p1, loop)) || !dim(m.Coefficient(*p1, j)) || !dim(m.Coefficient(*pc, i)) || !dim(m.Coefficient(*pc, j)))
			return;
		if (kernel->dim == 3) {
			// a leading batch index (Implementations.cpp:575-633 appends it to the indices of A, B and C; an operand with
			// fewer dimensions is shared): extent, then the strides of A, B and C along it
			const Node* t = kernel->index_nodes[2];
			if (!dim(m.Extent(t)) || !dim(m.Coefficient(*p0, t)) || !dim(m.Coefficient(*p1, t)) || !dim(m.Coefficient(*pc, t))) return;
		}
		match.buffers = {m.BindingOf(store->memory), m.BindingOf(A->memory), m.BindingOf(B->memory)};
		if (tail_load) match.buffers.push_back(m.BindingOf(tail_load->memory));
	} else {
		return;
	}
	for (int b : match.buffers)
		if (b < 0) return;
	for (auto& c : m.conditions) {
		auto lhs = m.ToDim(c.first), rhs = m.ToDim(c.second);
		if (!lhs || !rhs) return;
		match.conditions.push_back({*lhs, *rhs});
	}
	kernel->match = match;
}

// The two kernels of a lowered row softmax that are not plain reductions (tests/autograd_test.py:29-31 composes
// m = max(x), e = exp(x - m), y = e / sum(e); kernel fusion puts exp(x - m) into the loop of the sum and into the
// last element-wise kernel):
//   ExpSum      acc = 0; loop k { acc += exp(load X - load M) }; store acc     (M addressed by the row alone; in the
//               split form of Optimization.cpp:469-510 the padding select wraps the load or the whole term)
//   Normalise   store Y[r, c] = exp(load X[r, c] - load M[r]) / load Z[r], or (op "log") (load X - load M) - log(load Z)
// Neither is served on its own. The kernel manager follows a program's dispatches and, when max -> ExpSum -> sum ->
// Normalise arrive in that order on the same tensors, runs the fused softmax primitive in their place.
static void MatchSoftmaxPiece(Kernel* kernel) {
	if (!kernel->dispatch_guard || !kernel->group_memory.empty() || kernel->index_nodes.size() != (size_t)kernel->dim) return;
	if (kernel->dim != 1 && kernel->dim != 2) return;
	const Node* acc = nullptr;
	const Node* loop = nullptr;
	const Node* store = nullptr;
	std::vector<const Node*> loads;
	for (const Node* c : kernel->dispatch_guard->children) {
		if (!IsStatement(c)) continue;
		const std::string op = c->op->name;
		if (op == "load" && !c->local_memory_op && !store) loads.push_back(c);
		else if (op == "const" && !acc && !loop && !store) acc = c;
		else if (op == "loop" && acc && !loop && !store) loop = c;
		else if (op == "store" && !store && !c->local_memory_op) store = c;
		else return;
	}
	if (!store || store->inputs.size() != 1 || (acc != nullptr) != (loop != nullptr)) return;
	auto is = [](const Node* n, const char* name, size_t inputs) { return n && std::string(n->op->name) == name && n->inputs.size() == inputs && !n->modified; };
	auto is_load = [](const Node* n) { return n && std::string(n->op->name) == "load" && !n->local_memory_op; };
	Matcher m(kernel);
	m.loop = loop;
	IdiomMatch match;
	auto dim = [&](const std::optional<Poly>& p) -> bool {
		if (!p) return false;
		auto d = m.ToDim(*p);
		if (!d) return false;
		match.dims.push_back(*d);
		return true;
	};
	auto address = [&](const Node* mem_op) -> std::optional<Poly> {
		if (!mem_op->index) return Constant(0);
		auto p = m.ToPoly(mem_op->index);
		if (!p || !m.Offset(*p).t.empty()) return std::nullopt;
		return p;
	};
	// exp(load X - load M), the loads possibly behind a padding select that never pads
	const Node* LX = nullptr;
	const Node* LM = nullptr;
	auto strip = [&](const Node* v) -> const Node* {
		if (is(v, "ternary", 3) && std::string(v->inputs[1]->op->name) == "const" && m.NeverTrue(v->inputs[0])) return v->inputs[2];
		return v;
	};
	auto exp_of_difference = [&](const Node* e) -> bool {
		e = strip(e);
		if (!is(e, "exp", 1) || !is(e->inputs[0], "sub", 2)) return false;
		LX = strip(e->inputs[0]->inputs[0]);
		LM = e->inputs[0]->inputs[1];
		return is_load(LX) && is_load(LM) && LX->type == TFType_Float && LM->type == TFType_Float && LX->memory != LM->memory;
	};
	if (!loop && kernel->dim == 2 && loads.size() == 2) {
		// the softmax with e = exp(x - m) as a tensor of its own: E[r, c] = exp(X[r, c] - m[r]), and later Y[r, c] = E[r, c] / z[r]
		const Node* v = store->inputs[0];
		const Node *first = nullptr, *second = nullptr;
		if (exp_of_difference(v)) {
			match.kind = IdiomMatch::ExpDiff;
			first = LX, second = LM;
		} else if (is(v, "div", 2) && is_load(v->inputs[0]) && is_load(v->inputs[1]) && v->inputs[0]->type == TFType_Float && v->inputs[1]->type == TFType_Float) {
			match.kind = IdiomMatch::DivideRows;
			first = v->inputs[0], second = v->inputs[1];
		} else {
			return;
		}
		for (const Node* l : {first, second})
			if (std::find(loads.begin(), loads.end(), l) == loads.end() || l->memory == store->memory) return;
		if (first->memory == second->memory) return;
		const Node* c = kernel->index_nodes[0];
		const Node* r = kernel->index_nodes[1];
		if (!dim(m.Extent(c)) || !dim(m.Extent(r))) return;
		for (const Node* op : {first, store, second}) {
			auto p = address(op);
			if (!p || !dim(m.Coefficient(*p, c)) || !dim(m.Coefficient(*p, r))) return;
		}
		match.buffers = {m.BindingOf(store->memory), m.BindingOf(first->memory), m.BindingOf(second->memory)};
	} else if (!loop) {
		if (kernel->dim != 2 || loads.size() != 3) return;
		const Node* v = store->inputs[0];
		const Node* LZ = nullptr;
		if (is(v, "div", 2) && exp_of_difference(v->inputs[0])) {
			LZ = v->inputs[1];  // exp(x - m) / z
		} else if (is(v, "sub", 2) && is(v->inputs[0], "sub", 2) && is(v->inputs[1], "log", 1)) {
			// (x - m) - log(z): the last kernel of a log-softmax (tests/autograd_test.py:29-31)
			LX = v->inputs[0]->inputs[0];
			LM = v->inputs[0]->inputs[1];
			LZ = v->inputs[1]->inputs[0];
			if (!is_load(LX) || !is_load(LM) || LX->type != TFType_Float || LM->type != TFType_Float || LX->memory == LM->memory) return;
			match.op = "log";
		} else {
			return;
		}
		if (!is_load(LZ) || LZ->type != TFType_Float) return;
		for (const Node* l : {LX, LM, LZ})
			if (std::find(loads.begin(), loads.end(), l) == loads.end() || l->memory == store->memory) return;
		if (LZ->memory == LX->memory || LZ->memory == LM->memory) return;
		const Node* c = kernel->index_nodes[0];
		const Node* r = kernel->index_nodes[1];
		match.kind = IdiomMatch::Normalise;
		if (!dim(m.Extent(c)) || !dim(m.Extent(r))) return;
		for (const Node* op : {LX, store, LM, LZ}) {
			auto p = address(op);
			if (!p || !dim(m.Coefficient(*p, c)) || !dim(m.Coefficient(*p, r))) return;
		}
		match.buffers = {m.BindingOf(store->memory), m.BindingOf(LX->memory), m.BindingOf(LM->memory), m.BindingOf(LZ->memory)};
	} else {
		if (acc->type != TFType_Float || acc->data != Bits(0.0f)) return;
		const Node* step = loop->inputs[2];
		if (std::string(step->op->name) != "const" || (int)step->data != 1) return;
		const Node* update = nullptr;
		for (const Node* c : loop->children) {
			if (!IsStatement(c)) continue;
			const std::string op = c->op->name;
			if (op == "load" && !c->local_memory_op && !update) loads.push_back(c);
			else if (op == "set" && c->memory == acc && !update) update = c;
			else return;
		}
		if (!update || loads.size() != 2 || store->inputs[0] != acc) return;
		const Node* combine = update->inputs[0];
		if (!is(combine, "add", 2)) return;
		const Node* value = combine->inputs[0] == acc ? combine->inputs[1] : combine->inputs[1] == acc ? combine->inputs[0] : nullptr;
		if (!value || !exp_of_difference(value)) return;
		for (const Node* l : {LX, LM})
			if (std::find(loads.begin(), loads.end(), l) == loads.end() || l->memory == store->memory) return;
		const Node* t = kernel->index_nodes[0];
		auto in = address(LX), out = address(store), mx = address(LM);
		auto T = m.Extent(t), K = m.Extent(loop);
		if (!in || !out || !mx || !T || !K) return;
		auto out_k = m.Coefficient(*out, loop);
		if (!out_k || !out_k->t.empty()) return;
		match.kind = IdiomMatch::ExpSum;
		// as a reduction: T, K, input per thread / per step, output per thread, [outer extent, input, output per outer index];
		// then the maxima's strides per thread, per step [, per outer index]
		if (!dim(T) || !dim(K) || !dim(m.Coefficient(*in, t)) || !dim(m.Coefficient(*in, loop)) || !dim(m.Coefficient(*out, t))) return;
		if (kernel->dim == 2) {
			const Node* t1 = kernel->index_nodes[1];
			if (!dim(m.Extent(t1)) || !dim(m.Coefficient(*in, t1)) || !dim(m.Coefficient(*out, t1))) return;
		}
		if (!dim(m.Coefficient(*mx, t)) || !dim(m.Coefficient(*mx, loop))) return;
		if (kernel->dim == 2 && !dim(m.Coefficient(*mx, kernel->index_nodes[1]))) return;
		match.buffers = {m.BindingOf(store->memory), m.BindingOf(LX->memory), m.BindingOf(LM->memory)};
	}
	for (int b : match.buffers)
		if (b < 0) return;
	for (auto& c : m.conditions) {
		auto lhs = m.ToDim(c.first), rhs = m.ToDim(c.second);
		if (!lhs || !rhs) return;
		match.conditions.push_back({*lhs, *rhs});
	}
	kernel->match = match;
}

}  // namespace tfhost
