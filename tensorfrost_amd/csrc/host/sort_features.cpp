// What a kernel does, in the terms a `Radix sort` region is followed by (shim/hip_sort_region.cpp).
//
// tf.sort.radix (Python/TensorFrost/sort.py:38-187) reaches the backend as whatever kernels the compiler's passes cut
// it into: which element-wise operations share a kernel is decided by KernelScope (Compiler/Graph/Scope.cpp:5-35,
// 165-188: adjacent operations of exactly the same shape merge unless one loads or stores what the other produces),
// values computed element-wise may be copied into the kernels that load them, host scalars reach a kernel as whatever
// expression of the loop variable the host evaluated. None of that changes what the region computes. So instead of
// comparing whole kernels with templates, this file looks in a kernel's tree for the three things the region's
// result depends on, each found by what it computes, not by how its tree is spelled:
//
//   * element-wise copies  dst[i] = f(src[i])  where f, EVALUATED on probe words, is the identity or one of the
//     order-preserving key maps (sort.py:52-72) -- the prologue `keys = tf.copy(keys)`, `values = tf.copy(values)`,
//     alone, fused into one kernel, or fused with the map (:78-87);
//   * digit extraction  (load(keys, ...) >> shift) & mask  with shift a polynomial of the kernel's host scalars
//     (GetBits, :93-94), wherever it ended up;
//   * the scatter of a pass (:133-169): the one kernel written as an explicit `tf.kernel` block, so its body is one
//     kernel under any partitioning: group memory + barriers, and as its only global effects
//     keys_out[d] = keys_in[e], values_out[d] = values_in[e] behind `e < n`, e the thread's own element.
#include <cstring>
#include <unordered_set>

#include "address_poly.h"
#include "host_program.h"
#include "sort_composition.h"

namespace tfhost {

namespace {

using namespace address_poly;
using tfhip::SortFeatures;

bool Is(const Node* n, const char* op) { return n && std::strcmp(n->op->name, op) == 0; }
bool IsInteger(const Node* n) { return n->type == TFType_Int || n->type == TFType_Uint; }

// The value behind bit copies and conversions between the two 32-bit integer types.
const Node* StripCasts(const Node* n) {
	for (int depth = 0; n && depth < 16; depth++) {
		if ((Is(n, "asuint") || Is(n, "asint") || Is(n, "asfloat") || Is(n, "copy")) && n->inputs.size() == 1 && n->inputs[0]->type != TFType_Bool)
			n = n->inputs[0];
		else if ((Is(n, "uint") || Is(n, "int")) && n->inputs.size() == 1 && IsInteger(n->inputs[0]))
			n = n->inputs[0];
		else
			break;
	}
	return n;
}

// Where a scattered store lands, behind the conversions and the clamp that address finalisation wraps around a
// user-given index (Compiler/Steps/GraphOps.cpp:989-1043): two stores land on the same element when this is the same node.
const Node* TargetRoot(const Node* n) {
	for (int depth = 0; n && depth < 8; depth++) {
		const Node* inner = StripCasts(n);
		if (Is(inner, "clamp") && inner->inputs.size() == 3) inner = inner->inputs[0];
		if (inner == n) break;
		n = inner;
	}
	return n;
}

bool IsGlobalLoad(const Node* n) { return Is(n, "load") && !n->local_memory_op && n->memory && Is(n->memory, "memory"); }

void Walk(const Node* n, const std::function<void(const Node*)>& visit) {
	visit(n);
	for (const Node* c : n->children) Walk(c, visit);
}

// The global loads a value is computed from.
void LoadsOf(const Node* n, std::unordered_set<const Node*>& loads, std::unordered_set<const Node*>& seen, bool& opaque, int depth = 0) {
	if (!n || !seen.insert(n).second) return;
	if (depth > 64 || n->modified) {
		opaque = true;
		return;
	}
	if (Is(n, "load")) {
		if (IsGlobalLoad(n))
			loads.insert(n);
		else
			opaque = true;
		return;
	}
	if (n->op->cls == OpClass::Memory || n->op->cls == OpClass::Special) {
		if (!Is(n, "variable")) opaque = true;
		return;
	}
	for (const Node* in : n->inputs) LoadsOf(in, loads, seen, opaque, depth + 1);
}

// The value as a function of the word `probe` loads: true and *out on success; false when anything else than
// constants and operations on words takes part.
bool Evaluate(const Node* n, const Node* probe, uint32_t x, uint32_t* out, int depth = 0) {
	if (!n || depth > 48) return false;
	if (n == probe) {
		*out = x;
		return true;
	}
	if (n->modified) return false;
	if (Is(n, "const")) {
		*out = n->data;
		return true;
	}
	if (n->inputs.empty() || n->inputs.size() > 3 || n->op->cls == OpClass::Memory || n->op->cls == OpClass::Special) return false;
	uint32_t arg[3] = {0, 0, 0};
	for (size_t i = 0; i < n->inputs.size(); i++)
		if (!Evaluate(n->inputs[i], probe, x, &arg[i], depth + 1)) return false;
	ScalarFn fn = FindScalarFn(n->op->name, n->inputs[0]->type, n->type);
	if (!fn) return false;
	try {
		*out = fn(arg[0], arg[1], arg[2]);
	} catch (...) {
		return false;
	}
	return true;
}

uint32_t MapWord(int map, uint32_t x) {
	const uint32_t sign = 0x80000000u;
	switch (map) {
		case 0: return x;
		case 1: return x ^ ((x >> 31) == 1u ? 0xFFFFFFFFu : sign);  // map_float_to_uint
		case 2: return x ^ sign;                                    // map_int_to_uint = map_uint_to_int
		default: return x ^ ((x >> 31) == 0u ? 0xFFFFFFFFu : sign); // map_uint_to_float
	}
}

// Which of the maps the value is, as a function of the loaded word; -1 for any other function.
int MapOf(const Node* value, const Node* load) {
	static const std::vector<uint32_t> probes = [] {
		std::vector<uint32_t> p = {0u, 1u, 2u, 0x7FFFFFFFu, 0x80000000u, 0x80000001u, 0xFFFFFFFFu, 0xFFFFFFFEu, 0x3F800000u, 0xBF800000u, 0x7F800000u, 0xFF800000u,
		                           0x00000001u, 0x80000000u, 0x7FC00000u, 0x00800000u, 0x80800000u, 0x55555555u, 0xAAAAAAAAu};
		uint32_t s = 0x9E3779B9u;
		for (int i = 0; i < 256; i++) {
			s = s * 747796405u + 2891336453u;
			p.push_back(((s >> ((s >> 28u) + 4u)) ^ s) * 277803737u);
		}
		return p;
	}();
	int candidates = 0xF;
	for (uint32_t x : probes) {
		uint32_t y;
		if (!Evaluate(value, load, x, &y)) return -1;
		for (int m = 0; m < 4; m++)
			if (MapWord(m, x) != y) candidates &= ~(1 << m);
		if (!candidates) return -1;
	}
	for (int m = 0; m < 4; m++)
		if (candidates & (1 << m)) return m;
	return -1;
}

struct Analysis {
	const Kernel* kernel;
	Matcher m;
	std::vector<const Node*> global_stores, global_atomics, barriers, digit_nodes;
	bool has_group_memory = false;

	explicit Analysis(const Kernel* k) : kernel(k), m(k) {
		Walk(k->root, [&](const Node* n) {
			if (Is(n, "store") && !n->local_memory_op) global_stores.push_back(n);
			if (n->op->cls == OpClass::Memory && !Is(n, "load") && !Is(n, "store") && !n->local_memory_op) global_atomics.push_back(n);
			if (Is(n, "group_barrier")) barriers.push_back(n);
			if (Is(n, "group_memory")) has_group_memory = true;
			if (Is(n, "and") && n->inputs.size() == 2 && n->type != TFType_Bool) digit_nodes.push_back(n);
		});
	}

	// The flat element a thread stands for: index_0 in a one-dimensional kernel, index_1 * extent_0 + index_0 in a
	// two-dimensional one whose inner extent is a constant (the scatter's [groups, 128]).
	std::optional<Poly> Element() {
		if (kernel->index_nodes.empty() || kernel->index_nodes.size() != (size_t)kernel->dim) return std::nullopt;
		if (kernel->dim == 1) return Leaf(kernel->index_nodes[0]);
		if (kernel->dim == 2) {
			auto inner = m.ToPoly(kernel->shape_nodes[0]);
			if (!inner || inner->t.size() != 1 || !inner->t.begin()->first.empty()) return std::nullopt;  // a constant
			return Add(Leaf(kernel->index_nodes[0]), Mul(Leaf(kernel->index_nodes[1]), *inner), 1);
		}
		return std::nullopt;
	}

	bool AddressIs(const Node* address, const Poly& want) {
		if (!address) return false;
		auto p = m.ToPoly(address);
		return p && *p == want;
	}

	// (load >> shift) & mask in either operand order, mask = 2^b - 1.
	bool AsDigit(const Node* n, const Node** load, DimExpr* shift, uint32_t* mask) {
		n = StripCasts(n);
		if (!Is(n, "and") || n->inputs.size() != 2) return false;
		for (int side = 0; side < 2; side++) {
			const Node* c = StripCasts(n->inputs[side]);
			const Node* shifted = StripCasts(n->inputs[1 - side]);
			if (!Is(c, "const") || c->modified || !IsInteger(c)) continue;
			const uint32_t msk = c->data;
			if (msk == 0 || (msk & (msk + 1u)) != 0) continue;
			const Node* word = shifted;
			Poly amount = Constant(0);
			if (Is(shifted, "rshift") && shifted->inputs.size() == 2) {
				word = StripCasts(shifted->inputs[0]);
				auto s = m.ToPoly(StripCasts(shifted->inputs[1]));
				if (!s) continue;
				amount = *s;
			}
			if (!IsGlobalLoad(word)) continue;
			auto dim = m.ToDim(amount);  // fails when the amount moves with a thread index
			if (!dim) continue;
			*load = word;
			*shift = *dim;
			*mask = msk;
			return true;
		}
		return false;
	}
};

}  // namespace

void AnalyzeSortFeatures(Kernel* kernel) {
	kernel->sort = SortFeatures();
	if (!kernel->root || !kernel->primitive.empty() || !kernel->dispatch_guard) return;
	Analysis a(kernel);
	SortFeatures f;

	for (const Node* n : a.digit_nodes) {
		const Node* load = nullptr;
		SortFeatures::Digit d;
		if (!a.AsDigit(n, &load, &d.shift, &d.mask)) continue;
		d.keys = a.m.BindingOf(load->memory);
		if (d.keys >= 0) f.digits.push_back(d);
	}

	auto element = a.Element();

	// Element-wise copies: one-dimensional kernels whose stores all write the thread's own element.
	if (element && kernel->dim == 1 && !a.global_stores.empty() && a.global_atomics.empty() && a.barriers.empty() && !a.has_group_memory) {
		auto extent = a.m.Extent(kernel->index_nodes[0]);
		auto extent_dim = extent ? a.m.ToDim(*extent) : std::nullopt;
		bool all = (bool)extent_dim;
		for (const Node* store : a.global_stores) {
			if (!all) break;
			all = false;
			if (store->parent != kernel->dispatch_guard || !a.AddressIs(store->index, *element) || store->inputs.size() != 1) break;
			std::unordered_set<const Node*> loads, seen;
			bool opaque = false;
			LoadsOf(store->inputs[0], loads, seen, opaque);
			if (opaque || loads.size() != 1) break;
			const Node* load = *loads.begin();
			if (!a.AddressIs(load->index, *element)) break;
			SortFeatures::Copy c;
			c.map = MapOf(store->inputs[0], load);
			c.dst = a.m.BindingOf(store->memory);
			c.src = a.m.BindingOf(load->memory);
			c.extent = *extent_dim;
			if (c.map < 0 || c.dst < 0 || c.src < 0 || c.dst == c.src) break;
			f.copies.push_back(c);
			all = true;
		}
		// a buffer written twice, or written and read, is no plain copy
		for (size_t i = 0; all && i < f.copies.size(); i++)
			for (size_t j = 0; j < f.copies.size(); j++)
				if ((i != j && f.copies[i].dst == f.copies[j].dst) || f.copies[i].dst == f.copies[j].src) all = false;
		if (!a.m.conditions.empty()) all = false;  // an address that is the element only for some dispatches
		f.copies_only = all;
		if (!all) f.copies.clear();
	}

	// The scatter.
	if (element && a.has_group_memory && !a.barriers.empty() && a.global_atomics.empty() && (a.global_stores.size() == 1 || a.global_stores.size() == 2)) {
		bool ok = true;
		const Node* target = TargetRoot(a.global_stores[0]->index);
		const Node* scope = a.global_stores[0]->parent;
		struct Move {
			int dst, src;
			const Node* load;
		};
		std::vector<Move> moves;
		for (const Node* store : a.global_stores) {
			const Node* value = store->inputs.size() == 1 ? StripCasts(store->inputs[0]) : nullptr;
			if (!value || !target || TargetRoot(store->index) != target || store->parent != scope || !IsGlobalLoad(value) || !a.AddressIs(value->index, *element)) {
				ok = false;
				break;
			}
			moves.push_back({a.m.BindingOf(store->memory), a.m.BindingOf(value->memory), value});
		}
		// where the element lands is not a function of the thread index alone
		if (ok && a.m.ToPoly(target)) ok = false;
		// behind `element < n`
		DimExpr n_dim;
		if (ok) {
			ok = false;
			for (const Node* up = scope; up && up != kernel->dispatch_guard; up = up->parent) {
				if (!Is(up, "if") || up->inputs.size() != 1) continue;
				const Node* c = up->inputs[0];
				if (!Is(c, "lt") || c->inputs.size() != 2 || !a.AddressIs(c->inputs[0], *element)) continue;
				auto limit = a.m.ToPoly(c->inputs[1]);
				auto dim = limit ? a.m.ToDim(*limit) : std::nullopt;
				if (!dim) continue;
				n_dim = *dim;
				ok = true;
				break;
			}
		}
		// the keys are the moved words a digit is taken of
		int key_move = -1;
		SortFeatures::Digit digit;
		if (ok) {
			for (const Node* n : a.digit_nodes) {
				const Node* load = nullptr;
				SortFeatures::Digit d;
				if (!a.AsDigit(n, &load, &d.shift, &d.mask)) continue;
				for (size_t k = 0; k < moves.size(); k++)
					if (moves[k].load == load) {
						if (key_move >= 0 && key_move != (int)k) ok = false;
						key_move = (int)k;
						digit = d;
					}
			}
			if (key_move < 0) ok = false;
		}
		if (ok) {
			for (auto& mv : moves)
				if (mv.dst < 0 || mv.src < 0 || mv.dst >= (int)kernel->read_write_memory.size() || mv.src < (int)kernel->read_write_memory.size()) ok = false;
			if (moves.size() == 2 && (moves[0].dst == moves[1].dst || moves[0].src == moves[1].src)) ok = false;
			if (kernel->read_write_memory.size() != moves.size()) ok = false;  // it writes nothing else
		}
		if (ok) {
			f.scatter = true;
			f.keys_out = moves[key_move].dst;
			f.keys_in = moves[key_move].src;
			if (moves.size() == 2) {
				f.values_out = moves[1 - key_move].dst;
				f.values_in = moves[1 - key_move].src;
			}
			f.scatter_shift = digit.shift;
			f.scatter_mask = digit.mask;
			f.scatter_n = n_dim;
		}
	}
	kernel->sort = f;
}

}  // namespace tfhost
