// Integer expressions of a kernel as polynomials over its thread indices, a loop variable and its host scalars.
//
// After index finalisation (Compiler/Steps/GraphOps.cpp:989-1043,1091-1186) every address in a kernel is integer
// arithmetic over block / thread indices, loop variables and the host scalars bound as kernel variables. Expanding such
// an expression into a polynomial separates "how it moves with each index" (the coefficient of that index: a stride)
// from "where it starts" (the index-free part), both as polynomials in the host scalars alone, which a dispatch can
// evaluate from its variable words (DimExpr). Used by the whole-kernel idiom matcher (idiom_matcher.cpp) and by the
// analysis of the kernels of a `Radix sort` region (sort_features.cpp).
#pragma once

#include <algorithm>
#include <map>
#include <optional>
#include <unordered_map>

#include "tf_ir.h"

namespace tfhost {
namespace address_poly {

using Mono = std::vector<const Node*>;  // product of leaves, sorted by address
struct Poly {
	std::map<Mono, long> t;
	void Trim() {
		for (auto it = t.begin(); it != t.end();) it = it->second == 0 ? t.erase(it) : std::next(it);
	}
	bool operator==(const Poly& o) const { return t == o.t; }
};

inline Poly Constant(long c) {
	Poly p;
	if (c != 0) p.t[{}] = c;
	return p;
}
inline Poly Leaf(const Node* n) {
	Poly p;
	p.t[{n}] = 1;
	return p;
}
inline Poly Add(const Poly& a, const Poly& b, long sign) {
	Poly r = a;
	for (auto& kv : b.t) r.t[kv.first] += sign * kv.second;
	r.Trim();
	return r;
}
inline Poly Mul(const Poly& a, const Poly& b) {
	Poly r;
	for (auto& x : a.t)
		for (auto& y : b.t) {
			Mono m(x.first);
			m.insert(m.end(), y.first.begin(), y.first.end());
			std::sort(m.begin(), m.end());
			r.t[m] += x.second * y.second;
		}
	r.Trim();
	return r;
}

struct Matcher {
	const Kernel* kernel;
	const Node* loop = nullptr;
	std::unordered_map<const Node*, int> index_of;     // thread-index node -> dimension
	std::unordered_map<const Node*, int> variable_of;  // `variable` node -> position in the variable block

	explicit Matcher(const Kernel* k) : kernel(k) {
		for (size_t i = 0; i < k->index_nodes.size(); i++) index_of[k->index_nodes[i]] = (int)i;
		for (size_t i = 0; i < k->variables.size(); i++) variable_of[k->variables[i].node] = (int)i;
	}

	bool IsIndexLeaf(const Node* n) const { return index_of.count(n) || n == loop; }

	// Facts the match relies on that only a dispatch can confirm: lhs <= rhs for the dispatch's host scalars.
	std::vector<std::pair<Poly, Poly>> conditions;

	// Every leaf is a non-negative quantity (indices, extents), so non-negative coefficients mean p >= 0.
	static bool NonNegative(const Poly& p) {
		for (auto& kv : p.t)
			if (kv.second < 0) return false;
		return true;
	}

	// Largest value of p over the index ranges: every index leaf at its extent minus one (p must be NonNegative).
	std::optional<Poly> MaxOf(const Poly& p) {
		Poly r;
		for (auto& kv : p.t) {
			Poly term = Constant(kv.second);
			for (const Node* f : kv.first) {
				if (IsIndexLeaf(f)) {
					auto e = Extent(f);
					if (!e) return std::nullopt;
					term = Mul(term, Add(*e, Constant(1), -1));
				} else {
					term = Mul(term, Leaf(f));
				}
			}
			r = Add(r, term, 1);
		}
		return r;
	}

	// value <= limit for every thread and loop step? Structurally, or as a condition on the dispatch.
	bool BoundedBy(const Poly& value, const Poly& limit) {
		if (!NonNegative(value)) return false;
		auto mx = MaxOf(value);
		if (!mx) return false;
		if (!(*mx == limit)) conditions.push_back({*mx, limit});
		return true;
	}

	// A boolean that is false for every thread and loop step: the out-of-bounds test the reference wraps around
	// loads of reshaped tensors (ConstantOutOfBounds, Implementations.cpp:56-69): false || (i < 0 || i >= n) || ...
	bool NeverTrue(const Node* c, int depth = 0) {
		if (!c || depth > 16) return false;
		const std::string op = c->op->name;
		if (op == "const") return c->type == TFType_Bool && c->data == 0 && !c->modified;
		if (op == "or" && c->inputs.size() == 2) return NeverTrue(c->inputs[0], depth + 1) && NeverTrue(c->inputs[1], depth + 1);
		if ((op == "lt" || op == "gte") && c->inputs.size() == 2) {
			auto a = ToPoly(c->inputs[0]), b = ToPoly(c->inputs[1]);
			if (!a || !b || !NonNegative(*a)) return false;
			if (op == "lt") return b->t.empty();                     // a < 0 with a >= 0
			return BoundedBy(*a, Add(*b, Constant(1), -1));          // a >= b  is false when max a <= b - 1
		}
		return false;
	}

	// Extent of a thread index or of the loop variable (which must start at zero), as a polynomial.
	std::optional<Poly> Extent(const Node* leaf) {
		if (leaf == loop) {
			auto b = ToPoly(loop->inputs[0]);
			if (!b || !b->t.empty()) return std::nullopt;
			return ToPoly(loop->inputs[1]);
		}
		auto it = index_of.find(leaf);
		if (it == index_of.end() || (size_t)it->second >= kernel->shape_nodes.size()) return std::nullopt;
		return ToPoly(kernel->shape_nodes[it->second]);
	}

	std::optional<Poly> ToPoly(const Node* n, int depth = 0) {
		if (!n || depth > 48) return std::nullopt;
		if (IsIndexLeaf(n) || variable_of.count(n)) return Leaf(n);
		const std::string op = n->op->name;
		if (n->modified) return std::nullopt;
		if (op == "const") {
			if (n->type != TFType_Int && n->type != TFType_Uint) return std::nullopt;
			return Constant((long)(int)n->data);
		}
		if ((op == "add" || op == "sub" || op == "mul") && n->inputs.size() == 2 && (n->type == TFType_Int || n->type == TFType_Uint)) {
			auto a = ToPoly(n->inputs[0], depth + 1), b = ToPoly(n->inputs[1], depth + 1);
			if (!a || !b) return std::nullopt;
			return op == "mul" ? Mul(*a, *b) : Add(*a, *b, op == "add" ? 1 : -1);
		}
		if ((op == "int" || op == "uint" || op == "copy") && n->inputs.size() == 1 && (n->inputs[0]->type == TFType_Int || n->inputs[0]->type == TFType_Uint))
			return ToPoly(n->inputs[0], depth + 1);
		if (op == "clamp" && n->inputs.size() == 3) {
			// clamp(e, 0, hi) is the identity when 0 <= e <= hi: by construction for a guarded thread index or a loop
			// variable against its own extent, otherwise as a condition the dispatch has to meet
			auto e = ToPoly(n->inputs[0], depth + 1), lo = ToPoly(n->inputs[1], depth + 1), hi = ToPoly(n->inputs[2], depth + 1);
			if (e && lo && hi && lo->t.empty() && BoundedBy(*e, *hi)) return e;
		}
		return std::nullopt;
	}

	// Coefficient of `leaf` in p as a polynomial free of index leaves; fails on terms such as leaf^2 or leaf*other_index.
	std::optional<Poly> Coefficient(const Poly& p, const Node* leaf) {
		Poly c;
		for (auto& kv : p.t) {
			long count = std::count(kv.first.begin(), kv.first.end(), leaf);
			if (count == 0) continue;
			if (count > 1) return std::nullopt;
			Mono rest;
			for (const Node* f : kv.first) {
				if (f == leaf) continue;
				if (IsIndexLeaf(f)) return std::nullopt;
				rest.push_back(f);
			}
			c.t[rest] += kv.second;
		}
		c.Trim();
		return c;
	}

	// Part of p that contains none of the index leaves (the operand's constant offset).
	Poly Offset(const Poly& p) {
		Poly c;
		for (auto& kv : p.t)
			if (std::none_of(kv.first.begin(), kv.first.end(), [&](const Node* f) { return IsIndexLeaf(f); })) c.t[kv.first] = kv.second;
		return c;
	}

	std::optional<DimExpr> ToDim(const Poly& p) {
		DimExpr d;
		for (auto& kv : p.t) {
			std::vector<int> vars;
			for (const Node* f : kv.first) {
				auto it = variable_of.find(f);
				if (it == variable_of.end()) return std::nullopt;
				vars.push_back(it->second);
			}
			d.terms.push_back({vars, kv.second});
		}
		return d;
	}

	int BindingOf(const Node* memory) const {
		auto all = kernel->MemoryBindings();
		for (size_t i = 0; i < all.size(); i++)
			if (all[i] == memory) return (int)i;
		return -1;
	}
};

}  // namespace address_poly
}  // namespace tfhost
