// What the index finalisation of the compiler's passes leaves at the top of a kernel's tree, found again by walking
// that tree.
//
// TensorFrost's `Kernel` (Compiler/KernelGen.h:17-46) carries the kernel node, three binding maps, the group
// memory set and the Shape arguments of the kernel node; the thread-group size hangs on the kernel node itself
// (`Node::group_size`, Compiler/Graph/Node.h:73). The thread indices, the extents they are tested against and the
// `if` that guards the body are ordinary nodes that IR::LinearBlockModeIndices and ComputeIndicesFromBlockIndex
// (Compiler/Steps/GraphOps.cpp:1136-1186, 1091-1134) put first among the kernel's children:
//
//     block_id, block_thread_id<k>, blocks_shape_<k> = (shape_k + G_k - 1) / G_k, ...
//     index_<k> = out_block_k * G_k + block_thread_id<k>        (k < number of group axes; else out_block_k)
//     is_inside_dispatch = index_0 < shape_0 && index_1 < shape_1 && ...
//     if (is_inside_dispatch) { body }
//
// The HIP emitter and the idiom matcher reason from `0 <= index_k < shape_k` inside that `if`, so they need those
// nodes by role. Debug names are not relied on (the reference can strip them, Generators.cpp:52-55): the guard is the
// kernel's last direct child when that is an `if` over a conjunction of `<` comparisons whose left sides are built
// from block_id / block_thread_id.
#include <functional>
#include <stdexcept>
#include <string>

#include "tf_ir.h"

namespace tfhost {

namespace {

bool Is(const Node* n, const char* op) { return n && std::string(n->op->name) == op; }

// Whether the value is computed from block_thread_id<k> (k < 0: from block_id or any block_thread_id).
bool MovesWith(const Node* n, int k, int depth = 0) {
	if (!n || depth > 256) return false;
	if (Is(n, "block_thread_id")) return k < 0 || (int)n->data == k;
	if (Is(n, "block_id")) return k < 0;
	for (const Node* in : n->inputs)
		if (MovesWith(in, k, depth + 1)) return true;
	return false;
}

void SplitConjunction(const Node* n, bool top, std::vector<const Node*>& out) {
	// The passes name only the whole condition; a named `and` below it is a value of the program's own.
	if (Is(n, "and") && n->type == TFType_Bool && n->inputs.size() == 2 && (top || n->debug_name.empty())) {
		SplitConjunction(n->inputs[0], false, out);
		SplitConjunction(n->inputs[1], false, out);
	} else {
		out.push_back(n);
	}
}

// G from `x * G + block_thread_id<k>` in either operand order; a group extent of 1 is printed as
// `x + block_thread_id<k>` (x, the block's own index, is never a product with a constant); 0 if the index has
// neither form.
int GroupExtentOf(const Node* index, int k) {
	if (!Is(index, "add") || index->inputs.size() != 2) return 0;
	for (int side = 0; side < 2; side++) {
		const Node* tid = index->inputs[side];
		const Node* scaled = index->inputs[1 - side];
		if (!Is(tid, "block_thread_id") || (int)tid->data != k) continue;
		if (Is(scaled, "mul") && scaled->inputs.size() == 2)
			for (const Node* f : scaled->inputs)
				if (Is(f, "const") && !f->modified && (int)f->data > 0) return (int)f->data;
		return 1;
	}
	return 0;
}

}  // namespace

void DeriveKernelGeometry(Kernel* kernel) {
	if (!kernel || !kernel->root) throw std::runtime_error("DeriveKernelGeometry: the kernel has no tree");
	kernel->index_nodes.clear();
	kernel->shape_nodes.clear();
	kernel->dispatch_guard = nullptr;

	// The guard: the last direct child, an `if` over index_k < shape_k terms.
	Node* guard = kernel->root->children.empty() ? nullptr : kernel->root->children.back();
	std::vector<const Node*> terms;
	if (guard && Is(guard, "if") && guard->inputs.size() == 1) {
		SplitConjunction(guard->inputs[0], true, terms);
		for (const Node* t : terms)
			if (!Is(t, "lt") || t->inputs.size() != 2 || !MovesWith(t->inputs[0], -1)) guard = nullptr;
	} else {
		guard = nullptr;
	}
	if (!guard) {
		// A kernel without a dispatch shape has no index arithmetic (GraphOps.cpp:1220-1223): nothing to find.
		if (kernel->dim < 1) kernel->dim = (int)kernel->group_size.size() > 0 ? (int)kernel->group_size.size() : 1;
		return;
	}

	// Index k is the one that moves with block_thread_id<k>; kernel dimensions beyond the group's axes follow in the
	// order of their comparisons.
	const size_t dims = terms.size();
	std::vector<const Node*> by_axis(dims, nullptr);
	std::vector<bool> placed(dims, false);
	for (size_t k = 0; k < dims && k < 3; k++)
		for (size_t t = 0; t < dims; t++)
			if (!placed[t] && MovesWith(terms[t]->inputs[0], (int)k)) {
				by_axis[k] = terms[t];
				placed[t] = true;
				break;
			}
	size_t next = 0;
	for (size_t t = 0; t < dims; t++) {
		if (placed[t]) continue;
		bool grouped = false;
		for (int g = 0; g < 3; g++) grouped |= MovesWith(terms[t]->inputs[0], g);
		if (grouped) throw std::runtime_error("DeriveKernelGeometry: two indices of the dispatch guard move with the same block_thread_id");
		while (next < dims && by_axis[next]) next++;
		if (next == dims) throw std::runtime_error("DeriveKernelGeometry: the dispatch guard has more comparisons than dimensions");
		by_axis[next] = terms[t];
		placed[t] = true;
	}
	for (size_t k = 0; k < dims; k++) {
		if (!by_axis[k]) throw std::runtime_error("DeriveKernelGeometry: no index of the dispatch guard moves with block_thread_id" + std::to_string(k));
		kernel->index_nodes.push_back(const_cast<Node*>(by_axis[k])->inputs[0]);
		kernel->shape_nodes.push_back(const_cast<Node*>(by_axis[k])->inputs[1]);
	}
	kernel->dispatch_guard = guard;

	if (kernel->dim >= 1 && (size_t)kernel->dim != dims)
		throw std::runtime_error("DeriveKernelGeometry: the kernel has " + std::to_string(kernel->dim) + " Shape arguments but its dispatch guard tests " +
		                         std::to_string(dims) + " indices");
	kernel->dim = (int)dims;

	// Thread-group extents from the index arithmetic; the kernel node's own group_size, where given, has to agree.
	std::vector<int> group;
	for (size_t k = 0; k < dims && k < 3; k++) {
		const int g = GroupExtentOf(kernel->index_nodes[k], (int)k);
		if (g == 0) break;
		group.push_back(g);
	}
	if (kernel->group_size.empty()) {
		if (group.empty()) throw std::runtime_error("DeriveKernelGeometry: no thread-group size on the kernel node and none in its index arithmetic");
		kernel->group_size = group;
	} else {
		for (size_t k = 0; k < group.size() && k < kernel->group_size.size(); k++)
			if (group[k] != kernel->group_size[k])
				throw std::runtime_error("DeriveKernelGeometry: index_" + std::to_string(k) + " is computed with a group extent of " + std::to_string(group[k]) +
				                         " but the kernel node says " + std::to_string(kernel->group_size[k]));
	}
}

}  // namespace tfhost
