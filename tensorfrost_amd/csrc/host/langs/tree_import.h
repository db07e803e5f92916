// Reads one kernel out of the compiler's own tree into the form the HIP emitter works on.
//
// The emitter, the idiom matcher and the sort-composition fingerprints consume tfhost::Kernel / tfhost::Node
// (tf_ir.h). TensorFrost hands a code generator something else (Backend/CodeGen/Generators.cpp:9-23 passes
// `Program*, Kernel*`):
//
//   Kernel   Compiler/KernelGen.h:17-46     root (the `kernel` node); variables, read_write_memory, read_only_memory as
//                                           map<Node*, size_t> from the host-side node to its slot; group_memory as
//                                           set<Node*>; shape = the kernel node's Shape arguments (NodeArguments)
//   Node     Compiler/Graph/Node.h:58-75    a child / next list under its parent (placeholders end a list, :84-86),
//                                           `op->name_`, `args` (ArgumentManager, Compiler/Graph/Arguments.h:44-230:
//                                           Get / Has / Count by ArgType and position, OutputCount), `format.type`,
//                                           `data` (vector<uint>), `flags` (NodeProp::Modified, LocalMemoryOp),
//                                           debug_name, var_name, group_size (on the kernel node)
//
// Inside a kernel an argument may point at a node OUTSIDE it: a host scalar, which Compiler/KernelGen.cpp:41-52 has put
// into `variables` (the reference prints it as var_<name>, Generators.h:95-97), or the `memory` node of a bound tensor.
// Here each of those becomes a node of its own in the kernel (`variable`, `memory`), in slot order.
//
// What the reference's Kernel does not hold but the emitter needs -- thread-index nodes, the extents they are tested
// against, the `if (is_inside_dispatch)` node -- is found in the tree afterwards by DeriveKernelGeometry
// (kernel_geometry.cpp), which also checks `dim` (= number of Shape arguments) and `group_size` (= the kernel node's)
// against the index arithmetic.
//
// The importer is a template over the tree's types so that the same code is compiled twice: against the reference's
// headers (langs/reference_side/HIP.cpp, `Tree` = TensorFrost's Node / Kernel / ArgType / NodeProp) and, in the test
// suite, against a mirror of those classes that can be filled from a tfhost tree, which is how it is executed where the
// compiler itself cannot be built.
#pragma once

#include <map>
#include <set>
#include <stdexcept>
#include <string>
#include <unordered_map>
#include <vector>

#include "../tf_ir.h"

namespace tfhost {

template <class Tree>
class KernelImporter {
	using RNode = typename Tree::Node;
	using RKernel = typename Tree::Kernel;
	using ArgType = typename Tree::ArgType;
	using NodeProp = typename Tree::NodeProp;

 public:
	explicit KernelImporter(Program* into) : program_(into) {}

	// The kernel as a new kernel of the program given to the constructor. Throws std::runtime_error with the node's
	// name when the tree is not in post-lowering form (an operation a kernel cannot contain, several Index arguments
	// on a memory operation, an argument that is neither in the kernel nor bound to it).
	Kernel* Import(const RKernel* kernel) {
		if (!kernel || !kernel->root) throw std::runtime_error("ImportKernel: no kernel node");
		auto owned = std::make_unique<Kernel>();
		Kernel* k = owned.get();
		program_->kernels_.push_back(std::move(owned));
		seen_.clear();

		// Bound tensors and host scalars, by slot.
		for (RNode* memory : BySlot(kernel->read_write_memory, "read_write_memory")) k->read_write_memory.push_back(Bind(memory, "memory", TFType_Uint));
		for (RNode* memory : BySlot(kernel->read_only_memory, "read_only_memory")) k->read_only_memory.push_back(Bind(memory, "memory", TFType_Uint));
		for (RNode* scalar : BySlot(kernel->variables, "variables")) {
			Node* v = Bind(scalar, "variable", TypeOf(scalar));
			k->variables.push_back({v, v->debug_name, v->type});
		}

		// The tree: nodes first, arguments second (an argument may be defined later in the list than its user only for
		// `set`, but nothing here depends on that).
		k->root = Translate(kernel->root, nullptr);
		Wire(kernel->root);

		// Group memory in the order of the tree (the reference keeps a set ordered by address).
		CollectGroupMemory(k->root, kernel->group_memory, k);
		if (k->group_memory.size() != kernel->group_memory.size()) throw std::runtime_error("ImportKernel: a group_memory node of the kernel is not in its tree");

		k->group_size.assign(kernel->root->group_size.begin(), kernel->root->group_size.end());
		k->dim = (int)kernel->shape.size();
		DeriveKernelGeometry(k);

		// The extents the guard tests are the kernel node's Shape arguments, wherever those reached the kernel as host scalars.
		for (size_t d = 0; d < k->shape_nodes.size() && d < kernel->shape.size(); d++) {
			auto arg = kernel->shape.find({ArgType::Shape, (int)d});
			if (arg == kernel->shape.end()) throw std::runtime_error("ImportKernel: the kernel has no Shape argument " + std::to_string(d));
			auto bound = seen_.find(arg->second);
			if (bound != seen_.end() && kernel->variables.count(arg->second) && bound->second != k->shape_nodes[d])
				throw std::runtime_error("ImportKernel: index_" + std::to_string(d) + " is not tested against the kernel's Shape argument " + std::to_string(d));
		}
		return k;
	}

 private:
	Program* program_;
	std::unordered_map<const RNode*, Node*> seen_;

	static TFType TypeOf(const RNode* n) { return (TFType)(int)n->format.type; }

	// A list of children ends at a placeholder (Node::valid, Compiler/Graph/Node.h:88-90, which is not a const member)
	// or, for the dispatch guard, at a null `next` (GraphOps.cpp:1263-1271).
	static bool IsNode(const RNode* n) { return n != nullptr && !n->flags.has(NodeProp::Placeholder); }

	static std::vector<RNode*> BySlot(const std::map<RNode*, size_t>& slots, const char* what) {
		std::vector<RNode*> ordered(slots.size(), nullptr);
		for (auto& [node, slot] : slots) {
			if (slot >= ordered.size() || ordered[slot]) throw std::runtime_error(std::string("ImportKernel: the slots of ") + what + " are not 0..n-1");
			ordered[slot] = node;
		}
		return ordered;
	}

	Node* NewNode(const std::string& op, TFType type) {
		auto node = std::make_unique<Node>();
		node->op = &FindOperation(op);  // throws "IR Operation not defined" for anything a lowered kernel cannot contain
		node->type = type;
		Node* raw = node.get();
		program_->nodes.push_back(std::move(node));
		return raw;
	}

	// A node outside the kernel that the kernel is bound to: it keeps the name the host program knows it by
	// (GenerateNodeNames, Generators.cpp:46-91, runs before any kernel is generated).
	Node* Bind(const RNode* outside, const char* op, TFType type) {
		if (!outside) throw std::runtime_error("ImportKernel: empty binding slot");
		if (seen_.count(outside)) throw std::runtime_error("ImportKernel: " + outside->var_name + " is bound twice");
		Node* n = NewNode(op, type);
		n->debug_name = !outside->var_name.empty() ? outside->var_name : outside->debug_name;
		seen_[outside] = n;
		return n;
	}

	Node* Translate(const RNode* from, Node* parent) {
		Node* n = NewNode(from->op->name_, TypeOf(from));
		n->parent = parent;
		n->data = from->data.empty() ? 0u : (uint32_t)from->data[0];
		n->debug_name = from->debug_name;
		n->modified = from->flags.has(NodeProp::Modified);
		n->local_memory_op = from->flags.has(NodeProp::LocalMemoryOp);
		// Whether a value may be substituted into its single user is decided by the number of argument slots that
		// name it (Generators.h:111-112 reads ArgumentManager::OutputCount).
		n->use_count = (int)from->args.OutputCount();
		seen_[from] = n;
		for (const RNode* c = from->child; IsNode(c); c = c->next) n->children.push_back(Translate(c, n));
		return n;
	}

	Node* Resolve(const RNode* user, const RNode* argument) {
		auto it = seen_.find(argument);
		if (it != seen_.end() && it->second->parent == nullptr && it->second->op->cls == OpClass::Special) it->second->use_count++;  // a binding: counted here
		if (it == seen_.end())
			throw std::runtime_error("ImportKernel: an argument of " + user->var_name + " (" + user->op->name_ + ") is neither inside the kernel nor bound to it: " +
			                         argument->var_name + " (" + argument->op->name_ + ")");
		return it->second;
	}

	void Wire(const RNode* from) {
		Node* n = seen_.at(from);
		const auto& args = from->args;
		const int inputs = args.Count(ArgType::Input);
		for (int i = 0; i < inputs; i++) n->inputs.push_back(Resolve(from, args.Get(ArgType::Input, i)));
		const int indices = args.Count(ArgType::Index);
		if (indices > 1) throw std::runtime_error("ImportKernel: " + from->var_name + " still has " + std::to_string(indices) + " Index arguments (memory indexing not finalised)");
		if (indices == 1) n->index = Resolve(from, args.Get(ArgType::Index, 0));
		if (args.Has(ArgType::Memory, 0)) n->memory = Resolve(from, args.Get(ArgType::Memory, 0));
		for (const RNode* c = from->child; IsNode(c); c = c->next) Wire(c);
	}

	void CollectGroupMemory(Node* n, const std::set<RNode*>& declared, Kernel* k) {
		if (std::string(n->op->name) == "group_memory") {
			for (RNode* g : declared)
				if (seen_.at(g) == n) k->group_memory.push_back(n);
		}
		for (Node* c : n->children) CollectGroupMemory(c, declared, k);
	}
};

}  // namespace tfhost
