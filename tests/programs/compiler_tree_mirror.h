// Test double for the compiler-side classes the HIP kernel importer reads (langs/tree_import.h): the members and
// accessors it touches, under the names they have in TensorFrost --
//   Node             Compiler/Graph/Node.h:58-96       parent / child / next / prev, op->name_, flags.has, args, format.type,
//                                                     data, debug_name, var_name, group_size; a placeholder ends every list
//   ArgumentManager  Compiler/Graph/Arguments.h:44-230 Get / Has / Count by (ArgType, position), OutputCount
//   Kernel           Compiler/KernelGen.h:17-46        root, variables / read_write_memory / read_only_memory as
//                                                     map<Node*, size_t>, group_memory as set<Node*>, shape as map<ArgID, Node*>
// -- so that KernelImporter<Tree>, the template that a TensorFrost build instantiates with the real classes, can be
// instantiated and RUN here, where the compiler cannot be built. This is not a build of the reference: nothing of its
// code is in it, and whether the real classes offer these members with these meanings is what compiling
// csrc/reference_side/Backend/CodeGen/Langs/HIP.cpp against the reference's headers checks (test_import_against_reference.py).
//
// ExportKernel fills a mirror from a kernel of this repository's IR the way the passes would have left it: bound
// tensors and host scalars are nodes OUTSIDE the kernel node (host-side `memory` nodes and scalar values) held in
// std::maps keyed by node address with their slot as the value (Compiler/KernelGen.cpp:16-65), the lists end in placeholders
// except the dispatch guard's own list position, whose `next` is null (GraphOps.cpp:1263-1271), and the derived fields
// of tfhost::Kernel (index / shape nodes, guard, dim) are NOT carried over.
#pragma once

#include <array>
#include <map>
#include <memory>
#include <set>
#include <stdexcept>
#include <string>
#include <unordered_map>
#include <vector>

#include "tf_ir.h"

namespace mirror {

enum class ArgType { Input, Index, Shape, Memory, None, Count };

// Enumerators in the order of Compiler/Graph/Node.h:9-28.
enum class NodeProp {
	Placeholder, Modified, IsStatic, OutputMemory, InputShapeDim, InputShapeMemory, InputMemory, InputMemoryList, KeepDims, DetachGrad, PassGrad,
	NoLoadFusion, NoCopyFusion, StopFusion, HintMaxValue, HintMinValue, LocalMemoryOp, Count,
};

using ArgID = std::pair<ArgType, int>;

struct Operation {
	std::string name_;
};

struct DataFormat {
	TFType type = TFType_Float;
	size_t size = 32;
};

class NodeProps {
	std::array<bool, (size_t)NodeProp::Count> set_{};

 public:
	void set(NodeProp p) { set_[(size_t)p] = true; }
	void remove(NodeProp p) { set_[(size_t)p] = false; }
	bool has(NodeProp p) const { return set_[(size_t)p]; }
};

class Node;

class ArgumentManager {
	std::map<ArgID, Node*> inputs_;
	std::map<ArgType, int> counts_;
	size_t outputs_ = 0;

 public:
	void AddArgument(ArgType type, int index, Node* node);
	bool Has(ArgType type, int index = 0) const { return inputs_.count({type, index}) != 0; }
	Node* Get(ArgType type, int index = 0) const {
		auto it = inputs_.find({type, index});
		if (it == inputs_.end()) throw std::runtime_error("Argument at index " + std::to_string(index) + " not found");
		return it->second;
	}
	int Count(ArgType type) const {
		auto it = counts_.find(type);
		return it == counts_.end() ? 0 : it->second;
	}
	size_t OutputCount() const { return outputs_; }
	void AddOutput() { outputs_++; }
};

class Node {
 public:
	std::string name, var_name, debug_name;
	Node *parent = nullptr, *child = nullptr, *next = nullptr, *prev = nullptr;
	const Operation* op = nullptr;
	NodeProps flags;
	ArgumentManager args;
	DataFormat format;
	std::vector<unsigned> data;
	std::vector<int> group_size;

	Node() { flags.set(NodeProp::Placeholder); }
	bool valid() { return !flags.has(NodeProp::Placeholder); }
};

inline void ArgumentManager::AddArgument(ArgType type, int index, Node* node) {
	if (!inputs_.count({type, index})) counts_[type]++;
	inputs_[{type, index}] = node;
	node->args.AddOutput();
}

class Kernel {
 public:
	Node* root = nullptr;
	std::map<Node*, size_t> variables, read_write_memory, read_only_memory;
	std::set<Node*> group_memory;
	std::map<ArgID, Node*> shape;
};

struct Tree {
	using Node = mirror::Node;
	using Kernel = mirror::Kernel;
	using ArgType = mirror::ArgType;
	using NodeProp = mirror::NodeProp;
};

// Owns the nodes of one exported kernel.
struct Exported {
	Kernel kernel;
	std::vector<std::unique_ptr<Node>> nodes;
	std::map<std::string, std::unique_ptr<Operation>> operations;
};

// reverse_slots: the bindings get their slots in reverse order, to show that the importer goes by slot and not by the
// order in which the maps hold their nodes.
std::unique_ptr<Exported> ExportKernel(const tfhost::Kernel* kernel, bool reverse_slots);

}  // namespace mirror
