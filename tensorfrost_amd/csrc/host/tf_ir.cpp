#include "tf_ir.h"

#include <algorithm>
#include <functional>
#include <unordered_map>

namespace tfhost {

// Post-lowering operations and how they print, restated from the table at
// TensorFrost/Compiler/Operations.cpp:23-179 (name, code string, class). Algorithm and Gradient
// entries never survive the passes and are left out.
static const OpInfo kOps[] = {
    // host side (Operations.cpp:25-48)
    {"host", "", OpClass::Special},
    {"reshape", "reshape", OpClass::Special},
    {"assert", "assert_tensor", OpClass::Special},
    {"input_shape", "", OpClass::Special},
    {"deallocate", "", OpClass::Special},
    {"region_begin", "region_begin", OpClass::Special},
    {"region_end", "region_end", OpClass::Special},
    {"print_value", "print_value", OpClass::Special},
    {"assert_value", "assert_value", OpClass::Special},
    // kernels
    {"kernel", "", OpClass::Special},
    {"loop", "", OpClass::Special},
    {"if", "", OpClass::Special},
    {"break", "break", OpClass::Keyword},
    {"continue", "continue", OpClass::Keyword},
    {"discard", "discard", OpClass::Keyword},
    {"group_barrier", "group_barrier", OpClass::Function},
    {"memory", "", OpClass::Special},
    {"group_memory", "", OpClass::Special},
    {"local_memory", "", OpClass::Special},
    {"variable", "", OpClass::Special},  // a host scalar read through the kernel's variable block
    {"load", "", OpClass::Memory},
    {"store", "", OpClass::Memory},
    {"set", "", OpClass::Set},
    {"InterlockedAdd", "InterlockedAdd", OpClass::Memory},
    {"InterlockedMin", "InterlockedMin", OpClass::Memory},
    {"InterlockedMax", "InterlockedMax", OpClass::Memory},
    {"InterlockedAnd", "InterlockedAnd", OpClass::Memory},
    {"InterlockedOr", "InterlockedOr", OpClass::Memory},
    {"InterlockedXor", "InterlockedXor", OpClass::Memory},
    {"InterlockedAdd_Prev", "InterlockedAdd_Prev", OpClass::Memory},
    {"block_thread_id", "block_thread_id", OpClass::DimensionIndex},
    {"block_id", "block_id", OpClass::Variable},
    {"copy", "", OpClass::Copy},
    {"add", "+", OpClass::Operator},
    {"sub", "-", OpClass::Operator},
    {"mul", "*", OpClass::Operator},
    {"div", "/", OpClass::Operator},
    {"mod", "%", OpClass::Operator},
    {"lshift", "<<", OpClass::Operator},
    {"rshift", ">>", OpClass::Operator},
    {"and", "&", OpClass::Operator},
    {"or", "|", OpClass::Operator},
    {"xor", "^", OpClass::Operator},
    {"eq", "==", OpClass::Operator},
    {"neq", "!=", OpClass::Operator},
    {"lt", "<", OpClass::Operator},
    {"lte", "<=", OpClass::Operator},
    {"gt", ">", OpClass::Operator},
    {"gte", ">=", OpClass::Operator},
    {"notb", "!", OpClass::UnaryOperator},
    {"not", "~", OpClass::UnaryOperator},
    {"neg", "-", OpClass::UnaryOperator},
    {"uint", "uint", OpClass::TypeCast},
    {"int", "int", OpClass::TypeCast},
    {"float", "float", OpClass::TypeCast},
    {"bool", "bool", OpClass::TypeCast},
    {"asuint", "asuint", OpClass::TypeReinterpret},
    {"asint", "asint", OpClass::TypeReinterpret},
    {"asfloat", "asfloat", OpClass::TypeReinterpret},
    {"asbool", "asbool", OpClass::TypeReinterpret},
    {"min", "min", OpClass::Function},
    {"max", "max", OpClass::Function},
    {"abs", "abs", OpClass::Function},
    {"sign", "sign", OpClass::Function},
    {"ceil", "ceil", OpClass::Function},
    {"floor", "floor", OpClass::Function},
    {"round", "round", OpClass::Function},
    {"frac", "frac", OpClass::Function},
    {"exp", "exp", OpClass::Function},
    {"exp2", "exp2", OpClass::Function},
    {"log", "log", OpClass::Function},
    {"log2", "log2", OpClass::Function},
    {"sqrt", "sqrt", OpClass::Function},
    {"rsqrt", "rsqrt", OpClass::Function},
    {"rcp", "rcp", OpClass::Function},
    {"sin", "sin", OpClass::Function},
    {"cos", "cos", OpClass::Function},
    {"tan", "tan", OpClass::Function},
    {"asin", "asin", OpClass::Function},
    {"acos", "acos", OpClass::Function},
    {"atan", "atan", OpClass::Function},
    {"sinh", "sinh", OpClass::Function},
    {"cosh", "cosh", OpClass::Function},
    {"tanh", "tanh", OpClass::Function},
    {"pcg", "pcg", OpClass::Function},
    {"reversebits", "reversebits", OpClass::Function},
    {"pcgf", "pcgf", OpClass::Function},
    {"pow", "pow", OpClass::Function},
    {"atan2", "atan2", OpClass::Function},
    {"modf", "modf", OpClass::Function},
    {"step", "step", OpClass::Function},
    {"clamp", "clamp", OpClass::Function},
    {"lerp", "lerp", OpClass::Function},
    {"fma", "fma", OpClass::Function},
    {"smoothstep", "smoothstep", OpClass::Function},
    {"ternary", "", OpClass::TernaryOperator},
    {"const", "", OpClass::Constant},
};

const OpInfo& FindOperation(const std::string& name) {
	static const std::unordered_map<std::string, const OpInfo*> map = [] {
		std::unordered_map<std::string, const OpInfo*> m;
		for (const OpInfo& op : kOps) m[op.name] = &op;
		return m;
	}();
	auto it = map.find(name);
	if (it == map.end()) throw std::runtime_error("IR Operation not defined: " + name);
	return *it->second;
}

const std::string& Node::name() const {
	static thread_local std::string s;
	s = op->name;
	return s;
}

Kernel* Program::AddPrimitive(const std::string& name, size_t n_tensors, size_t n_variables) {
	auto k = std::make_unique<Kernel>();
	k->primitive = name;
	k->primitive_tensors = n_tensors;
	k->primitive_variables = n_variables;
	k->idiom = "primitive:" + name;
	Kernel* raw = k.get();
	kernels_.push_back(std::move(k));
	return raw;
}

// ---- the tail of a matmul kernel as a kernel of its own -----------------------------------------------------------

namespace {

void CollectNodes(const Node* n, std::vector<const Node*>& order, std::unordered_map<const Node*, Node*>& seen) {
	if (!n || seen.count(n)) return;
	seen[n] = nullptr;
	order.push_back(n);
	for (const Node* x : n->inputs) CollectNodes(x, order, seen);
	CollectNodes(n->index, order, seen);
	CollectNodes(n->memory, order, seen);
	for (const Node* c : n->children) CollectNodes(c, order, seen);
}

}  // namespace

Kernel* CloneKernel(Program* program, const Kernel* kernel, std::unordered_map<const Node*, Node*>* mapping) {
	std::vector<const Node*> order;
	std::unordered_map<const Node*, Node*> copy;
	CollectNodes(kernel->root, order, copy);
	for (Node* m : kernel->MemoryBindings()) CollectNodes(m, order, copy);
	for (auto& v : kernel->variables) CollectNodes(v.node, order, copy);
	for (const Node* n : order) {
		auto node = std::make_unique<Node>(*n);
		copy[n] = node.get();
		program->nodes.push_back(std::move(node));
	}
	auto at = [&](const Node* n) -> Node* { return n ? copy.at(n) : nullptr; };
	for (const Node* n : order) {
		Node* c = copy[n];
		for (Node*& x : c->inputs) x = at(x);
		c->index = at(c->index);
		c->memory = at(c->memory);
		for (Node*& x : c->children) x = at(x);
		c->parent = n->parent && copy.count(n->parent) ? copy[n->parent] : nullptr;
		c->var_name.clear();
	}
	auto k = std::make_unique<Kernel>();
	k->root = at(kernel->root);
	for (auto& v : kernel->variables) k->variables.push_back({at(v.node), v.name, v.type});
	for (Node* m : kernel->read_write_memory) k->read_write_memory.push_back(at(m));
	for (Node* m : kernel->read_only_memory) k->read_only_memory.push_back(at(m));
	for (Node* m : kernel->group_memory) k->group_memory.push_back(at(m));
	k->group_size = kernel->group_size;
	k->dim = kernel->dim;
	for (Node* n : kernel->index_nodes) k->index_nodes.push_back(at(n));
	for (Node* n : kernel->shape_nodes) k->shape_nodes.push_back(at(n));
	k->dispatch_guard = at(kernel->dispatch_guard);
	if (mapping) *mapping = copy;
	Kernel* raw = k.get();
	program->kernels_.push_back(std::move(k));
	return raw;
}

Kernel* MakeMatmulTailKernel(Program* program, const Kernel* kernel, const Node* accumulator, const Node* loop) {
	if (kernel->dim != 2 || kernel->index_nodes.size() != 2 || kernel->shape_nodes.size() != 2) throw std::runtime_error("matmul tail: kernel is not two-dimensional");
	std::unordered_map<const Node*, Node*> copy;
	Kernel* k = CloneKernel(program, kernel, &copy);
	auto at = [&](const Node* n) -> Node* { return n ? copy.at(n) : nullptr; };
	auto fresh = [&](const Node& from) {
		auto node = std::make_unique<Node>(from);
		Node* raw = node.get();
		program->nodes.push_back(std::move(node));
		return raw;
	};
	Node* acc = at(accumulator);
	Node* gone = at(loop);
	Node* scope = gone->parent;
	if (!scope || acc->parent != scope) throw std::runtime_error("matmul tail: accumulator and loop are not siblings");
	// What the loop body used is used once less (the emitter inlines values by their use count).
	std::function<void(Node*)> release = [&](Node* n) {
		for (Node* x : n->inputs) x->use_count--;
		if (n->index) n->index->use_count--;
		if (n->memory) n->memory->use_count--;
		for (Node* c : n->children) release(c);
	};
	release(gone);
	scope->children.erase(std::find(scope->children.begin(), scope->children.end(), gone));

	Node* product = fresh(Node());
	product->op = &FindOperation("memory");
	product->type = TFType_Uint;
	product->debug_name = "matmul_product";
	k->read_only_memory.push_back(product);
	auto binary = [&](const char* op, Node* a, Node* b) {
		Node* n = fresh(Node());
		n->op = &FindOperation(op);
		n->type = TFType_Int;
		n->inputs = {a, b};
		a->use_count++;
		b->use_count++;
		n->parent = scope;
		return n;
	};
	Node* row_offset = binary("mul", k->index_nodes[1], k->shape_nodes[0]);
	Node* address = binary("add", row_offset, k->index_nodes[0]);
	auto where = std::find(scope->children.begin(), scope->children.end(), acc);
	scope->children.insert(where, {row_offset, address});
	acc->op = &FindOperation("load");
	acc->inputs.clear();
	acc->memory = product;
	acc->index = address;
	acc->data = 0;
	acc->modified = false;
	acc->local_memory_op = false;
	product->use_count++;
	address->use_count++;
	return k;
}

// ---- builder ---------------------------------------------------------------------------------------

KernelBuilder::KernelBuilder(Program* program, int shape_dim, std::vector<int> group) : NodeBuilder(program), kernel_(new Kernel()) {
	if (shape_dim < 1) throw std::runtime_error("kernel needs at least one dimension");
	kernel_->dim = shape_dim;
	if (group.empty()) {
		switch (shape_dim) {
			case 1: group = {256}; break;
			case 2: group = {16, 16}; break;
			default: group = {8, 8, 8}; break;
		}
	}
	if (group.size() > 3 || (int)group.size() > shape_dim) throw std::runtime_error("invalid group dimensionality");
	kernel_->group_size = group;
	Node* root = NewNode("kernel", TFType_None);
	kernel_->root = root;
	scope_stack_.push_back(root);
}

Node* NodeBuilder::NewNode(const std::string& op, TFType type) {
	auto node = std::make_unique<Node>();
	node->op = &FindOperation(op);
	node->type = type;
	Node* raw = node.get();
	program_->nodes.push_back(std::move(node));
	return raw;
}

void NodeBuilder::Append(Node* n) {
	Node* scope = scope_stack_.back();
	n->parent = scope;
	scope->children.push_back(n);
}

void NodeBuilder::Use(Node* user, V v) {
	if (!v.n) throw std::runtime_error("null value used as an argument of " + std::string(user->op->name));
	user->inputs.push_back(v.n);
	v.n->use_count++;
}

V KernelBuilder::Buffer(const std::string& name, bool read_only) {
	Node* n = NewNode("memory", TFType_Uint);
	n->debug_name = name;
	(read_only ? kernel_->read_only_memory : kernel_->read_write_memory).push_back(n);
	return V(n, this);
}

V KernelBuilder::Var(const std::string& name, TFType type) {
	Node* n = NewNode("variable", type);
	n->debug_name = name;
	kernel_->variables.push_back({n, name, type});
	return V(n, this);
}

V KernelBuilder::GroupMemory(const std::string& name, TFType type, int size) {
	Node* n = NewNode("group_memory", type);
	n->debug_name = name;
	n->data = (uint32_t)size;
	kernel_->group_memory.push_back(n);
	Append(n);
	return V(n, this);
}

V KernelBuilder::LocalMemory(const std::string& name, TFType type, int size) {
	Node* n = NewNode("local_memory", type);
	n->debug_name = name;
	n->data = (uint32_t)size;
	Append(n);
	return V(n, this);
}

V NodeBuilder::Const(float v) {
	Node* n = NewNode("const", TFType_Float);
	n->data = FloatBits(v);
	Append(n);
	return V(n, this);
}
V NodeBuilder::Const(int v) {
	Node* n = NewNode("const", TFType_Int);
	n->data = (uint32_t)v;
	Append(n);
	return V(n, this);
}
V NodeBuilder::ConstU(uint32_t v) {
	Node* n = NewNode("const", TFType_Uint);
	n->data = v;
	Append(n);
	return V(n, this);
}
V NodeBuilder::ConstB(bool v) {
	Node* n = NewNode("const", TFType_Bool);
	n->data = v ? 1u : 0u;
	Append(n);
	return V(n, this);
}

V NodeBuilder::Op(const std::string& name, std::vector<V> inputs, TFType type) {
	Node* n = NewNode(name, type);
	for (V& v : inputs) Use(n, v);
	Append(n);
	return V(n, this);
}

V NodeBuilder::Named(V v, const std::string& debug_name) {
	v.n->debug_name = debug_name;
	return v;
}

V KernelBuilder::BlockId() {
	Node* n = NewNode("block_id", TFType_Int);
	Append(n);
	return V(n, this);
}

V KernelBuilder::BlockThreadId(int k) {
	Node* n = NewNode("block_thread_id", TFType_Int);
	n->data = (uint32_t)k;
	Append(n);
	return V(n, this);
}

std::vector<V> KernelBuilder::ThreadIndices(const std::vector<V>& shape) {
	const int dims = (int)shape.size();
	if (dims != kernel_->dim) throw std::runtime_error("ThreadIndices: shape does not match the kernel dimensionality");
	const int block_dim = (int)kernel_->group_size.size();
	V block_index = BlockId();

	// blocks_shape_k = ceil(shape_k / group_k) for grouped dims, shape_k for the outer ones
	std::vector<V> blocks_shape;
	for (int i = 0; i < dims; i++) {
		V bs;
		if (i < block_dim) {
			V g = Const(kernel_->group_size[i]);
			bs = (shape[i] + g - Const(1)) / g;
		} else {
			bs = shape[i];
		}
		// Shape values that are plain kernel variables keep their own name.
		if (bs.n->op->cls != OpClass::Special) Named(bs, "blocks_shape_" + std::to_string(i));
		blocks_shape.push_back(bs);
	}

	// Tensor::IndicesFromFlatIndex over blocks_shape (innermost first).
	std::vector<V> out_block(dims);
	if (dims == 1) {
		out_block[0] = block_index;
	} else {
		std::vector<V> sizes(dims);
		sizes[0] = blocks_shape[0];
		for (int i = 1; i < dims - 1; i++) sizes[i] = sizes[i - 1] * blocks_shape[i];
		V temp;
		for (int i = 0; i < dims; i++) {
			V idx0 = block_index;
			if (i < dims - 1) idx0 = idx0 / sizes[dims - i - 2];
			if (i > 0) {
				temp = temp * blocks_shape[dims - i - 1];
				idx0 = idx0 - temp;
				if (i != dims - 1) temp = temp + idx0;
			} else {
				temp = idx0;
			}
			out_block[dims - i - 1] = idx0;
		}
	}

	std::vector<V> indices;
	for (int i = 0; i < dims; i++) {
		V idx = out_block[i];
		if (i < block_dim) idx = idx * Const(kernel_->group_size[i]) + BlockThreadId(i);
		if (idx.n->debug_name.empty() && idx.n->op->cls != OpClass::Variable) Named(idx, "index_" + std::to_string(i));
		indices.push_back(idx);
	}

	V inside = indices[0] < shape[0];
	for (int i = 1; i < dims; i++) inside = inside && (indices[i] < shape[i]);
	Named(inside, "is_inside_dispatch");
	OpenDispatchGuard(inside, indices, shape);
	return indices;
}

void KernelBuilder::OpenDispatchGuard(V inside, const std::vector<V>& indices, const std::vector<V>& shape) {
	if ((int)indices.size() != kernel_->dim || indices.size() != shape.size()) throw std::runtime_error("OpenDispatchGuard: one index and one extent per kernel dimension");
	if (kernel_->dispatch_guard) throw std::runtime_error("OpenDispatchGuard: the kernel already has its guard");
	Node* if_node = NewNode("if", TFType_None);
	if_node->debug_name = "if_inside_dispatch";
	Use(if_node, inside);
	Append(if_node);
	scope_stack_.push_back(if_node);
	kernel_->dispatch_guard = if_node;
	for (size_t i = 0; i < indices.size(); i++) {
		kernel_->index_nodes.push_back(indices[i].n);
		kernel_->shape_nodes.push_back(shape[i].n);
	}
}

V KernelBuilder::Load(V memory, V address, TFType type) {
	Node* n = NewNode("load", type);
	n->memory = memory.n;
	memory.n->use_count++;
	n->index = address.n;
	if (address.n) address.n->use_count++;
	n->local_memory_op = memory.n->op->name != std::string("memory");
	Append(n);
	return V(n, this);
}

void KernelBuilder::Store(V memory, V address, V value) {
	Node* n = NewNode("store", TFType_None);
	n->memory = memory.n;
	memory.n->use_count++;
	n->index = address.n;
	if (address.n) address.n->use_count++;
	n->local_memory_op = memory.n->op->name != std::string("memory");
	Use(n, value);
	Append(n);
}

V KernelBuilder::Atomic(const std::string& op, V memory, V address, V value, bool returns_previous) {
	Node* n = NewNode(op, returns_previous ? value.type() : TFType_None);
	if (n->op->cls != OpClass::Memory || op == "load" || op == "store") throw std::runtime_error(op + " is not an atomic operation");
	n->memory = memory.n;
	memory.n->use_count++;
	n->index = address.n;
	if (address.n) address.n->use_count++;
	n->local_memory_op = memory.n->op->name != std::string("memory");
	Use(n, value);
	Append(n);
	return V(n, this);
}

void NodeBuilder::Set(V target, V value) {
	Node* n = NewNode("set", TFType_None);
	n->memory = target.n;
	target.n->use_count++;
	target.n->modified = true;
	Use(n, value);
	Append(n);
}

void KernelBuilder::Barrier() {
	Node* n = NewNode("group_barrier", TFType_None);
	Append(n);
}

void NodeBuilder::Keyword(const std::string& name) {
	Node* n = NewNode(name, TFType_None);
	if (n->op->cls != OpClass::Keyword) throw std::runtime_error(name + " is not a keyword operation");
	Append(n);
}

void NodeBuilder::Loop(V begin, V end, V step, const std::function<void(V)>& body) {
	Node* n = NewNode("loop", TFType_Int);
	Use(n, begin);
	Use(n, end);
	Use(n, step);
	Append(n);
	scope_stack_.push_back(n);
	body(V(n, this));
	scope_stack_.pop_back();
}

void NodeBuilder::If(V cond, const std::function<void()>& body) {
	Node* n = NewNode("if", TFType_None);
	Use(n, cond);
	Append(n);
	scope_stack_.push_back(n);
	body();
	scope_stack_.pop_back();
}

V NodeBuilder::Accumulator(const std::string& idiom_name, TFType type, uint32_t init_bits) {
	Node* n = NewNode("const", type);
	n->data = init_bits;
	n->debug_name = idiom_name;
	n->modified = true;
	Append(n);
	return V(n, this);
}

V KernelBuilder::FlatIndex(const std::vector<V>& indices, const std::vector<V>& shape) {
	if (indices.empty()) return Const(0);
	V flat = indices[0];
	for (size_t i = 1; i < indices.size(); i++) flat = flat * shape[i] + indices[i];
	return flat;
}

V NodeBuilder::Clamp(V x, V lo, V hi) { return Op("clamp", {x, lo, hi}, x.type()); }

Kernel* KernelBuilder::Finish() {
	Kernel* k = kernel_.get();
	program_->kernels_.push_back(std::move(kernel_));
	return k;
}

// ---- operators ---------------------------------------------------------------------------------------

static V Bin(const char* op, V a, V b, bool compare = false) {
	if (!a.b) throw std::runtime_error("operand does not belong to a kernel");
	return a.b->Op(op, {a, b}, compare ? TFType_Bool : a.type());
}

V operator+(V a, V b) { return Bin("add", a, b); }
V operator-(V a, V b) { return Bin("sub", a, b); }
V operator*(V a, V b) { return Bin("mul", a, b); }
V operator/(V a, V b) { return Bin("div", a, b); }
V operator%(V a, V b) { return Bin("mod", a, b); }
V operator<<(V a, V b) { return Bin("lshift", a, b); }
V operator>>(V a, V b) { return Bin("rshift", a, b); }
V operator&(V a, V b) { return Bin("and", a, b); }
V operator|(V a, V b) { return Bin("or", a, b); }
V operator^(V a, V b) { return Bin("xor", a, b); }
V operator&&(V a, V b) { return Bin("and", a, b, true); }
V operator||(V a, V b) { return Bin("or", a, b, true); }
V operator<(V a, V b) { return Bin("lt", a, b, true); }
V operator<=(V a, V b) { return Bin("lte", a, b, true); }
V operator>(V a, V b) { return Bin("gt", a, b, true); }
V operator>=(V a, V b) { return Bin("gte", a, b, true); }
V operator==(V a, V b) { return Bin("eq", a, b, true); }
V operator!=(V a, V b) { return Bin("neq", a, b, true); }
V operator-(V a) { return a.b->Op("neg", {a}, a.type()); }
V operator!(V a) { return a.b->Op("notb", {a}, TFType_Bool); }
V operator~(V a) { return a.b->Op("not", {a}, a.type()); }
V Select(V cond, V a, V b) { return cond.b->Op("ternary", {cond, a, b}, a.type()); }
V ToFloat(V a) { return a.b->Op("float", {a}, TFType_Float); }
V ToInt(V a) { return a.b->Op("int", {a}, TFType_Int); }
V ToUint(V a) { return a.b->Op("uint", {a}, TFType_Uint); }
V AsFloat(V a) { return a.b->Op("asfloat", {a}, TFType_Float); }
V AsUint(V a) { return a.b->Op("asuint", {a}, TFType_Uint); }
V AsInt(V a) { return a.b->Op("asint", {a}, TFType_Int); }

static TFType FnType(const std::string& name, V a) {
	if (name == "pcgf") return TFType_Float;
	return a.type();
}
V Fn(const std::string& name, V a) { return a.b->Op(name, {a}, FnType(name, a)); }
V Fn(const std::string& name, V a, V b) { return a.b->Op(name, {a, b}, FnType(name, a)); }
V Fn(const std::string& name, V a, V b, V c) { return a.b->Op(name, {a, b, c}, FnType(name, a)); }

}  // namespace tfhost
