// HostBuilder: the host part of a program's tree (see tf_ir.h).
#include "host_program.h"
#include "tf_ir.h"

namespace tfhost {

HostBuilder::HostBuilder(Program* program) : NodeBuilder(program) {
	if (program->host_root) throw std::runtime_error("the program already has a host tree");
	Node* root = NewNode("host", TFType_None);
	program->host_root = root;
	scope_stack_.push_back(root);
}

V HostBuilder::DimValue(const Dim& d) {
	if (d.v.n) {
		if (d.v.type() != TFType_Int && d.v.type() != TFType_Uint) throw std::runtime_error("a tensor extent must be an integer host scalar");
		return d.v;
	}
	if (d.constant < 0) throw std::runtime_error("only an input may leave an extent open");
	return Const((int)d.constant);
}

void HostBuilder::SetShape(Node* n, const std::vector<Dim>& shape) {
	std::vector<V> values;
	for (const Dim& d : shape) values.push_back(DimValue(d));
	for (size_t i = values.size(); i-- > 0;) {  // Shape arguments are kept innermost first
		n->shape.push_back(values[i].n);
		values[i].n->use_count++;
	}
}

V HostBuilder::Input(const std::string& name, const std::vector<Dim>& shape, TFType type) {
	if (scope_stack_.size() != 1) throw std::runtime_error("inputs are declared at the top of the host program");
	const int index = (int)program_->input_nodes.size();
	std::vector<Dim> resolved;
	for (size_t i = 0; i < shape.size(); i++) {
		if (!shape[i].v.n && shape[i].constant < 0) {
			Node* s = NewNode("input_shape", TFType_Int);
			s->input_index = index;
			s->input_dim = (int)i;
			s->data = (uint32_t)shape.size();  // dimensions the input is declared with
			s->debug_name = name + "_shape" + std::to_string(i);
			Append(s);
			resolved.push_back(Dim(V(s, this)));
		} else {
			resolved.push_back(shape[i]);
		}
	}
	Node* n = NewNode("memory", type);
	n->input_index = index;
	n->debug_name = name;
	SetShape(n, resolved);
	Append(n);
	program_->input_nodes.push_back(n);
	return V(n, this);
}

std::vector<V> HostBuilder::Shape(V tensor) {
	std::vector<V> out;
	for (size_t i = tensor.n->shape.size(); i-- > 0;) out.push_back(V(tensor.n->shape[i], this));
	return out;
}

V HostBuilder::Allocate(const std::string& name, const std::vector<Dim>& shape, TFType type) {
	// extents first, so that they precede the node that uses them
	std::vector<Dim> resolved;
	for (const Dim& d : shape) resolved.push_back(Dim(DimValue(d)));
	Node* n = NewNode("memory", type);
	n->debug_name = name;
	SetShape(n, resolved);
	Append(n);
	return V(n, this);
}

static void RequireTensor(V t, const char* what) {
	const std::string op = t.n ? t.n->op->name : "";
	if (op != "memory" && op != "reshape" && op != "assert") throw std::runtime_error(std::string(what) + " needs a host tensor");
}

void HostBuilder::Deallocate(V tensor) {
	RequireTensor(tensor, "deallocate");
	Node* n = NewNode("deallocate", TFType_None);
	n->memory = tensor.n;
	tensor.n->use_count++;
	Append(n);
}

Node* HostBuilder::TensorNode(const std::string& op, V source, const std::string& name, const std::vector<Dim>& shape, TFType type) {
	RequireTensor(source, op.c_str());
	std::vector<Dim> resolved;
	for (const Dim& d : shape) resolved.push_back(Dim(DimValue(d)));
	Node* n = NewNode(op, type);
	n->debug_name = name;
	n->memory = source.n;
	source.n->use_count++;
	SetShape(n, resolved);
	Append(n);
	return n;
}

V HostBuilder::Reshape(V tensor, const std::string& name, const std::vector<Dim>& shape, TFType type) { return V(TensorNode("reshape", tensor, name, shape, type), this); }
V HostBuilder::AssertTensor(V tensor, const std::string& name, const std::vector<Dim>& shape, TFType type) { return V(TensorNode("assert", tensor, name, shape, type), this); }

V HostBuilder::Read(V tensor, V index, TFType type) {
	RequireTensor(tensor, "read");
	Node* n = NewNode("load", type);
	n->memory = tensor.n;
	tensor.n->use_count++;
	n->index = index.n;
	if (index.n) index.n->use_count++;
	Append(n);
	return V(n, this);
}

void HostBuilder::Write(V tensor, V index, V value) {
	RequireTensor(tensor, "write");
	Node* n = NewNode("store", TFType_None);
	n->memory = tensor.n;
	tensor.n->use_count++;
	n->index = index.n;
	if (index.n) index.n->use_count++;
	Use(n, value);
	Append(n);
}

void HostBuilder::Dispatch(Kernel* kernel, const std::vector<V>& read_write, const std::vector<V>& read_only, const std::vector<V>& variables,
                           const std::vector<Dim>& shape, std::vector<int> group) {
	if (!kernel) throw std::runtime_error("dispatch of a null kernel");
	const std::string label = kernel->primitive.empty() ? "kernel" : kernel->primitive;
	if (kernel->primitive.empty()) {
		if (read_write.size() != kernel->read_write_memory.size() || read_only.size() != kernel->read_only_memory.size())
			throw std::runtime_error("dispatch: the " + label + " binds " + std::to_string(kernel->read_write_memory.size()) + " + " + std::to_string(kernel->read_only_memory.size()) +
			                         " tensors, the dispatch passes " + std::to_string(read_write.size()) + " + " + std::to_string(read_only.size()));
		if (variables.size() != kernel->variables.size())
			throw std::runtime_error("dispatch: the kernel reads " + std::to_string(kernel->variables.size()) + " host scalars, the dispatch passes " + std::to_string(variables.size()));
		for (size_t i = 0; i < variables.size(); i++)
			if (variables[i].type() != kernel->variables[i].type)
				throw std::runtime_error("dispatch: host scalar " + kernel->variables[i].name + " has another type than the kernel's variable");
		if ((int)shape.size() != kernel->dim) throw std::runtime_error("dispatch: the shape does not have the kernel's dimensionality");
	} else {
		if (read_write.size() + read_only.size() != kernel->primitive_tensors || variables.size() != kernel->primitive_variables)
			throw std::runtime_error("dispatch: " + label + " takes " + std::to_string(kernel->primitive_tensors) + " tensors and " + std::to_string(kernel->primitive_variables) + " scalars");
	}
	for (const V& t : read_write) RequireTensor(t, "dispatch");
	for (const V& t : read_only) RequireTensor(t, "dispatch");
	if (group.empty()) group = kernel->group_size;
	if (group.empty()) group = shape.size() == 1 ? std::vector<int>{256} : shape.size() == 2 ? std::vector<int>{16, 16} : std::vector<int>{8, 8, 8};
	if (group.size() > shape.size()) throw std::runtime_error("dispatch: more group dimensions than shape dimensions");

	std::vector<Dim> resolved;
	for (const Dim& d : shape) resolved.push_back(Dim(DimValue(d)));
	Node* n = NewNode("kernel", TFType_None);
	n->dispatch = (int)program_->dispatches.size();
	DispatchBinding binding;
	binding.kernel = kernel;
	binding.group = group;
	for (const V& t : read_write) { binding.read_write.push_back(t.n); t.n->use_count++; }
	for (const V& t : read_only) { binding.read_only.push_back(t.n); t.n->use_count++; }
	for (const V& v : variables) { binding.variables.push_back(v.n); v.n->use_count++; }
	program_->dispatches.push_back(std::move(binding));
	SetShape(n, resolved);
	Append(n);
}

void HostBuilder::RegionBegin(const std::string& name) {
	Node* n = NewNode("region_begin", TFType_None);
	n->debug_name = name;
	Append(n);
}
void HostBuilder::RegionEnd(const std::string& name) {
	Node* n = NewNode("region_end", TFType_None);
	n->debug_name = name;
	Append(n);
}
void HostBuilder::AssertValue(const std::string& name, V condition) {
	Node* n = NewNode("assert_value", TFType_None);
	n->debug_name = name;
	Use(n, condition);
	Append(n);
}
void HostBuilder::PrintValue(const std::string& name, V value) {
	Node* n = NewNode("print_value", TFType_None);
	n->debug_name = name;
	Use(n, value);
	Append(n);
}

void HostBuilder::Output(V tensor) {
	RequireTensor(tensor, "an output");
	program_->output_nodes.push_back(tensor.n);
}

void HostBuilder::Finish() {
	program_->input_count = (int)program_->input_nodes.size();
	program_->output_count = (int)program_->output_nodes.size();
	std::shared_ptr<HostCode> code = LowerHostProgram(program_);
	program_->host_code = code;
	program_->execute_callback = [code](TFTensor* in, TFTensor* out, TFRuntime runtime) -> int { return RunHostCode(*code, in, out, runtime); };
}

}  // namespace tfhost
