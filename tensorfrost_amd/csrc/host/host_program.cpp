#include "host_program.h"

#include <cstdio>
#include <sstream>
#include <unordered_map>

namespace tfhost {

// ---- lowering ---------------------------------------------------------------------------------------------------

namespace {

bool IsTensorOp(const Node* n) {
	const std::string op = n->op->name;
	return op == "memory" || op == "reshape" || op == "assert";
}

struct Lowering {
	const Program* program;
	HostCode* code;
	std::unordered_map<const Node*, int> scalar_slot, tensor_slot;
	struct LoopScope {
		std::vector<size_t> breaks, continues;  // instructions whose jump target is patched when the loop closes
	};
	std::vector<LoopScope> loops;

	int NewScalar(const Node* n) {
		auto it = scalar_slot.find(n);
		if (it != scalar_slot.end()) return it->second;
		const int slot = code->scalar_slots++;
		scalar_slot[n] = slot;
		return slot;
	}
	int NewTensor(const Node* n) {
		const int slot = code->tensor_slots++;
		tensor_slot[n] = slot;
		return slot;
	}
	int Scalar(const Node* n, const Node* user) const {
		auto it = n ? scalar_slot.find(n) : scalar_slot.end();
		if (it == scalar_slot.end())
			throw std::runtime_error("Host program " + program->program_name + ": " + std::string(user->op->name) + " uses a host scalar that no earlier node of the host tree defines");
		return it->second;
	}
	int Tensor(const Node* n, const Node* user) const {
		auto it = n ? tensor_slot.find(n) : tensor_slot.end();
		if (it == tensor_slot.end())
			throw std::runtime_error("Host program " + program->program_name + ": " + std::string(user->op->name) + " names a tensor that no earlier node of the host tree defines");
		return it->second;
	}
	HostInstr& Emit(HostInstr::Code c) {
		code->instrs.emplace_back();
		code->instrs.back().code = c;
		return code->instrs.back();
	}
	std::vector<int> ShapeSlots(const Node* n) {  // outermost first
		std::vector<int> s;
		for (size_t i = n->shape.size(); i-- > 0;) s.push_back(Scalar(n->shape[i], n));
		code->max_dims = std::max(code->max_dims, s.size());
		return s;
	}

	void Scope(const Node* scope) {
		for (const Node* n : scope->children) Statement(n);
	}

	void Statement(const Node* n) {
		const std::string op = n->op->name;
		switch (n->op->cls) {
			case OpClass::Constant: {
				HostInstr& i = Emit(HostInstr::Const);
				i.dst = NewScalar(n);
				i.imm = n->data;
				i.type = n->type;
				return;
			}
			case OpClass::Operator:
			case OpClass::UnaryOperator:
			case OpClass::Function:
			case OpClass::TypeCast:
			case OpClass::TypeReinterpret:
			case OpClass::TernaryOperator:
			case OpClass::Copy: {
				if (op == "group_barrier") throw std::runtime_error("Host program " + program->program_name + ": group_barrier outside a kernel");
				if (n->inputs.empty() || n->inputs.size() > 3) throw std::runtime_error("Host program " + program->program_name + ": " + op + " with " + std::to_string(n->inputs.size()) + " inputs");
				const TFType operand = n->inputs[n->op->cls == OpClass::TernaryOperator ? 1 : 0]->type;
				ScalarFn fn = FindScalarFn(op, operand, n->type);
				if (!fn) throw std::runtime_error("Host program " + program->program_name + ": the host cannot evaluate " + op + " on this operand type");
				const int a = Scalar(n->inputs[0], n);
				const int b = n->inputs.size() > 1 ? Scalar(n->inputs[1], n) : -1;
				const int c = n->inputs.size() > 2 ? Scalar(n->inputs[2], n) : -1;
				HostInstr& i = Emit(HostInstr::Scalar);
				i.dst = NewScalar(n);
				i.a = a;
				i.b = b;
				i.c = c;
				i.fn = fn;
				i.type = n->type;
				i.name = op;
				return;
			}
			case OpClass::Set: {
				HostInstr& i = Emit(HostInstr::Copy);
				i.dst = Scalar(n->memory, n);
				i.a = Scalar(n->inputs.at(0), n);
				return;
			}
			case OpClass::Keyword: {
				if (loops.empty() || op == "discard") throw std::runtime_error("Host program " + program->program_name + ": " + op + " outside a host loop");
				Emit(HostInstr::Jump);
				(op == "break" ? loops.back().breaks : loops.back().continues).push_back(code->instrs.size() - 1);
				return;
			}
			case OpClass::Memory: {
				if (op == "load") {
					const int t = Tensor(n->memory, n), idx = n->index ? Scalar(n->index, n) : -1;
					HostInstr& i = Emit(HostInstr::Read);
					i.dst = NewScalar(n);
					i.a = t;
					i.b = idx;
					i.type = n->type;
				} else if (op == "store") {
					const int t = Tensor(n->memory, n), idx = n->index ? Scalar(n->index, n) : -1, v = Scalar(n->inputs.at(0), n);
					HostInstr& i = Emit(HostInstr::Write);
					i.a = t;
					i.b = idx;
					i.c = v;
				} else {
					throw std::runtime_error("Scatter operation not supported in non-kernel mode");  // Generators.cpp:459-461
				}
				return;
			}
			default: break;
		}

		// OpClass::Special
		if (op == "loop") {
			const int begin = Scalar(n->inputs.at(0), n), end = Scalar(n->inputs.at(1), n), step = Scalar(n->inputs.at(2), n);
			const int counter = NewScalar(n);
			const size_t enter = code->instrs.size();
			{
				HostInstr& i = Emit(HostInstr::LoopEnter);
				i.dst = counter;
				i.a = begin;
				i.b = end;
			}
			loops.emplace_back();
			const size_t body = code->instrs.size();
			Scope(n);
			const size_t next = code->instrs.size();
			{
				HostInstr& i = Emit(HostInstr::LoopNext);
				i.dst = counter;
				i.b = end;
				i.c = step;
				i.jump = (int)body;
			}
			const size_t after = code->instrs.size();
			code->instrs[enter].jump = (int)after;
			for (size_t at : loops.back().breaks) code->instrs[at].jump = (int)after;
			for (size_t at : loops.back().continues) code->instrs[at].jump = (int)next;
			loops.pop_back();
		} else if (op == "if") {
			const size_t test = code->instrs.size();
			Emit(HostInstr::JumpIfNot).a = Scalar(n->inputs.at(0), n);
			Scope(n);
			code->instrs[test].jump = (int)code->instrs.size();
		} else if (op == "input_shape") {
			HostInstr& i = Emit(HostInstr::InputShape);
			i.dst = NewScalar(n);
			i.input = n->input_index;
			i.dim = n->input_dim;
			i.expected_dims = (int)n->data;
			i.name = program->input_nodes.at(n->input_index)->debug_name;
			i.type = TFType_Int;
		} else if (op == "memory") {
			std::vector<int> shape = ShapeSlots(n);
			HostInstr& i = Emit(n->input_index >= 0 ? HostInstr::CheckInput : HostInstr::Allocate);
			i.dst = NewTensor(n);
			i.input = n->input_index;
			i.name = n->debug_name;
			i.shape = std::move(shape);
			i.type = n->type;
		} else if (op == "reshape" || op == "assert") {
			std::vector<int> shape = ShapeSlots(n);
			const int src = Tensor(n->memory, n);
			HostInstr& i = Emit(op == "reshape" ? HostInstr::Reshape : HostInstr::AssertTensor);
			i.dst = NewTensor(n);
			i.a = src;
			i.name = n->debug_name;
			i.shape = std::move(shape);
			i.type = n->type;
		} else if (op == "deallocate") {
			Emit(HostInstr::Deallocate).a = Tensor(n->memory, n);
		} else if (op == "kernel") {
			const DispatchBinding& d = program->dispatches.at(n->dispatch);
			std::vector<int> shape = ShapeSlots(n);
			HostInstr i;
			i.code = HostInstr::Dispatch;
			i.kernel = d.kernel;
			for (const Node* t : d.read_write) i.tensors.push_back(Tensor(t, n));
			i.read_write = i.tensors.size();
			for (const Node* t : d.read_only) i.tensors.push_back(Tensor(t, n));
			for (const Node* v : d.variables) i.variables.push_back(Scalar(v, n));
			i.shape = std::move(shape);
			i.group = d.group;
			code->max_tensors = std::max(code->max_tensors, i.tensors.size());
			code->max_variables = std::max(code->max_variables, i.variables.size() + 1);
			code->instrs.push_back(std::move(i));
		} else if (op == "region_begin" || op == "region_end") {
			Emit(op == "region_begin" ? HostInstr::RegionBegin : HostInstr::RegionEnd).name = n->debug_name;
		} else if (op == "assert_value" || op == "print_value") {
			const int a = Scalar(n->inputs.at(0), n);
			HostInstr& i = Emit(op == "assert_value" ? HostInstr::AssertValue : HostInstr::PrintValue);
			i.a = a;
			i.name = n->debug_name;
			i.type = n->inputs[0]->type;
		} else {
			throw std::runtime_error("Host program " + program->program_name + ": " + op + " cannot appear on the host");
		}
	}
};

}  // namespace

std::shared_ptr<HostCode> LowerHostProgram(const Program* program) {
	if (!program->host_root) throw std::runtime_error("Program " + program->program_name + " has no host tree");
	auto code = std::make_shared<HostCode>();
	code->program_name = program->program_name;
	code->inputs = (int)program->input_nodes.size();
	code->outputs = (int)program->output_nodes.size();
	Lowering lower{program, code.get(), {}, {}, {}};
	lower.Scope(program->host_root);
	for (size_t i = 0; i < program->output_nodes.size(); i++) {
		auto it = lower.tensor_slot.find(program->output_nodes[i]);
		if (it == lower.tensor_slot.end()) throw std::runtime_error("Host program " + program->program_name + ": output " + std::to_string(i) + " is no tensor of the host tree");
		HostInstr& out = lower.Emit(HostInstr::Output);
		out.imm = (uint32_t)i;
		out.a = it->second;
	}
	return code;
}

// ---- execution --------------------------------------------------------------------------------------------------

namespace {

const char* TypeLabel(TFType t) {
	switch (t) {
		case TFType_Float: return "Float";
		case TFType_Uint: return "Uint";
		case TFType_Int: return "Int";
		case TFType_Bool: return "Bool";
		default: return "None";
	}
}

size_t ElementCount(const size_t* shape, size_t dim) {
	size_t n = 1;
	for (size_t i = 0; i < dim; i++) n *= shape[i];
	return n;
}

// The tensor must have exactly this element type, rank and extents (tf.check_tensor, CPP.cpp:431-448).
void RequireTensorIs(const TFTensor& tensor, const std::string& name, const size_t* shape, size_t dim, TFType type) {
	if (tensor.format.type != type || tensor.format.size != 32)
		throw std::runtime_error("Invalid type for " + name + ". Expected " + TypeLabel(type) + ", got " + TypeLabel(tensor.format.type));
	if (tensor.dim != dim) throw std::runtime_error("Invalid number of dimensions for " + name + ". Expected " + std::to_string(dim) + ", got " + std::to_string(tensor.dim));
	for (size_t i = 0; i < dim; i++)
		if (tensor.shape[i] != shape[i] || shape[i] < 1)
			throw std::runtime_error("Invalid shape for dimension " + std::to_string(i) + " in " + name + ". Expected " + std::to_string(shape[i]) + ", got " + std::to_string(tensor.shape[i]));
}

}  // namespace

int RunHostCode(const HostCode& code, TFTensor* in, TFTensor* out, TFRuntime runtime) {
	std::vector<uint32_t> s((size_t)code.scalar_slots);
	std::vector<TFTensor> t((size_t)code.tensor_slots);
	std::vector<TFTensor> tensor_args(code.max_tensors);
	std::vector<uint32_t> variable_args(code.max_variables);
	std::vector<size_t> dims(code.max_dims);
	void* user = runtime.custom_data;

	// Extents come from signed host scalars; a negative one must not wrap into a huge size_t.
	auto gather = [&](const HostInstr& i, const char* what) -> size_t {
		for (size_t d = 0; d < i.shape.size(); d++) {
			const int32_t v = (int32_t)s[i.shape[d]];
			if (v < 1 && i.code == HostInstr::Allocate)
				throw std::runtime_error("Invalid shape on dimension " + std::to_string(d) + " for " + i.name + ". Expected positive integer, got " + std::to_string(v));
			if (v < 0) throw std::runtime_error(std::string("Negative extent on dimension ") + std::to_string(d) + " of " + what + " " + i.name);
			dims[d] = (size_t)v;
		}
		return i.shape.size();
	};

	const HostInstr* instrs = code.instrs.data();
	const size_t count = code.instrs.size();
	size_t pc = 0;
	while (pc < count) {
		const HostInstr& i = instrs[pc++];
		switch (i.code) {
			case HostInstr::Const: s[i.dst] = i.imm; break;
			case HostInstr::Scalar: s[i.dst] = i.fn(s[i.a], i.b >= 0 ? s[i.b] : 0u, i.c >= 0 ? s[i.c] : 0u); break;
			case HostInstr::Copy: s[i.dst] = s[i.a]; break;
			case HostInstr::InputShape: {
				const TFTensor& tensor = in[i.input];
				if ((int)tensor.dim != i.expected_dims)
					throw std::runtime_error("Invalid number of dimensions for " + i.name + ". Expected " + std::to_string(i.expected_dims) + ", got " + std::to_string(tensor.dim));
				s[i.dst] = (uint32_t)(int32_t)tensor.shape[i.dim];
				break;
			}
			case HostInstr::CheckInput: {
				const size_t dim = gather(i, "input");
				RequireTensorIs(in[i.input], i.name, dims.data(), dim, i.type);
				t[i.dst] = in[i.input];
				break;
			}
			case HostInstr::Allocate: {
				const size_t dim = gather(i, "tensor");
				t[i.dst] = runtime.alloc(i.name.c_str(), dims.data(), dim, TFDataFormat{i.type, 32}, user);
				break;
			}
			case HostInstr::Deallocate: runtime.dealloc(t[i.a], user); break;
			case HostInstr::Reshape: {
				// A second header on the same buffer. Like every tensor header the runtime hands out, the extents
				// array lives as long as the process (CPP.cpp:450-463, TensorMemory.cpp:69-82).
				const size_t dim = gather(i, "reshape");
				const TFTensor& src = t[i.a];
				const size_t have = ElementCount(src.shape, src.dim), want = ElementCount(dims.data(), dim);
				if (have != want) throw std::runtime_error("Cannot reshape " + i.name + ", expected " + std::to_string(want) + " elements, while input has " + std::to_string(have));
				size_t* kept = new size_t[dim];
				for (size_t d = 0; d < dim; d++) kept[d] = dims[d];
				t[i.dst] = TFTensor{src.buffer, TFDataFormat{i.type, 32}, dim, kept};
				break;
			}
			case HostInstr::AssertTensor: {
				const size_t dim = gather(i, "tensor");
				RequireTensorIs(t[i.a], i.name, dims.data(), dim, i.type);
				t[i.dst] = t[i.a];
				break;
			}
			case HostInstr::Read: s[i.dst] = runtime.readback(t[i.a], i.b >= 0 ? (size_t)(int32_t)s[i.b] : 0, user); break;
			case HostInstr::Write: runtime.writeback(t[i.a], i.b >= 0 ? (size_t)(int32_t)s[i.b] : 0, s[i.c], user); break;
			case HostInstr::Dispatch: {
				// Every tensor travels in the read-write list, written ones first, and the variable block ends with
				// the group index offset, 0 (CPP.cpp:482-501). Outer extents multiply; the innermost group.size()
				// extents are divided by their group size, rounding up (CPP.cpp:503-515).
				const size_t n_tensors = i.tensors.size(), n_variables = i.variables.size();
				for (size_t k = 0; k < n_tensors; k++) tensor_args[k] = t[i.tensors[k]];
				for (size_t k = 0; k < i.read_write; k++) tensor_args[k].buffer->up_to_date = false;
				for (size_t k = 0; k < n_variables; k++) variable_args[k] = s[i.variables[k]];
				variable_args[n_variables] = 0;
				const size_t dim = gather(i, "dispatch of kernel"), grouped = i.group.size();
				size_t groups = 1;
				for (size_t d = 0; d < dim; d++) {
					const size_t from_inner = dim - 1 - d;
					groups *= from_inner < grouped ? (dims[d] + (size_t)i.group[from_inner] - 1) / (size_t)i.group[from_inner] : dims[d];
				}
				TFDispatchInfo info{i.kernel->kernel_id_, n_tensors, tensor_args.data(), 0, nullptr, n_variables + 1, variable_args.data(), groups};
				runtime.dispatch(info, user);
				break;
			}
			case HostInstr::RegionBegin:
				if (runtime.region) runtime.region(i.name.c_str(), true, user);
				break;
			case HostInstr::RegionEnd:
				if (runtime.region) runtime.region(i.name.c_str(), false, user);
				break;
			case HostInstr::AssertValue:
				if (!s[i.a]) throw std::runtime_error("Assertion failed: " + i.name);
				break;
			case HostInstr::PrintValue: {
				const uint32_t w = s[i.a];
				float f;
				__builtin_memcpy(&f, &w, 4);
				if (i.type == TFType_Float)
					printf("%s: %g\n", i.name.c_str(), (double)f);
				else if (i.type == TFType_Int)
					printf("%s: %d\n", i.name.c_str(), (int)w);
				else
					printf("%s: %u\n", i.name.c_str(), w);
				break;
			}
			case HostInstr::LoopEnter:
				s[i.dst] = s[i.a];
				if (!((int32_t)s[i.dst] < (int32_t)s[i.b])) pc = (size_t)i.jump;
				break;
			case HostInstr::LoopNext:
				s[i.dst] = (uint32_t)((int32_t)s[i.dst] + (int32_t)s[i.c]);
				if ((int32_t)s[i.dst] < (int32_t)s[i.b]) pc = (size_t)i.jump;
				break;
			case HostInstr::JumpIfNot:
				if (!s[i.a]) pc = (size_t)i.jump;
				break;
			case HostInstr::Jump: pc = (size_t)i.jump; break;
			case HostInstr::Output: out[i.imm] = t[i.a]; break;
		}
	}
	return 0;
}

// ---- listing ----------------------------------------------------------------------------------------------------

std::string PrintHostCode(const HostCode& code) {
	std::ostringstream o;
	auto slots = [&](const std::vector<int>& v, const char* prefix, size_t from, size_t to) {
		std::string r = "{";
		for (size_t k = from; k < to; k++) r += (k > from ? ", " : "") + std::string(prefix) + std::to_string(v[k]);
		return r + "}";
	};
	for (size_t pc = 0; pc < code.instrs.size(); pc++) {
		const HostInstr& i = code.instrs[pc];
		o << pc << ": ";
		switch (i.code) {
			case HostInstr::Const: {
				float f;
				__builtin_memcpy(&f, &i.imm, 4);
				o << "s" << i.dst << " = ";
				if (i.type == TFType_Float)
					o << f;
				else if (i.type == TFType_Int)
					o << (int32_t)i.imm;
				else
					o << i.imm << "u";
				break;
			}
			case HostInstr::Scalar:
				o << "s" << i.dst << " = " << i.name << "(s" << i.a;
				if (i.b >= 0) o << ", s" << i.b;
				if (i.c >= 0) o << ", s" << i.c;
				o << ")";
				break;
			case HostInstr::Copy: o << "s" << i.dst << " = s" << i.a; break;
			case HostInstr::InputShape: o << "s" << i.dst << " = in[" << i.input << "].shape[" << i.dim << "]"; break;
			case HostInstr::CheckInput: o << "t" << i.dst << " = in[" << i.input << "]; tf.check_tensor(t" << i.dst << ", \"" << i.name << "\", " << slots(i.shape, "s", 0, i.shape.size()) << ", " << TypeLabel(i.type) << ")"; break;
			case HostInstr::Allocate: o << "t" << i.dst << " = tf.allocate(\"" << i.name << "\", " << slots(i.shape, "s", 0, i.shape.size()) << ", " << TypeLabel(i.type) << ")"; break;
			case HostInstr::Deallocate: o << "tf.deallocate(t" << i.a << ")"; break;
			case HostInstr::Reshape: o << "t" << i.dst << " = tf.reshape(t" << i.a << ", \"" << i.name << "\", " << slots(i.shape, "s", 0, i.shape.size()) << ", " << TypeLabel(i.type) << ")"; break;
			case HostInstr::AssertTensor: o << "t" << i.dst << " = tf.assert_tensor(t" << i.a << ", \"" << i.name << "\", " << slots(i.shape, "s", 0, i.shape.size()) << ", " << TypeLabel(i.type) << ")"; break;
			case HostInstr::Read: o << "s" << i.dst << " = tf.read(t" << i.a << ", " << (i.b >= 0 ? "s" + std::to_string(i.b) : std::string("0")) << ")"; break;
			case HostInstr::Write: o << "tf.write(t" << i.a << ", " << (i.b >= 0 ? "s" + std::to_string(i.b) : std::string("0")) << ", s" << i.c << ")"; break;
			case HostInstr::Dispatch: {
				std::string group = "{";
				for (size_t k = 0; k < i.group.size(); k++) group += (k ? ", " : "") + std::to_string(i.group[k]);
				o << "tf.dispatch(" << i.kernel->kernel_id_ << ", " << slots(i.tensors, "t", 0, i.read_write) << ", " << slots(i.tensors, "t", i.read_write, i.tensors.size()) << ", "
				  << slots(i.variables, "s", 0, i.variables.size()) << ", " << slots(i.shape, "s", 0, i.shape.size()) << ", " << group << "})";
				break;
			}
			case HostInstr::RegionBegin: o << "tf.region_begin(\"" << i.name << "\")"; break;
			case HostInstr::RegionEnd: o << "tf.region_end(\"" << i.name << "\")"; break;
			case HostInstr::AssertValue: o << "tf.assert_value(\"" << i.name << "\", s" << i.a << ")"; break;
			case HostInstr::PrintValue: o << "tf.print_value(\"" << i.name << "\", s" << i.a << ")"; break;
			case HostInstr::LoopEnter: o << "s" << i.dst << " = s" << i.a << "; if (!(s" << i.dst << " < s" << i.b << ")) goto " << i.jump; break;
			case HostInstr::LoopNext: o << "s" << i.dst << " += s" << i.c << "; if (s" << i.dst << " < s" << i.b << ") goto " << i.jump; break;
			case HostInstr::JumpIfNot: o << "if (!s" << i.a << ") goto " << i.jump; break;
			case HostInstr::Jump: o << "goto " << i.jump; break;
			case HostInstr::Output: o << "out[" << i.imm << "] = t" << i.a; break;
		}
		o << "\n";
	}
	return o.str();
}

}  // namespace tfhost
