// Runs the kernel importer a TensorFrost build would use (KernelImporter, langs/tree_import.h) and the search for the
// thread indices and the dispatch guard (DeriveKernelGeometry, kernel_geometry.cpp) on every kernel this repository
// can build: the kernel is exported into a mirror of the compiler's classes (compiler_tree_mirror.h), imported from
// there, and the imported kernel has to be emitted to the same text, with the same launch decisions, idiom match and
// sort role, as the kernel it came from.
#include <cstring>
#include <functional>
#include <sstream>

#include "compiler_tree_mirror.h"
#include "hip_generator.h"
#include "langs/tree_import.h"
#include "registry.h"
#include "sort_composition.h"

namespace mirror {

namespace {

struct Exporter {
	Exported* out;
	std::unordered_map<const tfhost::Node*, Node*> at;

	const Operation* Op(const std::string& name) {
		auto& slot = out->operations[name];
		if (!slot) slot = std::make_unique<Operation>(Operation{name});
		return slot.get();
	}
	Node* New() {
		out->nodes.push_back(std::make_unique<Node>());
		return out->nodes.back().get();
	}
	Node* Real(const tfhost::Node* from, const std::string& op) {
		Node* n = New();
		n->flags.remove(NodeProp::Placeholder);
		n->op = Op(op);
		n->name = op;
		n->format.type = from->type;
		n->data = {from->data};
		n->debug_name = from->debug_name;
		n->var_name = from->debug_name;
		if (from->modified) n->flags.set(NodeProp::Modified);
		if (from->local_memory_op) n->flags.set(NodeProp::LocalMemoryOp);
		at[from] = n;
		return n;
	}
	// The children of `from` as a child / next list under `to`, ended by a placeholder.
	void Children(const tfhost::Node* from, Node* to, const tfhost::Node* guard) {
		Node* prev = nullptr;
		for (const tfhost::Node* c : from->children) {
			Node* n = Real(c, c->op->name);
			n->parent = to;
			n->prev = prev;
			(prev ? prev->next : to->child) = n;
			prev = n;
			Children(c, n, guard);
		}
		Node* end = New();  // stays a placeholder
		end->parent = to;
		end->prev = prev;
		if (prev && from->children.back() == guard) {
			prev->next = nullptr;  // IR::FinalizeMemoryIndexing leaves the guard without a successor
		} else {
			(prev ? prev->next : to->child) = end;
		}
	}
	void Arguments(const tfhost::Node* from) {
		Node* n = at.at(from);
		for (size_t i = 0; i < from->inputs.size(); i++) n->args.AddArgument(ArgType::Input, (int)i, at.at(from->inputs[i]));
		if (from->index) n->args.AddArgument(ArgType::Index, 0, at.at(from->index));
		if (from->memory) n->args.AddArgument(ArgType::Memory, 0, at.at(from->memory));
		for (const tfhost::Node* c : from->children) Arguments(c);
	}
};

}  // namespace

std::unique_ptr<Exported> ExportKernel(const tfhost::Kernel* kernel, bool reverse_slots) {
	auto out = std::make_unique<Exported>();
	Exporter e{out.get(), {}};
	auto slot = [&](size_t i, size_t n) { return reverse_slots ? n - 1 - i : i; };
	// Host-side nodes the kernel is bound to.
	for (size_t i = 0; i < kernel->read_write_memory.size(); i++)
		out->kernel.read_write_memory[e.Real(kernel->read_write_memory[i], "memory")] = slot(i, kernel->read_write_memory.size());
	for (size_t i = 0; i < kernel->read_only_memory.size(); i++)
		out->kernel.read_only_memory[e.Real(kernel->read_only_memory[i], "memory")] = slot(i, kernel->read_only_memory.size());
	for (size_t i = 0; i < kernel->variables.size(); i++) {
		// a host scalar: whatever operation computed it on the host; the importer must not care
		Node* n = e.Real(kernel->variables[i].node, "add");
		n->var_name = kernel->variables[i].name;
		out->kernel.variables[n] = slot(i, kernel->variables.size());
	}
	Node* root = e.Real(kernel->root, "kernel");
	root->group_size = kernel->group_size;
	out->kernel.root = root;
	e.Children(kernel->root, root, kernel->dispatch_guard);
	e.Arguments(kernel->root);
	for (const tfhost::Node* g : kernel->group_memory) out->kernel.group_memory.insert(e.at.at(g));
	// The kernel node's Shape arguments: the host scalar where the extent is one, else a host-side constant.
	for (size_t d = 0; d < (size_t)kernel->dim; d++) {
		Node* extent = nullptr;
		if (d < kernel->shape_nodes.size()) {
			for (auto& v : kernel->variables)
				if (v.node == kernel->shape_nodes[d]) extent = e.at.at(v.node);
		}
		if (!extent) {
			extent = e.New();
			extent->flags.remove(NodeProp::Placeholder);
			extent->op = e.Op("const");
			extent->format.type = TFType_Int;
			extent->data = {0};
		}
		out->kernel.shape[{ArgType::Shape, (int)d}] = extent;
	}
	return out;
}

}  // namespace mirror

namespace {

using namespace tfhost;

std::string Describe(const HipKernelInfo& i) {
	std::ostringstream o;
	o << "idiom=" << i.idiom << " threads=" << i.hip_threads << " groups/block=" << i.groups_per_hip_block << " blocks/tile=" << i.hip_blocks_per_tile
	  << " lanes=" << i.lanes_per_thread << " tplg=" << i.threads_per_lane_group << " serial=" << i.serial_load_loops << " scalar=" << i.scalar_entry << ":"
	  << i.scalar_hip_threads << ":" << i.scalar_groups_per_hip_block << " batch=" << i.batch_entry << ":" << i.batch_capacity << ":" << i.batch_call_bytes
	  << " rw=" << i.read_write_count << " tensors=" << i.tensor_count << " vars=" << i.variable_count << " sort=" << i.sort.copies.size() << "/" << i.sort.copies_only << "/" << i.sort.digits.size() << "/" << i.sort.scatter << ":" << i.sort.keys_out << i.sort.values_out << i.sort.keys_in << i.sort.values_in << ":" << i.sort.scatter_mask << " tail=" << i.has_tail_kernel
	  << " dense=" << i.has_dense_variant << " match=" << (int)i.match.kind << "/" << i.match.op << "/" << i.match.is_float << " buffers=";
	for (int b : i.match.buffers) o << b << ",";
	o << " dims=" << i.match.dims.size() << " conditions=" << i.match.conditions.size() << " group=";
	for (int g : i.group_size) o << g << ",";
	return o.str();
}

// Position of a node in a pre-order walk of the kernel's tree (bindings first): how nodes of two copies are compared.
void Number(const Kernel* k, std::unordered_map<const Node*, int>& number) {
	int next = 0;
	for (const Node* m : k->MemoryBindings()) number[m] = next++;
	for (auto& v : k->variables) number[v.node] = next++;
	std::function<void(const Node*)> walk = [&](const Node* n) {
		number[n] = next++;
		for (const Node* c : n->children) walk(c);
	};
	walk(k->root);
}

std::string Geometry(const Kernel* k) {
	std::unordered_map<const Node*, int> number;
	Number(k, number);
	std::ostringstream o;
	o << "dim=" << k->dim << " group=";
	for (int g : k->group_size) o << g << ",";
	o << " guard=" << (k->dispatch_guard ? number.at(k->dispatch_guard) : -1) << " index=";
	for (const Node* n : k->index_nodes) o << number.at(n) << ",";
	o << " shape=";
	for (const Node* n : k->shape_nodes) o << number.at(n) << ",";
	return o.str();
}

// The checks for one kernel that has not been emitted yet. Returns "" or what differs.
std::string RoundTrip(Program* program, Kernel* kernel, const std::string& label) {
	// 1. the derived fields, found again in a copy that has lost them
	{
		Kernel* copy = CloneKernel(program, kernel);
		const std::string before = Geometry(copy);
		const bool had_guard = copy->dispatch_guard != nullptr;
		copy->index_nodes.clear();
		copy->shape_nodes.clear();
		copy->dispatch_guard = nullptr;
		if (had_guard) {  // a kernel without a guard keeps what its builder said: its tree has nothing to find
			copy->dim = 0;
			copy->group_size.clear();
		}
		DeriveKernelGeometry(copy);
		const std::string after = Geometry(copy);
		if (before != after) return label + ": DeriveKernelGeometry found [" + after + "], the builder recorded [" + before + "]";
	}
	// 2. through the compiler's classes and back
	Program imported_program;
	std::unique_ptr<mirror::Exported> exported = mirror::ExportKernel(kernel, false);
	KernelImporter<mirror::Tree> importer(&imported_program);
	Kernel* imported = importer.Import(&exported->kernel);
	if (Geometry(imported) != Geometry(kernel)) return label + ": imported geometry [" + Geometry(imported) + "] differs from [" + Geometry(kernel) + "]";
	if (KernelFingerprint(imported) != KernelFingerprint(kernel)) return label + ": the imported kernel has another fingerprint";

	size_t next_id = 1;
	auto give_id = [&next_id](Kernel* k) {
		k->kernel_id_ = next_id++;
		k->kernel_name_ = "kernel_" + std::to_string(k->kernel_id_);
	};
	Kernel* original = CloneKernel(program, kernel);  // the program's own kernel stays as built
	original->kernel_id_ = imported->kernel_id_ = 0;
	original->kernel_name_ = imported->kernel_name_ = "kernel_0";
	original->verbatim = imported->verbatim = kernel->verbatim;
	std::vector<Kernel*> a = GenerateHIPKernelFamily(program, original, give_id);
	next_id = 1;
	std::vector<Kernel*> b = GenerateHIPKernelFamily(&imported_program, imported, give_id);
	if (a.size() != b.size()) return label + ": " + std::to_string(b.size()) + " kernels emitted from the imported tree, " + std::to_string(a.size()) + " from the original";
	for (size_t i = 0; i < a.size(); i++) {
		if (a[i]->full_generated_code_ != b[i]->full_generated_code_) {
			// first differing line
			std::istringstream sa(a[i]->full_generated_code_), sb(b[i]->full_generated_code_);
			std::string la, lb;
			int line = 0;
			while (true) {
				const bool ha = (bool)std::getline(sa, la), hb = (bool)std::getline(sb, lb);
				line++;
				if (!ha && !hb) break;
				if (la != lb || ha != hb) break;
			}
			return label + " (member " + std::to_string(i) + "): emitted text differs at line " + std::to_string(line) + ":\n  original: " + la + "\n  imported: " + lb;
		}
		const std::string ia = Describe(MakeKernelInfo(a[i])), ib = Describe(MakeKernelInfo(b[i]));
		if (ia != ib) return label + " (member " + std::to_string(i) + "): kernel info differs:\n  original: " + ia + "\n  imported: " + ib;
		if (a[i]->var_names != b[i]->var_names || a[i]->var_types != b[i]->var_types) return label + ": variable block differs";
	}
	// 3. slots are honoured whatever order the maps hold them in
	{
		Program reversed_program;
		std::unique_ptr<mirror::Exported> reversed = mirror::ExportKernel(kernel, true);
		KernelImporter<mirror::Tree> again(&reversed_program);
		Kernel* r = again.Import(&reversed->kernel);
		auto names = [](const std::vector<Node*>& nodes) {
			std::vector<std::string> out;
			for (const Node* n : nodes) out.push_back(n->debug_name);
			return out;
		};
		auto reversed_names = [&](const std::vector<Node*>& nodes) {
			std::vector<std::string> out = names(nodes);
			return std::vector<std::string>(out.rbegin(), out.rend());
		};
		if (names(r->read_write_memory) != reversed_names(kernel->read_write_memory) || names(r->read_only_memory) != reversed_names(kernel->read_only_memory))
			return label + ": buffers are not bound by slot";
		for (size_t i = 0; i < r->variables.size(); i++)
			if (r->variables[i].name != kernel->variables[kernel->variables.size() - 1 - i].name) return label + ": variables are not bound by slot";
	}
	return "";
}

long Report(const std::string& text, long status, char* out, size_t cap) {
	if (out && cap) {
		std::strncpy(out, text.c_str(), cap - 1);
		out[cap - 1] = 0;
	}
	return status;
}

}  // namespace

// Round trip of every emitted kernel of a registered program. Returns the number of kernels checked, or -1 with the
// first difference in `out`.
extern "C" long tftest_import_roundtrip_program(const char* name, const int64_t* params, size_t n_params, char* out, size_t cap) {
	try {
		auto it = ProgramRegistry().find(name);
		if (it == ProgramRegistry().end()) return Report(std::string("Unknown program: ") + name, -1, out, cap);
		Program program;
		program.program_name = name;
		it->second(&program, std::vector<int64_t>(params, params + n_params));
		long checked = 0;
		const size_t count = program.kernels_.size();
		for (size_t i = 0; i < count; i++) {
			Kernel* kernel = program.kernels_[i].get();
			if (!kernel->primitive.empty()) continue;
			const std::string problem = RoundTrip(&program, kernel, std::string(name) + " kernel " + std::to_string(i));
			if (!problem.empty()) return Report(problem, -1, out, cap);
			checked++;
		}
		return Report("", checked, out, cap);
	} catch (const std::exception& e) {
		return Report(std::string("exception: ") + e.what(), -1, out, cap);
	}
}

// What the importer says about trees that are not in post-lowering form. `defect`: 0 an operation a kernel cannot
// contain, 1 two Index arguments on a load, 2 an argument outside the kernel that is not bound, 3 binding slots with a
// gap, 4 a group size on the kernel node that contradicts the index arithmetic. Returns 0 and the message in `out`
// when the importer refuses, -1 when it accepts.
extern "C" long tftest_import_defect(int defect, char* out, size_t cap) {
	try {
		Program program;
		KernelBuilder kb(&program, 1);
		V n = kb.Var("n", TFType_Int);
		V x = kb.Buffer("x", true);
		V y = kb.Buffer("y", false);
		std::vector<V> idx = kb.ThreadIndices({n});
		kb.Store(y, idx[0], kb.Load(x, idx[0], TFType_Float) * kb.Const(2.0f));
		Kernel* kernel = kb.Finish();
		std::unique_ptr<mirror::Exported> e = mirror::ExportKernel(kernel, false);
		mirror::Node* guard = nullptr;
		for (mirror::Node* c = e->kernel.root->child; c; c = c->next)
			if (c->op->name_ == "if") guard = c;
		mirror::Node* load = nullptr;
		for (mirror::Node* c = guard->child; c && c->valid(); c = c->next)
			if (c->op->name_ == "load") load = c;
		static mirror::Operation dim_id{"dim_id"};
		static mirror::Operation constant{"const"};
		mirror::Node stray;
		stray.flags.remove(mirror::NodeProp::Placeholder);
		stray.op = &constant;
		stray.var_name = "stray";
		switch (defect) {
			case 0: load->op = &dim_id; break;
			case 1: load->args.AddArgument(mirror::ArgType::Index, 1, load->args.Get(mirror::ArgType::Index, 0)); break;
			case 2: load->args.AddArgument(mirror::ArgType::Index, 0, &stray); break;
			case 3: e->kernel.read_write_memory.begin()->second = 5; break;
			case 4: e->kernel.root->group_size = {64}; break;
			default: return Report("unknown defect", -2, out, cap);
		}
		Program into;
		KernelImporter<mirror::Tree> importer(&into);
		importer.Import(&e->kernel);
		return Report("accepted", -1, out, cap);
	} catch (const std::exception& e) {
		return Report(e.what(), 0, out, cap);
	}
}

// The round trip for a kernel that is already built (kernel_text.cpp: kernels parsed from text the reference printed).
std::string ImportRoundTripOf(tfhost::Program* program, tfhost::Kernel* kernel, const std::string& label) { return RoundTrip(program, kernel, label); }
