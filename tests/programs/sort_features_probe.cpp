// What AnalyzeSortFeatures (csrc/host/sort_features.cpp) finds in the kernels of a registered program, as text: one
// line per emitted kernel. Lets the CPU tests check the analysis the `Radix sort` region is followed by without a GPU.
#include <cstring>
#include <sstream>

#include "registry.h"
#include "sort_composition.h"

namespace {

std::string Text(const tfhip::DimExpr& d) {
	std::ostringstream o;
	if (d.terms.empty()) o << "0";
	for (size_t t = 0; t < d.terms.size(); t++) {
		if (t) o << "+";
		o << d.terms[t].second;
		for (int v : d.terms[t].first) o << "*v" << v;
	}
	return o.str();
}

}  // namespace

// mutate: 0 nothing; 1 the scatter also stores the key into the scan table's neighbour... (see cases below). Each
// changes the scatter kernel of the composition so that it is no longer `move the element to a computed place`.
extern "C" long tftest_sort_features(const char* name, const int64_t* params, size_t n_params, int mutate, char* out, size_t cap) {
	using namespace tfhost;
	std::string text;
	long status = 0;
	try {
		auto it = ProgramRegistry().find(name);
		if (it == ProgramRegistry().end()) throw std::runtime_error(std::string("Unknown program: ") + name);
		Program program;
		it->second(&program, std::vector<int64_t>(params, params + n_params));
		const size_t count = program.kernels_.size();
		for (size_t i = 0; i < count; i++) {
			Kernel* k = program.kernels_[i].get();
			if (!k->primitive.empty()) continue;
			if (mutate && !k->group_memory.empty()) {
				// the scatter kernel: find its stores to global memory
				std::vector<Node*> stores;
				std::function<void(Node*)> walk = [&](Node* n) {
					if (std::string(n->op->name) == "store" && !n->local_memory_op) stores.push_back(n);
					for (Node* c : n->children) walk(c);
				};
				walk(k->root);
				if (stores.size() != 2) throw std::runtime_error("expected the scatter's two stores");
				switch (mutate) {
					case 1: stores[1]->index = stores[1]->inputs[0]->index; break;  // values go to their own element, not to the key's place
					case 2: stores[0]->inputs[0] = stores[1]->inputs[0]; break;    // both stores write the value
					case 3: {                                                     // the key is stored shifted by one bit
						KernelBuilder kb(&program, 1);
						Node* one = kb.ConstU(1u).n;
						Node* sh = (V(stores[0]->inputs[0], &kb) << V(one, &kb)).n;
						stores[0]->inputs[0] = sh;
						break;
					}
					case 4: stores[0]->op = &FindOperation("InterlockedAdd"); break;  // an atomic instead of a store
					default: throw std::runtime_error("unknown mutation");
				}
			}
			AnalyzeSortFeatures(k);
			const auto& f = k->sort;
			std::ostringstream o;
			o << "kernel " << i << ": copies=";
			for (auto& c : f.copies) o << "[" << c.dst << "<-" << c.src << " map" << c.map << " n=" << Text(c.extent) << "]";
			o << " only=" << f.copies_only << " digits=";
			for (auto& d : f.digits) o << "[b" << d.keys << ">>" << Text(d.shift) << "&" << d.mask << "]";
			o << " scatter=" << f.scatter;
			if (f.scatter) o << "[k" << f.keys_out << "<-" << f.keys_in << " v" << f.values_out << "<-" << f.values_in << " >>" << Text(f.scatter_shift) << "&" << f.scatter_mask << " n=" << Text(f.scatter_n) << "]";
			text += o.str() + "\n";
			status++;
		}
	} catch (const std::exception& e) {
		text = std::string("exception: ") + e.what();
		status = -1;
	}
	if (out && cap) {
		std::strncpy(out, text.c_str(), cap - 1);
		out[cap - 1] = 0;
	}
	return status;
}
