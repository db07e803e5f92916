// TensorFrost/Backend/CodeGen/Langs/HIP.cpp -- the HIP arm of the kernel-language switch.
//
// Stands beside Langs/CPP.cpp, Langs/GLSL.cpp and Langs/HLSL.cpp and has their contract (GenerateCPPKernel,
// Backend/CodeGen/Langs/CPP.cpp:720-779; GenerateGLSLKernel, Langs/GLSL.cpp:146-186): GenerateKernel
// (Backend/CodeGen/Generators.cpp:9-23) calls GenerateHIPKernel(program, kernel) once per kernel, after
// GenerateNodeNames has named the nodes and KernelManager::AddKernelID has numbered the kernel
// (Langs/CPP.cpp:557-566), and expects kernel->full_generated_code_, generated_header_ / _bindings_ / _main_,
// var_names and var_types filled.
//
// This file belongs to a TensorFrost checkout and is compiled there (it includes the compiler's headers); this
// repository keeps it under csrc/reference_side/ in the place it has in that tree and only runs the compiler over it
// where the reference's headers are present. It does three things:
//   1. reads the kernel out of the compiler's tree (KernelImporter over TensorFrost's own Node / Kernel / ArgType /
//      NodeProp, langs/tree_import.h) into the emitter's form;
//   2. runs the emitter on it (hip_generator.h), together with the further kernels a dispatch may need -- those get
//      kernel ids of their own from the same KernelManager and are compiled with the kernel they belong to;
//   3. copies the generated text back and hands the kernel manager what the emitter decided
//      (HipKernelManager::SetKernelInfo).
// The emitter's own sources (tf_ir, hip_generator, hip_prelude, idiom_matcher, kernel_geometry, hip_kernel_family,
// sort_composition; namespace tfhost) are compiled into the tree unchanged and know nothing of it.
#include <memory>
#include <string>
#include <unordered_map>
#include <vector>

#include "Compiler/KernelGen.h"
#include "Backend/KernelManager.h"
#include "Backend/Backends/HIP/HIP.h"

#include "hip_generator.h"
#include "langs/tree_import.h"

namespace TensorFrost {

// The compiler's types under the names KernelImporter asks for.
struct CompilerTree {
	using Node = TensorFrost::Node;
	using Kernel = TensorFrost::Kernel;
	using ArgType = TensorFrost::ArgType;
	using NodeProp = TensorFrost::NodeProp;
};

namespace {

// Per program: the imported kernels (the emitter's trees live as long as the program's text may be regenerated) and
// the kernels that exist only on the HIP side. The latter are `Kernel` objects without a tree: id, name and text are
// all that CompileKernel and the kernel manager read of them.
struct ImportedProgram {
	tfhost::Program trees;
	std::vector<std::unique_ptr<Kernel>> further_kernels;
	std::unordered_map<size_t, std::vector<Kernel*>> further_of;  // kernel id -> the kernels generated with it
};

std::unordered_map<Program*, std::unique_ptr<ImportedProgram>>& ImportedPrograms() {
	static std::unordered_map<Program*, std::unique_ptr<ImportedProgram>> programs;
	return programs;
}

void CopyGeneratedText(const tfhost::Kernel* from, Kernel* to) {
	to->full_generated_code_ = from->full_generated_code_;
	to->generated_header_ = from->generated_header_;
	to->generated_bindings_ = from->generated_bindings_;
	to->generated_main_ = from->generated_main_;
	to->var_names = from->var_names;
	to->var_types = from->var_types;
}

}  // namespace

void GenerateHIPKernel(Program* program, Kernel* kernel) {
	auto& slot = ImportedPrograms()[program];
	if (!slot) slot = std::make_unique<ImportedProgram>();
	ImportedProgram& imported = *slot;
	imported.trees.program_name = program->program_name;

	tfhost::KernelImporter<CompilerTree> importer(&imported.trees);
	tfhost::Kernel* tree = importer.Import(kernel);
	tree->kernel_id_ = kernel->kernel_id_;
	tree->kernel_name_ = kernel->kernel_name_;

	std::unordered_map<tfhost::Kernel*, Kernel*> holder_of;
	std::vector<tfhost::Kernel*> family = tfhost::GenerateHIPKernelFamily(&imported.trees, tree, [&](tfhost::Kernel* further) {
		imported.further_kernels.push_back(std::make_unique<Kernel>());
		Kernel* holder = imported.further_kernels.back().get();
		holder->root = nullptr;
		global_kernel_manager->AddKernelID(program, holder);
		holder->kernel_name_ = "kernel_" + to_string(holder->kernel_id_);
		further->kernel_id_ = holder->kernel_id_;
		further->kernel_name_ = holder->kernel_name_;
		holder_of[further] = holder;
		imported.further_of[kernel->kernel_id_].push_back(holder);
	});

	CopyGeneratedText(tree, kernel);
	for (auto& [further, holder] : holder_of) CopyGeneratedText(further, holder);
	if (auto* hip = dynamic_cast<HipKernelManager*>(global_kernel_manager))
		for (tfhost::Kernel* member : family) hip->SetKernelInfo(tfhost::MakeKernelInfo(member));
}

// The HIP arm of CompileKernels (Backend/Backend.cpp:75-94): the kernel, then the kernels generated with it.
void CompileHIPKernel(Program* program, Kernel* kernel) {
	auto* hip = dynamic_cast<HipKernelManager*>(global_kernel_manager);
	if (hip == nullptr) throw std::runtime_error("The HIP backend is not initialized");
	hip->CompileKernel(kernel);
	auto imported = ImportedPrograms().find(program);
	if (imported == ImportedPrograms().end()) return;
	auto further = imported->second->further_of.find(kernel->kernel_id_);
	if (further == imported->second->further_of.end()) return;
	for (Kernel* k : further->second) hip->CompileKernel(k);
}

// When a program is unloaded (Program::unload_callback, Compiler/KernelGen.h:52).
void ForgetHIPProgram(Program* program) { ImportedPrograms().erase(program); }

}  // namespace TensorFrost
