#include "registry.h"

namespace tfhost {

std::map<std::string, ProgramFactory>& ProgramRegistry() {
	static std::map<std::string, ProgramFactory> registry;
	return registry;
}

Program* CreateProgram(const std::string& name, const std::vector<int64_t>& params) {
	auto it = ProgramRegistry().find(name);
	if (it == ProgramRegistry().end()) throw std::runtime_error("Unknown program: " + name);
	if (current_backend == BackendType::NotInitialized) throw std::runtime_error("Backend not initialized");
	Program* program = new Program();
	program->program_name = name;
	try {
		it->second(program, params);
		GenerateCode(program);
		CompileKernels(program);
	} catch (...) {
		if (global_kernel_manager) global_kernel_manager->RemoveProgram(program);
		delete program;
		throw;
	}
	return program;
}

void DestroyProgram(Program* program) {
	if (!program) return;
	if (global_kernel_manager) {
		if (auto* hip = dynamic_cast<HipKernelManager*>(global_kernel_manager))
			for (auto& k : program->kernels_) hip->FreeKernel(k->kernel_id_);
		global_kernel_manager->RemoveProgram(program);
	}
	delete program;
}

}  // namespace tfhost
